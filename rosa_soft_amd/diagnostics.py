"""Selected-route inspection of the hard forward on the device.

The reference inspects a call through its PyTorch oracle
(``rosa_soft/testing.py:28-117``), which materialises ``O(T^2)`` tensors and is
therefore limited to toy shapes.  The HIP forward already knows, for every row,
which route it selected and how long the exact match was; this module exposes
exactly that, at training shapes, in the vocabulary of the reference's
``RosaSoftInspection`` (``selected_route_indices``, ``exact_suffix_lengths`` taken
at the selected route) and of the route statistics of
``examples/fit_soft_reference.py:419-459``.
"""

from dataclasses import dataclass
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import cabi
from .soft_contract import validate_rosa_soft_inputs, validate_rosa_soft_varlen_inputs


@dataclass(frozen=True)
class HardRouteInspection:
    """What the hard forward selected, per (token, head)."""

    selected_route_indices: Tensor   # int32, 0 = null route, else 1 <= a <= t (sequence-local)
    selected_suffix_lengths: Tensor  # int32, exact matched suffix length of that route, 0 = null
    effective_max_suffix_length: int

    @property
    def null_route_mask(self) -> Tensor:
        return self.selected_route_indices == 0

    def route_stats(self) -> dict:
        """Null-route rate and match-length summary (host floats)."""

        lengths = self.selected_suffix_lengths
        hit = lengths > 0
        hits = int(hit.sum())
        return {
            "null_rate": 1.0 - hits / max(lengths.numel(), 1),
            "mean_match_length": float(lengths[hit].float().mean()) if hits else 0.0,
            "max_match_length": int(lengths.max()) if lengths.numel() else 0,
            "saturated_rate": float((lengths >= self.effective_max_suffix_length).float().mean())
            if lengths.numel() else 0.0,
        }


@torch.no_grad()
def inspect_hard_routes(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    cu_seqlens: Optional[Tensor] = None,
    *,
    max_suffix_length: int = 32,
) -> Tuple[Tensor, HardRouteInspection]:
    """Run the hard forward on the device and return ``(output, inspection)``.

    Same inputs and validation as ``rosa_soft`` / ``rosa_soft_varlen``; the output
    equals theirs bit for bit.
    """

    if cu_seqlens is None:
        horizon = validate_rosa_soft_inputs(query, key, value, max_suffix_length, 1.0, 0.0, 1.0)
    else:
        horizon = validate_rosa_soft_varlen_inputs(
            query, key, value, cu_seqlens, max_suffix_length, 1.0, 0.0, 1.0
        )
    if not query.is_cuda:
        raise RuntimeError("inspect_hard_routes runs the HIP forward and needs device tensors")
    output, routes, lengths = cabi.hard_routes(
        query.contiguous(), key.contiguous(), value.contiguous(), max_suffix_length, cu_seqlens
    )
    return output, HardRouteInspection(
        selected_route_indices=routes,
        selected_suffix_lengths=lengths,
        effective_max_suffix_length=int(horizon),
    )
