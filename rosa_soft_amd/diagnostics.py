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


# ---------------------------------------------------------------------------
# summaries (the part of rosa_soft/diagnostics.py that needs no T x T tensor)
# ---------------------------------------------------------------------------

def _nan_scalar(like: Tensor) -> Tensor:
    return torch.full((), float("nan"), device=like.device, dtype=torch.float32)


def _quantile(values: Tensor, q: float) -> Tensor:
    """``torch.quantile`` (linear interpolation) without its limit of 16 M elements."""

    flat = values.flatten().float()
    if flat.numel() <= 1 << 24:
        return torch.quantile(flat, q)
    ordered = flat.sort().values
    position = q * (ordered.numel() - 1)
    low = int(position)
    high = min(low + 1, ordered.numel() - 1)
    return torch.lerp(ordered[low], ordered[high], position - low)


@dataclass(frozen=True)
class TensorGradientDiagnostics:
    """Scale and support of one gradient tensor (rosa_soft/diagnostics.py:80-88)."""

    l2_norm: Tensor
    rms: Tensor
    max_abs: Tensor
    finite_fraction: Tensor
    nonzero_fraction: Tensor
    feature_rms_cv: Tensor


@dataclass(frozen=True)
class RosaSoftGradientDiagnostics:
    """rosa_soft/diagnostics.py:91-110."""

    query: TensorGradientDiagnostics
    key: TensorGradientDiagnostics
    value: TensorGradientDiagnostics
    qk_to_value_norm_ratio: Tensor

    def as_float_dict(self) -> dict:
        values = {}
        for role in ("query", "key", "value"):
            summary = getattr(self, role)
            for name in summary.__dataclass_fields__:
                values[f"{role}_{name}"] = float(getattr(summary, name).detach().float().cpu())
        values["qk_to_value_norm_ratio"] = float(self.qk_to_value_norm_ratio.detach().float().cpu())
        return values


def _summarize_gradient(gradient: Tensor) -> TensorGradientDiagnostics:
    # rosa_soft/diagnostics.py:362-387: norms over the finite elements, the spread of the
    # per-feature rms (last axis) as a coefficient of variation
    values = gradient.detach().float()
    finite = torch.isfinite(values)
    kept = values.masked_select(finite)
    if kept.numel() == 0:
        l2_norm = rms = max_abs = spread = _nan_scalar(values)
    else:
        l2_norm = kept.norm()
        rms = kept.square().mean().sqrt()
        max_abs = kept.abs().max()
        feature_rms = values.square().mean(dim=tuple(range(values.ndim - 1))).sqrt()
        spread = feature_rms.std(unbiased=False) / feature_rms.mean().clamp_min(
            torch.finfo(torch.float32).tiny)
    return TensorGradientDiagnostics(
        l2_norm=l2_norm,
        rms=rms,
        max_abs=max_abs,
        finite_fraction=finite.float().mean(),
        nonzero_fraction=(finite & (values != 0)).float().mean(),
        feature_rms_cv=spread,
    )


@torch.no_grad()
def summarize_rosa_soft_gradients(grad_query: Tensor, grad_key: Tensor,
                                  grad_value: Tensor) -> RosaSoftGradientDiagnostics:
    """Scale, support and feature balance of the three gradients, and the ratio of the
    symbol-side norm to the value-side norm (rosa_soft/diagnostics.py:390-415); device tensors
    stay on the device."""

    query = _summarize_gradient(grad_query)
    key = _summarize_gradient(grad_key)
    value = _summarize_gradient(grad_value)
    qk_norm = (query.l2_norm.square() + key.l2_norm.square()).sqrt()
    if float(value.l2_norm) == 0.0:
        ratio = torch.where(qk_norm == 0, _nan_scalar(qk_norm),
                            torch.full_like(qk_norm, float("inf")))
    else:
        ratio = qk_norm / value.l2_norm
    return RosaSoftGradientDiagnostics(query=query, key=key, value=value,
                                       qk_to_value_norm_ratio=ratio)


@dataclass(frozen=True)
class HardRouteDiagnostics:
    """The fields of the reference's ``RosaSoftDiagnostics`` (rosa_soft/diagnostics.py:26-58)
    that the selected routes and the logits determine; its other fields summarise the T x T
    route probabilities of the oracle, which the device path never forms."""

    quantile: float
    route_rows: int
    hard_nonnull_route_fraction: Tensor
    hard_route_lag_mean: Tensor
    max_exact_suffix_length: Tensor
    query_positive_fraction: Tensor
    key_positive_fraction: Tensor
    query_bit_imbalance: Tensor
    key_bit_imbalance: Tensor
    query_sign_margin_mean: Tensor
    key_sign_margin_mean: Tensor
    query_sign_margin_low_quantile: Tensor
    key_sign_margin_low_quantile: Tensor
    query_softsign_derivative_mean: Tensor
    key_softsign_derivative_mean: Tensor

    def as_float_dict(self) -> dict:
        values = {"quantile": self.quantile, "route_rows": float(self.route_rows)}
        for name in self.__dataclass_fields__:
            if name not in values:
                values[name] = float(getattr(self, name).detach().float().cpu())
        return values


def _symbol_health(logits: Tensor, low_quantile: float):
    # rosa_soft/diagnostics.py:189-207
    logits = logits.float()
    positive = logits > 0
    per_bit = positive.float().mean(dim=tuple(range(logits.ndim - 1)))
    margins = logits.abs()
    return (
        positive.float().mean(),
        (2.0 * (per_bit - 0.5).abs()).mean(),
        margins.mean(),
        _quantile(margins, low_quantile),
        (1.0 + margins).square().reciprocal().mean(),
    )


@torch.no_grad()
def summarize_hard_routes(inspection: HardRouteInspection, query: Tensor, key: Tensor,
                          cu_seqlens: Optional[Tensor] = None,
                          quantile: float = 0.95) -> HardRouteDiagnostics:
    """Summarise an inspection of ``inspect_hard_routes`` and the logits it was made from.

    ``hard_route_lag_mean`` is the mean of ``t - route`` over the routed rows, ``t`` counted
    inside the row's sequence; ``max_exact_suffix_length`` the longest match of any row (the
    selected route is a longest one, so this is the maximum over all routes).
    """

    if isinstance(quantile, bool) or not isinstance(quantile, (int, float)):
        raise TypeError("quantile must be a real number")
    quantile = float(quantile)
    if not 0.0 <= quantile <= 1.0:  # (also false for NaN)
        raise ValueError("quantile must be in [0, 1]")
    routes = inspection.selected_route_indices
    lengths = inspection.selected_suffix_lengths
    # routes are [B, T, H] (dense) or [N, H] (packed): the row index runs along axis -2
    positions = torch.arange(routes.size(-2), device=routes.device)
    if cu_seqlens is not None:  # count inside the row's sequence
        offsets = cu_seqlens.to(routes.device).long()
        sequence = torch.searchsorted(offsets, positions, right=True) - 1
        positions = positions - offsets[sequence]
    positions = positions.unsqueeze(-1)
    routed = routes > 0
    lag = (positions - routes).masked_select(routed)
    query_health = _symbol_health(query, 1.0 - quantile)
    key_health = _symbol_health(key, 1.0 - quantile)
    return HardRouteDiagnostics(
        quantile=quantile,
        route_rows=routes.numel(),
        hard_nonnull_route_fraction=routed.float().mean(),
        hard_route_lag_mean=lag.float().mean() if lag.numel() else _nan_scalar(routes),
        max_exact_suffix_length=lengths.max() if lengths.numel() else torch.zeros(
            (), dtype=lengths.dtype, device=lengths.device),
        query_positive_fraction=query_health[0],
        key_positive_fraction=key_health[0],
        query_bit_imbalance=query_health[1],
        key_bit_imbalance=key_health[1],
        query_sign_margin_mean=query_health[2],
        key_sign_margin_mean=key_health[2],
        query_sign_margin_low_quantile=query_health[3],
        key_sign_margin_low_quantile=key_health[3],
        query_softsign_derivative_mean=query_health[4],
        key_softsign_derivative_mean=key_health[4],
    )
