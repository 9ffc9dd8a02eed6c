"""Public argument contract shared by the operator, its oracle and the tests.

Mirrors the behaviour of the reference's ``rosa_soft/soft_contract.py``:
defaults (``:12-15``), the dropout seed rule (``:18-31``), static control
validation (``:34-66``), dense and packed input validation (``:69-129``,
``:132-208``) and the float32 representability checks (``:211-248``).  Error
types and message texts are kept because callers and tests match on them.
"""

from __future__ import annotations

import math
import operator
from typing import Sequence

import torch
from torch import Tensor

ROSA_SOFT_DEFAULT_SCALE = 1.0
ROSA_SOFT_DEFAULT_DROPOUT_P = 0.0
ROSA_SOFT_DEFAULT_MISMATCH_SCALE = 3.0
ROSA_SOFT_NULL_ROUTE_SCORE = 0.5

_MAX_DROPOUT_P = 1.0 - 2.0**-24
_INT64_MAX = torch.iinfo(torch.int64).max


def make_dropout_seed(reference: Tensor, dropout_p: float, needs_backward: bool) -> Tensor:
    """Return the int64 seed tensor the backward pass is keyed on.

    Empty when no mask will ever be drawn (``dropout_p == 0`` or no backward),
    otherwise one scalar drawn from the generator of ``reference``'s device, so
    a no-grad or ``p == 0`` call never touches any RNG state.
    """

    wants_mask = needs_backward and float(dropout_p) != 0.0
    if not wants_mask:
        return torch.empty(0, dtype=torch.int64, device=reference.device)
    return torch.randint(0, _INT64_MAX, (), dtype=torch.int64, device=reference.device)


def _is_positive_finite(value) -> bool:
    if isinstance(value, bool):
        return False
    as_float = float(value)
    return math.isfinite(as_float) and as_float > 0.0


def _validate_static_controls(
    max_suffix_length: int,
    scale: float,
    dropout_p: float,
    mismatch_scale: float,
    sequence_length_bound: int,
) -> int:
    if isinstance(max_suffix_length, bool):
        raise TypeError("max_suffix_length must be an integer")
    try:
        horizon = operator.index(max_suffix_length)
    except TypeError as error:
        raise TypeError("max_suffix_length must be an integer") from error
    if horizon < 1:
        raise ValueError("max_suffix_length must be >= 1")
    if not _is_positive_finite(scale):
        raise ValueError("scale must be finite and > 0")
    dropout_ok = (
        not isinstance(dropout_p, bool)
        and math.isfinite(float(dropout_p))
        and 0.0 <= float(dropout_p) <= _MAX_DROPOUT_P
    )
    if not dropout_ok:
        raise ValueError("dropout_p must be finite and in [0, 1 - 2^-24]")
    if not _is_positive_finite(mismatch_scale):
        raise ValueError("mismatch_scale must be finite and > 0")
    return min(horizon, int(sequence_length_bound))


def _require(condition: bool, message: str) -> None:
    if not condition:
        raise ValueError(message)


def _same(values: Sequence) -> bool:
    return all(value == values[0] for value in values[1:])


def validate_rosa_soft_inputs(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    max_suffix_length: int,
    scale: float,
    dropout_p: float,
    mismatch_scale: float,
) -> int:
    """Check a dense ``(B, T, H, D)`` call; return ``min(max_suffix_length, T)``."""

    tensors = (query, key, value)
    _require(
        all(tensor.ndim == 4 for tensor in tensors),
        "query, key, and value must have shape (B, T, H, D)",
    )
    _require(
        _same([tuple(tensor.shape[:2]) for tensor in tensors]),
        "all inputs must share batch and sequence dimensions",
    )
    heads, value_heads = query.size(2), value.size(2)
    _require(heads == key.size(2), "query and key head counts must match")
    _require(
        heads >= 1 and value_heads >= 1,
        "query and value must have at least one head",
    )
    _require(
        heads % value_heads == 0,
        "query heads must be divisible by value heads",
    )
    _require(
        query.size(3) == key.size(3),
        "query and key symbol dimensions must match",
    )
    _require(
        query.size(0) >= 1 and query.size(1) >= 1 and value.size(3) >= 1,
        "batch, sequence, and value dimensions must be >= 1",
    )
    _require(
        1 <= query.size(3) <= 32,
        "query/key symbol dimension must be in [1, 32]",
    )
    _require(
        _same([tensor.device for tensor in tensors]),
        "all inputs must be on the same device",
    )
    _require(
        _same([tensor.dtype for tensor in tensors]),
        "all inputs must have the same dtype",
    )
    _require(
        all(tensor.is_floating_point() for tensor in tensors),
        "all inputs must be floating-point tensors",
    )
    return _validate_static_controls(
        max_suffix_length, scale, dropout_p, mismatch_scale, query.size(1)
    )


def check_cu_seqlens_values(offsets: Sequence[int], total_tokens: int) -> None:
    """Host-side check of packed-sequence offsets (start, end, monotone)."""

    _require(offsets[0] == 0, "cu_seqlens must start at zero")
    _require(
        offsets[-1] == total_tokens,
        "cu_seqlens must end at the packed token count",
    )
    _require(
        all(left <= right for left, right in zip(offsets, offsets[1:])),
        "cu_seqlens must be nondecreasing",
    )


def validate_rosa_soft_varlen_inputs(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    cu_seqlens: Tensor,
    max_suffix_length: int,
    scale: float,
    dropout_p: float,
    mismatch_scale: float,
) -> int:
    """Check a packed ``(N, H, D)`` call; return ``min(max_suffix_length, N)``.

    Offset *values* are inspected only when ``cu_seqlens`` lives on the host:
    reading device offsets would force a synchronisation, so the device path
    validates them inside the launch instead.
    """

    tensors = (query, key, value)
    _require(
        all(tensor.ndim == 3 for tensor in tensors),
        "query, key, and value must have shape (N, H, D)",
    )
    _require(
        _same([tensor.size(0) for tensor in tensors]),
        "all inputs must share the packed token dimension",
    )
    _require(query.size(0) >= 1, "packed token dimension must be >= 1")
    _require(
        query.size(2) == key.size(2),
        "query and key symbol dimensions must match",
    )
    heads, value_heads = query.size(1), value.size(1)
    _require(heads == key.size(1), "query and key head counts must match")
    _require(
        heads >= 1 and value_heads >= 1,
        "query and value must have at least one head",
    )
    _require(
        heads % value_heads == 0,
        "query heads must be divisible by value heads",
    )
    _require(
        1 <= query.size(2) <= 32,
        "query/key symbol dimension must be in [1, 32]",
    )
    _require(value.size(2) >= 1, "value dimension must be >= 1")
    _require(
        _same([tensor.device for tensor in (*tensors, cu_seqlens)]),
        "all inputs and cu_seqlens must be on the same device",
    )
    _require(
        _same([tensor.dtype for tensor in tensors]),
        "all floating-point inputs must have the same dtype",
    )
    _require(
        all(tensor.is_floating_point() for tensor in tensors),
        "query, key, and value must be floating-point tensors",
    )
    _require(
        cu_seqlens.ndim == 1 and cu_seqlens.numel() >= 2,
        "cu_seqlens must be a one-dimensional int32 tensor",
    )
    _require(cu_seqlens.dtype == torch.int32, "cu_seqlens must have dtype int32")
    if not cu_seqlens.is_cuda:
        check_cu_seqlens_values(cu_seqlens.tolist(), query.size(0))
    return _validate_static_controls(
        max_suffix_length, scale, dropout_p, mismatch_scale, query.size(0)
    )


def validate_fp32_surrogate_scalars(
    max_suffix_length: int,
    scale: float,
    dropout_p: float,
    mismatch_scale: float,
) -> None:
    """Reject controls whose float32 images (or products) leave the normal range.

    The device computes every score in float32, so ``scale``,
    ``mismatch_scale``, ``W * scale``, ``W * scale * mismatch_scale`` and
    ``1 / (1 - dropout_p)`` must all be finite normal float32 numbers.
    """

    limits = torch.finfo(torch.float32)
    scale = float(scale)
    mismatch_scale = float(mismatch_scale)
    if not (math.isfinite(scale) and limits.tiny <= scale <= limits.max):
        raise ValueError(
            "scale must be representable as a positive normal float32 value"
        )
    if scale > limits.max / float(max_suffix_length):
        raise ValueError("max_suffix_length * scale must fit in float32")
    inverse_keep = 1.0 / (1.0 - float(dropout_p))
    if not (math.isfinite(inverse_keep) and inverse_keep <= limits.max):
        raise ValueError("1 / (1 - dropout_p) must fit in float32")
    if not limits.tiny <= mismatch_scale <= limits.max:
        raise ValueError(
            "mismatch_scale must be representable as a positive normal "
            "float32 value"
        )
    if mismatch_scale > limits.max / (float(max_suffix_length) * scale):
        raise ValueError(
            "mismatch_scale * max_suffix_length * scale must fit in float32"
        )
