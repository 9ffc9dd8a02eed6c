"""Public ``rosa_soft`` / ``rosa_soft_varlen`` operators on the MI355X kernels.

Same call surface and behaviour as the reference's ``rosa_soft/soft.py``:
keyword-only controls with the same defaults (``:417-426``, ``:462-472``),
validation before anything is launched (``:29-100``), a no-grad fast path that
draws no seed (``:438-447``, ``:485-495``), one dropout seed per call drawn
from the device generator (``:449``), an autograd node that saves only the
inputs, the packed symbols and the seed (``:259-293``), a backward that asks
the device for exactly the gradients autograd needs (``:103-109``,
``:296-332``) and casts the float32 results back to the input dtype
(``:112-124``), and fake-tensor kernels for tracing (``:127-256``).

HIP tensors report ``is_cuda`` in PyTorch-ROCm, so the device checks read the
same as on the reference's platform.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor
from torch.autograd.function import once_differentiable

from .soft_contract import (
    ROSA_SOFT_DEFAULT_DROPOUT_P,
    ROSA_SOFT_DEFAULT_MISMATCH_SCALE,
    ROSA_SOFT_DEFAULT_SCALE,
    make_dropout_seed,
    validate_fp32_surrogate_scalars,
    validate_rosa_soft_inputs,
    validate_rosa_soft_varlen_inputs,
)

__all__ = [
    "ROSA_SOFT_DEFAULT_DROPOUT_P",
    "ROSA_SOFT_DEFAULT_MISMATCH_SCALE",
    "ROSA_SOFT_DEFAULT_SCALE",
    "rosa_soft",
    "rosa_soft_varlen",
]

_DEVICE_DTYPES = (torch.float32, torch.float16, torch.bfloat16)
_GRADIENT_BITS = (1, 2, 4)  # query, key, value


def _gradient_mask(needs_input_grad: Tuple[bool, ...]) -> int:
    return sum(bit for bit, need in zip(_GRADIENT_BITS, needs_input_grad[:3]) if need)


def _check_device_call(name: str, query: Tensor, horizon: int, scale, dropout_p, mismatch_scale) -> None:
    if not query.is_cuda:
        raise ValueError(f"{name} requires CUDA tensors")
    if query.dtype not in _DEVICE_DTYPES:
        raise ValueError(f"{name} supports float32, float16, and bfloat16")
    validate_fp32_surrogate_scalars(horizon, scale, dropout_p, mismatch_scale)


# ---------------------------------------------------------------------------
# shape functions for FakeTensor / torch.compile tracing
# ---------------------------------------------------------------------------

def _fake_forward_outputs(query: Tensor, value: Tensor, packed: bool):
    if packed:
        tokens, heads = query.shape[0], query.shape[1]
        output_shape, word_shape = (tokens, heads, value.shape[2]), (heads, tokens)
    else:
        batch, seq_len, heads = query.shape[0], query.shape[1], query.shape[2]
        output_shape, word_shape = (batch, seq_len, heads, value.shape[3]), (batch, heads, seq_len)
    return (
        query.new_empty(output_shape),
        query.new_empty(word_shape, dtype=torch.int32),
        query.new_empty(word_shape, dtype=torch.int32),
    )


def _fake_gradients(query: Tensor, key: Tensor, value: Tensor, gradient_mask: int):
    return tuple(
        tensor.new_empty(tensor.shape if gradient_mask & bit else (0,), dtype=torch.float32)
        for bit, tensor in zip(_GRADIENT_BITS, (query, key, value))
    )


@torch.library.register_fake("rosa_soft::hard_forward")
def _fake_hard_forward(query, key, value, max_suffix_length):
    return _fake_forward_outputs(query, value, packed=False)


@torch.library.register_fake("rosa_soft::hard_forward_varlen")
def _fake_hard_forward_varlen(query, key, value, cu_seqlens, max_suffix_length):
    return _fake_forward_outputs(query, value, packed=True)


@torch.library.register_fake("rosa_soft::surrogate_vjp_masked")
def _fake_surrogate_vjp_masked(
    query, key, value, grad_output, packed_query_symbols, packed_key_symbols, dropout_seed,
    max_suffix_length, scale, dropout_p, mismatch_scale, gradient_mask,
):
    return _fake_gradients(query, key, value, gradient_mask)


@torch.library.register_fake("rosa_soft::surrogate_vjp_varlen_masked")
def _fake_surrogate_vjp_varlen_masked(
    query, key, value, cu_seqlens, grad_output, packed_query_symbols, packed_key_symbols,
    dropout_seed, max_suffix_length, scale, dropout_p, mismatch_scale, gradient_mask,
):
    return _fake_gradients(query, key, value, gradient_mask)


# ---------------------------------------------------------------------------
# autograd nodes
# ---------------------------------------------------------------------------

def _cast_requested(gradients, inputs, needs_input_grad):
    return tuple(
        gradient.to(tensor.dtype) if need else None
        for gradient, tensor, need in zip(gradients, inputs, needs_input_grad)
    )


class _HardForwardSoftVjpFunction(torch.autograd.Function):
    """Dense layout: exact hard forward, surrogate backward."""

    @staticmethod
    def forward(ctx, query, key, value, dropout_seed, max_suffix_length, scale, dropout_p,
                mismatch_scale):
        output, packed_query, packed_key = torch.ops.rosa_soft.hard_forward(
            query, key, value, int(max_suffix_length)
        )
        ctx.controls = (int(max_suffix_length), float(scale), float(dropout_p), float(mismatch_scale))
        ctx.save_for_backward(query, key, value, packed_query, packed_key, dropout_seed)
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        query, key, value, packed_query, packed_key, dropout_seed = ctx.saved_tensors
        needs = ctx.needs_input_grad[:3]
        horizon, scale, dropout_p, mismatch_scale = ctx.controls
        gradients = torch.ops.rosa_soft.surrogate_vjp_masked(
            query, key, value, grad_output, packed_query, packed_key, dropout_seed,
            horizon, scale, dropout_p, mismatch_scale, _gradient_mask(needs),
        )
        return (*_cast_requested(gradients, (query, key, value), needs), None, None, None, None, None)


class _HardForwardSoftVjpVarlenFunction(torch.autograd.Function):
    """Packed layout: every sequence of ``cu_seqlens`` is an independent problem."""

    @staticmethod
    def forward(ctx, query, key, value, cu_seqlens, dropout_seed, max_suffix_length, scale,
                dropout_p, mismatch_scale):
        output, packed_query, packed_key = torch.ops.rosa_soft.hard_forward_varlen(
            query, key, value, cu_seqlens, int(max_suffix_length)
        )
        ctx.controls = (int(max_suffix_length), float(scale), float(dropout_p), float(mismatch_scale))
        ctx.save_for_backward(query, key, value, cu_seqlens, packed_query, packed_key, dropout_seed)
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        query, key, value, cu_seqlens, packed_query, packed_key, dropout_seed = ctx.saved_tensors
        needs = ctx.needs_input_grad[:3]
        horizon, scale, dropout_p, mismatch_scale = ctx.controls
        gradients = torch.ops.rosa_soft.surrogate_vjp_varlen_masked(
            query, key, value, cu_seqlens, grad_output, packed_query, packed_key, dropout_seed,
            horizon, scale, dropout_p, mismatch_scale, _gradient_mask(needs),
        )
        return (
            *_cast_requested(gradients, (query, key, value), needs),
            None, None, None, None, None, None,
        )


def _needs_backward(*tensors: Tensor) -> bool:
    return torch.is_grad_enabled() and any(tensor.requires_grad for tensor in tensors)


def _refuse_training_capture(name: str) -> None:
    """The no-grad forward can be recorded into a HIP graph; the training step cannot.

    Recording forward + surrogate backward with ``torch.cuda.graph`` ended in a host
    segmentation fault on this platform whose cause is not known, so the attempt is turned
    into an error before anything is launched.
    """

    if torch.compiler.is_compiling():  # tracing: nothing is being launched
        return
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError(
            f"{name}: the surrogate backward cannot be recorded into a HIP graph in this "
            "build; capture the forward under torch.no_grad() or run the training step eagerly"
        )


# ---------------------------------------------------------------------------
# public operators
# ---------------------------------------------------------------------------

def rosa_soft(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    *,
    max_suffix_length: int = 32,
    scale: float = ROSA_SOFT_DEFAULT_SCALE,
    dropout_p: float = ROSA_SOFT_DEFAULT_DROPOUT_P,
    mismatch_scale: float = ROSA_SOFT_DEFAULT_MISMATCH_SCALE,
) -> Tensor:
    """Exact hard ROSA forward with a dense attention-style surrogate VJP.

    ``query``/``key`` are ``(B, T, H, D)`` logits whose signs are the symbols
    (``D`` in 1..32), ``value`` is ``(B, T, Hv, Dv)`` with ``H % Hv == 0``.
    Returns ``(B, T, H, Dv)`` with entries in ``{-1, 0, +1}``.
    """

    horizon = validate_rosa_soft_inputs(
        query, key, value, max_suffix_length, scale, dropout_p, mismatch_scale
    )
    _check_device_call("rosa_soft", query, horizon, scale, dropout_p, mismatch_scale)
    if not _needs_backward(query, key, value):
        return torch.ops.rosa_soft.hard_forward(query, key, value, horizon)[0]
    _refuse_training_capture("rosa_soft")
    seed = make_dropout_seed(query, dropout_p, True)
    return _HardForwardSoftVjpFunction.apply(
        query, key, value, seed, horizon, float(scale), float(dropout_p), float(mismatch_scale)
    )


def rosa_soft_varlen(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    cu_seqlens: Tensor,
    *,
    max_suffix_length: int = 32,
    scale: float = ROSA_SOFT_DEFAULT_SCALE,
    dropout_p: float = ROSA_SOFT_DEFAULT_DROPOUT_P,
    mismatch_scale: float = ROSA_SOFT_DEFAULT_MISMATCH_SCALE,
) -> Tensor:
    """``rosa_soft`` applied independently to sequences packed along dim 0.

    ``query``/``key`` are ``(N, H, D)``, ``value`` is ``(N, Hv, Dv)`` and
    ``cu_seqlens`` is a device int32 tensor of ``S + 1`` cumulative offsets.
    """

    horizon = validate_rosa_soft_varlen_inputs(
        query, key, value, cu_seqlens, max_suffix_length, scale, dropout_p, mismatch_scale
    )
    _check_device_call("rosa_soft_varlen", query, horizon, scale, dropout_p, mismatch_scale)
    if not _needs_backward(query, key, value):
        return torch.ops.rosa_soft.hard_forward_varlen(query, key, value, cu_seqlens, horizon)[0]
    _refuse_training_capture("rosa_soft_varlen")
    seed = make_dropout_seed(query, dropout_p, True)
    return _HardForwardSoftVjpVarlenFunction.apply(
        query, key, value, cu_seqlens, seed, horizon, float(scale), float(dropout_p),
        float(mismatch_scale),
    )
