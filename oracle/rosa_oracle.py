"""Dense PyTorch restatement of the reference RosaSoft equations (TEST ORACLE).

This file is test infrastructure.  It is imported only by ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``; the
shipped operator never routes through it.

It restates, equation by equation, what the reference computes in
``rosa_soft/soft_reference.py`` (all line numbers below refer to that file
unless another file is named):

* sign symbols ``z(x) = +1 if x > 0 else -1`` with the softsign Jacobian
  ``1 / (1 + |x|)^2`` (``:87-105``);
* exact suffix lengths ``L(t, a)`` and latest-longest route selection with the
  "length zero never wins" rule (``:116-132``, ``:197-231``, ``:295-333``);
* local match gates ``exp(-ms * mismatching_bits / D)`` (``:135-164``);
* raw suffix evidence ``S(t, a) = sum_l prod_{r<l} gate(t-r, a-r)`` with at
  most ``min(W, a)`` terms (``:167-186``);
* the concave transform ``U(S) = (sqrt(2)+1)(sqrt(1+S) - 1)`` (``:189-194``);
* candidate-normalised logits: null ``0.5 * scale``, route ``scale * U - log t``
  and the row softmax (``:234-271``);
* the counter-hash dropout mask (``:362-447``), with the batch coordinate
  offset used by the packed layout (``:683-698``);
* the value carrier ``y(t) = sum_a d p z(v_a)`` whose autograd VJP is *the*
  surrogate gradient (``:336-359``, ``:479-556``).

Differences from the reference that are deliberate and do not change results:
the dropout seed is an explicit integer argument (the reference draws it from
the device generator), a ``head_offset`` lets one (batch, head-group) slice of
a large problem be checked alone, the exact suffix lengths come from an
integer run-length recurrence instead of float products, and the selected
route indices are returned (the reference exposes them only through
``rosa_soft/testing.py:50-117``).

Pinned by ``tests/test_oracle_known_answers.py`` against the known answers
held by the reference's own tests and against brute force; the keep-mask bit
pattern and the end-to-end gradients are additionally pinned by the vectors in
``tests/golden/``.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import numpy as np
import torch
from torch import Tensor

SQRT_UTILITY_SCALE = math.sqrt(2.0) + 1.0
NULL_ROUTE_SCORE = 0.5

_U32 = np.uint64(0xFFFFFFFF)
_MIX_A = np.uint64(0x7FEB352D)
_MIX_B = np.uint64(0x846CA68B)
# Salts of (batch, head, query position, route) in that order.
_SALT_BATCH = 0xA511E9B3
_SALT_HEAD = 0x63D83595
_SALT_ROW = 0xB5297A4D
_SALT_ROUTE = 0x68E31DA4
_SALT_SEED_HIGH = 0x9E3779B9


# --------------------------------------------------------------------------
# symbols
# --------------------------------------------------------------------------

def hard_sign(x: Tensor) -> Tensor:
    """``+1`` where ``x > 0`` else ``-1`` (zeros, NaN and ``-inf`` map to -1)."""

    one = torch.ones((), dtype=x.dtype, device=x.device)
    return torch.where(x > 0, one, -one)


class _SignWithSoftsignJacobian(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits: Tensor) -> Tensor:
        ctx.save_for_backward(logits)
        return hard_sign(logits)

    @staticmethod
    def backward(ctx, upstream: Tensor) -> Tensor:
        (logits,) = ctx.saved_tensors
        return upstream / (1.0 + logits.abs()).square()


def sign_ste(x: Tensor) -> Tensor:
    return _SignWithSoftsignJacobian.apply(x)


def pack_symbols(x: Tensor) -> Tensor:
    """Pack the sign bits of the last axis (width 1..32) into int64 words.

    Bit ``i`` of the word is ``x[..., i] > 0``; this is the layout of the
    reference's packed symbol tensors (``rosa_soft_kernels.cu:202-241``).
    """

    width = x.size(-1)
    weights = (1 << torch.arange(width, dtype=torch.int64, device=x.device))
    return ((x > 0).to(torch.int64) * weights).sum(dim=-1)


# --------------------------------------------------------------------------
# hard forward
# --------------------------------------------------------------------------

def exact_suffix_lengths(query: Tensor, key: Tensor, max_suffix_length: int) -> Tensor:
    """``L[b, h, t, a]`` for routes ``1 <= a <= t``; zero elsewhere.

    ``L(t, a)`` is the largest ``l <= min(W, a)`` with ``q[t-r] == k[a-1-r]``
    for every ``r < l``, evaluated by the run-length recurrence
    ``L(t, a) = eq(t, a) * min(L(t-1, a-1) + 1, W)``.
    """

    q_words = pack_symbols(query).permute(0, 2, 1)  # [B, H, T]
    k_words = pack_symbols(key).permute(0, 2, 1)
    batch, heads, seq_len = q_words.shape
    lengths = torch.zeros(batch, heads, seq_len, seq_len, dtype=torch.int64)
    if seq_len < 2:
        return lengths
    # eq[t, a] for a >= 1 compares q[t] with k[a - 1]
    equal = q_words.unsqueeze(-1) == k_words[..., :-1].unsqueeze(-2)  # [B,H,T,T-1]
    route = torch.arange(1, seq_len)
    for t in range(1, seq_len):
        causal = route <= t
        previous = lengths[:, :, t - 1, :-1]  # L(t-1, a-1) for a = 1..T-1
        run = torch.clamp(previous + 1, max=int(max_suffix_length))
        lengths[:, :, t, 1:] = torch.where(
            equal[:, :, t] & causal, run, torch.zeros_like(run)
        )
    return lengths


def select_routes(lengths: Tensor) -> Tensor:
    """Latest-longest route per row; 0 (null) when no route matched at all."""

    seq_len = lengths.size(-1)
    route = torch.arange(seq_len, dtype=torch.int64)
    # lexicographic (length, route) maximum; route 0 has length 0
    score = lengths * seq_len + route
    best = score.argmax(dim=-1)
    best_length = lengths.gather(-1, best.unsqueeze(-1)).squeeze(-1)
    return torch.where(best_length > 0, best, torch.zeros_like(best))


def hard_forward(
    query: Tensor, key: Tensor, value: Tensor, max_suffix_length: int
) -> Tuple[Tensor, Tensor, Tensor]:
    """Return ``(output [B,T,H,Dv], routes [B,H,T], lengths [B,H,T,T])``."""

    lengths = exact_suffix_lengths(query, key, max_suffix_length)
    routes = select_routes(lengths)
    heads = query.size(2)
    group = heads // value.size(2)
    signs = hard_sign(value.to(torch.float32))  # [B, T, Hv, Dv]
    signs = signs.repeat_interleave(group, dim=2).permute(0, 2, 1, 3)  # [B,H,T,Dv]
    picked = signs.gather(
        2, routes.unsqueeze(-1).expand(-1, -1, -1, signs.size(-1))
    )
    picked = torch.where(
        (routes > 0).unsqueeze(-1), picked, torch.zeros_like(picked)
    )
    return picked.permute(0, 2, 1, 3).to(value.dtype), routes, lengths


# --------------------------------------------------------------------------
# dropout hash
# --------------------------------------------------------------------------

def _avalanche(state: np.ndarray) -> np.ndarray:
    state = state & _U32
    state ^= state >> np.uint64(16)
    state = (state * _MIX_A) & _U32
    state ^= state >> np.uint64(15)
    state = (state * _MIX_B) & _U32
    state ^= state >> np.uint64(16)
    return state


def dropout_uniforms(
    seed: int,
    batch_ids: Sequence[int],
    head_ids: Sequence[int],
    rows: int,
    routes: int,
) -> np.ndarray:
    """24-bit uniforms ``u[b, h, t, a]`` of the counter hash, as float32.

    The hash chains route, row, head and batch (innermost first), then the low
    and high seed words; ``u = (state >> 8) * 2^-24``.
    """

    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    a = np.arange(routes, dtype=np.uint64).reshape(1, 1, 1, routes)
    t = np.arange(rows, dtype=np.uint64).reshape(1, 1, rows, 1)
    h = np.asarray(list(head_ids), dtype=np.uint64).reshape(1, -1, 1, 1)
    b = np.asarray(list(batch_ids), dtype=np.uint64).reshape(-1, 1, 1, 1)
    state = _avalanche(a ^ np.uint64(_SALT_ROUTE))
    state = _avalanche(state ^ t ^ np.uint64(_SALT_ROW))
    state = _avalanche(state ^ h ^ np.uint64(_SALT_HEAD))
    state = _avalanche(state ^ b ^ np.uint64(_SALT_BATCH))
    state = _avalanche(state ^ np.uint64(seed & 0xFFFFFFFF))
    state = _avalanche(state ^ np.uint64(seed >> 32) ^ np.uint64(_SALT_SEED_HIGH))
    return (state >> np.uint64(8)).astype(np.float32) * np.float32(2.0**-24)


def dropout_keep_mask(
    seed: int,
    dropout_p: float,
    batch_ids: Sequence[int],
    head_ids: Sequence[int],
    rows: int,
    routes: int,
) -> np.ndarray:
    """Boolean keep mask: keep iff ``u >= float32(dropout_p)``."""

    uniforms = dropout_uniforms(seed, batch_ids, head_ids, rows, routes)
    return uniforms >= np.float32(dropout_p)


# --------------------------------------------------------------------------
# surrogate (dense, differentiable)
# --------------------------------------------------------------------------

def local_match_gates(query: Tensor, key: Tensor, mismatch_scale: float) -> Tensor:
    """``g[b, h, t, a]``: gate of query ``t`` against key ``a-1``; 0 off-support."""

    zq = sign_ste(query.permute(0, 2, 1, 3))  # [B,H,T,D]
    zk = sign_ste(key.permute(0, 2, 1, 3))
    seq_len = zq.size(2)
    agreement = torch.einsum("bhtd,bhsd->bhts", zq, zk[:, :, : seq_len - 1])
    mismatch_rate = 0.5 * (1.0 - agreement / zq.size(-1))
    gates = torch.exp(-float(mismatch_scale) * mismatch_rate)  # [B,H,T,T-1]
    t = torch.arange(seq_len).view(seq_len, 1)
    a = torch.arange(1, seq_len).view(1, seq_len - 1)
    gates = gates * (a <= t).to(gates.dtype)
    first_column = gates.new_zeros(*gates.shape[:-1], 1)
    return torch.cat((first_column, gates), dim=-1)


def suffix_evidence(gates: Tensor, max_suffix_length: int) -> Tensor:
    """``S = sum_{l=1..W} P_l`` with ``P_l(t, a) = g(t, a) P_{l-1}(t-1, a-1)``."""

    seq_len = gates.size(-1)
    total = gates
    product = gates
    for length in range(2, min(int(max_suffix_length), seq_len) + 1):
        shifted = torch.zeros_like(gates)
        shifted[..., 1:, 1:] = product[..., :-1, :-1]
        product = gates * shifted
        total = total + product
    return total


def suffix_utility(evidence: Tensor) -> Tensor:
    return SQRT_UTILITY_SCALE * (torch.sqrt(1.0 + evidence) - 1.0)


def route_probabilities(evidence: Tensor, scale: float) -> Tensor:
    """Row softmax over ``{null} + {1..t}`` with the ``-log t`` correction."""

    seq_len = evidence.size(-1)
    t = torch.arange(seq_len).view(seq_len, 1)
    a = torch.arange(seq_len).view(1, seq_len)
    candidates = (a >= 1) & (a <= t)
    count = t.clamp_min(1).to(evidence.dtype)
    logits = suffix_utility(evidence) * float(scale) - torch.log(count)
    null_logit = torch.full_like(logits, NULL_ROUTE_SCORE * float(scale))
    logits = torch.where(a == 0, null_logit, logits)
    logits = logits.masked_fill(~(candidates | (a == 0)), -math.inf)
    return torch.softmax(logits - logits.amax(dim=-1, keepdim=True), dim=-1)


@dataclass
class SurrogateInspection:
    lengths: Tensor
    routes: Tensor
    evidence: Tensor
    probabilities: Tensor
    keep: Optional[Tensor]


def _carrier(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    max_suffix_length: int,
    scale: float,
    dropout_p: float,
    mismatch_scale: float,
    seed: Optional[int],
    batch_ids: Sequence[int],
    head_ids: Sequence[int],
):
    heads = query.size(2)
    seq_len = query.size(1)
    gates = local_match_gates(query, key, mismatch_scale)
    evidence = suffix_evidence(gates, max_suffix_length)
    probabilities = route_probabilities(evidence, scale)
    weights = probabilities
    keep = None
    if float(dropout_p) != 0.0:
        if seed is None:
            raise ValueError("a dropout seed is required when dropout_p > 0")
        keep_np = dropout_keep_mask(
            seed, dropout_p, batch_ids, head_ids, seq_len, seq_len
        )
        keep = torch.from_numpy(keep_np)
        weights = weights * keep.to(weights.dtype) / (1.0 - float(dropout_p))
    group = heads // value.size(2)
    zv = sign_ste(value).repeat_interleave(group, dim=2).permute(0, 2, 1, 3)
    not_null = (torch.arange(seq_len) != 0).view(1, 1, seq_len, 1)
    zv = torch.where(not_null, zv, torch.zeros_like(zv))
    carrier = torch.einsum("bhta,bhad->bhtd", weights, zv).permute(0, 2, 1, 3)
    return carrier, evidence, probabilities, keep


def compute_dtype_for(dtype: torch.dtype) -> torch.dtype:
    if dtype in (torch.float16, torch.bfloat16):
        return torch.float32
    if dtype in (torch.float32, torch.float64):
        return dtype
    raise ValueError(
        "rosa_soft_reference supports float16, bfloat16, float32, and float64"
    )


def surrogate_vjp(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    grad_output: Tensor,
    *,
    max_suffix_length: int,
    scale: float = 1.0,
    dropout_p: float = 0.0,
    mismatch_scale: float = 3.0,
    seed: Optional[int] = None,
    batch_ids: Optional[Sequence[int]] = None,
    head_ids: Optional[Sequence[int]] = None,
    compute_dtype: Optional[torch.dtype] = None,
    needs: Tuple[bool, bool, bool] = (True, True, True),
) -> Tuple[Optional[Tensor], Optional[Tensor], Optional[Tensor]]:
    """Autograd VJP of the carrier w.r.t. ``(query, key, value)``.

    ``max_suffix_length`` must already be clamped to the sequence length.
    Gradients come back in ``compute_dtype`` (default: float32 for half
    inputs, else the input dtype).  ``batch_ids`` / ``head_ids`` are the
    dropout coordinates of the slices present (default ``range``).
    """

    work = compute_dtype or compute_dtype_for(query.dtype)
    batch_ids = list(range(query.size(0))) if batch_ids is None else list(batch_ids)
    head_ids = list(range(query.size(2))) if head_ids is None else list(head_ids)
    leaves = [
        tensor.detach().to(work).requires_grad_(need)
        for tensor, need in zip((query, key, value), needs)
    ]
    with torch.enable_grad():
        carrier, _, _, _ = _carrier(
            leaves[0], leaves[1], leaves[2], max_suffix_length, scale,
            dropout_p, mismatch_scale, seed, batch_ids, head_ids,
        )
        wanted = [leaf for leaf, need in zip(leaves, needs) if need]
        grads = torch.autograd.grad(carrier, wanted, grad_output.to(work))
    result = [None, None, None]
    iterator = iter(grads)
    for index, need in enumerate(needs):
        if need:
            result[index] = next(iterator)
    return tuple(result)


@torch.no_grad()
def inspect(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    *,
    max_suffix_length: int,
    scale: float = 1.0,
    dropout_p: float = 0.0,
    mismatch_scale: float = 3.0,
    seed: Optional[int] = None,
    compute_dtype: Optional[torch.dtype] = None,
) -> Tuple[Tensor, SurrogateInspection]:
    work = compute_dtype or compute_dtype_for(query.dtype)
    horizon = min(int(max_suffix_length), query.size(1))
    output, routes, lengths = hard_forward(query, key, value, horizon)
    _, evidence, probabilities, keep = _carrier(
        query.to(work), key.to(work), value.to(work), horizon, scale,
        dropout_p, mismatch_scale, seed,
        list(range(query.size(0))), list(range(query.size(2))),
    )
    return output, SurrogateInspection(lengths, routes, evidence, probabilities, keep)


# --------------------------------------------------------------------------
# operator-shaped wrappers (hard forward, surrogate backward)
# --------------------------------------------------------------------------

class _HardForwardSurrogateBackward(torch.autograd.Function):
    @staticmethod
    def forward(ctx, query, key, value, controls):
        ctx.controls = controls
        ctx.save_for_backward(query, key, value)
        output, _, _ = hard_forward(query, key, value, controls["max_suffix_length"])
        return output.to(query.dtype)

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        query, key, value = ctx.saved_tensors
        controls = ctx.controls
        grads = surrogate_vjp(
            query, key, value, grad_output,
            needs=tuple(ctx.needs_input_grad[:3]),
            **controls,
        )
        cast = tuple(
            None if grad is None else grad.to(tensor.dtype)
            for grad, tensor in zip(grads, (query, key, value))
        )
        return (*cast, None)


def rosa_soft_oracle(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    *,
    max_suffix_length: int = 32,
    scale: float = 1.0,
    dropout_p: float = 0.0,
    mismatch_scale: float = 3.0,
    seed: Optional[int] = None,
    batch_ids: Optional[Sequence[int]] = None,
    head_ids: Optional[Sequence[int]] = None,
    compute_dtype: Optional[torch.dtype] = None,
) -> Tensor:
    """Dense operator with the reference's semantics and an explicit seed."""

    compute_dtype_for(query.dtype)
    horizon = min(int(max_suffix_length), query.size(1))
    needs_backward = torch.is_grad_enabled() and any(
        tensor.requires_grad for tensor in (query, key, value)
    )
    if not needs_backward:
        return hard_forward(query, key, value, horizon)[0].to(query.dtype)
    controls = dict(
        max_suffix_length=horizon, scale=float(scale), dropout_p=float(dropout_p),
        mismatch_scale=float(mismatch_scale), seed=seed, batch_ids=batch_ids,
        head_ids=head_ids, compute_dtype=compute_dtype,
    )
    return _HardForwardSurrogateBackward.apply(query, key, value, controls)


def rosa_soft_varlen_oracle(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    cu_seqlens: Sequence[int],
    *,
    max_suffix_length: int = 32,
    scale: float = 1.0,
    dropout_p: float = 0.0,
    mismatch_scale: float = 3.0,
    seed: Optional[int] = None,
    compute_dtype: Optional[torch.dtype] = None,
) -> Tensor:
    """Packed layout: each segment is an independent dense call.

    The horizon is clamped to the packed token count first (as the reference
    does, ``soft_contract.py:202-208``) and then to each segment; empty
    segments produce nothing but still consume a sequence index, which is the
    dropout batch coordinate.
    """

    offsets = [int(v) for v in cu_seqlens]
    horizon = min(int(max_suffix_length), query.size(0))
    pieces = []
    for sequence, (start, end) in enumerate(zip(offsets[:-1], offsets[1:])):
        if start == end:
            continue
        pieces.append(
            rosa_soft_oracle(
                query[start:end].unsqueeze(0),
                key[start:end].unsqueeze(0),
                value[start:end].unsqueeze(0),
                max_suffix_length=horizon,
                scale=scale,
                dropout_p=dropout_p,
                mismatch_scale=mismatch_scale,
                seed=seed,
                batch_ids=[sequence],
                compute_dtype=compute_dtype,
            ).squeeze(0)
        )
    return torch.cat(pieces, dim=0)
