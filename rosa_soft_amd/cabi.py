"""ctypes binding of ``librosa_soft_hip.so`` (declared in ``include/rosa_soft_hip.h``).

This is the thinnest way to reach the kernels: tensors are passed as raw
device pointers and the current torch stream as ``hipStream_t``.  The operator
itself goes through the dispatcher extension (``rosa_soft_amd._C``); the parity
tests, ``bench.py`` and the route-index side channel use this module.  Loading
fails loudly when the library has not been built: there is no CPU fallback.
"""

from __future__ import annotations

import contextlib
import ctypes
import os
from typing import Optional, Sequence, Tuple

import torch
from torch import Tensor

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "librosa_soft_hip.so")

GRAD_QUERY, GRAD_KEY, GRAD_VALUE = 1, 2, 4

EXPORTED_SYMBOLS = (
    "rosa_hip_version",
    "rosa_hip_target",
    "rosa_hip_last_error",
    "rosa_hip_forward_workspace_bytes",
    "rosa_hip_vjp_workspace_bytes",
    "rosa_hip_set_record_budget",
    "rosa_hip_set_gradient_block_waves",
    "rosa_hip_set_gradient_piece_rows",
    "rosa_hip_set_forward_index",
    "rosa_hip_measure_atomic_rate",
    "rosa_hip_gradient_block_plan",
    "rosa_hip_gradient_piece_plan",
    "rosa_hip_hard_forward",
    "rosa_hip_hard_routes",
    "rosa_hip_hard_forward_bits",
    "rosa_hip_hard_forward_words",
    "rosa_hip_project_routed_bits",
    "rosa_hip_hard_forward_static",
    "rosa_hip_pack_symbols",
    "rosa_hip_surrogate_vjp",
    "rosa_hip_router_update",
    "rosa_hip_router_workspace_bytes",
    "rosa_hip_read_offset_error",
    "rosa_hip_stage_timing",
    "rosa_hip_stage_count",
    "rosa_hip_stage_name",
    "rosa_hip_stage_times",
    "rosa_hip_stage_totals",
)

_DTYPE_CODES = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


class RosaProblem(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int),
        ("B", ctypes.c_int),
        ("T", ctypes.c_int),
        ("N", ctypes.c_int),
        ("S", ctypes.c_int),
        ("H", ctypes.c_int),
        ("D", ctypes.c_int),
        ("Hv", ctypes.c_int),
        ("Dv", ctypes.c_int),
        ("W", ctypes.c_int),
        ("cu_seqlens", ctypes.c_void_p),
    ]


class RosaRouterUpdate(ctypes.Structure):
    """``rosa_router_update`` of ``include/rosa_soft_hip.h``."""

    _fields_ = [
        ("S", ctypes.c_int32),
        ("H", ctypes.c_int32),
        ("Hp", ctypes.c_int32),
        ("W", ctypes.c_int32),
        ("qk_bits", ctypes.c_int32),
        ("payload_bits", ctypes.c_int32),
        ("capacity", ctypes.c_int32),
        ("tokens", ctypes.c_int32),
        ("longest_chunk", ctypes.c_int32),
        ("uniform_chunk", ctypes.c_int32),
        ("chunk_offsets", ctypes.c_void_p),
        ("history_lengths", ctypes.c_void_p),
        ("query_history", ctypes.c_void_p),
        ("key_history", ctypes.c_void_p),
        ("payload_history", ctypes.c_void_p),
        ("query", ctypes.c_void_p),
        ("key", ctypes.c_void_p),
        ("payload", ctypes.c_void_p),
        ("output", ctypes.c_void_p),
        ("matched_key_end", ctypes.c_void_p),
        ("longest_total", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("history_lengths_out", ctypes.c_void_p),
    ]


_library: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Load the shared library and declare every prototype of the header."""

    global _library
    if _library is not None:
        return _library
    if not os.path.exists(LIBRARY_PATH):
        raise RuntimeError(
            f"{LIBRARY_PATH} is missing: build it with "
            "`python -c 'import __graft_entry__ as g; g.build()'` or `python setup.py build_ext --inplace`"
        )
    library = ctypes.CDLL(LIBRARY_PATH)
    problem_p = ctypes.POINTER(RosaProblem)
    vp = ctypes.c_void_p
    library.rosa_hip_version.restype = ctypes.c_int
    library.rosa_hip_target.restype = ctypes.c_char_p
    library.rosa_hip_last_error.restype = ctypes.c_char_p
    library.rosa_hip_forward_workspace_bytes.restype = ctypes.c_size_t
    library.rosa_hip_forward_workspace_bytes.argtypes = [problem_p]
    library.rosa_hip_vjp_workspace_bytes.restype = ctypes.c_size_t
    library.rosa_hip_vjp_workspace_bytes.argtypes = [
        problem_p, ctypes.c_int, ctypes.c_float, ctypes.c_int,
    ]
    library.rosa_hip_set_gradient_block_waves.restype = None
    library.rosa_hip_set_gradient_block_waves.argtypes = [ctypes.c_int]
    library.rosa_hip_set_gradient_piece_rows.restype = None
    library.rosa_hip_set_gradient_piece_rows.argtypes = [ctypes.c_int]
    library.rosa_hip_set_forward_index.restype = None
    library.rosa_hip_set_forward_index.argtypes = [ctypes.c_int]
    library.rosa_hip_gradient_block_plan.restype = ctypes.c_int
    library.rosa_hip_gradient_block_plan.argtypes = [
        problem_p, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
        ctypes.POINTER(ctypes.c_size_t),
    ]
    library.rosa_hip_gradient_piece_plan.restype = ctypes.c_int
    library.rosa_hip_gradient_piece_plan.argtypes = [
        problem_p, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
    ]
    library.rosa_hip_measure_atomic_rate.restype = ctypes.c_int
    library.rosa_hip_measure_atomic_rate.argtypes = [
        vp, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double), vp,
    ]
    library.rosa_hip_set_record_budget.restype = None
    library.rosa_hip_set_record_budget.argtypes = [ctypes.c_size_t]
    library.rosa_hip_hard_forward.restype = ctypes.c_int
    library.rosa_hip_hard_forward.argtypes = [
        problem_p, vp, vp, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, vp,
    ]
    library.rosa_hip_hard_routes.restype = ctypes.c_int
    library.rosa_hip_hard_routes.argtypes = [
        problem_p, vp, vp, vp, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, vp,
    ]
    library.rosa_hip_hard_forward_bits.restype = ctypes.c_int
    library.rosa_hip_hard_forward_bits.argtypes = [
        problem_p, vp, vp, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, vp,
    ]
    library.rosa_hip_hard_forward_words.restype = ctypes.c_int
    library.rosa_hip_hard_forward_words.argtypes = [
        problem_p, vp, vp, vp, vp, vp, vp, vp, vp, ctypes.c_size_t, vp,
    ]
    library.rosa_hip_project_routed_bits.restype = ctypes.c_int
    library.rosa_hip_project_routed_bits.argtypes = [
        vp, vp, ctypes.c_int64, ctypes.c_int, ctypes.c_int, vp, ctypes.c_int, vp, vp, vp,
    ]
    library.rosa_hip_hard_forward_static.restype = ctypes.c_int
    library.rosa_hip_hard_forward_static.argtypes = [problem_p, vp, vp, vp, vp, vp, vp, vp, vp]
    library.rosa_hip_pack_symbols.restype = ctypes.c_int
    library.rosa_hip_pack_symbols.argtypes = [
        ctypes.c_int, vp, ctypes.c_int64, ctypes.c_int, vp, ctypes.c_int, vp,
    ]
    library.rosa_hip_router_workspace_bytes.restype = ctypes.c_size_t
    library.rosa_hip_router_workspace_bytes.argtypes = [ctypes.POINTER(RosaRouterUpdate)]
    library.rosa_hip_router_update.restype = ctypes.c_int
    library.rosa_hip_router_update.argtypes = [ctypes.POINTER(RosaRouterUpdate), vp]
    library.rosa_hip_surrogate_vjp.restype = ctypes.c_int
    library.rosa_hip_surrogate_vjp.argtypes = [
        problem_p, vp, vp, vp, vp, vp, vp, vp,
        ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int,
        vp, vp, vp, vp, ctypes.c_size_t, vp,
    ]
    library.rosa_hip_read_offset_error.restype = ctypes.c_int
    library.rosa_hip_read_offset_error.argtypes = [vp, vp]
    library.rosa_hip_stage_timing.restype = ctypes.c_int
    library.rosa_hip_stage_timing.argtypes = [ctypes.c_int]
    library.rosa_hip_stage_count.restype = ctypes.c_int
    library.rosa_hip_stage_name.restype = ctypes.c_char_p
    library.rosa_hip_stage_name.argtypes = [ctypes.c_int]
    library.rosa_hip_stage_times.restype = ctypes.c_int
    library.rosa_hip_stage_times.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_int]
    library.rosa_hip_stage_totals.restype = ctypes.c_int
    library.rosa_hip_stage_totals.argtypes = [
        ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_int), ctypes.c_int,
    ]
    _library = library
    return library


def _check(status: int, what: str) -> None:
    if status != 0:
        message = load().rosa_hip_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed with status {status}: {message}")


def make_problem(
    query: Tensor, value: Tensor, max_suffix_length: int, cu_seqlens: Optional[Tensor] = None
) -> RosaProblem:
    if query.dtype not in _DTYPE_CODES:
        raise ValueError("rosa_soft supports float32, float16, and bfloat16")
    problem = RosaProblem()
    problem.dtype = _DTYPE_CODES[query.dtype]
    if cu_seqlens is None:
        batch, seq_len, heads, width = query.shape
        problem.B, problem.T = batch, seq_len
        problem.N, problem.S = batch * seq_len, 0
        problem.Hv, problem.Dv = value.shape[2], value.shape[3]
        problem.cu_seqlens = None
        bound = seq_len
    else:
        tokens, heads, width = query.shape
        problem.B, problem.T = 0, 0
        problem.N, problem.S = tokens, cu_seqlens.numel() - 1
        problem.Hv, problem.Dv = value.shape[1], value.shape[2]
        problem.cu_seqlens = cu_seqlens.data_ptr()
        bound = tokens
    problem.H, problem.D = heads, width
    problem.W = min(int(max_suffix_length), bound)
    return problem


def _stream(tensor: Tensor) -> int:
    return torch.cuda.current_stream(tensor.device).cuda_stream


def _ptr(tensor: Optional[Tensor]):
    return None if tensor is None else tensor.data_ptr()


def hard_forward(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    max_suffix_length: int,
    cu_seqlens: Optional[Tensor] = None,
    want_routes: bool = True,
) -> Tuple[Tensor, Tensor, Tensor, Optional[Tensor]]:
    """Run the hard forward; returns ``(output, packed_q, packed_k, routes)``.

    Inputs must be contiguous device tensors.  ``routes`` (int32, in the packed
    symbol layout, sequence-local, 0 = null) is the index side channel.
    """

    library = load()
    assert query.is_cuda and query.is_contiguous() and key.is_contiguous() and value.is_contiguous()
    problem = make_problem(query, value, max_suffix_length, cu_seqlens)
    if cu_seqlens is None:
        word_shape = (problem.B, problem.H, problem.T)
        out_shape = (problem.B, problem.T, problem.H, problem.Dv)
    else:
        word_shape = (problem.H, problem.N)
        out_shape = (problem.N, problem.H, problem.Dv)
    with torch.cuda.device(query.device):
        output = torch.empty(out_shape, dtype=query.dtype, device=query.device)
        packed_q = torch.empty(word_shape, dtype=torch.int32, device=query.device)
        packed_k = torch.empty(word_shape, dtype=torch.int32, device=query.device)
        routes = torch.empty(word_shape, dtype=torch.int32, device=query.device) if want_routes else None
        size = library.rosa_hip_forward_workspace_bytes(ctypes.byref(problem))
        workspace = torch.empty(max(size, 256), dtype=torch.uint8, device=query.device)
        status = library.rosa_hip_hard_forward(
            ctypes.byref(problem), _ptr(query), _ptr(key), _ptr(value), _ptr(output),
            _ptr(packed_q), _ptr(packed_k), _ptr(routes), _ptr(workspace), workspace.numel(),
            _stream(query),
        )
    _check(status, "rosa_hip_hard_forward")
    return output, packed_q, packed_k, routes


def hard_forward_static(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    max_suffix_length: int,
    cu_seqlens: Optional[Tensor] = None,
    outputs: Optional[Tuple[Tensor, Tensor, Tensor, Tensor]] = None,
) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """``hard_forward`` through the entry point that allocates nothing.

    The library call takes no workspace (it uses the scratch array of its device image).
    ``outputs`` = ``(output, packed_q, packed_k, routes)`` are written in place when given,
    which is what a caller that cannot allocate does; otherwise they are created here.
    """

    library = load()
    assert query.is_cuda and query.is_contiguous() and key.is_contiguous() and value.is_contiguous()
    problem = make_problem(query, value, max_suffix_length, cu_seqlens)
    if cu_seqlens is None:
        word_shape = (problem.B, problem.H, problem.T)
        out_shape = (problem.B, problem.T, problem.H, problem.Dv)
    else:
        word_shape = (problem.H, problem.N)
        out_shape = (problem.N, problem.H, problem.Dv)
    with torch.cuda.device(query.device):
        if outputs is None:
            outputs = (
                torch.empty(out_shape, dtype=query.dtype, device=query.device),
                torch.empty(word_shape, dtype=torch.int32, device=query.device),
                torch.empty(word_shape, dtype=torch.int32, device=query.device),
                torch.empty(word_shape, dtype=torch.int32, device=query.device),
            )
        output, packed_q, packed_k, routes = outputs
        assert output.shape == out_shape and output.dtype == query.dtype and output.is_contiguous()
        assert all(w.shape == word_shape and w.dtype == torch.int32 and w.is_contiguous()
                   for w in (packed_q, packed_k, routes))
        status = library.rosa_hip_hard_forward_static(
            ctypes.byref(problem), _ptr(query), _ptr(key), _ptr(value), _ptr(output),
            _ptr(packed_q), _ptr(packed_k), _ptr(routes), _stream(query),
        )
    _check(status, "rosa_hip_hard_forward_static")
    return output, packed_q, packed_k, routes


def hard_forward_bits(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    max_suffix_length: int,
    cu_seqlens: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """Hard forward whose output leaves as bits: ``(sign_words, routed)``.

    ``sign_words`` is int32 ``[..., H, ceil(Dv/32)]`` (bit ``d`` of word ``w`` set iff output
    element ``32 w + d`` is +1) and ``routed`` uint8 ``[..., H]`` (1 where a route was
    selected); the leading axes are those of the inputs.  ``expand_output_bits`` turns them
    back into the ternary output.
    """

    library = load()
    assert query.is_cuda and query.is_contiguous() and key.is_contiguous() and value.is_contiguous()
    problem = make_problem(query, value, max_suffix_length, cu_seqlens)
    words = (problem.Dv + 31) // 32
    if cu_seqlens is None:
        word_shape = (problem.B, problem.H, problem.T)
        lead = (problem.B, problem.T, problem.H)
    else:
        word_shape = (problem.H, problem.N)
        lead = (problem.N, problem.H)
    with torch.cuda.device(query.device):
        sign_words = torch.empty((*lead, words), dtype=torch.int32, device=query.device)
        routed = torch.empty(lead, dtype=torch.uint8, device=query.device)
        packed_q = torch.empty(word_shape, dtype=torch.int32, device=query.device)
        packed_k = torch.empty(word_shape, dtype=torch.int32, device=query.device)
        size = library.rosa_hip_forward_workspace_bytes(ctypes.byref(problem))
        workspace = torch.empty(max(size, 256), dtype=torch.uint8, device=query.device)
        status = library.rosa_hip_hard_forward_bits(
            ctypes.byref(problem), _ptr(query), _ptr(key), _ptr(value), _ptr(sign_words),
            _ptr(routed), _ptr(packed_q), _ptr(packed_k), _ptr(workspace), workspace.numel(),
            _stream(query),
        )
    _check(status, "rosa_hip_hard_forward_bits")
    return sign_words, routed


def hard_forward_words(
    packed_q: Tensor,
    packed_k: Tensor,
    value: Tensor,
    max_suffix_length: int,
    symbol_bits: int,
    cu_seqlens: Optional[Tensor] = None,
    as_bits: bool = False,
):
    """Hard forward from symbol words a producer has already packed (no packing pass).

    ``packed_q`` / ``packed_k`` are int32 ``[B, H, T]`` (``[H, N]`` packed), bit ``i`` set iff
    logit ``i`` is positive; ``symbol_bits`` is their width ``D``.  Returns ``(output, routes)``
    or, with ``as_bits``, ``(sign_words, routed, routes)`` in the layout of
    ``hard_forward_bits``.
    """

    library = load()
    assert packed_q.is_cuda and packed_q.is_contiguous() and packed_k.is_contiguous()
    assert packed_q.dtype == torch.int32 and packed_k.dtype == torch.int32 and value.is_contiguous()
    heads = packed_q.shape[-2]
    # only the shapes of a query tensor are needed to describe the problem
    if cu_seqlens is None:
        shape = (packed_q.shape[0], packed_q.shape[2], heads, symbol_bits)
    else:
        shape = (packed_q.shape[1], heads, symbol_bits)
    query_like = torch.empty(shape, dtype=value.dtype, device="meta")
    problem = make_problem(query_like, value, max_suffix_length, cu_seqlens)
    lead = shape[:-1]
    with torch.cuda.device(value.device):
        routes = torch.empty(packed_q.shape, dtype=torch.int32, device=value.device)
        output = sign_words = routed = None
        if as_bits:
            words = (problem.Dv + 31) // 32
            sign_words = torch.empty((*lead, words), dtype=torch.int32, device=value.device)
            routed = torch.empty(lead, dtype=torch.uint8, device=value.device)
        else:
            output = torch.empty((*lead, problem.Dv), dtype=value.dtype, device=value.device)
        size = library.rosa_hip_forward_workspace_bytes(ctypes.byref(problem))
        workspace = torch.empty(max(size, 256), dtype=torch.uint8, device=value.device)
        status = library.rosa_hip_hard_forward_words(
            ctypes.byref(problem), _ptr(packed_q), _ptr(packed_k), _ptr(value), _ptr(output),
            _ptr(sign_words), _ptr(routed), _ptr(routes), _ptr(workspace), workspace.numel(),
            _stream(value),
        )
    _check(status, "rosa_hip_hard_forward_words")
    return (sign_words, routed, routes) if as_bits else (output, routes)


def project_routed_bits(sign_words: Tensor, routed: Tensor, value_dim: int, weight: Tensor,
                        residual: Optional[Tensor] = None) -> Tensor:
    """``residual + expand_output_bits(sign_words, routed).flatten(-2) @ weight.T`` in one kernel.

    ``weight`` is the bfloat16 ``[N, H * Dv]`` matrix of a linear layer; the result (and the
    optional ``residual``) is bfloat16 ``[..., N]`` over the leading axes of ``routed`` without
    its head axis.
    """

    library = load()
    assert sign_words.is_cuda and sign_words.is_contiguous() and routed.is_contiguous()
    assert weight.dtype == torch.bfloat16 and weight.is_contiguous() and weight.dim() == 2
    heads = routed.shape[-1]
    tokens = routed.numel() // heads
    width = weight.shape[0]
    assert weight.shape[1] == heads * value_dim
    lead = routed.shape[:-1]
    if residual is not None:
        assert residual.dtype == torch.bfloat16 and residual.is_contiguous()
        assert tuple(residual.shape) == (*lead, width)
    with torch.cuda.device(weight.device):
        out = torch.empty((*lead, width), dtype=torch.bfloat16, device=weight.device)
        status = library.rosa_hip_project_routed_bits(
            _ptr(sign_words), _ptr(routed), tokens, heads, value_dim, _ptr(weight), width,
            _ptr(residual), _ptr(out), _stream(weight),
        )
    _check(status, "rosa_hip_project_routed_bits")
    return out


def expand_output_bits(sign_words: Tensor, routed: Tensor, value_dim: int,
                       dtype: torch.dtype = torch.float32) -> Tensor:
    """Ternary output from the bit form of ``hard_forward_bits`` (what a consumer's prologue does)."""

    shifts = torch.arange(32, device=sign_words.device, dtype=torch.int32)
    bits = (sign_words.unsqueeze(-1) >> shifts) & 1          # [..., words, 32]
    bits = bits.reshape(*sign_words.shape[:-1], -1)[..., :value_dim]
    signs = bits.to(dtype) * 2 - 1
    return signs * (routed == 1).unsqueeze(-1).to(dtype)


def pack_symbols(logits: Tensor, symbol_dtype: torch.dtype = torch.uint8) -> Tensor:
    """Sign symbols of the last axis of a device tensor: bit ``i`` = ``logits[..., i] > 0``.

    ``symbol_dtype`` is ``torch.uint8`` (widths up to 8, the streaming router's symbols) or
    ``torch.int32`` (widths up to 32).  One launch; the result has the shape of ``logits``
    without its last axis.
    """

    library = load()
    if logits.dtype not in _DTYPE_CODES:
        raise ValueError("pack_symbols supports float32, float16, and bfloat16")
    if symbol_dtype not in (torch.uint8, torch.int32):
        raise ValueError("symbols are stored as uint8 or int32")
    assert logits.is_cuda
    logits = logits.contiguous()
    bits = logits.size(-1)
    rows = logits.numel() // max(bits, 1)
    with torch.cuda.device(logits.device):
        symbols = torch.empty(logits.shape[:-1], dtype=symbol_dtype, device=logits.device)
        status = library.rosa_hip_pack_symbols(
            _DTYPE_CODES[logits.dtype], _ptr(logits), rows, bits, _ptr(symbols),
            1 if symbol_dtype == torch.uint8 else 4, _stream(logits),
        )
    _check(status, "rosa_hip_pack_symbols")
    return symbols


def hard_routes(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    max_suffix_length: int,
    cu_seqlens: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Hard forward with its selection: ``(output, routes, lengths)``.

    ``routes`` and ``lengths`` are int32 in the layout of the inputs without the
    feature axis (``[B, T, H]`` dense, ``[N, H]`` packed): the selected route
    index local to its sequence (0 = null route) and the exact matched suffix
    length of that route (0 for the null route).
    """

    library = load()
    assert query.is_cuda and query.is_contiguous() and key.is_contiguous() and value.is_contiguous()
    problem = make_problem(query, value, max_suffix_length, cu_seqlens)
    if cu_seqlens is None:
        word_shape = (problem.B, problem.H, problem.T)
        out_shape = (problem.B, problem.T, problem.H, problem.Dv)
    else:
        word_shape = (problem.H, problem.N)
        out_shape = (problem.N, problem.H, problem.Dv)
    with torch.cuda.device(query.device):
        output = torch.empty(out_shape, dtype=query.dtype, device=query.device)
        words = [torch.empty(word_shape, dtype=torch.int32, device=query.device) for _ in range(4)]
        size = library.rosa_hip_forward_workspace_bytes(ctypes.byref(problem))
        workspace = torch.empty(max(size, 256), dtype=torch.uint8, device=query.device)
        status = library.rosa_hip_hard_routes(
            ctypes.byref(problem), _ptr(query), _ptr(key), _ptr(value), _ptr(output),
            _ptr(words[0]), _ptr(words[1]), _ptr(words[2]), _ptr(words[3]), _ptr(workspace),
            workspace.numel(), _stream(query),
        )
    _check(status, "rosa_hip_hard_routes")
    # head-major words -> the layout of the inputs
    if cu_seqlens is None:
        routes, lengths = (w.permute(0, 2, 1).contiguous() for w in words[2:])
    else:
        routes, lengths = (w.t().contiguous() for w in words[2:])
    return output, routes, lengths


def surrogate_vjp(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    grad_output: Tensor,
    packed_q: Tensor,
    packed_k: Tensor,
    dropout_seed: Optional[Tensor],
    max_suffix_length: int,
    scale: float,
    dropout_p: float,
    mismatch_scale: float,
    gradient_mask: int = 7,
    cu_seqlens: Optional[Tensor] = None,
    workspace: Optional[Tensor] = None,
) -> Tuple[Optional[Tensor], Optional[Tensor], Optional[Tensor]]:
    """Run the surrogate VJP; returns float32 ``(grad_q, grad_k, grad_v)``."""

    library = load()
    problem = make_problem(query, value, max_suffix_length, cu_seqlens)
    p32 = torch.tensor(float(dropout_p), dtype=torch.float32)
    inverse_keep = float(torch.tensor(1.0, dtype=torch.float32) / (1.0 - p32))
    with torch.cuda.device(query.device):
        grads = [
            torch.empty(t.shape, dtype=torch.float32, device=query.device)
            if gradient_mask & bit
            else None
            for bit, t in zip((1, 2, 4), (query, key, value))
        ]
        size = library.rosa_hip_vjp_workspace_bytes(
            ctypes.byref(problem), gradient_mask, float(scale), int(dropout_p > 0)
        )
        if workspace is None or workspace.numel() < size:
            workspace = torch.empty(max(size, 256), dtype=torch.uint8, device=query.device)
        status = library.rosa_hip_surrogate_vjp(
            ctypes.byref(problem), _ptr(query), _ptr(key), _ptr(value), _ptr(grad_output),
            _ptr(packed_q), _ptr(packed_k),
            _ptr(dropout_seed) if dropout_p > 0 else None,
            float(scale), float(p32), inverse_keep, float(mismatch_scale), int(gradient_mask),
            _ptr(grads[0]), _ptr(grads[1]), _ptr(grads[2]),
            _ptr(workspace), workspace.numel(), _stream(query),
        )
    _check(status, "rosa_hip_surrogate_vjp")
    return tuple(grads)


def vjp_workspace_bytes(query: Tensor, value: Tensor, max_suffix_length: int,
                        cu_seqlens: Optional[Tensor] = None, dropout: bool = False) -> int:
    problem = make_problem(query, value, max_suffix_length, cu_seqlens)
    return int(load().rosa_hip_vjp_workspace_bytes(ctypes.byref(problem), 7, 1.0, int(dropout)))


def router_update(update: RosaRouterUpdate, device: torch.device) -> Optional[Tensor]:
    """Enqueue one streaming-router update on the current stream of ``device``.

    ``update.longest_total`` must be set.  Returns the workspace the update uses (or ``None``):
    the launches are stream-ordered, so the caller keeps it alive until they have run.
    """

    workspace = None
    # (the device guard costs a decoding step several microseconds: only where it changes anything)
    guard = (torch.cuda.device(device) if torch.cuda.current_device() != device.index
             else contextlib.nullcontext())
    with guard:
        # (chunks of up to 8 tokens never use a workspace: decoding steps skip the query)
        size = (int(load().rosa_hip_router_workspace_bytes(ctypes.byref(update)))
                if update.longest_chunk > 8 else 0)
        if size > 0:
            workspace = torch.empty(size, dtype=torch.uint8, device=device)
            update.workspace = workspace.data_ptr()
            update.workspace_bytes = size
        status = load().rosa_hip_router_update(
            ctypes.byref(update), torch.cuda.current_stream(device).cuda_stream
        )
    _check(status, "rosa_hip_router_update")
    return workspace


def set_record_budget(limit_bytes: Optional[int]) -> None:
    """Bound the chunk records of the backward workspace (``None`` restores the default)."""

    load().rosa_hip_set_record_budget(ctypes.c_size_t(-1).value if limit_bytes is None
                                      else int(limit_bytes))


def set_gradient_block_waves(waves: Optional[int]) -> None:
    """Waves per block of the gradient kernel: 1, 2, or ``None`` for the library's choice."""

    load().rosa_hip_set_gradient_block_waves(0 if waves is None else int(waves))


def set_gradient_piece_rows(rows: Optional[int]) -> None:
    """Rows of a piece of a band in the gradient kernel: a number, -1 for never, or ``None``
    for the library's choice by shape."""

    load().rosa_hip_set_gradient_piece_rows(0 if rows is None else int(rows))


def set_forward_index(mode: Optional[str]) -> None:
    """How the hard forward finds its routes: ``None`` (the library's choice: an index of the
    keys where the shape suits it), ``"scan"`` (always the scan over all routes),
    ``"handed_back"`` (the index with every row block handed back to the scan) or ``"always"``
    (the index at every shape); the last two are for tests."""

    modes = {None: 0, "scan": 1, "handed_back": 2, "always": 3}
    load().rosa_hip_set_forward_index(modes[mode])


def gradient_block_plan(query: Tensor, value: Tensor, max_suffix_length: int,
                        cu_seqlens: Optional[Tensor] = None) -> dict:
    """Launch form of the gradient kernel for a problem: waves per block, row queue, LDS bytes,
    and the rows of a piece of a band (0: whole bands) with the work items per band."""

    problem = make_problem(query, value, max_suffix_length, cu_seqlens)
    waves, queue, lds = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_size_t(0)
    status = load().rosa_hip_gradient_block_plan(
        ctypes.byref(problem), ctypes.byref(waves), ctypes.byref(queue), ctypes.byref(lds))
    _check(status, "rosa_hip_gradient_block_plan")
    piece_rows, pieces = ctypes.c_int(0), ctypes.c_int(1)
    status = load().rosa_hip_gradient_piece_plan(
        ctypes.byref(problem), ctypes.byref(piece_rows), ctypes.byref(pieces))
    _check(status, "rosa_hip_gradient_piece_plan")
    return dict(waves=waves.value, row_queue=bool(queue.value), lds_bytes=lds.value,
                piece_rows=piece_rows.value, pieces=pieces.value)


def measure_atomic_rate(row_floats: int, columns: int = 16, device: str = "cuda:0") -> float:
    """Row segments per second of global float atomics in the gradient flush's pattern."""

    buffer = torch.zeros(1 << 26, dtype=torch.float32, device=device)  # 256 MiB
    rate = ctypes.c_double(0.0)
    status = load().rosa_hip_measure_atomic_rate(
        _ptr(buffer), buffer.numel() * 4, int(row_floats), int(columns), ctypes.byref(rate),
        _stream(buffer),
    )
    _check(status, "rosa_hip_measure_atomic_rate")
    return rate.value


def stage_timing(enable: bool) -> None:
    """Switch per-stage HIP event timing of the library on or off."""

    _check(load().rosa_hip_stage_timing(1 if enable else 0), "rosa_hip_stage_timing")


def stage_times() -> dict:
    """Elapsed milliseconds per stage of the last call (waits for its events)."""

    library = load()
    count = library.rosa_hip_stage_count()
    buffer = (ctypes.c_float * count)()
    _check(library.rosa_hip_stage_times(buffer, count), "rosa_hip_stage_times")
    return {
        library.rosa_hip_stage_name(i).decode(): float(buffer[i])
        for i in range(count)
        if buffer[i] >= 0.0
    }


def stage_totals() -> dict:
    """``{stage: (summed milliseconds, runs)}`` of the calls since timing was enabled or the
    totals were last read (waits for their events, then starts a new sum).  At most the last
    64 runs of a stage are summed; ``runs`` says how many were."""

    library = load()
    count = library.rosa_hip_stage_count()
    buffer = (ctypes.c_float * count)()
    runs = (ctypes.c_int * count)()
    _check(library.rosa_hip_stage_totals(buffer, runs, count), "rosa_hip_stage_totals")
    return {
        library.rosa_hip_stage_name(i).decode(): (float(buffer[i]), int(runs[i]))
        for i in range(count)
        if runs[i] > 0
    }
