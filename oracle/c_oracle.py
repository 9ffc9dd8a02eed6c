"""ctypes front end of ``librosa_oracle.so`` (TEST ORACLE, never shipped).

Loads the float64 row-streamed C restatement built from ``rosa_oracle.c`` and
offers dense and packed helpers working on CPU torch tensors.  Only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` import this module.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Sequence, Tuple

import numpy as np
import torch
from torch import Tensor

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librosa_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``librosa_oracle.so`` with the Makefile next to this file."""

    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB_PATH


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    f32p = ctypes.POINTER(ctypes.c_float)
    f64p = ctypes.POINTER(ctypes.c_double)
    i32p = ctypes.POINTER(ctypes.c_int32)
    lib.rosa_oracle_hard_forward.restype = ctypes.c_int
    lib.rosa_oracle_hard_forward.argtypes = [
        f32p, f32p, f32p, *([ctypes.c_int] * 7), f32p, i32p, i32p,
    ]
    lib.rosa_oracle_surrogate_vjp.restype = ctypes.c_int
    lib.rosa_oracle_surrogate_vjp.argtypes = [
        f32p, f32p, f32p, f32p, *([ctypes.c_int] * 7),
        ctypes.c_double, ctypes.c_double, ctypes.c_double,
        ctypes.c_int, ctypes.c_uint64, i32p, ctypes.c_int,
        f64p, f64p, f64p,
    ]
    lib.rosa_oracle_dropout_uniform.restype = ctypes.c_float
    lib.rosa_oracle_dropout_uniform.argtypes = [
        ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
        ctypes.c_uint32,
    ]
    lib.rosa_oracle_num_threads.restype = ctypes.c_int
    lib.rosa_oracle_set_threads.argtypes = [ctypes.c_int]
    _lib = lib
    return lib


def _f32(tensor: Tensor) -> np.ndarray:
    return np.ascontiguousarray(tensor.detach().cpu().to(torch.float32).numpy())


def _ptr(array: Optional[np.ndarray], ctype):
    if array is None:
        return ctypes.cast(None, ctypes.POINTER(ctype))
    return array.ctypes.data_as(ctypes.POINTER(ctype))


def num_threads() -> int:
    return int(load().rosa_oracle_num_threads())


def set_threads(count: int) -> None:
    load().rosa_oracle_set_threads(int(count))


def dropout_uniform(seed: int, batch: int, head: int, row: int, route: int) -> float:
    return float(
        load().rosa_oracle_dropout_uniform(
            int(seed) & 0xFFFFFFFFFFFFFFFF, batch, head, row, route
        )
    )


def hard_forward(
    query: Tensor, key: Tensor, value: Tensor, max_suffix_length: int
) -> Tuple[Tensor, Tensor, Tensor]:
    """Dense hard forward: ``(output, routes [B,H,T], best_length [B,H,T])``."""

    lib = load()
    batch, seq_len, heads, width = query.shape
    value_heads, value_dim = value.shape[2], value.shape[3]
    horizon = min(int(max_suffix_length), seq_len)
    q, k, v = _f32(query), _f32(key), _f32(value)
    out = np.empty((batch, seq_len, heads, value_dim), dtype=np.float32)
    routes = np.empty((batch, heads, seq_len), dtype=np.int32)
    lengths = np.empty((batch, heads, seq_len), dtype=np.int32)
    status = lib.rosa_oracle_hard_forward(
        _ptr(q, ctypes.c_float), _ptr(k, ctypes.c_float), _ptr(v, ctypes.c_float),
        batch, seq_len, heads, width, value_heads, value_dim, horizon,
        _ptr(out, ctypes.c_float), _ptr(routes, ctypes.c_int32),
        _ptr(lengths, ctypes.c_int32),
    )
    if status != 0:
        raise RuntimeError(f"rosa_oracle_hard_forward failed with status {status}")
    return (
        torch.from_numpy(out).to(query.dtype),
        torch.from_numpy(routes),
        torch.from_numpy(lengths),
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
    head_offset: int = 0,
    needs: Tuple[bool, bool, bool] = (True, True, True),
) -> Tuple[Optional[Tensor], Optional[Tensor], Optional[Tensor]]:
    """Dense surrogate VJP in float64; gradients are float64 tensors."""

    lib = load()
    batch, seq_len, heads, width = query.shape
    value_heads, value_dim = value.shape[2], value.shape[3]
    horizon = min(int(max_suffix_length), seq_len)
    q, k, v, go = _f32(query), _f32(key), _f32(value), _f32(grad_output)
    ids = np.asarray(
        list(range(batch)) if batch_ids is None else list(batch_ids), dtype=np.int32
    )
    grads = [
        np.empty(shape, dtype=np.float64) if need else None
        for need, shape in zip(needs, (q.shape, k.shape, v.shape))
    ]
    status = lib.rosa_oracle_surrogate_vjp(
        _ptr(q, ctypes.c_float), _ptr(k, ctypes.c_float), _ptr(v, ctypes.c_float),
        _ptr(go, ctypes.c_float),
        batch, seq_len, heads, width, value_heads, value_dim, horizon,
        float(scale), float(dropout_p), float(mismatch_scale),
        0 if seed is None else 1,
        0 if seed is None else int(seed) & 0xFFFFFFFFFFFFFFFF,
        _ptr(ids, ctypes.c_int32), int(head_offset),
        _ptr(grads[0], ctypes.c_double), _ptr(grads[1], ctypes.c_double),
        _ptr(grads[2], ctypes.c_double),
    )
    if status != 0:
        raise RuntimeError(f"rosa_oracle_surrogate_vjp failed with status {status}")
    return tuple(None if g is None else torch.from_numpy(g) for g in grads)


def varlen_hard_forward(
    query: Tensor, key: Tensor, value: Tensor, cu_seqlens: Sequence[int],
    max_suffix_length: int,
) -> Tuple[Tensor, Tensor]:
    """Packed hard forward: ``(output [N,H,Dv], routes [H,N])`` (routes are
    segment-local, 0 = null)."""

    offsets = [int(x) for x in cu_seqlens]
    horizon = min(int(max_suffix_length), query.size(0))
    output = torch.zeros(query.size(0), query.size(1), value.size(2), dtype=query.dtype)
    routes = torch.zeros(query.size(1), query.size(0), dtype=torch.int32)
    for start, end in zip(offsets[:-1], offsets[1:]):
        if start == end:
            continue
        out, rts, _ = hard_forward(
            query[start:end].unsqueeze(0), key[start:end].unsqueeze(0),
            value[start:end].unsqueeze(0), horizon,
        )
        output[start:end] = out[0]
        routes[:, start:end] = rts[0]
    return output, routes


def varlen_surrogate_vjp(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    cu_seqlens: Sequence[int],
    grad_output: Tensor,
    *,
    max_suffix_length: int,
    scale: float = 1.0,
    dropout_p: float = 0.0,
    mismatch_scale: float = 3.0,
    seed: Optional[int] = None,
    head_offset: int = 0,
    needs: Tuple[bool, bool, bool] = (True, True, True),
):
    """Packed surrogate VJP: each segment independent, batch coordinate of the
    dropout hash = sequence index (empty segments still count)."""

    offsets = [int(x) for x in cu_seqlens]
    horizon = min(int(max_suffix_length), query.size(0))
    grads = [
        torch.zeros(t.shape, dtype=torch.float64) if need else None
        for t, need in zip((query, key, value), needs)
    ]
    for sequence, (start, end) in enumerate(zip(offsets[:-1], offsets[1:])):
        if start == end:
            continue
        piece = surrogate_vjp(
            query[start:end].unsqueeze(0), key[start:end].unsqueeze(0),
            value[start:end].unsqueeze(0), grad_output[start:end].unsqueeze(0),
            max_suffix_length=horizon, scale=scale, dropout_p=dropout_p,
            mismatch_scale=mismatch_scale, seed=seed, batch_ids=[sequence],
            head_offset=head_offset, needs=needs,
        )
        for total, part in zip(grads, piece):
            if total is not None:
                total[start:end] = part[0]
    return tuple(grads)
