"""CPU restatement of the packed hard-routing contract of ``RosaRuntime`` (test infrastructure).

Nothing outside ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline
leg may import this module.

The contract (``rosa_soft/csrc/rosa_runtime.cpp:34-227`` — the per-(slot, head) suffix
automaton — and ``:333-487`` — ``update_packed``): symbols are bytes masked to ``qk_bits`` /
``payload_bits``; for the query at position ``t`` of a slot, among all key end positions
``e < t`` take the one with the longest common suffix of ``query[..t]`` and ``key[..e]``,
capped at ``max_suffix_length`` and at the available history, the latest on ties; a zero
length is the null route.  The answer is ``e`` (``-1`` for null) and the payload symbol at
``e + 1`` (``0`` for null).  The reference's own tests state it as the brute force of
``tests/test_runtime.py:19-77``; this file is that definition restated with numpy, plus a
streaming wrapper that feeds chunks to it the way ``update_packed`` is called.

Pinned by ``tests/test_router_oracle.py``: the reference's own runtime built from its source
(``oracle/_ref/librosa_runtime_ref.so``, see ``reference_runtime``) on seeded batches, chunked
and packed; the hand-derived answers of the reference's
finite-horizon example (``tests/test_runtime.py:166-217``), exhaustive agreement with an
independent formulation (run lengths by dynamic programming along diagonals) on all binary
strings of length four, and the relation to the training hard forward.
"""

from typing import List, Optional, Sequence, Tuple

import numpy as np


def route_slot(query: np.ndarray, key: np.ndarray, payload: np.ndarray, horizon: int,
               group: int) -> Tuple[np.ndarray, np.ndarray]:
    """One slot: ``query``/``key`` ``[T, H]``, ``payload`` ``[T, Hp]`` (already masked).

    Returns ``(output [T, H] uint8, matched_key_end [T, H] int64)``.
    """

    tokens, heads = query.shape
    output = np.zeros((tokens, heads), dtype=np.uint8)
    ends = np.full((tokens, heads), -1, dtype=np.int64)
    for head in range(heads):
        q = query[:, head]
        k = key[:, head]
        for t in range(tokens):
            best_length, best_end = 0, -1
            for e in range(t):
                limit = min(horizon, t + 1, e + 1)
                length = 0
                while length < limit and q[t - length] == k[e - length]:
                    length += 1
                if length > 0 and length >= best_length:  # latest among the longest
                    best_length, best_end = length, e
            if best_end >= 0:
                ends[t, head] = best_end
                output[t, head] = payload[best_end + 1, head // group]
    return output, ends


class StreamingRouter:
    """Chunk-by-chunk driver with the call shape of ``update_packed``."""

    def __init__(self, num_heads: int, num_payload_heads: int, qk_bits: int, payload_bits: int,
                 max_suffix_length: int) -> None:
        assert num_heads % num_payload_heads == 0
        self.heads, self.payload_heads = num_heads, num_payload_heads
        self.qk_mask, self.payload_mask = (1 << qk_bits) - 1, (1 << payload_bits) - 1
        self.horizon = max_suffix_length
        self.histories: Optional[List[List[np.ndarray]]] = None

    def update_packed(self, query: np.ndarray, key: np.ndarray, payload: np.ndarray,
                      offsets: Sequence[int]) -> Tuple[np.ndarray, np.ndarray]:
        """``query``/``key`` ``[total, H]``, ``payload`` ``[total, Hp]``, ``offsets`` ``[S + 1]``."""

        slots = len(offsets) - 1
        if self.histories is None:
            self.histories = [
                [np.zeros((0, self.heads), np.uint8), np.zeros((0, self.heads), np.uint8),
                 np.zeros((0, self.payload_heads), np.uint8)] for _ in range(slots)
            ]
        assert slots == len(self.histories), "slot count is fixed after the first update"
        output = np.zeros((query.shape[0], self.heads), dtype=np.uint8)
        ends = np.full((query.shape[0], self.heads), -1, dtype=np.int64)
        group = self.heads // self.payload_heads
        for slot in range(slots):
            begin, end = offsets[slot], offsets[slot + 1]
            history = self.histories[slot]
            old = history[0].shape[0]
            history[0] = np.concatenate([history[0], query[begin:end] & self.qk_mask])
            history[1] = np.concatenate([history[1], key[begin:end] & self.qk_mask])
            history[2] = np.concatenate([history[2], payload[begin:end] & self.payload_mask])
            # routing the whole history again and keeping the new rows is the definition
            slot_output, slot_ends = route_slot(history[0], history[1], history[2], self.horizon,
                                                group)
            output[begin:end] = slot_output[old:]
            ends[begin:end] = slot_ends[old:]
        return output, ends


def route_dense(query: np.ndarray, key: np.ndarray, payload: np.ndarray, qk_bits: int,
                payload_bits: int, max_suffix_length: int) -> Tuple[np.ndarray, np.ndarray]:
    """Dense ``[B, T, H]`` / ``[B, T, Hp]`` one-shot call."""

    batch, tokens, heads = query.shape
    router = StreamingRouter(heads, payload.shape[2], qk_bits, payload_bits, max_suffix_length)
    offsets = [slot * tokens for slot in range(batch + 1)]
    output, ends = router.update_packed(
        query.reshape(batch * tokens, heads), key.reshape(batch * tokens, heads),
        payload.reshape(batch * tokens, -1), offsets,
    )
    return output.reshape(batch, tokens, heads), ends.reshape(batch, tokens, heads)


def reference_runtime():
    """``torch.classes.rosa_soft.RosaRuntime`` of the reference, if ``make -C oracle ref`` built it.

    The class is compiled from ``/root/reference/rosa_soft/csrc/rosa_runtime.cpp`` where it
    lies; returns ``None`` when the library is absent.
    """

    import os

    import torch

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref",
                        "librosa_runtime_ref.so")
    if not os.path.exists(path):
        return None
    torch.ops.load_library(path)
    return torch.classes.rosa_soft.RosaRuntime
