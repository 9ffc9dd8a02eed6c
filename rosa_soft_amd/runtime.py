"""Device-resident packed hard router with the interface of ``rosa_soft.RosaRuntime``.

The reference's deployment runtime (``rosa_soft/runtime.py:311-856`` over
``rosa_soft/csrc/rosa_runtime.cpp``) stages every update to the host and walks one
suffix automaton per (slot, head) on CPU threads.  On MI355X the same contract —
exact latest-longest routing of a stream of 1..8-bit query/key/payload symbols,
chunk by chunk, with ``matched_key_end_positions`` — is served from HBM: every
(slot, head) keeps its symbols as bytes on the device and an update routes the
new rows against all earlier keys with the kernel of the training forward
(``rosa_hip_router_update``).  Nothing is computed on the host; without the HIP
library and a GPU the class raises.

Interface kept from the reference: constructor arguments and checks, ``update``
(sign logits) and ``update_packed`` (uint8 symbols) for dense ``[B, T, H]`` and
packed ``[total, H]`` + ``cu_seqlens`` inputs, grouped payload heads, fixed slot
count after the first update, ``sequence_ids`` reorder checks, ``return_packed`` /
``output_dtype`` unpacking with an exact-zero null route, ``async_op`` work handles,
``reset``, ``close``, context manager, ``state``.  Results come back on the device of
the inputs (host inputs are copied to the GPU and back).

Differences, all consequences of having no automaton: ``stats`` /
``memory_stats`` count stored symbols instead of automaton states and edges, and
``state_dict`` / ``load_state_dict`` work (the state is three byte tensors and the
slot lengths) where the reference raises ``NotImplementedError``.
"""

from __future__ import annotations

import operator
from typing import Any, Dict, Optional, Sequence, Tuple

import torch
from torch import Tensor

from . import cabi

__all__ = ["RosaRuntime"]


def _as_int(name: str, value: Any) -> int:
    """A Python int from anything that indexes exactly (numpy and torch integer scalars
    included); booleans and everything else are a TypeError naming the argument."""

    indexes = not isinstance(value, bool) and hasattr(type(value), "__index__")
    if not indexes:
        raise TypeError(f"{name} must be an integer")
    return int(operator.index(value))


def _pack_sign_bits(logits: Tensor, device: torch.device) -> Tensor:
    """uint8 symbols on ``device``: bit i = logits[..., i] > 0 (rosa_soft/runtime.py:130-146).

    One kernel of the library (``rosa_hip_pack_symbols``); host logits are moved to the
    device first, so nothing is computed on the host.
    """

    if not logits.is_floating_point():
        raise TypeError("unpacked RosaRuntime inputs must be floating-point")
    bits = logits.size(-1)
    if not 1 <= bits <= 8:
        raise ValueError(f"RosaRuntime supports 1..8 bits, got {bits}")
    logits = logits.to(device)
    if logits.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        # wider than the kernel reads (float64): only the sign matters, and a narrowing cast
        # would flush positives below the float32 range to zero, so hand over +-1 instead
        logits = torch.where(logits > 0, 1.0, -1.0).to(torch.float32)
    return cabi.pack_symbols(logits, torch.uint8)


def _unpack_sign_bits(packed: Tensor, bits: int, dtype: torch.dtype) -> Tensor:
    shifts = torch.arange(bits, device=packed.device, dtype=torch.int16)
    binary = ((packed.to(torch.int16).unsqueeze(-1) >> shifts) & 1).to(dtype)
    return binary.mul(2).sub(1)


_ID_DTYPES = frozenset({torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64})


def _slot_ids(sequence_ids, slot_count: int) -> Optional[Tuple[int, ...]]:
    """The caller's slot labels as a tuple of distinct ints, one per slot, or None when no
    labels were given (checks and messages of rosa_soft/runtime.py:149-176)."""

    if sequence_ids is None:
        return None
    if isinstance(sequence_ids, Tensor):
        if sequence_ids.ndim != 1:
            raise ValueError("sequence_ids must be a 1D tensor")
        if sequence_ids.dtype not in _ID_DTYPES:
            raise TypeError("sequence_ids must contain integers")
        items = sequence_ids.detach().cpu().tolist()
    elif isinstance(sequence_ids, Sequence) and not isinstance(sequence_ids, (str, bytes)):
        items = sequence_ids
    else:
        raise TypeError("sequence_ids must be an integer sequence")
    ids = tuple(_as_int("sequence_ids", item) for item in items)
    if len(ids) != slot_count:
        raise ValueError(f"sequence_ids must contain one ID per slot ({slot_count})")
    if len(frozenset(ids)) < len(ids):
        raise ValueError("sequence_ids must be unique")
    return ids


def _flatten_packed(query: Tensor, key: Tensor, payload: Tensor, cu_seqlens: Optional[Tensor]):
    """Token-major ``[total, H]`` views, host offsets, the output shape and the layout flag."""

    if any(tensor.dtype != torch.uint8 for tensor in (query, key, payload)):
        raise TypeError("packed RosaRuntime inputs must have dtype torch.uint8")
    if query.shape != key.shape:
        raise ValueError(f"packed query/key shapes differ: {query.shape} vs {key.shape}")
    if not (query.device == key.device == payload.device):
        raise ValueError("all packed inputs must be on the same device")
    if cu_seqlens is None:
        if query.ndim != 3 or payload.ndim != 3:
            raise ValueError("dense packed inputs must have shapes [B, T, H] and [B, T, H_v]")
        if query.shape[:2] != payload.shape[:2]:
            raise ValueError("dense query and payload dimensions B,T must match")
        slots, tokens, _ = query.shape
        if slots < 1:
            raise ValueError("dense batch size must be >= 1")
        offsets = [slot * tokens for slot in range(slots + 1)]
        return (
            query.reshape(slots * tokens, query.size(2)).contiguous(),
            key.reshape(slots * tokens, key.size(2)).contiguous(),
            payload.reshape(slots * tokens, payload.size(2)).contiguous(),
            offsets, tuple(payload.shape), True,
        )
    if query.ndim != 2 or payload.ndim != 2:
        raise ValueError("varlen packed inputs must have shapes [total, H] and [total, H_v]")
    if query.size(0) != payload.size(0):
        raise ValueError("varlen query and payload token counts must match")
    if cu_seqlens.ndim != 1:
        raise ValueError("cu_seqlens must be a 1D tensor")
    if cu_seqlens.numel() < 2:
        raise ValueError("cu_seqlens must describe at least one sequence")
    if cu_seqlens.dtype not in (torch.int32, torch.int64):
        raise TypeError("cu_seqlens must have dtype int32 or int64")
    offsets = [int(item) for item in cu_seqlens.to(device="cpu").tolist()]
    # the native checks of the reference (rosa_runtime.cpp:229-264, 283-303)
    if offsets[0] != 0:
        raise RuntimeError("cu_seqlens[0] must be 0")
    if any(after < before for before, after in zip(offsets[:-1], offsets[1:])):
        raise RuntimeError("cu_seqlens must be monotonic")
    if offsets[-1] != query.size(0):
        raise RuntimeError("query has wrong total token dimension")
    return query.contiguous(), key.contiguous(), payload.contiguous(), offsets, \
        tuple(payload.shape), False


class _RuntimeWork:
    """Handle of an enqueued update: ``wait()`` returns ``(output, matched_key_end_positions)``."""

    def __init__(self, result: Tuple[Tensor, Tensor], done: Optional[torch.cuda.Event],
                 stream: Optional[torch.cuda.Stream]) -> None:
        self._result = result
        self._done = done
        self._stream = stream

    def wait(self) -> Tuple[Tensor, Tensor]:
        if self._done is not None and self._stream is not None:
            # make the caller's stream see the side stream's results
            torch.cuda.current_stream(self._result[0].device).wait_event(self._done)
            self._done = None
        return self._result


class RosaRuntime:
    """Packed deployment runtime for exact hard routing, resident on the GPU.

    This is the 1..8-bit packed deployment subset of the training contract
    (``rosa_soft/runtime.py:311-318``).  It preserves exact latest-longest matching.
    Runtime slots are fixed by the first update; supplying ``sequence_ids`` on that
    update enables reorder checks.
    """

    _INITIAL_CAPACITY = 256

    def __init__(
        self,
        num_heads: int,
        num_payload_heads: Optional[int] = None,
        qk_bits: int = 8,
        payload_bits: int = 8,
        max_suffix_length: int = 32,
        *,
        device: Optional[torch.device] = None,
    ) -> None:
        if num_payload_heads is None:
            num_payload_heads = num_heads
        self._num_heads = _as_int("num_heads", num_heads)
        self._num_payload_heads = _as_int("num_payload_heads", num_payload_heads)
        self._qk_bits = _as_int("qk_bits", qk_bits)
        self._payload_bits = _as_int("payload_bits", payload_bits)
        self._max_suffix_length = _as_int("max_suffix_length", max_suffix_length)
        for name, width in (("qk_bits", self._qk_bits), ("payload_bits", self._payload_bits)):
            if not 1 <= width <= 8:
                raise ValueError(
                    f"{name} must be in [1, 8]; RosaRuntime implements only the packed 1..8-bit "
                    "deployment subset of the RosaSoft training contract"
                )
        # the native constructor's checks (rosa_runtime.cpp:306-331)
        if self._num_heads <= 0:
            raise RuntimeError("num_heads must be positive")
        if self._num_payload_heads <= 0:
            raise RuntimeError("num_payload_heads must be positive")
        if self._num_heads % self._num_payload_heads != 0:
            raise RuntimeError("num_heads must be divisible by num_payload_heads")
        if not 0 < self._max_suffix_length <= 2**31 - 1:
            raise RuntimeError("max_suffix_length must be in [1, int32_max]")
        cabi.load()  # fails loudly when the HIP library is not built
        if not torch.cuda.is_available():
            raise RuntimeError("RosaRuntime routes on the GPU and no device is available")
        self._device = torch.device("cuda", torch.cuda.current_device()) if device is None \
            else torch.device(device)
        self._state = "OPEN"
        self._clear()

    # ------------------------------------------------------------------ properties

    @property
    def num_heads(self) -> int:
        return self._num_heads

    @property
    def num_payload_heads(self) -> int:
        return self._num_payload_heads

    @property
    def qk_bits(self) -> int:
        return self._qk_bits

    @property
    def payload_bits(self) -> int:
        return self._payload_bits

    @property
    def max_suffix_length(self) -> int:
        return self._max_suffix_length

    @property
    def state(self) -> str:
        return self._state

    # ------------------------------------------------------------------ lifecycle

    def _clear(self) -> None:
        self._slot_count = -1
        self._sequence_ids: Optional[Tuple[int, ...]] = None
        self._slots_initialized = False
        self._lengths: list = []            # host mirror of the per-slot history lengths
        self._device_lengths: Optional[Tensor] = None   # [S] int32, advanced by the library
        self._capacity = 0
        self._query_history: Optional[Tensor] = None    # [S, H, capacity] uint8
        self._key_history: Optional[Tensor] = None      # [S, H, capacity] uint8
        self._payload_history: Optional[Tensor] = None  # [S, Hp, capacity] uint8
        self._last_update = None            # event recorded after the latest update's launches
        self._last_stream = None            # ... and the stream they went to

    def _require_open(self) -> None:
        if self._state != "OPEN":
            raise RuntimeError(f"RosaRuntime is {self._state.lower()}")

    def close(self) -> None:
        if self._state == "CLOSED":
            return
        self._clear()
        self._state = "CLOSED"

    def reset(self) -> None:
        self._require_open()
        self._clear()

    def __enter__(self) -> "RosaRuntime":
        self._require_open()
        return self

    def __exit__(self, exc_type, exc, traceback) -> None:
        self.close()

    # ------------------------------------------------------------------ statistics

    def stats(self) -> Tuple[int, int, int]:
        """Stored key, query and payload symbols (rosa_soft/runtime.py:552-555 counts automaton
        states, edges and payload symbols; the third entry means the same thing)."""

        self._require_open()
        tokens = sum(self._lengths)
        return (tokens * self._num_heads, tokens * self._num_heads,
                tokens * self._num_payload_heads)

    def memory_stats(self) -> Dict[str, int]:
        self._require_open()
        tokens = sum(self._lengths)
        logical = tokens * (2 * self._num_heads + self._num_payload_heads)
        slots = max(self._slot_count, 0)
        return {
            # the reference's names (rosa_soft/runtime.py:557-576); its states and edges belong
            # to suffix automata, which this runtime does not build: the stored key and query
            # symbols stand in their place, as in stats()
            "states": tokens * self._num_heads,
            "edges": tokens * self._num_heads,
            "automata": slots * self._num_heads,
            "key_symbols": tokens * self._num_heads,
            "query_symbols": tokens * self._num_heads,
            "payload_symbols": tokens * self._num_payload_heads,
            "sequences": slots,
            "logical_bytes": logical,
            "capacity_bytes":
                slots * self._capacity * (2 * self._num_heads + self._num_payload_heads),
        }

    def state_dict(self) -> Dict[str, Any]:
        self._require_open()
        longest = max(self._lengths, default=0)
        histories = {}
        for name in ("_query_history", "_key_history", "_payload_history"):
            tensor = getattr(self, name)
            histories[name[1:]] = None if tensor is None else tensor[..., :longest].cpu()
        return {
            "config": (self._num_heads, self._num_payload_heads, self._qk_bits,
                       self._payload_bits, self._max_suffix_length),
            "lengths": list(self._lengths),
            "sequence_ids": self._sequence_ids,
            "slots_initialized": self._slots_initialized,
            **histories,
        }

    def load_state_dict(self, state_dict: Dict[str, Any]) -> None:
        self._require_open()
        config = (self._num_heads, self._num_payload_heads, self._qk_bits,
                  self._payload_bits, self._max_suffix_length)
        if tuple(state_dict["config"]) != config:
            raise ValueError("state_dict was written by a runtime with another configuration")
        self._clear()
        self._lengths = [int(item) for item in state_dict["lengths"]]
        self._sequence_ids = state_dict["sequence_ids"]
        self._slots_initialized = bool(state_dict["slots_initialized"])
        if state_dict["key_history"] is None:
            return
        self._slot_count = len(self._lengths)
        stored = state_dict["key_history"].size(-1)
        self._grow(max(stored, 1))
        # (the kernels rely on stored symbols within their declared width, as updates store them)
        widths = {"query_history": self._qk_bits, "key_history": self._qk_bits,
                  "payload_history": self._payload_bits}
        for name, bits in widths.items():
            symbols = state_dict[name].to(self._device)
            getattr(self, "_" + name)[..., :stored] = symbols & ((1 << bits) - 1)

    # ------------------------------------------------------------------ updates

    def update(self, query_logits: Tensor, key_logits: Tensor, payload_logits: Tensor,
               cu_seqlens: Optional[Tensor] = None, *, stream=None, async_op: bool = False,
               return_packed: bool = False, sequence_ids=None):
        if query_logits.shape != key_logits.shape:
            raise ValueError(f"query/key shapes differ: {query_logits.shape} vs {key_logits.shape}")
        if query_logits.size(-1) != self.qk_bits:
            raise ValueError("query/key last dimension must equal qk_bits")
        if payload_logits.size(-1) != self.payload_bits:
            raise ValueError("payload last dimension must equal payload_bits")
        expected_rank = 4 if cu_seqlens is None else 3
        if query_logits.ndim != expected_rank or payload_logits.ndim != expected_rank:
            layout = "dense" if cu_seqlens is None else "varlen"
            raise ValueError(f"{layout} inputs have the wrong rank for RosaRuntime")
        if not (query_logits.device == key_logits.device == payload_logits.device):
            raise ValueError("all inputs must be on the same device")
        self._require_open()
        # the symbols are packed on the router's device, results return to the caller's
        return self._update_symbols(
            _pack_sign_bits(query_logits, self._device), _pack_sign_bits(key_logits, self._device),
            _pack_sign_bits(payload_logits, self._device), cu_seqlens, stream=stream,
            async_op=async_op, return_packed=return_packed, output_dtype=payload_logits.dtype,
            sequence_ids=sequence_ids, caller_device=payload_logits.device,
        )

    def update_packed(self, query_symbols: Tensor, key_symbols: Tensor, payload_symbols: Tensor,
                      cu_seqlens: Optional[Tensor] = None, *, stream=None,
                      async_op: bool = False, return_packed: bool = True,
                      output_dtype: torch.dtype = torch.float32, sequence_ids=None):
        return self._update_symbols(
            query_symbols, key_symbols, payload_symbols, cu_seqlens, stream=stream,
            async_op=async_op, return_packed=return_packed, output_dtype=output_dtype,
            sequence_ids=sequence_ids, caller_device=payload_symbols.device,
        )

    def _update_symbols(self, query_symbols: Tensor, key_symbols: Tensor, payload_symbols: Tensor,
                        cu_seqlens: Optional[Tensor], *, stream, async_op: bool,
                        return_packed: bool, output_dtype: torch.dtype, sequence_ids,
                        caller_device: torch.device):
        query, key, payload, offsets, output_shape, dense = _flatten_packed(
            query_symbols, key_symbols, payload_symbols, cu_seqlens
        )
        if query.size(1) != self.num_heads:
            raise ValueError("packed query/key head count must equal num_heads")
        if payload.size(1) != self.num_payload_heads:
            raise ValueError("packed payload head count must equal num_payload_heads")
        slot_count = len(offsets) - 1
        normalized_ids = _slot_ids(sequence_ids, slot_count)
        if stream is not None and caller_device.type != "cuda":
            raise ValueError("stream requires CUDA inputs")
        if stream is not None and stream.device != caller_device:
            raise ValueError("stream and inputs must use the same CUDA device")
        if not return_packed and not torch.empty((), dtype=output_dtype).is_floating_point():
            raise TypeError("output_dtype must be floating-point when unpacking")
        self._require_open()
        self._check_sequence_ids(normalized_ids)
        if self._slot_count == -1:
            self._slot_count = slot_count
            self._lengths = [0] * slot_count
        elif slot_count != self._slot_count:
            raise RuntimeError("RosaRuntime slot count is fixed after the first update")

        run_stream = stream if (stream is not None and caller_device == self._device) else None
        done = None
        if run_stream is not None:
            run_stream.wait_stream(torch.cuda.current_stream(self._device))
        with torch.cuda.stream(run_stream) if run_stream is not None else _NullContext():
            # Updates are serialised whatever streams they are given (the reference's
            # runtime does the same): this one starts after the previous one has finished
            # with the histories, including a growth copy.
            working_stream = torch.cuda.current_stream(self._device)
            if self._last_update is not None and working_stream != self._last_stream:
                working_stream.wait_event(self._last_update)
            output, ends = self._route(
                query.to(self._device), key.to(self._device), payload.to(self._device), offsets
            )
            if dense:
                output = output.reshape(output_shape[0], output_shape[1], self.num_heads)
                ends = ends.reshape(output_shape[0], output_shape[1], self.num_heads)
            if not return_packed:
                unpacked = _unpack_sign_bits(output, self.payload_bits, output_dtype)
                output = torch.where(
                    ends.unsqueeze(-1) >= 0, unpacked,
                    torch.zeros((), dtype=output_dtype, device=self._device),
                )
            # (one event, recorded anew by every update; an update on the stream of the one
            # before it is ordered by the stream itself)
            if self._last_update is None:
                self._last_update = torch.cuda.Event()
            self._last_update.record(working_stream)
            self._last_stream = working_stream
            if caller_device != self._device:
                output, ends = output.to(caller_device), ends.to(caller_device)
            if run_stream is not None:
                done = torch.cuda.Event()
                done.record(run_stream)
                for tensor in (output, ends):
                    tensor.record_stream(torch.cuda.current_stream(self._device))
        work = _RuntimeWork((output, ends), done, run_stream)
        return work if async_op else work.wait()

    # ------------------------------------------------------------------ internals

    def _check_sequence_ids(self, sequence_ids: Optional[Tuple[int, ...]]) -> None:
        # rosa_soft/runtime.py:513-535
        if not self._slots_initialized:
            self._slots_initialized = True
            self._sequence_ids = sequence_ids
            return
        if self._sequence_ids is None:
            if sequence_ids is not None:
                raise RuntimeError(
                    "sequence_ids checking must be enabled on the first update after "
                    "construction or reset"
                )
            return
        if sequence_ids is None:
            raise RuntimeError("sequence_ids are required because slot checking is enabled")
        if sequence_ids != self._sequence_ids:
            raise RuntimeError("sequence_ids changed; RosaRuntime slots are fixed")

    def _grow(self, needed: int) -> None:
        """Make every run hold at least ``needed`` symbols (doubling, contents kept)."""

        if needed <= self._capacity:
            return
        capacity = max(self._INITIAL_CAPACITY, self._capacity)
        while capacity < needed:
            capacity *= 2
        if capacity > 2**31 - 1:
            raise RuntimeError("ROSA sequence length exceeded int32 range")
        shapes = {
            "_query_history": (self._slot_count, self._num_heads, capacity),
            "_key_history": (self._slot_count, self._num_heads, capacity),
            "_payload_history": (self._slot_count, self._num_payload_heads, capacity),
        }
        for name, shape in shapes.items():
            grown = torch.zeros(shape, dtype=torch.uint8, device=self._device)
            old = getattr(self, name)
            if old is not None:
                grown[..., : self._capacity] = old
            setattr(self, name, grown)
        self._capacity = capacity

    def _route(self, query: Tensor, key: Tensor, payload: Tensor, offsets) -> Tuple[Tensor, Tensor]:
        tokens = query.size(0)
        output = torch.empty((tokens, self._num_heads), dtype=torch.uint8, device=self._device)
        ends = torch.empty((tokens, self._num_heads), dtype=torch.int64, device=self._device)
        if tokens == 0:
            return output, ends
        chunk_lengths = [after - before for before, after in zip(offsets[:-1], offsets[1:])]
        self._grow(max(old + new for old, new in zip(self._lengths, chunk_lengths)))
        if self._device_lengths is None:
            # two arrays taking turns: an update reads one and writes the advanced lengths to the
            # other, which makes a decoding step one launch
            self._device_lengths = torch.tensor(self._lengths, dtype=torch.int32).to(self._device)
            self._device_lengths_next = torch.empty_like(self._device_lengths)
        uniform = all(length == chunk_lengths[0] for length in chunk_lengths)
        tables = None if uniform else torch.tensor(offsets, dtype=torch.int32).to(self._device)
        update = cabi.RosaRouterUpdate()
        update.S, update.H, update.Hp = self._slot_count, self._num_heads, self._num_payload_heads
        update.W = min(self._max_suffix_length, 2**31 - 1)
        update.qk_bits, update.payload_bits = self._qk_bits, self._payload_bits
        update.capacity = self._capacity
        update.tokens = tokens
        update.longest_chunk = max(chunk_lengths)
        update.uniform_chunk = chunk_lengths[0] if uniform else 0
        update.chunk_offsets = None if uniform else tables.data_ptr()
        update.history_lengths = self._device_lengths.data_ptr()
        update.history_lengths_out = self._device_lengths_next.data_ptr()
        update.query_history = self._query_history.data_ptr()
        update.key_history = self._key_history.data_ptr()
        update.payload_history = self._payload_history.data_ptr()
        update.query, update.key, update.payload = \
            query.data_ptr(), key.data_ptr(), payload.data_ptr()
        update.output, update.matched_key_end = output.data_ptr(), ends.data_ptr()
        update.longest_total = max(old + new for old, new in zip(self._lengths, chunk_lengths))
        workspace = cabi.router_update(update, self._device)
        # stream-ordered launches: keep what they read alive until they have run
        for held in (tables, workspace):
            if held is not None:
                held.record_stream(torch.cuda.current_stream(self._device))
        self._device_lengths, self._device_lengths_next = \
            self._device_lengths_next, self._device_lengths
        self._lengths = [old + new for old, new in zip(self._lengths, chunk_lengths)]
        return output, ends


class _NullContext:
    def __enter__(self):
        return None

    def __exit__(self, *args):
        return False
