"""Device-resident ``RosaRuntime`` against the CPU oracle (needs a real MI355X).

Mirrors the reference's ``tests/test_runtime.py:96-420``: same shapes, seeds and properties,
with the brute-force definition (``oracle/router_oracle.py``) as the expected side.
"""

import numpy as np
import pytest
import torch

from oracle import router_oracle

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"


@pytest.fixture(scope="module")
def rosa():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import rosa_soft_amd

    assert rosa_soft_amd.BUILD_CAPABILITIES.rosa_runtime
    return rosa_soft_amd


def random_packed(shape, bits, seed):
    return torch.randint(0, 1 << bits, shape, dtype=torch.uint8,
                         generator=torch.Generator().manual_seed(seed))


def expect_dense(query, key, payload, qk_bits, payload_bits, horizon):
    output, ends = router_oracle.route_dense(query.numpy(), key.numpy(), payload.numpy(), qk_bits,
                                             payload_bits, horizon)
    return torch.from_numpy(output), torch.from_numpy(ends)


@pytest.mark.parametrize("horizon", [1, 2, 5, 64])
def test_packed_dense_matches_oracle(rosa, horizon):
    batch, tokens, heads, payload_heads, bits = 2, 19, 4, 2, 4
    query = random_packed((batch, tokens, heads), bits, 1)
    key = random_packed((batch, tokens, heads), bits, 2)
    payload = random_packed((batch, tokens, payload_heads), bits, 3)
    want = expect_dense(query, key, payload, bits, bits, horizon)
    with rosa.RosaRuntime(heads, payload_heads, bits, bits, horizon) as runtime:
        got = runtime.update_packed(query.to(DEVICE), key.to(DEVICE), payload.to(DEVICE))
        stats = runtime.stats()
    assert got[0].dtype == torch.uint8 and got[1].dtype == torch.int64
    assert got[0].device.type == "cuda"
    assert torch.equal(got[0].cpu(), want[0]) and torch.equal(got[1].cpu(), want[1])
    assert stats[2] == batch * payload_heads * tokens


@pytest.mark.parametrize("horizon", [1, 2, 4])
def test_binary_length_four_state_space(rosa, horizon):
    patterns = torch.tensor([[(code >> shift) & 1 for shift in range(4)] for code in range(16)],
                            dtype=torch.uint8).unsqueeze(-1)
    query = patterns.repeat_interleave(16, dim=0)
    key = patterns.repeat(16, 1, 1)
    payload = torch.arange(4, dtype=torch.uint8).view(1, 4, 1).expand(256, -1, -1).contiguous()
    want = expect_dense(query, key, payload, 1, 2, horizon)
    with rosa.RosaRuntime(1, 1, 1, 2, horizon) as runtime:
        got = runtime.update_packed(query.to(DEVICE), key.to(DEVICE), payload.to(DEVICE))
    assert torch.equal(got[0].cpu(), want[0]) and torch.equal(got[1].cpu(), want[1])


def test_finite_horizon_changes_route_and_host_inputs_come_back_on_the_host(rosa):
    query = torch.zeros(1, 6, 1, dtype=torch.uint8)
    key = torch.tensor([[[0], [0], [0], [1], [0], [0]]], dtype=torch.uint8)
    payload = torch.tensor([[[1], [2], [3], [4], [5], [6]]], dtype=torch.uint8)
    answers = {1: ([0, 2, 3, 4, 4, 6], [-1, 0, 1, 2, 2, 4]), 4: ([0, 2, 3, 4, 4, 4], [-1, 0, 1, 2, 2, 2])}
    for horizon, (want_output, want_ends) in answers.items():
        with rosa.RosaRuntime(1, 1, 1, 3, horizon) as runtime:
            output, ends = runtime.update_packed(query, key, payload)
        assert output.device.type == "cpu" and ends.device.type == "cpu"
        assert output.reshape(-1).tolist() == want_output
        assert ends.reshape(-1).tolist() == want_ends


def test_varlen_and_grouped_payload_heads(rosa):
    lengths = [4, 9, 0, 6]
    offsets = torch.tensor([0, 4, 13, 13, 19], dtype=torch.int32)
    heads, payload_heads, bits, horizon = 6, 3, 3, 4
    total = sum(lengths)
    query = random_packed((total, heads), bits, 4)
    key = random_packed((total, heads), bits, 5)
    payload = random_packed((total, payload_heads), bits, 6)
    router = router_oracle.StreamingRouter(heads, payload_heads, bits, bits, horizon)
    want = router.update_packed(query.numpy(), key.numpy(), payload.numpy(), offsets.tolist())
    with rosa.RosaRuntime(heads, payload_heads, bits, bits, horizon) as runtime:
        got = runtime.update_packed(query.to(DEVICE), key.to(DEVICE), payload.to(DEVICE),
                                    cu_seqlens=offsets)
    assert torch.equal(got[0].cpu(), torch.from_numpy(want[0]))
    assert torch.equal(got[1].cpu(), torch.from_numpy(want[1]))


def test_chunked_updates_equal_one_shot_and_histories_grow(rosa):
    # 700 tokens per slot: several 64-row blocks per chunk, unaligned chunk starts, and the
    # history outgrows its first allocation twice
    batch, tokens, heads, payload_heads, bits, horizon = 2, 700, 3, 1, 2, 9
    query = random_packed((batch, tokens, heads), bits, 7)
    key = random_packed((batch, tokens, heads), bits, 8)
    payload = random_packed((batch, tokens, payload_heads), 5, 9)
    want = expect_dense(query, key, payload, bits, 5, horizon)
    with rosa.RosaRuntime(heads, payload_heads, bits, 5, horizon) as one_shot:
        whole = one_shot.update_packed(query.to(DEVICE), key.to(DEVICE), payload.to(DEVICE))
    assert torch.equal(whole[0].cpu(), want[0]) and torch.equal(whole[1].cpu(), want[1])
    chunks = [0, 3, 11, 200, 201, 457, 640, tokens]
    outputs, positions = [], []
    with rosa.RosaRuntime(heads, payload_heads, bits, 5, horizon) as chunked:
        for begin, end in zip(chunks[:-1], chunks[1:]):
            output, ends = chunked.update_packed(
                query[:, begin:end].to(DEVICE), key[:, begin:end].to(DEVICE),
                payload[:, begin:end].to(DEVICE),
            )
            outputs.append(output)
            positions.append(ends)
        assert chunked.memory_stats()["payload_symbols"] == batch * payload_heads * tokens
    assert torch.equal(torch.cat(outputs, dim=1).cpu(), want[0])
    assert torch.equal(torch.cat(positions, dim=1).cpu(), want[1])


def test_single_token_decode_steps(rosa):
    heads, bits, horizon, tokens = 2, 1, 6, 90
    query = random_packed((1, tokens, heads), bits, 17)
    key = random_packed((1, tokens, heads), bits, 18)
    payload = random_packed((1, tokens, heads), 8, 19)
    want = expect_dense(query, key, payload, bits, 8, horizon)
    ends = []
    with rosa.RosaRuntime(heads, heads, bits, 8, horizon) as runtime:
        for t in range(tokens):
            step = runtime.update_packed(query[:, t:t + 1].to(DEVICE), key[:, t:t + 1].to(DEVICE),
                                         payload[:, t:t + 1].to(DEVICE))
            ends.append(step[1])
    assert torch.equal(torch.cat(ends, dim=1).cpu(), want[1])


def test_unpacked_null_route_is_exact_zero_and_logit_interface(rosa):
    # reference tests/test_runtime.py:318-345
    query = torch.ones(1, 5, 1, 2, device=DEVICE)
    key = -torch.ones_like(query)
    payload = torch.ones(1, 5, 1, 3, device=DEVICE)
    with rosa.RosaRuntime(1, 1, 2, 3, 3) as runtime:
        output, ends = runtime.update(query, key, payload)
    assert output.shape == (1, 5, 1, 3) and output.dtype == torch.float32
    assert torch.count_nonzero(output) == 0 and torch.all(ends == -1)
    with rosa.RosaRuntime(1, 1, 2, 3, 3) as runtime:
        output, ends = runtime.update(query, query, payload)
    assert torch.equal(output[0, 1:], torch.ones(4, 1, 3, device=DEVICE))
    assert ends.reshape(-1).tolist() == [-1, 0, 1, 2, 3]


def test_lifecycle_slot_and_sequence_id_checks(rosa):
    symbols = torch.zeros(2, 3, 1, dtype=torch.uint8, device=DEVICE)
    runtime = rosa.RosaRuntime(1, 1, 1, 1, 2)
    assert runtime.state == "OPEN"
    runtime.update_packed(symbols, symbols, symbols, sequence_ids=[7, 9])
    with pytest.raises(RuntimeError, match="sequence_ids changed"):  # checked before the slots
        runtime.update_packed(symbols[:1], symbols[:1], symbols[:1], sequence_ids=[7])
    with pytest.raises(RuntimeError, match="sequence_ids are required"):
        runtime.update_packed(symbols, symbols, symbols)
    with pytest.raises(RuntimeError, match="sequence_ids changed"):
        runtime.update_packed(symbols, symbols, symbols, sequence_ids=[9, 7])
    with pytest.raises(ValueError, match="must be unique"):
        runtime.update_packed(symbols, symbols, symbols, sequence_ids=[7, 7])
    runtime.reset()
    assert runtime.stats() == (0, 0, 0)
    runtime.update_packed(symbols[:1], symbols[:1], symbols[:1])
    with pytest.raises(RuntimeError, match="slot count is fixed"):
        runtime.update_packed(symbols, symbols, symbols)
    with pytest.raises(RuntimeError, match="first update"):
        runtime.update_packed(symbols[:1], symbols[:1], symbols[:1], sequence_ids=[1])
    with pytest.raises(TypeError, match="torch.uint8"):
        runtime.update_packed(symbols.int(), symbols.int(), symbols.int())
    with pytest.raises(ValueError, match="head count must equal num_heads"):
        wide = torch.zeros(1, 3, 2, dtype=torch.uint8, device=DEVICE)
        runtime.update_packed(wide, wide, wide)
    runtime.close()
    assert runtime.state == "CLOSED"
    with pytest.raises(RuntimeError, match="closed"):
        runtime.update_packed(symbols[:1], symbols[:1], symbols[:1])
    runtime.close()  # idempotent
    with pytest.raises(ValueError, match=r"qk_bits must be in \[1, 8\]"):
        rosa.RosaRuntime(1, 1, 9, 1, 1)
    with pytest.raises(RuntimeError, match="divisible"):
        rosa.RosaRuntime(3, 2, 1, 1, 1)


def test_state_dict_round_trip_and_async_handle(rosa):
    heads, bits, horizon = 2, 3, 5
    query = random_packed((1, 60, heads), bits, 31)
    key = random_packed((1, 60, heads), bits, 32)
    payload = random_packed((1, 60, 1), bits, 33)
    want = expect_dense(query, key, payload, bits, bits, horizon)
    first = rosa.RosaRuntime(heads, 1, bits, bits, horizon)
    first.update_packed(query[:, :25].to(DEVICE), key[:, :25].to(DEVICE), payload[:, :25].to(DEVICE))
    saved = first.state_dict()
    first.close()
    second = rosa.RosaRuntime(heads, 1, bits, bits, horizon)
    second.load_state_dict(saved)
    side = torch.cuda.Stream(device=DEVICE)
    work = second.update_packed(query[:, 25:].to(DEVICE), key[:, 25:].to(DEVICE),
                                payload[:, 25:].to(DEVICE), stream=side, async_op=True)
    output, ends = work.wait()
    torch.cuda.synchronize()
    assert torch.equal(ends.cpu(), want[1][:, 25:]) and torch.equal(output.cpu(), want[0][:, 25:])
    second.close()


def test_history_beyond_65535_tokens_matches_the_dense_forward(rosa):
    # past 65535 tokens of history the route scan switches from its 32-bit key to the 64-bit
    # one; the expected routes come from the training forward's oracle on the same symbols
    from oracle import c_oracle

    tokens, bits, horizon = 66000, 2, 40
    query = random_packed((1, tokens, 1), bits, 11)
    key = random_packed((1, tokens, 1), bits, 12)
    payload = random_packed((1, tokens, 1), bits, 13)

    def signs(symbols):
        planes = (symbols.unsqueeze(-1) >> torch.arange(bits, dtype=torch.uint8)) & 1
        return planes.to(torch.float32) * 2.0 - 1.0  # [1, tokens, 1, bits]

    _, routes, _ = c_oracle.hard_forward(signs(query), signs(key), signs(payload), horizon)
    routes = routes.reshape(-1).to(torch.int64)
    want_ends = torch.where(routes > 0, routes - 1, torch.full_like(routes, -1))
    want_output = torch.where(routes > 0, payload.reshape(-1)[routes.clamp(min=0)].to(torch.int64),
                              torch.zeros_like(routes))
    with rosa.RosaRuntime(1, 1, bits, bits, horizon) as runtime:
        pieces = []
        for begin, end in ((0, 40000), (40000, 65999), (65999, tokens)):
            got = runtime.update_packed(query[:, begin:end].to(DEVICE), key[:, begin:end].to(DEVICE),
                                        payload[:, begin:end].to(DEVICE))
            pieces.append((got[0].cpu().reshape(-1), got[1].cpu().reshape(-1)))
    output = torch.cat([piece[0] for piece in pieces]).to(torch.int64)
    ends = torch.cat([piece[1] for piece in pieces])
    assert int(ends.max()) > 65535
    assert torch.equal(ends, want_ends)
    assert torch.equal(output, want_output)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_chunkings_match_the_dense_definition(rosa, seed):
    # random symbol widths, horizons, head groupings and chunk boundaries: chunks of up to 8
    # rows take the per-row kernel, longer ones the row-block scan
    import random

    rng = random.Random(seed)
    for case in range(10):
        batch = rng.choice([1, 2, 3])
        payload_heads = rng.choice([1, 2])
        heads = payload_heads * rng.choice([1, 2])
        bits = rng.choice([1, 2, 3, 8])
        payload_bits = rng.choice([1, 4, 8])
        horizon = rng.choice([1, 2, 5, 17, 64, 200])
        tokens = rng.choice([1, 9, 64, 65, 130, 300])
        query = random_packed((batch, tokens, heads), bits, 100 * seed + 3 * case)
        key = random_packed((batch, tokens, heads), bits, 100 * seed + 3 * case + 1)
        payload = random_packed((batch, tokens, payload_heads), payload_bits, 100 * seed + 3 * case + 2)
        want = expect_dense(query, key, payload, bits, payload_bits, horizon)
        cuts = sorted({0, tokens, *(rng.randrange(0, tokens + 1) for _ in range(rng.choice([0, 2, 6])))})
        outputs, positions = [], []
        with rosa.RosaRuntime(heads, payload_heads, bits, payload_bits, horizon) as runtime:
            for begin, end in zip(cuts[:-1], cuts[1:]):
                output, ends = runtime.update_packed(
                    query[:, begin:end].to(DEVICE), key[:, begin:end].to(DEVICE),
                    payload[:, begin:end].to(DEVICE))
                outputs.append(output)
                positions.append(ends)
        label = f"seed {seed} case {case}: cuts {cuts}"
        assert torch.equal(torch.cat(outputs, dim=1).cpu(), want[0]), label
        assert torch.equal(torch.cat(positions, dim=1).cpu(), want[1]), label


def test_logit_updates_pack_on_the_device_and_match_packed_updates(rosa):
    """``update`` (sign logits, every float dtype, host or device) routes exactly like
    ``update_packed`` on the symbols ``bit i = logit[..., i] > 0``; host inputs come back on
    the host (reference rosa_soft/runtime.py:130-146, tests/test_runtime.py:318-345)."""

    batch, tokens, heads, payload_heads, horizon = 2, 37, 4, 2, 6
    generator = torch.Generator().manual_seed(50)
    for qk_bits, payload_bits, dtype in ((8, 8, torch.float32), (3, 5, torch.float16),
                                         (1, 7, torch.bfloat16), (8, 2, torch.float64)):
        logits = [torch.randn(batch, tokens, h, bits, generator=generator).to(dtype)
                  for h, bits in ((heads, qk_bits), (heads, qk_bits), (payload_heads, payload_bits))]
        logits[0][0, 3, 1, 0] = 0.0            # zero, NaN and -inf quantise to bit 0, +inf to 1
        logits[1][1, 5, 0, 0] = float("nan")
        logits[2][0, 7, 1, 0] = float("-inf")
        logits[2][0, 8, 1, 0] = float("inf")
        if dtype == torch.float64:
            # positives and negatives below the float32 range keep their sign bit
            logits[0][1, 2, 0, 1] = 1e-300
            logits[1][1, 2, 0, 1] = -1e-300
            logits[2][1, 9, 0, 1] = 1e-300
        symbols = []
        for tensor in logits:
            weights = 1 << torch.arange(tensor.size(-1), dtype=torch.int64)
            symbols.append(((tensor > 0).long() * weights).sum(-1).to(torch.uint8))
        want = expect_dense(*symbols, qk_bits, payload_bits, horizon)
        for place in (DEVICE, "cpu"):
            with rosa.RosaRuntime(heads, payload_heads, qk_bits, payload_bits, horizon) as runtime:
                output, ends = runtime.update(*(t.to(place) for t in logits), return_packed=True)
            assert output.device.type == torch.device(place).type
            assert torch.equal(output.cpu(), want[0]) and torch.equal(ends.cpu(), want[1])


def test_many_slots_and_heads_in_one_update(rosa):
    # slots * heads beyond the 65535 blocks of a grid's second dimension
    slots, tokens, heads, bits, horizon = 1100, 9, 64, 2, 4
    query = random_packed((slots, tokens, heads), bits, 61)
    key = random_packed((slots, tokens, heads), bits, 62)
    payload = random_packed((slots, tokens, heads), bits, 63)
    want = expect_dense(query, key, payload, bits, bits, horizon)
    with rosa.RosaRuntime(heads, heads, bits, bits, horizon) as runtime:
        first = runtime.update_packed(query[:, :8].to(DEVICE), key[:, :8].to(DEVICE),
                                      payload[:, :8].to(DEVICE))
        last = runtime.update_packed(query[:, 8:].to(DEVICE), key[:, 8:].to(DEVICE),
                                     payload[:, 8:].to(DEVICE))     # decode-sized chunk
    got_output = torch.cat([first[0], last[0]], dim=1).cpu()
    got_ends = torch.cat([first[1], last[1]], dim=1).cpu()
    assert torch.equal(got_output, want[0]) and torch.equal(got_ends, want[1])


def test_updates_on_different_streams_are_serialised(rosa):
    heads, bits, horizon = 2, 2, 7
    query = random_packed((1, 3000, heads), bits, 71)
    key = random_packed((1, 3000, heads), bits, 72)
    payload = random_packed((1, 3000, 1), bits, 73)
    want = expect_dense(query, key, payload, bits, bits, horizon)
    q, k, p = (t.to(DEVICE) for t in (query, key, payload))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=DEVICE) for _ in range(3)]
    pieces = []
    with rosa.RosaRuntime(heads, 1, bits, bits, horizon) as runtime:
        bounds = [0, 1500, 1501, 2600, 3000]
        for index, (begin, end) in enumerate(zip(bounds[:-1], bounds[1:])):
            stream = streams[index % 3] if index != 2 else None
            pieces.append(runtime.update_packed(q[:, begin:end], k[:, begin:end], p[:, begin:end],
                                                stream=stream, async_op=True))
        results = [work.wait() for work in pieces]
        torch.cuda.synchronize()
    assert torch.equal(torch.cat([r[0] for r in results], dim=1).cpu(), want[0])
    assert torch.equal(torch.cat([r[1] for r in results], dim=1).cpu(), want[1])


@pytest.mark.parametrize("pattern", ["random", "period7", "constant"])
def test_long_chunks_route_through_the_index_of_the_keys(rosa, pattern):
    # chunks beyond 8 rows on histories of 512 tokens or more take the index of the keys
    # (8- and 6-bit symbols here); periodic and constant inputs hand their row blocks back.
    # The scan over all routes gives the expectation (the oracle as well where it is quick).
    from rosa_soft_amd import cabi

    batch, tokens, heads, payload_heads = 2, 1500, 4, 2
    for bits in (8, 6):
        query = random_packed((batch, tokens, heads), bits, 50 + bits)
        key = random_packed((batch, tokens, heads), bits, 60 + bits)
        if pattern == "period7":
            key = key[:, :7].repeat(1, tokens // 7 + 1, 1)[:, :tokens].contiguous()
            query = torch.roll(key, 1, dims=1).contiguous()
        elif pattern == "constant":
            key = torch.full_like(key, 3)
            query = torch.full_like(query, 3)
        else:
            # a repeated stretch, so that long runs and ties exist
            key[:, 900:1300] = key[:, 100:500]
            query[:, 901:1300] = key[:, 900:1299]
        payload = random_packed((batch, tokens, payload_heads), 8, 70 + bits)
        results = {}
        for mode in ("scan", None, "handed_back"):
            outputs, positions = [], []
            cabi.set_forward_index(mode)
            try:
                with rosa.RosaRuntime(heads, payload_heads, bits, 8, 40) as runtime:
                    for begin, end in [(0, 700), (700, 705), (705, 1400), (1400, 1500)]:
                        output, ends = runtime.update_packed(
                            query[:, begin:end].to(DEVICE), key[:, begin:end].to(DEVICE),
                            payload[:, begin:end].to(DEVICE))
                        outputs.append(output)
                        positions.append(ends)
            finally:
                cabi.set_forward_index(None)
            results[mode] = (torch.cat(outputs, dim=1).cpu(), torch.cat(positions, dim=1).cpu())
        for mode in (None, "handed_back"):
            assert torch.equal(results[mode][0], results["scan"][0]), (bits, mode)
            assert torch.equal(results[mode][1], results["scan"][1]), (bits, mode)
        assert int((results["scan"][1] >= 0).sum()) > 0
        if pattern == "random" and bits == 8:
            want = expect_dense(query, key, payload, bits, 8, 40)
            assert torch.equal(results[None][0], want[0]) and torch.equal(results[None][1], want[1])


def test_ragged_long_chunks_route_through_the_index_of_the_keys(rosa):
    heads, payload_heads, bits = 3, 3, 8
    lengths = [[600, 0, 900], [700, 650, 9], [64, 800, 300]]  # per update, per slot
    totals = [sum(step[slot] for step in lengths) for slot in range(3)]
    streams = []
    for slot, total in enumerate(totals):
        query = random_packed((1, total, heads), bits, 80 + slot)
        key = random_packed((1, total, heads), bits, 90 + slot)
        payload = random_packed((1, total, payload_heads), bits, 100 + slot)
        streams.append((query, key, payload, expect_dense(query, key, payload, bits, bits, 33)))
    done = [0, 0, 0]
    with rosa.RosaRuntime(heads, payload_heads, bits, bits, 33) as runtime:
        for step in lengths:
            parts = [[s[i][0, done[slot]:done[slot] + step[slot]] for slot, s in enumerate(streams)]
                     for i in range(3)]
            offsets = [0]
            for length in step:
                offsets.append(offsets[-1] + length)
            output, ends = runtime.update_packed(
                torch.cat(parts[0]).to(DEVICE), torch.cat(parts[1]).to(DEVICE),
                torch.cat(parts[2]).to(DEVICE), cu_seqlens=torch.tensor(offsets, dtype=torch.int32))
            for slot, s in enumerate(streams):
                rows = slice(offsets[slot], offsets[slot + 1])
                want = s[3]
                assert torch.equal(output[rows].cpu(), want[0][0, done[slot]:done[slot] + step[slot]])
                assert torch.equal(ends[rows].cpu(), want[1][0, done[slot]:done[slot] + step[slot]])
                done[slot] += step[slot]


# --------------------------------------------------------------------------- the reference's
# interface tests (tests/test_runtime.py:344-1008) restated for the device runtime

def test_packed_inputs_ignore_bits_above_the_declared_width(rosa):
    generator = torch.Generator().manual_seed(19)
    query = torch.randint(0, 2, (2, 32, 3), dtype=torch.uint8, generator=generator)
    key = torch.randint(0, 2, query.shape, dtype=torch.uint8, generator=generator)
    payload = torch.randint(0, 4, (2, 32, 1), dtype=torch.uint8, generator=generator)
    query_high = torch.randint(0, 128, query.shape, dtype=torch.uint8, generator=generator).mul_(2)
    key_high = torch.randint(0, 128, key.shape, dtype=torch.uint8, generator=generator).mul_(2)
    payload_high = torch.randint(0, 64, payload.shape, dtype=torch.uint8, generator=generator).mul_(4)
    with rosa.RosaRuntime(3, 1, 1, 2, 5) as canonical:
        want = canonical.update_packed(query.to(DEVICE), key.to(DEVICE), payload.to(DEVICE))
    with rosa.RosaRuntime(3, 1, 1, 2, 5) as noisy:
        got = noisy.update_packed((query | query_high).to(DEVICE), (key | key_high).to(DEVICE),
                                  (payload | payload_high).to(DEVICE))
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_grouped_payload_history_is_stored_once_per_payload_head(rosa):
    batch, tokens, heads, payload_heads = 3, 7, 6, 2
    query = random_packed((batch, tokens, heads), 2, 32)
    key = random_packed((batch, tokens, heads), 2, 33)
    payload = random_packed((batch, tokens, payload_heads), 3, 34)
    with rosa.RosaRuntime(heads, payload_heads, 2, 3, 4) as runtime:
        got = runtime.update_packed(query.to(DEVICE), key.to(DEVICE), payload.to(DEVICE))
        stats = runtime.stats()
        detailed = runtime.memory_stats()
    want = expect_dense(query, key, payload, 2, 3, 4)
    assert torch.equal(got[0].cpu(), want[0]) and torch.equal(got[1].cpu(), want[1])
    assert stats[2] == batch * tokens * payload_heads
    assert detailed["payload_symbols"] == stats[2]
    assert detailed["automata"] == batch * heads and detailed["sequences"] == batch


def test_long_chunked_history_preserves_global_successor_positions(rosa):
    # one symbol throughout: every row matches the key before it as far as the horizon reaches,
    # and the latest route wins, so row t answers with the payload at t and the end position t - 1
    chunk_tokens, heads = 16_384, 2
    query = torch.zeros(1, chunk_tokens, heads, dtype=torch.uint8, device=DEVICE)
    key = torch.zeros_like(query)
    payload = (torch.arange(chunk_tokens * 2, dtype=torch.int64).remainder(2).to(torch.uint8)
               .view(1, chunk_tokens * 2, 1).to(DEVICE))
    with rosa.RosaRuntime(heads, 1, qk_bits=1, payload_bits=1, max_suffix_length=32) as runtime:
        first = runtime.update_packed(query, key, payload[:, :chunk_tokens])
        second = runtime.update_packed(query, key, payload[:, chunk_tokens:])
        stats = runtime.memory_stats()
    output = torch.cat((first[0], second[0]), dim=1)
    ends = torch.cat((first[1], second[1]), dim=1)
    want_output = payload.expand(-1, -1, heads).clone()
    want_output[:, 0] = 0
    want_ends = (torch.arange(chunk_tokens * 2, dtype=torch.int64, device=DEVICE) - 1
                 ).view(1, -1, 1).expand(-1, -1, heads)
    assert torch.equal(output, want_output) and torch.equal(ends, want_ends)
    assert stats["payload_symbols"] == chunk_tokens * 2
    assert stats["sequences"] == 1 and stats["automata"] == heads


def test_constructor_names_and_read_only_configuration(rosa):
    import inspect

    parameters = inspect.signature(rosa.RosaRuntime).parameters
    assert tuple(parameters)[:5] == (
        "num_heads", "num_payload_heads", "qk_bits", "payload_bits", "max_suffix_length")
    # (what this runtime adds, the device of its histories, is optional)
    assert all(p.default is not inspect.Parameter.empty for p in list(parameters.values())[5:])
    expected = dict(num_heads=4, num_payload_heads=2, qk_bits=3, payload_bits=5, max_suffix_length=7)
    runtime = rosa.RosaRuntime(**expected)
    try:
        for name, value in expected.items():
            assert getattr(runtime, name) == value
            with pytest.raises(AttributeError):
                setattr(runtime, name, value + 1)
            assert getattr(runtime, name) == value
    finally:
        runtime.close()


def test_closed_runtime_rejects_statistics_and_updates(rosa):
    runtime = rosa.RosaRuntime(1, 1, 1, 1, 1)
    runtime.close()
    runtime.close()
    packed = torch.zeros(1, 1, 1, dtype=torch.uint8, device=DEVICE)
    with pytest.raises(RuntimeError, match="closed"):
        runtime.stats()
    with pytest.raises(RuntimeError, match="closed"):
        runtime.update_packed(packed, packed, packed)


def test_empty_dense_update_and_empty_batches(rosa):
    packed = torch.empty(2, 0, 1, dtype=torch.uint8, device=DEVICE)
    with rosa.RosaRuntime(1, 1, 1, 1, 3) as runtime:
        output, ends = runtime.update_packed(packed, packed, packed)
        assert runtime.stats()[2] == 0
    assert output.shape == (2, 0, 1) and ends.shape == (2, 0, 1)
    none = torch.empty(0, 3, 1, dtype=torch.uint8, device=DEVICE)
    varlen = torch.empty(0, 1, dtype=torch.uint8, device=DEVICE)
    with rosa.RosaRuntime(1, 1, 1, 1, 2) as runtime:
        with pytest.raises(ValueError, match="batch"):
            runtime.update_packed(none, none, none)
        with pytest.raises(ValueError, match="at least one sequence"):
            runtime.update_packed(varlen, varlen, varlen, cu_seqlens=torch.tensor([0]))


@pytest.mark.parametrize("name,args", [
    ("num_heads", (1.5,)),
    ("qk_bits", (1, None, True)),
    ("max_suffix_length", (1, None, 1, 1, False)),
])
def test_constructor_rejects_values_that_are_not_integers(rosa, name, args):
    with pytest.raises(TypeError, match=name):
        rosa.RosaRuntime(*args)


@pytest.mark.parametrize("qk_bits,payload_bits", [(0, 1), (9, 1), (1, 0), (1, 9)])
def test_symbol_widths_are_limited_to_one_through_eight(rosa, qk_bits, payload_bits):
    with pytest.raises(ValueError, match=r"in \[1, 8\]"):
        rosa.RosaRuntime(1, 1, qk_bits, payload_bits, 1)


def test_update_on_a_side_stream_matches_blocking_and_snapshots_its_inputs(rosa):
    query = random_packed((1, 32, 2), 3, 20).to(DEVICE)
    key = random_packed((1, 32, 2), 3, 21).to(DEVICE)
    payload = random_packed((1, 32, 1), 3, 22).to(DEVICE)
    with rosa.RosaRuntime(2, 1, 3, 3, 4) as blocking:
        want = blocking.update_packed(query, key, payload)
    stream = torch.cuda.Stream()
    with rosa.RosaRuntime(2, 1, 3, 3, 4) as asynchronous:
        work = asynchronous.update_packed(query, key, payload, stream=stream, async_op=True)
        # the caller may reuse its tensors as soon as the call returns
        query.fill_(7)
        key.zero_()
        payload.fill_(6)
        got = work.wait()
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_router_update_with_an_understated_longest_total_falls_back_to_the_scan(rosa):
    # the C ABI takes the longest history + chunk length from the caller; a run that is longer
    # than stated has no room in the index and must be routed by the scan, not out of bounds
    import ctypes

    from rosa_soft_amd import cabi

    tokens, capacity = 600, 1024
    query = random_packed((tokens, 1), 8, 5).to(DEVICE)
    key = random_packed((tokens, 1), 8, 6).to(DEVICE)
    key[300:500] = key[20:220]
    query[301:500] = key[300:499]
    payload = random_packed((tokens, 1), 8, 7).to(DEVICE)

    def run(longest_total, mode):
        lengths = torch.zeros(1, dtype=torch.int32, device=DEVICE)
        histories = [torch.zeros(1, 1, capacity, dtype=torch.uint8, device=DEVICE) for _ in range(3)]
        output = torch.empty(tokens, 1, dtype=torch.uint8, device=DEVICE)
        ends = torch.empty(tokens, 1, dtype=torch.int64, device=DEVICE)
        update = cabi.RosaRouterUpdate(
            S=1, H=1, Hp=1, W=64, qk_bits=8, payload_bits=8, capacity=capacity, tokens=tokens,
            longest_chunk=tokens, uniform_chunk=tokens, longest_total=longest_total)
        update.history_lengths = lengths.data_ptr()
        update.query_history, update.key_history, update.payload_history = (
            h.data_ptr() for h in histories)
        update.query, update.key, update.payload = query.data_ptr(), key.data_ptr(), payload.data_ptr()
        update.output, update.matched_key_end = output.data_ptr(), ends.data_ptr()
        cabi.set_forward_index(mode)
        try:
            workspace = cabi.router_update(update, torch.device(DEVICE))
        finally:
            cabi.set_forward_index(None)
        torch.cuda.synchronize()
        return output, ends, workspace

    want_output, want_ends, _ = run(tokens, "scan")
    assert int((want_ends >= 0).sum()) > 200
    for stated in (tokens, 512):
        output, ends, workspace = run(stated, None)
        assert workspace is not None
        assert torch.equal(output, want_output) and torch.equal(ends, want_ends), stated


def test_loaded_state_is_reduced_to_the_declared_symbol_widths(rosa):
    # a state dictionary with bits above the widths (written by hand, or damaged) must behave
    # like the same state without them: long chunks then go through the index of the keys,
    # which buckets stored symbols by their value
    heads, bits, horizon, tokens = 2, 6, 9, 700
    query = random_packed((1, 2 * tokens, heads), bits, 41)
    key = random_packed((1, 2 * tokens, heads), bits, 42)
    payload = random_packed((1, 2 * tokens, 1), bits, 43)
    want = expect_dense(query, key, payload, bits, bits, horizon)
    with rosa.RosaRuntime(heads, 1, bits, bits, horizon) as first:
        first.update_packed(query[:, :tokens].to(DEVICE), key[:, :tokens].to(DEVICE),
                            payload[:, :tokens].to(DEVICE))
        saved = first.state_dict()
    for name in ("query_history", "key_history", "payload_history"):
        saved[name] = saved[name] | 0xC0
    with rosa.RosaRuntime(heads, 1, bits, bits, horizon) as second:
        second.load_state_dict(saved)
        output, ends = second.update_packed(query[:, tokens:].to(DEVICE), key[:, tokens:].to(DEVICE),
                                            payload[:, tokens:].to(DEVICE))
    assert torch.equal(ends.cpu(), want[1][:, tokens:])
    assert torch.equal(output.cpu(), want[0][:, tokens:])


def test_decoding_steps_in_place_and_through_the_single_launch_agree(rosa):
    # the C ABI advances `history_lengths` in place unless `history_lengths_out` is given; the
    # runtime gives it (a decoding step is then one launch).  Both against the oracle, with
    # chunks of 1, 3 and 8 rows after a prefill, ragged across two slots.
    from rosa_soft_amd import cabi

    heads, payload_heads, bits, horizon, capacity = 4, 2, 3, 6, 256
    steps = [[40, 37], [1, 1], [3, 0], [8, 5], [1, 2]]  # rows per slot, per update
    totals = [sum(step[slot] for step in steps) for slot in range(2)]
    streams = []
    for slot, total in enumerate(totals):
        q = random_packed((1, total, heads), bits, 200 + slot)
        k = random_packed((1, total, heads), bits, 210 + slot)
        p = random_packed((1, total, payload_heads), bits, 220 + slot)
        streams.append((q[0], k[0], p[0], expect_dense(q, k, p, bits, bits, horizon)))

    def updates():
        done = [0, 0]
        for step in steps:
            parts = [torch.cat([s[i][done[slot]:done[slot] + step[slot]] for slot, s in enumerate(streams)])
                     for i in range(3)]
            want_output = torch.cat([s[3][0][0, done[slot]:done[slot] + step[slot]]
                                     for slot, s in enumerate(streams)])
            want_ends = torch.cat([s[3][1][0, done[slot]:done[slot] + step[slot]]
                                   for slot, s in enumerate(streams)])
            offsets = [0, step[0], step[0] + step[1]]
            yield parts, offsets, want_output, want_ends
            done = [done[slot] + step[slot] for slot in range(2)]

    # in place, straight through the C ABI
    lengths = torch.zeros(2, dtype=torch.int32, device=DEVICE)
    histories = [torch.zeros(2, n, capacity, dtype=torch.uint8, device=DEVICE)
                 for n in (heads, heads, payload_heads)]
    for (query, key, payload), offsets, want_output, want_ends in updates():
        tokens = offsets[-1]
        query, key, payload = (t.to(DEVICE).contiguous() for t in (query, key, payload))
        table = torch.tensor(offsets, dtype=torch.int32, device=DEVICE)
        output = torch.empty(tokens, heads, dtype=torch.uint8, device=DEVICE)
        ends = torch.empty(tokens, heads, dtype=torch.int64, device=DEVICE)
        update = cabi.RosaRouterUpdate(
            S=2, H=heads, Hp=payload_heads, W=horizon, qk_bits=bits, payload_bits=bits,
            capacity=capacity, tokens=tokens, longest_chunk=max(offsets[1], offsets[2] - offsets[1]),
            uniform_chunk=0, longest_total=capacity)
        update.chunk_offsets = table.data_ptr()
        update.history_lengths = lengths.data_ptr()
        update.query_history, update.key_history, update.payload_history = (
            h.data_ptr() for h in histories)
        update.query, update.key, update.payload = query.data_ptr(), key.data_ptr(), payload.data_ptr()
        update.output, update.matched_key_end = output.data_ptr(), ends.data_ptr()
        cabi.router_update(update, torch.device(DEVICE))
        torch.cuda.synchronize()
        assert torch.equal(output.cpu(), want_output) and torch.equal(ends.cpu(), want_ends)
    assert lengths.tolist() == totals
    # the runtime: lengths to the other array, decoding steps in one launch
    with rosa.RosaRuntime(heads, payload_heads, bits, bits, horizon) as runtime:
        for (query, key, payload), offsets, want_output, want_ends in updates():
            output, ends = runtime.update_packed(
                query.to(DEVICE), key.to(DEVICE), payload.to(DEVICE),
                cu_seqlens=torch.tensor(offsets, dtype=torch.int32))
            assert torch.equal(output.cpu(), want_output) and torch.equal(ends.cpu(), want_ends)
        histories_after = (runtime._query_history, runtime._key_history, runtime._payload_history)
        for mine, theirs in zip(histories, histories_after):
            width = min(mine.size(-1), theirs.size(-1), max(totals))
            assert torch.equal(mine[..., :width], theirs[..., :width])
