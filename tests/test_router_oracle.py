"""Pins ``oracle/router_oracle.py`` (CPU only)."""

import itertools

import numpy as np
import torch

from oracle import router_oracle


def test_finite_horizon_example_has_the_hand_derived_answers():
    # reference tests/test_runtime.py:166-217: all-zero queries against keys 0 0 0 1 0 0 and
    # payloads 1..6.  Horizon 1: each row takes the latest earlier zero key.  Horizon 4: rows
    # 4 and 5 prefer the three-long match ending at key 2 over the one-long match at key 4.
    query = np.zeros((1, 6, 1), dtype=np.uint8)
    key = np.array([0, 0, 0, 1, 0, 0], dtype=np.uint8).reshape(1, 6, 1)
    payload = np.arange(1, 7, dtype=np.uint8).reshape(1, 6, 1)
    output, ends = router_oracle.route_dense(query, key, payload, 1, 3, 1)
    assert ends.reshape(-1).tolist() == [-1, 0, 1, 2, 2, 4]
    assert output.reshape(-1).tolist() == [0, 2, 3, 4, 4, 6]
    output, ends = router_oracle.route_dense(query, key, payload, 1, 3, 4)
    assert ends.reshape(-1).tolist() == [-1, 0, 1, 2, 2, 2]
    assert output.reshape(-1).tolist() == [0, 2, 3, 4, 4, 4]


def _diagonal_dp(query, key, horizon):
    """Independent formulation: run(t, e) = q[t]==k[e] ? min(run(t-1, e-1) + 1, W) : 0."""

    tokens = len(query)
    ends = [-1] * tokens
    run = [[0] * tokens for _ in range(tokens)]
    for t in range(tokens):
        best = 0
        for e in range(t):
            if query[t] == key[e]:
                previous = run[t - 1][e - 1] if (t > 0 and e > 0) else 0
                run[t][e] = min(previous + 1, horizon)
            if run[t][e] > 0 and run[t][e] >= best:
                best, ends[t] = run[t][e], e
    return ends


def test_all_binary_strings_of_length_four_agree_with_the_diagonal_recurrence():
    # the state space of reference tests/test_runtime.py:138-163
    for horizon in (1, 2, 4):
        for q_bits, k_bits in itertools.product(range(16), repeat=2):
            query = np.array([(q_bits >> i) & 1 for i in range(4)], dtype=np.uint8)
            key = np.array([(k_bits >> i) & 1 for i in range(4)], dtype=np.uint8)
            payload = np.arange(4, dtype=np.uint8)
            _, ends = router_oracle.route_slot(
                query.reshape(4, 1), key.reshape(4, 1), payload.reshape(4, 1), horizon, 1
            )
            assert ends.reshape(-1).tolist() == _diagonal_dp(query, key, horizon)


def test_masks_groups_and_chunking():
    rng = np.random.default_rng(5)
    query = rng.integers(0, 256, (2, 17, 4), dtype=np.uint8)
    key = rng.integers(0, 256, (2, 17, 4), dtype=np.uint8)
    payload = rng.integers(0, 256, (2, 17, 2), dtype=np.uint8)
    output, ends = router_oracle.route_dense(query, key, payload, 2, 3, 5)
    # only the masked bits take part
    again, ends_again = router_oracle.route_dense(query & 3, key & 3, payload & 7, 2, 3, 5)
    assert np.array_equal(output, again) and np.array_equal(ends, ends_again)
    assert output.max() <= 7
    # chunked updates equal the one-shot call (reference tests/test_runtime.py:266-316)
    router = router_oracle.StreamingRouter(4, 2, 2, 3, 5)
    pieces = []
    for begin, end in ((0, 3), (3, 4), (4, 11), (11, 17)):
        flat = lambda x: x[:, begin:end].reshape(-1, x.shape[2])
        width = end - begin
        pieces.append(router.update_packed(flat(query), flat(key), flat(payload), [0, width, 2 * width]))
    chunked = np.concatenate([p[1].reshape(2, -1, 4) for p in pieces], axis=1)
    assert np.array_equal(chunked, ends)


def test_router_equals_the_training_hard_forward(c_oracle):
    # reference tests/test_runtime.py:190-217: symbols from sign bits, payload bits as +-1
    rng = np.random.default_rng(11)
    tokens, heads, bits, value_bits, horizon = 40, 2, 2, 3, 6
    query = rng.integers(0, 1 << bits, (1, tokens, heads), dtype=np.uint8)
    key = rng.integers(0, 1 << bits, (1, tokens, heads), dtype=np.uint8)
    payload = rng.integers(0, 1 << value_bits, (1, tokens, 1), dtype=np.uint8)
    output, ends = router_oracle.route_dense(query, key, payload, bits, value_bits, horizon)

    def logits(symbols, width):
        planes = [((symbols >> i) & 1).astype(np.float32) * 2 - 1 for i in range(width)]
        return torch.from_numpy(np.stack(planes, axis=-1))

    hard, routes, _ = c_oracle.hard_forward(
        logits(query, bits), logits(key, bits), logits(payload, value_bits), horizon
    )
    assert np.array_equal(routes.permute(0, 2, 1).numpy() - 1, ends)
    unpacked = logits(output, value_bits)
    unpacked[torch.from_numpy(ends < 0)] = 0.0
    assert torch.equal(unpacked, hard)


def test_oracle_equals_the_reference_runtime_built_from_source():
    # oracle/_ref/librosa_runtime_ref.so is the reference's rosa_runtime.cpp compiled as is
    import pytest

    native = router_oracle.reference_runtime()
    if native is None:
        pytest.skip("oracle/_ref is not built (make -C oracle ref)")
    rng = np.random.default_rng(3)
    for heads, payload_heads, qk_bits, payload_bits, horizon, lengths in (
        (4, 2, 4, 4, 5, [19, 19]),
        (6, 3, 3, 3, 4, [4, 9, 0, 6]),
        (2, 1, 1, 8, 64, [130]),
        (1, 1, 8, 1, 1, [40, 1]),
    ):
        total = sum(lengths)
        offsets = [0] + list(np.cumsum(lengths))
        query = rng.integers(0, 256, (total, heads), dtype=np.uint8)
        key = rng.integers(0, 256, (total, heads), dtype=np.uint8)
        payload = rng.integers(0, 256, (total, payload_heads), dtype=np.uint8)
        mine = router_oracle.StreamingRouter(heads, payload_heads, qk_bits, payload_bits, horizon)
        theirs = native(heads, payload_heads, qk_bits, payload_bits, horizon)
        # two updates: the second continues every slot's history
        for part in range(2):
            want = theirs.update_packed(torch.tensor(offsets, dtype=torch.int64),
                                        torch.from_numpy(query), torch.from_numpy(key),
                                        torch.from_numpy(payload))
            got = mine.update_packed(query, key, payload, offsets)
            assert np.array_equal(got[0], want[0].numpy()), (heads, horizon, part)
            assert np.array_equal(got[1], want[1].numpy()), (heads, horizon, part)
            query, key, payload = key.copy(), query.copy(), payload[::-1].copy()
