"""The benchmark configurations at their full sizes on a real MI355X.

The whole problem runs on the device; the CPU oracle then checks a slice that
it can finish in seconds.  (batch, value-head group) units are independent, so
a slice with the right dropout coordinates reproduces the full problem's
numbers for that unit.  Size-independent properties are checked on everything.
"""

import pytest
import torch

import bench

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"


@pytest.fixture(scope="module")
def cabi():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from rosa_soft_amd import cabi as module

    module.load()
    return module


def close(got, want, label):
    got = got.detach().cpu().double()
    assert torch.isfinite(got).all(), label
    tolerance = 1e-4 * want.abs() + 1e-5 * want.abs().max()
    excess = ((got - want).abs() - tolerance).max().item()
    assert excess <= 0.0, f"{label}: exceeds tolerance by {excess:.3e} (max|want| {want.abs().max():.3e})"


def run_full(cabi, name, seed):
    config, query, key, value, cu = bench.make_workload(name, DEVICE)
    generator = torch.Generator().manual_seed(99)
    out_shape = (*query.shape[:-1], config["Dv"])
    grad_output = torch.randn(out_shape, generator=generator).to(query.dtype).to(DEVICE)
    out, pq, pk, routes = cabi.hard_forward(query, key, value, config["W"], cu)
    seed_tensor = torch.tensor(seed, dtype=torch.int64, device=DEVICE) if config["p"] > 0 else None
    grads = cabi.surrogate_vjp(
        query, key, value, grad_output, pq, pk, seed_tensor, config["W"], 1.0, config["p"],
        config["ms"], 7, cu,
    )
    torch.cuda.synchronize()
    return config, (query, key, value, grad_output, cu), out, routes, grads


def check_properties(config, tensors, out, grads):
    query, key, value, grad_output, cu = tensors
    assert set(out.float().unique().tolist()) <= {-1.0, 0.0, 1.0}
    for g in grads:
        assert torch.isfinite(g).all()
    if cu is None:
        assert torch.count_nonzero(out[:, 0]) == 0        # row 0 has only the null route
        assert torch.count_nonzero(grads[0][:, 0]) == 0   # no suffix reaches query row 0
        assert torch.count_nonzero(grads[1][:, -1]) == 0  # the last key is never compared
        assert torch.count_nonzero(grads[2][:, 0]) == 0   # value 0 is never a candidate
    else:
        offsets = cu.tolist()
        for start, end in zip(offsets[:-1], offsets[1:]):
            if end > start:
                assert torch.count_nonzero(out[start]) == 0
                assert torch.count_nonzero(grads[0][start]) == 0
                assert torch.count_nonzero(grads[1][end - 1]) == 0
                assert torch.count_nonzero(grads[2][start]) == 0


def dense_slice_check(c_oracle, config, tensors, out, routes, grads, batch, value_head, seed):
    query, key, value, grad_output, _ = (t.cpu() if t is not None else None for t in tensors)
    group = config["H"] // config["Hv"]
    heads = slice(value_head * group, (value_head + 1) * group)
    q = query[batch:batch + 1, :, heads]
    k = key[batch:batch + 1, :, heads]
    v = value[batch:batch + 1, :, value_head:value_head + 1]
    go = grad_output[batch:batch + 1, :, heads]
    want_out, want_routes, _ = c_oracle.hard_forward(q, k, v, config["W"])
    assert torch.equal(out[batch:batch + 1, :, heads].cpu().float(), want_out.float())
    assert torch.equal(routes[batch:batch + 1, heads].cpu(), want_routes)
    want = c_oracle.surrogate_vjp(
        q, k, v, go, max_suffix_length=config["W"], dropout_p=config["p"],
        mismatch_scale=config["ms"], seed=seed if config["p"] > 0 else None,
        batch_ids=[batch], head_offset=value_head * group,
    )
    close(grads[0][batch:batch + 1, :, heads], want[0], "grad_query")
    close(grads[1][batch:batch + 1, :, heads], want[1], "grad_key")
    close(grads[2][batch:batch + 1, :, value_head:value_head + 1], want[2], "grad_value")


def test_config1_whole_problem(cabi, c_oracle):
    seed = 11
    config, tensors, out, routes, grads = run_full(cabi, "config1", seed)
    check_properties(config, tensors, out, grads)
    query, key, value, grad_output, _ = (t.cpu() if t is not None else None for t in tensors)
    want_out, want_routes, _ = c_oracle.hard_forward(query, key, value, config["W"])
    assert torch.equal(out.cpu(), want_out) and torch.equal(routes.cpu(), want_routes)
    want = c_oracle.surrogate_vjp(query, key, value, grad_output, max_suffix_length=config["W"])
    for got, expected, label in zip(grads, want, ("gq", "gk", "gv")):
        close(got, expected, label)


@pytest.mark.parametrize(
    "name,batch,value_head",
    [("config2", 1, 5), ("metric", 0, 3), ("config3", 2, 7), ("config4", 0, 3)],
)
def test_dense_configs_full_size(cabi, c_oracle, name, batch, value_head):
    seed = 0x1234ABCD5678EF01
    config, tensors, out, routes, grads = run_full(cabi, name, seed)
    check_properties(config, tensors, out, grads)
    dense_slice_check(c_oracle, config, tensors, out, routes, grads, batch, value_head, seed)
    if name == "config4":
        # the motif makes long matches the rule: most rows route somewhere
        assert float((routes > 0).float().mean()) > 0.9


def test_packed_config5_full_size(cabi, c_oracle):
    seed = 0x0FEDCBA987654321
    config, tensors, out, routes, grads = run_full(cabi, "config5", seed)
    check_properties(config, tensors, out, grads)
    query, key, value, grad_output, cu = (t.cpu() for t in tensors)
    offsets = cu.tolist()
    group = config["H"] // config["Hv"]
    # sequences 0 (1024 tokens) and 4 (512 tokens), and the longest one, 5 (8192 tokens: the
    # long bands, two symbol tiles, dropout), each with all heads of one value group
    for sequence, value_head in ((0, 2), (4, 2), (5, 6)):
        heads = slice(value_head * group, (value_head + 1) * group)
        start, end = offsets[sequence], offsets[sequence + 1]
        q = query[start:end, heads].unsqueeze(0)
        k = key[start:end, heads].unsqueeze(0)
        v = value[start:end, value_head:value_head + 1].unsqueeze(0)
        go = grad_output[start:end, heads].unsqueeze(0)
        want_out, want_routes, _ = c_oracle.hard_forward(q, k, v, config["W"])
        assert torch.equal(out[start:end, heads].cpu().float(), want_out[0].float())
        assert torch.equal(routes[heads, start:end].cpu(), want_routes[0])
        want = c_oracle.surrogate_vjp(
            q, k, v, go, max_suffix_length=config["W"], dropout_p=config["p"],
            mismatch_scale=config["ms"], seed=seed, batch_ids=[sequence],
            head_offset=value_head * group,
        )
        close(grads[0][start:end, heads], want[0][0], "grad_query")
        close(grads[1][start:end, heads], want[1][0], "grad_key")
        close(grads[2][start:end, value_head:value_head + 1], want[2][0], "grad_value")
    # forward routes of the second longest sequence for one head
    start, end = offsets[1], offsets[2]
    want_out, want_routes, _ = c_oracle.hard_forward(
        query[start:end, 17:18].unsqueeze(0), key[start:end, 17:18].unsqueeze(0),
        value[start:end, 2:3].unsqueeze(0), config["W"],
    )
    assert torch.equal(routes[17:18, start:end].cpu(), want_routes[0])


def test_one_long_sequence_three_ways(cabi):
    """One sequence of 32 768 tokens (four heads): few, long bands, the shape for which the
    gradient kernel cuts bands into pieces.  No oracle finishes this size; the three ways the
    kernel can get its state must agree with each other instead: chunk records with pieces
    (the default here), chunk records with whole bands, and no records at all (forward sweeps
    from two levels of checkpoints).  Accumulation order differs, so the comparison is to the
    bar of the parity tests, widened by two for two device results."""

    T, H, D, Hv, Dv, W = 32768, 4, 8, 2, 8, 64
    generator = torch.Generator(device=DEVICE).manual_seed(2024)
    query = torch.randn(1, T, H, D, device=DEVICE, generator=generator)
    key = torch.randn(1, T, H, D, device=DEVICE, generator=generator)
    key[:, 5000:5400] = query[:, 4000:4400]  # a long exact match in the middle
    value = torch.randn(1, T, Hv, Dv, device=DEVICE, generator=generator)
    grad_output = torch.randn(1, T, H, Dv, device=DEVICE, generator=generator)
    seed = torch.tensor(77, dtype=torch.int64, device=DEVICE)
    out, packed_q, packed_k, routes = cabi.hard_forward(query, key, value, W)
    plan = cabi.gradient_block_plan(query, value, W)
    assert plan["pieces"] > 1

    def backward():
        grads = cabi.surrogate_vjp(query, key, value, grad_output, packed_q, packed_k, seed, W,
                                   1.0, 0.1, 3.0, 7)
        torch.cuda.synchronize()
        return grads

    try:
        pieces = backward()
        cabi.set_gradient_piece_rows(-1)
        whole = backward()
        cabi.set_gradient_piece_rows(None)
        cabi.set_record_budget(0)
        swept = backward()
    finally:
        cabi.set_gradient_piece_rows(None)
        cabi.set_record_budget(None)
    assert int((routes > 0).sum()) > T  # matches were found
    for name, a, b, c in zip(("grad_query", "grad_key", "grad_value"), pieces, whole, swept):
        assert torch.isfinite(a).all() and float(a.abs().max()) > 0, name
        for other, label in ((b, "whole bands"), (c, "no records")):
            tolerance = 2e-4 * a.abs() + 2e-5 * a.abs().max()
            excess = float(((a - other).abs() - tolerance).max())
            assert excess <= 0.0, f"{name} against {label}: exceeds tolerance by {excess:.3e}"
    # structural zeros: first query row, last key row, first value row
    assert torch.count_nonzero(pieces[0][:, 0]) == 0
    assert torch.count_nonzero(pieces[1][:, -1]) == 0
    assert torch.count_nonzero(pieces[2][:, 0]) == 0


def test_stage_totals_cover_a_loop_of_calls_without_a_wait_per_call(cabi):
    device = torch.device("cuda:0")
    generator = torch.Generator(device=device).manual_seed(9)
    query = torch.randn(1, 256, 4, 8, device=device, generator=generator)
    key = torch.randn(1, 256, 4, 8, device=device, generator=generator)
    value = torch.randn(1, 256, 2, 8, device=device, generator=generator)
    cabi.stage_timing(True)
    try:
        for _ in range(3):
            cabi.hard_forward(query, key, value, 16)
        totals = cabi.stage_totals()
        assert set(totals) == {"hard_forward"}
        milliseconds, runs = totals["hard_forward"]
        assert runs == 3 and milliseconds > 0.0
        last = cabi.stage_times()
        assert last == {}  # reading the totals started a new sum
        for _ in range(70):  # more runs than the library keeps events for
            cabi.hard_forward(query, key, value, 16)
        assert cabi.stage_times()["hard_forward"] > 0.0
        milliseconds, runs = cabi.stage_totals()["hard_forward"]
        assert runs == 64 and milliseconds > 0.0
        assert cabi.stage_totals() == {}
    finally:
        cabi.stage_timing(False)
