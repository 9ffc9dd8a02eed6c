"""Parity of the HIP path against the CPU oracle (needs a real MI355X).

The kernels are driven through the C ABI (``rosa_soft_amd.cabi``); the last
section goes through the public operators and the dispatcher.  Bars:

* hard forward, packed symbols and route indices: bit-exact;
* gradients: ``|got - want| <= 1e-4 * |want| + 1e-5 * max|want|`` against the
  float64 streamed oracle for every input dtype at the C-ABI level (the
  kernels compute in float32 whatever the input type), and the reference's own
  half-precision bars ``(3e-3, 3e-3)`` / ``(2e-2, 2e-2)`` after the public
  operator has cast gradients to float16 / bfloat16.
"""

import ctypes

import numpy as np
import pytest
import torch

from tests.conftest import nonzero_randn

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"


@pytest.fixture(scope="module")
def cabi():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from rosa_soft_amd import cabi as module

    module.load()
    return module


@pytest.fixture(params=[None, 2], ids=["waves_by_shape", "two_wave_blocks"])
def block_waves(request, cabi):
    """Both forms of the gradient kernel: the library's choice (one wave per block at these
    sizes) and blocks of two waves that own neighbouring bands and exchange tiles in LDS."""

    cabi.set_gradient_block_waves(request.param)
    yield request.param
    cabi.set_gradient_block_waves(None)


def assert_gradients_close(got, want, label="", slack=1.0):
    got = got.detach().cpu().double()
    want = want.double()
    assert torch.isfinite(got).all(), label
    tolerance = slack * (1e-4 * want.abs() + 1e-5 * want.abs().max())
    excess = ((got - want).abs() - tolerance).max().item()
    assert excess <= 0.0, f"{label}: exceeds tolerance by {excess:.3e} (max|want| {want.abs().max():.3e})"


def make_case(B, T, H, D, Hv, Dv, dtype=torch.float32, seed=0, pattern="random"):
    query = nonzero_randn((B, T, H, D), seed=seed + 1).to(dtype)
    key = nonzero_randn((B, T, H, D), seed=seed + 2).to(dtype)
    value = nonzero_randn((B, T, Hv, Dv), seed=seed + 3).to(dtype)
    grad_output = nonzero_randn((B, T, H, Dv), seed=seed + 4, floor=0.0).to(dtype)
    if pattern == "shifted":  # long near-exact matches along one diagonal
        key = query.roll(3, dims=1).clone()
        key[:, ::7] = -key[:, ::7]
    elif pattern == "all_match":
        query = torch.ones_like(query)
        key = torch.ones_like(key)
    elif pattern == "periodic":
        period = nonzero_randn((B, 5, H, D), seed=seed + 9).to(dtype)
        reps = (T + 4) // 5
        key = period.repeat(1, reps, 1, 1)[:, :T].clone()
        query = key.clone()
    return query, key, value, grad_output


def run_device(cabi, query, key, value, grad_output, W, scale=1.0, p=0.0, ms=3.0, seed=None,
               mask=7, cu_seqlens=None):
    q, k, v, go = (t.to(DEVICE).contiguous() for t in (query, key, value, grad_output))
    offsets = None if cu_seqlens is None else torch.tensor(cu_seqlens, dtype=torch.int32, device=DEVICE)
    out, pq, pk, routes = cabi.hard_forward(q, k, v, W, offsets)
    seed_tensor = None if seed is None else torch.tensor(seed, dtype=torch.int64, device=DEVICE)
    grads = cabi.surrogate_vjp(q, k, v, go, pq, pk, seed_tensor, W, scale, p, ms, mask, offsets)
    torch.cuda.synchronize()
    return out, pq, pk, routes, grads


# --------------------------------------------------------------------------- forward

FORWARD_CASES = [
    # B, T, H, D, Hv, Dv, W, dtype, pattern
    (1, 1, 1, 1, 1, 1, 1, torch.float32, "random"),
    (2, 33, 2, 4, 1, 5, 8, torch.float32, "random"),
    (1, 64, 2, 2, 2, 3, 64, torch.float32, "random"),
    (1, 65, 1, 1, 1, 7, 1000, torch.float16, "random"),
    (2, 257, 4, 3, 2, 12, 16, torch.bfloat16, "random"),
    (1, 200, 2, 5, 1, 9, 31, torch.float32, "shifted"),
    (1, 300, 2, 32, 2, 4, 40, torch.float32, "shifted"),
    (1, 193, 1, 8, 1, 8, 128, torch.float32, "all_match"),
    (1, 150, 2, 7, 1, 70, 9, torch.float16, "periodic"),
    (1, 700, 3, 2, 3, 33, 64, torch.bfloat16, "random"),
]


@pytest.mark.parametrize("B,T,H,D,Hv,Dv,W,dtype,pattern", FORWARD_CASES)
def test_hard_forward_is_bit_exact(cabi, c_oracle, B, T, H, D, Hv, Dv, W, dtype, pattern):
    query, key, value, _ = make_case(B, T, H, D, Hv, Dv, dtype, seed=T, pattern=pattern)
    q, k, v = (t.to(DEVICE) for t in (query, key, value))
    out, pq, pk, routes = cabi.hard_forward(q, k, v, W)
    torch.cuda.synchronize()
    want_out, want_routes, _ = c_oracle.hard_forward(query, key, value, W)
    assert out.dtype == dtype and out.shape == (B, T, H, Dv)
    assert torch.equal(out.cpu().float(), want_out.float())
    assert torch.equal(routes.cpu(), want_routes)
    # packed symbols: bit i = x[..., i] > 0, head-major [B, H, T] (reference
    # tests/test_soft_cuda.py:80-98)
    weights = 1 << torch.arange(D, dtype=torch.int64)
    want_pq = ((query > 0).long() * weights).sum(-1).permute(0, 2, 1)
    want_pk = ((key > 0).long() * weights).sum(-1).permute(0, 2, 1)
    assert pq.shape == (B, H, T) and pq.stride() == (H * T, T, 1) and pq.dtype == torch.int32
    assert torch.equal(pq.cpu().long() & 0xFFFFFFFF, want_pq)
    assert torch.equal(pk.cpu().long() & 0xFFFFFFFF, want_pk)
    assert set(out.cpu().float().unique().tolist()) <= {-1.0, 0.0, 1.0}


def test_sign_policy_for_zero_and_non_finite_inputs(cabi, c_oracle):
    # zeros, -0, NaN and -inf quantise to -1, +inf to +1 (reference
    # docs/CONCEPT.md:27-33, tests/test_soft_cuda.py:570-611)
    query = nonzero_randn((1, 40, 1, 4), seed=1)
    key = query.roll(1, dims=1).clone()
    specials = torch.tensor([0.0, -0.0, float("nan"), float("-inf"), float("inf")])
    query[0, 5:10, 0, 0] = specials
    key[0, 6:11, 0, 1] = specials
    value = nonzero_randn((1, 40, 1, 3), seed=2)
    value[0, 7, 0] = torch.tensor([0.0, float("nan"), float("inf")])
    out, _, _, routes = cabi.hard_forward(query.to(DEVICE), key.to(DEVICE), value.to(DEVICE), 8)
    want_out, want_routes, _ = c_oracle.hard_forward(query, key, value, 8)
    assert torch.equal(out.cpu(), want_out) and torch.equal(routes.cpu(), want_routes)


# --------------------------------------------------------------------------- gradients

VJP_CASES = [
    # B, T, H, D, Hv, Dv, W, scale, p, ms, dtype, pattern
    (1, 33, 2, 16, 1, 5, 16, 1.0, 0.0, 3.0, torch.float32, "random"),
    (2, 130, 4, 8, 2, 8, 16, 1.0, 0.0, 3.0, torch.float32, "random"),
    (1, 257, 2, 3, 2, 12, 300, 1.3, 0.0, 2.0, torch.float32, "random"),
    (1, 160, 1, 1, 1, 4, 160, 1.0, 0.0, 3.0, torch.float32, "random"),
    (2, 200, 4, 8, 2, 8, 16, 1.0, 0.25, 3.0, torch.float32, "random"),
    (1, 96, 2, 4, 1, 6, 12, 0.25, 0.9, 1.0, torch.float32, "random"),
    (1, 700, 2, 2, 1, 40, 64, 1.0, 0.0, 3.0, torch.float32, "shifted"),
    (1, 300, 2, 1, 1, 4, 300, 1.0, 0.0, 3.0, torch.float32, "shifted"),
    (1, 600, 1, 8, 1, 8, 128, 1.0, 0.0, 3.0, torch.float32, "all_match"),
    (1, 260, 2, 6, 2, 17, 40, 0.7, 0.1, 9.0, torch.float32, "periodic"),
    (1, 160, 1, 16, 1, 33, 32, 4.0, 0.1, 9.0, torch.bfloat16, "random"),
    (2, 140, 2, 32, 2, 64, 24, 1.0, 0.0, 3.0, torch.float16, "shifted"),
    (1, 1200, 2, 8, 1, 8, 128, 1.0, 0.1, 3.0, torch.float32, "random"),
    (1, 180, 2, 8, 2, 8, 32, 10.0, 0.0, 3.0, torch.float32, "shifted"),   # row-maximum pass
    (1, 120, 1, 4, 1, 4, 8, 30.0, 0.2, 0.5, torch.float32, "periodic"),  # row-maximum pass
    (1, 90, 2, 4, 1, 70, 12, 1.0, 0.1, 3.0, torch.float32, "random"),    # two value slices
    (1, 70, 2, 3, 2, 130, 8, 1.0, 0.0, 3.0, torch.bfloat16, "shifted"),  # three value slices
    # second symbol tile 4 bits wide, second value tile 8 wide: both flushed on all lanes
    (1, 150, 2, 20, 1, 24, 20, 1.0, 0.1, 3.0, torch.float32, "random"),
    (2, 97, 2, 24, 2, 20, 12, 1.0, 0.0, 3.0, torch.float32, "shifted"),
]


def test_hard_forward_beyond_65535_rows_uses_the_64_bit_key(cabi, c_oracle):
    # sequences of 65536 rows and more no longer fit (run, route) into 32 bits: the scan
    # switches to a 64-bit key and the maximum; narrow symbols give long runs and many ties
    T, W = 66000, 40
    query = nonzero_randn((1, T, 1, 2), seed=1)
    key = nonzero_randn((1, T, 1, 2), seed=2)
    value = nonzero_randn((1, T, 1, 3), seed=3)
    out, _, _, routes = cabi.hard_forward(*(t.to(DEVICE) for t in (query, key, value)), W)
    torch.cuda.synchronize()
    want_out, want_routes, _ = c_oracle.hard_forward(query, key, value, W)
    assert int(want_routes.max()) > 65535
    assert torch.equal(routes.cpu(), want_routes)
    assert torch.equal(out.cpu(), want_out)


@pytest.mark.parametrize("B,T,H,D,Hv,Dv,W,scale,p,ms,dtype,pattern", VJP_CASES)
def test_surrogate_vjp_matches_oracle(cabi, c_oracle, block_waves, B, T, H, D, Hv, Dv, W, scale,
                                      p, ms, dtype, pattern):
    query, key, value, grad_output = make_case(B, T, H, D, Hv, Dv, dtype, seed=7 * T + D, pattern=pattern)
    seed = 0x5DEECE66D1234567 if p > 0 else None
    out, _, _, _, grads = run_device(cabi, query, key, value, grad_output, W, scale, p, ms, seed)
    want = c_oracle.surrogate_vjp(
        query, key, value, grad_output, max_suffix_length=W, scale=scale, dropout_p=p,
        mismatch_scale=ms, seed=seed,
    )
    # A float32 logit of magnitude L = scale * U(W) reaches the exponent through three
    # roundings of relative size 2^-24 (the square root, its product with the gain, the
    # row's exponent shift of the same magnitude), i.e. up to ~2e-7 * L, and the softmax
    # Jacobian multiplies that by `scale` once more, so gradients move by up to
    # ~2e-7 * scale * L relative to their own scale (the float32 reference kernels share
    # this limit).  The bar 1e-5 * max|want| widens accordingly, to 2.5e-7 * scale * L.
    longest_logit = scale * 2.4142 * ((1.0 + min(W, T)) ** 0.5 - 1.0)
    slack = max(1.0, scale * longest_logit / 40.0)
    for name, got, expected in zip(("grad_query", "grad_key", "grad_value"), grads, want):
        assert got.dtype == torch.float32 and got.shape == expected.shape
        assert_gradients_close(got, expected, name, slack)
    # structural zeros (first query row, last key row, first value row)
    assert torch.count_nonzero(grads[0][:, 0]) == 0
    assert torch.count_nonzero(grads[1][:, -1]) == 0
    assert torch.count_nonzero(grads[2][:, 0]) == 0


@pytest.mark.parametrize("mask", range(1, 8))
def test_gradient_masks(cabi, c_oracle, block_waves, mask):
    # reference tests/test_soft_cuda.py:510-567
    query, key, value, grad_output = make_case(1, 70, 2, 5, 1, 6, seed=mask)
    seed = 4242 + mask
    _, _, _, _, grads = run_device(cabi, query, key, value, grad_output, 9, 1.0, 0.3, 3.0, seed, mask)
    want = c_oracle.surrogate_vjp(
        query, key, value, grad_output, max_suffix_length=9, dropout_p=0.3, seed=seed
    )
    for bit, got, expected in zip((1, 2, 4), grads, want):
        if mask & bit:
            assert_gradients_close(got, expected)
        else:
            assert got is None


def test_dropout_seed_halves_and_replay(cabi):
    query, key, value, grad_output = make_case(1, 90, 2, 4, 2, 4, seed=3)
    low = run_device(cabi, query, key, value, grad_output, 8, p=0.5, seed=7)[4]
    again = run_device(cabi, query, key, value, grad_output, 8, p=0.5, seed=7)[4]
    high = run_device(cabi, query, key, value, grad_output, 8, p=0.5, seed=(1 << 32) + 7)[4]
    for a, b in zip(low, again):  # accumulation order is free: compare to tolerance
        torch.testing.assert_close(a, b, rtol=2e-6, atol=2e-7)
    assert any(not torch.allclose(a, b) for a, b in zip(low, high))


def test_every_causal_value_is_credited_and_singleton_is_zero(cabi):
    # reference tests/test_soft_cuda.py:693-713, tests/test_soft_reference.py:436-444
    query = torch.ones(1, 6, 2, 3)
    key = -torch.ones(1, 6, 2, 3)
    value = nonzero_randn((1, 6, 1, 4), seed=50)
    out, _, _, _, grads = run_device(cabi, query, key, value, torch.ones(1, 6, 2, 4), 4)
    assert torch.count_nonzero(out) == 0
    assert torch.all(grads[2][:, 1:].abs().sum(dim=(0, 2, 3)) > 0)
    ones = torch.ones(1, 1, 1, 1)
    out, _, _, _, grads = run_device(cabi, ones, ones, ones, ones, 1)
    assert torch.count_nonzero(out) == 0
    assert all(torch.count_nonzero(g) == 0 for g in grads)


# --------------------------------------------------------------------------- packed layout

PACKED_CASES = [
    # lengths, H, D, Hv, Dv, W, p, dtype
    ([5, 0, 7, 1, 12], 2, 3, 1, 4, 4, 0.3, torch.float32),
    ([1, 2, 127, 0, 128, 129], 2, 4, 2, 5, 160, 0.0, torch.float32),
    ([64, 65, 63], 4, 8, 2, 8, 16, 0.2, torch.bfloat16),
    ([300, 40, 0, 0, 513], 2, 2, 1, 33, 32, 0.1, torch.float16),
    # single-token sequences between longer ones, odd starts: the head-major accumulators of
    # narrow gradient rows (two neighbouring rows per atomic segment, rows stored one slot down)
    ([1, 1, 67, 1, 3, 130], 3, 8, 1, 8, 8, 0.2, torch.float32),
]


@pytest.mark.parametrize("lengths,H,D,Hv,Dv,W,p,dtype", PACKED_CASES)
def test_packed_layout_matches_oracle(cabi, c_oracle, block_waves, lengths, H, D, Hv, Dv, W, p,
                                      dtype):
    # reference tests/test_soft_varlen.py:42-141, :392-475, :860-915
    offsets = [0, *np.cumsum(lengths).tolist()]
    total = offsets[-1]
    query = nonzero_randn((total, H, D), seed=50).to(dtype)
    key = nonzero_randn((total, H, D), seed=51).to(dtype)
    if D <= 2:
        key = query.roll(2, dims=0).clone()
    value = nonzero_randn((total, Hv, Dv), seed=52).to(dtype)
    grad_output = nonzero_randn((total, H, Dv), seed=53, floor=0.0).to(dtype)
    seed = 987654321 if p > 0 else None
    out, pq, pk, routes, grads = run_device(
        cabi, query, key, value, grad_output, W, 1.0, p, 3.0, seed, 7, offsets
    )
    want_out, want_routes = c_oracle.varlen_hard_forward(query, key, value, offsets, W)
    assert out.shape == (total, H, Dv) and pq.shape == (H, total)
    assert torch.equal(out.cpu().float(), want_out.float())
    assert torch.equal(routes.cpu(), want_routes)
    want = c_oracle.varlen_surrogate_vjp(
        query, key, value, offsets, grad_output, max_suffix_length=W, dropout_p=p, seed=seed
    )
    for got, expected in zip(grads, want):
        assert_gradients_close(got, expected)
    for start, end in zip(offsets[:-1], offsets[1:]):
        if end > start:
            assert torch.count_nonzero(grads[2][start]) == 0
            assert torch.count_nonzero(grads[1][end - 1]) == 0
            assert torch.count_nonzero(grads[0][start]) == 0


def test_packed_equals_dense_batch_with_same_seed(cabi):
    # reference tests/test_soft_varlen.py:304-389
    B, T, H, D, Hv, Dv = 3, 70, 2, 4, 1, 5
    query, key, value, grad_output = make_case(B, T, H, D, Hv, Dv, seed=11)
    dense = run_device(cabi, query, key, value, grad_output, 12, p=0.4, seed=99)
    flat = [t.reshape(B * T, *t.shape[2:]) for t in (query, key, value, grad_output)]
    packed = run_device(cabi, *flat, 12, p=0.4, seed=99, cu_seqlens=[0, T, 2 * T, 3 * T])
    assert torch.equal(dense[0].reshape(B * T, H, Dv), packed[0])
    assert torch.equal(dense[3].permute(1, 0, 2).reshape(H, B * T), packed[3])
    for a, b in zip(dense[4], packed[4]):
        torch.testing.assert_close(a.reshape(b.shape), b, rtol=2e-5, atol=2e-6)


def test_invalid_device_offsets_poison_the_results(cabi, c_oracle):
    """Offsets the host cannot see are checked on the device.  Invalid ones touch no token
    (no fault), set the workspace flag and turn every output and gradient element into
    NaN; valid ones leave the results exactly as the oracle has them.  (The reference
    aborts the process: rosa_soft_kernels.cu:287-308, tests/test_soft_varlen.py:181-226.)"""

    total, H, D, Dv = 40, 2, 4, 3
    query = nonzero_randn((total, H, D), seed=1)
    key = nonzero_randn((total, H, D), seed=3)
    value = nonzero_randn((total, 1, Dv), seed=2)
    grad_output = nonzero_randn((total, H, Dv), seed=4, floor=0.0)
    q, k, v, go = (t.to(DEVICE) for t in (query, key, value, grad_output))
    library = cabi.load()
    stream = torch.cuda.current_stream().cuda_stream
    for offsets, bad in (([0, 10, 40], 0), ([0, 30, 20, 40], 1), ([0, 10, 50], 1), ([2, 40], 1),
                         ([0, 10, 39], 1), ([0, -3, 40], 1), ([0, 0, 40, 40], 0)):
        cu = torch.tensor(offsets, dtype=torch.int32, device=DEVICE)
        problem = cabi.make_problem(q, v, 8, cu)
        size = library.rosa_hip_forward_workspace_bytes(ctypes.byref(problem))
        workspace = torch.zeros(size, dtype=torch.uint8, device=DEVICE)
        out = torch.empty(total, H, Dv, device=DEVICE)
        words = torch.empty(2, H, total, dtype=torch.int32, device=DEVICE)
        status = library.rosa_hip_hard_forward(
            ctypes.byref(problem), q.data_ptr(), k.data_ptr(), v.data_ptr(),
            out.data_ptr(), words[0].data_ptr(), words[1].data_ptr(), None,
            workspace.data_ptr(), size, stream,
        )
        assert status == 0
        assert library.rosa_hip_read_offset_error(workspace.data_ptr(), stream) == bad
        grads = cabi.surrogate_vjp(q, k, v, go, words[0], words[1], None, 8, 1.0, 0.0, 3.0, 7, cu)
        torch.cuda.synchronize()
        if bad:
            assert bool(torch.isnan(out).all())
            assert all(bool(torch.isnan(g).all()) for g in grads)
        else:
            want_out, _ = c_oracle.varlen_hard_forward(query, key, value, offsets, 8)
            assert torch.equal(out.cpu(), want_out.float())
            want = c_oracle.varlen_surrogate_vjp(query, key, value, offsets, grad_output,
                                                 max_suffix_length=8)
            for g, w in zip(grads, want):
                assert_gradients_close(g, w, f"offsets {offsets}")


def test_packed_record_budget_on_both_sides_of_the_device_decision(cabi, c_oracle):
    """Packed layouts size the chunk records for the worst split of N tokens, capped by the
    budget, and decide on the device (workspace header word 3) whether the records of the
    actual lengths fit.  A budget that holds the actual records but not the worst case
    must use them; one that is non-zero but too small must fall back to recomputation;
    both must give the oracle's gradients."""

    lengths, H, D, Hv, Dv, W, p, seed = [70, 0, 1, 300, 129], 2, 3, 2, 5, 16, 0.1, 4711
    total = sum(lengths)
    query, key, value, grad_output = (t[0] for t in make_case(1, total, H, D, Hv, Dv, seed=5))
    offsets = [0] + list(np.cumsum(lengths))
    want = c_oracle.varlen_surrogate_vjp(query, key, value, offsets, grad_output,
                                         max_suffix_length=W, dropout_p=p, seed=seed)

    def band_steps(length):  # (row, band) steps of one (sequence, head)
        if length < 2:
            return 0
        bands = (length - 2) // 64 + 1
        return bands * (length - 1) - 32 * bands * (bands - 1)

    record_bytes = 4 * (96 + 32)  # S and a 16-bit window count of 64 diagonals + 16 keep bits per lane
    slots = lambda parts: (H * sum(band_steps(n) for n in parts)) // 16 \
        + H * sum((n + 63) // 64 for n in parts) + 1
    needed, worst = slots(lengths) * record_bytes, slots([total]) * record_bytes
    assert needed < worst
    q, k, v, go = (t.to(DEVICE).contiguous() for t in (query, key, value, grad_output))
    cu = torch.tensor(offsets, dtype=torch.int32, device=DEVICE)
    seed_tensor = torch.tensor(seed, dtype=torch.int64, device=DEVICE)
    _, pq, pk, _ = cabi.hard_forward(q, k, v, W, cu)
    sizes = {}
    try:
        for label, budget, fits in (("enough", needed + record_bytes, 1), ("short", needed // 2, 0),
                                    ("one record", record_bytes, 0)):
            cabi.set_record_budget(budget)
            sizes[label] = cabi.vjp_workspace_bytes(q, v, W, cu, dropout=True)
            workspace = torch.zeros(sizes[label], dtype=torch.uint8, device=DEVICE)
            grads = cabi.surrogate_vjp(q, k, v, go, pq, pk, seed_tensor, W, 1.0, p, 3.0, 7, cu,
                                       workspace=workspace)
            torch.cuda.synchronize()
            header = workspace[:16].view(torch.int32).cpu().tolist()
            assert header[0] == 0 and header[3] == fits, (label, header)
            for name, got, expected in zip("qkv", grads, want):
                assert_gradients_close(got, expected, f"{label} d{name}")
        cabi.set_record_budget(None)
        full = cabi.vjp_workspace_bytes(q, v, W, cu, dropout=True)
    finally:
        cabi.set_record_budget(None)
    assert sizes["one record"] < sizes["short"] < sizes["enough"] < full


# --------------------------------------------------------------------------- the operator's edges as bits

@pytest.mark.parametrize("bits", [1, 2, 3, 4, 7, 8, 16, 27, 32])
def test_pack_symbols_matches_the_closed_form(cabi, bits):
    # bit i = x[..., i] > 0; zero, -0, NaN and -inf give 0, +inf gives 1 (reference
    # rosa_soft_kernels.cu:202-241, rosa_soft/runtime.py:130-146)
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        logits = nonzero_randn((3, 41, 5, bits), seed=bits).to(dtype)
        flat = logits.view(-1)
        flat[:5] = torch.tensor([0.0, -0.0, float("nan"), float("-inf"), float("inf")]).to(dtype)
        weights = 1 << torch.arange(bits, dtype=torch.int64)
        want = ((logits > 0).long() * weights).sum(-1)
        words = cabi.pack_symbols(logits.to(DEVICE), torch.int32)
        assert words.shape == (3, 41, 5) and words.dtype == torch.int32
        assert torch.equal(words.cpu().long() & 0xFFFFFFFF, want)
        if bits <= 8:
            symbols = cabi.pack_symbols(logits.to(DEVICE), torch.uint8)
            assert symbols.dtype == torch.uint8 and torch.equal(symbols.cpu().long(), want)
        else:
            with pytest.raises(RuntimeError, match="symbol width"):
                cabi.pack_symbols(logits.to(DEVICE), torch.uint8)
    empty = cabi.pack_symbols(torch.empty(0, 4, bits, device=DEVICE), torch.int32)
    assert empty.shape == (0, 4)


@pytest.mark.parametrize("B,T,H,D,Hv,Dv,W,dtype,pattern", FORWARD_CASES)
def test_bit_form_of_the_output_expands_to_the_oracle_output(cabi, c_oracle, B, T, H, D, Hv, Dv,
                                                            W, dtype, pattern):
    query, key, value, _ = make_case(B, T, H, D, Hv, Dv, dtype, seed=T, pattern=pattern)
    q, k, v = (t.to(DEVICE) for t in (query, key, value))
    sign_words, routed = cabi.hard_forward_bits(q, k, v, W)
    torch.cuda.synchronize()
    want_out, want_routes, _ = c_oracle.hard_forward(query, key, value, W)
    assert sign_words.shape == (B, T, H, (Dv + 31) // 32) and routed.shape == (B, T, H)
    assert torch.equal(routed.cpu().bool(), (want_routes > 0).permute(0, 2, 1))
    assert set(routed.cpu().unique().tolist()) <= {0, 1}
    got = cabi.expand_output_bits(sign_words, routed, Dv)
    assert torch.equal(got.cpu(), want_out.float())
    # words of the null route and the bits beyond Dv are zero
    assert int((sign_words.cpu()[~routed.cpu().bool()] != 0).sum()) == 0
    if Dv % 32:
        last = sign_words.cpu()[..., -1].long() & 0xFFFFFFFF
        assert int((last >> (Dv % 32)).sum()) == 0


def test_bit_form_of_the_packed_output_and_its_invalid_offset_marker(cabi, c_oracle):
    offsets = [0, 9, 9, 70, 71, 130]
    query = nonzero_randn((130, 4, 6), seed=1)
    key = nonzero_randn((130, 4, 6), seed=2)
    value = nonzero_randn((130, 2, 40), seed=3)
    q, k, v = (t.to(DEVICE) for t in (query, key, value))
    cu = torch.tensor(offsets, dtype=torch.int32, device=DEVICE)
    sign_words, routed = cabi.hard_forward_bits(q, k, v, 12, cu)
    want_out, _ = c_oracle.varlen_hard_forward(query, key, value, offsets, 12)
    assert torch.equal(cabi.expand_output_bits(sign_words, routed, 40).cpu(), want_out)
    bad = torch.tensor([0, 80, 60, 130], dtype=torch.int32, device=DEVICE)
    sign_words, routed = cabi.hard_forward_bits(q, k, v, 12, bad)
    assert bool((routed == 0xFF).all()) and int(sign_words.abs().sum()) == 0


# --------------------------------------------------------------------------- golden vectors on the device

def test_device_matches_reference_golden_vectors(cabi):
    """GPU results against the vectors written by the reference's own oracle."""

    import os

    from tests.golden import make_reference_vectors as gold

    vectors = np.load(os.path.join(os.path.dirname(gold.__file__), "reference_vectors.npz"))
    bars = {"float32": (2e-4, 2e-6), "float16": (3e-3, 3e-3), "bfloat16": (2e-2, 2e-2)}
    for name, case in gold.DENSE_CASES.items():
        B, T, H, D, Hv, Dv, W, scale, p, ms, dtype, seed = case
        q, k, v, go = gold.dense_inputs(case)
        out, _, _, _, grads = run_device(cabi, q, k, v, go, W, scale, p, ms, seed)
        assert torch.equal(out.cpu().float(), torch.from_numpy(vectors[name + "/out"].astype(np.float32)))
        rtol, atol = bars[dtype]
        for label, got in zip(("gq", "gk", "gv"), grads):
            want = torch.from_numpy(vectors[name + "/" + label])
            torch.testing.assert_close(got.cpu(), want, rtol=rtol, atol=atol)
    for name, case in gold.VARLEN_CASES.items():
        lengths, H, D, Hv, Dv, W, scale, p, ms, dtype, _ = case
        q, k, v, go = gold.varlen_inputs(case)
        offsets = [0, *np.cumsum(lengths).tolist()]
        seed = int(vectors[name + "/seed"][0])
        out, _, _, _, grads = run_device(cabi, q, k, v, go, W, scale, p, ms, seed, 7, offsets)
        assert torch.equal(out.cpu().float(), torch.from_numpy(vectors[name + "/out"].astype(np.float32)))
        rtol, atol = bars[dtype]
        for label, got in zip(("gq", "gk", "gv"), grads):
            torch.testing.assert_close(got.cpu(), torch.from_numpy(vectors[name + "/" + label]), rtol=rtol, atol=atol)


# --------------------------------------------------------------------------- selection side channel

@pytest.mark.parametrize("B,T,H,D,Hv,Dv,W,pattern", [
    (2, 130, 2, 4, 1, 5, 16, "random"),
    (1, 300, 2, 3, 2, 4, 40, "shifted"),
    (1, 193, 1, 8, 1, 8, 128, "all_match"),
    (1, 150, 2, 2, 1, 7, 9, "periodic"),
])
def test_selected_routes_and_suffix_lengths_match_oracle(cabi, c_oracle, B, T, H, D, Hv, Dv, W,
                                                         pattern):
    # selected_route_indices and the exact suffix length at the selected route, the part of
    # the reference's inspection (rosa_soft/testing.py:28-117) the device can report
    from rosa_soft_amd.diagnostics import inspect_hard_routes

    query, key, value, _ = make_case(B, T, H, D, Hv, Dv, seed=T + 3, pattern=pattern)
    output, inspection = inspect_hard_routes(
        query.to(DEVICE), key.to(DEVICE), value.to(DEVICE), max_suffix_length=W
    )
    want_out, want_routes, want_lengths = c_oracle.hard_forward(query, key, value, W)
    assert torch.equal(output.cpu(), want_out)
    assert inspection.selected_route_indices.shape == (B, T, H)
    assert torch.equal(inspection.selected_route_indices.cpu(), want_routes.permute(0, 2, 1))
    assert torch.equal(inspection.selected_suffix_lengths.cpu(), want_lengths.permute(0, 2, 1))
    assert inspection.effective_max_suffix_length == min(W, T)
    stats = inspection.route_stats()
    assert 0.0 <= stats["null_rate"] <= 1.0 and stats["max_match_length"] <= min(W, T)
    # the null route has length 0 and only the null route has
    assert torch.equal(inspection.null_route_mask, inspection.selected_suffix_lengths == 0)


def test_selected_routes_of_a_packed_batch(cabi, c_oracle):
    from rosa_soft_amd.diagnostics import inspect_hard_routes

    lengths = [5, 0, 70, 1, 129]
    total = sum(lengths)
    query = nonzero_randn((total, 2, 3), seed=21)
    key = nonzero_randn((total, 2, 3), seed=22)
    value = nonzero_randn((total, 1, 4), seed=23)
    offsets = torch.tensor([0] + list(np.cumsum(lengths)), dtype=torch.int32)
    output, inspection = inspect_hard_routes(
        query.to(DEVICE), key.to(DEVICE), value.to(DEVICE), offsets.to(DEVICE), max_suffix_length=12
    )
    assert inspection.selected_route_indices.shape == (total, 2)
    for start, length in zip(offsets[:-1].tolist(), lengths):
        if length == 0:
            continue
        piece = slice(start, start + length)
        want_out, want_routes, want_lengths = c_oracle.hard_forward(
            query[piece].unsqueeze(0), key[piece].unsqueeze(0), value[piece].unsqueeze(0), 12
        )
        assert torch.equal(output[piece].cpu(), want_out[0])
        assert torch.equal(inspection.selected_route_indices[piece].cpu(), want_routes[0].t())
        assert torch.equal(inspection.selected_suffix_lengths[piece].cpu(), want_lengths[0].t())


# --------------------------------------------------------------------------- bounded workspace

@pytest.mark.parametrize("B,T,H,D,Hv,Dv,W,p,pattern,lengths", [
    (2, 330, 2, 4, 1, 6, 24, 0.2, "random", None),
    (1, 400, 1, 8, 1, 8, 128, 0.0, "all_match", None),
    (1, 0, 2, 3, 2, 5, 16, 0.1, "random", [70, 0, 1, 300, 129]),
])
def test_backward_without_chunk_records_recomputes_to_the_same_gradients(
        cabi, c_oracle, block_waves, B, T, H, D, Hv, Dv, W, p, pattern, lengths):
    # with the records forbidden the gradient pass sweeps forward again and hashes again
    seed = 99 if p > 0 else None
    if lengths is None:
        query, key, value, grad_output = make_case(B, T, H, D, Hv, Dv, seed=T, pattern=pattern)
        offsets = None
    else:
        total = sum(lengths)
        query, key, value, grad_output = (t[0] for t in make_case(1, total, H, D, Hv, Dv, seed=5))
        offsets = [0] + list(np.cumsum(lengths))
    cabi.set_record_budget(None)
    _, _, _, _, with_records = run_device(cabi, query, key, value, grad_output, W, 1.0, p, 3.0, seed,
                                          cu_seqlens=offsets)
    full = cabi.vjp_workspace_bytes(query.to(DEVICE), value.to(DEVICE), W,
                                    None if offsets is None else
                                    torch.tensor(offsets, dtype=torch.int32, device=DEVICE))
    cabi.set_record_budget(0)
    try:
        small = cabi.vjp_workspace_bytes(query.to(DEVICE), value.to(DEVICE), W,
                                         None if offsets is None else
                                         torch.tensor(offsets, dtype=torch.int32, device=DEVICE))
        _, _, _, _, without = run_device(cabi, query, key, value, grad_output, W, 1.0, p, 3.0, seed,
                                         cu_seqlens=offsets)
    finally:
        cabi.set_record_budget(None)
    # without records the workspace loses them and gains one fallback checkpoint per staged
    # segment and resident wave: smaller at training sizes, not necessarily at these
    assert small != full
    if lengths is None:
        want = c_oracle.surrogate_vjp(query, key, value, grad_output, max_suffix_length=W,
                                      dropout_p=p, seed=seed)
        for name, got, expected in zip(("grad_query", "grad_key", "grad_value"), without, want):
            assert_gradients_close(got, expected, name)
    # both ways of getting the state give the same gradients up to summation order
    for got, expected in zip(without, with_records):
        assert_gradients_close(got, expected.cpu())


# --------------------------------------------------------------------------- pieces of bands

PIECE_CASES = [
    # B, T, H, D, Hv, Dv, W, p, dtype, pattern, piece_rows, mask, lengths
    # a match of the whole sequence: every piece starts inside it, the halo (W - 1 rows,
    # rounded up to chunks) is longer than the pieces
    (1, 400, 1, 8, 1, 8, 128, 0.0, torch.float32, "all_match", 64, 7, None),
    (1, 530, 2, 2, 2, 32, 256, 0.0, torch.float16, "all_match", 128, 7, None),
    (1, 450, 2, 4, 1, 6, 40, 0.0, torch.float32, "shifted", 64, 7, None),
    (1, 450, 2, 4, 1, 6, 40, 0.25, torch.float32, "shifted", 96, 7, None),
    (1, 333, 2, 7, 1, 20, 9, 0.0, torch.float16, "periodic", 64, 7, None),
    (1, 333, 1, 3, 1, 8, 600, 0.1, torch.float32, "periodic", 64, 7, None),
    (2, 700, 3, 20, 3, 33, 64, 0.1, torch.bfloat16, "random", 192, 7, None),
    # value width above 64: two slices, each a run of both passes with its own pieces
    (1, 260, 2, 9, 1, 70, 24, 0.2, torch.float32, "shifted", 64, 7, None),
    # window beyond the sequence: the halo of every piece reaches the band's end
    (1, 200, 1, 8, 1, 8, 1000, 0.0, torch.float32, "periodic", 64, 7, None),
    # one gradient at a time: without symbol gradients the pieces take no halo
    (1, 300, 2, 5, 1, 6, 33, 0.2, torch.float32, "shifted", 64, 4, None),
    (1, 300, 2, 5, 1, 6, 33, 0.2, torch.float32, "shifted", 64, 1, None),
    (1, 300, 2, 5, 1, 6, 33, 0.2, torch.float32, "shifted", 64, 2, None),
    # packed sequences: pieces past the end of a short sequence's bands are empty work items
    (1, 0, 2, 3, 2, 5, 16, 0.1, torch.float32, "random", 64, 7, [70, 0, 1, 300, 129]),
    (1, 0, 2, 8, 1, 8, 150, 0.0, torch.float32, "all_match", 64, 7, [257, 64, 390]),
]


@pytest.mark.parametrize("records", [True, False], ids=["records", "no_records"])
@pytest.mark.parametrize("B,T,H,D,Hv,Dv,W,p,dtype,pattern,piece_rows,mask,lengths", PIECE_CASES)
def test_bands_cut_into_pieces_match_oracle(cabi, c_oracle, records, B, T, H, D, Hv, Dv, W, p,
                                            dtype, pattern, piece_rows, mask, lengths):
    """The gradient kernel cuts long bands into pieces when a shape has few of them; forced
    here at test sizes.  A piece restarts the reverse recurrences W - 1 rows below its last
    row and leaves its first 64 columns' partial sums to the piece above: long matches that
    cross every cut are the cases that would show a wrong halo or a lost partial sum."""

    seed = 31337 if p > 0 else None
    if lengths is None:
        query, key, value, grad_output = make_case(B, T, H, D, Hv, Dv, dtype, seed=T + W,
                                                   pattern=pattern)
        offsets = None
    else:
        total = sum(lengths)
        query, key, value, grad_output = (
            t[0] for t in make_case(1, total, H, D, Hv, Dv, dtype, seed=total, pattern=pattern))
        offsets = [0] + [int(x) for x in np.cumsum(lengths)]
    cabi.set_gradient_piece_rows(piece_rows)
    cabi.set_record_budget(None if records else 0)
    try:
        _, _, _, _, grads = run_device(cabi, query, key, value, grad_output, W, 1.0, p, 3.0, seed,
                                       mask, offsets)
        cabi.set_gradient_piece_rows(-1)
        _, _, _, _, whole = run_device(cabi, query, key, value, grad_output, W, 1.0, p, 3.0, seed,
                                       mask, offsets)
    finally:
        cabi.set_gradient_piece_rows(None)
        cabi.set_record_budget(None)
    if lengths is None:
        want = c_oracle.surrogate_vjp(query, key, value, grad_output, max_suffix_length=W,
                                      dropout_p=p, seed=seed)
    else:
        want = c_oracle.varlen_surrogate_vjp(query, key, value, offsets, grad_output,
                                             max_suffix_length=W, dropout_p=p, seed=seed)
    longest_logit = 2.4142 * ((1.0 + min(W, max(T, max(lengths or [0])))) ** 0.5 - 1.0)
    slack = max(1.0, longest_logit / 40.0)
    for bit, name, got, unsplit, expected in zip((1, 2, 4), ("grad_query", "grad_key", "grad_value"),
                                                 grads, whole, want):
        if not mask & bit:
            assert got is None
            continue
        assert_gradients_close(got, expected, name, slack)
        assert_gradients_close(got, unsplit.cpu(), name + " against whole bands", slack)


def test_atomic_rate_measurement_is_plausible_and_checks_its_arguments(cabi):
    """The measurement behind the gradient kernel's second bound: float atomics in the flush
    pattern (16 rows of a tile per step) run at some tens of G row segments per second on
    an MI355X whatever the number of live columns; bad arguments are refused with a status."""

    full = cabi.measure_atomic_rate(512, 16)
    half = cabi.measure_atomic_rate(512, 8)
    assert 2e9 < full < 2e11, full
    assert 0.5 < half / full < 2.0, (half, full)  # segments, not lanes, bound the rate
    with pytest.raises(RuntimeError, match="row_floats"):
        cabi.measure_atomic_rate(8, 8)
    with pytest.raises(RuntimeError, match="columns"):
        cabi.measure_atomic_rate(512, 17)


@pytest.mark.parametrize("T,H,D,Dv,W,ms,seed", [
    (200, 2, 5, 8, 2, 1.0, 93),
    (128, 2, 8, 8, 1, 1.0, 96),
    (191, 2, 8, 4, 500, 1.0, 59),
])
def test_value_gradient_keeps_its_margin_with_split_weights(cabi, c_oracle, T, H, D, Dv, W, ms,
                                                            seed):
    """dV sums route weights that run on the bfloat16 matrix pipe as two terms.  Short windows
    leave large weights on the early routes of many rows; a split whose leading term was
    truncated instead of rounded cost these cases their whole margin (errors at 1.1 to 1.6
    times the bar).  With both terms rounded the error stays below half of it."""

    query, key, value, grad_output = make_case(2, T, H, D, 1, Dv, seed=seed)
    _, _, _, _, grads = run_device(cabi, query, key, value, grad_output, W, 1.0, 0.0, ms)
    want = c_oracle.surrogate_vjp(query, key, value, grad_output, max_suffix_length=W, scale=1.0,
                                  dropout_p=0.0, mismatch_scale=ms, seed=None)
    assert_gradients_close(grads[2], want[2], "dv", slack=0.7)
    assert_gradients_close(grads[0], want[0], "dq")
    assert_gradients_close(grads[1], want[1], "dk")
