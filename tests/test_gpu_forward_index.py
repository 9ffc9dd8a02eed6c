"""The hard forward through the index of the keys (route_candidates_kernel) gives the routes of
the scan over all routes (hard_route_kernel), which are those of the reference's forward kernel
(rosa_soft_kernels.cu:367-531: longest matched suffix, latest route on ties, null route for a
zero run), bit for bit: at shapes below the sizes the library picks the index for by itself,
with every row block handed back to the scan, on inputs whose row blocks exceed their budget,
and with symbols wide enough to be bucketed by a hash."""

import pytest
import torch

from tests.conftest import nonzero_randn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cabi():
    from rosa_soft_amd import cabi as module

    module.load()
    yield module
    module.set_forward_index(None)


def _pattern_inputs(pattern, batch, length, heads, bits, seed):
    query = nonzero_randn((batch, length, heads, bits), dtype=torch.float32, seed=seed)
    key = nonzero_randn((batch, length, heads, bits), dtype=torch.float32, seed=seed + 1)
    if pattern == "random":
        return query, key
    if pattern == "constant":
        return torch.ones_like(query), torch.ones_like(key)
    if pattern.startswith("period"):
        period = int(pattern[len("period"):])
        motif = nonzero_randn((batch, period, heads, bits), dtype=torch.float32, seed=seed + 2)
        key = motif.repeat(1, length // period + 1, 1, 1)[:, :length].contiguous()
        return key.clone(), key
    assert pattern == "echo"
    # the second half of the keys repeats the first, and the queries follow the keys one
    # step behind: long runs, with an earlier and a later route of the same length
    half = length // 2
    key[:, half:2 * half] = key[:, :half]
    query[:, 1:] = key[:, :-1]
    generator = torch.Generator().manual_seed(seed + 3)
    noise = torch.rand(batch, length, heads, 1, generator=generator) < 0.02
    return torch.where(noise, -query, query).contiguous(), key.contiguous()


DENSE_CASES = [
    # batch, length, heads, bits, value heads, value width, window, pattern
    (2, 700, 4, 8, 2, 8, 16, "random"),
    (1, 1500, 3, 6, 3, 4, 1, "random"),
    (1, 2100, 2, 12, 1, 8, 2100, "random"),
    (2, 513, 2, 32, 2, 16, 7, "random"),       # buckets by hash
    (1, 900, 2, 20, 1, 8, 40, "echo"),         # buckets by hash, long runs
    (3, 65, 2, 7, 1, 8, 4, "random"),
    (1, 1, 1, 8, 1, 8, 3, "random"),
    (1, 2, 1, 8, 1, 8, 3, "random"),
    (2, 300, 2, 1, 2, 8, 9, "random"),         # two symbols
    (2, 300, 2, 3, 1, 8, 300, "random"),
    (1, 1200, 2, 8, 2, 8, 500, "period5"),     # every row block exceeds its budget
    (1, 1200, 2, 8, 1, 8, 64, "period300"),    # small buckets, long runs
    (2, 640, 2, 9, 2, 8, 640, "constant"),     # one bucket
    (1, 2048, 4, 8, 2, 8, 128, "echo"),
    (1, 4096, 2, 10, 1, 8, 33, "echo"),
]


@pytest.mark.parametrize("case", DENSE_CASES, ids=lambda c: "-".join(str(x) for x in c))
def test_indexed_forward_equals_the_scan_and_the_oracle(cabi, c_oracle, case):
    batch, length, heads, bits, value_heads, width, window, pattern = case
    device = torch.device("cuda:0")
    query, key = _pattern_inputs(pattern, batch, length, heads, bits, seed=17 * length + bits)
    value = nonzero_randn((batch, length, value_heads, width), dtype=torch.float32, seed=5)
    want_output, want_routes, _ = c_oracle.hard_forward(query, key, value, window)
    q, k, v = query.to(device), key.to(device), value.to(device)
    for mode in ("scan", "always", "handed_back", None):
        cabi.set_forward_index(mode)
        output, _, _, routes = cabi.hard_forward(q, k, v, window)
        assert torch.equal(routes.cpu(), want_routes), mode
        assert torch.equal(output.cpu(), want_output), mode
    cabi.set_forward_index(None)


@pytest.mark.parametrize("bits,window", [(8, 16), (6, 1), (24, 700), (2, 5)])
def test_indexed_forward_of_packed_sequences_equals_the_scan(cabi, bits, window):
    device = torch.device("cuda:0")
    lengths = [700, 1, 0, 513, 64, 2, 65, 1100, 0, 129]
    total = sum(lengths)
    offsets = torch.tensor([0] + torch.tensor(lengths).cumsum(0).tolist(), dtype=torch.int32,
                           device=device)
    query = nonzero_randn((total, 3, bits), dtype=torch.float32, seed=bits).to(device)
    key = nonzero_randn((total, 3, bits), dtype=torch.float32, seed=bits + 1).to(device)
    # a repeated stretch inside the longest sequence, so that long runs exist
    begin = sum(lengths[:7])
    key[begin + 500:begin + 900] = key[begin + 50:begin + 450]
    query[begin + 501:begin + 900] = key[begin + 500:begin + 899]
    value = nonzero_randn((total, 3, 8), dtype=torch.float32, seed=3).to(device)
    cabi.set_forward_index("scan")
    want_output, _, _, want_routes = cabi.hard_forward(query, key, value, window, offsets)
    assert int((want_routes > 0).sum()) > 0
    for mode in ("always", "handed_back", None):
        cabi.set_forward_index(mode)
        output, _, _, routes = cabi.hard_forward(query, key, value, window, offsets)
        assert torch.equal(routes, want_routes), mode
        assert torch.equal(output, want_output), mode
    cabi.set_forward_index(None)


def test_indexed_forward_through_the_entry_point_that_allocates_nothing(cabi):
    device = torch.device("cuda:0")
    query = nonzero_randn((2, 900, 4, 8), dtype=torch.float32, seed=41).to(device)
    key = nonzero_randn((2, 900, 4, 8), dtype=torch.float32, seed=42).to(device)
    value = nonzero_randn((2, 900, 2, 8), dtype=torch.float32, seed=43).to(device)
    cabi.set_forward_index("scan")
    want_output, _, _, want_routes = cabi.hard_forward(query, key, value, 32)
    cabi.set_forward_index("always")
    try:
        output, _, _, routes = cabi.hard_forward_static(query, key, value, 32)
    finally:
        cabi.set_forward_index(None)
    assert torch.equal(routes, want_routes) and torch.equal(output, want_output)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [
    # batch, length, heads, bits, value heads, value width
    (2, 37, 3, 8, 3, 8),      # symbols and rows of whole 16-byte pieces, a block across two batches
    (1, 130, 5, 16, 1, 24),
    (3, 16, 2, 32, 2, 64),
    (2, 50, 4, 4, 2, 4),      # whole pieces in float32 only
    (1, 70, 2, 5, 2, 3),      # never whole pieces: one lane per symbol, one thread per element
])
def test_packed_words_and_gathered_output_of_every_kernel_variant(cabi, c_oracle, dtype, shape):
    batch, length, heads, bits, value_heads, width = shape
    device = torch.device("cuda:0")
    query = nonzero_randn((batch, length, heads, bits), dtype=dtype, seed=1)
    key = nonzero_randn((batch, length, heads, bits), dtype=dtype, seed=2)
    value = nonzero_randn((batch, length, value_heads, width), dtype=dtype, seed=3)
    output, packed_q, packed_k, routes = cabi.hard_forward(
        query.to(device), key.to(device), value.to(device), 6)
    weights = (1 << torch.arange(bits, dtype=torch.int64))
    for packed, source in ((packed_q, query), (packed_k, key)):
        want = ((source.float() > 0).to(torch.int64) * weights).sum(-1).permute(0, 2, 1)
        assert torch.equal(packed.cpu().to(torch.int64) & 0xffffffff, want)
    want_output, want_routes, _ = c_oracle.hard_forward(query, key, value, 6)
    assert torch.equal(routes.cpu(), want_routes)
    assert torch.equal(output.cpu(), want_output)
    # packed sequences: the same tokens as one sequence per batch entry
    offsets = torch.arange(batch + 1, dtype=torch.int32, device=device) * length
    flat = [x.to(device).flatten(0, 1).contiguous() for x in (query, key, value)]
    output_packed, words_q, _, _ = cabi.hard_forward(flat[0], flat[1], flat[2], 6, offsets)
    assert torch.equal(output_packed.cpu(), want_output.flatten(0, 1))
    assert torch.equal(words_q.cpu().view(heads, batch, length).permute(1, 0, 2), packed_q.cpu())


def test_indexed_forward_over_the_random_sweep_of_shapes(cabi, c_oracle):
    """The forward of 300 cases of the sweep's case generator (symbol widths 1 to 32, lengths
    around the 64-row blocks, random, shifted, periodic and constant inputs, three dtypes,
    packed batches with empty sequences) with the index at every shape, against the oracle."""

    import random

    import numpy as np

    from tests.test_gpu_parity import make_case
    from tests.test_gpu_sweep import SHORT, draw_case, draw_run

    device = torch.device("cuda:0")
    rng = random.Random(4242)
    cabi.set_forward_index("always")
    try:
        for index in range(300):
            c = draw_case(rng, SHORT + [511, 777, 1024])
            _, parts = draw_run(rng, c)
            label = f"case {index}: {c} {parts}"
            if not c["packed"]:
                q, k, v, _ = make_case(c["B"], c["T"], c["H"], c["D"], c["Hv"], c["Dv"], c["dtype"],
                                       seed=index, pattern=c["pattern"])
                want_out, want_routes, _ = c_oracle.hard_forward(q, k, v, c["W"])
                out, _, _, routes = cabi.hard_forward(q.to(device), k.to(device), v.to(device), c["W"])
            else:
                offsets = [0, *np.cumsum(parts).tolist()]
                total = offsets[-1]
                q = nonzero_randn((total, c["H"], c["D"]), seed=index + 1).to(c["dtype"])
                k = nonzero_randn((total, c["H"], c["D"]), seed=index + 2).to(c["dtype"])
                if c["pattern"] != "random":
                    k = q.roll(2, dims=0).clone()
                v = nonzero_randn((total, c["Hv"], c["Dv"]), seed=index + 3).to(c["dtype"])
                want_out, want_routes = c_oracle.varlen_hard_forward(q, k, v, offsets, c["W"])
                out, _, _, routes = cabi.hard_forward(
                    q.to(device), k.to(device), v.to(device), c["W"],
                    torch.tensor(offsets, dtype=torch.int32, device=device))
            assert torch.equal(routes.cpu(), want_routes), label
            assert torch.equal(out.cpu().float(), want_out.float()), label
    finally:
        cabi.set_forward_index(None)


@pytest.mark.parametrize("bits", [8, 12, 30])
def test_indexed_forward_of_one_long_sequence_equals_the_scan(cabi, bits):
    # 32 768 tokens: 32 passes of the index build, 4 096 buckets (by hash at 30 bits), and with
    # 8-bit symbols buckets of 128 routes; a repeated stretch gives runs up to the window
    device = torch.device("cuda:0")
    length = 32768
    query = nonzero_randn((1, length, 2, bits), dtype=torch.float32, seed=bits).to(device)
    key = nonzero_randn((1, length, 2, bits), dtype=torch.float32, seed=bits + 1).to(device)
    key[:, 20000:26000] = key[:, 3000:9000]
    query[:, 20001:26000] = key[:, 20000:25999]
    value = nonzero_randn((1, length, 1, 8), dtype=torch.float32, seed=3).to(device)
    cabi.set_forward_index("scan")
    try:
        want_output, _, _, want_routes = cabi.hard_forward(query, key, value, 300)
        cabi.set_forward_index(None)
        output, _, _, routes = cabi.hard_forward(query, key, value, 300)
    finally:
        cabi.set_forward_index(None)
    assert int((want_routes > 0).sum()) > length // 4
    assert torch.equal(routes, want_routes) and torch.equal(output, want_output)
