"""The hard forward through the entry point that allocates nothing (needs a real MI355X).

``rosa_hip_hard_forward_static`` keeps its workspace in an array of the library's device
image instead of taking one from the caller.  It must give exactly what
``rosa_hip_hard_forward`` gives, call after call on the same GPU: the array keeps the
previous call's contents, so a second, smaller problem runs over stale data.
"""

import ctypes

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


def both_ways(cabi, query, key, value, horizon, offsets=None, routed=True):
    q, k, v = (t.to(DEVICE).contiguous() for t in (query, key, value))
    cu = None if offsets is None else torch.tensor(offsets, dtype=torch.int32, device=DEVICE)
    want = cabi.hard_forward(q, k, v, horizon, cu)
    # outputs exist before the call: the entry point itself must not need an allocation
    outputs = tuple(torch.full_like(t, 77) for t in want)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(DEVICE)
    got = cabi.hard_forward_static(q, k, v, horizon, cu, outputs=outputs)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(DEVICE) == before
    assert torch.equal(got[0].isnan(), want[0].isnan())
    assert torch.equal(got[0].nan_to_num(nan=5.0), want[0].nan_to_num(nan=5.0))
    # with invalid offsets no row is routed and the route tensors keep what they held
    for a, b in zip(got[1:] if routed else got[1:3], want[1:]):
        assert torch.equal(a, b)
    return got


def test_two_calls_in_a_row_the_second_smaller(cabi, c_oracle):
    # dense, then a smaller dense problem, then packed sequences with empty ones, then a tiny one
    query = nonzero_randn((2, 700, 4, 5), seed=1)
    key = query.roll(2, dims=1).clone()
    key[:, ::9] = -key[:, ::9]
    value = nonzero_randn((2, 700, 2, 9), seed=2)
    first = both_ways(cabi, query, key, value, 48)
    want_out, want_routes, _ = c_oracle.hard_forward(query, key, value, 48)
    assert torch.equal(first[0].cpu(), want_out) and torch.equal(first[3].cpu(), want_routes)
    assert int((first[3] > 0).sum()) > 0

    small = [t[:1, :130].contiguous() for t in (query, key, value)]
    second = both_ways(cabi, *small, 48)
    want_out, want_routes, _ = c_oracle.hard_forward(*small, 48)
    assert torch.equal(second[0].cpu(), want_out) and torch.equal(second[3].cpu(), want_routes)

    offsets = [0, 40, 40, 300, 301, 520]
    packed = [t[0, :520].to(torch.bfloat16).contiguous() for t in (query, key, value)]
    third = both_ways(cabi, *packed, 16, offsets)
    want_out, want_routes = c_oracle.varlen_hard_forward(*packed, offsets, 16)
    assert torch.equal(third[0].cpu(), want_out) and torch.equal(third[3].cpu(), want_routes)

    tiny = [t[:1, :3].contiguous() for t in (query, key, value)]
    both_ways(cabi, *tiny, 2)
    # invalid device offsets after valid ones: NaN output, as with the caller's workspace
    bad = both_ways(cabi, *packed, 16, [0, 300, 200, 520], routed=False)
    assert bool(torch.isnan(bad[0].float()).all())
    both_ways(cabi, *packed, 16, offsets)


def test_sizes_beyond_the_static_scratch_are_rejected(cabi):
    # 16 MiB hold the routes of about 4.19 M (token, head) pairs; nothing is launched beyond
    query = torch.empty(1, 70000, 64, 1, device=DEVICE)
    value = torch.empty(1, 70000, 1, 1, device=DEVICE)
    with pytest.raises(RuntimeError, match="static scratch"):
        cabi.hard_forward_static(query, query, value, 4)
    library = cabi.load()
    problem = cabi.make_problem(query[:, :100], value[:, :100], 4)
    assert library.rosa_hip_hard_forward_static(
        ctypes.byref(problem), None, None, None, None, None, None, None, None) != 0


def test_static_forward_records_into_a_hip_graph_after_a_first_call_outside(cabi):
    """The callers this entry point exists for record it into a HIP graph.  Its first call on
    a device looks up the address of the scratch array, which is not a stream operation and
    must therefore happen before the recording; after that the call is launches only.  Every
    replay is checked against eager work done between the replays, on inputs rewritten in
    place, and neither torch's allocator nor the device's free memory moves."""

    generator = torch.Generator(device=DEVICE).manual_seed(77)
    q = torch.randn(2, 300, 4, 6, device=DEVICE, generator=generator)
    k = torch.randn(2, 300, 4, 6, device=DEVICE, generator=generator)
    v = torch.randn(2, 300, 2, 10, device=DEVICE, generator=generator)
    want = cabi.hard_forward(q, k, v, 32)
    outputs = tuple(torch.full_like(t, 77) for t in want)
    cabi.hard_forward_static(q, k, v, 32, outputs=outputs)  # the first call: outside
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cabi.hard_forward_static(q, k, v, 32, outputs=outputs)
    torch.cuda.synchronize()
    free_bytes = torch.cuda.mem_get_info(DEVICE)[0]
    for _ in range(3):
        q.copy_(torch.randn(q.shape, device=DEVICE, generator=generator))
        k.copy_(q.roll(1, dims=1))
        want = cabi.hard_forward(q, k, v, 32)
        for tensor in outputs:
            tensor.fill_(77)
        torch.cuda.synchronize()
        allocated = torch.cuda.memory_allocated(DEVICE)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(DEVICE) == allocated
        for got, expected in zip(outputs, want):
            assert torch.equal(got, expected)
        assert int((outputs[3] > 0).sum()) > 0
    # (torch's cache may have grown for the eager calls' workspaces; the replays take nothing)
    assert torch.cuda.mem_get_info(DEVICE)[0] >= free_bytes - (64 << 20)
