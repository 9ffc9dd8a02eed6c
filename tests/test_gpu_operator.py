"""The public operators and the dispatcher on a real MI355X.

Restates the behavioural checks of the reference's device tests
(tests/test_soft_cuda.py, tests/test_soft_varlen.py, tests/test_soft_integration.py)
for the parts that sit above the kernels: autograd wiring, seeds, dtype casts,
error surfaces, tracing.
"""

import pytest
import torch

from tests.conftest import nonzero_randn

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"
INT64_MAX = torch.iinfo(torch.int64).max


@pytest.fixture(scope="module")
def rosa():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import rosa_soft_amd

    assert rosa_soft_amd.BUILD_CAPABILITIES.variant == "rocm"
    return rosa_soft_amd


def device_inputs(B=2, T=48, H=4, D=8, Hv=2, Dv=5, dtype=torch.float32, seed=0):
    query = nonzero_randn((B, T, H, D), seed=seed + 1).to(dtype)
    key = nonzero_randn((B, T, H, D), seed=seed + 2).to(dtype)
    value = nonzero_randn((B, T, Hv, Dv), seed=seed + 3).to(dtype)
    grad_output = nonzero_randn((B, T, H, Dv), seed=seed + 4, floor=0.0).to(dtype)
    return query, key, value, grad_output


def next_device_seed(manual_seed):
    """The seed the operator will draw after torch.cuda.manual_seed(manual_seed)."""

    torch.cuda.manual_seed(manual_seed)
    drawn = int(torch.randint(0, INT64_MAX, (), dtype=torch.int64, device=DEVICE))
    torch.cuda.manual_seed(manual_seed)
    return drawn


@pytest.mark.parametrize(
    "dtype,rtol,atol",
    [(torch.float32, 1e-4, 1e-6), (torch.float16, 3e-3, 3e-3), (torch.bfloat16, 2e-2, 2e-2)],
)
@pytest.mark.parametrize("dropout_p", [0.0, 0.3])
def test_operator_matches_oracle_end_to_end(rosa, c_oracle, dtype, rtol, atol, dropout_p):
    # reference tests/test_soft_cuda.py:141-207, :424-507
    query, key, value, grad_output = device_inputs(dtype=dtype, seed=5)
    seed = next_device_seed(1234) if dropout_p > 0 else None
    leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
    output = rosa.rosa_soft(*leaves, max_suffix_length=12, scale=1.2, dropout_p=dropout_p)
    grads = torch.autograd.grad(output, leaves, grad_output.to(DEVICE))
    want_out, _, _ = c_oracle.hard_forward(query, key, value, 12)
    assert output.dtype == dtype and torch.equal(output.detach().cpu(), want_out)
    want = c_oracle.surrogate_vjp(
        query, key, value, grad_output, max_suffix_length=12, scale=1.2, dropout_p=dropout_p,
        seed=seed,
    )
    for got, expected in zip(grads, want):
        assert got.dtype == dtype
        torch.testing.assert_close(
            got.cpu().double(), expected, rtol=rtol, atol=max(atol, 1e-5 * float(expected.abs().max()))
        )


def test_packed_operator_matches_oracle(rosa, c_oracle):
    offsets = [0, 9, 9, 40, 41, 100]
    query = nonzero_randn((100, 4, 6), seed=1)
    key = nonzero_randn((100, 4, 6), seed=2)
    value = nonzero_randn((100, 2, 7), seed=3)
    grad_output = nonzero_randn((100, 4, 7), seed=4, floor=0.0)
    seed = next_device_seed(77)
    leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
    # a non-contiguous view of the offsets (reference tests/test_soft_varlen.py:918-957)
    cu = torch.tensor([[o, -1] for o in offsets], dtype=torch.int32, device=DEVICE)[:, 0]
    assert not cu.is_contiguous()
    output = rosa.rosa_soft_varlen(*leaves, cu, max_suffix_length=10, dropout_p=0.25, mismatch_scale=9.0)
    grads = torch.autograd.grad(output, leaves, grad_output.to(DEVICE))
    want_out, _ = c_oracle.varlen_hard_forward(query, key, value, offsets, 10)
    assert torch.equal(output.detach().cpu(), want_out)
    want = c_oracle.varlen_surrogate_vjp(
        query, key, value, offsets, grad_output, max_suffix_length=10, dropout_p=0.25,
        mismatch_scale=9.0, seed=seed,
    )
    for got, expected in zip(grads, want):
        torch.testing.assert_close(
            got.cpu().double(), expected, rtol=1e-4, atol=1e-5 * float(expected.abs().max())
        )


def test_invalid_device_offsets_give_nan_at_the_operator(rosa):
    """The reference kills the process on bad device cu_seqlens (tests/test_soft_varlen.py:
    181-226); here the operator returns, and the mistake shows as NaN in the output, in every
    gradient and therefore in any loss built on them.  Half-precision outputs carry it too."""

    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        query = nonzero_randn((64, 2, 4), seed=1).to(dtype)
        key = nonzero_randn((64, 2, 4), seed=2).to(dtype)
        value = nonzero_randn((64, 1, 5), seed=3).to(dtype)
        for offsets in ([0, 50, 30, 64], [0, 20, 70], [1, 64]):
            cu = torch.tensor(offsets, dtype=torch.int32, device=DEVICE)
            leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
            output = rosa.rosa_soft_varlen(*leaves, cu, max_suffix_length=8, dropout_p=0.1)
            assert output.shape == (64, 2, 5) and bool(torch.isnan(output).all())
            grads = torch.autograd.grad(output, leaves, torch.ones_like(output))
            assert all(bool(torch.isnan(g).all()) for g in grads)
            with torch.no_grad():
                quiet = rosa.rosa_soft_varlen(*leaves, cu, max_suffix_length=8)
            assert bool(torch.isnan(quiet).all())
        good = torch.tensor([0, 20, 64], dtype=torch.int32, device=DEVICE)
        leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
        output = rosa.rosa_soft_varlen(*leaves, good, max_suffix_length=8)
        grads = torch.autograd.grad(output, leaves, torch.ones_like(output))
        assert bool(torch.isfinite(output).all())
        assert all(bool(torch.isfinite(g).all()) for g in grads)


def test_no_grad_path_draws_no_seed_and_equals_train_forward(rosa):
    # reference tests/test_soft_cuda.py:745-810
    query, key, value, _ = device_inputs(seed=9)
    q, k, v = (t.to(DEVICE) for t in (query, key, value))
    state = torch.cuda.get_rng_state(0)
    with torch.no_grad():
        quiet = rosa.rosa_soft(q, k, v, dropout_p=0.5)
    plain = rosa.rosa_soft(q, k, v, dropout_p=0.5)  # no leaf requires grad
    assert torch.equal(state, torch.cuda.get_rng_state(0))
    leaves = [t.clone().requires_grad_() for t in (q, k, v)]
    trained = rosa.rosa_soft(*leaves, dropout_p=0.0)
    assert torch.equal(state, torch.cuda.get_rng_state(0))  # p = 0 draws nothing either
    assert torch.equal(quiet, trained.detach()) and torch.equal(plain, quiet)
    rosa.rosa_soft(*leaves, dropout_p=0.5)
    assert not torch.equal(state, torch.cuda.get_rng_state(0))


def test_only_requested_gradients_and_noncontiguous_inputs(rosa, c_oracle):
    # reference tests/test_soft_cuda.py:548-567, :813-846
    query = nonzero_randn((2, 4, 20, 3), seed=60).transpose(1, 2)
    key = nonzero_randn((2, 4, 20, 3), seed=61).transpose(1, 2)
    value = nonzero_randn((2, 2, 20, 5), seed=62).transpose(1, 2)
    q = query.to(DEVICE).requires_grad_()
    k = key.to(DEVICE)
    v = value.to(DEVICE).requires_grad_()
    assert not q.is_contiguous()
    output = rosa.rosa_soft(q, k, v, max_suffix_length=5)
    assert output.shape == (2, 20, 4, 5)
    output.float().square().mean().backward()
    assert q.grad is not None and v.grad is not None and k.grad is None
    want_out, _, _ = c_oracle.hard_forward(query, key, value, 5)
    grad_output = 2.0 * want_out / want_out.numel()
    want = c_oracle.surrogate_vjp(query, key, value, grad_output, max_suffix_length=5)
    torch.testing.assert_close(q.grad.cpu().double(), want[0], rtol=1e-4, atol=1e-5 * float(want[0].abs().max()))
    torch.testing.assert_close(v.grad.cpu().double(), want[2], rtol=1e-4, atol=1e-5 * float(want[2].abs().max()))


def test_repeatability_within_reduction_order(rosa):
    # reference tests/test_soft_cuda.py:745-769
    query, key, value, grad_output = device_inputs(T=200, seed=21)

    def run():
        leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
        output = rosa.rosa_soft(*leaves, max_suffix_length=16)
        return output, torch.autograd.grad(output, leaves, grad_output.to(DEVICE))

    first, second = run(), run()
    assert torch.equal(first[0], second[0])
    for a, b in zip(first[1], second[1]):
        torch.testing.assert_close(a, b, rtol=2e-6, atol=2e-7)


def test_backward_is_once_differentiable_and_flagged_nondeterministic(rosa):
    # reference tests/test_soft_cuda.py:976-1007
    query, key, value, _ = device_inputs(T=16, seed=3)
    leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
    output = rosa.rosa_soft(*leaves)
    gradients = torch.autograd.grad(output.sum(), leaves, create_graph=True)
    assert all(not gradient.requires_grad for gradient in gradients)
    torch.use_deterministic_algorithms(True)
    try:
        output = rosa.rosa_soft(*leaves)
        with pytest.raises(RuntimeError, match="deterministic"):
            output.sum().backward()
    finally:
        torch.use_deterministic_algorithms(False)


def test_raw_operator_error_surface(rosa):
    # reference tests/test_soft_cuda.py:113-124, :888-973
    query, key, value, grad_output = (t.to(DEVICE) for t in device_inputs(T=12, seed=4))
    ops = torch.ops.rosa_soft
    out, pq, pk = ops.hard_forward(query, key, value, 8)
    empty = torch.empty(0, dtype=torch.int64, device=DEVICE)

    def vjp(**changes):
        args = dict(
            query=query, key=key, value=value, grad_output=grad_output, pq=pq, pk=pk, seed=empty,
            W=8, scale=1.0, p=0.0, ms=3.0, mask=7,
        )
        args.update(changes)
        return ops.surrogate_vjp_masked(
            args["query"], args["key"], args["value"], args["grad_output"], args["pq"], args["pk"],
            args["seed"], args["W"], args["scale"], args["p"], args["ms"], args["mask"],
        )

    assert all(g.dtype == torch.float32 for g in vjp())
    with pytest.raises(RuntimeError, match="packed_query_symbols head mismatch"):
        vjp(pq=pq[:, :2])
    with pytest.raises(RuntimeError, match="scalar exactly"):
        vjp(p=0.5)
    with pytest.raises(RuntimeError, match="scalar exactly"):
        vjp(seed=torch.zeros((), dtype=torch.int64, device=DEVICE))
    with pytest.raises(RuntimeError, match="int64"):
        vjp(p=0.5, seed=torch.zeros((), dtype=torch.int32, device=DEVICE))
    with pytest.raises(RuntimeError, match="CUDA"):
        vjp(p=0.5, seed=torch.zeros((), dtype=torch.int64))
    with pytest.raises(RuntimeError, match="scale"):
        vjp(scale=0.0)
    with pytest.raises(RuntimeError, match="max_suffix_length"):
        vjp(W=0)
    with pytest.raises(RuntimeError, match="mismatch_scale"):
        vjp(ms=float("inf"))
    with pytest.raises(RuntimeError, match=r"\[1, 7\]"):
        vjp(mask=0)
    with pytest.raises(RuntimeError, match="grad_output shape mismatch"):
        vjp(grad_output=grad_output[:, :-1])
    grads = vjp(mask=2)
    assert grads[0].shape == (0,) and grads[2].shape == (0,) and grads[1].shape == key.shape
    with pytest.raises(RuntimeError, match="cu_seqlens must be int32"):
        ops.hard_forward_varlen(
            query[0], key[0], value[0], torch.tensor([0, 12], device=DEVICE), 4
        )


def test_saturated_and_non_finite_logits_follow_the_jacobian(rosa):
    # reference tests/test_soft_cuda.py:570-663: +-inf logits get exactly zero
    # gradient, huge logits a vanishing one, everything else stays finite.
    query, key, value, grad_output = device_inputs(T=24, seed=8)
    query[0, 3, 0, 0] = float("inf")
    key[0, 2, 1, 1] = float("-inf")
    value[0, 5, 0, 2] = 1e30
    leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
    output = rosa.rosa_soft(*leaves, max_suffix_length=6)
    grads = torch.autograd.grad(output, leaves, grad_output.to(DEVICE))
    assert all(torch.isfinite(g).all() for g in grads)
    assert float(grads[0][0, 3, 0, 0]) == 0.0 and float(grads[1][0, 2, 1, 1]) == 0.0
    assert abs(float(grads[2][0, 5, 0, 2])) < 1e-30


def test_traces_under_torch_compile_aot_eager(rosa):
    # reference tests/test_soft_cuda.py:1010-1048
    query, key, value, grad_output = device_inputs(T=20, seed=12)

    def step(q, k, v):
        return rosa.rosa_soft(q, k, v, max_suffix_length=6, scale=1.1)

    compiled = torch.compile(step, backend="aot_eager", fullgraph=True)
    eager_leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
    traced_leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
    eager = step(*eager_leaves)
    traced = compiled(*traced_leaves)
    assert torch.equal(eager, traced)
    go = grad_output.to(DEVICE)
    for a, b in zip(
        torch.autograd.grad(eager, eager_leaves, go), torch.autograd.grad(traced, traced_leaves, go)
    ):
        torch.testing.assert_close(a, b, rtol=2e-6, atol=2e-7)


def test_autocast_gradscaler_and_checkpoint_replay(rosa):
    # reference tests/test_soft_integration.py:15-174
    from torch.utils.checkpoint import checkpoint

    torch.manual_seed(0)
    width, heads, symbol, value_dim = 32, 4, 8, 8
    project = torch.nn.Linear(width, heads * symbol * 2 + 2 * value_dim).to(DEVICE)
    tokens = torch.randn(2, 40, width, device=DEVICE)

    def block(x, dropout_p):
        mixed = project(x)
        q, k, v = mixed.split([heads * symbol, heads * symbol, 2 * value_dim], dim=-1)
        q = q.reshape(2, 40, heads, symbol)
        k = k.reshape(2, 40, heads, symbol)
        v = v.reshape(2, 40, 2, value_dim)
        return rosa.rosa_soft(q, k, v, max_suffix_length=8, dropout_p=dropout_p)

    scaler = torch.amp.GradScaler("cuda")
    with torch.autocast("cuda", dtype=torch.float16):
        output = block(tokens, 0.0)
        loss = output.float().square().mean()
    assert output.dtype == torch.float16
    scaler.scale(loss).backward()
    assert all(torch.isfinite(p.grad).all() for p in project.parameters())
    assert any(float(p.grad.abs().sum()) > 0 for p in project.parameters())

    def run(use_checkpoint):
        project.zero_grad()
        torch.cuda.manual_seed(31)
        x = tokens.clone().requires_grad_()
        if use_checkpoint:
            out = checkpoint(block, x, 0.4, use_reentrant=False, preserve_rng_state=True)
        else:
            out = block(x, 0.4)
        out.float().square().mean().backward()
        return out.detach(), x.grad.clone(), project.weight.grad.clone()

    plain, replayed = run(False), run(True)
    assert torch.equal(plain[0], replayed[0])
    torch.testing.assert_close(plain[1], replayed[1], rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(plain[2], replayed[2], rtol=1e-5, atol=1e-7)


def test_no_grad_forward_replays_from_a_hip_graph(rosa):
    # every replay is checked against eager work done between the replays, on new inputs
    # written in place
    query, key, value, _ = device_inputs(T=300, seed=21)
    q, k, v = (t.to(DEVICE) for t in (query, key, value))
    generator = torch.Generator(device=DEVICE).manual_seed(5)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            rosa.rosa_soft(q, k, v, max_suffix_length=32)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = rosa.rosa_soft(q, k, v, max_suffix_length=32)
        for _ in range(4):
            q.copy_(torch.randn(q.shape, device=DEVICE, generator=generator))
            want = rosa.rosa_soft(q, k, v, max_suffix_length=32).clone()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(captured, want)


def test_recording_the_training_step_into_a_graph_is_refused(rosa):
    query, key, value, _ = device_inputs(seed=22)
    leaves = [t.to(DEVICE).requires_grad_() for t in (query, key, value)]
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="cannot be recorded into a HIP graph"):
        with torch.cuda.graph(graph):
            rosa.rosa_soft(*leaves, max_suffix_length=12)
    # the stream is usable again afterwards
    output = rosa.rosa_soft(*leaves, max_suffix_length=12)
    assert output.shape == (2, 48, 4, 5)
    # the exported backward operator refuses by itself, before it allocates or launches
    q, k, v = (t.detach() for t in leaves)
    _, pq, pk = torch.ops.rosa_soft.hard_forward(q, k, v, 12)
    grad_output = torch.ones_like(output.detach())
    empty = torch.empty(0, dtype=torch.int64, device=DEVICE)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="cannot be recorded into a HIP graph"):
        with torch.cuda.graph(graph):
            torch.ops.rosa_soft.surrogate_vjp_masked(
                q, k, v, grad_output, pq, pk, empty, 12, 1.0, 0.0, 3.0, 7)
    gradients = torch.ops.rosa_soft.surrogate_vjp_masked(
        q, k, v, grad_output, pq, pk, empty, 12, 1.0, 0.0, 3.0, 7)
    assert all(bool(torch.isfinite(g).all()) for g in gradients)
