"""Behaviours the reference's own device tests pin, restated against the HIP operators: what the
backward controls may change (tests/test_soft_cuda.py:666-690), that the dense backward finds a
useful route by gradient descent (:716-743), the window clamp and the parameter checks
(:849-885), loss scaling on a float16 tail (tests/test_soft_integration.py:175-216), and, for
packed sequences, that nothing crosses a sequence boundary and that the first value of a sequence
is never routed (tests/test_soft_varlen.py:78-147), grouped heads with non-contiguous inputs and
offsets (:923-955), and the sequence-count limit (:234-254)."""

import math

import pytest
import torch

from tests.conftest import nonzero_randn

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"


@pytest.fixture(scope="module")
def rosa():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import rosa_soft_amd

    assert rosa_soft_amd.BUILD_CAPABILITIES.variant == "rocm"
    return rosa_soft_amd


def _gradients(operator, inputs, grad_output, *extra, **controls):
    leaves = tuple(t.detach().clone().to(DEVICE).requires_grad_() for t in inputs)
    output = operator(*leaves, *extra, **controls)
    gradients = torch.autograd.grad(output, leaves, grad_output.to(DEVICE))
    return output.detach(), gradients


def test_backward_controls_change_the_gradients_and_never_the_output(rosa):
    inputs = (nonzero_randn((1, 10, 2, 5), seed=70), nonzero_randn((1, 10, 2, 5), seed=71),
              nonzero_randn((1, 10, 1, 3), seed=72))
    grad_output = nonzero_randn((1, 10, 2, 3), seed=73)

    def run(scale, mismatch_scale):
        return _gradients(rosa.rosa_soft, inputs, grad_output, max_suffix_length=6, scale=scale,
                          mismatch_scale=mismatch_scale)

    base_output, base_gradients = run(2.0, 3.0)
    for output, gradients in (run(0.7, 3.0), run(2.0, 7.0)):
        assert torch.equal(output, base_output)
        assert any(not torch.allclose(got, base) for got, base in zip(gradients, base_gradients))


@pytest.mark.parametrize("seed", range(6))
def test_gradient_descent_on_one_query_logit_finds_the_useful_route(rosa, seed):
    # the last row can only match the first key, whose successor holds the wanted value, if its
    # one query logit turns positive: the surrogate gradient must push it there within six steps
    torch.manual_seed(seed)
    length = 33
    logit = torch.nn.Parameter(torch.tensor(-0.5, device=DEVICE))
    optimizer = torch.optim.SGD([logit], lr=1.0)
    steps = 0
    for steps in range(1, 13):
        optimizer.zero_grad(set_to_none=True)
        query = torch.ones(1, length, 1, 1, device=DEVICE)
        query[0, -1, 0, 0] = logit
        key = -torch.ones_like(query)
        key[:, 0] = 1
        value = -torch.ones_like(query)
        value[:, 1] = 1
        output = rosa.rosa_soft(query, key, value, max_suffix_length=1, scale=2.0, mismatch_scale=3.0)
        (output[0, -1, 0, 0] - 1).square().backward()
        optimizer.step()
        if logit.item() > 0:
            break
    assert steps <= 6 and logit.item() > 0


def test_a_window_beyond_the_sequence_is_the_whole_sequence_and_must_be_an_integer(rosa):
    inputs = tuple(t.to(DEVICE) for t in (nonzero_randn((1, 7, 1, 3), seed=110),
                                          nonzero_randn((1, 7, 1, 3), seed=111),
                                          nonzero_randn((1, 7, 1, 2), seed=112)))
    whole = rosa.rosa_soft(*inputs, max_suffix_length=7)
    huge = rosa.rosa_soft(*inputs, max_suffix_length=10 ** 9)
    assert torch.equal(whole, huge)
    for invalid in (True, 1.5):
        with pytest.raises(TypeError, match="integer"):
            rosa.rosa_soft(*inputs, max_suffix_length=invalid)


@pytest.mark.parametrize("controls,message", [
    ({"max_suffix_length": 0}, "max_suffix_length"),
    ({"scale": True}, "scale"),
    ({"scale": 0.0}, "scale"),
    ({"scale": 1e-300}, "scale"),
    ({"scale": 1e300}, "scale"),
    ({"dropout_p": True}, "dropout_p"),
    ({"dropout_p": -0.1}, "dropout_p"),
    ({"dropout_p": 1.0}, "dropout_p"),
    ({"dropout_p": math.nan}, "dropout_p"),
    ({"dropout_p": math.inf}, "dropout_p"),
    ({"mismatch_scale": 0.0}, "mismatch_scale"),
    ({"mismatch_scale": True}, "mismatch_scale"),
    ({"mismatch_scale": 1e-300}, "mismatch_scale"),
    ({"mismatch_scale": 1e300}, "mismatch_scale"),
])
def test_controls_outside_their_range_are_rejected_on_the_device_path(rosa, controls, message):
    tensor = torch.ones(1, 5, 1, 1, device=DEVICE)
    with pytest.raises(ValueError, match=message):
        rosa.rosa_soft(tensor, tensor, tensor, **controls)


def _final_row_value_gradient(rosa, dtype, loss_scale=1.0):
    tokens = 40
    query = torch.ones(1, tokens, 1, 4, device=DEVICE, dtype=dtype, requires_grad=True)
    key = torch.ones_like(query, requires_grad=True)
    value = torch.arange(tokens, device=DEVICE, dtype=dtype).reshape(1, tokens, 1, 1).requires_grad_()
    output = rosa.rosa_soft(query, key, value, max_suffix_length=32)
    (output[0, -1, 0, 0] * loss_scale).backward()
    return value.grad.detach().float().flatten() / loss_scale


def test_loss_scaling_brings_a_float16_tail_gradient_closer_to_float32(rosa):
    plain = _final_row_value_gradient(rosa, torch.float16)
    scaled = _final_row_value_gradient(rosa, torch.float16, loss_scale=1024.0)
    exact = _final_row_value_gradient(rosa, torch.float32)
    # position zero is the null value and never receives a route gradient
    assert torch.count_nonzero(exact[1:]) == exact.numel() - 1
    assert torch.count_nonzero(scaled[1:]) == scaled.numel() - 1
    assert torch.linalg.vector_norm(scaled - exact) < torch.linalg.vector_norm(plain - exact)


def _offsets(values):
    return torch.tensor(values, dtype=torch.int32, device=DEVICE)


def test_packed_sequences_do_not_see_each_other(rosa):
    inputs = (nonzero_randn((9, 1, 3), seed=10), nonzero_randn((9, 1, 3), seed=11),
              nonzero_randn((9, 1, 2), seed=12))
    grad_output = nonzero_randn((9, 1, 2), seed=13)
    offsets = _offsets([0, 4, 9])

    def run(tensors):
        return _gradients(rosa.rosa_soft_varlen, tensors, grad_output, offsets, max_suffix_length=5,
                          scale=2.0, mismatch_scale=9.0)

    base_output, base_gradients = run(inputs)
    changed = tuple(t.clone() for t in inputs)
    for tensor in changed:
        tensor[:4].mul_(-2.0)
    changed_output, changed_gradients = run(changed)
    assert torch.equal(changed_output[4:], base_output[4:])
    for got, base in zip(changed_gradients, base_gradients):
        # (the sums of the second sequence are the same terms in an order that the atomics choose)
        torch.testing.assert_close(got[4:], base[4:], rtol=1e-5, atol=1e-6 * float(base.abs().max()))
        assert not torch.allclose(got[:4], base[:4])


def test_the_first_value_of_a_packed_sequence_is_never_routed(rosa):
    query = nonzero_randn((7, 1, 2), seed=20).to(DEVICE).requires_grad_()
    key = nonzero_randn((7, 1, 2), seed=21).to(DEVICE).requires_grad_()
    value = nonzero_randn((7, 1, 3), seed=22).to(DEVICE).requires_grad_()
    output = rosa.rosa_soft_varlen(query, key, value, _offsets([0, 1, 4, 7]))
    output.sum().backward()
    assert torch.count_nonzero(output[[0, 1, 4]]) == 0
    assert torch.count_nonzero(value.grad[[0, 1, 4]]) == 0


def test_packed_grouped_heads_with_strided_inputs_and_offsets(rosa, c_oracle):
    total = 11
    query = nonzero_randn((total, 5, 4), seed=60).to(DEVICE).transpose(1, 2).requires_grad_()
    key = nonzero_randn((total, 5, 4), seed=61).to(DEVICE).transpose(1, 2).requires_grad_()
    value = nonzero_randn((total, 3, 2), seed=62).to(DEVICE).transpose(1, 2).requires_grad_()
    storage = _offsets([0, -1, 4, -1, 11])
    offsets = storage[::2]
    assert not offsets.is_contiguous() and not query.is_contiguous()
    output = rosa.rosa_soft_varlen(query, key, value, offsets, max_suffix_length=6)
    output.sum().backward()
    assert output.shape == (total, 4, 3)
    assert all(t.grad is not None and torch.isfinite(t.grad).all() for t in (query, key, value))
    want, _ = c_oracle.varlen_hard_forward(query.detach().cpu().contiguous(),
                                           key.detach().cpu().contiguous(),
                                           value.detach().cpu().contiguous(), [0, 4, 11], 6)
    assert torch.equal(output.detach().cpu(), want)


def test_more_packed_sequences_than_the_kernels_can_index_are_refused(rosa):
    query = torch.ones(1, 1, 2, device=DEVICE)
    value = torch.ones(1, 1, 2, device=DEVICE)
    offsets = torch.zeros(1, dtype=torch.int32, device=DEVICE).expand(2_147_483_521)
    with pytest.raises(RuntimeError, match="number of packed sequences is too large"):
        torch.ops.rosa_soft.hard_forward_varlen(query, query.clone(), value, offsets, 1)


# The shapes and controls of the reference's device tests that aim at single paths of its
# kernels (large value widths with only the query gradient, the query-utility cache, key
# aggregation over 512 and 1 024 rows, a window of one with 64-wide values, dropout, the three
# dtypes): batch, length, heads, bits, value heads, value width, window, scale, dropout,
# mismatch scale, gradient mask (1 query, 2 key, 4 value), dtype
DENSE_SHAPES_OF_THE_REFERENCE = [
    *[(1, 9, 2, 4, 1, width, 6, 1.4, p, 3.0, 1, torch.float32)   # test_soft_cuda.py:210-264
      for width in (32, 64, 128) for p in (0.0, 0.2)],
    (1, 129, 1, 8, 1, 64, 8, 1.4, 0.0, 3.0, 1, torch.float32),    # :267-315
    *[(1, 512, 1, 8, 1, 8, 32, 1.2, p, 3.0, 2, torch.float32) for p in (0.0, 0.2)],   # :318-366
    *[(1, 1024, 1, 8, 1, 8, 32, 1.2, p, 3.0, 3, torch.float32) for p in (0.0, 0.2)],
    *[(1, 67, 2, 8, 1, 64, 1, 1.4, p, 3.0, 4, torch.float32) for p in (0.0, 0.2)],    # :368-420
    *[(1, 9, 2, 4, 1, 3, 6, 1.5, p, 4.0, 7, torch.float32) for p in (0.1, 0.5)],      # :423-466
    *[(1, 7, 2, 5, 1, 3, 5, 1.4, 0.0, 2.6, 7, dtype)                                  # :468-509
      for dtype in (torch.float16, torch.bfloat16)],
]


@pytest.mark.parametrize("case", DENSE_SHAPES_OF_THE_REFERENCE,
                         ids=lambda c: "-".join(str(x).replace("torch.", "") for x in c))
def test_dense_shapes_of_the_reference_device_tests(c_oracle, case):
    from rosa_soft_amd import cabi
    from tests.test_gpu_parity import assert_gradients_close, make_case, run_device

    batch, length, heads, bits, value_heads, width, window, scale, p, ms, mask, dtype = case
    query, key, value, grad_output = make_case(batch, length, heads, bits, value_heads, width,
                                               dtype, seed=length + width)
    seed = 24680 if p > 0 else None
    out, _, _, routes, grads = run_device(cabi, query, key, value, grad_output, window, scale, p,
                                          ms, seed, mask)
    want_out, want_routes, _ = c_oracle.hard_forward(query, key, value, window)
    assert torch.equal(routes.cpu(), want_routes) and torch.equal(out.cpu().float(), want_out.float())
    want = c_oracle.surrogate_vjp(query, key, value, grad_output, max_suffix_length=window,
                                  scale=scale, dropout_p=p, mismatch_scale=ms, seed=seed)
    for bit, got, expected, name in zip((1, 2, 4), grads, want, "qkv"):
        if mask & bit:
            assert_gradients_close(got, expected, f"d{name}")


# lengths, heads, bits, value width, window, scale, dropout, mismatch scale
PACKED_SHAPES_OF_THE_REFERENCE = [
    *[((3, 0, 5, 2), 2, 3, 2, 4, 1.3, p, 7.0) for p in (0.0, 0.2)],   # test_soft_varlen.py:396-480
    *[((256,), 1, 8, 3, 4, 1.2, p, 3.0) for p in (0.0, 0.2)],          # :482-560
    ((256,), 1, 8, 64, 4, 1.2, 0.2, 3.0),                              # :562-640
    ((257,), 2, 8, 3, 9, 1.4, 0.2, 3.0),                               # :642-713
    ((1027,), 1, 4, 1, 2, 1.4, 0.2, 3.0),                              # :715-786
    *[((67,), 2, 8, 64, 9, 1.2, p, 3.0) for p in (0.0, 0.2)],          # :788-862
]


@pytest.mark.parametrize("case", PACKED_SHAPES_OF_THE_REFERENCE, ids=lambda c: str(c))
def test_packed_shapes_of_the_reference_device_tests(c_oracle, case):
    import numpy as np

    from rosa_soft_amd import cabi
    from tests.test_gpu_parity import assert_gradients_close, run_device

    lengths, heads, bits, width, window, scale, p, ms = case
    offsets = [0, *np.cumsum(lengths).tolist()]
    total = offsets[-1]
    query = nonzero_randn((total, heads, bits), seed=40)
    key = nonzero_randn((total, heads, bits), seed=41)
    value = nonzero_randn((total, 1, width), seed=42)
    grad_output = nonzero_randn((total, heads, width), seed=43, floor=0.0)
    seed = 13579 if p > 0 else None
    out, _, _, routes, grads = run_device(cabi, query, key, value, grad_output, window, scale, p,
                                          ms, seed, 7, offsets)
    want_out, want_routes = c_oracle.varlen_hard_forward(query, key, value, offsets, window)
    assert torch.equal(routes.cpu(), want_routes) and torch.equal(out.cpu().float(), want_out.float())
    want = c_oracle.varlen_surrogate_vjp(query, key, value, offsets, grad_output,
                                         max_suffix_length=window, scale=scale, dropout_p=p,
                                         mismatch_scale=ms, seed=seed)
    for got, expected, name in zip(grads, want, "qkv"):
        assert_gradients_close(got, expected, f"d{name}")


@pytest.mark.parametrize("varlen", [False, True])
def test_mixed_precision_projections_and_a_gradient_scaler(rosa, varlen):
    # tests/test_soft_integration.py:15-90: float16 logits out of autocast projections, dropout,
    # a scaled loss, finite parameter gradients, an optimizer step
    torch.manual_seed(3)
    width, heads, bits, value_width, tokens = 6, 2, 3, 2, 9
    projections = [torch.nn.Linear(width, n, device=DEVICE)
                   for n in (heads * bits, heads * bits, value_width)]
    parameters = [p for layer in projections for p in layer.parameters()]
    optimizer = torch.optim.SGD(parameters, lr=0.01)
    scaler = torch.amp.GradScaler("cuda", init_scale=128.0)
    source = torch.randn(tokens, width, device=DEVICE)
    optimizer.zero_grad(set_to_none=True)
    with torch.autocast("cuda", dtype=torch.float16):
        query = projections[0](source).reshape(tokens, heads, bits)
        key = projections[1](source).reshape(tokens, heads, bits)
        value = projections[2](source).reshape(tokens, 1, value_width)
        if varlen:
            output = rosa.rosa_soft_varlen(query, key, value, _offsets([0, 4, tokens]),
                                           max_suffix_length=5, dropout_p=0.1)
        else:
            output = rosa.rosa_soft(query.unsqueeze(0), key.unsqueeze(0), value.unsqueeze(0),
                                    max_suffix_length=5, dropout_p=0.1)
        loss = output.float().square().mean()
    assert query.dtype == torch.float16 and output.dtype == torch.float16
    scaler.scale(loss).backward()
    scaler.unscale_(optimizer)
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in parameters)
    before = [p.detach().clone() for p in parameters]
    scaler.step(optimizer)
    scaler.update()
    assert any(not torch.equal(p, old) for p, old in zip(parameters, before))


@pytest.mark.parametrize("varlen", [False, True])
@pytest.mark.parametrize("dropout_p", [0.0, 0.2])
def test_activation_checkpointing_replays_the_same_outputs_and_gradients(rosa, varlen, dropout_p):
    # tests/test_soft_integration.py:93-172: the recomputed forward draws the same dropout seed
    from torch.utils.checkpoint import checkpoint

    generator = torch.Generator(device=DEVICE).manual_seed(100)
    inputs = (torch.randn(9, 1, 3, generator=generator, device=DEVICE),
              torch.randn(9, 1, 3, generator=generator, device=DEVICE),
              torch.randn(9, 1, 2, generator=generator, device=DEVICE))
    offsets = _offsets([0, 4, 9])

    def operator(*tensors):
        if varlen:
            return rosa.rosa_soft_varlen(*tensors, offsets, max_suffix_length=5, dropout_p=dropout_p)
        return rosa.rosa_soft(*(t.unsqueeze(0) for t in tensors), max_suffix_length=5,
                              dropout_p=dropout_p).squeeze(0)

    def run(use_checkpoint):
        torch.cuda.manual_seed(101)
        leaves = tuple(t.detach().clone().requires_grad_() for t in inputs)
        if use_checkpoint:
            output = checkpoint(operator, *leaves, use_reentrant=False, preserve_rng_state=True)
        else:
            output = operator(*leaves)
        return output.detach(), torch.autograd.grad(output.sum(), leaves)

    direct_output, direct_gradients = run(False)
    replayed_output, replayed_gradients = run(True)
    assert torch.equal(replayed_output, direct_output)
    for replayed, direct in zip(replayed_gradients, direct_gradients):
        torch.testing.assert_close(replayed, direct, rtol=2e-5, atol=2e-6)


def test_training_without_dropout_draws_nothing_from_the_generator_and_repeats(rosa):
    # tests/test_soft_cuda.py:745-769
    inputs = (nonzero_randn((1, 8, 2, 4), seed=90), nonzero_randn((1, 8, 2, 4), seed=91),
              nonzero_randn((1, 8, 1, 3), seed=92))
    grad_output = nonzero_randn((1, 8, 2, 3), seed=93)
    state = torch.cuda.get_rng_state()
    first = _gradients(rosa.rosa_soft, inputs, grad_output, max_suffix_length=5)
    assert torch.equal(state, torch.cuda.get_rng_state())
    torch.cuda.manual_seed(123456)
    second = _gradients(rosa.rosa_soft, inputs, grad_output, max_suffix_length=5)
    assert torch.equal(first[0], second[0])
    for left, right in zip(first[1], second[1]):
        torch.testing.assert_close(left, right, rtol=2e-6, atol=2e-7)


def test_dropout_is_seeded_by_the_generator_and_touches_only_the_backward(rosa):
    # tests/test_soft_cuda.py:772-810
    inputs = (nonzero_randn((1, 8, 2, 4), seed=94), nonzero_randn((1, 8, 2, 4), seed=95),
              nonzero_randn((1, 8, 1, 3), seed=96))
    grad_output = nonzero_randn((1, 8, 2, 3), seed=97)

    def run(seed):
        torch.cuda.manual_seed(seed)
        return _gradients(rosa.rosa_soft, inputs, grad_output, max_suffix_length=5, dropout_p=0.5)

    first, replay, changed = run(98), run(98), run(99)
    assert torch.equal(first[0], replay[0]) and torch.equal(first[0], changed[0])
    for want, got in zip(first[1], replay[1]):
        torch.testing.assert_close(want, got, rtol=2e-6, atol=2e-7)
    assert any(not torch.allclose(want, got) for want, got in zip(first[1], changed[1]))
    state = torch.cuda.get_rng_state()
    with torch.no_grad():
        rosa.rosa_soft(*(t.to(DEVICE) for t in inputs), dropout_p=0.5)
    assert torch.equal(state, torch.cuda.get_rng_state())


def test_strided_inputs_and_a_sequence_of_one_token(rosa):
    # tests/test_soft_cuda.py:813-846
    query = nonzero_randn((2, 3, 9, 4), seed=100).to(DEVICE).transpose(1, 2)
    key = nonzero_randn((2, 3, 9, 4), seed=101).to(DEVICE).transpose(1, 2)
    value = nonzero_randn((2, 1, 9, 5), seed=102).to(DEVICE).transpose(1, 2)
    leaves = tuple(t.requires_grad_() for t in (query, key, value))
    output = rosa.rosa_soft(*leaves, max_suffix_length=7)
    output.backward(torch.randn_like(output))
    assert output.shape == (2, 9, 3, 5)
    assert all(t.grad is not None and torch.isfinite(t.grad).all() for t in leaves)
    single = tuple(torch.ones(2, 1, heads, width, device=DEVICE, requires_grad=True)
                   for heads, width in ((2, 3), (2, 3), (1, 4)))
    single_output = rosa.rosa_soft(*single)
    gradients = torch.autograd.grad(single_output.sum(), single)
    assert torch.equal(single_output, torch.zeros_like(single_output))
    assert all(torch.equal(g, torch.zeros_like(g)) for g in gradients)


def _oracle_gradients(inputs, grad_output, **controls):
    from oracle.rosa_oracle import rosa_soft_oracle

    leaves = tuple(t.detach().clone().cpu().requires_grad_() for t in inputs)
    output = rosa_soft_oracle(*leaves, **controls)
    return output.detach(), torch.autograd.grad(output, leaves, grad_output.cpu())


def test_non_finite_logits_follow_the_policy_of_the_oracle(rosa):
    # tests/test_soft_cuda.py:570-611: infinities and a NaN among the logits and values; the
    # output is the oracle's, the gradients are NaN where the oracle's are and close elsewhere
    inf, nan = math.inf, math.nan
    query = torch.tensor([[[[inf, -0.5]], [[0.4, -inf]], [[nan, -1.0]]]])
    key = torch.tensor([[[[-1.0, inf]], [[-inf, -0.7]], [[0.2, 0.3]]]])
    value = torch.tensor([[[[inf, -1.0]], [[-inf, 0.2]], [[0.5, -0.4]]]])
    grad_output = nonzero_randn((1, 3, 1, 2), seed=60)
    controls = dict(max_suffix_length=3, scale=1.0, mismatch_scale=3.0)
    want, want_gradients = _oracle_gradients((query, key, value), grad_output, **controls)
    got, got_gradients = _gradients(rosa.rosa_soft, (query, key, value), grad_output, **controls)
    assert torch.equal(got.cpu(), want)
    for observed, reference in zip(got_gradients, want_gradients):
        observed = observed.cpu()
        assert torch.equal(torch.isnan(observed), torch.isnan(reference))
        finite = torch.isfinite(observed) & torch.isfinite(reference)
        torch.testing.assert_close(observed[finite], reference[finite], rtol=2e-5, atol=2e-6)


def test_softsign_jacobian_from_tiny_to_saturated_logits(rosa):
    # tests/test_soft_cuda.py:614-663: magnitudes from 1e-6 to 1e8 in every position
    magnitudes = torch.tensor([1e-6, -1e-3, 0.2, -1.0, 10.0, -100.0, 1e4, -1e8])
    length = magnitudes.numel()
    query = torch.stack([magnitudes.roll(i) for i in range(length)]).reshape(1, length, 1, -1)
    key = torch.stack([magnitudes.flip(0).roll(i) for i in range(length)]).reshape_as(query)
    value = torch.stack([magnitudes[:5].roll(i) for i in range(length)]).reshape(1, length, 1, 5)
    grad_output = torch.stack([(magnitudes[:5].abs() + 1e-4).roll(-i)
                               for i in range(length)]).reshape_as(value)
    controls = dict(max_suffix_length=7, scale=1.7, mismatch_scale=3.0)
    _, want_gradients = _oracle_gradients((query, key, value), grad_output, **controls)
    _, got_gradients = _gradients(rosa.rosa_soft, (query, key, value), grad_output, **controls)
    for observed, reference in zip(got_gradients, want_gradients):
        torch.testing.assert_close(observed.cpu(), reference, rtol=4e-5, atol=3e-6)
