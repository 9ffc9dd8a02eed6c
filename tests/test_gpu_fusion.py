"""The operator's neighbours in the reference's caller (examples/fit_soft_reference.py:374-417):
the hard forward from symbol words a projection has already packed, and the output projection
fed with the bit form of the operator's result."""

import pytest
import torch

from tests.conftest import nonzero_randn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cabi():
    from rosa_soft_amd import cabi as module

    module.load()
    return module


def _inputs(shape, value_shape, dtype, seed):
    device = torch.device("cuda:0")
    query = nonzero_randn(shape, dtype=dtype, seed=seed).to(device)
    key = nonzero_randn(shape, dtype=dtype, seed=seed + 1).to(device)
    value = nonzero_randn(value_shape, dtype=dtype, seed=seed + 2).to(device)
    return query, key, value


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_forward_from_packed_words_equals_the_forward(cabi, dtype):
    # few symbol bits, so that most rows find a route
    query, key, value = _inputs((2, 300, 4, 3), (2, 300, 2, 10), dtype, 5)
    output, packed_q, packed_k, routes = cabi.hard_forward(query, key, value, 7)
    again, routes_again = cabi.hard_forward_words(packed_q, packed_k, value, 7, symbol_bits=3)
    assert torch.equal(again, output) and torch.equal(routes_again, routes)
    sign_words, routed = cabi.hard_forward_bits(query, key, value, 7)
    words_again, routed_again, _ = cabi.hard_forward_words(packed_q, packed_k, value, 7,
                                                           symbol_bits=3, as_bits=True)
    assert torch.equal(words_again, sign_words) and torch.equal(routed_again, routed)
    assert int((routes > 0).sum()) > 0 and int((routes == 0).sum()) > 0


def test_packed_forward_from_packed_words(cabi):
    lengths = [1, 70, 0, 129]
    tokens = sum(lengths)
    cu_seqlens = torch.tensor([0, 1, 71, 71, 200], dtype=torch.int32, device="cuda:0")
    query, key, value = _inputs((tokens, 2, 2), (tokens, 2, 8), torch.float16, 9)
    output, packed_q, packed_k, routes = cabi.hard_forward(query, key, value, 5, cu_seqlens)
    again, routes_again = cabi.hard_forward_words(packed_q, packed_k, value, 5, symbol_bits=2,
                                                  cu_seqlens=cu_seqlens)
    assert torch.equal(again, output) and torch.equal(routes_again, routes)


def _projection_reference(cabi, sign_words, routed, value_dim, weight, residual):
    expanded = cabi.expand_output_bits(sign_words, routed, value_dim, torch.float32)
    product = expanded.flatten(-2) @ weight.float().t()
    return product + (residual.float() if residual is not None else 0.0)


@pytest.mark.parametrize("heads,value_dim,width,tokens_shape,with_residual", [
    (64, 8, 128, (2, 200), True),       # the metric shape's heads: four heads per 32-wide step
    (8, 16, 64, (1, 300), False),
    (4, 32, 192, (3, 129), True),
    (32, 64, 256, (1, 513), True),      # configuration 3's heads: two steps per head
    (2, 96, 64, (1, 70), False),        # three words per head
])
def test_projection_of_the_bit_form_matches_the_expanded_product(cabi, heads, value_dim, width,
                                                                  tokens_shape, with_residual):
    device = torch.device("cuda:0")
    batch, length = tokens_shape
    # two symbol bits: a good share of the rows takes a route, the rest the null route
    query, key, value = _inputs((batch, length, heads, 2), (batch, length, heads, value_dim),
                                torch.bfloat16, 21)
    sign_words, routed = cabi.hard_forward_bits(query, key, value, 9)
    assert 0 < int((routed == 1).sum()) < routed.numel()
    generator = torch.Generator(device=device).manual_seed(3)
    weight = (torch.randn(width, heads * value_dim, device=device, generator=generator) /
              (heads * value_dim) ** 0.5).to(torch.bfloat16)
    residual = (torch.randn(batch, length, width, device=device, generator=generator)
                .to(torch.bfloat16) if with_residual else None)
    got = cabi.project_routed_bits(sign_words, routed, value_dim, weight, residual)
    want = _projection_reference(cabi, sign_words, routed, value_dim, weight, residual)
    assert got.shape == want.shape and got.dtype == torch.bfloat16
    # products of +-1 or 0 with bfloat16 weights are exact and sums are float32: the only
    # rounding is that of the result to bfloat16
    torch.testing.assert_close(got.float(), want, rtol=2.0 ** -8, atol=1e-6 * float(want.abs().max()))


def test_projection_at_the_shape_of_configuration_3(cabi):
    device = torch.device("cuda:0")
    query, key, value = _inputs((4, 4096, 32, 16), (4, 4096, 32, 64), torch.bfloat16, 33)
    sign_words, routed = cabi.hard_forward_bits(query, key, value, 32)
    generator = torch.Generator(device=device).manual_seed(4)
    weight = (torch.randn(2048, 2048, device=device, generator=generator) / 45.0).to(torch.bfloat16)
    residual = torch.randn(4, 4096, 2048, device=device, generator=generator).to(torch.bfloat16)
    got = cabi.project_routed_bits(sign_words, routed, 64, weight, residual)
    want = _projection_reference(cabi, sign_words, routed, 64, weight, residual)
    torch.testing.assert_close(got.float(), want, rtol=2.0 ** -8, atol=1e-6 * float(want.abs().max()))


def test_projection_refuses_shapes_it_does_not_tile(cabi):
    device = torch.device("cuda:0")
    routed = torch.ones(4, 3, dtype=torch.uint8, device=device)
    words = torch.zeros(4, 3, 1, dtype=torch.int32, device=device)
    weight = torch.zeros(64, 3 * 12, dtype=torch.bfloat16, device=device)
    with pytest.raises(RuntimeError, match="value width"):
        cabi.project_routed_bits(words, routed, 12, weight)
    weight = torch.zeros(48, 3 * 32, dtype=torch.bfloat16, device=device)
    with pytest.raises(RuntimeError, match="multiple of 64"):
        cabi.project_routed_bits(words, routed, 32, weight)


def test_projection_refuses_pointers_it_cannot_load_in_whole_vectors(cabi):
    device = torch.device("cuda:0")
    routed = torch.ones(8, 4, dtype=torch.uint8, device=device)
    words = torch.zeros(8, 4, 1, dtype=torch.int32, device=device)
    # a contiguous matrix that starts 2 bytes into its allocation
    weight = torch.zeros(64 * 32 + 1, dtype=torch.bfloat16, device=device)[1:].view(64, 32)
    assert weight.is_contiguous() and weight.data_ptr() % 16 != 0
    with pytest.raises(RuntimeError, match="aligned"):
        cabi.project_routed_bits(words, routed, 8, weight)
