"""The summaries of rosa_soft_amd/diagnostics.py: the gradient summary with the cases of the
reference's tests (tests/test_diagnostics.py:205-253) on the CPU, and the summary of the selected
routes against a direct count on the oracle's routes on the GPU."""

import math

import pytest
import torch

from rosa_soft_amd.diagnostics import (summarize_hard_routes, summarize_rosa_soft_gradients,
                                       inspect_hard_routes)
from tests.conftest import nonzero_randn


def test_gradient_summary_reports_scale_support_and_feature_balance():
    summary = summarize_rosa_soft_gradients(
        torch.tensor([[[[1.0, 0.0], [3.0, 0.0]]]]),
        torch.tensor([[[[0.0, 2.0], [0.0, 4.0]]]]),
        torch.ones(1, 1, 1, 2),
    )
    values = summary.as_float_dict()
    assert summary.query.l2_norm == torch.sqrt(torch.tensor(10.0))
    assert summary.key.l2_norm == torch.sqrt(torch.tensor(20.0))
    assert summary.value.l2_norm == torch.sqrt(torch.tensor(2.0))
    assert summary.query.finite_fraction == 1 and summary.value.finite_fraction == 1
    assert summary.query.nonzero_fraction == 0.5 and summary.key.nonzero_fraction == 0.5
    assert summary.value.nonzero_fraction == 1
    assert summary.query.feature_rms_cv == 1 and summary.key.feature_rms_cv == 1
    assert summary.value.feature_rms_cv == 0
    assert summary.query.rms == torch.sqrt(torch.tensor(2.5)) and summary.key.max_abs == 4
    assert summary.qk_to_value_norm_ratio == torch.sqrt(torch.tensor(15.0))
    assert set(values) == {
        f"{role}_{metric}" for role in ("query", "key", "value")
        for metric in summary.query.__dataclass_fields__
    } | {"qk_to_value_norm_ratio"}


def test_gradient_summary_surfaces_non_finite_elements_and_a_zero_value_gradient():
    summary = summarize_rosa_soft_gradients(
        torch.tensor([1.0, float("nan")]), torch.tensor([float("inf"), 0.0]), torch.zeros(2))
    assert summary.query.finite_fraction == 0.5 and summary.key.finite_fraction == 0.5
    assert summary.query.l2_norm == 1 and summary.key.l2_norm == 0
    assert summary.value.l2_norm == 0
    assert math.isinf(float(summary.qk_to_value_norm_ratio))
    nothing = summarize_rosa_soft_gradients(torch.zeros(3), torch.zeros(3), torch.zeros(3))
    assert math.isnan(float(nothing.qk_to_value_norm_ratio))
    lost = summarize_rosa_soft_gradients(torch.full((2,), float("nan")), torch.ones(2), torch.ones(2))
    assert math.isnan(float(lost.query.l2_norm)) and lost.query.finite_fraction == 0


@pytest.mark.gpu
@pytest.mark.parametrize("packed", [False, True])
def test_summary_of_the_selected_routes_equals_a_direct_count(c_oracle, packed):
    device = torch.device("cuda:0")
    heads, bits, window = 3, 3, 6
    if packed:
        lengths = [40, 0, 1, 90]
        offsets = [0, 40, 40, 41, 131]
        query = nonzero_randn((131, heads, bits), seed=1)
        key = nonzero_randn((131, heads, bits), seed=2)
        value = nonzero_randn((131, 1, 4), seed=3)
        _, want_routes = c_oracle.varlen_hard_forward(query, key, value, offsets, window)  # [H, N]
        want_routes = want_routes.t()
        local = torch.cat([torch.arange(n) for n in lengths]).unsqueeze(-1)
        cu_seqlens = torch.tensor(offsets, dtype=torch.int32, device=device)
    else:
        query = nonzero_randn((2, 70, heads, bits), seed=1)
        key = nonzero_randn((2, 70, heads, bits), seed=2)
        value = nonzero_randn((2, 70, 1, 4), seed=3)
        _, want_routes, _ = c_oracle.hard_forward(query, key, value, window)  # [B, H, T]
        want_routes = want_routes.permute(0, 2, 1)
        local = torch.arange(70).unsqueeze(-1)
        cu_seqlens = None
    _, inspection = inspect_hard_routes(query.to(device), key.to(device), value.to(device),
                                        cu_seqlens, max_suffix_length=window)
    summary = summarize_hard_routes(inspection, query.to(device), key.to(device), cu_seqlens,
                                    quantile=0.9)
    assert torch.equal(inspection.selected_route_indices.cpu(), want_routes)
    routed = want_routes > 0
    lag = (local - want_routes)[routed].float().mean()
    assert summary.route_rows == want_routes.numel()
    torch.testing.assert_close(summary.hard_nonnull_route_fraction.cpu(), routed.float().mean())
    torch.testing.assert_close(summary.hard_route_lag_mean.cpu(), lag)
    assert int(summary.max_exact_suffix_length) == int(inspection.selected_suffix_lengths.max())
    assert 1 <= int(summary.max_exact_suffix_length) <= window
    for name, logits in (("query", query), ("key", key)):
        margins = logits.abs()
        values = summary.as_float_dict()
        assert values[f"{name}_positive_fraction"] == pytest.approx(float((logits > 0).float().mean()))
        per_bit = (logits > 0).float().flatten(0, -2).mean(0)
        assert values[f"{name}_bit_imbalance"] == pytest.approx(float((2 * (per_bit - 0.5).abs()).mean()), rel=1e-5)
        assert values[f"{name}_sign_margin_mean"] == pytest.approx(float(margins.mean()), rel=1e-5)
        assert values[f"{name}_sign_margin_low_quantile"] == pytest.approx(
            float(torch.quantile(margins.flatten(), 0.1)), rel=1e-5)
        assert values[f"{name}_softsign_derivative_mean"] == pytest.approx(
            float((1 + margins).square().reciprocal().mean()), rel=1e-5)
    with pytest.raises(ValueError, match="quantile"):
        summarize_hard_routes(inspection, query, key, cu_seqlens, quantile=1.5)
    with pytest.raises(TypeError, match="quantile"):
        summarize_hard_routes(inspection, query, key, cu_seqlens, quantile=True)


def test_quantile_beyond_the_size_limit_of_torch_quantile_interpolates_the_same_way():
    from rosa_soft_amd.diagnostics import _quantile

    generator = torch.Generator().manual_seed(5)
    small = torch.rand(1000, generator=generator)
    for q in (0.0, 0.05, 0.5, 0.999, 1.0):
        ordered = small.sort().values
        position = q * (small.numel() - 1)
        low = int(position)
        high = min(low + 1, small.numel() - 1)
        by_hand = torch.lerp(ordered[low], ordered[high], position - low)
        torch.testing.assert_close(_quantile(small, q), by_hand)
    large = torch.rand((1 << 24) + 5, generator=generator)
    assert 0.049 < float(_quantile(large, 0.05)) < 0.051
