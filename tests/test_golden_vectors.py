"""Checks both CPU oracles against vectors written by the reference's oracle.

``tests/golden/reference_vectors.npz`` was produced by
``tests/golden/make_reference_vectors.py`` from the reference's pure-PyTorch
operator; it pins the two things no closed form reaches: the keep-mask bit
pattern and the end-to-end gradient composition (dense and packed).
"""

import os

import numpy as np
import pytest
import torch

from oracle import rosa_oracle as ro
from tests.golden import make_reference_vectors as gold

VECTORS = np.load(os.path.join(os.path.dirname(gold.__file__), "reference_vectors.npz"))

# gradient tolerances against the reference's float32 dense autograd
TOLERANCE = {
    "float32": dict(rtol=2e-4, atol=2e-6),
    "float16": dict(rtol=3e-3, atol=3e-3),
    "bfloat16": dict(rtol=2e-2, atol=2e-2),
}


@pytest.mark.parametrize(
    "name,seed,p,batch_offset,batch,heads,rows,routes",
    [
        ("mask_a", 7, 0.5, 0, 1, 1, 1, 4096),
        ("mask_b", 0x0123456789ABCDEF, 0.1, 3, 2, 5, 9, 33),
        ("mask_c", (1 << 62) + 12345, 0.9, 40, 1, 64, 17, 17),
    ],
)
def test_keep_mask_bit_pattern(name, seed, p, batch_offset, batch, heads, rows, routes, c_oracle):
    expected = np.unpackbits(VECTORS[name])[: batch * heads * rows * routes].astype(bool)
    expected = expected.reshape(batch, heads, rows, routes)
    batch_ids = [batch_offset + b for b in range(batch)]
    got = ro.dropout_keep_mask(seed, p, batch_ids, range(heads), rows, routes)
    assert np.array_equal(got, expected)
    # the C form, sampled
    rng = np.random.default_rng(0)
    for _ in range(200):
        b, h, t, a = (int(rng.integers(n)) for n in (batch, heads, rows, routes))
        u = c_oracle.dropout_uniform(seed, batch_ids[b], h, t, a)
        assert (np.float32(u) >= np.float32(p)) == bool(expected[b, h, t, a])


@pytest.mark.parametrize("name", sorted(gold.DENSE_CASES))
def test_dense_end_to_end_matches_reference(name, c_oracle):
    case = gold.DENSE_CASES[name]
    B, T, H, D, Hv, Dv, W, scale, p, ms, dtype, seed = case
    q, k, v, go = gold.dense_inputs(case)
    controls = dict(max_suffix_length=min(W, T), scale=scale, dropout_p=p, mismatch_scale=ms, seed=seed)
    expected_out = torch.from_numpy(VECTORS[name + "/out"].astype(np.float32))
    out_py, _, _ = ro.hard_forward(q, k, v, min(W, T))
    out_c, _, _ = c_oracle.hard_forward(q, k, v, W)
    assert torch.equal(out_py.float(), expected_out)
    assert torch.equal(out_c.float(), expected_out)
    streamed = c_oracle.surrogate_vjp(q, k, v, go, **controls)
    dense = ro.surrogate_vjp(q, k, v, go, compute_dtype=torch.float64, **controls) if T <= 64 else None
    for index, label in enumerate(("gq", "gk", "gv")):
        want = torch.from_numpy(VECTORS[name + "/" + label]).double()
        torch.testing.assert_close(streamed[index], want, **TOLERANCE[dtype])
        if dense is not None:
            torch.testing.assert_close(dense[index], want, **TOLERANCE[dtype])


@pytest.mark.parametrize("name", sorted(gold.VARLEN_CASES))
def test_packed_end_to_end_matches_reference(name, c_oracle):
    case = gold.VARLEN_CASES[name]
    lengths, H, D, Hv, Dv, W, scale, p, ms, dtype, _ = case
    q, k, v, go = gold.varlen_inputs(case)
    offsets = [0, *np.cumsum(lengths).tolist()]
    seed = int(VECTORS[name + "/seed"][0])
    out, _ = c_oracle.varlen_hard_forward(q, k, v, offsets, W)
    assert torch.equal(out.float(), torch.from_numpy(VECTORS[name + "/out"].astype(np.float32)))
    grads = c_oracle.varlen_surrogate_vjp(
        q, k, v, offsets, go, max_suffix_length=W, scale=scale, dropout_p=p,
        mismatch_scale=ms, seed=seed,
    )
    for index, label in enumerate(("gq", "gk", "gv")):
        want = torch.from_numpy(VECTORS[name + "/" + label]).double()
        torch.testing.assert_close(grads[index], want, **TOLERANCE[dtype])
