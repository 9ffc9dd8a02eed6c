"""Writes the golden vectors in this folder from the reference's own oracle.

Run once, by hand, in a container that has the reference checkout:

    python tests/golden/make_reference_vectors.py [/root/reference]

It imports the reference's pure-PyTorch oracle (``rosa_soft/soft_reference.py``)
only for the two things that no known answer, closed form or brute force in
``tests/test_oracle_known_answers.py`` can pin:

1. the exact keep-mask bit pattern of its attention dropout for given
   ``(seed, batch, head, row, route)`` coordinates (a swapped coordinate order
   or salt would pass every statistical check), and
2. its end-to-end gradients (composition order of the ``-log t`` correction,
   null score, dropout normalisation, grouped-head summation), dense and
   packed, with and without dropout, float32 and bfloat16.

Inputs are regenerated from seeds by ``tests/test_golden_vectors.py`` with the
same generator calls, so only outputs are stored.  The files hold numbers
only; nothing of the reference's code is written anywhere.
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def seeded(shape, seed, dtype=torch.float32):
    generator = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=generator, dtype=torch.float32).to(dtype)


DENSE_CASES = {
    # name: (B, T, H, D, Hv, Dv, W, scale, p, ms, dtype, seed)
    "config1_fp32": (1, 256, 4, 4, 4, 8, 16, 1.0, 0.0, 3.0, "float32", None),
    "grouped_dropout_fp32": (2, 48, 4, 8, 2, 5, 12, 1.5, 0.25, 3.0, "float32", 0x1F2E3D4C5B6A7988),
    "wide_bf16": (1, 40, 2, 32, 1, 6, 40, 0.7, 0.0, 9.0, "bfloat16", None),
    "narrow_fp16_dropout": (1, 64, 2, 1, 2, 3, 64, 1.0, 0.5, 2.0, "float16", 77),
}

VARLEN_CASES = {
    # name: (lengths, H, D, Hv, Dv, W, scale, p, ms, dtype, seed)
    "varlen_dropout_fp32": ([7, 0, 19, 1, 12], 4, 4, 2, 3, 6, 1.0, 0.3, 3.0, "float32", 0xABCDEF0123456789 & (2**63 - 1)),
}


def dense_inputs(case):
    B, T, H, D, Hv, Dv, W, scale, p, ms, dtype, seed = case
    dt = getattr(torch, dtype)
    return (
        seeded((B, T, H, D), 1000, dt),
        seeded((B, T, H, D), 1001, dt),
        seeded((B, T, Hv, Dv), 1002, dt),
        seeded((B, T, H, Dv), 1003, dt),
    )


def varlen_inputs(case):
    lengths, H, D, Hv, Dv, W, scale, p, ms, dtype, seed = case
    dt = getattr(torch, dtype)
    N = sum(lengths)
    return (
        seeded((N, H, D), 2000, dt),
        seeded((N, H, D), 2001, dt),
        seeded((N, Hv, Dv), 2002, dt),
        seeded((N, H, Dv), 2003, dt),
    )


def main():
    reference_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    sys.dont_write_bytecode = True
    sys.path.insert(0, reference_root)
    from rosa_soft import soft_reference as ref  # noqa: E402

    arrays = {}

    # 1. keep masks
    mask_cases = {
        "mask_a": (7, 0.5, 0, 1, 1, 1, 4096),
        "mask_b": (0x0123456789ABCDEF, 0.1, 3, 2, 5, 9, 33),
        "mask_c": ((1 << 62) + 12345, 0.9, 40, 1, 64, 17, 17),
    }
    for name, (seed, p, batch_offset, batch, heads, rows, routes) in mask_cases.items():
        weights = torch.ones(batch, heads, rows, routes)
        dropped = ref._apply_attention_dropout(
            weights, p, torch.tensor(seed, dtype=torch.int64), batch_offset
        )
        arrays[name] = np.packbits(dropped.ne(0).numpy().reshape(-1))

    # 2. dense end-to-end
    for name, case in DENSE_CASES.items():
        B, T, H, D, Hv, Dv, W, scale, p, ms, dtype, seed = case
        q, k, v, go = dense_inputs(case)
        leaves = [x.clone().requires_grad_() for x in (q, k, v)]
        seed_tensor = (
            torch.empty(0, dtype=torch.int64)
            if seed is None
            else torch.tensor(seed, dtype=torch.int64)
        )
        out = ref._rosa_soft_reference_with_seed(
            *leaves, seed_tensor, min(W, T), scale, p, ms, 0
        )
        grads = torch.autograd.grad(out, leaves, go)
        arrays[name + "/out"] = out.detach().float().numpy().astype(np.int8)
        for label, grad in zip(("gq", "gk", "gv"), grads):
            arrays[name + "/" + label] = grad.float().numpy()

    # 3. packed end-to-end through the public packed entry point; the seed it
    # draws from the global CPU generator is reproduced by drawing it first.
    for name, case in VARLEN_CASES.items():
        lengths, H, D, Hv, Dv, W, scale, p, ms, dtype, seed = case
        q, k, v, go = varlen_inputs(case)
        offsets = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32)
        torch.manual_seed(4242)
        drawn = int(torch.randint(0, torch.iinfo(torch.int64).max, (), dtype=torch.int64))
        torch.manual_seed(4242)
        leaves = [x.clone().requires_grad_() for x in (q, k, v)]
        out = ref.rosa_soft_varlen_reference(
            *leaves, offsets, max_suffix_length=W, scale=scale, dropout_p=p, mismatch_scale=ms
        )
        grads = torch.autograd.grad(out, leaves, go)
        arrays[name + "/seed"] = np.asarray([drawn], dtype=np.int64)
        arrays[name + "/out"] = out.detach().float().numpy().astype(np.int8)
        for label, grad in zip(("gq", "gk", "gv"), grads):
            arrays[name + "/" + label] = grad.float().numpy()

    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **arrays)
    print("wrote", path, os.path.getsize(path), "bytes;", len(arrays), "arrays")


if __name__ == "__main__":
    main()
