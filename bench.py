"""Throughput of the rosa_soft training step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload metric]

A step is one forward + backward of the public operator over one batch of
synthetic inputs already resident in HBM: ``rosa_soft`` (or
``rosa_soft_varlen``), loss ``output.float().square().mean()``, ``backward()``.
The default workload is the one the headline metric is quoted on:
B=2, T=4096, H=64, D=8 float32 with the remaining controls of the reference's
README configuration (value_heads=16, value_dim=8, max_suffix_length=128,
dropout_p=0.1, mismatch_scale=3.0).  One JSON line is printed.

Besides whole-step tokens/s the line carries

* ``fwd_tokens_per_s``: forward-only (no-grad) tokens/s;
* ``roofline``: the dominant kernel (``vjp_gradients``) priced by the matrix flops it
  performs, ``2 * pairs * (2 D + 2 Dv)`` (utilities, dV, dK, dQ), over its average launch
  time, measured with HIP events recorded by the library on the stream the kernel runs on,
  against the MI355X fp32 matrix peak; the same for the row-statistics kernel
  (``2 * pairs * Dv``) and for the whole backward (``2 * pairs * (3 D + 2 Dv)`` over the sum
  of its stages); ``traffic`` and ``issue`` are counter figures read from the rocprofv3
  summaries under ``profiles/`` for this workload (absent where none was taken);
* ``kernels``: average milliseconds and achieved HBM GB/s (algorithmic bytes)
  of every stage;
* ``configs`` (default workload only): ms per step, forward ms and the roofline fractions
  of configurations 1 to 5, timed by the same run;
* ``cpu_baseline``: the float64 C oracle timed on a bounded slice of the same workload on
  this box's host cores and scaled by pair count, with ``pytorch`` (the pure-PyTorch
  restatement of ``rosa_soft_reference``, forward + backward, configuration 1 at full
  shape) and ``router`` (the reference's own CPU ``RosaRuntime`` built from its source,
  forward only, the metric shape's 8-bit symbols) beside it.
"""

from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FP32_MATRIX_PEAK_TFLOPS = 157.3
# vector ALU: 256 CUs x 4 SIMDs x 16 lanes per clock at the 2.4 GHz peak engine clock
VALU_PEAK_LANE_OPS = 256 * 4 * 16 * 2.4e9

# name: dense  -> dict(B, T, H, D, Hv, Dv, W, p, ms, dtype, pattern)
#       packed -> dict(lengths, H, D, Hv, Dv, W, p, ms, dtype)
WORKLOADS = {
    "metric": dict(B=2, T=4096, H=64, D=8, Hv=16, Dv=8, W=128, p=0.1, ms=3.0, dtype="float32"),
    "metric_p0": dict(B=2, T=4096, H=64, D=8, Hv=16, Dv=8, W=128, p=0.0, ms=3.0, dtype="float32"),
    "config1": dict(B=1, T=256, H=4, D=4, Hv=4, Dv=8, W=16, p=0.0, ms=3.0, dtype="float32"),
    "config2": dict(B=2, T=1024, H=64, D=8, Hv=16, Dv=8, W=128, p=0.1, ms=3.0, dtype="float32"),
    "config3": dict(B=4, T=4096, H=32, D=16, Hv=32, Dv=64, W=32, p=0.0, ms=3.0, dtype="bfloat16"),
    "config4": dict(B=1, T=8192, H=16, D=2, Hv=16, Dv=32, W=256, p=0.0, ms=3.0, dtype="float16",
                    pattern="motif"),
    "config5": dict(lengths=[1024, 7168, 2048, 4096, 512, 8192, 3072, 6656], H=64, D=32, Hv=8,
                    Dv=32, W=64, p=0.1, ms=9.0, dtype="bfloat16"),
}


def make_workload(name: str, device="cpu"):
    """Seeded synthetic inputs of a named configuration, built in their final dtype.

    Returns ``(config, query, key, value, cu_seqlens_or_None)``.  A private
    generator is used so that the result does not depend on global RNG state.
    """

    config = dict(WORKLOADS[name])
    dtype = getattr(torch, config["dtype"])
    generator = torch.Generator().manual_seed(1234 + sorted(WORKLOADS).index(name))
    randn = lambda *shape: torch.randn(*shape, generator=generator)
    if "lengths" in config:
        total = sum(config["lengths"])
        query = randn(total, config["H"], config["D"]).to(dtype)
        key = randn(total, config["H"], config["D"]).to(dtype)
        value = randn(total, config["Hv"], config["Dv"]).to(dtype)
        offsets = [0]
        for length in config["lengths"]:
            offsets.append(offsets[-1] + length)
        cu_seqlens = torch.tensor(offsets, dtype=torch.int32)
        return config, query.to(device), key.to(device), value.to(device), cu_seqlens.to(device)
    B, T, H, D = config["B"], config["T"], config["H"], config["D"]
    if config.get("pattern") == "motif":
        # per head a random 64-step motif tiled over T, 10 % of positions
        # sign-flipped; query = key + N(0, 0.1), rounded to the final dtype
        motif = randn(B, 64, H, D)
        key = motif.repeat(1, (T + 63) // 64, 1, 1)[:, :T].clone()
        flip = torch.rand(B, T, H, 1, generator=generator) < 0.10
        key = torch.where(flip, -key, key).to(dtype)
        query = (key.float() + 0.1 * randn(B, T, H, D)).to(dtype)
    else:
        query = randn(B, T, H, D).to(dtype)
        key = randn(B, T, H, D).to(dtype)
    value = randn(B, T, config["Hv"], config["Dv"]).to(dtype)
    return config, query.to(device), key.to(device), value.to(device), None


def pair_count(config) -> int:
    if "lengths" in config:
        return config["H"] * sum(n * (n - 1) // 2 for n in config["lengths"])
    return config["B"] * config["H"] * config["T"] * (config["T"] - 1) // 2


def token_count(config) -> int:
    return sum(config["lengths"]) if "lengths" in config else config["B"] * config["T"]


def algorithmic_bytes(config) -> dict:
    """Bytes each stage must move at least once (inputs read, outputs written)."""

    tokens = token_count(config)
    item = 4 if config["dtype"] == "float32" else 2
    symbols = tokens * config["H"] * config["D"]
    values = tokens * config["Hv"] * config["Dv"]
    outputs = tokens * config["H"] * config["Dv"]
    words = tokens * config["H"] * 4
    forward = 2 * symbols * item + 2 * words + values * item + outputs * item
    backward = (2 * symbols + values + outputs) * item + 2 * words + (2 * symbols + values) * 4
    return dict(forward=forward, backward=backward)


def run_step(rosa, config, leaves, cu_seqlens):
    controls = dict(
        max_suffix_length=config["W"], scale=1.0, dropout_p=config["p"],
        mismatch_scale=config["ms"],
    )
    for leaf in leaves:
        leaf.grad = None
    if cu_seqlens is None:
        output = rosa.rosa_soft(*leaves, **controls)
    else:
        output = rosa.rosa_soft_varlen(*leaves, cu_seqlens, **controls)
    loss = output.float().square().mean()
    loss.backward()
    return loss


def cpu_baseline(name: str, budget_seconds: float = 25.0) -> dict:
    """Time the CPU oracle (a port, float64, OpenMP) on a slice of the workload.

    The slice is one batch element, a prefix of the sequence and a number of
    value-head groups chosen so that the run takes about 10 to 30 s; its time
    is scaled by the pair count to the whole workload.
    """

    from oracle import c_oracle

    config, query, key, value, cu_seqlens = make_workload(name)
    if cu_seqlens is not None:
        start, end = int(cu_seqlens[0]), int(cu_seqlens[1])
        query, key, value = (t[start:end].unsqueeze(0) for t in (query, key, value))
    group = config["H"] // config["Hv"]
    threads = c_oracle.num_threads()
    rows = min(query.size(1), 512)
    groups = 1  # value-head groups in the slice
    elapsed = 0.0
    while True:
        heads = groups * group
        q, k = (t[:1, :rows, :heads].contiguous() for t in (query, key))
        v = value[:1, :rows, :groups].contiguous()
        grad_output = torch.ones(1, rows, heads, config["Dv"]) / (rows * heads * config["Dv"])
        begin = time.perf_counter()
        out, _, _ = c_oracle.hard_forward(q, k, v, config["W"])
        forward_seconds = time.perf_counter() - begin
        c_oracle.surrogate_vjp(
            q, k, v, (2.0 * out.float() * grad_output), max_suffix_length=config["W"],
            dropout_p=config["p"], mismatch_scale=config["ms"], seed=12345 if config["p"] > 0 else None,
        )
        elapsed = time.perf_counter() - begin
        if elapsed * 4.0 > budget_seconds:
            break
        if rows < query.size(1):  # first grow the sequence prefix (work grows 4x) ...
            rows = min(query.size(1), rows * 2)
        elif groups < config["Hv"]:  # ... then the number of value-head groups
            groups = min(config["Hv"], groups * 4)
        else:
            break
    group = groups * group
    slice_pairs = group * rows * (rows - 1) // 2
    seconds_full = elapsed * pair_count(config) / max(slice_pairs, 1)
    return dict(
        value=token_count(config) / seconds_full,
        unit="tokens/s",
        cores=threads,
        kind="port",
        sample=(
            f"float64 C oracle, fwd+bwd, 1 batch x {group} heads x first {rows} rows "
            f"({slice_pairs} pairs, {elapsed:.2f} s, forward {forward_seconds:.3f} s), "
            f"extrapolated x{pair_count(config) / max(slice_pairs, 1):.1f} by pair count"
        ),
        extrapolation_factor=pair_count(config) / max(slice_pairs, 1),
    )



def measure_workload(name: str, steps: int, warmup: int) -> dict:
    """Time `steps` training steps and as many no-grad forwards of one configuration."""

    import rosa_soft_amd
    from rosa_soft_amd import cabi

    assert rosa_soft_amd.BUILD_CAPABILITIES.variant == "rocm", "HIP extension is not built"
    device = torch.device("cuda:0")
    config, query, key, value, cu_seqlens = make_workload(name, device)
    leaves = [t.requires_grad_() for t in (query, key, value)]
    cabi.stage_timing(True)
    for _ in range(warmup):
        run_step(rosa_soft_amd, config, leaves, cu_seqlens)
    torch.cuda.synchronize()
    cabi.stage_totals()  # the warm-up's events: read and dropped
    begin = time.perf_counter()
    for _ in range(steps):
        run_step(rosa_soft_amd, config, leaves, cu_seqlens)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - begin
    # the library recorded its stage events on the launch stream during the timed steps and
    # the host waited for none of them; they are read only now
    stage_means = {stage: total / runs for stage, (total, runs) in cabi.stage_totals().items()}
    cabi.stage_timing(False)

    def forward():
        if cu_seqlens is None:
            return rosa_soft_amd.rosa_soft(query, key, value, max_suffix_length=config["W"])
        return rosa_soft_amd.rosa_soft_varlen(query, key, value, cu_seqlens,
                                              max_suffix_length=config["W"])

    with torch.no_grad():
        for _ in range(2):
            forward()
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for _ in range(steps):
            forward()
        torch.cuda.synchronize()
        forward_ms = 1e3 * (time.perf_counter() - begin) / steps
    plan = cabi.gradient_block_plan(query, value, config["W"], cu_seqlens)
    return dict(
        name=name, config=config, steps=steps, warmup=warmup,
        ms_per_step=1e3 * elapsed / steps, forward_ms=forward_ms,
        stage_ms=stage_means,
        gradient_block_plan=plan,
    )


def roofline_fractions(measured: dict) -> dict:
    """Matrix flops each backward kernel performs over that kernel's own time.

    Per (row, route) pair the backward contracts five times: the utilities go x sign(v)
    (2 Dv flop; both backward kernels need them), dV (2 Dv), dK and dQ (2 D each) in the
    gradient kernel, and q x k (2 D), which this build evaluates as xor + popcount on packed
    words and therefore does not count for any kernel.  All fractions are against the
    MI355X float32 matrix peak, whatever pipe executes the products.
    """

    config, stage_ms = measured["config"], measured["stage_ms"]
    pairs = pair_count(config)
    D, Dv = config["D"], config["Dv"]
    flops = {
        "vjp_gradients": 2.0 * pairs * (2 * D + 2 * Dv),
        "vjp_row_stats": 2.0 * pairs * Dv,
    }
    out = {}
    for stage, work in flops.items():
        ms = stage_ms.get(stage)
        if ms:
            tflops = work / (ms * 1e-3) / 1e12
            out[stage] = dict(ms=ms, flop=work, tflops=tflops, frac=tflops / FP32_MATRIX_PEAK_TFLOPS)
    backward_ms = sum(ms for stage, ms in stage_ms.items() if stage.startswith("vjp_"))
    if backward_ms > 0:
        work = 2.0 * pairs * (3 * D + 2 * Dv)  # the per-pair figure of the five contractions
        tflops = work / (backward_ms * 1e-3) / 1e12
        out["whole_backward"] = dict(ms=backward_ms, flop=work, tflops=tflops,
                                     frac=tflops / FP32_MATRIX_PEAK_TFLOPS)
    return out


def algorithmic_lane_ops(config) -> dict:
    """Vector lane operations per (row, route) pair that the diagonal recurrence itself needs,
    one per arithmetic instruction of a lane, whatever its issue rate (32-bit integer
    multiplies and sqrt/exp2/rsq take four issue slots each on CDNA4, which the count ignores).

    Row statistics: gate (xor, popcount, table) 3, suffix score 1, window term 2, logit
    (sqrt, fma, exp2) 3, normaliser and expectation sums 2, utility 1 = 12; the dropout hash adds
    five rounds of (xor, multiply, shift, xor, multiply), the closing fold and the compare, 28.
    Gradients: the same replay without the sums 9, probability 1, keep bit and utility 2,
    route adjoint (rsq, two products) 3, weight as two bfloat16 terms 4, reverse carry 1,
    window sum 2, gate adjoint 1, its two bfloat16 terms 4 = 27.
    """

    hashed = 28 if config["p"] > 0 else 0
    return {"vjp_row_stats": 12 + hashed, "vjp_gradients": 27}


def valu_fractions(measured: dict) -> dict:
    """The vector-ALU roof of the two backward kernels: algorithmic lane operations per pair
    (`algorithmic_lane_ops`) x pairs over the kernel's time, against the VALU peak."""

    pairs = pair_count(measured["config"])
    out = {}
    for stage, per_pair in algorithmic_lane_ops(measured["config"]).items():
        ms = measured["stage_ms"].get(stage)
        if ms:
            rate = per_pair * pairs / (ms * 1e-3)
            out[stage] = dict(lane_ops_per_pair=per_pair, achieved=rate / 1e12,
                              peak=VALU_PEAK_LANE_OPS / 1e12, unit="T lane-op/s",
                              frac=rate / VALU_PEAK_LANE_OPS)
    return out


def atomic_row_segments(config, plan: dict) -> int:
    """64-byte row segments the float atomics of one gradient-kernel launch touch.

    Global float atomics are bounded by the row segments they touch, not by their number
    (`rosa_hip_measure_atomic_rate`).  A band of 64 diagonals with n rows adds n completed
    rows of dQ and n completed columns of dK and dV to memory, a row or column of w floats
    being ceil(4 w / 64) segments; a block of two waves adds the columns of its two bands
    once, and with the row queue also the rows they share.
    """

    lengths = config.get("lengths") or [config["T"]] * config["B"]
    D, Dv = config["D"], config["Dv"]
    # rows of at most 8 floats are accumulated head-major, where two neighbouring rows
    # share a segment and leave in one instruction
    symbol_segments = 0.5 if D <= 8 else -(-4 * D // 64)
    value_segments = 0.5 if Dv <= 8 else sum(
        -(-4 * min(64, Dv - first) // 64) for first in range(0, Dv, 64))
    rows = columns = 0
    piece_rows = plan.get("piece_rows", 0)
    for length in lengths:
        steps = [length - 1 - 64 * band for band in range((length + 63) // 64)]
        steps = [n for n in steps if n > 0]
        if piece_rows > 0:
            # every piece but the first of a band flushes four more column tiles (64 columns)
            columns += sum(64 * ((n - 1) // piece_rows) for n in steps)
        if plan["waves"] == 2:
            leads = steps[0::2]
            columns += sum(leads)
            rows += sum(leads) if plan["row_queue"] else sum(steps)
        else:
            columns += sum(steps)
            rows += sum(steps)
    return int(config["H"] * (columns * (symbol_segments + value_segments) + rows * symbol_segments))


def config_summary(measured: dict) -> dict:
    config = measured["config"]
    tokens = token_count(config)
    fractions = roofline_fractions(measured)
    return dict(
        workload=", ".join(f"{k}={v}" for k, v in config.items()),
        steps=measured["steps"],
        ms_per_step=round(measured["ms_per_step"], 4),
        fwd_ms=round(measured["forward_ms"], 4),
        tokens_per_s=round(tokens / (measured["ms_per_step"] * 1e-3), 1),
        fwd_tokens_per_s=round(tokens / (measured["forward_ms"] * 1e-3), 1),
        vjp_gradients_ms=round(measured["stage_ms"].get("vjp_gradients", float("nan")), 4),
        vjp_row_stats_ms=round(measured["stage_ms"].get("vjp_row_stats", float("nan")), 4),
        vjp_gradients_frac=round(fractions.get("vjp_gradients", {}).get("frac", float("nan")), 4),
        vjp_gradients_valu_frac=round(
            valu_fractions(measured).get("vjp_gradients", {}).get("frac", float("nan")), 4),
        whole_backward_frac=round(fractions.get("whole_backward", {}).get("frac", float("nan")), 4),
        waves_per_block=measured["gradient_block_plan"]["waves"],
        band_pieces=measured["gradient_block_plan"].get("pieces", 1),
        atomic_row_segments=atomic_row_segments(config, measured["gradient_block_plan"]),
    )


PROFILE_FIGURE = re.compile(r"^bench: (\w+) = ([-+0-9.eE]+)\s*$", re.MULTILINE)
PROFILE_SOURCE = re.compile(r"^bench-source: ([0-9a-f]{16})\s*$", re.MULTILINE)


def kernel_source_digest() -> str:
    """Digest of the HIP source and flags the library is built from; the counter summaries
    under profiles/ carry the digest of what they measured."""

    from rosa_soft_amd import _build

    return _build.source_digest()


def profile_figures(workload: str) -> dict:
    """Counter figures of a workload's dominant kernel, read from the committed summaries.

    The rocprofv3 summaries under profiles/ end in lines `bench: name = value`; those are
    what a counter run measured for this workload (HBM bytes per launch of the gradient
    kernel, busy fractions of the VALU and matrix pipes, issued matrix instructions).
    A workload without summaries yields an empty dict, never a guess; `stale` is set when a
    summary was taken from another version of the kernel source than the one in the tree.
    """

    figures = {}
    stale = False
    for suffix in ("backward_hbm_traffic", "backward_issue_counters"):
        path = os.path.join(ROOT, "profiles", f"{workload}_{suffix}.md")
        if os.path.exists(path):
            with open(path) as handle:
                text = handle.read()
            for name, value in PROFILE_FIGURE.findall(text):
                figures[name] = float(value)
            stale = stale or PROFILE_SOURCE.findall(text) != [kernel_source_digest()]
    if figures:
        figures["stale"] = stale
    return figures


def training_record(args) -> dict:
    measured = measure_workload(args.workload, args.steps, args.warmup)
    config, stage_ms = measured["config"], measured["stage_ms"]
    tokens = token_count(config)
    pairs = pair_count(config)
    ms_per_step, forward_ms = measured["ms_per_step"], measured["forward_ms"]
    bytes_needed = algorithmic_bytes(config)
    fractions = roofline_fractions(measured)
    backward_ms = fractions.get("whole_backward", {}).get("ms", 0.0)
    kernels = {stage: dict(ms=round(ms, 4)) for stage, ms in stage_ms.items()}
    if "hard_forward" in stage_ms:
        kernels["hard_forward"]["hbm_gbs"] = round(
            bytes_needed["forward"] / (stage_ms["hard_forward"] * 1e-3) / 1e9, 2
        )
        kernels["hard_forward"]["gpairs_per_s"] = round(pairs / (stage_ms["hard_forward"] * 1e-3) / 1e9, 2)
    if backward_ms > 0:
        kernels["vjp_total"] = dict(
            ms=round(backward_ms, 4),
            hbm_gbs=round(bytes_needed["backward"] / (backward_ms * 1e-3) / 1e9, 2),
            gpairs_per_s=round(pairs / (backward_ms * 1e-3) / 1e9, 2),
        )
    dominant = fractions.get("vjp_gradients", dict(tflops=float("nan"), frac=float("nan"), flop=0.0))
    figures = profile_figures(args.workload)
    roofline = {
        "kernel": "vjp_gradients_kernel",
        "bound": "mfma",
        "achieved": dominant["tflops"],
        "peak": FP32_MATRIX_PEAK_TFLOPS,
        "unit": "TFLOP/s",
        "frac": dominant["frac"],
        "traffic": figures.get("traffic_bytes_per_launch"),
        "flop_per_launch": dominant["flop"],
        "row_stats_kernel": fractions.get("vjp_row_stats"),
        "whole_backward": fractions.get("whole_backward"),
        "note": "achieved = the matrix flops this kernel performs per launch, "
                "2*pairs*(2D+2Dv) (utilities, dV, dK, dQ; q.k is xor+popcount here), over its "
                "mean launch time from HIP events on the launch stream; whole_backward = "
                "2*pairs*(3D+2Dv) over the sum of the backward stages; traffic and issue are "
                "read from the rocprofv3 summaries under profiles/ (null when this workload "
                "has none)",
    }
    valu = valu_fractions(measured)
    roofline["valu"] = dict(valu.get("vjp_gradients", {}), row_stats_kernel=valu.get("vjp_row_stats"),
                            note="algorithmic vector lane operations per pair (stated in "
                                 "algorithmic_lane_ops) x pairs / kernel time, against 256 CUs x 4 "
                                 "SIMDs x 16 lanes x 2.4 GHz; the roof that binds at D = Dv = 8")
    if figures:
        roofline["issue"] = {k: v for k, v in figures.items()
                             if k not in ("traffic_bytes_per_launch", "stale")}
        roofline["profile_figures_stale"] = figures["stale"]
    # the other bound of the gradient kernel: its global float atomics, priced against the
    # rate measured on this GPU in this run
    from rosa_soft_amd import cabi

    plan = measured["gradient_block_plan"]
    segments = atomic_row_segments(config, plan)
    row_floats = config["Hv"] * config["Dv"]
    rate = cabi.measure_atomic_rate(max(row_floats, 16), min(16, config["Dv"]))
    roofline["atomics"] = {
        "row_segments_per_launch": segments,
        "segments_per_s_measured": rate,
        "floor_ms": 1e3 * segments / rate,
        "kernel_ms": stage_ms.get("vjp_gradients"),
        "waves_per_block": plan["waves"],
        "row_queue": plan["row_queue"],
        "note": "global float atomics are bounded by the 64-byte row segments they touch; "
                "the rate is measured by rosa_hip_measure_atomic_rate in the flush pattern",
    }
    return {
        "metric": "fwd+bwd tokens/sec",
        "value": tokens / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if config["dtype"] == "float32" else config["dtype"],
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: " + ", ".join(f"{k}={v}" for k, v in config.items()),
            "loss": "output.float().square().mean()",
            "tokens_per_step": tokens,
            "pairs_per_step": pairs,
        },
        "fwd_tokens_per_s": tokens / (forward_ms * 1e-3),
        "fwd_ms": forward_ms,
        "roofline": roofline,
        "kernels": kernels,
    }


def pytorch_cpu_baseline(budget_seconds: float = 8.0) -> dict:
    """The pure-PyTorch restatement of rosa_soft_reference (oracle/rosa_oracle.py), forward +
    backward on configuration 1 at its full shape, on this box's host cores (the reference's
    own CPU-runnable case: rosa_soft/soft_reference.py:596-635)."""

    from oracle import rosa_oracle

    config, query, key, value, _ = make_workload("config1")
    leaves = [t.clone().requires_grad_() for t in (query, key, value)]
    repeats, elapsed = 0, 0.0
    while (elapsed < budget_seconds and repeats < 50) or repeats < 2:
        for leaf in leaves:
            leaf.grad = None
        begin = time.perf_counter()
        output = rosa_oracle.rosa_soft_oracle(
            *leaves, max_suffix_length=config["W"], scale=1.0, dropout_p=config["p"],
            mismatch_scale=config["ms"])
        output.square().mean().backward()
        if repeats > 0:  # the first pass warms the allocator and the thread pool
            elapsed += time.perf_counter() - begin
        repeats += 1
    timed = repeats - 1
    return dict(
        value=timed * token_count(config) / elapsed, unit="tokens/s",
        cores=torch.get_num_threads(), kind="port",
        sample=(f"oracle/rosa_oracle.py (dense PyTorch restatement), fwd+bwd, config1 at full "
                f"shape ({', '.join(f'{k}={v}' for k, v in config.items())}), {timed} repeats in "
                f"{elapsed:.2f} s, torch threads {torch.get_num_threads()}"),
    )


def router_cpu_baseline() -> dict:
    """The reference's RosaRuntime (its rosa_runtime.cpp built under oracle/_ref), forward only,
    on the metric shape's 8-bit symbols: the CPU counterpart of the hard forward
    (benchmarks/rosa_runtime.py:15-46)."""

    config = RUNTIME_WORKLOADS["runtime_prefill"]
    query, key, payload = runtime_symbols(config, config["T"], 7)
    return runtime_cpu_baseline(config, query, key, payload)


RUNTIME_WORKLOADS = {
    # the metric shape served by the device-resident hard router: one prefill update
    "runtime_prefill": dict(S=2, T=4096, H=64, Hp=16, qk_bits=8, payload_bits=8, W=128),
    # 8 slots with 4096 tokens of history each, then single-token updates
    "runtime_decode": dict(S=8, T=4096, H=64, Hp=16, qk_bits=8, payload_bits=8, W=128, decode=64),
}


def runtime_symbols(config, tokens, seed):
    generator = torch.Generator().manual_seed(seed)
    draw = lambda heads, bits: torch.randint(
        0, 1 << bits, (config["S"], tokens, heads), dtype=torch.uint8, generator=generator)
    return (draw(config["H"], config["qk_bits"]), draw(config["H"], config["qk_bits"]),
            draw(config["Hp"], config["payload_bits"]))


def runtime_cpu_baseline(config, query, key, payload) -> dict:
    """The reference's own CPU runtime (built from its source under oracle/_ref) on the same
    prefill, repeated until about ten seconds have passed."""

    from oracle import router_oracle

    native = router_oracle.reference_runtime()
    if native is None:
        return dict(value=None, unit="tokens/s", cores=0, kind="reference",
                    sample="oracle/_ref is not built")
    slots, tokens, heads = query.shape
    offsets = torch.arange(0, (slots + 1) * tokens, tokens, dtype=torch.int64)
    flat = lambda x: x.reshape(slots * tokens, x.size(2)).contiguous()
    repeats, elapsed = 0, 0.0
    while elapsed < 10.0 and repeats < 200:
        runtime = native(heads, payload.size(2), config["qk_bits"], config["payload_bits"],
                         config["W"])
        begin = time.perf_counter()
        runtime.update_packed(offsets, flat(query), flat(key), flat(payload))
        elapsed += time.perf_counter() - begin
        repeats += 1
    return dict(
        value=repeats * slots * tokens / elapsed, unit="tokens/s",
        cores=torch.get_num_threads(), kind="reference",
        sample=(f"rosa_runtime.cpp update_packed, {slots} slots x {tokens} tokens x {heads} heads, "
                f"{repeats} repeats in {elapsed:.2f} s (OpenMP over slots x heads)"),
    )


def run_runtime_workload(args) -> None:
    """Streaming hard router: prefill or decode throughput of the device-resident runtime."""

    import rosa_soft_amd

    config = RUNTIME_WORKLOADS[args.workload]
    device = torch.device("cuda:0")
    query, key, payload = (t.to(device) for t in runtime_symbols(config, config["T"], 7))
    decode = config.get("decode", 0)
    make = lambda: rosa_soft_amd.RosaRuntime(config["H"], config["Hp"], config["qk_bits"],
                                             config["payload_bits"], config["W"])
    begin_event = torch.cuda.Event(enable_timing=True)
    end_event = torch.cuda.Event(enable_timing=True)
    timed_ms = 0.0
    if decode:
        step_q, step_k, step_p = (t.to(device) for t in runtime_symbols(config, decode, 8))
        for step in range(args.warmup + args.steps):
            runtime = make()
            runtime.update_packed(query, key, payload)
            torch.cuda.synchronize()
            begin_event.record()
            for t in range(decode):
                runtime.update_packed(step_q[:, t:t + 1], step_k[:, t:t + 1], step_p[:, t:t + 1])
            end_event.record()
            torch.cuda.synchronize()
            if step >= args.warmup:
                timed_ms += begin_event.elapsed_time(end_event)
            runtime.close()
        tokens = config["S"] * decode
    else:
        for step in range(args.warmup + args.steps):
            runtime = make()
            torch.cuda.synchronize()
            begin_event.record()
            runtime.update_packed(query, key, payload)
            end_event.record()
            torch.cuda.synchronize()
            if step >= args.warmup:
                timed_ms += begin_event.elapsed_time(end_event)
            runtime.close()
        tokens = config["S"] * config["T"]
    ms_per_step = timed_ms / args.steps
    pairs = config["S"] * config["H"] * (
        decode * config["T"] if decode else config["T"] * (config["T"] - 1) // 2)
    record = {
        "metric": "router tokens/sec", "value": tokens / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: " + ", ".join(f"{k}={v}" for k, v in config.items()),
                   "tokens_per_step": tokens, "pairs_per_step": pairs},
        "gpairs_per_s": pairs / (ms_per_step * 1e-3) / 1e9,
    }
    if not args.no_cpu_baseline and not decode:
        record["cpu_baseline"] = runtime_cpu_baseline(config, query.cpu(), key.cpu(), payload.cpu())
    print(json.dumps(record))


FUSED_WORKLOADS = {
    # the projection behind the operator at the shape of config 3 (B4 T4096 H32 Dv64, bfloat16)
    # with a square model width: out = residual + y @ W^T, y the operator's ternary output
    "fused_output": dict(B=4, T=4096, H=32, D=16, Hv=32, Dv=64, W=32, N=2048),
}

BF16_MATRIX_PEAK = 2.5e15  # dense bfloat16 matrix peak of MI355X, FLOP/s


def run_fused_workload(args) -> None:
    """Hard forward in bit form + output projection fed with the bits, against the expanded
    tensor + a library product (what the reference's caller does)."""

    from rosa_soft_amd import cabi

    config = FUSED_WORKLOADS[args.workload]
    device = torch.device("cuda:0")
    generator = torch.Generator(device=device).manual_seed(4321)
    shape = lambda *dims: torch.randn(*dims, device=device, generator=generator).to(torch.bfloat16)
    query = shape(config["B"], config["T"], config["H"], config["D"])
    key = shape(config["B"], config["T"], config["H"], config["D"])
    value = shape(config["B"], config["T"], config["Hv"], config["Dv"])
    width = config["N"]
    depth = config["H"] * config["Dv"]
    weight = (shape(width, depth).float() / depth ** 0.5).to(torch.bfloat16)
    residual = shape(config["B"], config["T"], width)
    sign_words, routed = cabi.hard_forward_bits(query, key, value, config["W"])
    begin_event = torch.cuda.Event(enable_timing=True)
    end_event = torch.cuda.Event(enable_timing=True)

    def timed(step) -> float:
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        begin_event.record()
        for _ in range(args.steps):
            step()
        end_event.record()
        torch.cuda.synchronize()
        return begin_event.elapsed_time(end_event) / args.steps

    fused_ms = timed(lambda: cabi.project_routed_bits(sign_words, routed, config["Dv"], weight, residual))
    library_ms = timed(lambda: torch.addmm(
        residual.flatten(0, 1),
        cabi.expand_output_bits(sign_words, routed, config["Dv"], torch.bfloat16).flatten(0, 1).flatten(1),
        weight.t()))
    tokens = config["B"] * config["T"]
    flops = 2.0 * tokens * depth * width
    record = {
        "metric": "output projection from the bit form, tokens/sec",
        "value": tokens / (fused_ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": fused_ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: " + ", ".join(f"{k}={v}" for k, v in config.items())},
        "roofline": {"bound": "mfma", "achieved": flops / (fused_ms * 1e-3) / 1e12,
                     "peak": BF16_MATRIX_PEAK / 1e12, "unit": "TFLOP/s",
                     "frac": flops / (fused_ms * 1e-3) / BF16_MATRIX_PEAK, "traffic": None},
        "expanded_tensor_plus_library_product_ms": library_ms,
    }
    print(json.dumps(record))


def main() -> None:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=10)
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--workload", default="metric",
                        choices=sorted(WORKLOADS) + sorted(RUNTIME_WORKLOADS) + sorted(FUSED_WORKLOADS))
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-configs", action="store_true",
                        help="skip the block that times configurations 1 to 5 beside the metric shape")
    parser.add_argument(
        "--copy-calibration", type=int, default=0, metavar="MIB",
        help="only run a plain device copy of MIB mebibytes three times (reference point for "
             "scaling the FETCH_SIZE / WRITE_SIZE counters of rocprofv3) and exit",
    )
    args = parser.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(
            "bench.py measures one GPU: this operator shards over (batch, value-head group) "
            "without any exchange and no multi-GPU path is built; run with --gpus 1",
            file=sys.stderr,
        )
        sys.exit(2)

    if args.copy_calibration > 0:
        source = torch.ones(args.copy_calibration << 18, dtype=torch.float32, device="cuda:0")
        target = torch.empty_like(source)
        for _ in range(3):
            target.copy_(source)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": source.numel() * 4, "copy_bytes_written": source.numel() * 4,
                          "launches": 3}))
        return

    if args.workload in RUNTIME_WORKLOADS:
        run_runtime_workload(args)
        return
    if args.workload in FUSED_WORKLOADS:
        run_fused_workload(args)
        return

    record = training_record(args)
    if not args.no_configs and args.workload == "metric":
        # the other configurations, timed by this same run (fewer steps each)
        record["configs"] = {
            name: config_summary(measure_workload(name, max(2, args.steps // 3), 2))
            for name in ("config1", "config2", "config3", "config4", "config5")
        }
    if not args.no_cpu_baseline:
        record["cpu_baseline"] = cpu_baseline(args.workload)
        if args.workload == "metric":
            record["cpu_baseline"]["pytorch"] = pytorch_cpu_baseline()
            record["cpu_baseline"]["router"] = router_cpu_baseline()
    print(json.dumps(record))


if __name__ == "__main__":
    main()
