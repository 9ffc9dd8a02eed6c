"""Host-side contract: validation, capabilities, schemas, C-ABI symbols (no GPU)."""

import ctypes
import math
import os
import re

import pytest
import torch

import rosa_soft_amd
from rosa_soft_amd import cabi, soft_contract

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_defaults_are_frozen():
    # reference tests/test_soft_reference.py:28-31
    assert soft_contract.ROSA_SOFT_DEFAULT_SCALE == 1.0
    assert soft_contract.ROSA_SOFT_DEFAULT_DROPOUT_P == 0.0
    assert soft_contract.ROSA_SOFT_DEFAULT_MISMATCH_SCALE == 3.0
    assert soft_contract.ROSA_SOFT_NULL_ROUTE_SCORE == 0.5


def _validate(**kwargs):
    tensor = torch.ones(1, 5, 1, 1)
    controls = dict(max_suffix_length=32, scale=1.0, dropout_p=0.0, mismatch_scale=3.0)
    controls.update(kwargs)
    horizon = soft_contract.validate_rosa_soft_inputs(tensor, tensor, tensor, **controls)
    soft_contract.validate_fp32_surrogate_scalars(
        horizon, controls["scale"], controls["dropout_p"], controls["mismatch_scale"]
    )
    return horizon


@pytest.mark.parametrize(
    ("kwargs", "message"),
    [
        ({"max_suffix_length": 0}, "max_suffix_length"),
        ({"scale": True}, "scale"),
        ({"scale": 0.0}, "scale"),
        ({"scale": math.inf}, "scale"),
        ({"scale": math.nan}, "scale"),
        ({"scale": 1e-300}, "scale"),
        ({"scale": 1e300}, "scale"),
        ({"dropout_p": True}, "dropout_p"),
        ({"dropout_p": -0.1}, "dropout_p"),
        ({"dropout_p": 1.0}, "dropout_p"),
        ({"dropout_p": math.nan}, "dropout_p"),
        ({"dropout_p": math.inf}, "dropout_p"),
        ({"mismatch_scale": 0.0}, "mismatch_scale"),
        ({"mismatch_scale": True}, "mismatch_scale"),
        ({"mismatch_scale": math.nan}, "mismatch_scale"),
        ({"mismatch_scale": math.inf}, "mismatch_scale"),
        ({"mismatch_scale": 1e-300}, "mismatch_scale"),
        ({"mismatch_scale": 1e300}, "mismatch_scale"),
    ],
)
def test_static_parameter_validation(kwargs, message):
    # reference tests/test_soft_reference.py:609-635
    with pytest.raises(ValueError, match=message):
        _validate(**kwargs)


def test_window_is_integral_and_clamped():
    # reference tests/test_soft_reference.py:565-583
    assert _validate(max_suffix_length=10**9) == 5
    assert _validate(max_suffix_length=3) == 3
    for invalid in (True, 1.5):
        with pytest.raises(TypeError, match="integer"):
            _validate(max_suffix_length=invalid)
    assert _validate(dropout_p=1.0 - 2.0**-24) == 5


def test_shape_head_bit_and_dtype_validation():
    # reference tests/test_soft_reference.py:651-670
    query = torch.ones(1, 3, 2, 4)
    key = torch.ones_like(query)
    value = torch.ones(1, 3, 1, 2)
    check = lambda q, k, v: soft_contract.validate_rosa_soft_inputs(q, k, v, 4, 1.0, 0.0, 3.0)
    with pytest.raises(ValueError, match="sequence"):
        check(query, key[:, :-1], value)
    with pytest.raises(ValueError, match="divisible"):
        check(query[:, :, :1], key[:, :, :1], value.repeat(1, 1, 2, 1))
    with pytest.raises(ValueError, match=r"\[1, 32\]"):
        check(torch.ones(1, 3, 1, 33), torch.ones(1, 3, 1, 33), value)
    with pytest.raises(ValueError, match="same dtype"):
        check(query.double(), key, value)
    with pytest.raises(ValueError, match="floating-point"):
        check(query.long(), key.long(), value.long())


def test_packed_validation_and_host_offsets():
    # reference tests/test_soft_varlen.py:144-178
    query = torch.ones(6, 2, 3)
    value = torch.ones(6, 1, 2)

    def check(offsets, dtype=torch.int32):
        return soft_contract.validate_rosa_soft_varlen_inputs(
            query, query, value, torch.tensor(offsets, dtype=dtype), 4, 1.0, 0.0, 3.0
        )

    assert check([0, 2, 2, 6]) == 4
    with pytest.raises(ValueError, match="start at zero"):
        check([1, 6])
    with pytest.raises(ValueError, match="end at the packed token count"):
        check([0, 5])
    with pytest.raises(ValueError, match="nondecreasing"):
        check([0, 4, 3, 6])
    with pytest.raises(ValueError, match="int32"):
        check([0, 6], dtype=torch.int64)
    with pytest.raises(ValueError, match="one-dimensional"):
        soft_contract.validate_rosa_soft_varlen_inputs(
            query, query, value, torch.tensor([[0, 6]], dtype=torch.int32), 4, 1.0, 0.0, 3.0
        )


def test_seed_rule_draws_only_when_needed():
    # reference rosa_soft/soft_contract.py:18-31, tests/test_soft_reference.py:468-490
    reference = torch.ones(1)
    state = torch.random.get_rng_state()
    assert soft_contract.make_dropout_seed(reference, 0.0, True).numel() == 0
    assert soft_contract.make_dropout_seed(reference, 0.5, False).numel() == 0
    assert torch.equal(state, torch.random.get_rng_state())
    seed = soft_contract.make_dropout_seed(reference, 0.5, True)
    assert seed.dtype == torch.int64 and seed.ndim == 0 and int(seed) >= 0
    assert not torch.equal(state, torch.random.get_rng_state())


def test_capabilities_and_public_surface():
    # reference tests/test_build_contract.py:276-334 (the variant set gains "rocm")
    caps = rosa_soft_amd.BUILD_CAPABILITIES
    assert caps.variant in {"reference", "rocm"}
    assert caps.compiled_extension and caps.rosa_soft_cuda and caps.variant == "rocm"
    assert caps.rosa_runtime is True  # the device-resident router ships with the HIP library
    with pytest.raises(Exception):
        caps.variant = "other"
    assert rosa_soft_amd.__all__ == [
        "__version__", "BUILD_CAPABILITIES", "RosaRuntime", "rosa_soft",
        "rosa_soft_reference", "rosa_soft_varlen", "rosa_soft_varlen_reference",
    ]
    if not torch.cuda.is_available():  # the router never falls back to the host
        with pytest.raises(RuntimeError, match="no device is available"):
            rosa_soft_amd.RosaRuntime(1, 1, 1, 1, 1)
    with pytest.raises(RuntimeError, match="test infrastructure"):
        rosa_soft_amd.rosa_soft_reference()


def test_exact_operator_schemas_and_dispatch_key():
    # reference tests/test_soft_cuda.py:1088-1102, tests/test_soft_varlen.py:281-301
    triple = "(Tensor output, Tensor packed_query_symbols, Tensor packed_key_symbols)"
    grads = "(Tensor grad_query, Tensor grad_key, Tensor grad_value)"
    expected = {
        "hard_forward": "rosa_soft::hard_forward(Tensor query, Tensor key, Tensor value, "
        f"int max_suffix_length) -> {triple}",
        "hard_forward_varlen": "rosa_soft::hard_forward_varlen(Tensor query, Tensor key, "
        f"Tensor value, Tensor cu_seqlens, int max_suffix_length) -> {triple}",
        "surrogate_vjp_masked": "rosa_soft::surrogate_vjp_masked(Tensor query, Tensor key, "
        "Tensor value, Tensor grad_output, Tensor packed_query_symbols, "
        "Tensor packed_key_symbols, Tensor dropout_seed, int max_suffix_length, float scale, "
        f"float dropout_p, float mismatch_scale, int gradient_mask) -> {grads}",
        "surrogate_vjp_varlen_masked": "rosa_soft::surrogate_vjp_varlen_masked(Tensor query, "
        "Tensor key, Tensor value, Tensor cu_seqlens, Tensor grad_output, "
        "Tensor packed_query_symbols, Tensor packed_key_symbols, Tensor dropout_seed, "
        "int max_suffix_length, float scale, float dropout_p, float mismatch_scale, "
        f"int gradient_mask) -> {grads}",
    }
    for name, schema in expected.items():
        assert str(getattr(torch.ops.rosa_soft, name).default._schema) == schema
        assert torch._C._dispatch_has_kernel_for_dispatch_key(f"rosa_soft::{name}", "CUDA")
    source = open(os.path.join(ROOT, "rosa_soft_amd", "csrc", "rosa_dispatch.cpp")).read()
    assert len(re.findall(r"\bm\.def\(", source)) == 4


def test_public_signatures():
    # reference tests/test_soft_cuda.py:1072-1086
    import inspect

    signature = inspect.signature(rosa_soft_amd.rosa_soft)
    assert list(signature.parameters) == [
        "query", "key", "value", "max_suffix_length", "scale", "dropout_p", "mismatch_scale",
    ]
    for name in ("max_suffix_length", "scale", "dropout_p", "mismatch_scale"):
        assert signature.parameters[name].kind is inspect.Parameter.KEYWORD_ONLY
    assert signature.parameters["max_suffix_length"].default == 32
    packed = inspect.signature(rosa_soft_amd.rosa_soft_varlen)
    assert list(packed.parameters)[:4] == ["query", "key", "value", "cu_seqlens"]


def test_fake_tensor_shapes():
    # reference tests/test_soft_cuda.py:100-111
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        query = torch.empty(2, 5, 4, 8, device="cuda", dtype=torch.bfloat16)
        value = torch.empty(2, 5, 2, 3, device="cuda", dtype=torch.bfloat16)
        out, pq, pk = torch.ops.rosa_soft.hard_forward(query, query, value, 3)
        assert out.shape == (2, 5, 4, 3) and out.dtype == torch.bfloat16
        assert pq.shape == pk.shape == (2, 4, 5) and pq.dtype == torch.int32
        assert pq.stride() == (20, 5, 1)
        grads = torch.ops.rosa_soft.surrogate_vjp_masked(
            query, query, value, out, pq, pk, torch.empty(0, dtype=torch.int64, device="cuda"),
            3, 1.0, 0.0, 3.0, 5,
        )
        assert grads[0].shape == query.shape and grads[0].dtype == torch.float32
        assert grads[1].shape == (0,) and grads[2].shape == value.shape
        tokens = torch.empty(7, 4, 8, device="cuda")
        packed_value = torch.empty(7, 2, 3, device="cuda")
        offsets = torch.empty(3, dtype=torch.int32, device="cuda")
        out, pq, _ = torch.ops.rosa_soft.hard_forward_varlen(tokens, tokens, packed_value, offsets, 3)
        assert out.shape == (7, 4, 3) and pq.shape == (4, 7)


def test_cpu_tensors_are_rejected_before_any_launch():
    # reference rosa_soft/soft.py:47-54
    tensor = torch.ones(1, 3, 1, 1)
    with pytest.raises(ValueError, match="CUDA"):
        rosa_soft_amd.rosa_soft(tensor, tensor, tensor)
    packed = torch.ones(3, 1, 1)
    with pytest.raises(ValueError, match="CUDA"):
        rosa_soft_amd.rosa_soft_varlen(packed, packed, packed, torch.tensor([0, 3], dtype=torch.int32))


def test_c_abi_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "rosa_soft_hip.h")).read()
    declared = set(re.findall(r"\b(rosa_hip_[a-z_]+)\s*\(", header))
    assert declared == set(cabi.EXPORTED_SYMBOLS)
    library = ctypes.CDLL(cabi.LIBRARY_PATH)
    for symbol in declared:
        assert hasattr(library, symbol), symbol
    loaded = cabi.load()
    assert loaded.rosa_hip_version() >= 100
    assert loaded.rosa_hip_target() == b"rocm-gfx950"
    # host-side arithmetic only: workspace sizes and argument rejection
    problem = cabi.RosaProblem(dtype=0, B=2, T=128, N=256, S=0, H=4, D=8, Hv=2, Dv=8, W=16)
    assert loaded.rosa_hip_forward_workspace_bytes(ctypes.byref(problem)) >= 256 * 4 * 4
    assert loaded.rosa_hip_vjp_workspace_bytes(ctypes.byref(problem), 7, 1.0, 0) > 0
    # the forward's workspace has room for the index of the keys: the source token of every
    # row (4 bytes), an entry per row (16) and the bucket offsets (at most 4 per row)
    rows = 256 * 4
    assert 20 * rows <= loaded.rosa_hip_forward_workspace_bytes(ctypes.byref(problem)) <= 26 * rows + 4096
    # beyond 64 M rows the workspace holds no index: 4 bytes per row and the tables
    huge = cabi.RosaProblem(dtype=0, B=1, T=1 << 21, N=1 << 21, S=0, H=64, D=8, Hv=2, Dv=8, W=16)
    assert loaded.rosa_hip_forward_workspace_bytes(ctypes.byref(huge)) <= 4 * (1 << 27) + 4096
    problem.D = 33
    assert loaded.rosa_hip_forward_workspace_bytes(ctypes.byref(problem)) == 0
    assert b"[1, 32]" in loaded.rosa_hip_last_error()
    # the router's workspace: only updates that route a long chunk through the index need one
    update = cabi.RosaRouterUpdate(S=2, H=4, Hp=2, W=16, qk_bits=8, payload_bits=8, capacity=4096,
                                   tokens=2 * 700, longest_chunk=700, uniform_chunk=700,
                                   longest_total=700)
    size = loaded.rosa_hip_router_workspace_bytes(ctypes.byref(update))
    assert 8 * 8 * 700 <= size <= 8 * 8 * 700 + 8 * 257 * 4 + 8192
    for field, value in (("longest_chunk", 8), ("qk_bits", 5), ("longest_total", 500)):
        other = cabi.RosaRouterUpdate(S=2, H=4, Hp=2, W=16, qk_bits=8, payload_bits=8,
                                      capacity=4096, tokens=2 * 700, longest_chunk=700,
                                      uniform_chunk=700, longest_total=700)
        setattr(other, field, value)
        assert loaded.rosa_hip_router_workspace_bytes(ctypes.byref(other)) == 0, field


def test_backward_workspace_sizes_at_training_shapes():
    """Host arithmetic of the backward workspace (no device call): the chunk records cost half
    a byte per pair with dropout, a packed layout is capped per token and head, and forbidding
    the records makes the workspace of a training shape much smaller."""

    from rosa_soft_amd import cabi

    loaded = cabi.load()
    size = lambda problem, dropout: loaded.rosa_hip_vjp_workspace_bytes(
        ctypes.byref(problem), 7, 1.0, int(dropout))
    metric = cabi.RosaProblem(dtype=0, B=2, T=4096, N=8192, S=0, H=64, D=8, Hv=16, Dv=8, W=128)
    pairs = 2 * 64 * 4096 * 4095 // 2
    cabi.set_record_budget(None)
    try:
        with_dropout, without_dropout = size(metric, True), size(metric, False)
        # (beside the records: staged grad_output rows, value words, row statistics and, per
        # resident wave of the gradient kernel, a ring of W + 1 rows of six bytes per lane)
        assert 0.5 * pairs < with_dropout < 0.5 * pairs + 250 * 2 ** 20
        assert 0.375 * pairs < without_dropout < 0.375 * pairs + 250 * 2 ** 20
        cabi.set_record_budget(0)
        assert size(metric, True) < 300 * 2 ** 20
        cabi.set_record_budget(None)
        # configuration 5: 32 768 packed tokens, 64 heads (cu_seqlens is not read by the query)
        packed = cabi.RosaProblem(dtype=2, B=0, T=0, N=32768, S=8, H=64, D=32, Hv=8, Dv=32, W=64)
        packed.cu_seqlens = 1  # any non-null address: the size query never dereferences it
        assert size(packed, True) < 1536 * 32768 * 64 + 400 * 2 ** 20
    finally:
        cabi.set_record_budget(None)


def test_gradient_launch_plan_follows_the_shape():
    """Host arithmetic of the gradient kernel's launch form (no device call): blocks of two
    waves where the tiles are wide and bands outnumber the resident waves, the row queue
    only while a block stays within its LDS share, and the process-wide override."""

    def plan(dtype, lead, D, Hv, Dv, W):
        query = torch.empty(*lead, D, dtype=dtype)
        value = torch.empty(*lead[:-1], Hv, Dv, dtype=dtype)
        return cabi.gradient_block_plan(query, value, W)

    metric = plan(torch.float32, (2, 4096, 64), 8, 16, 8, 128)
    assert metric["waves"] == 1 and not metric["row_queue"]
    # 8 192 bands on 3 072 resident waves: whole bands
    assert metric["piece_rows"] == 0 and metric["pieces"] == 1
    # configuration 4: 2 048 bands of up to 8 191 rows on 2 048 resident waves are cut into two
    # pieces of whole 32-row segments, each at least four windows long
    long_bands = plan(torch.float16, (1, 8192, 16), 2, 16, 32, 256)
    assert long_bands["waves"] == 1 and long_bands["pieces"] == 2
    assert long_bands["piece_rows"] == 4096 and long_bands["piece_rows"] >= 4 * 256
    try:
        cabi.set_gradient_piece_rows(-1)
        assert plan(torch.float16, (1, 8192, 16), 2, 16, 32, 256)["pieces"] == 1
        cabi.set_gradient_piece_rows(100)  # rounded up to whole segments
        forced = plan(torch.float32, (2, 4096, 64), 8, 16, 8, 128)
        assert forced["piece_rows"] == 128 and forced["pieces"] == 32
        cabi.set_gradient_block_waves(2)   # two-wave blocks walk whole bands
        assert plan(torch.float32, (2, 4096, 64), 8, 16, 8, 128)["pieces"] == 1
    finally:
        cabi.set_gradient_piece_rows(None)
        cabi.set_gradient_block_waves(None)
    config3 = plan(torch.bfloat16, (4, 4096, 32), 16, 32, 64, 32)
    assert config3["waves"] == 2 and config3["row_queue"]
    assert config3["lds_bytes"] <= 40 * 1024
    # float32 inputs of the same shape stage three terms per element: the queue no longer
    # fits the block's LDS share, the two waves stay
    wide = plan(torch.float32, (4, 4096, 32), 16, 32, 64, 32)
    assert wide["waves"] in (1, 2) and wide["lds_bytes"] <= 64 * 1024
    if wide["waves"] == 2:
        assert not wide["row_queue"] or wide["lds_bytes"] <= 40 * 1024
    small = plan(torch.bfloat16, (1, 1024, 4), 16, 4, 64, 32)  # 64 bands: one wave each
    assert small["waves"] == 1
    try:
        cabi.set_gradient_block_waves(2)
        forced = plan(torch.float32, (2, 4096, 64), 8, 16, 8, 128)
        assert forced["waves"] == 2
        cabi.set_gradient_block_waves(1)
        assert plan(torch.bfloat16, (4, 4096, 32), 16, 32, 64, 32)["waves"] == 1
    finally:
        cabi.set_gradient_block_waves(None)
    assert plan(torch.float32, (2, 4096, 64), 8, 16, 8, 128) == metric


def test_no_kernel_of_the_last_build_spills_or_uses_scratch():
    """The build records what the compiler reported per kernel.  Spilled vector registers and
    scratch memory are performance faults of the backward kernels (a reload waits behind
    every atomic in flight): none of the instantiations may have any."""

    from rosa_soft_amd import _build

    if not os.path.exists(_build.HIP_LIBRARY):
        pytest.skip("the HIP library is not built")
    import json

    # a library without the report of its own build (built by hand, or from another version
    # of the source) would let register regressions through unseen: that is a failure
    assert os.path.exists(_build.RESOURCE_REPORT), "library present but no resource report"
    with open(_build.RESOURCE_REPORT) as handle:
        report = json.load(handle)
    built_from = report.pop(_build.BUILD_RECORD, {}).get("source_digest")
    assert built_from == _build.source_digest(), (
        "the resource report (and the library beside it) was built from another version of "
        "the HIP source or other flags: rebuild")
    assert len(report) >= 100  # every instantiation of the backward kernels is listed
    offenders = {name: use for name, use in report.items()
                 if use.get("vgpr_spills", 0) or use.get("scratch_bytes", 0)}
    assert not offenders, offenders
    gradient = [use for name, use in report.items() if "vjp_gradients_kernel" in name]
    assert gradient and all(use["vgprs"] + use.get("agprs", 0) <= 512 for use in gradient)
    # Both backward kernels run at the speed their waves per SIMD allow, so the registers of
    # the instantiations the benchmark shapes use are pinned: the metric shape's gradient
    # kernel (one sign word, width 8, one symbol tile, single-wave blocks) fits three waves,
    # the row-statistics kernel four (three at width 64 with dropout).
    budget = {2: 256, 3: 168, 4: 128}
    for name, use in report.items():
        registers = use["vgprs"] + use.get("agprs", 0)
        if "vjp_gradients_kernelILi1ELi8ELi1E" in name or "vjp_gradients_kernelILi1ELi16ELi1E" in name:
            # (the form that walks pieces of bands, last template argument true, is compiled
            # for two waves: it only runs when the bands are too few to fill three)
            pieces = name.endswith("ELb1EEEvNS_9VjpParamsE")
            assert registers <= budget[2 if pieces else 3], (name, registers)
        if "vjp_row_stats_kernel" in name:
            wide_with_dropout = "ILi2ELi64E" in name and name.split("ILi2ELi64E")[1].startswith(("Lb0ELb1E", "Lb1ELb1E"))
            assert registers <= budget[3 if wide_with_dropout else 4], (name, registers)


def test_no_product_module_imports_the_oracle():
    package = os.path.join(ROOT, "rosa_soft_amd")
    for name in os.listdir(package):
        if name.endswith(".py"):
            text = open(os.path.join(package, name)).read()
            assert "import oracle" not in text and "from oracle" not in text, name
