"""In-tree build of the two native pieces (used by setup.py and __graft_entry__).

* ``librosa_soft_hip.so`` - HIP kernels + C ABI, compiled by hipcc for gfx950
  only (no CUDA path, no hipify step: the source is HIP).
* ``_C`` - the PyTorch dispatcher module, plain C++ compiled by g++ against the
  torch headers and linked to the library above.
"""

from __future__ import annotations

import hashlib
import json
import os
import re
import shlex
import subprocess
import sys
import sysconfig
from typing import Dict, List

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
ROCM_HOME = os.environ.get("ROCM_HOME", "/opt/rocm")
OFFLOAD_ARCH = "gfx950"

HIP_SOURCE = os.path.join(HERE, "csrc", "rosa_kernels.hip")
# the band kernels of the backward, compiled once per tile family (sign words per value
# column, padded value width, symbol tiles) so that the families build side by side
INSTANCES_SOURCE = os.path.join(HERE, "csrc", "rosa_vjp_instances.hip")
TILE_FAMILIES = [(1, 8, 1), (1, 8, 2), (1, 16, 1), (1, 16, 2), (1, 32, 1), (1, 32, 2),
                 (2, 64, 1), (2, 64, 2)]
HIP_HEADERS = [os.path.join(HERE, "csrc", name)
               for name in ("rosa_device_common.hpp", "rosa_vjp_bands.hpp")]
OBJECT_DIR = os.path.join(HERE, "build_objects")
HIP_LIBRARY = os.path.join(HERE, "librosa_soft_hip.so")
DISPATCH_SOURCE = os.path.join(HERE, "csrc", "rosa_dispatch.cpp")
# registers, spills, scratch and LDS of every kernel, as the compiler reported them
RESOURCE_REPORT = os.path.join(HERE, "kernel_resources.json")

# -packed-fp32-ops is switched off on purpose: some packed-FP32 forms have
# produced silently wrong results on this hardware generation.
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}", "-O3", "-std=c++17", "-fPIC",
    "-munsafe-fp-atomics", "-Wno-pass-failed",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def dispatcher_path() -> str:
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(HERE, "_C" + suffix)


RESOURCE_REMARK = re.compile(r"remark:\s+([A-Za-z /\[\]]+?):\s+(\S+) \[-Rpass-analysis=kernel-resource-usage\]")


def _run(command: List[str]) -> str:
    print("+", " ".join(shlex.quote(part) for part in command), flush=True)
    return _report(subprocess.run(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                                  text=True))


def _report(completed) -> str:
    """Print what a finished build step said, without the compiler's known noise."""

    noise = ("packed-fp32-ops", "is not a recognized feature", "kernel-resource-usage")
    if completed.returncode == 0:
        noise += ("In file included from",)  # the include trail of a remark
    lines, skip_excerpt = [], 0
    for line in completed.stdout.splitlines():
        if "kernel-resource-usage" in line and "Function Name" in line:
            skip_excerpt = 2  # the remark of a function is followed by a source excerpt
            continue
        if skip_excerpt and re.match(r"\s+(\d+ )?\|", line):
            skip_excerpt -= 1
            continue
        if not any(n in line for n in noise):
            lines.append(line)
    if lines:
        print("\n".join(lines), flush=True)
    if completed.returncode != 0:
        raise RuntimeError(f"build step failed with exit code {completed.returncode}")
    return completed.stdout


def kernel_resources(compiler_output: str) -> Dict[str, Dict[str, int]]:
    """Per kernel, what -Rpass-analysis=kernel-resource-usage reported: registers, spilled
    registers, scratch bytes per lane, static LDS bytes."""

    keys = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes",
            "VGPRs Spill": "vgpr_spills", "SGPRs Spill": "sgpr_spills",
            "LDS Size [bytes/block]": "lds_bytes", "Occupancy [waves/SIMD]": "waves_per_simd"}
    report: Dict[str, Dict[str, int]] = {}
    current = None
    for name, value in RESOURCE_REMARK.findall(compiler_output):
        name = name.strip()
        if name == "Function Name":
            current = report.setdefault(value, {})
        elif current is not None and name in keys and value.isdigit():
            current[keys[name]] = int(value)
    return report


# entry of the resource report that names what was compiled (see source_digest)
BUILD_RECORD = "__build__"


def source_digest() -> str:
    """First 16 hex digits of the SHA-256 of the HIP source and the compiler flags: what a
    resource report or a counter summary must name to speak for the library in the tree."""

    digest = hashlib.sha256()
    for path in (HIP_SOURCE, INSTANCES_SOURCE, *HIP_HEADERS):
        with open(path, "rb") as handle:
            digest.update(handle.read())
    digest.update(" ".join(HIPCC_FLAGS).encode())
    return digest.hexdigest()[:16]


def build_hip_library() -> str:
    """Compile the main translation unit and the eight tile families side by side, then link.

    One compiler process per translation unit; the families take one to two minutes each,
    which is also the build's wall time on eight cores."""

    from concurrent.futures import ThreadPoolExecutor

    hipcc = os.path.join(ROCM_HOME, "bin", "hipcc")
    digest = source_digest()  # of what the compilers are about to read
    os.makedirs(OBJECT_DIR, exist_ok=True)
    jobs = [([hipcc, *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", "-c", HIP_SOURCE],
             os.path.join(OBJECT_DIR, "rosa_kernels.o"))]
    for nvw, dvp, symbol_tiles in TILE_FAMILIES:
        jobs.append(([hipcc, *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage",
                      f"-DROSA_FAMILY_NVW={nvw}", f"-DROSA_FAMILY_DVP={dvp}",
                      f"-DROSA_FAMILY_DT={symbol_tiles}", "-c", INSTANCES_SOURCE],
                     os.path.join(OBJECT_DIR, f"rosa_vjp_{nvw}_{dvp}_{symbol_tiles}.o")))

    def compile_one(job):
        command = [*job[0], "-o", job[1]]
        print("+", " ".join(shlex.quote(part) for part in command), flush=True)
        return subprocess.run(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)

    workers = max(1, min(len(jobs), os.cpu_count() or 1, 16))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        finished = list(pool.map(compile_one, jobs))
    output = "".join(_report(completed) for completed in finished)
    _run([hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC",
          *(job[1] for job in jobs), "-o", HIP_LIBRARY])
    report = kernel_resources(output)
    report[BUILD_RECORD] = {"source_digest": digest}
    with open(RESOURCE_REPORT, "w") as handle:
        json.dump(report, handle, indent=0, sort_keys=True)
    spilling = sorted(name for name, use in report.items()
                      if use.get("vgpr_spills", 0) or use.get("scratch_bytes", 0))
    print(f"{len(report) - 1} kernels; spilling vector registers or using scratch: "
          f"{spilling if spilling else 'none'}", flush=True)
    return HIP_LIBRARY


def build_dispatcher() -> str:
    from torch.utils import cpp_extension

    include_flags = [f"-I{path}" for path in cpp_extension.include_paths()]
    include_flags += [f"-I{ROCM_HOME}/include", f"-I{sysconfig.get_paths()['include']}"]
    library_flags = [f"-L{path}" for path in cpp_extension.library_paths()]
    torch_lib = cpp_extension.library_paths()[0]
    output = dispatcher_path()
    command = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C",
        "-D_GLIBCXX_USE_CXX11_ABI=1",
        *include_flags, DISPATCH_SOURCE, "-o", output,
        *library_flags, f"-L{HERE}", "-lrosa_soft_hip",
        "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
        f"-L{ROCM_HOME}/lib", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}", f"-Wl,-rpath,{ROCM_HOME}/lib",
    ]
    _run(command)
    return output


def build_all() -> None:
    build_hip_library()
    build_dispatcher()


if __name__ == "__main__":
    build_all()
    sys.exit(0)
