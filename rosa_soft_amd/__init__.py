"""MI355X-native ``rosa_soft`` / ``rosa_soft_varlen`` training operators.

Package surface modelled on the reference's ``rosa_soft/__init__.py``: the
compiled dispatcher module is optional at import time (``:20-30``), the four
``rosa_soft::`` operators are probed on the dispatch key HIP tensors use
(``:41-57``), a partial registration is rejected (``:60-69``), and a frozen
``BUILD_CAPABILITIES`` record says what this build can do (``:105-118``).  A
working build reports ``variant == "rocm"``.  Without the compiled module the
operators are placeholders that raise (``:121-179``): there is no CPU or
PyTorch fallback behind the public names.
"""

from __future__ import annotations

import importlib as _importlib
from dataclasses import dataclass as _dataclass

import torch as _torch

from .soft_contract import (
    ROSA_SOFT_DEFAULT_DROPOUT_P as _DEFAULT_DROPOUT_P,
    ROSA_SOFT_DEFAULT_MISMATCH_SCALE as _DEFAULT_MISMATCH_SCALE,
    ROSA_SOFT_DEFAULT_SCALE as _DEFAULT_SCALE,
)

__version__ = "0.1.0"

_DISPATCH_KEY = "CUDA"  # PyTorch-ROCm dispatches HIP tensors on this key
_OPERATORS = (
    "hard_forward",
    "hard_forward_varlen",
    "surrogate_vjp_masked",
    "surrogate_vjp_varlen_masked",
)


def _load_compiled_extension():
    name = f"{__name__}._C"
    try:
        return _importlib.import_module(name)
    except ModuleNotFoundError as error:
        if error.name != name:
            raise
        return None


def _has_dispatch_kernel(operator: str, dispatch_key: str) -> bool:
    try:
        return bool(_torch._C._dispatch_has_kernel_for_dispatch_key(operator, dispatch_key))
    except RuntimeError:
        return False


def _probe_operators(compiled: bool):
    return tuple(
        compiled and _has_dispatch_kernel(f"rosa_soft::{operator}", _DISPATCH_KEY)
        for operator in _OPERATORS
    )


def _require_complete_registration(flags) -> bool:
    if any(flags) and not all(flags):
        raise RuntimeError(
            "rosa_soft_amd._C loaded with an incomplete operator registration; "
            "the extension is stale or incompatible with this package"
        )
    return all(flags)


_C = _load_compiled_extension()
_has_compiled_extension = _C is not None
_has_device_operators = _require_complete_registration(_probe_operators(_has_compiled_extension))


@_dataclass(frozen=True, slots=True)
class BuildCapabilities:
    variant: str
    compiled_extension: bool
    rosa_runtime: bool
    rosa_soft_cuda: bool


BUILD_CAPABILITIES = BuildCapabilities(
    variant="rocm" if _has_device_operators else "reference",
    compiled_extension=_has_compiled_extension,
    rosa_runtime=_has_device_operators,
    rosa_soft_cuda=_has_device_operators,
)


def _raise_unavailable(feature: str, hint: str) -> None:
    raise RuntimeError(
        f"{feature} is unavailable in the {BUILD_CAPABILITIES.variant!r} "
        f"rosa_soft_amd build. {hint}"
    )


_BUILD_HINT = (
    "Build the gfx950 extension in-tree with `python setup.py build_ext --inplace` "
    "(needs hipcc from ROCm)."
)

if _has_device_operators:
    from .soft import rosa_soft, rosa_soft_varlen
else:

    def rosa_soft(query, key, value, *, max_suffix_length=32, scale=_DEFAULT_SCALE,
                  dropout_p=_DEFAULT_DROPOUT_P, mismatch_scale=_DEFAULT_MISMATCH_SCALE):
        _raise_unavailable("rosa_soft training operator", _BUILD_HINT)

    def rosa_soft_varlen(query, key, value, cu_seqlens, *, max_suffix_length=32,
                         scale=_DEFAULT_SCALE, dropout_p=_DEFAULT_DROPOUT_P,
                         mismatch_scale=_DEFAULT_MISMATCH_SCALE):
        _raise_unavailable("rosa_soft_varlen training operator", _BUILD_HINT)


if _has_device_operators:
    from .runtime import RosaRuntime
else:

    class RosaRuntime:
        """The device-resident hard router needs the HIP library."""

        def __init__(self, *args, **kwargs):
            _raise_unavailable("RosaRuntime", _BUILD_HINT)


def rosa_soft_reference(*args, **kwargs):
    _raise_unavailable(
        "rosa_soft_reference",
        "The pure-PyTorch restatement is test infrastructure (oracle/rosa_oracle.py) "
        "and is deliberately not reachable from the product package.",
    )


def rosa_soft_varlen_reference(*args, **kwargs):
    _raise_unavailable(
        "rosa_soft_varlen_reference",
        "The pure-PyTorch restatement is test infrastructure (oracle/rosa_oracle.py) "
        "and is deliberately not reachable from the product package.",
    )


__all__ = [
    "__version__",
    "BUILD_CAPABILITIES",
    "RosaRuntime",
    "rosa_soft",
    "rosa_soft_reference",
    "rosa_soft_varlen",
    "rosa_soft_varlen_reference",
]
