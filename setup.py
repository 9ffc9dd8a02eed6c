"""Packaging for rosa_soft_amd: builds the gfx950 HIP library and the dispatcher module.

The reference's setup.py chooses between a pure, a CPU and a CUDA build through
``ROSA_BUILD_EXTENSION`` / ``USE_CUDA`` (reference ``setup.py:50-96``).  This
build has one native variant, ``rocm``: ``ROSA_BUILD_EXTENSION=0`` skips it (the
package then reports ``variant == "reference"`` and the operators raise),
anything else builds it with hipcc for gfx950.  There is no CUDA path.
"""

import importlib.util
import os

from setuptools import Command, find_packages, setup
from setuptools.command.build_py import build_py

HERE = os.path.dirname(os.path.abspath(__file__))


def _load_build_module():
    spec = importlib.util.spec_from_file_location(
        "_rosa_build", os.path.join(HERE, "rosa_soft_amd", "_build.py")
    )
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def _wants_extension() -> bool:
    choice = os.environ.get("ROSA_BUILD_EXTENSION", "1")
    if choice not in ("0", "1"):
        raise SystemExit("ROSA_BUILD_EXTENSION must be 0 or 1")
    return choice == "1"


class BuildRocmExtension(Command):
    description = "compile librosa_soft_hip.so (hipcc, gfx950) and the _C dispatcher module in-tree"
    user_options = [("inplace", "i", "build in the source tree (always the case)")]
    boolean_options = ["inplace"]

    def initialize_options(self):
        self.inplace = True

    def finalize_options(self):
        pass

    def run(self):
        if _wants_extension():
            _load_build_module().build_all()


class BuildPyWithExtension(build_py):
    def run(self):
        self.run_command("build_ext")
        super().run()


setup(
    name="rosa_soft_amd",
    version="0.1.0",
    description="MI355X-native rosa_soft / rosa_soft_varlen training operators",
    packages=find_packages(include=["rosa_soft_amd", "rosa_soft_amd.*"]),
    package_data={"rosa_soft_amd": ["*.so", "csrc/*"]},
    python_requires=">=3.10",
    install_requires=["torch>=2.10"],
    cmdclass={"build_ext": BuildRocmExtension, "build_py": BuildPyWithExtension},
)
