"""Packaging of the MI355X build of the ``qfactory`` package.

Counterpart of the reference's setup.py (setup.py:11-23: packages qfactory, qfactory/core, qfactory/jit with
``include/**/*`` as package data).  Besides the kernel headers the package needs, at run time, the sources of
libqfactory_hip.so (``csrc/*.hip``, compiled by ``qfactory.native.build()`` with hipcc), the source of the
allocate-and-launch extension (``csrc/qf_fastpath.cpp``, ``qfactory.fastpath.build()``) and the C-ABI headers the
generated translation units include (``<checkout>/include/*.h``).  In a checkout both live outside the package
directory; a built distribution carries copies inside it (``qfactory/csrc``, ``qfactory/abi``), which is where
``qfactory.native`` and ``qfactory.jit.compiler`` look first.

    pip install -e <checkout>/qfactory-ae_amd          # editable: files stay where they are
    pip install <checkout>/qfactory-ae_amd             # regular: sources and headers are copied into the package
"""
import glob
import os
import shutil
import subprocess

import setuptools
from setuptools.command.build_py import build_py

HERE = os.path.dirname(os.path.abspath(__file__))


class build_py_with_native_sources(build_py):
    def run(self):
        super().run()
        pkg = os.path.join(self.build_lib, "qfactory")
        for sub, pattern in (("csrc", os.path.join(HERE, "csrc", "*.hip")),
                             ("csrc", os.path.join(HERE, "csrc", "*.cpp")),
                             ("abi", os.path.join(HERE, "..", "include", "*.h"))):
            os.makedirs(os.path.join(pkg, sub), exist_ok=True)
            for path in glob.glob(pattern):
                shutil.copy2(path, os.path.join(pkg, sub, os.path.basename(path)))


if __name__ == "__main__":
    try:
        revision = subprocess.check_output(["git", "rev-parse", "--short", "HEAD"], cwd=HERE).decode().strip()
    except Exception:
        revision = "unknown"
    setuptools.setup(
        name="qfactory",
        version=f"0.0.1+mi355x.{revision}",
        description="QFactory quantized linear layers on MI355X (gfx950): hipcc JIT of hand-written HIP kernels",
        packages=["qfactory", "qfactory.core", "qfactory.jit", "qfactory.integrations"],
        package_dir={"": "."},
        package_data={"qfactory": ["include/*.h"], "qfactory.core": ["*.json"]},
        python_requires=">=3.9",
        cmdclass={"build_py": build_py_with_native_sources},
    )
