"""Packaging of the Python front-end together with the HIP library it loads.

``pip install .`` (or ``python setup.py build``) compiles ``mops_amd/csrc`` with
hipcc for gfx950 through its Makefile and ships ``mops_amd/lib/libmops.so`` as
package data, the way the reference's wheels carry their ``libmops.so``
(python/mops/setup.py of lab-cosmo/mops builds it with CMake).
"""
import os
import shutil
import subprocess

from setuptools import setup
from setuptools.command.build_py import build_py

ROOT = os.path.dirname(os.path.abspath(__file__))


class build_py_with_library(build_py):
    def run(self):
        subprocess.run(["make", "-C", os.path.join(ROOT, "mops_amd", "csrc"), "-j8"], check=True)
        try:
            import torch  # noqa: F401
        except ImportError:
            print("torch is not installed: torch.ops.mops.* will be registered from Python when it is")
        else:
            import sys

            subprocess.run([sys.executable, os.path.join(ROOT, "mops_amd", "csrc", "build_torch_ops.py")], check=True)
        super().run()
        # the C / C++ headers travel inside the package, where cmake/mops/mops-config.cmake looks first
        target = os.path.join(self.build_lib, "mops_amd", "include")
        shutil.rmtree(target, ignore_errors=True)
        shutil.copytree(os.path.join(ROOT, "include"), target)


setup(
    name="mops-amd",
    version="0.1.0",
    description="lab-cosmo/mops operations on AMD MI355X (gfx950): HIP kernels behind the mops C ABI",
    packages=["mops_amd"],
    package_data={"mops_amd": ["lib/libmops.so", "lib/libmops_amd_torch.so", "cmake/mops/*.cmake"]},
    python_requires=">=3.9",
    install_requires=["numpy"],
    extras_require={"torch": ["torch"]},
    cmdclass={"build_py": build_py_with_library},
)
