"""Builds the C++ torch operators: mops_amd/csrc/torch_ops.cpp -> mops_amd/lib/libmops_amd_torch.so

    python mops_amd/csrc/build_torch_ops.py

Host code only (g++): the operators call libmops.so, which holds the HIP kernels, and link
against the PyTorch this interpreter imports. mops_amd/torch.py loads the result if it is
there and registers the operators from Python otherwise.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIBRARY_DIR = os.path.join(ROOT, "mops_amd", "lib")
OUTPUT = os.path.join(LIBRARY_DIR, "libmops_amd_torch.so")


def build():
    import torch
    from torch.utils import cpp_extension

    if not os.path.exists(os.path.join(LIBRARY_DIR, "libmops.so")):
        raise RuntimeError("build mops_amd/lib/libmops.so first (make -C mops_amd/csrc)")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    build_dir = os.path.join(HERE, "build")
    os.makedirs(build_dir, exist_ok=True)
    target = os.path.join(build_dir, "torch_ops.o")
    includes = [os.path.join(ROOT, "include"), os.path.join(rocm, "include")] + cpp_extension.include_paths()
    compile_command = [
        "g++", "-std=c++17", "-O2", "-fPIC", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        *["-I" + path for path in includes], "-c", os.path.join(HERE, "torch_ops.cpp"), "-o", target,
    ]  # fmt: skip
    link_command = [
        "g++", "-shared", "-o", OUTPUT, target, "-L" + LIBRARY_DIR, "-lmops", "-L" + torch_lib, "-ltorch",
        "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-L" + os.path.join(rocm, "lib"), "-lamdhip64",
        "-Wl,--no-undefined", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib,
    ]  # fmt: skip
    for command in (compile_command, link_command):
        done = subprocess.run(command, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if done.returncode != 0:
            raise RuntimeError(f"{' '.join(command)} failed:\n{done.stdout[-4000:]}")
    return OUTPUT


if __name__ == "__main__":
    print("built", build())
    sys.exit(0)
