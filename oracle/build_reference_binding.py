"""Compiles the reference's torch binding against THIS repository's library (test infrastructure).

    python oracle/build_reference_binding.py      ->  oracle/_ref/libmops_torch.so

mops-torch (mops-torch/src/*.cpp of lab-cosmo/mops) is the reference's own caller of the
operations: it registers torch.ops.mops.* with their autograd functions and calls the
`mops::` / `mops::cuda::` templates of <mops.hpp> (mops-torch/src/opsa.cpp:30-60). Its sources
are complete without the reference's build system, so they are compiled where they lie under
/root/reference, unchanged, with g++, against include/ and mops_amd/lib/libmops.so of this
repository. The result is not an oracle for arithmetic: tests/test_reference_binding.py uses it
to run the reference's operators, unmodified, on top of the HIP kernels. (The reference LIBRARY
itself cannot be compiled this way: its translation units include mops/exports.h, which only its
CMake configuration generates.)

Nothing is copied from the reference; the only output is oracle/_ref/libmops_torch.so, which git
ignores. Does nothing, successfully, where /root/reference is absent.
"""
import os
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE = "/root/reference/mops-torch"
OUTPUT_DIR = os.path.join(ROOT, "oracle", "_ref")
OUTPUT = os.path.join(OUTPUT_DIR, "libmops_torch.so")


def build():
    source_dir = os.path.join(REFERENCE, "src")
    if not os.path.isdir(source_dir):
        print("reference sources are not here: nothing to build")
        return None
    import torch
    from torch.utils import cpp_extension

    library_dir = os.path.join(ROOT, "mops_amd", "lib")
    if not os.path.exists(os.path.join(library_dir, "libmops.so")):
        raise RuntimeError("build mops_amd/lib/libmops.so first (make -C mops_amd/csrc)")
    sources = sorted(name for name in os.listdir(source_dir) if name.endswith(".cpp"))
    includes = [os.path.join(REFERENCE, "include"), os.path.join(ROOT, "include")] + cpp_extension.include_paths()
    # MOPS_CUDA_ENABLED: what the reference's build defines when its device path is compiled in
    # (mops-torch/src/opsa.cpp:48-66); it turns on the calls of mops::cuda::*
    flags = ["-std=c++17", "-O1", "-fPIC", "-DMOPS_CUDA_ENABLED",
             f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    flags += ["-I" + path for path in includes]
    os.makedirs(OUTPUT_DIR, exist_ok=True)
    with tempfile.TemporaryDirectory(dir=OUTPUT_DIR) as objects:

        def compile_one(name):
            target = os.path.join(objects, name + ".o")
            done = subprocess.run(
                ["g++", *flags, "-c", os.path.join(source_dir, name), "-o", target],
                stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
            )
            if done.returncode != 0:
                raise RuntimeError(f"{name} does not compile against include/:\n{done.stdout[-4000:]}")
            return target

        with ThreadPoolExecutor(max_workers=4) as pool:
            targets = list(pool.map(compile_one, sources))
        torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
        linked = subprocess.run(
            ["g++", "-shared", "-o", OUTPUT, *targets, "-L" + library_dir, "-lmops", "-L" + torch_lib,
             "-ltorch", "-ltorch_cpu", "-lc10", "-Wl,--no-undefined",
             "-Wl,-rpath,$ORIGIN/../../mops_amd/lib", "-Wl,-rpath," + torch_lib],
            stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
        )
        if linked.returncode != 0:
            raise RuntimeError(f"link failed:\n{linked.stdout[-4000:]}")
    print("built", OUTPUT)
    return OUTPUT


if __name__ == "__main__":
    build()
    sys.exit(0)
