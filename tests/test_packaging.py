"""The library as other build systems find it: the CMake package `mops` (target `mops`, as the
reference exports it, mops/CMakeLists.txt:224-257) and the files setup.py ships."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CONFIG_DIR = os.path.join(ROOT, "mops_amd", "cmake", "mops")
LIBRARY = os.path.join(ROOT, "mops_amd", "lib", "libmops.so")

CONSUMER_CMAKE = """
cmake_minimum_required(VERSION 3.16)
project(consumer CXX)
find_package(mops 0.1 CONFIG REQUIRED)
add_executable(consumer main.cpp)
target_link_libraries(consumer mops)
"""

# the C ABI and the C++ API through the same headers the reference installs; no GPU needed:
# the host entry point refuses, with status 1 and a message
CONSUMER_MAIN = """
#include <cstdio>
#include <stdexcept>
#include "mops.h"
#include "mops.hpp"

int main() {
    float value = 0;
    int32_t index = 0;
    mops_tensor_3d_f32_t output{&value, {1, 1, 1}};
    mops_tensor_2d_f32_t A{&value, {1, 1}};
    mops_tensor_2d_f32_t B{&value, {1, 1}};
    mops_tensor_1d_i32_t indices{&index, {1}};
    int status = mops_outer_product_scatter_add_f32(output, A, B, indices);
    std::printf("status %d: %s\\n", status, mops_get_last_error_message());
    try {
        mops::outer_product_scatter_add<double>({nullptr, {0, 0, 0}}, {nullptr, {0, 0}}, {nullptr, {0, 0}}, {nullptr, {0}});
    } catch (const std::runtime_error& error) {
        std::printf("c++: %s\\n", error.what());
    }
    return 0;
}
"""


@pytest.mark.skipif(shutil.which("cmake") is None, reason="cmake is not installed")
@pytest.mark.skipif(not os.path.exists(LIBRARY), reason="libmops.so is not built")
def test_cmake_consumer_links_the_imported_target(tmp_path):
    source = tmp_path / "source"
    build = tmp_path / "build"
    source.mkdir()
    (source / "CMakeLists.txt").write_text(CONSUMER_CMAKE)
    (source / "main.cpp").write_text(CONSUMER_MAIN)
    configure = subprocess.run(
        ["cmake", "-S", str(source), "-B", str(build), f"-Dmops_DIR={CONFIG_DIR}", "-DCMAKE_BUILD_TYPE=Release"],
        capture_output=True, text=True,
    )
    assert configure.returncode == 0, configure.stdout + configure.stderr
    compiled = subprocess.run(["cmake", "--build", str(build)], capture_output=True, text=True)
    assert compiled.returncode == 0, compiled.stdout + compiled.stderr
    ran = subprocess.run([str(build / "consumer")], capture_output=True, text=True)
    assert ran.returncode == 0, ran.stdout + ran.stderr
    assert "status 1: " in ran.stdout and "device path only" in ran.stdout
    assert "c++: " in ran.stdout


def test_version_file_accepts_the_reference_version(tmp_path):
    if shutil.which("cmake") is None:
        pytest.skip("cmake is not installed")
    script = tmp_path / "probe.cmake"
    script.write_text(
        f"""
set(PACKAGE_FIND_VERSION 0.1.0)
set(PACKAGE_FIND_VERSION_MAJOR 0)
set(PACKAGE_FIND_VERSION_MINOR 1)
include({CONFIG_DIR}/mops-config-version.cmake)
message("compatible=${{PACKAGE_VERSION_COMPATIBLE}} exact=${{PACKAGE_VERSION_EXACT}}")
set(PACKAGE_FIND_VERSION 0.2.0)
set(PACKAGE_FIND_VERSION_MINOR 2)
include({CONFIG_DIR}/mops-config-version.cmake)
message("other=${{PACKAGE_VERSION_COMPATIBLE}}")
"""
    )
    result = subprocess.run(["cmake", "-P", str(script)], capture_output=True, text=True)
    text = result.stdout + result.stderr
    assert "compatible=TRUE exact=TRUE" in text and "other=FALSE" in text


@pytest.mark.skipif(not os.path.exists(LIBRARY), reason="libmops.so is not built")
def test_setup_ships_library_headers_and_cmake_files(tmp_path):
    """`setup.py build_py` (what `pip install .` runs) puts the library, the headers and the CMake
    package into the package directory."""
    import sys

    built = subprocess.run(
        [sys.executable, "setup.py", "-q", "build_py", "--build-lib", str(tmp_path)],
        cwd=ROOT, capture_output=True, text=True,
    )
    assert built.returncode == 0, built.stdout + built.stderr
    package = tmp_path / "mops_amd"
    for relative in ("lib/libmops.so", "lib/libmops_amd_torch.so", "include/mops.h", "include/mops/opsa.hpp", "cmake/mops/mops-config.cmake",
                     "cmake/mops/mops-config-version.cmake", "torch.py"):
        assert (package / relative).exists(), relative
