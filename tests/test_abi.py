"""The C-ABI boundary, without a GPU: exported symbols, argument lists, error contract.

No compute call is made here (the library is the device path only); the
host-memory entry points validate their arguments exactly like the
reference's and then report that host arithmetic is not part of this library,
which is enough to pin statuses and messages.
"""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from mops_amd._c_api import SIGNATURES, _KINDS
from mops_amd.status import MopsError

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")


@pytest.fixture(scope="module")
def preprocessed_header():
    result = subprocess.run(
        ["gcc", "-E", "-P", "-I" + INCLUDE, os.path.join(INCLUDE, "mops.h")],
        capture_output=True, text=True, check=True,
    )  # fmt: skip
    return result.stdout.replace('__attribute__((visibility("default")))', "")


@pytest.fixture(scope="module")
def prototypes(preprocessed_header):
    """{symbol: [C type of every parameter]} of every function include/mops.h declares."""
    found = {}
    pattern = re.compile(r"(?:int|void\s*\*|const char\s*\*)\s*(mops_\w+)\s*\(([^)]*)\)\s*;")
    for name, parameters in pattern.findall(preprocessed_header):
        types = []
        for parameter in parameters.split(","):
            parameter = parameter.strip()
            if parameter in ("", "void"):
                continue
            types.append(" ".join(parameter.split()[:-1]) if " " in parameter else parameter)
        found[name] = types
    return found


@pytest.fixture(scope="module")
def libraries():
    from mops_amd._c_lib import device_library, host_library

    return device_library(), host_library()


def test_header_declares_the_reference_abi(prototypes):
    # mops/include/mops/*.h of the reference: 5 operations x {fwd, vjp, vjp_vjp}
    # x {f32, f64} x {host, cuda} + the error message getter
    reference = [name for name in prototypes if not name.startswith("mops_amd_")]
    assert len(reference) == 61
    for function in SIGNATURES:
        for tag in ("f32", "f64"):
            assert f"mops_{function}_{tag}" in prototypes
            assert f"mops_cuda_{function}_{tag}" in prototypes
    assert "mops_get_last_error_message" in prototypes


def test_library_exports_every_declared_symbol(prototypes, libraries):
    device, _ = libraries
    missing = [name for name in prototypes if not hasattr(device.cdll, name)]
    assert not missing


def test_library_exports_nothing_else():
    path = os.path.join(ROOT, "mops_amd", "lib", "libmops.so")
    listing = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True)
    c_symbols = sorted(
        line.split()[-1] for line in listing.stdout.splitlines() if re.search(r" T mops_\w+$", line)
    )
    result = subprocess.run(
        ["gcc", "-E", "-P", "-I" + INCLUDE, os.path.join(INCLUDE, "mops.h")],
        capture_output=True, text=True, check=True,
    )  # fmt: skip
    declared = sorted(set(re.findall(r"\b(mops_\w+)\s*\(", result.stdout)))
    assert c_symbols == declared


def test_python_argument_lists_match_the_header(prototypes):
    struct_of = {
        ("R1", "f32"): "mops_tensor_1d_f32_t", ("R2", "f32"): "mops_tensor_2d_f32_t",
        ("R3", "f32"): "mops_tensor_3d_f32_t", ("Q3", "f32"): "mops_tensor_2d_f32_t",
        ("R1", "f64"): "mops_tensor_1d_f64_t", ("R2", "f64"): "mops_tensor_2d_f64_t",
        ("R3", "f64"): "mops_tensor_3d_f64_t", ("Q3", "f64"): "mops_tensor_2d_f64_t",
    }  # fmt: skip
    for function, signature in SIGNATURES.items():
        for tag in ("f32", "f64"):
            expected = [
                f"mops_tensor_{_KINDS[kind][0]}d_i32_t" if _KINDS[kind][1] else struct_of[(kind, tag)]
                for kind, _ in signature
            ]
            for prefix in ("mops_", "mops_cuda_"):
                assert prototypes[f"{prefix}{function}_{tag}"] == expected, (prefix, function, tag)


def test_struct_layout_is_pointer_then_int64_extents(preprocessed_header):
    # mops/include/mops/tensor.h:11-49 of the reference
    for ndim in (1, 2, 3):
        for tag, ctype in (("f32", "float"), ("f64", "double")):
            pattern = rf"struct mops_tensor_{ndim}d_{tag}_t\s*{{\s*{ctype}\s*\*\s*(?:__restrict__\s*)?data;\s*int64_t shape\[{ndim}\];"
            assert re.search(pattern, preprocessed_header), (ndim, tag)
    for ndim in (1, 2):
        pattern = rf"struct mops_tensor_{ndim}d_i32_t\s*{{\s*int32_t\s*\*\s*(?:__restrict__\s*)?data;\s*int64_t shape\[{ndim}\];"
        assert re.search(pattern, preprocessed_header), ndim


def opsa_arguments(n_a=4, n_b=4, index_dtype=np.int32, dtype=np.float64):
    return (
        np.zeros((3, 2, 2), dtype), np.zeros((n_a, 2), dtype), np.zeros((n_b, 2), dtype),
        np.zeros(n_a, index_dtype),
    )  # fmt: skip


def test_status_and_message_of_a_shape_error(libraries):
    _, host = libraries
    with pytest.raises(MopsError) as error:
        host.call("outer_product_scatter_add", *opsa_arguments(n_a=4, n_b=5))
    assert error.value.status == 1
    # message format of mops/src/internal/checks/utils.hpp:32-36
    assert str(error.value) == (
        "Dimension mismatch: the sizes of A along dimension 0 and B along dimension 0 must match in "
        "cpu_outer_product_scatter_add"
    )
    assert host.last_error() == str(error.value)


def test_index_out_of_bounds_message(libraries):
    _, host = libraries
    output, A, B, index = opsa_arguments()
    index[:] = [0, 1, 2, 3]
    with pytest.raises(MopsError) as error:
        host.call("outer_product_scatter_add", output, A, B, index)
    assert error.value.status == 1
    assert "Index array indices_output in operation cpu_outer_product_scatter_add contains elements up to 3" in str(
        error.value
    )


def test_negative_extent_is_rejected(libraries):
    from mops_amd._c_api import STRUCTS

    _, host = libraries
    function = host.function("outer_product_scatter_add", "f64")
    output = STRUCTS[(3, "f64")]()
    output.shape[0] = -1
    status = function(output, STRUCTS[(2, "f64")](), STRUCTS[(2, "f64")](), STRUCTS[(1, "i32")]())
    assert status == 1
    assert "does not fit in size_t" in host.last_error()


def test_host_arithmetic_is_refused_loudly(libraries):
    _, host = libraries
    with pytest.raises(MopsError) as error:
        host.call("outer_product_scatter_add", *opsa_arguments())
    assert error.value.status == 1
    assert "device path only" in str(error.value)


def test_vjp_without_any_gradient_is_a_no_op(libraries):
    _, host = libraries
    output, A, B, index = opsa_arguments()
    host.call("outer_product_scatter_add_vjp", None, None, output, A, B, index)


def test_not_implemented_second_derivatives(libraries):
    # mops/src/opsaw/cpu.tpp:133-150, mops/src/sasaw/cpu.tpp:173-194
    device, host = libraries
    for library in (host, device):
        symbol = getattr(library.cdll, library.prefix + "outer_product_scatter_add_with_weights_vjp_vjp_f32")
        assert symbol is not None


def test_amd_additions_have_c_linkage(libraries):
    device, _ = libraries
    assert device.cdll.mops_amd_set_synchronous(1) in (0, 1)
    assert device.cdll.mops_amd_set_stream(None) == 0
    assert device.cdll.mops_amd_get_stream() in (None, 0)
    assert device.cdll.mops_amd_kernel_timing(0) in (0, 1)
    total = ctypes.c_double(-1.0)
    launches = ctypes.c_int64(-1)
    assert device.cdll.mops_amd_kernel_time(ctypes.byref(total), ctypes.byref(launches)) == 0
    assert (total.value, launches.value) == (0.0, 0)
