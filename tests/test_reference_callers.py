"""The reference's own C++ callers built against this library.

mops-torch (mops-torch/src/*.cpp of lab-cosmo/mops) includes <mops.hpp> and calls the
`mops::` / `mops::cuda::` templates directly (mops-torch/src/opsa.cpp:30-66). The recipe
oracle/build_reference_binding.py compiles its sources, where they lie and unchanged, against
the headers in include/ and links them against libmops.so with undefined symbols forbidden:
every template the callers use exists with the argument types and orders they use.

Here (no GPU): the binding is loaded into torch in a separate process; the operator schemas are
the reference's, and a call with host tensors reaches this library's host entry point (which
refuses: device path only). On a GPU: the reference's operators and their autograd functions
run on top of the HIP kernels and are checked against the oracle.
"""
import importlib.util
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import support

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINDING = os.path.join(ROOT, "oracle", "_ref", "libmops_torch.so")
REFERENCE_SOURCES = "/root/reference/mops-torch/src"

HOST_PROBE = r"""
import sys
import torch
torch.ops.load_library(sys.argv[1])
for name in ("homogeneous_polynomial_evaluation", "sparse_accumulation_of_products", "outer_product_scatter_add",
             "outer_product_scatter_add_with_weights", "sparse_accumulation_scatter_add_with_weights"):
    print("schema", getattr(torch.ops.mops, name).default._schema)
A = torch.ones(4, 2, dtype=torch.float64)
B = torch.ones(4, 3, dtype=torch.float64)
P = torch.zeros(4, dtype=torch.int32)
try:
    torch.ops.mops.outer_product_scatter_add(A, B, P, 2)
    print("call returned")
except RuntimeError as error:
    print("call raised:", str(error).splitlines()[0])
"""

# runs torch.ops.mops.<function> of the reference's binding on cuda:0: forward, backward, and the
# backward of the backward; arrays in, arrays out
DEVICE_PROBE = r"""
import sys
import numpy as np
import torch
torch.ops.load_library(sys.argv[1])
data = np.load(sys.argv[2])
function = str(data["function"])
names = [str(n) for n in data["argument_names"]]
differentiable = [str(n) for n in data["differentiable"]]
device = torch.device("cuda:0")
arguments = []
for name in names:
    value = data[name]
    if value.ndim == 0:
        arguments.append(int(value))
        continue
    tensor = torch.from_numpy(value).to(device)
    if name in differentiable:
        tensor.requires_grad_(True)
    arguments.append(tensor)
output = getattr(torch.ops.mops, function)(*arguments)
grad_output = torch.from_numpy(data["grad_output"]).to(device).requires_grad_(True)
wanted = [a for a, n in zip(arguments, names) if n in differentiable]
gradients = torch.autograd.grad(output, wanted, grad_output, create_graph=True)
results = {"output": output.detach().cpu().numpy()}
for name, gradient in zip(differentiable, gradients):
    results["grad_" + name] = gradient.detach().cpu().numpy()
if bool(data["second_order"]):
    contracted = sum((torch.from_numpy(data["grad_grad_" + n]).to(device) * g).sum() for n, g in zip(differentiable, gradients))
    second = torch.autograd.grad(contracted, [grad_output] + wanted)
    for name, value in zip(["grad_output"] + differentiable, second):
        results["second_" + name] = value.detach().cpu().numpy()
np.savez(sys.argv[3], **results)
print("done")
"""


def _recipe():
    spec = importlib.util.spec_from_file_location(
        "build_reference_binding", os.path.join(ROOT, "oracle", "build_reference_binding.py")
    )
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


@pytest.mark.skipif(not os.path.isdir(REFERENCE_SOURCES), reason="reference sources are not here")
def test_reference_torch_binding_builds_and_loads(tmp_path):
    from tests.test_torch_ops import SCHEMAS

    assert _recipe().build() == BINDING
    probe = subprocess.run([sys.executable, "-c", HOST_PROBE, BINDING], capture_output=True, text=True, cwd=str(tmp_path))
    assert probe.returncode == 0, probe.stdout + probe.stderr
    printed = [line[len("schema "):] for line in probe.stdout.splitlines() if line.startswith("schema ")]
    assert sorted(printed) == sorted(SCHEMAS.values())
    assert "call raised:" in probe.stdout and "device path only" in probe.stdout


CASES = {
    "hpe": lambda: support.hpe_case(31, np.float64, I=70, nA=8, J=40, K=3),
    "sap": lambda: support.sap_case(32, np.float64, I=200, nA=13, nB=7, K=150, nO=20),
    "opsa": lambda: support.opsa_case(33, np.float64, J=500, K=13, L=20, n_out=25, allow_empty=True),
}


@pytest.mark.gpu
@pytest.mark.skipif(not os.path.exists(BINDING), reason="oracle/_ref/libmops_torch.so was not built")
@pytest.mark.parametrize("op", list(CASES))
def test_reference_operators_run_on_the_hip_kernels(oracle, tmp_path, op):
    """The reference has device branches for HPE, SAP and OPSA (none for the weighted operations:
    mops-torch/src/opsaw.cpp:53, sasaw.cpp:90), and for the double backward of SAP only
    (mops-torch/src/sap.cpp:275-320; opsa.cpp:227-233 and hpe.cpp:181-184 refuse on a device before
    they reach the library). Its operators and autograd functions, compiled from its own sources,
    against the oracle."""
    spec = support.OPS[op]
    case = support.add_cotangents(CASES[op](), op)
    names = list(spec.inputs) + (["output_size"] if op in ("sap", "opsa") else [])
    arrays = {name: np.asarray(case[name]) for name in names}
    arrays["grad_output"] = case["grad_output"]
    for name in spec.differentiable:
        arrays["grad_grad_" + name] = case["grad_grad_" + name]
    np.savez(
        tmp_path / "in.npz", function=spec.function, argument_names=names, differentiable=list(spec.differentiable),
        second_order=op == "sap", **arrays,
    )
    probe = subprocess.run(
        [sys.executable, "-c", DEVICE_PROBE, BINDING, str(tmp_path / "in.npz"), str(tmp_path / "out.npz")],
        capture_output=True, text=True, cwd=str(tmp_path),
    )
    assert probe.returncode == 0, probe.stdout + probe.stderr
    results = np.load(tmp_path / "out.npz")
    support.assert_close(results["output"], support.cpu_forward(oracle, op, case), np.float64, f"{op} forward")
    first = support.cpu_vjp(oracle, op, case)
    for name in spec.differentiable:
        support.assert_close(results["grad_" + name], first[name], np.float64, f"{op} grad_{name}")
    if op != "sap":
        return
    second = support.cpu_vjp_vjp(oracle, op, case)
    for name in ["grad_output"] + list(spec.differentiable):
        support.assert_close(results["second_" + name], second[name], np.float64, f"{op} second order {name}")
