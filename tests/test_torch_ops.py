"""torch.ops.mops.*: schemas (as mops-torch/src/register.cpp of the reference), values, autograd."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import mops_amd.torch  # noqa: F401  (registers the operators)
from tests import support

SCHEMAS = {
    "homogeneous_polynomial_evaluation": "mops::homogeneous_polynomial_evaluation(Tensor A, Tensor C, Tensor indices_A) -> Tensor",
    "outer_product_scatter_add": "mops::outer_product_scatter_add(Tensor A, Tensor B, Tensor indices_output, int output_size) -> Tensor",
    "sparse_accumulation_of_products": "mops::sparse_accumulation_of_products(Tensor A, Tensor B, Tensor C, Tensor indices_A, Tensor indices_B, Tensor indices_output, int output_size) -> Tensor",
    "outer_product_scatter_add_with_weights": "mops::outer_product_scatter_add_with_weights(Tensor A, Tensor B, Tensor W, Tensor indices_W, Tensor indices_output) -> Tensor",
    "sparse_accumulation_scatter_add_with_weights": "mops::sparse_accumulation_scatter_add_with_weights(Tensor A, Tensor B, Tensor C, Tensor W, Tensor indices_A, Tensor indices_W_1, Tensor indices_W_2, Tensor indices_output_1, Tensor indices_output_2, int output_size) -> Tensor",
}  # fmt: skip

SMALL = {
    "hpe": lambda d: support.hpe_case(11, d, I=9, nA=5, J=12, K=3),
    "sap": lambda d: support.sap_case(12, d, I=70, nA=4, nB=3, K=15, nO=5),
    "opsa": lambda d: support.opsa_case(13, d, J=50, K=3, L=4, n_out=6, allow_empty=True),
    "opsaw": lambda d: support.opsaw_case(14, d, E=50, K=3, L=4, n_nodes=6, allow_empty=True),
    "sasaw": lambda d: support.sasaw_case(15, d, E=40, nA=3, L=4, n_nodes=5, n2=3, n3=4, N=11, allow_empty=True),
}  # fmt: skip


def arguments(op, case):
    """Arguments of torch.ops.mops.<op> in schema order."""
    tensors = [case[name] for name in support.OPS[op].inputs]
    if op in ("sap", "opsa", "sasaw"):
        tensors.append(case["output_size"])
    return tensors


def test_schemas_match_the_reference():
    for name, schema in SCHEMAS.items():
        assert str(getattr(torch.ops.mops, name).default._schema) == schema


def test_cpp_operators_are_used_when_built():
    """mops_amd/lib/libmops_amd_torch.so (mops_amd/csrc/torch_ops.cpp), if there, is what registers the operators."""
    built = os.path.exists(mops_amd.torch.CPP_OPERATORS_PATH)
    forced = os.environ.get("MOPS_AMD_TORCH_PYTHON_OPS", "0") not in ("", "0")
    assert mops_amd.torch.OPERATORS_FROM == ("c++" if built and not forced else "python")


@pytest.mark.gpu
@pytest.mark.skipif(mops_amd.torch.OPERATORS_FROM != "c++", reason="this process already runs the Python operators")
def test_python_operators_in_a_process_of_their_own():
    """The operators registered from Python (the fallback without the C++ library): the same tests, in a
    process that is told to use them."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    environment = dict(os.environ, MOPS_AMD_TORCH_PYTHON_OPS="1")
    done = subprocess.run(
        [sys.executable, "-m", "pytest", os.path.join(root, "tests", "test_torch_ops.py"), "-m", "gpu", "-q", "-x",
         "-p", "no:cacheprovider"],
        cwd=root, env=environment, capture_output=True, text=True,
    )
    assert done.returncode == 0, done.stdout[-3000:] + done.stderr[-2000:]
    assert " passed" in done.stdout


def test_host_tensors_are_refused():
    case = SMALL["opsa"](np.float64)
    tensors = [torch.from_numpy(v) if isinstance(v, np.ndarray) else v for v in arguments("opsa", case)]
    with pytest.raises(RuntimeError, match="device path only"):
        torch.ops.mops.outer_product_scatter_add(*tensors)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("op", list(SMALL))
def test_operator_values(oracle, device, op, dtype):
    case = SMALL[op](dtype)
    expected = support.cpu_forward(oracle, op, case)
    on_device = support.to_device(case, device)
    operator = getattr(torch.ops.mops, support.OPS[op].function)
    actual = operator(*arguments(op, on_device))
    support.assert_close(actual.cpu().numpy(), expected, dtype, op)


@pytest.mark.gpu
@pytest.mark.parametrize("op", list(SMALL))
def test_operator_gradients(oracle, device, op):
    """Backward of the operator = the oracle's vjp; and torch's own finite-difference gradcheck."""
    case = SMALL[op](np.float64)
    expected = support.cpu_vjp(oracle, op, case)
    on_device = support.to_device(case, device)
    spec = support.OPS[op]
    for name in spec.differentiable:
        on_device[name].requires_grad_(True)
    operator = getattr(torch.ops.mops, spec.function)
    output = operator(*arguments(op, on_device))
    output.backward(on_device["grad_output"])
    for name in spec.differentiable:
        support.assert_close(on_device[name].grad.cpu().numpy(), expected[name], np.float64, f"{op} grad_{name}")
    for name in spec.differentiable:
        on_device[name].grad = None
    assert torch.autograd.gradcheck(operator, arguments(op, on_device), fast_mode=True)


@pytest.mark.gpu
def test_only_requested_gradients_are_computed(device):
    case = support.to_device(SMALL["opsaw"](np.float64), device)
    case["B"].requires_grad_(True)
    output = torch.ops.mops.outer_product_scatter_add_with_weights(*arguments("opsaw", case))
    output.sum().backward()
    assert case["B"].grad is not None and case["A"].grad is None and case["W"].grad is None


@pytest.mark.gpu
@pytest.mark.parametrize("op", support.SECOND_ORDER)
def test_operator_second_derivatives(oracle, device, op):
    """Double backward = the oracle's vjp_vjp; torch's gradgradcheck as the reference's own tests
    (python/mops-torch/tests/{hpe,sap,opsa}.py)."""
    case = support.add_cotangents(SMALL[op](np.float64), op)
    expected = support.cpu_vjp_vjp(oracle, op, case)
    on_device = support.to_device(case, device)
    spec = support.OPS[op]
    for name in spec.differentiable + ["grad_output"]:
        on_device[name].requires_grad_(True)
    operator = getattr(torch.ops.mops, spec.function)
    output = operator(*arguments(op, on_device))
    wanted = [on_device[name] for name in spec.differentiable]
    gradients = torch.autograd.grad(output, wanted, on_device["grad_output"], create_graph=True)
    contracted = sum((on_device["grad_grad_" + n] * g).sum() for n, g in zip(spec.differentiable, gradients))
    second = torch.autograd.grad(contracted, [on_device["grad_output"]] + wanted)
    for name, value in zip(["grad_output"] + spec.differentiable, second):
        support.assert_close(value.cpu().numpy(), expected[name], np.float64, f"{op} second order {name}")
    assert torch.autograd.gradgradcheck(operator, arguments(op, on_device), fast_mode=True)


class ScriptedHpe(torch.nn.Module):
    def forward(self, A, C, indices_A):
        return torch.ops.mops.homogeneous_polynomial_evaluation(A, C, indices_A)


class ScriptedSap(torch.nn.Module):
    def forward(self, A, B, C, indices_A, indices_B, indices_output, output_size: int):
        return torch.ops.mops.sparse_accumulation_of_products(
            A, B, C, indices_A, indices_B, indices_output, output_size
        )


class ScriptedOpsa(torch.nn.Module):
    def forward(self, A, B, indices_output, output_size: int):
        return torch.ops.mops.outer_product_scatter_add(A, B, indices_output, output_size)


class ScriptedOpsaw(torch.nn.Module):
    def forward(self, A, B, W, indices_W, indices_output):
        return torch.ops.mops.outer_product_scatter_add_with_weights(A, B, W, indices_W, indices_output)


class ScriptedSasaw(torch.nn.Module):
    def forward(
        self, A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, output_size: int
    ):
        return torch.ops.mops.sparse_accumulation_scatter_add_with_weights(
            A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, output_size
        )


SCRIPTED = {"hpe": ScriptedHpe, "sap": ScriptedSap, "opsa": ScriptedOpsa, "opsaw": ScriptedOpsaw, "sasaw": ScriptedSasaw}


@pytest.mark.parametrize("op", list(SCRIPTED))
def test_modules_can_be_scripted(op):
    """Scripting resolves the operator against its schema (no GPU needed), as
    python/mops-torch/tests/torchscript.py:7-260 of the reference does for every operation."""
    scripted = torch.jit.script(SCRIPTED[op]())
    assert "mops::" + support.OPS[op].function in str(scripted.graph)


@pytest.mark.gpu
@pytest.mark.parametrize("op", list(SCRIPTED))
def test_torchscript_save_and_load(oracle, device, tmp_path, op):
    """A scripted module of every operation survives save / load and gives the oracle's values
    and gradients."""
    case = SMALL[op](np.float64)
    on_device = support.to_device(case, device)
    spec = support.OPS[op]
    scripted = torch.jit.script(SCRIPTED[op]())
    path = str(tmp_path / f"{op}.pt")
    scripted.save(path)
    loaded = torch.jit.load(path)
    actual = loaded(*arguments(op, on_device))
    support.assert_close(actual.cpu().numpy(), support.cpu_forward(oracle, op, case), np.float64, f"scripted {op}")
    for name in spec.differentiable:
        on_device[name].requires_grad_(True)
    loaded(*arguments(op, on_device)).backward(on_device["grad_output"])
    expected = support.cpu_vjp(oracle, op, case)
    for name in spec.differentiable:
        support.assert_close(
            on_device[name].grad.cpu().numpy(), expected[name], np.float64, f"scripted {op} grad_{name}"
        )
