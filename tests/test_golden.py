"""Known-answer fixtures (tests/golden/golden.npz) against the oracle and the HIP path.

The fixture's expected values come from dense float64 torch formulations and
torch.autograd (tests/golden/make_golden.py), code that shares nothing with
oracle/ or mops_amd/csrc. The inputs are exact in float32, so both precisions
are checked against the same float64 answers, at the north star's bar (the
oracle itself is within 0.02 of it on every fixture).
"""
import os

import numpy as np
import pytest

from tests import support
from tests.support import OPS, assert_close

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden.npz")
DTYPES = [np.float32, np.float64]


def load_cases():
    data = np.load(GOLDEN, allow_pickle=False)
    cases = {}
    for key in data.files:
        op, name, side, field = key.split("/")
        entry = cases.setdefault(f"{op}/{name}", {"in": {}, "out": {}})
        entry[side][field] = data[key]
    return cases


CASES = load_cases()


def typed_case(name, dtype):
    case = {}
    for key, value in CASES[name]["in"].items():
        if value.ndim == 0:
            case[key] = int(value)
        elif value.dtype == np.float64:
            case[key] = np.ascontiguousarray(value.astype(dtype))
        else:
            case[key] = np.ascontiguousarray(value)
    if name.startswith("opsaw"):
        case["output_size"] = case["W"].shape[0]
    return case


def test_fixture_inputs_are_exact_in_float32():
    for name, entry in CASES.items():
        for key, value in entry["in"].items():
            if value.dtype == np.float64:
                assert np.array_equal(value.astype(np.float32).astype(np.float64), value), (name, key)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_against_golden(oracle, name, dtype):
    op = name.split("/")[0]
    case = typed_case(name, dtype)
    expected = CASES[name]["out"]
    assert_close(support.cpu_forward(oracle, op, case), expected["output"], dtype, f"{name} output")
    gradients = support.cpu_vjp(oracle, op, case)
    for key in OPS[op].differentiable:
        assert_close(gradients[key], expected["grad_" + key], dtype, f"{name} grad_{key}")
    if op in support.SECOND_ORDER:
        second = support.cpu_vjp_vjp(oracle, op, case)
        assert_close(second["grad_output"], expected["grad_grad_output"], dtype, f"{name} grad_grad_output")
        for key in OPS[op].differentiable:
            assert_close(second[key], expected[f"grad_{key}_2"], dtype, f"{name} grad_{key}_2")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "f64"])
@pytest.mark.parametrize("name", sorted(CASES))
def test_hip_against_golden(device, name, dtype):
    op = name.split("/")[0]
    case = support.to_device(typed_case(name, dtype), device)
    expected = CASES[name]["out"]
    output = support.hip_forward(op, case).cpu().numpy()
    assert_close(output, expected["output"], dtype, f"{name} output")
    gradients = support.hip_vjp(op, case)
    for key in OPS[op].differentiable:
        assert_close(gradients[key].cpu().numpy(), expected["grad_" + key], dtype, f"{name} grad_{key}")
    if op in support.SECOND_ORDER:
        second = support.hip_vjp_vjp(op, case)
        assert_close(
            second["grad_output"].cpu().numpy(), expected["grad_grad_output"], dtype, f"{name} grad_grad_output"
        )
        for key in OPS[op].differentiable:
            assert_close(second[key].cpu().numpy(), expected[f"grad_{key}_2"], dtype, f"{name} grad_{key}_2")
