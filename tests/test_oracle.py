"""Pins of the CPU oracle (no GPU needed).

The reference ships no golden vectors and its library cannot be compiled in
this build (it needs a CMake-generated header), so the oracle is pinned
against what the mathematics fixes, with checks chosen so that a dropped
term, a swapped index or a transposed operand fails at least one of them:

* dense numpy formulations that share no code with it (einsum / add.at);
* special cases with textbook answers (order 0 and 1 polynomials, a single
  segment = one matrix product, identity-like tables);
* every vjp against central finite differences of the oracle's own forward
  and against the adjoint identity <vjp(g), dx> = <g, J dx> using linearity;
* the second-order functions (vjp_vjp of HPE, SAP, OPSA) against central
  differences of the pinned vjps, against the forward pass by linearity, and
  with absent cotangents against zero cotangents;
* empty segments give exact zeros; unsorted scatter indices are accepted;
* the committed golden vectors (tests/golden).
"""
import numpy as np
import pytest

from tests import support
from tests.support import OPS, assert_close, cpu_forward, cpu_vjp

DTYPES = [np.float32, np.float64]

SMALL = {
    "hpe": lambda seed, dtype: support.hpe_case(seed, dtype, I=37, nA=11, J=53, K=3),
    "sap": lambda seed, dtype: support.sap_case(seed, dtype, I=45, nA=6, nB=5, K=70, nO=8),
    "opsa": lambda seed, dtype: support.opsa_case(seed, dtype, J=90, K=5, L=7, n_out=12, allow_empty=True),
    "opsaw": lambda seed, dtype: support.opsaw_case(seed, dtype, E=90, K=5, L=7, n_nodes=12, allow_empty=True),
    "sasaw": lambda seed, dtype: support.sasaw_case(
        seed, dtype, E=80, nA=5, L=6, n_nodes=11, n2=4, n3=3, N=40, allow_empty=True
    ),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("op", list(OPS))
def test_forward_matches_dense_formulation(oracle, op, dtype):
    case = SMALL[op](1, dtype)
    assert_close(cpu_forward(oracle, op, case), OPS[op].dense(case), dtype, op)


@pytest.mark.parametrize("op", list(OPS))
def test_vjp_matches_finite_differences(oracle, op):
    """d<g, f(x)>/dx by central differences, float64."""
    case = SMALL[op](2, np.float64)
    gradients = cpu_vjp(oracle, op, case)
    g = case["grad_output"]
    h = 1e-6
    rng = np.random.default_rng(7)
    for name in OPS[op].differentiable:
        x = case[name]
        for _ in range(12):
            position = tuple(rng.integers(0, s) for s in x.shape)
            saved = x[position]
            x[position] = saved + h
            plus = np.sum(g * cpu_forward(oracle, op, case))
            x[position] = saved - h
            minus = np.sum(g * cpu_forward(oracle, op, case))
            x[position] = saved
            numeric = (plus - minus) / (2 * h)
            analytic = gradients[name][position]
            assert abs(numeric - analytic) <= 1e-6 * max(1.0, abs(numeric)), (op, name, position)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("op", ["sap", "opsa", "opsaw", "sasaw"])
def test_vjp_adjoint_identity(oracle, op, dtype):
    """These operations are linear in each argument separately, so
    f(.., x + dx, ..) - f(.., x, ..) = J_x dx exactly and
    <vjp_x(g), dx> must equal <g, f(dx in place of x)>."""
    case = SMALL[op](3, dtype)
    rng = np.random.default_rng(11)
    gradients = cpu_vjp(oracle, op, case)
    for name in OPS[op].differentiable:
        dx = rng.normal(size=case[name].shape).astype(dtype)
        swapped = dict(case)
        swapped[name] = dx
        right = np.sum(case["grad_output"].astype(np.float64) * cpu_forward(oracle, op, swapped))
        left = np.sum(gradients[name].astype(np.float64) * dx)
        scale = np.sum(np.abs(gradients[name].astype(np.float64) * dx))
        assert abs(left - right) <= support.TOLERANCE[np.dtype(dtype)] * 50 * scale, (op, name)


def test_hpe_order_zero_and_one(oracle):
    rng = np.random.default_rng(5)
    A = rng.normal(size=(19, 6))
    C = rng.normal(size=9)
    # order 0: every monomial is its coefficient
    case = {"A": A, "C": C, "indices_A": np.zeros((9, 0), dtype=np.int32), "grad_output": np.ones(19)}
    np.testing.assert_allclose(cpu_forward(oracle, "hpe", case), np.full(19, C.sum()), rtol=1e-14)
    assert np.all(cpu_vjp(oracle, "hpe", case)["A"] == 0.0)
    # order 1: a matrix-vector product with the coefficients scattered by feature
    P = rng.integers(0, 6, size=(9, 1)).astype(np.int32)
    case = {"A": A, "C": C, "indices_A": P, "grad_output": rng.normal(size=19)}
    weights = np.zeros(6)
    np.add.at(weights, P[:, 0], C)
    np.testing.assert_allclose(cpu_forward(oracle, "hpe", case), A @ weights, rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(
        cpu_vjp(oracle, "hpe", case)["A"], np.outer(case["grad_output"], weights), rtol=1e-12, atol=1e-13
    )


def test_hpe_repeated_factor_gradient(oracle):
    """x0^2 * x1: d/dx0 = 2 x0 x1, d/dx1 = x0^2 (a repeated index counts twice)."""
    A = np.array([[3.0, 5.0], [-2.0, 0.5]])
    case = {
        "A": A,
        "C": np.array([1.5]),
        "indices_A": np.array([[0, 0, 1]], dtype=np.int32),
        "grad_output": np.array([1.0, 2.0]),
    }
    np.testing.assert_allclose(cpu_forward(oracle, "hpe", case), 1.5 * A[:, 0] ** 2 * A[:, 1])
    expected = np.stack([1.5 * 2 * A[:, 0] * A[:, 1], 1.5 * A[:, 0] ** 2], axis=1) * case["grad_output"][:, None]
    np.testing.assert_allclose(cpu_vjp(oracle, "hpe", case)["A"], expected)


def test_opsa_single_segment_is_a_matrix_product(oracle):
    rng = np.random.default_rng(9)
    A = rng.normal(size=(23, 4))
    B = rng.normal(size=(23, 6))
    case = {
        "A": A, "B": B, "indices_output": np.zeros(23, dtype=np.int32), "output_size": 1,
        "grad_output": rng.normal(size=(1, 4, 6)),
    }  # fmt: skip
    np.testing.assert_allclose(cpu_forward(oracle, "opsa", case)[0], A.T @ B, rtol=1e-12, atol=1e-13)
    g = case["grad_output"][0]
    grads = cpu_vjp(oracle, "opsa", case)
    np.testing.assert_allclose(grads["A"], B @ g.T, rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(grads["B"], A @ g, rtol=1e-12, atol=1e-13)


def test_opsaw_unit_weights_is_opsa(oracle):
    case = SMALL["opsaw"](4, np.float64)
    case["W"][:] = 1.0
    plain = {k: case[k] for k in ("A", "B", "indices_output", "grad_output")}
    plain["output_size"] = case["W"].shape[0]
    # not bit-equal: with fused multiply-add, a*b*1 + o rounds a*b first
    np.testing.assert_allclose(
        cpu_forward(oracle, "opsaw", case), cpu_forward(oracle, "opsa", plain), rtol=1e-13, atol=1e-14
    )


def test_sasaw_reduces_to_opsaw(oracle):
    """With a one-entry table, A of width 1 and W of depth 1,
    SASAW is OPSAW with K = 1 scaled by C."""
    rng = np.random.default_rng(21)
    E, L, n = 40, 5, 7
    case = support.sasaw_case(6, np.float64, E=E, nA=1, L=L, n_nodes=n, n2=1, n3=1, N=1)
    case["C"][:] = 2.5
    out = cpu_forward(oracle, "sasaw", case)
    opsaw = {
        "A": case["A"], "B": case["B"], "W": case["W"][:, 0, :], "indices_W": case["indices_W_1"],
        "indices_output": case["indices_output_1"],
    }  # fmt: skip
    np.testing.assert_allclose(
        out[:, 0, :], 2.5 * cpu_forward(oracle, "opsaw", opsaw)[:, 0, :], rtol=1e-13, atol=1e-14
    )
    del rng


@pytest.mark.parametrize("op", ["opsa", "opsaw", "sasaw"])
def test_rows_without_edges_are_exactly_zero(oracle, op):
    case = SMALL[op](8, np.float64)
    key = "indices_output_1" if op == "sasaw" else "indices_output"
    index = case[key]
    index[index == 1] = 2  # the reference's "no neighbours" construction
    case[key] = np.sort(index)
    out = cpu_forward(oracle, op, case)
    assert np.all(out[1] == 0.0)
    assert_close(out, OPS[op].dense(case), np.float64, op)


@pytest.mark.parametrize("op", ["opsa", "opsaw", "sasaw"])
def test_unsorted_scatter_index_on_the_host(oracle, op):
    """The host algorithm buckets rows, so the scatter index need not be sorted."""
    case = SMALL[op](10, np.float64)
    key = "indices_output_1" if op == "sasaw" else "indices_output"
    rng = np.random.default_rng(3)
    case[key] = rng.permutation(case[key])
    assert_close(cpu_forward(oracle, op, case), OPS[op].dense(case), np.float64, op)


def test_sap_unsorted_output_index(oracle):
    case = support.sap_case(12, np.float64, I=33, nA=4, nB=3, K=50, nO=6, sort_output=False)
    assert_close(cpu_forward(oracle, "sap", case), OPS["sap"].dense(case), np.float64, "sap")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("op", ["hpe", "sap"])
def test_batch_remainder_rows(oracle, op, dtype):
    """Batch sizes that are not a multiple of the SIMD block (and smaller than one)."""
    for rows in (1, 3, 8, 13):
        case = SMALL[op](rows, dtype)
        for key in ("A", "B", "grad_output"):
            if key in case:
                case[key] = np.ascontiguousarray(case[key][:rows])
        assert_close(cpu_forward(oracle, op, case), OPS[op].dense(case), dtype, f"{op} rows={rows}")


@pytest.mark.parametrize("op", list(OPS))
def test_skipped_gradients(oracle, op):
    case = SMALL[op](14, np.float64)
    full = cpu_vjp(oracle, op, case)
    for name in OPS[op].differentiable:
        only = cpu_vjp(oracle, op, case, wanted=[name])
        np.testing.assert_array_equal(only[name], full[name])
        assert all(v is None for k, v in only.items() if k != name)
    # nothing requested: a no-op, not an error
    cpu_vjp(oracle, op, case, wanted=[])


def test_first_occurrences_definition(oracle):
    index = np.array([0, 0, 0, 1, 1, 1, 2, 2], dtype=np.int32)
    out = np.empty(2 * 3, dtype=np.int32)
    oracle.cdll.mops_oracle_first_occurrences(index.ctypes.data, len(index), 3, out.ctypes.data)
    assert out[:3].tolist() == [0, 3, 6]  # the documented example of the reference
    assert out[3:].tolist() == [3, 6, 8]
    index = np.array([1, 1, 4], dtype=np.int32)
    out = np.empty(2 * 6, dtype=np.int32)
    oracle.cdll.mops_oracle_first_occurrences(index.ctypes.data, len(index), 6, out.ctypes.data)
    assert out[:6].tolist() == [-1, 0, -1, -1, 2, -1]
    assert out[6:].tolist() == [-1, 2, -1, -1, 3, -1]


# --------------------------------------------------------------------------
# second order: the vjp of the vjp
# --------------------------------------------------------------------------
def _contracted_vjp(oracle, op, case):
    """s(grad_output, A, B) = sum over inputs of <grad_grad_x, vjp_x>, in float64."""
    gradients = cpu_vjp(oracle, op, case)
    return sum(np.sum(case["grad_grad_" + name] * gradients[name]) for name in OPS[op].differentiable)


@pytest.mark.parametrize("op", support.SECOND_ORDER)
def test_vjp_vjp_matches_finite_differences_of_the_vjp(oracle, op):
    """grad_grad_output, grad_A_2, grad_B_2 are the derivatives of
    s = <grad_grad_A, grad_A> + <grad_grad_B, grad_B> with respect to
    grad_output, A and B; s is evaluated with the (pinned) vjp."""
    case = support.add_cotangents(SMALL[op](5, np.float64), op)
    second = support.cpu_vjp_vjp(oracle, op, case)
    h = 1e-6
    rng = np.random.default_rng(13)
    for name in ["grad_output"] + OPS[op].differentiable:
        x = case[name]
        assert second[name].shape == x.shape
        for _ in range(12):
            position = tuple(rng.integers(0, s) for s in x.shape)
            saved = x[position]
            x[position] = saved + h
            plus = _contracted_vjp(oracle, op, case)
            x[position] = saved - h
            minus = _contracted_vjp(oracle, op, case)
            x[position] = saved
            numeric = (plus - minus) / (2 * h)
            analytic = second[name][position]
            assert abs(numeric - analytic) <= 2e-6 * max(1.0, abs(numeric)), (op, name, position)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("op", ["sap", "opsa"])
def test_grad_grad_output_is_two_forward_passes(oracle, op, dtype):
    """Bilinear operations: grad_grad_output = f(grad_grad_A, B) + f(A, grad_grad_B)."""
    case = support.add_cotangents(SMALL[op](6, dtype), op)
    second = support.cpu_vjp_vjp(oracle, op, case)
    first = dict(case, A=case["grad_grad_A"])
    other = dict(case, B=case["grad_grad_B"])
    expected = cpu_forward(oracle, op, first).astype(np.float64) + cpu_forward(oracle, op, other)
    assert_close(second["grad_output"], expected, dtype, op)


@pytest.mark.parametrize("op", support.SECOND_ORDER)
def test_vjp_vjp_absent_cotangents_and_skipped_outputs(oracle, op):
    case = support.add_cotangents(SMALL[op](7, np.float64), op)
    everything = support.cpu_vjp_vjp(oracle, op, case)
    names = OPS[op].differentiable
    # an absent cotangent counts as zero
    for absent in names:
        have = [n for n in names if n != absent]
        zeroed = dict(case)
        zeroed["grad_grad_" + absent] = np.zeros_like(case["grad_grad_" + absent])
        expected = support.cpu_vjp_vjp(oracle, op, zeroed)
        actual = support.cpu_vjp_vjp(oracle, op, case, have=have)
        for key in expected:
            assert np.array_equal(actual[key], expected[key]), (op, absent, key)
    # every output can be computed alone and gives the same values
    for alone in ["grad_output"] + names:
        actual = support.cpu_vjp_vjp(oracle, op, case, wanted=[alone])
        assert np.array_equal(actual[alone], everything[alone]), (op, alone)
        assert all(value is None for key, value in actual.items() if key != alone)
