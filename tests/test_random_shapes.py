"""Random shapes and sizes, HIP kernels against the oracle.

Shapes are drawn (fixed seed) from lists that straddle the limits at which the library changes
kernels: 16 / 17 and 32 / 33 values of a component or feature index, 64 / 65 columns, one row or
edge, 47 / 49 edges per node, 4000 nodes, tables of 2047 / 2049 entries, the row counts at which
SAP's wavefronts start to walk. Every output and gradient is compared with the oracle run in
float64 on the same (already rounded) inputs.

Bar: max|x - exact| / max|exact| <= 1e-5 in float32 and <= 1e-12 in float64 (the north star's),
except where the oracle itself, run in the dtype of the kernels, is further than a quarter of
that from the float64 result: a sum that cancels (one edge, forty terms of either sign) is as far
off in any order of summation, and the kernel then has to be within four times the oracle's own
error. In float64 there is nothing more exact to calibrate against, so sums of thousands of terms
that cancel get 1e-11.
"""
import numpy as np
import pytest

from tests import support
from tests.support import OPS, cpu_forward, cpu_vjp, hip_forward, hip_vjp, relative_error, to_device

pytestmark = pytest.mark.gpu

BUILDERS = {
    "hpe": support.hpe_case,
    "sap": support.sap_case,
    "opsa": support.opsa_case,
    "opsaw": support.opsaw_case,
    "sasaw": support.sasaw_case,
}
CASES_PER_OPERATION = 30


def _draw(op, rng):
    def pick(*choices):
        return int(choices[rng.integers(0, len(choices))])

    if op == "hpe":
        return dict(I=pick(1, 63, 65, 1000, 4097), nA=pick(1, 3, 17, 100, 257), J=pick(1, 7, 300, 2000), K=pick(0, 1, 2, 3, 4, 5, 6))
    if op == "sap":
        return dict(
            I=pick(1, 17, 129, 5000, 66000, 140001, 270000), nA=pick(1, 4, 13, 16, 17, 25), nB=pick(1, 3, 7, 16, 17),
            K=pick(1, 30, 900, 2047, 2049), nO=pick(1, 4, 16, 20, 33, 64, 65), sort_output=bool(rng.integers(0, 2)),
        )
    if op == "opsa":
        J = pick(1, 100, 5000, 60000)
        return dict(J=J, K=pick(1, 4, 13, 16, 17, 32, 33), L=pick(1, 4, 20, 32, 33, 64, 65, 130), n_out=max(1, J // pick(1, 3, 30, 700)), allow_empty=True)
    if op == "opsaw":
        E = pick(1, 100, 5000, 60000)
        return dict(E=E, K=pick(1, 4, 13, 16, 17, 32, 33), L=pick(1, 4, 32, 33, 64, 65, 130), n_nodes=max(1, E // pick(1, 3, 30, 47, 49, 700)), allow_empty=True)
    E = pick(1, 100, 5000, 60000, 200000)
    return dict(
        E=E, nA=pick(1, 4, 9, 16, 17), L=pick(1, 4, 16, 32, 33, 64, 65, 100), n_nodes=max(1, E // pick(1, 3, 20, 30, 47, 49, 700)),
        n2=pick(1, 3, 4, 9, 16, 17), n3=pick(1, 4, 5, 9, 16, 17), N=pick(1, 40, 250, 900), allow_empty=True,
    )


@pytest.mark.parametrize("op", list(BUILDERS))
def test_random_shapes(oracle, device, op):
    rng = np.random.default_rng({"hpe": 11, "sap": 12, "opsa": 13, "opsaw": 14, "sasaw": 15}[op])
    for number in range(CASES_PER_OPERATION):
        shape = _draw(op, rng)
        seed = int(rng.integers(0, 1 << 30))
        dtype = np.float64 if op == "hpe" or rng.integers(0, 2) else np.float32
        what = f"{op} {np.dtype(dtype).name} seed={seed} {shape}"
        print(f"case {number}: {what}", flush=True)
        case = BUILDERS[op](seed, dtype, **shape)
        exact_case = {
            key: value.astype(np.float64) if isinstance(value, np.ndarray) and value.dtype == np.float32 else value
            for key, value in case.items()
        }
        on_device = to_device(case, device)

        def check(actual, exact, same_dtype, name):
            if dtype == np.float32:
                bar = max(1e-5, 4.0 * relative_error(same_dtype, exact))
            else:
                bar = 1e-11
            error = relative_error(actual, exact)
            assert error <= bar, f"{what} {name}: {error:.3e} > {bar:.3e}"

        exact = cpu_forward(oracle, op, exact_case)
        same = cpu_forward(oracle, op, case) if dtype == np.float32 else exact
        check(hip_forward(op, on_device).cpu().numpy(), exact, same, "output")
        gradients = hip_vjp(op, on_device)
        exact = cpu_vjp(oracle, op, exact_case)
        same = cpu_vjp(oracle, op, case) if dtype == np.float32 else exact
        for key in OPS[op].differentiable:
            check(gradients[key].cpu().numpy(), exact[key], same[key], f"grad_{key}")
