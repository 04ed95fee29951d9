"""Random shapes and sizes, HIP kernels against the oracle.

Shapes are drawn (fixed seed) from lists that straddle the limits at which the library changes
kernels: 16 / 17 and 32 / 33 values of a component or feature index, 64 / 65 columns, one row or
edge, 47 / 49 edges per node, 4000 nodes, tables of 2047 / 2049 entries, the row counts at which
SAP's wavefronts start to walk. Every output and gradient is compared with the oracle run in
float64 on the same (already rounded) inputs.

Bar: max|x - exact| / max|exact| <= 1e-5 in float32 and <= 1e-12 in float64 (the north star's),
except where the sum itself is measured to be ill-conditioned (support.calibrated_bar): in float32
where the oracle run in float32 is itself further than a quarter of 1e-5 from the float64 result
(a sum that cancels, one edge and forty terms of either sign, is as far off in any order of
summation; the kernel then has to be within four times the oracle's own error); in float64 where
the sum of the absolute values of the terms is more than 1100 times the largest result. The bar
applied to every comparison is printed with its reason.
"""
import numpy as np
import pytest

from tests import support
from tests.support import OPS, cpu_forward, cpu_vjp, hip_forward, hip_vjp, to_device

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
        return dict(I=pick(1, 63, 65, 1000, 4097), nA=pick(1, 3, 17, 100, 257), J=pick(1, 7, 300, 2000), K=pick(0, 1, 2, 3, 4, 5, 6, 7, 10))
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
        exact_case = support.in_float64(case)
        absolute = support.magnitudes(case)
        on_device = to_device(case, device)

        def check(actual, exact, same_dtype, term_magnitudes, name):
            error, bar, reason = support.assert_calibrated(
                actual, exact, dtype, f"{what} {name}", same_dtype=same_dtype, term_magnitudes=term_magnitudes
            )
            if bar != support.TOLERANCE[np.dtype(dtype)]:
                print(f"    {name}: error {error:.2e}, bar {bar:.2e}: {reason}", flush=True)

        exact = cpu_forward(oracle, op, exact_case)
        same = cpu_forward(oracle, op, case) if dtype == np.float32 else None
        sums = cpu_forward(oracle, op, absolute) if dtype == np.float64 else None
        check(hip_forward(op, on_device).cpu().numpy(), exact, same, sums, "output")
        gradients = hip_vjp(op, on_device)
        exact = cpu_vjp(oracle, op, exact_case)
        same = cpu_vjp(oracle, op, case) if dtype == np.float32 else {}
        sums = cpu_vjp(oracle, op, absolute) if dtype == np.float64 else {}
        for key in OPS[op].differentiable:
            check(gradients[key].cpu().numpy(), exact[key], same.get(key), sums.get(key), f"grad_{key}")
