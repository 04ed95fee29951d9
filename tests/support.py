"""Shared helpers of the test-suite.

* loading the CPU oracle (``oracle/liboracle.so``, test infrastructure);
* seeded input generators, including the BASELINE configurations;
* closed-form numpy formulations of the five operations that share no code
  with either the oracle or the HIP kernels (dense einsum / ``np.add.at``),
  used to pin the oracle;
* the error norm the parity bar is written in.
"""
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_PATH = os.path.join(ROOT, "oracle", "liboracle.so")

#: parity bar of the north star: max|x - ref| / max|ref|
TOLERANCE = {np.dtype("float32"): 1e-5, np.dtype("float64"): 1e-12}

_oracle = None


def oracle_library():
    """The CPU oracle as a :py:class:`mops_amd._c_api.Library`."""
    global _oracle
    if _oracle is None:
        import ctypes

        from mops_amd._c_api import Library

        if not os.path.exists(ORACLE_PATH):
            raise RuntimeError(f"{ORACLE_PATH} is missing: run `make -C oracle`")
        _oracle = Library(ORACLE_PATH, "mops_oracle_", "mops_oracle_get_last_error_message")
        _oracle.cdll.mops_oracle_first_occurrences.argtypes = [
            ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
        ]  # fmt: skip
        _oracle.cdll.mops_oracle_first_occurrences.restype = ctypes.c_int
        _oracle.cdll.mops_oracle_num_threads.restype = ctypes.c_int
    return _oracle


def relative_error(actual, expected):
    """Norm-wise error max|a - e| / max|e| (signed sums cancel element-wise)."""
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    assert actual.shape == expected.shape, (actual.shape, expected.shape)
    if expected.size == 0:
        return 0.0
    scale = np.max(np.abs(expected))
    difference = np.max(np.abs(actual - expected))
    if scale == 0.0:
        return difference
    return difference / scale


def assert_close(actual, expected, dtype, what="", factor=1.0):
    error = relative_error(actual, expected)
    bound = TOLERANCE[np.dtype(dtype)] * factor
    assert error <= bound, f"{what}: relative error {error:.3e} above {bound:.1e}"


def in_float64(case):
    """The same (already rounded) inputs as float64 arrays."""
    return {
        key: value.astype(np.float64) if isinstance(value, np.ndarray) and value.dtype == np.float32 else value
        for key, value in case.items()
    }


def magnitudes(case):
    """``case`` in float64 with every floating-point value replaced by its absolute value: an
    operation applied to it gives, element by element, the sum of the absolute values of the terms
    whose signed sum the operation gives on ``case`` (every operation here is a sum of products)."""
    return {
        key: np.abs(value.astype(np.float64)) if isinstance(value, np.ndarray) and value.dtype.kind == "f" else value
        for key, value in case.items()
    }


def calibrated_bar(dtype, exact, same_dtype=None, term_magnitudes=None):
    """The bar a kernel's result is held to, and the reason as text.

    The north star's bar (1e-5 / 1e-12, norm-wise) unless the sum itself is ill-conditioned, which
    is MEASURED, never assumed:

    * float32: ``same_dtype`` is the oracle run in float32 on the same inputs and ``exact`` the
      oracle in float64. Where the oracle's own float32 error exceeds a quarter of 1e-5, no order
      of summation does better than that error's scale, and the bar is four times it.
    * float64: nothing more exact is at hand, so the conditioning is measured instead:
      ``term_magnitudes`` is the operation applied to the absolute values (``magnitudes``), and
      kappa = max(sum |terms|) / max|sum terms|. Rounding moves a sum by at least eps * sum|terms|
      whatever the order, so the bar is max(1e-12, 8 eps kappa): 1e-12 up to kappa = 1100.
    """
    dtype = np.dtype(dtype)
    base = TOLERANCE[dtype]
    if dtype == np.float32 and same_dtype is not None:
        own = relative_error(same_dtype, exact)
        if 4.0 * own > base:
            return 4.0 * own, f"4 x the float32 oracle's own error {own:.2e}"
        return base, f"north star (float32 oracle's own error {own:.2e})"
    if dtype == np.float64 and term_magnitudes is not None and np.size(exact):
        scale = float(np.max(np.abs(exact)))
        kappa = float(np.max(term_magnitudes)) / scale if scale > 0 else np.inf
        widened = 8.0 * np.finfo(np.float64).eps * kappa
        if widened > base:
            return widened, f"8 eps kappa, kappa = {kappa:.3g}"
        return base, f"north star (kappa = {kappa:.3g})"
    return base, "north star"


def assert_calibrated(actual, exact, dtype, what, same_dtype=None, term_magnitudes=None):
    bar, reason = calibrated_bar(dtype, exact, same_dtype, term_magnitudes)
    error = relative_error(actual, exact)
    assert error <= bar, f"{what}: relative error {error:.3e} above {bar:.3e} ({reason})"
    return error, bar, reason


# --------------------------------------------------------------------------
# input generators
# --------------------------------------------------------------------------
def segments(rng, n_out, n_in, allow_empty=False):
    """Sorted scatter index: segment lengths ~ Poisson(n_in / n_out), adjusted to sum to n_in."""
    mean = max(n_in / max(n_out, 1), 1.0)
    lengths = rng.poisson(mean, size=n_out)
    floor = 0 if allow_empty else 1
    lengths = np.maximum(lengths, floor)
    while lengths.sum() != n_in:
        row = rng.integers(n_out)
        if lengths.sum() < n_in:
            lengths[row] += 1
        elif lengths[row] > floor:
            lengths[row] -= 1
    return np.repeat(np.arange(n_out), lengths).astype(np.int32)


def hpe_case(seed, dtype, I=1000, nA=100, J=2000, K=4):
    rng = np.random.default_rng(seed)
    return {
        "A": rng.uniform(-1, 1, size=(I, nA)).astype(dtype),
        "C": rng.normal(size=J).astype(dtype),
        "indices_A": rng.integers(0, max(nA, 1), size=(J, K)).astype(np.int32),
        "grad_output": rng.normal(size=I).astype(dtype),
    }


def sap_case(seed, dtype, I=32000, nA=13, nB=7, K=900, nO=20, sort_output=True):
    rng = np.random.default_rng(seed)
    PO = rng.integers(0, nO, size=K)
    if sort_output:
        PO = np.sort(PO)
    return {
        "A": rng.normal(size=(I, nA)).astype(dtype),
        "B": rng.normal(size=(I, nB)).astype(dtype),
        "C": rng.normal(size=K).astype(dtype),
        "indices_A": rng.integers(0, nA, size=K).astype(np.int32),
        "indices_B": rng.integers(0, nB, size=K).astype(np.int32),
        "indices_output": PO.astype(np.int32),
        "output_size": nO,
        "grad_output": rng.normal(size=(I, nO)).astype(dtype),
    }


def opsa_case(seed, dtype, J=60000, K=13, L=20, n_out=2000, allow_empty=False):
    rng = np.random.default_rng(seed)
    return {
        "A": rng.normal(size=(J, K)).astype(dtype),
        "B": rng.normal(size=(J, L)).astype(dtype),
        "indices_output": segments(rng, n_out, J, allow_empty),
        "output_size": n_out,
        "grad_output": rng.normal(size=(n_out, K, L)).astype(dtype),
    }


def opsaw_case(seed, dtype, E=60000, K=13, L=32, n_nodes=2000, allow_empty=False):
    rng = np.random.default_rng(seed)
    return {
        "A": rng.normal(size=(E, K)).astype(dtype),
        "B": rng.normal(size=(E, L)).astype(dtype),
        "W": rng.normal(size=(n_nodes, L)).astype(dtype),
        "indices_W": rng.integers(0, n_nodes, size=E).astype(np.int32),
        "indices_output": segments(rng, n_nodes, E, allow_empty),
        "grad_output": rng.normal(size=(n_nodes, K, L)).astype(dtype),
    }


def sasaw_case(seed, dtype, E=60000, nA=9, L=32, n_nodes=2000, n2=9, n3=9, N=250, allow_empty=False):
    rng = np.random.default_rng(seed)
    return {
        "A": rng.normal(size=(E, nA)).astype(dtype),
        "B": rng.normal(size=(E, L)).astype(dtype),
        "C": rng.normal(size=N).astype(dtype),
        "W": rng.normal(size=(n_nodes, n2, L)).astype(dtype),
        "indices_A": rng.integers(0, nA, size=N).astype(np.int32),
        "indices_W_1": rng.integers(0, n_nodes, size=E).astype(np.int32),
        "indices_W_2": rng.integers(0, n2, size=N).astype(np.int32),
        "indices_output_1": segments(rng, n_nodes, E, allow_empty),
        "indices_output_2": rng.integers(0, n3, size=N).astype(np.int32),
        "output_size": n3,
        "grad_output": rng.normal(size=(n_nodes, n3, L)).astype(dtype),
    }


# --------------------------------------------------------------------------
# closed forms in float64 numpy (independent of oracle and kernels)
# --------------------------------------------------------------------------
def dense_hpe(A, C, indices_A):
    A = A.astype(np.float64)
    monomials = np.prod(A[:, indices_A], axis=2) if indices_A.shape[1] > 0 else np.ones(
        (A.shape[0], indices_A.shape[0])
    )
    return monomials @ C.astype(np.float64)


def dense_sap(A, B, C, indices_A, indices_B, indices_output, output_size):
    A, B, C = (x.astype(np.float64) for x in (A, B, C))
    terms = C[None, :] * A[:, indices_A] * B[:, indices_B]
    selector = np.zeros((len(C), output_size))
    selector[np.arange(len(C)), indices_output] = 1.0
    return terms @ selector


def dense_opsa(A, B, indices_output, output_size):
    A, B = A.astype(np.float64), B.astype(np.float64)
    out = np.zeros((output_size, A.shape[1], B.shape[1]))
    np.add.at(out, indices_output, np.einsum("jk,jl->jkl", A, B))
    return out


def dense_opsaw(A, B, W, indices_W, indices_output):
    return dense_opsa(A, B.astype(np.float64) * W.astype(np.float64)[indices_W], indices_output, W.shape[0])


def dense_sasaw(
    A, B, C, W, indices_A, indices_W_1, indices_W_2, indices_output_1, indices_output_2, output_size
):
    A, B, C, W = (x.astype(np.float64) for x in (A, B, C, W))
    # per edge and table entry: [E, N, L]
    terms = (C[None, :] * A[:, indices_A])[:, :, None] * B[:, None, :] * W[indices_W_1][:, indices_W_2, :]
    per_edge = np.zeros((A.shape[0], output_size, B.shape[1]))
    np.add.at(per_edge, (slice(None), indices_output_2), terms)
    out = np.zeros((W.shape[0], output_size, B.shape[1]))
    np.add.at(out, indices_output_1, per_edge)
    return out


# --------------------------------------------------------------------------
# one table that knows how to call every operation through the C ABI
# --------------------------------------------------------------------------
class Op:
    def __init__(self, name, function, inputs, differentiable, output_shape, dense):
        self.name = name
        self.function = function
        self.inputs = inputs  # ABI order of the forward inputs
        self.differentiable = differentiable  # inputs that have a gradient, ABI order
        self.output_shape = output_shape
        self.dense = dense


OPS = {
    "hpe": Op(
        "hpe",
        "homogeneous_polynomial_evaluation",
        ["A", "C", "indices_A"],
        ["A"],
        lambda c: (c["A"].shape[0],),
        lambda c: dense_hpe(c["A"], c["C"], c["indices_A"]),
    ),
    "sap": Op(
        "sap",
        "sparse_accumulation_of_products",
        ["A", "B", "C", "indices_A", "indices_B", "indices_output"],
        ["A", "B"],
        lambda c: (c["A"].shape[0], c["output_size"]),
        lambda c: dense_sap(
            c["A"], c["B"], c["C"], c["indices_A"], c["indices_B"], c["indices_output"], c["output_size"]
        ),
    ),
    "opsa": Op(
        "opsa",
        "outer_product_scatter_add",
        ["A", "B", "indices_output"],
        ["A", "B"],
        lambda c: (c["output_size"], c["A"].shape[1], c["B"].shape[1]),
        lambda c: dense_opsa(c["A"], c["B"], c["indices_output"], c["output_size"]),
    ),
    "opsaw": Op(
        "opsaw",
        "outer_product_scatter_add_with_weights",
        ["A", "B", "W", "indices_W", "indices_output"],
        ["A", "B", "W"],
        lambda c: (c["W"].shape[0], c["A"].shape[1], c["B"].shape[1]),
        lambda c: dense_opsaw(c["A"], c["B"], c["W"], c["indices_W"], c["indices_output"]),
    ),
    "sasaw": Op(
        "sasaw",
        "sparse_accumulation_scatter_add_with_weights",
        ["A", "B", "C", "W", "indices_A", "indices_W_1", "indices_W_2", "indices_output_1",
         "indices_output_2"],
        ["A", "B", "W"],
        lambda c: (c["W"].shape[0], c["output_size"], c["B"].shape[1]),
        lambda c: dense_sasaw(
            c["A"], c["B"], c["C"], c["W"], c["indices_A"], c["indices_W_1"], c["indices_W_2"],
            c["indices_output_1"], c["indices_output_2"], c["output_size"],
        ),
    ),
}  # fmt: skip


def cpu_forward(library, op, case):
    """Run the forward of ``op`` on numpy arrays through ``library``."""
    op = OPS[op]
    output = np.full(op.output_shape(case), np.nan, dtype=case["A"].dtype)
    library.call(op.function, output, *[case[name] for name in op.inputs])
    return output


def cpu_vjp(library, op, case, wanted=None):
    """Run the vjp of ``op``; returns {input name: gradient or None}."""
    op = OPS[op]
    wanted = op.differentiable if wanted is None else wanted
    gradients = [
        np.full(case[name].shape, np.nan, dtype=case[name].dtype) if name in wanted else None
        for name in op.differentiable
    ]
    library.call(
        op.function + "_vjp", *gradients, case["grad_output"], *[case[name] for name in op.inputs]
    )
    return dict(zip(op.differentiable, gradients))


SECOND_ORDER = ["hpe", "sap", "opsa"]  # operations that have a vjp_vjp


def add_cotangents(case, op, seed=99):
    """Adds grad_grad_<input> (cotangents of the vjp's outputs) to ``case``."""
    rng = np.random.default_rng(seed)
    for name in OPS[op].differentiable:
        case["grad_grad_" + name] = rng.normal(size=case[name].shape).astype(case[name].dtype)
    return case


def _vjp_vjp_arguments(op, case, have, wanted, empty_like):
    """ABI order: grad_grad_output, grad_<x>_2 ..., grad_grad_<x> ..., grad_output, inputs."""
    have = op.differentiable if have is None else have
    wanted = ["grad_output"] + op.differentiable if wanted is None else wanted
    outputs = {"grad_output": empty_like(case["grad_output"]) if "grad_output" in wanted else None}
    for name in op.differentiable:
        outputs[name] = empty_like(case[name]) if name in wanted else None
    cotangents = [case["grad_grad_" + name] if name in have else None for name in op.differentiable]
    arguments = (
        [outputs["grad_output"]]
        + [outputs[name] for name in op.differentiable]
        + cotangents
        + [case["grad_output"]]
        + [case[name] for name in op.inputs]
    )
    return outputs, arguments


def cpu_vjp_vjp(library, op, case, have=None, wanted=None):
    """Second-order function; returns {"grad_output": grad_grad_output, input name: grad_<name>_2}.

    ``have``: the inputs whose cotangent grad_grad_<name> is passed (others null);
    ``wanted``: which of "grad_output" and the input names are computed.
    """
    op = OPS[op]
    outputs, arguments = _vjp_vjp_arguments(
        op, case, have, wanted, lambda x: np.full(x.shape, np.nan, dtype=x.dtype)
    )
    library.call(op.function + "_vjp_vjp", *arguments)
    return outputs


def hip_vjp_vjp(op, case_on_device, have=None, wanted=None):
    import torch

    from mops_amd._c_lib import device_library

    op = OPS[op]
    outputs, arguments = _vjp_vjp_arguments(
        op, case_on_device, have, wanted, lambda x: torch.full_like(x, float("nan"))
    )
    library = device_library()
    _bind_stream(library, case_on_device["A"].device)
    library.call(op.function + "_vjp_vjp", *arguments)
    return outputs


def to_device(case, device):
    import torch

    return {
        key: torch.from_numpy(value).to(device) if isinstance(value, np.ndarray) else value
        for key, value in case.items()
    }


def hip_forward(op, case_on_device, poison=True):
    """Forward of ``op`` through the device C ABI on torch tensors."""
    import torch

    from mops_amd._c_lib import device_library

    op = OPS[op]
    A = case_on_device["A"]
    output = torch.empty(op.output_shape(case_on_device), dtype=A.dtype, device=A.device)
    if poison:
        output.fill_(float("nan"))  # the library must overwrite every element
    library = device_library()
    _bind_stream(library, A.device)
    library.call(op.function, output, *[case_on_device[name] for name in op.inputs])
    return output


def hip_vjp(op, case_on_device, wanted=None, poison=True):
    import torch

    from mops_amd._c_lib import device_library

    op = OPS[op]
    wanted = op.differentiable if wanted is None else wanted
    gradients = []
    for name in op.differentiable:
        if name in wanted:
            g = torch.empty_like(case_on_device[name])
            if poison:
                g.fill_(float("nan"))
            gradients.append(g)
        else:
            gradients.append(None)
    library = device_library()
    _bind_stream(library, case_on_device["A"].device)
    library.call(
        op.function + "_vjp",
        *gradients,
        case_on_device["grad_output"],
        *[case_on_device[name] for name in op.inputs],
    )
    return dict(zip(op.differentiable, gradients))


def _bind_stream(library, device):
    import torch

    torch.cuda.set_device(device)
    library.cdll.mops_amd_set_stream(torch.cuda.current_stream(device).cuda_stream)
    library.cdll.mops_amd_set_synchronous(1)
