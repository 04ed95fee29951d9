"""The error contract of all fifteen functions, table-driven.

The tables below restate, by hand and per operation, the ORDER and the tensor
names of the reference's checks
(``mops/src/internal/checks/{hpe,sap,opsa,opsaw,sasaw}.hpp`` of lab-cosmo/mops)
and the message formats of ``mops/src/internal/checks/utils.hpp:32-36,64-75``.
They share nothing with ``mops_amd/csrc/checks.hpp``. Every extent of every
argument is then perturbed in turn; a small evaluator walks the table and says
which check fails first, and the library must fail with exactly that text.
The same walk runs on the ``mops_cuda_*`` entry points (GPU, size checks only:
as in the reference the values of device index tensors are not inspected), and
the Python front-end's ``TypeError`` / ``ValueError`` texts
(``python/mops/src/mops/checks.py:9-34``, asserted per operation by
``python/mops/tests/{hpe,sap,opsa,opsaw,sasaw}.py``) are checked at the end.

Oddities of the reference that are part of the observable text and must stay:
HPE's first check names the output ``grad_output`` (``checks/hpe.hpp:16``);
SASAW bounds ``indices_W_2`` by ``B.shape[1]`` (``checks/sasaw.hpp:33``);
OPSAW and SASAW require ``W.shape[0] == output.shape[0]``; the negative-index
message reads "negative-valuedindices".
"""
import numpy as np
import pytest

from mops_amd._c_api import _KINDS, SIGNATURES
from mops_amd.status import MopsError

# (tensor, axis, tensor, axis) in the order the reference compares them; the
# forward output appears under the name the reference prints for it.
FORWARD_SIZE_CHECKS = {
    # checks/hpe.hpp:16-17
    "homogeneous_polynomial_evaluation": [("A", 0, "grad_output", 0), ("C", 0, "indices_A", 0)],
    # checks/sap.hpp:19-23
    "sparse_accumulation_of_products": [
        ("A", 0, "B", 0), ("A", 0, "output", 0), ("C", 0, "indices_A", 0), ("C", 0, "indices_B", 0),
        ("C", 0, "indices_output", 0),
    ],
    # checks/opsa.hpp:16-19
    "outer_product_scatter_add": [
        ("A", 0, "B", 0), ("A", 1, "output", 1), ("B", 1, "output", 2), ("A", 0, "indices_output", 0),
    ],
    # checks/opsaw.hpp:18-24
    "outer_product_scatter_add_with_weights": [
        ("A", 0, "B", 0), ("A", 1, "output", 1), ("B", 1, "output", 2), ("A", 0, "indices_output", 0),
        ("A", 0, "indices_W", 0), ("W", 0, "output", 0), ("B", 1, "W", 1),
    ],
    # checks/sasaw.hpp:22-29
    "sparse_accumulation_scatter_add_with_weights": [
        ("A", 0, "B", 0), ("W", 0, "output", 0), ("B", 1, "W", 2), ("C", 0, "indices_A", 0),
        ("C", 0, "indices_W_2", 0), ("C", 0, "indices_output_2", 0), ("A", 0, "indices_output_1", 0),
        ("A", 0, "indices_W_1", 0),
    ],
}  # fmt: skip

# (index tensor, (tensor, axis) whose extent bounds it), in the reference's order
INDEX_CHECKS = {
    "homogeneous_polynomial_evaluation": [("indices_A", ("A", 1))],
    "sparse_accumulation_of_products": [
        ("indices_A", ("A", 1)), ("indices_B", ("B", 1)), ("indices_output", ("output", 1)),
    ],
    "outer_product_scatter_add": [("indices_output", ("output", 0))],
    "outer_product_scatter_add_with_weights": [
        ("indices_output", ("output", 0)), ("indices_W", ("output", 0)),
    ],
    "sparse_accumulation_scatter_add_with_weights": [
        ("indices_A", ("A", 1)), ("indices_W_1", ("output", 0)), ("indices_W_2", ("B", 1)),
        ("indices_output_1", ("output", 0)), ("indices_output_2", ("output", 1)),
    ],
}  # fmt: skip

# optional outputs of the derivative levels and the tensor each must have the shape of,
# in the reference's order
GRADIENT_CHECKS = {
    "_vjp": lambda wrt: [("grad_" + name, name) for name in wrt],
    "_vjp_vjp": lambda wrt: (
        [("grad_grad_output", "grad_output")]
        + [("grad_" + name + "_2", name) for name in wrt]
        + [("grad_grad_" + name, name) for name in wrt]
    ),
}
DIFFERENTIABLE = {
    "homogeneous_polynomial_evaluation": ["A"],
    "sparse_accumulation_of_products": ["A", "B"],
    "outer_product_scatter_add": ["A", "B"],
    "outer_product_scatter_add_with_weights": ["A", "B", "W"],
    "sparse_accumulation_scatter_add_with_weights": ["A", "B", "W"],
}

# consistent small shapes (every extent distinct where the checks allow it, so
# that a check on the wrong axis cannot pass by accident)
BASE_SHAPES = {
    "homogeneous_polynomial_evaluation": {
        "output": (6,), "A": (6, 5), "C": (7,), "indices_A": (7, 3),
    },
    "sparse_accumulation_of_products": {
        "output": (6, 4), "A": (6, 5), "B": (6, 3), "C": (7,), "indices_A": (7,), "indices_B": (7,),
        "indices_output": (7,),
    },
    "outer_product_scatter_add": {"output": (4, 5, 3), "A": (6, 5), "B": (6, 3), "indices_output": (6,)},
    "outer_product_scatter_add_with_weights": {
        "output": (4, 5, 3), "A": (6, 5), "B": (6, 3), "W": (4, 3), "indices_W": (6,), "indices_output": (6,),
    },
    "sparse_accumulation_scatter_add_with_weights": {
        "output": (4, 2, 3), "A": (6, 5), "B": (6, 3), "C": (7,), "W": (4, 8, 3), "indices_A": (7,),
        "indices_W_1": (6,), "indices_W_2": (7,), "indices_output_1": (6,), "indices_output_2": (7,),
    },
}  # fmt: skip

LEVELS = ["", "_vjp", "_vjp_vjp"]


def shapes_of(operation, level):
    """Shapes by C parameter name of ``operation + level``, all consistent."""
    base = dict(BASE_SHAPES[operation])
    if level == "":
        return base
    shapes = {name: shape for name, shape in base.items() if name != "output"}
    shapes["grad_output"] = base["output"]
    for gradient, like in GRADIENT_CHECKS[level](DIFFERENTIABLE[operation]):
        shapes[gradient] = shapes[like]
    return shapes


def size_checks(operation, level):
    """All extent comparisons of ``operation + level`` in the reference's order."""
    shapes = shapes_of(operation, level)
    checks = []
    if level != "":
        for gradient, like in GRADIENT_CHECKS[level](DIFFERENTIABLE[operation]):
            for axis in range(len(shapes[like])):
                checks.append((gradient, axis, like, axis))
    # the forward checks print their fixed names at every level (the vjp levels pass
    # grad_output where the forward pass has its output: checks/sap.hpp:57 and siblings)
    output_names = ("output", "grad_output") if operation.startswith("homog") else ("output",)
    for first, axis_1, second, axis_2 in FORWARD_SIZE_CHECKS[operation]:
        actual = second
        if second in output_names:
            actual = "output" if level == "" else "grad_output"
        checks.append((first, axis_1, second, axis_2, actual))
    return [check if len(check) == 5 else check + (check[2],) for check in checks]


def first_failure(operation, level, shapes, prefix, absent=()):
    """Message of the first failing extent comparison, or None."""
    for first, axis_1, printed, axis_2, second in size_checks(operation, level):
        if first in absent:
            continue  # a gradient that is not requested is not compared
        if shapes[first][axis_1] != shapes[second][axis_2]:
            return (
                f"Dimension mismatch: the sizes of {first} along dimension {axis_1} and {printed} along "
                f"dimension {axis_2} must match in {prefix}{operation}{level}"
            )
    return None


def make_arguments(function, shapes, make_float, make_index, absent=()):
    arguments = []
    for kind, name in SIGNATURES[function]:
        if name in absent:
            arguments.append(None)
        elif _KINDS[kind][1]:
            arguments.append(make_index(shapes[name]))
        else:
            arguments.append(make_float(shapes[name]))
    return arguments


def perturbations(operation, level):
    shapes = shapes_of(operation, level)
    for name, shape in shapes.items():
        for axis in range(len(shape)):
            changed = dict(shapes)
            changed[name] = shape[:axis] + (shape[axis] + 1,) + shape[axis + 1 :]
            yield f"{name}[{axis}]+1", changed


ALL_FUNCTIONS = [(operation, level) for operation in FORWARD_SIZE_CHECKS for level in LEVELS]


@pytest.fixture(scope="module")
def host():
    from mops_amd._c_lib import host_library

    return host_library()


def optional_arguments(operation, level):
    """Tensors that may be absent (null data): they are compared only when given."""
    if level == "":
        return ()
    return tuple(g for g, _ in GRADIENT_CHECKS[level](DIFFERENTIABLE[operation]))


@pytest.mark.parametrize("operation,level", ALL_FUNCTIONS)
def test_host_size_mismatch_texts(host, operation, level):
    function = operation + level
    if level == "_vjp_vjp" and "with_weights" in operation:
        # mops/src/opsaw/cpu.tpp:133-150, mops/src/sasaw/cpu.tpp:173-194: no checks, no arithmetic
        shapes = shapes_of(operation, level)
        arguments = make_arguments(
            function, shapes, lambda s: np.zeros(s, np.float64), lambda s: np.zeros(s, np.int32)
        )
        with pytest.raises(MopsError, match="Not implemented"):
            host.call(function, *arguments)
        return
    seen = set()
    # once with every optional tensor given, once with none of them (their comparisons come
    # first and would hide the later ones)
    for absent in ((), optional_arguments(operation, level)):
        for what, shapes in perturbations(operation, level):
            expected = first_failure(operation, level, shapes, "cpu_", absent)
            arguments = make_arguments(
                function, shapes, lambda s: np.zeros(s, np.float64), lambda s: np.zeros(s, np.int32), absent
            )
            if level != "" and len(absent) > 0 and expected is None:
                # nothing requested and nothing wrong: a no-op that succeeds
                if all(name in absent for name in requested_outputs(operation, level)):
                    try:
                        host.call(function, *arguments)
                    except MopsError as error:
                        assert "device path only" in str(error), (what, str(error))
                    continue
            with pytest.raises(MopsError) as error:
                host.call(function, *arguments)
            assert error.value.status == 1
            if expected is None:
                # an extent nothing compares: validation passes, host arithmetic is refused
                assert "device path only" in str(error.value), (what, str(error.value))
            else:
                assert str(error.value) == expected, (what, absent)
                seen.add(expected)
    # every comparison of the table was reached by some perturbation
    reachable = {
        f"Dimension mismatch: the sizes of {c[0]} along dimension {c[1]} and {c[2]} along "
        f"dimension {c[3]} must match in cpu_{function}"
        for c in size_checks(operation, level)
    }
    assert seen == reachable, reachable - seen


def requested_outputs(operation, level):
    gradients = [g for g, _ in GRADIENT_CHECKS[level](DIFFERENTIABLE[operation])]
    if level == "_vjp":
        return gradients
    return [g for g in gradients if g == "grad_grad_output" or g.endswith("_2")]


@pytest.mark.parametrize("operation,level", [(o, l) for o, l in ALL_FUNCTIONS if l != ""])
def test_host_gradients_that_are_not_requested_are_not_compared(host, operation, level):
    function = operation + level
    gradients = [g for g, _ in GRADIENT_CHECKS[level](DIFFERENTIABLE[operation])]
    outputs = [g for g in gradients if not g.startswith("grad_grad_") or g == "grad_grad_output"]
    shapes = shapes_of(operation, level)
    for skipped in outputs:
        changed = dict(shapes)
        changed[skipped] = tuple(extent + 1 for extent in shapes[skipped])  # would fail if compared
        arguments = make_arguments(
            function, changed, lambda s: np.zeros(s, np.float64), lambda s: np.zeros(s, np.int32),
            absent=(skipped,),
        )  # fmt: skip
        try:
            host.call(function, *arguments)  # nothing else requested: a no-op
        except MopsError as error:
            assert "Dimension mismatch" not in str(error), (skipped, str(error))


@pytest.mark.parametrize("operation,level", ALL_FUNCTIONS)
def test_host_index_range_texts(host, operation, level):
    function = operation + level
    if level == "_vjp_vjp" and "with_weights" in operation:
        pytest.skip("throws 'Not implemented' before any check, as the reference")
    shapes = shapes_of(operation, level)
    output_name = "output" if level == "" else "grad_output"
    for position, (index_name, (bound_tensor, bound_axis)) in enumerate(INDEX_CHECKS[operation]):
        bound_tensor = output_name if bound_tensor == "output" else bound_tensor
        bound = shapes[bound_tensor][bound_axis]

        def run(values):
            arguments = []
            for kind, name in SIGNATURES[function]:
                if _KINDS[kind][1]:
                    index = np.zeros(shapes[name], np.int32)
                    if name == index_name:
                        index.reshape(-1)[: len(values)] = values
                    arguments.append(index)
                else:
                    arguments.append(np.zeros(shapes[name], np.float64))
            with pytest.raises(MopsError) as error:
                host.call(function, *arguments)
            assert error.value.status == 1
            return str(error.value)

        too_large = (
            f"Index array {index_name} in operation cpu_{function} contains elements up to {bound}; this would "
            f"cause out-of-bounds accesses. With the provided parameters, it can only contain elements up to "
            f"{bound - 1}"
        )
        negative = f"Index array {index_name} in operation cpu_{function} contains negative-valuedindices"
        assert run([bound]) == too_large
        assert run([-1]) == negative
        assert run([-3, bound]) == too_large  # the upper bound is tested first (utils.hpp:63-76)
        assert "Index array" not in run([bound - 1])  # the largest valid value


def test_sasaw_bounds_its_second_weight_index_by_the_columns_of_B(host):
    # checks/sasaw.hpp:33: W has 8 components along its second axis but B has 3 columns
    operation = "sparse_accumulation_scatter_add_with_weights"
    shapes = shapes_of(operation, "")
    assert shapes["W"][1] == 8 and shapes["B"][1] == 3
    arguments = []
    for kind, name in SIGNATURES[operation]:
        if _KINDS[kind][1]:
            index = np.zeros(shapes[name], np.int32)
            if name == "indices_W_2":
                index[0] = 5  # inside W's second axis, beyond B's columns
            arguments.append(index)
        else:
            arguments.append(np.zeros(shapes[name], np.float64))
    with pytest.raises(MopsError) as error:
        host.call(operation, *arguments)
    assert str(error.value) == (
        "Index array indices_W_2 in operation cpu_sparse_accumulation_scatter_add_with_weights contains "
        "elements up to 5; this would cause out-of-bounds accesses. With the provided parameters, it can "
        "only contain elements up to 2"
    )


def test_hpe_names_its_output_grad_output(host):
    # checks/hpe.hpp:16
    with pytest.raises(MopsError) as error:
        host.call(
            "homogeneous_polynomial_evaluation", np.zeros(5), np.zeros((6, 5)), np.zeros(7),
            np.zeros((7, 3), np.int32),
        )  # fmt: skip
    assert str(error.value) == (
        "Dimension mismatch: the sizes of A along dimension 0 and grad_output along dimension 0 must match in "
        "cpu_homogeneous_polynomial_evaluation"
    )


@pytest.mark.gpu
@pytest.mark.parametrize("operation,level", ALL_FUNCTIONS)
def test_device_size_mismatch_texts(operation, level):
    """The same walk on ``mops_cuda_*``: the comparison fails before anything is launched."""
    import torch

    from mops_amd._c_lib import device_library

    device = torch.device("cuda:0")
    library = device_library()
    function = operation + level
    if level == "_vjp_vjp" and "with_weights" in operation:
        pytest.skip("throws 'Not implemented' before any check, as the reference")
    checked = 0
    for what, shapes in perturbations(operation, level):
        expected = first_failure(operation, level, shapes, "cuda_")
        if expected is None:
            continue  # would run kernels on inconsistent shapes: not part of this test
        arguments = make_arguments(
            function, shapes, lambda s: torch.zeros(s, dtype=torch.float32, device=device),
            lambda s: torch.zeros(s, dtype=torch.int32, device=device),
        )  # fmt: skip
        with pytest.raises(MopsError) as error:
            library.call(function, *arguments)
        assert error.value.status == 1
        assert str(error.value) == expected, what
        checked += 1
    assert checked >= len(FORWARD_SIZE_CHECKS[operation])


# --------------------------------------------------------------------------
# the Python front-end (python/mops/src/mops/checks.py:9-34)
# --------------------------------------------------------------------------
def front_end_arguments(operation):
    shapes = BASE_SHAPES[operation]
    arguments = []
    for kind, name in SIGNATURES[operation][1:]:
        dtype = np.int32 if _KINDS[kind][1] else np.float64
        arguments.append(np.zeros(shapes[name], dtype))
    if operation == "outer_product_scatter_add":
        arguments.append(shapes["output"][0])
    elif operation == "sparse_accumulation_of_products":
        arguments.append(shapes["output"][1])
    elif operation == "sparse_accumulation_scatter_add_with_weights":
        arguments.append(shapes["output"][1])
    return arguments


@pytest.mark.parametrize("operation", list(FORWARD_SIZE_CHECKS))
def test_front_end_type_and_dimension_texts(operation):
    import mops_amd

    function = getattr(mops_amd, operation)
    names = [name for _, name in SIGNATURES[operation][1:]]
    for position, name in enumerate(names):
        arguments = front_end_arguments(operation)
        is_index = arguments[position].dtype == np.int32

        # wrong dtype (python/mops/tests/opsa.py:44-51 and siblings)
        wrong = front_end_arguments(operation)
        wrong[position] = wrong[position].astype(np.float64 if is_index else np.int32)
        got = "float64" if is_index else "int32"
        with pytest.raises(TypeError) as error:
            function(*wrong)
        assert str(error.value) == f"Wrong dtype for {name} in {operation}: got {got}"

        # one dimension too many (python/mops/tests/opsa.py:54-63 and siblings)
        wrong = front_end_arguments(operation)
        ndim = wrong[position].ndim
        wrong[position] = wrong[position][..., np.newaxis]
        with pytest.raises(ValueError) as error:
            function(*wrong)
        assert str(error.value) == (
            f"`{name}` must be a {ndim}D array in {operation}, got a {ndim + 1}D array instead"
        )

        # not an array at all
        wrong = front_end_arguments(operation)
        wrong[position] = [1, 2, 3]
        with pytest.raises(TypeError) as error:
            function(*wrong)
        assert str(error.value) == f"`{name}` must be an array in {operation}, got <class 'list'>"


@pytest.mark.parametrize(
    "operation", ["outer_product_scatter_add", "sparse_accumulation_of_products",
                  "sparse_accumulation_scatter_add_with_weights"],
)  # fmt: skip
def test_front_end_output_size_texts(operation):
    import mops_amd

    function = getattr(mops_amd, operation)
    arguments = front_end_arguments(operation)
    arguments[-1] = "4"
    with pytest.raises(TypeError) as error:
        function(*arguments)
    assert str(error.value) == f"`output_size` must be a scalar in {operation}, got <class 'str'>"
    arguments[-1] = 4.0
    with pytest.raises(TypeError) as error:
        function(*arguments)
    assert str(error.value) == f"Wrong dtype for output_size in {operation}: got <class 'float'>"


def test_front_end_size_mismatch_and_out_of_bounds_reach_the_library():
    # python/mops/tests/sasaw.py:215-260
    import mops_amd

    operation = "sparse_accumulation_scatter_add_with_weights"
    arguments = front_end_arguments(operation)
    names = [name for _, name in SIGNATURES[operation][1:]]
    arguments[names.index("indices_output_1")] = arguments[names.index("indices_output_1")][:5]
    with pytest.raises(MopsError) as error:
        getattr(mops_amd, operation)(*arguments)
    assert str(error.value) == (
        "Dimension mismatch: the sizes of A along dimension 0 and indices_output_1 along dimension 0 must match "
        "in cpu_sparse_accumulation_scatter_add_with_weights"
    )
    arguments = front_end_arguments(operation)
    arguments[names.index("indices_output_1")][0] = 4
    with pytest.raises(MopsError) as error:
        getattr(mops_amd, operation)(*arguments)
    assert str(error.value) == (
        "Index array indices_output_1 in operation cpu_sparse_accumulation_scatter_add_with_weights contains "
        "elements up to 4; this would cause out-of-bounds accesses. With the provided parameters, it can only "
        "contain elements up to 3"
    )


def test_front_end_refuses_tensors_on_different_devices_before_any_launch():
    """A host array beside a device tensor must raise, not reach a kernel (no GPU needed:
    the host branch is tested with a CPU tensor first and a fake device tensor cannot exist)."""
    import torch

    from mops_amd import ops

    class Probe:
        called = False

    def forbidden(*a, **k):
        Probe.called = True
        raise AssertionError("the library must not be called")

    # the first tensor in host memory, another claims to be on the GPU: meta tensors stand in
    # for device tensors here (they have a device that is not the CPU and no data)
    A = torch.zeros((6, 5), dtype=torch.float64)
    B = torch.zeros((6, 3), dtype=torch.float64, device="meta")
    index = torch.zeros(6, dtype=torch.int32)
    original = ops._dispatch.on_device
    ops._dispatch.on_device = lambda t: ops._dispatch.is_torch(t) and t.device.type != "cpu"
    try:
        with pytest.raises(ValueError, match="`B` is on meta but the first tensor is in host memory"):
            ops._call("outer_product_scatter_add", A, [torch.zeros((4, 5, 3), dtype=torch.float64), A, B, index])
    finally:
        ops._dispatch.on_device = original
    assert not Probe.called


@pytest.mark.gpu
def test_front_end_refuses_host_arrays_beside_device_tensors():
    import torch

    import mops_amd

    device = torch.device("cuda:0")
    A = torch.zeros((6, 5), dtype=torch.float32, device=device)
    B = torch.zeros((6, 3), dtype=torch.float32)  # left on the host by mistake
    index = torch.zeros(6, dtype=torch.int32, device=device)
    with pytest.raises(ValueError, match="`B` is on cpu but the first tensor is on cuda:0"):
        mops_amd.outer_product_scatter_add(A, B, index, 4)
    with pytest.raises(TypeError, match="`indices_output` must be a torch tensor on cuda:0"):
        mops_amd.outer_product_scatter_add(A, B.to(device), np.zeros(6, np.int32), 4)
