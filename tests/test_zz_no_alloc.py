"""The entry point that allocates nothing, against the entry point it is a variant of.

``mops_amd_sparse_accumulation_scatter_add_with_weights_vjp_no_alloc_f32`` (include/mops/amd.h)
keeps the temporaries of its kernels in an array that is part of the library's device code
instead of the per-thread scratch block. Called through the C ABI, twice in a row, the second
time with a smaller input (the array then still holds the first call's lists), and compared bit
for bit with ``mops_cuda_sparse_accumulation_scatter_add_with_weights_vjp_f32`` and, to the
float32 bar, with the oracle. And the property the entry point exists for: no device memory
is allocated by a call, and a call can be captured into a HIP graph and replayed.
"""
import ctypes

import numpy as np
import pytest

from tests import support

pytestmark = pytest.mark.gpu

FUNCTION = "sparse_accumulation_scatter_add_with_weights_vjp"
SYMBOL = "mops_amd_" + FUNCTION + "_no_alloc_f32"


def no_alloc_call(library, *tensors):
    from mops_amd._c_api import _KINDS, SIGNATURES, STRUCTS, view
    from mops_amd.status import MopsError

    signature = SIGNATURES[FUNCTION]
    symbol = getattr(library.cdll, SYMBOL)
    symbol.restype = ctypes.c_int
    symbol.argtypes = [STRUCTS[(_KINDS[kind][0], "i32" if _KINDS[kind][1] else "f32")] for kind, _ in signature]
    status = symbol(*[view(tensor, kind, "f32") for (kind, _), tensor in zip(signature, tensors)])
    if status != 0:
        raise MopsError(library.last_error(), status)


def gradients_of(library, case, entry, wanted=("A", "B", "W")):
    import torch

    spec = support.OPS["sasaw"]
    gradients = [
        torch.full_like(case[name], float("nan")) if name in wanted else None for name in spec.differentiable
    ]
    arguments = [*gradients, case["grad_output"], *[case[name] for name in spec.inputs]]
    if entry == "no_alloc":
        no_alloc_call(library, *arguments)
    else:
        library.call(FUNCTION, *arguments)
    torch.cuda.synchronize()
    return dict(zip(spec.differentiable, gradients))


def test_two_calls_in_a_row_the_second_smaller(oracle, device):
    import torch

    from mops_amd._c_lib import device_library

    library = device_library()
    support._bind_stream(library, device)
    cases = [
        support.sasaw_case(41, np.float32, E=6000, nA=9, L=32, n_nodes=200, allow_empty=True),
        support.sasaw_case(42, np.float32, E=900, nA=9, L=32, n_nodes=50, allow_empty=True),
    ]
    for number, host_case in enumerate(cases):
        case = support.to_device(host_case, device)
        print(f"no-alloc call {number}: E={host_case['A'].shape[0]}", flush=True)
        got = gradients_of(library, case, "no_alloc")
        want = gradients_of(library, case, "existing")
        expected = support.cpu_vjp(oracle, "sasaw", host_case)
        for name in ("A", "B", "W"):
            assert torch.equal(got[name], want[name]), (number, name)
            support.assert_close(got[name].cpu().numpy(), expected[name], np.float32, f"call {number} grad_{name}")
    # a subset of the gradients, again on the array the calls above used
    case = support.to_device(cases[0], device)
    for wanted in (("W",), ("A", "B"), ("B",)):
        got = gradients_of(library, case, "no_alloc", wanted)
        want = gradients_of(library, case, "existing", wanted)
        for name in wanted:
            assert torch.equal(got[name], want[name]), (wanted, name)


def test_nodes_beyond_the_slots(oracle, device):
    """Graphs of this size list the senders' edges by arrival, on counters that have to start at
    zero: here they lie in the built-in array, behind whatever an earlier call left there."""
    import torch

    from mops_amd._c_lib import device_library

    library = device_library()
    support._bind_stream(library, device)
    host_case = support.sasaw_case(44, np.float32, E=40000, nA=4, L=20, n_nodes=7000, n2=3, n3=4, N=30, allow_empty=True)
    case = support.to_device(host_case, device)
    expected = support.cpu_vjp(oracle, "sasaw", host_case)
    for number in range(2):
        print(f"no-alloc call {number} with 7000 nodes", flush=True)
        got = gradients_of(library, case, "no_alloc")
        want = gradients_of(library, case, "existing")
        for name in ("A", "B", "W"):
            assert torch.equal(got[name], want[name]), (number, name)
            support.assert_close(got[name].cpu().numpy(), expected[name], np.float32, f"call {number} grad_{name}")


def test_shapes_beyond_the_built_in_array_are_refused(device):
    import torch

    from mops_amd._c_lib import device_library
    from mops_amd.status import MopsError

    library = device_library()
    support._bind_stream(library, device)
    # 9000 nodes: the lists of the senders' edges alone need more than 4 MiB
    host_case = support.sasaw_case(43, np.float32, E=9000, nA=2, L=4, n_nodes=9000, n2=2, n3=2, N=3, allow_empty=True)
    case = support.to_device(host_case, device)
    with pytest.raises(MopsError, match="bytes of temporary memory, the built-in array holds 4194304"):
        gradients_of(library, case, "no_alloc")
    # the shape checks of the existing entry point come first, with its texts
    case["B"] = torch.zeros((8999, 4), dtype=torch.float32, device=device)
    with pytest.raises(MopsError, match="Dimension mismatch: the sizes of A along dimension 0 and B along dimension 0"):
        gradients_of(library, case, "no_alloc")


@pytest.mark.parametrize(
    "shape",
    [
        # the senders' edges in slots
        dict(E=6000, nA=9, L=32, n_nodes=200),
        # more than 4000 nodes: listed by arrival, on counters inside the built-in array
        dict(E=30000, nA=4, L=16, n_nodes=6000, n2=4, n3=4, N=30),
    ],
    ids=["slots", "by_arrival"],
)
def test_captured_into_a_graph_and_free_of_allocations(device, shape):
    """Asynchronous calls inside a stream capture (where an allocation, a stream or event creation
    or a wait would end the capture with an error), replayed twice with eager calls in between,
    against the eager results; the free device memory is the same before and after eager calls,
    also with kernel timing switched on (which the entry point switches off for its own length)."""
    import torch

    from mops_amd._c_lib import device_library

    library = device_library()
    host_case = support.sasaw_case(45, np.float32, allow_empty=True, **shape)
    case = support.to_device(host_case, device)
    support._bind_stream(library, device)
    eager = gradients_of(library, case, "existing")
    torch.cuda.synchronize()

    spec = support.OPS["sasaw"]
    captured = [torch.full_like(case[name], float("nan")) for name in spec.differentiable]
    arguments = [*captured, case["grad_output"], *[case[name] for name in spec.inputs]]

    # no allocation by eager calls: what the driver reports as free does not move
    previous_timing = library.cdll.mops_amd_kernel_timing(1)
    try:
        no_alloc_call(library, *arguments)  # (loads the code object's array on first use)
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info(device)
        for _ in range(5):
            no_alloc_call(library, *arguments)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info(device)
        total = ctypes.c_double(0.0)
        launches = ctypes.c_int64(-1)
        assert library.cdll.mops_amd_kernel_time(ctypes.byref(total), ctypes.byref(launches)) == 0
    finally:
        library.cdll.mops_amd_kernel_timing(previous_timing)
    assert free_after == free_before
    assert launches.value == 0  # no events were taken for this entry point
    for got, name in zip(captured, spec.differentiable):
        assert torch.equal(got, eager[name]), name

    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    graph = torch.cuda.CUDAGraph()
    try:
        with torch.cuda.stream(stream):
            library.cdll.mops_amd_set_stream(ctypes.c_void_p(stream.cuda_stream))
            library.cdll.mops_amd_set_synchronous(0)
            with torch.cuda.graph(graph, stream=stream):
                no_alloc_call(library, *arguments)
    finally:
        support._bind_stream(library, device)
    torch.cuda.synchronize()
    for replay in range(2):
        for tensor in captured:
            tensor.fill_(float("nan"))
        other = gradients_of(library, case, "no_alloc")  # eager work on the same array in between
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, name in zip(captured, spec.differentiable):
            assert torch.equal(got, eager[name]), (replay, name)
            assert torch.equal(other[name], eager[name]), (replay, name)


def test_degenerate_shapes_give_zero_gradients(device):
    """No columns, no table entries: every sum is empty, as with the existing entry point."""
    import torch

    from mops_amd._c_lib import device_library

    library = device_library()
    support._bind_stream(library, device)
    for shape in (dict(L=0), dict(N=0)):
        host_case = support.sasaw_case(46, np.float32, **{**dict(E=300, nA=3, L=8, n_nodes=20, n2=3, n3=3, N=10), **shape})
        case = support.to_device(host_case, device)
        got = gradients_of(library, case, "no_alloc")
        want = gradients_of(library, case, "existing")
        for name in ("A", "B", "W"):
            assert torch.equal(got[name], want[name]), (shape, name)
            assert not torch.isnan(got[name]).any()
