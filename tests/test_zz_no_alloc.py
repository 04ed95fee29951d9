"""The entry point that allocates nothing, against the entry point it is a variant of.

``mops_amd_sparse_accumulation_scatter_add_with_weights_vjp_no_alloc_f32`` (include/mops/amd.h)
keeps the temporaries of its kernels in an array that is part of the library's device code
instead of the per-thread scratch block. Called through the C ABI, twice in a row, the second
time with a smaller input (the array then still holds the first call's lists), and compared bit
for bit with ``mops_cuda_sparse_accumulation_scatter_add_with_weights_vjp_f32`` and, to the
float32 bar, with the oracle.
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
