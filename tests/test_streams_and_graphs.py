"""Calls on caller-owned streams: capture into a HIP graph and replay, and two host threads at once.

The library launches on the stream named with mops_amd_set_stream (per host
thread) and, in asynchronous mode, neither allocates nor synchronises once its
scratch block has its size, so a call can be captured; SASAW's vjp forks to a
side stream and joins again inside the call, which a capture has to follow.
"""
import ctypes
import threading

import numpy as np
import pytest
import torch

from tests import support
from tests.support import OPS

pytestmark = pytest.mark.gpu

CASES = {
    "hpe": lambda d: support.hpe_case(21, d, I=300, nA=20, J=150, K=3),
    "sap": lambda d: support.sap_case(22, d, I=700, nA=13, nB=7, K=300, nO=20),
    "opsa": lambda d: support.opsa_case(23, d, J=2000, K=13, L=20, n_out=70, allow_empty=True),
    "opsaw": lambda d: support.opsaw_case(24, d, E=2000, K=13, L=32, n_nodes=70, allow_empty=True),
    "sasaw": lambda d: support.sasaw_case(25, d, E=2000, nA=9, L=32, n_nodes=70, allow_empty=True),
    # paths with more than one kernel per call and with scratch memory between them:
    # segments cut into pieces and added up (OPSA forward of long segments)
    "opsa_pooling": lambda d: support.opsa_case(26, d, J=6000, K=13, L=20, n_out=8),
    # blocks of 64 columns, grad_A added to by one launch after the other
    "sasaw_many_columns": lambda d: support.sasaw_case(27, d, E=1500, nA=9, L=160, n_nodes=50, allow_empty=True),
    # more than 4000 nodes: the senders' edges listed by arrival, on counters that every replay must find at zero
    "opsaw_many_senders": lambda d: support.opsaw_case(29, d, E=30000, K=4, L=16, n_nodes=9000, allow_empty=True),
    "sasaw_many_senders": lambda d: support.sasaw_case(28, d, E=30000, nA=4, L=16, n_nodes=16000, n2=4, n3=4, N=30, allow_empty=True),
}


def _operation(name):
    return name.split("_")[0]


def _call(op, case):
    import mops_amd

    op = _operation(op)
    spec = OPS[op]
    forward = getattr(mops_amd, spec.function)
    backward = getattr(mops_amd, spec.function + "_vjp")
    arguments = [case[name] for name in spec.inputs]
    if op in ("sap", "opsa", "sasaw"):
        arguments.append(case["output_size"])
    output = forward(*arguments)
    gradients = backward(case["grad_output"], *[case[name] for name in spec.inputs])
    gradients = gradients if isinstance(gradients, (tuple, list)) else (gradients,)
    return [output, *gradients]


@pytest.mark.parametrize("op", list(CASES))
def test_graph_replays_match_eager_calls(device, op):
    case = support.to_device(CASES[op](np.float32), device)
    eager = [t.clone() for t in _call(op, case)]
    torch.cuda.synchronize()

    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        _call(op, case)  # the scratch block takes its size outside the capture
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            captured = _call(op, case)
    torch.cuda.synchronize()
    for replay in range(3):
        for tensor in captured:
            tensor.fill_(float("nan"))
        # eager work of the program between the replays
        other = _call(op, case)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want, again in zip(captured, eager, other):
            assert torch.equal(got, want), (op, replay)
            assert torch.equal(again, want), (op, replay)


@pytest.mark.parametrize("op", sorted(support.SECOND_ORDER))
def test_second_order_calls_replayed_from_a_graph(device, op):
    """With both cotangents given, the second-order functions of these shapes launch kernels only (no
    temporary from the stream's memory pool), so they can be captured; replays against eager calls."""
    from mops_amd._c_lib import device_library

    library = device_library()
    spec = OPS[op]
    case = support.to_device(support.add_cotangents(CASES[op](np.float64), op), device)

    def call():
        library.cdll.mops_amd_set_stream(torch.cuda.current_stream(device).cuda_stream)
        library.cdll.mops_amd_set_synchronous(0)
        outputs, arguments = support._vjp_vjp_arguments(
            spec, case, None, None, lambda x: torch.full_like(x, float("nan"))
        )
        library.call(spec.function + "_vjp_vjp", *arguments)
        return outputs

    try:
        eager = {key: value.clone() for key, value in call().items()}
        torch.cuda.synchronize()
        stream = torch.cuda.Stream(device=device)
        stream.wait_stream(torch.cuda.current_stream(device))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            call()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                captured = call()
        torch.cuda.synchronize()
        for replay in range(2):
            for tensor in captured.values():
                tensor.fill_(float("nan"))
            other = call()  # eager work between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for key in eager:
                assert torch.equal(captured[key], eager[key]), (op, key, replay)
                assert torch.equal(other[key], eager[key]), (op, key, replay)
    finally:
        support._bind_stream(library, device)


def test_two_host_threads_on_their_own_streams(oracle, device):
    """Two host threads, each on a stream of its own, call different operations at the same time:
    the per-thread state (stream, scratch block, error message) keeps them apart, and both get
    the oracle's results."""
    results = {}
    errors = []
    ready = threading.Barrier(2)

    def worker(op):
        try:
            host_case = CASES[op](np.float32)
            case = support.to_device(host_case, device)
            stream = torch.cuda.Stream(device=device)
            ready.wait()
            with torch.cuda.stream(stream):
                first = [t.clone() for t in _call(op, case)]
                for _ in range(20):
                    again = _call(op, case)
                stream.synchronize()
            results[op] = (host_case, first, all(torch.equal(a, b) for a, b in zip(first, again)))
        except Exception as error:  # pragma: no cover - reported below
            errors.append((op, repr(error)))
            ready.abort()

    threads = [threading.Thread(target=worker, args=(op,)) for op in ("opsaw", "sasaw")]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join()
    assert not errors, errors
    for op in ("opsaw", "sasaw"):
        host_case, first, repeatable = results[op]
        assert repeatable, op
        spec = OPS[op]
        support.assert_close(first[0].cpu().numpy(), support.cpu_forward(oracle, op, host_case), np.float32, op)
        expected = support.cpu_vjp(oracle, op, host_case)
        for name, got in zip(spec.differentiable, first[1:]):
            support.assert_close(got.cpu().numpy(), expected[name], np.float32, f"{op} grad_{name}")


def test_threads_that_end_hand_their_scratch_block_on(device):
    """A thread's scratch block goes to the next new thread instead of being lost."""
    from mops_amd._c_lib import device_library

    library = device_library()
    library.cdll.mops_amd_scratch_capacity.restype = ctypes.c_int64
    library.cdll.mops_amd_reserve_scratch.argtypes = [ctypes.c_int64]
    seen = []

    def worker(reserve):
        torch.cuda.set_device(device)
        if reserve:
            assert library.cdll.mops_amd_reserve_scratch(3 << 20) == 0
        else:
            # the first use of the state takes over what an ended thread left
            assert library.cdll.mops_amd_reserve_scratch(1) == 0
        seen.append(library.cdll.mops_amd_scratch_capacity())

    for reserve in (True, False):
        thread = threading.Thread(target=worker, args=(reserve,))
        thread.start()
        thread.join()
    assert seen[0] >= 3 << 20
    assert seen[1] == seen[0]


def test_growing_the_scratch_block_during_a_capture_is_refused(device):
    """No allocation can happen while a stream is being captured: the call fails with a message
    instead (a host-side check; nothing is launched)."""
    from mops_amd._c_lib import device_library

    library = device_library()
    library.cdll.mops_amd_scratch_capacity.restype = ctypes.c_int64
    library.cdll.mops_amd_reserve_scratch.argtypes = [ctypes.c_int64]
    torch.cuda.set_device(device)
    library.cdll.mops_amd_set_stream(torch.cuda.current_stream(device).cuda_stream)
    assert library.cdll.mops_amd_reserve_scratch(1) == 0
    capacity = library.cdll.mops_amd_scratch_capacity()
    assert capacity >= 1 << 20

    marker = torch.zeros(16, device=device)
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            library.cdll.mops_amd_set_stream(stream.cuda_stream)
            library.cdll.mops_amd_set_synchronous(0)
            marker.add_(1.0)
            within = library.cdll.mops_amd_reserve_scratch(capacity)  # fits: fine during a capture
            status = library.cdll.mops_amd_reserve_scratch(4 * capacity)
            message = library.last_error()
    library.cdll.mops_amd_set_stream(torch.cuda.current_stream(device).cuda_stream)
    assert within == 0
    assert status == 1
    assert "being captured" in message and "before capturing" in message
    assert library.cdll.mops_amd_scratch_capacity() == capacity  # untouched
    graph.replay()
    torch.cuda.synchronize()
    assert float(marker[0]) == 1.0


def test_a_block_that_a_graph_names_outlives_a_later_growth(device):
    """Eager calls with larger shapes after a capture must not free the block the graph uses."""
    from mops_amd._c_lib import device_library

    library = device_library()
    library.cdll.mops_amd_scratch_capacity.restype = ctypes.c_int64
    library.cdll.mops_amd_reserve_scratch.argtypes = [ctypes.c_int64]
    op = "opsa_pooling"  # pieces of long segments meet in scratch memory
    case = support.to_device(CASES[op](np.float32), device)
    eager = [t.clone() for t in _call(op, case)]
    torch.cuda.synchronize()
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        _call(op, case)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            captured = _call(op, case)
    torch.cuda.synchronize()
    library.cdll.mops_amd_set_stream(torch.cuda.current_stream(device).cuda_stream)
    before = library.cdll.mops_amd_scratch_capacity()
    assert library.cdll.mops_amd_reserve_scratch(8 * before) == 0  # grows: the old block is kept
    assert library.cdll.mops_amd_scratch_capacity() >= 8 * before
    filler = torch.full((before // 4,), float("nan"), device=device)  # would land in a freed block
    for tensor in captured:
        tensor.fill_(float("nan"))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    for got, want in zip(captured, eager):
        assert torch.equal(got, want)
    del filler


@pytest.mark.parametrize(
    "op,point", [("opsaw_many_senders", "opsaw_vjp_after_listing"), ("sasaw_many_senders", "sasaw_vjp_after_listing")]
)
def test_a_call_that_fails_between_two_launches_does_not_spoil_the_next(device, monkeypatch, op, point):
    """The senders' edges of large graphs are listed by a launch that counts in counters which the
    launch that uses the lists sets back to zero. A call that fails on the host between the two
    leaves counts behind; the library marks its counters on the host and clears them at the start
    of the next call. The failure is requested from the host (MOPS_AMD_TEST_FAIL_AT): every
    kernel that was enqueued runs to its end."""
    from mops_amd.status import MopsError

    case = support.to_device(CASES[op](np.float32), device)
    good = [t.clone() for t in _call(op, case)]
    torch.cuda.synchronize()
    monkeypatch.setenv("MOPS_AMD_TEST_FAIL_AT", point)
    with pytest.raises(MopsError, match="failure requested by MOPS_AMD_TEST_FAIL_AT"):
        _call(op, case)
    torch.cuda.synchronize()
    monkeypatch.delenv("MOPS_AMD_TEST_FAIL_AT")
    for attempt in range(2):
        again = _call(op, case)
        torch.cuda.synchronize()
        for got, want in zip(again, good):
            assert torch.equal(got, want), (op, attempt)
