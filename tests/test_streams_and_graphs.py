"""Calls on caller-owned streams: capture into a HIP graph and replay, and two host threads at once.

The library launches on the stream named with mops_amd_set_stream (per host
thread) and, in asynchronous mode, neither allocates nor synchronises once its
scratch block has its size, so a call can be captured; SASAW's vjp forks to a
side stream and joins again inside the call, which a capture has to follow.
"""
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
    # edges ordered by sender on a side stream (edges x nodes / 4 beyond the in-kernel gather)
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


def test_two_host_threads_on_their_own_streams(device):
    """The per-thread state (stream, scratch block, error message) keeps two callers apart."""
    results = {}
    errors = []

    def worker(op):
        try:
            case = support.to_device(CASES[op](np.float32), device)
            stream = torch.cuda.Stream(device=device)
            with torch.cuda.stream(stream):
                first = [t.clone() for t in _call(op, case)]
                for _ in range(20):
                    again = _call(op, case)
                stream.synchronize()
                results[op] = all(torch.equal(a, b) for a, b in zip(first, again))
        except Exception as error:  # pragma: no cover - reported below
            errors.append((op, repr(error)))

    threads = [threading.Thread(target=worker, args=(op,)) for op in ("opsaw", "sasaw")]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join()
    assert not errors, errors
    assert results == {"opsaw": True, "sasaw": True}
