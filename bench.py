"""Benchmark of the mops device path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--all/--no-all]

Prints ONE JSON line. The headline workload is BASELINE configuration 1
(sparse accumulation of products, float32: A[32000,13], B[32000,7], 900
products, 20 outputs); one "step" is its forward followed by its vjp with
respect to A and B. ``value`` is algorithmic bytes of a step (every input read
once, every output written once) divided by the wall time per step, inputs
resident in HBM, inputs rotated through more than 256 MB of distinct buffers so
that the 256 MB Infinity Cache cannot serve them.

Per-kernel figures (``roofline`` for the dominant kernel of the headline, and
``per_op`` for every BASELINE configuration, forward and vjp separately) are
device times: the launches of one function over the rotating buffers are
captured into a HIP graph and the replay is timed with HIP events on the
stream the kernels run on, which removes the Python / ctypes launch overhead
from the measurement. The time is per call of the function, i.e. it contains
every kernel the call launches (first_occurrences, the sender regrouping, the
table regrouping), not only the main one.

``cpu_baseline`` times the CPU oracle (a port of the reference's OpenMP
algorithm, oracle/oracle.cpp) on the same headline workload on this machine's
host cores for about ten seconds.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X, published
ROTATE_BYTES = 320 * 1024 * 1024  # > 256 MB Infinity Cache
# HBM bytes per launch of the main SAP f32 kernels from two rocprofv3 --pmc
# runs (profiles/all_ops_baseline_shapes_hbm_traffic.txt): FETCH_SIZE x 1.9993
# (the factor a 64 MiB element-wise pass gives) + WRITE_SIZE x 1.0, in KiB.
# forward: 1742.5 and 2500.0; vjp: 3099.8 and 2500.0.
MEASURED_TRAFFIC_BYTES = {"forward": 6094000, "vjp": 8888000}


def nbytes(arrays):
    return int(sum(a.nbytes for a in arrays))


def algorithmic_bytes(op, case, kind):
    """Every input read once + every output written once (index tensors included)."""
    from tests.support import OPS

    spec = OPS[op]
    inputs = [case[name] for name in spec.inputs]
    if kind == "forward":
        out_elements = int(np.prod(spec.output_shape(case)))
        return nbytes(inputs) + out_elements * case["A"].dtype.itemsize
    grads = [case[name] for name in spec.differentiable]
    return nbytes(inputs) + case["grad_output"].nbytes + nbytes(grads)


def build_configs():
    from tests import support

    return [
        ("c0", "hpe", np.float64, support.hpe_case(0, np.float64)),
        ("c1", "sap", np.float32, support.sap_case(1, np.float32)),
        ("c1", "sap", np.float64, support.sap_case(1, np.float64)),
        ("c2", "opsa", np.float32, support.opsa_case(2, np.float32)),
        ("c2", "opsa", np.float64, support.opsa_case(2, np.float64)),
        ("c3", "opsaw", np.float32, support.opsaw_case(3, np.float32)),
        ("c4", "sasaw", np.float32, support.sasaw_case(4, np.float32)),
        ("c4", "sasaw", np.float64, support.sasaw_case(4, np.float64)),
        # beyond the BASELINE shapes: feature counts that fill whole 16-wide matrix tiles
        ("wide", "opsa", np.float32, support.opsa_case(5, np.float32, K=32, L=64)),
        ("wide", "opsaw", np.float32, support.opsaw_case(6, np.float32, K=32, L=64)),
        # many rows: HPE with a lane per row (forward) and by feature (vjp)
        ("many_rows", "hpe", np.float64, support.hpe_case(10, np.float64, I=20000, nA=50, J=4000, K=3)),
        # 128 feature channels: the kernels take them in blocks of 64 columns
        ("wide128", "opsa", np.float32, support.opsa_case(7, np.float32, K=16, L=128)),
        ("wide128", "opsaw", np.float32, support.opsaw_case(8, np.float32, K=16, L=128)),
        ("wide128", "sasaw", np.float32, support.sasaw_case(9, np.float32, L=128)),
    ]


class DeviceWorkload:
    """One operation with its inputs replicated over enough buffer sets to defeat the caches."""

    def __init__(self, op, case, device):
        import torch

        from mops_amd._c_lib import device_library
        from tests.support import OPS, to_device

        self.op = op
        self.spec = OPS[op]
        self.case = case
        self.library = device_library()
        per_set = algorithmic_bytes(op, case, "forward") + algorithmic_bytes(op, case, "vjp")
        self.n_sets = max(2, int(np.ceil(ROTATE_BYTES / per_set)))
        self.sets = []
        for _ in range(self.n_sets):
            tensors = to_device(case, device)
            tensors = {k: (v.clone() if hasattr(v, "clone") else v) for k, v in tensors.items()}
            A = tensors["A"]
            tensors["output"] = torch.empty(self.spec.output_shape(case), dtype=A.dtype, device=device)
            for name in self.spec.differentiable:
                tensors["grad_" + name] = torch.empty_like(tensors[name])
            self.sets.append(tensors)
        self.cursor = 0
        self.rotate = True

    def _next(self):
        if not self.rotate:
            return self.sets[0]  # the same buffers every call: whatever the caches keep stays
        tensors = self.sets[self.cursor]
        self.cursor = (self.cursor + 1) % self.n_sets
        return tensors

    def forward(self):
        t = self._next()
        self.library.call(self.spec.function, t["output"], *[t[n] for n in self.spec.inputs])

    def vjp(self):
        t = self._next()
        self.library.call(
            self.spec.function + "_vjp",
            *[t["grad_" + n] for n in self.spec.differentiable],
            t["grad_output"],
            *[t[n] for n in self.spec.inputs],
        )

    def step(self):
        self.forward()
        self.vjp()


def bind_library_to_torch_stream(device):
    import torch

    from mops_amd._c_lib import device_library

    library = device_library()
    torch.cuda.set_device(device)
    library.cdll.mops_amd_set_stream(torch.cuda.current_stream(device).cuda_stream)
    library.cdll.mops_amd_set_synchronous(0)
    return library


def device_time_per_call(function, calls, replays, device):
    """Average device time (seconds) of one call of ``function``.

    ``calls`` consecutive calls are captured into a HIP graph; the graph is
    replayed ``replays`` times between two HIP events on the capture stream's
    parent (torch's current) stream.
    """
    import torch

    for _ in range(3):
        function()  # warm up: allocates the library's scratch block outside the capture
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    captured = True
    try:
        with torch.cuda.stream(stream):
            bind_library_to_torch_stream(device)
            function()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                bind_library_to_torch_stream(device)
                for _ in range(calls):
                    function()
    except Exception as error:  # pragma: no cover - depends on the runtime
        captured = False
        sys.stderr.write(f"graph capture failed ({error}); timing eager launches instead\n")
    bind_library_to_torch_stream(device)
    torch.cuda.synchronize()

    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    if captured:
        graph.replay()
        torch.cuda.synchronize()
        start.record()
        for _ in range(replays):
            graph.replay()
        stop.record()
    else:
        start.record()
        for _ in range(replays * calls):
            function()
        stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / (replays * calls), captured


def capture_steps(workload, steps, device):
    """A HIP graph holding ``steps`` consecutive steps of ``workload`` (None if capture fails)."""
    import torch

    for _ in range(3):
        workload.step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
    try:
        with torch.cuda.stream(stream):
            bind_library_to_torch_stream(device)
            workload.step()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                bind_library_to_torch_stream(device)
                for _ in range(steps):
                    workload.step()
    except Exception as error:  # pragma: no cover - depends on the runtime
        sys.stderr.write(f"graph capture failed ({error}); timing eager launches instead\n")
        graph = None
    bind_library_to_torch_stream(device)
    torch.cuda.synchronize()
    return graph


def main_kernel_time(library, function, calls):
    """Average duration (seconds) of the main kernel of ``function`` over ``calls`` eager calls.

    The library attaches a pair of HIP events to that kernel's launch on the
    stream it launches it on (mops_amd_kernel_timing in include/mops/amd.h).
    """
    import ctypes

    import torch

    function()
    torch.cuda.synchronize()
    library.cdll.mops_amd_kernel_timing(1)
    try:
        for _ in range(calls):
            function()
        total = ctypes.c_double(0.0)
        launches = ctypes.c_int64(0)
        status = library.cdll.mops_amd_kernel_time(ctypes.byref(total), ctypes.byref(launches))
    finally:
        library.cdll.mops_amd_kernel_timing(0)
    if status != 0 or launches.value == 0:
        return None, 0
    return total.value * 1e-3 / launches.value, launches.value


def cpu_time(function, seconds, max_calls):
    function()
    function()
    times = []
    begin = time.perf_counter()
    while len(times) < max_calls and (time.perf_counter() - begin < seconds or len(times) < 3):
        t0 = time.perf_counter()
        function()
        times.append(time.perf_counter() - t0)
    return times


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=2000)
    parser.add_argument("--warmup", type=int, default=100)
    parser.add_argument("--cpu-seconds", type=float, default=10.0)
    parser.add_argument("--no-per-op", action="store_true", help="only the headline workload")
    parser.add_argument(
        "--profile",
        choices=["hpe", "sap", "opsa", "opsaw", "sasaw", "all"],
        help="for rocprofv3: run 50 eager forward+vjp calls of the operation(s) at the BASELINE "
        "shapes (all their dtypes) and 20 element-wise passes over 64 MiB (read 64 MiB, write 64 MiB) as a yardstick for the HBM "
        "counters, print nothing, exit",
    )
    args = parser.parse_args()

    if args.gpus != 1:
        sys.stderr.write(
            "bench.py measures one GPU: every box of this build has a single MI355X and the five "
            "operations have no multi-GPU path (they would shard over rows / receivers, one gather and one "
            "reduce-scatter of the weights per call). "
            "Run with --gpus 1.\n"
        )
        sys.exit(2)

    import torch

    from tests import support

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs a GPU (the device library has no CPU fallback)\n")
        sys.exit(2)
    device = torch.device("cuda:0")
    bind_library_to_torch_stream(device)
    oracle = support.oracle_library()
    configs = build_configs()

    if args.profile:
        for config, op_name, _, op_case in configs:
            if config.startswith("c") and args.profile in (op_name, "all"):
                w = DeviceWorkload(op_name, op_case, device)
                for _ in range(50):
                    w.step()
                torch.cuda.synchronize()
                del w
                torch.cuda.empty_cache()
        source = torch.empty(64 * 1024 * 1024 // 4, dtype=torch.float32, device=device).normal_()
        target = torch.empty_like(source)
        for _ in range(20):
            torch.mul(source, 2.0, out=target)  # reads 64 MiB, writes 64 MiB
        torch.cuda.synchronize()
        return

    # ---------------- headline: c1 SAP f32, forward + vjp -------------------
    # The K timed steps are replays of HIP graphs that hold `steps_per_graph`
    # steps each (the launch-bound loop is what graphs are for); what does not
    # fill a whole graph is launched eagerly inside the same timed region.
    _, op, dtype, case = configs[1]
    workload = DeviceWorkload(op, case, device)
    step_bytes = algorithmic_bytes(op, case, "forward") + algorithmic_bytes(op, case, "vjp")
    steps_per_graph = max(1, min(workload.n_sets // 2, args.steps))
    graph = capture_steps(workload, steps_per_graph, device)
    for _ in range(args.warmup):
        workload.step()
    torch.cuda.synchronize()
    begin = time.perf_counter()
    done = 0
    if graph is not None:
        while done + steps_per_graph <= args.steps:
            graph.replay()
            done += steps_per_graph
    while done < args.steps:
        workload.step()
        done += 1
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - begin
    ms_per_step = elapsed / args.steps * 1e3
    value = step_bytes / (elapsed / args.steps) / 1e9

    # ---------------- device time per function ------------------------------
    per_op = []
    selected = configs if not args.no_per_op else [configs[1]]
    for config, op_name, op_dtype, op_case in selected:
        w = workload if (op_name, op_dtype) == (op, dtype) else DeviceWorkload(op_name, op_case, device)
        for kind, function in (("forward", w.forward), ("vjp", w.vjp)):
            calls = min(w.n_sets, 64)
            seconds, captured = device_time_per_call(function, calls, 20, device)
            abytes = algorithmic_bytes(op_name, op_case, kind)
            entry = {
                "config": config,
                "op": op_name,
                "dtype": np.dtype(op_dtype).name,
                "function": kind,
                "device_us": round(seconds * 1e6, 3),
                "algorithmic_bytes": abytes,
                "GBps": round(abytes / seconds / 1e9, 1),
                "hbm_frac": round(abytes / seconds / 1e9 / HBM_PEAK_GBS, 4),
                "timed": "hip-graph replay, HIP events" if captured else "eager launches, HIP events",
            }
            w.rotate = False
            warm_seconds, _ = device_time_per_call(function, calls, 20, device)
            w.rotate = True
            entry["device_us_same_buffers"] = round(warm_seconds * 1e6, 3)
            if not args.no_per_op:
                cpu_function = (
                    (lambda c=op_case, o=op_name: support.cpu_forward(oracle, o, c))
                    if kind == "forward"
                    else (lambda c=op_case, o=op_name: support.cpu_vjp(oracle, o, c))
                )
                times = cpu_time(cpu_function, 0.5, 20)
                entry["cpu_ms"] = round(float(np.median(times)) * 1e3, 3)
                entry["cpu_GBps"] = round(abytes / float(np.median(times)) / 1e9, 3)
            per_op.append(entry)
        if w is not workload:
            del w
            torch.cuda.empty_cache()

    # ---------------- roofline of the dominant kernel -----------------------
    # At this shape each call is one kernel (mops_amd/csrc/sap_mfma.hip), timed
    # with a pair of HIP events that the library hands to the launch itself
    # (hipExtLaunchKernelGGL stamps them with the begin and the end of that
    # kernel on the stream it runs on). Consecutive eager calls from Python
    # cannot be used instead: the interpreter needs longer per call than the
    # kernel runs.
    library = bind_library_to_torch_stream(device)
    kernels = {}
    for kind, function, name in (
        ("forward", workload.forward, "mops::amd::sap_mfma::(anonymous namespace)::forward_kernel<float, 2, 2>"),
        ("vjp", workload.vjp, "mops::amd::sap_mfma::(anonymous namespace)::vjp_kernel<float, 5>"),
    ):
        seconds, launches = main_kernel_time(library, function, 400)
        kernels[kind] = (seconds, launches, name)
    dominant_kind = max(kernels, key=lambda k: kernels[k][0] or 0.0)
    kernel_seconds, kernel_launches, kernel_name = kernels[dominant_kind]
    kernel_bytes = algorithmic_bytes(op, case, dominant_kind)
    if kernel_seconds is None:
        headline_entries = [e for e in per_op if e["op"] == op and e["dtype"] == np.dtype(dtype).name]
        entry = max(headline_entries, key=lambda e: e["device_us"])
        kernel_seconds = entry["device_us"] * 1e-6
    achieved = kernel_bytes / kernel_seconds / 1e9
    roofline = {
        "bound": "hbm",
        "kernel": kernel_name,
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get(dominant_kind),
        "algorithmic_bytes_per_launch": kernel_bytes,
        "avg_launch_us": round(kernel_seconds * 1e6, 3),
        "launches_timed": kernel_launches,
        "timed": "HIP events attached to the kernel launch (start/stop of that kernel on its launch stream), "
        "eager launches, rotating inputs",
        "other_kernel_us": {
            kind: None if kernels[kind][0] is None else round(kernels[kind][0] * 1e6, 3) for kind in kernels
        },
    }

    # ---------------- CPU baseline on the headline workload -----------------
    def cpu_step():
        support.cpu_forward(oracle, op, case)
        support.cpu_vjp(oracle, op, case)

    times = cpu_time(cpu_step, args.cpu_seconds, 100000)
    cpu_seconds = float(np.median(times))
    threads = int(oracle.cdll.mops_oracle_num_threads())
    cpu_baseline = {
        "value": round(step_bytes / cpu_seconds / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{len(times)} steps of the same workload (median {cpu_seconds * 1e3:.2f} ms/step) "
        f"in {sum(times):.1f} s, OpenMP threads = {threads}",
    }

    result = {
        "metric": "per-op fwd+vjp GB/s & % HBM roofline (fp32/fp64), 1 MI355X vs host CPU",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[1]: sparse_accumulation_of_products f32, A[32000,13] "
            "B[32000,7] C[900] sorted indices_output in [0,20); one step = forward + vjp(A, B); "
            f"inputs rotated over {workload.n_sets} buffer sets; timed as replays of HIP graphs of "
            f"{steps_per_graph} steps",
            "algorithmic_bytes_per_step": step_bytes,
            "value_is": "algorithmic bytes per step / wall time per step",
        },
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "per_op": per_op,
        "device": torch.cuda.get_device_name(0),
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
