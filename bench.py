"""Benchmark of the mops device path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--extra-shapes] [--no-per-op]

Prints ONE JSON line. One "step" is the forward pass followed by the vjp of
ALL eight operation x dtype combinations of the BASELINE configurations
(configs[0] HPE f64; configs[1] SAP f32, f64; configs[2] OPSA f32, f64;
configs[3] OPSAW f32; configs[4] SASAW f32, f64): sixteen calls. ``value`` is
the algorithmic bytes of a step (every input read once, every output written
once, index tensors included) divided by the wall time per step, inputs
resident in HBM and rotated over buffer sets of more than 256 MB per operation
so that the Infinity Cache cannot serve them. The timed region is an integer
number of replays of one HIP graph that holds a divisor of K steps, so the
figure does not depend on K.

``per_op`` has one entry per function: the device time of a call (every kernel
the call launches; HIP-graph replays between HIP events), the same with the
same buffers every call (``device_us_same_buffers``), the time a plain copy
kernel takes to read and write exactly the tensors the call reads and writes
(``copy_us``: the yardstick; ``frac_of_copy`` = copy_us / device_us), and the
CPU oracle on the host cores. ``roofline`` is the kernel with the most time in
a step; ``roofline_per_op`` lists the main kernel of every call. Their
durations come from pairs of HIP events that the library puts around that
kernel on the stream it launches it on (mops_amd_kernel_timing in
include/mops/amd.h); ``traffic`` is read from the rocprofv3 counter summary in
profiles/ (kernels are matched by name).

``cpu_baseline`` times the CPU oracle (a port of the reference's OpenMP
algorithm, oracle/oracle.cpp) on the same step on this machine's host cores,
with all threads and with one.
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X, published
ROTATE_BYTES = 320 * 1024 * 1024  # > 256 MB Infinity Cache
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "all_ops_baseline_shapes_hbm_traffic.txt")

# The kernel that does the arithmetic of each call at the BASELINE shapes, as
# rocprofv3 prints it (a prefix; {T} = float / double). Used to label the
# per-kernel figures and to find the kernel in the counter summary.
MAIN_KERNELS = {
    ("hpe", "forward"): "forward_ordered_kernel<{T}, 4>",
    ("hpe", "vjp"): "vjp_ordered_kernel<{T}, 4, true>",
    ("sap", "forward"): "sap_mfma::forward_kernel<{T}, 2, 2>",
    ("sap", "vjp"): "sap_mfma::vjp_kernel<{T}, 5>",
    ("opsa", "forward"): "forward_kernel<{T}, 2, false, true>",
    ("opsa", "vjp"): "edge_rows_vjp_kernel<{T}, 1, 2, false, true, false, false>",
    ("opsaw", "forward"): "forward_kernel<{T}, 2, true, true>",
    ("opsaw", "vjp"): "edge_rows_vjp_kernel<{T}, 1, 2, true, true, false, true>",
    ("sasaw", "forward"): {
        "float": "sasaw_segments::contract_kernel<float, 9, true, 32>",
        "double": "sasaw_segments::contract_kernel<double, 9, true, 64>",
    },
    ("sasaw", "vjp"): {
        "float": "sasaw_segments::gradients_kernel<float, 9, true, true, false>",
        "double": "sasaw_segments::gradients_kernel<double, 9, true, true, false>",
    },
}


def main_kernel_name(op, kind, type_name):
    """Name of the main kernel of ``op``'s ``kind`` call for elements of C++ type ``type_name``."""
    entry = MAIN_KERNELS.get((op, kind), "?")
    if isinstance(entry, dict):
        return entry[type_name]
    return entry.format(T=type_name)


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


def build_configs(extra):
    from tests import support

    configs = [
        ("c0", "hpe", np.float64, support.hpe_case(0, np.float64)),
        ("c1", "sap", np.float32, support.sap_case(1, np.float32)),
        ("c1", "sap", np.float64, support.sap_case(1, np.float64)),
        ("c2", "opsa", np.float32, support.opsa_case(2, np.float32)),
        ("c2", "opsa", np.float64, support.opsa_case(2, np.float64)),
        ("c3", "opsaw", np.float32, support.opsaw_case(3, np.float32)),
        ("c4", "sasaw", np.float32, support.sasaw_case(4, np.float32)),
        ("c4", "sasaw", np.float64, support.sasaw_case(4, np.float64)),
    ]
    if extra:
        configs += [
            # beyond the BASELINE shapes: feature counts that fill whole 16-wide matrix tiles
            ("wide", "opsa", np.float32, support.opsa_case(5, np.float32, K=32, L=64)),
            ("wide", "opsaw", np.float32, support.opsaw_case(6, np.float32, K=32, L=64)),
            # many rows: HPE with a lane per row (forward) and by feature (vjp)
            ("many_rows", "hpe", np.float64, support.hpe_case(10, np.float64, I=20000, nA=50, J=4000, K=3)),
            # 128 feature channels
            ("wide128", "opsa", np.float32, support.opsa_case(7, np.float32, K=16, L=128)),
            ("wide128", "opsaw", np.float32, support.opsaw_case(8, np.float32, K=16, L=128)),
            ("wide128", "sasaw", np.float32, support.sasaw_case(9, np.float32, L=128)),
        ]
    return configs


class Span(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("bytes", ctypes.c_int64)]


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

    # the copy yardstick on the tensors the call reads and writes
    def _copy(self, read_names, write_names):
        t = self._next()
        reads = (Span * len(read_names))(*[Span(t[n].data_ptr(), t[n].numel() * t[n].element_size()) for n in read_names])
        writes = (Span * len(write_names))(
            *[Span(t[n].data_ptr(), t[n].numel() * t[n].element_size()) for n in write_names]
        )
        status = self.library.cdll.mops_amd_copy_yardstick(reads, len(read_names), writes, len(write_names))
        if status != 0:
            raise RuntimeError(self.library.last_error())

    def copy_forward(self):
        self._copy(list(self.spec.inputs), ["output"])

    def copy_vjp(self):
        self._copy(["grad_output", *self.spec.inputs], ["grad_" + n for n in self.spec.differentiable])


def bind_library_to_torch_stream(device):
    import torch

    from mops_amd._c_lib import device_library

    library = device_library()
    torch.cuda.set_device(device)
    library.cdll.mops_amd_set_stream(ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream))
    library.cdll.mops_amd_set_synchronous(0)
    return library


def capture(function, calls, device):
    """A HIP graph of ``calls`` consecutive calls of ``function`` (None if the capture fails)."""
    import torch

    for _ in range(3):
        function()  # warm up: the library's scratch block takes its size outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream(device=device)
    stream.wait_stream(torch.cuda.current_stream(device))
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
        sys.stderr.write(f"graph capture failed ({error}); timing eager launches instead\n")
        graph = None
    bind_library_to_torch_stream(device)
    torch.cuda.synchronize()
    return graph


def device_time_per_call(function, calls, replays, device):
    """Average device time (seconds) of one call of ``function``: replays of a graph of ``calls``
    calls between two HIP events on the stream the replays are launched on."""
    import torch

    graph = capture(function, calls, device)
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    if graph is not None:
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
    return start.elapsed_time(stop) * 1e-3 / (replays * calls), graph is not None


def main_kernel_time(library, function, calls):
    """Average duration (seconds) of the main kernel of ``function`` over ``calls`` eager calls,
    from the pairs of HIP events the library records around it on its launch stream."""
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
    times = []
    begin = time.perf_counter()
    while len(times) < max_calls and (time.perf_counter() - begin < seconds or len(times) < 2):
        t0 = time.perf_counter()
        function()
        times.append(time.perf_counter() - t0)
    return times


def cpu_model():
    try:
        with open("/proc/cpuinfo") as handle:
            for line in handle:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def measured_traffic(kernel_prefix):
    """HBM bytes per launch of the kernel whose name starts with ``kernel_prefix``, from the
    rocprofv3 counter summary under profiles/ (last column of its table: total MB), or None."""
    try:
        with open(TRAFFIC_FILE) as handle:
            lines = handle.read().split("\n")
    except OSError:
        return None
    # (the summary cuts long names: compare without the closing bracket of the template list)
    prefix = kernel_prefix[:95].rstrip(">")
    for line in lines:
        if line.startswith(prefix):
            columns = re.findall(r"[-+]?\d+\.\d+", line[len(prefix):])
            if len(columns) >= 5:
                return int(round(float(columns[-1]) * 1e6))
    return None


def largest_divisor(n, limit):
    for candidate in range(min(n, limit), 0, -1):
        if n % candidate == 0:
            return candidate
    return 1


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=200)
    parser.add_argument("--warmup", type=int, default=20)
    parser.add_argument("--cpu-seconds", type=float, default=10.0)
    parser.add_argument("--no-per-op", action="store_true", help="only the headline step")
    parser.add_argument("--extra-shapes", action="store_true", help="per_op also for shapes beyond the BASELINE ones")
    parser.add_argument(
        "--profile",
        choices=["hpe", "sap", "opsa", "opsaw", "sasaw", "all"],
        help="for rocprofv3: run 50 eager forward+vjp calls of the operation(s) at the BASELINE "
        "shapes (all their dtypes), each followed by the copy yardstick on the same tensors, and 20 element-wise "
        "passes over 64 MiB (read 64 MiB, write 64 MiB) as a yardstick for the HBM counters, print nothing, exit",
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
    library = bind_library_to_torch_stream(device)
    library.cdll.mops_amd_copy_yardstick.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32]
    oracle = support.oracle_library()
    configs = build_configs(args.extra_shapes)
    baseline = [c for c in configs if c[0].startswith("c")]

    if args.profile:
        for config, op_name, _, op_case in baseline:
            if args.profile in (op_name, "all"):
                w = DeviceWorkload(op_name, op_case, device)
                for _ in range(50):
                    w.forward()
                    w.copy_forward()
                    w.vjp()
                    w.copy_vjp()
                torch.cuda.synchronize()
                del w
                torch.cuda.empty_cache()
        source = torch.empty(64 * 1024 * 1024 // 4, dtype=torch.float32, device=device).normal_()
        target = torch.empty_like(source)
        for _ in range(20):
            torch.mul(source, 2.0, out=target)  # reads 64 MiB, writes 64 MiB
        torch.cuda.synchronize()
        return

    # ---------------- headline: one step = forward + vjp of all eight combinations ----------
    workloads = {}
    for config, op_name, op_dtype, op_case in baseline:
        workloads[(config, op_name, np.dtype(op_dtype).name)] = DeviceWorkload(op_name, op_case, device)
    step_bytes = sum(
        algorithmic_bytes(w.op, w.case, "forward") + algorithmic_bytes(w.op, w.case, "vjp") for w in workloads.values()
    )

    def step():
        for w in workloads.values():
            w.step()

    steps_per_graph = largest_divisor(args.steps, 8)
    graph = capture(step, steps_per_graph, device)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    begin = time.perf_counter()
    if graph is not None:
        for _ in range(args.steps // steps_per_graph):
            graph.replay()
    else:
        for _ in range(args.steps):
            step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - begin
    seconds_per_step = elapsed / args.steps
    value = step_bytes / seconds_per_step / 1e9

    # ---------------- per function: call, copy yardstick, main kernel, CPU ------------------
    per_op = []
    roofline_per_op = []
    selected = [] if args.no_per_op else configs
    for config, op_name, op_dtype, op_case in selected:
        key = (config, op_name, np.dtype(op_dtype).name)
        w = workloads.get(key) or DeviceWorkload(op_name, op_case, device)
        type_name = "float" if op_dtype == np.float32 else "double"
        for kind, function, copy in (("forward", w.forward, w.copy_forward), ("vjp", w.vjp, w.copy_vjp)):
            calls = min(w.n_sets, 64)
            seconds, captured = device_time_per_call(function, calls, 20, device)
            copy_seconds, _ = device_time_per_call(copy, calls, 20, device)
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
                "copy_us": round(copy_seconds * 1e6, 3),
                "frac_of_copy": round(copy_seconds / seconds, 3),
                "timed": "hip-graph replay, HIP events" if captured else "eager launches, HIP events",
            }
            w.rotate = False
            warm_seconds, _ = device_time_per_call(function, calls, 20, device)
            w.rotate = True
            entry["device_us_same_buffers"] = round(warm_seconds * 1e6, 3)
            cpu_function = (
                (lambda c=op_case, o=op_name: support.cpu_forward(oracle, o, c))
                if kind == "forward"
                else (lambda c=op_case, o=op_name: support.cpu_vjp(oracle, o, c))
            )
            times = cpu_time(cpu_function, 0.4, 20)
            entry["cpu_ms"] = round(float(np.median(times)) * 1e3, 3)
            entry["cpu_GBps"] = round(abytes / float(np.median(times)) / 1e9, 3)
            per_op.append(entry)

            if config.startswith("c"):
                kernel_seconds, launches = main_kernel_time(library, function, 200)
                name = main_kernel_name(op_name, kind, type_name)
                timed_by = "HIP events around the kernel on its launch stream, eager calls, rotating inputs"
                if kernel_seconds is None:
                    # this call's kernels carry no events: the whole call as one interval
                    kernel_seconds, launches = seconds, calls * 20
                    timed_by = "whole call (all its kernels) as HIP-graph replays between HIP events"
                roofline_per_op.append(
                    {
                        "config": config,
                        "op": op_name,
                        "dtype": np.dtype(op_dtype).name,
                        "function": kind,
                        "kernel": name,
                        "avg_us": round(kernel_seconds * 1e6, 3),
                        "launches_timed": launches,
                        "algorithmic_bytes_per_launch": abytes,
                        "achieved_GBps": round(abytes / kernel_seconds / 1e9, 1),
                        "frac": round(abytes / kernel_seconds / 1e9 / HBM_PEAK_GBS, 4),
                        "traffic": measured_traffic(name),
                        "timed": timed_by,
                    }
                )
        if key not in workloads:
            del w
            torch.cuda.empty_cache()

    # ---------------- roofline of the kernel with the most time in a step -------------------
    if roofline_per_op:
        dominant = max(roofline_per_op, key=lambda e: e["avg_us"])
    else:
        # --no-per-op: only the kernel that dominated the last full run is timed
        w = workloads[("c4", "sasaw", "float64")]
        kernel_seconds, launches = main_kernel_time(library, w.vjp, 200)
        abytes = algorithmic_bytes("sasaw", w.case, "vjp")
        if kernel_seconds is None:
            kernel_seconds, _ = device_time_per_call(w.vjp, w.n_sets, 20, device)
            launches = w.n_sets * 20
        name = main_kernel_name("sasaw", "vjp", "double")
        dominant = {
            "config": "c4", "op": "sasaw", "dtype": "float64", "function": "vjp", "kernel": name,
            "avg_us": round(kernel_seconds * 1e6, 3), "launches_timed": launches,
            "algorithmic_bytes_per_launch": abytes, "achieved_GBps": round(abytes / kernel_seconds / 1e9, 1),
            "frac": round(abytes / kernel_seconds / 1e9 / HBM_PEAK_GBS, 4), "traffic": measured_traffic(name),
            "timed": "HIP events around the kernel on its launch stream",
        }  # fmt: skip
    roofline = {
        "bound": "hbm",
        "kernel": dominant["kernel"],
        "of": f"{dominant['config']} {dominant['op']} {dominant['dtype']} {dominant['function']}",
        "achieved": dominant["achieved_GBps"],
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": dominant["frac"],
        "traffic": dominant["traffic"],
        "traffic_from": os.path.relpath(TRAFFIC_FILE, ROOT),
        "algorithmic_bytes_per_launch": dominant["algorithmic_bytes_per_launch"],
        "avg_launch_us": dominant["avg_us"],
        "launches_timed": dominant["launches_timed"],
        "timed": dominant["timed"],
    }

    # ---------------- CPU baseline on the same step ------------------------------------------
    def cpu_step():
        for w in workloads.values():
            support.cpu_forward(oracle, w.op, w.case)
            support.cpu_vjp(oracle, w.op, w.case)

    threads = int(oracle.cdll.mops_oracle_num_threads())
    times = cpu_time(cpu_step, args.cpu_seconds, 100000)
    cpu_seconds = float(np.median(times))
    oracle.cdll.mops_oracle_set_num_threads(1)
    single = cpu_time(cpu_step, args.cpu_seconds, 100000)
    oracle.cdll.mops_oracle_set_num_threads(threads)
    single_seconds = float(np.median(single))
    cpu_baseline = {
        "value": round(step_bytes / cpu_seconds / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "cpu_model": cpu_model(),
        "sample": f"{len(times)} steps of the same workload (all eight combinations, forward + vjp; median "
        f"{cpu_seconds * 1e3:.1f} ms/step) in {sum(times):.1f} s, OpenMP threads = {threads}",
        "one_thread": {
            "value": round(step_bytes / single_seconds / 1e9, 3),
            "unit": "GB/s",
            "cores": 1,
            "sample": f"{len(single)} steps (median {single_seconds * 1e3:.1f} ms/step) in {sum(single):.1f} s",
        },
    }

    result = {
        "metric": "per-op fwd+vjp GB/s & % HBM roofline (fp32/fp64), 1 MI355X vs host CPU",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(seconds_per_step * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32+f64",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[0..4], every operation x dtype they name: HPE f64 (c0), SAP f32 + f64 (c1), "
            "OPSA f32 + f64 (c2), OPSAW f32 (c3), SASAW f32 + f64 (c4); one step = forward + vjp of all eight "
            f"(sixteen calls); inputs rotated over > 320 MB of buffer sets per operation; timed as "
            f"{args.steps // steps_per_graph} replays of one HIP graph of {steps_per_graph} steps",
            "algorithmic_bytes_per_step": step_bytes,
            "value_is": "algorithmic bytes per step / wall time per step",
        },
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "roofline_per_op": roofline_per_op,
        "per_op": per_op,
        "device": torch.cuda.get_device_name(0),
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
