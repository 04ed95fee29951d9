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

The step is timed ``--repetitions`` times (25 by default), each repetition
being exactly ``--steps`` steps between two host synchronisations;
``ms_per_step`` and ``value`` are the MEDIAN repetition, ``repetitions`` holds
the minimum, median and maximum.

``per_op`` has one entry per function: the device time of a call (every kernel
the call launches; HIP-graph replays between HIP events), the same with the
same buffers every call (``device_us_same_buffers``), two copy yardsticks timed
the same way (``copy_spans_us``: a copy kernel that reads and writes exactly
the tensors the call reads and writes; ``copy_flat_us``: one flat grid-stride
copy, 16 bytes per lane, of the same number of bytes read and written;
``copy_us`` is the smaller of the two and ``frac_of_copy`` = copy_us /
device_us), the useful floating-point operations of the call (``flops``: the
factored count, see ``useful_flops``) with ``flop_frac`` = flops / device time
/ the vector-or-matrix peak of the dtype, and the CPU oracle on the host cores.
``per_op_scaled`` is the same (without the CPU leg) at 16 to 100 times the rows
or edges of the BASELINE shapes: sizes at which a launch lasts long enough to
be bound by bandwidth or arithmetic rather than by latency.

``per_op_second_order`` times the vjp_vjp functions (HPE, SAP, OPSA) at the
BASELINE shapes; they are not part of a step.

``roofline`` is the kernel with the most time in a step; ``roofline_per_op``
lists the main kernel of every call. Their durations come from pairs of HIP
events that the library puts around that kernel on the stream it launches it on
(mops_amd_kernel_timing in include/mops/amd.h). Each entry carries both
fractions (``hbm_frac`` of 8 TB/s on the algorithmic bytes, ``flop_frac`` of
the dtype's peak on the useful flops) and ``bound`` = the ceiling that is the
nearer one for that kernel's shape (the larger of bytes / 8 TB/s and flops /
peak); ``frac`` is the fraction of THAT ceiling. ``traffic`` is read from the
rocprofv3 counter summary in profiles/ (kernels are matched by name), so it is
as fresh as that file.

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
FLOP_PEAK_TFLOPS = {"float32": 157.3, "float64": 78.6}  # MI355X, published (vector = dense matrix for these types)
ROTATE_BYTES = 320 * 1024 * 1024  # > 256 MB Infinity Cache
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "all_ops_baseline_shapes_hbm_traffic.txt")

# The kernel that does the arithmetic of each call at the BASELINE shapes, as
# rocprofv3 prints it (a prefix; {T} = float / double). Used to label the
# per-kernel figures and to find the kernel in the counter summary.
MAIN_KERNELS = {
    ("hpe", "forward"): "hpe::forward_ordered_kernel<{T}, 4>",
    ("hpe", "vjp"): "hpe::vjp_ordered_kernel<{T}, 4, true>",
    ("sap", "forward"): "sap_mfma::forward_kernel<{T}, 2, 2, false, 2>",
    ("sap", "vjp"): "sap_mfma::vjp_kernel<{T}, 5, 2>",
    ("opsa", "forward"): "opsa::forward_kernel<{T}, 2, false, true, true>",
    ("opsa", "vjp"): "opsa::edge_rows_vjp_kernel<{T}, 1, 2, false, true, false, false>",
    ("opsaw", "forward"): "opsa::forward_kernel<{T}, 2, true, true, true>",
    ("opsaw", "vjp"): "opsa::edge_rows_vjp_kernel<{T}, 1, 2, true, true, false, true>",
    ("sasaw", "forward"): {
        "float": "sasaw_segments::contract_kernel<float, 9, true, 32, false>",
        "double": "sasaw_segments::contract_kernel<double, 9, true, 64, false>",
    },
    ("sasaw", "vjp"): {
        "float": "sasaw_segments::gradients_kernel<float, 9, true, true, false, false>",
        "double": "sasaw_segments::gradients_kernel<double, 9, true, true, false, false>",
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


def useful_flops(op, case, kind):
    """Floating-point operations of one call in the cheapest formulation known (what a kernel
    must do, not what it pads to): a multiply and an add count one each.

    HPE       forward I J (K + 1); vjp I J (K^2 + 1) (every factor's partial product afresh)
    SAP       forward 3 I K; vjp 5 I K
    OPSA      forward 2 J K L; vjp 4 J K L
    OPSAW     forward E L + 2 E K L (b * w once per edge);
              vjp 4 E K L + 3 E L (t = sum_k g A once, then grad_B = t w, grad_W = t b)
    SASAW     with the table factored out of the sum over edges (per node Z = sum_e a (b w), then
              O = D Z with the N table entries): forward E (2 nA n2 L + n2 L) + 2 nodes N L;
              vjp three such contractions (grad_A, grad_B, grad_W) and two passes over the table:
              3 E 2 nA n2 L + E (4 n2 L) + 4 nodes N L
    """
    A = case["A"]
    if op == "hpe":
        I, (J, K) = A.shape[0], case["indices_A"].shape
        return I * J * (K + 1) if kind == "forward" else I * J * (K * K + 1)
    if op == "sap":
        I, K = A.shape[0], case["C"].shape[0]
        return (3 if kind == "forward" else 5) * I * K
    if op == "opsa":
        J, K, L = A.shape[0], A.shape[1], case["B"].shape[1]
        return (2 if kind == "forward" else 4) * J * K * L
    if op == "opsaw":
        E, K, L = A.shape[0], A.shape[1], case["B"].shape[1]
        return E * L + 2 * E * K * L if kind == "forward" else 4 * E * K * L + 3 * E * L
    if op == "sasaw":
        E, nA, L = A.shape[0], A.shape[1], case["B"].shape[1]
        nodes, n2 = case["W"].shape[0], case["W"].shape[1]
        N = case["C"].shape[0]
        if kind == "forward":
            return E * (2 * nA * n2 * L + n2 * L) + 2 * nodes * N * L
        return 3 * E * 2 * nA * n2 * L + E * 4 * n2 * L + 4 * nodes * N * L
    raise ValueError(op)


def ceilings(abytes, flops, dtype_name, seconds):
    """Both roofline fractions of a call or launch that took ``seconds``, and which ceiling binds."""
    peak = FLOP_PEAK_TFLOPS[dtype_name]
    hbm_seconds = abytes / (HBM_PEAK_GBS * 1e9)
    flop_seconds = flops / (peak * 1e12)
    bound = "hbm" if hbm_seconds >= flop_seconds else "mfma"
    return {
        "hbm_frac": round(hbm_seconds / seconds, 4),
        "flops": int(flops),
        "TFLOPs": round(flops / seconds / 1e12, 3),
        "flop_peak_TFLOPs": peak,
        "flop_frac": round(flop_seconds / seconds, 4),
        "bound": bound,
        "frac": round(max(hbm_seconds, flop_seconds) / seconds, 4),
    }


def build_scaled_configs():
    """16 to 100 times the rows or edges of the BASELINE shapes, same feature counts."""
    from tests import support

    return [
        ("c0x100", "hpe", np.float64, lambda: support.hpe_case(0, np.float64, I=100000)),
        ("c1x31", "sap", np.float32, lambda: support.sap_case(1, np.float32, I=1000000)),
        ("c1x31", "sap", np.float64, lambda: support.sap_case(1, np.float64, I=1000000)),
        ("c2x16", "opsa", np.float32, lambda: support.opsa_case(2, np.float32, J=1000000, n_out=33000)),
        ("c2x16", "opsa", np.float64, lambda: support.opsa_case(2, np.float64, J=1000000, n_out=33000)),
        ("c3x16", "opsaw", np.float32, lambda: support.opsaw_case(3, np.float32, E=1000000, n_nodes=33000)),
        ("c4x16", "sasaw", np.float32, lambda: support.sasaw_case(4, np.float32, E=1000000, n_nodes=33000)),
        ("c4x16", "sasaw", np.float64, lambda: support.sasaw_case(4, np.float64, E=1000000, n_nodes=33000)),
    ]


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


class Yardstick:
    """The two copy kernels of mops_amd/lib/libmops_yardstick.so (a library of the benchmark's
    own, built from mops_amd/csrc/yardstick.hip; not part of libmops.so)."""

    def __init__(self, device):
        import torch

        path = os.path.join(ROOT, "mops_amd", "lib", "libmops_yardstick.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `make -C mops_amd/csrc`")
        self.cdll = ctypes.CDLL(path)
        self.cdll.mops_yardstick_copy_spans.argtypes = [
            ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p,
        ]  # fmt: skip
        self.cdll.mops_yardstick_copy_flat.argtypes = [
            ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
        ]  # fmt: skip
        self.device = device
        self.torch = torch
        self.pool = None
        self.cursor = 0

    def _stream(self):
        return ctypes.c_void_p(self.torch.cuda.current_stream(self.device).cuda_stream)

    def spans(self, reads, writes):
        status = self.cdll.mops_yardstick_copy_spans(reads, len(reads), writes, len(writes), self._stream())
        if status != 0:
            raise RuntimeError(f"mops_yardstick_copy_spans: HIP error {status}")

    def flat(self, read_bytes, write_bytes):
        """One flat copy that reads ``read_bytes`` and writes ``write_bytes`` (rounded up to 16),
        at a place of a pool of more than 320 MB that moves on with every call."""
        read_bytes = (read_bytes + 15) // 16 * 16
        write_bytes = (write_bytes + 15) // 16 * 16
        both = (read_bytes + write_bytes + 255) // 256 * 256
        need = max(2 * ROTATE_BYTES, 2 * both)
        if self.pool is None or self.pool.numel() < need:
            self.pool = None
            self.torch.cuda.empty_cache()
            self.pool = self.torch.zeros(need, dtype=self.torch.uint8, device=self.device)
            self.cursor = 0
        if self.cursor + both > self.pool.numel():
            self.cursor = 0
        base = self.pool.data_ptr() + self.cursor
        self.cursor += both
        status = self.cdll.mops_yardstick_copy_flat(
            ctypes.c_void_p(base), read_bytes, ctypes.c_void_p(base + read_bytes), write_bytes, self._stream()
        )
        if status != 0:
            raise RuntimeError(f"mops_yardstick_copy_flat: HIP error {status}")


class DeviceWorkload:
    """One operation with its inputs replicated over enough buffer sets to defeat the caches."""

    yardstick = None  # a Yardstick, set by main()

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

    # the copy yardsticks: on the tensors the call reads and writes, and flat
    def _names(self, kind):
        if kind == "forward":
            return list(self.spec.inputs), ["output"]
        return ["grad_output", *self.spec.inputs], ["grad_" + n for n in self.spec.differentiable]

    def _copy(self, kind):
        t = self._next()
        read_names, write_names = self._names(kind)
        reads = (Span * len(read_names))(*[Span(t[n].data_ptr(), t[n].numel() * t[n].element_size()) for n in read_names])
        writes = (Span * len(write_names))(
            *[Span(t[n].data_ptr(), t[n].numel() * t[n].element_size()) for n in write_names]
        )
        self.yardstick.spans(reads, writes)

    def _flat(self, kind):
        t = self.sets[0]
        read_names, write_names = self._names(kind)
        self.yardstick.flat(
            sum(t[n].numel() * t[n].element_size() for n in read_names),
            sum(t[n].numel() * t[n].element_size() for n in write_names),
        )

    def copy_forward(self):
        self._copy("forward")

    def copy_vjp(self):
        self._copy("vjp")

    def flat_forward(self):
        self._flat("forward")

    def flat_vjp(self):
        self._flat("vjp")


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
    parser.add_argument(
        "--profile-scaled", action="store_true",
        help="with --profile: the scaled shapes (per_op_scaled) instead of the BASELINE ones, 10 eager forward+vjp "
        "calls each, every call followed by the flat copy of the same number of bytes",
    )  # fmt: skip
    parser.add_argument("--repetitions", type=int, default=25, help="how often the region of --steps steps is timed")
    parser.add_argument("--no-scaled", action="store_true", help="leave per_op_scaled out")
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
    DeviceWorkload.yardstick = Yardstick(device)
    oracle = support.oracle_library()
    configs = build_configs(args.extra_shapes)
    baseline = [c for c in configs if c[0].startswith("c")]

    if args.profile:
        for config, op_name, _, op_case in [] if args.profile_scaled else baseline:
            if args.profile in (op_name, "all"):
                w = DeviceWorkload(op_name, op_case, device)
                for _ in range(50):
                    w.forward()
                    w.copy_forward()
                    w.flat_forward()
                    w.vjp()
                    w.copy_vjp()
                    w.flat_vjp()
                torch.cuda.synchronize()
                del w
                torch.cuda.empty_cache()
        if args.profile_scaled:
            for config, op_name, _, make_case in build_scaled_configs():
                if args.profile in (op_name, "all"):
                    w = DeviceWorkload(op_name, make_case(), device)
                    for _ in range(10):
                        w.forward()
                        w.flat_forward()
                        w.vjp()
                        w.flat_vjp()
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
    region_seconds = []
    for _ in range(max(1, args.repetitions)):
        torch.cuda.synchronize()
        begin = time.perf_counter()
        if graph is not None:
            for _ in range(args.steps // steps_per_graph):
                graph.replay()
        else:
            for _ in range(args.steps):
                step()
        torch.cuda.synchronize()
        region_seconds.append(time.perf_counter() - begin)
    seconds_per_step = float(np.median(region_seconds)) / args.steps
    value = step_bytes / seconds_per_step / 1e9
    step_flops = {"float32": 0, "float64": 0}
    for (_, _, dtype_name), w in workloads.items():
        step_flops[dtype_name] += useful_flops(w.op, w.case, "forward") + useful_flops(w.op, w.case, "vjp")

    # ---------------- per function: call, copy yardsticks, main kernel, CPU ------------------
    def measure(config, op_name, op_dtype, op_case, w, kind, with_cpu):
        function = w.forward if kind == "forward" else w.vjp
        copy = w.copy_forward if kind == "forward" else w.copy_vjp
        flat = w.flat_forward if kind == "forward" else w.flat_vjp
        dtype_name = np.dtype(op_dtype).name
        calls = min(w.n_sets, 64)
        seconds, captured = device_time_per_call(function, calls, 20, device)
        spans_seconds, _ = device_time_per_call(copy, calls, 20, device)
        flat_seconds, _ = device_time_per_call(flat, calls, 20, device)
        copy_seconds = min(spans_seconds, flat_seconds)
        abytes = algorithmic_bytes(op_name, op_case, kind)
        flops = useful_flops(op_name, op_case, kind)
        entry = {
            "config": config,
            "op": op_name,
            "dtype": dtype_name,
            "function": kind,
            "device_us": round(seconds * 1e6, 3),
            "algorithmic_bytes": abytes,
            "GBps": round(abytes / seconds / 1e9, 1),
            **ceilings(abytes, flops, dtype_name, seconds),
            "copy_us": round(copy_seconds * 1e6, 3),
            "copy_spans_us": round(spans_seconds * 1e6, 3),
            "copy_flat_us": round(flat_seconds * 1e6, 3),
            "frac_of_copy": round(copy_seconds / seconds, 3),
            "timed": "hip-graph replay, HIP events" if captured else "eager launches, HIP events",
        }
        w.rotate = False
        warm_seconds, _ = device_time_per_call(function, calls, 20, device)
        w.rotate = True
        entry["device_us_same_buffers"] = round(warm_seconds * 1e6, 3)
        if with_cpu:
            cpu_function = (
                (lambda c=op_case, o=op_name: support.cpu_forward(oracle, o, c))
                if kind == "forward"
                else (lambda c=op_case, o=op_name: support.cpu_vjp(oracle, o, c))
            )
            times = cpu_time(cpu_function, 0.4, 20)
            entry["cpu_ms"] = round(float(np.median(times)) * 1e3, 3)
            entry["cpu_GBps"] = round(abytes / float(np.median(times)) / 1e9, 3)
        return entry, seconds, calls

    per_op = []
    roofline_per_op = []
    selected = [] if args.no_per_op else configs
    for config, op_name, op_dtype, op_case in selected:
        key = (config, op_name, np.dtype(op_dtype).name)
        w = workloads.get(key) or DeviceWorkload(op_name, op_case, device)
        type_name = "float" if op_dtype == np.float32 else "double"
        for kind in ("forward", "vjp"):
            entry, seconds, calls = measure(config, op_name, op_dtype, op_case, w, kind, True)
            per_op.append(entry)
            function = w.forward if kind == "forward" else w.vjp
            abytes = entry["algorithmic_bytes"]

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
                        **ceilings(abytes, entry["flops"], np.dtype(op_dtype).name, kernel_seconds),
                        "traffic": measured_traffic(name),
                        "timed": timed_by,
                    }
                )
        if key not in workloads:
            del w
            torch.cuda.empty_cache()

    # ---------------- the same at sizes that can reach a ceiling -------------------------------
    per_op_scaled = []
    if not (args.no_per_op or args.no_scaled):
        for config, op_name, op_dtype, make_case in build_scaled_configs():
            op_case = make_case()
            w = DeviceWorkload(op_name, op_case, device)
            for kind in ("forward", "vjp"):
                entry, _, _ = measure(config, op_name, op_dtype, op_case, w, kind, False)
                entry["shape"] = {name: list(np.shape(op_case[name])) for name in w.spec.inputs}
                per_op_scaled.append(entry)
            del w, op_case
            torch.cuda.empty_cache()

    # ---------------- second-order functions (not part of the step) ----------------
    per_op_second_order = []
    if not args.no_per_op:
        for config, op_name, op_dtype, op_case in baseline:
            if op_name not in support.SECOND_ORDER:
                continue
            case = support.add_cotangents(dict(op_case), op_name)
            on_device = support.to_device(case, device)
            spec = support.OPS[op_name]
            outputs, arguments = support._vjp_vjp_arguments(
                spec, on_device, None, None, lambda x: torch.empty_like(x)
            )

            def second_order(arguments=arguments, spec=spec):
                library.call(spec.function + "_vjp_vjp", *arguments)

            # (at these shapes the functions take no temporary, so they can be captured like the
            # first-order calls; device_time_per_call falls back to eager calls where a capture fails)
            for _ in range(3):
                second_order()
            torch.cuda.synchronize()
            seconds, captured = device_time_per_call(second_order, 20, 10, device)
            per_op_second_order.append(
                {
                    "config": config,
                    "op": op_name,
                    "dtype": np.dtype(op_dtype).name,
                    "function": "vjp_vjp",
                    "device_us": round(seconds * 1e6, 3),
                    "timed": ("hip-graph replay" if captured else "eager launches") + ", HIP events, the same buffers every call",
                }
            )
            del on_device, outputs, arguments
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
            **ceilings(abytes, useful_flops("sasaw", w.case, "vjp"), "float64", kernel_seconds),
            "traffic": measured_traffic(name),
            "timed": "HIP events around the kernel on its launch stream",
        }  # fmt: skip
    # the ceiling that binds this kernel's shape: bytes / 8 TB/s against useful flops / peak
    if dominant["bound"] == "hbm":
        achieved, peak, unit = dominant["achieved_GBps"], HBM_PEAK_GBS, "GB/s"
    else:
        achieved, peak, unit = dominant["TFLOPs"], dominant["flop_peak_TFLOPs"], "TFLOP/s"
    roofline = {
        "bound": dominant["bound"],
        "kernel": dominant["kernel"],
        "of": f"{dominant['config']} {dominant['op']} {dominant['dtype']} {dominant['function']}",
        "achieved": achieved,
        "peak": peak,
        "unit": unit,
        "frac": dominant["frac"],
        "hbm": {"achieved": dominant["achieved_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dominant["hbm_frac"]},
        "flop": {
            "achieved": dominant["TFLOPs"], "peak": dominant["flop_peak_TFLOPs"], "unit": "TFLOP/s",
            "frac": dominant["flop_frac"], "useful_flops_per_launch": dominant["flops"],
        },  # fmt: skip
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
        "repetitions": {
            "count": len(region_seconds),
            "each": f"{args.steps} steps between two host synchronisations",
            "ms_per_step_min": round(min(region_seconds) / args.steps * 1e3, 5),
            "ms_per_step_median": round(float(np.median(region_seconds)) / args.steps * 1e3, 5),
            "ms_per_step_max": round(max(region_seconds) / args.steps * 1e3, 5),
        },
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
            "value_is": "algorithmic bytes per step / wall time per step (median repetition)",
            "useful_flops_per_step": step_flops,
            "step_flop_frac": round(
                sum(step_flops[d] / (FLOP_PEAK_TFLOPS[d] * 1e12) for d in step_flops) / seconds_per_step, 4
            ),
        },
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
        "roofline_per_op": roofline_per_op,
        "per_op": per_op,
        "per_op_scaled": per_op_scaled,
        "per_op_second_order": per_op_second_order,
        "device": torch.cuda.get_device_name(0),
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
