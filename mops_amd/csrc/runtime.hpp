// Host-side plumbing shared by every device operation: HIP error handling,
// the per-thread stream / synchronisation settings, launch helpers and the
// scratch-memory cache.
#ifndef MOPS_AMD_RUNTIME_HPP
#define MOPS_AMD_RUNTIME_HPP

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>

#include <hip/hip_runtime.h>

namespace mops::amd {

/// Throw std::runtime_error naming `what` when `status` is not hipSuccess.
/// (The reference prints and calls exit() on a device error,
/// mops/src/internal/cuda_utils.cuh:11-24; throwing lets the C ABI report
/// status 1 instead of killing the caller's process.)
void check_hip(hipError_t status, const char* what);

#define MOPS_HIP_CHECK(expression) ::mops::amd::check_hip((expression), #expression)

/// Stream that device work of the calling thread is enqueued on.
hipStream_t current_stream();
void set_current_stream(hipStream_t stream);

/// Whether device entry points wait for their kernels before returning.
bool synchronous();
bool set_synchronous(bool value);

/// Check the launch that was just issued, then wait for the stream if the
/// calling thread is in synchronous mode. Called once at the end of every
/// device entry point.
void finish_call(const char* operation);

/// Scratch device memory of at least `bytes` bytes, 256-byte aligned, valid
/// until the next call of this function on the same thread. The block is
/// cached per thread and grows on demand (growing frees the old block, which
/// waits for the device; a block that was handed out while a stream was being
/// captured is kept until the process ends instead, because the graph names
/// it). Growing while the thread's stream is being captured throws. When the
/// calling thread switches to another stream, the new stream waits on the
/// device for the previous call that used the block, so two streams never
/// share the block at the same time. A thread that ends leaves its block to
/// the next new thread.
void* scratch(size_t bytes);
/// Bytes of the calling thread's scratch block (0: none yet).
size_t scratch_capacity();

/// Counters that come with the scratch block: SCRATCH_COUNTERS integers of 32
/// bits in front of the memory scratch() returned (call it first, in the same
/// call of the library). They are zero when the block is made, and every kernel
/// that counts in them sets what it has used back to zero before it ends, so
/// that the next launch finds zeros without a launch that clears them (also
/// the next replay of a graph the launches were captured into).
/// A call that fails between a launch that counts and the launch that reads
/// and clears would leave counts behind for the next call. The host keeps a
/// mark per block for that: a call takes the counters by holding a
/// ScratchCounters for as long as it enqueues work; the mark is set from the
/// object's construction until its destruction in the ordinary way, and stays
/// when the object is destroyed by an exception on its way out of the call.
/// scratch() clears the counters with a launch of its own when it finds the
/// mark. A graph that was captured earlier does not pass through scratch():
/// after a failed call, make one eager call that succeeds
/// (mops_amd_reserve_scratch(0) will do) before replaying it.
constexpr size_t SCRATCH_COUNTERS = size_t(1) << 18;
class ScratchCounters {
public:
    ScratchCounters();
    ~ScratchCounters();
    ScratchCounters(const ScratchCounters&) = delete;
    ScratchCounters& operator=(const ScratchCounters&) = delete;
    int32_t* data() const;

private:
    void* resources_ = nullptr;
    int exceptions_;
    bool capturing_ = false;
    bool before_ = false;
};

/// Throws when the environment variable MOPS_AMD_TEST_FAIL_AT names `name`:
/// lets a test make a call fail on the host between two of its launches (every
/// kernel that was enqueued still runs to its end).
void test_failure_point(const char* name);

/// A second stream of the calling thread, for a kernel of a call that does not
/// depend on the call's other kernels and leaves room on the device beside
/// them. Construction makes the side stream wait for everything enqueued on
/// `main` so far; destruction makes `main` wait for everything enqueued on the
/// side stream, so that for the caller the call still happens on `main` alone
/// (also when `main` is being captured into a graph: the side stream joins the
/// capture and leaves it again). Default stream priority.
class SideStream {
public:
    explicit SideStream(hipStream_t main);
    ~SideStream();
    SideStream(const SideStream&) = delete;
    SideStream& operator=(const SideStream&) = delete;
    hipStream_t get() const { return side_; }

private:
    hipStream_t main_;
    hipStream_t side_ = nullptr;
    hipEvent_t joined_ = nullptr;
};

/// Device time of an operation's main kernel, for benchmarks that want the
/// duration of one kernel and not of the whole call. While a thread has
/// kernel timing on (set_kernel_timing), every MainKernelTimer in scope of a
/// launch records a pair of HIP events around it on the stream it is launched
/// on; collect_kernel_time waits for them and adds the intervals up. Streams
/// that are being captured into a graph are left alone.
class MainKernelTimer {
public:
    explicit MainKernelTimer(hipStream_t stream);
    ~MainKernelTimer();
    MainKernelTimer(const MainKernelTimer&) = delete;
    MainKernelTimer& operator=(const MainKernelTimer&) = delete;

private:
    hipStream_t stream_;
    hipEvent_t stop_ = nullptr;
};
/// The same for a launch through hipExtLaunchKernelGGL, which takes the two
/// events itself and has them stamped with the begin and the end of that
/// kernel: no event packets of their own in the stream, so the interval is the
/// kernel's duration as a profiler reports it. Both are null when timing is off
/// or the stream is being captured.
struct LaunchEvents {
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};
LaunchEvents launch_events(hipStream_t stream);
bool set_kernel_timing(bool value);
/// Sum (milliseconds) and number of the intervals recorded since the last
/// call on this thread.
void collect_kernel_time(double* milliseconds, int64_t* launches);

/// Compute units of the current device (asked for once per device).
int32_t compute_units();

/// ceil(a / b) for positive b.
inline size_t ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

/// Round `bytes` up to a multiple of 256 so that consecutive carve-outs of
/// one scratch block keep every sub-buffer aligned for 128-bit accesses.
inline size_t align256(size_t bytes) { return (bytes + 255) & ~static_cast<size_t>(255); }

/// Convert a size to the 32-bit signed range the kernels index with.
int32_t narrow_i32(size_t value, const char* what);

/// True when the environment asks for index validation on the device path
/// (MOPS_AMD_CHECK_INDICES=1): index tensors are then copied to the host and
/// checked for range (and the scatter index for sortedness) on every call.
bool validate_device_indices();

} // namespace mops::amd

#endif
