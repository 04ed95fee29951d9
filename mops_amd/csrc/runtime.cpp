#include "runtime.hpp"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <exception>
#include <limits>
#include <mutex>
#include <utility>
#include <vector>

namespace mops::amd {

// (sender_buckets.hip: a launch that sets `count` integers to zero; usable while a stream is captured)
void clear_counters(int32_t* counters, size_t count, hipStream_t stream);

void check_hip(hipError_t status, const char* what) {
    if (status != hipSuccess) {
        throw std::runtime_error(
            std::string("HIP error in ") + what + ": " + hipGetErrorString(status)
        );
    }
}

namespace {

// Device objects of one calling thread. They outlive the thread: when it ends
// they go to a process-wide pool (no HIP call is made from a thread's exit
// path, where the HIP runtime may already be gone) and the next new thread
// takes them over, so short-lived worker threads do not leak device memory.
struct Resources {
    // scratch cache
    void* block = nullptr;
    size_t capacity = 0;
    int device = -1;
    hipStream_t block_stream = nullptr; // stream of the block's latest user
    bool block_in_graph = false;        // handed out while a stream was being captured
    hipEvent_t last_use = nullptr;      // recorded behind the latest eager call that used the block
    bool last_use_recorded = false;
    // The counters in front of the block were handed to a call that has not reached its end
    // (finish_call) yet. Found set at the start of the next call, it means that a call failed
    // between a launch that counts and the launch that reads and clears: the counters may hold
    // anything and are cleared before they are handed out again.
    bool counters_dirty = false;
    // blocks a captured graph may still name: kept until the process ends
    std::vector<void*> retired;

    // side stream and its two events, per device
    struct Side {
        int device;
        hipStream_t stream;
        hipEvent_t forked;
        hipEvent_t joined;
    };
    std::vector<Side> sides;

    // timing events
    std::vector<hipEvent_t> spare;
};

struct Pool {
    std::mutex mutex;
    std::vector<Resources*> idle;
};

Pool& pool() {
    static Pool* instance = new Pool(); // never destroyed: threads may end after main returns
    return *instance;
}

struct ThreadState {
    hipStream_t stream = nullptr;
    bool synchronous = true;
    Resources* resources = nullptr;

    // this call
    bool used_scratch = false;
    bool capturing = false;

    // kernel timing
    bool timing = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> recorded;

    Resources& res() {
        if (resources == nullptr) {
            Pool& p = pool();
            std::lock_guard<std::mutex> lock(p.mutex);
            if (!p.idle.empty()) {
                resources = p.idle.back();
                p.idle.pop_back();
            }
        }
        if (resources == nullptr) {
            resources = new Resources();
        }
        return *resources;
    }

    ~ThreadState() {
        if (resources == nullptr) {
            return;
        }
        for (auto& pair : recorded) {
            resources->spare.push_back(pair.first);
            resources->spare.push_back(pair.second);
        }
        Pool& p = pool();
        std::lock_guard<std::mutex> lock(p.mutex);
        p.idle.push_back(resources);
    }
};

hipEvent_t take_event(ThreadState& st) {
    auto& spare = st.res().spare;
    if (!spare.empty()) {
        hipEvent_t event = spare.back();
        spare.pop_back();
        return event;
    }
    hipEvent_t event = nullptr;
    MOPS_HIP_CHECK(hipEventCreate(&event));
    return event;
}

ThreadState& state() {
    static thread_local ThreadState instance;
    return instance;
}

bool is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    MOPS_HIP_CHECK(hipStreamIsCapturing(stream, &capture));
    return capture != hipStreamCaptureStatusNone;
}

} // namespace

hipStream_t current_stream() { return state().stream; }

void set_current_stream(hipStream_t stream) { state().stream = stream; }

bool synchronous() { return state().synchronous; }

bool set_synchronous(bool value) {
    bool previous = state().synchronous;
    state().synchronous = value;
    return previous;
}

namespace {
void record_last_use(Resources& res, hipStream_t stream, const char* operation) {
    if (res.last_use == nullptr) {
        check_hip(hipEventCreateWithFlags(&res.last_use, hipEventDisableTiming), operation);
    }
    check_hip(hipEventRecord(res.last_use, stream), operation);
    res.last_use_recorded = true;
}
} // namespace

void finish_call(const char* operation) {
    check_hip(hipGetLastError(), operation);
    auto& st = state();
    if (st.used_scratch) {
        // so that another stream (of this thread later, or of the thread that
        // inherits the block) can wait for this call without the host waiting
        st.used_scratch = false;
        Resources& res = st.res();
        if (!st.capturing) {
            record_last_use(res, st.stream, operation);
        }
    }
    if (st.synchronous) {
        check_hip(hipStreamSynchronize(st.stream), operation);
    }
}

SideStream::SideStream(hipStream_t main) : main_(main) {
    auto& st = state();
    int device = 0;
    MOPS_HIP_CHECK(hipGetDevice(&device));
    Resources::Side* side = nullptr;
    auto& sides = st.res().sides;
    for (auto& candidate : sides) {
        if (candidate.device == device) {
            side = &candidate;
        }
    }
    if (side == nullptr) {
        Resources::Side created{device, nullptr, nullptr, nullptr};
        MOPS_HIP_CHECK(hipStreamCreateWithFlags(&created.stream, hipStreamNonBlocking));
        MOPS_HIP_CHECK(hipEventCreateWithFlags(&created.forked, hipEventDisableTiming));
        MOPS_HIP_CHECK(hipEventCreateWithFlags(&created.joined, hipEventDisableTiming));
        sides.push_back(created);
        side = &sides.back();
    }
    side_ = side->stream;
    joined_ = side->joined;
    MOPS_HIP_CHECK(hipEventRecord(side->forked, main_));
    MOPS_HIP_CHECK(hipStreamWaitEvent(side_, side->forked, 0));
}

SideStream::~SideStream() {
    if (hipEventRecord(joined_, side_) == hipSuccess) {
        (void)hipStreamWaitEvent(main_, joined_, 0);
    }
}

MainKernelTimer::MainKernelTimer(hipStream_t stream) : stream_(stream) {
    auto& st = state();
    if (!st.timing) {
        return;
    }
    if (is_capturing(stream)) {
        return;
    }
    hipEvent_t start = take_event(st);
    stop_ = take_event(st);
    MOPS_HIP_CHECK(hipEventRecord(start, stream));
    st.recorded.emplace_back(start, stop_);
}

MainKernelTimer::~MainKernelTimer() {
    if (stop_ != nullptr) {
        (void)hipEventRecord(stop_, stream_);
    }
}

LaunchEvents launch_events(hipStream_t stream) {
    auto& st = state();
    LaunchEvents events;
    if (!st.timing) {
        return events;
    }
    if (is_capturing(stream)) {
        return events;
    }
    events.start = take_event(st);
    events.stop = take_event(st);
    st.recorded.emplace_back(events.start, events.stop);
    return events;
}

bool set_kernel_timing(bool value) {
    bool previous = state().timing;
    state().timing = value;
    return previous;
}

void collect_kernel_time(double* milliseconds, int64_t* launches) {
    auto& st = state();
    double total = 0.0;
    for (auto& pair : st.recorded) {
        MOPS_HIP_CHECK(hipEventSynchronize(pair.second));
        float elapsed = 0.0f;
        MOPS_HIP_CHECK(hipEventElapsedTime(&elapsed, pair.first, pair.second));
        total += elapsed;
        st.res().spare.push_back(pair.first);
        st.res().spare.push_back(pair.second);
    }
    *milliseconds = total;
    *launches = static_cast<int64_t>(st.recorded.size());
    st.recorded.clear();
}

void* scratch(size_t bytes) {
    auto& st = state();
    Resources& res = st.res();
    int device = 0;
    MOPS_HIP_CHECK(hipGetDevice(&device));
    // st.stream is the stream of this call: the caller named it and keeps it alive
    st.capturing = is_capturing(st.stream);

    if (res.block != nullptr && (device != res.device || bytes > res.capacity)) {
        if (st.capturing) {
            // Allocating would end the capture, and the graph would keep the
            // address of a block that the next growth frees.
            throw std::runtime_error(
                "mops: this call needs " + std::to_string(bytes) + " bytes of scratch memory but the calling "
                "thread holds " + std::to_string(res.capacity) + " and its stream is being captured into a graph; "
                "make one call with the largest shapes on this thread before capturing"
            );
        }
        if (res.block_in_graph) {
            // a captured graph may replay kernels that name this block
            res.retired.push_back(res.block);
        } else {
            // hipFree waits for the device, so nothing can still be using the block
            int restore = device;
            MOPS_HIP_CHECK(hipSetDevice(res.device));
            MOPS_HIP_CHECK(hipFree(res.block));
            MOPS_HIP_CHECK(hipSetDevice(restore));
        }
        res.block = nullptr;
        res.capacity = 0;
        res.block_in_graph = false;
        res.last_use_recorded = false;
    }

    if (res.block == nullptr) {
        if (st.capturing) {
            throw std::runtime_error(
                "mops: this call needs scratch memory and the calling thread has none yet, but its stream is being "
                "captured into a graph; make one call with the largest shapes on this thread before capturing"
            );
        }
        size_t capacity = bytes + bytes / 2;
        if (capacity < (size_t(1) << 20)) {
            capacity = size_t(1) << 20;
        }
        constexpr size_t counter_bytes = SCRATCH_COUNTERS * sizeof(int32_t);
        MOPS_HIP_CHECK(hipMalloc(&res.block, counter_bytes + capacity));
        // (not in a captured graph: a stream that is being captured got its error above)
        MOPS_HIP_CHECK(hipMemsetAsync(res.block, 0, counter_bytes, st.stream));
        res.capacity = capacity;
        res.device = device;
        res.counters_dirty = false;
        // another stream that takes the block over waits for the clearing, also when this call
        // fails before its end
        record_last_use(res, st.stream, "scratch");
    } else if (res.block_stream != st.stream && res.last_use_recorded && !st.capturing) {
        // The previous user of the block ran on another stream: this stream
        // waits (on the device, not the host) for the event recorded behind
        // it. The previous stream itself is not touched: its owner may have
        // destroyed it. A stream that is being captured cannot wait for an
        // event outside its graph, and its work does not run now anyway;
        // ordering graph replays against eager calls is the caller's business.
        MOPS_HIP_CHECK(hipStreamWaitEvent(st.stream, res.last_use, 0));
    }
    if (res.counters_dirty) {
        // A call that had the counters did not reach its end: what it enqueued may have counted
        // without the reader that clears. No event was recorded behind it, so when it ran on
        // another stream the host waits for the device (this happens after a failure only).
        if (!st.capturing && res.block_stream != st.stream) {
            MOPS_HIP_CHECK(hipDeviceSynchronize());
        }
        clear_counters(static_cast<int32_t*>(res.block), SCRATCH_COUNTERS, st.stream);
        // (a clearing that was only captured has not run: the next eager call still has to clear)
        res.counters_dirty = st.capturing;
    }
    res.block_stream = st.stream;
    res.block_in_graph = res.block_in_graph || st.capturing;
    st.used_scratch = true;
    return static_cast<char*>(res.block) + SCRATCH_COUNTERS * sizeof(int32_t);
}

ScratchCounters::ScratchCounters() : exceptions_(std::uncaught_exceptions()) {
    auto& st = state();
    if (!st.used_scratch || st.resources == nullptr || st.resources->block == nullptr) {
        throw std::runtime_error("mops: ScratchCounters without scratch() in the same call");
    }
    resources_ = st.resources;
    capturing_ = st.capturing;
    before_ = st.resources->counters_dirty;
    // until this object goes away in the ordinary way: a call that fails in between leaves the
    // mark for the next one
    st.resources->counters_dirty = true;
}

ScratchCounters::~ScratchCounters() {
    if (std::uncaught_exceptions() > exceptions_) {
        return; // the call is failing: what it enqueued may have counted without the reader
    }
    // Every launch of the call is enqueued, the readers that clear the counters included.
    // (Captured launches have not run: the counters are as they were.)
    static_cast<Resources*>(resources_)->counters_dirty = capturing_ ? before_ : false;
}

int32_t* ScratchCounters::data() const { return static_cast<int32_t*>(static_cast<Resources*>(resources_)->block); }

void test_failure_point(const char* name) {
    const char* wanted = std::getenv("MOPS_AMD_TEST_FAIL_AT");
    if (wanted != nullptr && std::string(wanted) == name) {
        throw std::runtime_error(std::string("mops: failure requested by MOPS_AMD_TEST_FAIL_AT at '") + name + "'");
    }
}

size_t scratch_capacity() {
    auto& st = state();
    return st.resources == nullptr ? 0 : st.resources->capacity;
}

int32_t compute_units() {
    static std::atomic<int> cached[64];
    int device = 0;
    MOPS_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= 64) {
        return 256;
    }
    int count = cached[device].load(std::memory_order_relaxed);
    if (count == 0) {
        MOPS_HIP_CHECK(hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device));
        count = std::max(count, 1);
        cached[device].store(count, std::memory_order_relaxed);
    }
    return count;
}

int32_t narrow_i32(size_t value, const char* what) {
    if (value > static_cast<size_t>(std::numeric_limits<int32_t>::max())) {
        throw std::runtime_error(
            std::string(what) + " = " + std::to_string(value) +
            " does not fit the 32-bit indexing of the device kernels"
        );
    }
    return static_cast<int32_t>(value);
}

bool validate_device_indices() {
    const char* value = std::getenv("MOPS_AMD_CHECK_INDICES");
    return value != nullptr && value[0] != '\0' && value[0] != '0';
}

} // namespace mops::amd
