#include "runtime.hpp"

#include <cstdlib>
#include <limits>
#include <utility>
#include <vector>

namespace mops::amd {

void check_hip(hipError_t status, const char* what) {
    if (status != hipSuccess) {
        throw std::runtime_error(
            std::string("HIP error in ") + what + ": " + hipGetErrorString(status)
        );
    }
}

namespace {

struct ThreadState {
    hipStream_t stream = nullptr;
    bool synchronous = true;

    // scratch cache
    void* block = nullptr;
    size_t capacity = 0;
    int device = -1;
    hipStream_t block_stream = nullptr;

    // side stream and its two events, per device
    struct Side {
        int device;
        hipStream_t stream;
        hipEvent_t forked;
        hipEvent_t joined;
    };
    std::vector<Side> sides;

    // kernel timing
    bool timing = false;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> recorded;
    std::vector<hipEvent_t> spare;
};

hipEvent_t take_event(ThreadState& st) {
    if (!st.spare.empty()) {
        hipEvent_t event = st.spare.back();
        st.spare.pop_back();
        return event;
    }
    hipEvent_t event = nullptr;
    MOPS_HIP_CHECK(hipEventCreate(&event));
    return event;
}

ThreadState& state() {
    // Deliberately never destroyed: at thread or process exit the HIP runtime
    // may already be gone, and freeing device memory then would fault.
    static thread_local ThreadState* instance = new ThreadState();
    return *instance;
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

void finish_call(const char* operation) {
    check_hip(hipGetLastError(), operation);
    auto& st = state();
    if (st.synchronous) {
        check_hip(hipStreamSynchronize(st.stream), operation);
    }
}

SideStream::SideStream(hipStream_t main) : main_(main) {
    auto& st = state();
    int device = 0;
    MOPS_HIP_CHECK(hipGetDevice(&device));
    ThreadState::Side* side = nullptr;
    for (auto& candidate : st.sides) {
        if (candidate.device == device) {
            side = &candidate;
        }
    }
    if (side == nullptr) {
        ThreadState::Side created{device, nullptr, nullptr, nullptr};
        MOPS_HIP_CHECK(hipStreamCreateWithFlags(&created.stream, hipStreamNonBlocking));
        MOPS_HIP_CHECK(hipEventCreateWithFlags(&created.forked, hipEventDisableTiming));
        MOPS_HIP_CHECK(hipEventCreateWithFlags(&created.joined, hipEventDisableTiming));
        st.sides.push_back(created);
        side = &st.sides.back();
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
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    MOPS_HIP_CHECK(hipStreamIsCapturing(stream, &capture));
    if (capture != hipStreamCaptureStatusNone) {
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
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    MOPS_HIP_CHECK(hipStreamIsCapturing(stream, &capture));
    if (capture != hipStreamCaptureStatusNone) {
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
        st.spare.push_back(pair.first);
        st.spare.push_back(pair.second);
    }
    *milliseconds = total;
    *launches = static_cast<int64_t>(st.recorded.size());
    st.recorded.clear();
}

void* scratch(size_t bytes) {
    auto& st = state();
    int device = 0;
    MOPS_HIP_CHECK(hipGetDevice(&device));

    if (st.block != nullptr && (device != st.device || bytes > st.capacity)) {
        // hipFree waits for the device, so nothing can still be using the block
        int restore = device;
        MOPS_HIP_CHECK(hipSetDevice(st.device));
        MOPS_HIP_CHECK(hipFree(st.block));
        MOPS_HIP_CHECK(hipSetDevice(restore));
        st.block = nullptr;
        st.capacity = 0;
    }

    if (st.block == nullptr) {
        size_t capacity = bytes + bytes / 2;
        if (capacity < (size_t(1) << 20)) {
            capacity = size_t(1) << 20;
        }
        MOPS_HIP_CHECK(hipMalloc(&st.block, capacity));
        st.capacity = capacity;
        st.device = device;
        st.block_stream = st.stream;
    } else if (st.block_stream != st.stream) {
        // The previous user of the block ran on another stream: let it finish
        // before this stream overwrites the block. Streams that are being
        // captured into a graph cannot be waited for (and their work does not
        // run now anyway); ordering graph replays is the caller's business.
        hipStreamCaptureStatus previous = hipStreamCaptureStatusNone;
        hipStreamCaptureStatus next = hipStreamCaptureStatusNone;
        // the previous stream may have been destroyed by its owner meanwhile:
        // then there is nothing left to wait for
        bool previous_alive = hipStreamIsCapturing(st.block_stream, &previous) == hipSuccess;
        if (!previous_alive) {
            (void)hipGetLastError();
        }
        MOPS_HIP_CHECK(hipStreamIsCapturing(st.stream, &next));
        if (previous_alive && previous == hipStreamCaptureStatusNone &&
            next == hipStreamCaptureStatusNone) {
            MOPS_HIP_CHECK(hipStreamSynchronize(st.block_stream));
        }
        st.block_stream = st.stream;
    }
    return st.block;
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
