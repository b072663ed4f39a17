#include "Utilities/Common/Stream.h"

#include <atomic>
#include <vector>

using ThorImplementation::ScopedGpu;

struct Stream::State {
    void* handle = nullptr;
    int gpuNum = 0;
    uint64_t id = 0;
    std::mutex failureMutex;
    std::exception_ptr firstFailure;

    ~State() {
        if (handle != nullptr) (void)thorhip_stream_destroy(handle);
    }
};

struct Stream::PendingHostCall {
    HostFn function;
    std::unique_ptr<HostFunctionArgsBase> args;
    std::shared_ptr<State> owner;
};

static std::atomic<uint64_t> nextStreamId{1};

// Finished host calls wait here until an application thread destroys them.  Never destructed: callbacks may still arrive
// while the process shuts down.
namespace {
struct FinishedCalls {
    std::mutex mutex;
    std::vector<void*> calls;
};
FinishedCalls& finishedCalls() {
    static FinishedCalls* list = new FinishedCalls;
    return *list;
}
}  // namespace

void Stream::drainFinishedHostCalls() {
    std::vector<void*> calls;
    {
        FinishedCalls& list = finishedCalls();
        std::lock_guard<std::mutex> lock(list.mutex);
        calls.swap(list.calls);
    }
    for (void* raw : calls) delete static_cast<PendingHostCall*>(raw);
}

Stream::Stream(int gpuNum, Priority) {
    // Priorities are accepted for source compatibility; every stream is created at the default priority.
    ScopedGpu scoped(gpuNum);
    auto s = std::make_shared<State>();
    THOR_HIP_CHECK(thorhip_stream_create(&s->handle));
    s->gpuNum = gpuNum;
    s->id = nextStreamId.fetch_add(1);
    state = std::move(s);
}

Stream::Stream(ThorImplementation::TensorPlacement placement, Priority priority)
    : Stream(placement.getMemDevice() == ThorImplementation::TensorPlacement::MemDevices::GPU ? placement.getDeviceNum() : 0, priority) {}

void* Stream::getStream() const {
    THOR_THROW_IF_FALSE(state != nullptr);
    return state->handle;
}

int Stream::getGpuNum() const {
    THOR_THROW_IF_FALSE(state != nullptr);
    return state->gpuNum;
}

uint64_t Stream::getId() const {
    THOR_THROW_IF_FALSE(state != nullptr);
    return state->id;
}

Event Stream::putEvent(bool enableTiming, bool) const {
    Event event(getGpuNum(), enableTiming);
    THOR_HIP_CHECK(thorhip_event_record(event.getEvent(), state->handle));
    return event;
}

void Stream::putEvent(Event& event, bool enableTiming, bool) const {
    if (!event.isInitialized()) event = Event(getGpuNum(), enableTiming);
    THOR_HIP_CHECK(thorhip_event_record(event.getEvent(), state->handle));
}

void Stream::waitEvent(Event event) const {
    THOR_THROW_IF_FALSE(state != nullptr && event.isInitialized());
    THOR_HIP_CHECK(thorhip_stream_wait_event(state->handle, event.getEvent()));
}

void Stream::synchronize() const {
    THOR_THROW_IF_FALSE(state != nullptr);
    THOR_HIP_CHECK(thorhip_stream_synchronize(state->handle));
    drainFinishedHostCalls();
    std::exception_ptr failure;
    {
        std::lock_guard<std::mutex> lock(state->failureMutex);
        std::swap(failure, state->firstFailure);
    }
    if (failure) std::rethrow_exception(failure);
}

void Stream::deviceSynchronize(int gpuNum) {
    ScopedGpu scoped(gpuNum);
    THOR_HIP_CHECK(thorhip_device_synchronize());
}

void Stream::hostFunctionTrampoline(void* raw) noexcept {
    PendingHostCall* call = static_cast<PendingHostCall*>(raw);
    try {
        call->function(call->args.get());
    } catch (...) {
        std::lock_guard<std::mutex> lock(call->owner->failureMutex);
        if (!call->owner->firstFailure) call->owner->firstFailure = std::current_exception();
    }
    // This runs on the runtime's callback thread: destroying the arguments here could free device or pinned memory (the
    // tensors a copy keeps alive), which blocks on the very stream that is executing this callback.  Park them instead.
    try {
        FinishedCalls& list = finishedCalls();
        std::lock_guard<std::mutex> lock(list.mutex);
        list.calls.push_back(call);
    } catch (...) {
        // out of memory while parking: leak the call rather than release memory on this thread
    }
}

void Stream::enqueueHostFunction(HostFn function, std::unique_ptr<HostFunctionArgsBase>&& args) {
    THOR_THROW_IF_FALSE(state != nullptr && function != nullptr);
    drainFinishedHostCalls();
    auto* call = new PendingHostCall{function, std::move(args), state};
    const int rc = thorhip_stream_enqueue_host_function(state->handle, &Stream::hostFunctionTrampoline, call);
    if (rc != 0) {
        delete call;
        ThorImplementation::hipCheck(rc, "thorhip_stream_enqueue_host_function");
    }
}
