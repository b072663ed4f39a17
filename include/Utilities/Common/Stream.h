// Shared-ownership handle of one HIP stream on one GPU (reference: Utilities/Common/Stream.h:35-116).
//
// Copies refer to the same stream.  Host callbacks enqueued with enqueueHostFunction never let an exception cross the
// C callback boundary: the first exception is captured and rethrown by synchronize(), as in the reference
// (Stream.h:63-66,107-108).  Every stream is created at the default priority.
#pragma once

#include "DeepLearning/Implementation/Tensor/TensorPlacement.h"
#include "Utilities/Common/Event.h"

#include <cstdint>
#include <exception>
#include <functional>
#include <memory>
#include <mutex>
#include <string>

struct HostFunctionArgsBase {
    virtual ~HostFunctionArgsBase() = default;
};

class Stream {
   public:
    enum class Priority { HIGH = 3, REGULAR = 4, LOW = 5 };

    Stream() = default;
    explicit Stream(int gpuNum, Priority priority = Priority::REGULAR);
    explicit Stream(ThorImplementation::TensorPlacement placement, Priority priority = Priority::REGULAR);
    virtual ~Stream() = default;

    // The raw stream handle as the C ABI expects it (hipStream_t behind void*).
    void* getStream() const;
    operator void*() const { return getStream(); }

    Event putEvent(bool enableTiming = false, bool expectingHostToWaitOnThisOne = false) const;
    void putEvent(Event& event, bool enableTiming = false, bool expectingHostToWaitOnThisOne = false) const;
    void waitEvent(Event event) const;
    void synchronize() const;
    static void deviceSynchronize(int gpuNum);

    typedef void (*HostFn)(void*);
    void enqueueHostFunction(HostFn function, std::unique_ptr<HostFunctionArgsBase>&& args);
    // The arguments of a finished host function (and the tensors they keep alive) are destroyed on an application thread,
    // never on the runtime's callback thread, where releasing device or pinned memory is not allowed.  synchronize(),
    // enqueueHostFunction() and tensor allocation drain the list; it may also be drained explicitly.
    static void drainFinishedHostCalls();

    bool operator==(const Stream& other) const { return state != nullptr && state == other.state; }
    int getGpuNum() const;
    bool isInitialized() const { return state != nullptr; }
    uint64_t getId() const;
    virtual std::string getObjectName() const { return "Stream"; }

   private:
    struct State;
    struct PendingHostCall;
    static void hostFunctionTrampoline(void* raw) noexcept;
    std::shared_ptr<State> state;
};
