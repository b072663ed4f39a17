// Shared-ownership HIP event handle (the reference's Utilities/Common/Event.h counterpart).
#pragma once

#include "Utilities/Common/ScopedGpu.h"

#include <memory>

class Event {
   public:
    Event() = default;
    explicit Event(int gpuNum, bool enableTiming = false) {
        ThorImplementation::ScopedGpu scoped(gpuNum);
        void* handle = nullptr;
        THOR_HIP_CHECK(thorhip_event_create(&handle, enableTiming ? 1 : 0));
        state = std::shared_ptr<State>(new State{handle, gpuNum}, [](State* s) {
            (void)thorhip_event_destroy(s->handle);
            delete s;
        });
    }

    bool isInitialized() const { return state != nullptr; }
    void* getEvent() const { return state ? state->handle : nullptr; }
    int getGpuNum() const { return state ? state->gpuNum : -1; }

    void synchronize() const {
        if (state) THOR_HIP_CHECK(thorhip_event_synchronize(state->handle));
    }

    // Milliseconds between this (earlier) event and `later`; both must have been created with timing enabled.
    float synchronizeAndReportElapsedTimeInMilliseconds(const Event& later) const {
        float ms = 0.0f;
        later.synchronize();
        THOR_HIP_CHECK(thorhip_event_elapsed_ms(&ms, state->handle, later.state->handle));
        return ms;
    }

   private:
    struct State {
        void* handle;
        int gpuNum;
    };
    std::shared_ptr<State> state;
};
