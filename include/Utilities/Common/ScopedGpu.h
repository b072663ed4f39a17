// Makes `gpuNum` the calling thread's current device for the lifetime of the object and restores the previous one.
#pragma once

#include "Utilities/HipDriver/HipDriverApi.h"

namespace ThorImplementation {

class ScopedGpu {
   public:
    explicit ScopedGpu(int gpuNum) {
        THOR_HIP_CHECK(thorhip_get_device(&previous));
        if (previous != gpuNum) {
            THOR_HIP_CHECK(thorhip_set_device(gpuNum));
            switched = true;
        }
    }
    ~ScopedGpu() {
        if (switched) (void)thorhip_set_device(previous);
    }
    ScopedGpu(const ScopedGpu&) = delete;
    ScopedGpu& operator=(const ScopedGpu&) = delete;

   private:
    int previous = 0;
    bool switched = false;
};

}  // namespace ThorImplementation
