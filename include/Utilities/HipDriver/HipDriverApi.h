// Exception-throwing C++ face of the thorhip C ABI.  This is the only way host code reaches the GPU: it plays the role
// the dlopen()ed CUDA driver table plays in the reference (Utilities/CudaDriver/CudaDrivertApi.h:9-158) and, like the
// reference's check macros (Utilities/Expression/CudaHelpers.h:22-92), turns failure codes into std::runtime_error.
#pragma once

#include "thorhip.h"

#include <stdexcept>
#include <string>

namespace ThorImplementation {

inline void hipCheck(int rc, const char* what) {
    if (rc != 0) {
        throw std::runtime_error(std::string(what) + " failed (" + std::to_string(rc) + "): " + thorhip_last_error());
    }
}

#define THOR_HIP_CHECK(call) ::ThorImplementation::hipCheck((call), #call)

}  // namespace ThorImplementation
