// Internal: handle structs and the exception -> error-code bridge of the flat C binding.
#pragma once

#include "thor_c_api.h"

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"
#include "Utilities/TensorOperations/Cub/CubReduction.h"

#include <algorithm>
#include <memory>
#include <stdexcept>
#include <string>

struct thor_stream {
    Stream stream;
};
struct thor_tensor {
    ThorImplementation::Tensor tensor;
};
struct thor_stamped_reduction {
    std::shared_ptr<ThorImplementation::StampedCubReduction> stamped;
};
struct thor_stamped_arg_reduction {
    std::shared_ptr<ThorImplementation::StampedCubArgReduction> stamped;
};
struct thor_stamped_segmented_reduction {
    std::shared_ptr<ThorImplementation::StampedCubSegmentedReduction> value;     // exactly one of the two is set
    std::shared_ptr<ThorImplementation::StampedCubSegmentedArgReduction> arg;
};

namespace thor_capi {
std::string& lastError();
void recordCurrentException();
int copyOut(const std::string& text, char* buffer, size_t capacity, size_t* needed);

template <typename T>
void require(T* handle, const char* what) {
    if (handle == nullptr) throw std::invalid_argument(std::string("NULL ") + what + " handle");
}
}  // namespace thor_capi

// body runs inside try; an exception becomes return value -1 (or nullptr) plus thor_last_error()
#define THOR_CAPI_TRY_INT(...)                     \
    try {                                          \
        __VA_ARGS__                                \
        return 0;                                  \
    } catch (...) {                                \
        ::thor_capi::recordCurrentException();     \
        return -1;                                 \
    }

#define THOR_CAPI_TRY_PTR(...)                     \
    try {                                          \
        __VA_ARGS__                                \
    } catch (...) {                                \
        ::thor_capi::recordCurrentException();     \
        return nullptr;                            \
    }
