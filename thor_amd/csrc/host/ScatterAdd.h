// Internal: flat scatter-add, the second half of the gradient of min / max scans.
#pragma once

#include "Utilities/Expression/StampedEquation.h"

#include <cstdint>
#include <memory>
#include <optional>
#include <vector>

namespace ThorImplementation {

// output[:] = 0 (FP32, dense).  Kernel argument: output.
std::shared_ptr<StampedEquation> stampScatterClear(const Tensor& output, int deviceNum);
// output[indices[i]] += updates[i] for every i whose index lies inside the output (0xFFFFFFFF and anything else out of range is
// skipped), and, given the offsets [B + 1] of a row partition, only for i in [offsets[0], offsets[B]).  updates FP32, indices
// UINT32, same element count; output FP32.  Kernel arguments: updates, indices, [offsets], output.
std::shared_ptr<StampedEquation> stampScatterAdd(const Tensor& updates, const Tensor& indices, const Tensor& output, const std::optional<Tensor>& offsets,
                                                 int deviceNum);

// output[offset + sum(c[k] * strides[k])] = gradient[c] for every coordinate c of `dims` (gradient dense FP32 of that shape,
// output dense FP32).  Throws when two coordinates address one element or any leaves the output.  Kernel arguments: gradient, output.
std::shared_ptr<StampedEquation> stampViewScatter(const Tensor& gradient, const Tensor& output, const std::vector<uint64_t>& dims,
                                                  const std::vector<uint64_t>& strides, uint64_t offset, int deviceNum);

}  // namespace ThorImplementation
