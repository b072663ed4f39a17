// Internal: the kernel behind Expression::takeAlongAxis.
#pragma once

#include "Utilities/Expression/StampedEquation.h"

#include <cstdint>
#include <memory>

namespace ThorImplementation {

// output[c] = values[c with its coordinate along `axis` replaced by indices[c]]; `output` has the shape of `indices`, which
// matches `values` on every other axis.  Indices are UINT32 or UINT64; one past the end and beyond reads the last element
// of the axis (no access leaves the tensor).  All dense.  Kernel arguments: values, indices, output.
std::shared_ptr<StampedEquation> stampTakeAlongAxis(const Tensor& values, const Tensor& indices, const Tensor& output, uint64_t axis, int deviceNum);

}  // namespace ThorImplementation
