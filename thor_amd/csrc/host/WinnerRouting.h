// Internal: the kernel that spreads the gradient of a min/max reduction to the winners of its windows.
#pragma once

#include "Utilities/Expression/StampedEquation.h"

#include <cstdint>
#include <memory>
#include <vector>

namespace ThorImplementation {

// `winners` holds, per reduction window (numbered row-major over the kept axes of `operandDims`), the UINT32 position of
// the winning element inside the window (row-major over `reducedAxes`, sorted).  `outputGradient` holds one value per
// window, `routed` has the operand's element count.  All dense; arguments of the kernel: winners, gradient, routed.
std::shared_ptr<StampedEquation> stampWinnerRouting(const Tensor& winners, const Tensor& outputGradient, const Tensor& routed,
                                                    const std::vector<uint64_t>& operandDims, const std::vector<uint64_t>& reducedAxes, int deviceNum);

}  // namespace ThorImplementation
