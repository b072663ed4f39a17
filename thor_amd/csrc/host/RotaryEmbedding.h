// Internal: the kernel behind Expression::rotaryPositionEmbedding.
#pragma once

#include "Utilities/Expression/Expression.h"
#include "Utilities/Expression/StampedEquation.h"

#include <cstdint>
#include <memory>
#include <optional>

namespace ThorImplementation {

// output = values with every pair of the rotary part of the head dimension turned by position * frequency(pair); the rest of
// the head dimension is copied.  `node` carries the ROPE parameters.  positionIds (any numeric dtype, one element per
// element of the sequence axis) replace coordinate + offset; effectiveLength (one element) replaces the extent of the sequence
// axis in the Dynamic-NTK and LongRoPE rules.  All tensors dense.  Kernel arguments: values, [ids], [length], output.
std::shared_ptr<StampedEquation> stampRotaryEmbedding(const Tensor& values, const std::optional<Tensor>& positionIds,
                                                      const std::optional<Tensor>& effectiveLength, const Tensor& output, const ExprNode& node,
                                                      int deviceNum);

}  // namespace ThorImplementation
