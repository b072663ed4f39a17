// Internal: the dimensions of every node of an expression graph, given the dimensions of the tensors bound to its inputs
// (NumPy-style right-aligned broadcasting for elementwise nodes; reductions, shape ops and ragged ops by their own rules).
#pragma once

#include "Utilities/Expression/Expression.h"

#include <cstdint>
#include <functional>
#include <vector>

namespace ThorImplementation {

// `inputDims(slot)` returns the dimensions bound to that input slot.  Scalars have rank 0.  Throws std::runtime_error when
// operands do not broadcast or an axis is out of range.
std::vector<std::vector<uint64_t>> inferExpressionShapes(const PhysicalExpression& expr,
                                                           const std::function<std::vector<uint64_t>(uint32_t)>& inputDims);

}  // namespace ThorImplementation
