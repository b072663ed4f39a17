// Internal: differentiation of a forward graph whose dtypes have been resolved for the tensors actually bound, so that the
// backward graph undoes casts to, and delivers gradients in, the dtypes of those tensors.
#pragma once

#include "Utilities/Expression/AutoDiff.h"

namespace ThorImplementation {

// `typed_forward` is a copy of *forward_outputs.expr (same node numbering) after resolveOutputsDTypesInPlace; the upstream
// names are taken as validated.
PhysicalOutputs buildBackwardOutputsTyped(const PhysicalOutputs& forward_outputs, const PhysicalExpression& typed_forward,
                                          const std::vector<std::string>& wrt_names,
                                          const std::optional<std::unordered_map<std::string, std::string>>& upstream_input_names_by_output,
                                          const std::unordered_map<std::string, std::vector<uint64_t>>& forward_input_dims,
                                          bool accumulate_grad_outputs);

}  // namespace ThorImplementation
