// Reverse-mode differentiation of Expression graphs: builds, as another Expression graph, the gradients of the forward
// outputs with respect to named tensor inputs.  The result goes through the same compiler as any other expression, so
// the gradient of a fused elementwise chain is again one fused kernel and un-broadcasting is an ordinary reduction stage
// (reference: Utilities/Expression/AutoDiff.h:13-41, AutoDiff.cpp:2486-2581,3690-5932).
//
// Gradient outputs are named "<input>_grad", in the order of `wrt_names` (all tensor inputs when empty), and have the
// shape of the input.  The upstream gradient of each forward output is either an extra input of the backward graph (its
// name given by the caller) or, for a single output with no name given, implicit ones: the gradient of the sum of the
// output's elements.
//
// Differentiable here: + - * / pow, min/max (ties split evenly), neg, abs, the exponentials, logarithms, sqrt,
// trigonometric, hyperbolic and error functions, normcdf, lgamma/tgamma, where, cast (straight through, back to the
// operand's dtype), reshape/unsqueeze/squeeze/transpose, reduce_sum/mean/prod/norm1/norm2, reduce_min/max (the first
// winner in logical order takes the gradient), softmax and log-softmax, segmented sum/mean and segmented broadcast over a
// row partition, and ragged runtime extents.  Rounding, comparison and logical ops, arg reductions, strided views,
// segmented min/max and digamma have no backward rule and throw when a gradient reaches them.
#pragma once

#include "Utilities/Expression/Expression.h"

#include <optional>
#include <string>
#include <unordered_map>
#include <vector>

namespace ThorImplementation {

inline constexpr const char* DEFAULT_BACKWARD_UPSTREAM_INPUT_NAME = "__grad_output";

// With `forward_input_dims` (by input name) every gradient has exactly the shape of its input: contributions to an operand that
// the forward op broadcast are summed back, gradients of reductions are expanded.  Without them (the reference's shape-free form)
// nothing is expanded or summed back - the implicit seed is the scalar 1, contributions keep the shape broadcasting gives them -
// which is the gradient itself for graphs whose operands all have one shape; reshapes, squeezing reductions, means, min / max
// reductions, softmax, strided views and segmented ops need shapes and throw std::runtime_error ("... requires forward shape
// information.").  FusedEquation::compileBackward always builds with the shapes of the tensors it is stamped with.
PhysicalOutputs buildBackwardOutputs(const PhysicalOutputs& forward_outputs, const std::vector<std::string>& wrt_names = {},
                                     const std::optional<std::string>& upstream_input_name = std::nullopt,
                                     const std::optional<std::unordered_map<std::string, std::vector<uint64_t>>>& forward_input_dims = std::nullopt,
                                     bool accumulate_grad_outputs = false);

// Explicit upstream gradient input per forward output (may name a subset: outputs without an entry contribute nothing).
PhysicalOutputs buildBackwardOutputs(const PhysicalOutputs& forward_outputs, const std::vector<std::string>& wrt_names,
                                     const std::unordered_map<std::string, std::string>& upstream_input_names_by_output,
                                     const std::optional<std::unordered_map<std::string, std::vector<uint64_t>>>& forward_input_dims = std::nullopt,
                                     bool accumulate_grad_outputs = false);

// As above, with the runtime dtype of each upstream gradient input (by forward-output name; an input named without its dtype
// throws): the seed's INPUT node carries it, so dtype resolution of the backward graph starts from the tensor that will be bound.
PhysicalOutputs buildBackwardOutputs(const PhysicalOutputs& forward_outputs, const std::vector<std::string>& wrt_names,
                                     const std::unordered_map<std::string, std::string>& upstream_input_names_by_output,
                                     const std::unordered_map<std::string, DataType>& upstream_input_dtypes_by_output,
                                     const std::optional<std::unordered_map<std::string, std::vector<uint64_t>>>& forward_input_dims = std::nullopt,
                                     bool accumulate_grad_outputs = false);

// As above, with upstream gradients that are values of the forward graph itself (node indices by forward-output name; they take
// precedence over an input named for the same output).
PhysicalOutputs buildBackwardOutputs(const PhysicalOutputs& forward_outputs, const std::vector<std::string>& wrt_names,
                                     const std::unordered_map<std::string, std::string>& upstream_input_names_by_output,
                                     const std::unordered_map<std::string, uint32_t>& upstream_node_indices_by_output,
                                     const std::optional<std::unordered_map<std::string, std::vector<uint64_t>>>& forward_input_dims = std::nullopt,
                                     bool accumulate_grad_outputs = false);

// Validation shared with FusedEquation::compileBackward, which defers the graph construction until shapes are bound.
std::vector<std::string> normalizeBackwardWrtNames(const PhysicalExpression& forward_expr, const std::vector<std::string>& wrt_names);
std::optional<std::unordered_map<std::string, std::string>> normalizeBackwardUpstreamNames(const PhysicalOutputs& forward_outputs,
                                                                                             const std::optional<std::string>& upstream_input_name);
std::unordered_map<std::string, std::string> normalizeBackwardUpstreamNames(
    const PhysicalOutputs& forward_outputs, const std::unordered_map<std::string, std::string>& upstream_input_names_by_output);

}  // namespace ThorImplementation
