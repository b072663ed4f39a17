// FusedEquation: a compiled Expression.  compile() only captures the graph; the first stamp()/run() with concrete
// tensors resolves dtypes, infers shapes, splits the graph into stages at reduction boundaries, generates gfx950
// source for each fused stage, compiles it with hipRTC and binds tensors.  Plans are cached per (dtypes, shapes,
// strides, alignment) and kernels process-wide per source text
// (reference: Utilities/Expression/FusedEquation.h:574-632; FusedEquation.cpp:6828-6887,7014-7064,8885-9353,10760-10905).
#pragma once

#include "Utilities/Cache/LruCache.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "Utilities/Expression/Expression.h"
#include "Utilities/Expression/StampedEquation.h"

#include <memory>
#include <optional>
#include <string>
#include <unordered_map>
#include <vector>

namespace ThorImplementation {

struct PlannedGraph;  // dtype-resolved, de-duplicated graph with its stage split (internal)

class FusedEquation {
   public:
    static FusedEquation compile(const PhysicalExpression& expr, int device_num);
    static FusedEquation compile(const PhysicalOutputs& outputs, int device_num);

    // Binds tensors and returns a plan whose run() only launches.  Outputs are allocated here unless the caller passes
    // them in `preallocated_outputs` (shape and dtype are validated).
    // `tensor_scalar_inputs` binds the equation's tensorRuntimeScalar inputs to elements of device buffers.
    // `requestedOutputShapes` (reference: FusedEquation.h:594-599, FusedEquation.cpp:3152-3174): the dimensions the caller wants an
    // output tensor to carry.  They must be the dimensions the expression gives it up to axes of extent 1 (a row-reduction's
    // [N, 1] asked for as [N]); anything else throws "Output tensor dimensions are incompatible with the fused equation
    // result."  A preallocated output of that name is checked against the request and keeps its own dimensions.
    [[nodiscard]] StampedExecutionPlan stamp(const std::unordered_map<std::string, Tensor>& inputs, const Stream& stream,
                                             const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs = {},
                                             const std::unordered_map<std::string, Tensor>& preallocated_outputs = {},
                                             const std::unordered_map<std::string, std::vector<uint64_t>>& requestedOutputShapes = {}) const;
    [[nodiscard]] StampedExecutionPlan stampSingleOutput(const std::unordered_map<std::string, Tensor>& inputs, const Stream& stream,
                                                         const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs = {},
                                                         const std::optional<Tensor>& preallocated_output = {},
                                                         const std::vector<uint64_t>& requestedOutputShape = {}) const;

    // Convenience: bind, launch into caller-provided outputs.  Restricted, as in the reference, to expressions that
    // lower to fused kernels only (no reduction stage) -- use stamp() otherwise.
    void run(const Tensor& input, Tensor& output, Stream& stream) const;
    void run(const std::unordered_map<std::string, Tensor>& inputs, Tensor& output, Stream& stream) const;
    void run(const std::unordered_map<std::string, Tensor>& inputs, const std::unordered_map<std::string, float>& scalar_inputs, Tensor& output,
             Stream& stream) const;
    void run(const Tensor& input, std::unordered_map<std::string, Tensor>& outputs, Stream& stream) const;
    void run(const std::unordered_map<std::string, Tensor>& inputs, std::unordered_map<std::string, Tensor>& outputs, Stream& stream) const;
    void run(const std::unordered_map<std::string, Tensor>& inputs, const std::unordered_map<std::string, float>& scalar_inputs,
             std::unordered_map<std::string, Tensor>& outputs, Stream& stream) const;

    // The equation of the gradients of this equation's outputs with respect to the named tensor inputs (all of them when
    // `wrt_names` is empty): outputs "<input>_grad", inputs the forward inputs plus one upstream gradient per forward
    // output (named by the caller; with no name given, a single output's upstream gradient is implicit ones) and, with
    // `accumulate_grad_outputs`, the running "<input>_grad" tensors the new gradients are added to.  The gradient graph is
    // built when tensors are bound, since undoing broadcasts needs their shapes; names are validated here.
    [[nodiscard]] FusedEquation compileBackward(const std::vector<std::string>& wrt_names = {},
                                                const std::optional<std::string>& upstream_input_name = std::nullopt,
                                                bool accumulate_grad_outputs = false) const;
    [[nodiscard]] FusedEquation compileBackward(const std::vector<std::string>& wrt_names,
                                                const std::unordered_map<std::string, std::string>& upstream_input_names_by_output,
                                                bool accumulate_grad_outputs = false) const;

    std::vector<std::string> getOutputNames() const;
    [[nodiscard]] const PhysicalOutputs& physicalOutputs() const { return outputs_template; }

    std::vector<uint64_t> getOutputShape(const Tensor& input) const;
    std::vector<uint64_t> getOutputShape(const std::unordered_map<std::string, Tensor>& inputs) const;
    std::unordered_map<std::string, std::vector<uint64_t>> getOutputShapes(const Tensor& input) const;
    std::unordered_map<std::string, std::vector<uint64_t>> getOutputShapes(const std::unordered_map<std::string, Tensor>& inputs) const;
    std::unordered_map<std::string, std::vector<uint64_t>> getOutputShapes(
        const std::unordered_map<std::string, Tensor>& inputs, const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs) const;
    std::unordered_map<std::string, DataType> getOutputDataTypes(const std::unordered_map<std::string, Tensor>& inputs) const;
    std::unordered_map<std::string, DataType> getOutputDataTypes(const std::unordered_map<std::string, Tensor>& inputs,
                                                                 const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs) const;

    // NumPy-style right-aligned broadcast of the input shapes; returns true when any input needs broadcasting.
    static bool resolveLayout(std::vector<Tensor>& inputs, std::vector<uint64_t>& outputDimensions);

    int getDeviceNum() const { return device_num; }

   private:
    FusedEquation(PhysicalOutputs outputs_template, int device_num);

    // `inputs` plus one single-element view per tensor-scalar binding (validated)
    std::unordered_map<std::string, Tensor> withTensorScalars(const std::unordered_map<std::string, Tensor>& inputs,
                                                              const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs) const;
    std::shared_ptr<PlannedGraph> plannedGraphFor(const std::vector<DataType>& root_dtypes) const;
    std::vector<DataType> rootDTypes(const std::unordered_map<std::string, Tensor>& inputs) const;
    StampedExecutionPlan stampImpl(const std::unordered_map<std::string, Tensor>& inputs, const Stream& stream,
                                   const std::unordered_map<std::string, Tensor>& preallocated_outputs, bool fusedKernelsOnly,
                                   const std::unordered_map<std::string, std::vector<uint64_t>>& requestedOutputShapes = {}) const;

    struct BackwardRecipe;  // a backward equation before shapes are known: the forward graph and what to differentiate
    FusedEquation(std::shared_ptr<BackwardRecipe> recipe, int device_num);
    // the equation for the shapes and dtypes of `inputs`, and the subset of `inputs` it reads
    std::shared_ptr<const FusedEquation> backwardFor(const std::unordered_map<std::string, Tensor>& inputs,
                                                     std::unordered_map<std::string, Tensor>& used) const;

    std::shared_ptr<BackwardRecipe> backward;  // set on equations made by compileBackward; outputs_template is empty then
    PhysicalOutputs outputs_template;
    std::vector<NamedInput> root_inputs;
    int device_num;
    // dtype key -> planned graph; full binding key -> stamped plan recipe is rebuilt per stamp (allocation is per stamp)
    std::shared_ptr<LruCacheThreadSafe<std::string, std::shared_ptr<PlannedGraph>>> planned_graph_cache;
};

}  // namespace ThorImplementation
