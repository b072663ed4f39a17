// Flat C binding, part 2: Expression, Outputs, FusedEquation, StampedExecutionPlan.
#include "capi_internal.h"

#include "Utilities/Expression/FusedEquation.h"

#include <functional>
#include <limits>
#include <unordered_map>

using namespace ThorImplementation;
using namespace thor_capi;

struct thor_expr {
    Expression expr;
};
struct thor_outputs {
    Outputs outputs;
};
struct thor_fused_equation {
    FusedEquation equation;
};
struct thor_plan {
    StampedExecutionPlan plan;
};

namespace {

std::optional<DataType> optionalDType(int code) {
    if (code < 0) return std::nullopt;
    (void)dataTypeName(static_cast<DataType>(code));
    return static_cast<DataType>(code);
}

std::vector<uint64_t> u64s(const uint64_t* p, int n) { return std::vector<uint64_t>(p, p + (n > 0 ? n : 0)); }

const std::unordered_map<std::string, std::function<Expression(const Expression&)>>& unaryMethods() {
    static const std::unordered_map<std::string, std::function<Expression(const Expression&)>> table = {
#define M(name) {#name, [](const Expression& e) { return e.name(); }}
        M(abs), M(ceil), M(floor), M(round), M(trunc), M(sin), M(cos), M(tan), M(csc), M(sec), M(cot), M(asin), M(acos), M(atan), M(acsc),
        M(asec), M(acot), M(sinh), M(cosh), M(tanh), M(csch), M(sech), M(coth), M(asinh), M(acosh), M(atanh), M(acsch), M(asech), M(acoth),
        M(erf), M(erfc), M(erfcx), M(erfinv), M(erfcinv), M(tgamma), M(lgamma), M(digamma), M(ln), M(log1p), M(log2), M(log10), M(exp), M(expm1),
        M(exp2), M(exp10), M(sqrt), M(normcdf), M(sigmoid), M(softplus), M(selu), M(gelu), M(mish), M(relu6), M(hardSwish), M(swish),
        M(logicalNot), M(transpose),
#undef M
        {"neg", [](const Expression& e) { return -e; }},
        {"elu", [](const Expression& e) { return e.elu(); }},
        {"hardTanh", [](const Expression& e) { return e.hardTanh(); }},
        {"threshold", [](const Expression& e) { return e.threshold(); }},
    };
    return table;
}

const std::unordered_map<std::string, std::function<Expression(const Expression&, const Expression&)>>& binaryMethods() {
    static const std::unordered_map<std::string, std::function<Expression(const Expression&, const Expression&)>> table = {
        {"add", [](const Expression& a, const Expression& b) { return a + b; }},
        {"sub", [](const Expression& a, const Expression& b) { return a - b; }},
        {"mul", [](const Expression& a, const Expression& b) { return a * b; }},
        {"div", [](const Expression& a, const Expression& b) { return a / b; }},
        {"pow", [](const Expression& a, const Expression& b) { return a.pow(b); }},
        {"min", [](const Expression& a, const Expression& b) { return a.min(b); }},
        {"max", [](const Expression& a, const Expression& b) { return a.max(b); }},
        {"equal", [](const Expression& a, const Expression& b) { return a.equal(b); }},
        {"notEqual", [](const Expression& a, const Expression& b) { return a.notEqual(b); }},
        {"lessThan", [](const Expression& a, const Expression& b) { return a.lessThan(b); }},
        {"lessEqual", [](const Expression& a, const Expression& b) { return a.lessEqual(b); }},
        {"greaterThan", [](const Expression& a, const Expression& b) { return a.greaterThan(b); }},
        {"greaterEqual", [](const Expression& a, const Expression& b) { return a.greaterEqual(b); }},
        {"logicalAnd", [](const Expression& a, const Expression& b) { return a.logicalAnd(b); }},
        {"logicalOr", [](const Expression& a, const Expression& b) { return a.logicalOr(b); }},
        {"dotProduct", [](const Expression& a, const Expression& b) { return a.dotProduct(b); }},
    };
    return table;
}

std::unordered_map<std::string, Tensor> tensorMap(const char* const* names, const thor_tensor_t* tensors, int count) {
    std::unordered_map<std::string, Tensor> map;
    for (int i = 0; i < count; ++i) {
        if (names[i] == nullptr || tensors[i] == nullptr) throw std::invalid_argument("NULL name or tensor in a named tensor list");
        map.emplace(names[i], tensors[i]->tensor);
    }
    return map;
}

std::unordered_map<std::string, float> scalarMap(const char* const* names, const float* values, int count) {
    std::unordered_map<std::string, float> map;
    for (int i = 0; i < count; ++i) map.emplace(names[i], values[i]);
    return map;
}

}  // namespace

extern "C" {

thor_expr_t thor_expr_input(const char* name, int compute_dtype, int output_dtype) {
    THOR_CAPI_TRY_PTR(return new thor_expr{Expression::input(name ? name : "", optionalDType(compute_dtype), optionalDType(output_dtype))};)
}
thor_expr_t thor_expr_runtime_scalar(const char* name, int compute_dtype, int output_dtype) {
    THOR_CAPI_TRY_PTR(return new thor_expr{Expression::runtimeScalar(name ? name : "", optionalDType(compute_dtype), optionalDType(output_dtype))};)
}
thor_expr_t thor_expr_tensor_runtime_scalar(const char* name, int compute_dtype, int output_dtype) {
    THOR_CAPI_TRY_PTR(return new thor_expr{Expression::tensorRuntimeScalar(name ? name : "", optionalDType(compute_dtype), optionalDType(output_dtype))};)
}
thor_expr_t thor_expr_scalar(double value) { THOR_CAPI_TRY_PTR(return new thor_expr{Expression(value)};) }
thor_expr_t thor_expr_fill(double value, const uint64_t* dims, int rank, int output_dtype) {
    THOR_CAPI_TRY_PTR(return new thor_expr{Expression::fill(value, u64s(dims, rank), optionalDType(output_dtype))};)
}

thor_expr_t thor_expr_binary(const char* method, thor_expr_t lhs, thor_expr_t rhs) {
    THOR_CAPI_TRY_PTR(require(lhs, "expression"); require(rhs, "expression");
                      auto it = binaryMethods().find(method ? method : "");
                      if (it == binaryMethods().end()) throw std::invalid_argument(std::string("Unknown binary Expression method: ") + (method ? method : "(null)"));
                      return new thor_expr{it->second(lhs->expr, rhs->expr)};)
}

thor_expr_t thor_expr_ragged(const char* method, thor_expr_t values, thor_expr_t offsets, uint64_t batch_size, uint64_t max_active_values,
                             uint64_t elements_per_value) {
    THOR_CAPI_TRY_PTR(
        require(values, "expression"); require(offsets, "expression"); const std::string m = method ? method : "";
        if (m == "segmented_broadcast" || m == "segmented_broadcast_normalized") {
            return new thor_expr{Expression::segmentedBroadcast(values->expr, offsets->expr, batch_size, max_active_values, elements_per_value,
                                                                m == "segmented_broadcast_normalized")};
        }
        if (m == "ragged_extent") {
            return new thor_expr{values->expr.withRaggedRuntimeExtent(offsets->expr, batch_size, max_active_values, elements_per_value)};
        }
        ExprOp op;
        if (m == "segment_sum") op = ExprOp::SEGMENTED_REDUCE_SUM;
        else if (m == "segment_min") op = ExprOp::SEGMENTED_REDUCE_MIN;
        else if (m == "segment_max") op = ExprOp::SEGMENTED_REDUCE_MAX;
        else if (m == "segment_mean") op = ExprOp::SEGMENTED_REDUCE_MEAN;
        else throw std::invalid_argument("Unknown ragged Expression method: " + m);
        return new thor_expr{Expression::segmentedReduceWithRaggedMetadata(values->expr, offsets->expr, op, batch_size, max_active_values,
                                                                           elements_per_value == 0 ? 1 : elements_per_value)};)
}

thor_expr_t thor_expr_unary(const char* method, thor_expr_t input) {
    THOR_CAPI_TRY_PTR(require(input, "expression");
                      auto it = unaryMethods().find(method ? method : "");
                      if (it == unaryMethods().end()) throw std::invalid_argument(std::string("Unknown unary Expression method: ") + (method ? method : "(null)"));
                      return new thor_expr{it->second(input->expr)};)
}

thor_expr_t thor_expr_unary_params(const char* method, thor_expr_t input, double p0, double p1) {
    THOR_CAPI_TRY_PTR(
        require(input, "expression");
        const std::string m = method ? method : "";
        if (m == "elu") return new thor_expr{input->expr.elu(p0)};
        if (m == "hardTanh") return new thor_expr{input->expr.hardTanh(p0, p1)};
        if (m == "threshold") return new thor_expr{input->expr.threshold(p0, p1)};
        if (m == "log") return new thor_expr{input->expr.log(p0)};
        if (m == "clamp") return new thor_expr{input->expr.clamp(p0, p1)};
        if (m == "softmax" || m == "logSoftmax") {  // p0: 0 fast, 1 accurate; p1: 0 instance, 1 channel
            if ((p0 != 0.0 && p0 != 1.0) || (p1 != 0.0 && p1 != 1.0)) throw std::invalid_argument("Unknown softmax algorithm or mode.");
            const SoftmaxMode mode = p1 == 0.0 ? SoftmaxMode::Instance : SoftmaxMode::Channel;
            if (m == "logSoftmax") return new thor_expr{input->expr.logSoftmax(mode)};
            return new thor_expr{input->expr.softmax(p0 == 0.0 ? SoftmaxAlgorithm::Fast : SoftmaxAlgorithm::Accurate, mode)};
        }
        throw std::invalid_argument("Unknown parameterised Expression method: " + m);)
}

thor_expr_t thor_expr_where(thor_expr_t condition, thor_expr_t true_value, thor_expr_t false_value) {
    THOR_CAPI_TRY_PTR(require(condition, "expression"); require(true_value, "expression"); require(false_value, "expression");
                      return new thor_expr{Expression::where(condition->expr, true_value->expr, false_value->expr)};)
}
thor_expr_t thor_expr_cast(thor_expr_t input, int dtype) {
    THOR_CAPI_TRY_PTR(require(input, "expression"); (void)dataTypeSizeInBytes(static_cast<DataType>(dtype));
                      return new thor_expr{input->expr.cast(static_cast<DataType>(dtype))};)
}
thor_expr_t thor_expr_with_dtypes(thor_expr_t input, int compute_dtype, int output_dtype) {
    THOR_CAPI_TRY_PTR(require(input, "expression");
                      return new thor_expr{input->expr.withDTypes(optionalDType(compute_dtype), optionalDType(output_dtype))};)
}

thor_expr_t thor_expr_reduce(const char* method, thor_expr_t input, const uint64_t* axes, int num_axes, const uint64_t* squeeze_axes,
                             int num_squeeze_axes) {
    THOR_CAPI_TRY_PTR(
        require(input, "expression");
        static const std::unordered_map<std::string, ExprOp> ops = {
            {"reduce_sum", ExprOp::REDUCE_SUM},     {"reduce_prod", ExprOp::REDUCE_PROD},   {"reduce_min", ExprOp::REDUCE_MIN},
            {"reduce_max", ExprOp::REDUCE_MAX},     {"reduce_mean", ExprOp::REDUCE_AVG},    {"reduce_norm1", ExprOp::REDUCE_NORM1},
            {"reduce_norm2", ExprOp::REDUCE_NORM2}, {"argmin", ExprOp::REDUCE_ARGMIN},      {"argmax", ExprOp::REDUCE_ARGMAX}};
        auto it = ops.find(method ? method : "");
        if (it == ops.end()) throw std::invalid_argument(std::string("Unknown reduction method: ") + (method ? method : "(null)"));
        return new thor_expr{input->expr.reduction(it->second, u64s(axes, num_axes), u64s(squeeze_axes, num_squeeze_axes), std::nullopt)};)
}
thor_expr_t thor_expr_strided_view(thor_expr_t input, const uint64_t* dims, const uint64_t* strides, int rank, uint64_t element_offset) {
    THOR_CAPI_TRY_PTR(require(input, "expression"); if (rank < 0 || (rank > 0 && (!dims || !strides))) throw std::invalid_argument("strided view needs dims and strides.");
                      return new thor_expr{input->expr.stridedView(std::vector<uint64_t>(dims, dims + rank), std::vector<uint64_t>(strides, strides + rank),
                                                                   element_offset)};)
}
thor_expr_t thor_expr_scan(thor_expr_t input, thor_expr_t offsets, int op, int64_t axis, int inclusive, int reverse) {
    THOR_CAPI_TRY_PTR(require(input, "input"); if (op < 0 || op > 5) throw std::invalid_argument("scan op must be 0..5");
                      const ScanOp scanOp = static_cast<ScanOp>(op);
                      if (offsets) return new thor_expr{input->expr.segmentedScan(offsets->expr, scanOp, inclusive != 0, reverse != 0)};
                      return new thor_expr{reverse ? input->expr.reverseScan(scanOp, axis, inclusive != 0) : input->expr.scan(scanOp, axis, inclusive != 0)};)
}
thor_expr_t thor_expr_take_along_axis(thor_expr_t input, thor_expr_t indices, int64_t axis) {
    THOR_CAPI_TRY_PTR(require(input, "input"); require(indices, "indices"); return new thor_expr{input->expr.takeAlongAxis(indices->expr, axis)};)
}
thor_expr_t thor_expr_rope(thor_expr_t input, thor_expr_t position_ids, thor_expr_t effective_sequence_length, const thor_rope_options* options) {
    THOR_CAPI_TRY_PTR(
        require(input, "input"); if (!options) throw std::invalid_argument("rope needs options.");
        if (options->scaling_kind < 0 || options->scaling_kind > 5) throw std::invalid_argument("rope scaling_kind must be 0..5");
        if (options->num_long_rope_factors > 0 && (!options->long_rope_short_factors || !options->long_rope_long_factors)) {
            throw std::invalid_argument("rope needs both LongRoPE factor lists.");
        }
        RotaryPositionEmbeddingOptions o;
        o.sequence_axis = options->sequence_axis; o.head_dim_axis = options->head_dim_axis; o.rotary_dim = options->rotary_dim; o.base = options->base;
        o.position_offset = options->position_offset; o.interleaved = options->interleaved != 0; o.inverse = options->inverse != 0;
        o.scaling_kind = static_cast<RotaryScalingKind>(options->scaling_kind); o.scaling_factor = options->scaling_factor;
        o.original_max_position_embeddings = options->original_max_position_embeddings;
        if (options->attention_factor > 0.0) o.attention_factor = options->attention_factor;
        o.yarn_beta_fast = options->yarn_beta_fast; o.yarn_beta_slow = options->yarn_beta_slow;
        o.llama3_low_freq_factor = options->llama3_low_freq_factor; o.llama3_high_freq_factor = options->llama3_high_freq_factor;
        if (options->num_long_rope_factors > 0) {
            o.long_rope_short_factors.assign(options->long_rope_short_factors, options->long_rope_short_factors + options->num_long_rope_factors);
            o.long_rope_long_factors.assign(options->long_rope_long_factors, options->long_rope_long_factors + options->num_long_rope_factors);
        }
        o.output_dtype = optionalDType(options->output_dtype); o.compute_dtype = optionalDType(options->compute_dtype);
        if (position_ids && effective_sequence_length) {
            return new thor_expr{input->expr.rotaryPositionEmbeddingWithPositionIdsAndEffectiveSequenceLength(position_ids->expr, effective_sequence_length->expr, o)};
        }
        if (position_ids) return new thor_expr{input->expr.rotaryPositionEmbeddingWithPositionIds(position_ids->expr, o)};
        if (effective_sequence_length) return new thor_expr{input->expr.rotaryPositionEmbeddingWithEffectiveSequenceLength(effective_sequence_length->expr, o)};
        return new thor_expr{input->expr.rotaryPositionEmbedding(o)};)
}
thor_expr_t thor_expr_reshape(thor_expr_t input, const uint64_t* dims, int rank) {
    THOR_CAPI_TRY_PTR(require(input, "expression"); return new thor_expr{input->expr.reshape(u64s(dims, rank))};)
}
thor_expr_t thor_expr_unsqueeze(thor_expr_t input, const uint64_t* axes, int num_axes) {
    THOR_CAPI_TRY_PTR(require(input, "expression"); return new thor_expr{input->expr.unsqueeze(u64s(axes, num_axes))};)
}
thor_expr_t thor_expr_squeeze(thor_expr_t input, const uint64_t* axes, int num_axes) {
    THOR_CAPI_TRY_PTR(require(input, "expression"); return new thor_expr{input->expr.squeeze(u64s(axes, num_axes))};)
}
void thor_expr_destroy(thor_expr_t expr) { delete expr; }
int thor_expr_num_nodes(thor_expr_t expr) { return expr ? static_cast<int>(expr->expr.expression().nodes.size()) : -1; }
int thor_expr_canonical(thor_expr_t expr, char* buffer, size_t capacity, size_t* needed) {
    THOR_CAPI_TRY_INT(require(expr, "expression"); copyOut(canonicalize(expr->expr.expression()), buffer, capacity, needed);)
}

thor_outputs_t thor_outputs_create(const char* const* names, const thor_expr_t* exprs, int count) {
    THOR_CAPI_TRY_PTR(
        std::vector<std::pair<std::string, Expression>> named;
        for (int i = 0; i < count; ++i) {
            if (names[i] == nullptr || exprs[i] == nullptr) throw std::invalid_argument("NULL name or expression in thor_outputs_create");
            named.emplace_back(names[i], exprs[i]->expr);
        }
        return new thor_outputs{Expression::outputs(named)};)
}
void thor_outputs_destroy(thor_outputs_t outputs) { delete outputs; }
thor_outputs_t thor_outputs_conditional(thor_expr_t predicate, thor_outputs_t then_outputs, const thor_expr_t* elif_predicates,
                                        const thor_outputs_t* elif_outputs, int num_elif, thor_outputs_t else_outputs) {
    THOR_CAPI_TRY_PTR(
        require(predicate, "predicate"); require(then_outputs, "then outputs"); require(else_outputs, "else outputs");
        if (num_elif <= 0) return new thor_outputs{Outputs::ifElse(predicate->expr, then_outputs->outputs, else_outputs->outputs)};
        std::vector<std::pair<Expression, Outputs>> branches;
        for (int i = 0; i < num_elif; ++i) {
            if (elif_predicates[i] == nullptr || elif_outputs[i] == nullptr) throw std::invalid_argument("NULL elif predicate or outputs");
            branches.emplace_back(elif_predicates[i]->expr, elif_outputs[i]->outputs);
        }
        return new thor_outputs{Outputs::ifElifElse(predicate->expr, then_outputs->outputs, branches, else_outputs->outputs)};)
}

// ---- FusedEquation ------------------------------------------------------------------------------------------------------------
thor_fused_equation_t thor_fused_equation_compile(thor_outputs_t outputs, int device_num) {
    THOR_CAPI_TRY_PTR(require(outputs, "outputs"); return new thor_fused_equation{FusedEquation::compile(outputs->outputs.physicalOutputs(), device_num)};)
}
thor_fused_equation_t thor_fused_equation_compile_backward(thor_fused_equation_t eq, const char* const* wrt_names, int num_wrt,
                                                           const char* const* upstream_output_names, const char* const* upstream_input_names,
                                                           int num_upstream, int accumulate_grad_outputs) {
    THOR_CAPI_TRY_PTR(
        require(eq, "equation"); std::vector<std::string> wrt; for (int i = 0; i < num_wrt; ++i) wrt.emplace_back(wrt_names[i]);
        if (num_upstream == 0) return new thor_fused_equation{eq->equation.compileBackward(wrt, std::nullopt, accumulate_grad_outputs != 0)};
        if (!upstream_input_names) throw std::invalid_argument("upstream_input_names is null");
        if (!upstream_output_names) {
            if (num_upstream != 1) throw std::invalid_argument("a single upstream input name needs num_upstream == 1");
            return new thor_fused_equation{eq->equation.compileBackward(wrt, std::string(upstream_input_names[0]), accumulate_grad_outputs != 0)};
        }
        std::unordered_map<std::string, std::string> byOutput;
        for (int i = 0; i < num_upstream; ++i) byOutput[upstream_output_names[i]] = upstream_input_names[i];
        return new thor_fused_equation{eq->equation.compileBackward(wrt, byOutput, accumulate_grad_outputs != 0)};)
}
void thor_fused_equation_destroy(thor_fused_equation_t eq) { delete eq; }
int thor_fused_equation_num_outputs(thor_fused_equation_t eq) { return eq ? static_cast<int>(eq->equation.getOutputNames().size()) : -1; }
int thor_fused_equation_output_name(thor_fused_equation_t eq, int index, char* buffer, size_t capacity) {
    THOR_CAPI_TRY_INT(require(eq, "equation"); copyOut(eq->equation.getOutputNames().at(index), buffer, capacity, nullptr);)
}

thor_plan_t thor_fused_equation_stamp(thor_fused_equation_t eq, const char* const* input_names, const thor_tensor_t* inputs, int num_inputs,
                                      const char* const* preallocated_names, const thor_tensor_t* preallocated, int num_preallocated,
                                      thor_stream_t stream) {
    THOR_CAPI_TRY_PTR(require(eq, "equation"); require(stream, "stream");
                      return new thor_plan{eq->equation.stamp(tensorMap(input_names, inputs, num_inputs), stream->stream, {},
                                                              tensorMap(preallocated_names, preallocated, num_preallocated))};)
}

thor_plan_t thor_fused_equation_stamp_with_tensor_scalars(thor_fused_equation_t eq, const char* const* input_names, const thor_tensor_t* inputs,
                                                          int num_inputs, const char* const* scalar_names, const thor_tensor_t* scalar_buffers,
                                                          const uint64_t* scalar_byte_offsets, const int* scalar_dtypes, int num_scalars,
                                                          const char* const* preallocated_names, const thor_tensor_t* preallocated,
                                                          int num_preallocated, thor_stream_t stream) {
    THOR_CAPI_TRY_PTR(require(eq, "equation"); require(stream, "stream"); std::unordered_map<std::string, TensorScalarBinding> bindings;
                      for (int i = 0; i < num_scalars; ++i) {
                          require(scalar_buffers[i], "tensor scalar buffer");
                          bindings[scalar_names[i]] = TensorScalarBinding{scalar_buffers[i]->tensor, scalar_byte_offsets ? scalar_byte_offsets[i] : 0,
                                                                          static_cast<DataType>(scalar_dtypes[i])};
                      } return new thor_plan{eq->equation.stamp(tensorMap(input_names, inputs, num_inputs), stream->stream, bindings,
                                                                tensorMap(preallocated_names, preallocated, num_preallocated))};)
}

int thor_fused_equation_run(thor_fused_equation_t eq, const char* const* input_names, const thor_tensor_t* inputs, int num_inputs,
                            const char* const* scalar_names, const float* scalars, int num_scalars, const char* const* output_names,
                            const thor_tensor_t* outputs, int num_outputs, thor_stream_t stream) {
    THOR_CAPI_TRY_INT(require(eq, "equation"); require(stream, "stream");
                      std::unordered_map<std::string, Tensor> outs = tensorMap(output_names, outputs, num_outputs);
                      eq->equation.run(tensorMap(input_names, inputs, num_inputs), scalarMap(scalar_names, scalars, num_scalars), outs, stream->stream);)
}

int thor_fused_equation_output_shape(thor_fused_equation_t eq, const char* const* input_names, const thor_tensor_t* inputs, int num_inputs,
                                     const char* output_name, uint64_t* dims_out, int* rank_out, int* dtype_out) {
    THOR_CAPI_TRY_INT(
        require(eq, "equation");
        const auto map = tensorMap(input_names, inputs, num_inputs);
        const auto shapes = eq->equation.getOutputShapes(map);
        const auto dtypes = eq->equation.getOutputDataTypes(map);
        auto it = shapes.find(output_name ? output_name : "");
        if (it == shapes.end()) throw std::runtime_error(std::string("No such output: ") + (output_name ? output_name : "(null)"));
        if (rank_out) *rank_out = static_cast<int>(it->second.size());
        if (dims_out) std::copy(it->second.begin(), it->second.end(), dims_out);
        if (dtype_out) *dtype_out = static_cast<int>(dtypes.at(it->first));)
}

// ---- StampedExecutionPlan --------------------------------------------------------------------------------------------------------
void thor_plan_destroy(thor_plan_t plan) { delete plan; }
int thor_plan_run(thor_plan_t plan) { THOR_CAPI_TRY_INT(require(plan, "plan"); plan->plan.run();) }
int thor_plan_run_with_scalars(thor_plan_t plan, const char* const* scalar_names, const float* scalars, int num_scalars) {
    THOR_CAPI_TRY_INT(require(plan, "plan"); plan->plan.run(scalarMap(scalar_names, scalars, num_scalars));)
}
int thor_plan_run_on(thor_plan_t plan, thor_stream_t stream) {
    THOR_CAPI_TRY_INT(require(plan, "plan"); require(stream, "stream"); plan->plan.runOn(stream->stream);)
}
thor_tensor_t thor_plan_output(thor_plan_t plan, const char* name) {
    THOR_CAPI_TRY_PTR(require(plan, "plan"); return new thor_tensor{name ? plan->plan.output(name) : plan->plan.output()};)
}
int thor_plan_num_stages(thor_plan_t plan) { return plan ? static_cast<int>(plan->plan.stages().size()) : -1; }
int thor_plan_stage_kind(thor_plan_t plan, int stage, char* buffer, size_t capacity) {
    THOR_CAPI_TRY_INT(require(plan, "plan"); copyOut(plan->plan.stageKindNames().at(stage), buffer, capacity, nullptr);)
}
int thor_plan_stage_source(thor_plan_t plan, int stage, char* buffer, size_t capacity, size_t* needed) {
    THOR_CAPI_TRY_INT(require(plan, "plan"); const StampedExecutionStage& s = plan->plan.stages().at(stage);
                      copyOut(s.kernel ? s.kernel->getCompiledKernel()->source()
                                       : (s.fused_reduction ? s.fused_reduction->getLaunchPlan().mainKernel->source() : std::string()),
                              buffer, capacity, needed);)
}
int thor_plan_stage_description(thor_plan_t plan, int stage, char* buffer, size_t capacity) {
    THOR_CAPI_TRY_INT(
        require(plan, "plan"); const StampedExecutionStage& s = plan->plan.stages().at(stage);
        std::string text;
        if (s.kernel) text = s.kernel->getDescription();
        if (s.reduction) text = s.reduction->getStamped()->getKernelVariant();
        if (s.fused_reduction) text = s.fused_reduction->getDescription();
        if (s.segmented_reduction) text = s.segmented_reduction->getStamped()->getKernelVariant();
        if (s.segmented_arg_reduction) text = s.segmented_arg_reduction->getKernelVariant();
        if (s.segmented_broadcast) text = s.segmented_broadcast->getKernelVariant();
        if (s.scan) text = s.scan->getKernelVariant();
        copyOut(text, buffer, capacity, nullptr);)
}
uint64_t thor_plan_flop_count(thor_plan_t plan) { return plan ? plan->plan.flopCount() : 0; }
uint64_t thor_compiled_kernel_count(void) { return compiledKernelCount(); }

}  // extern "C"
