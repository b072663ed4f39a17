// Expression: an immutable DAG of elementwise, broadcast, cast, shape and reduction operations over named tensor
// inputs, built with ordinary C++ operators and lowered by FusedEquation into gfx950 kernels.
//
// The public surface (class names, method names, argument meaning, the ExprOp numbering and the way activations
// decompose into primitive nodes) follows the reference so that its callers compile against this header unchanged:
// Utilities/Expression/Expression.h:32-148 (ops), :231-371 (node), :516-1075 (API), :1077-1115 (stable activations),
// Utilities/Expression/Expression.cpp:4176-4193,5185-5190 (activation macros).
//
// Operations of the reference that sit outside this path (matmul, convolution, attention, RMSNorm, embedding, cuDNN softmax,
// user kernels) keep their ExprOp codes so serialized graphs stay readable, but have no builder here and are rejected by
// the compiler.
#pragma once

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"

#include <cstdint>
#include <initializer_list>
#include <memory>
#include <optional>
#include <set>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace ThorImplementation {

class Expression;
class Outputs;

// clang-format off
enum class ExprOp : uint16_t {
    INPUT = 3, RUNTIME_SCALAR, TENSOR_RUNTIME_SCALAR, SCALAR_FP,
    ADD, SUB, MUL, DIV, POW,
    EQUAL, NOT_EQUAL, LESS, LESS_EQUAL, GREATER, GREATER_EQUAL,
    LOGICAL_AND, LOGICAL_OR, LOGICAL_NOT, CAST, WHERE,
    NEG, ABS, CEIL, FLOOR, ROUND, TRUNC,
    SIN, COS, TAN, ASIN, ACOS, ATAN, SINH, COSH, ASINH, ACOSH, ATANH,
    ERF, ERFC, ERFCX, ERFINV, ERFCINV, TGAMMA, LGAMMA, DIGAMMA,
    EXP, EXPM1, EXP2, EXP10, LN, LOG1P, LOG2, LOG10, SQRT, TANH, NORMCDF,
    ROPE, SOFTMAX, FILL, RESHAPE, STRIDED_VIEW, STRIDED_VIEW_BACKWARD, UNSQUEEZE, SQUEEZE, TRANSPOSE, TAKE_ALONG_AXIS,
    MIN, MAX, MIN_GRAD_LEFT, MIN_GRAD_RIGHT, MAX_GRAD_LEFT, MAX_GRAD_RIGHT,
    MATMUL, GEMM, CONV2D, CONV2D_BACKWARD_DATA, CONV2D_BACKWARD_FILTER, CONV3D, CONV3D_BACKWARD_DATA, CONV3D_BACKWARD_FILTER,
    REDUCE_SUM, REDUCE_PROD, REDUCE_MIN, REDUCE_MAX, REDUCE_ARGMIN, REDUCE_ARGMAX,
    REDUCE_MIN_BACKWARD, REDUCE_MAX_BACKWARD, SCAN_MIN_BACKWARD, SCAN_MAX_BACKWARD,
    SEGMENTED_SCAN_MIN_BACKWARD, SEGMENTED_SCAN_MAX_BACKWARD,
    REDUCE_AVG, REDUCE_NORM1, REDUCE_NORM2,
    SCAN, RMSNORM, RMSNORM_BACKWARD_X, RMSNORM_BACKWARD_SCALE,
    ATTENTION, ATTENTION_BACKWARD_Q, ATTENTION_BACKWARD_K, ATTENTION_BACKWARD_V, ATTENTION_BACKWARD_BIAS,
    EMBEDDING_LOOKUP, CUDA_KERNEL_OUTPUT, SEGMENTED_SCAN,
    SEGMENTED_REDUCE_SUM, SEGMENTED_REDUCE_MIN, SEGMENTED_REDUCE_MAX, RAGGED_VALUEWISE_EXTENT, SEGMENTED_REDUCE_MEAN,
    SEGMENTED_BROADCAST, SEGMENTED_REDUCE_MIN_BACKWARD, SEGMENTED_REDUCE_MAX_BACKWARD,
};
// clang-format on

inline bool isValueReductionOp(ExprOp op) {
    switch (op) {
        case ExprOp::REDUCE_SUM:
        case ExprOp::REDUCE_PROD:
        case ExprOp::REDUCE_MIN:
        case ExprOp::REDUCE_MAX:
        case ExprOp::REDUCE_AVG:
        case ExprOp::REDUCE_NORM1:
        case ExprOp::REDUCE_NORM2:
            return true;
        default:
            return false;
    }
}
// Softmax spellings of the reference (it takes cuDNN's enums: Expression.h:736-738 there).  Channel = over axis 1 for every
// other coordinate (NCHW semantics; the last axis of an [N, C] matrix), Instance = over every axis but the first.
enum class SoftmaxAlgorithm : uint8_t { Fast = 0, Accurate = 1, Log = 2 };
enum class SoftmaxMode : uint8_t { Instance = 0, Channel = 1 };
}  // namespace ThorImplementation

// The two enumerations the reference's softmax signatures are spelled with (Expression.h:736-738 there; they come from cudnn.h),
// under cuDNN's type names, enumerator names and values, so that a caller written against the reference compiles unchanged:
// `x.softmax(CUDNN_SOFTMAX_ACCURATE, CUDNN_SOFTMAX_MODE_CHANNEL)`.  They are names only: nothing of cuDNN is used or needed.
enum cudnnSoftmaxAlgorithm_t { CUDNN_SOFTMAX_FAST = 0, CUDNN_SOFTMAX_ACCURATE = 1, CUDNN_SOFTMAX_LOG = 2 };
enum cudnnSoftmaxMode_t { CUDNN_SOFTMAX_MODE_INSTANCE = 0, CUDNN_SOFTMAX_MODE_CHANNEL = 1 };

namespace ThorImplementation {

// Prefix scans along the last axis (Expression.h:181-193 there).  ArgMin / ArgMax return the UINT32 flattened index of the
// element that holds the running minimum / maximum (the first one among equals), 0xFFFFFFFF where the prefix is empty.
enum class ScanOp : uint8_t { Sum = 0, Min = 1, Max = 2, Product = 3, ArgMin = 4, ArgMax = 5 };
enum class ScanMode : uint8_t { Exclusive = 0, Inclusive = 1 };
inline bool isArgScanOp(ScanOp op) { return op == ScanOp::ArgMin || op == ScanOp::ArgMax; }

// Rotary position embedding (Expression.h:150-218 there).  Pair j of the rotary part of the head dimension turns by
// position * frequency(j); the scaling kinds only change the frequencies (and, for Linear, the position).
enum class RotaryScalingKind : uint8_t { None = 0, Linear = 1, DynamicNTK = 2, Yarn = 3, LongRope = 4, Llama3 = 5 };
struct RotaryPositionEmbeddingOptions {
    uint32_t sequence_axis = 2;
    uint32_t head_dim_axis = 3;
    uint64_t rotary_dim = 0;  // 0 = the whole head dimension
    double base = 10000.0;
    int64_t position_offset = 0;
    bool interleaved = false;  // pairs (2j, 2j + 1) instead of (j, j + rotary_dim / 2)
    bool inverse = false;      // turns the other way (the transpose of the rotation)
    RotaryScalingKind scaling_kind = RotaryScalingKind::None;
    double scaling_factor = 1.0;
    uint64_t original_max_position_embeddings = 0;
    std::optional<double> attention_factor = std::nullopt;
    double yarn_beta_fast = 32.0;
    double yarn_beta_slow = 1.0;
    double llama3_low_freq_factor = 1.0;
    double llama3_high_freq_factor = 4.0;
    std::vector<double> long_rope_short_factors;
    std::vector<double> long_rope_long_factors;
    std::optional<DataType> output_dtype = std::nullopt;
    // The arithmetic dtype: FP32 (the default) is the only one the rotation kernels have; anything else is refused with
    // std::invalid_argument when the node is built.
    std::optional<DataType> compute_dtype = std::nullopt;
    // A permission, not a request (the reference's planner MAY rotate a private producer's output in place when it is set;
    // its default is off because out of place benchmarked faster).  This build never uses the permission: the rotation
    // always writes a tensor of its own, which is one of the behaviours the flag allows.
    bool allow_in_place_materialization = false;
};

// reduction_axes entry standing for "every axis except axis 0"
constexpr uint64_t kReduceAllAxesButFirst = UINT64_MAX - 1;

inline bool isArgReductionOp(ExprOp op) { return op == ExprOp::REDUCE_ARGMIN || op == ExprOp::REDUCE_ARGMAX; }
inline bool isReductionOp(ExprOp op) { return isValueReductionOp(op) || isArgReductionOp(op); }

// Ops over a ragged batch: lhs holds values, rhs the row-partition offsets [B + 1] (UINT32 / UINT64), which are structure,
// not data: they take no part in dtype promotion or broadcasting.
inline bool isSegmentedReduceOp(ExprOp op) {
    return op == ExprOp::SEGMENTED_REDUCE_SUM || op == ExprOp::SEGMENTED_REDUCE_MIN || op == ExprOp::SEGMENTED_REDUCE_MAX ||
           op == ExprOp::SEGMENTED_REDUCE_MEAN;
}
// Gradient of a min/max reduction: lhs is the reduced operand, rhs the gradient of the reduction's output; the element of each
// reduction window that won (the first in logical order among equals) takes the window's gradient, every other element 0.
inline bool isWinnerRoutingOp(ExprOp op) { return op == ExprOp::REDUCE_MIN_BACKWARD || op == ExprOp::REDUCE_MAX_BACKWARD; }
// Views of the operand's storage: nothing is computed, consumers read through the view's strides.
inline bool isStorageViewOp(ExprOp op) { return op == ExprOp::STRIDED_VIEW || op == ExprOp::TRANSPOSE; }
// SCAN: lhs scanned along its last axis.  SEGMENTED_SCAN: lhs = values [N], rhs = row-partition offsets [B + 1]; every segment
// is scanned on its own.
inline bool isScanOp(ExprOp op) { return op == ExprOp::SCAN || op == ExprOp::SEGMENTED_SCAN; }
// Gradient of a min / max scan (AutoDiff.cpp:5743-5760 there): lhs = the scanned operand, rhs = the FP32 gradient of the scan's
// output, aux = the offsets of a segmented scan.  Every position's gradient goes to the element that held the running
// minimum / maximum there (the first among equals); the result is FP32, shaped like the operand.
inline bool isScanBackwardOp(ExprOp op) {
    return op == ExprOp::SCAN_MIN_BACKWARD || op == ExprOp::SCAN_MAX_BACKWARD || op == ExprOp::SEGMENTED_SCAN_MIN_BACKWARD ||
           op == ExprOp::SEGMENTED_SCAN_MAX_BACKWARD;
}
// Gradient of a per-segment min / max (AutoDiff.cpp:5630-5700 there): lhs = the packed values [N, D...], rhs = the FP32 gradient
// of the reduction's output [B, D...], aux = the offsets.  Each segment's gradient goes to the row that won the column (the
// lowest row among equals); every other element, and every row outside the partition, gets 0.  FP32, shaped like the values.
inline bool isSegmentWinnerRoutingOp(ExprOp op) { return op == ExprOp::SEGMENTED_REDUCE_MIN_BACKWARD || op == ExprOp::SEGMENTED_REDUCE_MAX_BACKWARD; }
// Stages that read up to three dense tensors (lhs, rhs, aux) and scatter gradients into a cleared FP32 tensor.
// STRIDED_VIEW_BACKWARD (AutoDiff.cpp:2100-2125 there): lhs = the FP32 gradient of a view (shaped like the view); the result has
// the operand's shape (fill_dims), holds the gradient at the elements the view addresses (view_dims / view_strides /
// view_element_offset) and 0 everywhere else.  Views that address an element twice are rejected.
inline bool isScatterRoutingOp(ExprOp op) { return isScanBackwardOp(op) || isSegmentWinnerRoutingOp(op) || op == ExprOp::STRIDED_VIEW_BACKWARD; }
inline bool isRaggedOp(ExprOp op) {
    return isSegmentedReduceOp(op) || op == ExprOp::SEGMENTED_BROADCAST || op == ExprOp::RAGGED_VALUEWISE_EXTENT;
}

// One vertex of the DAG.  Children are indices into PhysicalExpression::nodes and always precede their consumer.
struct ExprNode {
    ExprOp op = ExprOp::SCALAR_FP;
    uint32_t lhs = UINT32_MAX;
    uint32_t rhs = UINT32_MAX;
    uint32_t aux = UINT32_MAX;         // third operand (WHERE: lhs = condition, rhs = true value, aux = false value)
    uint32_t input_slot = UINT32_MAX;  // INPUT / RUNTIME_SCALAR only
    double scalar_fp = 0.0;            // SCALAR_FP / FILL only

    // INPUT / RUNTIME_SCALAR: dtype of the value actually bound at stamp time (filled in by dtype resolution).
    std::optional<DataType> input_tensor_dtype;
    // Value semantics: the dtype the node's value has in the graph, and the dtype its arithmetic runs in.
    std::optional<DataType> output_dtype;
    std::optional<DataType> compute_dtype;

    std::vector<uint64_t> reduction_axes;  // reductions: empty = all axes
    std::vector<uint64_t> squeeze_axes;    // reductions and SQUEEZE; {UINT64_MAX} = every singleton axis
    std::vector<uint64_t> unsqueeze_axes;
    std::vector<uint64_t> reshape_dims;    // one entry may be UINT64_MAX = inferred
    std::vector<uint64_t> fill_dims;
    // STRIDED_VIEW: shape, strides and first element of the view, in elements of the operand's storage
    std::vector<uint64_t> view_dims, view_strides;
    uint64_t view_element_offset = 0;
    // SCAN / SEGMENTED_SCAN: scan_axis UINT64_MAX = the last axis
    ScanOp scan_op = ScanOp::Sum;
    ScanMode scan_mode = ScanMode::Inclusive;
    uint64_t scan_axis = UINT64_MAX;
    bool scan_reverse = false;
    // ROPE (Expression.h:293-318 there): lhs = values; rhs = position ids (rope_position_ids_node there: one absolute
    // position per element of the sequence axis) and aux = effective sequence length (rope_effective_sequence_length_node
    // there: one element, read on the device at run time), UINT32_MAX where absent.
    uint32_t rope_sequence_axis = 2;
    uint32_t rope_head_dim_axis = 3;
    uint64_t rope_rotary_dim = 0;
    double rope_base = 10000.0;
    int64_t rope_position_offset = 0;
    bool rope_interleaved = false;
    bool rope_inverse = false;
    RotaryScalingKind rope_scaling_kind = RotaryScalingKind::None;
    double rope_scaling_factor = 1.0;
    uint64_t rope_original_max_position_embeddings = 0;
    double rope_attention_factor = 1.0;
    double rope_yarn_beta_fast = 32.0;
    double rope_yarn_beta_slow = 1.0;
    double rope_llama3_low_freq_factor = 1.0;
    double rope_llama3_high_freq_factor = 4.0;
    std::vector<double> rope_long_rope_short_factors;
    std::vector<double> rope_long_rope_long_factors;
    SoftmaxAlgorithm softmax_algorithm = SoftmaxAlgorithm::Accurate;  // SOFTMAX only
    SoftmaxMode softmax_mode = SoftmaxMode::Channel;

    // Ragged ops (reference: Expression.h:336-343 there): the batch size B, the capacity of the packed values tensor in
    // rows, and the elements one row holds.  Zero batch size = not given (segmented reductions take both from the bound
    // tensors then).
    uint64_t ragged_runtime_batch_size = 0;
    uint64_t ragged_runtime_max_active_values = 0;
    uint64_t ragged_runtime_elements_per_value = 1;
    bool segmented_broadcast_normalize_by_length = false;
};

// The axes a reduction node reduces for an input of `rank` dimensions: sorted, unique, validated ({} = all).
std::vector<uint64_t> resolveReductionAxes(const std::vector<uint64_t>& reduction_axes, size_t rank);

struct NamedInput {
    enum class Kind : uint8_t { Tensor, RuntimeScalarFp32, TensorRuntimeScalar };
    std::string name;
    uint32_t slot = 0;
    Kind kind = Kind::Tensor;
};

struct NamedOutput {
    std::string name;
    uint32_t node_idx = UINT32_MAX;
};

struct PhysicalExpression {
    std::vector<ExprNode> nodes;
    std::vector<NamedInput> inputs;
    uint32_t output_node = UINT32_MAX;

    uint32_t numInputs() const { return static_cast<uint32_t>(inputs.size()); }
    uint32_t getOrCreateInputSlot(const std::string& name, NamedInput::Kind kind = NamedInput::Kind::Tensor);
    std::set<std::string> getInputNames() const {
        std::set<std::string> names;
        for (const NamedInput& in : inputs) names.insert(in.name);
        return names;
    }
};

struct PhysicalOutputs {
    std::shared_ptr<PhysicalExpression> expr;
    std::vector<NamedOutput> outputs;
};

class Outputs {
   public:
    const std::shared_ptr<PhysicalExpression>& expression() const { return expr; }
    const std::vector<NamedOutput>& namedOutputs() const { return outputs; }
    PhysicalOutputs physicalOutputs() const;
    static Outputs fromPhysicalOutputs(PhysicalOutputs physicalOutputs);

    // Outputs that take, name by name, the then-branch's value where `predicate` (a single element, read on the device at every
    // run) is nonzero and the else-branch's value otherwise (reference: Expression.h:474-483, Expression.cpp:5342-5390 there).
    // The reference runs one branch through a conditional graph node; this build evaluates both branches and selects element
    // by element (`where(predicate != 0, then, else)`), which gives the same outputs for these side-effect-free expressions -
    // values of the branch not taken, NaNs included, never reach an output - usually inside one fused kernel, and the same
    // gradients (a gradient flows into the branch that was taken).  The result is an ordinary Outputs: isConditional() is false
    // and a stamped plan shows the stages of the selection, not a Conditional stage.
    static Outputs conditional(const Expression& predicate, const Outputs& then_outputs, const Outputs& else_outputs);
    static Outputs ifElse(const Expression& predicate, const Outputs& then_outputs, const Outputs& else_outputs) {
        return conditional(predicate, then_outputs, else_outputs);
    }
    static Outputs ifElifElse(const Expression& predicate, const Outputs& then_outputs, const std::vector<std::pair<Expression, Outputs>>& elif_branches,
                              const Outputs& else_outputs);
    bool isConditional() const { return false; }

   private:
    Outputs(std::shared_ptr<PhysicalExpression> expr, std::vector<NamedOutput> outputs) : expr(std::move(expr)), outputs(std::move(outputs)) {}
    std::shared_ptr<PhysicalExpression> expr;
    std::vector<NamedOutput> outputs;
    friend class Expression;
};

class Expression {
   public:
    Expression(double value);  // implicit on purpose: `x + 2.0`

    // One of a small pool of helper streams of `gpu_num`, handed out in turn (reference: Expression.h:518, Expression.cpp:48-55).
    // Stamped plans run their independent branches on them.  The pool holds as many streams as a process has hardware queues
    // (4): more streams would share queues and overlap nothing more.  Streams are created on first use, at default priority.
    static Stream& getNextHelperStream(uint32_t gpu_num);

    static Expression input(const std::string& name, std::optional<DataType> compute_dtype = std::nullopt,
                            std::optional<DataType> output_dtype = std::nullopt);
    static Expression runtimeScalar(const std::string& name, std::optional<DataType> compute_dtype = std::nullopt,
                                    std::optional<DataType> output_dtype = std::nullopt);
    // A scalar read from device memory at every run (bound with a TensorScalarBinding at stamp time); like a runtime scalar
    // it takes no part in dtype promotion (Expression.cpp:3101-3120 there).
    static Expression tensorRuntimeScalar(const std::string& name, std::optional<DataType> compute_dtype = std::nullopt,
                                          std::optional<DataType> output_dtype = std::nullopt);
    static Expression constantScalar(double value);
    static Expression fill(double value, const std::vector<uint64_t>& dims, std::optional<DataType> output_dtype = std::nullopt);

    static Outputs outputs(const std::vector<std::pair<std::string, Expression>>& named_exprs);
    static Outputs outputs(std::initializer_list<std::pair<std::string, Expression>> named_exprs);

    static Expression fromPhysicalNode(std::shared_ptr<PhysicalExpression> expr, uint32_t nodeIndex);
    PhysicalExpression expression() const;
    std::set<std::string> getInputNames() const;
    bool isSameLogicalNode(const Expression& other) const {
        return expr && other.expr && expr.get() == other.expr.get() && nodeIndex == other.nodeIndex;
    }

    // ---- arithmetic, comparison, logic --------------------------------------------------------------------------
    Expression operator+(const Expression& other) const;
    Expression operator-(const Expression& other) const;
    Expression operator*(const Expression& other) const;
    Expression operator/(const Expression& other) const;
    Expression operator-() const;
    Expression operator!() const;
    Expression operator==(const Expression& other) const;
    Expression operator!=(const Expression& other) const;
    Expression operator<(const Expression& other) const;
    Expression operator<=(const Expression& other) const;
    Expression operator>(const Expression& other) const;
    Expression operator>=(const Expression& other) const;

    Expression equal(const Expression& other) const;
    Expression notEqual(const Expression& other) const;
    Expression lessThan(const Expression& other) const;
    Expression lessEqual(const Expression& other) const;
    Expression greaterThan(const Expression& other) const;
    Expression greaterEqual(const Expression& other) const;
    Expression logicalAnd(const Expression& other) const;
    Expression logicalOr(const Expression& other) const;
    Expression logicalNot() const;
    Expression pow(const Expression& exponent) const;
    Expression min(const Expression& other) const;
    Expression max(const Expression& other) const;
    Expression cast(DataType output_dtype) const;
    Expression select(const Expression& true_value, const Expression& false_value) const;

    static Expression equal(const Expression& lhs, const Expression& rhs) { return lhs.equal(rhs); }
    static Expression notEqual(const Expression& lhs, const Expression& rhs) { return lhs.notEqual(rhs); }
    static Expression lessThan(const Expression& lhs, const Expression& rhs) { return lhs.lessThan(rhs); }
    static Expression lessEqual(const Expression& lhs, const Expression& rhs) { return lhs.lessEqual(rhs); }
    static Expression greaterThan(const Expression& lhs, const Expression& rhs) { return lhs.greaterThan(rhs); }
    static Expression greaterEqual(const Expression& lhs, const Expression& rhs) { return lhs.greaterEqual(rhs); }
    static Expression logicalAnd(const Expression& lhs, const Expression& rhs) { return lhs.logicalAnd(rhs); }
    static Expression logicalOr(const Expression& lhs, const Expression& rhs) { return lhs.logicalOr(rhs); }
    static Expression logicalNot(const Expression& input) { return input.logicalNot(); }
    static Expression cast(const Expression& input, DataType output_dtype) { return input.cast(output_dtype); }
    static Expression where(const Expression& condition, const Expression& true_value, const Expression& false_value);
    static Expression select(const Expression& condition, const Expression& true_value, const Expression& false_value) {
        return where(condition, true_value, false_value);
    }

    // ---- unary math: one primitive node each ----------------------------------------------------------------------
    Expression abs() const;
    Expression ceil() const;
    Expression floor() const;
    Expression round() const;
    Expression trunc() const;
    Expression sin() const;
    Expression cos() const;
    Expression tan() const;
    Expression asin() const;
    Expression acos() const;
    Expression atan() const;
    Expression sinh() const;
    Expression cosh() const;
    Expression tanh() const;
    Expression asinh() const;
    Expression acosh() const;
    Expression atanh() const;
    Expression erf() const;
    Expression erfc() const;
    Expression erfcx() const;
    Expression erfinv() const;
    Expression erfcinv() const;
    Expression tgamma() const;
    Expression lgamma() const;
    Expression digamma() const;
    Expression exp() const;
    Expression expm1() const;
    Expression exp2() const;
    Expression exp10() const;
    Expression ln() const;
    Expression log1p() const;
    Expression log2() const;
    Expression log10() const;
    Expression sqrt() const;
    static Expression sqrt(const Expression& expr) { return expr.sqrt(); }
    Expression normcdf() const;

    // ---- compositions of the primitives above ---------------------------------------------------------------------
    Expression csc() const;
    Expression sec() const;
    Expression cot() const;
    Expression acsc() const;
    Expression asec() const;
    Expression acot() const;
    Expression csch() const;
    Expression sech() const;
    Expression coth() const;
    Expression acsch() const;
    Expression asech() const;
    Expression acoth() const;
    Expression log(double base) const;
    Expression clamp(const Expression& lower_bound, const Expression& upper_bound) const;
    Expression clamp(double lower_bound, double upper_bound) const;
    static Expression clamp(const Expression& input, const Expression& lower_bound, const Expression& upper_bound) {
        return input.clamp(lower_bound, upper_bound);
    }
    static Expression clamp(const Expression& input, double lower_bound, double upper_bound) { return input.clamp(lower_bound, upper_bound); }

    // Numerically stable activation shapes.
    Expression sigmoid() const;
    Expression softplus() const;
    Expression elu(double alpha = 1.0) const;
    Expression selu() const;
    Expression gelu() const;
    Expression mish() const;
    Expression relu6() const;
    Expression hardTanh(double min_value = -1.0, double max_value = 1.0) const;
    Expression hardSwish() const;
    Expression threshold(double threshold = 0.0, double value = 0.0) const;
    Expression swish() const;

    // softmax / log-softmax over the channel axis (or over everything but the batch axis), fp32 arithmetic, result in
    // the input's dtype (fp16 for fp8 inputs).  Lowered to max / exp / sum / divide, which a [N, C] input runs as one
    // register-resident row kernel.
    Expression softmax(SoftmaxAlgorithm algorithm = SoftmaxAlgorithm::Accurate, SoftmaxMode mode = SoftmaxMode::Channel) const;
    Expression logSoftmax(SoftmaxMode mode = SoftmaxMode::Channel) const;
    // the reference's spelling of the same two (the enumerators map one to one)
    Expression softmax(cudnnSoftmaxAlgorithm_t algorithm, cudnnSoftmaxMode_t mode = CUDNN_SOFTMAX_MODE_CHANNEL) const {
        return softmax(static_cast<SoftmaxAlgorithm>(algorithm), static_cast<SoftmaxMode>(mode));
    }
    Expression logSoftmax(cudnnSoftmaxMode_t mode) const { return logSoftmax(static_cast<SoftmaxMode>(mode)); }

    // ---- shape -------------------------------------------------------------------------------------------------------
    Expression reshape(const std::vector<uint64_t>& new_dims) const;
    Expression unsqueeze(const std::vector<uint64_t>& unsqueeze_axes) const;
    Expression squeeze(const std::vector<uint64_t>& squeeze_axes) const;
    // A view of the operand's storage (reference: Expression.cpp:3769-3787 there): `strides_elements` and `element_offset`
    // address the storage of the tensor the operand resolves to, not the logical index space of an earlier view.  Nothing is
    // copied; kernels read through the strides.
    Expression stridedView(const std::vector<uint64_t>& dims, const std::vector<uint64_t>& strides_elements, uint64_t element_offset = 0) const;
    // The gradient of stridedView(view_dims, view_strides_elements, view_element_offset) of a tensor shaped source_dims: this
    // expression is the FP32 gradient of the view; the result is FP32, shaped source_dims, zero where the view does not reach.
    Expression stridedViewBackward(const std::vector<uint64_t>& source_dims, const std::vector<uint64_t>& view_dims,
                                   const std::vector<uint64_t>& view_strides_elements, uint64_t view_element_offset = 0) const;
    Expression aliasView(const std::vector<uint64_t>& dims, const std::vector<uint64_t>& strides_elements, uint64_t element_offset = 0) const {
        return stridedView(dims, strides_elements, element_offset);
    }
    // The last two axes exchanged (rank >= 2), as a view.
    Expression transpose() const;
    // Prefix scans along the last axis (axis = -1 or the index of the last axis), and over the segments of a row partition
    // (values [N], offsets [B + 1]); `reverse` scans from the end of every row / segment.  Values are UINT32, FP16, BF16 or
    // FP32 and keep their dtype; arg scans return UINT32 (Expression.h:640-700, Expression.cpp:3866-3960 there).
    Expression scan(ScanOp op = ScanOp::Sum, int64_t axis = -1, bool inclusive = true) const;
    static Expression scan(const Expression& input, ScanOp op, int64_t axis = -1, bool inclusive = true) { return input.scan(op, axis, inclusive); }
    Expression exclusiveScanSum(int64_t axis = -1) const { return scan(ScanOp::Sum, axis, false); }
    Expression inclusiveScanSum(int64_t axis = -1) const { return scan(ScanOp::Sum, axis, true); }
    static Expression exclusiveScanSum(const Expression& input, int64_t axis = -1) { return input.scan(ScanOp::Sum, axis, false); }
    static Expression inclusiveScanSum(const Expression& input, int64_t axis = -1) { return input.scan(ScanOp::Sum, axis, true); }
    static Expression prefixCount(const Expression& mask, bool inclusive = true, int64_t axis = -1) { return mask.prefixCount(inclusive, axis); }
    Expression reverseScan(ScanOp op, int64_t axis = -1, bool inclusive = true) const;
    Expression prefixCount(bool inclusive = true, int64_t axis = -1) const;  // running count of non-zero elements, UINT32
    std::pair<Expression, Expression> scanWithIndices(ScanOp op, int64_t axis = -1, bool inclusive = true) const;  // {values, indices}, Min / Max
    Expression segmentedScan(const Expression& offsets, ScanOp op = ScanOp::Sum, bool inclusive = true, bool reverse = false) const;
    static Expression segmentedScan(const Expression& input, const Expression& offsets, ScanOp op, bool inclusive = true, bool reverse = false) {
        return input.segmentedScan(offsets, op, inclusive, reverse);
    }
    static Expression segmentedScanWithRaggedMetadata(const Expression& input, const Expression& offsets, ScanOp op, bool inclusive, bool reverse,
                                                      uint64_t ragged_batch_size, uint64_t ragged_max_active_values);
    std::pair<Expression, Expression> segmentedScanWithIndices(const Expression& offsets, ScanOp op, bool inclusive = true, bool reverse = false) const;
    // Gather along one axis (the last one for axis = -1): the result has the shape of `indices` (UINT32 / UINT64), which
    // matches this tensor on every other axis; result[c] = this[c with the axis coordinate replaced by indices[c]]
    // (Expression.h:676-677, Expression.cpp:3856-3865 there).  The axis is kept in reduction_axes ({UINT64_MAX} = last).
    Expression takeAlongAxis(const Expression& indices, int64_t axis = -1) const;
    static Expression takeAlongAxis(const Expression& input, const Expression& indices, int64_t axis = -1) { return input.takeAlongAxis(indices, axis); }

    // Rotary position embedding of every [sequence, head dimension] plane of the operand (Expression.h:650-675,
    // Expression.cpp:4334-4507 there).  Explicit position ids (any numeric dtype, one per element of the sequence axis) replace
    // coordinate + position_offset; the effective sequence length (one element) replaces the extent of the sequence axis in
    // the Dynamic-NTK and LongRoPE rules.  Arithmetic is fp32; the result has output_dtype or the operand's dtype.
    Expression rotaryPositionEmbedding(RotaryPositionEmbeddingOptions options = {}) const;
    Expression rope(RotaryPositionEmbeddingOptions options = {}) const { return rotaryPositionEmbedding(std::move(options)); }
    static Expression rotaryPositionEmbedding(const Expression& input, RotaryPositionEmbeddingOptions options = {}) {
        return input.rotaryPositionEmbedding(std::move(options));
    }
    static Expression rope(const Expression& input, RotaryPositionEmbeddingOptions options = {}) { return input.rotaryPositionEmbedding(std::move(options)); }
    Expression rotaryPositionEmbeddingWithEffectiveSequenceLength(const Expression& effective_sequence_length,
                                                                  RotaryPositionEmbeddingOptions options = {}) const;
    Expression rotaryPositionEmbeddingWithPositionIds(const Expression& position_ids, RotaryPositionEmbeddingOptions options = {}) const;
    Expression rotaryPositionEmbeddingWithPositionIdsAndEffectiveSequenceLength(const Expression& position_ids,
                                                                                const Expression& effective_sequence_length,
                                                                                RotaryPositionEmbeddingOptions options = {}) const;

    // ---- reductions: fp32 accumulation, reduced axes kept as 1 unless listed in squeeze_axes ------------------------
    Expression reduction(ExprOp op, const std::vector<uint64_t>& reduction_axes, const std::vector<uint64_t>& squeeze_axes,
                         std::optional<DataType> compute_dtype) const;
    Expression reduce_sum(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                          std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression reduce_prod(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                           std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression reduce_min(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                          std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression reduce_max(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                          std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression reduce_mean(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                           std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression reduce_norm1(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                            std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression reduce_norm2(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                            std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression argmin(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                      std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression argmax(const std::vector<uint64_t>& reduction_axes = {}, const std::vector<uint64_t>& squeeze_axes = {},
                      std::optional<DataType> compute_dtype = std::nullopt) const;
    Expression dotProduct(const Expression& other, std::optional<DataType> compute_dtype = std::nullopt) const;
    static Expression dotProduct(const Expression& lhs, const Expression& rhs, std::optional<DataType> compute_dtype = std::nullopt);

    // ---- ragged batches: values [N, D...] packed row after row, offsets [B + 1] read on the device at run time -------------
    // Per-segment sum / min / max / mean -> [B, D...] in the values' dtype, fp32 accumulation (reference: Expression.cpp:3962-4008).
    static Expression segmentedReduceWithRaggedMetadata(const Expression& input, const Expression& offsets, ExprOp op, uint64_t ragged_batch_size,
                                                        uint64_t ragged_max_active_values, uint64_t ragged_elements_per_value = 1);
    Expression segmentedReduceSum(const Expression& offsets) const { return segmentedReduceSum(*this, offsets); }
    Expression segmentedReduceMin(const Expression& offsets) const { return segmentedReduceMin(*this, offsets); }
    Expression segmentedReduceMax(const Expression& offsets) const { return segmentedReduceMax(*this, offsets); }
    Expression segmentedReduceMean(const Expression& offsets) const { return segmentedReduceMean(*this, offsets); }
    static Expression segmentedReduceSum(const Expression& input, const Expression& offsets);
    static Expression segmentedReduceMin(const Expression& input, const Expression& offsets);
    static Expression segmentedReduceMax(const Expression& input, const Expression& offsets);
    static Expression segmentedReduceMean(const Expression& input, const Expression& offsets);
    // Per-segment values [B, D...] -> rows [max_active_values, D...]: every row of segment b receives values[b] (divided by
    // the segment's length on request); rows of no segment are undefined (RaggedExpression.cpp:421-430 there).
    static Expression segmentedBroadcast(const Expression& per_segment_values, const Expression& offsets, uint64_t batch_size,
                                         uint64_t max_active_values, uint64_t elements_per_value, bool normalize_by_segment_length);
    // Identity on the values that limits the kernel producing them to the first offsets[batch_size] rows; the rest of the
    // output tensor keeps its contents (Expression.cpp:4010-4032 there).  `offsets` has to be a direct input.
    Expression withRaggedRuntimeExtent(const Expression& offsets, uint64_t batch_size, uint64_t max_active_values, uint64_t elements_per_value) const;

    // ---- dtype overrides on the root node ----------------------------------------------------------------------------
    Expression withDTypes(std::optional<DataType> compute_dtype = std::nullopt, std::optional<DataType> output_dtype = std::nullopt) const;
    Expression withComputeDType(DataType compute_dtype) const { return withDTypes(compute_dtype, std::nullopt); }
    Expression withOutputDType(DataType output_dtype) const { return withDTypes(std::nullopt, output_dtype); }

    // This expression with every use of the tensor input `input_name` reading `replacement` instead.
    Expression substituteInput(const std::string& input_name, const Expression& replacement) const;

    static bool isLeafOp(ExprOp op);
    static bool isUnaryOp(ExprOp op);
    static bool isBinaryOp(ExprOp op);
    static bool isTernaryOp(ExprOp op);

   private:
    friend class Outputs;
    Expression(std::shared_ptr<PhysicalExpression> expr, uint32_t nodeIndex) : expr(std::move(expr)), nodeIndex(nodeIndex) {}
    static Expression unaryOp(const Expression& input, ExprOp op);
    static Expression binaryOp(const Expression& lhs, const Expression& rhs, ExprOp op);
    static Expression ternaryOp(const Expression& a, const Expression& b, const Expression& c, ExprOp op);
    static Expression ropeOp(const Expression& input, const Expression* position_ids, const Expression* effective_sequence_length, ExprNode node);

    std::shared_ptr<PhysicalExpression> expr;
    uint32_t nodeIndex = UINT32_MAX;
};

std::string opName(ExprOp op);
bool isCommutative(ExprOp op);
std::string formatFloatCanonical(double x);
// Every parameter of a ROPE node as text (two rotations with the same text and operands are the same computation).
std::string ropeKey(const ExprNode& n);
// Canonical text of the sub-DAG below `nodeIndex` (commutative operands ordered, shared sub-trees memoised): two graphs
// with the same text compute the same function of the same input slots.
std::string canonicalizeNode(const PhysicalExpression& expr, uint32_t nodeIndex, std::unordered_map<uint32_t, std::string>& memo);
std::string canonicalize(const PhysicalExpression& expr);
std::string canonicalize(const PhysicalOutputs& outputs);
std::string expressionHash(const PhysicalOutputs& outputs);

}  // namespace ThorImplementation
