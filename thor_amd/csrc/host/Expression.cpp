// Graph construction for Expression (reference behaviour: Utilities/Expression/Expression.cpp:3057-3296,3604-3722,
// 4176-4193,5084-5310).  Every operator builds a fresh PhysicalExpression holding copies of its operands' sub-DAGs with
// the input slots merged by name; nodes shared inside one operand are copied once.
#include "Utilities/Expression/Expression.h"

#include <algorithm>
#include <array>
#include <atomic>
#include <mutex>
#include <cmath>
#include <cstdio>
#include <functional>
#include <limits>
#include <sstream>
#include <stdexcept>
#include <unordered_set>

namespace ThorImplementation {

namespace {
struct HelperStreams {
    static constexpr uint32_t kPerGpu = 4;
    std::array<Stream, kPerGpu> streams;
    std::atomic<uint32_t> next{0};
};
}  // namespace

Stream& Expression::getNextHelperStream(uint32_t gpu_num) {
    static std::mutex mutex;
    // never destroyed: at process exit the device runtime may be gone before static destructors run
    static std::vector<std::unique_ptr<HelperStreams>>& pools = *new std::vector<std::unique_ptr<HelperStreams>>();
    HelperStreams* pool = nullptr;
    {
        std::lock_guard<std::mutex> lock(mutex);
        if (pools.size() <= gpu_num) pools.resize(gpu_num + 1);
        if (!pools[gpu_num]) {
            pools[gpu_num] = std::make_unique<HelperStreams>();
            for (Stream& s : pools[gpu_num]->streams) s = Stream(static_cast<int>(gpu_num));
        }
        pool = pools[gpu_num].get();
    }
    return pool->streams[pool->next.fetch_add(1, std::memory_order_relaxed) % HelperStreams::kPerGpu];
}


uint32_t PhysicalExpression::getOrCreateInputSlot(const std::string& name, NamedInput::Kind kind) {
    for (const NamedInput& in : inputs) {
        if (in.name == name) {
            if (in.kind != kind) throw std::runtime_error("Input kind mismatch for input: " + name);
            return in.slot;
        }
    }
    const uint32_t slot = static_cast<uint32_t>(inputs.size());
    inputs.push_back(NamedInput{name, slot, kind});
    return slot;
}

PhysicalOutputs Outputs::physicalOutputs() const {
    if (!expr) throw std::runtime_error("Outputs has no backing expression graph.");
    return PhysicalOutputs{expr, outputs};
}

Outputs Outputs::fromPhysicalOutputs(PhysicalOutputs physicalOutputs) {
    if (!physicalOutputs.expr) throw std::runtime_error("Outputs::fromPhysicalOutputs requires a non-null PhysicalExpression.");
    return Outputs(std::move(physicalOutputs.expr), std::move(physicalOutputs.outputs));
}

namespace {

void validateUserInputName(const std::string& name) {
    if (name.empty()) throw std::invalid_argument("Expression input names must not be empty.");
    if (name.rfind("__", 0) == 0) throw std::invalid_argument("Expression input names starting with '__' are reserved: " + name);
}

// Copies sub-DAGs into `dst`, keeping one copy per (source graph, source node) and one input slot per name.
class GraphMerger {
   public:
    explicit GraphMerger(PhysicalExpression& dst) : dst(dst) {
        for (const NamedInput& in : dst.inputs) slotByName[in.name] = in.slot;
    }

    // `replacedInput` (may be null): tensor inputs of that name are not copied; their consumers read node `replacement` of dst instead
    uint32_t absorb(const PhysicalExpression& src, uint32_t root, const std::string* replacedInput = nullptr, uint32_t replacement = UINT32_MAX) {
        if (root >= src.nodes.size()) throw std::runtime_error("Expression node index is out of range.");
        std::unordered_map<uint32_t, uint32_t> substitutionMemo;
        std::unordered_map<uint32_t, uint32_t>& memo = replacedInput ? substitutionMemo : memos[&src];
        // children precede parents, so an ascending sweep over the reachable set needs no recursion
        std::vector<char> needed(root + 1, 0);
        needed[root] = 1;
        for (uint32_t i = root + 1; i-- > 0;) {
            if (!needed[i]) continue;
            const ExprNode& n = src.nodes[i];
            for (uint32_t child : {n.lhs, n.rhs, n.aux}) {
                if (child == UINT32_MAX) continue;
                if (child >= i) throw std::runtime_error("Expression graph is not topologically ordered.");
                needed[child] = 1;
            }
        }
        for (uint32_t i = 0; i <= root; ++i) {
            if (!needed[i] || memo.count(i)) continue;
            ExprNode copy = src.nodes[i];
            if (replacedInput && copy.op == ExprOp::INPUT && copy.input_slot < src.inputs.size() && src.inputs[copy.input_slot].name == *replacedInput) {
                memo[i] = replacement;
                continue;
            }
            if (copy.lhs != UINT32_MAX) copy.lhs = memo.at(copy.lhs);
            if (copy.rhs != UINT32_MAX) copy.rhs = memo.at(copy.rhs);
            if (copy.aux != UINT32_MAX) copy.aux = memo.at(copy.aux);
            if (copy.op == ExprOp::INPUT || copy.op == ExprOp::RUNTIME_SCALAR || copy.op == ExprOp::TENSOR_RUNTIME_SCALAR) {
                if (copy.input_slot >= src.inputs.size()) throw std::runtime_error("Input slot out of range while combining expressions.");
                const NamedInput& in = src.inputs[copy.input_slot];
                auto it = slotByName.find(in.name);
                if (it == slotByName.end()) {
                    const uint32_t slot = static_cast<uint32_t>(dst.inputs.size());
                    dst.inputs.push_back(NamedInput{in.name, slot, in.kind});
                    it = slotByName.emplace(in.name, slot).first;
                } else if (dst.inputs[it->second].kind != in.kind) {
                    throw std::runtime_error("Input kind mismatch while combining expressions for input: " + in.name);
                }
                copy.input_slot = it->second;
            }
            memo[i] = static_cast<uint32_t>(dst.nodes.size());
            dst.nodes.push_back(std::move(copy));
        }
        return memo.at(root);
    }

   private:
    PhysicalExpression& dst;
    std::unordered_map<std::string, uint32_t> slotByName;
    std::unordered_map<const PhysicalExpression*, std::unordered_map<uint32_t, uint32_t>> memos;
};

std::vector<uint64_t> sortedUnique(std::vector<uint64_t> v) {
    std::sort(v.begin(), v.end());
    v.erase(std::unique(v.begin(), v.end()), v.end());
    return v;
}

}  // namespace

// ---- leaves ------------------------------------------------------------------------------------------------------------
Expression::Expression(double value) {
    expr = std::make_shared<PhysicalExpression>();
    ExprNode node;
    node.op = ExprOp::SCALAR_FP;
    node.scalar_fp = value;
    expr->nodes.push_back(node);
    expr->output_node = nodeIndex = 0;
}

Expression Expression::constantScalar(double value) { return Expression(value); }

static Expression makeLeaf(ExprOp op, NamedInput::Kind kind, const std::string& name, std::optional<DataType> compute_dtype,
                           std::optional<DataType> output_dtype, std::shared_ptr<PhysicalExpression>& out) {
    validateUserInputName(name);
    out = std::make_shared<PhysicalExpression>();
    ExprNode node;
    node.op = op;
    node.input_slot = out->getOrCreateInputSlot(name, kind);
    node.output_dtype = output_dtype;
    node.compute_dtype = compute_dtype;
    out->nodes.push_back(node);
    out->output_node = 0;
    return Expression::fromPhysicalNode(out, 0);
}

Expression Expression::input(const std::string& name, std::optional<DataType> compute_dtype, std::optional<DataType> output_dtype) {
    std::shared_ptr<PhysicalExpression> out;
    return makeLeaf(ExprOp::INPUT, NamedInput::Kind::Tensor, name, compute_dtype, output_dtype, out);
}

Expression Expression::runtimeScalar(const std::string& name, std::optional<DataType> compute_dtype, std::optional<DataType> output_dtype) {
    std::shared_ptr<PhysicalExpression> out;
    return makeLeaf(ExprOp::RUNTIME_SCALAR, NamedInput::Kind::RuntimeScalarFp32, name, compute_dtype, output_dtype, out);
}

Expression Expression::tensorRuntimeScalar(const std::string& name, std::optional<DataType> compute_dtype, std::optional<DataType> output_dtype) {
    std::shared_ptr<PhysicalExpression> out;
    return makeLeaf(ExprOp::TENSOR_RUNTIME_SCALAR, NamedInput::Kind::TensorRuntimeScalar, name, compute_dtype, output_dtype, out);
}

Expression Expression::fill(double value, const std::vector<uint64_t>& dims, std::optional<DataType> output_dtype) {
    if (dims.empty()) throw std::invalid_argument("Expression::fill requires non-empty concrete dimensions; use constantScalar for a scalar.");
    for (uint64_t d : dims) {
        if (d == 0 || d == std::numeric_limits<uint64_t>::max()) throw std::invalid_argument("Expression::fill requires concrete non-zero dimensions.");
    }
    auto out = std::make_shared<PhysicalExpression>();
    ExprNode node;
    node.op = ExprOp::FILL;
    node.scalar_fp = value;
    node.fill_dims = dims;
    node.output_dtype = output_dtype;
    out->nodes.push_back(node);
    out->output_node = 0;
    return Expression(out, 0);
}

Expression Expression::fromPhysicalNode(std::shared_ptr<PhysicalExpression> expr, uint32_t nodeIndex) {
    if (!expr) throw std::invalid_argument("Expression::fromPhysicalNode requires a non-null PhysicalExpression.");
    if (nodeIndex >= expr->nodes.size()) throw std::out_of_range("Expression::fromPhysicalNode node index is out of range.");
    return Expression(std::move(expr), nodeIndex);
}

PhysicalExpression Expression::expression() const {
    if (!expr) throw std::runtime_error("Expression has no underlying graph.");
    PhysicalExpression out = *expr;
    out.output_node = nodeIndex;
    return out;
}

std::set<std::string> Expression::getInputNames() const {
    if (!expr) throw std::runtime_error("Expression has no underlying graph.");
    // only the inputs reachable from this node
    std::set<std::string> names;
    std::vector<char> seen(nodeIndex + 1, 0);
    seen[nodeIndex] = 1;
    for (uint32_t i = nodeIndex + 1; i-- > 0;) {
        if (!seen[i]) continue;
        const ExprNode& n = expr->nodes[i];
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != UINT32_MAX) seen[c] = 1;
        if (n.input_slot != UINT32_MAX) names.insert(expr->inputs.at(n.input_slot).name);
    }
    return names;
}

// ---- combinators -------------------------------------------------------------------------------------------------------
Expression Expression::unaryOp(const Expression& input, ExprOp op) {
    if (!input.expr) throw std::runtime_error("Cannot apply unary op to empty expression");
    auto out = std::make_shared<PhysicalExpression>();
    GraphMerger merger(*out);
    ExprNode node;
    node.op = op;
    node.lhs = merger.absorb(*input.expr, input.nodeIndex);
    out->nodes.push_back(node);
    out->output_node = static_cast<uint32_t>(out->nodes.size() - 1);
    return Expression(out, out->output_node);
}

Expression Expression::binaryOp(const Expression& lhs, const Expression& rhs, ExprOp op) {
    if (!lhs.expr || !rhs.expr) throw std::runtime_error("Cannot combine empty expressions");
    auto out = std::make_shared<PhysicalExpression>();
    GraphMerger merger(*out);
    ExprNode node;
    node.op = op;
    node.lhs = merger.absorb(*lhs.expr, lhs.nodeIndex);
    node.rhs = merger.absorb(*rhs.expr, rhs.nodeIndex);
    out->nodes.push_back(node);
    out->output_node = static_cast<uint32_t>(out->nodes.size() - 1);
    return Expression(out, out->output_node);
}

Expression Expression::ternaryOp(const Expression& a, const Expression& b, const Expression& c, ExprOp op) {
    if (!a.expr || !b.expr || !c.expr) throw std::runtime_error("Cannot combine empty expressions");
    auto out = std::make_shared<PhysicalExpression>();
    GraphMerger merger(*out);
    ExprNode node;
    node.op = op;
    node.lhs = merger.absorb(*a.expr, a.nodeIndex);
    node.rhs = merger.absorb(*b.expr, b.nodeIndex);
    node.aux = merger.absorb(*c.expr, c.nodeIndex);
    out->nodes.push_back(node);
    out->output_node = static_cast<uint32_t>(out->nodes.size() - 1);
    return Expression(out, out->output_node);
}

Outputs Expression::outputs(const std::vector<std::pair<std::string, Expression>>& named_exprs) {
    if (named_exprs.empty()) throw std::runtime_error("Expression::outputs requires at least one named output.");
    auto merged = std::make_shared<PhysicalExpression>();
    GraphMerger merger(*merged);
    std::vector<NamedOutput> outs;
    std::unordered_set<std::string> seen;
    for (const auto& [name, e] : named_exprs) {
        if (name.empty()) throw std::runtime_error("Output name cannot be empty.");
        if (!seen.insert(name).second) throw std::runtime_error("Duplicate output name: " + name);
        if (!e.expr) throw std::runtime_error("Output expression has no backing PhysicalExpression.");
        outs.push_back(NamedOutput{name, merger.absorb(*e.expr, e.nodeIndex)});
    }
    merged->output_node = outs.back().node_idx;
    return Outputs(std::move(merged), std::move(outs));
}

Outputs Outputs::conditional(const Expression& predicate, const Outputs& then_outputs, const Outputs& else_outputs) {
    if (then_outputs.outputs.empty() || else_outputs.outputs.empty()) {
        throw std::runtime_error("Outputs::conditional requires non-empty then and else branches.");
    }
    bool sameNames = then_outputs.outputs.size() == else_outputs.outputs.size();
    for (size_t i = 0; sameNames && i < then_outputs.outputs.size(); ++i) sameNames = then_outputs.outputs[i].name == else_outputs.outputs[i].name;
    if (!sameNames) throw std::runtime_error("Outputs::conditional requires then/else branches to expose the same output names in the same order.");
    const Expression taken = predicate.notEqual(Expression(0.0));
    std::vector<std::pair<std::string, Expression>> selected;
    for (size_t i = 0; i < then_outputs.outputs.size(); ++i) {
        const Expression whenTrue(then_outputs.expr, then_outputs.outputs[i].node_idx), whenFalse(else_outputs.expr, else_outputs.outputs[i].node_idx);
        selected.emplace_back(then_outputs.outputs[i].name, Expression::where(taken, whenTrue, whenFalse));
    }
    return Expression::outputs(selected);
}

Outputs Outputs::ifElifElse(const Expression& predicate, const Outputs& then_outputs, const std::vector<std::pair<Expression, Outputs>>& elif_branches,
                            const Outputs& else_outputs) {
    if (elif_branches.empty()) throw std::runtime_error("Outputs::ifElifElse requires at least one elif branch.");
    Outputs chained = else_outputs;
    for (auto it = elif_branches.rbegin(); it != elif_branches.rend(); ++it) chained = conditional(it->first, it->second, chained);
    return conditional(predicate, then_outputs, chained);
}

Outputs Expression::outputs(std::initializer_list<std::pair<std::string, Expression>> named_exprs) {
    return outputs(std::vector<std::pair<std::string, Expression>>(named_exprs));
}

// ---- operators -----------------------------------------------------------------------------------------------------------
Expression Expression::operator+(const Expression& o) const { return binaryOp(*this, o, ExprOp::ADD); }
Expression Expression::operator-(const Expression& o) const { return binaryOp(*this, o, ExprOp::SUB); }
Expression Expression::operator*(const Expression& o) const { return binaryOp(*this, o, ExprOp::MUL); }
Expression Expression::operator/(const Expression& o) const { return binaryOp(*this, o, ExprOp::DIV); }
Expression Expression::operator-() const { return unaryOp(*this, ExprOp::NEG); }
Expression Expression::operator!() const { return logicalNot(); }
Expression Expression::operator==(const Expression& o) const { return equal(o); }
Expression Expression::operator!=(const Expression& o) const { return notEqual(o); }
Expression Expression::operator<(const Expression& o) const { return lessThan(o); }
Expression Expression::operator<=(const Expression& o) const { return lessEqual(o); }
Expression Expression::operator>(const Expression& o) const { return greaterThan(o); }
Expression Expression::operator>=(const Expression& o) const { return greaterEqual(o); }

Expression Expression::equal(const Expression& o) const { return binaryOp(*this, o, ExprOp::EQUAL); }
Expression Expression::notEqual(const Expression& o) const { return binaryOp(*this, o, ExprOp::NOT_EQUAL); }
Expression Expression::lessThan(const Expression& o) const { return binaryOp(*this, o, ExprOp::LESS); }
Expression Expression::lessEqual(const Expression& o) const { return binaryOp(*this, o, ExprOp::LESS_EQUAL); }
Expression Expression::greaterThan(const Expression& o) const { return binaryOp(*this, o, ExprOp::GREATER); }
Expression Expression::greaterEqual(const Expression& o) const { return binaryOp(*this, o, ExprOp::GREATER_EQUAL); }
Expression Expression::logicalAnd(const Expression& o) const { return binaryOp(*this, o, ExprOp::LOGICAL_AND); }
Expression Expression::logicalOr(const Expression& o) const { return binaryOp(*this, o, ExprOp::LOGICAL_OR); }
Expression Expression::logicalNot() const { return unaryOp(*this, ExprOp::LOGICAL_NOT); }
Expression Expression::pow(const Expression& e) const { return binaryOp(*this, e, ExprOp::POW); }
Expression Expression::min(const Expression& o) const { return binaryOp(*this, o, ExprOp::MIN); }
Expression Expression::max(const Expression& o) const { return binaryOp(*this, o, ExprOp::MAX); }

Expression Expression::cast(DataType output_dtype) const {
    Expression result = unaryOp(*this, ExprOp::CAST);
    ExprNode& node = result.expr->nodes[result.nodeIndex];
    node.output_dtype = output_dtype;
    node.compute_dtype = output_dtype;
    return result;
}

Expression Expression::where(const Expression& condition, const Expression& true_value, const Expression& false_value) {
    return ternaryOp(condition, true_value, false_value, ExprOp::WHERE);
}
Expression Expression::select(const Expression& true_value, const Expression& false_value) const { return where(*this, true_value, false_value); }

#define THOR_UNARY(method, OP) \
    Expression Expression::method() const { return unaryOp(*this, ExprOp::OP); }
THOR_UNARY(abs, ABS)
THOR_UNARY(ceil, CEIL)
THOR_UNARY(floor, FLOOR)
THOR_UNARY(round, ROUND)
THOR_UNARY(trunc, TRUNC)
THOR_UNARY(sin, SIN)
THOR_UNARY(cos, COS)
THOR_UNARY(tan, TAN)
THOR_UNARY(asin, ASIN)
THOR_UNARY(acos, ACOS)
THOR_UNARY(atan, ATAN)
THOR_UNARY(sinh, SINH)
THOR_UNARY(cosh, COSH)
THOR_UNARY(tanh, TANH)
THOR_UNARY(asinh, ASINH)
THOR_UNARY(acosh, ACOSH)
THOR_UNARY(atanh, ATANH)
THOR_UNARY(erf, ERF)
THOR_UNARY(erfc, ERFC)
THOR_UNARY(erfcx, ERFCX)
THOR_UNARY(erfinv, ERFINV)
THOR_UNARY(erfcinv, ERFCINV)
THOR_UNARY(tgamma, TGAMMA)
THOR_UNARY(lgamma, LGAMMA)
THOR_UNARY(digamma, DIGAMMA)
THOR_UNARY(exp, EXP)
THOR_UNARY(expm1, EXPM1)
THOR_UNARY(exp2, EXP2)
THOR_UNARY(exp10, EXP10)
THOR_UNARY(ln, LN)
THOR_UNARY(log1p, LOG1P)
THOR_UNARY(log2, LOG2)
THOR_UNARY(log10, LOG10)
THOR_UNARY(sqrt, SQRT)
THOR_UNARY(normcdf, NORMCDF)
#undef THOR_UNARY

// reciprocal / inverse-reciprocal trigonometry: 1 / f(x) and f(1 / x)
Expression Expression::csc() const { return constantScalar(1.0) / sin(); }
Expression Expression::sec() const { return constantScalar(1.0) / cos(); }
Expression Expression::cot() const { return constantScalar(1.0) / tan(); }
Expression Expression::csch() const { return constantScalar(1.0) / sinh(); }
Expression Expression::sech() const { return constantScalar(1.0) / cosh(); }
Expression Expression::coth() const { return constantScalar(1.0) / tanh(); }
Expression Expression::acsc() const { return (constantScalar(1.0) / *this).asin(); }
Expression Expression::asec() const { return (constantScalar(1.0) / *this).acos(); }
Expression Expression::acot() const { return (constantScalar(1.0) / *this).atan(); }
Expression Expression::acsch() const { return (constantScalar(1.0) / *this).asinh(); }
Expression Expression::asech() const { return (constantScalar(1.0) / *this).acosh(); }
Expression Expression::acoth() const { return (constantScalar(1.0) / *this).atanh(); }

Expression Expression::log(double base) const {
    if (base <= 0.0 || base == 1.0) {
        throw std::runtime_error("log base must be positive and not equal to 1, received base = " + std::to_string(base));
    }
    return ln() / constantScalar(std::log(base));
}

Expression Expression::clamp(const Expression& lower_bound, const Expression& upper_bound) const { return max(lower_bound).min(upper_bound); }
Expression Expression::clamp(double lower_bound, double upper_bound) const {
    if (lower_bound > upper_bound) throw std::invalid_argument("Expression::clamp requires lower_bound <= upper_bound.");
    return clamp(constantScalar(lower_bound), constantScalar(upper_bound));
}

// sigmoid(x) = exp(-max(-x, 0)) / (1 + exp(-|x|)): finite for both signs of large |x|
Expression Expression::sigmoid() const {
    const Expression negated = -*this;
    const Expression numerator = (-negated.max(Expression(0.0))).exp();
    const Expression denominator = Expression(1.0) + (-abs()).exp();
    return numerator / denominator;
}
// log(1 + e^x) = max(x, 0) + log1p(e^-|x|)
Expression Expression::softplus() const { return max(Expression(0.0)) + (-abs()).exp().log1p(); }
// expm1 of min(x, 0) never evaluates e^x for positive x and keeps precision near zero
Expression Expression::elu(double alpha) const { return max(Expression(0.0)) + (min(Expression(0.0)).expm1() * Expression(alpha)); }
Expression Expression::selu() const {
    return (max(Expression(0.0)) * Expression(1.05070098)) + (min(Expression(0.0)).expm1() * Expression(1.758099326));
}
Expression Expression::gelu() const { return *this * normcdf(); }
Expression Expression::mish() const { return *this * softplus().tanh(); }
Expression Expression::relu6() const { return max(Expression(0.0)).min(Expression(6.0)); }
Expression Expression::hardTanh(double min_value, double max_value) const {
    if (min_value > max_value) throw std::invalid_argument("Expression::hardTanh requires min_value <= max_value.");
    return max(Expression(min_value)).min(Expression(max_value));
}
Expression Expression::hardSwish() const { return *this * ((*this + Expression(3.0)).relu6() / Expression(6.0)); }
Expression Expression::threshold(double threshold, double value) const {
    return where(*this > Expression(threshold), *this, Expression(value));
}
Expression Expression::swish() const { return *this * sigmoid(); }

Expression Expression::softmax(SoftmaxAlgorithm algorithm, SoftmaxMode mode) const {
    if (algorithm == SoftmaxAlgorithm::Log) {
        throw std::invalid_argument("Expression::softmax computes ordinary softmax; use Expression::logSoftmax for the log form.");
    }
    Expression out = unaryOp(*this, ExprOp::SOFTMAX);
    out.expr->nodes[out.nodeIndex].softmax_algorithm = algorithm;
    out.expr->nodes[out.nodeIndex].softmax_mode = mode;
    return out;
}

Expression Expression::logSoftmax(SoftmaxMode mode) const {
    Expression out = unaryOp(*this, ExprOp::SOFTMAX);
    out.expr->nodes[out.nodeIndex].softmax_algorithm = SoftmaxAlgorithm::Log;
    out.expr->nodes[out.nodeIndex].softmax_mode = mode;
    return out;
}

std::vector<uint64_t> resolveReductionAxes(const std::vector<uint64_t>& reduction_axes, size_t rank) {
    std::vector<uint64_t> out;
    if (reduction_axes.empty()) {
        for (uint64_t a = 0; a < rank; ++a) out.push_back(a);
    } else if (reduction_axes.size() == 1 && reduction_axes[0] == kReduceAllAxesButFirst) {
        if (rank < 2) throw std::runtime_error("Reduction axis out of range.");
        for (uint64_t a = 1; a < rank; ++a) out.push_back(a);
    } else {
        out = reduction_axes;
        std::sort(out.begin(), out.end());
        out.erase(std::unique(out.begin(), out.end()), out.end());
    }
    for (uint64_t a : out)
        if (a >= rank) throw std::runtime_error("Reduction axis out of range.");
    return out;
}

// ---- shape ---------------------------------------------------------------------------------------------------------------
Expression Expression::reshape(const std::vector<uint64_t>& new_dims) const {
    if (new_dims.empty()) throw std::invalid_argument("Expression::reshape requires at least one dimension.");
    if (std::count(new_dims.begin(), new_dims.end(), std::numeric_limits<uint64_t>::max()) > 1) {
        throw std::invalid_argument("Expression::reshape supports at most one infer-dimension marker.");
    }
    Expression out = unaryOp(*this, ExprOp::RESHAPE);
    out.expr->nodes[out.nodeIndex].reshape_dims = new_dims;
    return out;
}

Expression Expression::unsqueeze(const std::vector<uint64_t>& axes) const {
    Expression out = unaryOp(*this, ExprOp::UNSQUEEZE);
    out.expr->nodes[out.nodeIndex].unsqueeze_axes = sortedUnique(axes);
    return out;
}

Expression Expression::squeeze(const std::vector<uint64_t>& axes) const {
    Expression out = unaryOp(*this, ExprOp::SQUEEZE);
    out.expr->nodes[out.nodeIndex].squeeze_axes = sortedUnique(axes);
    return out;
}

// ---- reductions -----------------------------------------------------------------------------------------------------------
Expression Expression::reduction(ExprOp op, const std::vector<uint64_t>& reduction_axes, const std::vector<uint64_t>& squeeze_axes,
                                 std::optional<DataType> compute_dtype) const {
    if (!isReductionOp(op)) throw std::invalid_argument("Expression::reduction requires a reduction op.");
    if (compute_dtype.has_value() && compute_dtype.value() != DataType::FP32) {
        throw std::runtime_error("Reductions accumulate in FP32; requested compute dtype " + std::string(dataTypeName(compute_dtype.value())) +
                                 " is not supported.");
    }
    Expression out = unaryOp(*this, op);
    ExprNode& node = out.expr->nodes[out.nodeIndex];
    node.reduction_axes = reduction_axes;
    node.squeeze_axes = squeeze_axes;
    node.compute_dtype = DataType::FP32;
    if (isArgReductionOp(op)) node.output_dtype = DataType::UINT32;
    return out;
}

#define THOR_REDUCTION(method, OP)                                                                                           \
    Expression Expression::method(const std::vector<uint64_t>& axes, const std::vector<uint64_t>& squeeze,                    \
                                  std::optional<DataType> compute_dtype) const {                                              \
        return reduction(ExprOp::OP, axes, squeeze, compute_dtype);                                                           \
    }
THOR_REDUCTION(reduce_sum, REDUCE_SUM)
THOR_REDUCTION(reduce_prod, REDUCE_PROD)
THOR_REDUCTION(reduce_min, REDUCE_MIN)
THOR_REDUCTION(reduce_max, REDUCE_MAX)
THOR_REDUCTION(reduce_mean, REDUCE_AVG)
THOR_REDUCTION(reduce_norm1, REDUCE_NORM1)
THOR_REDUCTION(reduce_norm2, REDUCE_NORM2)
THOR_REDUCTION(argmin, REDUCE_ARGMIN)
THOR_REDUCTION(argmax, REDUCE_ARGMAX)
#undef THOR_REDUCTION

Expression Expression::dotProduct(const Expression& other, std::optional<DataType> compute_dtype) const {
    return dotProduct(*this, other, compute_dtype);
}
Expression Expression::dotProduct(const Expression& lhs, const Expression& rhs, std::optional<DataType> compute_dtype) {
    return (lhs * rhs).reduce_sum({}, {UINT64_MAX}, compute_dtype);
}

Expression Expression::withDTypes(std::optional<DataType> compute_dtype, std::optional<DataType> output_dtype) const {
    if (!expr) throw std::runtime_error("Cannot override dtypes on an empty expression");
    auto out = std::make_shared<PhysicalExpression>();
    GraphMerger merger(*out);
    const uint32_t root = merger.absorb(*expr, nodeIndex);
    out->output_node = root;
    if (compute_dtype.has_value()) out->nodes[root].compute_dtype = compute_dtype;
    if (output_dtype.has_value()) out->nodes[root].output_dtype = output_dtype;
    return Expression(out, root);
}

Expression Expression::stridedView(const std::vector<uint64_t>& dims, const std::vector<uint64_t>& strides_elements, uint64_t element_offset) const {
    if (!expr) throw std::runtime_error("Cannot create a strided view from an empty expression");
    if (dims.empty() || dims.size() != strides_elements.size()) {
        throw std::invalid_argument("Expression::stridedView requires dimensions and strides with the same non-zero rank.");
    }
    for (uint64_t d : dims) {
        if (d == std::numeric_limits<uint64_t>::max()) throw std::invalid_argument("Expression::stridedView does not support infer-dimension markers.");
        if (d == 0) throw std::invalid_argument("Expression::stridedView does not support zero-sized dimensions.");
    }
    Expression out = unaryOp(*this, ExprOp::STRIDED_VIEW);
    ExprNode& node = out.expr->nodes[out.nodeIndex];
    node.view_dims = dims;
    node.view_strides = strides_elements;
    node.view_element_offset = element_offset;
    return out;
}

// The gradient of a strided view as an expression of its own (reference: Expression.cpp:3789-3835 there): `this` is the gradient,
// shaped like the view; the result is FP32, shaped like the viewed tensor, zero where the view does not reach.
Expression Expression::stridedViewBackward(const std::vector<uint64_t>& source_dims, const std::vector<uint64_t>& view_dims,
                                           const std::vector<uint64_t>& view_strides_elements, uint64_t view_element_offset) const {
    if (!expr) throw std::runtime_error("Cannot create a strided-view backward from an empty expression");
    if (source_dims.empty()) throw std::invalid_argument("Expression::stridedViewBackward requires non-empty source dimensions.");
    if (view_dims.empty() || view_dims.size() != view_strides_elements.size()) {
        throw std::invalid_argument("Expression::stridedViewBackward requires view dimensions and strides with the same non-zero rank.");
    }
    uint64_t denseTail = 1;
    for (size_t axis = view_dims.size(); axis-- > 0;) {
        if (view_dims[axis] == 0 || view_dims[axis] == std::numeric_limits<uint64_t>::max() || view_strides_elements[axis] < denseTail) {
            throw std::invalid_argument("Expression::stridedViewBackward requires canonical non-overlapping row-major-like strides.");
        }
        if (denseTail > std::numeric_limits<uint64_t>::max() / view_dims[axis]) {
            throw std::overflow_error("Expression::stridedViewBackward view element count overflows uint64_t.");
        }
        denseTail *= view_dims[axis];
    }
    uint64_t sourceElements = 1;
    for (uint64_t d : source_dims) {
        if (d == 0 || d == std::numeric_limits<uint64_t>::max()) {
            throw std::invalid_argument("Expression::stridedViewBackward requires concrete non-zero source dimensions.");
        }
        if (sourceElements > std::numeric_limits<uint64_t>::max() / d) throw std::overflow_error("Expression::stridedViewBackward source element count overflows uint64_t.");
        sourceElements *= d;
    }
    uint64_t last = view_element_offset;
    for (size_t axis = 0; axis < view_dims.size(); ++axis) last += (view_dims[axis] - 1) * view_strides_elements[axis];
    if (last >= sourceElements) throw std::invalid_argument("Expression::stridedViewBackward view reaches past the source tensor.");
    Expression out = unaryOp(*this, ExprOp::STRIDED_VIEW_BACKWARD);
    ExprNode& node = out.expr->nodes[out.nodeIndex];
    node.view_dims = view_dims;
    node.view_strides = view_strides_elements;
    node.view_element_offset = view_element_offset;
    node.fill_dims = source_dims;
    node.output_dtype = DataType::FP32;
    return out;
}

// Every use of the tensor input `input_name` reads `replacement` instead (reference: Expression.cpp:3173-3198 there).  The result's
// inputs are those of the replacement and the remaining ones of this expression, merged by name.
Expression Expression::substituteInput(const std::string& input_name, const Expression& replacement) const {
    if (input_name.empty()) throw std::invalid_argument("Expression::substituteInput requires a non-empty input name.");
    if (!expr) throw std::runtime_error("Expression::substituteInput called on an expression with no underlying graph.");
    if (!replacement.expr) throw std::runtime_error("Expression::substituteInput replacement has no underlying graph.");
    if (replacement.nodeIndex >= replacement.expr->nodes.size()) throw std::runtime_error("Expression::substituteInput replacement node index is out of range.");
    if (nodeIndex >= expr->nodes.size()) throw std::runtime_error("Expression::substituteInput source node index is out of range.");
    auto out = std::make_shared<PhysicalExpression>();
    GraphMerger merger(*out);
    const uint32_t replacementRoot = merger.absorb(*replacement.expr, replacement.nodeIndex);
    const uint32_t root = merger.absorb(*expr, nodeIndex, &input_name, replacementRoot);
    out->output_node = root;
    return Expression(out, root);
}

// ---- scans -----------------------------------------------------------------------------------------------------------------
namespace {
void validateScanOp(ScanOp op, const char* api) {
    if (static_cast<uint8_t>(op) > static_cast<uint8_t>(ScanOp::ArgMax)) throw std::invalid_argument(std::string(api) + " received an unsupported ScanOp.");
}
ScanOp indexOpOf(ScanOp op, const char* api) {
    if (op == ScanOp::Min) return ScanOp::ArgMin;
    if (op == ScanOp::Max) return ScanOp::ArgMax;
    throw std::invalid_argument(std::string(api) + " supports only ScanOp::Min and ScanOp::Max.");
}
}  // namespace

Expression Expression::scan(ScanOp op, int64_t axis, bool inclusive) const {
    if (axis < -1) throw std::invalid_argument("Expression::scan currently supports only axis=-1 or an explicit non-negative final axis.");
    validateScanOp(op, "Expression::scan");
    Expression out = unaryOp(*this, ExprOp::SCAN);
    ExprNode& node = out.expr->nodes[out.nodeIndex];
    node.scan_op = op;
    node.scan_mode = inclusive ? ScanMode::Inclusive : ScanMode::Exclusive;
    node.scan_axis = axis < 0 ? UINT64_MAX : static_cast<uint64_t>(axis);
    return out;
}

Expression Expression::reverseScan(ScanOp op, int64_t axis, bool inclusive) const {
    Expression out = scan(op, axis, inclusive);
    out.expr->nodes[out.nodeIndex].scan_reverse = true;
    return out;
}

Expression Expression::prefixCount(bool inclusive, int64_t axis) const { return cast(DataType::UINT32).scan(ScanOp::Sum, axis, inclusive); }

std::pair<Expression, Expression> Expression::scanWithIndices(ScanOp op, int64_t axis, bool inclusive) const {
    const ScanOp indexOp = indexOpOf(op, "Expression::scanWithIndices");
    return {scan(op, axis, inclusive), scan(indexOp, axis, inclusive)};
}

Expression Expression::segmentedScan(const Expression& offsets, ScanOp op, bool inclusive, bool reverse) const {
    validateScanOp(op, "Expression::segmentedScan");
    Expression out = binaryOp(*this, offsets, ExprOp::SEGMENTED_SCAN);
    ExprNode& node = out.expr->nodes[out.nodeIndex];
    node.scan_op = op;
    node.scan_mode = inclusive ? ScanMode::Inclusive : ScanMode::Exclusive;
    node.scan_axis = UINT64_MAX;
    node.scan_reverse = reverse;
    return out;
}

Expression Expression::segmentedScanWithRaggedMetadata(const Expression& input, const Expression& offsets, ScanOp op, bool inclusive, bool reverse,
                                                       uint64_t ragged_batch_size, uint64_t ragged_max_active_values) {
    if ((ragged_batch_size == 0) != (ragged_max_active_values == 0)) {
        throw std::invalid_argument("Segmented scan ragged metadata requires both batch size and max active values, or neither.");
    }
    Expression out = input.segmentedScan(offsets, op, inclusive, reverse);
    if (ragged_batch_size != 0) {
        ExprNode& node = out.expr->nodes.at(out.nodeIndex);
        node.ragged_runtime_batch_size = ragged_batch_size;
        node.ragged_runtime_max_active_values = ragged_max_active_values;
        node.ragged_runtime_elements_per_value = 1;
    }
    return out;
}

std::pair<Expression, Expression> Expression::segmentedScanWithIndices(const Expression& offsets, ScanOp op, bool inclusive, bool reverse) const {
    const ScanOp indexOp = indexOpOf(op, "Expression::segmentedScanWithIndices");
    return {segmentedScan(offsets, op, inclusive, reverse), segmentedScan(offsets, indexOp, inclusive, reverse)};
}

Expression Expression::takeAlongAxis(const Expression& indices, int64_t axis) const {
    if (axis < -1) throw std::invalid_argument("Expression::takeAlongAxis currently supports only axis=-1 or an explicit non-negative axis.");
    Expression out = binaryOp(*this, indices, ExprOp::TAKE_ALONG_AXIS);
    out.expr->nodes[out.nodeIndex].reduction_axes = {axis < 0 ? UINT64_MAX : static_cast<uint64_t>(axis)};
    return out;
}

// ---- rotary position embedding (Expression.cpp:4334-4507 there) -----------------------------------------------------------
namespace {
ExprNode ropeNodeFrom(const RotaryPositionEmbeddingOptions& options) {
    if (options.compute_dtype.has_value() && options.compute_dtype.value() != DataType::FP32) {
        // the rotation kernels work in FP32 whatever the storage dtype; another arithmetic dtype is refused rather than ignored
        throw std::invalid_argument(std::string("RoPE rotates in FP32: compute_dtype ") + dataTypeName(options.compute_dtype.value()) + " is not supported.");
    }
    if (options.base <= 0.0) throw std::runtime_error("RoPE base must be positive.");
    if (options.scaling_factor <= 0.0) throw std::runtime_error("RoPE scaling factor must be positive.");
    if (options.attention_factor.has_value() && options.attention_factor.value() <= 0.0) throw std::runtime_error("RoPE attention_factor must be positive.");
    if (options.rotary_dim != 0 && (options.rotary_dim & 1ull) != 0) throw std::runtime_error("RoPE rotary_dim must be even.");
    if (options.scaling_kind == RotaryScalingKind::DynamicNTK && options.original_max_position_embeddings == 0) {
        throw std::runtime_error("Dynamic-NTK RoPE scaling requires original_max_position_embeddings.");
    }
    if ((options.scaling_kind == RotaryScalingKind::Yarn || options.scaling_kind == RotaryScalingKind::LongRope ||
         options.scaling_kind == RotaryScalingKind::Llama3) &&
        options.original_max_position_embeddings == 0) {
        throw std::runtime_error("This RoPE scaling kind requires original_max_position_embeddings.");
    }
    if (options.scaling_kind == RotaryScalingKind::Yarn && (options.yarn_beta_fast <= 0.0 || options.yarn_beta_slow <= 0.0)) {
        throw std::runtime_error("YaRN RoPE scaling requires positive beta parameters.");
    }
    if (options.scaling_kind == RotaryScalingKind::Llama3 &&
        (options.llama3_low_freq_factor <= 0.0 || options.llama3_high_freq_factor <= 0.0 ||
         options.llama3_high_freq_factor <= options.llama3_low_freq_factor)) {
        throw std::runtime_error("Llama3 RoPE scaling requires 0 < low_freq_factor < high_freq_factor.");
    }
    if (options.scaling_kind == RotaryScalingKind::LongRope) {
        if (options.rotary_dim == 0) throw std::runtime_error("LongRoPE scaling requires an explicit rotary_dim.");
        const uint64_t expected = options.rotary_dim / 2;
        if (options.long_rope_short_factors.size() != expected || options.long_rope_long_factors.size() != expected) {
            throw std::runtime_error("LongRoPE scaling requires short/long factor lists of length rotary_dim / 2.");
        }
        for (double f : options.long_rope_short_factors)
            if (f <= 0.0) throw std::runtime_error("LongRoPE short factors must be positive.");
        for (double f : options.long_rope_long_factors)
            if (f <= 0.0) throw std::runtime_error("LongRoPE long factors must be positive.");
    }
    ExprNode node;
    node.op = ExprOp::ROPE;
    node.rope_sequence_axis = options.sequence_axis;
    node.rope_head_dim_axis = options.head_dim_axis;
    node.rope_rotary_dim = options.rotary_dim;
    node.rope_base = options.base;
    node.rope_position_offset = options.position_offset;
    node.rope_interleaved = options.interleaved;
    node.rope_inverse = options.inverse;
    node.rope_scaling_kind = options.scaling_kind;
    node.rope_scaling_factor = options.scaling_factor;
    node.rope_original_max_position_embeddings = options.original_max_position_embeddings;
    // the magnitude correction that goes with the stretched frequencies, unless the caller names one
    if (options.attention_factor.has_value()) {
        node.rope_attention_factor = options.attention_factor.value();
    } else if (options.scaling_kind == RotaryScalingKind::Yarn) {
        node.rope_attention_factor = options.scaling_factor <= 1.0 ? 1.0 : 0.1 * std::log(options.scaling_factor) + 1.0;
    } else if (options.scaling_kind == RotaryScalingKind::LongRope) {
        node.rope_attention_factor =
            options.scaling_factor <= 1.0
                ? 1.0
                : std::sqrt(1.0 + std::log(options.scaling_factor) / std::log(static_cast<double>(options.original_max_position_embeddings)));
    } else {
        node.rope_attention_factor = 1.0;
    }
    node.rope_yarn_beta_fast = options.yarn_beta_fast;
    node.rope_yarn_beta_slow = options.yarn_beta_slow;
    node.rope_llama3_low_freq_factor = options.llama3_low_freq_factor;
    node.rope_llama3_high_freq_factor = options.llama3_high_freq_factor;
    node.rope_long_rope_short_factors = options.long_rope_short_factors;
    node.rope_long_rope_long_factors = options.long_rope_long_factors;
    node.output_dtype = options.output_dtype;
    node.compute_dtype = options.compute_dtype;
    return node;
}
}  // namespace

Expression Expression::ropeOp(const Expression& input, const Expression* position_ids, const Expression* effective_sequence_length, ExprNode node) {
    if (!input.expr) throw std::runtime_error("Cannot build RoPE from an empty expression.");
    auto out = std::make_shared<PhysicalExpression>();
    GraphMerger merger(*out);
    // metadata first, so every operand precedes the rotation in the graph
    if (effective_sequence_length != nullptr) node.aux = merger.absorb(*effective_sequence_length->expr, effective_sequence_length->nodeIndex);
    if (position_ids != nullptr) node.rhs = merger.absorb(*position_ids->expr, position_ids->nodeIndex);
    node.lhs = merger.absorb(*input.expr, input.nodeIndex);
    out->nodes.push_back(std::move(node));
    out->output_node = static_cast<uint32_t>(out->nodes.size() - 1);
    return Expression(out, out->output_node);
}

Expression Expression::rotaryPositionEmbedding(RotaryPositionEmbeddingOptions options) const {
    if (!expr) throw std::runtime_error("Cannot build RoPE from an empty expression.");
    return ropeOp(*this, nullptr, nullptr, ropeNodeFrom(options));
}

Expression Expression::rotaryPositionEmbeddingWithEffectiveSequenceLength(const Expression& effective_sequence_length,
                                                                          RotaryPositionEmbeddingOptions options) const {
    if (!effective_sequence_length.expr) throw std::runtime_error("RoPE effective sequence length cannot be an empty expression.");
    // the scaling rules take the length as a floating-point number, whatever dtype the caller's metadata has
    const Expression length = effective_sequence_length.cast(DataType::FP32);
    return ropeOp(*this, nullptr, &length, ropeNodeFrom(options));
}

Expression Expression::rotaryPositionEmbeddingWithPositionIds(const Expression& position_ids, RotaryPositionEmbeddingOptions options) const {
    if (!position_ids.expr) throw std::runtime_error("RoPE position ids cannot be an empty expression.");
    if (options.position_offset != 0) {
        throw std::runtime_error("RoPE explicit position ids require position_offset == 0 because the ids are absolute positions.");
    }
    const Expression ids = position_ids.cast(DataType::FP32);
    return ropeOp(*this, &ids, nullptr, ropeNodeFrom(options));
}

Expression Expression::rotaryPositionEmbeddingWithPositionIdsAndEffectiveSequenceLength(const Expression& position_ids,
                                                                                        const Expression& effective_sequence_length,
                                                                                        RotaryPositionEmbeddingOptions options) const {
    if (!position_ids.expr) throw std::runtime_error("RoPE position ids cannot be an empty expression.");
    if (!effective_sequence_length.expr) throw std::runtime_error("RoPE effective sequence length cannot be an empty expression.");
    if (options.position_offset != 0) {
        throw std::runtime_error("RoPE explicit position ids require position_offset == 0 because the ids are absolute positions.");
    }
    const Expression ids = position_ids.cast(DataType::FP32);
    const Expression length = effective_sequence_length.cast(DataType::FP32);
    return ropeOp(*this, &ids, &length, ropeNodeFrom(options));
}

std::string ropeKey(const ExprNode& n) {
    std::string k = "seq=" + std::to_string(n.rope_sequence_axis) + ",dim=" + std::to_string(n.rope_head_dim_axis) + ",rotary=" + std::to_string(n.rope_rotary_dim) +
                    ",base=" + formatFloatCanonical(n.rope_base) + ",offset=" + std::to_string(n.rope_position_offset) +
                    (n.rope_interleaved ? ",interleaved" : "") + (n.rope_inverse ? ",inverse" : "") + ",kind=" + std::to_string(static_cast<int>(n.rope_scaling_kind)) +
                    ",factor=" + formatFloatCanonical(n.rope_scaling_factor) + ",max=" + std::to_string(n.rope_original_max_position_embeddings) +
                    ",attention=" + formatFloatCanonical(n.rope_attention_factor) + ",yarn=" + formatFloatCanonical(n.rope_yarn_beta_fast) + "/" +
                    formatFloatCanonical(n.rope_yarn_beta_slow) + ",llama3=" + formatFloatCanonical(n.rope_llama3_low_freq_factor) + "/" +
                    formatFloatCanonical(n.rope_llama3_high_freq_factor) + ",short=";
    for (double f : n.rope_long_rope_short_factors) k += formatFloatCanonical(f) + ";";
    k += ",long=";
    for (double f : n.rope_long_rope_long_factors) k += formatFloatCanonical(f) + ";";
    // which of the two optional operands is which (both ride in rhs / aux)
    k += std::string(",ids=") + (n.rhs != UINT32_MAX ? "1" : "0") + ",length=" + (n.aux != UINT32_MAX ? "1" : "0");
    return k;
}

Expression Expression::transpose() const {
    if (!expr) throw std::runtime_error("Cannot transpose an empty expression");
    return unaryOp(*this, ExprOp::TRANSPOSE);
}

// ---- ragged batches ------------------------------------------------------------------------------------------------------
Expression Expression::segmentedReduceWithRaggedMetadata(const Expression& input, const Expression& offsets, ExprOp op, uint64_t ragged_batch_size,
                                                         uint64_t ragged_max_active_values, uint64_t ragged_elements_per_value) {
    if (!isSegmentedReduceOp(op)) throw std::invalid_argument("segmentedReduceWithRaggedMetadata requires a segmented reduction op.");
    if ((ragged_batch_size == 0) != (ragged_max_active_values == 0)) {
        throw std::invalid_argument("Segmented reduction ragged metadata requires both batch size and max active values, or neither.");
    }
    if (ragged_elements_per_value == 0) throw std::invalid_argument("Segmented reduction ragged elements-per-value metadata must be non-zero.");
    Expression out = binaryOp(input, offsets, op);
    if (ragged_batch_size != 0) {
        ExprNode& node = out.expr->nodes.at(out.nodeIndex);
        node.ragged_runtime_batch_size = ragged_batch_size;
        node.ragged_runtime_max_active_values = ragged_max_active_values;
        node.ragged_runtime_elements_per_value = ragged_elements_per_value;
    }
    return out;
}

Expression Expression::segmentedReduceSum(const Expression& input, const Expression& offsets) {
    return segmentedReduceWithRaggedMetadata(input, offsets, ExprOp::SEGMENTED_REDUCE_SUM, 0, 0);
}
Expression Expression::segmentedReduceMin(const Expression& input, const Expression& offsets) {
    return segmentedReduceWithRaggedMetadata(input, offsets, ExprOp::SEGMENTED_REDUCE_MIN, 0, 0);
}
Expression Expression::segmentedReduceMax(const Expression& input, const Expression& offsets) {
    return segmentedReduceWithRaggedMetadata(input, offsets, ExprOp::SEGMENTED_REDUCE_MAX, 0, 0);
}
Expression Expression::segmentedReduceMean(const Expression& input, const Expression& offsets) {
    return segmentedReduceWithRaggedMetadata(input, offsets, ExprOp::SEGMENTED_REDUCE_MEAN, 0, 0);
}

Expression Expression::segmentedBroadcast(const Expression& per_segment_values, const Expression& offsets, uint64_t batch_size,
                                          uint64_t max_active_values, uint64_t elements_per_value, bool normalize_by_segment_length) {
    if (batch_size == 0 || max_active_values == 0 || elements_per_value == 0) {
        throw std::invalid_argument("Expression::segmentedBroadcast requires non-zero batch size, row capacity and elements per value.");
    }
    Expression out = binaryOp(per_segment_values, offsets, ExprOp::SEGMENTED_BROADCAST);
    ExprNode& node = out.expr->nodes.at(out.nodeIndex);
    node.ragged_runtime_batch_size = batch_size;
    node.ragged_runtime_max_active_values = max_active_values;
    node.ragged_runtime_elements_per_value = elements_per_value;
    node.segmented_broadcast_normalize_by_length = normalize_by_segment_length;
    return out;
}

Expression Expression::withRaggedRuntimeExtent(const Expression& offsets, uint64_t batch_size, uint64_t max_active_values,
                                               uint64_t elements_per_value) const {
    if (batch_size + 1 <= batch_size) throw std::invalid_argument("Expression::withRaggedRuntimeExtent batch size overflows offsets element count.");
    if (max_active_values == 0 || elements_per_value == 0) {
        throw std::invalid_argument("Expression::withRaggedRuntimeExtent requires non-zero maximum extent metadata.");
    }
    if (!offsets.expr || offsets.expr->nodes.at(offsets.nodeIndex).op != ExprOp::INPUT) {
        throw std::invalid_argument("Expression::withRaggedRuntimeExtent currently requires offsets to be a direct input expression.");
    }
    Expression out = binaryOp(*this, offsets, ExprOp::RAGGED_VALUEWISE_EXTENT);
    ExprNode& node = out.expr->nodes.at(out.nodeIndex);
    node.ragged_runtime_batch_size = batch_size;
    node.ragged_runtime_max_active_values = max_active_values;
    node.ragged_runtime_elements_per_value = elements_per_value;
    return out;
}

// ---- op classification ---------------------------------------------------------------------------------------------------
bool Expression::isLeafOp(ExprOp op) {
    return op == ExprOp::INPUT || op == ExprOp::RUNTIME_SCALAR || op == ExprOp::TENSOR_RUNTIME_SCALAR || op == ExprOp::SCALAR_FP ||
           op == ExprOp::FILL;
}

bool Expression::isBinaryOp(ExprOp op) {
    switch (op) {
        case ExprOp::ADD:
        case ExprOp::SUB:
        case ExprOp::MUL:
        case ExprOp::DIV:
        case ExprOp::POW:
        case ExprOp::EQUAL:
        case ExprOp::NOT_EQUAL:
        case ExprOp::LESS:
        case ExprOp::LESS_EQUAL:
        case ExprOp::GREATER:
        case ExprOp::GREATER_EQUAL:
        case ExprOp::LOGICAL_AND:
        case ExprOp::LOGICAL_OR:
        case ExprOp::MIN:
        case ExprOp::MAX:
        case ExprOp::MIN_GRAD_LEFT:
        case ExprOp::MIN_GRAD_RIGHT:
        case ExprOp::MAX_GRAD_LEFT:
        case ExprOp::MAX_GRAD_RIGHT:
            return true;
        default:
            return false;
    }
}

bool Expression::isTernaryOp(ExprOp op) { return op == ExprOp::WHERE; }

bool Expression::isUnaryOp(ExprOp op) {
    if (isLeafOp(op) || isBinaryOp(op) || isTernaryOp(op)) return false;
    if (isReductionOp(op)) return true;
    switch (op) {
        case ExprOp::LOGICAL_NOT:
        case ExprOp::CAST:
        case ExprOp::RESHAPE:
        case ExprOp::UNSQUEEZE:
        case ExprOp::SQUEEZE:
        case ExprOp::SOFTMAX:
            return true;
        default:
            return op >= ExprOp::NEG && op <= ExprOp::NORMCDF;
    }
}

// ---- canonical text -------------------------------------------------------------------------------------------------------
std::string opName(ExprOp op) {
    static const std::unordered_map<uint16_t, const char*> names = {
        {(uint16_t)ExprOp::INPUT, "input"}, {(uint16_t)ExprOp::RUNTIME_SCALAR, "runtime_scalar"},
        {(uint16_t)ExprOp::TENSOR_RUNTIME_SCALAR, "tensor_runtime_scalar"}, {(uint16_t)ExprOp::SCALAR_FP, "scalar"},
        {(uint16_t)ExprOp::ADD, "add"}, {(uint16_t)ExprOp::SUB, "sub"}, {(uint16_t)ExprOp::MUL, "mul"}, {(uint16_t)ExprOp::DIV, "div"},
        {(uint16_t)ExprOp::POW, "pow"}, {(uint16_t)ExprOp::EQUAL, "eq"}, {(uint16_t)ExprOp::NOT_EQUAL, "ne"}, {(uint16_t)ExprOp::LESS, "lt"},
        {(uint16_t)ExprOp::LESS_EQUAL, "le"}, {(uint16_t)ExprOp::GREATER, "gt"}, {(uint16_t)ExprOp::GREATER_EQUAL, "ge"},
        {(uint16_t)ExprOp::LOGICAL_AND, "and"}, {(uint16_t)ExprOp::LOGICAL_OR, "or"}, {(uint16_t)ExprOp::LOGICAL_NOT, "not"},
        {(uint16_t)ExprOp::CAST, "cast"}, {(uint16_t)ExprOp::WHERE, "where"}, {(uint16_t)ExprOp::NEG, "neg"}, {(uint16_t)ExprOp::ABS, "abs"},
        {(uint16_t)ExprOp::CEIL, "ceil"}, {(uint16_t)ExprOp::FLOOR, "floor"}, {(uint16_t)ExprOp::ROUND, "round"},
        {(uint16_t)ExprOp::TRUNC, "trunc"}, {(uint16_t)ExprOp::SIN, "sin"}, {(uint16_t)ExprOp::COS, "cos"}, {(uint16_t)ExprOp::TAN, "tan"},
        {(uint16_t)ExprOp::ASIN, "asin"}, {(uint16_t)ExprOp::ACOS, "acos"}, {(uint16_t)ExprOp::ATAN, "atan"}, {(uint16_t)ExprOp::SINH, "sinh"},
        {(uint16_t)ExprOp::COSH, "cosh"}, {(uint16_t)ExprOp::ASINH, "asinh"}, {(uint16_t)ExprOp::ACOSH, "acosh"},
        {(uint16_t)ExprOp::ATANH, "atanh"}, {(uint16_t)ExprOp::ERF, "erf"}, {(uint16_t)ExprOp::ERFC, "erfc"}, {(uint16_t)ExprOp::ERFCX, "erfcx"},
        {(uint16_t)ExprOp::ERFINV, "erfinv"}, {(uint16_t)ExprOp::ERFCINV, "erfcinv"}, {(uint16_t)ExprOp::TGAMMA, "tgamma"},
        {(uint16_t)ExprOp::LGAMMA, "lgamma"}, {(uint16_t)ExprOp::DIGAMMA, "digamma"}, {(uint16_t)ExprOp::EXP, "exp"},
        {(uint16_t)ExprOp::EXPM1, "expm1"}, {(uint16_t)ExprOp::EXP2, "exp2"}, {(uint16_t)ExprOp::EXP10, "exp10"}, {(uint16_t)ExprOp::LN, "ln"},
        {(uint16_t)ExprOp::LOG1P, "log1p"}, {(uint16_t)ExprOp::LOG2, "log2"}, {(uint16_t)ExprOp::LOG10, "log10"}, {(uint16_t)ExprOp::SQRT, "sqrt"},
        {(uint16_t)ExprOp::TANH, "tanh"}, {(uint16_t)ExprOp::NORMCDF, "normcdf"}, {(uint16_t)ExprOp::SOFTMAX, "softmax"}, {(uint16_t)ExprOp::ROPE, "rope"}, {(uint16_t)ExprOp::SEGMENTED_REDUCE_MIN_BACKWARD, "segmented_reduce_min_backward"}, {(uint16_t)ExprOp::SEGMENTED_REDUCE_MAX_BACKWARD, "segmented_reduce_max_backward"}, {(uint16_t)ExprOp::STRIDED_VIEW_BACKWARD, "strided_view_backward"}, {(uint16_t)ExprOp::SCAN_MIN_BACKWARD, "scan_min_backward"}, {(uint16_t)ExprOp::SCAN_MAX_BACKWARD, "scan_max_backward"}, {(uint16_t)ExprOp::SEGMENTED_SCAN_MIN_BACKWARD, "segmented_scan_min_backward"}, {(uint16_t)ExprOp::SEGMENTED_SCAN_MAX_BACKWARD, "segmented_scan_max_backward"}, {(uint16_t)ExprOp::FILL, "fill"},
        {(uint16_t)ExprOp::RESHAPE, "reshape"}, {(uint16_t)ExprOp::UNSQUEEZE, "unsqueeze"}, {(uint16_t)ExprOp::SQUEEZE, "squeeze"},
        {(uint16_t)ExprOp::MIN, "min"}, {(uint16_t)ExprOp::MAX, "max"}, {(uint16_t)ExprOp::MIN_GRAD_LEFT, "min_grad_left"},
        {(uint16_t)ExprOp::MIN_GRAD_RIGHT, "min_grad_right"}, {(uint16_t)ExprOp::MAX_GRAD_LEFT, "max_grad_left"},
        {(uint16_t)ExprOp::MAX_GRAD_RIGHT, "max_grad_right"}, {(uint16_t)ExprOp::REDUCE_SUM, "reduce_sum"},
        {(uint16_t)ExprOp::REDUCE_PROD, "reduce_prod"}, {(uint16_t)ExprOp::REDUCE_MIN, "reduce_min"}, {(uint16_t)ExprOp::REDUCE_MAX, "reduce_max"},
        {(uint16_t)ExprOp::REDUCE_ARGMIN, "argmin"}, {(uint16_t)ExprOp::REDUCE_ARGMAX, "argmax"}, {(uint16_t)ExprOp::REDUCE_AVG, "reduce_mean"},
        {(uint16_t)ExprOp::REDUCE_NORM1, "reduce_norm1"}, {(uint16_t)ExprOp::REDUCE_NORM2, "reduce_norm2"},
        {(uint16_t)ExprOp::SEGMENTED_REDUCE_SUM, "segmented_reduce_sum"}, {(uint16_t)ExprOp::SEGMENTED_REDUCE_MIN, "segmented_reduce_min"},
        {(uint16_t)ExprOp::SEGMENTED_REDUCE_MAX, "segmented_reduce_max"}, {(uint16_t)ExprOp::SEGMENTED_REDUCE_MEAN, "segmented_reduce_mean"},
        {(uint16_t)ExprOp::STRIDED_VIEW, "strided_view"}, {(uint16_t)ExprOp::TRANSPOSE, "transpose"},
        {(uint16_t)ExprOp::TAKE_ALONG_AXIS, "take_along_axis"}, {(uint16_t)ExprOp::SCAN, "scan"}, {(uint16_t)ExprOp::SEGMENTED_SCAN, "segmented_scan"}, {(uint16_t)ExprOp::REDUCE_MIN_BACKWARD, "reduce_min_backward"}, {(uint16_t)ExprOp::REDUCE_MAX_BACKWARD, "reduce_max_backward"},
        {(uint16_t)ExprOp::SEGMENTED_BROADCAST, "segmented_broadcast"}, {(uint16_t)ExprOp::RAGGED_VALUEWISE_EXTENT, "ragged_valuewise_extent"},
    };
    auto it = names.find(static_cast<uint16_t>(op));
    return it == names.end() ? "op" + std::to_string(static_cast<int>(op)) : it->second;
}

bool isCommutative(ExprOp op) {
    switch (op) {
        case ExprOp::ADD:
        case ExprOp::MUL:
        case ExprOp::MIN:
        case ExprOp::MAX:
        case ExprOp::EQUAL:
        case ExprOp::NOT_EQUAL:
        case ExprOp::LOGICAL_AND:
        case ExprOp::LOGICAL_OR:
            return true;
        default:
            return false;
    }
}

std::string formatFloatCanonical(double x) {
    char buffer[64];
    std::snprintf(buffer, sizeof buffer, "%.17g", x);
    return buffer;
}

static std::string axesText(const std::vector<uint64_t>& v) {
    std::string s = "[";
    for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + std::to_string(v[i]);
    return s + "]";
}

std::string canonicalizeNode(const PhysicalExpression& expr, uint32_t nodeIndex, std::unordered_map<uint32_t, std::string>& memo) {
    auto hit = memo.find(nodeIndex);
    if (hit != memo.end()) return hit->second;
    const ExprNode& n = expr.nodes.at(nodeIndex);
    std::string text = opName(n.op);
    auto dtypes = [&] {
        std::string s;
        if (n.output_dtype) s += std::string(":o=") + dataTypeName(*n.output_dtype);
        if (n.compute_dtype) s += std::string(":c=") + dataTypeName(*n.compute_dtype);
        if (n.input_tensor_dtype) s += std::string(":i=") + dataTypeName(*n.input_tensor_dtype);
        return s;
    };
    if (n.op == ExprOp::INPUT || n.op == ExprOp::RUNTIME_SCALAR || n.op == ExprOp::TENSOR_RUNTIME_SCALAR) {
        text += "#" + std::to_string(n.input_slot) + dtypes();
    } else if (n.op == ExprOp::SCALAR_FP) {
        text += "(" + formatFloatCanonical(n.scalar_fp) + ")" + dtypes();
    } else if (n.op == ExprOp::FILL) {
        text += "(" + formatFloatCanonical(n.scalar_fp) + "," + axesText(n.fill_dims) + ")" + dtypes();
    } else {
        std::vector<std::string> kids;
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != UINT32_MAX) kids.push_back(canonicalizeNode(expr, c, memo));
        if (isCommutative(n.op) && kids.size() == 2 && kids[1] < kids[0]) std::swap(kids[0], kids[1]);
        text += dtypes();
        if (n.op == ExprOp::TAKE_ALONG_AXIS) text += ":axis=" + axesText(n.reduction_axes);
        if (n.op == ExprOp::ROPE) text += ":" + ropeKey(n);
        if (isScanBackwardOp(n.op)) {
            text += std::string(n.scan_mode == ScanMode::Inclusive ? ":inclusive" : ":exclusive") + (n.scan_reverse ? ":reverse" : "");
        }
        if (isScanOp(n.op)) {
            static const char* const scanNames[] = {"sum", "min", "max", "product", "arg_min", "arg_max"};
            text += std::string(":") + scanNames[static_cast<int>(n.scan_op)] + (n.scan_mode == ScanMode::Inclusive ? ":inclusive" : ":exclusive") +
                    (n.scan_reverse ? ":reverse" : "") + ":axis=" + (n.scan_axis == UINT64_MAX ? std::string("last") : std::to_string(n.scan_axis));
        }
        if (isReductionOp(n.op) || isWinnerRoutingOp(n.op)) text += ":axes=" + axesText(n.reduction_axes) + ":squeeze=" + axesText(n.squeeze_axes);
        if (n.op == ExprOp::RESHAPE) text += ":dims=" + axesText(n.reshape_dims);
        if (n.op == ExprOp::UNSQUEEZE) text += ":axes=" + axesText(n.unsqueeze_axes);
        if (n.op == ExprOp::SQUEEZE) text += ":axes=" + axesText(n.squeeze_axes);
        if (n.op == ExprOp::STRIDED_VIEW_BACKWARD) text += ":into=" + axesText(n.fill_dims);
        if (n.op == ExprOp::STRIDED_VIEW || n.op == ExprOp::STRIDED_VIEW_BACKWARD) {
            text += ":dims=" + axesText(n.view_dims) + ":strides=" + axesText(n.view_strides) + ":offset=" + std::to_string(n.view_element_offset);
        }
        if (isRaggedOp(n.op)) {
            text += ":ragged=[" + std::to_string(n.ragged_runtime_batch_size) + "," + std::to_string(n.ragged_runtime_max_active_values) + "," +
                    std::to_string(n.ragged_runtime_elements_per_value) + "]";
            if (n.op == ExprOp::SEGMENTED_BROADCAST) text += n.segmented_broadcast_normalize_by_length ? ":normalized" : "";
        }
        if (n.op == ExprOp::SOFTMAX) {
            text += std::string(":alg=") + std::to_string(static_cast<int>(n.softmax_algorithm)) + ":mode=" + std::to_string(static_cast<int>(n.softmax_mode));
        }
        text += "(";
        for (size_t i = 0; i < kids.size(); ++i) text += (i ? "," : "") + kids[i];
        text += ")";
    }
    memo[nodeIndex] = text;
    return text;
}

std::string canonicalize(const PhysicalExpression& expr) {
    std::unordered_map<uint32_t, std::string> memo;
    return canonicalizeNode(expr, expr.output_node, memo);
}

std::string canonicalize(const PhysicalOutputs& outputs) {
    if (!outputs.expr) throw std::runtime_error("canonicalize requires a non-null expression graph.");
    std::unordered_map<uint32_t, std::string> memo;
    std::vector<std::string> parts;
    for (const NamedOutput& o : outputs.outputs) parts.push_back(o.name + "=" + canonicalizeNode(*outputs.expr, o.node_idx, memo));
    std::sort(parts.begin(), parts.end());
    std::string text;
    for (const std::string& p : parts) text += p + ";";
    return text;
}

std::string expressionHash(const PhysicalOutputs& outputs) {
    // FNV-1a over the canonical text, printed as 16 hex digits
    const std::string text = canonicalize(outputs);
    uint64_t h = 1469598103934665603ull;
    for (unsigned char c : text) {
        h ^= c;
        h *= 1099511628211ull;
    }
    char buffer[32];
    std::snprintf(buffer, sizeof buffer, "%016llx", static_cast<unsigned long long>(h));
    return buffer;
}

}  // namespace ThorImplementation
