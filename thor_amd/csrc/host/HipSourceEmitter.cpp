#include "HipSourceEmitter.h"

#include "ReductionPlanner.h"  // deviceTypeName
#include "thorhip_numeric_embed.h"

#include <algorithm>
#include <cstdlib>
#include <iomanip>
#include <limits>
#include <optional>
#include <sstream>
#include <stdexcept>

namespace ThorImplementation {

namespace {

bool isFloatHeld(DataType d) {  // dtypes whose in-kernel value lives in a `float`
    return d == DataType::FP32 || d == DataType::BF16 || d == DataType::FP8_E4M3 || d == DataType::FP8_E5M2;
}
bool isIntegral(DataType d) {
    switch (d) {
        case DataType::INT8:
        case DataType::INT16:
        case DataType::INT32:
        case DataType::INT64:
        case DataType::UINT8:
        case DataType::UINT16:
        case DataType::UINT32:
        case DataType::UINT64:
            return true;
        default:
            return false;
    }
}

const char* unaryFunction(ExprOp op) {
    switch (op) {
        case ExprOp::ABS: return "fabsf";
        case ExprOp::CEIL: return "ceilf";
        case ExprOp::FLOOR: return "floorf";
        case ExprOp::ROUND: return "roundf";
        case ExprOp::TRUNC: return "truncf";
        case ExprOp::SIN: return "sinf";
        case ExprOp::COS: return "cosf";
        case ExprOp::TAN: return "tanf";
        case ExprOp::ASIN: return "asinf";
        case ExprOp::ACOS: return "acosf";
        case ExprOp::ATAN: return "atanf";
        case ExprOp::SINH: return "sinhf";
        case ExprOp::COSH: return "coshf";
        case ExprOp::ASINH: return "asinhf";
        case ExprOp::ACOSH: return "acoshf";
        case ExprOp::ATANH: return "atanhf";
        case ExprOp::ERF: return "erff";
        case ExprOp::ERFC: return "erfcf";
        case ExprOp::ERFCX: return "erfcxf";
        case ExprOp::ERFINV: return "erfinvf";
        case ExprOp::ERFCINV: return "erfcinvf";
        case ExprOp::TGAMMA: return "tgammaf";
        case ExprOp::LGAMMA: return "lgammaf";
        case ExprOp::DIGAMMA: return "thor::digammaf";
        case ExprOp::EXP: return "expf";
        case ExprOp::EXPM1: return "expm1f";
        case ExprOp::EXP2: return "exp2f";
        case ExprOp::EXP10: return "exp10f";
        case ExprOp::LN: return "logf";
        case ExprOp::LOG1P: return "log1pf";
        case ExprOp::LOG2: return "log2f";
        case ExprOp::LOG10: return "log10f";
        case ExprOp::SQRT: return "sqrtf";
        case ExprOp::TANH: return "tanhf";
        case ExprOp::NORMCDF: return "normcdff";
        default: return nullptr;
    }
}

uint64_t opFlops(ExprOp op) {
    switch (op) {
        case ExprOp::ADD:
        case ExprOp::SUB:
        case ExprOp::MUL:
        case ExprOp::NEG:
        case ExprOp::ABS:
        case ExprOp::MIN:
        case ExprOp::MAX:
            return 1;
        case ExprOp::DIV:
        case ExprOp::SQRT:
            return 4;
        case ExprOp::CAST:
        case ExprOp::RESHAPE:
        case ExprOp::SQUEEZE:
        case ExprOp::UNSQUEEZE:
            return 0;
        default:
            return unaryFunction(op) ? 8 : 1;
    }
}

bool isConstZero(const PhysicalExpression& e, uint32_t n) {
    double v;
    return tryFoldConstant(e, n, v) && v == 0.0;
}
bool isConstOne(const PhysicalExpression& e, uint32_t n) {
    double v;
    return tryFoldConstant(e, n, v) && v == 1.0;
}

// x + 0, 0 + x, x - 0, x * 1, 1 * x, x / 1 and pure shape ops evaluate to their operand
bool aliasSource(const PhysicalExpression& e, uint32_t nodeIndex, uint32_t& source) {
    const ExprNode& n = e.nodes[nodeIndex];
    switch (n.op) {
        case ExprOp::RESHAPE:
        case ExprOp::UNSQUEEZE:
        case ExprOp::SQUEEZE:
        case ExprOp::RAGGED_VALUEWISE_EXTENT:  // the values themselves; the extent limits the kernel, not the arithmetic
            source = n.lhs;
            return true;
        case ExprOp::ADD:
            if (isConstZero(e, n.lhs)) return source = n.rhs, true;
            if (isConstZero(e, n.rhs)) return source = n.lhs, true;
            return false;
        case ExprOp::SUB:
            if (isConstZero(e, n.rhs)) return source = n.lhs, true;
            return false;
        case ExprOp::MUL:
            if (isConstOne(e, n.lhs)) return source = n.rhs, true;
            if (isConstOne(e, n.rhs)) return source = n.lhs, true;
            return false;
        case ExprOp::DIV:
            if (isConstOne(e, n.rhs)) return source = n.lhs, true;
            return false;
        default:
            return false;
    }
}

}  // namespace

const char* valueCType(DataType dtype) {
    switch (dtype) {
        case DataType::FP32:
        case DataType::BF16:
        case DataType::FP8_E4M3:
        case DataType::FP8_E5M2:
            return "float";
        case DataType::FP16: return "_Float16";
        case DataType::FP64: return "double";
        case DataType::BOOLEAN: return "bool";
        case DataType::INT8: return "thor::i8";
        case DataType::INT16: return "thor::i16";
        case DataType::INT32: return "thor::i32";
        case DataType::INT64: return "thor::i64";
        case DataType::UINT8: return "thor::u8";
        case DataType::UINT16: return "thor::u16";
        case DataType::UINT32: return "thor::u32";
        case DataType::UINT64: return "thor::u64";
        default: break;
    }
    throw std::runtime_error(std::string("No in-kernel value type for dtype ") + dataTypeName(dtype));
}

std::string floatLiteral(double value) {
    // nine significant digits and an `f` suffix: the literal text the reference prints for the same constant
    if (value != value) return "__builtin_nanf(\"\")";
    if (value == std::numeric_limits<double>::infinity()) return "__builtin_inff()";
    if (value == -std::numeric_limits<double>::infinity()) return "(-__builtin_inff())";
    std::ostringstream oss;
    oss << std::setprecision(9) << std::defaultfloat << value;
    std::string s = oss.str();
    if (s.find('.') == std::string::npos && s.find('e') == std::string::npos && s.find('E') == std::string::npos) s += ".0";
    return s + "f";
}

std::string castValueExpr(const std::string& x, DataType from, DataType to) {
    if (from == to) return x;
    // every conversion goes through the fp32 image of the source value, as `static_cast` chains do in the reference
    std::string asFloat;
    if (isFloatHeld(from)) {
        asFloat = x;
    } else if (from == DataType::INT64 || from == DataType::UINT64) {
        // not the cast: its expansion shifts 64 bits by a register amount, which this device gets wrong in one register placement
        asFloat = "thor::toFloat((" + std::string(from == DataType::INT64 ? "thor::i64" : "thor::u64") + ")(" + x + "))";
    } else if (from == DataType::FP16 || isIntegral(from) || from == DataType::FP64) {
        asFloat = "(float)(" + x + ")";
    } else if (from == DataType::BOOLEAN) {
        asFloat = "((" + x + ") ? 1.0f : 0.0f)";
    } else {
        throw std::runtime_error(std::string("Unsupported cast source dtype in fused stage emitter: ") + dataTypeName(from));
    }
    switch (to) {
        case DataType::FP32: return asFloat;
        case DataType::FP16: return "thor::halfFromFloat(" + asFloat + ")";
        case DataType::BF16: return "thor::roundBf16(" + asFloat + ")";
        case DataType::FP8_E4M3: return "thor::roundE4m3(" + asFloat + ")";
        case DataType::FP8_E5M2: return "thor::roundE5m2(" + asFloat + ")";
        case DataType::BOOLEAN: return "((" + asFloat + ") != 0.0f)";
        case DataType::FP64: return "(double)(" + asFloat + ")";
        default:
            if (isIntegral(to)) {
                if (isIntegral(from)) return std::string("(") + valueCType(to) + ")(" + x + ")";
                return std::string("(") + valueCType(to) + ")(" + asFloat + ")";
            }
    }
    throw std::runtime_error(std::string("Unsupported cast destination dtype in fused stage emitter: ") + dataTypeName(to));
}

std::string storageToValueExpr(const std::string& x, DataType dtype) {
    switch (dtype) {
        case DataType::FP16: return "thor::asHalf(" + x + ")";
        case DataType::BF16:
        case DataType::FP8_E4M3:
        case DataType::FP8_E5M2:
            return "thor::toFloat(" + x + ")";
        case DataType::BOOLEAN: return "((" + x + ").bits != 0)";
        default: return x;
    }
}

std::string valueToStorageExpr(const std::string& x, DataType dtype) {
    switch (dtype) {
        case DataType::FP16: return "thor::fromHalf(" + x + ")";
        case DataType::BF16: return "thor::bf16FromExact(" + x + ")";  // bf16 values are held as floats that need no rounding
        case DataType::FP8_E4M3: return "thor::toE4m3(" + x + ")";
        case DataType::FP8_E5M2: return "thor::toE5m2(" + x + ")";
        case DataType::BOOLEAN: return "thor::makeBoolean(" + x + ")";
        default: return x;
    }
}

DataType emittedValueDType(const ExprNode& node) {
    if (Expression::isLeafOp(node.op)) {
        if (!node.output_dtype) throw std::runtime_error("Leaf node without a resolved output dtype.");
        return *node.output_dtype;
    }
    if (!node.compute_dtype) throw std::runtime_error("Node without a resolved compute dtype.");
    return *node.compute_dtype;
}

bool tryFoldConstant(const PhysicalExpression& expr, uint32_t nodeIndex, double& value) {
    const ExprNode& n = expr.nodes.at(nodeIndex);
    switch (n.op) {
        case ExprOp::SCALAR_FP:
        case ExprOp::FILL:
            value = n.scalar_fp;
            return true;
        case ExprOp::RESHAPE:
        case ExprOp::UNSQUEEZE:
        case ExprOp::SQUEEZE:
            return tryFoldConstant(expr, n.lhs, value);
        case ExprOp::NEG:
            if (!tryFoldConstant(expr, n.lhs, value)) return false;
            value = -value;
            return true;
        case ExprOp::ADD:
        case ExprOp::SUB:
        case ExprOp::MUL:
        case ExprOp::DIV: {
            double a, b;
            if (!tryFoldConstant(expr, n.lhs, a) || !tryFoldConstant(expr, n.rhs, b)) return false;
            value = n.op == ExprOp::ADD ? a + b : n.op == ExprOp::SUB ? a - b : n.op == ExprOp::MUL ? a * b : a / b;
            return true;
        }
        default:
            return false;
    }
}

namespace {
// exp(-max(-x, 0)) evaluated in fp32 - the numerator of the reference's overflow-safe sigmoid, exp(-max(-x, 0)) / (1 + exp(-|x|))
// (Expression.cpp:3261-3296 there).  For x < 0 its argument -(-x) is x = -|x| bit for bit; otherwise (x >= 0, -0, NaN: the
// maximum ignores a NaN) the argument is -0 and the value exactly 1.  Written as `x < 0 ? exp(-|x|) : 1` it gives the same
// bits and shares its exponential with the denominator's: one exponential per sigmoid instead of two.
bool isExpOfMinusPositivePart(const PhysicalExpression& expr, uint32_t nodeIndex, uint32_t& x) {
    auto fp32 = [&](uint32_t i) { return i != UINT32_MAX && emittedValueDType(expr.nodes[i]) == DataType::FP32; };
    const ExprNode& e = expr.nodes[nodeIndex];
    if (e.op != ExprOp::EXP || !fp32(nodeIndex) || !fp32(e.lhs)) return false;
    if (std::getenv("THOR_SIGMOID_TWO_EXPONENTIALS")) return false;  // diagnostic switch: the literal form, for A/B runs
    const ExprNode& outer = expr.nodes[e.lhs];
    if (outer.op != ExprOp::NEG || !fp32(outer.lhs)) return false;
    const ExprNode& larger = expr.nodes[outer.lhs];
    if (larger.op != ExprOp::MAX) return false;
    for (int side = 0; side < 2; ++side) {
        const uint32_t negated = side == 0 ? larger.lhs : larger.rhs, zero = side == 0 ? larger.rhs : larger.lhs;
        double constant;
        if (!tryFoldConstant(expr, zero, constant) || constant != 0.0 || !fp32(negated)) continue;
        const ExprNode& inner = expr.nodes[negated];
        if (inner.op != ExprOp::NEG || inner.lhs == UINT32_MAX) continue;
        x = inner.lhs;
        return true;
    }
    return false;
}
}  // namespace

BodyEmitter::BodyEmitter(const PhysicalExpression& expr)
    : expr(expr), valueDType(expr.nodes.size()), names(expr.nodes.size()), rowDivisors(expr.nodes.size()) {}

void BodyEmitter::defineSource(uint32_t node, DataType dtype, const std::string& name) {
    valueDType[node] = dtype;
    names[node] = name.empty() ? "t" + std::to_string(node) : name;
}

std::string BodyEmitter::ref(uint32_t child, DataType target) const {
    double folded;
    if (!valueDType[child].has_value() && tryFoldConstant(expr, child, folded)) {
        return castValueExpr(floatLiteral(folded), DataType::FP32, target);
    }
    if (!valueDType[child].has_value()) throw std::logic_error("Fused stage emitter referenced a value before its definition.");
    return castValueExpr(names[child], valueDType[child].value(), target);
}

std::vector<uint32_t> BodyEmitter::collect(const std::vector<uint32_t>& roots) const {
    std::vector<char> need(expr.nodes.size(), 0);
    std::vector<uint32_t> stack(roots.begin(), roots.end());
    while (!stack.empty()) {
        const uint32_t n = stack.back();
        stack.pop_back();
        if (need[n] || valueDType[n].has_value()) continue;
        double folded;
        if (tryFoldConstant(expr, n, folded)) continue;
        need[n] = 1;
        const ExprNode& node = expr.nodes[n];
        if (node.op == ExprOp::RAGGED_VALUEWISE_EXTENT) {
            stack.push_back(node.lhs);  // the offsets are read as the kernel's extent, not as a value
            continue;
        }
        for (uint32_t c : {node.lhs, node.rhs, node.aux})
            if (c != UINT32_MAX) stack.push_back(c);
    }
    std::vector<uint32_t> order;
    for (uint32_t i = 0; i < need.size(); ++i)
        if (need[i]) order.push_back(i);
    return order;
}

uint64_t BodyEmitter::emit(std::string& out, uint32_t nodeIndex, const std::string& indent) {
    const ExprNode& n = expr.nodes[nodeIndex];
    const DataType dtype = emittedValueDType(n);
    const std::string name = "t" + std::to_string(nodeIndex);
    const std::string decl = indent + "const " + valueCType(dtype) + " " + name + " = ";
    auto define = [&] {
        valueDType[nodeIndex] = dtype;
        names[nodeIndex] = name;
    };
    if (n.op == ExprOp::RUNTIME_SCALAR) {
        out += decl + castValueExpr("s" + std::to_string(n.input_slot), DataType::FP32, dtype) + ";\n";
        define();
        return 0;
    }
    if (n.op == ExprOp::INPUT) throw std::runtime_error("Fused stage reads an input that was not bound as a kernel operand.");
    uint32_t source;
    uint64_t flops = 0;
    if (aliasSource(expr, nodeIndex, source)) {
        out += decl + ref(source, dtype) + ";\n";
    } else if (n.op == ExprOp::CAST) {
        out += decl + ref(n.lhs, dtype) + ";\n";
    } else if (n.op == ExprOp::WHERE) {
        out += decl + "(" + ref(n.lhs, DataType::BOOLEAN) + " ? " + ref(n.rhs, dtype) + " : " + ref(n.aux, dtype) + ");\n";
        flops = 1;
    } else if (Expression::isBinaryOp(n.op)) {
        out += decl + binary(n, dtype) + ";\n";
        flops = opFlops(n.op);
    } else if (uint32_t x; isExpOfMinusPositivePart(expr, nodeIndex, x) && defined(x)) {
        const std::string value = ref(x, DataType::FP32);
        out += decl + "((" + value + " < 0.0f) ? expf((-fabsf(" + value + "))) : 1.0f);\n";
        flops = opFlops(n.op);
    } else {
        out += decl + unary(n, dtype) + ";\n";
        flops = opFlops(n.op);
    }
    define();
    return flops;
}

std::string BodyEmitter::unary(const ExprNode& n, DataType c) const {
    if (n.op == ExprOp::NEG) {
        if (c == DataType::FP32 || c == DataType::FP16 || c == DataType::BF16) return "(-" + ref(n.lhs, c) + ")";
        return castValueExpr("(-" + ref(n.lhs, DataType::FP32) + ")", DataType::FP32, c);
    }
    if (n.op == ExprOp::LOGICAL_NOT) {
        if (c == DataType::BOOLEAN) return "(!" + ref(n.lhs, DataType::BOOLEAN) + ")";
        return "(!(" + ref(n.lhs, DataType::FP32) + " != 0.0f))";
    }
    if (const char* fn = unaryFunction(n.op)) {
        // evaluated on an fp32 copy of the operand and converted back to the compute dtype
        return castValueExpr(std::string(fn) + "(" + ref(n.lhs, DataType::FP32) + ")", DataType::FP32, c);
    }
    throw std::runtime_error("Unsupported unary op in fused stage emitter: " + opName(n.op));
}

std::string BodyEmitter::binary(const ExprNode& n, DataType c) const {
    const bool native = c == DataType::FP32 || c == DataType::FP16 || c == DataType::BF16;
    auto arithmetic = [&](const char* op) {
        if (native || (n.op == ExprOp::SUB && (c == DataType::UINT32 || c == DataType::UINT64))) {
            const std::string text = "(" + ref(n.lhs, c) + " " + op + " " + ref(n.rhs, c) + ")";
            // bf16 arithmetic: exact fp32 operation on bf16 operands, then one rounding to bf16
            return c == DataType::BF16 ? "thor::roundBf16" + text : text;
        }
        return castValueExpr("(" + ref(n.lhs, DataType::FP32) + " " + op + " " + ref(n.rhs, DataType::FP32) + ")", DataType::FP32, c);
    };
    const std::string a = ref(n.lhs, DataType::FP32), b = ref(n.rhs, DataType::FP32);
    switch (n.op) {
        case ExprOp::ADD: return arithmetic("+");
        case ExprOp::SUB: return arithmetic("-");
        case ExprOp::MUL: return arithmetic("*");
        case ExprOp::DIV:
            if (c == DataType::FP32 && !rowDivisors[n.rhs].empty()) return rowDivisors[n.rhs] + ".divide(" + a + ")";
            return arithmetic("/");
        case ExprOp::POW: return castValueExpr("powf(" + a + ", " + b + ")", DataType::FP32, c);
        case ExprOp::MIN: return castValueExpr("fminf(" + a + ", " + b + ")", DataType::FP32, c);
        case ExprOp::MAX: return castValueExpr("fmaxf(" + a + ", " + b + ")", DataType::FP32, c);
        case ExprOp::EQUAL: return "(" + a + " == " + b + ")";
        case ExprOp::NOT_EQUAL: return "(" + a + " != " + b + ")";
        case ExprOp::LESS: return "(" + a + " < " + b + ")";
        case ExprOp::LESS_EQUAL: return "(" + a + " <= " + b + ")";
        case ExprOp::GREATER: return "(" + a + " > " + b + ")";
        case ExprOp::GREATER_EQUAL: return "(" + a + " >= " + b + ")";
        case ExprOp::LOGICAL_AND:
            if (c == DataType::BOOLEAN) return "(" + ref(n.lhs, c) + " && " + ref(n.rhs, c) + ")";
            return "((" + a + " != 0.0f) && (" + b + " != 0.0f))";
        case ExprOp::LOGICAL_OR:
            if (c == DataType::BOOLEAN) return "(" + ref(n.lhs, c) + " || " + ref(n.rhs, c) + ")";
            return "((" + a + " != 0.0f) || (" + b + " != 0.0f))";
        case ExprOp::MIN_GRAD_LEFT:
        case ExprOp::MAX_GRAD_RIGHT:
            return castValueExpr("((" + a + " < " + b + ") ? 1.0f : ((" + a + " > " + b + ") ? 0.0f : 0.5f))", DataType::FP32, c);
        case ExprOp::MIN_GRAD_RIGHT:
        case ExprOp::MAX_GRAD_LEFT:
            return castValueExpr("((" + a + " > " + b + ") ? 1.0f : ((" + a + " < " + b + ") ? 0.0f : 0.5f))", DataType::FP32, c);
        default: break;
    }
    throw std::runtime_error("Unsupported binary op in fused stage emitter: " + opName(n.op));
}

namespace {

struct CollapsedLayout {
    std::vector<uint64_t> dims;                       // collapsed output dims
    std::vector<std::vector<uint64_t>> operandStride;  // [operand][axis]
};

// Right-aligns every operand against the output shape (stride 0 on broadcast axes), then merges neighbouring axes that
// every operand and the dense output address as one longer axis.
CollapsedLayout collapseForBroadcast(const FusedKernelRequest& r) {
    const size_t rank = r.outputDims.size();
    std::vector<std::vector<uint64_t>> strides(r.operands.size(), std::vector<uint64_t>(rank, 0));
    for (size_t o = 0; o < r.operands.size(); ++o) {
        const KernelOperand& op = r.operands[o];
        if (op.dims.size() > rank) throw std::runtime_error("Fused stage operand has a higher rank than the stage output.");
        const size_t shift = rank - op.dims.size();
        for (size_t a = 0; a < op.dims.size(); ++a) {
            const uint64_t d = op.dims[a], outDim = r.outputDims[a + shift];
            if (d == outDim) {
                strides[o][a + shift] = d == 1 ? 0 : op.strides[a];
            } else if (d == 1) {
                strides[o][a + shift] = 0;
            } else {
                throw std::runtime_error("Fused stage operand shape does not broadcast to the stage output shape.");
            }
        }
    }
    std::vector<uint64_t> outStride(rank, 1);
    for (size_t a = rank; a-- > 1;) outStride[a - 1] = outStride[a] * r.outputDims[a];

    CollapsedLayout c;
    c.operandStride.assign(r.operands.size(), {});
    std::vector<uint64_t> outC;
    for (size_t a = 0; a < rank; ++a) {
        const uint64_t d = r.outputDims[a];
        if (d == 1) continue;
        bool merge = !c.dims.empty();
        if (merge) {
            for (size_t o = 0; o < r.operands.size() && merge; ++o) merge = c.operandStride[o].back() == d * strides[o][a];
            merge = merge && outC.back() == d * outStride[a];
        }
        if (merge) {
            c.dims.back() *= d;
            for (size_t o = 0; o < r.operands.size(); ++o) c.operandStride[o].back() = strides[o][a];
            outC.back() = outStride[a];
        } else {
            c.dims.push_back(d);
            for (size_t o = 0; o < r.operands.size(); ++o) c.operandStride[o].push_back(strides[o][a]);
            outC.push_back(outStride[a]);
        }
    }
    if (c.dims.empty()) {
        c.dims.push_back(1);
        for (auto& s : c.operandStride) s.push_back(0);
    }
    return c;
}

}  // namespace

EmittedKernel emitFusedKernel(const FusedKernelRequest& r) {
    if (!r.expr || r.outputs.empty()) throw std::runtime_error("Fused stage needs an expression and at least one output.");
    const PhysicalExpression& expr = *r.expr;
    EmittedKernel k;
    k.numel = 1;
    for (uint64_t d : r.outputDims) k.numel *= d;
    k.numelIs64 = k.numel >= (1ull << 31);
    const char* indexType = k.numelIs64 ? "unsigned long long" : "unsigned int";

    // flat when every operand has the output's element count, is dense, and agrees on the non-singleton dims
    auto stripOnes = [](const std::vector<uint64_t>& d) {
        std::vector<uint64_t> out;
        for (uint64_t v : d)
            if (v != 1) out.push_back(v);
        return out;
    };
    const std::vector<uint64_t> outCore = stripOnes(r.outputDims);
    k.flat = true;
    // a single-element operand (a scalar kept in device memory) is read at [0] and does not decide the kernel's form
    std::vector<char> single(r.operands.size(), 0);
    for (size_t o = 0; o < r.operands.size(); ++o) {
        uint64_t count = 1;
        for (uint64_t d : r.operands[o].dims) count *= d;
        single[o] = count == 1 && k.numel > 1;
    }
    for (size_t o = 0; o < r.operands.size(); ++o) {
        const KernelOperand& op = r.operands[o];
        if (single[o]) continue;
        uint64_t expected = 1;
        bool dense = true;
        for (size_t a = op.dims.size(); a-- > 0;) {
            if (op.dims[a] != 1 && op.strides[a] != expected) dense = false;
            expected *= op.dims[a];
        }
        if (!dense || stripOnes(op.dims) != outCore) k.flat = false;
    }

    // widest element decides the vector length: one 16-byte access for it, narrower operands move fewer bytes
    uint32_t widest = 1;
    for (size_t o = 0; o < r.operands.size(); ++o)
        if (!single[o]) widest = std::max(widest, dataTypeSizeInBytes(r.operands[o].storageDType));
    for (const KernelOutput& out : r.outputs) widest = std::max(widest, dataTypeSizeInBytes(out.storageDType));
    int vec = static_cast<int>(16 / widest);

    CollapsedLayout layout;
    if (!k.flat) layout = collapseForBroadcast(r);
    auto fits = [&](int v) {
        for (const KernelOutput& out : r.outputs)
            if (out.alignmentBytes % (static_cast<uint64_t>(v) * dataTypeSizeInBytes(out.storageDType)) != 0) return false;
        // operands only have to be aligned to their element: a vector of an operand that begins inside a word (a view a few
        // elements into its storage, rows whose pitch no vector divides) is read where it lies, at the rate of aligned loads
        for (size_t o = 0; o < r.operands.size(); ++o)
            if (!single[o] && r.operands[o].alignmentBytes % dataTypeSizeInBytes(r.operands[o].storageDType) != 0) return false;
        if (k.flat) return true;
        if (layout.dims.back() % v != 0) return false;
        if (r.extent.has_value() && r.extent->elementsPerValue % v != 0) return false;  // a vector never straddles the last active row
        for (size_t o = 0; o < r.operands.size(); ++o)
            if (layout.operandStride[o].back() > 1) return false;  // neither contiguous nor broadcast along the innermost axis
        return true;
    };
    while (vec > 1 && !fits(vec)) vec /= 2;
    // which operands are read with aligned vector loads at the chosen length
    auto operandAligned = [&](size_t o, int v) {
        if (r.operands[o].alignmentBytes % (static_cast<uint64_t>(v) * dataTypeSizeInBytes(r.operands[o].storageDType)) != 0) return false;
        if (!k.flat)
            for (size_t a = 0; a + 1 < layout.operandStride[o].size(); ++a)
                if (layout.operandStride[o][a] % v != 0) return false;
        return true;
    };
    auto vectorLoad = [&](size_t o, int v) { return operandAligned(o, v) ? ".loadStream(" : ".loadStreamUnaligned("; };

    // Operands whose contiguous axis is another axis of the output than the innermost one (transposes, permuted views): read
    // through LDS tiles, so that both the operand and the output are addressed along their own contiguous axis.
    int tileAxis = -1;
    std::vector<char> viaTile(r.operands.size(), 0);
    if (!k.flat && layout.dims.size() >= 2 && !r.extent.has_value() && r.gathers.empty()) {
        bool consistent = true;
        for (size_t o = 0; o < r.operands.size() && consistent; ++o) {
            const std::vector<uint64_t>& st = layout.operandStride[o];
            if (st.back() <= 1) continue;
            int axis = -1;
            for (size_t a = 0; a + 1 < st.size(); ++a)
                if (st[a] == 1 && layout.dims[a] > 1) axis = static_cast<int>(a);
            if (axis < 0) continue;  // contiguous nowhere: strided scalar reads
            if (tileAxis >= 0 && tileAxis != axis) consistent = false;
            tileAxis = axis;
            viaTile[o] = 1;
        }
        if (!consistent || tileAxis < 0 || layout.dims[tileAxis] < 16 || layout.dims.back() < 16) tileAxis = -1;
    }
    const bool tiled = tileAxis >= 0;
    if (tiled) vec = 1;
    // An innermost extent (or an operand's stride) that no vector length divides: the lanes still own vectors of the dense
    // output, which may straddle rows; operands laid out like the output are read as vectors too, the others element by
    // element at coordinates that are carried along the vector.
    bool straddling = false;
    std::vector<char> likeOutput(r.operands.size(), 0);
    if (!k.flat && !tiled && vec == 1 && !r.extent.has_value() && r.gathers.empty() && k.numel >= 4096) {
        int wide = static_cast<int>(16 / widest);
        std::vector<uint64_t> dense(layout.dims.size(), 1);
        for (size_t a = layout.dims.size(); a-- > 1;) dense[a - 1] = dense[a] * layout.dims[a];
        for (size_t o = 0; o < r.operands.size(); ++o) {
            likeOutput[o] = !single[o];
            for (size_t a = 0; a < layout.dims.size(); ++a)
                if (layout.dims[a] > 1 && layout.operandStride[o][a] != dense[a]) likeOutput[o] = 0;
        }
        auto aligned = [&](int v) {
            for (const KernelOutput& out : r.outputs)
                if (out.alignmentBytes % (static_cast<uint64_t>(v) * dataTypeSizeInBytes(out.storageDType)) != 0) return false;
            return true;  // (operands are read where they lie)
        };
        while (wide > 1 && !aligned(wide)) wide /= 2;
        if (wide > 1) {
            straddling = true;
            vec = wide;
        }
    }
    k.vec = vec;
    k.passNumel = k.flat;

    // 16-bit float arithmetic must round after every operation, so mul+add fusion is only allowed in all-fp32 kernels
    k.fastContract = true;
    BodyEmitter probe(expr);
    for (const KernelOperand& op : r.operands) probe.defineSource(op.node, DataType::FP32);
    for (const GatherOperand& g : r.gathers) probe.defineSource(g.node, DataType::FP32);
    std::vector<uint32_t> roots;
    for (const KernelOutput& out : r.outputs) roots.push_back(out.node);
    for (uint32_t n : probe.collect(roots)) {
        const DataType c = emittedValueDType(expr.nodes[n]);
        if (c == DataType::FP16 || c == DataType::BF16) k.fastContract = false;
    }

    std::ostringstream s;
    s << thor_embed::kDevicePrelude;
    const int threads = 256;  // 128 to 1024 threads per block measure the same on MI355X (C1 at 2^28: 5.95-6.13 TB/s)
    k.threads = static_cast<uint32_t>(threads);
    s << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void fused_kernel(";
    for (size_t o = 0; o < r.operands.size(); ++o) s << "const " << deviceTypeName(r.operands[o].storageDType) << "* in" << o << ", ";
    if (!r.gathers.empty() && !k.flat) throw std::runtime_error("Gathered per-segment operands need a kernel without broadcasting.");
    for (size_t g = 0; g < r.gathers.size(); ++g) {
        s << "const " << deviceTypeName(r.gathers[g].storageDType) << "* g" << g << ", const unsigned int* gid" << g << ", ";
        if (r.gathers[g].normalize) s << "const " << (r.gathers[g].offsetsAre64 ? "unsigned long long" : "unsigned int") << "* goff" << g << ", ";
    }
    if (r.extent.has_value()) s << "const " << (r.extent->offsetsAre64 ? "unsigned long long" : "unsigned int") << "* extentOffsets, ";
    for (uint32_t slot : r.scalarSlots) s << "float s" << slot << ", ";
    for (size_t o = 0; o < r.outputs.size(); ++o) {
        s << deviceTypeName(r.outputs[o].storageDType) << "* out" << o;
        if (o + 1 < r.outputs.size() || k.passNumel) s << ", ";
    }
    if (k.passNumel) s << indexType << (r.extent.has_value() ? " capacity" : " numel");
    s << ") {\n";
    s << "    typedef " << indexType << " index_t;\n";
    if (r.extent.has_value()) {
        // only the rows the partition covers now are computed; the rest of the outputs keeps its contents
        s << "    const unsigned long long active = (unsigned long long)extentOffsets[" << r.extent->batchSize << "ull] * " << r.extent->elementsPerValue
          << "ull;\n";
        if (k.flat) s << "    const index_t numel = active < (unsigned long long)capacity ? (index_t)active : capacity;\n";
    }
    s << "    constexpr int V = " << vec << ";\n";

    // body text for one element; `load(o)` and `store(o, value)` differ between the vector and the scalar form
    uint64_t flops = 0;
    // the element a gathered operand contributes at flat index `index`: the storage word, and the segment it came from
    auto gatherValue = [&](size_t g, const std::string& word, const std::string& segment) {
        const GatherOperand& op = r.gathers[g];
        std::string value = storageToValueExpr(word, op.storageDType);
        if (op.normalize) {
            // fp32 division by the segment's length, rounded once to the storage dtype (through fp16 for e5m2), as the
            // materialised broadcast stores it
            std::string quotient = "(" + castValueExpr(value, op.storageDType, DataType::FP32) + " / thor::toFloat(goff" + std::to_string(g) + "[" + segment +
                                   " + 1] - goff" + std::to_string(g) + "[" + segment + "]))";
            if (op.storageDType == DataType::FP8_E5M2) quotient = "thor::roundF16(" + quotient + ")";
            value = storageToValueExpr(valueToStorageExpr(castValueExpr(quotient, DataType::FP32, op.storageDType), op.storageDType), op.storageDType);
        }
        return value;
    };
    auto emitBody = [&](const std::string& indent, auto loadExpr, auto storeStmt, auto gatherExpr) {
        std::string body;
        BodyEmitter emitter(expr);
        for (size_t g = 0; g < r.gathers.size(); ++g) {
            const GatherOperand& op = r.gathers[g];
            const DataType valueDType = expr.nodes[op.node].output_dtype.value();
            const std::string value = castValueExpr(gatherExpr(g, body, indent), op.storageDType, valueDType);
            body += indent + "const " + valueCType(valueDType) + " t" + std::to_string(op.node) + " = " + value + ";\n";
            emitter.defineSource(op.node, valueDType);
        }
        for (size_t o = 0; o < r.operands.size(); ++o) {
            const KernelOperand& op = r.operands[o];
            const ExprNode& node = expr.nodes[op.node];
            const DataType valueDType = node.output_dtype.value();
            std::string value = storageToValueExpr(loadExpr(o), op.storageDType);
            value = castValueExpr(value, op.storageDType, valueDType);
            body += indent + "const " + valueCType(valueDType) + " t" + std::to_string(op.node) + " = " + value + ";\n";
            emitter.defineSource(op.node, valueDType);
        }
        uint64_t bodyFlops = 0;
        for (uint32_t n : emitter.collect(roots)) bodyFlops += emitter.emit(body, n, indent);
        for (size_t o = 0; o < r.outputs.size(); ++o) {
            const ExprNode& node = expr.nodes[r.outputs[o].node];
            const DataType outDType = node.output_dtype.value();
            if (outDType != r.outputs[o].storageDType) throw std::runtime_error("Fused stage output tensor dtype differs from the node's output dtype.");
            const std::string value = emitter.ref(r.outputs[o].node, outDType);
            body += indent + storeStmt(o, valueToStorageExpr(value, outDType)) + "\n";
        }
        flops = bodyFlops;
        return body;
    };

    // segment of flat element `index` for gather g (clamped: rows outside every segment hold no defined index)
    auto segmentOf = [&](size_t g, const std::string& index) {
        const GatherOperand& op = r.gathers[g];
        const std::string id = "gid" + std::to_string(g) + "[(unsigned long long)(" + index + ") / " + std::to_string(op.elementsPerValue) + "ull]";
        return "((unsigned long long)(" + id + " < " + std::to_string(op.segments) + "u ? " + id + " : " + std::to_string(op.segments - 1) + "u))";
    };
    auto gatherPerElement = [&](const std::string& index) {
        return [&, index](size_t g, std::string& body, const std::string& indent) {
            const std::string seg = "gs" + std::to_string(g);
            body += indent + "const unsigned long long " + seg + " = " + segmentOf(g, index) + ";\n";
            const std::string word = "g" + std::to_string(g) + "[" + seg + " * " + std::to_string(r.gathers[g].elementsPerValue) + "ull + (unsigned long long)(" +
                                     index + ") % " + std::to_string(r.gathers[g].elementsPerValue) + "ull]";
            return gatherValue(g, word, seg);
        };
    };
    auto noGather = [](size_t, std::string&, const std::string&) -> std::string { throw std::logic_error("gather in a broadcast kernel"); };

    if (k.flat) {
        s << "    const index_t base = ((index_t)blockIdx.x * " << threads << "u + threadIdx.x) * V;\n";
        s << "    if (base >= numel) return;\n";
        if (vec > 1) {
            s << "    if (base + V <= numel) {\n";
            // a whole vector lies in one row when the row length is a multiple of the vector: one index read, one vector load
            std::vector<char> hoisted(r.gathers.size(), 0);
            for (size_t g = 0; g < r.gathers.size(); ++g) {
                const GatherOperand& op = r.gathers[g];
                hoisted[g] = op.elementsPerValue % vec == 0 && op.alignmentBytes % (static_cast<uint64_t>(vec) * dataTypeSizeInBytes(op.storageDType)) == 0;
                if (!hoisted[g]) continue;
                s << "        const unsigned long long gs" << g << " = " << segmentOf(g, "base") << ";\n";
                s << "        thor::Pack<" << deviceTypeName(op.storageDType) << ", V> gp" << g << ";\n";
                s << "        gp" << g << ".load(g" << g << " + gs" << g << " * " << op.elementsPerValue << "ull + (unsigned long long)base % " << op.elementsPerValue
                  << "ull);\n";
            }
            auto gatherInVector = [&](size_t g, std::string& body, const std::string& indent) {
                if (hoisted[g]) return gatherValue(g, "gp" + std::to_string(g) + ".v[k]", "gs" + std::to_string(g));
                return gatherPerElement("base + k")(g, body, indent);
            };
            for (size_t o = 0; o < r.operands.size(); ++o) {
                if (single[o]) continue;
                s << "        thor::Pack<" << deviceTypeName(r.operands[o].storageDType) << ", V> p" << o << ";\n";
                s << "        p" << o << vectorLoad(o, vec) << "in" << o << " + base);\n";
            }
            for (size_t o = 0; o < r.outputs.size(); ++o) s << "        thor::Pack<" << deviceTypeName(r.outputs[o].storageDType) << ", V> q" << o << ";\n";
            s << "#pragma unroll\n        for (int k = 0; k < V; ++k) {\n";
            s << emitBody(
                "            ", [&](size_t o) { return single[o] ? "in" + std::to_string(o) + "[0]" : "p" + std::to_string(o) + ".v[k]"; },
                [](size_t o, const std::string& v) { return "q" + std::to_string(o) + ".v[k] = " + v + ";"; }, gatherInVector);
            s << "        }\n";
            for (size_t o = 0; o < r.outputs.size(); ++o) s << "        q" << o << ".storeStream(out" << o << " + base);\n";
            s << "        return;\n    }\n";
        }
        s << "    const index_t end = (base + V < numel) ? base + V : numel;\n";
        s << "    for (index_t e = base; e < end; ++e) {\n";
        s << emitBody(
            "        ", [&](size_t o) { return "in" + std::to_string(o) + (single[o] ? "[0]" : "[e]"); },
            [](size_t o, const std::string& v) { return "out" + std::to_string(o) + "[e] = " + v + ";"; }, gatherPerElement("e"));
        s << "    }\n";
        const uint64_t lanes = (k.numel + vec - 1) / vec;
        k.gridX = static_cast<uint32_t>(std::max<uint64_t>((lanes + threads - 1) / threads, 1));
        k.description = "flat(vec=" + std::to_string(vec) + ")";
    } else if (tiled) {
        // block = one 64 x (64 * VB) tile of the (tile axis, innermost axis) plane at fixed other coordinates; 256 threads = 4 rows
        // of 64; a thread handles VB adjacent innermost elements (4 bytes of the widest type) per row
        const std::vector<uint64_t>& dims = layout.dims;
        const size_t rank = dims.size(), A = static_cast<size_t>(tileAxis), B = rank - 1;
        std::vector<uint64_t> outStride(rank, 1);
        for (size_t a = rank; a-- > 1;) outStride[a - 1] = outStride[a] * dims[a];
        int vb = std::max(1, 4 / static_cast<int>(widest));
        auto vectorFits = [&](int v) {
            if (dims[B] % v != 0) return false;
            for (const KernelOutput& out : r.outputs)
                if (out.alignmentBytes % (static_cast<uint64_t>(v) * dataTypeSizeInBytes(out.storageDType)) != 0) return false;
            for (size_t o = 0; o < r.operands.size(); ++o) {
                const std::vector<uint64_t>& st = layout.operandStride[o];
                if (viaTile[o] || st[B] != 1) continue;
                if (r.operands[o].alignmentBytes % (static_cast<uint64_t>(v) * dataTypeSizeInBytes(r.operands[o].storageDType)) != 0) return false;
                for (size_t a = 0; a < B; ++a)
                    if (st[a] % v != 0) return false;
            }
            return true;
        };
        while (vb > 1 && !vectorFits(vb)) vb /= 2;
        const uint64_t tileB = 64ull * vb;
        const uint64_t tilesA = (dims[A] + 63) / 64, tilesB = (dims[B] + tileB - 1) / tileB;
        uint64_t blocks = tilesA * tilesB;
        s << "    constexpr int PITCH = 65;\n    constexpr int VB = " << vb << ";\n";
        s << "    const unsigned tx = threadIdx.x % 64u, ty = threadIdx.x / 64u;\n";
        s << "    unsigned long long rest = blockIdx.x;\n";
        // tiles are numbered along diagonals: blocks that run together then differ in both coordinates, so neither the
        // reads (rows a pitch apart) nor the writes of a power-of-two matrix queue up on one memory channel
        s << "    const unsigned long long tileB = rest % " << tilesB << "ull;\n    rest /= " << tilesB << "ull;\n";
        s << "    const unsigned long long b0 = tileB * " << tileB << "ull;\n";
        s << "    const unsigned long long a0 = ((rest + tileB) % " << tilesA << "ull) * 64ull;\n    rest /= " << tilesA << "ull;\n";
        for (size_t a = rank; a-- > 0;) {
            if (a == A || a == B) continue;
            s << "    const unsigned long long c" << a << " = rest % " << dims[a] << "ull;\n    rest /= " << dims[a] << "ull;\n";
            blocks *= dims[a];
        }
        auto baseOf = [&](const std::vector<uint64_t>& st) {
            std::string text = "0ull";
            for (size_t a = 0; a < rank; ++a)
                if (a != A && a != B && st[a] != 0) text += " + c" + std::to_string(a) + " * " + std::to_string(st[a]) + "ull";
            return text;
        };
        for (size_t o = 0; o < r.operands.size(); ++o) s << "    const unsigned long long base" << o << " = " << baseOf(layout.operandStride[o]) << ";\n";
        s << "    const unsigned long long outBase = " << baseOf(outStride) << ";\n";
        for (size_t o = 0; o < r.operands.size(); ++o) {
            if (!viaTile[o]) continue;
            const char* type = deviceTypeName(r.operands[o].storageDType);
            s << "    __shared__ " << type << " tile" << o << "[64 * VB * PITCH];\n";
            s << "#pragma unroll\n    for (int i = 0; i < 16 * VB; ++i) {\n";
            s << "        const unsigned long long a = a0 + tx, b = b0 + ty + 4u * i;\n";
            s << "        if (a < " << dims[A] << "ull && b < " << dims[B] << "ull) tile" << o << "[(ty + 4u * i) * PITCH + tx] = in" << o << "[base" << o
              << " + a + b * " << layout.operandStride[o][B] << "ull];\n    }\n";
        }
        s << "    __syncthreads();\n";
        s << "#pragma unroll 4\n    for (int i = 0; i < 16; ++i) {\n";
        s << "        const unsigned long long a = a0 + ty + 4u * i, b = b0 + tx * VB;\n";
        s << "        if (a >= " << dims[A] << "ull || b >= " << dims[B] << "ull) continue;\n";
        for (size_t o = 0; o < r.operands.size(); ++o) {
            if (viaTile[o]) continue;
            const std::vector<uint64_t>& st = layout.operandStride[o];
            const char* type = deviceTypeName(r.operands[o].storageDType);
            const std::string address = "in" + std::to_string(o) + " + base" + std::to_string(o) + " + a * " + std::to_string(st[A]) + "ull + b * " +
                                        std::to_string(st[B]) + "ull";
            if (st[B] == 1) {
                s << "        thor::Pack<" << type << ", VB> p" << o << ";\n        p" << o << ".loadStream(" << address << ");\n";
            } else if (st[B] == 0) {
                s << "        const " << type << " b" << o << " = *(" << address << ");\n";
            }
        }
        for (size_t o = 0; o < r.outputs.size(); ++o) s << "        thor::Pack<" << deviceTypeName(r.outputs[o].storageDType) << ", VB> q" << o << ";\n";
        s << "#pragma unroll\n        for (int k = 0; k < VB; ++k) {\n";
        s << emitBody(
            "            ",
            [&](size_t o) {
                const std::vector<uint64_t>& st = layout.operandStride[o];
                if (viaTile[o]) return "tile" + std::to_string(o) + "[(tx * VB + k) * PITCH + ty + 4u * i]";
                if (st[B] == 1) return "p" + std::to_string(o) + ".v[k]";
                if (st[B] == 0) return "b" + std::to_string(o);
                return "in" + std::to_string(o) + "[base" + std::to_string(o) + " + a * " + std::to_string(st[A]) + "ull + (b + k) * " + std::to_string(st[B]) + "ull]";
            },
            [](size_t o, const std::string& v) { return "q" + std::to_string(o) + ".v[k] = " + v + ";"; }, noGather);
        s << "        }\n";
        for (size_t o = 0; o < r.outputs.size(); ++o)
            s << "        q" << o << ".storeStream(out" << o << " + outBase + a * " << outStride[A] << "ull + b);\n";
        s << "    }\n";
        if (blocks >= (1ull << 31)) throw std::runtime_error("Tiled fused kernel would need more blocks than a grid holds.");
        k.gridX = static_cast<uint32_t>(blocks);
        k.vec = vb;
        k.description = "tiled(axis=" + std::to_string(tileAxis) + "/" + std::to_string(rank) + ",tile=64x" + std::to_string(tileB) + ")";
    } else if (straddling) {
        const std::vector<uint64_t>& dims = layout.dims;
        const size_t rank = dims.size();
        s << "    const index_t base = ((index_t)blockIdx.x * " << threads << "u + threadIdx.x) * V;\n";
        s << "    if (base >= " << k.numel << "ull) return;\n";
        // coordinates of element `base`; element base + k is reached by adding one k times, with carries
        s << "    index_t rest = base;\n";
        for (size_t a = rank; a-- > 0;) {
            if (a == 0) {
                s << "    index_t c0 = rest;\n";
            } else {
                s << "    index_t c" << a << " = rest % " << dims[a] << "u;\n    rest /= " << dims[a] << "u;\n";
            }
        }
        auto offsetOf = [&](size_t o) {
            std::string text = "0ull";
            for (size_t a = 0; a < rank; ++a)
                if (layout.operandStride[o][a] != 0 && dims[a] > 1) text += " + (unsigned long long)c" + std::to_string(a) + " * " + std::to_string(layout.operandStride[o][a]) + "ull";
            return text;
        };
        std::string advance = "        ++c" + std::to_string(rank - 1) + ";\n";
        for (size_t a = rank; a-- > 1;)
            advance += "        if (c" + std::to_string(a) + " == " + std::to_string(dims[a]) + "u) { c" + std::to_string(a) + " = 0; ++c" + std::to_string(a - 1) + "; }\n";
        s << "    if (base + V <= " << k.numel << "ull) {\n";
        for (size_t o = 0; o < r.operands.size(); ++o) {
            if (!likeOutput[o]) continue;
            s << "        thor::Pack<" << deviceTypeName(r.operands[o].storageDType) << ", V> p" << o << ";\n        p" << o << vectorLoad(o, vec) << "in" << o << " + base);\n";
        }
        // broadcast operands that are contiguous along the innermost axis: one vector when the lane's elements stay inside
        // a row of theirs, element by element (at the carried coordinates) in the lanes whose vector wraps
        std::vector<char> rowVector(r.operands.size(), 0);
        for (size_t o = 0; o < r.operands.size(); ++o) {
            if (single[o] || likeOutput[o] || layout.operandStride[o][rank - 1] != 1 || dims[rank - 1] < static_cast<uint64_t>(vec)) continue;
            rowVector[o] = 1;
            s << "        const bool inRow" << o << " = c" << (rank - 1) << " + V <= " << dims[rank - 1] << "u;\n";
            s << "        thor::Pack<" << deviceTypeName(r.operands[o].storageDType) << ", V> pb" << o << ";\n";
            s << "        if (inRow" << o << ") pb" << o << ".loadUnaligned(in" << o << " + " << offsetOf(o) << ");\n";
        }
        for (size_t o = 0; o < r.outputs.size(); ++o) s << "        thor::Pack<" << deviceTypeName(r.outputs[o].storageDType) << ", V> q" << o << ";\n";
        s << "#pragma unroll\n        for (int k = 0; k < V; ++k) {\n";
        s << emitBody(
            "            ",
            [&](size_t o) {
                if (single[o]) return "in" + std::to_string(o) + "[0]";
                if (likeOutput[o]) return "p" + std::to_string(o) + ".v[k]";
                if (rowVector[o]) return "(inRow" + std::to_string(o) + " ? pb" + std::to_string(o) + ".v[k] : in" + std::to_string(o) + "[" + offsetOf(o) + "])";
                return "in" + std::to_string(o) + "[" + offsetOf(o) + "]";
            },
            [](size_t o, const std::string& v) { return "q" + std::to_string(o) + ".v[k] = " + v + ";"; }, noGather);
        s << advance;
        s << "        }\n";
        for (size_t o = 0; o < r.outputs.size(); ++o) s << "        q" << o << ".storeStream(out" << o << " + base);\n";
        s << "        return;\n    }\n";
        s << "    for (index_t e = base; e < " << k.numel << "ull; ++e) {\n";
        s << emitBody(
            "        ",
            [&](size_t o) {
                if (single[o]) return "in" + std::to_string(o) + "[0]";
                if (likeOutput[o]) return "in" + std::to_string(o) + "[e]";
                return "in" + std::to_string(o) + "[" + offsetOf(o) + "]";
            },
            [](size_t o, const std::string& v) { return "out" + std::to_string(o) + "[e] = " + v + ";"; }, noGather);
        s << advance;
        s << "    }\n";
        const uint64_t lanes = (k.numel + vec - 1) / vec;
        k.gridX = static_cast<uint32_t>(std::max<uint64_t>((lanes + threads - 1) / threads, 1));
        k.description = "broadcast(axes=" + std::to_string(rank) + ",vec=" + std::to_string(vec) + ",vectors_straddle_rows)";
    } else {
        std::vector<uint64_t> dims = layout.dims;
        dims.back() /= vec;  // the innermost axis is walked in vectors
        uint64_t lanes = 1;
        for (uint64_t d : dims) lanes *= d;
        s << "    const index_t lane = (index_t)blockIdx.x * " << threads << "u + threadIdx.x;\n";
        s << "    if (lane >= " << lanes << "ull) return;\n";
        if (r.extent.has_value()) s << "    if ((unsigned long long)lane * V >= active) return;\n";
        s << "    index_t rest = lane;\n";
        for (size_t a = dims.size(); a-- > 0;) {
            if (a == 0) {
                s << "    const index_t c0 = rest;\n";
            } else {
                s << "    const index_t c" << a << " = rest % " << dims[a] << "u;\n    rest /= " << dims[a] << "u;\n";
            }
        }
        for (size_t o = 0; o < r.operands.size(); ++o) {
            const std::vector<uint64_t>& st = layout.operandStride[o];
            s << "    const unsigned long long off" << o << " = 0ull";
            for (size_t a = 0; a < st.size(); ++a) {
                if (st[a] == 0) continue;
                const uint64_t step = (a + 1 == st.size()) ? st[a] * vec : st[a];
                s << " + (unsigned long long)c" << a << " * " << step << "ull";
            }
            s << ";\n";
        }
        s << "    const unsigned long long outOff = (unsigned long long)lane * V;\n";
        for (size_t o = 0; o < r.operands.size(); ++o) {
            const bool contiguous = layout.operandStride[o].back() == 1;
            const char* type = deviceTypeName(r.operands[o].storageDType);
            if (contiguous && vec > 1) {
                s << "    thor::Pack<" << type << ", V> p" << o << ";\n    p" << o << vectorLoad(o, vec) << "in" << o << " + off" << o << ");\n";
            } else {
                s << "    const " << type << " b" << o << " = in" << o << "[off" << o << "];\n";
            }
        }
        for (size_t o = 0; o < r.outputs.size(); ++o) s << "    thor::Pack<" << deviceTypeName(r.outputs[o].storageDType) << ", V> q" << o << ";\n";
        s << "#pragma unroll\n    for (int k = 0; k < V; ++k) {\n";
        s << emitBody(
            "        ",
            [&](size_t o) {
                const bool contiguous = layout.operandStride[o].back() == 1;
                return (contiguous && vec > 1) ? "p" + std::to_string(o) + ".v[k]" : "b" + std::to_string(o);
            },
            [](size_t o, const std::string& v) { return "q" + std::to_string(o) + ".v[k] = " + v + ";"; }, noGather);
        s << "    }\n";
        for (size_t o = 0; o < r.outputs.size(); ++o) s << "    q" << o << ".storeStream(out" << o << " + outOff);\n";
        k.gridX = static_cast<uint32_t>(std::max<uint64_t>((lanes + threads - 1) / threads, 1));
        k.description = "broadcast(axes=" + std::to_string(dims.size()) + ",vec=" + std::to_string(vec) + ")";
    }
    s << "}\n";
    k.source = s.str();
    k.flopsPerElement = flops;
    return k;
}

}  // namespace ThorImplementation
