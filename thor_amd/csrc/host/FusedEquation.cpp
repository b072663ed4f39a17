// Planning and stamping of compiled expressions: dtype resolution, de-duplication, the split into stages at reduction
// boundaries, shape inference, output allocation and kernel generation per stage
// (reference behaviour: Utilities/Expression/EquationCompiler.cpp:6572-7879 planExecution,
//  Utilities/Expression/FusedEquation.cpp:666-710 broadcasting, :6828-6887 per-dtype compilation, :8885-9353 stamp,
//  :10760-10905 convenience run).
#include "Utilities/Expression/FusedEquation.h"

#include "AutoDiffInternal.h"
#include "CubScanInternal.h"
#include "HipSourceEmitter.h"
#include "IndexGather.h"
#include "RotaryEmbedding.h"
#include "ScatterAdd.h"
#include "ReductionPlanner.h"
#include "RowFusion.h"
#include "ShapeInference.h"
#include "WinnerRouting.h"
#include "Utilities/Common/ScopedGpu.h"
#include "Utilities/Expression/ExpressionDTypeResolution.h"

#include <algorithm>
#include <cstdlib>
#include <functional>
#include <limits>
#include <map>
#include <numeric>
#include <sstream>
#include <stdexcept>

namespace ThorImplementation {

struct PlannedGraph {
    // Gather: a SEGMENTED_BROADCAST that only fused kernels consume: they read the per-segment tensor through a
    // row -> segment index instead of a materialised [rows, E] copy
    enum class Role : uint8_t { Inline, InputSource, Materialized, View, Gather };
    PhysicalExpression expr;  // dtype-resolved, de-duplicated, reachable nodes only
    std::vector<NamedOutput> outputs;
    std::vector<Role> role;
    std::vector<uint32_t> level;  // Materialized nodes: position in the dependency order
};

namespace {

using Role = PlannedGraph::Role;

bool isShapeOnly(ExprOp op) { return op == ExprOp::RESHAPE || op == ExprOp::UNSQUEEZE || op == ExprOp::SQUEEZE || isStorageViewOp(op); }
bool isReductionStorage(DataType d) {
    return d == DataType::FP8_E4M3 || d == DataType::FP8_E5M2 || d == DataType::FP16 || d == DataType::BF16 || d == DataType::FP32;
}

std::string axesKey(const std::vector<uint64_t>& v) {
    std::string s;
    for (uint64_t a : v) s += std::to_string(a) + ",";
    return s;
}

std::string structuralKey(const ExprNode& n) {
    std::ostringstream k;
    k << static_cast<int>(n.op) << "|" << n.lhs << "|" << n.rhs << "|" << n.aux << "|" << n.input_slot << "|" << formatFloatCanonical(n.scalar_fp)
      << "|" << (n.input_tensor_dtype ? static_cast<int>(*n.input_tensor_dtype) : -1) << "|" << (n.output_dtype ? static_cast<int>(*n.output_dtype) : -1)
      << "|" << (n.compute_dtype ? static_cast<int>(*n.compute_dtype) : -1) << "|" << axesKey(n.reduction_axes) << "|" << axesKey(n.squeeze_axes)
      << "|" << axesKey(n.unsqueeze_axes) << "|" << axesKey(n.reshape_dims) << "|" << axesKey(n.fill_dims) << "|" << n.ragged_runtime_batch_size << "|"
      << n.ragged_runtime_max_active_values << "|" << n.ragged_runtime_elements_per_value << "|" << n.segmented_broadcast_normalize_by_length << "|"
      << axesKey(n.view_dims) << "|" << axesKey(n.view_strides) << "|" << n.view_element_offset << "|" << static_cast<int>(n.scan_op) << "|"
      << static_cast<int>(n.scan_mode) << "|" << n.scan_axis << "|" << n.scan_reverse;
    if (n.op == ExprOp::ROPE) k << "|" << ropeKey(n);
    return k.str();
}

// Rebuilds the reachable part of a resolved graph without duplicate nodes and with explicit CAST nodes wherever a
// tensor consumer (reduction, shape op, named output) needs an input in a dtype its bound tensor does not have.
class GraphBuilder {
   public:
    explicit GraphBuilder(const PhysicalExpression& src) : src(src) { out.inputs = src.inputs; }

    uint32_t add(ExprNode node) {
        if (isCommutative(node.op) && node.rhs != UINT32_MAX && node.rhs < node.lhs) std::swap(node.lhs, node.rhs);
        const std::string key = structuralKey(node);
        auto it = byKey.find(key);
        if (it != byKey.end()) return it->second;
        const uint32_t idx = static_cast<uint32_t>(out.nodes.size());
        out.nodes.push_back(std::move(node));
        byKey.emplace(key, idx);
        return idx;
    }

    uint32_t castOf(uint32_t child, DataType dtype) {
        ExprNode cast;
        cast.op = ExprOp::CAST;
        cast.lhs = child;
        cast.output_dtype = dtype;
        cast.compute_dtype = dtype;
        return add(cast);
    }

    // index (in the new graph) of a node that can stand for `child` as a tensor of its value dtype
    uint32_t asTensorOperand(uint32_t child, bool forReduction) {
        const ExprNode& c = out.nodes[child];
        DataType valueDType = c.output_dtype.value();
        if (forReduction && !isReductionStorage(valueDType)) return castOf(child, DataType::FP32);
        if (c.op == ExprOp::INPUT && c.input_tensor_dtype.value() != valueDType) return castOf(child, valueDType);
        return child;
    }

    // softmax(x) = exp(x - max) / sum(exp(x - max)) over the channel axis (or every axis but the first), in fp32, converted
    // once to the node's output dtype; Fast skips the max, Log returns (x - max) - ln(sum).  `node.lhs` is already translated.
    uint32_t lowerSoftmax(const ExprNode& node) {
        const uint32_t x = asTensorOperand(node.lhs, true);
        const std::vector<uint64_t> axes = node.softmax_mode == SoftmaxMode::Channel ? std::vector<uint64_t>{1} : std::vector<uint64_t>{kReduceAllAxesButFirst};
        auto make = [&](ExprOp op, uint32_t lhs, uint32_t rhs = UINT32_MAX) {
            ExprNode n;
            n.op = op;
            n.lhs = lhs;
            n.rhs = rhs;
            n.compute_dtype = DataType::FP32;
            n.output_dtype = DataType::FP32;
            if (isReductionOp(op)) n.reduction_axes = axes;
            return add(n);
        };
        uint32_t shifted = x;
        if (node.softmax_algorithm != SoftmaxAlgorithm::Fast) shifted = make(ExprOp::SUB, x, make(ExprOp::REDUCE_MAX, x));
        const uint32_t e = make(ExprOp::EXP, shifted);
        const uint32_t sum = make(ExprOp::REDUCE_SUM, e);
        const uint32_t result = node.softmax_algorithm == SoftmaxAlgorithm::Log ? make(ExprOp::SUB, shifted, make(ExprOp::LN, sum)) : make(ExprOp::DIV, e, sum);
        const DataType outDType = node.output_dtype.value();
        return outDType == DataType::FP32 ? result : castOf(result, outDType);
    }

    uint32_t translate(uint32_t srcIndex) {
        auto it = remap.find(srcIndex);
        if (it != remap.end()) return it->second;
        ExprNode node = src.nodes.at(srcIndex);
        // a scalar in device memory is bound as a one-element tensor: from here on an input like any other
        if (node.op == ExprOp::TENSOR_RUNTIME_SCALAR) node.op = ExprOp::INPUT;
        if (node.lhs != UINT32_MAX) node.lhs = translate(node.lhs);
        if (node.rhs != UINT32_MAX) node.rhs = translate(node.rhs);
        if (node.aux != UINT32_MAX) node.aux = translate(node.aux);
        if (node.op == ExprOp::SOFTMAX) {
            const uint32_t idx = lowerSoftmax(node);
            remap.emplace(srcIndex, idx);
            return idx;
        }
        if (node.op == ExprOp::CAST) {
            // a conversion of a computed value to the dtype it already has is that value (inputs and views keep theirs: it
            // is what copies them into a tensor of their own)
            const ExprNode& child = out.nodes[node.lhs];
            if (!Expression::isLeafOp(child.op) && !isShapeOnly(child.op) && child.output_dtype == node.output_dtype) {
                remap.emplace(srcIndex, node.lhs);
                return node.lhs;
            }
        }
        if (isReductionOp(node.op) || isSegmentedReduceOp(node.op)) {
            node.lhs = asTensorOperand(node.lhs, true);
        } else if (isWinnerRoutingOp(node.op)) {
            node.lhs = asTensorOperand(node.lhs, true);  // read by an arg reduction
            node.rhs = asTensorOperand(node.rhs, false);
        } else if (isScanOp(node.op)) {
            // the scan kernels stream dense storage
            node.lhs = asTensorOperand(node.lhs, false);
            if (isStorageViewOp(out.nodes[node.lhs].op)) node.lhs = castOf(node.lhs, out.nodes[node.lhs].output_dtype.value());
            if (node.op == ExprOp::SEGMENTED_SCAN) node.rhs = asTensorOperand(node.rhs, false);
        } else if (node.op == ExprOp::ROPE || isScatterRoutingOp(node.op)) {
            // the rotation kernel addresses dense storage; position ids and the effective length are small tensors it reads
            for (uint32_t* operand : {&node.lhs, &node.rhs, &node.aux}) {
                if (*operand == UINT32_MAX) continue;
                // a conversion of a bound tensor to the dtype it already has would only copy it: these kernels read the tensor itself
                const ExprNode& asked = out.nodes[*operand];
                if (asked.op == ExprOp::CAST && out.nodes[asked.lhs].op == ExprOp::INPUT && out.nodes[asked.lhs].output_dtype == asked.output_dtype &&
                    out.nodes[asked.lhs].input_tensor_dtype == asked.output_dtype) {
                    *operand = asked.lhs;
                }
                *operand = asTensorOperand(*operand, false);
                if (isStorageViewOp(out.nodes[*operand].op)) *operand = castOf(*operand, out.nodes[*operand].output_dtype.value());
            }
        } else if (node.op == ExprOp::TAKE_ALONG_AXIS) {
            node.lhs = asTensorOperand(node.lhs, false);
            node.rhs = asTensorOperand(node.rhs, false);
            // the gather addresses dense storage: a strided view is copied into a dense tensor first
            if (isStorageViewOp(out.nodes[node.lhs].op)) node.lhs = castOf(node.lhs, out.nodes[node.lhs].output_dtype.value());
            if (isStorageViewOp(out.nodes[node.rhs].op)) node.rhs = castOf(node.rhs, out.nodes[node.rhs].output_dtype.value());
        } else if (node.op == ExprOp::SEGMENTED_BROADCAST) {
            node.lhs = asTensorOperand(node.lhs, false);
        } else if (isShapeOnly(node.op)) {
            double folded;
            if (!tryFoldConstant(out, node.lhs, folded)) node.lhs = asTensorOperand(node.lhs, false);
        }
        if ((isSegmentedReduceOp(node.op) || node.op == ExprOp::SEGMENTED_BROADCAST) && isStorageViewOp(out.nodes[node.lhs].op)) {
            // the segment kernels stream dense rows: a strided view is gathered into a dense tensor first (an identity kernel)
            node.lhs = castOf(node.lhs, out.nodes[node.lhs].output_dtype.value());
        }
        const uint32_t idx = add(std::move(node));
        remap.emplace(srcIndex, idx);
        return idx;
    }

    const PhysicalExpression& src;
    PhysicalExpression out;
    std::unordered_map<std::string, uint32_t> byKey;
    std::unordered_map<uint32_t, uint32_t> remap;
};

bool isTensorRole(Role r) { return r != Role::Inline; }

// Tensor sources (inputs, materialised values, views) that the value of `root` is computed from without crossing
// another materialised value.
void collectSources(const PlannedGraph& g, uint32_t root, std::vector<uint32_t>& sources, std::vector<uint32_t>& scalarSlots) {
    std::vector<char> seen(g.expr.nodes.size(), 0);
    std::vector<uint32_t> stack;
    const ExprNode& r = g.expr.nodes[root];
    // the offsets under a runtime-extent marker are the kernel's extent, not one of its value sources
    auto valueChildren = [](const ExprNode& n) {
        return n.op == ExprOp::RAGGED_VALUEWISE_EXTENT ? std::vector<uint32_t>{n.lhs} : std::vector<uint32_t>{n.lhs, n.rhs, n.aux};
    };
    for (uint32_t c : valueChildren(r))
        if (c != UINT32_MAX) stack.push_back(c);
    if (r.op == ExprOp::RUNTIME_SCALAR) scalarSlots.push_back(r.input_slot);
    while (!stack.empty()) {
        const uint32_t n = stack.back();
        stack.pop_back();
        if (seen[n]) continue;
        seen[n] = 1;
        if (isTensorRole(g.role[n])) {
            sources.push_back(n);
            continue;
        }
        const ExprNode& node = g.expr.nodes[n];
        if (node.op == ExprOp::RUNTIME_SCALAR) scalarSlots.push_back(node.input_slot);
        for (uint32_t c : valueChildren(node))
            if (c != UINT32_MAX) stack.push_back(c);
    }
    std::sort(sources.begin(), sources.end());
    sources.erase(std::unique(sources.begin(), sources.end()), sources.end());
    std::sort(scalarSlots.begin(), scalarSlots.end());
    scalarSlots.erase(std::unique(scalarSlots.begin(), scalarSlots.end()), scalarSlots.end());
}

uint32_t baseOfView(const PlannedGraph& g, uint32_t node) {
    // the tensor a source stands on: views and gathers lead to the tensor they read
    while (g.role[node] == Role::View || g.role[node] == Role::Gather) node = g.expr.nodes[node].lhs;
    return node;
}

// Can the consumer read a per-segment value through the segment index?  Only work that ends up inside a flat fused kernel.
bool consumesGather(const ExprNode& consumer) {
    if (consumer.op == ExprOp::RAGGED_VALUEWISE_EXTENT || consumer.op == ExprOp::WHERE || consumer.op == ExprOp::CAST) return true;
    if (isReductionOp(consumer.op) || isRaggedOp(consumer.op) || isShapeOnly(consumer.op) || consumer.op == ExprOp::SOFTMAX || isWinnerRoutingOp(consumer.op) ||
        consumer.op == ExprOp::TAKE_ALONG_AXIS || consumer.op == ExprOp::ROPE || isScatterRoutingOp(consumer.op) || isScanOp(consumer.op)) {
        return false;
    }
    return Expression::isBinaryOp(consumer.op) || Expression::isUnaryOp(consumer.op);
}

std::vector<uint64_t> broadcastDims(const std::vector<uint64_t>& a, const std::vector<uint64_t>& b) {
    const size_t rank = std::max(a.size(), b.size());
    std::vector<uint64_t> out(rank, 1);
    for (size_t i = 0; i < rank; ++i) {
        const uint64_t da = i < rank - a.size() ? 1 : a[i - (rank - a.size())];
        const uint64_t db = i < rank - b.size() ? 1 : b[i - (rank - b.size())];
        if (da != db && da != 1 && db != 1) {
            throw std::runtime_error("Expression operands are not broadcast-compatible.");
        }
        out[i] = std::max(da, db);
    }
    return out;
}

std::vector<uint64_t> reshapeDims(const std::vector<uint64_t>& in, const std::vector<uint64_t>& requested) {
    uint64_t total = 1, known = 1;
    for (uint64_t d : in) total *= d;
    std::vector<uint64_t> out = requested;
    int infer = -1;
    for (size_t i = 0; i < out.size(); ++i) {
        if (out[i] == std::numeric_limits<uint64_t>::max()) {
            infer = static_cast<int>(i);
        } else {
            known *= out[i];
        }
    }
    if (infer >= 0) {
        if (known == 0 || total % known != 0) throw std::runtime_error("Expression::reshape cannot infer the marked dimension.");
        out[infer] = total / known;
        known *= out[infer];
    }
    if (known != total) throw std::runtime_error("Expression::reshape changes the number of elements.");
    return out;
}

std::vector<uint64_t> sortedAxesOrAll(const std::vector<uint64_t>& axes, size_t rank) { return resolveReductionAxes(axes, rank); }

}  // namespace

std::vector<std::vector<uint64_t>> inferExpressionShapes(const PhysicalExpression& expr,
                                                           const std::function<std::vector<uint64_t>(uint32_t)>& inputDims) {
    std::vector<std::vector<uint64_t>> dims(expr.nodes.size());
    for (uint32_t i = 0; i < expr.nodes.size(); ++i) {
        const ExprNode& n = expr.nodes[i];
        switch (n.op) {
            case ExprOp::INPUT:
            case ExprOp::TENSOR_RUNTIME_SCALAR:  // bound as a one-element tensor
                dims[i] = inputDims(n.input_slot);
                break;
            case ExprOp::RUNTIME_SCALAR:
            case ExprOp::SCALAR_FP:
                dims[i] = {};
                break;
            case ExprOp::FILL:
                dims[i] = n.fill_dims;
                break;
            case ExprOp::RESHAPE:
                dims[i] = reshapeDims(dims[n.lhs], n.reshape_dims);
                break;
            case ExprOp::UNSQUEEZE: {
                const size_t rank = dims[n.lhs].size() + n.unsqueeze_axes.size();
                std::vector<uint64_t> out;
                size_t src = 0;
                for (size_t a = 0; a < rank; ++a) {
                    if (std::binary_search(n.unsqueeze_axes.begin(), n.unsqueeze_axes.end(), a)) {
                        out.push_back(1);
                    } else {
                        if (src >= dims[n.lhs].size()) throw std::runtime_error("unsqueeze axes are invalid for the input rank.");
                        out.push_back(dims[n.lhs][src++]);
                    }
                }
                for (uint64_t a : n.unsqueeze_axes)
                    if (a >= rank) throw std::runtime_error("unsqueeze axes are invalid for the input rank.");
                dims[i] = out;
                break;
            }
            case ExprOp::STRIDED_VIEW:
                dims[i] = n.view_dims;
                break;
            case ExprOp::TRANSPOSE:
                if (dims[n.lhs].size() < 2) throw std::runtime_error("Expression::transpose requires a tensor of rank 2 or more.");
                dims[i] = dims[n.lhs];
                std::swap(dims[i][dims[i].size() - 1], dims[i][dims[i].size() - 2]);
                break;
            case ExprOp::SQUEEZE:
                dims[i] = StampedEquation::computeReductionOutputDims(dims[n.lhs], {}, n.squeeze_axes.empty() ? std::vector<uint64_t>{UINT64_MAX} : n.squeeze_axes);
                break;
            case ExprOp::RAGGED_VALUEWISE_EXTENT:
                dims[i] = dims[n.lhs];
                break;
            case ExprOp::SEGMENTED_REDUCE_SUM:
            case ExprOp::SEGMENTED_REDUCE_MIN:
            case ExprOp::SEGMENTED_REDUCE_MAX:
            case ExprOp::SEGMENTED_REDUCE_MEAN: {
                // values [N, D...] and offsets [B + 1] -> [B, D...]
                if (dims[n.lhs].empty() || dims[n.rhs].size() != 1 || dims[n.rhs][0] < 2) {
                    throw std::runtime_error("Segmented reduction requires values [N, D...] and offsets [B + 1] with at least one segment.");
                }
                if (n.ragged_runtime_batch_size != 0 && dims[n.rhs][0] != n.ragged_runtime_batch_size + 1) {
                    throw std::runtime_error("Segmented reduction offsets do not have the ragged descriptor's batch size + 1 entries.");
                }
                dims[i] = dims[n.lhs];
                dims[i][0] = dims[n.rhs][0] - 1;
                break;
            }
            case ExprOp::SEGMENTED_BROADCAST: {
                // per-segment values [B, D...] -> rows [capacity, D...]
                if (dims[n.lhs].empty() || dims[n.rhs].size() != 1 || dims[n.rhs][0] != dims[n.lhs][0] + 1) {
                    throw std::runtime_error("Segmented broadcast requires per-segment values [B, D...] and offsets [B + 1].");
                }
                if (n.ragged_runtime_max_active_values == 0) throw std::runtime_error("Segmented broadcast is missing its row capacity.");
                dims[i] = dims[n.lhs];
                dims[i][0] = n.ragged_runtime_max_active_values;
                break;
            }
            case ExprOp::SCAN:
                if (dims[n.lhs].empty()) throw std::runtime_error("Expression::scan requires a tensor of rank 1 or more.");
                if (n.scan_axis != UINT64_MAX && n.scan_axis != dims[n.lhs].size() - 1) {
                    throw std::runtime_error("Expression::scan currently supports only axis=-1 or an explicit non-negative final axis.");
                }
                dims[i] = dims[n.lhs];
                break;
            case ExprOp::SEGMENTED_SCAN: {
                uint64_t elements = 1;
                for (uint64_t d : dims[n.lhs]) elements *= d;
                if (dims[n.lhs].empty() || elements != dims[n.lhs][0] || dims[n.rhs].size() != 1 || dims[n.rhs][0] < 2) {
                    throw std::runtime_error("Segmented scan requires values [N] (one element per row) and offsets [B + 1] with at least one segment.");
                }
                if (n.ragged_runtime_batch_size != 0 && dims[n.rhs][0] != n.ragged_runtime_batch_size + 1) {
                    throw std::runtime_error("Segmented scan offsets do not have the ragged descriptor's batch size + 1 entries.");
                }
                dims[i] = dims[n.lhs];
                break;
            }
            case ExprOp::STRIDED_VIEW_BACKWARD:
                if (dims[n.lhs] != n.view_dims) throw std::runtime_error("Strided view backward requires a gradient shaped like the view.");
                dims[i] = n.fill_dims;
                break;
            case ExprOp::SEGMENTED_REDUCE_MIN_BACKWARD:
            case ExprOp::SEGMENTED_REDUCE_MAX_BACKWARD: {
                const std::vector<uint64_t>& values = dims[n.lhs];
                if (n.aux == UINT32_MAX || values.empty() || dims[n.aux].size() != 1 || dims[n.aux][0] < 2) {
                    throw std::runtime_error("Segmented ragged min/max backward requires values [N,D...], output [B,D...], and offsets [B+1].");
                }
                std::vector<uint64_t> segments = values;
                segments[0] = dims[n.aux][0] - 1;
                if (dims[n.rhs] != segments) throw std::runtime_error("Segmented ragged min/max backward requires values [N,D...], output [B,D...], and offsets [B+1].");
                dims[i] = values;
                break;
            }
            case ExprOp::SCAN_MIN_BACKWARD:
            case ExprOp::SCAN_MAX_BACKWARD:
            case ExprOp::SEGMENTED_SCAN_MIN_BACKWARD:
            case ExprOp::SEGMENTED_SCAN_MAX_BACKWARD: {
                if (dims[n.rhs] != dims[n.lhs]) throw std::runtime_error("Scan min/max backward requires a gradient shaped like the scanned operand.");
                const bool segmented = n.op == ExprOp::SEGMENTED_SCAN_MIN_BACKWARD || n.op == ExprOp::SEGMENTED_SCAN_MAX_BACKWARD;
                if (segmented != (n.aux != UINT32_MAX)) throw std::runtime_error("Scan min/max backward: offsets go with segmented scans only.");
                if (!segmented && n.scan_axis != UINT64_MAX && n.scan_axis != dims[n.lhs].size() - 1) {
                    throw std::runtime_error("Expression::scan currently supports only the last axis.");
                }
                dims[i] = dims[n.lhs];
                break;
            }
            case ExprOp::ROPE: {
                const std::vector<uint64_t>& in = dims[n.lhs];
                if (n.rope_sequence_axis >= in.size() || n.rope_head_dim_axis >= in.size() || n.rope_sequence_axis == n.rope_head_dim_axis) {
                    throw std::runtime_error("RoPE sequence and head-dimension axes must be distinct axes of the input.");
                }
                const uint64_t headDim = in[n.rope_head_dim_axis];
                const uint64_t rotary = n.rope_rotary_dim == 0 ? headDim : n.rope_rotary_dim;
                if (rotary == 0 || rotary > headDim || (rotary & 1ull) != 0) {
                    throw std::runtime_error("RoPE rotary_dim must be even and no larger than the head dimension.");
                }
                if (n.rope_scaling_kind == RotaryScalingKind::LongRope && n.rope_long_rope_short_factors.size() != rotary / 2) {
                    throw std::runtime_error("LongRoPE scaling requires short/long factor lists of length rotary_dim / 2.");
                }
                auto elements = [&](uint32_t node) {
                    uint64_t e = 1;
                    for (uint64_t d : dims[node]) e *= d;
                    return e;
                };
                if (n.rhs != UINT32_MAX && elements(n.rhs) != in[n.rope_sequence_axis]) {
                    throw std::runtime_error("RoPE position ids must hold one position per element of the sequence axis.");
                }
                if (n.aux != UINT32_MAX && elements(n.aux) != 1) throw std::runtime_error("RoPE effective sequence length must be a single element.");
                dims[i] = in;
                break;
            }
            case ExprOp::TAKE_ALONG_AXIS:
                if (dims[n.lhs].empty() || dims[n.rhs].empty()) throw std::runtime_error("take_along_axis requires non-scalar input and indices tensors.");
                if (dims[n.lhs].size() != dims[n.rhs].size()) throw std::runtime_error("take_along_axis input and indices must have the same rank.");
                dims[i] = dims[n.rhs];
                break;
            case ExprOp::REDUCE_MIN_BACKWARD:
            case ExprOp::REDUCE_MAX_BACKWARD: {
                // operand-shaped; the gradient holds one element per reduction window
                const std::vector<uint64_t> windows = StampedEquation::computeReductionOutputDims(
                    dims[n.lhs], sortedAxesOrAll(n.reduction_axes, dims[n.lhs].size()), n.squeeze_axes);
                uint64_t expected = 1, got = 1;
                for (uint64_t d : windows) expected *= d;
                for (uint64_t d : dims[n.rhs]) got *= d;
                if (expected != got) throw std::runtime_error("Min/max reduction backward: the gradient does not have the reduction's output shape.");
                dims[i] = dims[n.lhs];
                break;
            }
            default:
                if (isReductionOp(n.op)) {
                    const std::vector<uint64_t> axes = sortedAxesOrAll(n.reduction_axes, dims[n.lhs].size());
                    dims[i] = StampedEquation::computeReductionOutputDims(dims[n.lhs], axes, n.squeeze_axes);
                } else if (n.op == ExprOp::WHERE) {
                    dims[i] = broadcastDims(broadcastDims(dims[n.lhs], dims[n.rhs]), dims[n.aux]);
                } else if (Expression::isBinaryOp(n.op)) {
                    dims[i] = broadcastDims(dims[n.lhs], dims[n.rhs]);
                } else {
                    dims[i] = dims[n.lhs];
                }
        }
    }
    return dims;
}

namespace {

std::vector<std::vector<uint64_t>> inferShapes(const PlannedGraph& g, const std::vector<Tensor>& boundInputs) {
    return inferExpressionShapes(g.expr, [&](uint32_t slot) { return boundInputs.at(slot).getDimensions(); });
}

std::vector<uint64_t> orScalarShape(const std::vector<uint64_t>& dims) { return dims.empty() ? std::vector<uint64_t>{1} : dims; }

CubReductionOp valueReductionOp(ExprOp op) {
    switch (op) {
        case ExprOp::REDUCE_SUM: return CubReductionOp::Sum;
        case ExprOp::REDUCE_PROD: return CubReductionOp::Product;
        case ExprOp::REDUCE_MIN: return CubReductionOp::Min;
        case ExprOp::REDUCE_MAX: return CubReductionOp::Max;
        case ExprOp::REDUCE_AVG: return CubReductionOp::Mean;
        case ExprOp::REDUCE_NORM1: return CubReductionOp::L1Norm;
        case ExprOp::REDUCE_NORM2: return CubReductionOp::L2Norm;
        default: break;
    }
    throw std::runtime_error("Not a value reduction op.");
}

// THOR_DISABLE_ROW_FUSION=1 (or THOR_DISABLE_STAGE_FUSION=1) selects the staged plan: one stage per reduction and per
// elementwise group, like the reference's lowering.
bool stageFusionEnabled() {
    for (const char* name : {"THOR_DISABLE_ROW_FUSION", "THOR_DISABLE_STAGE_FUSION"}) {
        const char* env = std::getenv(name);
        if (env && env[0] == '1') return false;
    }
    return true;
}

}  // namespace

// ---- FusedEquation --------------------------------------------------------------------------------------------------------------
FusedEquation::FusedEquation(PhysicalOutputs outputs, int device_num)
    : outputs_template(std::move(outputs)),
      root_inputs(outputs_template.expr ? outputs_template.expr->inputs : std::vector<NamedInput>{}),
      device_num(device_num),
      planned_graph_cache(std::make_shared<LruCacheThreadSafe<std::string, std::shared_ptr<PlannedGraph>>>(128)) {}

FusedEquation FusedEquation::compile(const PhysicalExpression& expr, int device_num) {
    if (expr.output_node >= expr.nodes.size()) throw std::runtime_error("FusedEquation::compile requires a valid output node.");
    PhysicalOutputs outputs;
    outputs.expr = std::make_shared<PhysicalExpression>(expr);
    outputs.outputs.push_back(NamedOutput{"output", expr.output_node});
    return compile(outputs, device_num);
}

FusedEquation FusedEquation::compile(const PhysicalOutputs& outputs, int device_num) {
    if (!outputs.expr) throw std::runtime_error("FusedEquation::compile requires a non-null expression graph.");
    if (outputs.outputs.empty()) throw std::runtime_error("FusedEquation::compile requires at least one output.");
    for (const NamedOutput& o : outputs.outputs) {
        if (o.node_idx >= outputs.expr->nodes.size()) throw std::runtime_error("FusedEquation::compile output node index is out of range.");
    }
    int count = 0;
    THOR_HIP_CHECK(thorhip_device_count(&count));
    if (device_num < 0 || (count > 0 && device_num >= count)) {
        throw std::runtime_error("FusedEquation::compile: no such GPU: " + std::to_string(device_num));
    }
    // private copy: later edits of the caller's graph must not reach the compiled equation
    PhysicalOutputs copy;
    copy.expr = std::make_shared<PhysicalExpression>(*outputs.expr);
    copy.outputs = outputs.outputs;
    return FusedEquation(std::move(copy), device_num);
}

std::vector<std::string> FusedEquation::getOutputNames() const {
    std::vector<std::string> names;
    for (const NamedOutput& o : outputs_template.outputs) names.push_back(o.name);
    return names;
}

std::vector<DataType> FusedEquation::rootDTypes(const std::unordered_map<std::string, Tensor>& inputs) const {
    std::vector<DataType> dtypes(root_inputs.size(), DataType::FP32);
    for (const NamedInput& in : root_inputs) {
        if (in.kind == NamedInput::Kind::RuntimeScalarFp32) continue;
        auto it = inputs.find(in.name);
        if (it == inputs.end()) throw std::runtime_error("Missing required input tensor: " + in.name);
        if (!it->second.isInitialized()) throw std::runtime_error("Input tensor is not initialized: " + in.name);
        dtypes[in.slot] = it->second.getDataType();
    }
    for (const auto& [name, tensor] : inputs) {
        (void)tensor;
        bool known = false;
        for (const NamedInput& in : root_inputs) known = known || in.name == name;
        if (!known) throw std::runtime_error("Unexpected input tensor for this equation: " + name);
    }
    return dtypes;
}

std::shared_ptr<PlannedGraph> FusedEquation::plannedGraphFor(const std::vector<DataType>& root_dtypes) const {
    std::string key = stageFusionEnabled() ? "fused:" : "staged:";  // roles differ between the two kinds of plan
    for (DataType d : root_dtypes) key += std::to_string(static_cast<int>(d)) + ",";
    return planned_graph_cache->getOrCreate(key, [&] {
        PhysicalOutputs resolved;
        resolved.expr = std::make_shared<PhysicalExpression>(*outputs_template.expr);
        resolved.outputs = outputs_template.outputs;
        resolveOutputsDTypesInPlace(resolved, root_dtypes);

        auto graph = std::make_shared<PlannedGraph>();
        GraphBuilder builder(*resolved.expr);
        for (const NamedOutput& o : resolved.outputs) {
            uint32_t idx = builder.translate(o.node_idx);
            // a named output that is only an input in another dtype becomes an explicit cast
            idx = builder.asTensorOperand(idx, false);
            graph->outputs.push_back(NamedOutput{o.name, idx});
        }
        graph->expr = std::move(builder.out);
        graph->expr.output_node = graph->outputs.back().node_idx;

        const size_t count = graph->expr.nodes.size();
        graph->role.assign(count, Role::Inline);
        graph->level.assign(count, 0);
        auto ensureTensor = [&](uint32_t n) {
            if (graph->role[n] == Role::Inline) graph->role[n] = Role::Materialized;
        };
        for (uint32_t i = 0; i < count; ++i) {
            const ExprNode& n = graph->expr.nodes[i];
            if (n.op == ExprOp::INPUT) {
                graph->role[i] = Role::InputSource;
            } else if (isReductionOp(n.op)) {
                graph->role[i] = Role::Materialized;
                ensureTensor(n.lhs);
            } else if (n.op == ExprOp::SCAN) {
                graph->role[i] = Role::Materialized;
                ensureTensor(n.lhs);
            } else if (isSegmentedReduceOp(n.op) || n.op == ExprOp::SEGMENTED_BROADCAST || isWinnerRoutingOp(n.op) || n.op == ExprOp::TAKE_ALONG_AXIS ||
                       n.op == ExprOp::SEGMENTED_SCAN) {
                graph->role[i] = Role::Materialized;
                ensureTensor(n.lhs);
                ensureTensor(n.rhs);
            } else if (n.op == ExprOp::ROPE || isScatterRoutingOp(n.op)) {
                graph->role[i] = Role::Materialized;
                for (uint32_t operand : {n.lhs, n.rhs, n.aux})
                    if (operand != UINT32_MAX) ensureTensor(operand);
            } else if (n.op == ExprOp::RAGGED_VALUEWISE_EXTENT) {
                // the kernel that produces these values stops at the rows the partition covers
                graph->role[i] = Role::Materialized;
                ensureTensor(n.rhs);
            } else if (isShapeOnly(n.op)) {
                double folded;
                if (isStorageViewOp(n.op) || !tryFoldConstant(graph->expr, i, folded)) {
                    ensureTensor(n.lhs);
                    graph->role[i] = Role::View;
                }
            }
        }
        for (const NamedOutput& o : graph->outputs) ensureTensor(o.node_idx);

        if (stageFusionEnabled()) {
            std::vector<char> named(count, 0), fusable(count, 1), used(count, 0);
            for (const NamedOutput& o : graph->outputs) named[o.node_idx] = 1;
            for (uint32_t i = 0; i < count; ++i) {
                const ExprNode& n = graph->expr.nodes[i];
                for (uint32_t c : {n.lhs, n.rhs, n.aux}) {
                    if (c == UINT32_MAX || graph->expr.nodes[c].op != ExprOp::SEGMENTED_BROADCAST) continue;
                    used[c] = 1;
                    if (!consumesGather(n) || (n.op == ExprOp::RAGGED_VALUEWISE_EXTENT && n.rhs == c)) fusable[c] = 0;
                }
            }
            for (uint32_t i = 0; i < count; ++i) {
                if (graph->expr.nodes[i].op == ExprOp::SEGMENTED_BROADCAST && used[i] && fusable[i] && !named[i]) graph->role[i] = Role::Gather;
            }
            // An elementwise value that only one rotation reads is computed inside the rotation's kernel, element by element.
            for (uint32_t r = 0; r < count; ++r) {
                const ExprNode& rope = graph->expr.nodes[r];
                if (rope.op != ExprOp::ROPE) continue;
                const uint32_t m = rope.lhs;
                const ExprNode& operand = graph->expr.nodes[m];
                const bool elementwise = Expression::isBinaryOp(operand.op) || operand.op == ExprOp::WHERE || operand.op == ExprOp::CAST ||
                                         (Expression::isUnaryOp(operand.op) && !isReductionOp(operand.op) && !isShapeOnly(operand.op) && operand.op != ExprOp::SOFTMAX);
                if (graph->role[m] != Role::Materialized || named[m] || !elementwise) continue;
                bool ok = true;
                for (uint32_t j = 0; j < count && ok; ++j) {
                    const ExprNode& consumer = graph->expr.nodes[j];
                    if (j != r && (consumer.lhs == m || consumer.rhs == m || consumer.aux == m)) ok = false;
                }
                if (rope.rhs == m || rope.aux == m) ok = false;
                if (ok) graph->role[m] = Role::Inline;
            }
            // An elementwise value that only segmented reductions over one partition need as a tensor is never stored: the
            // reduction evaluates it in registers (per-segment values of the same partition are read once per segment), and
            // elementwise consumers recompute it.
            for (uint32_t r = 0; r < count; ++r) {
                const ExprNode& reduce = graph->expr.nodes[r];
                if (!isSegmentedReduceOp(reduce.op)) continue;
                const uint32_t m = reduce.lhs;
                const ExprNode& operand = graph->expr.nodes[m];
                const bool elementwise = Expression::isBinaryOp(operand.op) || operand.op == ExprOp::WHERE || operand.op == ExprOp::CAST ||
                                         (Expression::isUnaryOp(operand.op) && !isReductionOp(operand.op) && !isShapeOnly(operand.op) && operand.op != ExprOp::SOFTMAX);
                if (graph->role[m] != Role::Materialized || named[m] || !elementwise) continue;
                bool ok = true;
                for (uint32_t j = 0; j < count && ok; ++j) {
                    const ExprNode& consumer = graph->expr.nodes[j];
                    if (consumer.lhs != m && consumer.rhs != m && consumer.aux != m) continue;
                    if (isSegmentedReduceOp(consumer.op)) {
                        ok = consumer.lhs == m && consumer.rhs == reduce.rhs;
                    } else {
                        ok = consumesGather(consumer) && !(consumer.op == ExprOp::RAGGED_VALUEWISE_EXTENT && consumer.rhs == m);
                    }
                }
                // everything below m, down to tensors: elementwise work and broadcasts over the same partition
                std::vector<uint32_t> stack{m};
                std::vector<char> seen(count, 0);
                while (ok && !stack.empty()) {
                    const uint32_t v = stack.back();
                    stack.pop_back();
                    if (seen[v]) continue;
                    seen[v] = 1;
                    const ExprNode& node = graph->expr.nodes[v];
                    if (node.op == ExprOp::SEGMENTED_BROADCAST) {
                        ok = graph->role[v] != Role::Gather || (node.rhs == reduce.rhs && !node.segmented_broadcast_normalize_by_length);
                        continue;
                    }
                    if (v != m && graph->role[v] != Role::Inline) continue;
                    if (node.op == ExprOp::FILL || node.op == ExprOp::RAGGED_VALUEWISE_EXTENT) ok = false;
                    for (uint32_t c : {node.lhs, node.rhs, node.aux})
                        if (c != UINT32_MAX) stack.push_back(c);
                }
                if (ok) graph->role[m] = Role::Inline;
            }
        }

        // dependency levels: a materialised value runs after every materialised value it reads
        for (uint32_t i = 0; i < count; ++i) {
            if (graph->role[i] != Role::Materialized) continue;
            std::vector<uint32_t> sources, scalars;
            if (isReductionOp(graph->expr.nodes[i].op)) {
                sources.push_back(graph->expr.nodes[i].lhs);
            } else if (graph->expr.nodes[i].op == ExprOp::SCAN) {
                sources.push_back(graph->expr.nodes[i].lhs);
            } else if (graph->expr.nodes[i].op == ExprOp::ROPE || isScatterRoutingOp(graph->expr.nodes[i].op)) {
                for (uint32_t operand : {graph->expr.nodes[i].lhs, graph->expr.nodes[i].rhs, graph->expr.nodes[i].aux}) {
                    if (operand == UINT32_MAX) continue;
                    if (graph->role[operand] == Role::Inline) {
                        collectSources(*graph, operand, sources, scalars);  // evaluated inside the rotation
                    } else {
                        sources.push_back(operand);
                    }
                }
            } else if (isWinnerRoutingOp(graph->expr.nodes[i].op) || graph->expr.nodes[i].op == ExprOp::TAKE_ALONG_AXIS ||
                       graph->expr.nodes[i].op == ExprOp::SEGMENTED_SCAN) {
                sources.push_back(graph->expr.nodes[i].lhs);
                sources.push_back(graph->expr.nodes[i].rhs);
            } else if (isSegmentedReduceOp(graph->expr.nodes[i].op) || graph->expr.nodes[i].op == ExprOp::SEGMENTED_BROADCAST) {
                const uint32_t operand = graph->expr.nodes[i].lhs;
                if (graph->role[operand] == Role::Inline) {
                    collectSources(*graph, operand, sources, scalars);  // evaluated inside the reduction
                } else {
                    sources.push_back(operand);
                }
                sources.push_back(graph->expr.nodes[i].rhs);
            } else {
                collectSources(*graph, i, sources, scalars);
            }
            uint32_t level = 0;
            for (uint32_t s : sources) {
                const uint32_t base = baseOfView(*graph, s);
                if (graph->role[base] == Role::Materialized) level = std::max(level, graph->level[base] + 1);
            }
            graph->level[i] = level;
        }
        return graph;
    });
}

bool FusedEquation::resolveLayout(std::vector<Tensor>& inputs, std::vector<uint64_t>& outputDimensions) {
    if (inputs.empty()) throw std::runtime_error("resolveLayout requires at least one input tensor.");
    std::vector<uint64_t> dims;
    for (const Tensor& t : inputs) dims = broadcastDims(dims, t.getDimensions());
    outputDimensions = dims;
    bool broadcast = false;
    for (const Tensor& t : inputs) broadcast = broadcast || t.getDimensions() != dims;
    return broadcast;
}

std::unordered_map<std::string, Tensor> FusedEquation::withTensorScalars(const std::unordered_map<std::string, Tensor>& inputs,
                                                                         const std::unordered_map<std::string, TensorScalarBinding>& bindings) const {
    if (bindings.empty()) return inputs;
    std::unordered_map<std::string, Tensor> merged = inputs;
    for (const auto& [name, binding] : bindings) {
        bool declared = false;
        for (const NamedInput& in : root_inputs) declared = declared || (in.name == name && in.kind == NamedInput::Kind::TensorRuntimeScalar);
        if (!declared) throw std::runtime_error("Unexpected tensor-runtime-scalar input for this equation: " + name);
        if (inputs.count(name)) throw std::runtime_error("Input '" + name + "' is bound both as a tensor and as a tensor-runtime-scalar.");
        if (!binding.buffer.isInitialized()) throw std::runtime_error("Tensor-runtime-scalar buffer is not initialized for " + name + ".");
        if (binding.buffer.getDataType() != binding.sourceDType) {
            throw std::runtime_error("Tensor-runtime-scalar binding for " + name + " must use a backing buffer with the same dtype as the scalar source dtype.");
        }
        const uint64_t elementBytes = dataTypeSizeInBytes(binding.sourceDType);
        if (elementBytes == 0 || binding.byteOffset % elementBytes != 0) {
            throw std::runtime_error("Tensor-runtime-scalar binding byte offset is not element-aligned for " + name + ".");
        }
        if (!binding.buffer.isDenseContiguous() || binding.byteOffset + elementBytes > binding.buffer.getTotalNumElements() * elementBytes) {
            throw std::runtime_error("Tensor-runtime-scalar binding exceeds backing buffer size for " + name + ".");
        }
        Tensor flat = binding.buffer;
        flat.reshape({binding.buffer.getTotalNumElements()});
        merged.emplace(name, flat.aliasView({1}, {1}, binding.byteOffset / elementBytes));
    }
    return merged;
}

StampedExecutionPlan FusedEquation::stamp(const std::unordered_map<std::string, Tensor>& inputs, const Stream& stream,
                                          const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs,
                                          const std::unordered_map<std::string, Tensor>& preallocated_outputs,
                                          const std::unordered_map<std::string, std::vector<uint64_t>>& requestedOutputShapes) const {
    return stampImpl(withTensorScalars(inputs, tensor_scalar_inputs), stream, preallocated_outputs, false, requestedOutputShapes);
}

StampedExecutionPlan FusedEquation::stampSingleOutput(const std::unordered_map<std::string, Tensor>& inputs, const Stream& stream,
                                                      const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs,
                                                      const std::optional<Tensor>& preallocated_output,
                                                      const std::vector<uint64_t>& requestedOutputShape) const {
    if (outputs_template.outputs.size() != 1) throw std::runtime_error("stampSingleOutput requires an equation with exactly one output.");
    std::unordered_map<std::string, Tensor> pre;
    if (preallocated_output.has_value()) pre.emplace(outputs_template.outputs[0].name, preallocated_output.value());
    std::unordered_map<std::string, std::vector<uint64_t>> requested;
    if (!requestedOutputShape.empty()) requested.emplace(outputs_template.outputs[0].name, requestedOutputShape);
    return stampImpl(withTensorScalars(inputs, tensor_scalar_inputs), stream, pre, false, requested);
}

namespace {
// equal once axes of extent 1 are dropped (reference: outputDimensionsMatchIgnoringSingletons, FusedEquation.cpp:3170-3174)
bool sameDimensionsIgnoringSingletons(const std::vector<uint64_t>& a, const std::vector<uint64_t>& b) {
    std::vector<uint64_t> x, y;
    for (uint64_t d : a)
        if (d != 1) x.push_back(d);
    for (uint64_t d : b)
        if (d != 1) y.push_back(d);
    return x == y;
}
}  // namespace

StampedExecutionPlan FusedEquation::stampImpl(const std::unordered_map<std::string, Tensor>& inputs, const Stream& stream,
                                              const std::unordered_map<std::string, Tensor>& preallocated, bool fusedKernelsOnly,
                                              const std::unordered_map<std::string, std::vector<uint64_t>>& requestedOutputShapes) const {
    if (!stream.isInitialized()) throw std::runtime_error("FusedEquation::stamp requires an initialized stream.");
    if (stream.getGpuNum() != device_num) throw std::runtime_error("FusedEquation::stamp: the stream belongs to another GPU than the equation.");
    if (backward) {
        std::unordered_map<std::string, Tensor> used;
        const std::shared_ptr<const FusedEquation> equation = backwardFor(inputs, used);
        return equation->stampImpl(used, stream, preallocated, fusedKernelsOnly, requestedOutputShapes);
    }
    const std::vector<DataType> dtypes = rootDTypes(inputs);
    const std::shared_ptr<PlannedGraph> graph = plannedGraphFor(dtypes);
    const PhysicalExpression& expr = graph->expr;
    const TensorPlacement gpuPlacement(TensorPlacement::MemDevices::GPU, device_num);

    std::vector<Tensor> bound(root_inputs.size());
    for (const NamedInput& in : root_inputs) {
        if (in.kind == NamedInput::Kind::RuntimeScalarFp32) continue;
        const Tensor& t = inputs.at(in.name);
        if (t.getPlacement() != gpuPlacement) throw std::runtime_error("Input tensor '" + in.name + "' does not live on the equation's GPU.");
        bound[in.slot] = t;
    }
    for (const auto& [name, tensor] : preallocated) {
        bool known = false;
        for (const NamedOutput& o : graph->outputs) known = known || o.name == name;
        if (!known) throw std::runtime_error("Preallocated output '" + name + "' is not an output of this equation.");
        if (!tensor.isInitialized() || tensor.getPlacement() != gpuPlacement) {
            throw std::runtime_error("Preallocated output '" + name + "' must be an initialized tensor on the equation's GPU.");
        }
    }

    const std::vector<std::vector<uint64_t>> dims = inferShapes(*graph, bound);
    ScopedGpu scoped(device_num);

    // ---- tensors of every tensor-role node --------------------------------------------------------------------------
    std::vector<Tensor> tensorOf(expr.nodes.size());
    std::unordered_map<uint32_t, std::string> outputNameOfNode;
    for (const NamedOutput& o : graph->outputs) outputNameOfNode.emplace(o.node_idx, o.name);  // first name wins for allocation

    auto allocateFor = [&](uint32_t node) {
        const DataType dtype = expr.nodes[node].output_dtype.value();
        const std::vector<uint64_t> shape = orScalarShape(dims[node]);
        auto named = outputNameOfNode.find(node);
        if (named != outputNameOfNode.end()) {
            auto pre = preallocated.find(named->second);
            if (pre != preallocated.end()) {
                const Tensor& t = pre->second;
                if (t.getDataType() != dtype) {
                    throw std::runtime_error("Preallocated output '" + named->second + "' has dtype " + dataTypeName(t.getDataType()) +
                                             " but the expression produces " + dataTypeName(dtype) + ".");
                }
                if (t.getDimensions() != shape) {
                    throw std::runtime_error("Preallocated output '" + named->second + "' has shape " + t.dimensionsToString() +
                                             " but the expression produces " + TensorDescriptor(dtype, shape).toString() + ".");
                }
                if (!t.isDenseContiguous()) throw std::runtime_error("Preallocated output '" + named->second + "' must be dense.");
                return t;
            }
        }
        return Tensor(gpuPlacement, TensorDescriptor(dtype, shape));
    };

    auto viewOf = [&](uint32_t node) {
        const Tensor& base = tensorOf[expr.nodes[node].lhs];
        const ExprNode& v = expr.nodes[node];
        if (v.op == ExprOp::STRIDED_VIEW) {
            // strides and offset address the storage the operand resolves to
            if (!base.isDenseContiguous()) throw std::runtime_error("Expression::stridedView needs a dense operand: compose the strides of nested views first.");
            return base.aliasView(v.view_dims, v.view_strides, v.view_element_offset);
        }
        if (v.op == ExprOp::TRANSPOSE) {
            std::vector<uint64_t> d = base.getDimensions(), st = base.getStridesElements();
            if (d.size() < 2) throw std::runtime_error("Expression::transpose requires a tensor of rank 2 or more.");
            std::swap(d[d.size() - 1], d[d.size() - 2]);
            std::swap(st[st.size() - 1], st[st.size() - 2]);
            return base.aliasView(d, st, 0);
        }
        if (!base.isDenseContiguous()) throw std::runtime_error("Shape operations on a non-dense tensor view are not supported.");
        Tensor view = base;
        view.reshape(orScalarShape(dims[node]));
        return view;
    };

    // ---- stages in level order -----------------------------------------------------------------------------------------
    // Elementwise values are grouped into kernels by shape (and ragged extent).  With the shapes known, a stored value that
    // another value of the same group reads directly need not come back from memory: both run in one kernel, which keeps the
    // producer's value in registers and stores it as well.  That holds when the stored value is the computed one (storage
    // dtype = arithmetic dtype) and the consumer does not read it through a view.
    auto groupKeyOf = [&](uint32_t i) {
        const ExprNode& n = expr.nodes[i];
        std::vector<uint64_t> key = orScalarShape(dims[i]);
        if (n.op == ExprOp::RAGGED_VALUEWISE_EXTENT) {
            // kernels of ragged values stop at the partition's last row, so they are grouped by partition as well
            key.push_back(UINT64_MAX);
            key.push_back(n.rhs);
            key.push_back(n.ragged_runtime_batch_size);
            key.push_back(n.ragged_runtime_elements_per_value);
        }
        return key;
    };
    auto runsInFusedKernel = [&](uint32_t i) {
        const ExprOp op = expr.nodes[i].op;
        return graph->role[i] == Role::Materialized && !isReductionOp(op) && !isSegmentedReduceOp(op) && op != ExprOp::SEGMENTED_BROADCAST &&
               !isWinnerRoutingOp(op) && op != ExprOp::TAKE_ALONG_AXIS && op != ExprOp::ROPE && !isScatterRoutingOp(op) && !isScanOp(op) && op != ExprOp::INPUT;
    };
    std::vector<uint32_t> levelOf = graph->level;
    if (stageFusionEnabled()) {
        for (uint32_t i = 0; i < expr.nodes.size(); ++i) {
            if (graph->role[i] != Role::Materialized) continue;
            const ExprNode& n = expr.nodes[i];
            std::vector<uint32_t> sources, scalars;
            if (isReductionOp(n.op)) {
                sources.push_back(n.lhs);
            } else if (n.op == ExprOp::SCAN) {
                sources = {n.lhs};
            } else if (n.op == ExprOp::ROPE || isScatterRoutingOp(n.op)) {
                for (uint32_t operand : {n.lhs, n.rhs, n.aux}) {
                    if (operand == UINT32_MAX) continue;
                    if (graph->role[operand] == Role::Inline) {
                        collectSources(*graph, operand, sources, scalars);
                    } else {
                        sources.push_back(operand);
                    }
                }
            } else if (isWinnerRoutingOp(n.op) || n.op == ExprOp::TAKE_ALONG_AXIS || n.op == ExprOp::SEGMENTED_SCAN) {
                sources = {n.lhs, n.rhs};
            } else if (isSegmentedReduceOp(n.op) || n.op == ExprOp::SEGMENTED_BROADCAST) {
                if (graph->role[n.lhs] == Role::Inline) {
                    collectSources(*graph, n.lhs, sources, scalars);
                } else {
                    sources.push_back(n.lhs);
                }
                sources.push_back(n.rhs);
            } else {
                collectSources(*graph, i, sources, scalars);
            }
            uint32_t level = 0;
            for (uint32_t s : sources) {
                const uint32_t base = baseOfView(*graph, s);
                if (graph->role[base] != Role::Materialized) continue;
                const bool sameKernel = s == base && runsInFusedKernel(i) && runsInFusedKernel(base) && groupKeyOf(base) == groupKeyOf(i) &&
                                        expr.nodes[base].output_dtype.value() == emittedValueDType(expr.nodes[base]);
                level = std::max(level, levelOf[base] + (sameKernel ? 0 : 1));
            }
            levelOf[i] = level;
        }
    }
    uint32_t maxLevel = 0;
    for (uint32_t i = 0; i < expr.nodes.size(); ++i)
        if (graph->role[i] == Role::Materialized) maxLevel = std::max(maxLevel, levelOf[i]);

    for (uint32_t i = 0; i < expr.nodes.size(); ++i) {
        if (graph->role[i] == Role::InputSource) tensorOf[i] = bound[expr.nodes[i].input_slot];
    }
    // views of inputs can be resolved right away; views of materialised values are resolved after their stage
    auto resolveViewsUpTo = [&]() {
        for (uint32_t i = 0; i < expr.nodes.size(); ++i) {
            if (graph->role[i] == Role::View && !tensorOf[i].isInitialized() && tensorOf[expr.nodes[i].lhs].isInitialized()) tensorOf[i] = viewOf(i);
        }
    };
    resolveViewsUpTo();

    std::vector<StampedExecutionStage> stages;
    std::vector<int> stageOfNode(expr.nodes.size(), -1);
    auto dependenciesOf = [&](const std::vector<uint32_t>& sources) {
        std::vector<uint32_t> deps;
        for (uint32_t s : sources) {
            const int st = stageOfNode[baseOfView(*graph, s)];
            if (st >= 0) deps.push_back(static_cast<uint32_t>(st));
        }
        std::sort(deps.begin(), deps.end());
        deps.erase(std::unique(deps.begin(), deps.end()), deps.end());
        return deps;
    };

    std::vector<char> done(expr.nodes.size(), 0);
    std::map<std::pair<uint32_t, uint64_t>, std::pair<Tensor, uint32_t>> segmentIds;  // (offsets node, row capacity) -> index tensor, its stage
    std::unordered_map<uint32_t, uint32_t> materialisedGather;                        // gather node -> the stage that wrote its rows
    const bool stageFusion = stageFusionEnabled() && !fusedKernelsOnly;
    std::vector<uint8_t> roles(graph->role.size());
    for (size_t i = 0; i < roles.size(); ++i) roles[i] = static_cast<uint8_t>(graph->role[i]);
    RowFusionContext context{expr, graph->outputs, root_inputs, roles, dims, tensorOf, done, stages, stageOfNode, allocateFor, device_num, stream};
    if (stageFusion) {
        // Recognise chains of last-axis reductions and row-wise elementwise work over one [rows, R] input and emit them
        // as one kernel that keeps each row in registers.
        tryRowFusion(context);
        resolveViewsUpTo();
    }

    // One fused elementwise kernel for values of one shape (and one ragged extent): gathers its sources, emits and compiles the
    // kernel, allocates the outputs and appends the stage.
    auto emitFusedGroup = [&](const std::vector<uint32_t>& nodes) {
        FusedKernelRequest request;
        request.expr = &expr;
        const std::vector<uint64_t> shape = orScalarShape(dims[nodes.front()]);
        request.outputDims = shape;
        std::optional<Tensor> extentOffsets;
        if (expr.nodes[nodes.front()].op == ExprOp::RAGGED_VALUEWISE_EXTENT) {
            const ExprNode& marker = expr.nodes[nodes.front()];
            extentOffsets = tensorOf[marker.rhs];
            if (!extentOffsets->isInitialized() || !extentOffsets->isDenseContiguous() ||
                extentOffsets->getTotalNumElements() != marker.ragged_runtime_batch_size + 1) {
                throw std::runtime_error("Ragged runtime extent offsets must be a dense tensor with batch size + 1 entries.");
            }
            uint64_t elements = 1;
            for (uint64_t d : shape) elements *= d;
            if (elements != marker.ragged_runtime_max_active_values * marker.ragged_runtime_elements_per_value) {
                throw std::runtime_error("Ragged values do not have the shape [max active values, elements per value] their descriptor states.");
            }
            request.extent = RaggedExtent{marker.ragged_runtime_batch_size, marker.ragged_runtime_elements_per_value,
                                          extentOffsets->getDataType() == DataType::UINT64};
        }
        std::vector<uint32_t> sources, scalarSlots;
        for (uint32_t node : nodes) {
            std::vector<uint32_t> s, sc;
            if (isTensorRole(graph->role[node]) && expr.nodes[node].op == ExprOp::INPUT) {
                s.push_back(node);
            } else {
                collectSources(*graph, node, s, sc);
            }
            sources.insert(sources.end(), s.begin(), s.end());
            scalarSlots.insert(scalarSlots.end(), sc.begin(), sc.end());
        }
        std::sort(sources.begin(), sources.end());
        sources.erase(std::unique(sources.begin(), sources.end()), sources.end());
        // a value this kernel computes itself is used from registers (its own sources are listed through its membership)
        sources.erase(std::remove_if(sources.begin(), sources.end(),
                                     [&](uint32_t s) {
                                         return graph->role[s] == Role::Materialized && !done[s] && std::find(nodes.begin(), nodes.end(), s) != nodes.end();
                                     }),
                      sources.end());
        std::sort(scalarSlots.begin(), scalarSlots.end());
        scalarSlots.erase(std::unique(scalarSlots.begin(), scalarSlots.end()), scalarSlots.end());

        // Per-segment values reach a flat kernel through the row -> segment index; a kernel that broadcasts other operands
        // gets them as a materialised [rows, E] tensor instead.
        auto stripOnes = [](const std::vector<uint64_t>& d) {
            std::vector<uint64_t> out;
            for (uint64_t v : d)
                if (v != 1) out.push_back(v);
            return out;
        };
        bool flatGroup = true;
        for (uint32_t s : sources) {
            if (graph->role[s] == Role::Gather) continue;
            flatGroup = flatGroup && tensorOf[s].isInitialized() && tensorOf[s].isDenseContiguous() && stripOnes(orScalarShape(dims[s])) == stripOnes(shape);
        }
        std::vector<uint32_t> extraDependencies;
        std::vector<Tensor> inputTensors, gatherTensors;
        for (uint32_t s : sources) {
            if (graph->role[s] == Role::Gather && !tensorOf[s].isInitialized()) {
                const ExprNode& g = expr.nodes[s];
                const Tensor& perSegment = tensorOf[g.lhs];
                const Tensor& offsets = tensorOf[g.rhs];
                if (!perSegment.isInitialized() || !offsets.isInitialized()) throw std::logic_error("Gathered per-segment values have not been produced yet.");
                if (flatGroup && perSegment.isDenseContiguous() && offsets.isDenseContiguous()) {
                    const uint64_t capacity = g.ragged_runtime_max_active_values;
                    auto key = std::make_pair(g.rhs, capacity);
                    auto found = segmentIds.find(key);
                    if (found == segmentIds.end()) {
                        Tensor ids(gpuPlacement, TensorDescriptor(DataType::UINT32, {capacity}));
                        StampedExecutionStage stage;
                        stage.kind = StampedExecutionStage::Kind::SegmentedBroadcast;
                        stage.gpu_num = device_num;
                        stage.segmented_broadcast = stampSegmentIds(offsets, ids, stream);
                        found = segmentIds.emplace(key, std::make_pair(ids, static_cast<uint32_t>(stages.size()))).first;
                        stages.push_back(std::move(stage));
                    }
                    GatherOperand gather;
                    gather.node = s;
                    gather.storageDType = perSegment.getDataType();
                    gather.elementsPerValue = g.ragged_runtime_elements_per_value;
                    gather.segments = g.ragged_runtime_batch_size;
                    gather.normalize = g.segmented_broadcast_normalize_by_length;
                    gather.offsetsAre64 = offsets.getDataType() == DataType::UINT64;
                    gather.alignmentBytes = pointerAlignment(perSegment.getMemPtr());
                    if (perSegment.getTotalNumElements() != gather.segments * gather.elementsPerValue ||
                        offsets.getTotalNumElements() != gather.segments + 1) {
                        throw std::runtime_error("Segmented broadcast operands do not have the shapes [B, E] and [B + 1] of their ragged descriptor.");
                    }
                    request.gathers.push_back(gather);
                    gatherTensors.push_back(perSegment);
                    gatherTensors.push_back(found->second.first);
                    if (gather.normalize) gatherTensors.push_back(offsets);
                    extraDependencies.push_back(found->second.second);
                    continue;
                }
                // not a flat kernel: materialise the broadcast once and read it like any other tensor
                Tensor rows(gpuPlacement, TensorDescriptor(g.output_dtype.value(), orScalarShape(dims[s])));
                StampedExecutionStage stage;
                stage.kind = StampedExecutionStage::Kind::SegmentedBroadcast;
                stage.gpu_num = device_num;
                stage.dependency_stage_indices = dependenciesOf({g.lhs, g.rhs});
                stage.segmented_broadcast = stampSegmentedBroadcast(perSegment, offsets, rows, g.segmented_broadcast_normalize_by_length, stream);
                tensorOf[s] = rows;
                materialisedGather[s] = static_cast<uint32_t>(stages.size());
                stages.push_back(std::move(stage));
            }
            if (materialisedGather.count(s)) extraDependencies.push_back(materialisedGather.at(s));
            const Tensor& t = tensorOf[s];
            if (!t.isInitialized()) throw std::logic_error("Fused stage reads a value that has not been produced yet.");
            KernelOperand operand;
            operand.node = s;
            operand.storageDType = t.getDataType();
            operand.dims = orScalarShape(dims[s]);
            operand.strides = t.getStridesElements();
            if (operand.strides.size() != operand.dims.size()) throw std::logic_error("Operand rank does not match its tensor.");
            operand.alignmentBytes = pointerAlignment(t.getMemPtr());
            request.operands.push_back(operand);
            inputTensors.push_back(t);
        }
        request.scalarSlots = scalarSlots;
        std::vector<Tensor> outputTensors;
        for (uint32_t node : nodes) {
            Tensor out = allocateFor(node);
            KernelOutput ko;
            ko.node = node;
            ko.storageDType = out.getDataType();
            ko.alignmentBytes = pointerAlignment(out.getMemPtr());
            request.outputs.push_back(ko);
            outputTensors.push_back(out);
            tensorOf[node] = out;
        }
        const EmittedKernel emitted = emitFusedKernel(request);
        std::shared_ptr<CompiledKernel> kernel = compileKernel(emitted.source, emitted.kernelName, device_num, emitted.fastContract);

        inputTensors.insert(inputTensors.end(), gatherTensors.begin(), gatherTensors.end());  // pointer arguments after the operands
        if (extentOffsets.has_value()) inputTensors.push_back(extentOffsets.value());
        std::vector<size_t> inputArgIndex(inputTensors.size()), outputArgIndex(outputTensors.size());
        std::iota(inputArgIndex.begin(), inputArgIndex.end(), 0);
        std::vector<StampedEquation::ScalarArgument> scalarArgs;
        size_t next = inputTensors.size();
        for (uint32_t slot : scalarSlots) scalarArgs.push_back({root_inputs.at(slot).name, next++});
        for (size_t o = 0; o < outputTensors.size(); ++o) outputArgIndex[o] = next++;

        StampedExecutionStage stage;
        stage.kind = StampedExecutionStage::Kind::FusedKernel;
        stage.gpu_num = device_num;
        stage.dependency_stage_indices = dependenciesOf(sources);
        stage.dependency_stage_indices.insert(stage.dependency_stage_indices.end(), extraDependencies.begin(), extraDependencies.end());
        std::sort(stage.dependency_stage_indices.begin(), stage.dependency_stage_indices.end());
        stage.dependency_stage_indices.erase(std::unique(stage.dependency_stage_indices.begin(), stage.dependency_stage_indices.end()),
                                             stage.dependency_stage_indices.end());
        stage.kernel = std::make_shared<StampedEquation>(kernel, inputTensors, outputTensors, scalarArgs, inputArgIndex, outputArgIndex, next,
                                                         emitted.passNumel, emitted.numel, emitted.numelIs64, emitted.gridX, emitted.threads,
                                                         emitted.flopsPerElement * emitted.numel, emitted.description + " [" + kernel->kernelName + "]");
        for (uint32_t node : nodes) {
            stageOfNode[node] = static_cast<int>(stages.size());
            done[node] = 1;
        }
        stages.push_back(std::move(stage));
    };

    // A segmented reduction whose operand is an elementwise expression: the reduction kernel evaluates the expression in
    // registers.  Sources are tensors of the operand's shape, single elements, and per-segment tensors that the expression
    // broadcasts over the same partition (read once per segment and trailing element).  False = cannot be done this way.
    auto stampSegmentedReductionOfExpression = [&](uint32_t node) -> bool {
        const ExprNode& n = expr.nodes[node];
        const uint32_t operand = n.lhs;
        const Tensor& offsets = tensorOf[n.rhs];
        std::vector<uint32_t> sources, scalarSlots;
        collectSources(*graph, operand, sources, scalarSlots);
        const std::vector<uint64_t> valueShape = orScalarShape(dims[operand]);
        if (valueShape.empty() || !offsets.isInitialized() || !offsets.isDenseContiguous()) return false;
        uint64_t trailing = 1;
        for (size_t a = 1; a < valueShape.size(); ++a) trailing *= valueShape[a];
        const uint64_t rows = valueShape[0], segments = offsets.getTotalNumElements() - 1;
        auto stripOnes = [](const std::vector<uint64_t>& d) {
            std::vector<uint64_t> out;
            for (uint64_t v : d)
                if (v != 1) out.push_back(v);
            return out;
        };
        using SourceKind = ReductionKernelRequest::Source::Kind;
        ReductionKernelRequest request;
        request.segmented = true;
        request.segments = segments;
        request.segmentedRows = rows;
        request.trailing = trailing;
        request.offsetsAre64 = offsets.getDataType() == DataType::UINT64;
        request.deviceNum = device_num;
        request.inputAlignmentBytes = 256;
        request.geometry.path = CubReductionPath::OffsetSegmented;
        request.geometry.rank = static_cast<uint32_t>(valueShape.size());
        request.geometry.input_elements = rows * trailing;
        request.geometry.output_elements = segments * trailing;
        request.geometry.reduction_size = rows;
        request.geometry.output_dimensions = orScalarShape(dims[node]);
        request.geometry.squeezed_output_dimensions = request.geometry.output_dimensions;
        request.scalarSlots = scalarSlots;

        BodyEmitter body(expr);
        std::string text;
        for (uint32_t slot : scalarSlots) text += "        const float s" + std::to_string(slot) + " = s.s" + std::to_string(slot) + ";\n";
        std::vector<Tensor> inputs;
        bool anyVector = false;
        for (uint32_t s : sources) {
            Tensor t;
            SourceKind kind;
            if (graph->role[s] == Role::Gather && !tensorOf[s].isInitialized()) {
                const ExprNode& g = expr.nodes[s];
                t = tensorOf[g.lhs];
                if (g.rhs != n.rhs || g.segmented_broadcast_normalize_by_length || !t.isInitialized() || !t.isDenseContiguous() ||
                    t.getTotalNumElements() != segments * trailing) {
                    return false;
                }
                kind = SourceKind::Kept;
            } else {
                t = tensorOf[s];
                if (!t.isInitialized() || !t.isDenseContiguous()) return false;
                if (stripOnes(orScalarShape(dims[s])) == stripOnes(valueShape)) {
                    kind = SourceKind::Vector;
                } else if (t.getTotalNumElements() == 1) {
                    kind = SourceKind::Scalar;
                } else {
                    return false;
                }
            }
            const size_t index = inputs.size();
            ReductionKernelRequest::Source source;
            source.storage = t.getDataType();
            source.kind = kind;
            request.sources.push_back(source);
            if (kind == SourceKind::Vector) {
                request.inputAlignmentBytes = std::min(request.inputAlignmentBytes, pointerAlignment(t.getMemPtr()));
                anyVector = true;
            }
            inputs.push_back(t);
            const DataType valueDType = expr.nodes[s].output_dtype.value();
            const std::string raw = kind == SourceKind::Vector ? "l.p" + std::to_string(index) + ".v[k]" : "kk.z" + std::to_string(index);
            text += "        const " + std::string(valueCType(valueDType)) + " t" + std::to_string(s) + " = " +
                    castValueExpr(storageToValueExpr(raw, t.getDataType()), t.getDataType(), valueDType) + ";\n";
            body.defineSource(s, valueDType);
        }
        if (!anyVector) return false;
        uint64_t flopsPerElement = 1;
        for (uint32_t v : body.collect({operand})) flopsPerElement += body.emit(text, v, "        ");
        // the staged plan would have stored the operand in its output dtype: round there before accumulating in fp32
        const DataType storedDType = expr.nodes[operand].output_dtype.value();
        ReductionKernelRequest::Value value;
        value.op = n.op == ExprOp::SEGMENTED_REDUCE_SUM   ? CubReductionOp::Sum
                   : n.op == ExprOp::SEGMENTED_REDUCE_MIN ? CubReductionOp::Min
                   : n.op == ExprOp::SEGMENTED_REDUCE_MAX ? CubReductionOp::Max
                                                          : CubReductionOp::Mean;
        value.outputDType = n.output_dtype.value();
        value.expression = castValueExpr(body.ref(operand, storedDType), storedDType, DataType::FP32);
        request.values.push_back(value);
        request.prologue = text;
        request.inputDType = inputs.front().getDataType();

        ReductionLaunchPlan plan = buildReductionKernels(request);
        std::optional<Tensor> workspace = allocateReductionWorkspace(plan, gpuPlacement, stream);
        Tensor output = allocateFor(node);
        std::vector<std::string> scalarNames;
        for (uint32_t slot : scalarSlots) scalarNames.push_back(root_inputs.at(slot).name);
        StampedExecutionStage stage;
        stage.kind = StampedExecutionStage::Kind::FusedReduction;
        stage.gpu_num = device_num;
        sources.push_back(n.rhs);
        stage.dependency_stage_indices = dependenciesOf(sources);
        plan.variant = "fused_segmented_reduction(sources=" + std::to_string(inputs.size()) + ") " + plan.variant;
        stage.fused_reduction = std::make_shared<StampedFusedReduction>(std::move(plan), inputs, scalarNames, std::vector<Tensor>{output}, std::vector<Tensor>{},
                                                                        workspace, flopsPerElement * rows * trailing, offsets);
        tensorOf[node] = output;
        stageOfNode[node] = static_cast<int>(stages.size());
        stages.push_back(std::move(stage));
        done[node] = 1;
        return true;
    };

    // The two statistics of a segment softmax in one pass over the values: `node` is the segment maximum of a tensor x, and a
    // segment sum over the same partition of exp(x - broadcast(maximum)) (fp32 arithmetic, nothing else in between) is waiting
    // further up.  One segment kernel with a {maximum, sum of exponentials} accumulator writes both.  False = not that pattern.
    auto stampSegmentSoftmaxStatistics = [&](uint32_t node) -> bool {
        const ExprNode& n = expr.nodes[node];
        if (n.op != ExprOp::SEGMENTED_REDUCE_MAX || graph->role[n.lhs] == Role::Inline) return false;
        uint32_t sumNode = UINT32_MAX;
        for (uint32_t j = node + 1; j < expr.nodes.size() && sumNode == UINT32_MAX; ++j) {
            const ExprNode& sum = expr.nodes[j];
            if (done[j] || sum.op != ExprOp::SEGMENTED_REDUCE_SUM || graph->role[j] != Role::Materialized || sum.rhs != n.rhs) continue;
            if (sum.lhs == UINT32_MAX || graph->role[sum.lhs] != Role::Inline) continue;
            const ExprNode& e = expr.nodes[sum.lhs];
            if (e.op != ExprOp::EXP || emittedValueDType(e) != DataType::FP32 || e.output_dtype != DataType::FP32 || graph->role[e.lhs] != Role::Inline) continue;
            const ExprNode& d = expr.nodes[e.lhs];
            if (d.op != ExprOp::SUB || emittedValueDType(d) != DataType::FP32 || d.lhs != n.lhs || d.rhs == UINT32_MAX) continue;
            const ExprNode& g = expr.nodes[d.rhs];
            if (g.op != ExprOp::SEGMENTED_BROADCAST || graph->role[d.rhs] != Role::Gather || g.lhs != node || g.rhs != n.rhs ||
                g.segmented_broadcast_normalize_by_length) {
                continue;
            }
            sumNode = j;
        }
        if (sumNode == UINT32_MAX) return false;
        const Tensor& values = tensorOf[n.lhs];
        const Tensor& offsets = tensorOf[n.rhs];
        if (!values.isInitialized() || !values.isDenseContiguous() || !offsets.isInitialized() || !offsets.isDenseContiguous()) return false;
        const std::vector<uint64_t> valueShape = orScalarShape(dims[n.lhs]);
        if (valueShape.empty()) return false;
        uint64_t trailing = 1;
        for (size_t a = 1; a < valueShape.size(); ++a) trailing *= valueShape[a];
        const uint64_t rows = valueShape[0], segments = offsets.getTotalNumElements() - 1;
        ReductionKernelRequest request;
        request.segmented = true;
        request.segments = segments;
        request.segmentedRows = rows;
        request.trailing = trailing;
        request.offsetsAre64 = offsets.getDataType() == DataType::UINT64;
        request.deviceNum = device_num;
        request.inputAlignmentBytes = pointerAlignment(values.getMemPtr());
        request.geometry.path = CubReductionPath::OffsetSegmented;
        request.geometry.rank = static_cast<uint32_t>(valueShape.size());
        request.geometry.input_elements = rows * trailing;
        request.geometry.output_elements = segments * trailing;
        request.geometry.reduction_size = rows;
        request.geometry.output_dimensions = orScalarShape(dims[node]);
        request.geometry.squeezed_output_dimensions = request.geometry.output_dimensions;
        ReductionKernelRequest::Source source;
        source.storage = values.getDataType();
        source.kind = ReductionKernelRequest::Source::Kind::Vector;
        request.sources.push_back(source);
        const DataType valueDType = expr.nodes[n.lhs].output_dtype.value();
        request.prologue = "        const float x0 = " +
                           castValueExpr(castValueExpr(storageToValueExpr("l.p0.v[k]", values.getDataType()), values.getDataType(), valueDType), valueDType,
                                         DataType::FP32) +
                           ";\n";
        request.values.push_back({CubReductionOp::Max, n.output_dtype.value(), "x0"});
        request.values.push_back({CubReductionOp::Sum, expr.nodes[sumNode].output_dtype.value(), "x0"});
        request.onlineSoftmax = true;
        request.inputDType = values.getDataType();

        ReductionLaunchPlan plan = buildReductionKernels(request);
        std::optional<Tensor> workspace = allocateReductionWorkspace(plan, gpuPlacement, stream);
        Tensor maxima = allocateFor(node), sums = allocateFor(sumNode);
        StampedExecutionStage stage;
        stage.kind = StampedExecutionStage::Kind::FusedReduction;
        stage.gpu_num = device_num;
        stage.dependency_stage_indices = dependenciesOf({n.lhs, n.rhs});
        plan.variant = "segment_softmax_statistics(max, sum of exp in one pass) " + plan.variant;
        stage.fused_reduction = std::make_shared<StampedFusedReduction>(std::move(plan), std::vector<Tensor>{values}, std::vector<std::string>{},
                                                                        std::vector<Tensor>{maxima, sums}, std::vector<Tensor>{}, workspace,
                                                                        4 * rows * trailing, offsets);
        tensorOf[node] = maxima;
        tensorOf[sumNode] = sums;
        stageOfNode[node] = stageOfNode[sumNode] = static_cast<int>(stages.size());
        stages.push_back(std::move(stage));
        done[node] = done[sumNode] = 1;
        return true;
    };

    for (uint32_t level = 0; level <= maxLevel; ++level) {
        if (stageFusion) {
            // Reductions over one shape and axes whose inputs exist by now (or are elementwise functions of such tensors
            // that nothing else needs) run as one pass.
            tryReductionFusion(context);
            resolveViewsUpTo();
        }
        // fused values of this level, grouped by output shape so that one kernel shares the loads
        std::map<std::vector<uint64_t>, std::vector<uint32_t>> fusedGroups;
        for (uint32_t i = 0; i < expr.nodes.size(); ++i) {
            if (graph->role[i] != Role::Materialized || levelOf[i] != level || done[i]) continue;
            const ExprNode& n = expr.nodes[i];
            if (isSegmentedReduceOp(n.op) || n.op == ExprOp::SEGMENTED_BROADCAST) {
                if (fusedKernelsOnly) {
                    throw std::runtime_error(
                        "FusedEquation::run() only supports expressions that lower to fused kernels; this expression has a segmented stage. "
                        "Use stamp() and run the returned plan.");
                }
                if (isSegmentedReduceOp(n.op) && graph->role[n.lhs] == Role::Inline) {
                    if (stampSegmentedReductionOfExpression(i)) continue;
                    emitFusedGroup({n.lhs});  // operands the reduction cannot evaluate by itself: store the values first
                }
                if (stageFusion && stampSegmentSoftmaxStatistics(i)) continue;
                const Tensor& values = tensorOf[n.lhs];
                const Tensor& offsets = tensorOf[n.rhs];
                Tensor output = allocateFor(i);
                StampedExecutionStage stage;
                stage.gpu_num = device_num;
                stage.dependency_stage_indices = dependenciesOf({n.lhs, n.rhs});
                if (n.op == ExprOp::SEGMENTED_BROADCAST) {
                    stage.kind = StampedExecutionStage::Kind::SegmentedBroadcast;
                    stage.segmented_broadcast = stampSegmentedBroadcast(values, offsets, output, n.segmented_broadcast_normalize_by_length, stream);
                } else {
                    const CubReductionOp op = n.op == ExprOp::SEGMENTED_REDUCE_SUM   ? CubReductionOp::Sum
                                              : n.op == ExprOp::SEGMENTED_REDUCE_MIN ? CubReductionOp::Min
                                              : n.op == ExprOp::SEGMENTED_REDUCE_MAX ? CubReductionOp::Max
                                                                                     : CubReductionOp::Mean;
                    stage.kind = StampedExecutionStage::Kind::SegmentedReduction;
                    // the partition is read on the device every time the plan runs: nothing about it is fixed here
                    stage.segmented_reduction = std::make_shared<StampedSegmentedReductionStage>(
                        CubSegmentedReduction(op, n.output_dtype.value()).stampRuntimeOffsets(values, output, offsets, stream));
                }
                tensorOf[i] = output;
                stageOfNode[i] = static_cast<int>(stages.size());
                stages.push_back(std::move(stage));
                done[i] = 1;
                continue;
            }
            if (isScanOp(n.op)) {
                if (fusedKernelsOnly) {
                    throw std::runtime_error(
                        "FusedEquation::run() only supports expressions that lower to fused kernels; this expression has a scan stage. "
                        "Use stamp() and run the returned plan.");
                }
                const Tensor& values = tensorOf[n.lhs];
                if (!values.isDenseContiguous()) throw std::runtime_error("Expression scan needs a dense operand.");
                Tensor scanned = allocateFor(i);
                ScanRequest request;
                request.dtype = values.getDataType();
                request.total = values.getTotalNumElements();
                request.deviceNum = device_num;
                const bool arg = isArgScanOp(n.scan_op);
                request.op = arg ? (n.scan_op == ScanOp::ArgMin ? 1 : 2) : static_cast<int>(n.scan_op);
                request.writeValue = !arg;
                request.writeIndex = arg;
                // a min / max scan and the arg scan of the same operand (scanWithIndices) are one pass with two outputs
                uint32_t partner = UINT32_MAX;
                if (request.op == 1 || request.op == 2) {
                    const ScanOp wanted = arg ? (request.op == 1 ? ScanOp::Min : ScanOp::Max) : (request.op == 1 ? ScanOp::ArgMin : ScanOp::ArgMax);
                    for (uint32_t j = i + 1; j < expr.nodes.size() && partner == UINT32_MAX; ++j) {
                        const ExprNode& m = expr.nodes[j];
                        if (!done[j] && graph->role[j] == Role::Materialized && levelOf[j] == level && m.op == n.op && m.lhs == n.lhs && m.rhs == n.rhs &&
                            m.scan_op == wanted && m.scan_mode == n.scan_mode && m.scan_reverse == n.scan_reverse) {
                            partner = j;
                        }
                    }
                }
                Tensor partnerOutput;
                if (partner != UINT32_MAX) {
                    partnerOutput = allocateFor(partner);
                    request.writeValue = request.writeIndex = true;
                }
                request.inclusive = n.scan_mode == ScanMode::Inclusive;
                request.reverse = n.scan_reverse;
                request.alignmentBytes = std::min(pointerAlignment(values.getMemPtr()), pointerAlignment(scanned.getMemPtr()));
                if (partner != UINT32_MAX) request.alignmentBytes = std::min(request.alignmentBytes, pointerAlignment(partnerOutput.getMemPtr()));
                std::optional<Tensor> offsets;
                std::vector<uint32_t> stageSources{n.lhs};
                if (n.op == ExprOp::SEGMENTED_SCAN) {
                    offsets = tensorOf[n.rhs];
                    if (!offsets->isDenseContiguous()) throw std::runtime_error("Segmented scan needs dense offsets.");
                    request.row = 0;
                    request.segments = offsets->getTotalNumElements() - 1;
                    request.offsets64 = offsets->getDataType() == DataType::UINT64;
                    stageSources.push_back(n.rhs);
                } else {
                    request.row = dims[n.lhs].back();
                    request.segments = request.total / request.row;
                }
                const std::shared_ptr<const CubScanKernels> kernels = buildScanKernels(request);
                Tensor temp(gpuPlacement, TensorDescriptor(DataType::UINT8, {std::max<uint64_t>(kernels->tempBytes, 1)}));
                StampedExecutionStage stage;
                stage.kind = StampedExecutionStage::Kind::Scan;
                stage.gpu_num = device_num;
                stage.dependency_stage_indices = dependenciesOf(stageSources);
                if (partner != UINT32_MAX) {
                    stage.scan = std::make_shared<StampedScan>(kernels, values, offsets, temp, arg ? partnerOutput : scanned, arg ? scanned : partnerOutput);
                    tensorOf[partner] = partnerOutput;
                    stageOfNode[partner] = static_cast<int>(stages.size());
                    done[partner] = 1;
                } else {
                    stage.scan = std::make_shared<StampedScan>(kernels, values, offsets, temp, scanned, arg);
                }
                tensorOf[i] = scanned;
                stageOfNode[i] = static_cast<int>(stages.size());
                stages.push_back(std::move(stage));
                done[i] = 1;
                continue;
            }
            if (n.op == ExprOp::STRIDED_VIEW_BACKWARD) {
                const Tensor& gradient = tensorOf[n.lhs];
                if (!gradient.isDenseContiguous()) throw std::runtime_error("Strided view backward needs a dense gradient.");
                Tensor routed = allocateFor(i);
                StampedExecutionStage clearStage;
                clearStage.kind = StampedExecutionStage::Kind::FusedKernel;
                clearStage.gpu_num = device_num;
                clearStage.kernel = stampScatterClear(routed, device_num);
                const uint32_t clearIndex = static_cast<uint32_t>(stages.size());
                stages.push_back(std::move(clearStage));
                StampedExecutionStage placeStage;
                placeStage.kind = StampedExecutionStage::Kind::FusedKernel;
                placeStage.gpu_num = device_num;
                placeStage.dependency_stage_indices = dependenciesOf({n.lhs});
                placeStage.dependency_stage_indices.push_back(clearIndex);
                placeStage.kernel = stampViewScatter(gradient, routed, n.view_dims, n.view_strides, n.view_element_offset, device_num);
                tensorOf[i] = routed;
                stageOfNode[i] = static_cast<int>(stages.size());
                stages.push_back(std::move(placeStage));
                done[i] = 1;
                continue;
            }
            if (isSegmentWinnerRoutingOp(n.op)) {
                if (fusedKernelsOnly) {
                    throw std::runtime_error(
                        "FusedEquation::run() only supports expressions that lower to fused kernels; this expression has a reduction stage. "
                        "Use stamp() and run the returned plan.");
                }
                // the row that won every (segment, column), as a flattened index into the values; then each segment's gradient added
                // into that element of a cleared FP32 tensor (destinations are distinct, so nothing is actually summed)
                const Tensor& values = tensorOf[n.lhs];
                const Tensor& gradient = tensorOf[n.rhs];
                const Tensor& offsets = tensorOf[n.aux];
                if (!values.isDenseContiguous() || !gradient.isDenseContiguous() || !offsets.isDenseContiguous()) {
                    throw std::runtime_error("Segmented min/max backward needs dense operands.");
                }
                if (values.getTotalNumElements() >= 0xffffffffull) throw std::runtime_error("Segmented min/max backward: UINT32 winners cannot address this many values.");
                Tensor winners(gpuPlacement, TensorDescriptor(DataType::UINT32, gradient.getDimensions()));
                const CubSegmentedArgReduction find(n.op == ExprOp::SEGMENTED_REDUCE_MAX_BACKWARD ? CubArgReductionOp::ArgMax : CubArgReductionOp::ArgMin, DataType::UINT32);
                StampedExecutionStage findStage;
                findStage.kind = StampedExecutionStage::Kind::SegmentedReduction;
                findStage.gpu_num = device_num;
                findStage.dependency_stage_indices = dependenciesOf({n.lhs, n.aux});
                findStage.segmented_arg_reduction = find.stampRuntimeOffsets(values, winners, offsets, stream);
                const uint32_t findIndex = static_cast<uint32_t>(stages.size());
                stages.push_back(std::move(findStage));
                Tensor routed = allocateFor(i);
                StampedExecutionStage clearStage;
                clearStage.kind = StampedExecutionStage::Kind::FusedKernel;
                clearStage.gpu_num = device_num;
                clearStage.kernel = stampScatterClear(routed, device_num);
                const uint32_t clearIndex = static_cast<uint32_t>(stages.size());
                stages.push_back(std::move(clearStage));
                StampedExecutionStage addStage;
                addStage.kind = StampedExecutionStage::Kind::FusedKernel;
                addStage.gpu_num = device_num;
                addStage.dependency_stage_indices = dependenciesOf({n.rhs});
                addStage.dependency_stage_indices.push_back(findIndex);
                addStage.dependency_stage_indices.push_back(clearIndex);
                addStage.kernel = stampScatterAdd(gradient, winners, routed, std::nullopt, device_num);
                tensorOf[i] = routed;
                stageOfNode[i] = static_cast<int>(stages.size());
                stages.push_back(std::move(addStage));
                done[i] = 1;
                continue;
            }
            if (isScanBackwardOp(n.op)) {
                if (fusedKernelsOnly) {
                    throw std::runtime_error(
                        "FusedEquation::run() only supports expressions that lower to fused kernels; this expression has a scan stage. "
                        "Use stamp() and run the returned plan.");
                }
                // which element held the running minimum / maximum at every position (an arg scan), then every position's gradient
                // added into that element of a cleared FP32 tensor
                const Tensor& values = tensorOf[n.lhs];
                const Tensor& gradient = tensorOf[n.rhs];
                if (!values.isDenseContiguous() || !gradient.isDenseContiguous()) throw std::runtime_error("Scan min/max backward needs dense operands.");
                const bool segmented = n.aux != UINT32_MAX;
                Tensor winners(gpuPlacement, TensorDescriptor(DataType::UINT32, values.getDimensions()));
                ScanRequest request;
                request.dtype = values.getDataType();
                request.total = values.getTotalNumElements();
                request.deviceNum = device_num;
                request.op = (n.op == ExprOp::SCAN_MIN_BACKWARD || n.op == ExprOp::SEGMENTED_SCAN_MIN_BACKWARD) ? 1 : 2;
                request.writeValue = false;
                request.writeIndex = true;
                request.inclusive = n.scan_mode == ScanMode::Inclusive;
                request.reverse = n.scan_reverse;
                request.alignmentBytes = std::min(pointerAlignment(values.getMemPtr()), pointerAlignment(winners.getMemPtr()));
                std::optional<Tensor> offsets;
                std::vector<uint32_t> scanSources{n.lhs};
                if (segmented) {
                    offsets = tensorOf[n.aux];
                    if (!offsets->isDenseContiguous()) throw std::runtime_error("Segmented scan needs dense offsets.");
                    request.row = 0;
                    request.segments = offsets->getTotalNumElements() - 1;
                    request.offsets64 = offsets->getDataType() == DataType::UINT64;
                    scanSources.push_back(n.aux);
                } else {
                    request.row = dims[n.lhs].back();
                    request.segments = request.total / request.row;
                }
                if (!segmented && gradient.getDataType() == DataType::FP32 && n.output_dtype.value() == DataType::FP32) {
                    // rows that fit one block: winners, the sums of the gradient over the positions each of them won, and the
                    // gradient of the operand in one launch (every element is written, so nothing is cleared first)
                    Tensor routed = allocateFor(i);
                    ScanRequest oneLaunch = request;
                    oneLaunch.route = true;
                    oneLaunch.alignmentBytes = std::min({pointerAlignment(values.getMemPtr()), pointerAlignment(gradient.getMemPtr()), pointerAlignment(routed.getMemPtr())});
                    if (scanRouteFits(oneLaunch)) {
                        StampedExecutionStage routeStage;
                        routeStage.kind = StampedExecutionStage::Kind::Scan;
                        routeStage.gpu_num = device_num;
                        routeStage.dependency_stage_indices = dependenciesOf({n.lhs, n.rhs});
                        routeStage.scan = std::make_shared<StampedScan>(StampedScan::routing(buildScanKernels(oneLaunch), values, gradient, routed));
                        tensorOf[i] = routed;
                        stageOfNode[i] = static_cast<int>(stages.size());
                        stages.push_back(std::move(routeStage));
                        done[i] = 1;
                        continue;
                    }
                }
                const std::shared_ptr<const CubScanKernels> kernels = buildScanKernels(request);
                Tensor temp(gpuPlacement, TensorDescriptor(DataType::UINT8, {std::max<uint64_t>(kernels->tempBytes, 1)}));
                StampedExecutionStage scanStage;
                scanStage.kind = StampedExecutionStage::Kind::Scan;
                scanStage.gpu_num = device_num;
                scanStage.dependency_stage_indices = dependenciesOf(scanSources);
                scanStage.scan = std::make_shared<StampedScan>(kernels, values, offsets, temp, winners, /*indexOutput=*/true);
                const uint32_t scanIndex = static_cast<uint32_t>(stages.size());
                stages.push_back(std::move(scanStage));
                Tensor routed = allocateFor(i);
                StampedExecutionStage clearStage;
                clearStage.kind = StampedExecutionStage::Kind::FusedKernel;
                clearStage.gpu_num = device_num;
                clearStage.kernel = stampScatterClear(routed, device_num);
                const uint32_t clearIndex = static_cast<uint32_t>(stages.size());
                stages.push_back(std::move(clearStage));
                StampedExecutionStage addStage;
                addStage.kind = StampedExecutionStage::Kind::FusedKernel;
                addStage.gpu_num = device_num;
                addStage.dependency_stage_indices = dependenciesOf({n.rhs});
                addStage.dependency_stage_indices.push_back(scanIndex);
                addStage.dependency_stage_indices.push_back(clearIndex);
                addStage.kernel = stampScatterAdd(gradient, winners, routed, offsets, device_num);
                tensorOf[i] = routed;
                stageOfNode[i] = static_cast<int>(stages.size());
                stages.push_back(std::move(addStage));
                done[i] = 1;
                continue;
            }
            if (n.op == ExprOp::ROPE) {
                const std::vector<uint64_t> shape = orScalarShape(dims[i]);
                RopeFusion fusion;
                std::vector<uint32_t> operands;
                // Elementwise statements for `root` over tensors of the rotated shape (placeholders "@<tag><index>@" stand for their
                // loaded elements), runtime scalars and, in an epilogue, the rotated value.  False: something else is involved.
                auto buildPiece = [&](uint32_t root, bool epilogue, RopeFusion::Piece& piece, std::vector<uint32_t>& pieceSources) -> bool {
                    std::vector<uint32_t> sources, scalarSlots;
                    collectSources(*graph, root, sources, scalarSlots);
                    BodyEmitter body(expr);
                    std::string text;
                    bool readsRotation = false;
                    for (uint32_t source : sources) {
                        if (epilogue && source == i) {
                            body.defineSource(i, n.output_dtype.value(), "@R@");
                            readsRotation = true;
                            continue;
                        }
                        const Tensor& t = tensorOf[source];
                        if (!done[source] && expr.nodes[source].op != ExprOp::INPUT && graph->role[source] != Role::InputSource) return false;
                        if (!t.isInitialized() || !t.isDenseContiguous() || t.getDimensions() != shape) return false;
                        const DataType valueDType = expr.nodes[source].output_dtype.value();
                        const std::string raw = std::string("@") + (epilogue ? "E" : "P") + std::to_string(piece.tensors.size()) + "@";
                        text += "const " + std::string(valueCType(valueDType)) + " t" + std::to_string(source) + " = " +
                                castValueExpr(storageToValueExpr(raw, t.getDataType()), t.getDataType(), valueDType) + ";\n";
                        body.defineSource(source, valueDType);
                        piece.tensors.push_back(t);
                        pieceSources.push_back(source);
                    }
                    if (epilogue && !readsRotation) return false;
                    if (piece.tensors.empty() && !epilogue) return false;
                    piece.contract = true;
                    for (uint32_t v : body.collect({root})) {
                        const ExprNode& node = expr.nodes[v];
                        const bool elementwise = Expression::isBinaryOp(node.op) || node.op == ExprOp::WHERE || node.op == ExprOp::CAST ||
                                                 node.op == ExprOp::RUNTIME_SCALAR || node.op == ExprOp::SCALAR_FP ||
                                                 (Expression::isUnaryOp(node.op) && !isReductionOp(node.op) && !isShapeOnly(node.op) && node.op != ExprOp::SOFTMAX);
                        if (!elementwise) return false;
                        const DataType c = emittedValueDType(node);
                        if (c == DataType::FP16 || c == DataType::BF16) piece.contract = false;
                        fusion.extraFlopsPerElement += body.emit(text, v, "");
                    }
                    piece.statements = text;
                    const DataType stored = expr.nodes[root].output_dtype.value();
                    piece.value = epilogue ? valueToStorageExpr(body.ref(root, stored), stored) : castValueExpr(body.ref(root, stored), stored, DataType::FP32);
                    for (uint32_t slot : scalarSlots) {
                        if (std::find(fusion.scalarSlots.begin(), fusion.scalarSlots.end(), slot) == fusion.scalarSlots.end()) {
                            fusion.scalarSlots.push_back(slot);
                            fusion.scalarNames.push_back(root_inputs.at(slot).name);
                        }
                    }
                    return true;
                };
                // the operand: a tensor, or elementwise work the planner left to this kernel
                Tensor shapeCarrier;
                if (graph->role[n.lhs] == Role::Inline) {
                    RopeFusion saved = fusion;
                    RopeFusion::Piece piece;
                    std::vector<uint32_t> pieceSources;
                    if (stageFusion && buildPiece(n.lhs, false, piece, pieceSources)) {
                        fusion.operandDType = expr.nodes[n.lhs].output_dtype.value();
                        shapeCarrier = piece.tensors.front();
                        fusion.prologue = std::move(piece);
                        operands = pieceSources;
                    } else {
                        fusion = saved;
                        emitFusedGroup({n.lhs});  // store the operand first
                    }
                }
                if (!fusion.prologue.has_value()) {
                    operands = {n.lhs};
                    shapeCarrier = tensorOf[n.lhs];
                }
                if (n.rhs != UINT32_MAX) operands.push_back(n.rhs);
                if (n.aux != UINT32_MAX) operands.push_back(n.aux);
                // the consumer: when one elementwise value (of this shape, nothing else unfinished under it) is all that reads the
                // rotation, this kernel computes and stores that value instead
                uint32_t stored = i;
                if (stageFusion && outputNameOfNode.find(i) == outputNameOfNode.end()) {
                    uint32_t reader = UINT32_MAX;
                    bool single = true;
                    for (uint32_t j = 0; j < expr.nodes.size() && single; ++j) {
                        if (j == i || !isTensorRole(graph->role[j]) || done[j]) continue;
                        const ExprNode& candidate = expr.nodes[j];
                        std::vector<uint32_t> sources, scalars;
                        if (runsInFusedKernel(j)) {
                            collectSources(*graph, j, sources, scalars);
                        } else {
                            for (uint32_t c : {candidate.lhs, candidate.rhs, candidate.aux})
                                if (c != UINT32_MAX) sources.push_back(c);
                            // (a value an inline operand of another stage reads also counts as read by that stage)
                            std::vector<uint32_t> deeper;
                            for (uint32_t c : sources)
                                if (graph->role[c] == Role::Inline) collectSources(*graph, c, deeper, scalars);
                            sources.insert(sources.end(), deeper.begin(), deeper.end());
                        }
                        if (std::find(sources.begin(), sources.end(), i) == sources.end()) continue;
                        if (reader != UINT32_MAX || !runsInFusedKernel(j) || candidate.op == ExprOp::RAGGED_VALUEWISE_EXTENT || orScalarShape(dims[j]) != shape) {
                            single = false;
                        } else {
                            reader = j;
                        }
                    }
                    if (single && reader != UINT32_MAX) {
                        RopeFusion saved = fusion;
                        RopeFusion::Piece piece;
                        std::vector<uint32_t> pieceSources;
                        if (buildPiece(reader, true, piece, pieceSources)) {
                            fusion.rotatedDType = n.output_dtype.value();
                            fusion.epilogue = std::move(piece);
                            operands.insert(operands.end(), pieceSources.begin(), pieceSources.end());
                            stored = reader;
                        } else {
                            fusion = saved;
                        }
                    }
                }
                Tensor result = allocateFor(stored);
                StampedExecutionStage stage;
                stage.kind = StampedExecutionStage::Kind::FusedKernel;
                stage.gpu_num = device_num;
                stage.dependency_stage_indices = dependenciesOf(operands);
                stage.kernel = stampRotaryEmbedding(shapeCarrier, n.rhs != UINT32_MAX ? std::optional<Tensor>(tensorOf[n.rhs]) : std::nullopt,
                                                    n.aux != UINT32_MAX ? std::optional<Tensor>(tensorOf[n.aux]) : std::nullopt, result, n, device_num, fusion);
                tensorOf[stored] = result;
                stageOfNode[stored] = static_cast<int>(stages.size());
                stageOfNode[i] = static_cast<int>(stages.size());
                stages.push_back(std::move(stage));
                done[i] = 1;
                done[stored] = 1;
                continue;
            }
            if (n.op == ExprOp::TAKE_ALONG_AXIS) {
                const uint64_t rank = dims[n.lhs].size();
                const uint64_t axis = n.reduction_axes.empty() || n.reduction_axes.front() == UINT64_MAX ? rank - 1 : n.reduction_axes.front();
                if (axis >= rank) throw std::runtime_error("take_along_axis axis is out of range for the input rank.");
                Tensor gathered = allocateFor(i);
                StampedExecutionStage stage;
                stage.kind = StampedExecutionStage::Kind::FusedKernel;
                stage.gpu_num = device_num;
                stage.dependency_stage_indices = dependenciesOf({n.lhs, n.rhs});
                stage.kernel = stampTakeAlongAxis(tensorOf[n.lhs], tensorOf[n.rhs], gathered, axis, device_num);
                tensorOf[i] = gathered;
                stageOfNode[i] = static_cast<int>(stages.size());
                stages.push_back(std::move(stage));
                done[i] = 1;
                continue;
            }
            if (isWinnerRoutingOp(n.op)) {
                if (fusedKernelsOnly) {
                    throw std::runtime_error(
                        "FusedEquation::run() only supports expressions that lower to fused kernels; this expression has a reduction stage. "
                        "Use stamp() and run the returned plan.");
                }
                // winners of the forward reduction (an index per window), then one pass that spreads the gradient
                const Tensor& operand = tensorOf[n.lhs];
                const std::vector<uint64_t> axes64 = sortedAxesOrAll(n.reduction_axes, dims[n.lhs].size());
                std::vector<uint32_t> axes(axes64.begin(), axes64.end());
                CubArgReductionOutputOptions options;
                options.produce_value = false;
                options.produce_index = true;
                options.index_output_dtype = DataType::UINT32;
                const CubArgReduction reduction(n.op == ExprOp::REDUCE_MAX_BACKWARD ? CubArgReductionOp::ArgMax : CubArgReductionOp::ArgMin, axes, options);
                Tensor winners(gpuPlacement, TensorDescriptor(DataType::UINT32, StampedEquation::computeReductionOutputDims(dims[n.lhs], axes64, {})));
                StampedExecutionStage find;
                find.kind = StampedExecutionStage::Kind::ArgMinMax;
                find.gpu_num = device_num;
                find.dependency_stage_indices = dependenciesOf({n.lhs});
                find.arg_minmax = std::make_shared<StampedArgMinMax>(reduction.stamp(operand, std::nullopt, winners, stream));
                const uint32_t findStage = static_cast<uint32_t>(stages.size());
                stages.push_back(std::move(find));

                Tensor gradient = tensorOf[n.rhs];
                if (!gradient.isDenseContiguous()) throw std::runtime_error("Min/max reduction backward needs a dense gradient tensor.");
                Tensor routed = allocateFor(i);
                StampedExecutionStage spread;
                spread.kind = StampedExecutionStage::Kind::ReduceMinMaxBackward;
                spread.gpu_num = device_num;
                spread.dependency_stage_indices = dependenciesOf({n.rhs});
                spread.dependency_stage_indices.push_back(findStage);
                std::sort(spread.dependency_stage_indices.begin(), spread.dependency_stage_indices.end());
                spread.kernel = stampWinnerRouting(winners, gradient, routed, dims[n.lhs], axes64, device_num);
                tensorOf[i] = routed;
                stageOfNode[i] = static_cast<int>(stages.size());
                stages.push_back(std::move(spread));
                done[i] = 1;
                continue;
            }
            if (!isReductionOp(n.op)) {
                fusedGroups[groupKeyOf(i)].push_back(i);
                continue;
            }
            if (fusedKernelsOnly) {
                throw std::runtime_error(
                    "FusedEquation::run() only supports expressions that lower to fused kernels; this expression has a reduction stage. "
                    "Use stamp() and run the returned plan.");
            }
            const Tensor& input = tensorOf[n.lhs];
            std::vector<uint32_t> axes;
            for (uint64_t a : sortedAxesOrAll(n.reduction_axes, dims[n.lhs].size())) axes.push_back(static_cast<uint32_t>(a));
            Tensor output = allocateFor(i);
            StampedExecutionStage stage;
            stage.gpu_num = device_num;
            stage.dependency_stage_indices = dependenciesOf({n.lhs});
            if (isArgReductionOp(n.op)) {
                CubArgReductionOutputOptions options;
                options.produce_value = false;
                options.produce_index = true;
                options.index_output_dtype = n.output_dtype.value();
                const CubArgReduction reduction(n.op == ExprOp::REDUCE_ARGMAX ? CubArgReductionOp::ArgMax : CubArgReductionOp::ArgMin, axes, options);
                stage.kind = StampedExecutionStage::Kind::ArgMinMax;
                stage.arg_minmax = std::make_shared<StampedArgMinMax>(reduction.stamp(input, std::nullopt, output, stream));
            } else {
                const CubReduction reduction(valueReductionOp(n.op), axes, n.output_dtype.value());
                stage.kind = StampedExecutionStage::Kind::Reduction;
                stage.reduction = std::make_shared<StampedReduction>(reduction.stamp(input, output, stream));
            }
            tensorOf[i] = output;
            stageOfNode[i] = static_cast<int>(stages.size());
            stages.push_back(std::move(stage));
            done[i] = 1;
        }

        for (auto& [groupKey, nodes] : fusedGroups) emitFusedGroup(nodes);
        resolveViewsUpTo();
    }

    // ---- final outputs ---------------------------------------------------------------------------------------------------
    std::unordered_map<std::string, Tensor> finalOutputs;
    for (const NamedOutput& o : graph->outputs) {
        Tensor produced = tensorOf[o.node_idx];
        if (!produced.isInitialized()) throw std::logic_error("Output '" + o.name + "' was not produced by any stage.");
        auto pre = preallocated.find(o.name);
        if (pre != preallocated.end() && pre->second != produced && pre->second.getMemPtr() != produced.getMemPtr()) {
            // the value lives elsewhere (an input, a view, or another name's tensor): copy it into the caller's tensor
            if (pre->second.getTotalNumElements() != produced.getTotalNumElements() || pre->second.getDataType() != produced.getDataType()) {
                throw std::runtime_error("Preallocated output '" + o.name + "' does not match the shape or dtype the expression produces.");
            }
            StampedExecutionStage copy;
            copy.kind = StampedExecutionStage::Kind::Copy;
            copy.gpu_num = device_num;
            copy.copySource = produced;
            copy.copyDestination = pre->second;
            const int st = stageOfNode[baseOfView(*graph, o.node_idx)];
            if (st >= 0) copy.dependency_stage_indices.push_back(static_cast<uint32_t>(st));
            stages.push_back(std::move(copy));
            produced = pre->second;
        }
        auto requested = requestedOutputShapes.find(o.name);
        if (requested != requestedOutputShapes.end() && !requested->second.empty()) {
            if (!sameDimensionsIgnoringSingletons(produced.getDimensions(), requested->second)) {
                throw std::runtime_error("Output tensor dimensions are incompatible with the fused equation result.");
            }
            // a caller's own tensor keeps its dimensions; a tensor allocated here is handed out with the requested ones
            if (pre == preallocated.end() && produced.isDenseContiguous() && produced.getDimensions() != requested->second) produced.reshape(requested->second);
        }
        finalOutputs.emplace(o.name, produced);
    }
    for (const auto& [name, shape] : requestedOutputShapes) {
        if (!shape.empty() && finalOutputs.find(name) == finalOutputs.end()) throw std::runtime_error("Requested output shape names '" + name + "', which is not an output of this equation.");
    }
    return StampedExecutionPlan(std::move(stages), std::move(finalOutputs), stream);
}

// ---- backward equations -------------------------------------------------------------------------------------------------------------
struct FusedEquation::BackwardRecipe {
    PhysicalOutputs forward;
    std::vector<std::string> wrt;
    std::optional<std::unordered_map<std::string, std::string>> upstreamByOutput;
    bool accumulate = false;
    // shapes and dtypes of the forward inputs -> the equation differentiated for them
    LruCacheThreadSafe<std::string, std::shared_ptr<const FusedEquation>> specialised{64};
};

FusedEquation::FusedEquation(std::shared_ptr<BackwardRecipe> recipe, int device_num)
    : backward(std::move(recipe)),
      device_num(device_num),
      planned_graph_cache(std::make_shared<LruCacheThreadSafe<std::string, std::shared_ptr<PlannedGraph>>>(1)) {
    // what may be bound: the forward inputs, the upstream gradients and the running gradients; what is produced
    root_inputs = backward->forward.expr->inputs;
    auto addInput = [&](const std::string& name) {
        for (const NamedInput& in : root_inputs)
            if (in.name == name) return;
        root_inputs.push_back(NamedInput{name, static_cast<uint32_t>(root_inputs.size()), NamedInput::Kind::Tensor});
    };
    if (backward->upstreamByOutput.has_value()) {
        for (const NamedOutput& o : backward->forward.outputs) {
            auto it = backward->upstreamByOutput->find(o.name);
            if (it != backward->upstreamByOutput->end()) addInput(it->second);
        }
    }
    for (const std::string& name : backward->wrt) {
        if (backward->accumulate) addInput(name + "_grad");
        outputs_template.outputs.push_back(NamedOutput{name + "_grad", UINT32_MAX});
    }
}

FusedEquation FusedEquation::compileBackward(const std::vector<std::string>& wrt_names, const std::optional<std::string>& upstream_input_name,
                                             bool accumulate_grad_outputs) const {
    if (backward) throw std::runtime_error("compileBackward of a backward equation is not supported.");
    auto recipe = std::make_shared<BackwardRecipe>();
    recipe->forward = outputs_template;
    recipe->wrt = normalizeBackwardWrtNames(*outputs_template.expr, wrt_names);
    recipe->upstreamByOutput = normalizeBackwardUpstreamNames(outputs_template, upstream_input_name);
    recipe->accumulate = accumulate_grad_outputs;
    if (outputs_template.outputs.size() > 1 && !recipe->upstreamByOutput.has_value()) {
        throw std::runtime_error(
            "buildBackwardOutputs for multi-output forward equations requires an explicit upstream seed map. The map may be partial when "
            "some outputs have no incoming gradient.");
    }
    return FusedEquation(std::move(recipe), device_num);
}

FusedEquation FusedEquation::compileBackward(const std::vector<std::string>& wrt_names,
                                             const std::unordered_map<std::string, std::string>& upstream_input_names_by_output,
                                             bool accumulate_grad_outputs) const {
    if (backward) throw std::runtime_error("compileBackward of a backward equation is not supported.");
    auto recipe = std::make_shared<BackwardRecipe>();
    recipe->forward = outputs_template;
    recipe->wrt = normalizeBackwardWrtNames(*outputs_template.expr, wrt_names);
    recipe->upstreamByOutput = normalizeBackwardUpstreamNames(outputs_template, upstream_input_names_by_output);
    if (recipe->upstreamByOutput->empty()) {
        throw std::runtime_error("buildBackwardOutputs explicit upstream seed map must contain at least one forward output.");
    }
    recipe->accumulate = accumulate_grad_outputs;
    return FusedEquation(std::move(recipe), device_num);
}

std::shared_ptr<const FusedEquation> FusedEquation::backwardFor(const std::unordered_map<std::string, Tensor>& inputs,
                                                                std::unordered_map<std::string, Tensor>& used) const {
    const PhysicalExpression& forward = *backward->forward.expr;
    for (const auto& [name, tensor] : inputs) {
        (void)tensor;
        bool known = false;
        for (const NamedInput& in : root_inputs) known = known || in.name == name;
        if (!known) throw std::runtime_error("Unexpected input tensor for this equation: " + name);
    }
    // the forward inputs fix the shapes and dtypes the gradients are built for
    std::string key;
    std::vector<DataType> dtypes(forward.inputs.size(), DataType::FP32);
    std::unordered_map<std::string, std::vector<uint64_t>> dimsByName;
    for (const NamedInput& in : forward.inputs) {
        if (in.kind == NamedInput::Kind::RuntimeScalarFp32) continue;
        auto it = inputs.find(in.name);
        if (it == inputs.end()) throw std::runtime_error("Missing required input tensor: " + in.name);
        if (!it->second.isInitialized()) throw std::runtime_error("Input tensor is not initialized: " + in.name);
        dtypes[in.slot] = it->second.getDataType();
        dimsByName[in.name] = it->second.getDimensions();
        key += in.name + ":" + std::to_string(static_cast<int>(dtypes[in.slot])) + ":" + axesKey(it->second.getDimensions()) + ";";
    }
    const std::shared_ptr<const FusedEquation> equation = backward->specialised.getOrCreate(key, [&] {
        PhysicalOutputs typed;
        typed.expr = std::make_shared<PhysicalExpression>(forward);
        typed.outputs = backward->forward.outputs;
        resolveOutputsDTypesInPlace(typed, dtypes);
        const PhysicalOutputs gradients =
            buildBackwardOutputsTyped(backward->forward, *typed.expr, backward->wrt, backward->upstreamByOutput, dimsByName, backward->accumulate);
        return std::shared_ptr<const FusedEquation>(new FusedEquation(compile(gradients, device_num)));
    });
    for (const NamedInput& in : equation->root_inputs) {
        if (in.kind == NamedInput::Kind::RuntimeScalarFp32) continue;
        auto it = inputs.find(in.name);
        if (it == inputs.end()) throw std::runtime_error("Missing required input tensor: " + in.name);
        used.emplace(in.name, it->second);
    }
    return equation;
}

// ---- convenience run ---------------------------------------------------------------------------------------------------------------
void FusedEquation::run(const Tensor& input, Tensor& output, Stream& stream) const {
    if (root_inputs.size() != 1) throw std::runtime_error("run(input, output) requires an equation with exactly one input.");
    run(std::unordered_map<std::string, Tensor>{{root_inputs[0].name, input}}, output, stream);
}

void FusedEquation::run(const std::unordered_map<std::string, Tensor>& inputs, Tensor& output, Stream& stream) const {
    run(inputs, std::unordered_map<std::string, float>{}, output, stream);
}

void FusedEquation::run(const std::unordered_map<std::string, Tensor>& inputs, const std::unordered_map<std::string, float>& scalar_inputs,
                        Tensor& output, Stream& stream) const {
    if (outputs_template.outputs.size() != 1) throw std::runtime_error("run(..., output) requires an equation with exactly one output.");
    std::unordered_map<std::string, Tensor> outputs{{outputs_template.outputs[0].name, output}};
    run(inputs, scalar_inputs, outputs, stream);
}

void FusedEquation::run(const Tensor& input, std::unordered_map<std::string, Tensor>& outputs, Stream& stream) const {
    if (root_inputs.size() != 1) throw std::runtime_error("run(input, outputs) requires an equation with exactly one input.");
    run(std::unordered_map<std::string, Tensor>{{root_inputs[0].name, input}}, outputs, stream);
}

void FusedEquation::run(const std::unordered_map<std::string, Tensor>& inputs, std::unordered_map<std::string, Tensor>& outputs, Stream& stream) const {
    run(inputs, std::unordered_map<std::string, float>{}, outputs, stream);
}

void FusedEquation::run(const std::unordered_map<std::string, Tensor>& inputs, const std::unordered_map<std::string, float>& scalar_inputs,
                        std::unordered_map<std::string, Tensor>& outputs, Stream& stream) const {
    for (const NamedOutput& o : outputs_template.outputs) {
        if (!outputs.count(o.name)) throw std::runtime_error("Missing output tensor: " + o.name);
    }
    const StampedExecutionPlan plan = stampImpl(inputs, stream, outputs, true);
    for (const std::string& name : plan.runtimeScalarNames()) {
        if (!scalar_inputs.count(name)) throw std::runtime_error("Missing runtime scalar input: " + name);
    }
    plan.runOn(stream, scalar_inputs);
}

// ---- shape / dtype queries -----------------------------------------------------------------------------------------------------------
std::unordered_map<std::string, std::vector<uint64_t>> FusedEquation::getOutputShapes(const std::unordered_map<std::string, Tensor>& inputs) const {
    if (backward) {
        std::unordered_map<std::string, Tensor> used;
        const std::shared_ptr<const FusedEquation> equation = backwardFor(inputs, used);
        return equation->getOutputShapes(used);
    }
    const std::shared_ptr<PlannedGraph> graph = plannedGraphFor(rootDTypes(inputs));
    std::vector<Tensor> bound(root_inputs.size());
    for (const NamedInput& in : root_inputs)
        if (in.kind != NamedInput::Kind::RuntimeScalarFp32) bound[in.slot] = inputs.at(in.name);
    const std::vector<std::vector<uint64_t>> dims = inferShapes(*graph, bound);
    std::unordered_map<std::string, std::vector<uint64_t>> out;
    for (const NamedOutput& o : graph->outputs) out.emplace(o.name, orScalarShape(dims[o.node_idx]));
    return out;
}

std::unordered_map<std::string, std::vector<uint64_t>> FusedEquation::getOutputShapes(const Tensor& input) const {
    if (root_inputs.size() != 1) throw std::runtime_error("getOutputShapes(input) requires an equation with exactly one input.");
    return getOutputShapes(std::unordered_map<std::string, Tensor>{{root_inputs[0].name, input}});
}

std::vector<uint64_t> FusedEquation::getOutputShape(const std::unordered_map<std::string, Tensor>& inputs) const {
    if (outputs_template.outputs.size() != 1) throw std::runtime_error("getOutputShape requires an equation with exactly one output.");
    return getOutputShapes(inputs).begin()->second;
}

std::vector<uint64_t> FusedEquation::getOutputShape(const Tensor& input) const {
    if (outputs_template.outputs.size() != 1) throw std::runtime_error("getOutputShape requires an equation with exactly one output.");
    return getOutputShapes(input).begin()->second;
}

std::unordered_map<std::string, std::vector<uint64_t>> FusedEquation::getOutputShapes(
    const std::unordered_map<std::string, Tensor>& inputs, const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs) const {
    return getOutputShapes(withTensorScalars(inputs, tensor_scalar_inputs));
}
std::unordered_map<std::string, DataType> FusedEquation::getOutputDataTypes(
    const std::unordered_map<std::string, Tensor>& inputs, const std::unordered_map<std::string, TensorScalarBinding>& tensor_scalar_inputs) const {
    return getOutputDataTypes(withTensorScalars(inputs, tensor_scalar_inputs));
}

std::unordered_map<std::string, DataType> FusedEquation::getOutputDataTypes(const std::unordered_map<std::string, Tensor>& inputs) const {
    if (backward) {
        std::unordered_map<std::string, Tensor> used;
        const std::shared_ptr<const FusedEquation> equation = backwardFor(inputs, used);
        return equation->getOutputDataTypes(used);
    }
    const std::shared_ptr<PlannedGraph> graph = plannedGraphFor(rootDTypes(inputs));
    std::unordered_map<std::string, DataType> out;
    for (const NamedOutput& o : graph->outputs) out.emplace(o.name, graph->expr.nodes[o.node_idx].output_dtype.value());
    return out;
}

}  // namespace ThorImplementation
