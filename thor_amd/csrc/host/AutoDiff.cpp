// Reverse-mode differentiation of Expression graphs (behaviour of the reference: Utilities/Expression/AutoDiff.cpp:2486-2581
// name validation, :3690-3800 seeds, :4000-5075 per-op rules, :5790-5932 gradient outputs).
//
// One sweep over the forward nodes from last to first.  Every node that lies between a requested input and a seeded
// output owns an adjoint with exactly the node's shape; a rule turns it into contributions to the node's operands, each
// summed back to the operand's shape where the forward op broadcast it.  Forward values the rules need are copied into
// the backward graph once.
#include "Utilities/Expression/AutoDiff.h"

#include "AutoDiffInternal.h"
#include "ShapeInference.h"

#include <algorithm>
#include <cmath>
#include <stdexcept>
#include <unordered_set>

namespace ThorImplementation {

namespace {

typedef std::vector<uint64_t> Dims;
constexpr uint32_t kNone = UINT32_MAX;

uint64_t elementCount(const Dims& d) {
    uint64_t n = 1;
    for (uint64_t x : d) n *= x;
    return n;
}

Dims broadcastOf(const Dims& a, const Dims& b) {
    const size_t rank = std::max(a.size(), b.size());
    Dims out(rank, 1);
    for (size_t i = 0; i < rank; ++i) {
        const uint64_t da = i < rank - a.size() ? 1 : a[i - (rank - a.size())];
        const uint64_t db = i < rank - b.size() ? 1 : b[i - (rank - b.size())];
        if (da != db && da != 1 && db != 1) throw std::runtime_error("Autodiff: gradient operands are not broadcast-compatible.");
        out[i] = std::max(da, db);
    }
    return out;
}

// The backward graph under construction: nodes are appended in dependency order and every node's shape is tracked.
class BackwardGraph {
   public:
    // shapeless: the caller gave no dimensions; no shape is tracked and nothing is expanded or summed back
    BackwardGraph(const PhysicalExpression& forward, const std::vector<Dims>& forwardDims, bool shapeless = false)
        : shapeless(shapeless), forward(forward), forwardDims(forwardDims) {}

    const bool shapeless;
    PhysicalExpression graph;
    std::vector<Dims> dims;

    const Dims& dimsOf(uint32_t node) const { return dims.at(node); }

    // forward value of node `f`, copied with everything it depends on (once)
    uint32_t value(uint32_t f) {
        auto known = copied.find(f);
        if (known != copied.end()) return known->second;
        std::vector<char> needed(f + 1, 0);
        needed[f] = 1;
        for (uint32_t i = f + 1; i-- > 0;) {
            if (!needed[i] || copied.count(i)) continue;
            const ExprNode& n = forward.nodes[i];
            for (uint32_t c : {n.lhs, n.rhs, n.aux})
                if (c != kNone) needed[c] = 1;
        }
        for (uint32_t i = 0; i <= f; ++i) {
            if (!needed[i] || copied.count(i)) continue;
            ExprNode copy = forward.nodes[i];
            if (copy.lhs != kNone) copy.lhs = copied.at(copy.lhs);
            if (copy.rhs != kNone) copy.rhs = copied.at(copy.rhs);
            if (copy.aux != kNone) copy.aux = copied.at(copy.aux);
            if (copy.input_slot != kNone) {
                const NamedInput& in = forward.inputs.at(copy.input_slot);
                copy.input_slot = graph.getOrCreateInputSlot(in.name, in.kind);
            }
            copied[i] = push(std::move(copy), forwardDims[i]);
        }
        return copied.at(f);
    }

    uint32_t scalar(double v) {
        ExprNode n;
        n.op = ExprOp::SCALAR_FP;
        n.scalar_fp = v;
        return push(std::move(n), {});
    }
    uint32_t fill(double v, const Dims& d, std::optional<DataType> dtype = std::nullopt) {
        ExprNode n;
        n.op = ExprOp::FILL;
        n.scalar_fp = v;
        n.fill_dims = d;
        n.output_dtype = dtype;
        return push(std::move(n), d);
    }
    uint32_t input(const std::string& name) {
        ExprNode n;
        n.op = ExprOp::INPUT;
        n.input_slot = graph.getOrCreateInputSlot(name, NamedInput::Kind::Tensor);
        return push(std::move(n), {});  // the caller sets the shape it expects
    }
    uint32_t unary(ExprOp op, uint32_t a) {
        ExprNode n;
        n.op = op;
        n.lhs = a;
        return push(std::move(n), dims[a]);
    }
    uint32_t binary(ExprOp op, uint32_t a, uint32_t b) {
        ExprNode n;
        n.op = op;
        n.lhs = a;
        n.rhs = b;
        return push(std::move(n), shapeless ? Dims{} : broadcastOf(dims[a], dims[b]));
    }
    uint32_t add(uint32_t a, uint32_t b) { return binary(ExprOp::ADD, a, b); }
    uint32_t sub(uint32_t a, uint32_t b) { return binary(ExprOp::SUB, a, b); }
    uint32_t mul(uint32_t a, uint32_t b) { return binary(ExprOp::MUL, a, b); }
    uint32_t div(uint32_t a, uint32_t b) { return binary(ExprOp::DIV, a, b); }
    uint32_t neg(uint32_t a) { return unary(ExprOp::NEG, a); }
    uint32_t scaled(uint32_t a, double factor) { return mul(a, scalar(factor)); }
    uint32_t where(uint32_t condition, uint32_t a, uint32_t b) {
        ExprNode n;
        n.op = ExprOp::WHERE;
        n.lhs = condition;
        n.rhs = a;
        n.aux = b;
        return push(std::move(n), broadcastOf(broadcastOf(dims[condition], dims[a]), dims[b]));
    }
    uint32_t cast(uint32_t a, DataType dtype) {
        ExprNode n;
        n.op = ExprOp::CAST;
        n.lhs = a;
        n.output_dtype = dtype;
        n.compute_dtype = dtype;
        return push(std::move(n), dims[a]);
    }
    uint32_t reshape(uint32_t a, const Dims& d) {
        if (dims[a] == d) return a;
        if (elementCount(dims[a]) != elementCount(d)) throw std::logic_error("Autodiff: reshape of a gradient changes its element count.");
        ExprNode n;
        n.op = ExprOp::RESHAPE;
        n.lhs = a;
        n.reshape_dims = d;
        return push(std::move(n), d);
    }
    uint32_t transpose(uint32_t a) {
        Dims d = dims[a];
        if (d.size() >= 2) std::swap(d[d.size() - 1], d[d.size() - 2]);
        ExprNode n;
        n.op = ExprOp::TRANSPOSE;
        n.lhs = a;
        return push(std::move(n), d);
    }
    // sum over `axes` (kept as size-1 axes), then drop the axes listed in `squeeze`
    uint32_t reduceSum(uint32_t a, const Dims& axes, const Dims& squeeze) {
        ExprNode n;
        n.op = ExprOp::REDUCE_SUM;
        n.lhs = a;
        n.reduction_axes = axes;
        n.squeeze_axes = squeeze;
        n.compute_dtype = DataType::FP32;
        Dims d = dims[a];
        for (uint64_t axis : axes) d[axis] = 1;
        Dims kept;
        for (uint64_t i = 0; i < d.size(); ++i)
            if (!std::binary_search(squeeze.begin(), squeeze.end(), i)) kept.push_back(d[i]);
        if (kept.empty()) kept.push_back(1);
        return push(std::move(n), kept);
    }
    uint32_t softmax(uint32_t a, SoftmaxAlgorithm algorithm, SoftmaxMode mode) {
        ExprNode n;
        n.op = ExprOp::SOFTMAX;
        n.lhs = a;
        n.softmax_algorithm = algorithm;
        n.softmax_mode = mode;
        return push(std::move(n), dims[a]);
    }
    // min/max routing: the element of `source` that won the forward reduction takes `outputGrad`'s value
    uint32_t routeToWinner(ExprOp op, uint32_t source, uint32_t outputGrad, const ExprNode& forwardReduction) {
        ExprNode n;
        n.op = op;
        n.lhs = source;
        n.rhs = outputGrad;
        n.reduction_axes = forwardReduction.reduction_axes;
        n.squeeze_axes = forwardReduction.squeeze_axes;
        return push(std::move(n), dims[source]);
    }
    uint32_t segmentedReduce(ExprOp op, uint32_t values, uint32_t offsets, const ExprNode& like) {
        ExprNode n;
        n.op = op;
        n.lhs = values;
        n.rhs = offsets;
        n.ragged_runtime_batch_size = like.ragged_runtime_batch_size;
        n.ragged_runtime_max_active_values = like.ragged_runtime_max_active_values;
        n.ragged_runtime_elements_per_value = like.ragged_runtime_elements_per_value;
        Dims d = dims[values];
        d[0] = dims[offsets].at(0) - 1;
        return push(std::move(n), d);
    }
    uint32_t segmentedBroadcast(uint32_t perSegment, uint32_t offsets, uint64_t rows, bool normalize) {
        const Dims& segmentDims = dims[perSegment];
        ExprNode n;
        n.op = ExprOp::SEGMENTED_BROADCAST;
        n.lhs = perSegment;
        n.rhs = offsets;
        n.ragged_runtime_batch_size = segmentDims.at(0);
        n.ragged_runtime_max_active_values = rows;
        n.ragged_runtime_elements_per_value = elementCount(segmentDims) / segmentDims.at(0);
        n.segmented_broadcast_normalize_by_length = normalize;
        Dims d = segmentDims;
        d[0] = rows;
        return push(std::move(n), d);
    }
    // the scan `like` describes, over `values` (and the same offsets), in the other direction
    uint32_t oppositeScan(uint32_t values, uint32_t offsets, const ExprNode& like) {
        ExprNode n;
        n.op = like.op;
        n.lhs = values;
        n.rhs = offsets;
        n.scan_op = like.scan_op;
        n.scan_mode = like.scan_mode;
        n.scan_axis = like.scan_axis;
        n.scan_reverse = !like.scan_reverse;
        n.ragged_runtime_batch_size = like.ragged_runtime_batch_size;
        n.ragged_runtime_max_active_values = like.ragged_runtime_max_active_values;
        n.ragged_runtime_elements_per_value = like.ragged_runtime_elements_per_value;
        return push(std::move(n), dims[values]);
    }
    // the gradient of the strided view `like` of an operand shaped `operandDims`
    uint32_t viewGradient(uint32_t gradient, const ExprNode& like, const Dims& operandDims) {
        ExprNode n;
        n.op = ExprOp::STRIDED_VIEW_BACKWARD;
        n.lhs = gradient;
        n.view_dims = like.view_dims;
        n.view_strides = like.view_strides;
        n.view_element_offset = like.view_element_offset;
        n.fill_dims = operandDims;
        n.output_dtype = DataType::FP32;
        return push(std::move(n), operandDims);
    }
    // the gradient of the per-segment min / max `like`: packed values, FP32 gradient of the segments, offsets
    uint32_t segmentWinnerGradient(uint32_t values, uint32_t gradient, uint32_t offsets, const ExprNode& like) {
        ExprNode n;
        n.op = like.op == ExprOp::SEGMENTED_REDUCE_MIN ? ExprOp::SEGMENTED_REDUCE_MIN_BACKWARD : ExprOp::SEGMENTED_REDUCE_MAX_BACKWARD;
        n.lhs = values;
        n.rhs = gradient;
        n.aux = offsets;
        n.ragged_runtime_batch_size = like.ragged_runtime_batch_size;
        n.ragged_runtime_max_active_values = like.ragged_runtime_max_active_values;
        n.ragged_runtime_elements_per_value = like.ragged_runtime_elements_per_value;
        n.output_dtype = DataType::FP32;
        return push(std::move(n), dims[values]);
    }
    // the gradient of the min / max scan `like`: operand, FP32 upstream gradient, offsets of a segmented scan
    uint32_t scanWinnerGradient(uint32_t operand, uint32_t gradient, uint32_t offsets, const ExprNode& like) {
        ExprNode n;
        const bool smallest = like.scan_op == ScanOp::Min;
        n.op = like.op == ExprOp::SEGMENTED_SCAN ? (smallest ? ExprOp::SEGMENTED_SCAN_MIN_BACKWARD : ExprOp::SEGMENTED_SCAN_MAX_BACKWARD)
                                                 : (smallest ? ExprOp::SCAN_MIN_BACKWARD : ExprOp::SCAN_MAX_BACKWARD);
        n.lhs = operand;
        n.rhs = gradient;
        n.aux = offsets;
        n.scan_op = like.scan_op;
        n.scan_mode = like.scan_mode;
        n.scan_axis = like.scan_axis;
        n.scan_reverse = like.scan_reverse;
        n.ragged_runtime_batch_size = like.ragged_runtime_batch_size;
        n.ragged_runtime_max_active_values = like.ragged_runtime_max_active_values;
        n.ragged_runtime_elements_per_value = like.ragged_runtime_elements_per_value;
        n.output_dtype = DataType::FP32;
        return push(std::move(n), dims[operand]);
    }
    // the rotation `like` describes turned the other way, over `values` (same position ids and effective length)
    uint32_t oppositeRope(uint32_t values, uint32_t positionIds, uint32_t effectiveLength, const ExprNode& like) {
        ExprNode n = like;
        n.lhs = values;
        n.rhs = positionIds;
        n.aux = effectiveLength;
        n.rope_inverse = !like.rope_inverse;
        n.output_dtype.reset();
        n.input_tensor_dtype.reset();
        return push(std::move(n), dims[values]);
    }
    uint32_t raggedExtent(uint32_t values, uint32_t offsets, const ExprNode& like) {
        ExprNode n;
        n.op = ExprOp::RAGGED_VALUEWISE_EXTENT;
        n.lhs = values;
        n.rhs = offsets;
        n.ragged_runtime_batch_size = like.ragged_runtime_batch_size;
        n.ragged_runtime_max_active_values = like.ragged_runtime_max_active_values;
        n.ragged_runtime_elements_per_value = like.ragged_runtime_elements_per_value;
        return push(std::move(n), dims[values]);
    }

    // `a`, which broadcasts against `target`, brought to exactly `target`: expanded where it is smaller, summed over the
    // axes along which the forward op broadcast the operand
    uint32_t sumToShape(uint32_t a, const Dims& target) {
        if (shapeless || dims[a] == target) return a;
        const Dims full = broadcastOf(dims[a], target);
        if (dims[a] != full) a = add(a, fill(0.0, full));
        if (full == target) return a;
        const size_t lead = full.size() - target.size();
        Dims axes, squeeze;
        for (size_t i = 0; i < full.size(); ++i) {
            if (i < lead) {
                axes.push_back(i);
                squeeze.push_back(i);
            } else if (target[i - lead] == 1 && full[i] != 1) {
                axes.push_back(i);
            }
        }
        uint32_t out = axes.empty() ? a : reduceSum(a, axes, squeeze);
        return reshape(out, target);
    }

    void setDims(uint32_t node, const Dims& d) { dims.at(node) = d; }

   private:
    uint32_t push(ExprNode&& n, const Dims& d) {
        graph.nodes.push_back(std::move(n));
        dims.push_back(d);
        return static_cast<uint32_t>(graph.nodes.size() - 1);
    }

    const PhysicalExpression& forward;
    const std::vector<Dims>& forwardDims;
    std::unordered_map<uint32_t, uint32_t> copied;
};

std::string noRule(ExprOp op) { return "Thor expressions autodiff does not support backward for op " + opName(op) + "."; }

bool usesRowPartition(ExprOp op) { return isRaggedOp(op) || op == ExprOp::SEGMENTED_SCAN; }

// input names that feed row-partition offsets: structure, not data
std::unordered_set<std::string> rowPartitionInputs(const PhysicalExpression& forward) {
    std::unordered_set<std::string> names;
    std::vector<char> metadata(forward.nodes.size(), 0);
    for (const ExprNode& n : forward.nodes)
        if (usesRowPartition(n.op) && n.rhs != kNone) metadata[n.rhs] = 1;
    for (uint32_t i = static_cast<uint32_t>(forward.nodes.size()); i-- > 0;) {
        if (!metadata[i]) continue;
        const ExprNode& n = forward.nodes[i];
        if (n.op == ExprOp::INPUT) names.insert(forward.inputs.at(n.input_slot).name);
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != kNone) metadata[c] = 1;
    }
    return names;
}

// `typed` is the forward graph (same node numbering) after dtype resolution, when the caller has one: the dtypes that casts
// are undone to and that gradients are delivered in come from it.
PhysicalOutputs differentiate(const PhysicalOutputs& forwardOutputs, const PhysicalExpression* typed, const std::vector<std::string>& wrtNames,
                              const std::optional<std::unordered_map<std::string, std::string>>& upstreamByOutput,
                              const std::optional<std::unordered_map<std::string, Dims>>& inputDimsByName, bool accumulate,
                              const std::unordered_map<std::string, DataType>* seedDTypes = nullptr,
                              const std::unordered_map<std::string, uint32_t>* seedNodes = nullptr) {
    if (!forwardOutputs.expr) throw std::runtime_error("buildBackwardOutputs requires non-null forward_outputs.expr.");
    const PhysicalExpression& forward = *forwardOutputs.expr;
    if (typed && typed->nodes.size() != forward.nodes.size()) throw std::logic_error("Autodiff: the dtype-resolved graph does not match the forward graph.");
    auto dtypeOf = [&](uint32_t node) -> const std::optional<DataType>& { return (typed ? *typed : forward).nodes[node].output_dtype; };
    for (const NamedOutput& o : forwardOutputs.outputs) {
        if (o.node_idx >= forward.nodes.size()) throw std::runtime_error("Forward output node index is out of range in buildBackwardOutputs.");
    }
    const std::vector<std::string> wrt = normalizeBackwardWrtNames(forward, wrtNames);
    const std::unordered_set<std::string> partitionInputs = rowPartitionInputs(forward);
    for (const std::string& name : wrt) {
        if (partitionInputs.count(name)) throw std::runtime_error("Ragged row-partition offsets are metadata and are not differentiable: " + name);
    }
    if (forwardOutputs.outputs.size() > 1 && !upstreamByOutput.has_value()) {
        throw std::runtime_error(
            "buildBackwardOutputs for multi-output forward equations requires an explicit upstream seed map. The map may be partial when "
            "some outputs have no incoming gradient.");
    }
    if (upstreamByOutput.has_value() && upstreamByOutput->empty() && !(seedNodes && !seedNodes->empty())) {
        throw std::runtime_error("buildBackwardOutputs explicit upstream seed map must contain at least one forward output.");
    }
    // Without the dimensions of the forward inputs (the reference's shape-free form, AutoDiff.cpp:3756,3829-3870 there) no
    // gradient is expanded over reduced axes or summed back over broadcast ones: every contribution keeps the shape that
    // broadcasting gives it, the implicit seed is the scalar 1, and a gradient nothing reaches is the scalar 0.  That is the
    // gradient itself for graphs whose operands all have one shape; rules that cannot be written without shapes throw.
    const bool shapeless = !inputDimsByName.has_value();
    const std::vector<Dims> fdims = shapeless ? std::vector<Dims>(forward.nodes.size())
                                              : inferExpressionShapes(forward, [&](uint32_t slot) {
                                                    const std::string& name = forward.inputs.at(slot).name;
                                                    auto it = inputDimsByName->find(name);
                                                    if (it == inputDimsByName->end()) {
                                                        throw std::runtime_error("buildBackwardOutputs is missing the dimensions of forward input: " + name);
                                                    }
                                                    return it->second;
                                                });
    auto needsShapes = [&](const char* what) {
        if (shapeless) throw std::runtime_error(std::string("AutoDiff ") + what + " backward requires forward shape information.");
    };

    // nodes through which a requested input is reached
    std::unordered_set<std::string> wanted(wrt.begin(), wrt.end());
    std::vector<char> reaches(forward.nodes.size(), 0);
    for (uint32_t i = 0; i < forward.nodes.size(); ++i) {
        const ExprNode& n = forward.nodes[i];
        if (n.op == ExprOp::INPUT) {
            reaches[i] = wanted.count(forward.inputs.at(n.input_slot).name) ? 1 : 0;
            continue;
        }
        // offsets are structure: nothing flows through the rhs of a ragged op
        const bool ragged = usesRowPartition(n.op);
        const bool rope = n.op == ExprOp::ROPE;  // position ids and the effective length are structure as well
        for (uint32_t c : {n.lhs, ragged || rope ? kNone : n.rhs, rope ? kNone : n.aux})
            if (c != kNone && reaches[c]) reaches[i] = 1;
    }

    BackwardGraph b(forward, fdims, shapeless);
    std::vector<uint32_t> adjoint(forward.nodes.size(), kNone);
    auto contribute = [&](uint32_t child, uint32_t contribution) {
        if (child == kNone || !reaches[child]) return;
        const uint32_t shaped = b.sumToShape(contribution, fdims[child]);
        adjoint[child] = adjoint[child] == kNone ? shaped : b.add(adjoint[child], shaped);
    };

    for (const NamedOutput& o : forwardOutputs.outputs) {
        if (!reaches[o.node_idx]) continue;
        uint32_t seed;
        if (upstreamByOutput.has_value()) {
            const auto node = seedNodes ? seedNodes->find(o.name) : decltype(seedNodes->find(o.name)){};
            auto it = upstreamByOutput->find(o.name);
            if (seedNodes && node != seedNodes->end()) {
                // the upstream gradient is a value of the forward graph itself
                if (node->second >= forward.nodes.size()) throw std::runtime_error("buildBackwardOutputs upstream node index is out of range for output: " + o.name);
                seed = b.value(node->second);
            } else if (it != upstreamByOutput->end()) {
                seed = b.input(it->second);
                b.setDims(seed, fdims[o.node_idx]);
                if (seedDTypes) {
                    auto dtype = seedDTypes->find(o.name);
                    if (dtype == seedDTypes->end()) {
                        throw std::runtime_error("buildBackwardOutputs received an upstream gradient input without its runtime dtype for output: " + o.name);
                    }
                    b.graph.nodes[seed].output_dtype = dtype->second;
                }
            } else {
                continue;  // a partial map: this output received no gradient
            }
        } else if (shapeless) {
            seed = b.scalar(1.0);
        } else {
            seed = b.fill(1.0, fdims[o.node_idx].empty() ? Dims{1} : fdims[o.node_idx]);
        }
        adjoint[o.node_idx] = adjoint[o.node_idx] == kNone ? seed : b.add(adjoint[o.node_idx], seed);
    }

    for (uint32_t i = static_cast<uint32_t>(forward.nodes.size()); i-- > 0;) {
        if (adjoint[i] == kNone || !reaches[i]) continue;
        const ExprNode& n = forward.nodes[i];
        const uint32_t g = adjoint[i];
        const bool toLhs = n.lhs != kNone && reaches[n.lhs];
        const bool toRhs = n.rhs != kNone && reaches[n.rhs];
        auto x = [&] { return b.value(n.lhs); };
        auto y = [&] { return b.value(i); };
        // g * f'(x) for a unary op, f' given as a node
        auto chain = [&](uint32_t derivative) { contribute(n.lhs, b.mul(g, derivative)); };
        auto sign = [&](uint32_t v) {
            const uint32_t minus = b.neg(v);
            return b.sub(b.binary(ExprOp::MAX_GRAD_LEFT, v, minus), b.binary(ExprOp::MAX_GRAD_RIGHT, v, minus));  // -1, 0 (also for NaN: 0.5 - 0.5), 1
        };
        // the gradient of a reduction's output, shaped like the reduced operand with size-1 reduced axes, then expanded
        auto expandedOverReducedAxes = [&](uint32_t node) {
            if (shapeless) {
                // a reduction that kept its axes broadcasts back by itself; squeezed axes cannot be put back without the rank
                if (!n.squeeze_axes.empty()) needsShapes("squeezing reduction");
                return node;
            }
            Dims keptAsOnes = fdims[n.lhs];
            for (uint64_t axis : resolveReductionAxes(n.reduction_axes, keptAsOnes.size())) keptAsOnes[axis] = 1;
            return b.sumToShape(b.reshape(node, keptAsOnes), fdims[n.lhs]);
        };

        switch (n.op) {
            case ExprOp::INPUT:
            case ExprOp::RUNTIME_SCALAR:
            case ExprOp::TENSOR_RUNTIME_SCALAR:
            case ExprOp::SCALAR_FP:
            case ExprOp::FILL:
                break;

            case ExprOp::ADD:
                contribute(n.lhs, g);
                contribute(n.rhs, g);
                break;
            case ExprOp::SUB:
                contribute(n.lhs, g);
                if (toRhs) contribute(n.rhs, b.neg(g));
                break;
            case ExprOp::MUL:
                if (toLhs) contribute(n.lhs, b.mul(g, b.value(n.rhs)));
                if (toRhs) contribute(n.rhs, b.mul(g, b.value(n.lhs)));
                break;
            case ExprOp::DIV:
                if (toLhs) contribute(n.lhs, b.div(g, b.value(n.rhs)));
                if (toRhs) contribute(n.rhs, b.neg(b.div(b.mul(g, y()), b.value(n.rhs))));  // -g * (a / b) / b
                break;
            case ExprOp::POW:
                if (toLhs) {
                    const uint32_t exponent = b.value(n.rhs);
                    contribute(n.lhs, b.mul(g, b.mul(exponent, b.binary(ExprOp::POW, x(), b.sub(exponent, b.scalar(1.0))))));
                }
                if (toRhs) contribute(n.rhs, b.mul(g, b.mul(y(), b.unary(ExprOp::LN, x()))));
                break;
            case ExprOp::MIN:
            case ExprOp::MAX: {
                const bool isMin = n.op == ExprOp::MIN;
                if (toLhs) contribute(n.lhs, b.mul(g, b.binary(isMin ? ExprOp::MIN_GRAD_LEFT : ExprOp::MAX_GRAD_LEFT, x(), b.value(n.rhs))));
                if (toRhs) contribute(n.rhs, b.mul(g, b.binary(isMin ? ExprOp::MIN_GRAD_RIGHT : ExprOp::MAX_GRAD_RIGHT, x(), b.value(n.rhs))));
                break;
            }
            case ExprOp::WHERE:
                if (toRhs) contribute(n.rhs, b.where(b.value(n.lhs), g, b.scalar(0.0)));
                if (n.aux != kNone && reaches[n.aux]) contribute(n.aux, b.where(b.value(n.lhs), b.scalar(0.0), g));
                break;
            case ExprOp::CAST: {
                // straight through, delivered in the operand's dtype when that is known
                const std::optional<DataType>& source = dtypeOf(n.lhs);
                contribute(n.lhs, source.has_value() ? b.cast(g, source.value()) : g);
                break;
            }

            case ExprOp::NEG: contribute(n.lhs, b.neg(g)); break;
            case ExprOp::ABS: chain(sign(x())); break;
            case ExprOp::EXP: chain(y()); break;
            case ExprOp::EXP2: chain(b.scaled(y(), std::log(2.0))); break;
            case ExprOp::EXP10: chain(b.scaled(y(), std::log(10.0))); break;
            case ExprOp::EXPM1: chain(b.add(y(), b.scalar(1.0))); break;
            case ExprOp::LN: contribute(n.lhs, b.div(g, x())); break;
            case ExprOp::LOG2: contribute(n.lhs, b.div(g, b.scaled(x(), std::log(2.0)))); break;
            case ExprOp::LOG10: contribute(n.lhs, b.div(g, b.scaled(x(), std::log(10.0)))); break;
            case ExprOp::LOG1P: contribute(n.lhs, b.div(g, b.add(x(), b.scalar(1.0)))); break;
            case ExprOp::SQRT: contribute(n.lhs, b.div(g, b.scaled(y(), 2.0))); break;
            case ExprOp::SIN: chain(b.unary(ExprOp::COS, x())); break;
            case ExprOp::COS: chain(b.neg(b.unary(ExprOp::SIN, x()))); break;
            case ExprOp::TAN: chain(b.add(b.mul(y(), y()), b.scalar(1.0))); break;
            case ExprOp::TANH: chain(b.sub(b.scalar(1.0), b.mul(y(), y()))); break;
            case ExprOp::SINH: chain(b.unary(ExprOp::COSH, x())); break;
            case ExprOp::COSH: chain(b.unary(ExprOp::SINH, x())); break;
            case ExprOp::ASIN: contribute(n.lhs, b.div(g, b.unary(ExprOp::SQRT, b.sub(b.scalar(1.0), b.mul(x(), x()))))); break;
            case ExprOp::ACOS: contribute(n.lhs, b.neg(b.div(g, b.unary(ExprOp::SQRT, b.sub(b.scalar(1.0), b.mul(x(), x())))))); break;
            case ExprOp::ATAN: contribute(n.lhs, b.div(g, b.add(b.mul(x(), x()), b.scalar(1.0)))); break;
            case ExprOp::ASINH: contribute(n.lhs, b.div(g, b.unary(ExprOp::SQRT, b.add(b.mul(x(), x()), b.scalar(1.0))))); break;
            case ExprOp::ACOSH: contribute(n.lhs, b.div(g, b.unary(ExprOp::SQRT, b.sub(b.mul(x(), x()), b.scalar(1.0))))); break;
            case ExprOp::ATANH: contribute(n.lhs, b.div(g, b.sub(b.scalar(1.0), b.mul(x(), x())))); break;
            case ExprOp::ERF: chain(b.scaled(b.unary(ExprOp::EXP, b.neg(b.mul(x(), x()))), 2.0 / std::sqrt(M_PI))); break;
            case ExprOp::ERFC: chain(b.scaled(b.unary(ExprOp::EXP, b.neg(b.mul(x(), x()))), -2.0 / std::sqrt(M_PI))); break;
            case ExprOp::ERFCX: chain(b.sub(b.scaled(b.mul(x(), y()), 2.0), b.scalar(2.0 / std::sqrt(M_PI)))); break;
            case ExprOp::ERFINV: chain(b.scaled(b.unary(ExprOp::EXP, b.mul(y(), y())), std::sqrt(M_PI) / 2.0)); break;
            case ExprOp::ERFCINV: chain(b.scaled(b.unary(ExprOp::EXP, b.mul(y(), y())), -std::sqrt(M_PI) / 2.0)); break;
            case ExprOp::NORMCDF: chain(b.scaled(b.unary(ExprOp::EXP, b.scaled(b.mul(x(), x()), -0.5)), 1.0 / std::sqrt(2.0 * M_PI))); break;
            case ExprOp::LGAMMA: chain(b.unary(ExprOp::DIGAMMA, x())); break;
            case ExprOp::TGAMMA: chain(b.mul(y(), b.unary(ExprOp::DIGAMMA, x()))); break;

            case ExprOp::RESHAPE:
            case ExprOp::UNSQUEEZE:
            case ExprOp::SQUEEZE:
                needsShapes("reshape");
                contribute(n.lhs, b.reshape(g, fdims[n.lhs]));
                break;
            case ExprOp::TRANSPOSE:
                contribute(n.lhs, b.transpose(g));
                break;
            case ExprOp::STRIDED_VIEW:
                // the gradient lands on the elements the view addresses, 0 elsewhere (Utilities/Expression/AutoDiff.cpp:2100-2125 there);
                // a view of a view addresses storage that is not the operand's own index space
                if (isStorageViewOp(forward.nodes[n.lhs].op)) throw std::runtime_error(noRule(n.op) + " The operand is itself a view.");
                needsShapes("strided view");
                contribute(n.lhs, b.viewGradient(b.cast(g, DataType::FP32), n, fdims[n.lhs]));
                break;

            case ExprOp::REDUCE_SUM:
                contribute(n.lhs, expandedOverReducedAxes(g));
                break;
            case ExprOp::REDUCE_AVG: {
                needsShapes("reduce_mean");
                const uint64_t count = elementCount(fdims[n.lhs]) / elementCount(fdims[i]);
                contribute(n.lhs, b.div(expandedOverReducedAxes(g), b.scalar(static_cast<double>(count))));
                break;
            }
            case ExprOp::REDUCE_NORM1:
                contribute(n.lhs, b.mul(expandedOverReducedAxes(g), sign(x())));
                break;
            case ExprOp::REDUCE_NORM2:
                contribute(n.lhs, b.div(b.mul(expandedOverReducedAxes(g), x()), expandedOverReducedAxes(y())));
                break;
            case ExprOp::REDUCE_PROD:
                // product of the others = product / element: valid where no reduced element is zero
                contribute(n.lhs, b.div(b.mul(expandedOverReducedAxes(g), expandedOverReducedAxes(y())), x()));
                break;
            case ExprOp::REDUCE_MIN:
            case ExprOp::REDUCE_MAX:
                needsShapes("reduce_min / reduce_max");
                contribute(n.lhs, b.routeToWinner(n.op == ExprOp::REDUCE_MIN ? ExprOp::REDUCE_MIN_BACKWARD : ExprOp::REDUCE_MAX_BACKWARD, x(), g, n));
                break;

            case ExprOp::SOFTMAX: {
                needsShapes("softmax");
                const Dims& d = fdims[n.lhs];
                if (d.size() < 2) throw std::runtime_error("Autodiff for softmax expects tensors of rank 2 or more.");
                Dims axes;
                if (n.softmax_mode == SoftmaxMode::Channel) {
                    axes = {1};
                } else {
                    for (uint64_t a = 1; a < d.size(); ++a) axes.push_back(a);
                }
                if (n.softmax_algorithm == SoftmaxAlgorithm::Log) {
                    // y = x - logsumexp(x): dx = g - softmax(x) * sum(g)
                    const uint32_t probabilities = b.softmax(x(), SoftmaxAlgorithm::Accurate, n.softmax_mode);
                    contribute(n.lhs, b.sub(g, b.mul(probabilities, b.reduceSum(g, axes, {}))));
                } else {
                    // dx = y * (g - sum(g * y))
                    contribute(n.lhs, b.mul(y(), b.sub(g, b.reduceSum(b.mul(g, y()), axes, {}))));
                }
                break;
            }

            case ExprOp::SEGMENTED_REDUCE_SUM:
            case ExprOp::SEGMENTED_REDUCE_MEAN:
                // every row of a segment receives the segment's gradient (divided by the segment's length for a mean)
                needsShapes("segmented reduction");
                contribute(n.lhs, b.segmentedBroadcast(g, b.value(n.rhs), fdims[n.lhs].at(0), n.op == ExprOp::SEGMENTED_REDUCE_MEAN));
                break;
            case ExprOp::SEGMENTED_REDUCE_MIN:
            case ExprOp::SEGMENTED_REDUCE_MAX:
                // each segment's gradient goes to the row that won the column (Utilities/Expression/AutoDiff.cpp:5630-5700 there)
                contribute(n.lhs, b.segmentWinnerGradient(x(), b.cast(g, DataType::FP32), b.value(n.rhs), n));
                break;
            case ExprOp::SEGMENTED_BROADCAST:
                needsShapes("segmented broadcast");
                contribute(n.lhs, b.segmentedReduce(n.segmented_broadcast_normalize_by_length ? ExprOp::SEGMENTED_REDUCE_MEAN : ExprOp::SEGMENTED_REDUCE_SUM,
                                                    g, b.value(n.rhs), n));
                break;
            case ExprOp::RAGGED_VALUEWISE_EXTENT:
                contribute(n.lhs, b.raggedExtent(g, b.value(n.rhs), n));
                break;
            case ExprOp::SCAN:
            case ExprOp::SEGMENTED_SCAN:
                // element j feeds every later prefix (the later ones only, when exclusive): its gradient is the same scan of the
                // upstream gradient run from the other end
                if (n.scan_op == ScanOp::Sum) {
                    contribute(n.lhs, b.oppositeScan(g, n.op == ExprOp::SEGMENTED_SCAN ? b.value(n.rhs) : kNone, n));
                } else if (n.scan_op == ScanOp::Min || n.scan_op == ScanOp::Max) {
                    // every position hands its gradient to the element that held the running minimum / maximum there
                    // (Utilities/Expression/AutoDiff.cpp:5743-5760 there)
                    contribute(n.lhs, b.scanWinnerGradient(x(), b.cast(g, DataType::FP32), n.op == ExprOp::SEGMENTED_SCAN ? b.value(n.rhs) : kNone, n));
                } else {
                    throw std::runtime_error("Thor expressions autodiff currently supports backward only for sum/min/max scan.");
                }
                break;

            case ExprOp::ROPE:
                // y = a R x with R a rotation: the gradient is a R^T g, the same rotation turned the other way
                // (Utilities/Expression/AutoDiff.cpp:4672-4693 there)
                contribute(n.lhs, b.oppositeRope(g, n.rhs != kNone ? b.value(n.rhs) : kNone, n.aux != kNone ? b.value(n.aux) : kNone, n));
                break;

            default:
                throw std::runtime_error(noRule(n.op));
        }
    }

    // ---- gradient outputs ---------------------------------------------------------------------------------------------
    PhysicalOutputs result;
    std::unordered_map<uint32_t, uint32_t> timesNamed;  // one gradient value may answer for several inputs
    std::vector<NamedOutput> named;
    for (const std::string& name : wrt) {
        uint32_t slot = kNone;
        for (const NamedInput& in : forward.inputs)
            if (in.name == name) slot = in.slot;
        uint32_t total = kNone, firstNode = kNone;
        for (uint32_t i = 0; i < forward.nodes.size(); ++i) {
            const ExprNode& n = forward.nodes[i];
            if (n.op != ExprOp::INPUT || n.input_slot != slot) continue;
            if (firstNode == kNone) firstNode = i;
            if (adjoint[i] != kNone) total = total == kNone ? adjoint[i] : b.add(total, adjoint[i]);
        }
        if (firstNode == kNone) throw std::runtime_error("No INPUT node found for requested gradient input: " + name);
        const Dims shape = fdims[firstNode].empty() ? Dims{1} : fdims[firstNode];
        const std::optional<DataType>& dtype = dtypeOf(firstNode);
        const std::string outputName = name + "_grad";
        if (total == kNone) total = shapeless ? b.scalar(0.0) : b.fill(0.0, shape, dtype);
        if (accumulate) {
            const uint32_t running = b.input(outputName);
            b.setDims(running, shape);
            total = b.add(running, total);
        }
        // a node of its own per name, so that two names never share one tensor
        const uint32_t repeats = timesNamed[total]++;
        uint32_t terminal = total;
        for (uint32_t r = 0; r < repeats; ++r) terminal = b.add(terminal, b.scalar(0.0));
        terminal = dtype.has_value() ? b.cast(terminal, dtype.value()) : b.add(terminal, shapeless ? b.scalar(0.0) : b.fill(0.0, shape));
        named.push_back(NamedOutput{outputName, terminal});
    }
    result.expr = std::make_shared<PhysicalExpression>(std::move(b.graph));
    result.expr->output_node = named.back().node_idx;
    result.outputs = std::move(named);
    return result;
}

}  // namespace

std::vector<std::string> normalizeBackwardWrtNames(const PhysicalExpression& forward, const std::vector<std::string>& wrtNames) {
    std::vector<std::string> out;
    if (wrtNames.empty()) {
        const std::unordered_set<std::string> partitionInputs = rowPartitionInputs(forward);
        for (const NamedInput& in : forward.inputs)
            if (in.kind == NamedInput::Kind::Tensor && !partitionInputs.count(in.name)) out.push_back(in.name);
        return out;
    }
    std::unordered_set<std::string> seen;
    for (const std::string& name : wrtNames) {
        if (!seen.insert(name).second) throw std::runtime_error("Duplicate wrt input name passed to compileBackward: " + name);
        const NamedInput* found = nullptr;
        for (const NamedInput& in : forward.inputs)
            if (in.name == name) found = &in;
        if (!found) throw std::runtime_error("Requested gradient for unknown input: " + name);
        if (found->kind != NamedInput::Kind::Tensor) {
            throw std::runtime_error("compileBackward only supports gradients with respect to tensor inputs. Got runtime scalar input: " + name);
        }
        out.push_back(name);
    }
    return out;
}

std::optional<std::unordered_map<std::string, std::string>> normalizeBackwardUpstreamNames(const PhysicalOutputs& forwardOutputs,
                                                                                             const std::optional<std::string>& upstreamName) {
    if (!upstreamName.has_value()) return std::nullopt;
    if (forwardOutputs.outputs.size() != 1) {
        throw std::runtime_error("compileBackward single upstream input name overload only supports exactly one forward output.");
    }
    if (upstreamName->empty()) throw std::runtime_error("compileBackward explicit upstream input name cannot be empty.");
    for (const NamedInput& in : forwardOutputs.expr->inputs) {
        if (in.name == upstreamName.value()) {
            throw std::runtime_error("compileBackward explicit upstream input name collides with an existing forward input: " + upstreamName.value());
        }
    }
    return std::unordered_map<std::string, std::string>{{forwardOutputs.outputs[0].name, upstreamName.value()}};
}

std::unordered_map<std::string, std::string> normalizeBackwardUpstreamNames(const PhysicalOutputs& forwardOutputs,
                                                                             const std::unordered_map<std::string, std::string>& byOutput) {
    if (!forwardOutputs.expr) throw std::runtime_error("compileBackward upstream-input validation requires non-null forward expr.");
    for (const auto& [outputName, upstreamName] : byOutput) {
        bool known = false;
        for (const NamedOutput& o : forwardOutputs.outputs) known = known || o.name == outputName;
        if (!known) throw std::runtime_error("compileBackward explicit upstream map contains unknown forward output: " + outputName);
        if (upstreamName.empty()) throw std::runtime_error("compileBackward explicit upstream input name cannot be empty for output: " + outputName);
        for (const NamedInput& in : forwardOutputs.expr->inputs) {
            if (in.name == upstreamName) {
                throw std::runtime_error("compileBackward explicit upstream input name collides with an existing forward input: " + upstreamName);
            }
        }
    }
    return byOutput;
}

PhysicalOutputs buildBackwardOutputs(const PhysicalOutputs& forwardOutputs, const std::vector<std::string>& wrtNames,
                                     const std::optional<std::string>& upstreamName,
                                     const std::optional<std::unordered_map<std::string, std::vector<uint64_t>>>& inputDims, bool accumulate) {
    if (!forwardOutputs.expr) throw std::runtime_error("buildBackwardOutputs requires non-null forward_outputs.expr.");
    return differentiate(forwardOutputs, nullptr, wrtNames, normalizeBackwardUpstreamNames(forwardOutputs, upstreamName), inputDims, accumulate);
}

PhysicalOutputs buildBackwardOutputs(const PhysicalOutputs& forwardOutputs, const std::vector<std::string>& wrtNames,
                                     const std::unordered_map<std::string, std::string>& upstreamByOutput,
                                     const std::optional<std::unordered_map<std::string, std::vector<uint64_t>>>& inputDims, bool accumulate) {
    return differentiate(forwardOutputs, nullptr, wrtNames, normalizeBackwardUpstreamNames(forwardOutputs, upstreamByOutput), inputDims, accumulate);
}

PhysicalOutputs buildBackwardOutputs(const PhysicalOutputs& forwardOutputs, const std::vector<std::string>& wrtNames,
                                     const std::unordered_map<std::string, std::string>& upstreamByOutput,
                                     const std::unordered_map<std::string, DataType>& upstreamDTypesByOutput,
                                     const std::optional<std::unordered_map<std::string, std::vector<uint64_t>>>& inputDims, bool accumulate) {
    return differentiate(forwardOutputs, nullptr, wrtNames, normalizeBackwardUpstreamNames(forwardOutputs, upstreamByOutput), inputDims, accumulate,
                         &upstreamDTypesByOutput);
}

PhysicalOutputs buildBackwardOutputs(const PhysicalOutputs& forwardOutputs, const std::vector<std::string>& wrtNames,
                                     const std::unordered_map<std::string, std::string>& upstreamByOutput,
                                     const std::unordered_map<std::string, uint32_t>& upstreamNodeIndicesByOutput,
                                     const std::optional<std::unordered_map<std::string, std::vector<uint64_t>>>& inputDims, bool accumulate) {
    if (upstreamByOutput.empty() && !upstreamNodeIndicesByOutput.empty()) {
        // seeds given as forward nodes only: the name map may be empty then
        return differentiate(forwardOutputs, nullptr, wrtNames, std::unordered_map<std::string, std::string>{}, inputDims, accumulate, nullptr,
                             &upstreamNodeIndicesByOutput);
    }
    return differentiate(forwardOutputs, nullptr, wrtNames, normalizeBackwardUpstreamNames(forwardOutputs, upstreamByOutput), inputDims, accumulate, nullptr,
                         &upstreamNodeIndicesByOutput);
}

PhysicalOutputs buildBackwardOutputsTyped(const PhysicalOutputs& forwardOutputs, const PhysicalExpression& typedForward,
                                          const std::vector<std::string>& wrtNames,
                                          const std::optional<std::unordered_map<std::string, std::string>>& upstreamByOutput,
                                          const std::unordered_map<std::string, std::vector<uint64_t>>& inputDims, bool accumulate) {
    return differentiate(forwardOutputs, &typedForward, wrtNames, upstreamByOutput, inputDims, accumulate);
}

}  // namespace ThorImplementation
