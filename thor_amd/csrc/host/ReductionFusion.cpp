#include "RowFusion.h"

#include "HipSourceEmitter.h"
#include "ReductionPlanner.h"

#include <algorithm>
#include <map>
#include <set>

namespace ThorImplementation {

namespace {

using Role = RowFusionContext::Role;
typedef ReductionKernelRequest::Source::Kind SourceKind;

CubReductionOp cubOpOf(ExprOp op) {
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
    throw std::logic_error("Not a value reduction op.");
}

bool isElementwise(ExprOp op) {
    if (isReductionOp(op) || op == ExprOp::RESHAPE || op == ExprOp::UNSQUEEZE || op == ExprOp::SQUEEZE) return false;
    return Expression::isBinaryOp(op) || op == ExprOp::WHERE || Expression::isUnaryOp(op);
}

uint64_t product(const std::vector<uint64_t>& d) {
    uint64_t n = 1;
    for (uint64_t v : d) n *= v;
    return n;
}

uint32_t viewBase(const RowFusionContext& ctx, uint32_t node) {
    while (ctx.role[node] == Role::View) node = ctx.expr.nodes[node].lhs;
    return node;
}

// One (shape, axes) geometry and what can be evaluated per element of it.
struct Geometry {
    std::vector<uint64_t> shape;
    std::vector<uint64_t> axes;  // sorted, unique
    uint64_t outputs = 1;

    bool reduced(size_t axis) const { return std::binary_search(axes.begin(), axes.end(), static_cast<uint64_t>(axis)); }
};

enum class Leaf : uint8_t { No, Vector, Scalar, Kept };

// How an existing tensor can be read inside the kernel.
Leaf leafKind(const RowFusionContext& ctx, uint32_t node, const Geometry& g) {
    const Tensor& t = ctx.tensorOf[node];
    if (!t.isInitialized() || !t.isDenseContiguous()) return Leaf::No;
    const std::vector<uint64_t>& d = ctx.dims[node];
    if (product(d) == 1) return Leaf::Scalar;
    if (d == g.shape) return Leaf::Vector;
    // a function of the output alone: extent 1 along every reduced axis; along a kept axis the full extent or 1 (broadcast there
    // too: a [C, 1, 1] bias under [N, C, H, W] -> [N, C])
    if (d.size() > g.shape.size()) return Leaf::No;
    const size_t shift = g.shape.size() - d.size();
    for (size_t a = 0; a < g.shape.size(); ++a) {
        const uint64_t extent = a < shift ? 1 : d[a - shift];
        if (g.reduced(a) ? extent != 1 : (extent != g.shape[a] && extent != 1)) return Leaf::No;
    }
    return Leaf::Kept;
}

// The offset of a Kept leaf's element as a C expression of `slot`, the output's number (row-major over the kept axes); empty
// when the leaf has one element per output in that order.
std::string keptOffsetOf(const std::vector<uint64_t>& d, const Geometry& g) {
    const size_t shift = g.shape.size() - d.size();
    bool identity = true;
    for (size_t a = 0; a < g.shape.size(); ++a)
        if (!g.reduced(a) && (a < shift ? 1 : d[a - shift]) != g.shape[a]) identity = false;
    if (identity) return std::string();
    std::string text;
    uint64_t after = 1;   // outputs per step of the kept axis at hand: the product of the kept extents after it
    uint64_t stride = 1;  // the leaf's own stride there: the product of its extents after it
    for (size_t a = g.shape.size(); a-- > 0;) {
        const uint64_t extent = a < shift ? 1 : d[a - shift];
        if (!g.reduced(a)) {
            if (extent != 1) {
                text += (text.empty() ? "" : " + ") + ("((slot / " + std::to_string(after) + "ull) % " + std::to_string(g.shape[a]) + "ull) * " + std::to_string(stride) + "ull");
            }
            after *= g.shape[a];
        }
        stride *= extent;
    }
    return text.empty() ? std::string("0") : text;
}

struct Analysis {
    const RowFusionContext& ctx;
    const Geometry& g;
    std::vector<int8_t> memo;  // -1 unknown, 0 no, 1 yes

    Analysis(const RowFusionContext& ctx, const Geometry& g) : ctx(ctx), g(g), memo(ctx.expr.nodes.size(), -1) {}

    // Can the value of `node` be produced per element inside the kernel (from tensors that exist now)?
    bool computable(uint32_t node) {
        if (memo[node] >= 0) return memo[node] == 1;
        memo[node] = 0;
        const ExprNode& n = ctx.expr.nodes[node];
        bool ok = false;
        if (ctx.tensorOf[node].isInitialized()) {
            ok = leafKind(ctx, node, g) != Leaf::No;
        } else if (ctx.done[node]) {
            ok = false;  // produced by another stage without a tensor of its own
        } else if (n.op == ExprOp::SCALAR_FP || n.op == ExprOp::RUNTIME_SCALAR) {
            ok = true;
        } else if (n.op == ExprOp::FILL) {
            double folded;
            ok = tryFoldConstant(ctx.expr, node, folded);
        } else if (isElementwise(n.op)) {
            const std::vector<uint64_t>& d = ctx.dims[node];
            ok = d == g.shape || product(d) == 1;  // broadcast intermediates of other shapes stay with the staged path
            for (uint32_t c : {n.lhs, n.rhs, n.aux})
                if (c != UINT32_MAX) ok = ok && computable(c);
        }
        memo[node] = ok ? 1 : 0;
        return ok;
    }
};

}  // namespace

void tryReductionFusion(RowFusionContext& ctx) {
    const PhysicalExpression& expr = ctx.expr;
    const size_t count = expr.nodes.size();

    std::vector<std::vector<uint32_t>> consumers(count);
    for (uint32_t i = 0; i < count; ++i) {
        const ExprNode& n = expr.nodes[i];
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != UINT32_MAX) consumers[c].push_back(i);
    }
    std::vector<char> isNamedOutput(count, 0);
    for (const NamedOutput& o : ctx.outputs) {
        isNamedOutput[o.node_idx] = 1;
        isNamedOutput[viewBase(ctx, o.node_idx)] = 1;
    }

    // group the pending value reductions by (shape of the reduced value, reduced axes)
    typedef std::pair<std::vector<uint64_t>, std::vector<uint64_t>> Key;
    std::map<Key, std::vector<uint32_t>> groups;
    for (uint32_t i = 0; i < count; ++i) {
        const ExprNode& n = expr.nodes[i];
        if (ctx.done[i] || !isValueReductionOp(n.op) || ctx.role[i] != Role::Materialized) continue;
        const std::vector<uint64_t>& shape = ctx.dims[n.lhs];
        if (shape.empty() || product(shape) < 2) continue;
        const std::vector<uint64_t> axes = resolveReductionAxes(n.reduction_axes, shape.size());
        groups[Key(shape, axes)].push_back(i);
    }

    const TensorPlacement gpuPlacement(TensorPlacement::MemDevices::GPU, ctx.deviceNum);
    for (auto& [key, candidates] : groups) {
        Geometry g;
        g.shape = key.first;
        g.axes = key.second;
        for (size_t a = 0; a < g.shape.size(); ++a)
            if (!g.reduced(a)) g.outputs *= g.shape[a];
        Analysis analysis(ctx, g);

        std::vector<uint32_t> reductions;
        for (uint32_t r : candidates)
            if (analysis.computable(expr.nodes[r].lhs)) reductions.push_back(r);
        if (reductions.empty()) continue;

        // ---- the nodes evaluated inside the kernel: everything below the operands down to existing tensors ---------------
        std::vector<char> inKernel(count, 0), isLeaf(count, 0);
        std::vector<uint32_t> stack;
        auto addRoot = [&](uint32_t root) {
            stack.push_back(root);
            while (!stack.empty()) {
                const uint32_t node = stack.back();
                stack.pop_back();
                if (inKernel[node] || isLeaf[node]) continue;
                if (ctx.tensorOf[node].isInitialized()) {
                    isLeaf[node] = 1;
                    continue;
                }
                inKernel[node] = 1;
                const ExprNode& n = expr.nodes[node];
                for (uint32_t c : {n.lhs, n.rhs, n.aux})
                    if (c != UINT32_MAX) stack.push_back(c);
            }
        };
        for (uint32_t r : reductions) addRoot(expr.nodes[r].lhs);

        // other same-shaped elementwise values that read one of the kernel's full-shape tensors ride along: the source is
        // read once for both
        std::vector<uint32_t> extraOutputs;
        for (uint32_t i = 0; i < count; ++i) {
            if (ctx.done[i] || inKernel[i] || ctx.role[i] != Role::Materialized || !isElementwise(expr.nodes[i].op)) continue;
            if (ctx.dims[i] != g.shape || !analysis.computable(i)) continue;
            // shares a vector source with the kernel?
            std::vector<char> seen(count, 0);
            std::vector<uint32_t> walk = {i};
            bool shares = false;
            while (!walk.empty() && !shares) {
                const uint32_t node = walk.back();
                walk.pop_back();
                if (seen[node]) continue;
                seen[node] = 1;
                if (ctx.tensorOf[node].isInitialized()) {
                    shares = isLeaf[node] && leafKind(ctx, node, g) == Leaf::Vector;
                    continue;
                }
                if (inKernel[node]) {
                    shares = true;
                    continue;
                }
                const ExprNode& n = expr.nodes[node];
                for (uint32_t c : {n.lhs, n.rhs, n.aux})
                    if (c != UINT32_MAX) walk.push_back(c);
            }
            if (shares) extraOutputs.push_back(i);
        }
        for (uint32_t e : extraOutputs) addRoot(e);

        // ---- which materialised kernel values must also reach memory ------------------------------------------------------
        std::set<uint32_t> reductionSet(reductions.begin(), reductions.end());
        std::vector<char> neededOutside(count, 0);
        for (uint32_t i = 0; i < count; ++i) {
            if (!inKernel[i]) continue;
            if (isNamedOutput[i]) neededOutside[i] = 1;
            for (uint32_t c : consumers[i])
                if (!inKernel[c] && !reductionSet.count(c)) neededOutside[i] = 1;
        }
        // an inline value needed outside is recomputed there from its tensor sources: those must exist
        for (uint32_t i = static_cast<uint32_t>(count); i-- > 0;) {
            if (!inKernel[i] || !neededOutside[i] || ctx.role[i] != Role::Inline) continue;
            const ExprNode& n = expr.nodes[i];
            for (uint32_t c : {n.lhs, n.rhs, n.aux})
                if (c != UINT32_MAX && inKernel[c]) neededOutside[c] = 1;
        }
        std::vector<uint32_t> stored;
        bool storable = true;
        for (uint32_t i = 0; i < count; ++i) {
            if (!inKernel[i] || ctx.role[i] != Role::Materialized || !neededOutside[i]) continue;
            if (ctx.dims[i] != g.shape) storable = false;  // a scalar intermediate cannot be written by a per-element pass
            stored.push_back(i);
        }
        if (!storable) continue;

        bool anyPrologue = false;
        for (uint32_t r : reductions) anyPrologue = anyPrologue || !ctx.tensorOf[expr.nodes[r].lhs].isInitialized();
        if (reductions.size() < 2 && !anyPrologue && stored.empty()) continue;  // a lone reduction of an existing tensor

        // ---- kernel request ------------------------------------------------------------------------------------------------
        std::vector<uint32_t> sourceNodes;
        std::set<uint32_t> scalarSet;
        for (uint32_t i = 0; i < count; ++i) {
            if (isLeaf[i]) sourceNodes.push_back(i);
            if (inKernel[i] && expr.nodes[i].op == ExprOp::RUNTIME_SCALAR) scalarSet.insert(expr.nodes[i].input_slot);
        }
        ReductionKernelRequest request;
        request.deviceNum = ctx.deviceNum;
        std::vector<uint32_t> axes32;
        for (uint64_t a : g.axes) axes32.push_back(static_cast<uint32_t>(a));
        request.geometry = CubReduction::analyzeGeometry(g.shape, axes32);
        request.scalarSlots.assign(scalarSet.begin(), scalarSet.end());
        request.inputAlignmentBytes = 256;
        BodyEmitter body(expr);
        std::string text;
        for (uint32_t slot : request.scalarSlots) text += "        const float s" + std::to_string(slot) + " = s.s" + std::to_string(slot) + ";\n";
        std::vector<Tensor> inputs;
        std::map<uint32_t, size_t> sourceIndex;
        bool anyVector = false;
        for (size_t i = 0; i < sourceNodes.size(); ++i) {
            const uint32_t node = sourceNodes[i];
            const Tensor& t = ctx.tensorOf[node];
            const Leaf kind = leafKind(ctx, node, g);
            ReductionKernelRequest::Source source;
            source.storage = t.getDataType();
            source.kind = kind == Leaf::Vector ? SourceKind::Vector : (kind == Leaf::Scalar ? SourceKind::Scalar : SourceKind::Kept);
            if (kind == Leaf::Kept) source.keptOffset = keptOffsetOf(ctx.dims[node], g);
            request.sources.push_back(source);
            if (kind == Leaf::Vector) {
                request.inputAlignmentBytes = std::min(request.inputAlignmentBytes, pointerAlignment(t.getMemPtr()));
                anyVector = true;
            }
            inputs.push_back(t);
            sourceIndex[node] = i;
            const DataType valueDType = expr.nodes[node].output_dtype.value();
            const std::string raw = kind == Leaf::Vector ? "l.p" + std::to_string(i) + ".v[k]" : "kk.z" + std::to_string(i);
            text += "        const " + std::string(valueCType(valueDType)) + " t" + std::to_string(node) + " = " +
                    castValueExpr(storageToValueExpr(raw, t.getDataType()), t.getDataType(), valueDType) + ";\n";
            body.defineSource(node, valueDType);
        }
        if (!anyVector) continue;  // nothing streams: leave it to the staged path
        uint64_t flopsPerElement = 0;
        for (uint32_t node = 0; node < count; ++node) {
            if (!inKernel[node]) continue;
            double folded;
            if (tryFoldConstant(expr, node, folded)) continue;
            flopsPerElement += body.emit(text, node, "        ");
            if (ctx.role[node] == Role::Materialized) {
                // the staged plan would have stored this value in its output dtype: round there before anything reads it
                const DataType storedDType = expr.nodes[node].output_dtype.value();
                if (body.dtypeOf(node) != storedDType) {
                    text += "        const " + std::string(valueCType(storedDType)) + " m" + std::to_string(node) + " = " + body.ref(node, storedDType) + ";\n";
                    body.defineSource(node, storedDType, "m" + std::to_string(node));
                }
            }
        }
        for (uint32_t r : reductions) {
            const ExprNode& rn = expr.nodes[r];
            ReductionKernelRequest::Value value;
            value.op = cubOpOf(rn.op);
            value.outputDType = rn.output_dtype.value();
            const uint32_t operand = rn.lhs;
            if (isLeaf[operand]) {
                // an existing tensor is read as the stand-alone reduction reads it: storage -> fp32
                const size_t i = sourceIndex.at(operand);
                const DataType storage = inputs[i].getDataType();
                value.expression = castValueExpr(storageToValueExpr("l.p" + std::to_string(i) + ".v[k]", storage), storage, DataType::FP32);
            } else {
                value.expression = body.ref(operand, DataType::FP32);
            }
            request.values.push_back(value);
            ++flopsPerElement;
        }
        for (uint32_t node : stored) {
            ReductionKernelRequest::Elementwise e;
            e.outputDType = expr.nodes[node].output_dtype.value();
            e.expression = valueToStorageExpr(body.ref(node, e.outputDType), e.outputDType);
            request.elementwise.push_back(e);
        }
        request.prologue = text;
        request.inputDType = inputs.front().getDataType();

        ReductionLaunchPlan plan = buildReductionKernels(request);
        std::optional<Tensor> workspace = allocateReductionWorkspace(plan, gpuPlacement, ctx.stream);
        std::vector<Tensor> outputs, elementwiseOutputs;
        for (uint32_t r : reductions) {
            Tensor out = ctx.allocateFor(r);
            ctx.tensorOf[r] = out;
            outputs.push_back(out);
        }
        for (uint32_t node : stored) {
            Tensor out = ctx.allocateFor(node);
            ctx.tensorOf[node] = out;
            elementwiseOutputs.push_back(out);
        }
        std::vector<std::string> scalarNames;
        for (uint32_t slot : request.scalarSlots) scalarNames.push_back(ctx.rootInputs.at(slot).name);

        StampedExecutionStage stage;
        stage.kind = StampedExecutionStage::Kind::FusedReduction;
        stage.gpu_num = ctx.deviceNum;
        for (uint32_t node : sourceNodes) {
            const int st = ctx.stageOfNode[viewBase(ctx, node)];
            if (st >= 0) stage.dependency_stage_indices.push_back(static_cast<uint32_t>(st));
        }
        plan.variant = "fused_reduction(values=" + std::to_string(reductions.size()) + ",sources=" + std::to_string(sourceNodes.size()) +
                       ",elementwise_outputs=" + std::to_string(stored.size()) + ") " + plan.variant;
        stage.fused_reduction = std::make_shared<StampedFusedReduction>(std::move(plan), inputs, scalarNames, outputs, elementwiseOutputs, workspace,
                                                                        flopsPerElement * product(g.shape));
        const int stageIndex = static_cast<int>(ctx.stages.size());
        for (uint32_t r : reductions) {
            ctx.done[r] = 1;
            ctx.stageOfNode[r] = stageIndex;
        }
        for (uint32_t i = 0; i < count; ++i) {
            if (!inKernel[i] || ctx.role[i] != Role::Materialized) continue;
            ctx.done[i] = 1;  // stored ones have a tensor now, the others are never materialised
            if (ctx.tensorOf[i].isInitialized()) ctx.stageOfNode[i] = stageIndex;
        }
        ctx.stages.push_back(std::move(stage));
    }
}

}  // namespace ThorImplementation
