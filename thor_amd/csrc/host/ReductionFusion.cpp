#include "RowFusion.h"

#include "HipSourceEmitter.h"
#include "ReductionPlanner.h"

#include <algorithm>
#include <map>
#include <set>

namespace ThorImplementation {

namespace {

using Role = RowFusionContext::Role;

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

// Tensor-role nodes and runtime scalar slots a value is computed from without crossing another tensor-role node.
void sourcesOf(const RowFusionContext& ctx, uint32_t root, std::set<uint32_t>& tensors, std::set<uint32_t>& scalarSlots) {
    std::vector<char> seen(ctx.expr.nodes.size(), 0);
    std::vector<uint32_t> stack;
    const ExprNode& r = ctx.expr.nodes[root];
    for (uint32_t c : {r.lhs, r.rhs, r.aux})
        if (c != UINT32_MAX) stack.push_back(c);
    while (!stack.empty()) {
        const uint32_t n = stack.back();
        stack.pop_back();
        if (seen[n]) continue;
        seen[n] = 1;
        const ExprNode& node = ctx.expr.nodes[n];
        if (node.op == ExprOp::RUNTIME_SCALAR) {
            scalarSlots.insert(node.input_slot);
            continue;
        }
        if (ctx.role[n] != Role::Inline) {
            tensors.insert(n);
            continue;
        }
        for (uint32_t c : {node.lhs, node.rhs, node.aux})
            if (c != UINT32_MAX) stack.push_back(c);
    }
}

struct Candidate {
    uint32_t reduction;
    uint32_t operand;
    bool inlined;  // the operand is evaluated inside the reduction kernel instead of being materialised
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

    auto usableSource = [&](uint32_t node, const std::vector<uint64_t>& shape) {
        const Tensor& t = ctx.tensorOf[node];
        if (!t.isInitialized() || !t.isDenseContiguous()) return false;
        return ctx.dims[node] == shape || product(ctx.dims[node]) == 1;
    };

    // group key: (shape of the reduced value, reduced axes)
    typedef std::pair<std::vector<uint64_t>, std::vector<uint64_t>> Key;
    std::map<Key, std::vector<Candidate>> groups;
    for (uint32_t i = 0; i < count; ++i) {
        const ExprNode& n = expr.nodes[i];
        if (ctx.done[i] || !isValueReductionOp(n.op) || ctx.role[i] != Role::Materialized) continue;
        const uint32_t operand = n.lhs;
        const std::vector<uint64_t>& shape = ctx.dims[operand];
        if (shape.empty() || product(shape) < 2) continue;
        std::vector<uint64_t> axes = n.reduction_axes;
        if (axes.empty())
            for (uint64_t a = 0; a < shape.size(); ++a) axes.push_back(a);
        std::sort(axes.begin(), axes.end());
        axes.erase(std::unique(axes.begin(), axes.end()), axes.end());

        Candidate candidate{i, operand, false};
        if (ctx.tensorOf[operand].isInitialized()) {
            if (!ctx.tensorOf[operand].isDenseContiguous()) continue;
        } else {
            if (ctx.done[operand] || ctx.role[operand] != Role::Materialized || !isElementwise(expr.nodes[operand].op)) continue;
            if (isNamedOutput[operand]) continue;
            bool onlyReductions = true;
            for (uint32_t c : consumers[operand]) onlyReductions = onlyReductions && isValueReductionOp(expr.nodes[c].op) && !ctx.done[c];
            if (!onlyReductions) continue;
            std::set<uint32_t> tensors, scalarSlots;
            sourcesOf(ctx, operand, tensors, scalarSlots);
            bool ok = !tensors.empty();
            bool anyFullShape = false;
            for (uint32_t t : tensors) {
                ok = ok && usableSource(t, shape);
                anyFullShape = anyFullShape || ctx.dims[t] == shape;
            }
            if (!ok || !anyFullShape) continue;
            candidate.inlined = true;
        }
        groups[Key(shape, axes)].push_back(candidate);
    }

    // an inlined operand must be inlined by every reduction that consumes it: drop operands some consumer could not take
    std::map<uint32_t, size_t> inlinedConsumers;
    for (const auto& [key, group] : groups)
        for (const Candidate& c : group)
            if (c.inlined) ++inlinedConsumers[c.operand];
    auto fullyInlined = [&](uint32_t operand) { return inlinedConsumers[operand] == consumers[operand].size(); };

    const TensorPlacement gpuPlacement(TensorPlacement::MemDevices::GPU, ctx.deviceNum);
    for (auto& [key, allCandidates] : groups) {
        std::vector<Candidate> group;
        for (const Candidate& c : allCandidates)
            if (!c.inlined || fullyInlined(c.operand)) group.push_back(c);
        bool anyInlined = false;
        for (const Candidate& c : group) anyInlined = anyInlined || c.inlined;
        if (group.size() < 2 && !anyInlined) continue;  // a lone reduction of an existing tensor: the stand-alone path

        const std::vector<uint64_t>& shape = key.first;
        std::vector<uint32_t> axes32;
        for (uint64_t a : key.second) axes32.push_back(static_cast<uint32_t>(a));

        // kernel sources: every tensor the prologues read, in node order
        std::set<uint32_t> tensorSet, scalarSet;
        for (const Candidate& c : group) {
            if (c.inlined) {
                sourcesOf(ctx, c.operand, tensorSet, scalarSet);
            } else {
                tensorSet.insert(c.operand);
            }
        }
        const std::vector<uint32_t> sourceNodes(tensorSet.begin(), tensorSet.end());
        ReductionKernelRequest request;
        request.deviceNum = ctx.deviceNum;
        request.geometry = CubReduction::analyzeGeometry(shape, axes32);
        request.scalarSlots.assign(scalarSet.begin(), scalarSet.end());
        request.inputAlignmentBytes = 256;
        BodyEmitter body(expr);
        std::string text;
        for (uint32_t slot : request.scalarSlots) text += "        const float s" + std::to_string(slot) + " = s.s" + std::to_string(slot) + ";\n";
        std::vector<Tensor> inputs;
        std::map<uint32_t, size_t> sourceIndex;
        for (size_t i = 0; i < sourceNodes.size(); ++i) {
            const uint32_t node = sourceNodes[i];
            const Tensor& t = ctx.tensorOf[node];
            const bool scalar = ctx.dims[node] != shape;
            request.sources.push_back({t.getDataType(), scalar});
            if (!scalar) request.inputAlignmentBytes = std::min(request.inputAlignmentBytes, pointerAlignment(t.getMemPtr()));
            inputs.push_back(t);
            sourceIndex[node] = i;
            const DataType valueDType = expr.nodes[node].output_dtype.value();
            const std::string raw = scalar ? "l.z" + std::to_string(i) : "l.p" + std::to_string(i) + ".v[k]";
            text += "        const " + std::string(valueCType(valueDType)) + " t" + std::to_string(node) + " = " +
                    castValueExpr(storageToValueExpr(raw, t.getDataType()), t.getDataType(), valueDType) + ";\n";
            body.defineSource(node, valueDType);
        }
        uint64_t flopsPerElement = 0;
        std::vector<uint32_t> roots;
        for (const Candidate& c : group)
            if (c.inlined) roots.push_back(c.operand);
        for (uint32_t node : body.collect(roots)) flopsPerElement += body.emit(text, node, "        ");
        bool strictRounding = false;
        for (const Candidate& c : group) {
            const ExprNode& r = expr.nodes[c.reduction];
            ReductionKernelRequest::Value value;
            value.op = cubOpOf(r.op);
            value.outputDType = r.output_dtype.value();
            if (c.inlined) {
                // the staged plan would have stored the operand in its output dtype: round there before accumulating
                const DataType stored = expr.nodes[c.operand].output_dtype.value();
                value.expression = castValueExpr(body.ref(c.operand, stored), stored, DataType::FP32);
                strictRounding = true;
            } else {
                const size_t i = sourceIndex.at(c.operand);
                const DataType storage = inputs[i].getDataType();
                value.expression = castValueExpr(storageToValueExpr("l.p" + std::to_string(i) + ".v[k]", storage), storage, DataType::FP32);
            }
            request.values.push_back(value);
            ++flopsPerElement;
        }
        (void)strictRounding;
        request.prologue = text;
        request.inputDType = inputs.front().getDataType();

        ReductionLaunchPlan plan = buildReductionKernels(request);
        std::optional<Tensor> workspace;
        if (plan.workspaceBytes > 0) workspace = Tensor(gpuPlacement, TensorDescriptor(DataType::UINT8, {plan.workspaceBytes}));
        std::vector<Tensor> outputs;
        for (const Candidate& c : group) {
            Tensor out = ctx.allocateFor(c.reduction);
            ctx.tensorOf[c.reduction] = out;
            outputs.push_back(out);
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
        plan.variant = "fused_reduction(values=" + std::to_string(group.size()) + ",sources=" + std::to_string(sourceNodes.size()) + ") " + plan.variant;
        stage.fused_reduction = std::make_shared<StampedFusedReduction>(std::move(plan), inputs, scalarNames, outputs, workspace,
                                                                        flopsPerElement * product(shape));
        const int stageIndex = static_cast<int>(ctx.stages.size());
        for (const Candidate& c : group) {
            ctx.done[c.reduction] = 1;
            ctx.stageOfNode[c.reduction] = stageIndex;
            if (c.inlined) ctx.done[c.operand] = 1;  // never materialised
        }
        ctx.stages.push_back(std::move(stage));
    }
}

}  // namespace ThorImplementation
