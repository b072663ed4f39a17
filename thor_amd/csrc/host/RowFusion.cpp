#include "RowFusion.h"

#include "HipSourceEmitter.h"
#include "ReductionPlanner.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "thorhip_numeric_embed.h"

#include <algorithm>
#include <cstdlib>
#include <functional>
#include <map>
#include <numeric>
#include <set>
#include <sstream>

namespace ThorImplementation {

namespace {

using Role = RowFusionContext::Role;

// How a value relates to the row geometry P = [..., R] (rows = prod(P[:-1])).
enum class Cls : uint8_t {
    Other,       // not expressible per row
    RowVec,      // dims == P: one value per element
    RowScalarK,  // dims == P with the last dim 1 (reduced axis kept)
    RowScalarS,  // dims == P[:-1] (reduced axis squeezed)
    ColVec,      // dims == [R] right-aligned ([1,...,1,R]): one value per column, shared by all rows
    Scalar,      // one element
};

bool isElem(Cls c) { return c == Cls::RowVec || c == Cls::ColVec; }
bool isUniform(Cls c) { return c == Cls::RowScalarK || c == Cls::RowScalarS || c == Cls::Scalar; }
bool isShapeOnly(ExprOp op) { return op == ExprOp::RESHAPE || op == ExprOp::UNSQUEEZE || op == ExprOp::SQUEEZE; }

uint64_t product(const std::vector<uint64_t>& d) {
    uint64_t n = 1;
    for (uint64_t v : d) n *= v;
    return n;
}

Cls classifyDims(const std::vector<uint64_t>& dims, const std::vector<uint64_t>& P) {
    if (product(dims) == 1) return Cls::Scalar;
    if (dims == P) return Cls::RowVec;
    const uint64_t R = P.back();
    if (dims.size() == P.size() && dims.back() == 1 && std::equal(dims.begin(), dims.end() - 1, P.begin())) return Cls::RowScalarK;
    bool col = !dims.empty() && dims.size() <= P.size() && dims.back() == R;
    for (size_t i = 0; col && i + 1 < dims.size(); ++i) col = dims[i] == 1;
    const bool squeezed = dims.size() + 1 == P.size() && std::equal(dims.begin(), dims.end(), P.begin());
    if (col && squeezed) return Cls::Other;  // rows == R makes [R] ambiguous: leave such graphs to the staged path
    if (col) return Cls::ColVec;
    if (squeezed) return Cls::RowScalarS;
    return Cls::Other;
}

const char* accumulatorFor(ExprOp op, int& finalize) {
    finalize = 0;
    switch (op) {
        case ExprOp::REDUCE_SUM: return "thor::ValueAcc<thor::SumOp>";
        case ExprOp::REDUCE_AVG: finalize = 1; return "thor::ValueAcc<thor::SumOp>";
        case ExprOp::REDUCE_NORM1: return "thor::ValueAcc<thor::AbsSumOp>";
        case ExprOp::REDUCE_NORM2: finalize = 2; return "thor::ValueAcc<thor::SquareSumOp>";
        case ExprOp::REDUCE_PROD: return "thor::ValueAcc<thor::ProductOp>";
        case ExprOp::REDUCE_MIN: return "thor::ValueAcc<thor::MinOp>";
        case ExprOp::REDUCE_MAX: return "thor::ValueAcc<thor::MaxOp>";
        default: return nullptr;
    }
}

struct Region {
    std::vector<uint64_t> P;
    uint64_t rows = 0, R = 0;
    std::vector<Cls> cls;
    std::vector<char> computable;   // value can live inside the row kernel (source or computed)
    std::vector<char> isSource;     // read from a tensor
    std::vector<char> member;       // computed by the kernel
    std::vector<char> stored;       // member whose value is written to memory
    std::vector<uint32_t> reductions;
};

bool isLastAxisReduction(const ExprNode& n, const std::vector<uint64_t>& inDims) {
    if (!isValueReductionOp(n.op) || inDims.empty()) return false;
    if (n.reduction_axes.empty()) return inDims.size() == 1;
    if (n.reduction_axes.size() == 1 && n.reduction_axes[0] == kReduceAllAxesButFirst) return inDims.size() == 2;
    std::vector<uint64_t> axes = n.reduction_axes;
    std::sort(axes.begin(), axes.end());
    axes.erase(std::unique(axes.begin(), axes.end()), axes.end());
    return axes.size() == 1 && axes[0] == inDims.size() - 1;
}

// Classifies every node against P and marks what the row kernel can hold.
void analyse(const RowFusionContext& ctx, Region& rg) {
    const size_t count = ctx.expr.nodes.size();
    rg.cls.assign(count, Cls::Other);
    rg.computable.assign(count, 0);
    rg.isSource.assign(count, 0);
    for (uint32_t i = 0; i < count; ++i) {
        const ExprNode& n = ctx.expr.nodes[i];
        const std::vector<uint64_t>& d = ctx.dims[i];
        if (ctx.done[i]) {
            // produced by an earlier fused stage: usable as a tensor source if it has a tensor
            if (ctx.tensorOf[i].isInitialized() && ctx.tensorOf[i].isDenseContiguous()) {
                rg.cls[i] = classifyDims(d, rg.P);
                rg.computable[i] = rg.isSource[i] = rg.cls[i] != Cls::Other;
            }
            continue;
        }
        if (n.op == ExprOp::INPUT || (ctx.role[i] == Role::View && ctx.tensorOf[i].isInitialized())) {
            const Tensor& t = ctx.tensorOf[i];
            if (t.isInitialized() && t.isDenseContiguous()) {
                rg.cls[i] = classifyDims(d, rg.P);
                rg.computable[i] = rg.isSource[i] = rg.cls[i] != Cls::Other;
            }
            continue;
        }
        if (n.op == ExprOp::SCALAR_FP || n.op == ExprOp::RUNTIME_SCALAR) {
            rg.cls[i] = Cls::Scalar;
            rg.computable[i] = 1;
            continue;
        }
        if (n.op == ExprOp::FILL) {
            double folded;
            if (tryFoldConstant(ctx.expr, i, folded)) {
                rg.cls[i] = classifyDims(d, rg.P);
                rg.computable[i] = rg.cls[i] != Cls::Other;
            }
            continue;
        }
        if (isReductionOp(n.op)) {
            if (rg.computable[n.lhs] && rg.cls[n.lhs] == Cls::RowVec && isLastAxisReduction(n, ctx.dims[n.lhs])) {
                const Cls c = classifyDims(d, rg.P);
                if (c == Cls::RowScalarK || c == Cls::RowScalarS) {
                    rg.cls[i] = c;
                    rg.computable[i] = 1;
                }
            }
            continue;
        }
        if (isShapeOnly(n.op)) {
            // only the moves between the kept and the squeezed form of a per-row value keep their meaning inside a row
            if (rg.computable[n.lhs] && isUniform(rg.cls[n.lhs])) {
                const Cls c = classifyDims(d, rg.P);
                if (isUniform(c)) {
                    rg.cls[i] = c;
                    rg.computable[i] = 1;
                }
            }
            continue;
        }
        // elementwise
        if (!(Expression::isBinaryOp(n.op) || n.op == ExprOp::WHERE || (Expression::isUnaryOp(n.op) && !isReductionOp(n.op)))) continue;
        bool ok = true, anySqueezed = false, anyAligned = false;
        for (uint32_t c : {n.lhs, n.rhs, n.aux}) {
            if (c == UINT32_MAX) continue;
            ok = ok && rg.computable[c];
            anySqueezed = anySqueezed || rg.cls[c] == Cls::RowScalarS;
            anyAligned = anyAligned || rg.cls[c] == Cls::RowVec || rg.cls[c] == Cls::RowScalarK || rg.cls[c] == Cls::ColVec;
        }
        if (!ok || (anySqueezed && anyAligned)) continue;
        const Cls c = classifyDims(d.empty() ? std::vector<uint64_t>{1} : d, rg.P);
        if (c == Cls::Other) continue;
        rg.cls[i] = c;
        rg.computable[i] = 1;
    }
}

// Tensor-role nodes a value is computed from without crossing another tensor-role node.
void sourcesOf(const RowFusionContext& ctx, uint32_t root, std::vector<uint32_t>& out) {
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
        if (ctx.role[n] != Role::Inline) {
            out.push_back(n);
            continue;
        }
        const ExprNode& node = ctx.expr.nodes[n];
        for (uint32_t c : {node.lhs, node.rhs, node.aux})
            if (c != UINT32_MAX) stack.push_back(c);
    }
}

uint32_t viewBase(const RowFusionContext& ctx, uint32_t node) {
    while (ctx.role[node] == Role::View) node = ctx.expr.nodes[node].lhs;
    return node;
}

bool buildRegion(const RowFusionContext& ctx, Region& rg) {
    const size_t count = ctx.expr.nodes.size();
    analyse(ctx, rg);
    rg.reductions.clear();
    for (uint32_t i = 0; i < count; ++i)
        if (!ctx.done[i] && rg.computable[i] && isReductionOp(ctx.expr.nodes[i].op)) rg.reductions.push_back(i);
    if (rg.reductions.empty()) return false;

    // members: computed nodes connected to a reduction, upstream (they feed it) or downstream (they consume it)
    std::vector<char> feeds(count, 0), consumes(count, 0);
    for (uint32_t r : rg.reductions) feeds[r] = consumes[r] = 1;
    for (uint32_t i = static_cast<uint32_t>(count); i-- > 0;) {
        if (!feeds[i]) continue;
        const ExprNode& n = ctx.expr.nodes[i];
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != UINT32_MAX && rg.computable[c] && !rg.isSource[c]) feeds[c] = 1;
    }
    for (uint32_t i = 0; i < count; ++i) {
        if (consumes[i] || !rg.computable[i] || rg.isSource[i]) continue;
        const ExprNode& n = ctx.expr.nodes[i];
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != UINT32_MAX && consumes[c]) consumes[i] = 1;
    }
    rg.member.assign(count, 0);
    for (uint32_t i = 0; i < count; ++i) {
        rg.member[i] = rg.computable[i] && !rg.isSource[i] && !ctx.done[i] && (feeds[i] || consumes[i]);
    }
    // a member must only depend on sources and members (feeds/consumes closure can leave out constants: pull them in)
    bool changed = true;
    while (changed) {
        changed = false;
        for (uint32_t i = 0; i < count; ++i) {
            if (!rg.member[i]) continue;
            const ExprNode& n = ctx.expr.nodes[i];
            for (uint32_t c : {n.lhs, n.rhs, n.aux}) {
                if (c == UINT32_MAX || rg.member[c] || rg.isSource[c]) continue;
                if (rg.computable[c] && !ctx.done[c]) {
                    rg.member[c] = 1;
                    changed = true;
                }
            }
        }
    }
    // views of inputs that classify as sources must already have tensors; every other dependency must be a member
    for (uint32_t i = 0; i < count; ++i) {
        if (!rg.member[i]) continue;
        const ExprNode& n = ctx.expr.nodes[i];
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != UINT32_MAX && !rg.member[c] && !rg.isSource[c]) return false;
    }

    // which materialised members have to reach memory: named outputs (also through views) and everything a stage
    // outside the region reads
    rg.stored.assign(count, 0);
    for (const NamedOutput& o : ctx.outputs) {
        const uint32_t base = viewBase(ctx, o.node_idx);
        if (rg.member[base] && ctx.role[base] == Role::Materialized) rg.stored[base] = 1;
    }
    for (uint32_t i = 0; i < count; ++i) {
        if (rg.member[i] || ctx.done[i]) continue;
        if (ctx.role[i] != Role::Materialized && ctx.role[i] != Role::View) continue;
        std::vector<uint32_t> src;
        if (ctx.role[i] == Role::View || isReductionOp(ctx.expr.nodes[i].op)) {
            src.push_back(ctx.expr.nodes[i].lhs);
        } else {
            sourcesOf(ctx, i, src);
        }
        for (uint32_t s : src) {
            const uint32_t base = viewBase(ctx, s);
            if (rg.member[base] && ctx.role[base] == Role::Materialized) rg.stored[base] = 1;
        }
    }
    // a member view that is itself outside-visible is handled through its base above; members that are views of
    // members stay aliases inside the kernel
    bool anyStored = false, anyElemMember = false;
    size_t memberReductions = 0;
    for (uint32_t i = 0; i < count; ++i) {
        anyStored = anyStored || rg.stored[i];
        anyElemMember = anyElemMember || (rg.member[i] && isElem(rg.cls[i]));
        memberReductions += rg.member[i] && isReductionOp(ctx.expr.nodes[i].op);
    }
    // One reduction of a tensor that already exists is what the stand-alone reduction kernels are tuned for (they can
    // split long rows over blocks).  Keeping rows on chip pays when it removes a materialised per-element value or a
    // second pass over the input.
    return anyStored && (anyElemMember || memberReductions >= 2);
}

struct Emission {
    std::string source;
    std::vector<uint32_t> sourceNodes;   // kernel operand order
    std::vector<uint32_t> scalarSlots;
    std::vector<uint32_t> storedNodes;   // kernel output order
    uint32_t threads = 256, gridX = 1;
    bool fastContract = true;
    uint64_t flops = 0;
    std::string description;
};

bool emitRegion(const RowFusionContext& ctx, const Region& rg, Emission& em) {
    const PhysicalExpression& expr = ctx.expr;
    const size_t count = expr.nodes.size();
    std::vector<uint32_t> members;
    for (uint32_t i = 0; i < count; ++i)
        if (rg.member[i]) members.push_back(i);

    // sources actually read by members; runtime scalars
    std::set<uint32_t> sourceSet, scalarSet;
    for (uint32_t m : members) {
        const ExprNode& n = expr.nodes[m];
        if (n.op == ExprOp::RUNTIME_SCALAR) scalarSet.insert(n.input_slot);
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != UINT32_MAX && rg.isSource[c]) sourceSet.insert(c);
    }
    em.sourceNodes.assign(sourceSet.begin(), sourceSet.end());
    em.scalarSlots.assign(scalarSet.begin(), scalarSet.end());
    for (uint32_t m : members)
        if (rg.stored[m]) em.storedNodes.push_back(m);

    // vector width: one 16-byte word of the widest streamed element type per lane (at least four elements); with bf16 in
    // and fp32 out that is an 8-byte load and a 16-byte store, measured 17 % faster than 16-byte loads with 32-byte stores
    uint32_t narrow = 8, wide = 1;
    auto consider = [&](DataType dt) {
        narrow = std::min(narrow, dataTypeSizeInBytes(dt));
        wide = std::max(wide, dataTypeSizeInBytes(dt));
    };
    for (uint32_t s : em.sourceNodes)
        if (isElem(rg.cls[s])) consider(ctx.tensorOf[s].getDataType());
    for (uint32_t m : em.storedNodes)
        if (isElem(rg.cls[m])) consider(expr.nodes[m].output_dtype.value());
    if (narrow > wide) return false;  // nothing streamed per element: not worth a row kernel
    int vec = static_cast<int>(std::max<uint32_t>(16 / wide, std::min<uint32_t>(4, 16 / narrow)));
    const int wantedVec = vec;
    while (vec > 1 && rg.R % vec != 0) vec /= 2;
    // pointers of existing tensors must allow the vector accesses (fresh allocations are 256-byte aligned)
    for (uint32_t s : em.sourceNodes) {
        if (!isElem(rg.cls[s])) continue;
        const uint64_t align = pointerAlignment(ctx.tensorOf[s].getMemPtr());
        while (vec > 1 && align % std::min<uint64_t>(16, static_cast<uint64_t>(vec) * dataTypeSizeInBytes(ctx.tensorOf[s].getDataType())) != 0) vec /= 2;
    }
    // A row length (or a pointer) that the vector does not fit: the lanes keep the full vector, read and written at addresses
    // that are only aligned to the element; the row's last vector overlaps the one before it (rows of 1001 or 50257).
    bool unaligned = false;
    if (vec < wantedVec && rg.R >= 4ull * static_cast<uint64_t>(wantedVec)) {
        vec = wantedVec;
        unaligned = true;
    }
    const uint64_t tail = rg.R % static_cast<uint64_t>(vec);
    // ---- phases ---------------------------------------------------------------------------------------------------------
    // elem nodes get the loop they are computed in; uniform nodes get the number of folds that must have happened
    std::vector<int> phase(count, 0);
    int lastElemPhase = 0;
    for (uint32_t m : members) {
        const ExprNode& n = expr.nodes[m];
        int p = 0;
        for (uint32_t c : {n.lhs, n.rhs, n.aux}) {
            if (c == UINT32_MAX || !rg.member[c]) continue;
            p = std::max(p, phase[c]);
        }
        if (isReductionOp(n.op)) {
            phase[m] = (rg.member[n.lhs] ? phase[n.lhs] : 0) + 1;  // available after the fold that follows its operand's loop
        } else {
            phase[m] = p;
        }
        if (isElem(rg.cls[m])) lastElemPhase = std::max(lastElemPhase, phase[m]);
    }
    int numLoops = lastElemPhase + 1;
    for (uint32_t r : rg.reductions)
        if (rg.member[r]) numLoops = std::max(numLoops, phase[r]);  // a loop must exist for every operand

    // elem values that cross loops are kept in register arrays
    std::vector<char> needsArray(count, 0);
    for (uint32_t m : members) {
        if (!isElem(rg.cls[m])) continue;
        const ExprNode& n = expr.nodes[m];
        for (uint32_t c : {n.lhs, n.rhs, n.aux})
            if (c != UINT32_MAX && rg.member[c] && isElem(rg.cls[c]) && phase[c] < phase[m]) needsArray[c] = 1;
    }

    // ---- lanes per row ---------------------------------------------------------------------------------------------------
    // about eight vectors per lane, more lanes when the row's registers (the loaded row plus every per-element value
    // that has to survive a fold) would not fit the budget a block of that size leaves per lane
    const uint64_t vectors = (rg.R + vec - 1) / vec;  // the last one is partial when tail != 0
    auto budget = [](uint64_t lanes) { return lanes <= 512 ? 160.0 : 96.0; };
    // Measured on MI355X (softmax and normalisation, rows of 128 to 8192 elements): two 16-byte vectors per lane up to one
    // 256-thread block per row is fastest; longer rows then take more vectors per lane until the row data reaches about
    // 64 registers, and only after that more lanes.
    const double softTarget = 64.0;
    const uint64_t vectorsPerLane = narrow < wide ? 4 : 2;  // narrow-side words are half words: take twice as many
    uint64_t T = 1, items = 0;
    auto sizeBlock = [&](bool withArrays) {
        double registersPerElement = 0.0;
        for (uint32_t sNode : em.sourceNodes)
            if (isElem(rg.cls[sNode])) registersPerElement += dataTypeSizeInBytes(ctx.tensorOf[sNode].getDataType()) / 4.0;
        for (uint32_t m : members) {
            if (!withArrays || !needsArray[m]) continue;
            const DataType dt = ctx.role[m] == Role::Materialized ? expr.nodes[m].output_dtype.value() : emittedValueDType(expr.nodes[m]);
            registersPerElement += std::max(1.0, dataTypeSizeInBytes(dt) / 4.0);  // 16-bit values sit in registers of their own
        }
        T = 1;
        while (T < 256 && T * vectorsPerLane < vectors) T <<= 1;
        while (T < 1024 && T < vectors && (vectors + T - 1) / T * vec * registersPerElement > softTarget) T <<= 1;
        while (T < 1024 && ((vectors + T - 1) / T * vec > 64 || (vectors + T - 1) / T * vec * registersPerElement > budget(T))) T <<= 1;
        if (const char* forced = std::getenv("THOR_ROW_THREADS")) {  // tuning switch: lanes per row (a power of two up to 1024)
            const uint64_t wanted = static_cast<uint64_t>(std::max(1, std::atoi(forced)));
            if ((wanted & (wanted - 1)) == 0 && wanted <= 1024 && (vectors + wanted - 1) / wanted * vec <= 64) T = wanted;
        }
        items = (vectors + T - 1) / T;
        return !(items * vec > 64 || items * vec * registersPerElement > budget(T));
    };
    // A row whose values would not fit next to it keeps only the row itself in registers: values that a later loop needs are
    // computed again there from the row (every per-element value is a function of the sources and of per-row values) -- for
    // softmax a second exponential per element instead of a register per element.
    bool recompute = false;
    if (!sizeBlock(true)) {
        if (!sizeBlock(false)) return false;  // the row does not fit one block's registers
        recompute = true;
        std::fill(needsArray.begin(), needsArray.end(), 0);
    }
    const bool subWave = T <= 64;
    const uint64_t threads = subWave ? 256 : T;
    const uint64_t rowsPerBlock = subWave ? 256 / T : 1;
    // A block that owns a row spends part of its life in folds and barriers with no load in flight.  THOR_ROW_TURNS (a tuning
    // switch) makes it take that many consecutive rows in turn, the loads of the next row issued before it works on the current
    // one (the row's sources are the only registers that double).  Measured, it loses: eight resident blocks per compute unit
    // already overlap one block's folds with the others' loads, and fewer, longer blocks overlap less - softmax bf16
    // [16384, 4096] 68 / 71 / 78 / 87 us with 1 / 2 / 4 / 8 rows in turn, normalisation fp32 [32768, 1024] 44.5 / 46.7 / 50.7 /
    // 51.6 us.  So the default is one row per block.
    uint64_t turns = 1;
    if (const char* forced = std::getenv("THOR_ROW_TURNS")) turns = subWave ? 1 : static_cast<uint64_t>(std::max(1, std::atoi(forced)));
    turns = std::min<uint64_t>(turns, std::max<uint64_t>(rg.rows / 2048, 1));  // not at the price of an idle compute unit
    for (uint32_t sNode : em.sourceNodes)
        if (rg.cls[sNode] == Cls::ColVec) turns = 1;  // operands shared by all rows are loaded once, ahead of everything
    const bool inTurns = turns > 1;
    em.threads = static_cast<uint32_t>(threads);
    em.gridX = static_cast<uint32_t>((rg.rows + rowsPerBlock * turns - 1) / (rowsPerBlock * turns));

    em.fastContract = true;
    for (uint32_t m : members) {
        const ExprNode& n = expr.nodes[m];
        if (!Expression::isLeafOp(n.op) && (n.compute_dtype == DataType::FP16 || n.compute_dtype == DataType::BF16)) em.fastContract = false;
    }
    // reductions fix their own accumulation order; contraction inside the elementwise part does not reorder them

    std::ostringstream s;
    s << thor_embed::kDevicePrelude;
    s << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void fused_row_kernel(";
    for (size_t o = 0; o < em.sourceNodes.size(); ++o) s << "const " << deviceTypeName(ctx.tensorOf[em.sourceNodes[o]].getDataType()) << "* in" << o << ", ";
    for (uint32_t slot : em.scalarSlots) s << "float s" << slot << ", ";
    for (size_t o = 0; o < em.storedNodes.size(); ++o) {
        s << deviceTypeName(expr.nodes[em.storedNodes[o]].output_dtype.value()) << "* out" << o << (o + 1 < em.storedNodes.size() ? ", " : "");
    }
    s << ") {\n";
    s << "    constexpr int T = " << T << ", V = " << vec << ", ITEMS = " << items << ";\n";
    s << "    constexpr unsigned long long R = " << rg.R << "ull, ROWS = " << rg.rows << "ull, VECTORS = " << vectors << "ull;\n";
    if (subWave) {
        s << "    const unsigned long long row = (unsigned long long)thor::xcdBlock<" << xcdRunLength(1) << ">(blockIdx.x, gridDim.x) * " << rowsPerBlock
          << "ull + threadIdx.x / T;\n";
        s << "    const int lane = threadIdx.x % T;\n";
    } else if (inTurns) {
        s << "    constexpr int TURNS = " << turns << ";\n";
        s << "    const unsigned long long firstRow = (unsigned long long)thor::xcdBlock<" << xcdRunLength(1) << ">(blockIdx.x, gridDim.x) * TURNS;\n"
             "    const int lane = threadIdx.x;\n";
    } else {
        s << "    const unsigned long long row = thor::xcdBlock<" << xcdRunLength(1) << ">(blockIdx.x, gridDim.x);\n    const int lane = threadIdx.x;\n";
    }
    // when every lane of every block has a whole vector of a real row, the bounds checks vanish at compile time
    const bool allLive = vectors % T == 0 && rg.rows % (rowsPerBlock * turns) == 0 && tail == 0;
    const std::string liveIf = allLive ? "" : "if (live[it]) ";
    // what depends on the row: emitted once, or at the top of every turn
    const std::string rowLines =
        std::string("    const bool rowLive = row < ROWS;\n    const unsigned long long rowIndex = rowLive ? row : 0ull;\n"
                    "    const unsigned long long rowBase = rowIndex * R;\n    bool live[ITEMS];\n"
                    "#pragma unroll\n    for (int it = 0; it < ITEMS; ++it) live[it] = rowLive && (unsigned long long)it * T + lane < VECTORS;\n");
    s << "    unsigned long long column[ITEMS];\n";
    s << "#pragma unroll\n    for (int it = 0; it < ITEMS; ++it) {\n        const unsigned long long v = (unsigned long long)it * T + lane;\n"
         "        column[it] = (v < VECTORS ? v : 0ull) * V;\n    }\n";
    if (!inTurns) s << rowLines;
    if (tail != 0) {
        // The row's last vector is read (and written) V - tail elements early, so that it ends with the row: it overlaps the
        // vector before it, folds skip the elements it shares with that one, and the stores write those twice with the same bits.
        s << "    int skip[ITEMS];\n#pragma unroll\n    for (int it = 0; it < ITEMS; ++it) {\n"
             "        const unsigned long long v = (unsigned long long)it * T + lane;\n"
             "        skip[it] = v + 1 == VECTORS ? " << (vec - tail) << " : 0;\n"
             "        if (v + 1 == VECTORS) column[it] = R - V;\n    }\n";
    }
    auto loadItem = [&](const std::string& pack, const std::string& address, bool stream) {
        return "        " + liveIf + pack + (unaligned ? (stream ? ".loadStreamUnaligned(" : ".loadUnaligned(") : (stream ? ".loadStream(" : ".load(")) + address + ");\n";
    };
    auto storeItem = [&](const std::string& pack, const std::string& address) {
        return "        " + liveIf + pack + ".storeStream(" + address + ");\n";  // the store instruction takes any alignment
    };

    // sources
    std::map<uint32_t, size_t> sourceIndex;
    for (size_t o = 0; o < em.sourceNodes.size(); ++o) sourceIndex[em.sourceNodes[o]] = o;
    BodyEmitter uniform(expr);  // values that exist once per row (function scope)
    std::string turnPrefetch, turnHandOver, turnUniform;  // in turns: the next row's loads, p = next, the row's own scalars
    for (size_t o = 0; o < em.sourceNodes.size(); ++o) {
        const uint32_t node = em.sourceNodes[o];
        const DataType storage = ctx.tensorOf[node].getDataType();
        const DataType valueDType = expr.nodes[node].output_dtype.value();
        const char* type = deviceTypeName(storage);
        if (isElem(rg.cls[node]) && inTurns && rg.cls[node] == Cls::RowVec) {
            // the first row's loads here; every turn then issues the next row's before it works on its own
            const std::string pack = "p" + std::to_string(o), in = "in" + std::to_string(o);
            const std::string guard = allLive ? "" : "if (firstRow < ROWS && (unsigned long long)it * T + lane < VECTORS) ";
            s << "    thor::Pack<" << type << ", V> " << pack << "[ITEMS];\n";
            s << "#pragma unroll\n    for (int it = 0; it < ITEMS; ++it) {\n        " << pack << "[it] = {};\n        " << guard << pack << "[it]"
              << (unaligned ? ".loadStreamUnaligned(" : ".loadStream(") << in << " + firstRow * R + column[it]);\n    }\n";
            const std::string nextGuard = allLive ? "if (turn + 1 < TURNS) " : "if (turn + 1 < TURNS && row + 1 < ROWS && (unsigned long long)it * T + lane < VECTORS) ";
            turnPrefetch += "    thor::Pack<" + std::string(type) + ", V> n" + pack + "[ITEMS];\n#pragma unroll\n    for (int it = 0; it < ITEMS; ++it) {\n        n" + pack +
                            "[it] = {};\n        " + nextGuard + "n" + pack + "[it]" + (unaligned ? ".loadStreamUnaligned(" : ".loadStream(") + in +
                            " + (row + 1) * R + column[it]);\n    }\n";
            turnHandOver += "#pragma unroll\n    for (int it = 0; it < ITEMS; ++it) " + pack + "[it] = n" + pack + "[it];\n";
        } else if (isElem(rg.cls[node])) {
            s << "    thor::Pack<" << type << ", V> p" << o << "[ITEMS];\n";
            s << "#pragma unroll\n    for (int it = 0; it < ITEMS; ++it) {\n        p" << o << "[it] = {};\n";
            if (rg.cls[node] == Cls::RowVec) {
                s << loadItem("p" + std::to_string(o) + "[it]", "in" + std::to_string(o) + " + rowBase + column[it]", true);
            } else {
                s << loadItem("p" + std::to_string(o) + "[it]", "in" + std::to_string(o) + " + column[it]", false);
            }
            s << "    }\n";
        } else {
            const std::string index = rg.cls[node] == Cls::Scalar ? "0" : "rowIndex";
            std::string value = castValueExpr(storageToValueExpr("in" + std::to_string(o) + "[" + index + "]", storage), storage, valueDType);
            const std::string line = "    const " + std::string(valueCType(valueDType)) + " t" + std::to_string(node) + " = " + value + ";\n";
            if (inTurns) {
                turnUniform += line;
            } else {
                s << line;
            }
            uniform.defineSource(node, valueDType);
        }
    }
    if (inTurns) {
        s << "#pragma unroll 1\n    for (int turn = 0; turn < TURNS; ++turn) {\n    const unsigned long long row = firstRow + turn;\n" << rowLines << turnPrefetch
          << turnUniform;
    }

    auto isStoredOutput = [&](uint32_t node) { return rg.stored[node] != 0; };
    std::map<uint32_t, size_t> outputIndex;
    for (size_t o = 0; o < em.storedNodes.size(); ++o) outputIndex[em.storedNodes[o]] = o;

    // uniform members in evaluation order, emitted once their fold count is reached
    auto emitUniformUpTo = [&](int foldsDone) {
        std::string text;
        for (uint32_t m : members) {
            if (!isUniform(rg.cls[m]) || isReductionOp(expr.nodes[m].op) || uniform.defined(m) || phase[m] > foldsDone) continue;
            double folded;
            if (tryFoldConstant(expr, m, folded)) continue;
            bool ready = true;
            for (uint32_t c : {expr.nodes[m].lhs, expr.nodes[m].rhs, expr.nodes[m].aux}) {
                if (c == UINT32_MAX) continue;
                double f2;
                if (!uniform.defined(c) && !tryFoldConstant(expr, c, f2)) ready = false;
            }
            if (!ready) continue;
            em.flops += uniform.emit(text, m, "    ");
            if (ctx.role[m] == Role::Materialized) {
                const DataType outDType = expr.nodes[m].output_dtype.value();
                if (uniform.dtypeOf(m) != outDType) {
                    text += "    const " + std::string(valueCType(outDType)) + " m" + std::to_string(m) + " = " + uniform.ref(m, outDType) + ";\n";
                    uniform.defineSource(m, outDType, "m" + std::to_string(m));
                }
            }
            if (isStoredOutput(m)) {
                const DataType outDType = expr.nodes[m].output_dtype.value();
                text += "    if (lane == 0 && rowLive) out" + std::to_string(outputIndex[m]) + "[row] = " +
                        valueToStorageExpr(uniform.ref(m, outDType), outDType) + ";\n";
            }
        }
        s << text;
    };
    emitUniformUpTo(0);

    for (uint32_t m : members) {
        if (needsArray[m]) {
            const DataType dt = ctx.role[m] == Role::Materialized ? expr.nodes[m].output_dtype.value() : emittedValueDType(expr.nodes[m]);
            s << "    " << valueCType(dt) << " v" << m << "[ITEMS][V];\n";
        }
    }

    std::map<uint32_t, std::string> rowDivisorOf;
    for (int loop = 0; loop < numLoops; ++loop) {
        // reductions whose operand is produced in this loop
        std::vector<uint32_t> folding;
        for (uint32_t r : rg.reductions) {
            if (!rg.member[r]) continue;
            const uint32_t operand = expr.nodes[r].lhs;
            const int operandLoop = rg.member[operand] ? phase[operand] : 0;
            if (operandLoop == loop) folding.push_back(r);
        }
        for (uint32_t r : folding) {
            int fin;
            s << "    " << accumulatorFor(expr.nodes[r].op, fin) << " acc" << r << ";\n    acc" << r << ".reset();\n";
        }
        std::vector<uint32_t> elemNodes;
        for (uint32_t m : members)
            if (isElem(rg.cls[m]) && phase[m] == loop) elemNodes.push_back(m);

        // fp32 divisions of per-element values by a per-row value: one reciprocal per row
        for (uint32_t m : elemNodes) {
            const ExprNode& n = expr.nodes[m];
            if (n.op != ExprOp::DIV || n.compute_dtype != DataType::FP32 || !uniform.defined(n.rhs) || rowDivisorOf.count(n.rhs)) continue;
            const std::string name = "d" + std::to_string(n.rhs);
            s << "    const thor::RowDivisor " << name << "(" << uniform.ref(n.rhs, DataType::FP32) << ");\n";
            rowDivisorOf[n.rhs] = name;
        }
        // The next row's registers are taken over before the last loop when that loop reads no source: the wait for those loads
        // then comes before this turn's stores are issued and does not have to sit through them.
        bool lastLoopReadsSources = recompute;
        for (uint32_t m : elemNodes)
            for (uint32_t c : {expr.nodes[m].lhs, expr.nodes[m].rhs, expr.nodes[m].aux})
                if (c != UINT32_MAX && rg.isSource[c] && rg.cls[c] == Cls::RowVec) lastLoopReadsSources = true;
        if (inTurns && loop == numLoops - 1 && !lastLoopReadsSources) {
            s << turnHandOver;
            turnHandOver.clear();
        }
        s << "#pragma unroll\n    for (int it = 0; it < ITEMS; ++it) {\n";
        std::vector<uint32_t> storedHere;
        for (uint32_t m : elemNodes)
            if (isStoredOutput(m)) storedHere.push_back(m);
        for (uint32_t m : storedHere) {
            s << "        thor::Pack<" << deviceTypeName(expr.nodes[m].output_dtype.value()) << ", V> q" << outputIndex[m] << ";\n";
        }
        BodyEmitter body(expr);
        // everything uniform that has been defined is visible; elem sources and earlier elem values are extracted on demand
        for (uint32_t i = 0; i < count; ++i)
            if (uniform.defined(i)) body.defineSource(i, uniform.dtypeOf(i), uniform.nameOf(i));
        for (const auto& [node, name] : rowDivisorOf) body.defineRowDivisor(node, name);
        std::string text;
        std::set<uint32_t> extracted;
        std::function<void(uint32_t)> extractRef;
        auto extract = [&](uint32_t c) {
            if (c == UINT32_MAX || body.defined(c) || extracted.count(c)) return;
            if (rg.isSource[c] && isElem(rg.cls[c])) {
                const size_t o = sourceIndex.at(c);
                const DataType storage = ctx.tensorOf[c].getDataType();
                const DataType valueDType = expr.nodes[c].output_dtype.value();
                const std::string value = castValueExpr(storageToValueExpr("p" + std::to_string(o) + "[it].v[k]", storage), storage, valueDType);
                text += "            const " + std::string(valueCType(valueDType)) + " t" + std::to_string(c) + " = " + value + ";\n";
                body.defineSource(c, valueDType);
                extracted.insert(c);
            } else if (rg.member[c] && isElem(rg.cls[c]) && phase[c] < loop && !recompute) {
                const DataType dt = ctx.role[c] == Role::Materialized ? expr.nodes[c].output_dtype.value() : emittedValueDType(expr.nodes[c]);
                text += "            const " + std::string(valueCType(dt)) + " t" + std::to_string(c) + " = v" + std::to_string(c) + "[it][k];\n";
                body.defineSource(c, dt);
                extracted.insert(c);
            } else if (rg.member[c] && isElem(rg.cls[c]) && phase[c] < loop) {
                // computed again from the row: the same statements as in its own loop (and the same rounding where it is stored)
                const ExprNode& n = expr.nodes[c];
                for (uint32_t child : {n.lhs, n.rhs, n.aux}) extractRef(child);
                double folded;
                if (tryFoldConstant(expr, c, folded)) {
                    const DataType dt = emittedValueDType(n);
                    text += "            const " + std::string(valueCType(dt)) + " t" + std::to_string(c) + " = " + castValueExpr(floatLiteral(folded), DataType::FP32, dt) + ";\n";
                    body.defineSource(c, dt);
                } else {
                    em.flops += body.emit(text, c, "            ") * rg.R;
                }
                if (ctx.role[c] == Role::Materialized) {
                    const DataType outDType = n.output_dtype.value();
                    if (body.dtypeOf(c) != outDType) {
                        text += "            const " + std::string(valueCType(outDType)) + " m" + std::to_string(c) + " = " + body.ref(c, outDType) + ";\n";
                        body.defineSource(c, outDType, "m" + std::to_string(c));
                    }
                }
                extracted.insert(c);
            }
        };
        extractRef = extract;
        for (uint32_t m : elemNodes) {
            const ExprNode& n = expr.nodes[m];
            for (uint32_t c : {n.lhs, n.rhs, n.aux}) extract(c);
            double folded;
            if (tryFoldConstant(expr, m, folded)) {
                const DataType dt = emittedValueDType(n);
                text += "            const " + std::string(valueCType(dt)) + " t" + std::to_string(m) + " = " +
                        castValueExpr(floatLiteral(folded), DataType::FP32, dt) + ";\n";
                body.defineSource(m, dt);
            } else {
                em.flops += body.emit(text, m, "            ") * rg.R;
            }
            if (ctx.role[m] == Role::Materialized) {
                const DataType outDType = n.output_dtype.value();
                if (body.dtypeOf(m) != outDType) {
                    text += "            const " + std::string(valueCType(outDType)) + " m" + std::to_string(m) + " = " + body.ref(m, outDType) + ";\n";
                    body.defineSource(m, outDType, "m" + std::to_string(m));
                }
            }
            if (needsArray[m]) text += "            v" + std::to_string(m) + "[it][k] = " + body.nameOf(m) + ";\n";
            if (isStoredOutput(m)) {
                const DataType outDType = n.output_dtype.value();
                text += "            q" + std::to_string(outputIndex[m]) + ".v[k] = " + valueToStorageExpr(body.ref(m, outDType), outDType) + ";\n";
            }
        }
        for (uint32_t r : folding) {
            const uint32_t operand = expr.nodes[r].lhs;
            extract(operand);
            text += "            a" + std::to_string(r) + "[k] = " + body.ref(operand, DataType::FP32) + ";\n";
            em.flops += rg.R;
        }
        for (uint32_t r : folding) s << "        float a" << r << "[V];\n";
        s << "#pragma unroll\n        for (int k = 0; k < V; ++k) {\n";
        s << text;
        s << "        }\n";
        if (!folding.empty()) {
            // one bounds decision per vector, not per element
            if (tail == 0) {
                s << "        " << liveIf << "{\n#pragma unroll\n            for (int k = 0; k < V; ++k) {\n";
                for (uint32_t r : folding) s << "                acc" << r << ".add(a" << r << "[k], 0u);\n";
                s << "            }\n        }\n";
            } else {
                s << "#pragma unroll\n        for (int k = 0; k < V; ++k) {\n            if (live[it] && k >= skip[it]) {\n";
                for (uint32_t r : folding) s << "                acc" << r << ".add(a" << r << "[k], 0u);\n";
                s << "            }\n        }\n";
            }
        }
        for (uint32_t m : storedHere) {
            const Cls c = rg.cls[m];
            s << storeItem("q" + std::to_string(outputIndex[m]), "out" + std::to_string(outputIndex[m]) + " + " + (c == Cls::RowVec ? "rowBase + " : "") + "column[it]");
        }
        s << "    }\n";
        // fold the lanes that share the row, then the values that depend on the results
        for (uint32_t r : folding) {
            int fin = 0;
            (void)accumulatorFor(expr.nodes[r].op, fin);
            if (subWave) {
                s << "    thor::groupReduce<T>(acc" << r << ");\n";
            } else {
                s << "    __shared__ " << accumulatorFor(expr.nodes[r].op, fin) << " scratch" << r << "[T / thor::kWave];\n";
                s << "    thor::blockReduce<T, true>(acc" << r << ", scratch" << r << ");\n";
            }
            const DataType outDType = expr.nodes[r].output_dtype.value();
            s << "    const " << valueCType(outDType) << " t" << r << " = "
              << castValueExpr("thor::finalizeValue<" + std::to_string(fin) + ">(acc" + std::to_string(r) + ".v, (float)R, 1.0f)", DataType::FP32, outDType)
              << ";\n";
            uniform.defineSource(r, outDType);
            if (isStoredOutput(r)) {
                s << "    if (lane == 0 && rowLive) out" << outputIndex[r] << "[row] = " << valueToStorageExpr("t" + std::to_string(r), outDType) << ";\n";
            }
        }
        emitUniformUpTo(loop + 1);
    }
    if (inTurns) s << turnHandOver << "    }\n";
    s << "}\n";
    // every member must have been produced
    for (uint32_t m : members) {
        if (isUniform(rg.cls[m]) && !uniform.defined(m)) {
            double folded;
            if (!tryFoldConstant(expr, m, folded)) return false;
        }
    }
    em.source = s.str();
    em.flops *= rg.rows;
    em.description = "row_fused(rows=" + std::to_string(rg.rows) + ",R=" + std::to_string(rg.R) + ",lanes_per_row=" + std::to_string(T) +
                     ",items=" + std::to_string(items) + ",vec=" + std::to_string(vec) + (inTurns ? ",rows_in_turn=" + std::to_string(turns) : "") +
                     (unaligned ? ",unaligned_vectors" : "") + (recompute ? ",values_recomputed" : "") + ",loops=" + std::to_string(numLoops) + ")";
    return true;
}

}  // namespace

void tryRowFusion(RowFusionContext& ctx) {
    const PhysicalExpression& expr = ctx.expr;
    // candidate geometries: the input shape of every last-axis value reduction
    std::vector<std::vector<uint64_t>> geometries;
    for (uint32_t i = 0; i < expr.nodes.size(); ++i) {
        const ExprNode& n = expr.nodes[i];
        if (!isReductionOp(n.op) || ctx.done[i]) continue;
        const std::vector<uint64_t>& in = ctx.dims[n.lhs];
        if (!isLastAxisReduction(n, in) || in.size() < 2 || in.back() < 2) continue;
        if (std::find(geometries.begin(), geometries.end(), in) == geometries.end()) geometries.push_back(in);
    }
    for (const std::vector<uint64_t>& P : geometries) {
        Region rg;
        rg.P = P;
        rg.R = P.back();
        rg.rows = product(P) / rg.R;
        if (rg.rows < 2) continue;
        if (!buildRegion(ctx, rg)) continue;
        Emission em;
        if (!emitRegion(ctx, rg, em)) continue;

        std::shared_ptr<CompiledKernel> kernel = compileKernel(em.source, "fused_row_kernel", ctx.deviceNum, em.fastContract);
        std::vector<Tensor> inputs, outputs;
        for (uint32_t sNode : em.sourceNodes) inputs.push_back(ctx.tensorOf[sNode]);
        for (uint32_t m : em.storedNodes) {
            Tensor out = ctx.allocateFor(m);
            ctx.tensorOf[m] = out;
            outputs.push_back(out);
        }
        std::vector<size_t> inputArgIndex(inputs.size()), outputArgIndex(outputs.size());
        std::iota(inputArgIndex.begin(), inputArgIndex.end(), 0);
        size_t next = inputs.size();
        std::vector<StampedEquation::ScalarArgument> scalarArgs;
        for (uint32_t slot : em.scalarSlots) scalarArgs.push_back({ctx.rootInputs.at(slot).name, next++});
        for (size_t o = 0; o < outputs.size(); ++o) outputArgIndex[o] = next++;

        StampedExecutionStage stage;
        stage.kind = StampedExecutionStage::Kind::FusedRowKernel;
        stage.gpu_num = ctx.deviceNum;
        for (uint32_t sNode : em.sourceNodes) {
            const int st = ctx.stageOfNode[viewBase(ctx, sNode)];
            if (st >= 0) stage.dependency_stage_indices.push_back(static_cast<uint32_t>(st));
        }
        stage.kernel = std::make_shared<StampedEquation>(kernel, inputs, outputs, scalarArgs, inputArgIndex, outputArgIndex, next, false,
                                                         rg.rows * rg.R, false, em.gridX, em.threads, em.flops, em.description + " [" + kernel->kernelName + "]");
        const int stageIndex = static_cast<int>(ctx.stages.size());
        for (uint32_t i = 0; i < expr.nodes.size(); ++i) {
            if (!rg.member[i]) continue;
            if (ctx.role[i] == Role::Materialized) {
                ctx.done[i] = 1;
                ctx.stageOfNode[i] = stageIndex;
            }
        }
        ctx.stages.push_back(std::move(stage));
    }
}

}  // namespace ThorImplementation
