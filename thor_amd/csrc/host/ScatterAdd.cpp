// Flat scatter-add: output[indices[i]] += updates[i] (the reference's contract: Utilities/Expression/FlatScatterAddKernel.h:17-30
// there, which sorts the destinations, reduces equal ones and applies the result with a sparse-vector library call).
//
// Here the destinations come from arg scans, so equal destinations sit next to each other in long runs (a running maximum
// changes rarely).  A wavefront first adds up every run of equal neighbouring destinations among its 64 elements with shuffles,
// then the last lane of each run issues one hardware fp32 atomic add; a row whose maximum never changes costs one atomic per
// wavefront instead of 64.  Sums of more than one wavefront's worth of values are added in the order the atomics arrive.
#include "ScatterAdd.h"

#include "ReductionPlanner.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "thorhip_numeric_embed.h"

#include <algorithm>
#include <sstream>
#include <utility>
#include <vector>
#include <stdexcept>

namespace ThorImplementation {

namespace {

std::string clearSource(uint64_t outputs, int clearVec) {
    std::ostringstream s;
    s << thor_embed::kDevicePrelude;
    s << "extern \"C\" __global__ __launch_bounds__(256) void thor_scatter_clear(float* __restrict__ out) {\n";
    s << "    const thor::u64 vector = (thor::u64)blockIdx.x * 256 + threadIdx.x;\n";
    s << "    if (vector >= " << outputs / clearVec << "ull) return;\n";
    s << "    thor::Pack<float, " << clearVec << "> zero = {};\n";
    s << "    zero.store(out + vector * " << clearVec << ");\n}\n";
    return s.str();
}

// offsetsType: empty = every update counts; else the updates outside [offsets[0], offsets[segments]) are skipped
std::string addSource(uint64_t updates, uint64_t outputs, const std::string& offsetsType, uint64_t segments, uint64_t stretch) {
    std::ostringstream s;
    s << thor_embed::kDevicePrelude;
    // x of the lane that CTRL names (a row shift or a row broadcast), 0 where there is no such lane or ROWS leaves the row out
    s << "template <int CTRL, int ROWS>\n__device__ __forceinline__ float thor_scatter_moved(float x) {\n";
    s << "    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, ROWS, 0xf, false));\n}\n";
    s << "extern \"C\" __global__ __launch_bounds__(256) void thor_scatter_add(const float* __restrict__ updates, const thor::u32* __restrict__ indices,\n";
    s << "                                                                   ";
    if (!offsetsType.empty()) s << "const " << offsetsType << "* __restrict__ offsets, ";
    s << "float* __restrict__ out) {\n";
    s << "    const int lane = threadIdx.x & 63;\n";
    if (!offsetsType.empty()) s << "    const thor::u64 first = (thor::u64)offsets[0], end = (thor::u64)offsets[" << segments << "];\n";
    // A wavefront owns a stretch of consecutive updates and walks it 64 at a time, the loads of four steps in flight.  The run
    // that reaches the end of a step is not added yet: its destination and partial sum are carried into the next step (both are
    // the same in every lane), joined with that step's first run when the destination continues, added otherwise.  A run then
    // costs one atomic per stretch it touches, however long it is.
    const std::string live = offsetsType.empty() ? "i < " + std::to_string(updates) + "ull" : "i < " + std::to_string(updates) + "ull && i >= first && i < end";
    s << "    constexpr int DEPTH = 4;\n";
    s << "    const thor::u64 wave = (thor::u64)blockIdx.x * 4 + (threadIdx.x >> 6);\n";
    s << "    const thor::u64 base = wave * " << stretch << "ull;\n";
    s << "    thor::u32 carriedKey = 0xffffffffu;\n    float carried = 0.0f;\n";
    s << "    for (thor::u64 step = 0; step < " << stretch / 64 << "ull; step += DEPTH) {\n";
    s << "        thor::u32 keys[DEPTH];\n        float values[DEPTH];\n";
    s << "#pragma unroll\n        for (int d = 0; d < DEPTH; ++d) {\n";
    s << "            const thor::u64 i = base + (step + d) * 64 + lane;\n";
    s << "            keys[d] = 0xffffffffu;\n            values[d] = 0.0f;\n";
    s << "            if (" << live << ") {\n                keys[d] = __builtin_nontemporal_load(indices + i);\n                values[d] = __builtin_nontemporal_load(updates + i);\n            }\n        }\n";
    s << "#pragma unroll\n        for (int d = 0; d < DEPTH; ++d) {\n";
    s << "            thor::u32 key = keys[d] < " << outputs << "ull ? keys[d] : 0xffffffffu;\n            float v = values[d];\n";
    // runs of equal neighbouring destinations inside the wavefront: bit l of `heads` = lane l starts a run
    s << "            const thor::u32 before = __shfl_up(key, 1);\n";
    s << "            const thor::u64 heads = __ballot(lane == 0 || before != key);\n";
    // the last head at or below this lane, from the 32-bit halves of the ballot (no 64-bit shift by a register amount: this
    // device gets those wrong when the amount sits in the last register a wavefront owns); lane 0 is always a head
    s << "            const thor::u32 headsLo = (thor::u32)heads, headsHi = (thor::u32)(heads >> 32);\n";
    s << "            const thor::u32 belowLo = lane >= 31 ? headsLo : headsLo & (0xffffffffu >> (31 - lane));\n";
    s << "            const thor::u32 belowHi = lane < 32 ? 0u : headsHi & (0xffffffffu >> (63 - lane));\n";
    s << "            const int start = belowHi ? 63 - __builtin_clz(belowHi) : 31 - __builtin_clz(belowLo);\n";
    // inclusive sums within each run, with data-parallel-primitive moves: 1, 2, 4, 8 lanes up inside rows of 16 (a lane without
    // a source receives 0), then the last lane of row 0 / 2 into row 1 / 3, then lane 31 into the upper half; a lane takes what
    // arrives only if its run reaches back that far
    s << "            { const float o = thor_scatter_moved<0x111, 0xf>(v); if (lane - 1 >= start) v += o; }\n";
    s << "            { const float o = thor_scatter_moved<0x112, 0xf>(v); if (lane - 2 >= start) v += o; }\n";
    s << "            { const float o = thor_scatter_moved<0x114, 0xf>(v); if (lane - 4 >= start) v += o; }\n";
    s << "            { const float o = thor_scatter_moved<0x118, 0xf>(v); if (lane - 8 >= start) v += o; }\n";
    s << "            { const float o = thor_scatter_moved<0x142, 0xa>(v); if ((lane & 16) != 0 && start < (lane & ~15)) v += o; }\n";
    s << "            { const float o = thor_scatter_moved<0x143, 0xc>(v); if (lane >= 32 && start < 32) v += o; }\n";
    // what the earlier steps carried: into this step's first run, or out to memory
    s << "            const thor::u32 firstKey = (thor::u32)__builtin_amdgcn_readfirstlane((int)key);\n";
    s << "            if (firstKey == carriedKey) {\n                if (start == 0) v += carried;\n";
    s << "            } else if (carriedKey != 0xffffffffu && lane == 0) {\n                unsafeAtomicAdd(out + carriedKey, carried);\n            }\n";
    s << "            carriedKey = (thor::u32)__builtin_amdgcn_readlane((int)key, 63);\n";
    s << "            carried = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));\n";
    s << "            const bool last = lane != 63 && (((lane + 1 < 32 ? headsLo : headsHi) >> ((lane + 1) & 31)) & 1u) != 0;\n";
    s << "            if (last && key != 0xffffffffu) unsafeAtomicAdd(out + key, v);\n        }\n    }\n";
    s << "    if (carriedKey != 0xffffffffu && lane == 0) unsafeAtomicAdd(out + carriedKey, carried);\n}\n";
    return s.str();
}

void requireDense(const Tensor& t, DataType dtype, const char* what) {
    if (!t.isInitialized() || !t.isDenseContiguous() || t.getDataType() != dtype) {
        throw std::runtime_error(std::string("Scatter-add requires a dense ") + dataTypeName(dtype) + " " + what + " tensor.");
    }
}

int clearVectorOf(const Tensor& output) {
    int vec = 4;
    while (vec > 1 && (output.getTotalNumElements() % vec != 0 || pointerAlignment(output.getMemPtr()) % (4ull * vec) != 0)) vec /= 2;
    return vec;
}

}  // namespace

std::shared_ptr<StampedEquation> stampScatterClear(const Tensor& output, int deviceNum) {
    requireDense(output, DataType::FP32, "output");
    const uint64_t outputs = output.getTotalNumElements();
    const int vec = clearVectorOf(output);
    const uint64_t blocks = (outputs / vec + 255) / 256;
    if (blocks > 0x7fffffffull) throw std::runtime_error("Scatter-add: the output is too large for one launch.");
    const std::shared_ptr<CompiledKernel> kernel = compileKernel(clearSource(outputs, vec), "thor_scatter_clear", deviceNum, /*fastContract=*/false);
    std::ostringstream description;
    description << "scatter_clear(n=" << outputs << ",vec=" << vec << ",grid=" << blocks << ") [" << kernel->kernelName << "]";
    return std::make_shared<StampedEquation>(kernel, std::vector<Tensor>{}, std::vector<Tensor>{output}, std::vector<StampedEquation::ScalarArgument>{},
                                             std::vector<size_t>{}, std::vector<size_t>{0}, 1, /*passNumel=*/false, outputs, outputs > UINT32_MAX,
                                             static_cast<uint32_t>(blocks), 256, /*flops=*/0, description.str());
}

std::shared_ptr<StampedEquation> stampScatterAdd(const Tensor& updates, const Tensor& indices, const Tensor& output, const std::optional<Tensor>& offsets,
                                                 int deviceNum) {
    requireDense(updates, DataType::FP32, "updates");
    requireDense(indices, DataType::UINT32, "indices");
    requireDense(output, DataType::FP32, "output");
    const uint64_t count = updates.getTotalNumElements(), outputs = output.getTotalNumElements();
    if (indices.getTotalNumElements() != count) throw std::runtime_error("Scatter-add requires one index per update.");
    if (outputs >= 0xffffffffull) throw std::runtime_error("Scatter-add: UINT32 indices cannot address an output this large.");
    // a wavefront's stretch: 2048 updates (a multiple of four steps of 64), shorter while that leaves fewer than 4096 blocks
    uint64_t stretch = 2048;
    while (stretch > 256 && (count + 4 * stretch - 1) / (4 * stretch) < 4096) stretch /= 2;
    const uint64_t blocks = (count + 4 * stretch - 1) / (4 * stretch);
    if (blocks > 0x7fffffffull) throw std::runtime_error("Scatter-add: too many updates for one launch.");
    std::string offsetsType;
    uint64_t segments = 0;
    if (offsets.has_value()) {
        if (!offsets->isInitialized() || !offsets->isDenseContiguous() || offsets->getTotalNumElements() < 2 ||
            (offsets->getDataType() != DataType::UINT32 && offsets->getDataType() != DataType::UINT64)) {
            throw std::runtime_error("Scatter-add requires dense UINT32 or UINT64 offsets [B + 1].");
        }
        offsetsType = offsets->getDataType() == DataType::UINT64 ? "thor::u64" : "thor::u32";
        segments = offsets->getTotalNumElements() - 1;
    }
    const std::shared_ptr<CompiledKernel> kernel = compileKernel(addSource(count, outputs, offsetsType, segments, stretch), "thor_scatter_add", deviceNum, /*fastContract=*/false);
    std::ostringstream description;
    description << "scatter_add(updates=" << count << ",into=" << outputs << ",stretch=" << stretch << ",grid=" << blocks << ") [" << kernel->kernelName << "]";
    std::vector<Tensor> inputs = {updates, indices};
    if (offsets.has_value()) inputs.push_back(*offsets);
    std::vector<size_t> inputArgs;
    for (size_t i = 0; i < inputs.size(); ++i) inputArgs.push_back(i);
    return std::make_shared<StampedEquation>(kernel, inputs, std::vector<Tensor>{output}, std::vector<StampedEquation::ScalarArgument>{}, inputArgs,
                                             std::vector<size_t>{inputs.size()}, inputs.size() + 1, /*passNumel=*/false, count, count > UINT32_MAX,
                                             static_cast<uint32_t>(blocks), 256, /*flops=*/0, description.str());
}

std::shared_ptr<StampedEquation> stampViewScatter(const Tensor& gradient, const Tensor& output, const std::vector<uint64_t>& dims,
                                                  const std::vector<uint64_t>& strides, uint64_t offset, int deviceNum) {
    requireDense(gradient, DataType::FP32, "gradient");
    requireDense(output, DataType::FP32, "output");
    if (dims.size() != strides.size() || dims.empty()) throw std::runtime_error("Strided view backward needs one stride per dimension.");
    uint64_t count = 1, last = offset;
    std::vector<std::pair<uint64_t, uint64_t>> byStride;  // (stride, extent) of the axes that move
    for (size_t k = 0; k < dims.size(); ++k) {
        if (dims[k] == 0) throw std::runtime_error("Strided view backward does not support zero-sized dimensions.");
        count *= dims[k];
        last += (dims[k] - 1) * strides[k];
        if (dims[k] > 1) byStride.emplace_back(strides[k], dims[k]);
    }
    if (gradient.getTotalNumElements() != count) throw std::runtime_error("Strided view backward requires a gradient shaped like the view.");
    if (last >= output.getTotalNumElements()) throw std::runtime_error("Strided view backward: the view leaves the operand's storage.");
    // no element twice: sorted by stride, every axis must step over everything the finer axes span
    std::sort(byStride.begin(), byStride.end());
    uint64_t span = 0;
    for (const auto& [stride, extent] : byStride) {
        if (stride == 0 || stride <= span) throw std::runtime_error("Strided view backward requires a view that addresses every element once.");
        span += (extent - 1) * stride;
    }
    const uint64_t blocks = (count + 255) / 256;
    if (blocks > 0x7fffffffull) throw std::runtime_error("Strided view backward: the view is too large for one launch.");
    std::ostringstream s;
    s << thor_embed::kDevicePrelude;
    s << "extern \"C\" __global__ __launch_bounds__(256) void thor_view_scatter(const float* __restrict__ gradient, float* __restrict__ out) {\n";
    s << "    const thor::u64 e = (thor::u64)blockIdx.x * 256 + threadIdx.x;\n";
    s << "    if (e >= " << count << "ull) return;\n";
    s << "    thor::u64 rest = e, at = " << offset << "ull;\n";
    for (size_t k = dims.size(); k-- > 0;) {
        if (dims[k] == 1) continue;
        s << "    at += (rest % " << dims[k] << "ull) * " << strides[k] << "ull;\n    rest /= " << dims[k] << "ull;\n";
    }
    s << "    out[at] = __builtin_nontemporal_load(gradient + e);\n}\n";
    const std::shared_ptr<CompiledKernel> kernel = compileKernel(s.str(), "thor_view_scatter", deviceNum, /*fastContract=*/false);
    std::ostringstream description;
    description << "view_scatter(elements=" << count << ",into=" << output.getTotalNumElements() << ",grid=" << blocks << ") [" << kernel->kernelName << "]";
    return std::make_shared<StampedEquation>(kernel, std::vector<Tensor>{gradient}, std::vector<Tensor>{output}, std::vector<StampedEquation::ScalarArgument>{},
                                             std::vector<size_t>{0}, std::vector<size_t>{1}, 2, /*passNumel=*/false, count, count > UINT32_MAX,
                                             static_cast<uint32_t>(blocks), 256, /*flops=*/0, description.str());
}

}  // namespace ThorImplementation
