// Backward of a min/max reduction: the winner of every reduction window takes the window's gradient, every other element
// zero.  The winners come from an arg reduction (an index per window, numbered row-major over the reduced axes, first among
// equals); this file generates the kernel that spreads the gradient: one pass that writes the operand-shaped output and
// reads one index and one gradient value per window (reference behaviour: Utilities/Expression/StampedEquation.cpp:3139-3160
// there pairs an index-producing reduction with a routing kernel the same way).
#include "WinnerRouting.h"

#include "ReductionPlanner.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "thorhip_numeric_embed.h"

#include <algorithm>
#include <sstream>
#include <stdexcept>

namespace ThorImplementation {

std::shared_ptr<StampedEquation> stampWinnerRouting(const Tensor& winners, const Tensor& outputGradient, const Tensor& routed,
                                                    const std::vector<uint64_t>& operandDims, const std::vector<uint64_t>& reducedAxes, int deviceNum) {
    if (!winners.isInitialized() || !outputGradient.isInitialized() || !routed.isInitialized()) {
        throw std::runtime_error("Min/max reduction backward requires initialized tensors.");
    }
    if (!winners.isDenseContiguous() || !outputGradient.isDenseContiguous() || !routed.isDenseContiguous()) {
        throw std::runtime_error("Min/max reduction backward requires dense tensors.");
    }
    if (winners.getDataType() != DataType::UINT32) throw std::runtime_error("Min/max reduction backward expects UINT32 winner indices.");

    // neighbouring axes of one kind (kept / reduced) act as one axis; size-1 axes drop out
    struct Group {
        uint64_t size;
        bool reduced;
    };
    std::vector<Group> groups;
    uint64_t total = 1, windows = 1, windowSize = 1;
    for (size_t axis = 0; axis < operandDims.size(); ++axis) {
        const uint64_t d = operandDims[axis];
        const bool reduced = std::binary_search(reducedAxes.begin(), reducedAxes.end(), axis);
        total *= d;
        (reduced ? windowSize : windows) *= d;
        if (d == 1) continue;
        if (!groups.empty() && groups.back().reduced == reduced) {
            groups.back().size *= d;
        } else {
            groups.push_back({d, reduced});
        }
    }
    if (routed.getTotalNumElements() != total || winners.getTotalNumElements() != windows || outputGradient.getTotalNumElements() != windows) {
        throw std::runtime_error("Min/max reduction backward: the gradient must hold one element per reduction window.");
    }
    if (windowSize > UINT32_MAX) throw std::runtime_error("Min/max reduction backward: a reduction window exceeds the UINT32 index range.");

    const uint32_t elementBytes = dataTypeSizeInBytes(routed.getDataType());
    int vec = static_cast<int>(16 / elementBytes);
    while (vec > 1 && (total % vec != 0 || pointerAlignment(routed.getMemPtr()) % (static_cast<uint64_t>(vec) * elementBytes) != 0)) vec /= 2;
    const bool wide = total > UINT32_MAX;
    const char* indexType = wide ? "thor::u64" : "thor::u32";
    const char* suffix = wide ? "ull" : "u";
    const uint64_t vectors = total / vec;
    const uint32_t threads = 256;
    const uint64_t blocks = (vectors + threads - 1) / threads;
    if (blocks > 0x7fffffffull) throw std::runtime_error("Min/max reduction backward: the operand is too large for one launch.");

    std::ostringstream s;
    s << thor_embed::kDevicePrelude;
    s << "extern \"C\" __global__ __launch_bounds__(256) void thor_route_winner(const thor::u32* winners, const " << deviceTypeName(outputGradient.getDataType())
      << "* gradient, " << deviceTypeName(routed.getDataType()) << "* routed) {\n";
    s << "    typedef " << deviceTypeName(routed.getDataType()) << " T;\n";
    s << "    const thor::u64 vector = (thor::u64)blockIdx.x * " << threads << " + threadIdx.x;\n";
    s << "    if (vector >= " << vectors << "ull) return;\n";
    s << "    const " << indexType << " first = (" << indexType << ")(vector * " << vec << ");\n";
    s << "    thor::Pack<T, " << vec << "> out;\n";
    s << "#pragma unroll\n    for (int k = 0; k < " << vec << "; ++k) {\n";
    s << "        " << indexType << " rest = first + k, window = 0, position = 0, c;\n";
    // innermost group first: coordinates peel off the flat index; kept coordinates number the window, reduced ones the position
    uint64_t windowStride = 1, positionStride = 1;
    for (size_t g = groups.size(); g-- > 0;) {
        const Group& group = groups[g];
        if (g == 0) {
            s << "        c = rest;\n";
        } else {
            s << "        c = rest % " << group.size << suffix << "; rest /= " << group.size << suffix << ";\n";
        }
        if (group.reduced) {
            s << "        position += c * " << positionStride << suffix << ";\n";
            positionStride *= group.size;
        } else {
            s << "        window += c * " << windowStride << suffix << ";\n";
            windowStride *= group.size;
        }
    }
    s << "        const float g = winners[window] == (thor::u32)position ? thor::toFloat(gradient[window]) : 0.0f;\n";
    s << "        out.v[k] = thor::fromFloat<T>(g);\n";
    s << "    }\n";
    s << "    out.storeStream(routed + first);\n}\n";

    const std::shared_ptr<CompiledKernel> kernel = compileKernel(s.str(), "thor_route_winner", deviceNum, /*fastContract=*/false);
    std::ostringstream description;
    description << "route_winner(windows=" << windows << ",window=" << windowSize << ",vec=" << vec << ",grid=" << blocks << ") [" << kernel->kernelName << "]";
    return std::make_shared<StampedEquation>(kernel, std::vector<Tensor>{winners, outputGradient}, std::vector<Tensor>{routed},
                                             std::vector<StampedEquation::ScalarArgument>{}, std::vector<size_t>{0, 1}, std::vector<size_t>{2}, 3,
                                             /*passNumel=*/false, total, wide, static_cast<uint32_t>(blocks), threads, /*flops=*/0, description.str());
}

}  // namespace ThorImplementation
