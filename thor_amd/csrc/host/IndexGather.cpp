// Expression::takeAlongAxis: a gather along one axis with a tensor of indices (reference behaviour:
// Utilities/Expression/CudaSourceEmitter.cpp:2343-2410 source index of an output element, FusedEquation.cpp:1049-1068 shapes).
// Neighbouring axes collapse to [outer, axis, inner]; a thread produces one vector of consecutive output elements: it loads
// their indices as one vector, gathers the values one by one and stores one vector.
#include "IndexGather.h"

#include "ReductionPlanner.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "thorhip_numeric_embed.h"

#include <algorithm>
#include <sstream>
#include <stdexcept>

namespace ThorImplementation {

std::shared_ptr<StampedEquation> stampTakeAlongAxis(const Tensor& values, const Tensor& indices, const Tensor& output, uint64_t axis, int deviceNum) {
    if (!values.isInitialized() || !indices.isInitialized() || !output.isInitialized()) throw std::runtime_error("take_along_axis requires initialized tensors.");
    const std::vector<uint64_t>& valueDims = values.getDimensions();
    const std::vector<uint64_t>& indexDims = indices.getDimensions();
    if (valueDims.empty() || indexDims.empty()) throw std::runtime_error("take_along_axis requires non-scalar input and indices tensors.");
    if (valueDims.size() != indexDims.size()) throw std::runtime_error("take_along_axis input and indices must have the same rank.");
    if (axis >= valueDims.size()) throw std::runtime_error("take_along_axis axis is out of range for the input rank.");
    uint64_t outer = 1, inner = 1;
    for (size_t d = 0; d < valueDims.size(); ++d) {
        if (d != axis && valueDims[d] != indexDims[d]) {
            throw std::runtime_error("take_along_axis input and indices dimensions must match except on the selected axis.");
        }
        if (valueDims[d] == 0 || indexDims[d] == 0) throw std::runtime_error("take_along_axis does not support zero-sized dimensions.");
        if (d < axis) outer *= valueDims[d];
        if (d > axis) inner *= valueDims[d];
    }
    if (indices.getDataType() != DataType::UINT32 && indices.getDataType() != DataType::UINT64) {
        throw std::runtime_error(std::string("take_along_axis indices must have UINT32 or UINT64 dtype, received: ") + dataTypeName(indices.getDataType()));
    }
    if (output.getDimensions() != indexDims) throw std::runtime_error("take_along_axis output must have the shape of the indices.");
    if (!values.isDenseContiguous() || !indices.isDenseContiguous() || !output.isDenseContiguous()) {
        throw std::runtime_error("take_along_axis requires dense tensors.");
    }
    const uint64_t along = valueDims[axis], taken = indexDims[axis];
    const uint64_t total = outer * taken * inner;
    const bool sameType = values.getDataType() == output.getDataType();
    const uint32_t outBytes = dataTypeSizeInBytes(output.getDataType());
    const uint32_t indexBytes = dataTypeSizeInBytes(indices.getDataType());
    int vec = static_cast<int>(16 / std::max(outBytes, indexBytes));
    while (vec > 1 && (total % vec != 0 || pointerAlignment(output.getMemPtr()) % (static_cast<uint64_t>(vec) * outBytes) != 0 ||
                       pointerAlignment(indices.getMemPtr()) % (static_cast<uint64_t>(vec) * indexBytes) != 0)) {
        vec /= 2;
    }
    const uint64_t vectors = total / vec;
    const uint32_t threads = 256;
    const uint64_t blocks = (vectors + threads - 1) / threads;
    if (blocks > 0x7fffffffull) throw std::runtime_error("take_along_axis: the output is too large for one launch.");
    const char* rawWord = outBytes == 1 ? "thor::u8" : outBytes == 2 ? "thor::u16" : "thor::u32";
    const std::string valueType = sameType ? rawWord : deviceTypeName(values.getDataType());
    const std::string outType = sameType ? rawWord : deviceTypeName(output.getDataType());
    const char* indexType = indices.getDataType() == DataType::UINT64 ? "thor::u64" : "thor::u32";

    std::ostringstream s;
    s << thor_embed::kDevicePrelude;
    s << "extern \"C\" __global__ __launch_bounds__(256) void thor_take_along_axis(const " << valueType << "* values, const " << indexType << "* indices, "
      << outType << "* out) {\n";
    s << "    const thor::u64 vector = (thor::u64)blockIdx.x * " << threads << " + threadIdx.x;\n";
    s << "    if (vector >= " << vectors << "ull) return;\n";
    s << "    const thor::u64 first = vector * " << vec << ";\n";
    s << "    thor::Pack<" << indexType << ", " << vec << "> chosen;\n    chosen.loadStream(indices + first);\n";
    s << "    thor::Pack<" << outType << ", " << vec << "> q;\n";
    s << "#pragma unroll\n    for (int k = 0; k < " << vec << "; ++k) {\n";
    s << "        const thor::u64 e = first + k;\n";
    s << "        const thor::u64 i = e % " << inner << "ull, o = e / " << inner * taken << "ull;\n";
    s << "        thor::u64 j = (thor::u64)chosen.v[k];\n";
    s << "        j = j < " << along << "ull ? j : " << along - 1 << "ull;\n";
    s << "        const " << valueType << " v = values[(o * " << along << "ull + j) * " << inner << "ull + i];\n";
    s << "        q.v[k] = " << (sameType ? "v" : "thor::fromFloat<" + outType + ">(thor::toFloat(v))") << ";\n";
    s << "    }\n    q.storeStream(out + first);\n}\n";

    const std::shared_ptr<CompiledKernel> kernel = compileKernel(s.str(), "thor_take_along_axis", deviceNum, /*fastContract=*/false);
    std::ostringstream description;
    description << "take_along_axis(outer=" << outer << ",axis=" << along << "->" << taken << ",inner=" << inner << ",vec=" << vec << ",grid=" << blocks << ") ["
                << kernel->kernelName << "]";
    return std::make_shared<StampedEquation>(kernel, std::vector<Tensor>{values, indices}, std::vector<Tensor>{output},
                                             std::vector<StampedEquation::ScalarArgument>{}, std::vector<size_t>{0, 1}, std::vector<size_t>{2}, 3,
                                             /*passNumel=*/false, total, total > UINT32_MAX, static_cast<uint32_t>(blocks), threads, /*flops=*/0,
                                             description.str());
}

}  // namespace ThorImplementation
