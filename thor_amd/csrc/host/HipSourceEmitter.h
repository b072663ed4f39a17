// Internal: generates gfx950 HIP source for one fused elementwise / broadcast stage of an expression
// (the counterpart of the reference's CudaSourceEmitter: Utilities/Expression/CudaSourceEmitter.cpp:1610-1959 casts and
// per-op expressions, :5730-5910 wide flat kernels, :7794-7944 shape-specialised broadcast kernels).
//
// Kernel shapes emitted here
//   flat       every tensor operand has the output's shape and is dense: one 16-byte vector per operand per lane,
//              non-temporal loads and stores, one vector per lane, element-wise tail; `numel` is a kernel argument so one
//              compiled kernel serves every size
//   broadcast  operands with broadcast (stride-0), permuted or strided axes: axes are collapsed jointly over all
//              operands, extents and strides are baked in as constants (divides by constants), and the innermost axis
//              is vectorised whenever every operand is either contiguous or broadcast along it
#pragma once

#include "Utilities/Expression/Expression.h"

#include <cstdint>
#include <optional>
#include <string>
#include <vector>

namespace ThorImplementation {

// A tensor read by the kernel: the graph node that stands for it, its storage dtype and its layout in elements.
struct KernelOperand {
    uint32_t node = UINT32_MAX;
    DataType storageDType = DataType::FP32;
    std::vector<uint64_t> dims;     // logical dims of the operand (rank <= output rank, right-aligned for broadcasting)
    std::vector<uint64_t> strides;  // elements, same rank as dims
    uint64_t alignmentBytes = 256;
};

struct KernelOutput {
    uint32_t node = UINT32_MAX;
    DataType storageDType = DataType::FP32;
    uint64_t alignmentBytes = 256;
};

// Kernels of a ragged batch compute only the first offsets[batchSize] * elementsPerValue elements; `offsets` is passed as a
// pointer after the operands and read on the device.
struct RaggedExtent {
    uint64_t batchSize = 0;
    uint64_t elementsPerValue = 1;
    bool offsetsAre64 = false;
};

// A per-segment tensor [B, E] read through a row -> segment index: element e of the output takes values[ids[e / E] * E + e % E]
// (the value a SEGMENTED_BROADCAST node would have materialised), divided by the segment's length when `normalize` is set.
// Kernel arguments: `const T* g<i>, const unsigned int* gid<i>` and, when normalised, `const OffsetT* goff<i>`.
struct GatherOperand {
    uint32_t node = UINT32_MAX;  // the SEGMENTED_BROADCAST node this stands for
    DataType storageDType = DataType::FP32;
    uint64_t elementsPerValue = 1;
    uint64_t segments = 1;
    bool normalize = false;
    bool offsetsAre64 = false;
    uint64_t alignmentBytes = 256;
};

struct FusedKernelRequest {
    const PhysicalExpression* expr = nullptr;
    std::vector<KernelOperand> operands;   // kernel arguments, in order
    std::vector<GatherOperand> gathers;    // then the gathered per-segment tensors (flat kernels only)
    std::optional<RaggedExtent> extent;    // then the offsets pointer of the runtime extent, when there is one
    std::vector<uint32_t> scalarSlots;     // runtime scalar input slots passed by value (float), after the operands
    std::vector<KernelOutput> outputs;     // then the outputs
    std::vector<uint64_t> outputDims;      // common logical shape of every output
};

struct EmittedKernel {
    std::string source;
    std::string kernelName = "fused_kernel";
    bool flat = true;
    bool passNumel = true;
    bool numelIs64 = false;
    int vec = 1;
    uint64_t numel = 0;
    uint32_t gridX = 1;
    uint32_t threads = 256;
    bool fastContract = true;  // fp32-only arithmetic: allow mul+add fusion like the reference's -fmad=true
    uint64_t flopsPerElement = 0;
    std::string description;
};

EmittedKernel emitFusedKernel(const FusedKernelRequest& request);

// ---- pieces shared with the row-fused emitter -------------------------------------------------------------------------
// C type a value of `dtype` is held in inside a kernel (bf16 / fp8 values live in a float that is exactly representable).
const char* valueCType(DataType dtype);
// Expression converting `expr` (a value of dtype `from`) into a value of dtype `to`.
std::string castValueExpr(const std::string& expr, DataType from, DataType to);
// Expression turning a loaded storage element into a value of the same dtype, and back.
std::string storageToValueExpr(const std::string& expr, DataType dtype);
std::string valueToStorageExpr(const std::string& expr, DataType dtype);
std::string floatLiteral(double value);
// dtype of the value a node evaluates to inside a kernel: leaves carry their output dtype, everything else its compute dtype
DataType emittedValueDType(const ExprNode& node);
bool tryFoldConstant(const PhysicalExpression& expr, uint32_t nodeIndex, double& value);

// Emits `const T tN = ...;` statements for elementwise nodes.  Values that already exist (kernel operands, results of
// earlier statements) are registered with their dtype and the C name that holds them; constants are folded on the host
// and printed as literals; x+0, x*1, x/1 and pure shape ops become aliases of their operand.
class BodyEmitter {
   public:
    explicit BodyEmitter(const PhysicalExpression& expr);
    void defineSource(uint32_t node, DataType dtype, const std::string& name = "");
    bool defined(uint32_t node) const { return valueDType[node].has_value(); }
    DataType dtypeOf(uint32_t node) const { return valueDType[node].value(); }
    const std::string& nameOf(uint32_t node) const { return names[node]; }
    // expression reading the value of `child` converted to dtype `target`
    std::string ref(uint32_t child, DataType target) const;
    // nodes (ascending) needed to evaluate `roots`, stopping at already defined values and at host-foldable constants
    std::vector<uint32_t> collect(const std::vector<uint32_t>& roots) const;
    // fp32 divisions by `node` are emitted as `name.divide(x)` (a thor::RowDivisor built once from the divisor's value)
    void defineRowDivisor(uint32_t node, const std::string& name) { rowDivisors[node] = name; }
    // appends the statement for one node (operands must be defined); returns the flops it costs per element
    uint64_t emit(std::string& out, uint32_t nodeIndex, const std::string& indent);

   private:
    std::string unary(const ExprNode& n, DataType c) const;
    std::string binary(const ExprNode& n, DataType c) const;
    const PhysicalExpression& expr;
    std::vector<std::optional<DataType>> valueDType;
    std::vector<std::string> names;
    std::vector<std::string> rowDivisors;
};

}  // namespace ThorImplementation
