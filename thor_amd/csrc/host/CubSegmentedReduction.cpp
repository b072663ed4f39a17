// Offset-segmented reductions: validation, stamping and launching (kernels: thor_device_reduce.h reduceSegments).
#include "ReductionPlanner.h"
#include "Utilities/Common/ScopedGpu.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "Utilities/TensorOperations/Cub/CubReduction.h"

#include <cstring>
#include <stdexcept>

namespace ThorImplementation {

namespace {

bool isFloatingStorage(DataType d) {
    return d == DataType::FP8_E4M3 || d == DataType::FP8_E5M2 || d == DataType::FP16 || d == DataType::BF16 || d == DataType::FP32;
}

void requireDenseGpu(const Tensor& t, const char* what) {
    if (!t.isInitialized()) throw std::invalid_argument(std::string("Segmented reduction ") + what + " tensor is not initialized.");
    if (t.getPlacement().getMemDevice() != TensorPlacement::MemDevices::GPU) {
        throw std::invalid_argument(std::string("Segmented reduction ") + what + " must be a GPU tensor.");
    }
    if (!t.isDenseContiguous()) throw std::invalid_argument(std::string("Segmented reduction ") + what + " must be dense and contiguous.");
}

bool overlaps(const Tensor& a, const Tensor& b) {
    const char* a0 = static_cast<const char*>(a.getMemPtr());
    const char* b0 = static_cast<const char*>(b.getMemPtr());
    return a0 < b0 + b.getArraySizeInBytes() && b0 < a0 + a.getArraySizeInBytes();
}

struct SegmentedShape {
    uint64_t rows = 0, trailing = 1, segments = 0;
    std::vector<uint64_t> outputDims;
};

// Shape and dtype contract shared by the value and the arg form.
SegmentedShape requireContract(const Tensor& input, const Tensor& offsets, const Stream& stream) {
    requireDenseGpu(input, "input");
    requireDenseGpu(offsets, "segment offsets");
    if (!stream.isInitialized() || stream.getGpuNum() != input.getPlacement().getDeviceNum()) {
        throw std::invalid_argument("Segmented reduction stream must belong to the input tensor's GPU.");
    }
    if (offsets.getPlacement() != input.getPlacement()) throw std::invalid_argument("Segment offsets must live on the input tensor's GPU.");
    if (!isFloatingStorage(input.getDataType())) {
        throw std::invalid_argument("Segmented reduction input must be fp8, fp16, bf16 or fp32.");
    }
    if (!CubSegmentedReduction::isOffsetDataTypeSupported(offsets.getDataType())) {
        throw std::invalid_argument("Segmented-reduction offsets must use UINT32 or UINT64.");
    }
    const std::vector<uint64_t> offsetDims = offsets.getDimensions();
    if (offsetDims.size() != 1 || offsetDims[0] < 2) {
        throw std::invalid_argument("Segmented-reduction offsets must be rank 1 with shape [num_segments + 1] and at least one segment.");
    }
    if (overlaps(input, offsets)) throw std::invalid_argument("Segment offsets must not alias the input tensor.");
    SegmentedShape shape;
    const std::vector<uint64_t> dims = input.getDimensions();
    shape.rows = dims[0];
    for (size_t a = 1; a < dims.size(); ++a) shape.trailing *= dims[a];
    shape.segments = offsetDims[0] - 1;
    shape.outputDims = dims;
    shape.outputDims[0] = shape.segments;
    return shape;
}

// Reads the offsets back and checks the row-partition contract: zero based, non-decreasing, within the rows.
void requireValidPartition(const Tensor& offsets, uint64_t rows, const Stream& stream) {
    Tensor host(TensorPlacement(TensorPlacement::MemDevices::CPU), TensorDescriptor(offsets.getDataType(), offsets.getDimensions()));
    host.copyFromAsync(offsets, stream);
    stream.synchronize();
    const uint64_t count = offsets.getTotalNumElements();
    auto at = [&](uint64_t i) -> uint64_t {
        return offsets.getDataType() == DataType::UINT64 ? host.getMemPtr<uint64_t>()[i] : host.getMemPtr<uint32_t>()[i];
    };
    if (at(0) != 0) throw std::invalid_argument("Segment offsets must start at 0.");
    for (uint64_t i = 1; i < count; ++i)
        if (at(i) < at(i - 1)) throw std::invalid_argument("Segment offsets must be non-decreasing.");
    if (at(count - 1) > rows) throw std::invalid_argument("Segment offsets exceed the number of input rows.");
}

void requireOutput(const Tensor& output, const Tensor& input, const SegmentedShape& shape, const char* what) {
    requireDenseGpu(output, what);
    if (output.getPlacement() != input.getPlacement()) throw std::invalid_argument(std::string("Segmented reduction ") + what + " must live on the input's GPU.");
    if (output.getDimensions() != shape.outputDims) {
        throw std::invalid_argument(std::string("Segmented reduction ") + what + " has shape " + output.dimensionsToString() + " but [" +
                                    std::to_string(shape.segments) + ", trailing input dims...] is required.");
    }
    if (overlaps(output, input)) throw std::invalid_argument(std::string("Segmented reduction ") + what + " must not alias the input.");
}

ReductionKernelRequest baseRequest(const Tensor& input, const Tensor& offsets, const SegmentedShape& shape, const Stream& stream) {
    ReductionKernelRequest request;
    request.segmented = true;
    request.segments = shape.segments;
    request.segmentedRows = shape.rows;
    request.trailing = shape.trailing;
    request.offsetsAre64 = offsets.getDataType() == DataType::UINT64;
    request.inputDType = input.getDataType();
    request.inputAlignmentBytes = pointerAlignment(input.getMemPtr());
    request.deviceNum = stream.getGpuNum();
    request.geometry.path = CubReductionPath::OffsetSegmented;
    request.geometry.rank = static_cast<uint32_t>(input.getDimensions().size());
    request.geometry.input_elements = shape.rows * shape.trailing;
    request.geometry.output_elements = shape.segments * shape.trailing;
    request.geometry.reduction_size = shape.rows;  // an upper bound; the divisor of a mean is the runtime row count
    request.geometry.output_dimensions = shape.outputDims;
    request.geometry.squeezed_output_dimensions = shape.outputDims;
    return request;
}

void launch(const ReductionLaunchPlan& plan, const Tensor& input, void* valueOut, void* indexOut, const std::optional<Tensor>& workspace,
            const Tensor& offsets, Stream& stream) {
    if (!stream.isInitialized() || stream.getGpuNum() != input.getPlacement().getDeviceNum()) {
        throw std::invalid_argument("Stamped segmented reduction must run on a stream of the GPU it was stamped for.");
    }
    ScopedGpu scoped(stream.getGpuNum());
    const void* in = input.getMemPtr();
    void* partials = workspace.has_value() ? const_cast<Tensor&>(workspace.value()).getMemPtr<char>() : nullptr;
    const void* offsetPointer = offsets.getMemPtr();
    float scale = 1.0f;
    if (plan.prepareKernel) {
        std::vector<void*> prepareArgs = {&partials, &offsetPointer};
        plan.prepareKernel->launch(plan.prepareGridX, 1, 1, plan.prepareThreads, stream.getStream(), prepareArgs);
    }
    std::vector<void*> args = {&in, &valueOut, &indexOut, &partials, &scale, &offsetPointer};
    plan.mainKernel->launch(plan.mainGridX, plan.mainGridY, 1, plan.mainThreads, stream.getStream(), args);
    if (plan.finishKernel) {
        const void* constPartials = partials;
        std::vector<void*> finishArgs = {&constPartials, &valueOut, &indexOut, &scale, &offsetPointer};
        plan.finishKernel->launch(plan.finishGridX, 1, 1, plan.finishThreads, stream.getStream(), finishArgs);
    }
}

std::optional<Tensor> workspaceFor(const ReductionLaunchPlan& plan, const Tensor& input) {
    if (plan.workspaceBytes == 0) return std::nullopt;
    return Tensor(input.getPlacement(), TensorDescriptor(DataType::UINT8, {plan.workspaceBytes}));
}

}  // namespace

// ---- values -----------------------------------------------------------------------------------------------------------------
CubSegmentedReduction::CubSegmentedReduction(CubReductionOp op, std::optional<DataType> output_dtype) : op(op), output_dtype(output_dtype) {
    if (op != CubReductionOp::Sum && op != CubReductionOp::Mean && op != CubReductionOp::Min && op != CubReductionOp::Max) {
        throw std::invalid_argument("Offset-segmented reduction supports sum, mean, min, and max.");
    }
    if (output_dtype.has_value() && !isFloatingStorage(output_dtype.value())) {
        throw std::invalid_argument("Offset-segmented reduction output dtype must be fp8, fp16, bf16 or fp32.");
    }
}

bool CubSegmentedReduction::isInputDataTypeSupported(DataType dtype) { return isFloatingStorage(dtype); }

std::shared_ptr<StampedCubSegmentedReduction> CubSegmentedReduction::stamp(const Tensor& input, const Tensor& segment_offsets,
                                                                           const Stream& stream) const {
    const SegmentedShape shape = requireContract(input, segment_offsets, stream);
    Tensor output(input.getPlacement(), TensorDescriptor(resolveOutputDataType(input.getDataType()), shape.outputDims));
    return stamp(input, output, segment_offsets, stream);
}

std::shared_ptr<StampedCubSegmentedReduction> CubSegmentedReduction::stamp(const Tensor& input, const Tensor& preallocated_output,
                                                                           const Tensor& segment_offsets, const Stream& stream) const {
    const SegmentedShape shape = requireContract(input, segment_offsets, stream);
    requireValidPartition(segment_offsets, shape.rows, stream);
    return stampValidated(input, preallocated_output, segment_offsets, stream);
}

std::shared_ptr<StampedCubSegmentedReduction> CubSegmentedReduction::stampRuntimeOffsets(const Tensor& input, const Tensor& preallocated_output,
                                                                                         const Tensor& segment_offsets, const Stream& stream) const {
    (void)requireContract(input, segment_offsets, stream);
    return stampValidated(input, preallocated_output, segment_offsets, stream);
}

std::shared_ptr<StampedCubSegmentedReduction> CubSegmentedReduction::stampValidated(const Tensor& input, const Tensor& output,
                                                                                    const Tensor& segment_offsets, const Stream& stream) const {
    const SegmentedShape shape = requireContract(input, segment_offsets, stream);
    requireOutput(output, input, shape, "output");
    if (!isFloatingStorage(output.getDataType())) throw std::invalid_argument("Segmented reduction output must be fp8, fp16, bf16 or fp32.");
    if (output_dtype.has_value() && output.getDataType() != output_dtype.value()) {
        throw std::invalid_argument("Preallocated segmented-reduction output dtype does not match the configured output dtype.");
    }
    if (overlaps(output, segment_offsets)) throw std::invalid_argument("Segmented reduction output must not alias the offsets.");
    ReductionKernelRequest request = baseRequest(input, segment_offsets, shape, stream);
    request.isArg = false;
    request.valueOp = op;
    request.valueOutputDType = output.getDataType();
    ScopedGpu scoped(stream.getGpuNum());
    ReductionLaunchPlan plan = buildReductionKernels(request);
    std::optional<Tensor> workspace = workspaceFor(plan, input);
    return std::shared_ptr<StampedCubSegmentedReduction>(new StampedCubSegmentedReduction(
        op, input, output, segment_offsets, shape.rows * shape.trailing, shape.segments, std::move(plan), std::move(workspace), stream));
}

void StampedCubSegmentedReduction::runOn(Stream& run_stream) const {
    launch(plan, input, output.getMemPtr(), nullptr, workspace, segment_offsets, run_stream);
}

// ---- arg ----------------------------------------------------------------------------------------------------------------------
CubSegmentedArgReduction::CubSegmentedArgReduction(CubArgReductionOp op, DataType index_output_dtype)
    : op(op), index_output_dtype(index_output_dtype) {
    if (op != CubArgReductionOp::ArgMin && op != CubArgReductionOp::ArgMax) throw std::invalid_argument("Unsupported arg reduction operation.");
    if (index_output_dtype != DataType::UINT32 && index_output_dtype != DataType::UINT64) {
        throw std::invalid_argument("Arg reduction index output dtype must be UINT32 or UINT64.");
    }
}

std::shared_ptr<StampedCubSegmentedArgReduction> CubSegmentedArgReduction::stamp(const Tensor& input, const Tensor& segment_offsets,
                                                                                 const Stream& stream) const {
    const SegmentedShape shape = requireContract(input, segment_offsets, stream);
    Tensor winners(input.getPlacement(), TensorDescriptor(index_output_dtype, shape.outputDims));
    return stamp(input, winners, segment_offsets, stream);
}

std::shared_ptr<StampedCubSegmentedArgReduction> CubSegmentedArgReduction::stamp(const Tensor& input, const Tensor& preallocated_index_output,
                                                                                 const Tensor& segment_offsets, const Stream& stream) const {
    const SegmentedShape shape = requireContract(input, segment_offsets, stream);
    requireValidPartition(segment_offsets, shape.rows, stream);
    return stampValidated(input, preallocated_index_output, segment_offsets, stream);
}

std::shared_ptr<StampedCubSegmentedArgReduction> CubSegmentedArgReduction::stampRuntimeOffsets(const Tensor& input,
                                                                                               const Tensor& preallocated_index_output,
                                                                                               const Tensor& segment_offsets,
                                                                                               const Stream& stream) const {
    (void)requireContract(input, segment_offsets, stream);
    return stampValidated(input, preallocated_index_output, segment_offsets, stream);
}

std::shared_ptr<StampedCubSegmentedArgReduction> CubSegmentedArgReduction::stampValidated(const Tensor& input, const Tensor& index_output,
                                                                                          const Tensor& segment_offsets,
                                                                                          const Stream& stream) const {
    const SegmentedShape shape = requireContract(input, segment_offsets, stream);
    requireOutput(index_output, input, shape, "index output");
    if (index_output.getDataType() != index_output_dtype) {
        throw std::invalid_argument("Segmented arg reduction index output dtype does not match the configured index dtype.");
    }
    if (index_output_dtype == DataType::UINT32 && shape.rows * shape.trailing > 0xffffffffull) {
        throw std::invalid_argument("UINT32 winner indices cannot address this input; use UINT64.");
    }
    if (overlaps(index_output, segment_offsets)) throw std::invalid_argument("Segmented reduction output must not alias the offsets.");
    ReductionKernelRequest request = baseRequest(input, segment_offsets, shape, stream);
    request.isArg = true;
    request.argOp = op;
    request.writeValue = false;
    request.writeIndex = true;
    request.indexOutputDType = index_output_dtype;
    request.valueOutputDType = DataType::FP32;
    ScopedGpu scoped(stream.getGpuNum());
    ReductionLaunchPlan plan = buildReductionKernels(request);
    std::optional<Tensor> workspace = workspaceFor(plan, input);
    return std::shared_ptr<StampedCubSegmentedArgReduction>(new StampedCubSegmentedArgReduction(
        op, input, index_output, segment_offsets, shape.rows * shape.trailing, shape.segments, std::move(plan), std::move(workspace), stream));
}

void StampedCubSegmentedArgReduction::runOn(Stream& run_stream) const {
    launch(plan, input, nullptr, index_output.getMemPtr(), workspace, segment_offsets, run_stream);
}

}  // namespace ThorImplementation
