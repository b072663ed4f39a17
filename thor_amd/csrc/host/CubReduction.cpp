// Host side of the dense reductions: argument validation, geometry analysis / path selection, kernel-shape planning,
// source generation for the shape-specialised wave64 kernels, stamping and launching
// (reference behaviour: Utilities/TensorOperations/Cub/CubReduction.cpp:40-74,718-912,926-979,1255-1448).
#include "Utilities/TensorOperations/Cub/CubReduction.h"

#include "ReductionPlanner.h"
#include "Utilities/Common/ScopedGpu.h"
#include "Utilities/Expression/CompiledEquation.h"

#include <algorithm>
#include <cmath>
#include <numeric>
#include <sstream>
#include <stdexcept>
#include <string>

namespace ThorImplementation {

namespace {

bool isReductionStorageDType(DataType dtype) {
    return dtype == DataType::FP8_E4M3 || dtype == DataType::FP8_E5M2 || dtype == DataType::FP16 || dtype == DataType::BF16 ||
           dtype == DataType::FP32;
}

void requireReductionStorageDType(DataType dtype, const char* role) {
    if (!isReductionStorageDType(dtype)) {
        throw std::invalid_argument(std::string("Tensor reduction does not support ") + role + " dtype " + dataTypeName(dtype) +
                                    ". Supported storage dtypes are fp8_e4m3, fp8_e5m2, fp16, bf16 and fp32.");
    }
}

void requireValidAxes(const std::vector<uint32_t>& axes) {
    if (axes.empty()) throw std::invalid_argument("Tensor reduction requires at least one reduction axis.");
    for (size_t i = 1; i < axes.size(); ++i) {
        if (axes[i] <= axes[i - 1]) throw std::invalid_argument("Tensor reduction axes must be unique and strictly increasing.");
    }
}

void requireGpuTensor(const Tensor& tensor, const char* name) {
    if (!tensor.isInitialized()) throw std::invalid_argument(std::string(name) + " must be initialized.");
    if (tensor.getPlacement().getMemDevice() != TensorPlacement::MemDevices::GPU) {
        throw std::invalid_argument(std::string(name) + " must be a GPU tensor.");
    }
}

void requireCompatibleStream(const Tensor& input, const Stream& stream) {
    if (!stream.isInitialized()) throw std::invalid_argument("Tensor reduction requires an initialized stream.");
    if (input.getPlacement().getDeviceNum() != stream.getGpuNum()) {
        throw std::invalid_argument("Tensor reduction stream must belong to the input tensor's GPU.");
    }
}

uint64_t checkedMultiply(uint64_t a, uint64_t b, const char* quantity) {
    if (b != 0 && a > std::numeric_limits<uint64_t>::max() / b) {
        throw std::invalid_argument(std::string("Tensor reduction ") + quantity + " overflows uint64_t.");
    }
    return a * b;
}

std::vector<uint64_t> denseStrides(const std::vector<uint64_t>& dims) {
    std::vector<uint64_t> strides(dims.size(), 1);
    uint64_t running = 1;
    for (size_t d = dims.size(); d-- > 0;) {
        strides[d] = running;
        running = checkedMultiply(running, dims[d], "input element count");
    }
    return strides;
}

// A stamped output may be the keep-dimension shape, the squeezed shape, or any shape with the same element count whose
// non-singleton dimensions match.
void requireOutputShape(const Tensor& output, const CubReductionGeometry& geometry, const char* name) {
    if (output.getTotalNumElements() != geometry.output_elements) {
        throw std::invalid_argument(std::string(name) + " has " + std::to_string(output.getTotalNumElements()) +
                                    " elements but the reduction produces " + std::to_string(geometry.output_elements) + ".");
    }
    if (!output.isDenseContiguous()) throw std::invalid_argument(std::string(name) + " must be dense.");
}

}  // namespace

// ---- CubReduction ----------------------------------------------------------------------------------------------------------
CubReduction::CubReduction(CubReductionOp op, uint32_t axis, std::optional<DataType> output_dtype, float output_scale)
    : CubReduction(op, std::vector<uint32_t>{axis}, output_dtype, output_scale) {}

CubReduction::CubReduction(CubReductionOp op, std::vector<uint32_t> axes, std::optional<DataType> output_dtype, float output_scale)
    : op(op), axes(std::move(axes)), output_dtype(output_dtype), output_scale(output_scale) {
    if (static_cast<uint8_t>(op) > static_cast<uint8_t>(CubReductionOp::L2Norm)) {
        throw std::invalid_argument("Unsupported tensor reduction operation.");
    }
    requireValidAxes(this->axes);
    if (output_dtype.has_value()) requireReductionStorageDType(output_dtype.value(), "output");
    if (!std::isfinite(output_scale)) throw std::invalid_argument("Tensor reduction output scale must be finite.");
}

DataType CubReduction::resolveOutputDataType(DataType input_dtype) const { return output_dtype.value_or(input_dtype); }

float CubReduction::getFp32EmptyReductionValue(CubReductionOp op) {
    switch (op) {
        case CubReductionOp::Sum:
        case CubReductionOp::Mean:
        case CubReductionOp::L1Norm:
        case CubReductionOp::L2Norm:
            return 0.0f;
        case CubReductionOp::Min:
            return std::numeric_limits<float>::infinity();
        case CubReductionOp::Max:
            return -std::numeric_limits<float>::infinity();
        case CubReductionOp::Product:
            return 1.0f;
    }
    throw std::invalid_argument("Unsupported tensor reduction operation.");
}

CubReductionGeometry CubReduction::analyzeGeometry(const std::vector<uint64_t>& input_dimensions, uint32_t axis) {
    return analyzeGeometry(input_dimensions, std::vector<uint32_t>{axis});
}

CubReductionGeometry CubReduction::analyzeGeometry(const std::vector<uint64_t>& input_dimensions, const std::vector<uint32_t>& axes) {
    return analyzeGeometry(input_dimensions, denseStrides(input_dimensions), axes);
}

CubReductionGeometry CubReduction::analyzeGeometry(const std::vector<uint64_t>& dims, const std::vector<uint64_t>& strides,
                                                    const std::vector<uint32_t>& axes) {
    if (dims.empty()) throw std::invalid_argument("Tensor reduction requires at least one input dimension.");
    if (dims.size() != strides.size()) throw std::invalid_argument("Tensor reduction input stride rank must match the input rank.");
    requireValidAxes(axes);
    if (axes.size() > dims.size()) throw std::invalid_argument("Tensor reduction has more reduction axes than input dimensions.");
    for (uint32_t axis : axes) {
        if (axis >= dims.size()) throw std::invalid_argument("Tensor reduction axis is outside the input rank.");
    }
    for (uint64_t d : dims) {
        if (d == 0) throw std::invalid_argument("Tensor reduction does not support zero-sized tensor dimensions.");
    }

    CubReductionGeometry g;
    g.axes = axes;
    g.rank = static_cast<uint32_t>(dims.size());
    g.reduction_size = 1;
    g.output_elements = 1;
    g.output_dimensions = dims;
    g.indexing.input_strides = strides;
    const std::vector<uint64_t> dense = denseStrides(dims);
    g.input_elements = dense.front() * dims.front();
    const bool isDense = strides == dense;

    size_t cursor = 0;
    for (uint32_t d = 0; d < dims.size(); ++d) {
        if (cursor < axes.size() && axes[cursor] == d) {
            g.output_dimensions[d] = 1;
            g.reduction_size = checkedMultiply(g.reduction_size, dims[d], "reduction element count");
            g.indexing.reduced_axes.push_back(d);
            g.indexing.reduced_dimensions.push_back(dims[d]);
            ++cursor;
        } else {
            g.output_elements = checkedMultiply(g.output_elements, dims[d], "output element count");
            g.squeezed_output_dimensions.push_back(dims[d]);
            g.indexing.retained_axes.push_back(d);
            g.indexing.retained_dimensions.push_back(dims[d]);
        }
    }
    if (g.squeezed_output_dimensions.empty()) g.squeezed_output_dimensions.push_back(1);
    if (g.input_elements > static_cast<uint64_t>(std::numeric_limits<int64_t>::max())) {
        throw std::invalid_argument("Tensor reduction input element count exceeds the int64 item-count limit.");
    }

    g.reduced_axes_are_contiguous = true;
    for (size_t i = 1; i < axes.size(); ++i) g.reduced_axes_are_contiguous = g.reduced_axes_are_contiguous && axes[i] == axes[i - 1] + 1;
    if (g.reduced_axes_are_contiguous) {
        g.outer_size = g.inner_size = 1;
        for (uint32_t d = 0; d < axes.front(); ++d) g.outer_size *= dims[d];
        for (uint32_t d = axes.back() + 1; d < dims.size(); ++d) g.inner_size *= dims[d];
        g.tiled_output_outer_stride = g.inner_size;
        g.tiled_output_inner_stride = 1;
    }

    const bool singleOutput = g.output_elements == 1;
    if (isDense) {
        if (singleOutput) {
            g.path = CubReductionPath::DeviceTransformReduce;
        } else if (g.reduced_axes_are_contiguous && g.inner_size == 1) {
            g.path = CubReductionPath::ContiguousFixedSegment;
        } else if (g.reduced_axes_are_contiguous) {
            g.path = CubReductionPath::TiledFixedSegment;
        } else {
            g.path = CubReductionPath::StridedFixedSegment;
        }
    } else if (singleOutput && dims.size() == 1) {
        g.path = CubReductionPath::DeviceTransformReduce;
        g.device_transform_uses_affine_stride = true;
        g.affine_input_stride = strides[0];
    } else {
        // Views are reduced where they lie: the strided path walks their logical coordinates without materialising.
        g.path = CubReductionPath::StridedFixedSegment;
    }
    if (g.path != CubReductionPath::DeviceTransformReduce && g.reduction_size > static_cast<uint64_t>(std::numeric_limits<int>::max())) {
        throw std::invalid_argument("Tensor reduction domain exceeds the fixed segment-size int limit.");
    }
    return g;
}

uint64_t CubReduction::mapLogicalReductionIndexToPhysicalIndex(const CubReductionGeometry& g, uint64_t output_index, uint64_t reduction_index) {
    if (output_index >= g.output_elements) throw std::out_of_range("Tensor reduction output index is outside the geometry.");
    if (reduction_index >= g.reduction_size) throw std::out_of_range("Tensor reduction reduction index is outside the geometry.");
    uint64_t offset = 0;
    for (size_t a = g.indexing.retained_axes.size(); a-- > 0;) {
        const uint64_t dim = g.indexing.retained_dimensions[a];
        offset += (output_index % dim) * g.indexing.input_strides[g.indexing.retained_axes[a]];
        output_index /= dim;
    }
    for (size_t a = g.indexing.reduced_axes.size(); a-- > 0;) {
        const uint64_t dim = g.indexing.reduced_dimensions[a];
        offset += (reduction_index % dim) * g.indexing.input_strides[g.indexing.reduced_axes[a]];
        reduction_index /= dim;
    }
    return offset;
}

size_t CubReduction::queryWorkspaceSizeInBytes(const TensorDescriptor& input_descriptor, const Stream& stream) const {
    requireReductionStorageDType(input_descriptor.getDataType(), "input");
    const CubReductionGeometry geometry = analyzeGeometry(input_descriptor.getDimensions(), axes);
    ReductionKernelRequest request;
    request.isArg = false;
    request.valueOp = op;
    request.inputDType = input_descriptor.getDataType();
    request.valueOutputDType = resolveOutputDataType(input_descriptor.getDataType());
    request.geometry = geometry;
    request.inputAlignmentBytes = 256;
    request.deviceNum = stream.getGpuNum();
    return planReductionShape(request).workspaceBytes;
}

std::shared_ptr<StampedCubReduction> CubReduction::stamp(const Tensor& input, const Stream& stream) const {
    requireGpuTensor(input, "Reduction input");
    requireReductionStorageDType(input.getDataType(), "input");
    const CubReductionGeometry geometry = analyzeGeometry(input.getDimensions(), input.getStridesElements(), axes);
    Tensor output(input.getPlacement(), TensorDescriptor(resolveOutputDataType(input.getDataType()), geometry.output_dimensions));
    return stamp(input, output, stream);
}

std::shared_ptr<StampedCubReduction> CubReduction::stamp(const Tensor& input, const Tensor& output, const Stream& stream) const {
    requireGpuTensor(input, "Reduction input");
    requireGpuTensor(output, "Reduction output");
    requireCompatibleStream(input, stream);
    requireReductionStorageDType(input.getDataType(), "input");
    requireReductionStorageDType(output.getDataType(), "output");
    if (output.getPlacement() != input.getPlacement()) throw std::invalid_argument("Reduction output must live on the input tensor's GPU.");
    if (output_dtype.has_value() && output.getDataType() != output_dtype.value()) {
        throw std::invalid_argument("Preallocated reduction output dtype does not match the configured output dtype.");
    }
    const CubReductionGeometry geometry = analyzeGeometry(input.getDimensions(), input.getStridesElements(), axes);
    requireOutputShape(output, geometry, "Reduction output");

    ReductionKernelRequest request;
    request.isArg = false;
    request.valueOp = op;
    request.inputDType = input.getDataType();
    request.valueOutputDType = output.getDataType();
    request.geometry = geometry;
    request.inputAlignmentBytes = pointerAlignment(input.getMemPtr());
    request.deviceNum = stream.getGpuNum();

    ScopedGpu scoped(stream.getGpuNum());
    ReductionLaunchPlan plan = buildReductionKernels(request);
    std::optional<Tensor> workspace = allocateReductionWorkspace(plan, input.getPlacement(), stream);
    return std::shared_ptr<StampedCubReduction>(
        new StampedCubReduction(op, geometry, input, output, std::move(plan), std::move(workspace), output_scale, stream));
}

namespace {
void launchPlan(const ReductionLaunchPlan& plan, const void* in, void* valueOut, void* indexOut, const std::optional<Tensor>& workspace,
                float scale, void* stream) {
    char* ws = workspace.has_value() ? const_cast<Tensor&>(workspace.value()).getMemPtr<char>() : nullptr;
    void* partials = ws;
    const void* input = in;
    std::vector<void*> args = {&input, &valueOut, &indexOut, &partials, &scale};
    plan.mainKernel->launch(plan.mainGridX, plan.mainGridY, 1, plan.mainThreads, stream, args);
    if (plan.finishKernel) {
        const void* constPartials = partials;
        std::vector<void*> finishArgs = {&constPartials, &valueOut, &indexOut, &scale};
        plan.finishKernel->launch(plan.finishGridX, 1, 1, plan.finishThreads, stream, finishArgs);
    }
}
}  // namespace

void StampedCubReduction::run() { runOn(stream, output_scale); }
void StampedCubReduction::run(float scale) { runOn(stream, scale); }
void StampedCubReduction::runOn(Stream& run_stream) const { runOn(run_stream, output_scale); }
void StampedCubReduction::runOn(Stream& run_stream, float scale) const {
    if (!run_stream.isInitialized() || run_stream.getGpuNum() != static_cast<int>(gpuNum())) {
        throw std::invalid_argument("Stamped reduction must run on a stream of the GPU it was stamped for.");
    }
    if (!std::isfinite(scale)) throw std::invalid_argument("Tensor reduction output scale must be finite.");
    ScopedGpu scoped(run_stream.getGpuNum());
    launchPlan(plan, input.getMemPtr(), output.getMemPtr(), nullptr, workspace, scale, run_stream.getStream());
}

// ---- CubArgReduction ---------------------------------------------------------------------------------------------------------
CubArgReduction::CubArgReduction(CubArgReductionOp op, uint32_t axis, CubArgReductionOutputOptions outputs)
    : CubArgReduction(op, std::vector<uint32_t>{axis}, outputs) {}

CubArgReduction::CubArgReduction(CubArgReductionOp op, std::vector<uint32_t> axes, CubArgReductionOutputOptions outputs)
    : op(op), axes(std::move(axes)), outputs(outputs) {
    if (op != CubArgReductionOp::ArgMin && op != CubArgReductionOp::ArgMax) throw std::invalid_argument("Unsupported arg reduction operation.");
    requireValidAxes(this->axes);
    if (!outputs.produce_value && !outputs.produce_index) throw std::invalid_argument("Arg reduction must produce a value or an index output.");
    if (outputs.index_output_dtype != DataType::UINT32 && outputs.index_output_dtype != DataType::UINT64) {
        throw std::invalid_argument("Arg reduction index output dtype must be UINT32 or UINT64.");
    }
    if (outputs.value_output_dtype.has_value()) requireReductionStorageDType(outputs.value_output_dtype.value(), "value output");
}

DataType CubArgReduction::resolveValueOutputDataType(DataType input_dtype) const { return outputs.value_output_dtype.value_or(input_dtype); }

float CubArgReduction::getFp32EmptyReductionValue(CubArgReductionOp op) {
    return op == CubArgReductionOp::ArgMin ? std::numeric_limits<float>::infinity() : -std::numeric_limits<float>::infinity();
}

std::shared_ptr<StampedCubArgReduction> CubArgReduction::stamp(const Tensor& input, const Stream& stream) const {
    return stamp(input, std::nullopt, std::nullopt, stream);
}

std::shared_ptr<StampedCubArgReduction> CubArgReduction::stamp(const Tensor& input, const std::optional<Tensor>& preValue,
                                                               const std::optional<Tensor>& preIndex, const Stream& stream) const {
    requireGpuTensor(input, "Arg reduction input");
    requireCompatibleStream(input, stream);
    requireReductionStorageDType(input.getDataType(), "input");
    const CubReductionGeometry geometry = CubReduction::analyzeGeometry(input.getDimensions(), input.getStridesElements(), axes);
    if (outputs.index_output_dtype == DataType::UINT32 && geometry.reduction_size > 0xffffffffull) {
        throw std::invalid_argument("Arg reduction domain does not fit a UINT32 index output.");
    }
    std::optional<Tensor> value, index;
    if (outputs.produce_value) {
        value = preValue.has_value() ? preValue.value()
                                     : Tensor(input.getPlacement(), TensorDescriptor(resolveValueOutputDataType(input.getDataType()),
                                                                                     geometry.output_dimensions));
        requireGpuTensor(value.value(), "Arg reduction value output");
        requireReductionStorageDType(value->getDataType(), "value output");
        requireOutputShape(value.value(), geometry, "Arg reduction value output");
    } else if (preValue.has_value()) {
        throw std::invalid_argument("A value output tensor was supplied but value output is disabled.");
    }
    if (outputs.produce_index) {
        index = preIndex.has_value() ? preIndex.value()
                                     : Tensor(input.getPlacement(), TensorDescriptor(outputs.index_output_dtype, geometry.output_dimensions));
        requireGpuTensor(index.value(), "Arg reduction index output");
        if (index->getDataType() != DataType::UINT32 && index->getDataType() != DataType::UINT64) {
            throw std::invalid_argument("Arg reduction index output dtype must be UINT32 or UINT64.");
        }
        requireOutputShape(index.value(), geometry, "Arg reduction index output");
    } else if (preIndex.has_value()) {
        throw std::invalid_argument("An index output tensor was supplied but index output is disabled.");
    }

    ReductionKernelRequest request;
    request.isArg = true;
    request.argOp = op;
    request.inputDType = input.getDataType();
    request.writeValue = value.has_value();
    request.writeIndex = index.has_value();
    request.valueOutputDType = value.has_value() ? value->getDataType() : DataType::FP32;
    request.indexOutputDType = index.has_value() ? index->getDataType() : DataType::UINT32;
    request.geometry = geometry;
    request.inputAlignmentBytes = pointerAlignment(input.getMemPtr());
    request.deviceNum = stream.getGpuNum();

    ScopedGpu scoped(stream.getGpuNum());
    ReductionLaunchPlan plan = buildReductionKernels(request);
    std::optional<Tensor> workspace = allocateReductionWorkspace(plan, input.getPlacement(), stream);
    return std::shared_ptr<StampedCubArgReduction>(
        new StampedCubArgReduction(op, geometry, input, std::move(value), std::move(index), std::move(plan), std::move(workspace), stream));
}

void StampedCubArgReduction::run() { runOn(stream); }
void StampedCubArgReduction::runOn(Stream& run_stream) const {
    if (!run_stream.isInitialized() || run_stream.getGpuNum() != static_cast<int>(gpuNum())) {
        throw std::invalid_argument("Stamped arg reduction must run on a stream of the GPU it was stamped for.");
    }
    ScopedGpu scoped(run_stream.getGpuNum());
    void* valuePtr = value_output.has_value() ? value_output->getMemPtr() : nullptr;
    void* indexPtr = index_output.has_value() ? index_output->getMemPtr() : nullptr;
    launchPlan(plan, input.getMemPtr(), valuePtr, indexPtr, workspace, 1.0f, run_stream.getStream());
}

}  // namespace ThorImplementation
