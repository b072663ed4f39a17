// Flat C binding, part 1: errors, Stream, Tensor, TypeConverter, CubReduction, CubArgReduction.
#include "capi_internal.h"

#include "CubScanInternal.h"
#include "ReductionPlanner.h"
#include "../device/thorhip_static_scratch.h"
#include "Utilities/Common/ScopedGpu.h"
#include "Utilities/Expression/SegmentedBroadcastKernel.h"
#include "Utilities/TensorOperations/Cub/CubDevicePrimitives.h"
#include "Utilities/TensorOperations/DataTypeConversions/TypeConverter.h"

#include <cstring>

using namespace ThorImplementation;

namespace thor_capi {
std::string& lastError() {
    static thread_local std::string slot;
    return slot;
}

void recordCurrentException() {
    try {
        throw;
    } catch (const std::invalid_argument& e) {
        lastError() = std::string("invalid_argument: ") + e.what();
    } catch (const std::out_of_range& e) {
        lastError() = std::string("out_of_range: ") + e.what();
    } catch (const std::logic_error& e) {
        lastError() = std::string("logic_error: ") + e.what();
    } catch (const std::runtime_error& e) {
        lastError() = std::string("runtime_error: ") + e.what();
    } catch (const std::exception& e) {
        lastError() = std::string("exception: ") + e.what();
    } catch (...) {
        lastError() = "exception: unknown";
    }
}

int copyOut(const std::string& text, char* buffer, size_t capacity, size_t* needed) {
    if (needed) *needed = text.size() + 1;
    if (buffer == nullptr || capacity == 0) return needed ? 0 : -1;
    const size_t n = std::min(text.size(), capacity - 1);
    std::memcpy(buffer, text.data(), n);
    buffer[n] = '\0';
    return text.size() + 1 <= capacity ? 0 : -2;
}
}  // namespace thor_capi

using namespace thor_capi;

namespace {
std::vector<uint32_t> axesOf(const uint32_t* axes, int n) { return std::vector<uint32_t>(axes, axes + (n > 0 ? n : 0)); }
std::vector<uint64_t> dimsOf(const uint64_t* dims, int n) { return std::vector<uint64_t>(dims, dims + (n > 0 ? n : 0)); }

CubReductionGeometry geometryOf(const uint64_t* dims, const uint64_t* strides, int rank, const uint32_t* axes, int num_axes) {
    if (strides == nullptr) return CubReduction::analyzeGeometry(dimsOf(dims, rank), axesOf(axes, num_axes));
    return CubReduction::analyzeGeometry(dimsOf(dims, rank), dimsOf(strides, rank), axesOf(axes, num_axes));
}
}  // namespace

extern "C" {

const char* thor_last_error(void) { return lastError().c_str(); }

// ---- Stream ---------------------------------------------------------------------------------------------------------------
thor_stream_t thor_stream_create(int gpu_num) {
    THOR_CAPI_TRY_PTR(return new thor_stream{Stream(gpu_num)};)
}
void thor_stream_destroy(thor_stream_t stream) { delete stream; }
int thor_stream_synchronize(thor_stream_t stream) {
    THOR_CAPI_TRY_INT(require(stream, "stream"); stream->stream.synchronize();)
}
void* thor_stream_raw(thor_stream_t stream) { return stream ? stream->stream.getStream() : nullptr; }
int thor_stream_gpu_num(thor_stream_t stream) { return stream ? stream->stream.getGpuNum() : -1; }

// ---- Tensor ---------------------------------------------------------------------------------------------------------------
thor_tensor_t thor_tensor_create(int device_type, int device_num, int dtype, const uint64_t* dims, int rank) {
    THOR_CAPI_TRY_PTR(
        if (rank <= 0 || dims == nullptr) throw std::invalid_argument("thor_tensor_create requires at least one dimension.");
        for (int i = 0; i < rank; ++i)
            if (dims[i] == 0) throw std::invalid_argument("Tensor dimensions must be non-zero.");
        const TensorPlacement placement(device_type == THOR_DEVICE_GPU ? TensorPlacement::MemDevices::GPU : TensorPlacement::MemDevices::CPU,
                                        device_type == THOR_DEVICE_GPU ? device_num : 0);
        (void)dataTypeSizeInBytes(static_cast<DataType>(dtype));
        return new thor_tensor{Tensor(placement, TensorDescriptor(static_cast<DataType>(dtype), dimsOf(dims, rank)))};)
}
thor_tensor_t thor_tensor_clone_handle(thor_tensor_t tensor) {
    THOR_CAPI_TRY_PTR(require(tensor, "tensor"); return new thor_tensor{tensor->tensor};)
}
void thor_tensor_destroy(thor_tensor_t tensor) { delete tensor; }
void* thor_tensor_mem_ptr(thor_tensor_t tensor) { return tensor ? tensor->tensor.getMemPtr() : nullptr; }
int thor_tensor_dtype(thor_tensor_t tensor) { return tensor ? static_cast<int>(tensor->tensor.getDataType()) : -1; }
int thor_tensor_rank(thor_tensor_t tensor) { return tensor ? static_cast<int>(tensor->tensor.getNumDimensions()) : -1; }
int thor_tensor_dims(thor_tensor_t tensor, uint64_t* dims_out) {
    THOR_CAPI_TRY_INT(require(tensor, "tensor"); const auto d = tensor->tensor.getDimensions(); std::copy(d.begin(), d.end(), dims_out);)
}
int thor_tensor_strides(thor_tensor_t tensor, uint64_t* strides_out) {
    THOR_CAPI_TRY_INT(require(tensor, "tensor"); const auto s = tensor->tensor.getStridesElements(); std::copy(s.begin(), s.end(), strides_out);)
}
uint64_t thor_tensor_num_elements(thor_tensor_t tensor) { return tensor ? tensor->tensor.getTotalNumElements() : 0; }
int thor_tensor_device_type(thor_tensor_t tensor) {
    if (!tensor) return -1;
    return tensor->tensor.getPlacement().getMemDevice() == TensorPlacement::MemDevices::GPU ? THOR_DEVICE_GPU : THOR_DEVICE_CPU;
}
int thor_tensor_device_num(thor_tensor_t tensor) { return tensor ? tensor->tensor.getPlacement().getDeviceNum() : -1; }
int thor_tensor_is_dense(thor_tensor_t tensor) { return tensor && tensor->tensor.isDenseContiguous() ? 1 : 0; }
int thor_tensor_copy_from_async(thor_tensor_t dest, thor_tensor_t source, thor_stream_t stream) {
    THOR_CAPI_TRY_INT(require(dest, "dest"); require(source, "source"); require(stream, "stream");
                      dest->tensor.copyFromAsync(source->tensor, stream->stream);)
}
int thor_tensor_memset_async(thor_tensor_t tensor, int byte_value, thor_stream_t stream) {
    THOR_CAPI_TRY_INT(require(tensor, "tensor"); require(stream, "stream");
                      tensor->tensor.memsetAsync(stream->stream, static_cast<int8_t>(byte_value));)
}
int thor_tensor_reshape(thor_tensor_t tensor, const uint64_t* dims, int rank) {
    THOR_CAPI_TRY_INT(require(tensor, "tensor"); tensor->tensor.reshape(dimsOf(dims, rank));)
}
thor_tensor_t thor_tensor_alias_view(thor_tensor_t tensor, const uint64_t* dims, const uint64_t* strides, int rank, uint64_t element_offset) {
    THOR_CAPI_TRY_PTR(require(tensor, "tensor");
                      return new thor_tensor{tensor->tensor.aliasView(dimsOf(dims, rank), dimsOf(strides, rank), element_offset)};)
}

// ---- TypeConverter ----------------------------------------------------------------------------------------------------------
int thor_convert_type(void* source, void* dest, int source_dtype, int dest_dtype, int64_t num_elements, thor_stream_t stream, int device_num) {
    THOR_CAPI_TRY_INT(require(stream, "stream");
                      if (source_dtype == dest_dtype) throw std::invalid_argument("convertType requires two different dtypes.");
                      if (num_elements < 0) throw std::invalid_argument("convertType requires a non-negative element count.");
                      TypeConverter::convertType(source, dest, static_cast<DataType>(source_dtype), static_cast<DataType>(dest_dtype),
                                                 static_cast<long>(num_elements), stream->stream, device_num);)
}
int thor_convert_type_cpu(const void* source, void* dest, int source_dtype, int dest_dtype, int64_t num_elements) {
    THOR_CAPI_TRY_INT(if (source_dtype == dest_dtype) throw std::invalid_argument("convertType requires two different dtypes.");
                      if (num_elements < 0) throw std::invalid_argument("convertType requires a non-negative element count.");
                      TypeConverter::cpuConvertNow(source, dest, static_cast<DataType>(source_dtype), static_cast<DataType>(dest_dtype),
                                                   static_cast<long>(num_elements));)
}

// ---- CubReduction -------------------------------------------------------------------------------------------------------------
int thor_reduction_analyze_geometry(const uint64_t* dims, const uint64_t* strides, int rank, const uint32_t* axes, int num_axes,
                                    thor_reduction_geometry* out) {
    THOR_CAPI_TRY_INT(
        if (out == nullptr) throw std::invalid_argument("thor_reduction_analyze_geometry: out is NULL");
        const CubReductionGeometry g = geometryOf(dims, strides, rank, axes, num_axes);
        if (g.rank > 16) throw std::invalid_argument("thor_reduction_analyze_geometry reports at most 16 dimensions.");
        std::memset(out, 0, sizeof *out);
        out->path = static_cast<int>(g.path);
        out->reduced_axes_are_contiguous = g.reduced_axes_are_contiguous;
        out->outer_size = g.outer_size;
        out->reduction_size = g.reduction_size;
        out->inner_size = g.inner_size;
        out->input_elements = g.input_elements;
        out->output_elements = g.output_elements;
        out->rank = static_cast<int>(g.rank);
        std::copy(g.output_dimensions.begin(), g.output_dimensions.end(), out->output_dimensions);
        out->squeezed_rank = static_cast<int>(g.squeezed_output_dimensions.size());
        std::copy(g.squeezed_output_dimensions.begin(), g.squeezed_output_dimensions.end(), out->squeezed_output_dimensions);
        out->device_transform_uses_affine_stride = g.device_transform_uses_affine_stride;
        out->affine_input_stride = g.affine_input_stride;)
}

int thor_reduction_map_index(const uint64_t* dims, const uint64_t* strides, int rank, const uint32_t* axes, int num_axes,
                             uint64_t output_index, uint64_t reduction_index, uint64_t* physical_index) {
    THOR_CAPI_TRY_INT(const CubReductionGeometry g = geometryOf(dims, strides, rank, axes, num_axes);
                      *physical_index = CubReduction::mapLogicalReductionIndexToPhysicalIndex(g, output_index, reduction_index);)
}

thor_stamped_reduction_t thor_reduction_stamp(int op, const uint32_t* axes, int num_axes, int output_dtype, float output_scale,
                                              thor_tensor_t input, thor_tensor_t preallocated_output, thor_stream_t stream) {
    THOR_CAPI_TRY_PTR(
        require(input, "input"); require(stream, "stream");
        std::optional<DataType> out;
        if (output_dtype >= 0) out = static_cast<DataType>(output_dtype);
        const CubReduction reduction(static_cast<CubReductionOp>(op), axesOf(axes, num_axes), out, output_scale);
        auto stamped = preallocated_output ? reduction.stamp(input->tensor, preallocated_output->tensor, stream->stream)
                                           : reduction.stamp(input->tensor, stream->stream);
        return new thor_stamped_reduction{stamped};)
}
void thor_stamped_reduction_destroy(thor_stamped_reduction_t r) { delete r; }
int thor_stamped_reduction_run(thor_stamped_reduction_t r) { THOR_CAPI_TRY_INT(require(r, "reduction"); r->stamped->run();) }
int thor_stamped_reduction_run_scaled(thor_stamped_reduction_t r, float scale) {
    THOR_CAPI_TRY_INT(require(r, "reduction"); r->stamped->run(scale);)
}
int thor_stamped_reduction_run_on(thor_stamped_reduction_t r, thor_stream_t stream) {
    THOR_CAPI_TRY_INT(require(r, "reduction"); require(stream, "stream"); r->stamped->runOn(stream->stream);)
}
thor_tensor_t thor_stamped_reduction_output(thor_stamped_reduction_t r) {
    THOR_CAPI_TRY_PTR(require(r, "reduction"); return new thor_tensor{r->stamped->getOutputTensor()};)
}
int thor_stamped_reduction_path(thor_stamped_reduction_t r) { return r ? static_cast<int>(r->stamped->getPath()) : -1; }
size_t thor_stamped_reduction_workspace_bytes(thor_stamped_reduction_t r) { return r ? r->stamped->getWorkspaceSizeInBytes() : 0; }
int thor_stamped_reduction_variant(thor_stamped_reduction_t r, char* buffer, size_t capacity) {
    THOR_CAPI_TRY_INT(require(r, "reduction"); copyOut(r->stamped->getKernelVariant(), buffer, capacity, nullptr);)
}

int thor_reduction_generate_source(int is_arg, int op, int input_dtype, int output_dtype, int index_dtype, const uint64_t* dims,
                                   const uint64_t* strides, int rank, const uint32_t* axes, int num_axes, char* buffer, size_t capacity,
                                   size_t* needed) {
    THOR_CAPI_TRY_INT(
        ReductionKernelRequest request;
        request.isArg = is_arg != 0;
        if (is_arg) {
            request.argOp = static_cast<CubArgReductionOp>(op);
            request.writeIndex = true;
            request.writeValue = true;
        } else {
            request.valueOp = static_cast<CubReductionOp>(op);
        }
        request.inputDType = static_cast<DataType>(input_dtype);
        request.valueOutputDType = static_cast<DataType>(output_dtype);
        request.indexOutputDType = static_cast<DataType>(index_dtype);
        request.geometry = geometryOf(dims, strides, rank, axes, num_axes);
        const ReductionShape shape = planReductionShape(request);
        copyOut(generateReductionSource(request, shape), buffer, capacity, needed);)
}

// ---- CubArgReduction --------------------------------------------------------------------------------------------------------------
thor_stamped_arg_reduction_t thor_arg_reduction_stamp(int op, const uint32_t* axes, int num_axes, int produce_value, int produce_index,
                                                      int value_output_dtype, int index_output_dtype, thor_tensor_t input,
                                                      thor_tensor_t preallocated_value, thor_tensor_t preallocated_index,
                                                      thor_stream_t stream) {
    THOR_CAPI_TRY_PTR(
        require(input, "input"); require(stream, "stream");
        CubArgReductionOutputOptions options;
        options.produce_value = produce_value != 0;
        options.produce_index = produce_index != 0;
        if (value_output_dtype >= 0) options.value_output_dtype = static_cast<DataType>(value_output_dtype);
        if (index_output_dtype >= 0) options.index_output_dtype = static_cast<DataType>(index_output_dtype);
        const CubArgReduction reduction(static_cast<CubArgReductionOp>(op), axesOf(axes, num_axes), options);
        std::optional<Tensor> value, index;
        if (preallocated_value) value = preallocated_value->tensor;
        if (preallocated_index) index = preallocated_index->tensor;
        return new thor_stamped_arg_reduction{reduction.stamp(input->tensor, value, index, stream->stream)};)
}
void thor_stamped_arg_reduction_destroy(thor_stamped_arg_reduction_t r) { delete r; }
int thor_stamped_arg_reduction_run(thor_stamped_arg_reduction_t r) { THOR_CAPI_TRY_INT(require(r, "arg reduction"); r->stamped->run();) }
thor_tensor_t thor_stamped_arg_reduction_value_output(thor_stamped_arg_reduction_t r) {
    if (!r || !r->stamped->getValueOutputTensor().has_value()) return nullptr;
    return new thor_tensor{r->stamped->getValueOutputTensor().value()};
}
thor_tensor_t thor_stamped_arg_reduction_index_output(thor_stamped_arg_reduction_t r) {
    if (!r || !r->stamped->getIndexOutputTensor().has_value()) return nullptr;
    return new thor_tensor{r->stamped->getIndexOutputTensor().value()};
}
int thor_stamped_arg_reduction_path(thor_stamped_arg_reduction_t r) { return r ? static_cast<int>(r->stamped->getPath()) : -1; }
int thor_stamped_arg_reduction_variant(thor_stamped_arg_reduction_t r, char* buffer, size_t capacity) {
    THOR_CAPI_TRY_INT(require(r, "arg reduction"); copyOut(r->stamped->getKernelVariant(), buffer, capacity, nullptr);)
}

thor_stamped_segmented_reduction_t thor_segmented_reduction_stamp(int is_arg, int op, int dtype, thor_tensor_t input, thor_tensor_t segment_offsets,
                                                                  thor_tensor_t preallocated_output, int runtime_offsets, thor_stream_t stream) {
    THOR_CAPI_TRY_PTR(
        require(input, "input"); require(segment_offsets, "segment offsets"); require(stream, "stream");
        if (runtime_offsets && !preallocated_output) throw std::invalid_argument("stampRuntimeOffsets requires a preallocated output.");
        auto handle = std::make_unique<thor_stamped_segmented_reduction>();
        if (is_arg) {
            const CubSegmentedArgReduction reduction(static_cast<CubArgReductionOp>(op), dtype >= 0 ? static_cast<DataType>(dtype) : DataType::UINT64);
            if (runtime_offsets) {
                handle->arg = reduction.stampRuntimeOffsets(input->tensor, preallocated_output->tensor, segment_offsets->tensor, stream->stream);
            } else if (preallocated_output) {
                handle->arg = reduction.stamp(input->tensor, preallocated_output->tensor, segment_offsets->tensor, stream->stream);
            } else {
                handle->arg = reduction.stamp(input->tensor, segment_offsets->tensor, stream->stream);
            }
        } else {
            const CubSegmentedReduction reduction(static_cast<CubReductionOp>(op),
                                                  dtype >= 0 ? std::optional<DataType>(static_cast<DataType>(dtype)) : std::nullopt);
            if (runtime_offsets) {
                handle->value = reduction.stampRuntimeOffsets(input->tensor, preallocated_output->tensor, segment_offsets->tensor, stream->stream);
            } else if (preallocated_output) {
                handle->value = reduction.stamp(input->tensor, preallocated_output->tensor, segment_offsets->tensor, stream->stream);
            } else {
                handle->value = reduction.stamp(input->tensor, segment_offsets->tensor, stream->stream);
            }
        }
        return handle.release();)
}
void thor_stamped_segmented_reduction_destroy(thor_stamped_segmented_reduction_t r) { delete r; }
int thor_stamped_segmented_reduction_run(thor_stamped_segmented_reduction_t r) {
    THOR_CAPI_TRY_INT(require(r, "segmented reduction"); if (r->value) r->value->run(); else r->arg->run();)
}
thor_tensor_t thor_stamped_segmented_reduction_output(thor_stamped_segmented_reduction_t r) {
    if (!r) return nullptr;
    return new thor_tensor{r->value ? r->value->getOutputTensor() : r->arg->getIndexOutputTensor()};
}
size_t thor_stamped_segmented_reduction_workspace_bytes(thor_stamped_segmented_reduction_t r) {
    if (!r) return 0;
    return r->value ? r->value->getWorkspaceSizeInBytes() : r->arg->getWorkspaceSizeInBytes();
}
int thor_stamped_segmented_reduction_variant(thor_stamped_segmented_reduction_t r, char* buffer, size_t capacity) {
    THOR_CAPI_TRY_INT(require(r, "segmented reduction");
                      copyOut(r->value ? r->value->getKernelVariant() : r->arg->getKernelVariant(), buffer, capacity, nullptr);)
}

int thor_segmented_broadcast(thor_tensor_t per_segment_values, thor_tensor_t segment_offsets, thor_tensor_t output, int normalize_by_segment_length,
                             thor_stream_t stream) {
    THOR_CAPI_TRY_INT(require(per_segment_values, "per-segment values"); require(segment_offsets, "segment offsets"); require(output, "output");
                      require(stream, "stream");
                      launchSegmentedBroadcast(per_segment_values->tensor, segment_offsets->tensor, output->tensor, normalize_by_segment_length != 0,
                                               stream->stream);)
}

int thor_select_flagged(thor_tensor_t input, thor_tensor_t flags, thor_tensor_t output, thor_tensor_t num_selected_out, uint64_t num_items,
                        thor_stream_t stream, char* variant, size_t variant_capacity) {
    THOR_CAPI_TRY_INT(require(input, "input"); require(flags, "flags"); require(output, "output"); require(num_selected_out, "num_selected_out");
                      require(stream, "stream");
                      const auto plan = prepareCubDeviceSelectFlagged(input->tensor, flags->tensor, output->tensor, num_selected_out->tensor, num_items);
                      cubDeviceSelectFlagged(plan, allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes), input->tensor, flags->tensor,
                                             output->tensor, num_selected_out->tensor, stream->stream);
                      if (variant) copyOut(cubSelectionKernelVariant(plan.kernels), variant, variant_capacity, nullptr);)
}

int thor_topk(thor_tensor_t keys_in, thor_tensor_t keys_out, thor_tensor_t values_in, thor_tensor_t values_out, uint64_t num_segments,
              uint64_t segment_size, uint64_t k, int largest, int segmented, thor_stream_t stream, char* variant, size_t variant_capacity) {
    THOR_CAPI_TRY_INT(
        require(keys_in, "keys_in"); require(keys_out, "keys_out"); require(stream, "stream");
        if ((values_in == nullptr) != (values_out == nullptr)) throw std::invalid_argument("top-k takes values_in and values_out together or neither");
        const CubTopKOrder order = largest ? CubTopKOrder::Largest : CubTopKOrder::Smallest;
        std::shared_ptr<const CubSelectionKernels> kernels;
        if (segmented) {
            if (values_in) {
                const auto plan = prepareCubDeviceSegmentedTopKPairs(keys_in->tensor, keys_out->tensor, values_in->tensor, values_out->tensor,
                                                                     num_segments, segment_size, k, order);
                cubDeviceSegmentedTopKPairs(plan, allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes), keys_in->tensor, keys_out->tensor,
                                            values_in->tensor, values_out->tensor, stream->stream);
                kernels = plan.kernels;
            } else {
                const auto plan = prepareCubDeviceSegmentedTopKKeys(keys_in->tensor, keys_out->tensor, num_segments, segment_size, k, order);
                cubDeviceSegmentedTopKKeys(plan, allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes), keys_in->tensor, keys_out->tensor,
                                           stream->stream);
                kernels = plan.kernels;
            }
        } else if (values_in) {
            const auto plan = prepareCubDeviceTopKPairs(keys_in->tensor, keys_out->tensor, values_in->tensor, values_out->tensor, segment_size, k, order);
            cubDeviceTopKPairs(plan, allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes), keys_in->tensor, keys_out->tensor,
                               values_in->tensor, values_out->tensor, stream->stream);
            kernels = plan.kernels;
        } else {
            const auto plan = prepareCubDeviceTopKKeys(keys_in->tensor, keys_out->tensor, segment_size, k, order);
            cubDeviceTopKKeys(plan, allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes), keys_in->tensor, keys_out->tensor, stream->stream);
            kernels = plan.kernels;
        }
        if (variant) copyOut(cubSelectionKernelVariant(kernels), variant, variant_capacity, nullptr);)
}

struct thor_selection_plan {
    int kind = 0;  // 0 select-flagged, 1 top-k keys, 2 top-k pairs, 3 row top-k keys, 4 row top-k pairs
    CubDeviceSelectFlaggedPlan select;
    CubDeviceTopKKeysPlan keys;
    CubDeviceTopKPairsPlan pairs;
    CubDeviceSegmentedTopKKeysPlan rowKeys;
    CubDeviceSegmentedTopKPairsPlan rowPairs;
    size_t tempBytes = 1;
    std::shared_ptr<const CubSelectionKernels> kernels;
};

thor_selection_plan_t thor_select_flagged_prepare(thor_tensor_t input, thor_tensor_t flags, thor_tensor_t output, thor_tensor_t num_selected_out,
                                                  uint64_t num_items) {
    THOR_CAPI_TRY_PTR(require(input, "input"); require(flags, "flags"); require(output, "output"); require(num_selected_out, "num_selected_out");
                      auto handle = std::make_unique<thor_selection_plan>();
                      handle->select = prepareCubDeviceSelectFlagged(input->tensor, flags->tensor, output->tensor, num_selected_out->tensor, num_items);
                      handle->tempBytes = handle->select.temp_storage_bytes; handle->kernels = handle->select.kernels; return handle.release();)
}

thor_selection_plan_t thor_topk_prepare(thor_tensor_t keys_in, thor_tensor_t keys_out, thor_tensor_t values_in, thor_tensor_t values_out,
                                        uint64_t num_segments, uint64_t segment_size, uint64_t k, int largest, int segmented) {
    THOR_CAPI_TRY_PTR(
        require(keys_in, "keys_in"); require(keys_out, "keys_out");
        if ((values_in == nullptr) != (values_out == nullptr)) throw std::invalid_argument("top-k takes values_in and values_out together or neither");
        const CubTopKOrder order = largest ? CubTopKOrder::Largest : CubTopKOrder::Smallest;
        auto handle = std::make_unique<thor_selection_plan>();
        if (segmented && values_in) {
            handle->kind = 4;
            handle->rowPairs = prepareCubDeviceSegmentedTopKPairs(keys_in->tensor, keys_out->tensor, values_in->tensor, values_out->tensor, num_segments,
                                                                  segment_size, k, order);
            handle->tempBytes = handle->rowPairs.temp_storage_bytes;
            handle->kernels = handle->rowPairs.kernels;
        } else if (segmented) {
            handle->kind = 3;
            handle->rowKeys = prepareCubDeviceSegmentedTopKKeys(keys_in->tensor, keys_out->tensor, num_segments, segment_size, k, order);
            handle->tempBytes = handle->rowKeys.temp_storage_bytes;
            handle->kernels = handle->rowKeys.kernels;
        } else if (values_in) {
            handle->kind = 2;
            handle->pairs = prepareCubDeviceTopKPairs(keys_in->tensor, keys_out->tensor, values_in->tensor, values_out->tensor, segment_size, k, order);
            handle->tempBytes = handle->pairs.temp_storage_bytes;
            handle->kernels = handle->pairs.kernels;
        } else {
            handle->kind = 1;
            handle->keys = prepareCubDeviceTopKKeys(keys_in->tensor, keys_out->tensor, segment_size, k, order);
            handle->tempBytes = handle->keys.temp_storage_bytes;
            handle->kernels = handle->keys.kernels;
        }
        return handle.release();)
}

size_t thor_selection_plan_temp_bytes(thor_selection_plan_t plan) { return plan ? plan->tempBytes : 0; }

int thor_selection_plan_run(thor_selection_plan_t plan, thor_tensor_t temp_storage, thor_tensor_t a, thor_tensor_t b, thor_tensor_t c, thor_tensor_t d,
                            thor_stream_t stream) {
    THOR_CAPI_TRY_INT(
        require(plan, "selection plan"); require(temp_storage, "temp_storage"); require(a, "first tensor"); require(b, "second tensor");
        require(stream, "stream");
        const bool four = plan->kind == 0 || plan->kind == 2 || plan->kind == 4;
        if (four) {
            require(c, "third tensor");
            require(d, "fourth tensor");
        }
        switch (plan->kind) {
            case 0: cubDeviceSelectFlagged(plan->select, temp_storage->tensor, a->tensor, b->tensor, c->tensor, d->tensor, stream->stream); break;
            case 1: cubDeviceTopKKeys(plan->keys, temp_storage->tensor, a->tensor, b->tensor, stream->stream); break;
            case 2: cubDeviceTopKPairs(plan->pairs, temp_storage->tensor, a->tensor, b->tensor, c->tensor, d->tensor, stream->stream); break;
            case 3: cubDeviceSegmentedTopKKeys(plan->rowKeys, temp_storage->tensor, a->tensor, b->tensor, stream->stream); break;
            default: cubDeviceSegmentedTopKPairs(plan->rowPairs, temp_storage->tensor, a->tensor, b->tensor, c->tensor, d->tensor, stream->stream); break;
        })
}

int thor_selection_plan_variant(thor_selection_plan_t plan, char* buffer, size_t capacity) {
    THOR_CAPI_TRY_INT(require(plan, "selection plan"); copyOut(cubSelectionKernelVariant(plan->kernels), buffer, capacity, nullptr);)
}

void thor_selection_plan_destroy(thor_selection_plan_t plan) { delete plan; }

int thor_scan(thor_tensor_t input, thor_tensor_t output, thor_tensor_t offsets, uint64_t num_items, uint64_t num_segments, uint64_t segment_size,
              int op, int arg, int inclusive, int reverse, thor_stream_t stream, char* variant, size_t variant_capacity) {
    THOR_CAPI_TRY_INT(
        require(input, "input"); require(output, "output"); require(stream, "stream");
        if (op < 0 || op > 3 || (arg != 0 && op != 1 && op != 2)) throw std::invalid_argument("scan op must be 0..3 (1 or 2 for arg scans)");
        const CubScanMode mode = inclusive ? CubScanMode::Inclusive : CubScanMode::Exclusive;
        const CubScanDirection direction = reverse ? CubScanDirection::Reverse : CubScanDirection::Forward;
        const CubScanOp valueOp = static_cast<CubScanOp>(op);
        const CubArgScanOp argOp = op == 1 ? CubArgScanOp::ArgMin : CubArgScanOp::ArgMax;
        const Tensor& in = input->tensor;
        Tensor& out = output->tensor;
        std::shared_ptr<const CubScanKernels> kernels;
        Tensor temp;
        if (offsets) {
            if (arg) {
                const auto plan = prepareCubDeviceSegmentedArgScan(in, out, offsets->tensor, num_items, num_segments, argOp, mode, direction);
                temp = allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes);
                cubDeviceSegmentedArgScan(plan, temp, in, out, offsets->tensor, stream->stream);
                kernels = plan.kernels;
            } else {
                const auto plan = prepareCubDeviceSegmentedScan(in, out, offsets->tensor, num_items, num_segments, valueOp, mode, direction);
                temp = allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes);
                cubDeviceSegmentedScan(plan, temp, in, out, offsets->tensor, stream->stream);
                kernels = plan.kernels;
            }
        } else if (segment_size > 0) {
            if (arg) {
                const auto plan = prepareCubDeviceSegmentedUniformArgScan(in, out, num_items, num_items / segment_size, segment_size, argOp, mode, direction);
                temp = allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes);
                cubDeviceSegmentedUniformArgScan(plan, temp, in, out, stream->stream);
                kernels = plan.kernels;
            } else {
                const auto plan = prepareCubDeviceSegmentedUniformScan(in, out, num_items, num_items / segment_size, segment_size, valueOp, mode, direction);
                temp = allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes);
                cubDeviceSegmentedUniformScan(plan, temp, in, out, stream->stream);
                kernels = plan.kernels;
            }
        } else if (arg) {
            const auto plan = prepareCubDeviceArgScan(in, out, num_items, argOp, mode, direction);
            temp = allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes);
            cubDeviceArgScan(plan, temp, in, out, stream->stream);
            kernels = plan.kernels;
        } else {
            const auto plan = prepareCubDeviceScan(in, out, num_items, valueOp, mode, direction);
            temp = allocateCubTemporaryStorage(plan.placement, plan.temp_storage_bytes);
            cubDeviceScan(plan, temp, in, out, stream->stream);
            kernels = plan.kernels;
        }
        // this entry point frees its temporary storage on return, which waits for the device anyway: waits between blocks that
        // gave up (and worked their totals out again, so the results are complete) are counted here
        scanWaitsRecovered(*kernels, temp.getMemPtr(), stream->stream);
        if (variant) copyOut(cubScanKernelVariant(kernels), variant, variant_capacity, nullptr);)
}

uint64_t thor_scan_waits_recovered(void) { return scanWaitsRecoveredTotal(); }

int thor_scan_no_alloc(thor_tensor_t input, thor_tensor_t output, thor_tensor_t offsets, uint64_t num_items, uint64_t num_segments,
                       uint64_t segment_size, int op, int arg, int inclusive, int reverse, thor_stream_t stream, char* variant, size_t variant_capacity) {
    THOR_CAPI_TRY_INT(
        require(input, "input"); require(output, "output"); require(stream, "stream");
        if (!input->tensor.isInitialized() || input->tensor.getPlacement().getMemDevice() != TensorPlacement::MemDevices::GPU) {
            throw std::invalid_argument("CUB scan requires initialized input and output tensors on a GPU.");
        }
        // the scratch block of the GPU that holds the tensors: looked up with that GPU current
        ScopedGpu scoped(static_cast<int>(input->tensor.getPlacement().getDeviceNum()));
        void* scratch = nullptr;
        size_t capacity = 0;
        if (thorhip::staticScratch(&scratch, &capacity) != 0) throw std::runtime_error(thorhip_last_error());
        const auto kernels = scanWithLoadedKernels(input->tensor, output->tensor, offsets ? &offsets->tensor : nullptr, num_items, num_segments, segment_size,
                                                   op, arg != 0, inclusive != 0, reverse != 0, scratch, capacity, stream->stream);
        if (variant) copyOut(cubScanKernelVariant(kernels), variant, variant_capacity, nullptr);)
}

}  // extern "C"
