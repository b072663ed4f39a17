// Dense tensor reductions over one or more axes -- sum, min, max, product, mean, L1 / L2 norm, argmin, argmax -- for
// MI355X.  The class and method names, the geometry analysis and its path names follow the reference's CUB-backed
// API so callers and tests carry over (Utilities/TensorOperations/Cub/CubReduction.h:16-153,175-234,412-537); the
// kernels underneath are wave64 HIP kernels specialised and compiled per shape at stamp time, not CUB.
//
// Contract kept from the reference: stamp() validates, plans, compiles, allocates the output and the workspace;
// run() / runOn() only launches.  Every path converts inputs to fp32, accumulates in fp32, finalises (mean division,
// L2 square root) in fp32, multiplies by the fp32 output scale and converts once to the output storage dtype.
// Min / max propagate NaN.  Arg reductions return the row-major position inside the reduction domain; NaN wins and
// the lowest index wins ties.
#pragma once

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"

#include <cstddef>
#include <cstdint>
#include <limits>
#include <memory>
#include <optional>
#include <string>
#include <vector>

namespace ThorImplementation {

struct CompiledKernel;

enum class CubReductionOp : uint8_t { Sum = 0, Min = 1, Max = 2, Product = 3, Mean = 4, L1Norm = 5, L2Norm = 6 };
enum class CubArgReductionOp : uint8_t { ArgMin = 0, ArgMax = 1 };

struct CubArgReductionOutputOptions {
    bool produce_value = true;
    bool produce_index = true;
    std::optional<DataType> value_output_dtype = std::nullopt;
    DataType index_output_dtype = DataType::UINT32;
};

// Which kernel family a geometry maps to.  The names are the reference's; here they mean:
//   DeviceTransformReduce   whole tensor (or a rank-1 strided view) -> one value: per-block partials, then a one-block finishing launch
//   ContiguousFixedSegment  [outer, R] rows, R contiguous: 1..64 lanes or one block per row
//   TiledFixedSegment       [outer, R, inner] with inner > 1: one lane per inner vector, R optionally split
//   StridedFixedSegment     anything else (disjoint axes, views): generated address arithmetic, R optionally split
//   OffsetSegmented         [N, D...] rows reduced over runtime row ranges (CubSegmentedReduction below)
enum class CubReductionPath : uint8_t {
    DeviceTransformReduce = 0,
    ContiguousFixedSegment = 1,
    TiledFixedSegment = 2,
    StridedFixedSegment = 3,
    OffsetSegmented = 4,
};

struct CubReductionIndexing {
    std::vector<uint32_t> reduced_axes;
    std::vector<uint32_t> retained_axes;
    std::vector<uint64_t> input_strides;
    std::vector<uint64_t> reduced_dimensions;
    std::vector<uint64_t> retained_dimensions;
};

struct CubReductionGeometry {
    std::vector<uint32_t> axes;
    uint32_t rank = 0;

    // When the reduced axes form one contiguous block of a dense tensor the input is [outer_size, reduction_size,
    // inner_size]; outer_size and inner_size stay zero otherwise.
    bool reduced_axes_are_contiguous = false;
    uint64_t outer_size = 0;
    uint64_t inner_size = 0;

    uint64_t input_elements = 0;
    uint64_t reduction_size = 0;
    uint64_t output_elements = 0;
    std::vector<uint64_t> output_dimensions;           // reduced axes kept as 1
    std::vector<uint64_t> squeezed_output_dimensions;  // reduced axes removed ({1} when nothing is left)
    CubReductionIndexing indexing;

    // A rank-1 view with a stride other than 1 (a matrix diagonal, a broadcast alias) still reduces to one value on
    // the whole-tensor path.
    bool device_transform_uses_affine_stride = false;
    uint64_t affine_input_stride = 1;

    uint64_t tiled_output_outer_stride = 0;
    uint64_t tiled_output_inner_stride = 0;

    CubReductionPath path = CubReductionPath::DeviceTransformReduce;
};

class StampedCubReduction;
class StampedCubArgReduction;

class CubReduction {
   public:
    CubReduction(CubReductionOp op, uint32_t axis, std::optional<DataType> output_dtype = std::nullopt, float output_scale = 1.0f);
    CubReduction(CubReductionOp op, std::vector<uint32_t> axes, std::optional<DataType> output_dtype = std::nullopt,
                 float output_scale = 1.0f);

    CubReductionOp getOperation() const { return op; }
    uint32_t getAxis() const { return axes.front(); }
    const std::vector<uint32_t>& getAxes() const { return axes; }
    std::optional<DataType> getConfiguredOutputDataType() const { return output_dtype; }
    float getOutputScale() const { return output_scale; }
    DataType resolveOutputDataType(DataType input_dtype) const;

    // The value an empty reduction domain would produce (sum/mean/norms 0, product 1, min +inf, max -inf).
    static float getFp32EmptyReductionValue(CubReductionOp op);

    static CubReductionGeometry analyzeGeometry(const std::vector<uint64_t>& input_dimensions, uint32_t axis);
    static CubReductionGeometry analyzeGeometry(const std::vector<uint64_t>& input_dimensions, const std::vector<uint32_t>& axes);
    static CubReductionGeometry analyzeGeometry(const std::vector<uint64_t>& input_dimensions,
                                                const std::vector<uint64_t>& input_strides, const std::vector<uint32_t>& axes);

    // Physical element offset of logical (output, reduction) coordinates; both are row-major flat indices.
    static uint64_t mapLogicalReductionIndexToPhysicalIndex(const CubReductionGeometry& geometry, uint64_t output_index,
                                                            uint64_t reduction_index);

    size_t queryWorkspaceSizeInBytes(const TensorDescriptor& input_descriptor, const Stream& stream) const;

    std::shared_ptr<StampedCubReduction> stamp(const Tensor& input, const Stream& stream) const;
    std::shared_ptr<StampedCubReduction> stamp(const Tensor& input, const Tensor& preallocated_output, const Stream& stream) const;

   private:
    CubReductionOp op;
    std::vector<uint32_t> axes;
    std::optional<DataType> output_dtype;
    float output_scale;
};

class CubArgReduction {
   public:
    CubArgReduction(CubArgReductionOp op, uint32_t axis, CubArgReductionOutputOptions outputs = {});
    CubArgReduction(CubArgReductionOp op, std::vector<uint32_t> axes, CubArgReductionOutputOptions outputs = {});

    CubArgReductionOp getOperation() const { return op; }
    uint32_t getAxis() const { return axes.front(); }
    const std::vector<uint32_t>& getAxes() const { return axes; }
    const CubArgReductionOutputOptions& getOutputOptions() const { return outputs; }
    DataType resolveValueOutputDataType(DataType input_dtype) const;
    static float getFp32EmptyReductionValue(CubArgReductionOp op);
    static uint64_t getEmptyReductionIndex() { return std::numeric_limits<uint64_t>::max(); }

    std::shared_ptr<StampedCubArgReduction> stamp(const Tensor& input, const Stream& stream) const;
    std::shared_ptr<StampedCubArgReduction> stamp(const Tensor& input, const std::optional<Tensor>& preallocated_value_output,
                                                  const std::optional<Tensor>& preallocated_index_output, const Stream& stream) const;

   private:
    CubArgReductionOp op;
    std::vector<uint32_t> axes;
    CubArgReductionOutputOptions outputs;
};

class StampedCubSegmentedReduction;
class StampedCubSegmentedArgReduction;

// Offset-segmented reduction of dense values [N, D...] -> [B, D...] (reference: CubReduction.h:236-330).  Segment i is the
// half-open row range [offsets[i], offsets[i + 1]) of a rank-1 UINT32 / UINT64 offsets tensor with B + 1 entries.  Inputs
// convert to fp32, all arithmetic is fp32.  Empty segments give getFp32EmptyReductionValue(); a mean divides by the
// segment's row count and is 0 for an empty segment.  Supported: sum, mean, min, max.  stamp() reads and validates the
// offsets (zero based, non-decreasing, within N); stampRuntimeOffsets() only checks shapes and dtypes, for offsets that
// are filled in later.  Either way the kernels read the offsets when they run, so the partition may change between runs.
class CubSegmentedReduction {
   public:
    explicit CubSegmentedReduction(CubReductionOp op, std::optional<DataType> output_dtype = std::nullopt);

    CubReductionOp getOperation() const { return op; }
    std::optional<DataType> getConfiguredOutputDataType() const { return output_dtype; }
    DataType resolveOutputDataType(DataType input_dtype) const { return output_dtype.value_or(input_dtype); }
    static bool isInputDataTypeSupported(DataType dtype);
    static bool isOffsetDataTypeSupported(DataType dtype) { return dtype == DataType::UINT32 || dtype == DataType::UINT64; }

    std::shared_ptr<StampedCubSegmentedReduction> stamp(const Tensor& input, const Tensor& segment_offsets, const Stream& stream) const;
    std::shared_ptr<StampedCubSegmentedReduction> stamp(const Tensor& input, const Tensor& preallocated_output, const Tensor& segment_offsets,
                                                        const Stream& stream) const;
    std::shared_ptr<StampedCubSegmentedReduction> stampRuntimeOffsets(const Tensor& input, const Tensor& preallocated_output,
                                                                      const Tensor& segment_offsets, const Stream& stream) const;

   private:
    std::shared_ptr<StampedCubSegmentedReduction> stampValidated(const Tensor& input, const Tensor& output, const Tensor& segment_offsets,
                                                                 const Stream& stream) const;
    CubReductionOp op;
    std::optional<DataType> output_dtype;
};

// Offset-segmented argmin / argmax over packed values [N, D...]: winners are global packed indices row * D + d, UINT64
// (default) or UINT32; NaN wins, the lowest index wins ties, empty segments give the all-ones index of the output dtype
// (reference: CubReduction.h:331-400).
class CubSegmentedArgReduction {
   public:
    explicit CubSegmentedArgReduction(CubArgReductionOp op, DataType index_output_dtype = DataType::UINT64);

    CubArgReductionOp getOperation() const { return op; }
    DataType getIndexOutputDataType() const { return index_output_dtype; }
    static bool isInputDataTypeSupported(DataType dtype) { return CubSegmentedReduction::isInputDataTypeSupported(dtype); }
    static bool isOffsetDataTypeSupported(DataType dtype) { return CubSegmentedReduction::isOffsetDataTypeSupported(dtype); }

    std::shared_ptr<StampedCubSegmentedArgReduction> stamp(const Tensor& input, const Tensor& segment_offsets, const Stream& stream) const;
    std::shared_ptr<StampedCubSegmentedArgReduction> stamp(const Tensor& input, const Tensor& preallocated_index_output,
                                                           const Tensor& segment_offsets, const Stream& stream) const;
    std::shared_ptr<StampedCubSegmentedArgReduction> stampRuntimeOffsets(const Tensor& input, const Tensor& preallocated_index_output,
                                                                         const Tensor& segment_offsets, const Stream& stream) const;

   private:
    std::shared_ptr<StampedCubSegmentedArgReduction> stampValidated(const Tensor& input, const Tensor& index_output, const Tensor& segment_offsets,
                                                                    const Stream& stream) const;
    CubArgReductionOp op;
    DataType index_output_dtype;
};

// The launch recipe a stamp produced: up to two kernels (main + fold of split partials) with fixed grids.
struct ReductionLaunchPlan {
    std::shared_ptr<CompiledKernel> mainKernel;
    std::shared_ptr<CompiledKernel> finishKernel;  // null unless the reduction domain was split across blocks
    std::shared_ptr<CompiledKernel> prepareKernel; // offset-segmented reductions over several chunks: runs before the main kernel
    uint32_t prepareGridX = 1, prepareThreads = 256;
    uint32_t mainGridX = 1, mainGridY = 1, mainThreads = 256;
    uint32_t finishGridX = 1, finishThreads = 256;
    size_t workspaceBytes = 0;  // per-block / per-share partials, then the ticket words
    size_t ticketOffset = 0, ticketBytes = 0;  // part of the workspace that must be zero before the first run (0 bytes: none)
    std::string variant;        // human-readable description of the chosen kernel shape
};

class StampedCubReduction {
   public:
    void run();
    void run(float output_scale);
    void runOn(Stream& run_stream) const;
    void runOn(Stream& run_stream, float output_scale) const;

    uint32_t gpuNum() const { return output.getPlacement().getDeviceNum(); }
    Tensor getInputTensor() const { return input; }
    Tensor getOutputTensor() const { return output; }
    CubReductionOp getOperation() const { return op; }
    CubReductionPath getPath() const { return geometry.path; }
    DataType getInputDataType() const { return input.getDataType(); }
    DataType getOutputDataType() const { return output.getDataType(); }
    DataType getAccumulatorDataType() const { return DataType::FP32; }
    const CubReductionGeometry& getGeometry() const { return geometry; }
    size_t getWorkspaceSizeInBytes() const { return plan.workspaceBytes; }
    float getOutputScale() const { return output_scale; }
    const std::string& getKernelVariant() const { return plan.variant; }

   private:
    friend class CubReduction;
    StampedCubReduction(CubReductionOp op, CubReductionGeometry geometry, const Tensor& input, const Tensor& output,
                        ReductionLaunchPlan plan, std::optional<Tensor> workspace, float output_scale, const Stream& stream)
        : op(op), geometry(std::move(geometry)), input(input), output(output), plan(std::move(plan)),
          workspace(std::move(workspace)), output_scale(output_scale), stream(stream) {}

    CubReductionOp op;
    CubReductionGeometry geometry;
    const Tensor input;
    mutable Tensor output;
    ReductionLaunchPlan plan;
    std::optional<Tensor> workspace;
    const float output_scale;
    Stream stream;
};

class StampedCubArgReduction {
   public:
    void run();
    void runOn(Stream& run_stream) const;

    uint32_t gpuNum() const { return input.getPlacement().getDeviceNum(); }
    CubArgReductionOp getOperation() const { return op; }
    CubReductionPath getPath() const { return geometry.path; }
    DataType getInputDataType() const { return input.getDataType(); }
    DataType getValueAccumulatorDataType() const { return DataType::FP32; }
    const CubReductionGeometry& getGeometry() const { return geometry; }
    size_t getWorkspaceSizeInBytes() const { return plan.workspaceBytes; }
    const std::optional<Tensor>& getValueOutputTensor() const { return value_output; }
    const std::optional<Tensor>& getIndexOutputTensor() const { return index_output; }
    const std::string& getKernelVariant() const { return plan.variant; }

   private:
    friend class CubArgReduction;
    StampedCubArgReduction(CubArgReductionOp op, CubReductionGeometry geometry, const Tensor& input, std::optional<Tensor> value_output,
                           std::optional<Tensor> index_output, ReductionLaunchPlan plan, std::optional<Tensor> workspace,
                           const Stream& stream)
        : op(op), geometry(std::move(geometry)), input(input), value_output(std::move(value_output)),
          index_output(std::move(index_output)), plan(std::move(plan)), workspace(std::move(workspace)), stream(stream) {}

    CubArgReductionOp op;
    CubReductionGeometry geometry;
    const Tensor input;
    mutable std::optional<Tensor> value_output;
    mutable std::optional<Tensor> index_output;
    ReductionLaunchPlan plan;
    std::optional<Tensor> workspace;
    Stream stream;
};

// Concrete offset-segmented reductions: run() launches only.
class StampedCubSegmentedReduction {
   public:
    void run() { runOn(stream); }
    void runOn(Stream& run_stream) const;

    uint32_t gpuNum() const { return input.getPlacement().getDeviceNum(); }
    Tensor getOutputTensor() const { return output; }
    CubReductionOp getOperation() const { return op; }
    CubReductionPath getPath() const { return CubReductionPath::OffsetSegmented; }
    DataType getInputDataType() const { return input.getDataType(); }
    DataType getOutputDataType() const { return output.getDataType(); }
    DataType getAccumulatorDataType() const { return DataType::FP32; }
    DataType getOffsetDataType() const { return segment_offsets.getDataType(); }
    uint64_t getNumItems() const { return num_items; }
    uint64_t getNumSegments() const { return num_segments; }
    size_t getWorkspaceSizeInBytes() const { return plan.workspaceBytes; }
    const std::string& getKernelVariant() const { return plan.variant; }

   private:
    friend class CubSegmentedReduction;
    StampedCubSegmentedReduction(CubReductionOp op, const Tensor& input, const Tensor& output, const Tensor& segment_offsets, uint64_t num_items,
                                 uint64_t num_segments, ReductionLaunchPlan plan, std::optional<Tensor> workspace, const Stream& stream)
        : op(op), input(input), output(output), segment_offsets(segment_offsets), num_items(num_items), num_segments(num_segments),
          plan(std::move(plan)), workspace(std::move(workspace)), stream(stream) {}

    CubReductionOp op;
    const Tensor input;
    mutable Tensor output;
    const Tensor segment_offsets;
    const uint64_t num_items, num_segments;
    ReductionLaunchPlan plan;
    std::optional<Tensor> workspace;
    Stream stream;
};

class StampedCubSegmentedArgReduction {
   public:
    void run() { runOn(stream); }
    void runOn(Stream& run_stream) const;

    uint32_t gpuNum() const { return input.getPlacement().getDeviceNum(); }
    Tensor getIndexOutputTensor() const { return index_output; }
    CubArgReductionOp getOperation() const { return op; }
    CubReductionPath getPath() const { return CubReductionPath::OffsetSegmented; }
    DataType getInputDataType() const { return input.getDataType(); }
    DataType getOffsetDataType() const { return segment_offsets.getDataType(); }
    uint64_t getNumItems() const { return num_items; }
    uint64_t getNumSegments() const { return num_segments; }
    size_t getWorkspaceSizeInBytes() const { return plan.workspaceBytes; }
    const std::string& getKernelVariant() const { return plan.variant; }

   private:
    friend class CubSegmentedArgReduction;
    StampedCubSegmentedArgReduction(CubArgReductionOp op, const Tensor& input, const Tensor& index_output, const Tensor& segment_offsets,
                                    uint64_t num_items, uint64_t num_segments, ReductionLaunchPlan plan, std::optional<Tensor> workspace,
                                    const Stream& stream)
        : op(op), input(input), index_output(index_output), segment_offsets(segment_offsets), num_items(num_items), num_segments(num_segments),
          plan(std::move(plan)), workspace(std::move(workspace)), stream(stream) {}

    CubArgReductionOp op;
    const Tensor input;
    mutable Tensor index_output;
    const Tensor segment_offsets;
    const uint64_t num_items, num_segments;
    ReductionLaunchPlan plan;
    std::optional<Tensor> workspace;
    Stream stream;
};

}  // namespace ThorImplementation
