// Device-wide prefix scans with the reference's plan / temporary-storage / run protocol
// (reference: Utilities/TensorOperations/Cub/CubDevicePrimitives.h:16-19,141-158,197-243,781-880,951-1012 and CubScan.cu,
// CubSegmentedScan.cu).  Only the scan family of that header is provided: flat scans, scans over segments of one size
// (rows) and scans over the segments of an offsets tensor, each as value scan (sum / min / max / product) and arg scan
// (arg-min / arg-max: UINT32 flattened index of the winning prefix element), inclusive or exclusive, forward or reverse.
//
// Values are UINT32 (exact, wrapping), FP32, FP16 or BF16.  16-bit floats accumulate in fp32 and round once at the
// store (the reference rounds at every combine, in an order its library chooses); min / max are selections and exact.
// Exclusive scans start every segment with the identity (0, 1, the largest / smallest value or +-inf); arg scans with
// 0xFFFFFFFF.  Min / max keep the earlier element among equals and take the first element as it is.  Rows past
// offsets[num_segments] are scanned as one more segment.  Sort, select, top-k, run-length encode and find are not built.
#pragma once

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"

#include <cstdint>
#include <memory>
#include <string>

namespace ThorImplementation {

enum class CubScanOp : uint8_t { Sum = 0, Min = 1, Max = 2, Product = 3 };
enum class CubArgScanOp : uint8_t { ArgMin = 0, ArgMax = 1 };
enum class CubScanMode : uint8_t { Exclusive = 0, Inclusive = 1 };
enum class CubScanDirection : uint8_t { Forward = 0, Reverse = 1 };

struct CubScanKernels;  // compiled kernels and launch shapes of one plan (internal)

struct CubDeviceScanPlan {
    TensorPlacement placement;
    DataType dtype = DataType::UINT32;
    uint64_t num_items = 0;
    CubScanOp op = CubScanOp::Sum;
    CubScanMode mode = CubScanMode::Exclusive;
    CubScanDirection direction = CubScanDirection::Forward;
    size_t temp_storage_bytes = 0;
    std::shared_ptr<const CubScanKernels> kernels;
};
struct CubDeviceArgScanPlan {
    TensorPlacement placement;
    DataType dtype = DataType::UINT32;
    uint64_t num_items = 0;
    CubArgScanOp op = CubArgScanOp::ArgMin;
    CubScanMode mode = CubScanMode::Inclusive;
    CubScanDirection direction = CubScanDirection::Forward;
    size_t temp_storage_bytes = 0;
    std::shared_ptr<const CubScanKernels> kernels;
};
struct CubDeviceSegmentedUniformScanPlan {
    TensorPlacement placement;
    DataType dtype = DataType::UINT32;
    uint64_t num_items = 0;
    uint64_t num_segments = 0;
    uint64_t segment_size = 0;
    CubScanOp op = CubScanOp::Sum;
    CubScanMode mode = CubScanMode::Exclusive;
    CubScanDirection direction = CubScanDirection::Forward;
    size_t temp_storage_bytes = 0;
    std::shared_ptr<const CubScanKernels> kernels;
};
struct CubDeviceSegmentedUniformArgScanPlan {
    TensorPlacement placement;
    DataType dtype = DataType::UINT32;
    uint64_t num_items = 0;
    uint64_t num_segments = 0;
    uint64_t segment_size = 0;
    CubArgScanOp op = CubArgScanOp::ArgMin;
    CubScanMode mode = CubScanMode::Inclusive;
    CubScanDirection direction = CubScanDirection::Forward;
    size_t temp_storage_bytes = 0;
    std::shared_ptr<const CubScanKernels> kernels;
};
struct CubDeviceSegmentedScanPlan {
    TensorPlacement placement;
    DataType dtype = DataType::UINT32;
    DataType offset_dtype = DataType::UINT32;
    uint64_t num_items = 0;
    uint64_t num_segments = 0;
    CubScanOp op = CubScanOp::Sum;
    CubScanMode mode = CubScanMode::Exclusive;
    CubScanDirection direction = CubScanDirection::Forward;
    size_t temp_storage_bytes = 0;
    std::shared_ptr<const CubScanKernels> kernels;
};
struct CubDeviceSegmentedArgScanPlan {
    TensorPlacement placement;
    DataType dtype = DataType::UINT32;
    DataType offset_dtype = DataType::UINT32;
    uint64_t num_items = 0;
    uint64_t num_segments = 0;
    CubArgScanOp op = CubArgScanOp::ArgMin;
    CubScanMode mode = CubScanMode::Inclusive;
    CubScanDirection direction = CubScanDirection::Forward;
    size_t temp_storage_bytes = 0;
    std::shared_ptr<const CubScanKernels> kernels;
};

[[nodiscard]] bool isCubScanDTypeSupported(DataType dtype);           // UINT32, FP16, BF16, FP32
[[nodiscard]] bool isCubSegmentOffsetDTypeSupported(DataType dtype);  // UINT32, UINT64
// UINT8 tensor of at least `bytes` bytes (at least one) on `placement`
[[nodiscard]] Tensor allocateCubTemporaryStorage(const TensorPlacement& placement, size_t bytes);

// ---- one scan over num_items elements ------------------------------------------------------------------------------------
[[nodiscard]] CubDeviceScanPlan prepareCubDeviceScan(const Tensor& input, const Tensor& output, uint64_t num_items, CubScanOp op, CubScanMode mode,
                                                     CubScanDirection direction = CubScanDirection::Forward);
[[nodiscard]] size_t cubDeviceScanTempBytes(const Tensor& input, const Tensor& output, uint64_t num_items, CubScanOp op, CubScanMode mode,
                                            CubScanDirection direction = CubScanDirection::Forward);
void cubDeviceScan(const CubDeviceScanPlan& plan, const Tensor& temp_storage, const Tensor& input, Tensor& output, Stream& stream);

[[nodiscard]] CubDeviceArgScanPlan prepareCubDeviceArgScan(const Tensor& input, const Tensor& output, uint64_t num_items, CubArgScanOp op,
                                                           CubScanMode mode, CubScanDirection direction = CubScanDirection::Forward);
[[nodiscard]] size_t cubDeviceArgScanTempBytes(const Tensor& input, const Tensor& output, uint64_t num_items, CubArgScanOp op, CubScanMode mode,
                                               CubScanDirection direction = CubScanDirection::Forward);
void cubDeviceArgScan(const CubDeviceArgScanPlan& plan, const Tensor& temp_storage, const Tensor& input, Tensor& output, Stream& stream);

// ---- num_segments scans over consecutive runs of segment_size elements -------------------------------------------------
[[nodiscard]] CubDeviceSegmentedUniformScanPlan prepareCubDeviceSegmentedUniformScan(const Tensor& input, const Tensor& output, uint64_t num_items,
                                                                                     uint64_t num_segments, uint64_t segment_size, CubScanOp op,
                                                                                     CubScanMode mode,
                                                                                     CubScanDirection direction = CubScanDirection::Forward);
[[nodiscard]] size_t cubDeviceSegmentedUniformScanTempBytes(const Tensor& input, const Tensor& output, uint64_t num_items, uint64_t num_segments,
                                                            uint64_t segment_size, CubScanOp op, CubScanMode mode,
                                                            CubScanDirection direction = CubScanDirection::Forward);
void cubDeviceSegmentedUniformScan(const CubDeviceSegmentedUniformScanPlan& plan, const Tensor& temp_storage, const Tensor& input, Tensor& output,
                                   Stream& stream);

[[nodiscard]] CubDeviceSegmentedUniformArgScanPlan prepareCubDeviceSegmentedUniformArgScan(const Tensor& input, const Tensor& output,
                                                                                           uint64_t num_items, uint64_t num_segments,
                                                                                           uint64_t segment_size, CubArgScanOp op, CubScanMode mode,
                                                                                           CubScanDirection direction = CubScanDirection::Forward);
[[nodiscard]] size_t cubDeviceSegmentedUniformArgScanTempBytes(const Tensor& input, const Tensor& output, uint64_t num_items, uint64_t num_segments,
                                                               uint64_t segment_size, CubArgScanOp op, CubScanMode mode,
                                                               CubScanDirection direction = CubScanDirection::Forward);
void cubDeviceSegmentedUniformArgScan(const CubDeviceSegmentedUniformArgScanPlan& plan, const Tensor& temp_storage, const Tensor& input,
                                      Tensor& output, Stream& stream);

// ---- scans over the segments [offsets[s], offsets[s + 1]) of an offsets tensor read on the device at every run -----------
[[nodiscard]] CubDeviceSegmentedScanPlan prepareCubDeviceSegmentedScan(const Tensor& input, const Tensor& output, const Tensor& segment_offsets,
                                                                       uint64_t num_items, uint64_t num_segments, CubScanOp op, CubScanMode mode,
                                                                       CubScanDirection direction = CubScanDirection::Forward);
[[nodiscard]] size_t cubDeviceSegmentedScanTempBytes(const Tensor& input, const Tensor& output, const Tensor& segment_offsets, uint64_t num_items,
                                                     uint64_t num_segments, CubScanOp op, CubScanMode mode,
                                                     CubScanDirection direction = CubScanDirection::Forward);
void cubDeviceSegmentedScan(const CubDeviceSegmentedScanPlan& plan, const Tensor& temp_storage, const Tensor& input, Tensor& output,
                            const Tensor& segment_offsets, Stream& stream);

[[nodiscard]] CubDeviceSegmentedArgScanPlan prepareCubDeviceSegmentedArgScan(const Tensor& input, const Tensor& output, const Tensor& segment_offsets,
                                                                             uint64_t num_items, uint64_t num_segments, CubArgScanOp op,
                                                                             CubScanMode mode,
                                                                             CubScanDirection direction = CubScanDirection::Forward);
[[nodiscard]] size_t cubDeviceSegmentedArgScanTempBytes(const Tensor& input, const Tensor& output, const Tensor& segment_offsets, uint64_t num_items,
                                                        uint64_t num_segments, CubArgScanOp op, CubScanMode mode,
                                                        CubScanDirection direction = CubScanDirection::Forward);
void cubDeviceSegmentedArgScan(const CubDeviceSegmentedArgScanPlan& plan, const Tensor& temp_storage, const Tensor& input, Tensor& output,
                               const Tensor& segment_offsets, Stream& stream);

// How a plan runs: chunk size, vector width, grid, number of launches (diagnostics and tests).
[[nodiscard]] std::string cubScanKernelVariant(const std::shared_ptr<const CubScanKernels>& kernels);

}  // namespace ThorImplementation
