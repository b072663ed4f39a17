// Device-wide primitives with the reference's plan / temporary-storage / run protocol
// (reference: Utilities/TensorOperations/Cub/CubDevicePrimitives.h:15-19,47-93,141-158,197-243,357-516,781-880,951-1012 and
// CubScan.cu, CubSegmentedScan.cu, CubSelect.cu, CubTopK.cu).  Provided: the scan family - flat scans, scans over segments of one
// size (rows) and scans over the segments of an offsets tensor, each as value scan (sum / min / max / product) and arg scan
// (arg-min / arg-max: UINT32 flattened index of the winning prefix element), inclusive or exclusive, forward or reverse -
// select-flagged (order-preserving compaction) and top-k (keys or key / index pairs; device-wide and per fixed-size row).
//
// Values are UINT32 (exact, wrapping), FP32, FP16 or BF16.  16-bit floats accumulate in fp32 and round once at the
// store (the reference rounds at every combine, in an order its library chooses); min / max are selections and exact.
// Exclusive scans start every segment with the identity (0, 1, the largest / smallest value or +-inf); arg scans with
// 0xFFFFFFFF.  Min / max keep the earlier element among equals and take the first element as it is.  Rows past
// offsets[num_segments] are scanned as one more segment.  Sort, run-length encode and find are not built.
#pragma once

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"

#include <cstdint>
#include <initializer_list>
#include <memory>
#include <string>

namespace ThorImplementation {

enum class CubScanOp : uint8_t { Sum = 0, Min = 1, Max = 2, Product = 3 };
enum class CubArgScanOp : uint8_t { ArgMin = 0, ArgMax = 1 };
enum class CubScanMode : uint8_t { Exclusive = 0, Inclusive = 1 };
enum class CubScanDirection : uint8_t { Forward = 0, Reverse = 1 };

enum class CubTopKOrder : uint8_t { Smallest = 0, Largest = 1 };

struct CubTemporaryStoragePlan {
    TensorPlacement placement;
    size_t bytes = 0;
};

struct CubScanKernels;       // compiled kernels and launch shapes of one plan (internal)
struct CubSelectionKernels;  // the same for select-flagged and top-k plans

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

// ---- select-flagged and top-k plans (reference: CubDevicePrimitives.h:47-93 there) ------------------------------------------------
struct CubDeviceTopKKeysPlan {
    TensorPlacement placement;
    DataType key_dtype = DataType::UINT8;
    uint64_t num_items = 0;
    uint64_t k = 0;
    CubTopKOrder order = CubTopKOrder::Largest;
    size_t temp_storage_bytes = 0;
    uint64_t key_alignment_bytes = 1;  // what the kernels assume of keys_in (not in the reference's struct)
    std::shared_ptr<const CubSelectionKernels> kernels;
};
struct CubDeviceTopKPairsPlan {
    TensorPlacement placement;
    DataType key_dtype = DataType::UINT8;
    DataType value_dtype = DataType::UINT32;
    uint64_t num_items = 0;
    uint64_t k = 0;
    CubTopKOrder order = CubTopKOrder::Largest;
    size_t temp_storage_bytes = 0;
    uint64_t key_alignment_bytes = 1;
    std::shared_ptr<const CubSelectionKernels> kernels;
};
struct CubDeviceSegmentedTopKKeysPlan {
    TensorPlacement placement;
    DataType key_dtype = DataType::UINT8;
    uint64_t num_segments = 0;
    uint64_t segment_size = 0;
    uint64_t k = 0;
    CubTopKOrder order = CubTopKOrder::Largest;
    size_t temp_storage_bytes = 0;
    std::shared_ptr<const CubSelectionKernels> kernels;
};
struct CubDeviceSegmentedTopKPairsPlan {
    TensorPlacement placement;
    DataType key_dtype = DataType::UINT8;
    DataType value_dtype = DataType::UINT32;
    uint64_t num_segments = 0;
    uint64_t segment_size = 0;
    uint64_t k = 0;
    CubTopKOrder order = CubTopKOrder::Largest;
    size_t temp_storage_bytes = 0;
    std::shared_ptr<const CubSelectionKernels> kernels;
};
struct CubDeviceSelectFlaggedPlan {
    TensorPlacement placement;
    DataType input_dtype = DataType::UINT8;
    DataType flag_dtype = DataType::BOOLEAN;
    uint64_t num_items = 0;
    size_t temp_storage_bytes = 0;
    uint64_t vector_elements = 1;  // 4: the kernels read input, flags and output in groups of four elements (not in the reference's struct)
    std::shared_ptr<const CubSelectionKernels> kernels;
};

[[nodiscard]] bool isCubScanDTypeSupported(DataType dtype);           // UINT32, FP16, BF16, FP32
[[nodiscard]] bool isCubSegmentOffsetDTypeSupported(DataType dtype);  // UINT32, UINT64
// UINT8 tensor of at least `bytes` bytes (at least one) on `placement`
// A temporary-storage requirement, so that several plans can share the largest block (reference: CubDevicePrimitives.h:21-24,284-287).
[[nodiscard]] CubTemporaryStoragePlan cubTemporaryStoragePlan(const TensorPlacement& placement, size_t bytes);
[[nodiscard]] CubTemporaryStoragePlan cubMaxTemporaryStoragePlan(std::initializer_list<CubTemporaryStoragePlan> plans);
[[nodiscard]] Tensor allocateCubTemporaryStorage(const TensorPlacement& placement, size_t bytes);
[[nodiscard]] Tensor allocateCubTemporaryStorage(const CubTemporaryStoragePlan& plan);

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
// Diagnostic: how many bounded waits between the blocks of the last run on `temp_storage` gave up.  Such a wait computes the
// totals it lacks from the input, in the order their owners would have, so a run's results are complete and the same bits either
// way; the count is 0 in normal operation (a block only waits for blocks that started before it).  Synchronises `stream`.
[[nodiscard]] uint32_t cubScanWaitsRecovered(const std::shared_ptr<const CubScanKernels>& kernels, const Tensor& temp_storage, Stream& stream);

// ---- top-k: the k largest (or smallest) keys, in no particular order; which of several equal keys at the boundary are taken is ----
// ---- not fixed (the reference asks its library for unsorted, not run-to-run deterministic output: CubTopK.cu:34-36 there) -----------
// Keys: UINT8 / INT8 / UINT16 / INT16 / UINT32 / INT32 / FP16 / BF16 / FP32 (floats order by their bits: -0 below +0, NaNs beyond
// the infinities); values of pairs: UINT32.  k is capped at num_items; outputs need min(num_items, k) elements.
[[nodiscard]] bool isCubTopKKeyDTypeSupported(DataType dtype);
[[nodiscard]] bool isCubTopKValueDTypeSupported(DataType dtype);
[[nodiscard]] bool isCubSelectValueDTypeSupported(DataType dtype);  // the top-k key dtypes
[[nodiscard]] bool isCubSelectFlagDTypeSupported(DataType dtype);   // BOOLEAN, UINT8

[[nodiscard]] CubDeviceTopKKeysPlan prepareCubDeviceTopKKeys(const Tensor& keys_in, const Tensor& keys_out, uint64_t num_items, uint64_t k,
                                                             CubTopKOrder order = CubTopKOrder::Largest);
[[nodiscard]] size_t cubDeviceTopKKeysTempBytes(const Tensor& keys_in, const Tensor& keys_out, uint64_t num_items, uint64_t k,
                                                CubTopKOrder order = CubTopKOrder::Largest);
void cubDeviceTopKKeys(const CubDeviceTopKKeysPlan& plan, const Tensor& temp_storage, const Tensor& keys_in, Tensor& keys_out, Stream& stream);
void cubDeviceTopKKeys(const Tensor& temp_storage, size_t temp_storage_bytes, const Tensor& keys_in, Tensor& keys_out, uint64_t num_items, uint64_t k,
                       Stream& stream, CubTopKOrder order = CubTopKOrder::Largest);

[[nodiscard]] CubDeviceTopKPairsPlan prepareCubDeviceTopKPairs(const Tensor& keys_in, const Tensor& keys_out, const Tensor& values_in,
                                                               const Tensor& values_out, uint64_t num_items, uint64_t k,
                                                               CubTopKOrder order = CubTopKOrder::Largest);
[[nodiscard]] size_t cubDeviceTopKPairsTempBytes(const Tensor& keys_in, const Tensor& keys_out, const Tensor& values_in, const Tensor& values_out,
                                                 uint64_t num_items, uint64_t k, CubTopKOrder order = CubTopKOrder::Largest);
void cubDeviceTopKPairs(const CubDeviceTopKPairsPlan& plan, const Tensor& temp_storage, const Tensor& keys_in, Tensor& keys_out,
                        const Tensor& values_in, Tensor& values_out, Stream& stream);
void cubDeviceTopKPairs(const Tensor& temp_storage, size_t temp_storage_bytes, const Tensor& keys_in, Tensor& keys_out, const Tensor& values_in,
                        Tensor& values_out, uint64_t num_items, uint64_t k, Stream& stream, CubTopKOrder order = CubTopKOrder::Largest);

// Rows of segment_size keys (at most 8192), k < segment_size keys out of each, written row after row.
[[nodiscard]] CubDeviceSegmentedTopKKeysPlan prepareCubDeviceSegmentedTopKKeys(const Tensor& keys_in, const Tensor& keys_out, uint64_t num_segments,
                                                                               uint64_t segment_size, uint64_t k,
                                                                               CubTopKOrder order = CubTopKOrder::Largest);
[[nodiscard]] size_t cubDeviceSegmentedTopKKeysTempBytes(const Tensor& keys_in, const Tensor& keys_out, uint64_t num_segments, uint64_t segment_size,
                                                         uint64_t k, CubTopKOrder order = CubTopKOrder::Largest);
void cubDeviceSegmentedTopKKeys(const CubDeviceSegmentedTopKKeysPlan& plan, const Tensor& temp_storage, const Tensor& keys_in, Tensor& keys_out,
                                Stream& stream);
void cubDeviceSegmentedTopKKeys(const Tensor& temp_storage, size_t temp_storage_bytes, const Tensor& keys_in, Tensor& keys_out, uint64_t num_segments,
                                uint64_t segment_size, uint64_t k, Stream& stream, CubTopKOrder order = CubTopKOrder::Largest);

[[nodiscard]] CubDeviceSegmentedTopKPairsPlan prepareCubDeviceSegmentedTopKPairs(const Tensor& keys_in, const Tensor& keys_out,
                                                                                 const Tensor& values_in, const Tensor& values_out,
                                                                                 uint64_t num_segments, uint64_t segment_size, uint64_t k,
                                                                                 CubTopKOrder order = CubTopKOrder::Largest);
[[nodiscard]] size_t cubDeviceSegmentedTopKPairsTempBytes(const Tensor& keys_in, const Tensor& keys_out, const Tensor& values_in,
                                                          const Tensor& values_out, uint64_t num_segments, uint64_t segment_size, uint64_t k,
                                                          CubTopKOrder order = CubTopKOrder::Largest);
void cubDeviceSegmentedTopKPairs(const CubDeviceSegmentedTopKPairsPlan& plan, const Tensor& temp_storage, const Tensor& keys_in, Tensor& keys_out,
                                 const Tensor& values_in, Tensor& values_out, Stream& stream);
void cubDeviceSegmentedTopKPairs(const Tensor& temp_storage, size_t temp_storage_bytes, const Tensor& keys_in, Tensor& keys_out,
                                 const Tensor& values_in, Tensor& values_out, uint64_t num_segments, uint64_t segment_size, uint64_t k, Stream& stream,
                                 CubTopKOrder order = CubTopKOrder::Largest);

// ---- select-flagged: output = the elements of input whose flag is nonzero, in input order; *num_selected_out (UINT32) = their count ----
[[nodiscard]] CubDeviceSelectFlaggedPlan prepareCubDeviceSelectFlagged(const Tensor& input, const Tensor& flags, const Tensor& output,
                                                                       const Tensor& num_selected_out, uint64_t num_items);
[[nodiscard]] size_t cubDeviceSelectFlaggedTempBytes(const Tensor& input, const Tensor& flags, const Tensor& output, const Tensor& num_selected_out,
                                                     uint64_t num_items);
void cubDeviceSelectFlagged(const CubDeviceSelectFlaggedPlan& plan, const Tensor& temp_storage, const Tensor& input, const Tensor& flags,
                            Tensor& output, Tensor& num_selected_out, Stream& stream);
void cubDeviceSelectFlagged(const Tensor& temp_storage, size_t temp_storage_bytes, const Tensor& input, const Tensor& flags, Tensor& output,
                            Tensor& num_selected_out, uint64_t num_items, Stream& stream);

[[nodiscard]] std::string cubSelectionKernelVariant(const std::shared_ptr<const CubSelectionKernels>& kernels);

}  // namespace ThorImplementation
