// Internal: one description of a scan (flat, rows, or the segments of an offsets tensor), its compiled kernels and launch.
#pragma once

#include "Utilities/Expression/CompiledEquation.h"
#include "Utilities/TensorOperations/Cub/CubDevicePrimitives.h"

#include <cstdint>
#include <memory>
#include <string>

namespace ThorImplementation {

struct ScanRequest {
    DataType dtype = DataType::FP32;
    uint64_t total = 0;     // elements
    uint64_t row = 0;       // length of every segment; 0 = segments come from an offsets tensor; total = one flat scan
    uint64_t segments = 1;  // offsets hold segments + 1 entries
    bool offsets64 = false;
    int op = 0;  // 0 sum, 1 min, 2 max, 3 product
    bool writeValue = true, writeIndex = false;
    bool inclusive = true, reverse = false;
    uint64_t alignmentBytes = 256;  // largest power of two (capped at 256) dividing the input and output addresses
    // Not a scan of its own: the gradient of the min / max scan described above, in one launch (reads the operand and an FP32
    // upstream gradient, writes the FP32 gradient of the operand).  Only for rows (row != 0) that fit a block's chunk; see
    // scanRouteFits.
    bool route = false;
    int deviceNum = 0;
};

struct CubScanKernels {
    ScanRequest request;
    std::shared_ptr<CompiledKernel> mainKernel, totalsKernel, carriesKernel, clearKernel, markKernel;
    uint64_t chunks = 1;
    uint32_t threads = 256;
    bool carry = false;
    bool lookback = false;    // chunks read what precedes them from totals the blocks publish to each other (one launch over the data)
    uint64_t clearWords = 0;  // 4-byte words at the start of the temporary storage that every run zeroes first
    size_t headsBytes = 0, statesBytes = 0, tempBytes = 1;
    std::string variant;
};

constexpr uint64_t kScanRouteMaxChunkElems = 8192;
// Whether buildScanKernels accepts `request` with route set (otherwise the gradient takes an arg scan and a scatter).
bool scanRouteFits(const ScanRequest& request);
// Launches the routing kernel of a request built with route set.
void launchScanRoute(const CubScanKernels& kernels, const void* input, const void* gradient, void* routed, Stream& stream);

// loadedOnly: take every kernel from the process-wide cache and throw std::runtime_error when one is missing, so that nothing is
// compiled or loaded (for callers that must not allocate).  A request whose temporary storage exceeds tempLimitBytes is rejected
// with std::invalid_argument before any kernel is looked up.
std::shared_ptr<const CubScanKernels> buildScanKernels(const ScanRequest& request, bool loadedOnly = false, size_t tempLimitBytes = ~size_t(0));
// `temp` holds at least kernels.tempBytes bytes; outValue / outIndex may be null when the request does not write them.
void launchScan(const CubScanKernels& kernels, const void* input, const void* offsets, void* temp, size_t tempBytes, void* outValue, void* outIndex,
                Stream& stream);

// How many waits of the last launch on `temp` gave up.  Scans that publish totals between blocks bound every wait so that each
// wavefront has an exit; a wait that gives up works the totals it lacks out again from the input, so the results are complete
// and the same bits either way: this is a diagnostic, not an error.  Waits for the stream, then reads one word of `temp`: for
// callers that synchronise anyway.  Always 0 for kernels that do not wait on each other.
uint32_t scanWaitsRecovered(const CubScanKernels& kernels, const void* temp, Stream& stream);
// The sum of what scanWaitsRecovered returned in this process (every thor_scan call adds its count).
uint64_t scanWaitsRecoveredTotal();

// One scan (flat: offsets null and segmentSize 0; rows of segmentSize; or the numSegments segments of *offsets) that compiles, loads
// and allocates nothing: its kernels must be in the process-wide cache already (std::runtime_error otherwise) and its temporary
// storage is the caller's block `temp` of tempCapacityBytes (std::invalid_argument when the request needs more).  Same validation,
// kernels and results as the plan / run entry points.
std::shared_ptr<const CubScanKernels> scanWithLoadedKernels(const Tensor& input, Tensor& output, const Tensor* offsets, uint64_t numItems,
                                                            uint64_t numSegments, uint64_t segmentSize, int op, bool arg, bool inclusive, bool reverse,
                                                            void* temp, size_t tempCapacityBytes, Stream& stream);

}  // namespace ThorImplementation
