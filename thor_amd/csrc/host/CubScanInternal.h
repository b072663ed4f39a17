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
    int deviceNum = 0;
};

struct CubScanKernels {
    ScanRequest request;
    std::shared_ptr<CompiledKernel> mainKernel, totalsKernel, carriesKernel, clearKernel, markKernel;
    uint64_t chunks = 1;
    uint32_t threads = 256;
    bool carry = false;
    size_t headsBytes = 0, statesBytes = 0, tempBytes = 1;
    std::string variant;
};

std::shared_ptr<const CubScanKernels> buildScanKernels(const ScanRequest& request);
// `temp` holds at least kernels.tempBytes bytes; outValue / outIndex may be null when the request does not write them.
void launchScan(const CubScanKernels& kernels, const void* input, const void* offsets, void* temp, size_t tempBytes, void* outValue, void* outIndex,
                Stream& stream);

}  // namespace ThorImplementation
