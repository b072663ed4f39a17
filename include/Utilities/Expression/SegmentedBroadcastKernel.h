// Broadcast of per-segment values [B, D...] onto the packed rows [N, D...] of a ragged batch (reference:
// Utilities/Expression/SegmentedBroadcastKernel.h:8-12).  Row r of segment b = [offsets[b], offsets[b + 1]) receives
// values[b], optionally divided by the segment's length (fp32 division, one rounding to the storage dtype); rows outside
// every segment are left as they are.  Offsets are UINT32 or UINT64 and are read when the kernel runs.  Values and output
// share one floating-point dtype (fp8, fp16, bf16, fp32) and one GPU; trailing dimensions may be shaped differently as
// long as the elements per value agree.  Errors are std::runtime_error, as in the reference.
#pragma once

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"

#include <memory>
#include <string>

namespace ThorImplementation {

struct CompiledKernel;

// The validated, compiled form: stampSegmentedBroadcast() does everything launchSegmentedBroadcast() does except the
// launch; runOn() only launches (what a stamped execution plan keeps per broadcast stage).
class StampedSegmentedBroadcast {
   public:
    StampedSegmentedBroadcast(std::shared_ptr<CompiledKernel> kernel, Tensor values, Tensor offsets, Tensor output, uint32_t gridX, std::string variant)
        : kernel(std::move(kernel)), values(std::move(values)), offsets(std::move(offsets)), output(std::move(output)), gridX(gridX),
          variant(std::move(variant)) {}
    void runOn(Stream& stream) const;
    Tensor getOutputTensor() const { return output; }
    const std::string& getKernelVariant() const { return variant; }

   private:
    std::shared_ptr<CompiledKernel> kernel;
    Tensor values, offsets, output;
    uint32_t gridX;
    std::string variant;
};

std::shared_ptr<StampedSegmentedBroadcast> stampSegmentedBroadcast(const Tensor& per_segment_values, const Tensor& segment_offsets, const Tensor& output,
                                                                   bool normalize_by_segment_length, const Stream& stream);

// ids[r] = the segment row r belongs to, for every row inside a segment (UINT32 [N]; other rows keep their contents).  The
// index fused kernels read per-segment values through.
std::shared_ptr<StampedSegmentedBroadcast> stampSegmentIds(const Tensor& segment_offsets, const Tensor& ids, const Stream& stream);

void launchSegmentedBroadcast(const Tensor& per_segment_values, const Tensor& segment_offsets, Tensor& output, bool normalize_by_segment_length,
                              Stream& stream);

}  // namespace ThorImplementation
