// Broadcast of per-segment values [B, D...] onto the packed rows [N, D...] of a ragged batch (reference:
// Utilities/Expression/SegmentedBroadcastKernel.h:8-12).  Row r of segment b = [offsets[b], offsets[b + 1]) receives
// values[b], optionally divided by the segment's length (fp32 division, one rounding to the storage dtype); rows outside
// every segment are left as they are.  Offsets are UINT32 or UINT64 and are read when the kernel runs.  Values and output
// share one floating-point dtype (fp8, fp16, bf16, fp32) and one GPU; trailing dimensions may be shaped differently as
// long as the elements per value agree.  Errors are std::runtime_error, as in the reference.
#pragma once

#include "DeepLearning/Implementation/Tensor/Tensor.h"
#include "Utilities/Common/Stream.h"

namespace ThorImplementation {

void launchSegmentedBroadcast(const Tensor& per_segment_values, const Tensor& segment_offsets, Tensor& output, bool normalize_by_segment_length,
                              Stream& stream);

}  // namespace ThorImplementation
