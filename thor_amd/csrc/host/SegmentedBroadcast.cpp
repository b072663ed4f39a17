// Segmented broadcast: validation, kernel specialisation and launch (kernel: thor_device_reduce.h broadcastSegments).
#include "Utilities/Expression/SegmentedBroadcastKernel.h"

#include "ReductionPlanner.h"
#include "Utilities/Cache/LruCache.h"
#include "Utilities/Common/ScopedGpu.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "thorhip_numeric_embed.h"

#include <algorithm>
#include <cstdlib>
#include <limits>
#include <sstream>
#include <stdexcept>

namespace ThorImplementation {

namespace {

uint64_t pow2Floor(uint64_t v) {
    uint64_t p = 1;
    while (p * 2 <= v) p *= 2;
    return p;
}

uint64_t pow2Ceil(uint64_t v) {
    uint64_t p = 1;
    while (p < v) p *= 2;
    return p;
}

const char* rawWordName(uint32_t bytes) { return bytes == 1 ? "thor::u8" : bytes == 2 ? "thor::u16" : "thor::u32"; }

}  // namespace

namespace {
std::shared_ptr<StampedSegmentedBroadcast> stampImpl(const Tensor& per_segment_values, const Tensor& segment_offsets, const Tensor& output,
                                                     bool normalize_by_segment_length, bool ids, const Stream& stream);
}

std::shared_ptr<StampedSegmentedBroadcast> stampSegmentedBroadcast(const Tensor& per_segment_values, const Tensor& segment_offsets, const Tensor& output,
                                                                   bool normalize_by_segment_length, const Stream& stream) {
    return stampImpl(per_segment_values, segment_offsets, output, normalize_by_segment_length, false, stream);
}

std::shared_ptr<StampedSegmentedBroadcast> stampSegmentIds(const Tensor& segment_offsets, const Tensor& ids, const Stream& stream) {
    if (!ids.isInitialized() || ids.getDataType() != DataType::UINT32 || ids.getDimensions().size() != 1) {
        throw std::runtime_error("Segment ids must be a UINT32 tensor of shape [rows].");
    }
    if (!segment_offsets.isInitialized() || segment_offsets.getDimensions().size() != 1 || segment_offsets.getDimensions()[0] < 2) {
        throw std::runtime_error("Segment ids require offsets [B+1] with at least one segment.");
    }
    // the values operand is not read in this mode; a [B] view of the ids tensor's dtype stands in for the shape checks
    Tensor standIn(ids.getPlacement(), TensorDescriptor(DataType::UINT32, {segment_offsets.getDimensions()[0] - 1}));
    return stampImpl(standIn, segment_offsets, ids, false, true, stream);
}

namespace {
std::shared_ptr<StampedSegmentedBroadcast> stampImpl(const Tensor& per_segment_values, const Tensor& segment_offsets, const Tensor& output,
                                                     bool normalize_by_segment_length, bool ids, const Stream& stream) {
    if (!per_segment_values.isInitialized() || !segment_offsets.isInitialized() || !output.isInitialized()) {
        throw std::runtime_error("Segmented broadcast requires initialized tensors.");
    }
    if (per_segment_values.getPlacement() != segment_offsets.getPlacement() || per_segment_values.getPlacement() != output.getPlacement()) {
        throw std::runtime_error("Segmented broadcast tensors must share one placement.");
    }
    if (per_segment_values.getPlacement().getMemDevice() != TensorPlacement::MemDevices::GPU || !stream.isInitialized() ||
        per_segment_values.getPlacement().getDeviceNum() != stream.getGpuNum()) {
        throw std::runtime_error("Segmented broadcast requires tensors on the execution GPU.");
    }
    if (per_segment_values.getDimensions().empty() || segment_offsets.getDimensions().size() != 1 || output.getDimensions().empty()) {
        throw std::runtime_error("Segmented broadcast requires per-segment values [B,D...], offsets [B+1], and output [N,D...].");
    }
    const uint64_t segments = per_segment_values.getDimensions()[0];
    if (segments == 0 || segments > static_cast<uint64_t>(std::numeric_limits<int32_t>::max())) {
        throw std::runtime_error("Segmented broadcast batch size is zero or exceeds the supported number of segments.");
    }
    if (segment_offsets.getDimensions()[0] != segments + 1) throw std::runtime_error("Segmented broadcast offsets must have shape [batch_size + 1].");
    if (per_segment_values.getDataType() != output.getDataType()) throw std::runtime_error("Segmented broadcast input and output dtypes must match.");
    if (!per_segment_values.isDenseContiguous() || !segment_offsets.isDenseContiguous() || !output.isDenseContiguous()) {
        throw std::runtime_error("Segmented broadcast requires dense tensors.");
    }
    const DataType offsetType = segment_offsets.getDataType();
    if (offsetType != DataType::UINT32 && offsetType != DataType::UINT64) throw std::runtime_error("Segmented broadcast offsets must use UINT32 or UINT64.");
    const DataType dtype = per_segment_values.getDataType();
    if (!ids && dtype != DataType::FP8_E4M3 && dtype != DataType::FP8_E5M2 && dtype != DataType::FP16 && dtype != DataType::BF16 && dtype != DataType::FP32) {
        throw std::runtime_error("Segmented broadcast requires a floating-point expression dtype.");
    }
    // Trailing dimensions may be reshaped between the two tensors ([B, 4] against [N, 2, 2]); the elements per value are
    // what has to agree.
    const uint64_t rows = output.getDimensions()[0];
    const uint64_t elementsPerValue = per_segment_values.getTotalNumElements() / segments;
    if (elementsPerValue == 0 || rows == 0 || output.getTotalNumElements() % rows != 0 || output.getTotalNumElements() / rows != elementsPerValue) {
        throw std::runtime_error("Segmented broadcast trailing dimensions produce an invalid elements-per-value extent.");
    }

    const uint32_t elementBytes = dataTypeSizeInBytes(dtype);
    const uint64_t alignment = std::min(pointerAlignment(per_segment_values.getMemPtr()), pointerAlignment(output.getMemPtr()));
    int vec = static_cast<int>(16 / elementBytes);
    while (vec > 1 && alignment % (static_cast<uint64_t>(vec) * elementBytes) != 0) vec /= 2;
    // about 32 KiB of output per block, fewer rows while that leaves under eight blocks per CU; always a multiple of 16 rows.
    // (Measured on [65 536, 64] fp32 -> [2^22, 64], 1 GiB written: 16 / 32 / 64 / 128 / 256 / 512 KiB per block take 214 / 179 / 184 / 199 /
    // 206 / 249 us: a block's search for its first segment and its window of offsets are round trips during which it stores nothing.)
    uint64_t chunkRows = std::max<uint64_t>(pow2Floor(std::max<uint64_t>(32768 / (elementsPerValue * elementBytes), 1)), 16);
    while (chunkRows > 16 && (rows + chunkRows - 1) / chunkRows < 2048) chunkRows /= 2;
    if (const char* env = std::getenv("THOR_BROADCAST_CHUNK_ROWS")) chunkRows = std::max<uint64_t>(pow2Floor(std::max<long>(std::atol(env), 16)), 16);  // tuning switch
    const uint64_t chunks = (rows + chunkRows - 1) / chunkRows;
    const uint64_t averageRows = std::max<uint64_t>(rows / segments, 1);
    const uint64_t window = std::min<uint64_t>(std::max<uint64_t>(pow2Ceil(2 * chunkRows / averageRows + 2), 16), 1024);

    // What decides the kernel's text: calls that stamp on every run (the one-call C entry point) look the built kernel up by
    // these few numbers instead of writing out and hashing a hundred kilobytes of source.
    std::ostringstream key;
    key << stream.getGpuNum() << ' ' << static_cast<int>(dtype) << ' ' << static_cast<int>(offsetType) << ' ' << elementsPerValue << ' ' << rows << ' ' << segments
        << ' ' << chunkRows << ' ' << vec << ' ' << window << ' ' << normalize_by_segment_length << ' ' << ids;
    static LruCacheThreadSafe<std::string, std::shared_ptr<CompiledKernel>> builtKernels(1024);
    std::shared_ptr<CompiledKernel> kernel;
    if (auto known = builtKernels.get(key.str())) kernel = *known;
    std::ostringstream s;
    if (!kernel) {
        s << thor_embed::kDevicePrelude << thor_embed::kReduceKernels;
        const std::string typeName = normalize_by_segment_length ? deviceTypeName(dtype) : rawWordName(elementBytes);
        s << "namespace gen {\nstruct Cfg {\n    typedef " << typeName << " T;\n    typedef " << (offsetType == DataType::UINT64 ? "thor::u64" : "thor::u32")
          << " OffsetT;\n    static constexpr thor::u64 kE = " << elementsPerValue << "ull;\n    static constexpr thor::u64 kRows = " << rows
          << "ull;\n    static constexpr thor::u64 kSegments = " << segments << "ull;\n    static constexpr thor::u64 kChunkRows = " << chunkRows
          << "ull;\n    static constexpr int kVec = " << vec << ";\n    static constexpr int kThreads = 256;\n    static constexpr int kWindow = " << window
          << ";\n    static constexpr bool kNormalize = " << (normalize_by_segment_length ? "true" : "false")
          << ";\n    static constexpr bool kViaHalf = " << (dtype == DataType::FP8_E5M2 ? "true" : "false") << ";\n    static constexpr bool kIds = "
          << (ids ? "true" : "false") << ";\n};\n}  // namespace gen\n";
        // eight wavefronts per SIMD: the fp32 form takes 65 vector registers unasked, one more than eight resident wavefronts allow
        // (2^26 rows in 65 536 segments, four alternating runs on one device: 181-186 -> 170-172 us)
        s << "extern \"C\" __global__ __launch_bounds__(256, 8) void thor_segmented_broadcast(const gen::Cfg::T* values, const void* offsets, gen::Cfg::T* out) "
             "{\n    thor::broadcastSegments<gen::Cfg>(values, static_cast<const gen::Cfg::OffsetT*>(offsets), out);\n}\n";
        kernel = compileKernel(s.str(), "thor_segmented_broadcast", stream.getGpuNum(), /*fastContract=*/false);
        kernel = builtKernels.getOrCreate(key.str(), [&] { return kernel; });
    }

    std::ostringstream variant;
    variant << (ids ? "segment_ids(chunk_rows=" : "segmented_broadcast(chunk_rows=") << chunkRows << ",window=" << window << ",vec=" << vec << ",grid=" << chunks << ") [" << kernel->kernelName
            << "]";
    return std::make_shared<StampedSegmentedBroadcast>(kernel, per_segment_values, segment_offsets, output, static_cast<uint32_t>(chunks), variant.str());
}
}  // namespace

void StampedSegmentedBroadcast::runOn(Stream& stream) const {
    if (!stream.isInitialized() || stream.getGpuNum() != static_cast<int>(output.getPlacement().getDeviceNum())) {
        throw std::runtime_error("Segmented broadcast requires tensors on the execution GPU.");
    }
    ScopedGpu scoped(stream.getGpuNum());
    const void* valuePointer = values.getMemPtr();
    const void* offsetPointer = offsets.getMemPtr();
    void* out = const_cast<Tensor&>(output).getMemPtr();
    std::vector<void*> args = {&valuePointer, &offsetPointer, &out};
    kernel->launch(gridX, 1, 1, 256, stream.getStream(), args);
}

void launchSegmentedBroadcast(const Tensor& per_segment_values, const Tensor& segment_offsets, Tensor& output, bool normalize_by_segment_length,
                              Stream& stream) {
    stampSegmentedBroadcast(per_segment_values, segment_offsets, output, normalize_by_segment_length, stream)->runOn(stream);
}

}  // namespace ThorImplementation
