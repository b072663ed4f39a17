// Select-flagged and top-k: validation, kernel specialisation and launch (kernels: device/thor_device_select.h; reference
// behaviour: Utilities/TensorOperations/Cub/CubSelect.cu:54-136 plan / run protocol, CubTopK.cu:333-735 the four top-k families,
// CubDevicePrimitiveSupport.cpp:116-182,225-330 argument checks and the fixed-size limits of the row form).
#include "Utilities/TensorOperations/Cub/CubDevicePrimitives.h"

#include "ReductionPlanner.h"
#include "Utilities/Common/ScopedGpu.h"
#include "Utilities/Expression/CompiledEquation.h"
#include "thorhip_numeric_embed.h"

#include "Utilities/Cache/LruCache.h"

#include <algorithm>
#include <cstdlib>
#include <limits>
#include <sstream>
#include <string>
#include <stdexcept>
#include <vector>

namespace ThorImplementation {

// What one plan launches.  kind 0: select-flagged (count, offsets, scatter); 1: device-wide top-k (init, then one counting pass
// per digit whose last block picks the digit, gather; `third` is not used; or, for long inputs, floor, collect, finish); 2: top-k of rows (one launch).  A plan with nothing to do (no items, k == 0) holds no kernels.
struct CubSelectionKernels {
    int kind = 0;
    int deviceNum = 0;
    std::shared_ptr<CompiledKernel> first, second, third, fourth;
    // device-wide top-k over candidates: the sample that sets their floor, the copying pass, the histogram and the gathering
    // pass over the candidates
    std::shared_ptr<CompiledKernel> floor, collect, finish;  // candidates: the three launches of a long input
    uint32_t floorBlocks = 0, finishBlocks = 0;
    uint64_t chunks = 0;          // blocks of the counting / scattering / gathering launches; rows for kind 2
    uint32_t histogramBlocks = 0;
    uint32_t threads = 256;
    int digits = 0;                                // passes of the device-wide selection
    std::vector<std::pair<uint32_t, uint32_t>> digitPlan;  // (shift, bits) from the most significant digit down
    size_t countsBytes = 0;  // select: chunk counts, then as many chunk bases
    size_t tempBytes = 1;
    std::string variant;
};

namespace {

constexpr uint64_t kRowTopKMaxSegment = 8192, kRowTopKMaxK = 8192;
constexpr uint32_t kSelectThreads = 256, kSelectRounds = 4;
constexpr uint32_t kGatherThreads = 256, kGatherItems = 8;  // vectors per thread
constexpr uint32_t kTopKBins = 2048, kTopKStateWords = 16;
constexpr uint64_t kTopKCompactMinItems = 1ull << 20;

size_t roundUp(size_t v, size_t to) { return (v + to - 1) / to * to; }

void requireDenseGpu(const Tensor& tensor, const char* name) {
    if (!tensor.isInitialized()) throw std::invalid_argument(std::string(name) + " must be initialized.");
    if (tensor.getPlacement().getMemDevice() != TensorPlacement::MemDevices::GPU) throw std::invalid_argument(std::string(name) + " must be a GPU tensor.");
    if (!tensor.isDenseContiguous()) throw std::invalid_argument(std::string(name) + " must be dense contiguous.");
}
void requireSamePlacement(const Tensor& a, const Tensor& b, const char* aName, const char* bName) {
    if (a.getPlacement() != b.getPlacement()) throw std::invalid_argument(std::string(aName) + " and " + bName + " must live on the same GPU placement.");
}
void requireStorage(const Tensor& tensor, const char* name, uint64_t items) {
    if (tensor.getTotalNumElements() < items) throw std::invalid_argument(std::string(name) + " has fewer elements than num_items.");
}
void requireCount(uint64_t value, const char* name) {
    if (value > static_cast<uint64_t>(std::numeric_limits<int64_t>::max())) throw std::invalid_argument(std::string(name) + " exceeds CUB's int64 count limit.");
}
void requireTemp(const Tensor& temp, const TensorPlacement& placement, size_t bytes) {
    requireDenseGpu(temp, "temp_storage");
    if (temp.getPlacement() != placement) throw std::invalid_argument("temp_storage must live on the same GPU placement as the operation tensors.");
    if (temp.getDataType() != DataType::UINT8) throw std::invalid_argument("temp_storage must have dtype uint8.");
    if (temp.getTotalNumElements() < bytes) throw std::invalid_argument("temp_storage has fewer bytes than temp_storage_bytes.");
}
void requireStream(const Stream& stream, const TensorPlacement& placement) {
    if (!stream.isInitialized() || stream.getGpuNum() != static_cast<int>(placement.getDeviceNum())) {
        throw std::invalid_argument("The stream must live on the GPU of the operation tensors.");
    }
}

const char* rawWordName(DataType dtype) {
    switch (dataTypeSizeInBytes(dtype)) {
        case 1: return "thor::u8";
        case 2: return "thor::u16";
        default: return "thor::u32";
    }
}
int keyKind(DataType dtype) {  // 0 unsigned, 1 signed, 2 float
    switch (dtype) {
        case DataType::INT8:
        case DataType::INT16:
        case DataType::INT32: return 1;
        case DataType::FP16:
        case DataType::BF16:
        case DataType::FP32: return 2;
        default: return 0;
    }
}

// ---- select-flagged --------------------------------------------------------------------------------------------------------------
void validateSelect(const Tensor& input, const Tensor& flags, const Tensor& output, const Tensor& numSelected, uint64_t numItems) {
    requireDenseGpu(input, "input");
    requireDenseGpu(flags, "flags");
    requireDenseGpu(output, "output");
    requireDenseGpu(numSelected, "num_selected_out");
    requireSamePlacement(input, flags, "input", "flags");
    requireSamePlacement(input, output, "input", "output");
    requireSamePlacement(input, numSelected, "input", "num_selected_out");
    requireStorage(input, "input", numItems);
    requireStorage(flags, "flags", numItems);
    requireStorage(output, "output", numItems);
    requireStorage(numSelected, "num_selected_out", 1);
    if (input.getDataType() != output.getDataType()) throw std::invalid_argument("CUB select input/output dtypes must match.");
    if (!isCubSelectValueDTypeSupported(input.getDataType())) {
        throw std::invalid_argument(std::string("Unsupported CUB select value dtype ") + dataTypeName(input.getDataType()) + ".");
    }
    if (!isCubSelectFlagDTypeSupported(flags.getDataType())) {
        throw std::invalid_argument(std::string("Unsupported CUB select flag dtype ") + dataTypeName(flags.getDataType()) + ".");
    }
    if (numSelected.getDataType() != DataType::UINT32) throw std::invalid_argument("CUB select num_selected_out must have dtype uint32.");
    if (numItems > static_cast<uint64_t>(std::numeric_limits<int32_t>::max())) {
        throw std::invalid_argument("CUB device primitive num_items exceeds CUB's int item-count limit.");
    }
}

std::shared_ptr<const CubSelectionKernels> buildSelectKernelsUncached(DataType dtype, uint64_t numItems, int deviceNum, uint32_t vec) {
    auto kernels = std::make_shared<CubSelectionKernels>();
    CubSelectionKernels& k = *kernels;
    k.kind = 0;
    k.deviceNum = deviceNum;
    k.threads = kSelectThreads;
    const uint64_t chunkElems = uint64_t(kSelectThreads) * vec * kSelectRounds;
    k.chunks = std::max<uint64_t>((numItems + chunkElems - 1) / chunkElems, 1);
    k.countsBytes = roundUp(k.chunks * 4, 256);
    k.tempBytes = 2 * k.countsBytes;
    std::ostringstream s;
    s << thor_embed::kDevicePrelude << thor_embed::kSelectKernels;
    s << "namespace gen {\nstruct Cfg {\n    typedef " << rawWordName(dtype) << " Word;\n    static constexpr thor::u64 kTotal = " << numItems
      << "ull;\n    static constexpr int kThreads = " << kSelectThreads << ";\n    static constexpr int kVec = " << vec
      << ";\n    static constexpr int kRounds = " << kSelectRounds << ";\n    static constexpr thor::u64 kChunks = " << k.chunks << "ull;\n};\n}  // namespace gen\n";
    s << "extern \"C\" __global__ __launch_bounds__(" << kSelectThreads
      << ") void thor_select_count(const thor::u8* flags, thor::u32* counts) { thor::selectCount<gen::Cfg>(flags, counts); }\n";
    s << "extern \"C\" __global__ __launch_bounds__(1024) void thor_select_offsets(const thor::u32* counts, thor::u32* bases, thor::u32* numSelected) {\n"
         "    thor::selectOffsets<gen::Cfg>(counts, bases, numSelected);\n}\n";
    s << "extern \"C\" __global__ __launch_bounds__(" << kSelectThreads
      << ") void thor_select_scatter(const gen::Cfg::Word* in, const thor::u8* flags, const thor::u32* bases, gen::Cfg::Word* out) {\n"
         "    thor::selectScatter<gen::Cfg>(in, flags, bases, out);\n}\n";
    const std::string source = s.str();
    k.first = compileKernel(source, "thor_select_count", deviceNum, /*fastContract=*/false);
    k.second = compileKernel(source, "thor_select_offsets", deviceNum, false);
    k.third = compileKernel(source, "thor_select_scatter", deviceNum, false);
    std::ostringstream v;
    v << "select-flagged word" << dataTypeSizeInBytes(dtype) * 8 << " vec" << vec << " chunks" << k.chunks << "x" << chunkElems << " launches3 ["
      << k.third->kernelName << "]";
    k.variant = v.str();
    return kernels;
}

// ---- top-k -----------------------------------------------------------------------------------------------------------------------
void validateTopKKeys(const Tensor& keysIn, const Tensor& keysOut, uint64_t numItems, uint64_t k) {
    requireDenseGpu(keysIn, "keys_in");
    requireDenseGpu(keysOut, "keys_out");
    requireSamePlacement(keysIn, keysOut, "keys_in", "keys_out");
    requireStorage(keysIn, "keys_in", numItems);
    requireStorage(keysOut, "keys_out", std::min(numItems, k));
    if (keysIn.getDataType() != keysOut.getDataType()) throw std::invalid_argument("CUB top-k key input/output dtypes must match.");
    if (!isCubTopKKeyDTypeSupported(keysIn.getDataType())) {
        throw std::invalid_argument(std::string("Unsupported CUB top-k key dtype ") + dataTypeName(keysIn.getDataType()) + ".");
    }
    requireCount(numItems, "num_items");
    requireCount(k, "k");
    // the kernels count keys in 32-bit words
    if (numItems > 0xffffffffull) throw std::invalid_argument("CUB top-k num_items exceeds the 32-bit counters of this implementation.");
}
void validateTopKPairs(const Tensor& keysIn, const Tensor& keysOut, const Tensor& valuesIn, const Tensor& valuesOut, uint64_t numItems, uint64_t k) {
    validateTopKKeys(keysIn, keysOut, numItems, k);
    requireDenseGpu(valuesIn, "values_in");
    requireDenseGpu(valuesOut, "values_out");
    requireSamePlacement(keysIn, valuesIn, "keys_in", "values_in");
    requireSamePlacement(keysIn, valuesOut, "keys_in", "values_out");
    requireStorage(valuesIn, "values_in", numItems);
    requireStorage(valuesOut, "values_out", std::min(numItems, k));
    if (valuesIn.getDataType() != valuesOut.getDataType()) throw std::invalid_argument("CUB top-k value input/output dtypes must match.");
    if (!isCubTopKValueDTypeSupported(valuesIn.getDataType())) {
        throw std::invalid_argument(std::string("Unsupported CUB top-k index value dtype ") + dataTypeName(valuesIn.getDataType()) + ".");
    }
}

uint64_t rowTopKTotalItems(uint64_t numSegments, uint64_t segmentSize) {
    if (segmentSize != 0 && numSegments > std::numeric_limits<uint64_t>::max() / segmentSize) {
        throw std::invalid_argument("CUB segmented top-k num_segments * segment_size overflows uint64_t.");
    }
    const uint64_t total = numSegments * segmentSize;
    if (total > static_cast<uint64_t>(std::numeric_limits<int32_t>::max())) {
        throw std::invalid_argument("CUB segmented top-k total item count exceeds the current CUB fixed-size implementation limit.");
    }
    return total;
}
uint64_t rowTopKOutputItems(uint64_t numSegments, uint64_t segmentSize, uint64_t k) {
    const uint64_t perSegment = std::min(segmentSize, k);
    if (perSegment != 0 && numSegments > std::numeric_limits<uint64_t>::max() / perSegment) {
        throw std::invalid_argument("CUB segmented top-k num_segments * k overflows uint64_t.");
    }
    requireCount(numSegments * perSegment, "num_segments * k");
    return numSegments * perSegment;
}
void validateRowTopKKeys(const Tensor& keysIn, const Tensor& keysOut, uint64_t numSegments, uint64_t segmentSize, uint64_t k) {
    requireDenseGpu(keysIn, "keys_in");
    requireDenseGpu(keysOut, "keys_out");
    requireSamePlacement(keysIn, keysOut, "keys_in", "keys_out");
    requireStorage(keysIn, "keys_in", rowTopKTotalItems(numSegments, segmentSize));
    requireStorage(keysOut, "keys_out", rowTopKOutputItems(numSegments, segmentSize, k));
    if (keysIn.getDataType() != keysOut.getDataType()) throw std::invalid_argument("CUB segmented top-k key input/output dtypes must match.");
    if (!isCubTopKKeyDTypeSupported(keysIn.getDataType())) {
        throw std::invalid_argument(std::string("Unsupported CUB segmented top-k key dtype ") + dataTypeName(keysIn.getDataType()) + ".");
    }
    requireCount(numSegments, "num_segments");
    requireCount(segmentSize, "segment_size");
    requireCount(k, "k");
    if (numSegments == 0 || k == 0) return;
    if (segmentSize == 0) throw std::invalid_argument("CUB segmented top-k segment_size must be nonzero when num_segments and k are nonzero.");
    if (segmentSize > kRowTopKMaxSegment) throw std::invalid_argument("CUB segmented top-k segment_size exceeds CUB's current fixed-size support limit.");
    if (k > kRowTopKMaxK) throw std::invalid_argument("CUB segmented top-k k exceeds CUB's current fixed-size support limit.");
    if (k >= segmentSize) throw std::invalid_argument("CUB segmented top-k currently requires k to be smaller than the fixed segment size.");
}
void validateRowTopKPairs(const Tensor& keysIn, const Tensor& keysOut, const Tensor& valuesIn, const Tensor& valuesOut, uint64_t numSegments,
                          uint64_t segmentSize, uint64_t k) {
    validateRowTopKKeys(keysIn, keysOut, numSegments, segmentSize, k);
    requireDenseGpu(valuesIn, "values_in");
    requireDenseGpu(valuesOut, "values_out");
    requireSamePlacement(keysIn, valuesIn, "keys_in", "values_in");
    requireSamePlacement(keysIn, valuesOut, "keys_in", "values_out");
    requireStorage(valuesIn, "values_in", rowTopKTotalItems(numSegments, segmentSize));
    requireStorage(valuesOut, "values_out", rowTopKOutputItems(numSegments, segmentSize, k));
    if (valuesIn.getDataType() != valuesOut.getDataType()) throw std::invalid_argument("CUB segmented top-k value input/output dtypes must match.");
    if (!isCubTopKValueDTypeSupported(valuesIn.getDataType())) {
        throw std::invalid_argument(std::string("Unsupported CUB segmented top-k index value dtype ") + dataTypeName(valuesIn.getDataType()) + ".");
    }
}

void writeKeyTraits(std::ostringstream& s, DataType dtype, bool largest, bool pairs) {
    s << "    typedef " << rawWordName(dtype) << " Raw;\n    static constexpr int kKind = " << keyKind(dtype)
      << ";\n    static constexpr int kBits = " << dataTypeSizeInBytes(dtype) * 8 << ";\n    static constexpr bool kLargest = " << (largest ? "true" : "false")
      << ";\n    static constexpr bool kPairs = " << (pairs ? "true" : "false") << ";\n";
}

std::vector<std::pair<uint32_t, uint32_t>> digitPlanFor(uint32_t keyBits) {
    if (keyBits == 32) return {{21, 11}, {10, 11}, {0, 10}};
    if (keyBits == 16) return {{8, 8}, {0, 8}};
    return {{0, 8}};
}

// numItems > 0 and 0 < k (already capped at numItems)
std::shared_ptr<const CubSelectionKernels> buildTopKKernelsUncached(DataType dtype, uint64_t numItems, uint64_t k, bool largest, bool pairs, int deviceNum,
                                                            uint64_t keyAlignmentBytes) {
    auto kernels = std::make_shared<CubSelectionKernels>();
    CubSelectionKernels& sel = *kernels;
    sel.kind = 1;
    sel.deviceNum = deviceNum;
    sel.threads = kGatherThreads;
    const uint32_t keyBytes = dataTypeSizeInBytes(dtype);
    sel.digitPlan = digitPlanFor(keyBytes * 8);
    sel.digits = static_cast<int>(sel.digitPlan.size());
    uint64_t vec = 16 / keyBytes;
    while (vec > 1 && (numItems % vec != 0 || keyAlignmentBytes % (vec * keyBytes) != 0)) vec /= 2;
    const uint64_t vectors = numItems / vec;
    const uint64_t chunkVectors = uint64_t(kGatherThreads) * kGatherItems;
    sel.chunks = (vectors + chunkVectors - 1) / chunkVectors;
    // enough striding blocks to keep every compute unit busy, few enough that the global histogram sees little contention
    sel.histogramBlocks = static_cast<uint32_t>(std::min<uint64_t>((vectors + 255) / 256, 2048));
    // Long inputs with more than one digit are read once, in three launches (the kernels' file describes them): a floor from a
    // sample, the pass over the input that lists the keys above the floor, and the output out of that list.
    // The sample: max(2^19, 128 k) keys in runs of 256 vectors spread evenly, 32 vectors per lane (8 when the input is too short
    // for that many runs of 256 vectors: larger wavefront samples give values that scatter less), 512 maxima per wavefront; every wavefront's
    // value is reached by floorRank = ceil(k / wavefronts) of its maxima.  Somewhat more than k * items / sample keys become
    // candidates (the smallest of the wavefronts' values lies below what the whole sample would give); the list has room for
    // a 32nd of the input.  When k is more than a 256th of the input the candidates would not fit: every digit then reads
    // the whole input.
    // (k beyond 2^18: the keys that share the k-th largest key's bucket, about a 40th of k, would be more than the last block of
    // the third launch holds in registers.)
    bool compact = sel.digits >= 2 && numItems >= kTopKCompactMinItems && numItems < (1ull << 32) && k * 256 <= numItems && k <= (1ull << 18);
    bool forced = false;
    if (const char* env = std::getenv("THOR_TOPK_CANDIDATES")) {  // tuning / test switch: "0" reads the whole input in every pass
        if (std::string(env) == "0") compact = false;
        // "1": also short inputs and large k, down to no sample at all (a floor of zero: every key is a candidate)
        if (std::string(env) == "1") compact = forced = sel.digits >= 2 && numItems < (1ull << 32);
    }
    uint64_t floorBlocks = 0, floorRank = 0, sampleRunStride = 0, kFloorItems = 8;
    if (compact) {
        const uint64_t sampleKeys = std::max<uint64_t>(uint64_t(1) << 19, 128 * k);
        if (vectors / (256 * 32) >= (sampleKeys + 256 * 32 * vec - 1) / (256 * 32 * vec)) kFloorItems = 32;
        if (const char* env = std::getenv("THOR_TOPK_SAMPLE_ITEMS")) kFloorItems = std::max(std::atoi(env) / 8, 1) * 8;  // tuning switch
        const uint64_t blockKeys = 256 * kFloorItems * vec;
        floorBlocks = std::min<uint64_t>({(sampleKeys + blockKeys - 1) / blockKeys, 512, vectors / (256 * kFloorItems)});
        if (const char* env = std::getenv("THOR_TOPK_SAMPLE_BLOCKS")) {  // tuning switch
            floorBlocks = std::min<uint64_t>(std::max<long>(std::atol(env), 1), vectors / (256 * kFloorItems));
        }
        if (floorBlocks != 0) {
            floorRank = (k + floorBlocks * 4 - 1) / (floorBlocks * 4);
            sampleRunStride = vectors / (floorBlocks * kFloorItems);  // >= 256: the runs do not overlap
        }
        if (floorBlocks == 0 || floorRank > 64 * 8 / 2) {  // a value that most of a wavefront's maxima must reach says little
            compact = forced;
            floorBlocks = 1;
            floorRank = 0;  // no sample: the floor is zero
            sampleRunStride = 0;
        }
    }
    uint64_t regions = 0, regionEntries = 0, ambiguous = 0;
    if (compact) {
        // Every block of the pass over the input ends with additions to the same few words of the shared histogram, a request
        // for room in the list and a ticket, and those are served one after the other: more blocks, longer tail.
        uint64_t limit = 1024;
        if (const char* env = std::getenv("THOR_TOPK_BLOCKS")) limit = std::max<long>(std::atol(env), 1);  // tuning switch
        sel.histogramBlocks = static_cast<uint32_t>(std::min<uint64_t>((vectors + 255) / 256, limit));
        // every wavefront of that pass owns room for its share of a 32nd of the input, at least 64 entries
        regions = uint64_t(sel.histogramBlocks) * (256 / 64);
        regionEntries = std::max<uint64_t>((numItems / 32 + regions - 1) / regions, 64);
        if (const char* env = std::getenv("THOR_TOPK_REGION")) regionEntries = std::max<long>(std::atol(env), 1);  // test switch: entries per wavefront
        ambiguous = 16384;
        if (const char* env = std::getenv("THOR_TOPK_AMBIGUOUS")) ambiguous = std::min<long>(std::max<long>(std::atol(env), 1), 16384);  // test switch: entries of the second list (at most what the last block holds in registers)
        // the third launch: a wavefront per batch of regions; the same blocks walk the whole input when a region overflowed
        long finishLimit = 256;
        if (const char* env = std::getenv("THOR_TOPK_FINISH_BLOCKS")) finishLimit = std::max<long>(std::atol(env), 1);  // tuning switch
        sel.finishBlocks = static_cast<uint32_t>(std::min<uint64_t>((regions + 15) / 16, static_cast<uint64_t>(finishLimit)));
        sel.floorBlocks = static_cast<uint32_t>(floorBlocks);
    }
    sel.tempBytes = (kTopKBins + kTopKStateWords) * 4;
    if (compact) sel.tempBytes += (floorBlocks * 4 + k + 2 * ambiguous + regions + regions * regionEntries * (pairs ? 2 : 1)) * 4;
    std::ostringstream s;
    s << thor_embed::kDevicePrelude << thor_embed::kSelectKernels;
    s << "namespace gen {\nstruct Cfg {\n";
    writeKeyTraits(s, dtype, largest, pairs);
    s << "    static constexpr thor::u64 kTotal = " << numItems << "ull;\n    static constexpr thor::u64 kK = " << k
      << "ull;\n    static constexpr int kVec = " << vec << ";\n    static constexpr int kThreads = " << kGatherThreads
      << ";\n    static constexpr int kItems = " << kGatherItems << ";\n    static constexpr bool kCompact = " << (compact ? "true" : "false")
      << ";\n    static constexpr thor::u32 kBucketBits = " << (std::getenv("THOR_TOPK_BUCKET_BITS") ? std::min(std::max(std::atoi(std::getenv("THOR_TOPK_BUCKET_BITS")), 3), 6) : 6)
      << ";\n    static constexpr int kWalkPerLane = " << (std::getenv("THOR_TOPK_WALK") ? std::max(std::atoi(std::getenv("THOR_TOPK_WALK")), 1) : 2)
      << ";\n    static constexpr int kCompactUnroll = " << (std::getenv("THOR_TOPK_COMPACT_UNROLL") ? std::max(std::atoi(std::getenv("THOR_TOPK_COMPACT_UNROLL")), 1) : 2)
      << ";\n    static constexpr thor::u32 kFloorBlocks = " << std::max<uint64_t>(floorBlocks, 1) << "u;\n    static constexpr int kFloorItems = " << kFloorItems
      << ";\n    static constexpr thor::u32 kFloorRank = " << floorRank << "u;\n    static constexpr thor::u64 kSampleRunStride = " << sampleRunStride
      << "ull;\n    static constexpr thor::u32 kRegion = " << regionEntries << "u;\n    static constexpr thor::u32 kRegions = " << regions
      << "u;\n    static constexpr thor::u32 kAmbiguous = " << ambiguous << "u;\n};\n}  // namespace gen\n";
    if (!compact) {
        s << "extern \"C\" __global__ __launch_bounds__(256) void thor_topk_init(thor::u32* temp) { thor::topkInit<gen::Cfg>(temp); }\n";
        // every counting pass ends with the pick of its digit, by the block that finishes last
        s << "extern \"C\" __global__ __launch_bounds__(256) void thor_topk_histogram(const gen::Cfg::Raw* keys, thor::u32* temp, thor::u32 shift, thor::u32 bits) {\n"
             "    thor::topkHistogram<gen::Cfg>(keys, temp, shift, bits);\n}\n";
        s << "extern \"C\" __global__ __launch_bounds__(" << kGatherThreads
          << ") void thor_topk_gather(const gen::Cfg::Raw* keys, const thor::u32* values, thor::u32* temp, gen::Cfg::Raw* outKeys, thor::u32* outValues) {\n"
             "    thor::topkGather<gen::Cfg>(keys, values, temp, outKeys, outValues);\n}\n";
    } else {
        s << "extern \"C\" __global__ __launch_bounds__(256) void thor_topk_floor(const gen::Cfg::Raw* keys, thor::u32* temp) {\n"
             "    thor::topkFloor<gen::Cfg>(keys, temp);\n}\n";
        s << "extern \"C\" __global__ __launch_bounds__(256) void thor_topk_collect(const gen::Cfg::Raw* keys, thor::u32* temp) {\n"
             "    thor::topkCollect<gen::Cfg>(keys, temp);\n}\n";
        s << "extern \"C\" __global__ __launch_bounds__(256) void thor_topk_finish(const gen::Cfg::Raw* keys, const thor::u32* values, thor::u32* temp, "
             "gen::Cfg::Raw* outKeys, thor::u32* outValues) {\n    thor::topkFinish<gen::Cfg>(keys, values, temp, outKeys, outValues);\n}\n";
    }
    const std::string source = s.str();
    int launches = 2 + sel.digits;  // init, one counting pass per digit, the gathering pass
    if (!compact) {
        sel.first = compileKernel(source, "thor_topk_init", deviceNum, false);
        sel.second = compileKernel(source, "thor_topk_histogram", deviceNum, false);
        sel.fourth = compileKernel(source, "thor_topk_gather", deviceNum, false);
    } else {
        sel.floor = compileKernel(source, "thor_topk_floor", deviceNum, false);
        sel.collect = compileKernel(source, "thor_topk_collect", deviceNum, false);
        sel.finish = compileKernel(source, "thor_topk_finish", deviceNum, false);
        launches = 3;
    }
    std::ostringstream v;
    v << "top-k radix-select bits" << keyBytes * 8 << " digits" << sel.digits << " vec" << vec << (largest ? " largest" : " smallest") << (pairs ? " pairs" : " keys")
      << " k" << k << " of " << numItems
      << (compact ? " candidates(sample=" + std::to_string(floorBlocks * 4) + "x" + std::to_string(64 * kFloorItems * vec) + ",rank=" + std::to_string(floorRank) +
                        ",regions=" + std::to_string(regions) + "x" + std::to_string(regionEntries) + ")"
                  : std::string())
      << " launches" << launches << " [" << (compact ? sel.collect : sel.second)->kernelName << "]";
    sel.variant = v.str();
    return kernels;
}

// numSegments > 0, 0 < k < segmentSize <= 8192
std::shared_ptr<const CubSelectionKernels> buildRowTopKKernelsUncached(DataType dtype, uint64_t numSegments, uint64_t segmentSize, uint64_t k, bool largest,
                                                               bool pairs, int deviceNum) {
    auto kernels = std::make_shared<CubSelectionKernels>();
    CubSelectionKernels& sel = *kernels;
    sel.kind = 2;
    sel.deviceNum = deviceNum;
    sel.threads = 256;
    sel.digits = static_cast<int>(digitPlanFor(dataTypeSizeInBytes(dtype) * 8).size());
    sel.chunks = numSegments;
    // Rows that a wavefront can hold (at most 64 keys per lane: 4096 keys) take the kernel with one wavefront per row and four
    // rows per block; longer rows the one with a block per row.  THOR_TOPK_ROW_KERNEL=block forces the latter (a test switch).
    const uint64_t vec = 16 / dataTypeSizeInBytes(dtype);
    const uint64_t vectorsPerLane = (segmentSize + 64 * vec - 1) / (64 * vec);
    const char* forced = std::getenv("THOR_TOPK_ROW_KERNEL");
    const bool wavePerRow = vectorsPerLane * vec <= 64 && !(forced && std::string(forced) == "block");
    const uint64_t items = wavePerRow ? vectorsPerLane : (segmentSize + 255) / 256;
    sel.chunks = wavePerRow ? (numSegments + 3) / 4 : numSegments;
    std::ostringstream s;
    s << thor_embed::kDevicePrelude << thor_embed::kSelectKernels;
    s << "namespace gen {\nstruct Cfg {\n";
    writeKeyTraits(s, dtype, largest, pairs);
    s << "    static constexpr thor::u32 kSegment = " << segmentSize << "u;\n    static constexpr thor::u64 kK = " << k
      << "ull;\n    static constexpr thor::u64 kRows = " << numSegments << "ull;\n    static constexpr int kVec = " << vec
      << ";\n    static constexpr int kThreads = 256;\n    static constexpr int kItems = " << items << ";\n};\n}  // namespace gen\n";
    // A wavefront of the one-per-row kernel spends most of its life waiting (the row's loads, then chains of votes and counts), so
    // what counts is how many of them a SIMD holds: the compiler is asked to leave room for as many as the row's registers
    // (two 16-bit images to a register) plus about 40 others allow.  Measured on [16384, 4096] bf16, k = 64 (wavefronts per SIMD
    // asked for -> time): none 38.1 us, 5 34.0, 6 31.6, 7 30.8, 8 37.1 (spills).  THOR_TOPK_ROW_WAVES overrides it (a tuning switch).
    const uint64_t rowRegisters = vectorsPerLane * vec / (dataTypeSizeInBytes(dtype) == 2 ? 2 : 1);
    const char* forcedWaves = std::getenv("THOR_TOPK_ROW_WAVES");
    const int wavesPerSimd = forcedWaves ? std::max(1, std::atoi(forcedWaves)) : static_cast<int>(std::min<uint64_t>(8, std::max<uint64_t>(1, 512 / (rowRegisters + 41))));
    s << "extern \"C\" __global__ __launch_bounds__(256" << (wavePerRow ? ", " + std::to_string(wavesPerSimd) : std::string())
      << ") void thor_topk_rows(const gen::Cfg::Raw* keys, const thor::u32* values, gen::Cfg::Raw* outKeys, "
         "thor::u32* outValues) {\n    thor::" << (wavePerRow ? "topkRowsWave" : "topkRows") << "<gen::Cfg>(keys, values, outKeys, outValues);\n}\n";
    sel.first = compileKernel(s.str(), "thor_topk_rows", deviceNum, false);
    std::ostringstream v;
    v << "row top-k " << (wavePerRow ? "bit-select wavefront-per-row" : "radix-select block-per-row") << " bits" << dataTypeSizeInBytes(dtype) * 8
      << (wavePerRow ? " vec" + std::to_string(vec) + "x" + std::to_string(items) + (k <= 64 && vectorsPerLane % 2 == 0 && segmentSize >= 32 * vec * vectorsPerLane && vectorsPerLane * vec > 16 ? " floor-candidates" : "")
                     : " digits" + std::to_string(sel.digits))
      << (largest ? " largest" : " smallest") << (pairs ? " pairs" : " keys") << " k" << k << " of "
      << segmentSize << " rows" << numSegments << " launches1 [" << sel.first->kernelName << "]";
    sel.variant = v.str();
    return kernels;
}

// Callers that prepare on every call (the one-call C entry points) find their kernels by the few numbers that decide the text,
// and by the tuning switches' values, instead of writing out and hashing a hundred kilobytes of source each time.
std::string requestKey(const char* family, std::initializer_list<uint64_t> numbers) {
    std::string key = family;
    for (uint64_t v : numbers) key += ' ' + std::to_string(v);
    for (const char* name : {"THOR_TOPK_CANDIDATES", "THOR_TOPK_REGION", "THOR_TOPK_AMBIGUOUS", "THOR_TOPK_BLOCKS", "THOR_TOPK_SAMPLE_BLOCKS", "THOR_TOPK_SAMPLE_ITEMS",
                             "THOR_TOPK_FINISH_BLOCKS", "THOR_TOPK_WALK", "THOR_TOPK_BUCKET_BITS", "THOR_TOPK_COMPACT_UNROLL", "THOR_TOPK_ROW_KERNEL", "THOR_TOPK_ROW_WAVES"}) {
        const char* value = std::getenv(name);
        key += '|';
        if (value) key += value;
    }
    return key;
}
LruCacheThreadSafe<std::string, std::shared_ptr<const CubSelectionKernels>>& builtSelections() {
    static LruCacheThreadSafe<std::string, std::shared_ptr<const CubSelectionKernels>> cache(1024);
    return cache;
}
template <typename Build>
std::shared_ptr<const CubSelectionKernels> builtOnce(const std::string& key, const Build& build) {
    if (auto known = builtSelections().get(key)) return *known;
    std::shared_ptr<const CubSelectionKernels> built = build();
    return builtSelections().getOrCreate(key, [&] { return built; });
}
std::shared_ptr<const CubSelectionKernels> buildSelectKernels(DataType dtype, uint64_t numItems, int deviceNum, uint32_t vec) {
    return builtOnce(requestKey("select", {static_cast<uint64_t>(dtype), numItems, static_cast<uint64_t>(deviceNum), vec}),
                     [&] { return buildSelectKernelsUncached(dtype, numItems, deviceNum, vec); });
}
std::shared_ptr<const CubSelectionKernels> buildTopKKernels(DataType dtype, uint64_t numItems, uint64_t k, bool largest, bool pairs, int deviceNum,
                                                            uint64_t keyAlignmentBytes) {
    // (the alignment only matters up to the 16 bytes of a vector)
    return builtOnce(requestKey("topk", {static_cast<uint64_t>(dtype), numItems, k, largest, pairs, static_cast<uint64_t>(deviceNum), std::min<uint64_t>(keyAlignmentBytes, 16)}),
                     [&] { return buildTopKKernelsUncached(dtype, numItems, k, largest, pairs, deviceNum, keyAlignmentBytes); });
}
std::shared_ptr<const CubSelectionKernels> buildRowTopKKernels(DataType dtype, uint64_t numSegments, uint64_t segmentSize, uint64_t k, bool largest,
                                                               bool pairs, int deviceNum) {
    return builtOnce(requestKey("rows", {static_cast<uint64_t>(dtype), numSegments, segmentSize, k, largest, pairs, static_cast<uint64_t>(deviceNum)}),
                     [&] { return buildRowTopKKernelsUncached(dtype, numSegments, segmentSize, k, largest, pairs, deviceNum); });
}

void launchTopK(const CubSelectionKernels& sel, const void* keysIn, const void* valuesIn, void* temp, void* keysOut, void* valuesOut, Stream& stream) {
    ScopedGpu scoped(sel.deviceNum);
    void* raw = stream.getStream();
    if (sel.kind == 2) {
        std::vector<void*> args = {&keysIn, &valuesIn, &keysOut, &valuesOut};
        sel.first->launch(static_cast<uint32_t>(sel.chunks), 1, 1, sel.threads, raw, args);
        return;
    }
    std::vector<void*> gatherArgs = {&keysIn, &valuesIn, &temp, &keysOut, &valuesOut};
    if (sel.collect) {
        std::vector<void*> readArgs = {&keysIn, &temp};
        sel.floor->launch(sel.floorBlocks, 1, 1, 256, raw, readArgs);
        sel.collect->launch(sel.histogramBlocks, 1, 1, 256, raw, readArgs);
        sel.finish->launch(sel.finishBlocks, 1, 1, 256, raw, gatherArgs);
        return;
    }
    std::vector<void*> initArgs = {&temp};
    sel.first->launch(1, 1, 1, 256, raw, initArgs);
    for (size_t d = 0; d < sel.digitPlan.size(); ++d) {
        uint32_t shift = sel.digitPlan[d].first, bits = sel.digitPlan[d].second;
        std::vector<void*> countArgs = {&keysIn, &temp, &shift, &bits};
        sel.second->launch(sel.histogramBlocks, 1, 1, 256, raw, countArgs);
    }
    sel.fourth->launch(static_cast<uint32_t>(sel.chunks), 1, 1, sel.threads, raw, gatherArgs);
}

void* tempPointer(const Tensor& temp) { return const_cast<Tensor&>(temp).getMemPtr(); }

}  // namespace

bool isCubTopKKeyDTypeSupported(DataType dtype) {
    switch (dtype) {
        case DataType::UINT8:
        case DataType::INT8:
        case DataType::UINT16:
        case DataType::INT16:
        case DataType::UINT32:
        case DataType::INT32:
        case DataType::FP16:
        case DataType::BF16:
        case DataType::FP32: return true;
        default: return false;
    }
}
bool isCubTopKValueDTypeSupported(DataType dtype) { return dtype == DataType::UINT32; }
bool isCubSelectValueDTypeSupported(DataType dtype) { return isCubTopKKeyDTypeSupported(dtype); }
bool isCubSelectFlagDTypeSupported(DataType dtype) { return dtype == DataType::BOOLEAN || dtype == DataType::UINT8; }

CubTemporaryStoragePlan cubTemporaryStoragePlan(const TensorPlacement& placement, size_t bytes) {
    if (placement.getMemDevice() != TensorPlacement::MemDevices::GPU) throw std::invalid_argument("CUB temporary storage must be planned on GPU placement.");
    CubTemporaryStoragePlan plan;
    plan.placement = placement;
    plan.bytes = std::max<size_t>(bytes, 1);
    return plan;
}
CubTemporaryStoragePlan cubMaxTemporaryStoragePlan(std::initializer_list<CubTemporaryStoragePlan> plans) {
    if (plans.size() == 0) throw std::invalid_argument("At least one CUB temporary-storage plan is required.");
    auto it = plans.begin();
    CubTemporaryStoragePlan combined = cubTemporaryStoragePlan(it->placement, it->bytes);
    for (++it; it != plans.end(); ++it) {
        if (it->placement != combined.placement) throw std::invalid_argument("All CUB temporary-storage plans must use the same GPU placement.");
        combined.bytes = std::max(combined.bytes, std::max<size_t>(it->bytes, 1));
    }
    return combined;
}
Tensor allocateCubTemporaryStorage(const CubTemporaryStoragePlan& plan) { return allocateCubTemporaryStorage(plan.placement, plan.bytes); }

std::string cubSelectionKernelVariant(const std::shared_ptr<const CubSelectionKernels>& kernels) { return kernels ? kernels->variant : std::string(); }

// ---- select-flagged --------------------------------------------------------------------------------------------------------------
CubDeviceSelectFlaggedPlan prepareCubDeviceSelectFlagged(const Tensor& input, const Tensor& flags, const Tensor& output, const Tensor& numSelected,
                                                         uint64_t numItems) {
    validateSelect(input, flags, output, numSelected, numItems);
    CubDeviceSelectFlaggedPlan plan;
    plan.placement = input.getPlacement();
    plan.input_dtype = input.getDataType();
    plan.flag_dtype = flags.getDataType();
    plan.num_items = numItems;
    // no items: the run only writes the zero count, with the offsets kernel of a one-chunk plan over no elements
    // the kernels are specialised for how the three streams are aligned: groups of four elements (four flag bytes) or single ones
    const uint64_t groupBytes = 4 * dataTypeSizeInBytes(plan.input_dtype);
    plan.vector_elements = pointerAlignment(input.getMemPtr()) % groupBytes == 0 && pointerAlignment(output.getMemPtr()) % groupBytes == 0 &&
                                   pointerAlignment(flags.getMemPtr()) % 4 == 0
                               ? 4
                               : 1;
    plan.kernels = buildSelectKernels(plan.input_dtype, numItems, static_cast<int>(plan.placement.getDeviceNum()), static_cast<uint32_t>(plan.vector_elements));
    plan.temp_storage_bytes = std::max<size_t>(plan.kernels->tempBytes, 1);
    return plan;
}
size_t cubDeviceSelectFlaggedTempBytes(const Tensor& input, const Tensor& flags, const Tensor& output, const Tensor& numSelected, uint64_t numItems) {
    return prepareCubDeviceSelectFlagged(input, flags, output, numSelected, numItems).temp_storage_bytes;
}
void cubDeviceSelectFlagged(const CubDeviceSelectFlaggedPlan& plan, const Tensor& temp, const Tensor& input, const Tensor& flags, Tensor& output,
                            Tensor& numSelected, Stream& stream) {
    validateSelect(input, flags, output, numSelected, plan.num_items);
    if (input.getPlacement() != plan.placement || input.getDataType() != plan.input_dtype || flags.getDataType() != plan.flag_dtype || !plan.kernels) {
        throw std::invalid_argument("CUB select-flagged plan is not compatible with the provided tensors.");
    }
    if (plan.vector_elements > 1) {
        const uint64_t bytes = plan.vector_elements * dataTypeSizeInBytes(plan.input_dtype);
        if (pointerAlignment(input.getMemPtr()) % bytes != 0 || pointerAlignment(output.getMemPtr()) % bytes != 0 ||
            pointerAlignment(flags.getMemPtr()) % plan.vector_elements != 0) {
            throw std::invalid_argument("CUB select-flagged plan was prepared for tensors aligned to four elements; these are not.");
        }
    }
    requireTemp(temp, plan.placement, plan.temp_storage_bytes);
    requireStream(stream, plan.placement);
    const CubSelectionKernels& k = *plan.kernels;
    ScopedGpu scoped(k.deviceNum);
    void* raw = stream.getStream();
    char* base = static_cast<char*>(tempPointer(temp));
    void* counts = base;
    void* bases = base + k.countsBytes;
    const void* in = const_cast<Tensor&>(input).getMemPtr();
    const void* flagBytes = const_cast<Tensor&>(flags).getMemPtr();
    void* out = output.getMemPtr();
    void* total = numSelected.getMemPtr();
    std::vector<void*> countArgs = {&flagBytes, &counts};
    const uint64_t chunksPerBlock = k.threads / 64;  // a wavefront counts a chunk
    k.first->launch(static_cast<uint32_t>((k.chunks + chunksPerBlock - 1) / chunksPerBlock), 1, 1, k.threads, raw, countArgs);
    std::vector<void*> offsetArgs = {&counts, &bases, &total};
    k.second->launch(1, 1, 1, 1024, raw, offsetArgs);
    if (plan.num_items == 0) return;
    std::vector<void*> scatterArgs = {&in, &flagBytes, &bases, &out};
    k.third->launch(static_cast<uint32_t>(k.chunks), 1, 1, k.threads, raw, scatterArgs);
}
void cubDeviceSelectFlagged(const Tensor& temp, size_t tempBytes, const Tensor& input, const Tensor& flags, Tensor& output, Tensor& numSelected,
                            uint64_t numItems, Stream& stream) {
    CubDeviceSelectFlaggedPlan plan = prepareCubDeviceSelectFlagged(input, flags, output, numSelected, numItems);
    if (tempBytes < plan.temp_storage_bytes) throw std::invalid_argument("temp_storage_bytes is smaller than the prepared CUB select-flagged requirement.");
    plan.temp_storage_bytes = tempBytes;
    cubDeviceSelectFlagged(plan, temp, input, flags, output, numSelected, stream);
}

// ---- device-wide top-k -------------------------------------------------------------------------------------------------------------
namespace {

template <typename Plan>
void fillTopKPlan(Plan& plan, const Tensor& keysIn, uint64_t numItems, uint64_t k, CubTopKOrder order, bool pairs) {
    plan.placement = keysIn.getPlacement();
    plan.key_dtype = keysIn.getDataType();
    plan.num_items = numItems;
    plan.k = k;
    plan.order = order;
    const uint64_t selected = std::min(numItems, k);
    if (selected != 0) {
        plan.key_alignment_bytes = std::min<uint64_t>(pointerAlignment(keysIn.getMemPtr()), 16);
        plan.kernels = buildTopKKernels(plan.key_dtype, numItems, selected, order == CubTopKOrder::Largest, pairs, static_cast<int>(plan.placement.getDeviceNum()),
                                        plan.key_alignment_bytes);
    }
    plan.temp_storage_bytes = plan.kernels ? plan.kernels->tempBytes : 1;
}

template <typename Plan>
void fillRowTopKPlan(Plan& plan, const Tensor& keysIn, uint64_t numSegments, uint64_t segmentSize, uint64_t k, CubTopKOrder order, bool pairs) {
    plan.placement = keysIn.getPlacement();
    plan.key_dtype = keysIn.getDataType();
    plan.num_segments = numSegments;
    plan.segment_size = segmentSize;
    plan.k = k;
    plan.order = order;
    if (numSegments != 0 && k != 0) {
        plan.kernels = buildRowTopKKernels(plan.key_dtype, numSegments, segmentSize, k, order == CubTopKOrder::Largest, pairs,
                                           static_cast<int>(plan.placement.getDeviceNum()));
    }
    plan.temp_storage_bytes = 1;
}

}  // namespace

CubDeviceTopKKeysPlan prepareCubDeviceTopKKeys(const Tensor& keysIn, const Tensor& keysOut, uint64_t numItems, uint64_t k, CubTopKOrder order) {
    validateTopKKeys(keysIn, keysOut, numItems, k);
    CubDeviceTopKKeysPlan plan;
    fillTopKPlan(plan, keysIn, numItems, k, order, false);
    return plan;
}
size_t cubDeviceTopKKeysTempBytes(const Tensor& keysIn, const Tensor& keysOut, uint64_t numItems, uint64_t k, CubTopKOrder order) {
    return prepareCubDeviceTopKKeys(keysIn, keysOut, numItems, k, order).temp_storage_bytes;
}
void cubDeviceTopKKeys(const CubDeviceTopKKeysPlan& plan, const Tensor& temp, const Tensor& keysIn, Tensor& keysOut, Stream& stream) {
    validateTopKKeys(keysIn, keysOut, plan.num_items, plan.k);
    if (keysIn.getPlacement() != plan.placement || keysIn.getDataType() != plan.key_dtype) {
        throw std::invalid_argument("CUB top-k-keys plan is not compatible with the provided tensors.");
    }
    if (pointerAlignment(keysIn.getMemPtr()) % plan.key_alignment_bytes != 0) {
        throw std::invalid_argument("CUB top-k-keys plan was prepared for keys with a stricter alignment than these have.");
    }
    requireTemp(temp, plan.placement, plan.temp_storage_bytes);
    requireStream(stream, plan.placement);
    if (!plan.kernels) return;
    launchTopK(*plan.kernels, const_cast<Tensor&>(keysIn).getMemPtr(), nullptr, tempPointer(temp), keysOut.getMemPtr(), nullptr, stream);
}
void cubDeviceTopKKeys(const Tensor& temp, size_t tempBytes, const Tensor& keysIn, Tensor& keysOut, uint64_t numItems, uint64_t k, Stream& stream,
                       CubTopKOrder order) {
    CubDeviceTopKKeysPlan plan = prepareCubDeviceTopKKeys(keysIn, keysOut, numItems, k, order);
    if (tempBytes < plan.temp_storage_bytes) throw std::invalid_argument("temp_storage_bytes is smaller than the prepared CUB top-k-keys requirement.");
    plan.temp_storage_bytes = tempBytes;
    cubDeviceTopKKeys(plan, temp, keysIn, keysOut, stream);
}

CubDeviceTopKPairsPlan prepareCubDeviceTopKPairs(const Tensor& keysIn, const Tensor& keysOut, const Tensor& valuesIn, const Tensor& valuesOut,
                                                 uint64_t numItems, uint64_t k, CubTopKOrder order) {
    validateTopKPairs(keysIn, keysOut, valuesIn, valuesOut, numItems, k);
    CubDeviceTopKPairsPlan plan;
    plan.value_dtype = valuesIn.getDataType();
    fillTopKPlan(plan, keysIn, numItems, k, order, true);
    return plan;
}
size_t cubDeviceTopKPairsTempBytes(const Tensor& keysIn, const Tensor& keysOut, const Tensor& valuesIn, const Tensor& valuesOut, uint64_t numItems,
                                   uint64_t k, CubTopKOrder order) {
    return prepareCubDeviceTopKPairs(keysIn, keysOut, valuesIn, valuesOut, numItems, k, order).temp_storage_bytes;
}
void cubDeviceTopKPairs(const CubDeviceTopKPairsPlan& plan, const Tensor& temp, const Tensor& keysIn, Tensor& keysOut, const Tensor& valuesIn,
                        Tensor& valuesOut, Stream& stream) {
    validateTopKPairs(keysIn, keysOut, valuesIn, valuesOut, plan.num_items, plan.k);
    if (keysIn.getPlacement() != plan.placement || keysIn.getDataType() != plan.key_dtype || valuesIn.getDataType() != plan.value_dtype) {
        throw std::invalid_argument("CUB top-k-pairs plan is not compatible with the provided tensors.");
    }
    if (pointerAlignment(keysIn.getMemPtr()) % plan.key_alignment_bytes != 0) {
        throw std::invalid_argument("CUB top-k-pairs plan was prepared for keys with a stricter alignment than these have.");
    }
    requireTemp(temp, plan.placement, plan.temp_storage_bytes);
    requireStream(stream, plan.placement);
    if (!plan.kernels) return;
    launchTopK(*plan.kernels, const_cast<Tensor&>(keysIn).getMemPtr(), const_cast<Tensor&>(valuesIn).getMemPtr(), tempPointer(temp), keysOut.getMemPtr(),
               valuesOut.getMemPtr(), stream);
}
void cubDeviceTopKPairs(const Tensor& temp, size_t tempBytes, const Tensor& keysIn, Tensor& keysOut, const Tensor& valuesIn, Tensor& valuesOut,
                        uint64_t numItems, uint64_t k, Stream& stream, CubTopKOrder order) {
    CubDeviceTopKPairsPlan plan = prepareCubDeviceTopKPairs(keysIn, keysOut, valuesIn, valuesOut, numItems, k, order);
    if (tempBytes < plan.temp_storage_bytes) throw std::invalid_argument("temp_storage_bytes is smaller than the prepared CUB top-k-pairs requirement.");
    plan.temp_storage_bytes = tempBytes;
    cubDeviceTopKPairs(plan, temp, keysIn, keysOut, valuesIn, valuesOut, stream);
}

// ---- top-k of rows ---------------------------------------------------------------------------------------------------------------
CubDeviceSegmentedTopKKeysPlan prepareCubDeviceSegmentedTopKKeys(const Tensor& keysIn, const Tensor& keysOut, uint64_t numSegments, uint64_t segmentSize,
                                                                 uint64_t k, CubTopKOrder order) {
    validateRowTopKKeys(keysIn, keysOut, numSegments, segmentSize, k);
    CubDeviceSegmentedTopKKeysPlan plan;
    fillRowTopKPlan(plan, keysIn, numSegments, segmentSize, k, order, false);
    return plan;
}
size_t cubDeviceSegmentedTopKKeysTempBytes(const Tensor& keysIn, const Tensor& keysOut, uint64_t numSegments, uint64_t segmentSize, uint64_t k,
                                           CubTopKOrder order) {
    return prepareCubDeviceSegmentedTopKKeys(keysIn, keysOut, numSegments, segmentSize, k, order).temp_storage_bytes;
}
void cubDeviceSegmentedTopKKeys(const CubDeviceSegmentedTopKKeysPlan& plan, const Tensor& temp, const Tensor& keysIn, Tensor& keysOut, Stream& stream) {
    validateRowTopKKeys(keysIn, keysOut, plan.num_segments, plan.segment_size, plan.k);
    if (keysIn.getPlacement() != plan.placement || keysIn.getDataType() != plan.key_dtype) {
        throw std::invalid_argument("CUB segmented top-k-keys plan is not compatible with the provided tensors.");
    }
    requireTemp(temp, plan.placement, plan.temp_storage_bytes);
    requireStream(stream, plan.placement);
    if (!plan.kernels) return;
    launchTopK(*plan.kernels, const_cast<Tensor&>(keysIn).getMemPtr(), nullptr, nullptr, keysOut.getMemPtr(), nullptr, stream);
}
void cubDeviceSegmentedTopKKeys(const Tensor& temp, size_t tempBytes, const Tensor& keysIn, Tensor& keysOut, uint64_t numSegments, uint64_t segmentSize,
                                uint64_t k, Stream& stream, CubTopKOrder order) {
    CubDeviceSegmentedTopKKeysPlan plan = prepareCubDeviceSegmentedTopKKeys(keysIn, keysOut, numSegments, segmentSize, k, order);
    if (tempBytes < plan.temp_storage_bytes) {
        throw std::invalid_argument("temp_storage_bytes is smaller than the prepared CUB segmented top-k-keys requirement.");
    }
    plan.temp_storage_bytes = tempBytes;
    cubDeviceSegmentedTopKKeys(plan, temp, keysIn, keysOut, stream);
}

CubDeviceSegmentedTopKPairsPlan prepareCubDeviceSegmentedTopKPairs(const Tensor& keysIn, const Tensor& keysOut, const Tensor& valuesIn,
                                                                   const Tensor& valuesOut, uint64_t numSegments, uint64_t segmentSize, uint64_t k,
                                                                   CubTopKOrder order) {
    validateRowTopKPairs(keysIn, keysOut, valuesIn, valuesOut, numSegments, segmentSize, k);
    CubDeviceSegmentedTopKPairsPlan plan;
    plan.value_dtype = valuesIn.getDataType();
    fillRowTopKPlan(plan, keysIn, numSegments, segmentSize, k, order, true);
    return plan;
}
size_t cubDeviceSegmentedTopKPairsTempBytes(const Tensor& keysIn, const Tensor& keysOut, const Tensor& valuesIn, const Tensor& valuesOut,
                                            uint64_t numSegments, uint64_t segmentSize, uint64_t k, CubTopKOrder order) {
    return prepareCubDeviceSegmentedTopKPairs(keysIn, keysOut, valuesIn, valuesOut, numSegments, segmentSize, k, order).temp_storage_bytes;
}
void cubDeviceSegmentedTopKPairs(const CubDeviceSegmentedTopKPairsPlan& plan, const Tensor& temp, const Tensor& keysIn, Tensor& keysOut,
                                 const Tensor& valuesIn, Tensor& valuesOut, Stream& stream) {
    validateRowTopKPairs(keysIn, keysOut, valuesIn, valuesOut, plan.num_segments, plan.segment_size, plan.k);
    if (keysIn.getPlacement() != plan.placement || keysIn.getDataType() != plan.key_dtype || valuesIn.getDataType() != plan.value_dtype) {
        throw std::invalid_argument("CUB segmented top-k-pairs plan is not compatible with the provided tensors.");
    }
    requireTemp(temp, plan.placement, plan.temp_storage_bytes);
    requireStream(stream, plan.placement);
    if (!plan.kernels) return;
    launchTopK(*plan.kernels, const_cast<Tensor&>(keysIn).getMemPtr(), const_cast<Tensor&>(valuesIn).getMemPtr(), nullptr, keysOut.getMemPtr(),
               valuesOut.getMemPtr(), stream);
}
void cubDeviceSegmentedTopKPairs(const Tensor& temp, size_t tempBytes, const Tensor& keysIn, Tensor& keysOut, const Tensor& valuesIn, Tensor& valuesOut,
                                 uint64_t numSegments, uint64_t segmentSize, uint64_t k, Stream& stream, CubTopKOrder order) {
    CubDeviceSegmentedTopKPairsPlan plan = prepareCubDeviceSegmentedTopKPairs(keysIn, keysOut, valuesIn, valuesOut, numSegments, segmentSize, k, order);
    if (tempBytes < plan.temp_storage_bytes) {
        throw std::invalid_argument("temp_storage_bytes is smaller than the prepared CUB segmented top-k-pairs requirement.");
    }
    plan.temp_storage_bytes = tempBytes;
    cubDeviceSegmentedTopKPairs(plan, temp, keysIn, keysOut, valuesIn, valuesOut, stream);
}

}  // namespace ThorImplementation
