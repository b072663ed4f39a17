// Prefix scans: validation, kernel specialisation and launch (kernels: device/thor_device_scan.h; reference behaviour:
// Utilities/TensorOperations/Cub/CubScan.cu:47-196 operators and identities, :314-420 plan / run protocol,
// CubSegmentedScan.cu for the uniform-segment and offset-segment forms).
#include "CubScanInternal.h"

#include "Utilities/Expression/StampedEquation.h"

#include "ReductionPlanner.h"
#include "Utilities/Common/ScopedGpu.h"
#include "thorhip_numeric_embed.h"
#include "Utilities/Cache/LruCache.h"

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <numeric>
#include <sstream>
#include <stdexcept>

namespace ThorImplementation {

namespace {

size_t roundUp(size_t v, size_t to) { return (v + to - 1) / to * to; }

const char* scanStorageName(DataType dtype) {
    switch (dtype) {
        case DataType::UINT32: return "thor::u32";
        case DataType::FP16: return "thor::f16";
        case DataType::BF16: return "thor::bf16";
        case DataType::FP32: return "float";
        default: break;
    }
    throw std::invalid_argument(std::string("Unsupported CUB scan dtype ") + dataTypeName(dtype) + ".");
}

struct ScanChunking {
    uint64_t vec = 1, threads = 256, items = 4, chunkElems = 0;
    bool carry = true;
    bool routable = false;  // a request with route set can run as it is
};

ScanChunking chooseScanChunking(const ScanRequest& r) {
    ScanChunking c;
    const bool ragged = r.row == 0;
    const uint32_t elementBytes = dataTypeSizeInBytes(r.dtype);
    c.vec = 16 / elementBytes;
    while (c.vec > 1 && (r.total % c.vec != 0 || r.alignmentBytes % (c.vec * std::max<uint32_t>(elementBytes, r.writeIndex || r.route ? 4 : elementBytes)) != 0)) {
        c.vec /= 2;
    }
    bool threadsForced = false;
    if (const char* env = std::getenv("THOR_SCAN_THREADS")) {  // tuning switch: 256, 512 or 1024 threads per block
        const long requested = std::atol(env);
        if (requested == 256 || requested == 512 || requested == 1024) {
            c.threads = static_cast<uint64_t>(requested);
            threadsForced = true;
        }
    }
    const uint64_t lanesWorth = c.threads * c.vec;
    uint64_t maxItems = 64 / (c.threads / 64) < 16 ? 64 / (c.threads / 64) : 16;
    // routing a gradient keeps an fp32 copy of the chunk in LDS: at most 32 KiB of it
    if (r.route) maxItems = std::min<uint64_t>(maxItems, kScanRouteMaxChunkElems / lanesWorth);
    c.chunkElems = lanesWorth * c.items;
    if (!ragged && maxItems > 0 && r.row <= lanesWorth * maxItems) {
        // chunks of whole rows: every chunk starts at a head and needs nothing from its predecessors
        const uint64_t step = c.vec / std::gcd(r.row, c.vec);  // rows per chunk must keep chunk starts on vector boundaries
        const uint64_t rowsPerChunk = std::max<uint64_t>(lanesWorth * std::min<uint64_t>(4, maxItems) / r.row / step * step, step);
        if (rowsPerChunk * r.row <= lanesWorth * maxItems) {
            c.chunkElems = rowsPerChunk * r.row;
            c.items = (c.chunkElems + lanesWorth - 1) / lanesWorth;
            c.carry = false;
        }
    }
    if (!c.carry && !threadsForced) {
        // A chunk of whole rows keeps its size; more threads hold fewer vectors each.  Measured on [8192, 8192] fp32 (256 / 512 /
        // 1024 threads): running sum 96 / 91 / 95 us, running arg-max 106 / 88 / 93 us, routed gradient 239 / 162 / 139 us - the
        // register arrays of the longer per-thread walks cost more residency than the extra wavefront totals.
        const uint64_t wanted = r.route ? 2 : 4;
        while (c.items > wanted && c.threads < 1024) {
            c.threads *= 2;
            c.items = (c.chunkElems + c.threads * c.vec - 1) / (c.threads * c.vec);
        }
    }
    c.routable = !c.carry && !ragged && (r.op == 1 || r.op == 2);
    if (c.carry) {
        // Chunks that wait for each other's totals: the fewer and larger, the fewer tickets and waits.  2^26 fp32 elements, flat:
        // 256 threads x 8 vectors 162 us, 512 x 8 127 us, 1024 x 4 117 us.  Shorter inputs keep the small chunks that fill the device.
        uint64_t threads = c.threads;
        if (!threadsForced && r.total >= 1024ull * 1024 * c.vec * 4) threads = 1024;
        const uint64_t wavesWorth = 64 / (threads / 64);
        c.threads = threads;
        c.items = std::min<uint64_t>(8, std::max<uint64_t>(std::min<uint64_t>(wavesWorth, 16), 1));
        c.chunkElems = c.threads * c.vec * c.items;
    }
    return c;
}

void writeScanTraits(std::ostringstream& s, const ScanRequest& r, bool isUnsigned, uint64_t threads, uint64_t vec, uint64_t items, uint64_t chunkElems,
                     const CubScanKernels& k) {
    // Waits between blocks are bounded so that every wavefront has an exit: 2^22 polls are seconds.  The test switch makes the
    // bound so small that waits give up, to exercise the way out: the wavefront works the missing totals out from the input.
    unsigned long waitLimit = 1ul << 22;
    if (const char* env = std::getenv("THOR_SCAN_WAIT_LIMIT")) waitLimit = std::min<unsigned long>(std::strtoul(env, nullptr, 10), 1ul << 30);
    s << "namespace gen {\nstruct Cfg {\n    typedef " << scanStorageName(r.dtype) << " T;\n    typedef " << (isUnsigned ? "thor::u32" : "float")
      << " Acc;\n    typedef " << (r.offsets64 ? "thor::u64" : "thor::u32") << " OffsetT;\n"
      << "    static constexpr bool kUnsigned = " << (isUnsigned ? "true" : "false") << ";\n    static constexpr int kOp = " << r.op
      << ";\n    static constexpr bool kArg = " << (r.writeIndex ? "true" : "false") << ";\n    static constexpr bool kInclusive = "
      << (r.inclusive ? "true" : "false") << ";\n    static constexpr bool kReverse = " << (r.reverse ? "true" : "false")
      << ";\n    static constexpr thor::u64 kTotal = " << r.total << "ull;\n    static constexpr thor::u64 kRow = " << r.row
      << "ull;\n    static constexpr thor::u64 kSegments = " << r.segments << "ull;\n    static constexpr int kThreads = " << threads
      << ";\n    static constexpr int kVec = " << vec << ";\n    static constexpr int kItems = " << items
      << ";\n    static constexpr thor::u64 kChunkElems = " << chunkElems << "ull;\n    static constexpr thor::u64 kChunks = " << k.chunks
      << "ull;\n    static constexpr bool kCarry = " << (k.carry ? "true" : "false") << ";\n    static constexpr bool kLookback = "
      << (k.lookback ? "true" : "false") << ";\n    static constexpr thor::u32 kWaitLimit = " << waitLimit << "u;\n    static constexpr thor::u64 kClearWords = " << k.clearWords
      << "ull;\n    static constexpr bool kWriteValue = "
      << (r.writeValue ? "true" : "false") << ";\n    static constexpr bool kWriteIndex = " << (r.writeIndex ? "true" : "false") << ";\n};\n}  // namespace gen\n";
}

}  // namespace

bool isCubScanDTypeSupported(DataType dtype) {
    return dtype == DataType::UINT32 || dtype == DataType::FP16 || dtype == DataType::BF16 || dtype == DataType::FP32;
}
bool isCubSegmentOffsetDTypeSupported(DataType dtype) { return dtype == DataType::UINT32 || dtype == DataType::UINT64; }

Tensor allocateCubTemporaryStorage(const TensorPlacement& placement, size_t bytes) {
    if (placement.getMemDevice() != TensorPlacement::MemDevices::GPU) throw std::invalid_argument("CUB temporary storage must be planned on GPU placement.");
    return Tensor(placement, TensorDescriptor(DataType::UINT8, {std::max<uint64_t>(bytes, 1)}));
}

namespace {
// The kernels of the requests seen so far, by request and by the switches that enter the generated source: a caller that repeats
// a request (a serving loop through the entry point that allocates nothing) gets them without the source being generated and
// hashed again.
const char* switchText(const char* name) {
    const char* value = std::getenv(name);
    return value ? value : "";
}
std::string requestKey(const ScanRequest& r) {
    char text[320];
    std::snprintf(text, sizeof text, "%d|%llu|%llu|%llu|%d|%d|%d%d%d%d%d|%llu|%d|%s|%s|%s", static_cast<int>(r.dtype), (unsigned long long)r.total,
                  (unsigned long long)r.row, (unsigned long long)r.segments, r.offsets64 ? 1 : 0, r.op, r.writeValue ? 1 : 0, r.writeIndex ? 1 : 0,
                  r.inclusive ? 1 : 0, r.reverse ? 1 : 0, r.route ? 1 : 0, (unsigned long long)r.alignmentBytes, r.deviceNum,
                  switchText("THOR_SCAN_WAIT_LIMIT"), switchText("THOR_SCAN_THREADS"), switchText("THOR_SCAN_PASSES"));
    return std::string(text) + "|" + switchText("THOR_SCAN_MIN_WAVES");
}
LruCacheThreadSafe<std::string, std::shared_ptr<const CubScanKernels>>& builtScans() {
    static LruCacheThreadSafe<std::string, std::shared_ptr<const CubScanKernels>> cache(1024);
    return cache;
}
std::shared_ptr<const CubScanKernels> buildScanKernelsUncached(const ScanRequest& r, bool loadedOnly, size_t tempLimitBytes);
}  // namespace

std::shared_ptr<const CubScanKernels> buildScanKernels(const ScanRequest& r, bool loadedOnly, size_t tempLimitBytes) {
    const std::string key = requestKey(r);
    if (auto known = builtScans().get(key)) {
        if ((*known)->tempBytes > tempLimitBytes) {
            throw std::invalid_argument("CUB scan: this request needs " + std::to_string((*known)->tempBytes) + " bytes of temporary storage, more than the " +
                                        std::to_string(tempLimitBytes) + " bytes of the fixed scratch block; use the allocating scan.");
        }
        return *known;
    }
    std::shared_ptr<const CubScanKernels> built = buildScanKernelsUncached(r, loadedOnly, tempLimitBytes);
    return builtScans().getOrCreate(key, [&] { return built; });
}

namespace {
std::shared_ptr<const CubScanKernels> buildScanKernelsUncached(const ScanRequest& r, bool loadedOnly, size_t tempLimitBytes) {
    if (!isCubScanDTypeSupported(r.dtype)) throw std::invalid_argument(std::string("Unsupported CUB scan dtype ") + dataTypeName(r.dtype) + ".");
    if (r.total == 0) throw std::invalid_argument("CUB scan requires at least one element.");
    if ((r.writeIndex || r.op == 1 || r.op == 2) && r.total > 0xfffffffeull) {
        throw std::invalid_argument("CUB min / max / arg scans index elements with UINT32: too many elements.");
    }
    const bool ragged = r.row == 0;
    if (!ragged && r.total % r.row != 0) throw std::invalid_argument("CUB uniform segmented scan requires num_items == num_segments * segment_size.");

    auto kernels = std::make_shared<CubScanKernels>();
    CubScanKernels& k = *kernels;
    k.request = r;
    const ScanChunking chunking = chooseScanChunking(r);
    if (r.route && !chunking.routable) {
        throw std::invalid_argument("CUB scan: the one-pass gradient routing needs a min / max scan over rows that fit one block's chunk.");
    }
    const uint64_t vec = chunking.vec, threads = chunking.threads, items = chunking.items, chunkElems = chunking.chunkElems;
    k.carry = chunking.carry;
    k.threads = static_cast<uint32_t>(threads);
    k.chunks = (r.total + chunkElems - 1) / chunkElems;
    if (k.chunks == 1) k.carry = false;
    if (k.chunks > 0x7fffffffull) throw std::invalid_argument("CUB scan: too many elements for one launch.");

    // Chunks that need what precedes them read it from totals that the blocks publish to each other (one pass over the data);
    // the fixed tree of those totals is three levels of 64, beyond which (or with THOR_SCAN_PASSES=3) separate launches
    // compute totals and carries first.
    const char* passes = std::getenv("THOR_SCAN_PASSES");
    k.lookback = k.carry && k.chunks <= 64ull * 64 * 64 && !(passes && std::atoi(passes) == 3);

    // temporary storage: head bitmap (ragged), then either the block of published totals (32 control words and two words per
    // chunk, group and super-group, 8 bytes each) or chunk totals and chunk carries
    k.headsBytes = ragged ? roundUp((r.total + 31) / 32 * 4, 256) : 0;
    if (k.lookback) {
        const uint64_t groups = (k.chunks + 63) / 64, supers = (groups + 63) / 64;
        k.statesBytes = roundUp(8 * (32 + 2 * (k.chunks + groups + supers)), 256);
        k.tempBytes = k.headsBytes + k.statesBytes;
        k.clearWords = k.tempBytes / 4;
    } else {
        k.statesBytes = k.carry ? roundUp(3 * k.chunks * 4, 256) : 0;
        k.tempBytes = std::max<size_t>(k.headsBytes + 2 * k.statesBytes, 1);
        k.clearWords = k.headsBytes / 4;
    }
    if (k.tempBytes > tempLimitBytes) {
        throw std::invalid_argument("CUB scan: this request needs " + std::to_string(k.tempBytes) + " bytes of temporary storage, more than the " +
                                    std::to_string(tempLimitBytes) + " bytes of the fixed scratch block; use the allocating scan.");
    }

    const bool isUnsigned = r.dtype == DataType::UINT32;
    if (r.route) {
        std::ostringstream s;
        s << thor_embed::kDevicePrelude << thor_embed::kScanKernels;
        writeScanTraits(s, r, isUnsigned, threads, vec, items, chunkElems, k);
        s << "extern \"C\" __global__ __launch_bounds__(" << threads
          << ") void thor_scan_route(const gen::Cfg::T* in, const float* gradient, float* routed) {\n    thor::scanRoute<gen::Cfg>(in, gradient, routed);\n}\n";
        k.mainKernel = compileKernel(s.str(), "thor_scan_route", r.deviceNum, /*fastContract=*/false);
        std::ostringstream v;
        v << "scan-route " << (r.op == 1 ? "min" : "max") << (r.inclusive ? " inclusive" : " exclusive") << (r.reverse ? " reverse" : "") << " rows" << r.row
          << " chunk" << chunkElems << " vec" << vec << " threads" << threads << " launches1 [" << k.mainKernel->kernelName << "]";
        k.variant = v.str();
        return kernels;
    }
    std::ostringstream s;
    s << thor_embed::kDevicePrelude << thor_embed::kScanKernels;
    writeScanTraits(s, r, isUnsigned, threads, vec, items, chunkElems, k);

    // Blocks of 1 024 threads whose chunks wait for each other: two of them fit a compute unit only within 64 vector registers.  The
    // head-aware value scans take about 93 and then run one block per compute unit, with nothing to cover a block's wait; asked
    // for eight wavefronts per SIMD the compiler spills a few registers instead (ragged running sum of 2^26 fp32: 137 -> 126 us;
    // kernels that fit anyway are unchanged).  Arg scans hold twice the state and are left alone, and with smaller blocks the
    // bound costs more than it gives (512 threads: 137 -> 209 us).  THOR_SCAN_MIN_WAVES=<n> asks for n, 0 for no bound.
    int minWaves = k.lookback && threads == 1024 && !r.writeIndex ? 8 : 0;
    if (const char* env = std::getenv("THOR_SCAN_MIN_WAVES")) minWaves = std::atoi(env);
    s << "extern \"C\" __global__ __launch_bounds__(" << threads << (minWaves > 0 ? ", " + std::to_string(minWaves) : std::string())
      << ") void thor_scan_main(const gen::Cfg::T* in, const thor::u32* heads, const void* carries, "
         "gen::Cfg::T* outValue, thor::u32* outIndex) {\n    thor::scanChunk<gen::Cfg, false>(in, heads, carries, nullptr, outValue, outIndex);\n}\n";
    if (k.carry && !k.lookback) {
        s << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void thor_scan_totals(const gen::Cfg::T* in, const thor::u32* heads, void* totals) {\n"
             "    thor::scanChunk<gen::Cfg, true>(in, heads, nullptr, totals, nullptr, nullptr);\n}\n";
        s << "extern \"C\" __global__ __launch_bounds__(1024) void thor_scan_carries(const void* totals, void* carries) {\n"
             "    thor::scanCarries<gen::Cfg>(totals, carries);\n}\n";
    }
    if (k.clearWords) s << "extern \"C\" __global__ __launch_bounds__(256) void thor_scan_clear(thor::u32* words) { thor::scanClear<gen::Cfg>(words); }\n";
    if (ragged) {
        s << "extern \"C\" __global__ __launch_bounds__(256) void thor_scan_mark_heads(const void* offsets, thor::u32* heads) {\n"
             "    thor::scanMarkHeads<gen::Cfg>(static_cast<const gen::Cfg::OffsetT*>(offsets), heads);\n}\n";
    }
    const std::string source = s.str();
    auto kernel = [&](const char* name) {
        if (!loadedOnly) return compileKernel(source, name, r.deviceNum, /*fastContract=*/false);
        std::shared_ptr<CompiledKernel> loaded = findLoadedKernel(source, name, r.deviceNum, false);
        if (!loaded) {
            throw std::runtime_error(std::string("CUB scan: kernel ") + name +
                                     " of this request is not loaded yet; an ordinary scan of the same dtype, operation, sizes and alignment - made "
                                     "with the same THOR_SCAN_WAIT_LIMIT / THOR_SCAN_THREADS / THOR_SCAN_PASSES in the environment - loads it.");
        }
        return loaded;
    };
    k.mainKernel = kernel("thor_scan_main");
    if (k.carry && !k.lookback) {
        k.totalsKernel = kernel("thor_scan_totals");
        k.carriesKernel = kernel("thor_scan_carries");
    }
    if (k.clearWords) k.clearKernel = kernel("thor_scan_clear");
    if (ragged) k.markKernel = kernel("thor_scan_mark_heads");
    std::ostringstream variant;
    variant << (ragged ? "segments" : r.row == r.total ? "flat" : "rows") << "(chunk=" << chunkElems << ",vec=" << vec << ",items=" << items << ",threads=" << threads
            << ",grid=" << k.chunks << (k.lookback ? ",passes=scan,published_totals" : k.carry ? ",passes=totals+carries+scan" : ",passes=scan") << (r.reverse ? ",reverse" : "") << ") ["
            << k.mainKernel->kernelName << "]";
    k.variant = variant.str();
    return kernels;
}
}  // namespace

void launchScan(const CubScanKernels& k, const void* input, const void* offsets, void* temp, size_t tempBytes, void* outValue, void* outIndex,
                Stream& stream) {
    if (!stream.isInitialized() || stream.getGpuNum() != k.request.deviceNum) throw std::invalid_argument("CUB scan stream must live on the plan's GPU.");
    if (tempBytes < k.tempBytes || (k.tempBytes > 1 && temp == nullptr)) throw std::invalid_argument("CUB scan temporary storage is too small for the plan.");
    ScopedGpu scoped(k.request.deviceNum);
    char* base = static_cast<char*>(temp);
    void* heads = k.headsBytes ? base : nullptr;
    void* totals = k.statesBytes ? base + k.headsBytes : nullptr;
    // with published totals the scan kernel's `carries` argument is the block they live in
    void* carries = k.lookback ? totals : k.statesBytes ? base + k.headsBytes + k.statesBytes : nullptr;
    void* raw = stream.getStream();
    if (k.markKernel && offsets == nullptr) throw std::invalid_argument("CUB segmented scan requires segment offsets.");
    if (k.clearKernel) {
        void* words = base;
        std::vector<void*> clearArgs = {&words};
        k.clearKernel->launch(static_cast<uint32_t>((k.clearWords + 255) / 256), 1, 1, 256, raw, clearArgs);
    }
    if (k.markKernel) {
        std::vector<void*> markArgs = {&offsets, &heads};
        k.markKernel->launch(static_cast<uint32_t>((k.request.segments + 1 + 255) / 256), 1, 1, 256, raw, markArgs);
    }
    if (k.totalsKernel) {
        std::vector<void*> totalsArgs = {&input, &heads, &totals};
        k.totalsKernel->launch(static_cast<uint32_t>(k.chunks), 1, 1, k.threads, raw, totalsArgs);
        std::vector<void*> carriesArgs = {&totals, &carries};
        k.carriesKernel->launch(1, 1, 1, 1024, raw, carriesArgs);
    }
    std::vector<void*> mainArgs = {&input, &heads, &carries, &outValue, &outIndex};
    k.mainKernel->launch(static_cast<uint32_t>(k.chunks), 1, 1, k.threads, raw, mainArgs);
}

namespace {
std::atomic<uint64_t> gWaitsRecovered{0};
}
uint64_t scanWaitsRecoveredTotal() { return gWaitsRecovered.load(); }

uint32_t scanWaitsRecovered(const CubScanKernels& k, const void* temp, Stream& stream) {
    if (!k.lookback || temp == nullptr) return 0;
    ScopedGpu scoped(k.request.deviceNum);
    uint32_t count = 0;
    // the second control word of the block of published totals, which follows the head bitmap
    const char* word = static_cast<const char*>(temp) + k.headsBytes + 8;
    if (thorhip_memcpy_async(&count, word, sizeof count, THORHIP_D2H, stream.getStream()) != 0 || thorhip_stream_synchronize(stream.getStream()) != 0) {
        throw std::runtime_error(std::string("CUB scan: reading the wait counter failed: ") + thorhip_last_error());
    }
    gWaitsRecovered += count;
    return count;
}

bool scanRouteFits(const ScanRequest& request) {
    ScanRequest routed = request;
    routed.route = true;
    return request.total != 0 && request.row != 0 && request.total % request.row == 0 && isCubScanDTypeSupported(request.dtype) &&
           chooseScanChunking(routed).routable;
}

void launchScanRoute(const CubScanKernels& k, const void* input, const void* gradient, void* routed, Stream& stream) {
    if (!k.request.route) throw std::invalid_argument("CUB scan: these kernels do not route a gradient.");
    if (!stream.isInitialized() || stream.getGpuNum() != k.request.deviceNum) throw std::invalid_argument("CUB scan stream must live on the plan's GPU.");
    ScopedGpu scoped(k.request.deviceNum);
    std::vector<void*> args = {&input, &gradient, &routed};
    k.mainKernel->launch(static_cast<uint32_t>(k.chunks), 1, 1, k.threads, stream.getStream(), args);
}

void StampedScan::runOn(Stream& stream) const {
    if (gradient.isInitialized()) {
        launchScanRoute(*kernels, input.getMemPtr(), gradient.getMemPtr(), const_cast<Tensor&>(values).getMemPtr(), stream);
        return;
    }
    launchScan(*kernels, input.getMemPtr(), offsets.has_value() ? offsets->getMemPtr() : nullptr, const_cast<Tensor&>(temp).getMemPtr(),
               temp.getTotalNumElements(), values.isInitialized() ? const_cast<Tensor&>(values).getMemPtr() : nullptr,
               indices.isInitialized() ? const_cast<Tensor&>(indices).getMemPtr() : nullptr, stream);
}
std::string StampedScan::getKernelVariant() const { return kernels->variant; }

std::string cubScanKernelVariant(const std::shared_ptr<const CubScanKernels>& kernels) { return kernels ? kernels->variant : std::string(); }
uint32_t cubScanWaitsRecovered(const std::shared_ptr<const CubScanKernels>& kernels, const Tensor& temp, Stream& stream) {
    if (!kernels || !temp.isInitialized()) return 0;
    return scanWaitsRecovered(*kernels, const_cast<Tensor&>(temp).getMemPtr(), stream);
}

// ---- the reference's plan / run entry points ----------------------------------------------------------------------------------
namespace {

struct Checked {
    ScanRequest request;
    TensorPlacement placement;
};

// shared validation (reference: validateExclusiveSum and the checks of each prepare function)
Checked check(const Tensor& input, const Tensor& output, const Tensor* offsets, uint64_t numItems, uint64_t numSegments, uint64_t segmentSize,
              bool uniform, bool arg) {
    if (!input.isInitialized() || !output.isInitialized()) throw std::invalid_argument("CUB scan requires initialized input and output tensors.");
    if (input.getPlacement().getMemDevice() != TensorPlacement::MemDevices::GPU || input.getPlacement() != output.getPlacement()) {
        throw std::invalid_argument("CUB scan input and output must live on the same GPU.");
    }
    if (!isCubScanDTypeSupported(input.getDataType())) {
        throw std::invalid_argument(std::string("Unsupported CUB scan dtype ") + dataTypeName(input.getDataType()) + ".");
    }
    if (arg ? output.getDataType() != DataType::UINT32 : output.getDataType() != input.getDataType()) {
        throw std::invalid_argument(arg ? "CUB arg scan output must be UINT32." : "CUB scan input and output dtypes must match.");
    }
    if (numItems == 0) throw std::invalid_argument("CUB scan requires at least one element.");
    if (input.getTotalNumElements() < numItems || output.getTotalNumElements() < numItems) {
        throw std::invalid_argument("CUB scan num_items exceeds the input or output tensor.");
    }
    if (!input.isDenseContiguous() || !output.isDenseContiguous()) throw std::invalid_argument("CUB scan requires dense tensors.");
    Checked c;
    c.placement = input.getPlacement();
    ScanRequest& r = c.request;
    r.dtype = input.getDataType();
    r.total = numItems;
    r.deviceNum = static_cast<int>(input.getPlacement().getDeviceNum());
    r.alignmentBytes = std::min(pointerAlignment(input.getMemPtr()), pointerAlignment(output.getMemPtr()));
    if (offsets) {
        if (!offsets->isInitialized() || offsets->getPlacement() != input.getPlacement() || !offsets->isDenseContiguous()) {
            throw std::invalid_argument("CUB segmented scan offsets must be a dense tensor on the input's GPU.");
        }
        if (!isCubSegmentOffsetDTypeSupported(offsets->getDataType())) throw std::invalid_argument("CUB segmented scan offsets must be UINT32 or UINT64.");
        if (numSegments == 0 || offsets->getTotalNumElements() < numSegments + 1) {
            throw std::invalid_argument("CUB segmented scan offsets must hold num_segments + 1 entries.");
        }
        r.row = 0;
        r.segments = numSegments;
        r.offsets64 = offsets->getDataType() == DataType::UINT64;
    } else if (uniform) {
        if (numSegments == 0 || segmentSize == 0 || numSegments * segmentSize != numItems) {
            throw std::invalid_argument("CUB uniform segmented scan requires num_items == num_segments * segment_size.");
        }
        r.row = segmentSize;
        r.segments = numSegments;
    } else {
        r.row = numItems;
        r.segments = 1;
    }
    return c;
}

void fill(ScanRequest& r, CubScanOp op, CubScanMode mode, CubScanDirection direction) {
    r.op = static_cast<int>(op);
    r.writeValue = true;
    r.writeIndex = false;
    r.inclusive = mode == CubScanMode::Inclusive;
    r.reverse = direction == CubScanDirection::Reverse;
}
void fill(ScanRequest& r, CubArgScanOp op, CubScanMode mode, CubScanDirection direction) {
    r.op = op == CubArgScanOp::ArgMin ? 1 : 2;
    r.writeValue = false;
    r.writeIndex = true;
    r.inclusive = mode == CubScanMode::Inclusive;
    r.reverse = direction == CubScanDirection::Reverse;
}

template <typename Plan>
void run(const Plan& plan, const Tensor& temp, const Tensor& input, Tensor& output, const Tensor* offsets, bool arg, Stream& stream) {
    if (!plan.kernels) throw std::invalid_argument("CUB scan plan was not prepared.");
    if (input.getDataType() != plan.dtype || input.getPlacement() != plan.placement || output.getPlacement() != plan.placement ||
        input.getTotalNumElements() < plan.num_items || output.getTotalNumElements() < plan.num_items) {
        throw std::invalid_argument("CUB scan tensors do not match the plan.");
    }
    if (std::min(pointerAlignment(input.getMemPtr()), pointerAlignment(output.getMemPtr())) < plan.kernels->request.alignmentBytes) {
        throw std::invalid_argument("CUB scan tensors are less aligned than the tensors the plan was prepared for.");
    }
    if (plan.temp_storage_bytes > 1 && (!temp.isInitialized() || temp.getPlacement() != plan.placement ||
                                        temp.getTotalNumElements() * dataTypeSizeInBytes(temp.getDataType()) < plan.temp_storage_bytes)) {
        throw std::invalid_argument("CUB scan temporary storage is too small for the plan.");
    }
    void* tempPtr = temp.isInitialized() ? const_cast<Tensor&>(temp).getMemPtr() : nullptr;
    const size_t tempBytes = temp.isInitialized() ? temp.getTotalNumElements() * dataTypeSizeInBytes(temp.getDataType()) : 1;
    launchScan(*plan.kernels, input.getMemPtr(), offsets ? offsets->getMemPtr() : nullptr, tempPtr, tempBytes, arg ? nullptr : output.getMemPtr(),
               arg ? output.getMemPtr() : nullptr, stream);
}

}  // namespace

std::shared_ptr<const CubScanKernels> scanWithLoadedKernels(const Tensor& input, Tensor& output, const Tensor* offsets, uint64_t numItems,
                                                            uint64_t numSegments, uint64_t segmentSize, int op, bool arg, bool inclusive, bool reverse,
                                                            void* temp, size_t tempCapacityBytes, Stream& stream) {
    if (op < 0 || op > 3 || (arg && op != 1 && op != 2)) throw std::invalid_argument("scan op must be 0..3 (1 or 2 for arg scans)");
    const bool uniform = offsets == nullptr && segmentSize > 0;
    Checked c = check(input, output, offsets, numItems, uniform ? numItems / segmentSize : numSegments, segmentSize, uniform, arg);
    const CubScanMode mode = inclusive ? CubScanMode::Inclusive : CubScanMode::Exclusive;
    const CubScanDirection direction = reverse ? CubScanDirection::Reverse : CubScanDirection::Forward;
    if (arg) {
        fill(c.request, op == 1 ? CubArgScanOp::ArgMin : CubArgScanOp::ArgMax, mode, direction);
    } else {
        fill(c.request, static_cast<CubScanOp>(op), mode, direction);
    }
    std::shared_ptr<const CubScanKernels> kernels = buildScanKernels(c.request, /*loadedOnly=*/true, tempCapacityBytes);
    launchScan(*kernels, input.getMemPtr(), offsets ? offsets->getMemPtr() : nullptr, temp, tempCapacityBytes, arg ? nullptr : output.getMemPtr(),
               arg ? output.getMemPtr() : nullptr, stream);
    return kernels;
}

#define THOR_SCAN_PLAN_COMMON(plan, checked, opValue, modeValue, directionValue) \
    plan.placement = checked.placement;                                          \
    plan.dtype = checked.request.dtype;                                          \
    plan.num_items = numItems;                                                   \
    plan.op = opValue;                                                           \
    plan.mode = modeValue;                                                       \
    plan.direction = directionValue;                                             \
    plan.kernels = buildScanKernels(checked.request);                            \
    plan.temp_storage_bytes = plan.kernels->tempBytes

CubDeviceScanPlan prepareCubDeviceScan(const Tensor& input, const Tensor& output, uint64_t numItems, CubScanOp op, CubScanMode mode,
                                       CubScanDirection direction) {
    Checked c = check(input, output, nullptr, numItems, 1, numItems, false, false);
    fill(c.request, op, mode, direction);
    CubDeviceScanPlan plan;
    THOR_SCAN_PLAN_COMMON(plan, c, op, mode, direction);
    return plan;
}
size_t cubDeviceScanTempBytes(const Tensor& input, const Tensor& output, uint64_t numItems, CubScanOp op, CubScanMode mode, CubScanDirection direction) {
    return prepareCubDeviceScan(input, output, numItems, op, mode, direction).temp_storage_bytes;
}
void cubDeviceScan(const CubDeviceScanPlan& plan, const Tensor& temp, const Tensor& input, Tensor& output, Stream& stream) {
    run(plan, temp, input, output, nullptr, false, stream);
}

CubDeviceArgScanPlan prepareCubDeviceArgScan(const Tensor& input, const Tensor& output, uint64_t numItems, CubArgScanOp op, CubScanMode mode,
                                             CubScanDirection direction) {
    Checked c = check(input, output, nullptr, numItems, 1, numItems, false, true);
    fill(c.request, op, mode, direction);
    CubDeviceArgScanPlan plan;
    THOR_SCAN_PLAN_COMMON(plan, c, op, mode, direction);
    return plan;
}
size_t cubDeviceArgScanTempBytes(const Tensor& input, const Tensor& output, uint64_t numItems, CubArgScanOp op, CubScanMode mode,
                                 CubScanDirection direction) {
    return prepareCubDeviceArgScan(input, output, numItems, op, mode, direction).temp_storage_bytes;
}
void cubDeviceArgScan(const CubDeviceArgScanPlan& plan, const Tensor& temp, const Tensor& input, Tensor& output, Stream& stream) {
    run(plan, temp, input, output, nullptr, true, stream);
}

CubDeviceSegmentedUniformScanPlan prepareCubDeviceSegmentedUniformScan(const Tensor& input, const Tensor& output, uint64_t numItems,
                                                                       uint64_t numSegments, uint64_t segmentSize, CubScanOp op, CubScanMode mode,
                                                                       CubScanDirection direction) {
    Checked c = check(input, output, nullptr, numItems, numSegments, segmentSize, true, false);
    fill(c.request, op, mode, direction);
    CubDeviceSegmentedUniformScanPlan plan;
    THOR_SCAN_PLAN_COMMON(plan, c, op, mode, direction);
    plan.num_segments = numSegments;
    plan.segment_size = segmentSize;
    return plan;
}
size_t cubDeviceSegmentedUniformScanTempBytes(const Tensor& input, const Tensor& output, uint64_t numItems, uint64_t numSegments, uint64_t segmentSize,
                                              CubScanOp op, CubScanMode mode, CubScanDirection direction) {
    return prepareCubDeviceSegmentedUniformScan(input, output, numItems, numSegments, segmentSize, op, mode, direction).temp_storage_bytes;
}
void cubDeviceSegmentedUniformScan(const CubDeviceSegmentedUniformScanPlan& plan, const Tensor& temp, const Tensor& input, Tensor& output,
                                   Stream& stream) {
    run(plan, temp, input, output, nullptr, false, stream);
}

CubDeviceSegmentedUniformArgScanPlan prepareCubDeviceSegmentedUniformArgScan(const Tensor& input, const Tensor& output, uint64_t numItems,
                                                                             uint64_t numSegments, uint64_t segmentSize, CubArgScanOp op,
                                                                             CubScanMode mode, CubScanDirection direction) {
    Checked c = check(input, output, nullptr, numItems, numSegments, segmentSize, true, true);
    fill(c.request, op, mode, direction);
    CubDeviceSegmentedUniformArgScanPlan plan;
    THOR_SCAN_PLAN_COMMON(plan, c, op, mode, direction);
    plan.num_segments = numSegments;
    plan.segment_size = segmentSize;
    return plan;
}
size_t cubDeviceSegmentedUniformArgScanTempBytes(const Tensor& input, const Tensor& output, uint64_t numItems, uint64_t numSegments,
                                                 uint64_t segmentSize, CubArgScanOp op, CubScanMode mode, CubScanDirection direction) {
    return prepareCubDeviceSegmentedUniformArgScan(input, output, numItems, numSegments, segmentSize, op, mode, direction).temp_storage_bytes;
}
void cubDeviceSegmentedUniformArgScan(const CubDeviceSegmentedUniformArgScanPlan& plan, const Tensor& temp, const Tensor& input, Tensor& output,
                                      Stream& stream) {
    run(plan, temp, input, output, nullptr, true, stream);
}

CubDeviceSegmentedScanPlan prepareCubDeviceSegmentedScan(const Tensor& input, const Tensor& output, const Tensor& offsets, uint64_t numItems,
                                                         uint64_t numSegments, CubScanOp op, CubScanMode mode, CubScanDirection direction) {
    Checked c = check(input, output, &offsets, numItems, numSegments, 0, false, false);
    fill(c.request, op, mode, direction);
    CubDeviceSegmentedScanPlan plan;
    THOR_SCAN_PLAN_COMMON(plan, c, op, mode, direction);
    plan.num_segments = numSegments;
    plan.offset_dtype = offsets.getDataType();
    return plan;
}
size_t cubDeviceSegmentedScanTempBytes(const Tensor& input, const Tensor& output, const Tensor& offsets, uint64_t numItems, uint64_t numSegments,
                                       CubScanOp op, CubScanMode mode, CubScanDirection direction) {
    return prepareCubDeviceSegmentedScan(input, output, offsets, numItems, numSegments, op, mode, direction).temp_storage_bytes;
}
void cubDeviceSegmentedScan(const CubDeviceSegmentedScanPlan& plan, const Tensor& temp, const Tensor& input, Tensor& output, const Tensor& offsets,
                            Stream& stream) {
    if (offsets.getDataType() != plan.offset_dtype || offsets.getTotalNumElements() < plan.num_segments + 1) {
        throw std::invalid_argument("CUB segmented scan offsets do not match the plan.");
    }
    run(plan, temp, input, output, &offsets, false, stream);
}

CubDeviceSegmentedArgScanPlan prepareCubDeviceSegmentedArgScan(const Tensor& input, const Tensor& output, const Tensor& offsets, uint64_t numItems,
                                                               uint64_t numSegments, CubArgScanOp op, CubScanMode mode,
                                                               CubScanDirection direction) {
    Checked c = check(input, output, &offsets, numItems, numSegments, 0, false, true);
    fill(c.request, op, mode, direction);
    CubDeviceSegmentedArgScanPlan plan;
    THOR_SCAN_PLAN_COMMON(plan, c, op, mode, direction);
    plan.num_segments = numSegments;
    plan.offset_dtype = offsets.getDataType();
    return plan;
}
size_t cubDeviceSegmentedArgScanTempBytes(const Tensor& input, const Tensor& output, const Tensor& offsets, uint64_t numItems, uint64_t numSegments,
                                          CubArgScanOp op, CubScanMode mode, CubScanDirection direction) {
    return prepareCubDeviceSegmentedArgScan(input, output, offsets, numItems, numSegments, op, mode, direction).temp_storage_bytes;
}
void cubDeviceSegmentedArgScan(const CubDeviceSegmentedArgScanPlan& plan, const Tensor& temp, const Tensor& input, Tensor& output,
                               const Tensor& offsets, Stream& stream) {
    if (offsets.getDataType() != plan.offset_dtype || offsets.getTotalNumElements() < plan.num_segments + 1) {
        throw std::invalid_argument("CUB segmented scan offsets do not match the plan.");
    }
    run(plan, temp, input, output, &offsets, true, stream);
}

}  // namespace ThorImplementation
