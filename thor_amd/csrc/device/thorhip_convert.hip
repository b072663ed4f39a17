// Type-converter kernels for gfx950 and the thorhip_convert entry point.
//
// Replaces TypeConverter::gpuConvertType and its 16 size-specialised kernels
// (Utilities/TensorOperations/DataTypeConversions/TypeConverterKernels.cu:39-823,906-936,965-1338,1340-1433).
//
// Design for MI355X: the conversion is a pure HBM stream (6 B/element for fp32<->16-bit), so each lane moves one
// 16-byte word of the wider type and the matching 8-byte word of the narrower one, with non-temporal hints, one slot per
// lane and as many 512-thread blocks as there are slots.  Measured on MI355X at 2^28 elements this shape (6.2 TB/s in
// both directions; a plain one-word-per-lane copy reaches 6.45 TB/s, a read-only stream 6.9 TB/s) beats 32-byte loads
// with 16-byte stores (6.15 TB/s narrowing, 4.6 TB/s widening), grid-stride loops capped at a few blocks per CU
// (5.3-5.9 TB/s) and cached loads/stores (5.4-5.8 TB/s); the loop
// remains so that a capped grid can be selected with THORHIP_CONVERT_BLOCKS_PER_CU.  A slot is a fixed, index-aligned
// group of VEC elements; slots that straddle the [begin, end) range are handled element-wise, so nothing outside the
// range is touched (the reference kernels over-read and over-write up to 15 elements into the tensor's 128-byte pad).
#include "thorhip.h"
#include "thorhip_internal.h"
#include "thorhip_numeric.h"

#include <cstdlib>
#include <mutex>

namespace {

using namespace thor;

constexpr int kBlockThreads = 512;

template <int BYTES>
struct Word;
template <>
struct Word<1> {
    typedef u8 type;
};
template <>
struct Word<2> {
    typedef u16 type;
};
template <>
struct Word<4> {
    typedef u32 type;
};
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
template <>
struct Word<8> {
    typedef u32x2 type;
};
template <>
struct Word<16> {
    typedef u32x4 type;
};

// Streaming store: written once, never read back by this kernel.  Words of 4 bytes and more are written through every
// cache level (sc0 sc1 = system scope) with the non-temporal hint; narrower words take the compiler's non-temporal store.
// The compiler's hazard checks do not look inside inline assembly: a store of more than 8 bytes still reads its data
// registers for two cycles after it issues, hence the two wait states (s_nop 1) behind the 16-byte form.
template <typename W>
__device__ __forceinline__ void streamStore(W* p, W w) {
    if constexpr (sizeof(W) == 16) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" : : "v"(p), "v"(w) : "memory");
    } else if constexpr (sizeof(W) == 8) {
        asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(w) : "memory");
    } else if constexpr (sizeof(W) == 4) {
        asm volatile("global_store_dword %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(w) : "memory");
    } else {
        __builtin_nontemporal_store(w, p);
    }
}

// The hardware deals consecutive workgroup ids round-robin to the 8 XCDs.  With this renumbering XCD x works on blocks
// [g*128 + x*16, g*128 + x*16 + 16) of every group g of 128 blocks: a contiguous 16-block run per XCD at any moment.  A
// bijection on [0, gridDim.x) when gridDim.x is a multiple of 128; the identity otherwise.
constexpr int kXcds = 8, kXcdRun = 16;
__device__ __forceinline__ long xcdBlock() {
    const long b = blockIdx.x;
    if (gridDim.x % (kXcds * kXcdRun) != 0) return b;
    const long within = b % (kXcds * kXcdRun);
    return b - within + (within % kXcds) * kXcdRun + within / kXcds;
}

// VEC elements of T moved as whole machine words of up to 16 bytes.
template <typename T, int VEC>
struct alignas((sizeof(T) * VEC) >= 16 ? 16 : (sizeof(T) * VEC)) Pack {
    static constexpr int kBytes = sizeof(T) * VEC;
    static constexpr int kWordBytes = kBytes >= 16 ? 16 : kBytes;
    static constexpr int kWords = kBytes / kWordBytes;
    typedef typename Word<kWordBytes>::type word_t;
    T v[VEC];

    __device__ __forceinline__ void load(const T* p) {
        const word_t* wp = reinterpret_cast<const word_t*>(p);
        word_t* mine = reinterpret_cast<word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) mine[w] = __builtin_nontemporal_load(wp + w);
    }
    // The same words at an address that is only aligned to the element (global memory takes any alignment; the access may
    // touch one more cache line).  The store below is an instruction spelled out, which takes any address as well.
    __device__ __forceinline__ void loadElementAligned(const T* p) {
        typedef word_t __attribute__((aligned(alignof(T)))) unaligned_word_t;
        const unaligned_word_t* wp = reinterpret_cast<const unaligned_word_t*>(p);
        word_t* mine = reinterpret_cast<word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) mine[w] = __builtin_nontemporal_load(wp + w);
    }
    __device__ __forceinline__ void store(T* p) const {
        word_t* wp = reinterpret_cast<word_t*>(p);
        const word_t* mine = reinterpret_cast<const word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) streamStore(wp + w, mine[w]);
    }
};

// Elements per slot: one 16-byte word of the wider type per lane (fp32 <-> 16-bit: a 16-byte access on the fp32 side and
// an 8-byte access on the other), never fewer than 4 elements.  Measured on MI355X at 2^28 elements this shape with 512
// threads per block streams fp32 -> fp16 about 3 % faster than 32-byte loads with 16-byte stores.
template <typename From, typename To>
struct Slot {
    static constexpr int kMin = sizeof(From) < sizeof(To) ? sizeof(From) : sizeof(To);
    static constexpr int kMax = sizeof(From) < sizeof(To) ? sizeof(To) : sizeof(From);
    static constexpr int kWide = 16 / kMax;
    static constexpr int kFloor = (16 / kMin) < 4 ? (16 / kMin) : 4;
    static constexpr int kVec = kWide > kFloor ? kWide : kFloor;
};

// Index-aligned slots [firstSlot, lastSlot) cover elements [begin, end).  UNROLL slots are in flight per lane.
template <typename From, typename To, int VEC, int UNROLL, bool WORD_ALIGNED = true>
__global__ __launch_bounds__(kBlockThreads) void convertSlots(const From* src, To* dst, long begin, long end, long firstSlot,
                                                               long lastSlot) {
    const long stride = (long)gridDim.x * kBlockThreads;
    for (long s0 = firstSlot + xcdBlock() * kBlockThreads + threadIdx.x; s0 < lastSlot; s0 += stride * UNROLL) {
        Pack<From, VEC> in[UNROLL];
        bool whole[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const long s = s0 + (long)u * stride;
            const long e0 = s * VEC;
            whole[u] = (s < lastSlot) && (e0 >= begin) && (e0 + VEC <= end);
            if (whole[u]) {
                if (WORD_ALIGNED) in[u].load(src + e0); else in[u].loadElementAligned(src + e0);
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const long s = s0 + (long)u * stride;
            const long e0 = s * VEC;
            if (whole[u]) {
                Pack<To, VEC> out;
#pragma unroll
                for (int k = 0; k < VEC; ++k) out.v[k] = convertElement<To>(in[u].v[k]);
                out.store(dst + e0);
            } else if (s < lastSlot) {
                // ragged first / last slot: element-wise, and read everything before writing so that an in-place
                // conversion between equally sized types stays correct
                From tmp[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    const long e = e0 + k;
                    if (e >= begin && e < end) tmp[k] = src[e];
                }
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    const long e = e0 + k;
                    if (e >= begin && e < end) dst[e] = convertElement<To>(tmp[k]);
                }
            }
        }
    }
}

// Element-wise fallback for buffers whose base address is not even aligned to the element.
template <typename From, typename To>
__global__ __launch_bounds__(kBlockThreads) void convertScalar(const From* src, To* dst, long begin, long end) {
    const long stride = (long)gridDim.x * kBlockThreads;
    for (long e = begin + (long)blockIdx.x * kBlockThreads + threadIdx.x; e < end; e += stride) dst[e] = convertElement<To>(src[e]);
}

// One block converts [0, count) in place between differently sized types: every lane reads all of its elements, the
// block synchronises, then every lane writes.  count is at most kStagedElements.
constexpr int kStagedPerThread = 8;
constexpr int kStagedElements = kBlockThreads * kStagedPerThread;
template <typename From, typename To>
__global__ __launch_bounds__(kBlockThreads) void convertStagedInPlace(const From* src, To* dst, long count) {
    From tmp[kStagedPerThread];
#pragma unroll
    for (int k = 0; k < kStagedPerThread; ++k) {
        const long e = (long)k * kBlockThreads + threadIdx.x;
        if (e < count) tmp[k] = src[e];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kStagedPerThread; ++k) {
        const long e = (long)k * kBlockThreads + threadIdx.x;
        if (e < count) dst[e] = convertElement<To>(tmp[k]);
    }
}

struct LaunchShape {
    int compute_units = 0;
    int blocks_per_cu = 0;
};

LaunchShape& launchShape() {
    static LaunchShape shape;
    static std::once_flag once;
    std::call_once(once, [] {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) {
            shape.compute_units = prop.multiProcessorCount;
        } else {
            (void)hipGetLastError();
            shape.compute_units = 256;
        }
        // 0 = one slot per lane (no cap); a positive value caps the grid at that many 256-thread blocks per CU.
        shape.blocks_per_cu = 0;
        if (const char* env = std::getenv("THORHIP_CONVERT_BLOCKS_PER_CU")) {
            const int v = std::atoi(env);
            if (v >= 0 && v <= 4096) shape.blocks_per_cu = v;
        }
    });
    return shape;
}

unsigned gridFor(long work_items, int unroll) {
    const LaunchShape& shape = launchShape();
    const long per_block = (long)kBlockThreads * unroll;
    long blocks = (work_items + per_block - 1) / per_block;
    const long cap = shape.blocks_per_cu > 0 ? (long)shape.compute_units * shape.blocks_per_cu : 0x7fffffffL;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    // whole groups of 128 blocks switch the XCD-aware numbering on; the blocks added find no slot and leave
    if (blocks >= 1024) blocks = (blocks + 127) / 128 * 128;
    return (unsigned)blocks;
}

template <typename T>
bool alignedTo(const T* p, size_t bytes) {
    return (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
}

// Out-of-place (or same-size in-place) conversion of elements [begin, end).
template <typename From, typename To>
int launchRange(const From* src, To* dst, long begin, long end, hipStream_t stream) {
    if (end <= begin) return 0;
    constexpr int VEC = Slot<From, To>::kVec;
    constexpr int UNROLL = 1;
    const size_t src_word = sizeof(From) * VEC >= 16 ? 16 : sizeof(From) * VEC;
    const size_t dst_word = sizeof(To) * VEC >= 16 ? 16 : sizeof(To) * VEC;
    if (alignedTo(src, src_word) && alignedTo(dst, dst_word)) {
        const long firstSlot = begin / VEC;
        const long lastSlot = (end + VEC - 1) / VEC;
        const unsigned grid = gridFor(lastSlot - firstSlot, UNROLL);
        hipLaunchKernelGGL((convertSlots<From, To, VEC, UNROLL>), dim3(grid), dim3(kBlockThreads), 0, stream, src, dst, begin, end,
                           firstSlot, lastSlot);
    } else if (alignedTo(src, sizeof(From)) && alignedTo(dst, sizeof(To))) {
        // Views that begin a few elements into their storage: the slots are counted from the word boundary below the
        // destination, so every store is a whole aligned word and the first and last slots are ragged.  When the source lies
        // the same number of elements past a word boundary it is aligned as well; else its words are read where they lie.
        // (2^27 fp32 -> fp16 one element in: 243 us element by element.)
        const long shift = (long)((reinterpret_cast<uintptr_t>(dst) % dst_word) / sizeof(To));
        const From* shiftedSrc = src - shift;
        To* shiftedDst = dst - shift;
        const long firstSlot = (begin + shift) / VEC;
        const long lastSlot = (end + shift + VEC - 1) / VEC;
        const unsigned grid = gridFor(lastSlot - firstSlot, UNROLL);
        if (alignedTo(shiftedSrc, src_word)) {
            hipLaunchKernelGGL((convertSlots<From, To, VEC, UNROLL, true>), dim3(grid), dim3(kBlockThreads), 0, stream, shiftedSrc, shiftedDst,
                               begin + shift, end + shift, firstSlot, lastSlot);
        } else {
            hipLaunchKernelGGL((convertSlots<From, To, VEC, UNROLL, false>), dim3(grid), dim3(kBlockThreads), 0, stream, shiftedSrc, shiftedDst,
                               begin + shift, end + shift, firstSlot, lastSlot);
        }
    } else {
        const unsigned grid = gridFor(end - begin, 1);
        hipLaunchKernelGGL((convertScalar<From, To>), dim3(grid), dim3(kBlockThreads), 0, stream, src, dst, begin, end);
    }
    THORHIP_TRY(hipGetLastError());
    return 0;
}

// In-place conversion between differently sized types.  Element i's destination bytes overlap the source bytes of other
// elements, so the range is cut into launches whose destination span is disjoint from their own source span; stream
// order between launches does the rest.  Narrowing walks upward from a staged first chunk with spans growing by the
// size ratio; widening walks downward and finishes with the staged chunk
// (TypeConverterKernels.cu:826-904,939-962 use the same geometric schedule).
template <typename From, typename To>
int launchInPlace(const From* src, To* dst, long n, hipStream_t stream) {
    constexpr long ss = sizeof(From), ds = sizeof(To);
    if (ds < ss) {
        long done = n < kStagedElements ? n : kStagedElements;
        hipLaunchKernelGGL((convertStagedInPlace<From, To>), dim3(1), dim3(kBlockThreads), 0, stream, src, dst, done);
        THORHIP_TRY(hipGetLastError());
        while (done < n) {
            // [done, next): destination bytes end at next*ds <= done*ss, the start of this launch's source bytes
            long next = done * ss / ds;
            if (next > n) next = n;
            if (int rc = launchRange<From, To>(src, dst, done, next, stream)) return rc;
            done = next;
        }
    } else {
        long top = n;
        while (top > kStagedElements) {
            // [low, top): destination bytes start at low*ds >= top*ss, the end of this launch's source bytes
            long low = (top * ss + ds - 1) / ds;
            if (low < kStagedElements) low = kStagedElements;  // a later start keeps the spans disjoint
            if (int rc = launchRange<From, To>(src, dst, low, top, stream)) return rc;
            top = low;
        }
        hipLaunchKernelGGL((convertStagedInPlace<From, To>), dim3(1), dim3(kBlockThreads), 0, stream, src, dst, top);
        THORHIP_TRY(hipGetLastError());
    }
    return 0;
}

template <typename From, typename To>
int convertPair(const void* src_v, void* dst_v, long n, hipStream_t stream) {
    const From* src = static_cast<const From*>(src_v);
    To* dst = static_cast<To*>(dst_v);
    if (src_v == dst_v) {
        if (sizeof(From) == sizeof(To)) return launchRange<From, To>(src, dst, 0, n, stream);
        return launchInPlace<From, To>(src, dst, n, stream);
    }
    const char* sb = static_cast<const char*>(src_v);
    const char* se = sb + n * (long)sizeof(From);
    const char* db = static_cast<const char*>(dst_v);
    const char* de = db + n * (long)sizeof(To);
    if (sb < de && db < se) {
        return thorhip::fail(-1, "thorhip_convert: source and destination overlap without being the same buffer");
    }
    return launchRange<From, To>(src, dst, 0, n, stream);
}

template <typename From>
int dispatchDst(const void* src, void* dst, int dst_dtype, long n, hipStream_t stream) {
    switch (dst_dtype) {
        case THORHIP_FP16:
            return convertPair<From, f16>(src, dst, n, stream);
        case THORHIP_BF16:
            return convertPair<From, bf16>(src, dst, n, stream);
        case THORHIP_FP8_E4M3:
            return convertPair<From, e4m3>(src, dst, n, stream);
        case THORHIP_FP8_E5M2:
            return convertPair<From, e5m2>(src, dst, n, stream);
        case THORHIP_FP32:
            return convertPair<From, float>(src, dst, n, stream);
        case THORHIP_FP64:
            return convertPair<From, double>(src, dst, n, stream);
        case THORHIP_INT8:
            return convertPair<From, i8>(src, dst, n, stream);
        case THORHIP_INT16:
            return convertPair<From, i16>(src, dst, n, stream);
        case THORHIP_INT32:
            return convertPair<From, i32>(src, dst, n, stream);
        case THORHIP_INT64:
            return convertPair<From, i64>(src, dst, n, stream);
        case THORHIP_UINT8:
            return convertPair<From, u8>(src, dst, n, stream);
        case THORHIP_UINT16:
            return convertPair<From, u16>(src, dst, n, stream);
        case THORHIP_UINT32:
            return convertPair<From, u32>(src, dst, n, stream);
        case THORHIP_UINT64:
            return convertPair<From, u64>(src, dst, n, stream);
        case THORHIP_BOOLEAN:
            return convertPair<From, boolean>(src, dst, n, stream);
        default:
            return thorhip::fail(-1, "thorhip_convert: unknown destination dtype %d", dst_dtype);
    }
}

}  // namespace

extern "C" {

int thorhip_dtype_size(int dtype) {
    switch (dtype) {
        case THORHIP_FP8_E4M3:
        case THORHIP_FP8_E5M2:
        case THORHIP_INT8:
        case THORHIP_UINT8:
        case THORHIP_BOOLEAN:
            return 1;
        case THORHIP_FP16:
        case THORHIP_BF16:
        case THORHIP_INT16:
        case THORHIP_UINT16:
            return 2;
        case THORHIP_FP32:
        case THORHIP_INT32:
        case THORHIP_UINT32:
            return 4;
        case THORHIP_FP64:
        case THORHIP_INT64:
        case THORHIP_UINT64:
            return 8;
        default:
            return -1;
    }
}

int thorhip_convert(const void* src, void* dst, int src_dtype, int dst_dtype, int64_t num_elements, void* stream_v) {
    THORHIP_REQUIRE(num_elements >= 0, "thorhip_convert: negative element count %lld", (long long)num_elements);
    THORHIP_REQUIRE(src_dtype != dst_dtype, "thorhip_convert: source and destination dtype are both %d", src_dtype);
    THORHIP_REQUIRE(thorhip_dtype_size(src_dtype) > 0, "thorhip_convert: unknown source dtype %d", src_dtype);
    THORHIP_REQUIRE(thorhip_dtype_size(dst_dtype) > 0, "thorhip_convert: unknown destination dtype %d", dst_dtype);
    if (num_elements == 0) return 0;
    THORHIP_REQUIRE(src != nullptr && dst != nullptr, "thorhip_convert: NULL buffer");
    hipStream_t stream = (hipStream_t)stream_v;
    const long n = (long)num_elements;
    switch (src_dtype) {
        case THORHIP_FP16:
            return dispatchDst<f16>(src, dst, dst_dtype, n, stream);
        case THORHIP_BF16:
            return dispatchDst<bf16>(src, dst, dst_dtype, n, stream);
        case THORHIP_FP8_E4M3:
            return dispatchDst<e4m3>(src, dst, dst_dtype, n, stream);
        case THORHIP_FP8_E5M2:
            return dispatchDst<e5m2>(src, dst, dst_dtype, n, stream);
        case THORHIP_FP32:
            return dispatchDst<float>(src, dst, dst_dtype, n, stream);
        case THORHIP_FP64:
            return dispatchDst<double>(src, dst, dst_dtype, n, stream);
        case THORHIP_INT8:
            return dispatchDst<i8>(src, dst, dst_dtype, n, stream);
        case THORHIP_INT16:
            return dispatchDst<i16>(src, dst, dst_dtype, n, stream);
        case THORHIP_INT32:
            return dispatchDst<i32>(src, dst, dst_dtype, n, stream);
        case THORHIP_INT64:
            return dispatchDst<i64>(src, dst, dst_dtype, n, stream);
        case THORHIP_UINT8:
            return dispatchDst<u8>(src, dst, dst_dtype, n, stream);
        case THORHIP_UINT16:
            return dispatchDst<u16>(src, dst, dst_dtype, n, stream);
        case THORHIP_UINT32:
            return dispatchDst<u32>(src, dst, dst_dtype, n, stream);
        case THORHIP_UINT64:
            return dispatchDst<u64>(src, dst, dst_dtype, n, stream);
        case THORHIP_BOOLEAN:
            return dispatchDst<boolean>(src, dst, dst_dtype, n, stream);
        default:
            return thorhip::fail(-1, "thorhip_convert: unknown source dtype %d", src_dtype);
    }
}

}  // extern "C"
