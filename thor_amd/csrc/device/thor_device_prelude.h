// Device-side building blocks shared by every run-time compiled kernel (placed after thorhip_numeric.h).
//
// wave64 throughout: a wavefront is 64 lanes, a 256-thread block is 4 wavefronts.  Reductions keep fp32 accumulators in
// registers, fold lanes with cross-lane shuffles, fold wavefronts through a few words of LDS, and fold blocks through
// a per-launch partials buffer that a small second launch folds -- no atomics, bit-reproducible for a fixed shape.
#pragma once

namespace thor {

typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// v >> s for s < 32 from shifts of the 32-bit halves.  A 64-bit vector shift by an amount held in a register has been measured
// to go wrong on MI355X when that register is the last one the wavefront owns (one result in ten), and the compiler does not
// avoid that placement, so device code here has no such shift: lane masks are counted with mbcnt, the rest goes through this.
__device__ __forceinline__ u64 shiftRightBelow32(u64 v, u32 s) {
    const u32 lo = (u32)v, hi = (u32)(v >> 32);
    const u32 mixed = s ? (lo >> s) | (hi << (32u - s)) : lo;
    return ((u64)(hi >> s) << 32) | mixed;
}

// ---- machine-word loads / stores of VEC elements --------------------------------------------------------------------
template <int BYTES>
struct WordOf;
template <>
struct WordOf<1> {
    typedef u8 type;
};
template <>
struct WordOf<2> {
    typedef u16 type;
};
template <>
struct WordOf<4> {
    typedef u32 type;
};
template <>
struct WordOf<8> {
    typedef u32x2 type;
};
template <>
struct WordOf<16> {
    typedef u32x4 type;
};

// A word that is written once and not read again by the kernel: written through every cache level (sc0 sc1 = system
// scope) with the non-temporal hint.  The per-XCD L2 then holds no dirty lines that it has to evict in bursts between
// the reads; measured on MI355X against the plain non-temporal store: fp32 -> fp16 streams 6.3 -> 6.55 TB/s, 2-byte in /
// 2-byte out 6.47 -> 6.62 TB/s, write-only 6.7 -> 6.95 TB/s, copies and 4-in / 1-out streams unchanged.  Words narrower
// than 4 bytes take the compiler's non-temporal store.
// The stores are inline assembly because the compiler offers no spelling for the scope bits of a plain store, and the
// compiler's hazard checks do not look inside assembly: a store of more than 8 bytes reads its data registers for two
// more cycles after it issues, so the 16-byte form is followed by two wait states (s_nop 1) before anything may
// overwrite them.  (Without them, a kernel with two stores in a row wrote stale registers now and then.)
template <typename W>
__device__ __forceinline__ void streamStoreWord(W* p, W w) {
#ifdef THOR_PLAIN_STREAM_STORES
    __builtin_nontemporal_store(w, p);
#else
    if constexpr (sizeof(W) == 16) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" : : "v"(p), "v"(w) : "memory");
    } else if constexpr (sizeof(W) == 8) {
        asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(w) : "memory");
    } else if constexpr (sizeof(W) == 4) {
        asm volatile("global_store_dword %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(w) : "memory");
    } else {
        __builtin_nontemporal_store(w, p);
    }
#endif
}

// Workgroup ids are dealt round-robin to the 8 XCDs (each with an L2 and a fabric port of its own).  With this numbering
// XCD x works on blocks [g * 8 * RUN + x * RUN, ... + RUN) of every group g of 8 * RUN blocks, a run of RUN adjacent
// blocks at any moment instead of every eighth block.  A bijection on [0, grid) when grid is a multiple of 8 * RUN, the
// identity otherwise (and for RUN <= 1).
template <int RUN>
__device__ __forceinline__ u32 xcdBlock(u32 block, u32 grid) {
    if (RUN <= 1 || grid % (8u * RUN) != 0) return block;
    const u32 within = block % (8u * RUN);
    return block - within + (within % 8u) * RUN + within / 8u;
}

template <typename T, int VEC>
struct alignas((sizeof(T) * VEC) >= 16 ? 16 : (sizeof(T) * VEC)) Pack {
    static constexpr int kBytes = sizeof(T) * VEC;
    static constexpr int kWordBytes = kBytes >= 16 ? 16 : kBytes;
    static constexpr int kWords = kBytes / kWordBytes;
    typedef typename WordOf<kWordBytes>::type word_t;
    T v[VEC];

    // streaming (non-temporal) access: data that is touched once should not displace reusable lines
    __device__ __forceinline__ void loadStream(const T* p) {
        const word_t* wp = reinterpret_cast<const word_t*>(p);
        word_t* mine = reinterpret_cast<word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) mine[w] = __builtin_nontemporal_load(wp + w);
    }
    // the same for an address that is only aligned to the element: one access of the same width (global memory takes any
    // alignment), which may touch a second cache line
    __device__ __forceinline__ void loadStreamUnaligned(const T* p) {
        typedef word_t __attribute__((aligned(alignof(T)))) unaligned_word_t;
        const unaligned_word_t* wp = reinterpret_cast<const unaligned_word_t*>(p);
        word_t* mine = reinterpret_cast<word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) mine[w] = __builtin_nontemporal_load(wp + w);
    }
    __device__ __forceinline__ void loadUnaligned(const T* p) {
        typedef word_t __attribute__((aligned(alignof(T)))) unaligned_word_t;
        const unaligned_word_t* wp = reinterpret_cast<const unaligned_word_t*>(p);
        word_t* mine = reinterpret_cast<word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) mine[w] = wp[w];
    }
    __device__ __forceinline__ void load(const T* p) {
        const word_t* wp = reinterpret_cast<const word_t*>(p);
        word_t* mine = reinterpret_cast<word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) mine[w] = wp[w];
    }
    __device__ __forceinline__ void storeStream(T* p) const {
        word_t* wp = reinterpret_cast<word_t*>(p);
        const word_t* mine = reinterpret_cast<const word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) streamStoreWord(wp + w, mine[w]);
    }
    __device__ __forceinline__ void store(T* p) const {
        word_t* wp = reinterpret_cast<word_t*>(p);
        const word_t* mine = reinterpret_cast<const word_t*>(v);
#pragma unroll
        for (int w = 0; w < kWords; ++w) wp[w] = mine[w];
    }
};

// ---- fp32 -> storage ---------------------------------------------------------------------------------------------------
template <typename To>
__device__ __forceinline__ To fromFloat(float x) {
    return Store<To>::from(x);
}
__device__ __forceinline__ float toFloat(boolean v) { return v.bits ? 1.0f : 0.0f; }
__device__ __forceinline__ float toFloat(u8 v) { return (float)v; }
__device__ __forceinline__ float toFloat(i8 v) { return (float)v; }
__device__ __forceinline__ float toFloat(u16 v) { return (float)v; }
__device__ __forceinline__ float toFloat(i16 v) { return (float)v; }
__device__ __forceinline__ float toFloat(u32 v) { return (float)v; }
__device__ __forceinline__ float toFloat(i32 v) { return (float)v; }
__device__ __forceinline__ float toFloat(u64 v) { return u64ToF32(v); }
__device__ __forceinline__ float toFloat(i64 v) { return i64ToF32(v); }

// fp16 values are held in native _Float16 registers inside fused kernels
__device__ __forceinline__ _Float16 asHalf(f16 h) { return __builtin_bit_cast(_Float16, h.bits); }
// fp32 -> fp16 value (round to nearest even, the hardware conversion), spelled as the instruction itself.  A plain
// `(_Float16)x` lets the vectoriser pair two conversions that feed packed fp16 arithmetic into a <2 x float> truncation,
// which this compiler cannot select once packed fp32 operations are switched off (it aborts: "Cannot select: v2f32 =
// bitcast", seen for x - ln(y) over fp16 vectors); the instruction keeps each conversion scalar and leaves the packed
// fp16 arithmetic around it alone.
__device__ __forceinline__ _Float16 halfFromFloat(float x) {
    _Float16 h;
    asm("v_cvt_f16_f32 %0, %1" : "=v"(h) : "v"(x));
    return h;
}
__device__ __forceinline__ f16 fromHalf(_Float16 h) {
    f16 r;
    r.bits = __builtin_bit_cast(u16, h);
    return r;
}
__device__ __forceinline__ boolean makeBoolean(bool b) {
    boolean r;
    r.bits = b ? 1 : 0;
    return r;
}

// value rounded through a 16-bit / 8-bit float and widened again (how a bf16 / fp8 compute step is modelled in fp32)
// (a NaN stays a NaN of the hardware's choosing here; bf16FromExact writes the canonical one when the value is stored)
__device__ __forceinline__ float roundBf16(float x) { return bitsF32((u32)bf16BitsRne(x) << 16); }
// Storage form of a float that already holds a bf16 value (every bf16-typed value inside a kernel does: loads widen
// exactly and every arithmetic result passes through roundBf16): the upper half of its bits; NaN stays canonical.
__device__ __forceinline__ bf16 bf16FromExact(float x) {
    bf16 r;
    r.bits = (x != x) ? (u16)0x7fffu : (u16)(f32Bits(x) >> 16);
    return r;
}
__device__ __forceinline__ float roundF16(float x) { return toFloat(toF16(x)); }
__device__ __forceinline__ float roundE4m3(float x) { return toFloat(toE4m3(x)); }
__device__ __forceinline__ float roundE5m2(float x) { return toFloat(toE5m2(x)); }

// Division of many values by one divisor that a whole row shares (a row sum, a standard deviation).  The reciprocal is
// taken once; each quotient is then x * r corrected by one fused residual step, with v_div_fixup supplying the IEEE
// results for zeros, infinities, NaNs and exponent overflow / underflow.  The result is within one unit in the last
// place of x / d and equal to it in all but rare cases, for a third of the instructions of a full division; divisors
// whose reciprocal would leave the normal range take the full division.
struct RowDivisor {
    float d, r;
    bool fast;
    __device__ __forceinline__ explicit RowDivisor(float divisor) : d(divisor), r(1.0f / divisor) {
        const float a = __builtin_fabsf(divisor);
        fast = a >= 0x1p-100f && a <= 0x1p100f;
    }
    __device__ __forceinline__ float divide(float x) const {
        if (fast) {
            const float q = x * r;
            const float residual = __builtin_fmaf(-d, q, x);
            return __builtin_amdgcn_div_fixupf(__builtin_fmaf(residual, r, q), d, x);
        }
        return x / d;
    }
};

// ---- reduction operators: fp32 accumulate -----------------------------------------------------------------------------
// Min / Max return the NaN operand when either side is NaN (unlike fminf / fmaxf).
struct SumOp {
    __device__ __forceinline__ static float identity() { return 0.0f; }
    __device__ __forceinline__ static float transform(float x) { return x; }
    __device__ __forceinline__ static float combine(float a, float b) { return a + b; }
};
struct AbsSumOp {
    __device__ __forceinline__ static float identity() { return 0.0f; }
    __device__ __forceinline__ static float transform(float x) { return __builtin_fabsf(x); }
    __device__ __forceinline__ static float combine(float a, float b) { return a + b; }
};
struct SquareSumOp {
    __device__ __forceinline__ static float identity() { return 0.0f; }
    __device__ __forceinline__ static float transform(float x) { return x * x; }
    __device__ __forceinline__ static float combine(float a, float b) { return a + b; }
};
struct ProductOp {
    __device__ __forceinline__ static float identity() { return 1.0f; }
    __device__ __forceinline__ static float transform(float x) { return x; }
    __device__ __forceinline__ static float combine(float a, float b) { return a * b; }
};
struct MinOp {
    __device__ __forceinline__ static float identity() { return __builtin_inff(); }
    __device__ __forceinline__ static float transform(float x) { return x; }
    // b replaces a when it is smaller or NaN; a NaN in a stays (no comparison with it holds): two compares and a select
    __device__ __forceinline__ static float combine(float a, float b) { return ((b < a) | (b != b)) ? b : a; }
};
struct MaxOp {
    __device__ __forceinline__ static float identity() { return -__builtin_inff(); }
    __device__ __forceinline__ static float transform(float x) { return x; }
    __device__ __forceinline__ static float combine(float a, float b) { return ((b > a) | (b != b)) ? b : a; }
};

// Partials that travel between blocks of one launch (ticket protocol of the reduction kernels) go through memory words that
// are written and read at device scope: relaxed atomic stores and loads of agent scope, which go past the per-XCD L2 instead
// of leaving a dirty or stale line in it.  (Partials for a finishing launch are plain stores: the launch boundary publishes them.)  A block that has waited for its own stores (partialsWritten) may then announce
// them with an atomic counter, and a reader that has seen the count needs no cache invalidation.
template <typename W>
__device__ __forceinline__ void storeDeviceWide(W* p, W w) {
    __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename W>
__device__ __forceinline__ W loadDeviceWide(const W* p) {
    return __hip_atomic_load(const_cast<W*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Waits until every store this wavefront has issued is acknowledged at the level it was written to.
__device__ __forceinline__ void partialsWritten() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Accumulator protocol used by every reduction kernel:
//   reset(), add(x, index), merge(other), shuffleXor(mask), and the fields a partial is stored as.
template <typename Op>
struct ValueAcc {
    float v;
    __device__ __forceinline__ void reset() { v = Op::identity(); }
    template <typename I>
    __device__ __forceinline__ void add(float x, I) {
        v = Op::combine(v, Op::transform(x));
    }
    __device__ __forceinline__ void merge(const ValueAcc& o) { v = Op::combine(v, o.v); }
    __device__ __forceinline__ ValueAcc shuffleXor(int mask) const {
        ValueAcc r;
        r.v = __shfl_xor(v, mask, kWave);
        return r;
    }
    // A partial of `slots` accumulators is one float array of that length.
    __device__ __forceinline__ static u64 partialBytes(u64 slots) { return ((slots * 4 + 7) / 8) * 8; }
    // DEVICE_WIDE: the partial is read by another block of the same launch (ticket protocol); otherwise by a later launch
    template <bool DEVICE_WIDE = false>
    __device__ __forceinline__ void storePartial(void* partials, u64 slot, u64) const {
        if (DEVICE_WIDE) storeDeviceWide(static_cast<float*>(partials) + slot, v);
        else static_cast<float*>(partials)[slot] = v;
    }
    template <bool DEVICE_WIDE = false>
    __device__ __forceinline__ void loadPartial(const void* partials, u64 slot, u64) {
        v = DEVICE_WIDE ? loadDeviceWide(static_cast<const float*>(partials) + slot) : static_cast<const float*>(partials)[slot];
    }
};

// The two statistics of a softmax in one pass: m = the maximum of the elements seen (NaN wins, like MaxOp) and
// s = the sum of exp(x - m) over them.  A new maximum rescales the sum gathered so far; merging rescales the side with the
// smaller maximum.  One exponential per element: with d = x - m, exp(-|d|) is the factor of the old sum (d > 0) or the new
// term (d <= 0).  Elements equal to -inf add nothing, so an empty accumulator is {-inf, 0}.  (The library's expf on purpose: a
// base-2 hardware exponential with a compensated argument is as accurate and a sixth of the instructions, but measured
// slower in the segment kernel, 574 against 340 us: the compiler overlaps more of them and residency drops to two wavefronts.)
struct OnlineSoftmaxAcc {
    float m, s;
    __device__ __forceinline__ void reset() {
        m = -__builtin_inff();
        s = 0.0f;
    }
    template <typename I>
    __device__ __forceinline__ void add(float x, I) {
        const float d = x - m;
        const float e = x == -__builtin_inff() ? 0.0f : expf(-fabsf(d));  // m == -inf, x finite: d = +inf, e = 0
        const bool rises = (d > 0.0f) | (x != x);
        s = rises ? s * e + 1.0f : s + e;
        m = MaxOp::combine(m, x);
    }
    // N elements at once (-inf marks "no element"): their maximum, then N independent base-2 hardware exponentials of
    // (x - maximum) * log2(e), then one merge.  The difference is formed before the scaling, so an exponent t carries a
    // relative error of 2^-24 and the term 2^t one of |t| * 4e-8 plus the instruction's own ulp: terms far below the
    // maximum are the inexact ones, and x * e^-x <= 1 / e bounds what they add to the sum's error at 2.2e-8 each.
    template <int N>
    __device__ __forceinline__ void addMany(const float (&x)[N]) {
        constexpr float kLog2e = 1.44269504f;
        float top = x[0];
#pragma unroll
        for (int u = 1; u < N; ++u) top = __builtin_fmaxf(top, x[u]);  // ignores NaNs: they come back through the sum
        const float base = top == -__builtin_inff() ? 0.0f : top;      // all -inf: every term is 2^-inf = 0
        float sum = 0.0f;
#pragma unroll
        for (int u = 0; u < N; ++u) sum += __builtin_amdgcn_exp2f((x[u] - base) * kLog2e);
        // a NaN sum: some x was NaN (then the maximum is NaN as well), or the maximum is +inf (inf - inf)
        if (sum != sum && top != __builtin_inff()) top = __builtin_nanf("");
        // merge {top, sum}: both sides rescaled to the common maximum the same way
        const float joint = MaxOp::combine(m, top);
        const float anchor = joint == -__builtin_inff() ? 0.0f : joint;
        s = s * __builtin_amdgcn_exp2f((m - anchor) * kLog2e) + sum * __builtin_amdgcn_exp2f((top - anchor) * kLog2e);
        m = joint;
    }
    __device__ __forceinline__ static float scaleTo(float from, float to) { return from == -__builtin_inff() ? 0.0f : expf(from - to); }
    __device__ __forceinline__ void merge(const OnlineSoftmaxAcc& o) {
        const float top = MaxOp::combine(m, o.m);
        s = s * scaleTo(m, top) + o.s * scaleTo(o.m, top);
        m = top;
    }
    __device__ __forceinline__ OnlineSoftmaxAcc shuffleXor(int mask) const {
        OnlineSoftmaxAcc r;
        r.m = __shfl_xor(m, mask, kWave);
        r.s = __shfl_xor(s, mask, kWave);
        return r;
    }
    // A partial of `slots` accumulators is two float arrays of that length, maxima first.
    __device__ __forceinline__ static u64 partialBytes(u64 slots) { return 2 * (((slots * 4 + 7) / 8) * 8); }
    template <bool DEVICE_WIDE = false>
    __device__ __forceinline__ void storePartial(void* partials, u64 slot, u64 slots) const {
        float* maxima = static_cast<float*>(partials);
        float* sums = reinterpret_cast<float*>(static_cast<char*>(partials) + ((slots * 4 + 7) / 8) * 8);
        if (DEVICE_WIDE) {
            storeDeviceWide(maxima + slot, m);
            storeDeviceWide(sums + slot, s);
        } else {
            maxima[slot] = m;
            sums[slot] = s;
        }
    }
    template <bool DEVICE_WIDE = false>
    __device__ __forceinline__ void loadPartial(const void* partials, u64 slot, u64 slots) {
        const float* maxima = static_cast<const float*>(partials);
        const float* sums = reinterpret_cast<const float*>(static_cast<const char*>(partials) + ((slots * 4 + 7) / 8) * 8);
        m = DEVICE_WIDE ? loadDeviceWide(maxima + slot) : maxima[slot];
        s = DEVICE_WIDE ? loadDeviceWide(sums + slot) : sums[slot];
    }
};

// Candidate {value, index}: NaN beats every number, equal values (and two NaNs) keep the lower index.  The empty
// candidate carries the all-ones index, so any real element wins against it.
template <bool IS_MAX, typename IndexT>
struct ArgAcc {
    float v;
    IndexT i;
    __device__ __forceinline__ void reset() {
        v = IS_MAX ? -__builtin_inff() : __builtin_inff();
        i = ~(IndexT)0;
    }
    __device__ __forceinline__ static bool better(float av, IndexT ai, float bv, IndexT bi) {
        // true when candidate a wins over candidate b.  Spelled without control flow: the lanes of a wavefront rarely agree.
        const bool an = av != av, bn = bv != bv;
        const bool strictA = IS_MAX ? (av > bv) : (av < bv);  // false whenever a NaN is involved
        const bool strictB = IS_MAX ? (bv > av) : (bv < av);
        const bool onlyA = an & !bn, onlyB = bn & !an;
        return onlyA | (!onlyB & (strictA | (!strictB & (ai <= bi))));
    }
    // Adds the next element of one thread's walk.  Every kernel visits its elements in increasing index order, so an
    // equal value never replaces the candidate: only a strictly better value, the first NaN, or the first element at all.
    template <typename I>
    __device__ __forceinline__ void add(float x, I index) {
        // strictly better, or the first NaN: "not (x no better than v)" holds for both, and a NaN that is held stays
        const bool noBetter = IS_MAX ? (x <= v) : (x >= v);
        const bool take = (!noBetter & (v == v)) | (i == ~(IndexT)0);
        v = take ? x : v;  // selects, not branches: lanes of a wavefront rarely agree
        i = take ? (IndexT)index : i;
    }
    __device__ __forceinline__ void merge(const ArgAcc& o) {
        const bool keep = better(v, i, o.v, o.i);
        v = keep ? v : o.v;
        i = keep ? i : o.i;
    }
    __device__ __forceinline__ ArgAcc shuffleXor(int mask) const {
        ArgAcc r;
        r.v = __shfl_xor(v, mask, kWave);
        if (sizeof(IndexT) == 8) {
            const u32 lo = __shfl_xor((u32)((u64)i & 0xffffffffu), mask, kWave);
            const u32 hi = __shfl_xor((u32)((u64)i >> 32), mask, kWave);
            r.i = (IndexT)(((u64)hi << 32) | lo);
        } else {
            r.i = (IndexT)__shfl_xor((u32)i, mask, kWave);
        }
        return r;
    }
    // A partial of `slots` candidates is a float array followed by an IndexT array of the same length.
    __device__ __forceinline__ static u64 partialBytes(u64 slots) { return ((slots * 4 + 7) / 8) * 8 + slots * sizeof(IndexT); }
    template <bool DEVICE_WIDE = false>
    __device__ __forceinline__ void storePartial(void* partials, u64 slot, u64 slots) const {
        float* values = static_cast<float*>(partials);
        IndexT* indices = reinterpret_cast<IndexT*>(static_cast<char*>(partials) + ((slots * 4 + 7) / 8) * 8);
        if (DEVICE_WIDE) {
            storeDeviceWide(values + slot, v);
            storeDeviceWide(indices + slot, i);
        } else {
            values[slot] = v;
            indices[slot] = i;
        }
    }
    template <bool DEVICE_WIDE = false>
    __device__ __forceinline__ void loadPartial(const void* partials, u64 slot, u64 slots) {
        const float* values = static_cast<const float*>(partials);
        const IndexT* indices = reinterpret_cast<const IndexT*>(static_cast<const char*>(partials) + ((slots * 4 + 7) / 8) * 8);
        v = DEVICE_WIDE ? loadDeviceWide(values + slot) : values[slot];
        i = DEVICE_WIDE ? loadDeviceWide(indices + slot) : indices[slot];
    }
};

// Folds the LANES (power of two, <= 64) consecutive lanes that share a result; every lane of the group ends up with it.
template <int LANES, typename Acc>
__device__ __forceinline__ void groupReduce(Acc& acc) {
#pragma unroll
    for (int mask = LANES / 2; mask >= 1; mask >>= 1) acc.merge(acc.shuffleXor(mask));
}

// Folds a whole block of THREADS threads (multiple of 64).  Returns the result in every thread of wavefront 0 (and in
// all threads when BROADCAST is set).  `scratch` must hold THREADS / 64 accumulators in LDS; without BROADCAST there is
// no trailing barrier, so a second fold in the same kernel needs its own scratch.
template <int THREADS, bool BROADCAST, typename Acc>
__device__ __forceinline__ void blockReduce(Acc& acc, Acc* scratch) {
    groupReduce<kWave>(acc);
    if (THREADS > kWave) {
        constexpr int kWaves = THREADS / kWave;
        const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
        if (lane == 0) scratch[wave] = acc;
        __syncthreads();
        if (wave == 0 || BROADCAST) {
            Acc other;
            other.reset();
            if (lane < kWaves) other = scratch[lane];
            groupReduce<kWave>(other);
            acc = other;
        }
        if (BROADCAST) __syncthreads();
    }
}

// ---- result finalisation -----------------------------------------------------------------------------------------------
// FINALIZE: 0 none, 1 divide by `divisor` (mean), 2 square root (L2 norm).  Then the fp32 scale, then one conversion.
template <int FINALIZE>
__device__ __forceinline__ float finalizeValue(float acc, float divisor, float scale) {
    float r = acc;
    if (FINALIZE == 1) r = (divisor == 0.0f) ? 0.0f : ((divisor == 1.0f) ? acc : acc / divisor);
    if (FINALIZE == 2) r = __builtin_sqrtf(acc);
    return r * scale;
}

// digamma(x) in fp32 with the reference's recipe (its emitted helper, Utilities/Expression/CudaSourceEmitter.cpp:679-722):
// poles at the non-positive integers give NaN, x <= 0 is reflected through psi(1-x) - pi/tan(pi x), the argument is
// walked up to x >= 8 with psi(x) = psi(x+1) - 1/x, and the asymptotic series is summed to the 1/x^10 term in the
// same order, so the rounding behaviour matches term for term.
__device__ inline float digammaf(float x) {
    if (x != x) return x;
    if (__builtin_isinf(x)) return x > 0.0f ? x : __builtin_nanf("");
    const float pi = 3.14159265358979323846f;
    float acc = 0.0f;
    if (x <= 0.0f) {
        if (x == floorf(x)) return __builtin_nanf("");
        acc -= pi / tanf(pi * x);
        x = 1.0f - x;
    }
    for (; x < 8.0f; x += 1.0f) acc -= 1.0f / x;
    const float r = 1.0f / x;
    const float r2 = r * r, r4 = r2 * r2;
    const float r6 = r4 * r2, r8 = r4 * r4;
    const float r10 = r8 * r2;
    acc += logf(x) - 0.5f * r;
    acc -= r2 * (1.0f / 12.0f);
    acc += r4 * (1.0f / 120.0f);
    acc -= r6 * (1.0f / 252.0f);
    acc += r8 * (1.0f / 240.0f);
    acc -= r10 * (1.0f / 132.0f);
    return acc;
}

}  // namespace thor
