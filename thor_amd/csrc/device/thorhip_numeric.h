// Storage-type tags and scalar conversions for gfx950 device code.
//
// The same text is compiled by hipcc into the library (type converter kernels) and handed to hipRTC in front of every
// generated expression / reduction kernel, so both families round identically.  It therefore may only use what both
// compilers provide without includes: builtins, _Float16 and plain integer arithmetic.
//
// Conversion rules restate `static_cast<To>(From)` of the reference's storage types
// (Utilities/TensorOperations/DataTypeConversions/TypeConverterKernels.cu:23-37,
//  Utilities/Common/LowPrecisionFloat.h:17-79): narrowing to fp16/bf16 is one round-to-nearest-even step with +-Inf on
// overflow and gradual underflow, NaN becomes the canonical 0x7fff; narrowing to fp8 saturates to the largest finite
// value (448 for e4m3, 57344 for e5m2); widening is exact.
#pragma once

namespace thor {

typedef unsigned char u8;
typedef unsigned short u16;
typedef unsigned int u32;
typedef unsigned long long u64;
typedef signed char i8;
typedef short i16;
typedef int i32;
typedef long long i64;

struct f16 {
    u16 bits;
};
struct bf16 {
    u16 bits;
};
struct e4m3 {
    u8 bits;
};
struct e5m2 {
    u8 bits;
};
struct boolean {
    u8 bits;
};

__device__ __forceinline__ u32 f32Bits(float x) { return __builtin_bit_cast(u32, x); }
__device__ __forceinline__ float bitsF32(u32 x) { return __builtin_bit_cast(float, x); }

// ---- widening (exact) ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float toFloat(float x) { return x; }
__device__ __forceinline__ float toFloat(f16 h) {
    // v_cvt_f32_f16 is exact for numbers; a NaN operand is replaced by the canonical quiet NaN.
    const float f = (float)__builtin_bit_cast(_Float16, h.bits);
    return ((h.bits & 0x7fffu) > 0x7c00u) ? bitsF32(0x7fffffffu) : f;
}
__device__ __forceinline__ float toFloat(bf16 h) { return bitsF32(((u32)h.bits) << 16); }
__device__ __forceinline__ float toFloat(e5m2 v) {
    // e5m2 is the top byte of an fp16 pattern
    const u16 hb = (u16)(((u32)v.bits) << 8);
    return (float)__builtin_bit_cast(_Float16, hb);
}
__device__ __forceinline__ float toFloat(e4m3 v) {
    const u32 mag = v.bits & 0x7fu;
    const u32 sign = ((u32)(v.bits & 0x80u)) << 24;
    if (mag == 0x7fu) return bitsF32(sign | 0x7fc00000u);
    const u32 e = mag >> 3, m = mag & 7u;
    float r;
    if (e == 0) {
        r = (float)m * 0.001953125f;  // m * 2^-9
    } else {
        r = bitsF32(((e + 120u) << 23) | (m << 20));
    }
    return bitsF32(f32Bits(r) | sign);
}

// ---- narrowing from fp32 (single RNE step) ----------------------------------------------------------------------------
__device__ __forceinline__ f16 toF16(float x) {
    // v_cvt_f16_f32: round-to-nearest-even, Inf on overflow, gradual underflow (fp16 denormals are always enabled).
    const u16 b = __builtin_bit_cast(u16, (_Float16)x);
    f16 r;
    r.bits = (x != x) ? (u16)0x7fffu : b;
    return r;
}

// v_cvt_pk_bf16_f32 (what the compiler selects for a float -> __bf16 truncation on gfx950): round-to-nearest-even with
// gradual underflow, equal to the integer formula (b + 0x7fff + ((b >> 16) & 1)) >> 16 on every one of the 2^32 - 2^24
// inputs that are not NaN; a NaN comes out as a quiet NaN that keeps its sign and upper payload.
__device__ __forceinline__ u16 bf16BitsRne(float x) { return __builtin_bit_cast(u16, (__bf16)x); }

__device__ __forceinline__ bf16 toBf16(float x) {
    bf16 r;
    r.bits = (x != x) ? (u16)0x7fffu : bf16BitsRne(x);
    return r;
}

// Generic small-format encoder on the magnitude bits of a finite, non-NaN fp32.  EBITS/MBITS/BIAS describe the target;
// MAXCODE is the largest finite code (values that round above it saturate to it).
template <int MBITS, int BIAS, u32 MAXCODE>
__device__ __forceinline__ u32 encodeSmallFloat(u32 abits) {
    // abits: fp32 magnitude bits, finite
    const int e = (int)(abits >> 23);
    const u32 m = abits & 0x7fffffu;
    const int emin = 1 - BIAS;          // smallest normal exponent of the target
    const int E = e - 127;              // unbiased fp32 exponent (e == 0 handled below: far below target range)
    if (e == 0) return 0u;              // fp32 subnormals are < 2^-126, far below half the smallest target subnormal
    u32 sig = m | 0x800000u;            // 24-bit significand, value = sig * 2^(E-23)
    int shift = 23 - MBITS;
    u32 base;
    if (E < emin) {
        shift += emin - E;
        base = 0u;
        if (shift > 25) return 0u;      // below half of the smallest subnormal (sig < 2^24)
    } else {
        base = ((u32)(E + BIAS - 1)) << MBITS;
    }
    const u32 q = sig >> shift;
    const u32 rem = sig & ((1u << shift) - 1u);
    const u32 half = 1u << (shift - 1);
    const u32 up = (rem > half || (rem == half && (q & 1u))) ? 1u : 0u;
    const u32 enc = base + q + up;
    return enc > MAXCODE ? MAXCODE : enc;
}

__device__ __forceinline__ e4m3 toE4m3(float x) {
    const u32 b = f32Bits(x);
    const u32 sign = (b >> 24) & 0x80u;
    const u32 ab = b & 0x7fffffffu;
    u32 code;
    if (ab > 0x7f800000u) {
        code = 0x7fu;
    } else if (ab >= 0x43e80000u) {  // >= 464: everything from the 448/480 midpoint upward, Inf included, saturates
        code = 0x7eu;
    } else {
        code = encodeSmallFloat<3, 7, 0x7eu>(ab);
    }
    e4m3 r;
    r.bits = (u8)(sign | code);
    return r;
}

__device__ __forceinline__ e5m2 toE5m2(float x) {
    const u32 b = f32Bits(x);
    const u32 sign = (b >> 24) & 0x80u;
    const u32 ab = b & 0x7fffffffu;
    u32 code;
    if (ab > 0x7f800000u) {
        code = 0x7fu;
    } else if (ab >= 0x47800000u) {  // >= 65536 (Inf included): saturate without touching the exponent arithmetic
        code = 0x7bu;
    } else {
        code = encodeSmallFloat<2, 15, 0x7bu>(ab);
    }
    e5m2 r;
    r.bits = (u8)(sign | code);
    return r;
}

// ---- sticky (round-to-odd) fp32 images of wider sources --------------------------------------------------------------
// Rounding a wider value first to fp32 with round-to-odd and then to an <= 11-bit significand with RNE gives the same
// result as one direct RNE step, which is what __double2half / __int2bfloat16_rn and friends specify.
__device__ __forceinline__ float f64ToF32RoundOdd(double d) {
    const float f = (float)d;
    if (!(d == d) || (double)f == d) return f;
    u32 b = f32Bits(f);
    const float af = __builtin_fabsf(f);
    const double ad = __builtin_fabs(d);
    if ((double)af > ad) b -= 1u;  // step the magnitude back to the truncated neighbour (also turns Inf into FLT_MAX)
    return bitsF32(b | 1u);
}

// The value, unknown to the optimiser: keeps it from widening the conversion of a 32-bit half back into the conversion of the
// 64-bit integer the half was taken from (whose expansion shifts 64 bits by a register amount, see below).
__device__ __forceinline__ u32 opaque(u32 x) {
    asm("" : "+v"(x));  // not volatile: a conversion whose result is unused still disappears
    return x;
}

__device__ __forceinline__ float u64ToF32RoundOdd(u64 v) {
    if (v < (1ull << 24)) return (float)opaque((u32)v);
    const int lz = __builtin_clzll(v);
    const int shift = 40 - lz;  // bits dropped below a 24-bit significand: 1..40
    // Shifts of 32-bit halves only.  A 64-bit vector shift by an amount held in a register has been measured to go wrong on
    // MI355X when that register is the last one the wavefront owns (one result in ten), and the compiler does not avoid it.
    const u32 lo = (u32)v, hi = (u32)(v >> 32);
    u32 sig, dropped;
    if (shift >= 32) {
        const u32 s = (u32)shift - 32u;
        sig = hi >> s;
        dropped = (hi & ((1u << s) - 1u)) | lo;
    } else {
        sig = (lo >> shift) | (hi << (32 - shift));
        dropped = lo & ((1u << shift) - 1u);
    }
    if (dropped) sig |= 1u;
    const u32 exp = (u32)(127 + 23 + shift);
    return bitsF32((exp << 23) | (sig & 0x7fffffu));
}

// Round-to-nearest-even fp32 of 64-bit integers, as the cast gives it, without the 64-bit shift by a register amount that the
// compiler's own expansion of the cast uses: the halves are normalised with 32-bit shifts, the bits that do not fit 32 become
// a sticky bit, the 32-bit conversion rounds once, and the scaling is exact.
__device__ __forceinline__ float u64ToF32(u64 v) {
    const u32 hi = (u32)(v >> 32), lo = (u32)v;
    if (hi == 0) return (float)opaque(lo);
    const u32 lz = (u32)__builtin_clz(hi);
    const u32 top = lz ? (hi << lz) | (lo >> (32u - lz)) : hi;
    const u32 rest = lo << lz;
    return __builtin_ldexpf((float)(top | (rest ? 1u : 0u)), 32 - (int)lz);
}
__device__ __forceinline__ float i64ToF32(i64 v) { return v < 0 ? -u64ToF32((u64)0 - (u64)v) : u64ToF32((u64)v); }

__device__ __forceinline__ float i64ToF32RoundOdd(i64 v) {
    if (v >= 0) return u64ToF32RoundOdd((u64)v);
    return -u64ToF32RoundOdd((u64)0 - (u64)v);
}

// ---- uniform front end: a carrier value per source class, a store per destination -------------------------------------
template <typename T>
struct Carrier;
template <>
struct Carrier<f16> {
    typedef float type;
};
template <>
struct Carrier<bf16> {
    typedef float type;
};
template <>
struct Carrier<e4m3> {
    typedef float type;
};
template <>
struct Carrier<e5m2> {
    typedef float type;
};
template <>
struct Carrier<float> {
    typedef float type;
};
template <>
struct Carrier<double> {
    typedef double type;
};
template <>
struct Carrier<i8> {
    typedef i32 type;
};
template <>
struct Carrier<i16> {
    typedef i32 type;
};
template <>
struct Carrier<i32> {
    typedef i32 type;
};
template <>
struct Carrier<i64> {
    typedef i64 type;
};
template <>
struct Carrier<u8> {
    typedef u32 type;
};
template <>
struct Carrier<u16> {
    typedef u32 type;
};
template <>
struct Carrier<u32> {
    typedef u32 type;
};
template <>
struct Carrier<u64> {
    typedef u64 type;
};
template <>
struct Carrier<boolean> {
    typedef u32 type;
};

__device__ __forceinline__ float carry(f16 v) { return toFloat(v); }
__device__ __forceinline__ float carry(bf16 v) { return toFloat(v); }
__device__ __forceinline__ float carry(e4m3 v) { return toFloat(v); }
__device__ __forceinline__ float carry(e5m2 v) { return toFloat(v); }
__device__ __forceinline__ float carry(float v) { return v; }
__device__ __forceinline__ double carry(double v) { return v; }
__device__ __forceinline__ i32 carry(i8 v) { return v; }
__device__ __forceinline__ i32 carry(i16 v) { return v; }
__device__ __forceinline__ i32 carry(i32 v) { return v; }
__device__ __forceinline__ i64 carry(i64 v) { return v; }
__device__ __forceinline__ u32 carry(u8 v) { return v; }
__device__ __forceinline__ u32 carry(u16 v) { return v; }
__device__ __forceinline__ u32 carry(u32 v) { return v; }
__device__ __forceinline__ u64 carry(u64 v) { return v; }
__device__ __forceinline__ u32 carry(boolean v) { return v.bits ? 1u : 0u; }

// fp32 image whose RNE narrowing equals the direct narrowing of the carrier value
__device__ __forceinline__ float narrowImage(float v) { return v; }
__device__ __forceinline__ float narrowImage(double v) { return f64ToF32RoundOdd(v); }
__device__ __forceinline__ float narrowImage(i32 v) { return f64ToF32RoundOdd((double)v); }
__device__ __forceinline__ float narrowImage(u32 v) { return f64ToF32RoundOdd((double)v); }
__device__ __forceinline__ float narrowImage(i64 v) { return i64ToF32RoundOdd(v); }
__device__ __forceinline__ float narrowImage(u64 v) { return u64ToF32RoundOdd(v); }

template <typename To>
struct Store;
template <>
struct Store<f16> {
    template <typename C>
    __device__ __forceinline__ static f16 from(C v) {
        return toF16(narrowImage(v));
    }
};
template <>
struct Store<bf16> {
    template <typename C>
    __device__ __forceinline__ static bf16 from(C v) {
        return toBf16(narrowImage(v));
    }
};
template <>
struct Store<e4m3> {
    template <typename C>
    __device__ __forceinline__ static e4m3 from(C v) {
        return toE4m3(narrowImage(v));
    }
};
template <>
struct Store<e5m2> {
    template <typename C>
    __device__ __forceinline__ static e5m2 from(C v) {
        return toE5m2(narrowImage(v));
    }
};
template <>
struct Store<boolean> {
    template <typename C>
    __device__ __forceinline__ static boolean from(C v) {
        boolean r;
        r.bits = (v != (C)0) ? 1 : 0;
        return r;
    }
};
#define THOR_PLAIN_STORE(T)                                    \
    template <>                                                \
    struct Store<T> {                                          \
        template <typename C>                                  \
        __device__ __forceinline__ static T from(C v) {        \
            return (T)v;                                       \
        }                                                      \
    };
template <>
struct Store<float> {
    template <typename C>
    __device__ __forceinline__ static float from(C v) {
        return (float)v;
    }
    __device__ __forceinline__ static float from(u64 v) { return u64ToF32(v); }
    __device__ __forceinline__ static float from(i64 v) { return i64ToF32(v); }
};
THOR_PLAIN_STORE(double)
THOR_PLAIN_STORE(i8)
THOR_PLAIN_STORE(i16)
THOR_PLAIN_STORE(i32)
THOR_PLAIN_STORE(i64)
THOR_PLAIN_STORE(u8)
THOR_PLAIN_STORE(u16)
THOR_PLAIN_STORE(u32)
THOR_PLAIN_STORE(u64)
#undef THOR_PLAIN_STORE

template <typename To, typename From>
__device__ __forceinline__ To convertElement(From v) {
    return Store<To>::from(carry(v));
}

}  // namespace thor
