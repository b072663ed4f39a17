/*
 * CPU oracle for the Thor hot path.  TEST INFRASTRUCTURE ONLY -- see thor_oracle.h for scope and pinning status.
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp; -mf16c only for the exhaustive hardware cross-check)
 */
#include "thor_oracle.h"

#include <math.h>
#include <omp.h>
#include <stdlib.h>
#include <string.h>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

/* ------------------------------------------------------------------------------------------------------------------
 * Generic IEEE-style narrowing.  One rounding step (round-to-nearest, ties-to-even) from an exact binary value
 * sig * 2^exp, which is what `static_cast<half>(float)` / `__float2half_rn` / `__float2bfloat16_rn` /
 * `__nv_cvt_float_to_fp8(..., __NV_SATFINITE, ...)` specify
 * (Utilities/TensorOperations/DataTypeConversions/TypeConverter.cpp:10-22, Utilities/Common/LowPrecisionFloat.h:17-79).
 * ------------------------------------------------------------------------------------------------------------------ */
typedef struct {
    int ebits, mbits, bias;
    int kind; /* 0: IEEE (overflow -> inf), 1: e4m3 saturate-to-finite (no inf, 0x7f NaN), 2: e5m2 saturate-to-finite */
} fmt_t;

static const fmt_t FMT_F16 = {5, 10, 15, 0};
static const fmt_t FMT_BF16 = {8, 7, 127, 0};
static const fmt_t FMT_E4M3 = {4, 3, 7, 1};
static const fmt_t FMT_E5M2 = {5, 2, 15, 2};

static uint32_t fmt_sign_bit(const fmt_t* f) { return 1u << (f->ebits + f->mbits); }
static uint32_t fmt_inf(const fmt_t* f) { return ((1u << f->ebits) - 1u) << f->mbits; }

static uint32_t fmt_overflow(const fmt_t* f) {
    if (f->kind == 0) return fmt_inf(f);
    if (f->kind == 1) return 0x7e; /* 448 */
    return 0x7b;                   /* 57344 */
}

static uint32_t fmt_nan(const fmt_t* f) {
    if (f->kind == 0) return fmt_inf(f) | ((1u << f->mbits) - 1u); /* 0x7fff for fp16 and bf16 */
    return 0x7f;
}

/* magnitude only; sig != 0 */
static uint32_t round_mag(uint64_t sig, int exp, const fmt_t* f) {
    int lz = __builtin_clzll(sig);
    sig <<= lz;
    exp -= lz;
    const int E = exp + 63; /* value in [2^E, 2^(E+1)) */
    const int emin = 1 - f->bias;
    const int emax_field = (1 << f->ebits) - 1;
    if (E + f->bias > emax_field + 1) return fmt_overflow(f);
    int shift = 63 - f->mbits;
    int subnormal = 0;
    if (E < emin) {
        shift += emin - E;
        subnormal = 1;
    }
    uint64_t q, rem, half;
    if (shift > 64) {
        return 0; /* below half of the smallest subnormal */
    } else if (shift == 64) {
        q = 0;
        rem = sig;
        half = 1ull << 63;
        /* rem in [2^63, 2^64): rem >= half always, equality only when sig == 2^63 exactly -> tie -> even (0) */
        return (rem > half) ? 1u : 0u;
    } else {
        q = sig >> shift;
        rem = sig & ((1ull << shift) - 1ull);
        half = 1ull << (shift - 1);
    }
    if (rem > half || (rem == half && (q & 1ull))) q += 1;
    uint64_t enc = subnormal ? q : (((uint64_t)(E + f->bias - 1)) << f->mbits) + q;
    uint32_t maxfinite = (f->kind == 1) ? 0x7e : (fmt_inf(f) - 1u);
    if (enc > maxfinite) return fmt_overflow(f);
    return (uint32_t)enc;
}

static uint32_t narrow_from_f32_bits(uint32_t x, const fmt_t* f) {
    const uint32_t sign = (x >> 31) ? fmt_sign_bit(f) : 0u;
    const uint32_t ax = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return (f->kind == 0) ? fmt_nan(f) : (fmt_nan(f) | sign);
    if (ax == 0x7f800000u) return sign | fmt_overflow(f);
    if (ax == 0) return sign;
    const uint32_t e = ax >> 23, m = ax & 0x7fffffu;
    if (e == 0) return sign | round_mag(m, -149, f);
    return sign | round_mag(m | 0x800000u, (int)e - 150, f);
}

static uint32_t narrow_from_f64(double d, const fmt_t* f) {
    uint64_t x;
    memcpy(&x, &d, 8);
    const uint32_t sign = (x >> 63) ? fmt_sign_bit(f) : 0u;
    const uint64_t ax = x & 0x7fffffffffffffffull;
    if (ax > 0x7ff0000000000000ull) return (f->kind == 0) ? fmt_nan(f) : (fmt_nan(f) | sign);
    if (ax == 0x7ff0000000000000ull) return sign | fmt_overflow(f);
    if (ax == 0) return sign;
    const uint64_t e = ax >> 52, m = ax & 0xfffffffffffffull;
    if (e == 0) return sign | round_mag(m, -1074, f);
    return sign | round_mag(m | (1ull << 52), (int)e - 1075, f);
}

static uint32_t narrow_from_i64(int64_t v, const fmt_t* f) {
    if (v == 0) return 0;
    const uint32_t sign = v < 0 ? fmt_sign_bit(f) : 0u;
    const uint64_t mag = v < 0 ? (uint64_t)0 - (uint64_t)v : (uint64_t)v;
    return sign | round_mag(mag, 0, f);
}

static uint32_t narrow_from_u64(uint64_t v, const fmt_t* f) { return v == 0 ? 0 : round_mag(v, 0, f); }

/* exact widening */
static double widen(uint32_t bits, const fmt_t* f) {
    const uint32_t sign = bits & fmt_sign_bit(f);
    const uint32_t mag = bits & (fmt_sign_bit(f) - 1u);
    const uint32_t e = mag >> f->mbits, m = mag & ((1u << f->mbits) - 1u);
    double v;
    if (f->kind == 1) {
        if (mag == 0x7f) return sign ? -NAN : NAN;
    } else if (e == (1u << f->ebits) - 1u) {
        if (m) return sign ? -NAN : NAN;
        return sign ? -INFINITY : INFINITY;
    }
    if (e == 0)
        v = ldexp((double)m, 1 - f->bias - f->mbits);
    else
        v = ldexp((double)(m | (1u << f->mbits)), (int)e - f->bias - f->mbits);
    return sign ? -v : v;
}

static uint32_t f32_bits(float x) {
    uint32_t b;
    memcpy(&b, &x, 4);
    return b;
}

uint16_t oracle_f32_to_f16_bits(float x) { return (uint16_t)narrow_from_f32_bits(f32_bits(x), &FMT_F16); }
uint16_t oracle_f32_to_bf16_bits(float x) { return (uint16_t)narrow_from_f32_bits(f32_bits(x), &FMT_BF16); }
uint8_t oracle_f32_to_e4m3_bits(float x) { return (uint8_t)narrow_from_f32_bits(f32_bits(x), &FMT_E4M3); }
uint8_t oracle_f32_to_e5m2_bits(float x) { return (uint8_t)narrow_from_f32_bits(f32_bits(x), &FMT_E5M2); }
uint16_t oracle_f64_to_f16_bits(double x) { return (uint16_t)narrow_from_f64(x, &FMT_F16); }
uint16_t oracle_f64_to_bf16_bits(double x) { return (uint16_t)narrow_from_f64(x, &FMT_BF16); }

/* fp16 -> fp32 widening is exact; a NaN operand becomes the canonical quiet NaN 0x7fffffff (PTX cvt.f32.f16 rule). */
float oracle_f16_bits_to_f32(uint16_t h) {
    if ((h & 0x7fffu) > 0x7c00u) {
        uint32_t q = 0x7fffffffu;
        float r;
        memcpy(&r, &q, 4);
        return r;
    }
    return (float)widen(h, &FMT_F16);
}

/* bf16 -> fp32 is a 16-bit left shift (__bfloat162float), NaN payloads included. */
float oracle_bf16_bits_to_f32(uint16_t h) {
    uint32_t b = ((uint32_t)h) << 16;
    float r;
    memcpy(&r, &b, 4);
    return r;
}

float oracle_e4m3_bits_to_f32(uint8_t v) { return (float)widen(v, &FMT_E4M3); }
float oracle_e5m2_bits_to_f32(uint8_t v) { return (float)widen(v, &FMT_E5M2); }

int oracle_dtype_size(int dtype) {
    switch (dtype) {
        case ORACLE_FP8_E4M3:
        case ORACLE_FP8_E5M2:
        case ORACLE_INT8:
        case ORACLE_UINT8:
        case ORACLE_BOOLEAN:
            return 1;
        case ORACLE_FP16:
        case ORACLE_BF16:
        case ORACLE_INT16:
        case ORACLE_UINT16:
            return 2;
        case ORACLE_FP32:
        case ORACLE_INT32:
        case ORACLE_UINT32:
            return 4;
        case ORACLE_FP64:
        case ORACLE_INT64:
        case ORACLE_UINT64:
            return 8;
        default:
            return -1;
    }
}

/* ------------------------------------------------------------------------------------------------------------------
 * Element conversion, `static_cast<To>(From)` semantics for every pair except ->e4m3 (saturate-to-finite helper)
 * (TypeConverter.cpp:10-22).  A value is carried as one of three exact classes.
 * ------------------------------------------------------------------------------------------------------------------ */
typedef struct {
    int cls; /* 0 float32-exact (payload f), 1 double (payload d), 2 signed (payload i), 3 unsigned (payload u) */
    float f;
    double d;
    int64_t i;
    uint64_t u;
} val_t;

static val_t load_val(const void* p, long idx, int dt) {
    val_t v;
    memset(&v, 0, sizeof v);
    switch (dt) {
        case ORACLE_FP16:
            v.cls = 0;
            v.f = oracle_f16_bits_to_f32(((const uint16_t*)p)[idx]);
            break;
        case ORACLE_BF16:
            v.cls = 0;
            v.f = oracle_bf16_bits_to_f32(((const uint16_t*)p)[idx]);
            break;
        case ORACLE_FP8_E4M3:
            v.cls = 0;
            v.f = oracle_e4m3_bits_to_f32(((const uint8_t*)p)[idx]);
            break;
        case ORACLE_FP8_E5M2:
            v.cls = 0;
            v.f = oracle_e5m2_bits_to_f32(((const uint8_t*)p)[idx]);
            break;
        case ORACLE_FP32:
            v.cls = 0;
            v.f = ((const float*)p)[idx];
            break;
        case ORACLE_FP64:
            v.cls = 1;
            v.d = ((const double*)p)[idx];
            break;
        case ORACLE_INT8:
            v.cls = 2;
            v.i = ((const int8_t*)p)[idx];
            break;
        case ORACLE_INT16:
            v.cls = 2;
            v.i = ((const int16_t*)p)[idx];
            break;
        case ORACLE_INT32:
            v.cls = 2;
            v.i = ((const int32_t*)p)[idx];
            break;
        case ORACLE_INT64:
            v.cls = 2;
            v.i = ((const int64_t*)p)[idx];
            break;
        case ORACLE_UINT8:
            v.cls = 3;
            v.u = ((const uint8_t*)p)[idx];
            break;
        case ORACLE_UINT16:
            v.cls = 3;
            v.u = ((const uint16_t*)p)[idx];
            break;
        case ORACLE_UINT32:
            v.cls = 3;
            v.u = ((const uint32_t*)p)[idx];
            break;
        case ORACLE_UINT64:
            v.cls = 3;
            v.u = ((const uint64_t*)p)[idx];
            break;
        case ORACLE_BOOLEAN:
            v.cls = 3;
            v.u = ((const uint8_t*)p)[idx] ? 1 : 0;
            break;
    }
    return v;
}

static uint32_t narrow_val(const val_t* v, const fmt_t* f) {
    switch (v->cls) {
        case 0:
            return narrow_from_f32_bits(f32_bits(v->f), f);
        case 1:
            return narrow_from_f64(v->d, f);
        case 2:
            return narrow_from_i64(v->i, f);
        default:
            return narrow_from_u64(v->u, f);
    }
}

static double val_as_double(const val_t* v) {
    switch (v->cls) {
        case 0:
            return (double)v->f;
        case 1:
            return v->d;
        case 2:
            return (double)v->i;
        default:
            return (double)v->u;
    }
}

/* float -> integer is C++ truncation toward zero; out-of-range is undefined in the reference, here it wraps through int64 */
static int64_t val_as_i64(const val_t* v) {
    switch (v->cls) {
        case 0:
            return (v->f != v->f) ? 0 : (int64_t)v->f;
        case 1:
            return (v->d != v->d) ? 0 : (int64_t)v->d;
        case 2:
            return v->i;
        default:
            return (int64_t)v->u;
    }
}

static uint64_t val_as_u64(const val_t* v) {
    switch (v->cls) {
        case 0:
            return (v->f != v->f) ? 0 : (v->f < 0 ? (uint64_t)(int64_t)v->f : (uint64_t)v->f);
        case 1:
            return (v->d != v->d) ? 0 : (v->d < 0 ? (uint64_t)(int64_t)v->d : (uint64_t)v->d);
        case 2:
            return (uint64_t)v->i;
        default:
            return v->u;
    }
}

static void store_val(void* p, long idx, int dt, const val_t* v) {
    switch (dt) {
        case ORACLE_FP16:
            ((uint16_t*)p)[idx] = (uint16_t)narrow_val(v, &FMT_F16);
            break;
        case ORACLE_BF16:
            ((uint16_t*)p)[idx] = (uint16_t)narrow_val(v, &FMT_BF16);
            break;
        case ORACLE_FP8_E4M3:
            ((uint8_t*)p)[idx] = (uint8_t)narrow_val(v, &FMT_E4M3);
            break;
        case ORACLE_FP8_E5M2:
            ((uint8_t*)p)[idx] = (uint8_t)narrow_val(v, &FMT_E5M2);
            break;
        case ORACLE_FP32:
            switch (v->cls) {
                case 0:
                    ((float*)p)[idx] = v->f;
                    break;
                case 1:
                    ((float*)p)[idx] = (float)v->d;
                    break;
                case 2:
                    ((float*)p)[idx] = (float)v->i;
                    break;
                default:
                    ((float*)p)[idx] = (float)v->u;
                    break;
            }
            break;
        case ORACLE_FP64:
            ((double*)p)[idx] = val_as_double(v);
            break;
        case ORACLE_INT8:
            ((int8_t*)p)[idx] = (int8_t)val_as_i64(v);
            break;
        case ORACLE_INT16:
            ((int16_t*)p)[idx] = (int16_t)val_as_i64(v);
            break;
        case ORACLE_INT32:
            ((int32_t*)p)[idx] = (int32_t)val_as_i64(v);
            break;
        case ORACLE_INT64:
            ((int64_t*)p)[idx] = val_as_i64(v);
            break;
        case ORACLE_UINT8:
            ((uint8_t*)p)[idx] = (uint8_t)val_as_u64(v);
            break;
        case ORACLE_UINT16:
            ((uint16_t*)p)[idx] = (uint16_t)val_as_u64(v);
            break;
        case ORACLE_UINT32:
            ((uint32_t*)p)[idx] = (uint32_t)val_as_u64(v);
            break;
        case ORACLE_UINT64:
            ((uint64_t*)p)[idx] = val_as_u64(v);
            break;
        case ORACLE_BOOLEAN: {
            int nz;
            switch (v->cls) {
                case 0:
                    nz = v->f != 0.0f;
                    break;
                case 1:
                    nz = v->d != 0.0;
                    break;
                case 2:
                    nz = v->i != 0;
                    break;
                default:
                    nz = v->u != 0;
                    break;
            }
            ((uint8_t*)p)[idx] = nz ? 1 : 0;
            break;
        }
    }
}

static void convert_range(const void* src, void* dst, int sdt, int ddt, long begin, long end, int reverse) {
    /* hot pairs get tight loops so the timed CPU baseline is not dominated by the generic dispatch */
    if (!reverse && sdt == ORACLE_FP32 && ddt == ORACLE_FP16) {
        const uint32_t* s = (const uint32_t*)src;
        uint16_t* d = (uint16_t*)dst;
        for (long i = begin; i < end; ++i) d[i] = (uint16_t)narrow_from_f32_bits(s[i], &FMT_F16);
        return;
    }
    if (!reverse && sdt == ORACLE_FP32 && ddt == ORACLE_BF16) {
        const uint32_t* s = (const uint32_t*)src;
        uint16_t* d = (uint16_t*)dst;
        for (long i = begin; i < end; ++i) d[i] = (uint16_t)narrow_from_f32_bits(s[i], &FMT_BF16);
        return;
    }
    if (!reverse && sdt == ORACLE_FP16 && ddt == ORACLE_FP32) {
        const uint16_t* s = (const uint16_t*)src;
        float* d = (float*)dst;
        for (long i = begin; i < end; ++i) d[i] = oracle_f16_bits_to_f32(s[i]);
        return;
    }
    if (!reverse && sdt == ORACLE_BF16 && ddt == ORACLE_FP32) {
        const uint16_t* s = (const uint16_t*)src;
        float* d = (float*)dst;
        for (long i = begin; i < end; ++i) d[i] = oracle_bf16_bits_to_f32(s[i]);
        return;
    }
    if (!reverse) {
        for (long i = begin; i < end; ++i) {
            val_t v = load_val(src, i, sdt);
            store_val(dst, i, ddt, &v);
        }
    } else {
        for (long i = end - 1; i >= begin; --i) {
            val_t v = load_val(src, i, sdt);
            store_val(dst, i, ddt, &v);
        }
    }
}

/* TypeConverter::cpuConvertTypeImpl (TypeConverter.cpp:899-942): out of place or same-size in place runs an OpenMP
 * static partition over numProcs = max(min(nprocs, n / 500000), 1) threads; in-place narrowing walks forward and
 * in-place widening walks backward on one thread. */
int oracle_convert(const void* src, void* dst, int sdt, int ddt, long n, int threads) {
    const int ss = oracle_dtype_size(sdt), ds = oracle_dtype_size(ddt);
    if (ss < 0 || ds < 0 || n < 0) return -1;
    if (n == 0) return 0;
    const int in_place = (src == dst);
    if (!in_place || ss == ds) {
        long procs = threads > 0 ? threads : omp_get_num_procs();
        if (threads <= 0) {
            long cap = n / 500000;
            if (procs > cap) procs = cap;
        }
        if (procs < 1) procs = 1;
        if (procs > 1) {
            const long per = (n + procs - 1) / procs;
#pragma omp parallel for schedule(static, 1) num_threads(procs)
            for (long t = 0; t < procs; ++t) {
                long b = t * per, e = b + per;
                if (e > n) e = n;
                if (b < e) convert_range(src, dst, sdt, ddt, b, e, 0);
            }
        } else {
            convert_range(src, dst, sdt, ddt, 0, n, 0);
        }
        return (int)procs;
    }
    convert_range(src, dst, sdt, ddt, 0, n, ds > ss);
    return 1;
}

/* ------------------------------------------------------------------------------------------------------------------
 * Exhaustive witnesses
 * ------------------------------------------------------------------------------------------------------------------ */
#if defined(__x86_64__)
__attribute__((target("f16c"))) static uint16_t hw_f32_to_f16(float x) {
    return (uint16_t)_mm_extract_epi16(_mm_cvtps_ph(_mm_set_ss(x), _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC), 0);
}
__attribute__((target("f16c"))) static float hw_f16_to_f32(uint16_t h) {
    return _mm_cvtss_f32(_mm_cvtph_ps(_mm_cvtsi32_si128(h)));
}
#endif

long oracle_check_f16_against_f16c(void) {
#if defined(__x86_64__)
    if (!__builtin_cpu_supports("f16c")) return -1;
    long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (long hi = 0; hi < 65536; ++hi) {
        for (uint32_t lo = 0; lo < 65536; ++lo) {
            uint32_t b = ((uint32_t)hi << 16) | lo;
            float x;
            memcpy(&x, &b, 4);
            uint16_t mine = (uint16_t)narrow_from_f32_bits(b, &FMT_F16);
            uint16_t hw = hw_f32_to_f16(x);
            if ((b & 0x7fffffffu) > 0x7f800000u) {
                /* F16C keeps sign and payload of NaNs; only require "NaN stays NaN" there */
                if ((hw & 0x7fffu) <= 0x7c00u || (mine & 0x7fffu) <= 0x7c00u) bad++;
            } else if (mine != hw) {
                bad++;
            }
        }
    }
    return bad;
#else
    return -1;
#endif
}

long oracle_check_f16_widen_against_f16c(void) {
#if defined(__x86_64__)
    if (!__builtin_cpu_supports("f16c")) return -1;
    long bad = 0;
    for (uint32_t h = 0; h < 65536; ++h) {
        float a = oracle_f16_bits_to_f32((uint16_t)h), b = hw_f16_to_f32((uint16_t)h);
        if ((h & 0x7fffu) > 0x7c00u) {
            if (a == a || b == b) bad++;
        } else if (memcmp(&a, &b, 4) != 0) {
            bad++;
        }
    }
    return bad;
#else
    return -1;
#endif
}

long oracle_check_bf16_against_addtrick(void) {
    long bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
    for (long hi = 0; hi < 65536; ++hi) {
        for (uint32_t lo = 0; lo < 65536; ++lo) {
            uint32_t b = ((uint32_t)hi << 16) | lo;
            uint16_t mine = (uint16_t)narrow_from_f32_bits(b, &FMT_BF16);
            uint16_t other;
            if ((b & 0x7fffffffu) > 0x7f800000u)
                other = 0x7fff;
            else
                other = (uint16_t)((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
            if (mine != other) bad++;
        }
    }
    return bad;
}

/* ------------------------------------------------------------------------------------------------------------------
 * Reductions (Utilities/TensorOperations/Cub/CubReductionOperation.cuh:60-164, CubReduction.cpp:718-734,
 * CubReductionSum.cu:10-119, CubReductionMax.cu:8-48) and arg reductions (CubArgReductionOperation.cuh:24-71).
 * ------------------------------------------------------------------------------------------------------------------ */
static float load_f32(const void* p, uint64_t idx, int dt) {
    switch (dt) {
        case ORACLE_FP32:
            return ((const float*)p)[idx];
        case ORACLE_FP16:
            return oracle_f16_bits_to_f32(((const uint16_t*)p)[idx]);
        case ORACLE_BF16:
            return oracle_bf16_bits_to_f32(((const uint16_t*)p)[idx]);
        case ORACLE_FP8_E4M3:
            return oracle_e4m3_bits_to_f32(((const uint8_t*)p)[idx]);
        case ORACLE_FP8_E5M2:
            return oracle_e5m2_bits_to_f32(((const uint8_t*)p)[idx]);
        default:
            return NAN;
    }
}

static int reduction_dtype_ok(int dt) {
    return dt == ORACLE_FP32 || dt == ORACLE_FP16 || dt == ORACLE_BF16 || dt == ORACLE_FP8_E4M3 || dt == ORACLE_FP8_E5M2;
}

typedef struct {
    int nk, nr;
    uint64_t kdims[16], kstr[16], rdims[16], rstr[16];
    uint64_t outputs, rsize;
} geom_t;

static int make_geom(const uint64_t* dims, const uint64_t* strides, int rank, const uint32_t* axes, int naxes, geom_t* g) {
    if (rank < 1 || rank > 16 || naxes < 1 || naxes > rank) return -1;
    g->nk = g->nr = 0;
    g->outputs = g->rsize = 1;
    int c = 0;
    for (int d = 0; d < rank; ++d) {
        if (dims[d] == 0) return -1;
        if (c < naxes && axes[c] == (uint32_t)d) {
            if (c > 0 && axes[c] <= axes[c - 1]) return -1;
            g->rdims[g->nr] = dims[d];
            g->rstr[g->nr++] = strides[d];
            g->rsize *= dims[d];
            ++c;
        } else {
            g->kdims[g->nk] = dims[d];
            g->kstr[g->nk++] = strides[d];
            g->outputs *= dims[d];
        }
    }
    return c == naxes ? 0 : -1;
}

static uint64_t offset_of(uint64_t flat, int n, const uint64_t* dims, const uint64_t* str) {
    uint64_t off = 0;
    for (int i = n - 1; i >= 0; --i) {
        off += (flat % dims[i]) * str[i];
        flat /= dims[i];
    }
    return off;
}

static float prop_min(float a, float b) { return a != a ? a : (b != b ? b : fminf(a, b)); }
static float prop_max(float a, float b) { return a != a ? a : (b != b ? b : fmaxf(a, b)); }

static void store_f32_as(void* out, uint64_t idx, int dt, float v) {
    val_t x;
    memset(&x, 0, sizeof x);
    x.cls = 0;
    x.f = v;
    store_val(out, (long)idx, dt, &x);
}

int oracle_reduce(int op, const void* in, int in_dtype, const uint64_t* dims, const uint64_t* strides, int rank,
                  const uint32_t* axes, int naxes, float scale, void* out, int out_dtype) {
    geom_t g;
    if (!reduction_dtype_ok(in_dtype) || !reduction_dtype_ok(out_dtype)) return -1;
    if (make_geom(dims, strides, rank, axes, naxes, &g)) return -1;
    if (op < ORACLE_SUM || op > ORACLE_L2) return -1;
#pragma omp parallel for schedule(static) if (g.outputs > 64)
    for (uint64_t o = 0; o < g.outputs; ++o) {
        const uint64_t base = offset_of(o, g.nk, g.kdims, g.kstr);
        float acc;
        switch (op) {
            case ORACLE_MIN:
                acc = INFINITY;
                break;
            case ORACLE_MAX:
                acc = -INFINITY;
                break;
            case ORACLE_PRODUCT:
                acc = 1.0f;
                break;
            default:
                acc = 0.0f;
                break;
        }
        for (uint64_t r = 0; r < g.rsize; ++r) {
            const float x = load_f32(in, base + offset_of(r, g.nr, g.rdims, g.rstr), in_dtype);
            switch (op) {
                case ORACLE_SUM:
                case ORACLE_MEAN:
                    acc = acc + x;
                    break;
                case ORACLE_L1:
                    acc = acc + fabsf(x);
                    break;
                case ORACLE_L2:
                    acc = acc + x * x;
                    break;
                case ORACLE_PRODUCT:
                    acc = acc * x;
                    break;
                case ORACLE_MIN:
                    acc = prop_min(acc, x);
                    break;
                case ORACLE_MAX:
                    acc = prop_max(acc, x);
                    break;
            }
        }
        if (op == ORACLE_MEAN) {
            const float div = (float)g.rsize;
            acc = (div == 0.0f) ? 0.0f : (div == 1.0f ? acc : acc / div);
        } else if (op == ORACLE_L2) {
            acc = sqrtf(acc);
        }
        store_f32_as(out, o, out_dtype, acc * scale);
    }
    return 0;
}

int oracle_reduce_f64(int op, const void* in, int in_dtype, const uint64_t* dims, const uint64_t* strides, int rank,
                      const uint32_t* axes, int naxes, double* out) {
    geom_t g;
    if (!reduction_dtype_ok(in_dtype)) return -1;
    if (make_geom(dims, strides, rank, axes, naxes, &g)) return -1;
    if (op < ORACLE_SUM || op > ORACLE_L2) return -1;
#pragma omp parallel for schedule(static) if (g.outputs > 64)
    for (uint64_t o = 0; o < g.outputs; ++o) {
        const uint64_t base = offset_of(o, g.nk, g.kdims, g.kstr);
        double acc = (op == ORACLE_MIN) ? INFINITY : (op == ORACLE_MAX) ? -INFINITY : (op == ORACLE_PRODUCT) ? 1.0 : 0.0;
        double comp = 0.0; /* Neumaier compensation for the additive ops */
        int saw_nan = 0;
        for (uint64_t r = 0; r < g.rsize; ++r) {
            const double x = (double)load_f32(in, base + offset_of(r, g.nr, g.rdims, g.rstr), in_dtype);
            double term = x;
            switch (op) {
                case ORACLE_L1:
                    term = fabs(x);
                    break;
                case ORACLE_L2:
                    term = x * x;
                    break;
                default:
                    break;
            }
            switch (op) {
                case ORACLE_SUM:
                case ORACLE_MEAN:
                case ORACLE_L1:
                case ORACLE_L2: {
                    const double t = acc + term;
                    if (fabs(acc) >= fabs(term))
                        comp += (acc - t) + term;
                    else
                        comp += (term - t) + acc;
                    acc = t;
                    break;
                }
                case ORACLE_PRODUCT:
                    acc *= x;
                    break;
                case ORACLE_MIN:
                    if (x != x) saw_nan = 1;
                    acc = fmin(acc, x);
                    break;
                case ORACLE_MAX:
                    if (x != x) saw_nan = 1;
                    acc = fmax(acc, x);
                    break;
            }
        }
        if (op == ORACLE_SUM || op == ORACLE_MEAN || op == ORACLE_L1 || op == ORACLE_L2) {
            if (isfinite(acc)) acc += comp;
        }
        if (op == ORACLE_MEAN) acc /= (double)g.rsize;
        if (op == ORACLE_L2) acc = sqrt(acc);
        if (saw_nan) acc = NAN;
        out[o] = acc;
    }
    return 0;
}

int oracle_arg_reduce(int op, const void* in, int in_dtype, const uint64_t* dims, const uint64_t* strides, int rank,
                      const uint32_t* axes, int naxes, uint64_t* index_out, float* value_out) {
    geom_t g;
    if (!reduction_dtype_ok(in_dtype)) return -1;
    if (make_geom(dims, strides, rank, axes, naxes, &g)) return -1;
    if (op != ORACLE_ARGMIN && op != ORACLE_ARGMAX) return -1;
#pragma omp parallel for schedule(static) if (g.outputs > 64)
    for (uint64_t o = 0; o < g.outputs; ++o) {
        const uint64_t base = offset_of(o, g.nk, g.kdims, g.kstr);
        uint64_t best_i = 0;
        float best_v = load_f32(in, base + offset_of(0, g.nr, g.rdims, g.rstr), in_dtype);
        for (uint64_t r = 1; r < g.rsize; ++r) {
            const float x = load_f32(in, base + offset_of(r, g.nr, g.rdims, g.rstr), in_dtype);
            /* candidate rule: NaN beats numbers, earlier index wins between equals and between NaNs */
            const int best_nan = best_v != best_v, x_nan = x != x;
            int take = 0;
            if (best_nan) {
                take = 0;
            } else if (x_nan) {
                take = 1;
            } else if (op == ORACLE_ARGMAX) {
                take = x > best_v;
            } else {
                take = x < best_v;
            }
            if (take) {
                best_v = x;
                best_i = r;
            }
        }
        index_out[o] = best_i;
        if (value_out) value_out[o] = best_v;
    }
    return 0;
}
