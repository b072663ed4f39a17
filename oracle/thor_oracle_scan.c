/*
 * CPU oracle, prefix scans.  TEST INFRASTRUCTURE ONLY: nothing in the shipped library links, loads or calls this file.
 *
 * A sequential, element-by-element walk with the reference's scan operators
 * (Utilities/TensorOperations/Cub/CubScan.cu:50-93): sum and product combine in the element type (16-bit floats: widen both
 * operands to fp32, add or multiply, round to the type - :52-68), min / max are selections that keep the earlier element
 * unless the later one is strictly smaller / larger (:70-90, comparisons of 16-bit floats on their fp32 values), UINT32
 * wraps.  Identities that open an exclusive scan (:92-196): 0, 1, the largest / smallest value of the type (+-inf for
 * floats, 0xFFFFFFFF / 0 for UINT32).  Arg scans return the flattened index of the element that holds the running extreme
 * (0xFFFFFFFF for the empty prefix of an exclusive scan).
 *
 * Pinning: the reference's scan tests' literal vectors (tests/golden/scan_kats.json), NumPy's sequential cumsum / cumprod /
 * minimum.accumulate / maximum.accumulate on random rows, and the pure-Python walk of oracle/__init__.py on small inputs
 * (tests/test_oracle_scans.py).  Unpinned: the order in which the reference's library combines partial sums (any order is a
 * valid result of the reference), NaN operands of min / max.
 */
#include "thor_oracle.h"

#include <math.h>
#include <string.h>

static float scan_load(const void* in, long i, int dtype) {
    switch (dtype) {
        case ORACLE_FP32: return ((const float*)in)[i];
        case ORACLE_FP16: return oracle_f16_bits_to_f32(((const uint16_t*)in)[i]);
        default: return oracle_bf16_bits_to_f32(((const uint16_t*)in)[i]);
    }
}

static float scan_round(float v, int dtype) {
    switch (dtype) {
        case ORACLE_FP32: return v;
        case ORACLE_FP16: return oracle_f16_bits_to_f32(oracle_f32_to_f16_bits(v));
        default: return oracle_bf16_bits_to_f32(oracle_f32_to_bf16_bits(v));
    }
}

static void scan_store(void* out, long i, int dtype, float v) {
    switch (dtype) {
        case ORACLE_FP32: ((float*)out)[i] = v; break;
        case ORACLE_FP16: ((uint16_t*)out)[i] = oracle_f32_to_f16_bits(v); break;
        default: ((uint16_t*)out)[i] = oracle_f32_to_bf16_bits(v); break;
    }
}

int oracle_scan(const void* in, int dtype, long n, const int64_t* bounds, long segments, int op, int inclusive, int reverse, void* out_values,
                uint32_t* out_index) {
    if (dtype != ORACLE_UINT32 && dtype != ORACLE_FP32 && dtype != ORACLE_FP16 && dtype != ORACLE_BF16) return -1;
    if (op < 0 || op > 3) return -2;
    const int integer = dtype == ORACLE_UINT32;
    if (out_values) memset(out_values, 0, (size_t)n * (size_t)oracle_dtype_size(dtype));
    if (out_index) memset(out_index, 0, (size_t)n * sizeof(uint32_t));
    for (long s = 0; s < segments; ++s) {
        const long begin = bounds[2 * s], end = bounds[2 * s + 1];
        if (begin < 0 || end > n || end < begin) return -3;
        int started = 0;
        uint32_t running_u = 0, winner = 0xFFFFFFFFu;
        float running_f = 0.0f;
        for (long k = 0; k < end - begin; ++k) {
            const long i = reverse ? end - 1 - k : begin + k;
            if (!inclusive) {
                if (out_index) out_index[i] = winner;
                if (out_values) {
                    if (integer) {
                        ((uint32_t*)out_values)[i] = started ? running_u : (op == 0 ? 0u : op == 3 ? 1u : op == 1 ? 0xFFFFFFFFu : 0u);
                    } else {
                        const float identity = op == 0 ? 0.0f : op == 3 ? 1.0f : op == 1 ? INFINITY : -INFINITY;
                        scan_store(out_values, i, dtype, started ? running_f : identity);
                    }
                }
            }
            if (integer) {
                const uint32_t x = ((const uint32_t*)in)[i];
                if (!started) {
                    running_u = x;
                    winner = (uint32_t)i;
                } else if (op == 0) {
                    running_u += x;
                } else if (op == 3) {
                    running_u *= x;
                } else if (op == 1 ? x < running_u : running_u < x) {
                    running_u = x;
                    winner = (uint32_t)i;
                }
            } else {
                const float x = scan_load(in, i, dtype);
                if (!started) {
                    running_f = x;
                    winner = (uint32_t)i;
                } else if (op == 0) {
                    running_f = scan_round(running_f + x, dtype);
                } else if (op == 3) {
                    running_f = scan_round(running_f * x, dtype);
                } else if (op == 1 ? x < running_f : running_f < x) {
                    running_f = x;
                    winner = (uint32_t)i;
                }
            }
            started = 1;
            if (inclusive) {
                if (out_index) out_index[i] = winner;
                if (out_values) {
                    if (integer) ((uint32_t*)out_values)[i] = running_u;
                    else scan_store(out_values, i, dtype, running_f);
                }
            }
        }
    }
    return 0;
}
