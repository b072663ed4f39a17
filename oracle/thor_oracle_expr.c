/*
 * CPU restatement of the BASELINE expression workloads (configs 1, 4, 5) for the timed CPU baseline and as a second
 * checker beside the float64 closed forms.  TEST INFRASTRUCTURE ONLY, like thor_oracle.c.
 *
 * The reference has no CPU evaluator for expressions (Utilities/Expression/EquationRunner.cpp:56-58 rejects non-GPU
 * tensors), so these loops restate what its generated kernels compute, node by node:
 *   - sigmoid(d) = exp(-max(-d,0)) / (1 + exp(-|d|))            Utilities/Expression/Expression.cpp:3261-3296
 *   - fp32 nodes evaluate with expf / IEEE divide                Utilities/Expression/CudaSourceEmitter.cpp:1749-1959
 *   - fp16 nodes round after every operation (__hmul2, __hadd2)  Utilities/Expression/CudaSourceEmitter.cpp:4373-4435
 *   - reductions accumulate in fp32, mean divides by (float)R    Utilities/TensorOperations/Cub/CubReductionOperation.cuh:60-129
 *   - softmax / normalisation are the composed stage plans       test/Utilities/Expression/CommonInputFusionTest.cpp:281-327
 * Pinning: tests/test_oracle_expressions.py checks every function against numpy float64 closed forms (fp32 results within
 * 2 ulp of the correctly rounded value for elementwise work, 1e-5 relative for sums) and the fp16 paths bit for bit against
 * numpy float16 arithmetic.  Row sums of configs 4a / 4b add by halving, the others one after the other.
 */
#include "thor_oracle.h"

#include <math.h>
#include <omp.h>
#include <string.h>

static float sigmoid_f32(float d) {
    const float a = expf(-fmaxf(-d, 0.0f));
    const float b = 1.0f + expf(-fabsf(d));
    return a / b;
}

/* fp32 sum of v[0..n) (of the squares when `squares` is set) by halving: the reference's reductions are library tree
 * reductions whose order is not specified (CubReductionOperation.cuh:2908-2956), so any fp32 order is a restatement; this
 * one keeps the rounding error at log2(n) ulps, where adding 4096 terms one after the other drifts by up to ~1e-5 relative. */
static float pairwise_sum(const float* v, long n, int squares) {
    if (n <= 8) {
        float s = 0.0f;
        for (long j = 0; j < n; ++j) s += squares ? v[j] * v[j] : v[j];
        return s;
    }
    const long half = n / 2;
    return pairwise_sum(v, half, squares) + pairwise_sum(v + half, n - half, squares);
}

/* config 1: out = (a*b + c) * sigmoid(d), fp32 */
int oracle_expr_config1(const float* a, const float* b, const float* c, const float* d, float* out, long n) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < n; ++i) {
        const float t = a[i] * b[i];
        const float u = t + c[i];
        out[i] = u * sigmoid_f32(d[i]);
    }
    return omp_get_max_threads();
}

/* config 4a: y = exp(x - rowmax) / rowsum, x bf16 (bit patterns), fp32 arithmetic, fp32 output */
int oracle_softmax_rows_bf16(const uint16_t* x, float* out, long rows, long cols) {
#pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        const uint16_t* xr = x + r * cols;
        float* yr = out + r * cols;
        float m = -INFINITY;
        for (long j = 0; j < cols; ++j) {
            const float v = oracle_bf16_bits_to_f32(xr[j]);
            m = (v != v || m != m) ? NAN : fmaxf(m, v);
        }
        for (long j = 0; j < cols; ++j) yr[j] = expf(oracle_bf16_bits_to_f32(xr[j]) - m);
        const float sum = pairwise_sum(yr, cols, 0);
        for (long j = 0; j < cols; ++j) yr[j] = yr[j] / sum;
    }
    return omp_get_max_threads();
}

/* config 4b: y = (x - mean) / sqrt(var + eps), population variance, fp32 */
int oracle_normalize_rows_f32(const float* x, float* out, long rows, long cols, float eps) {
#pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        const float* xr = x + r * cols;
        float* yr = out + r * cols;
        const float mean = pairwise_sum(xr, cols, 0) / (float)cols;
        for (long j = 0; j < cols; ++j) yr[j] = xr[j] - mean;
        const float sq = pairwise_sum(yr, cols, 1);
        const float denom = sqrtf(sq / (float)cols + eps);
        for (long j = 0; j < cols; ++j) yr[j] = yr[j] / denom;
    }
    return omp_get_max_threads();
}

static float round_f16(float v) { return oracle_f16_bits_to_f32(oracle_f32_to_f16_bits(v)); }

/* config 5a: y = max(x*scale + bias, 0) in fp16 arithmetic (one rounding per operation), NCHW with per-channel scale, bias */
int oracle_relu_scale_bias_f16(const uint16_t* x, const uint16_t* scale, const uint16_t* bias, uint16_t* out, long n, long c, long hw) {
#pragma omp parallel for schedule(static) collapse(2)
    for (long i = 0; i < n; ++i) {
        for (long ch = 0; ch < c; ++ch) {
            const float s = oracle_f16_bits_to_f32(scale[ch]), b = oracle_f16_bits_to_f32(bias[ch]);
            const uint16_t* xp = x + (i * c + ch) * hw;
            uint16_t* yp = out + (i * c + ch) * hw;
            for (long j = 0; j < hw; ++j) {
                const float prod = round_f16(oracle_f16_bits_to_f32(xp[j]) * s);
                const float sum = round_f16(prod + b);
                yp[j] = oracle_f32_to_f16_bits(fmaxf(sum, 0.0f));
            }
        }
    }
    return omp_get_max_threads();
}

/* config 5b: per-channel sum of x and of x*x (the product rounded to fp16 like a materialised fp16 stage), fp32 accumulate */
int oracle_channel_stats_f16(const uint16_t* x, float* sum, float* sumsq, long n, long c, long hw) {
#pragma omp parallel for schedule(static)
    for (long ch = 0; ch < c; ++ch) {
        float s = 0.0f, q = 0.0f;
        for (long i = 0; i < n; ++i) {
            const uint16_t* xp = x + (i * c + ch) * hw;
            for (long j = 0; j < hw; ++j) {
                const float v = oracle_f16_bits_to_f32(xp[j]);
                s += v;
                q += round_f16(v * v);
            }
        }
        sum[ch] = s;
        sumsq[ch] = q;
    }
    return omp_get_max_threads();
}

/* config 3 on the host cores: row sums, row maxima (NaN propagating) and row argmax (NaN wins, lowest index on ties) */
int oracle_rows_f32(const float* x, float* row_sum, float* row_max, uint32_t* row_argmax, long rows, long cols) {
#pragma omp parallel for schedule(static)
    for (long r = 0; r < rows; ++r) {
        const float* xr = x + r * cols;
        float s = 0.0f, m = xr[0];
        uint32_t at = 0;
        for (long j = 0; j < cols; ++j) {
            const float v = xr[j];
            s += v;
            const int m_nan = m != m, v_nan = v != v;
            if (!m_nan && (v_nan || v > m)) {
                m = v;
                at = (uint32_t)j;
            }
        }
        row_sum[r] = s;
        row_max[r] = m;
        row_argmax[r] = at;
    }
    return omp_get_max_threads();
}
