/*
 * CPU oracle for the Thor hot path (type conversion, dense reductions, arg reductions).
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls this file.  It exists so that
 * the HIP kernels can be checked against an independent CPU restatement of the reference semantics, and so that a
 * CPU baseline can be timed beside the GPU numbers.
 *
 * Every function names the reference file:line whose behaviour it restates (paths relative to the reference root).
 *
 * Pinning status (what independently confirms each function, see tests/test_oracle_*.py):
 *   - fp32<->fp16 conversion: exhaustive over all 2^32 fp32 bit patterns against the x86 F16C hardware converter,
 *     plus numpy float16 on edge vectors                                                   -> pinned
 *   - fp32<->bf16 conversion: exhaustive over all 2^32 patterns against the independent add-0x7fff formulation,
 *     plus torch CPU bfloat16 casts on edge vectors                                        -> pinned
 *   - fp8 e4m3 / e5m2: all 256 codes round-trip, monotone midpoints, reference KATs 448 / 57344
 *     (test/Utilities/TensorOperations/CubReductionDTypeAndLifecycleTest.cpp:205-222)       -> pinned for finite
 *     values; NaN sign/payload of the fp8 encoders is "parity unpinned" (only CUDA headers fix it)
 *   - NaN canonicalisation of the fp16/bf16 narrowing converters (0x7FFF) follows the PTX cvt rule; the reference
 *     tests do not exercise it -> "parity unpinned" for NaN payloads only
 *   - reductions / arg reductions: reference KAT arrays (CubReductionValueOperationsTest.cpp:23-100,
 *     CubArgReductionTest.cpp:154-188), numpy float64 closed forms, brute force on tiny shapes -> pinned
 */
#ifndef THOR_ORACLE_H
#define THOR_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Numeric codes follow DeepLearning/Implementation/Tensor/DataType.h:7-27. */
enum {
    ORACLE_FP16 = 10,
    ORACLE_FP32 = 11,
    ORACLE_FP64 = 12,
    ORACLE_INT8 = 13,
    ORACLE_INT16 = 14,
    ORACLE_INT32 = 15,
    ORACLE_INT64 = 16,
    ORACLE_UINT8 = 17,
    ORACLE_UINT16 = 18,
    ORACLE_UINT32 = 19,
    ORACLE_UINT64 = 20,
    ORACLE_BOOLEAN = 21,
    ORACLE_FP8_E4M3 = 22,
    ORACLE_FP8_E5M2 = 23,
    ORACLE_BF16 = 24
};

/* Utilities/TensorOperations/Cub/CubReduction.h:16-24 */
enum { ORACLE_SUM = 0, ORACLE_MIN = 1, ORACLE_MAX = 2, ORACLE_PRODUCT = 3, ORACLE_MEAN = 4, ORACLE_L1 = 5, ORACLE_L2 = 6 };
/* Utilities/TensorOperations/Cub/CubReduction.h:26-29 */
enum { ORACLE_ARGMIN = 0, ORACLE_ARGMAX = 1 };

int oracle_dtype_size(int dtype);

/* Scalar converters (bit level). */
uint16_t oracle_f32_to_f16_bits(float x);
float oracle_f16_bits_to_f32(uint16_t h);
uint16_t oracle_f32_to_bf16_bits(float x);
float oracle_bf16_bits_to_f32(uint16_t h);
uint8_t oracle_f32_to_e4m3_bits(float x);
float oracle_e4m3_bits_to_f32(uint8_t v);
uint8_t oracle_f32_to_e5m2_bits(float x);
float oracle_e5m2_bits_to_f32(uint8_t v);
uint16_t oracle_f64_to_f16_bits(double x);
uint16_t oracle_f64_to_bf16_bits(double x);

/* Array conversion, all 15x15 storage pairs, in place or out of place.
 * threads <= 0 : use the reference's rule numProcs = max(min(nprocs, n / 500000), 1).
 * Returns the number of threads used, or a negative value on an unsupported pair. */
int oracle_convert(const void* src, void* dst, int src_dtype, int dst_dtype, long n, int threads);

/* Exhaustive self checks used by the CPU test-suite.  Return the number of mismatching fp32 bit patterns
 * (0 == pinned) or -1 when the host CPU lacks the instruction used as the independent witness. */
long oracle_check_f16_against_f16c(void);
long oracle_check_bf16_against_addtrick(void);
long oracle_check_f16_widen_against_f16c(void);

/* Dense N-d reduction:  out[o] = store(out_dtype, finalize(reduce(transform(float(in[...])))) * scale).
 * dims/strides are in elements, rank entries; axes strictly increasing.  Accumulation is fp32 in row-major order of
 * the reduced coordinates; *_f64 variants accumulate in double and are the truth the GPU tolerance is judged against. */
int oracle_reduce(int op, const void* in, int in_dtype, const uint64_t* dims, const uint64_t* strides, int rank,
                  const uint32_t* axes, int naxes, float scale, void* out, int out_dtype);
int oracle_reduce_f64(int op, const void* in, int in_dtype, const uint64_t* dims, const uint64_t* strides, int rank,
                      const uint32_t* axes, int naxes, double* out);

/* Arg reduction: winning local flattened index inside the reduction domain (row-major over the reduced axes), NaN wins,
 * lowest index wins ties.  index_out is uint64; value_out (optional) is fp32. */
int oracle_arg_reduce(int op, const void* in, int in_dtype, const uint64_t* dims, const uint64_t* strides, int rank,
                      const uint32_t* axes, int naxes, uint64_t* index_out, float* value_out);

/* BASELINE expression workloads restated on the host (thor_oracle_expr.c); each returns the OpenMP thread count used. */
int oracle_expr_config1(const float* a, const float* b, const float* c, const float* d, float* out, long n);
int oracle_softmax_rows_bf16(const uint16_t* x, float* out, long rows, long cols);
int oracle_normalize_rows_f32(const float* x, float* out, long rows, long cols, float eps);
int oracle_relu_scale_bias_f16(const uint16_t* x, const uint16_t* scale, const uint16_t* bias, uint16_t* out, long n, long c, long hw);
int oracle_channel_stats_f16(const uint16_t* x, float* sum, float* sumsq, long n, long c, long hw);
int oracle_rows_f32(const float* x, float* row_sum, float* row_max, uint32_t* row_argmax, long rows, long cols);

/* Sequential prefix scan (thor_oracle_scan.c) of the `segments` ranges [bounds[2s], bounds[2s+1]) of a flat array of n
 * UINT32 / FP32 / FP16 / BF16 elements.  op: 0 sum, 1 min, 2 max, 3 product.  out_values (element type) and out_index (flattened
 * index of the running extreme; min / max only) may be NULL; elements outside every range are set to 0. */
int oracle_scan(const void* in, int dtype, long n, const int64_t* bounds, long segments, int op, int inclusive, int reverse, void* out_values,
                uint32_t* out_index);

#ifdef __cplusplus
}
#endif
#endif
