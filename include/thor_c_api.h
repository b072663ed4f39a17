/*
 * thor_c_api.h -- flat C binding of the host-side Thor API of this backend (Tensor, Stream, TypeConverter,
 * CubReduction / CubArgReduction, Expression, FusedEquation, StampedExecutionPlan).
 *
 * The reference exposes this surface to Python through a nanobind module
 * (bindings/python/src/core/physical/expression.cpp:602-2866, physical_tensor.cpp); this header is what a cgo / JNI /
 * ctypes / nanobind shim binds instead.  Each function names the C++ entry point of the reference it stands for.
 *
 * Conventions: opaque handles are created by *_create / builder functions and released with the matching *_destroy;
 * handles are independent references (destroying a tensor handle does not free storage another handle still uses).
 * Functions that can fail return 0 on success and a negative code otherwise, or NULL for handle-returning functions;
 * thor_last_error() then holds the message of the C++ exception, prefixed with its type
 * ("invalid_argument: ...", "runtime_error: ...", "logic_error: ...").
 */
#ifndef THOR_C_API_H
#define THOR_C_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct thor_tensor* thor_tensor_t;
typedef struct thor_stream* thor_stream_t;
typedef struct thor_stamped_reduction* thor_stamped_reduction_t;
typedef struct thor_stamped_arg_reduction* thor_stamped_arg_reduction_t;
typedef struct thor_stamped_segmented_reduction* thor_stamped_segmented_reduction_t;
typedef struct thor_selection_plan* thor_selection_plan_t;
typedef struct thor_expr* thor_expr_t;
typedef struct thor_outputs* thor_outputs_t;
typedef struct thor_fused_equation* thor_fused_equation_t;
typedef struct thor_plan* thor_plan_t;

enum { THOR_DEVICE_CPU = 1, THOR_DEVICE_GPU = 2 }; /* TensorPlacement::MemDevices */

const char* thor_last_error(void);

/* ---- Stream (Utilities/Common/Stream.h:35-116) ----------------------------------------------------------------------- */
thor_stream_t thor_stream_create(int gpu_num);
void thor_stream_destroy(thor_stream_t stream);
int thor_stream_synchronize(thor_stream_t stream);
void* thor_stream_raw(thor_stream_t stream); /* the hipStream_t, for thorhip_* calls */
int thor_stream_gpu_num(thor_stream_t stream);

/* ---- Tensor (DeepLearning/Implementation/Tensor/Tensor.h:54-264) ------------------------------------------------------- */
thor_tensor_t thor_tensor_create(int device_type, int device_num, int dtype, const uint64_t* dims, int rank);
thor_tensor_t thor_tensor_clone_handle(thor_tensor_t tensor);
void thor_tensor_destroy(thor_tensor_t tensor);
void* thor_tensor_mem_ptr(thor_tensor_t tensor);
int thor_tensor_dtype(thor_tensor_t tensor);
int thor_tensor_rank(thor_tensor_t tensor);
int thor_tensor_dims(thor_tensor_t tensor, uint64_t* dims_out);       /* rank entries */
int thor_tensor_strides(thor_tensor_t tensor, uint64_t* strides_out); /* rank entries, in elements */
uint64_t thor_tensor_num_elements(thor_tensor_t tensor);
int thor_tensor_device_type(thor_tensor_t tensor);
int thor_tensor_device_num(thor_tensor_t tensor);
int thor_tensor_is_dense(thor_tensor_t tensor);
/* Tensor::copyFromAsync: copies and, when dtypes differ, converts (Tensor.cpp:731-866) */
int thor_tensor_copy_from_async(thor_tensor_t dest, thor_tensor_t source, thor_stream_t stream);
int thor_tensor_memset_async(thor_tensor_t tensor, int byte_value, thor_stream_t stream);
int thor_tensor_reshape(thor_tensor_t tensor, const uint64_t* dims, int rank);
/* Tensor::aliasView (Tensor.cpp:617-660) */
thor_tensor_t thor_tensor_alias_view(thor_tensor_t tensor, const uint64_t* dims, const uint64_t* strides_elements, int rank,
                                     uint64_t element_offset);

/* ---- TypeConverter::convertType (TypeConverter.h:30-46); device_num == -1 converts on the host inside the stream ------ */
int thor_convert_type(void* source, void* dest, int source_dtype, int dest_dtype, int64_t num_elements, thor_stream_t stream,
                      int device_num);
/* synchronous host conversion, TypeConverter::cpuConvertTypeImpl (TypeConverter.cpp:899-942) */
int thor_convert_type_cpu(const void* source, void* dest, int source_dtype, int dest_dtype, int64_t num_elements);

/* ---- CubReduction (Utilities/TensorOperations/Cub/CubReduction.h:175-234,496-537) ------------------------------------- */
typedef struct thor_reduction_geometry {
    int path; /* CubReductionPath */
    int reduced_axes_are_contiguous;
    uint64_t outer_size, reduction_size, inner_size;
    uint64_t input_elements, output_elements;
    int rank;
    uint64_t output_dimensions[16];
    int squeezed_rank;
    uint64_t squeezed_output_dimensions[16];
    int device_transform_uses_affine_stride;
    uint64_t affine_input_stride;
} thor_reduction_geometry;

/* CubReduction::analyzeGeometry; strides == NULL means dense row-major */
int thor_reduction_analyze_geometry(const uint64_t* dims, const uint64_t* strides, int rank, const uint32_t* axes, int num_axes,
                                    thor_reduction_geometry* out);
/* CubReduction::mapLogicalReductionIndexToPhysicalIndex */
int thor_reduction_map_index(const uint64_t* dims, const uint64_t* strides, int rank, const uint32_t* axes, int num_axes,
                             uint64_t output_index, uint64_t reduction_index, uint64_t* physical_index);
/* CubReduction(op, axes, output_dtype, scale).stamp(input[, preallocated_output], stream); output_dtype < 0 = input dtype */
thor_stamped_reduction_t thor_reduction_stamp(int op, const uint32_t* axes, int num_axes, int output_dtype, float output_scale,
                                              thor_tensor_t input, thor_tensor_t preallocated_output, thor_stream_t stream);
void thor_stamped_reduction_destroy(thor_stamped_reduction_t r);
int thor_stamped_reduction_run(thor_stamped_reduction_t r);
int thor_stamped_reduction_run_scaled(thor_stamped_reduction_t r, float output_scale);
int thor_stamped_reduction_run_on(thor_stamped_reduction_t r, thor_stream_t stream);
thor_tensor_t thor_stamped_reduction_output(thor_stamped_reduction_t r);
int thor_stamped_reduction_path(thor_stamped_reduction_t r);
size_t thor_stamped_reduction_workspace_bytes(thor_stamped_reduction_t r);
int thor_stamped_reduction_variant(thor_stamped_reduction_t r, char* buffer, size_t capacity);
/* the generated HIP source for a geometry, without touching a GPU (host-only tests compile it with thorhip_compile) */
int thor_reduction_generate_source(int is_arg, int op, int input_dtype, int output_dtype, int index_dtype, const uint64_t* dims,
                                   const uint64_t* strides, int rank, const uint32_t* axes, int num_axes, char* buffer,
                                   size_t capacity, size_t* needed);

/* ---- CubArgReduction (CubReduction.h:412-487) ---------------------------------------------------------------------------- */
thor_stamped_arg_reduction_t thor_arg_reduction_stamp(int op, const uint32_t* axes, int num_axes, int produce_value, int produce_index,
                                                      int value_output_dtype, int index_output_dtype, thor_tensor_t input,
                                                      thor_tensor_t preallocated_value, thor_tensor_t preallocated_index,
                                                      thor_stream_t stream);
void thor_stamped_arg_reduction_destroy(thor_stamped_arg_reduction_t r);
int thor_stamped_arg_reduction_run(thor_stamped_arg_reduction_t r);
thor_tensor_t thor_stamped_arg_reduction_value_output(thor_stamped_arg_reduction_t r); /* NULL when not produced */
thor_tensor_t thor_stamped_arg_reduction_index_output(thor_stamped_arg_reduction_t r);
int thor_stamped_arg_reduction_path(thor_stamped_arg_reduction_t r);
int thor_stamped_arg_reduction_variant(thor_stamped_arg_reduction_t r, char* buffer, size_t capacity);

/* CubSegmentedReduction / CubSegmentedArgReduction (CubReduction.h:236-400 of the reference): values [N, D...] reduced over the row
 * ranges [offsets[i], offsets[i+1]) of a UINT32 / UINT64 offsets tensor.  is_arg = 0: op is a CubReductionOp (sum, mean, min, max),
 * dtype the output dtype (-1 = input dtype); is_arg = 1: op is a CubArgReductionOp, dtype the index dtype (UINT32 / UINT64, -1 = UINT64).
 * preallocated_output may be NULL unless runtime_offsets is set (then the offsets are not read at stamp time). */
thor_stamped_segmented_reduction_t thor_segmented_reduction_stamp(int is_arg, int op, int dtype, thor_tensor_t input, thor_tensor_t segment_offsets,
                                                                  thor_tensor_t preallocated_output, int runtime_offsets, thor_stream_t stream);
void thor_stamped_segmented_reduction_destroy(thor_stamped_segmented_reduction_t r);
int thor_stamped_segmented_reduction_run(thor_stamped_segmented_reduction_t r);
thor_tensor_t thor_stamped_segmented_reduction_output(thor_stamped_segmented_reduction_t r);
size_t thor_stamped_segmented_reduction_workspace_bytes(thor_stamped_segmented_reduction_t r);
int thor_stamped_segmented_reduction_variant(thor_stamped_segmented_reduction_t r, char* buffer, size_t capacity);

/* ---- segmented broadcast (Utilities/Expression/SegmentedBroadcastKernel.h:8-12) ------------------------------------------- */
/* output[r, :] = per_segment_values[b, :] for the rows r of segment b (divided by the segment length when
 * normalize_by_segment_length is nonzero); rows of no segment are left untouched.  Enqueued on `stream`. */
int thor_segmented_broadcast(thor_tensor_t per_segment_values, thor_tensor_t segment_offsets, thor_tensor_t output,
                             int normalize_by_segment_length, thor_stream_t stream);

/* Prefix scans (Utilities/TensorOperations/Cub/CubDevicePrimitives.h:781-880,951-1012 there): prepare, allocate the temporary
 * storage and run in one call.  op: 0 sum, 1 min, 2 max, 3 product; arg != 0 (op 1 or 2): output holds UINT32 flattened indices
 * of the winning prefix element.  Segments: offsets != NULL -> the num_segments segments of an offsets tensor; else
 * segment_size > 0 -> num_items / segment_size rows; else one scan.  `variant` (may be NULL) receives how the plan runs.
 * The call returns when the scan has run (it owns the temporary storage and frees it). */
int thor_scan(thor_tensor_t input, thor_tensor_t output, thor_tensor_t offsets, uint64_t num_items, uint64_t num_segments, uint64_t segment_size,
              int op, int arg, int inclusive, int reverse, thor_stream_t stream, char* variant, size_t variant_capacity);

/* Diagnostic (no counterpart in the reference, whose scans never return a partial result either): blocks of a one-launch scan
 * read the totals of earlier chunks from each other, and every such wait is bounded so that each wavefront has an exit.  A wait
 * that gives up computes the totals it lacks from the input in the order their owners would have, so every scan entry point -
 * thor_scan, thor_scan_no_alloc, the plan / run functions of CubDevicePrimitives.h, the Scan stage of a stamped Expression -
 * returns complete results, the same bits, whether or not a wait gave up.  This returns how many waits did so over all
 * thor_scan calls of the process so far (0 in normal operation: a block only waits for blocks that started before it). */
uint64_t thor_scan_waits_recovered(void);

/* Select-flagged (Utilities/TensorOperations/Cub/CubDevicePrimitives.h:87-93,490-516 there): output receives the elements of input
 * whose flag (BOOLEAN or UINT8) is nonzero, in input order, and *num_selected_out (UINT32) their number; prepare, allocate the
 * temporary storage and run in one call.  num_items == 0 writes a zero count. */
int thor_select_flagged(thor_tensor_t input, thor_tensor_t flags, thor_tensor_t output, thor_tensor_t num_selected_out, uint64_t num_items,
                        thor_stream_t stream, char* variant, size_t variant_capacity);

/* Top-k (CubDevicePrimitives.h:47-85,357-488 there): the k largest (largest != 0) or smallest keys, unordered; values_in /
 * values_out (UINT32, both or neither) travel with their keys.  segmented == 0: one selection over the first segment_size keys
 * (num_segments is ignored), k capped at that count.  segmented != 0: num_segments rows of segment_size <= 8192 keys each,
 * k < segment_size keys of every row written row after row. */
int thor_topk(thor_tensor_t keys_in, thor_tensor_t keys_out, thor_tensor_t values_in, thor_tensor_t values_out, uint64_t num_segments,
              uint64_t segment_size, uint64_t k, int largest, int segmented, thor_stream_t stream, char* variant, size_t variant_capacity);

/* The plan / temporary-storage / run protocol of the same primitives (prepareCubDevice..., ...TempBytes and the run functions that take
 * a plan, CubDevicePrimitives.h:357-516 there): prepare once, keep a UINT8 temporary-storage tensor of at least
 * thor_selection_plan_temp_bytes bytes (several plans may share the largest), run any number of times with nothing allocated.
 * thor_selection_plan_run takes the tensors in the order of the prepare call that made the plan: (input, flags, output,
 * num_selected_out) or (keys_in, keys_out, values_in, values_out; the values NULL for key-only plans). */
thor_selection_plan_t thor_select_flagged_prepare(thor_tensor_t input, thor_tensor_t flags, thor_tensor_t output, thor_tensor_t num_selected_out,
                                                  uint64_t num_items);
thor_selection_plan_t thor_topk_prepare(thor_tensor_t keys_in, thor_tensor_t keys_out, thor_tensor_t values_in, thor_tensor_t values_out,
                                        uint64_t num_segments, uint64_t segment_size, uint64_t k, int largest, int segmented);
size_t thor_selection_plan_temp_bytes(thor_selection_plan_t plan);
int thor_selection_plan_run(thor_selection_plan_t plan, thor_tensor_t temp_storage, thor_tensor_t a, thor_tensor_t b, thor_tensor_t c, thor_tensor_t d,
                            thor_stream_t stream);
int thor_selection_plan_variant(thor_selection_plan_t plan, char* buffer, size_t capacity);
void thor_selection_plan_destroy(thor_selection_plan_t plan);

/* thor_scan for callers that cannot allocate (work recorded under stream capture, serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  Same arguments, kernels and results as thor_scan, but the temporary
 * storage (segment-head bitmap, the totals that chunks publish to each other) is a fixed 4 MiB block of device memory that is part of the library's
 * code object, and nothing is compiled or loaded: no hipMalloc, hipFree, hipRTC or module load happens in this call.
 *   - The kernels of the request (dtype, operation, mode, direction, sizes, pointer alignment) must have been loaded by an earlier
 *     thor_scan (or a stamped Expression scan) with the same request in this process; otherwise the call fails and says so.
 *   - Requests that need more than 4 MiB of temporary storage fail with a message that gives both sizes.  Flat and row scans
 *     need about 16 bytes per chunk of 4 096 to 32 768 elements (fp32: up to ~2^31 elements); offset-segmented scans add one
 *     bit per element (up to ~2^24 elements).
 *   - Every call on one GPU uses that GPU's block.  A call leaves nothing behind that a later call depends on (the bitmap
 *     and the block of totals are cleared by the call's own first kernel), but two calls that overlap
 *     in time on one GPU - different streams, different threads - race on the block. */
int thor_scan_no_alloc(thor_tensor_t input, thor_tensor_t output, thor_tensor_t offsets, uint64_t num_items, uint64_t num_segments,
                       uint64_t segment_size, int op, int arg, int inclusive, int reverse, thor_stream_t stream, char* variant,
                       size_t variant_capacity);

/* ---- Expression (Utilities/Expression/Expression.h:516-1075) ------------------------------------------------------------- */
/* dtype arguments: a DataType code, or -1 for "not specified" */
thor_expr_t thor_expr_input(const char* name, int compute_dtype, int output_dtype);
thor_expr_t thor_expr_runtime_scalar(const char* name, int compute_dtype, int output_dtype);
thor_expr_t thor_expr_scalar(double value);
thor_expr_t thor_expr_fill(double value, const uint64_t* dims, int rank, int output_dtype);
/* `method` is the C++ method name: "add", "sub", "mul", "div", "pow", "min", "max", "equal", "notEqual", "lessThan",
 * "lessEqual", "greaterThan", "greaterEqual", "logicalAnd", "logicalOr" (binary); "neg", "logicalNot", "abs", "exp",
 * "sigmoid", "gelu", ... (unary; every unary method of Expression) */
thor_expr_t thor_expr_binary(const char* method, thor_expr_t lhs, thor_expr_t rhs);
/* Ragged batches (Expression::segmentedReduceWithRaggedMetadata / segmentedBroadcast / withRaggedRuntimeExtent): `method` is
 * "segment_sum", "segment_min", "segment_max", "segment_mean" (batch_size and max_active_values both zero = take them from the
 * bound tensors), "segmented_broadcast", "segmented_broadcast_normalized" or "ragged_extent". */
thor_expr_t thor_expr_ragged(const char* method, thor_expr_t values, thor_expr_t offsets, uint64_t batch_size, uint64_t max_active_values,
                             uint64_t elements_per_value);
thor_expr_t thor_expr_unary(const char* method, thor_expr_t input);
/* methods with numeric parameters: "elu"(alpha), "hardTanh"(min,max), "threshold"(threshold,value), "log"(base),
 * "clamp"(lo,hi) */
thor_expr_t thor_expr_unary_params(const char* method, thor_expr_t input, double p0, double p1);
thor_expr_t thor_expr_where(thor_expr_t condition, thor_expr_t true_value, thor_expr_t false_value);
thor_expr_t thor_expr_cast(thor_expr_t input, int dtype);
thor_expr_t thor_expr_with_dtypes(thor_expr_t input, int compute_dtype, int output_dtype);
/* `method`: "reduce_sum", "reduce_prod", "reduce_min", "reduce_max", "reduce_mean", "reduce_norm1", "reduce_norm2",
 * "argmin", "argmax"; num_axes == 0 reduces all axes; squeeze axis UINT64_MAX squeezes every singleton axis */
thor_expr_t thor_expr_reduce(const char* method, thor_expr_t input, const uint64_t* axes, int num_axes, const uint64_t* squeeze_axes,
                             int num_squeeze_axes);
/* Expression::stridedView: dims / strides / offset in elements of the operand's storage ("transpose" is a unary method). */
thor_expr_t thor_expr_strided_view(thor_expr_t input, const uint64_t* dims, const uint64_t* strides, int rank, uint64_t element_offset);
/* Expression::scan / segmentedScan (Expression.h:640-700 there): op 0 sum, 1 min, 2 max, 3 product, 4 arg-min, 5 arg-max;
 * offsets == NULL: scan along the last axis (axis -1 or its index); else a scan over the segments of the offsets expression */
thor_expr_t thor_expr_scan(thor_expr_t input, thor_expr_t offsets, int op, int64_t axis, int inclusive, int reverse);
/* Expression::takeAlongAxis(indices, axis) (Expression.h:676-677 there); axis = -1 is the last axis */
thor_expr_t thor_expr_take_along_axis(thor_expr_t input, thor_expr_t indices, int64_t axis);
/* Expression::rotaryPositionEmbedding and its WithPositionIds / WithEffectiveSequenceLength forms (Expression.h:196-218 options,
 * :650-675 builders there).  position_ids and effective_sequence_length may be NULL.  scaling_kind: 0 none, 1 linear, 2 dynamic
 * NTK, 3 YaRN, 4 LongRoPE, 5 Llama 3.  attention_factor <= 0 asks for the scaling kind's own; output_dtype / compute_dtype < 0
 * leave the choice to dtype resolution. */
typedef struct thor_rope_options {
    uint32_t sequence_axis;
    uint32_t head_dim_axis;
    uint64_t rotary_dim;
    double base;
    int64_t position_offset;
    int interleaved;
    int inverse;
    int scaling_kind;
    double scaling_factor;
    uint64_t original_max_position_embeddings;
    double attention_factor;
    double yarn_beta_fast;
    double yarn_beta_slow;
    double llama3_low_freq_factor;
    double llama3_high_freq_factor;
    const double* long_rope_short_factors;
    const double* long_rope_long_factors;
    uint64_t num_long_rope_factors;
    int output_dtype;
    int compute_dtype;
} thor_rope_options;
thor_expr_t thor_expr_rope(thor_expr_t input, thor_expr_t position_ids, thor_expr_t effective_sequence_length, const thor_rope_options* options);
thor_expr_t thor_expr_reshape(thor_expr_t input, const uint64_t* dims, int rank);
thor_expr_t thor_expr_unsqueeze(thor_expr_t input, const uint64_t* axes, int num_axes);
thor_expr_t thor_expr_squeeze(thor_expr_t input, const uint64_t* axes, int num_axes);
void thor_expr_destroy(thor_expr_t expr);
int thor_expr_num_nodes(thor_expr_t expr);
int thor_expr_canonical(thor_expr_t expr, char* buffer, size_t capacity, size_t* needed);

/* Expression::outputs({{name, expr}, ...}) */
thor_outputs_t thor_outputs_create(const char* const* names, const thor_expr_t* exprs, int count);
void thor_outputs_destroy(thor_outputs_t outputs);
/* Outputs::ifElse / ifElifElse (Expression.h:474-483 there): name by name the then-branch's value where the single-element predicate is
 * nonzero, else the next branch whose predicate is nonzero, else the else-branch.  num_elif may be 0 (plain if / else). */
thor_outputs_t thor_outputs_conditional(thor_expr_t predicate, thor_outputs_t then_outputs, const thor_expr_t* elif_predicates,
                                        const thor_outputs_t* elif_outputs, int num_elif, thor_outputs_t else_outputs);

/* ---- FusedEquation (Utilities/Expression/FusedEquation.h:574-632) --------------------------------------------------------- */
thor_fused_equation_t thor_fused_equation_compile(thor_outputs_t outputs, int device_num);
/* FusedEquation::compileBackward (Utilities/Expression/FusedEquation.h:580-586): the equation of the gradients "<input>_grad"
 * of `wrt_names` (all tensor inputs when num_wrt is 0).  num_upstream == 0: implicit ones as the upstream gradient of the single
 * output.  upstream_output_names == NULL and num_upstream == 1: upstream_input_names[0] names the upstream gradient input of the
 * single output.  Otherwise upstream_input_names[i] is the upstream gradient input of forward output upstream_output_names[i]. */
thor_fused_equation_t thor_fused_equation_compile_backward(thor_fused_equation_t eq, const char* const* wrt_names, int num_wrt,
                                                           const char* const* upstream_output_names, const char* const* upstream_input_names,
                                                           int num_upstream, int accumulate_grad_outputs);
void thor_fused_equation_destroy(thor_fused_equation_t eq);
int thor_fused_equation_num_outputs(thor_fused_equation_t eq);
int thor_fused_equation_output_name(thor_fused_equation_t eq, int index, char* buffer, size_t capacity);
/* FusedEquation::stamp(inputs, stream, {}, preallocated_outputs) */
thor_plan_t thor_fused_equation_stamp(thor_fused_equation_t eq, const char* const* input_names, const thor_tensor_t* inputs, int num_inputs,
                                      const char* const* preallocated_names, const thor_tensor_t* preallocated, int num_preallocated,
                                      thor_stream_t stream);
/* The same with tensorRuntimeScalar inputs bound to one element of a device buffer each (TensorScalarBinding,
 * Utilities/Expression/CompiledEquation.h:15-19 there): scalar_buffers[i] at scalar_byte_offsets[i], read as scalar_dtypes[i]. */
thor_plan_t thor_fused_equation_stamp_with_tensor_scalars(thor_fused_equation_t eq, const char* const* input_names, const thor_tensor_t* inputs,
                                                          int num_inputs, const char* const* scalar_names, const thor_tensor_t* scalar_buffers,
                                                          const uint64_t* scalar_byte_offsets, const int* scalar_dtypes, int num_scalars,
                                                          const char* const* preallocated_names, const thor_tensor_t* preallocated,
                                                          int num_preallocated, thor_stream_t stream);
/* Expression::tensorRuntimeScalar(name, compute_dtype, output_dtype) */
thor_expr_t thor_expr_tensor_runtime_scalar(const char* name, int compute_dtype, int output_dtype);
/* FusedEquation::run(inputs, scalar_inputs, outputs, stream): compile-if-needed and launch into caller tensors */
int thor_fused_equation_run(thor_fused_equation_t eq, const char* const* input_names, const thor_tensor_t* inputs, int num_inputs,
                            const char* const* scalar_names, const float* scalars, int num_scalars, const char* const* output_names,
                            const thor_tensor_t* outputs, int num_outputs, thor_stream_t stream);
/* FusedEquation::getOutputShapes / getOutputDataTypes for one named output */
int thor_fused_equation_output_shape(thor_fused_equation_t eq, const char* const* input_names, const thor_tensor_t* inputs, int num_inputs,
                                     const char* output_name, uint64_t* dims_out, int* rank_out, int* dtype_out);

/* ---- StampedExecutionPlan (Utilities/Expression/StampedEquation.h:1659-1780) ---------------------------------------------- */
void thor_plan_destroy(thor_plan_t plan);
int thor_plan_run(thor_plan_t plan);
int thor_plan_run_with_scalars(thor_plan_t plan, const char* const* scalar_names, const float* scalars, int num_scalars);
int thor_plan_run_on(thor_plan_t plan, thor_stream_t stream);
thor_tensor_t thor_plan_output(thor_plan_t plan, const char* name);
int thor_plan_num_stages(thor_plan_t plan);
/* StampedExecutionPlan::stageKindNames: "FusedKernel", "Reduction", "ArgMinMax", ... */
int thor_plan_stage_kind(thor_plan_t plan, int stage, char* buffer, size_t capacity);
/* generated HIP source of a stage's kernel (diagnostics and tests) */
int thor_plan_stage_source(thor_plan_t plan, int stage, char* buffer, size_t capacity, size_t* needed);
int thor_plan_stage_description(thor_plan_t plan, int stage, char* buffer, size_t capacity);
uint64_t thor_plan_flop_count(thor_plan_t plan);
/* number of run-time compilations since process start (cache-behaviour tests) */
uint64_t thor_compiled_kernel_count(void);

#ifdef __cplusplus
}
#endif
#endif /* THOR_C_API_H */
