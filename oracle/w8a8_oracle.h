/*
 * CPU restatement of the reference's W8A8 linear arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this file; it exists so the HIP path can be checked against an
 * independent scalar statement of the reference contract, and so a CPU
 * baseline can be timed next to the GPU.  Each function names the reference
 * file:line it restates (paths relative to the reference tree's native/).
 *
 * Parity status: every function below is pinned by the reference's own
 * known-answer vectors (tests/golden/reference_kats.json) and, where the
 * reference tree is available, by a byte comparison against the reference C
 * compiled from its own sources (oracle/_ref).  The optional f32 bias of
 * vxo_qlinear_rowscale_i8u8 has no reference counterpart (the reference's
 * requantizing linear has an accumulator-domain bias only), so no reference
 * vector can cover it; it is pinned instead by what its definition fixes:
 * hand-derived cases in which another order of the additions, a single
 * rounding or a reciprocal product give a different byte, and a seeded sweep
 * against the rule evaluated in exact rationals with explicit roundings
 * (tests/test_oracle.py).  With the bias absent the function is the
 * reference's per-row call and is pinned like the rest.
 */
#ifndef VXO_W8A8_ORACLE_H
#define VXO_W8A8_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Canonical dtype ids (include/volvoxai_enums.h:479-480). */
#define VXO_DTYPE_U8 5u
#define VXO_DTYPE_I8 6u

/* src/kernels/w8a8_affine.h:114-120 */
int32_t vxo_round_ties_even(float value);
/* src/kernels/w8a8_affine.h:125-131 */
int32_t vxo_requantize(float transformed, int32_t minimum, int32_t maximum,
                       int32_t nan_value);
/* src/kernels/w8a8_affine.h:139-144 */
float vxo_transform_accumulator(int64_t accumulator, float multiplier,
                                int32_t output_zero_point);
/* src/kernels/w8a8_affine.h:169-181 and src/backends/qlinear_multiplier.h:12-27 */
int vxo_multiplier(float input_scale, float weight_scale, float output_scale,
                   float* multiplier_out);

/* src/kernels/portable_inference_kernels.inc:968-1032.  Returns 1 handled,
 * 0 declined.  `accumulators`, when non-NULL, receives the int32 accumulator
 * (bias included) of every output element, row-major [rows, d_out]. */
int vxo_qlinear_i8u8(const void* input, const void* weight,
                     const int32_t* bias, const float* weight_scales,
                     const int32_t* weight_zero_points, void* output,
                     int32_t* accumulators, uint32_t rows, uint32_t d_in,
                     uint32_t d_out, float input_scale,
                     int32_t input_zero_point, float output_scale,
                     int32_t output_zero_point, uint32_t input_dtype,
                     uint32_t weight_dtype, uint32_t output_dtype);

/* Per-token activation scales: row m is its own reference QLinear call with
 * input_scale = row_scales[m], input zero point 0, I8 input
 * (portable_inference_kernels.inc:968-1032 called with rows = 1).  bias_i32
 * (may be NULL = 0) is the reference's accumulator-domain bias.  bias_f32
 * (may be NULL) is an EXTENSION with no reference counterpart: after the
 * reference transform t = f32(f32(acc)*mult) + f32(zp), the term
 * f32(bias_f32[n] / output_scale) is added with one more f32 rounding before
 * the saturating round.  With bias_f32 == NULL the bytes are the reference's.
 * A bias that is not finite declines the call, like an invalid scale. */
int vxo_qlinear_rowscale_i8u8(const int8_t* input, const void* weight,
                              const int32_t* bias_i32, const float* bias_f32,
                              const float* weight_scales,
                              const int32_t* weight_zero_points, void* output,
                              int32_t* accumulators, uint32_t rows,
                              uint32_t d_in, uint32_t d_out,
                              const float* row_scales, float output_scale,
                              int32_t output_zero_point, uint32_t weight_dtype,
                              uint32_t output_dtype);

/* src/kernels/packed_linear.h:108-116 */
int32_t vxo_packed_round_i8(float value);
/* Activation preparation of PackedLinear under DYNAMIC_I8
 * (src/kernels/packed_linear_ops.inc:1574-1597, 97-153).  Returns the
 * "finite" flag; on a non-finite row `prepared` is zeroed. */
int vxo_packed_prepare_i8(const float* input, uint32_t k, int8_t* prepared,
                          float* scale);

/* PackedLinear W8 / DYNAMIC_I8 (src/kernels/packed_linear_ops.inc:1545-1621,
 * row body :1493-1534).  packed: offset-binary I32 words [n, ceil(k/4)],
 * scales [n, ceil(k/group)], bias [n] or NULL, output [rows, n].
 * Returns 0 on success, -1 on a rejected descriptor (reference convention). */
int vxo_packed_linear_forward(const float* input, const uint32_t* packed,
                              const float* scales, const float* bias,
                              float* output, uint64_t rows, uint32_t k,
                              uint32_t n, uint32_t group_size);

/* Same arithmetic with the activation codes and per-row scales injected
 * (the "prepared A8" form the reference's CUDA route keeps in x[4]/x[5],
 * src/kernels/llm_ops.h:30-32).  row_finite may be NULL (all rows finite).
 * accumulators (optional) receives the full-K int32 sum of the group dots,
 * [rows, n]. */
int vxo_packed_linear_a8(const int8_t* activation, const float* row_scales,
                         const uint8_t* row_finite, const uint32_t* packed,
                         const float* scales, const float* bias, float* output,
                         int32_t* accumulators, uint64_t rows, uint32_t k,
                         uint32_t n, uint32_t group_size);

/* The same two routines for every packed width (weight_bits 2, 3, 4 or 8):
 * I32 words [n, vx_packed_words(k, bits)] (src/kernels/packed_linear_ops.inc:
 * 246-248); codes offset by half their range, lowest bits first, W3 a dense
 * bitstream (:249-254; integer dot :472-480; single-row body :1493-1504). */
int vxo_packed_linear_forward_bits(const float* input, const uint32_t* packed,
                                   const float* scales, const float* bias,
                                   float* output, uint64_t rows, uint32_t k,
                                   uint32_t n, uint32_t group_size,
                                   uint32_t weight_bits);
/* vx_packed_linear_forward restricted to its output window (VxLLMOpArgs
 * first_unit / unit_count, src/kernels/llm_ops.h:48-52; the bounds check, the row
 * range and the per-row column range of src/kernels/packed_linear_ops.inc:
 * 1550-1553, 1555, 1593-1596): units are elements of the row-major output,
 * unit_count 0 = all rows * n, elements outside the window are not written.
 * Pinned by the reference's own window cases (native/tests/
 * test_packed_linear_i8.c:186-188 and :263-278) against oracle/_ref. */
int vxo_packed_linear_forward_window(const float* input, const uint32_t* packed,
                                     const float* scales, const float* bias,
                                     float* output, uint64_t rows, uint32_t k,
                                     uint32_t n, uint32_t group_size,
                                     uint32_t weight_bits, uint64_t first_unit,
                                     uint64_t unit_count);
int vxo_packed_linear_a8_bits(const int8_t* activation, const float* row_scales,
                              const uint8_t* row_finite, const uint32_t* packed,
                              const float* scales, const float* bias,
                              float* output, int32_t* accumulators,
                              uint64_t rows, uint32_t k, uint32_t n,
                              uint32_t group_size, uint32_t weight_bits);

/* src/kernels/quantize_linear_ops.inc:156-169 (scalar rule), :234-254 */
int vxo_quantize_linear(const float* input, uint32_t elements, void* output,
                        float scale, int32_t zero_point, uint32_t dtype);
/* src/kernels/quantize_linear_ops.inc:9-16, :95-128 */
int vxo_dequantize_linear(const void* input, uint32_t elements, float scale,
                          int32_t zero_point, uint32_t dtype, float* output);
/* RequantizeLinear (portable_inference_kernels.inc:2437-2463): 1 done / 0 declined. */
int vxo_requantize_linear(const void* input, uint32_t elements, float input_scale,
                          int32_t input_zero_point, float output_scale, int32_t output_zero_point,
                          uint32_t input_dtype, uint32_t output_dtype, void* output);

/* src/training/quantization.c:142-160: symmetric per-tensor activation scale
 * s = f32(max|x| / 127.0) computed in double; 1.0 for an all-zero tensor. */
int vxo_ptq_symmetric_scale(const float* values, int64_t count, float* scale);
/* src/training/quantization.c:186-211: q = clamp(rne(x / s + zp)) in double. */
int vxo_ptq_quantize_i8(const float* values, int64_t count, float scale,
                        int32_t zero_point, int8_t* output);
/* src/training/quantization.c:391-414 */
int vxo_ptq_pack_bias_i32(const float* values, int32_t count,
                          float input_scale, const float* weight_scales,
                          int32_t* output);

/* docs/packed-linear-design.md:24-28: offset-binary W8 codes, LSB first. */
void vxo_pack_w8_words(const int8_t* weight, uint32_t n, uint32_t k,
                       uint32_t* packed);
/* W4 codes (values -8..7, stored +8), eight per word, lowest nibble first
 * (src/kernels/packed_linear_ops.inc:476-477). */
void vxo_pack_w4_words(const int8_t* weight, uint32_t n, uint32_t k,
                       uint32_t* packed);

/* src/kernels/embedding.inc:5-16 (ids must lie inside the table) */
void vxo_embedding_f32(const int32_t* tokens, const float* table, float* out,
                       uint32_t count, uint32_t d_model);
/* argmax_axis_typed with inner == 1 (src/kernels/reduction_argmax.inc:211-235) */
void vxo_argmax_rows_f32(const float* input, uint32_t rows, uint32_t n,
                         int32_t* indices);

/* Codes of any packed width below 8 (values in [-2^(bits-1), 2^(bits-1)) stored
 * + 2^(bits-1)), the layout packed_code() reads; the tail holds the zero code. */
void vxo_pack_low_bit_words(const int8_t* weight, uint32_t n, uint32_t k,
                            uint32_t bits, uint32_t* packed);

#ifdef __cplusplus
}
#endif
#endif
