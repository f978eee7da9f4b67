/*
 * vxhip_w8a8 -- MI355X (gfx950) W8A8 linear backend, C ABI.
 *
 * Plain C, no HIP types: every pointer is either a host pointer or an opaque
 * device address (void*), every handle is an opaque struct.  A C host (the
 * backend provider in volvoxai_amd/provider/) or any FFI can bind this header
 * directly.  File:line citations name the reference interface each entry
 * point stands in for (paths relative to the reference's native/ directory).
 *
 * Return convention: functions that mirror a reference kernel slot keep that
 * slot's convention (1 = handled, 0 = declined before any side effect, exactly
 * like VxQLinearI8U8Fn).  All other entry points return a VxHipStatus whose
 * values equal the reference's VxStatus codes (include/volvoxai_enums.h:264-288)
 * so a provider can return them unchanged.  vxhip_last_error() gives the
 * calling thread's last failure text.
 *
 * Scopes follow the provider contract (docs/backend-sdk.md:77-95):
 *   VxHipQLinear / VxHipPackedLinear  compiled scope, immutable after create,
 *                                     shareable by concurrent contexts;
 *   VxHipContext                      context scope, owns a stream and the
 *                                     mutable scratch; one thread at a time.
 */
#ifndef VXHIP_W8A8_H
#define VXHIP_W8A8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VXHIP_ABI_VERSION 1u

/* Canonical dtype ids (include/volvoxai_enums.h:479-480). */
#define VXHIP_DTYPE_U8 5u
#define VXHIP_DTYPE_I8 6u

typedef int32_t VxHipStatus;
#define VXHIP_OK                     0
#define VXHIP_INVALID_ARGUMENT      (-1)
#define VXHIP_OUT_OF_MEMORY         (-2)
#define VXHIP_BACKEND_UNAVAILABLE   (-6)
#define VXHIP_BACKEND_UNSUPPORTED   (-7)
#define VXHIP_EXECUTION_FAILED      (-10)
#define VXHIP_DEVICE_LOST           (-12)
#define VXHIP_INTERNAL              (-16)

typedef struct VxHipContext VxHipContext;
typedef struct VxHipQLinear VxHipQLinear;
typedef struct VxHipPackedLinear VxHipPackedLinear;

/* ---- library / device ------------------------------------------------- */

uint32_t vxhip_abi_version(void);
/* Number of visible gfx950 devices; 0 when none (a provider then answers
 * BACKEND_UNAVAILABLE from runtime_create, runtime/backend_sdk.c:206-213). */
int32_t vxhip_device_count(void);
/* "AMD Instinct MI355X (gfx950), 256 CU, ..." into buffer; VXHIP_OK or error. */
VxHipStatus vxhip_device_name(int32_t device, char* buffer, size_t capacity);
const char* vxhip_last_error(void);

/* ---- context scope ---------------------------------------------------- */

/* flags = VXHIP_CONTEXT_OWN_STREAM: the context creates and owns a stream
 * (`stream` is ignored).  flags = VXHIP_CONTEXT_BORROW_STREAM: work is enqueued
 * on the caller's hipStream_t passed as void* (NULL names the device's default
 * stream) and the caller owns its lifetime. */
#define VXHIP_CONTEXT_OWN_STREAM    0u
#define VXHIP_CONTEXT_BORROW_STREAM 1u
VxHipStatus vxhip_context_create(int32_t device, void* stream, uint32_t flags,
                                 VxHipContext** out_context);
void vxhip_context_destroy(VxHipContext* context);
VxHipStatus vxhip_context_synchronize(VxHipContext* context);

/* Recording and replay.  Between begin and end the launches this context's entry
 * points make are recorded instead of run; end hands back the recording,
 * instantiated; vxhip_replay_launch runs it on the context's stream.  The
 * reference's device route does the same with its forward pass
 * (native/src/backends/cuda/host/cuda_graph_lifecycle_host.inc:184-188
 * cuStreamBeginCapture, :236-262 instantiate and first launch, :285-290
 * replay).  What may be recorded: the *_forward*, prepare, row, attention,
 * gather and argmax entry points on device pointers, after the same calls have
 * run once unrecorded (that run sizes the context's scratch; a recording that
 * would have to grow it fails).  Not recordable: anything that copies to or from
 * the host or synchronizes (memcpy, fault_flags, the host-pointer drop-ins).
 * A replay reads and writes the device addresses of the recorded calls; values
 * that change between replays (ids, positions) live in device memory.  end with
 * out_replay NULL abandons the recording. */
typedef struct VxHipReplay VxHipReplay;
VxHipStatus vxhip_context_begin_recording(VxHipContext* context);
VxHipStatus vxhip_context_end_recording(VxHipContext* context,
                                        VxHipReplay** out_replay);
VxHipStatus vxhip_replay_launch(VxHipContext* context,
                                const VxHipReplay* replay);
void vxhip_replay_destroy(VxHipReplay* replay);
/* Kernel-variant id chosen by the last launch on this context, e.g.
 * "hip.qlinear.mfma-i8.t256x256" -- the string a provider reports as
 * route_evidence (runtime/public_api_model_lifecycle.inc:748-751). */
const char* vxhip_context_last_variant(const VxHipContext* context);
/* Device-side fault word accumulated by kernels; reading it synchronises the
 * stream.  0 = clean.  Bit 1: a requantization multiplier was not finite and
 * positive.  Bit 2: an embedding id outside the table (its row is zeros).
 * Bit 4: a cache position at or past max_seq was given to the rotary/attention
 * entry points (that token's caches and output are left untouched).  Bit 8: a
 * real-valued bias given to vxhip_qlinear_forward_rowscale was not finite.
 *
 * What the host can check it checks before anything is launched, and declines.
 * Values that live in device memory (the row scales and the real-valued bias of
 * vxhip_qlinear_forward_rowscale, token ids, cache positions) can only be checked
 * by the kernels: where the reference's CPU rule would decline the whole call
 * (src/kernels/w8a8_affine.h:169-181) the kernel raises the bit and still writes
 * output bytes, which are then meaningless.  The return value of such a call is
 * therefore provisional until this word has been read as 0.  The word is sticky:
 * it keeps every bit raised since the context was created or since the last
 * vxhip_context_clear_fault_flags. */
VxHipStatus vxhip_context_fault_flags(VxHipContext* context, uint32_t* flags);
/* Clears the fault word, ordered on the context's stream after the work already
 * enqueued (asynchronous; no counterpart in the reference). */
VxHipStatus vxhip_context_clear_fault_flags(VxHipContext* context);
/* Grows the context's scratch (activation staging, prepared rows) to at least
 * `bytes` now instead of inside a later call.  Entry points size the scratch by
 * themselves; a block that is outgrown is kept until vxhip_context_destroy, so a
 * HIP graph captured on this context stays valid when a later, larger call
 * grows it.  Reserving up front only avoids holding the outgrown blocks.  No
 * counterpart in the reference. */
VxHipStatus vxhip_context_reserve_scratch(VxHipContext* context, size_t bytes);
/* Layout of prepared activations (int8 codes) handed between entry points on
 * this context; no counterpart in the reference, whose prepared rows
 * (src/kernels/llm_ops.h:30-32) are row major.
 *   VXHIP_ACTIVATIONS_ROW_MAJOR (default): [rows, k] bytes.
 *   VXHIP_ACTIVATIONS_OPERAND32: calls with rows <= 32 exchange the codes in
 *     the order the streaming GEMV loads them: the 16-byte chunks of the rows
 *     interleaved, code j of row r at ((j / 16) * 32 + r) * 16 + j % 16.  Such a
 *     buffer ALWAYS holds 32 * ceil(k / 16) * 16 bytes, whatever `rows` is, and
 *     must be 16-byte aligned.  Calls with rows > 32 stay row major.
 * It applies to what vxhip_packed_prepare_i8, vxhip_rmsnorm_prepare_i8,
 * vxhip_add_rmsnorm_prepare_i8 and vxhip_swiglu_prepare_i8 write and to what
 * vxhip_packed_linear_forward_a8 reads.  With 32 rows the GEMVs of a decoder
 * layer run 0.5-2 us shorter each (a row-major load of one k-step touches 32
 * cache lines for its 1 KiB). */
#define VXHIP_ACTIVATIONS_ROW_MAJOR 0u
#define VXHIP_ACTIVATIONS_OPERAND32 1u
VxHipStatus vxhip_context_set_activation_layout(VxHipContext* context, uint32_t layout);
/* Bytes a prepared-activation buffer needs on this context for `rows` x k. */
size_t vxhip_context_prepared_bytes(const VxHipContext* context, uint32_t rows, uint32_t k);

/* ---- decoder glue around the PackedLinear calls ------------------------- */
/* The steps either side of the linears of a decoder layer (the components the
 * reference runs through src/kernels/softmax_rmsnorm.inc, src/kernels/llm_math.h
 * and src/kernels/attention_f32_core.h; its CUDA backend fuses the same pairs,
 * src/backends/cuda/kernels/cuda_forward_gemv_pair_kernels.inc:408,672).
 * Device pointers, asynchronous on the context's stream, f32 row-major. */

/* RMSNorm of rows [rows, d] (double accumulation and scaling, one rounding to
 * f32: softmax_rmsnorm.inc:3-17) followed by the activation preparation of
 * vxhip_packed_prepare_i8 on the normalized row.  normalized_dev may be NULL. */
VxHipStatus vxhip_rmsnorm_prepare_i8(VxHipContext* context, const float* input_dev,
                                     const float* gain_dev, uint32_t rows, uint32_t d,
                                     double eps, int8_t* prepared_dev,
                                     float* row_scales_dev, float* normalized_dev);
/* The same after the residual add: residual_dev [rows, d] += delta_dev in place
 * (one f32 add per element), then RMSNorm and preparation of the updated rows. */
VxHipStatus vxhip_add_rmsnorm_prepare_i8(VxHipContext* context, float* residual_dev,
                                         const float* delta_dev, const float* gain_dev,
                                         uint32_t rows, uint32_t d, double eps,
                                         int8_t* prepared_dev, float* row_scales_dev);
/* silu(gate) * up of gate_up [rows, 2*inter] (gate first), then the same
 * preparation.  activated_dev [rows, inter] may be NULL. */
VxHipStatus vxhip_swiglu_prepare_i8(VxHipContext* context, const float* gate_up_dev,
                                    uint32_t rows, uint32_t inter, int8_t* prepared_dev,
                                    float* row_scales_dev, float* activated_dev);
/* Non-interleaved rotary embedding (llm_math.h:256-274) of the q and k heads of
 * qkv [rows, t, (q_heads + 2*kv_heads) * head_dim] with cos/sin tables
 * [max_seq, head_dim], token i of every row at cache slot positions_dev[i];
 * rotated q to q_out [rows, t, q_heads, head_dim], rotated k and plain v into the
 * caches [rows, kv_heads, max_seq, head_dim]. */
VxHipStatus vxhip_rope_append_kv(VxHipContext* context, const float* qkv_dev,
                                 const float* cos_dev, const float* sin_dev,
                                 const int64_t* positions_dev, uint32_t rows, uint32_t t,
                                 uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                                 uint32_t max_seq, float* q_out_dev, float* k_cache_dev,
                                 float* v_cache_dev);
/* Grouped-query attention of q [rows, t, q_heads, head_dim] over the caches:
 * scores q.k * f32(1/sqrt(head_dim)), slots 0..positions_dev[i] visible to
 * token i, softmax, P.V; out [rows, t, q_heads * head_dim]. */
VxHipStatus vxhip_gqa_attention(VxHipContext* context, const float* q_dev,
                                const float* k_cache_dev, const float* v_cache_dev,
                                const int64_t* positions_dev, uint32_t rows, uint32_t t,
                                uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                                uint32_t max_seq, float* out_dev);

/* One decode step (one new token per row) of the two entry points above in a
 * single launch: rotates the q heads and the new k of qkv [rows, (q_heads +
 * 2*kv_heads) * head_dim] at cache slot position_dev[0], appends the rotated k
 * and the v to the caches at that slot, and attends over slots 0..position.
 * out [rows, q_heads * head_dim] holds the same bits as vxhip_rope_append_kv
 * followed by vxhip_gqa_attention with t = 1. */
VxHipStatus vxhip_rope_gqa_attention_decode(VxHipContext* context, const float* qkv_dev,
                                            const float* cos_dev, const float* sin_dev,
                                            const int64_t* position_dev, uint32_t rows,
                                            uint32_t q_heads, uint32_t kv_heads,
                                            uint32_t head_dim, uint32_t max_seq,
                                            float* k_cache_dev, float* v_cache_dev,
                                            float* out_dev);

/* Embedding lookup (src/kernels/embedding.inc:5-16): out [count, d_model] row i
 * = table [vocab, d_model] row tokens_dev[i] (int32 ids as in the reference).
 * An id outside the table gives a zero row and raises fault bit 2 of
 * vxhip_context_fault_flags (the reference reads out of bounds there). */
VxHipStatus vxhip_embedding_gather_f32(VxHipContext* context, const int32_t* tokens_dev,
                                       const float* table_dev, uint32_t count,
                                       uint32_t d_model, uint32_t vocab, float* out_dev);
/* ArgMax over the last axis of input [rows, n] (argmax_axis_typed with inner 1,
 * src/kernels/reduction_argmax.inc:211-235): strictly-greater scan, so the first
 * index wins ties, a NaN is never chosen and a NaN in element 0 keeps index 0.
 * indices_dev int32 [rows].  advance_dev (optional, no counterpart in the
 * reference) are up to 64 int64 counters incremented by one in the same launch:
 * a greedy decode loop keeps its position on the device that way. */
VxHipStatus vxhip_argmax_rows_f32(VxHipContext* context, const float* input_dev,
                                  uint32_t rows, uint32_t n, int32_t* indices_dev,
                                  int64_t* advance_dev, uint32_t advance_count);

/* Measurement aid with no counterpart in the reference: runs a register-only
 * v_mfma_i32_32x32x32_i8 loop (16 accumulators per wave, one wave per SIMD,
 * `rounds` x 16 MFMAs per wave) and reports the int8 rate it reached, the
 * shader clock it ran at and the launch time.  flags bit 0 feeds random 8-bit
 * operand bytes instead of constants; the clock the device then sustains is
 * the ceiling of any int8 GEMM on such data.  flags bit 1 runs the loop on
 * v_mfma_i32_16x16x64_i8 instead (two waves per SIMD with 16 accumulators of
 * four registers each: the same operations per round and SIMD), the
 * instruction of the large GEMM tiles.
 * Synchronises the context's stream. */
VxHipStatus vxhip_probe_mfma_rate(VxHipContext* context, uint32_t rounds,
                                  uint32_t flags, double* tops,
                                  double* shader_mhz, double* microseconds);
/* Its HBM counterpart, also without a counterpart in the reference: `launches`
 * launches of a kernel that only reads, each one whole buffer of bytes_each
 * bytes (16-byte aligned device pointers, taken in rotation so that a buffer
 * smaller than the 256 MB Infinity Cache is not served from it), timed
 * back to back; reports the rate per launch and the time of one.  This is the
 * ceiling of a bandwidth-bound kernel of that size on this device, launch ramp
 * and drain included.  Synchronises the context's stream. */
VxHipStatus vxhip_probe_stream_read(VxHipContext* context, const void* const* buffers_dev,
                                    uint32_t buffer_count, size_t bytes_each,
                                    uint32_t launches, double* gigabytes_per_second,
                                    double* microseconds);

/* A third measurement aid without a counterpart in the reference: whether the
 * matrix and the vector instructions of a SIMD run beside each other, which
 * bounds the dequantizing GEMM (two MFMAs and twelve vector instructions per
 * result tile and scale group of 128).  Four launches of `rounds` rounds, four
 * waves per SIMD, random operand bytes: [0] the MFMAs of a 64 x 32 wave tile
 * alone, [1] the folds of its accumulators alone, [2] both in every wave, [3]
 * even waves the MFMAs and odd waves the folds (half the work of each kind).
 * microseconds[4] and shader_mhz[4] (optional) receive time and clock of each.
 * constant_operands != 0: every operand byte is 1 instead of random (the matrix
 * pipes then draw less power and the clock stays higher).
 * Synchronises the context's stream. */
VxHipStatus vxhip_probe_mfma_valu_overlap(VxHipContext* context, uint32_t rounds,
                                          uint32_t constant_operands,
                                          double* microseconds,
                                          double* shader_mhz);

/* Device memory for hosts without HIP headers. */
VxHipStatus vxhip_device_malloc(size_t bytes, void** out_device_pointer);
void vxhip_device_free(void* device_pointer);
VxHipStatus vxhip_memcpy_to_device(VxHipContext* context, void* device_dst,
                                   const void* host_src, size_t bytes);
VxHipStatus vxhip_memcpy_to_host(VxHipContext* context, void* host_dst,
                                 const void* device_src, size_t bytes);

/* ---- QLinear / QMatMul / QGemm: requantizing epilogue ------------------ */

/* Weight prepack = the reference's vx_pack_q8_weight step
 * (src/kernels/packed_quant_gemm.c:237-392), redone for the int8 MFMA operand
 * layout.  All pointers are HOST pointers and are not retained.
 *   weight  [d_out, d_in] I8/U8 row-major, weight_scales/zero_points [d_out],
 *   bias    [d_out] int32 in the accumulator domain (may be NULL = 0). */
VxHipStatus vxhip_qlinear_create(const void* weight, const float* weight_scales,
                                 const int32_t* weight_zero_points,
                                 const int32_t* bias, uint32_t d_in,
                                 uint32_t d_out, uint32_t weight_dtype,
                                 VxHipQLinear** out_linear);
void vxhip_qlinear_destroy(VxHipQLinear* linear);
/* Bytes of device memory held by the compiled weight (attestation input). */
uint64_t vxhip_qlinear_resident_bytes(const VxHipQLinear* linear);
/* 1 if vxhip_qlinear_forward would accept these call scalars for this weight
 * (dtypes, scales, zero points, every requantization multiplier, and the int32
 * accumulator proof K*max|x-zx|*max|w-zw| + max|bias| <= INT32_MAX of
 * src/kernels/qlinear_w8a8_x86.c:80,92-99), else 0 with vxhip_last_error set.
 * Lets a provider refuse a graph at compile time, where the reference rejects
 * an unprovable fused operator (docs/w8a8-safetensors.md:158-175, item 8). */
int vxhip_qlinear_admits(const VxHipQLinear* linear, float input_scale,
                         int32_t input_zero_point, float output_scale,
                         int32_t output_zero_point, uint32_t input_dtype,
                         uint32_t output_dtype);

/* Canonical QLinear on resident buffers (the resident half of
 * cuda_graph_qlinear_i8u8, src/backends/cuda/host/
 * cuda_graph_quantized_linear_conv_host.inc:19-106; arithmetic of
 * qlinear_i8u8, src/kernels/portable_inference_kernels.inc:968-1032).
 * input_dev [rows,d_in], output_dev [rows,d_out] device pointers;
 * accumulators_dev optional int32 [rows,d_out] (bias included).
 * Asynchronous on the context stream.  Returns 1 handled / 0 declined. */
int vxhip_qlinear_forward(VxHipContext* context, const VxHipQLinear* linear,
                          const void* input_dev, void* output_dev,
                          int32_t* accumulators_dev, uint32_t rows,
                          float input_scale, int32_t input_zero_point,
                          float output_scale, int32_t output_zero_point,
                          uint32_t input_dtype, uint32_t output_dtype);

/* QLinear followed by the DequantizeLinear that reads its output, in one launch:
 * output_f32_dev [rows,d_out] = f32((q - dequant_zero_point) * dequant_scale) for
 * the byte q that vxhip_qlinear_forward writes (DequantizeLinear,
 * src/kernels/quantize_linear_ops.inc:9-16, applied in the linear's epilogue) --
 * the Q -> QLinear -> DQ sandwich of an exported W8A8 graph without the byte
 * tensor's round trip and its launch.  output_dev (optional) also receives the
 * bytes, for a graph in which another node reads them.  The dequantization
 * parameters are those of the DequantizeLinear node (in a valid package they
 * equal the tensor's output_scale / output_zero_point); a scale that is not
 * finite and positive or a zero point outside output_dtype declines.  The f32
 * values are bit-identical to vxhip_qlinear_forward + vxhip_dequantize_forward.
 * Returns 1 handled / 0 declined. */
int vxhip_qlinear_forward_dequantized(VxHipContext* context, const VxHipQLinear* linear,
                                      const void* input_dev, float* output_f32_dev,
                                      void* output_dev, uint32_t rows,
                                      float input_scale, int32_t input_zero_point,
                                      float output_scale, int32_t output_zero_point,
                                      uint32_t input_dtype, uint32_t output_dtype,
                                      float dequant_scale, int32_t dequant_zero_point);

/* The whole QuantizeLinear -> QLinear -> DequantizeLinear sandwich on resident f32
 * rows: input_f32_dev [rows,d_in] is quantized with the QLinear's own input
 * parameters (input_scale, input_zero_point, input_dtype: QuantizeLinear,
 * src/kernels/quantize_linear_ops.inc:156-169), multiplied, and written as
 * bytes (output_dev, optional) and / or dequantized f32 (output_f32_dev,
 * optional; parameters as in vxhip_qlinear_forward_dequantized) -- at least one
 * of the two.  One or two rows against weights without zero points run as one
 * launch (the streaming kernel quantizes the rows itself, route id ending in
 * "-prep"); otherwise the quantization is a launch of its own first.  The
 * results are bit-identical to the three operators in turn.
 * Returns 1 handled / 0 declined. */
int vxhip_qlinear_forward_f32(VxHipContext* context, const VxHipQLinear* linear,
                              const float* input_f32_dev, float* output_f32_dev,
                              void* output_dev, uint32_t rows,
                              float input_scale, int32_t input_zero_point,
                              float output_scale, int32_t output_zero_point,
                              uint32_t input_dtype, uint32_t output_dtype,
                              float dequant_scale, int32_t dequant_zero_point);

/* Per-token activation scales: row m behaves as its own canonical QLinear
 * call with input_scale = row_scales_dev[m], input zero point 0, I8 input.
 * bias_f32_dev (optional, [d_out]) is an extension with no reference
 * counterpart: f32(bias/output_scale) is added to the transformed value
 * before the saturating round; with it NULL the bytes equal the reference's.
 * Returns 1 handled / 0 declined. */
int vxhip_qlinear_forward_rowscale(VxHipContext* context,
                                   const VxHipQLinear* linear,
                                   const int8_t* input_dev,
                                   const float* row_scales_dev,
                                   const float* bias_f32_dev, void* output_dev,
                                   int32_t* accumulators_dev, uint32_t rows,
                                   float output_scale,
                                   int32_t output_zero_point,
                                   uint32_t output_dtype);

/* Drop-in for the VxW8A8Ops.qlinear_i8u8 slot: identical argument order and
 * meaning to VxQLinearI8U8Fn (src/backends/w8a8_device_ops.h:15-17), HOST
 * pointers, synchronous, on device 0.  The packed weight stays resident
 * between calls (see vxhip_resident_weights_clear); a call uploads the
 * activations, runs and downloads the outputs.
 * Returns 1 handled / 0 declined before any side effect. */
int vxhip_qlinear_i8u8(const void* input, const void* weight,
                       const float* weight_scales,
                       const int32_t* weight_zero_points, const int32_t* bias,
                       void* output, uint32_t rows, uint32_t d_in,
                       uint32_t d_out, float input_scale,
                       int32_t input_zero_point, float output_scale,
                       int32_t output_zero_point, uint32_t input_dtype,
                       uint32_t weight_dtype, uint32_t output_dtype);

/* ---- PackedLinear W8/W4 under DYNAMIC_I8: dequant + bias to f32 -------- */

/* packed_words [n, vx_packed_words(k, bits)] I32 words
 * (src/kernels/packed_linear_ops.inc:246-248): weight_bits 8 = offset-binary
 * bytes (code - 128), four per word; weight_bits 4 / 2 = nibbles (code - 8) /
 * bit pairs (code - 2), lowest first; weight_bits 3 = a dense bitstream over
 * the row (code - 4) (:249-254, 472-480).  scales [n, ceil(k/G)], bias [n] or
 * NULL, group_size in {32,64,128,256} (docs/packed-linear-design.md:24-32;
 * physical shapes as checked at src/runtime/engine_runtime_llm.inc:94-99).
 * Other widths return VXHIP_BACKEND_UNSUPPORTED.  HOST pointers, not retained.
 * Widths below 8 are held as four-bit weights in device memory. */
VxHipStatus vxhip_packed_linear_create(const uint32_t* packed_words,
                                       const float* scales, const float* bias,
                                       uint32_t k, uint32_t n,
                                       uint32_t group_size,
                                       uint32_t weight_bits,
                                       VxHipPackedLinear** out_linear);
void vxhip_packed_linear_destroy(VxHipPackedLinear* linear);
uint64_t vxhip_packed_linear_resident_bytes(const VxHipPackedLinear* linear);

/* Activation preparation (vx_packed_prepare_i8_*, src/kernels/
 * packed_linear_ops.inc:97-217; CUDA twin vx_packed_cuda_prepare,
 * src/backends/cuda/kernels/cuda_forward_llm_kernels.inc:195-252):
 * per-row absmax scale, round-half-even codes clamped to +-127, non-finite
 * rows flagged by a NaN scale.  Device pointers; asynchronous. */
VxHipStatus vxhip_packed_prepare_i8(VxHipContext* context,
                                    const float* input_dev, uint32_t rows,
                                    uint32_t k, int8_t* prepared_dev,
                                    float* row_scales_dev);

/* vx_packed_linear_forward with normalize==8, groups in {8, 4, 3, 2}
 * (src/kernels/packed_linear_ops.inc:1545-1621) on resident f32 rows.
 * One or two rows (the reference's single-row route, :1471-1535, which prepares
 * the row and multiplies in one call) run as one launch: the streaming kernel
 * prepares the rows itself (route id ends in "-prep"); more rows are prepared
 * by a launch of their own first.  The bits are the same either way.
 * Returns 0 on success, -1 on a rejected descriptor (reference convention). */
int vxhip_packed_linear_forward_f32(VxHipContext* context,
                                    const VxHipPackedLinear* linear,
                                    const float* input_dev, float* output_dev,
                                    uint32_t rows);

/* The same with the reference's output window (src/kernels/llm_ops.h:48-52,
 * src/kernels/packed_linear_ops.inc:1550-1553, 1593-1596) on resident tensors:
 * input_dev [rows, k] and output_dev [rows, n] are the whole tensors, units
 * [first_unit, first_unit + unit_count) of the row-major output are written
 * (unit_count 0: all of it), every other element keeps its value.  Only the
 * rows the window touches are computed; a window that begins or ends inside a
 * row is computed into the context's staging buffer and its elements copied
 * (one device-to-device copy on the context's stream).  Returns 0, or -1 for a
 * window that does not fit or a rejected descriptor. */
int vxhip_packed_linear_forward_f32_window(VxHipContext* context,
                                           const VxHipPackedLinear* linear,
                                           const float* input_dev,
                                           float* output_dev, uint32_t rows,
                                           uint64_t first_unit,
                                           uint64_t unit_count);

/* The fused single-row decode forms of the reference's device route
 * (native/src/backends/cuda/kernels/cuda_forward_gemv_pair_kernels.inc:
 * vx_cuda_rmsnorm_packed_linear_triple_decode_a8 :1136,
 * vx_cuda_rmsnorm_packed_linear_pair_silu_mul_decode_a8 :1424,
 * vx_cuda_packed_linear_pair_silu_mul_decode_a8 :408,
 * vx_cuda_packed_linear_add_decode_a8 :672), as one entry: the row operation in
 * front of the linear, the dynamic preparation, the linear and the residual add
 * behind it in ONE launch, for one or two rows.
 *   row_op VXHIP_ROW_OP_NONE:    input [rows, k]
 *          VXHIP_ROW_OP_RMSNORM: input [rows, k], gain [k], eps; the input is
 *                                f32(x * (1/sqrt(mean(x^2) + eps)) * gain), in double
 *          VXHIP_ROW_OP_SWIGLU:  input [rows, 2k] = [gate | up]; the input is
 *                                silu(gate) * up
 *   add_to_dev [rows, n] or NULL: output = add_to + (linear + bias); it may be
 *   output_dev itself (the residual stream updated in place).
 * The bits are those of the separate launches (vxhip_rmsnorm_prepare_i8 /
 * vxhip_swiglu_prepare_i8 / vxhip_packed_linear_forward_f32, then the add).
 * Returns 1 handled; 0 declined, nothing launched (more than two rows, k above
 * 4096 (8192 without RMSNorm), k below 1024 with RMSNorm, a panel count the
 * eight-wave kernel does not take): the caller runs the separate launches;
 * -1 on an invalid argument, which includes input rows that overlap the output
 * or the residual (every workgroup reads the whole rows while others already
 * store; add_to_dev == output_dev is the one overlap that is safe). */
#define VXHIP_ROW_OP_NONE 0u
#define VXHIP_ROW_OP_RMSNORM 1u
#define VXHIP_ROW_OP_SWIGLU 2u
int vxhip_packed_linear_forward_fused(VxHipContext* context,
                                      const VxHipPackedLinear* linear,
                                      const float* input_dev, uint32_t rows,
                                      uint32_t row_op, const float* gain_dev,
                                      double eps, const float* add_to_dev,
                                      float* output_dev);

/* 1 if vxhip_packed_linear_forward_fused would run a call of this description
 * (rows, row operation, with or without a residual) on this context, 0 if it
 * would decline; nothing is launched.  It is the launcher's own decision, made
 * without launching, so the two cannot disagree.  A caller that updates its
 * residual stream in place asks for every linear of a model once, up front: after
 * the first fused launch of a layer has overwritten the stream there is no way
 * back to the separate launches.  No counterpart in the reference. */
int vxhip_packed_linear_fused_takes(VxHipContext* context,
                                    const VxHipPackedLinear* linear,
                                    uint32_t rows, uint32_t row_op,
                                    int with_residual);

/* vxhip_packed_linear_forward_f32 for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): it has no counterpart in the reference.  Same arguments, same
 * arithmetic, same output bits; the prepared activations are staged in a fixed
 * 4 MiB array inside the library's device code instead of the context's
 * grow-only scratch, and the call makes no hipMalloc/hipFree.  The staging needs
 * 256 + 4 * rows (rounded up to 256) + max(rows, 32 when rows <= 32) * ceil16(k)
 * bytes; a call that needs more returns -1 with vxhip_last_error saying so
 * (for example rows = 256 at k = 14336 fits, rows = 2048 does not).  Each device
 * has one such array, shared by every context on it and keeping the last call's
 * contents: calls that overlap on one device (two streams, two threads) race.
 * The array's address is looked up when the first context on a device is
 * created, so the entry point itself performs no set-up. */
int vxhip_packed_linear_forward_f32_noalloc(VxHipContext* context,
                                            const VxHipPackedLinear* linear,
                                            const float* input_dev,
                                            float* output_dev, uint32_t rows);

/* Same arithmetic from already prepared activations (the x[4]/x[5] form of
 * src/kernels/llm_ops.h:30-32): int8 codes [rows,k] and one f32 scale per
 * row; a NaN scale marks a non-finite row (whole output row NaN).
 * accumulators_dev optional int32 [rows,n] = full-K sum of the group dots
 * (8-bit weights only). */
int vxhip_packed_linear_forward_a8(VxHipContext* context,
                                   const VxHipPackedLinear* linear,
                                   const int8_t* activation_dev,
                                   const float* row_scales_dev,
                                   float* output_dev,
                                   int32_t* accumulators_dev, uint32_t rows);

/* Field-for-field layout of the PackedLinear part of VxLLMOpArgs
 * (src/kernels/llm_ops.h:38-53) is not reproduced here; this one-shot HOST
 * entry takes the same values as plain arguments: x=input f32 [rows,k],
 * packed_weight, scale, bias (optional), y=out [rows,n], key_dim=k,
 * value_dim=n, rate=group_size, groups=weight_bits (8, 4, 3 or 2; 0 means 4
 * as in the reference), normalize=8, and the output window first_unit /
 * unit_count (src/kernels/llm_ops.h:48-52): units are elements of the row-major
 * output, [first_unit, first_unit + unit_count) are written and every other
 * element of `output` is left as it was; unit_count 0 stands for the whole
 * output ("a zero unit_count preserves whole-graph dispatch"); a window that
 * does not fit rows * n is refused (src/kernels/packed_linear_ops.inc:1550-1553).
 * `input` and `output` are the whole tensors, as in the reference.  The packed
 * weight stays resident between calls (see vxhip_resident_weights_clear).
 * Returns 0 / -1 like vx_llm_forward_f32 (src/kernels/llm_ops.inc:41-56). */
int vxhip_packed_linear_f32(const float* input, const uint32_t* packed_weight,
                            const float* scale, const float* bias,
                            float* output, uint64_t rows, int32_t key_dim,
                            int32_t value_dim, int32_t rate, int32_t groups,
                            int32_t normalize, uint64_t first_unit,
                            uint64_t unit_count);

/* The host-pointer entry points (vxhip_qlinear_i8u8, vxhip_packed_linear_f32) keep
 * the weights they are given resident on the device -- prepacked, with scales,
 * zero points and bias -- keyed by the host pointers, shape and type, as the
 * reference's device routes keep immutable inputs resident by host pointer
 * (src/backends/cuda/host/cuda_graph_quantized_linear_conv_host.inc:74-77), plus a
 * fingerprint of the bytes (the per-channel arrays whole, the weight's ends and a
 * few hundred samples), so a buffer that is refilled is packed again.  A caller
 * that rewrites individual weights in place clears the set.  Entries are dropped
 * least recently used first beyond 256 entries or VXHIP_RESIDENT_WEIGHT_BYTES
 * bytes (environment, default 4 GiB).  The two entry points may be called from
 * several threads at once: the resident set is shared, each calling thread
 * has a context of its own (stream, staging buffers), released when the
 * thread ends.  No counterpart in the reference's ABI. */
void vxhip_resident_weights_clear(void);
uint64_t vxhip_resident_weights_bytes(void);

/* ---- F32 <-> byte boundaries ------------------------------------------ */

/* VxQuantizeTypedI8U8Fn / VxDequantizeTypedI8U8Fn slots
 * (src/backends/w8a8_device_ops.h:31-32); arithmetic of
 * quantize_linear_typed / dequantize_linear_typed
 * (src/kernels/quantize_linear_ops.inc:234-254, 95-128).  HOST pointers,
 * synchronous, 1 handled / 0 declined. */
int vxhip_quantize_typed_f32_i8u8(const float* input, uint32_t elements,
                                  void* output, float scale,
                                  int32_t zero_point, uint32_t output_dtype);
int vxhip_dequantize_typed_i8u8_f32(const void* input, uint32_t elements,
                                    float scale, int32_t zero_point,
                                    uint32_t input_dtype, float* output);
/* Resident forms (device pointers, asynchronous on the context stream). */
int vxhip_quantize_forward(VxHipContext* context, const float* input_dev,
                           uint32_t elements, void* output_dev, float scale,
                           int32_t zero_point, uint32_t output_dtype);
int vxhip_dequantize_forward(VxHipContext* context, const void* input_dev,
                             uint32_t elements, float scale,
                             int32_t zero_point, uint32_t input_dtype,
                             float* output_dev);

/* RequantizeLinear, the byte-to-byte bridge between two per-tensor descriptors:
 * the VxCopyI8U8Fn slot `requantize_linear_i8u8` of VxW8A8Ops
 * (src/backends/w8a8_device_ops.h:33-34,116), arithmetic of
 * requantize_linear_i8u8 (src/kernels/portable_inference_kernels.inc:2437-2463):
 * multiplier = f32(input_scale / output_scale), then a rounded product, a
 * rounded sum with the output zero point, ties to even, saturation.  Declines
 * what the reference declines (dtypes, scales, zero points, a multiplier that is
 * not finite and positive) and, like its device forms
 * (src/backends/cuda/host/cuda_graph_quantized_boundary_shape_host.inc:246-281),
 * unequal counts and overlapping buffers.  HOST pointers, synchronous,
 * 1 handled / 0 declined; then the resident form. */
int vxhip_requantize_linear_i8u8(const void* input, uint32_t input_elements,
                                 void* output, uint32_t output_elements,
                                 float input_scale, int32_t input_zero_point,
                                 float output_scale, int32_t output_zero_point,
                                 uint32_t input_dtype, uint32_t output_dtype);
int vxhip_requantize_forward(VxHipContext* context, const void* input_dev,
                             uint32_t elements, void* output_dev,
                             float input_scale, int32_t input_zero_point,
                             float output_scale, int32_t output_zero_point,
                             uint32_t input_dtype, uint32_t output_dtype);

/* ---- kernel-variant table --------------------------------------------- */

/* Same record shape as VxKernelVariantRegistration
 * (src/generated/kernel_registry.h:75-82).  `backend` is 0
 * (VX_BACKEND_KIND_UNSPECIFIED): an external provider has no built-in kind
 * (tests/test_kernel_registry.c:60). */
typedef struct VxHipKernelVariant {
    const char* id;
    int32_t backend;
    int32_t operator_kind;
    const char* entrypoint_id;
    const char* predicate_id;
    const char* required_features;
    int32_t priority;
} VxHipKernelVariant;

const VxHipKernelVariant* vxhip_kernel_variants(size_t* out_count);

/* Tuning/diagnostic override: force a variant family by id prefix for the
 * calling thread's later launches ("" or NULL restores automatic choice).
 * A forced variant that cannot run the shape makes the launch decline. */
void vxhip_force_variant(const char* id_prefix);

#ifdef __cplusplus
}
#endif
#endif /* VXHIP_W8A8_H */
