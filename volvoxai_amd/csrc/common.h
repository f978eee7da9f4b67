// Internal declarations shared by the translation units of libvxhip_w8a8.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

#include "../../include/vxhip_w8a8.h"

namespace vxhip {

// ---- error reporting ----------------------------------------------------
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
VxHipStatus hip_status(hipError_t e, const char* what);

#define VXHIP_TRY(expr)                                            \
    do {                                                           \
        hipError_t vxhip_e_ = (expr);                              \
        if (vxhip_e_ != hipSuccess) return hip_status(vxhip_e_, #expr); \
    } while (0)

// ---- prepacked weight layout --------------------------------------------
// Signed int8 weights in MFMA operand order.  The matrix is cut into panels
// of 32 output channels and steps of 32 input channels; block (panel, step)
// is 1 KiB and holds, for lane l of a wavefront, the 16 bytes
//     W[32*panel + l%32][32*step + 16*(l/32) + 0..15]
// at byte offset 16*l.  One block is exactly one operand of
// v_mfma_i32_32x32x32_i8, and half a block pair is one operand of
// v_mfma_i32_16x16x64_i8.  Panels are padded to a multiple of 8 and steps to
// a multiple of 4 with zero weights, so tiles never need a weight-side bound.
//
// Four-bit weights (bits == 4) keep the same panels and the same 1 KiB blocks,
// but a block then covers the pair of steps (2t, 2t+1): byte j of lane l's 16
// holds W[32*panel + l%32][64*t + 16*(l/32) + j] in its low nibble and the
// weight 32 columns further on in its high nibble, both as 4-bit two's
// complement.  (w << 4) & 0xf0f0f0f0 and w & 0xf0f0f0f0 therefore turn a
// block into the two MFMA operands of its steps with every weight scaled by
// 16, which the exact integer dot undoes with an arithmetic shift.  `ksteps`
// counts blocks per panel in both forms.
struct PackedWeight {
    int8_t* data = nullptr;
    uint32_t n = 0, k = 0;
    uint32_t panels = 0;   // padded
    uint32_t ksteps = 0;   // padded; 1 KiB blocks per panel
    uint32_t bits = 8;
    size_t bytes() const { return (size_t)panels * ksteps * 1024u; }
};

constexpr uint32_t kPanelRows = 32, kStepK = 32, kPanelPad = 8, kStepPad = 4;
constexpr uint32_t kMaxGemvRows = 32;  // the MFMA operand has 32 row slots
constexpr uint32_t kMaxPrepRows = 2;   // f32 rows a GEMV workgroup prepares by itself (every workgroup repeats them; measured: one and two rows are faster that way than as two launches, four are not)

enum FaultBits : uint32_t {
    kFaultBadMultiplier = 1u,   // a requantization multiplier was not finite and positive
    kFaultBadToken = 2u,        // an embedding lookup was asked for a row outside the table
    kFaultBadPosition = 4u,     // a cache slot at or past max_seq was named: nothing read or written there
    kFaultBadBias = 8u,         // a real-valued bias of the per-token requantizing form was not finite
};

}  // namespace vxhip

struct VxHipContext {
    int device = 0;
    hipStream_t stream = nullptr;
    bool own_stream = false;
    // grow-only scratch (activation staging, per-channel parameters, prepared rows).  A block that
    // has been outgrown is kept until the context is destroyed: a HIP graph captured on this
    // context has the block's address baked into its kernel nodes and may be replayed later.
    void* scratch = nullptr;
    size_t scratch_bytes = 0;
    static constexpr int kRetiredSlots = 48;  // sizes at least double, so this is never reached
    void* retired[kRetiredSlots] = {};
    int retired_count = 0;
    uint32_t* fault_dev = nullptr;
    void* no_alloc_scratch = nullptr;  // this device's address of the fixed scratch array (api.hip), or null
    // Exhaustive exactness proofs of the short division sequences, one pair of mismatch
    // counters per divisor seen (the output scales of the calls made on this context).
    static constexpr int kDivisorSlots = 16;
    uint32_t* div_proof_dev = nullptr;          // [kDivisorSlots][2]
    uint32_t div_bits[kDivisorSlots] = {};      // bit pattern of the divisor proved in each slot
    int div_used = 0, div_next = 0;
    char last_variant[96] = "";  // a copy: the launchers' name buffers are per thread, not per context
    int cu_count = 0;
    uint32_t activation_layout = 0;  // VXHIP_ACTIVATIONS_*: what the prepare entry points write for rows <= 32
    // grow-only device staging of the host-pointer entry points' activations and outputs
    void* io_in = nullptr;
    void* io_out = nullptr;
    size_t io_in_bytes = 0, io_out_bytes = 0;
    bool recording = false;  // between vxhip_context_begin_recording and _end_recording: launches are recorded, not run
};

// The launches a context recorded, instantiated for replay.
struct VxHipReplay {
    int device = 0;
    hipGraphExec_t executable = nullptr;
};

struct VxHipQLinear {
    int device = 0;
    vxhip::PackedWeight w;
    uint32_t weight_dtype = 0;
    float* scales = nullptr;       // [n_pad]
    int32_t* zero_points = nullptr; // [n_pad], in the signed-byte domain
    int32_t* bias = nullptr;        // [n_pad]
    int32_t* weight_sums = nullptr; // [n_pad], sum over k of the signed bytes
    bool any_zero_point = false;
    float scale_min = 0.f, scale_max = 0.f;
    int64_t weight_abs_max = 0;     // max |w - zero_point|
    int64_t bias_abs_max = 0;
    uint64_t resident = 0;
};

struct VxHipPackedLinear {
    int device = 0;
    vxhip::PackedWeight w;
    uint32_t group_size = 0, groups = 0;
    float* scales_t = nullptr;  // [groups][n_pad], transposed so 4 channels are contiguous
    float* bias = nullptr;      // [n_pad] (zeros when the node has no bias)
    bool uniform_scales = false; // every channel's group scales are bit-equal (a per-channel scale replicated over the groups)
    uint64_t resident = 0;
};

namespace vxhip {

VxHipStatus ensure_scratch(VxHipContext* ctx, size_t bytes);
void set_last_variant(VxHipContext* ctx, const char* id);

// pack.hip ------------------------------------------------------------------
// raw_dev: [n] rows of `row_stride` bytes holding k weight bytes each.
// flip: XOR 0x80 (U8 or offset-binary source -> signed byte).
VxHipStatus pack_weight(hipStream_t stream, const uint8_t* raw_dev, size_t row_stride,
                        uint32_t n, uint32_t k, bool flip, PackedWeight* out);
// raw_dev: [n] rows of `row_words` I32 words of 2-, 3- or 4-bit codes, offset by half their range,
// lowest bits first; all are stored as four-bit weights (out->bits == 4).
VxHipStatus pack_weight_nibbles(hipStream_t stream, const uint32_t* raw_dev, uint32_t row_words,
                                uint32_t n, uint32_t k, uint32_t bits, PackedWeight* out);
VxHipStatus weight_row_stats(hipStream_t stream, const uint8_t* raw_dev, size_t row_stride,
                             uint32_t n, uint32_t k, bool flip, const int32_t* zero_points_signed,
                             int32_t* sums_dev, int32_t* absmax_dev /* single word */);

// boundary.hip ---------------------------------------------------------------
VxHipStatus launch_stage_activations(hipStream_t s, const void* x, uint32_t rows, uint32_t k,
                                     bool flip, int8_t* staged, uint32_t ld, int32_t* rowsum);
// Where code j of activation row `row` lives.  Row major: row * ld + j.  Operand order (at most
// 32 rows): the row's 16-byte chunks interleaved with those of the other rows,
// ((j / 16) * 32 + row) * 16 + j % 16, which is how a wavefront of the streaming GEMV wants them:
// the 64 lanes' loads of one k-step are then 1 KiB in a row (8 cache lines) instead of 32 bytes
// from each of 32 lines.  Such a buffer always holds 32 rows of ceil(k / 16) chunks.
struct ActivationLayout {
    uint32_t ld;
    uint32_t operand_order;
};
__host__ __device__ inline size_t activation_offset(ActivationLayout layout, uint32_t row, uint32_t j) {
    return layout.operand_order ? ((size_t)(j >> 4) * 32u + row) * 16u + (j & 15u) : (size_t)row * layout.ld + j;
}
constexpr uint32_t kOperandOrderRows = 32;

VxHipStatus launch_prepare_i8(hipStream_t s, const float* x, uint32_t rows, uint32_t k,
                              int8_t* prepared, ActivationLayout layout, float* scales);
// operand-order activations (rows <= 32, k codes each) back to row-major rows of ld bytes
VxHipStatus launch_unblock_activations(hipStream_t s, const int8_t* blocked, uint32_t rows, uint32_t k,
                                       int8_t* row_major, uint32_t ld);
VxHipStatus launch_requantize(hipStream_t s, const void* x, uint32_t n, void* y, float multiplier, int32_t zp_in,
                              int32_t zp_out, bool in_i8, bool out_i8);
VxHipStatus launch_fill_u32(hipStream_t s, uint32_t* p, uint32_t count, uint32_t value);
// Counts, over every f32 mantissa of the dividend, where the one- and the two-correction
// division by `divisor` differ from IEEE division: counters[0] and counters[1].
VxHipStatus launch_division_proof(hipStream_t s, float divisor, float recip, uint32_t* counters);
VxHipStatus launch_quantize(hipStream_t s, const float* x, uint32_t n, void* y, float scale,
                            int32_t zp, bool is_i8);
VxHipStatus launch_dequantize(hipStream_t s, const void* x, uint32_t n, float scale, int32_t zp,
                              bool is_i8, float* y);

// One description for both the GEMM and the GEMV launchers.
enum class Epilogue : int { RequantTensor = 0, RequantRow = 1, DequantF32 = 2 };

struct LinearArgs {
    Epilogue mode;
    const int8_t* x;        // signed activations [rows][ldx], or in operand order (GEMV only)
    // instead of x (GEMV, rows <= kMaxPrepRows): f32 rows of ldx elements which the kernel turns into codes
    // itself -- DequantF32: the dynamic per-row preparation; RequantTensor: the QuantizeLinear in front
    // of the QLinear (input_scale, input_zp; x_f32_unsigned: that node writes U8)
    const float* x_f32;
    uint32_t x_f32_unsigned;
    uint32_t ldx;
    uint32_t x_operand_order;  // see ActivationLayout; rows <= 32
    uint32_t x_flip_mask;      // GEMV only: 0x80808080 when x holds unsigned bytes (the kernel flips their top bits), else 0
    uint32_t rows, n, k;
    const int8_t* w;        // packed
    uint32_t panels, ksteps;
    uint32_t weight_bits;   // 8, or 4 (DequantF32 only): see PackedWeight
    // requant: per-channel arrays are padded to n_pad and 16-byte aligned
    const float* wscale;    // [n_pad] weight scales
    const int32_t* bias_i32;// [n_pad] accumulator-domain bias
    const int32_t* wsum;    // [n_pad] sum over k of the signed weight bytes
    const int32_t* zw;      // [n_pad] signed-domain weight zero points, null when all are zero
    const int32_t* rowsum;  // [rows] sum of signed activations (read only with zw)
    const float* row_scale; // [rows]  RequantRow / DequantF32: activation scales
    const float* bias_row;  // [n_pad] RequantRow: optional real-valued bias
    float input_scale;      // RequantTensor
    int32_t input_zp;       // RequantTensor, signed-byte domain
    float output_scale;
    float output_scale_recip;  // RN(1 / output_scale), correctly rounded by the host
    // [2] mismatch counts of the one- / two-correction division by output_scale (zero = proved
    // exact for every dividend mantissa); null = unproved, use IEEE division
    const uint32_t* div_proof;
    bool int_bias_zero;     // bias_i32 is all zeros
    float wscale_min, wscale_max;  // extremes of wscale[0..n)
    int32_t out_zp, out_lo, out_hi;
    // dequant
    const float* scales_t;  // [groups][n_pad]
    const float* bias_f32;  // [n_pad]
    uint32_t group_size, groups, n_pad;
    bool uniform_group_scales;  // scales_t[g][n] is the same for every g: a kernel may form s_a * s_w once
    // outputs
    void* y;                // int8/uint8 [rows][n] or float [rows][n]; may be null with acc_out or dq_out
    int32_t* acc_out;       // optional int32 [rows][n]
    // requant: optional float [rows][n], the requantized value dequantized again with the parameters
    // of the DequantizeLinear that reads it, f32((q - dq_zp) * dq_scale)
    float* dq_out;
    float dq_scale;
    int32_t dq_zp;
    uint32_t* fault;
    // (behind everything else: the kernels that do not use them find their arguments where they were)
    // what the kernel does to the f32 rows before it prepares them (DequantF32 only), the fused decode
    // forms of the reference's device route
    // (native/src/backends/cuda/kernels/cuda_forward_gemv_pair_kernels.inc:1136,1424,408,672):
    // row_gain: RMSNorm with this gain [k] and row_eps, as rmsnorm_prepare_kernel computes it;
    // row_swiglu: the rows are [gate | up] of 2k elements and the input is silu(gate) * up, as
    // swiglu_prepare_kernel computes it.  add_to [rows][n] (may be y itself): the output is
    // add_to + (linear + bias), the residual add behind the linear.
    const float* row_gain;
    double row_eps;
    uint32_t row_swiglu;
    const float* add_to;
    // set by the large-tile GEMM launchers for outputs of a size where it was measured to pay: the
    // output leaves the L2 as it is stored (store_stream) instead of with the write-back at the end
    uint32_t stream_out;
};

// gemm_mfma.hip / gemv_stream.hip: return the variant id that ran, or null if
// the shape is outside the kernel's domain (nothing launched).
const char* launch_gemm_mfma(hipStream_t s, const LinearArgs& a, int cu_count, const char* force);
// A kernel's dynamic-LDS limit is an attribute per device: raised once per device and kernel
// (`done` holds one bit per device ordinal; a racing second call only repeats the request).
inline bool raise_lds_limit(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return false;
    const uint64_t bit = 1ull << device;
    if (done.load(std::memory_order_acquire) & bit) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
    done.fetch_or(bit, std::memory_order_release);
    return true;
}

const char* launch_gemv_stream(hipStream_t s, const LinearArgs& a, int cu_count, const char* force);
// While on (per thread), launch_gemv_stream chooses as always and launches nothing: its result tells
// whether a call of that description would be taken.
void set_gemv_dry_run(bool on);

const char* forced_variant();

}  // namespace vxhip
