// Bandwidth-bound W8A8 linear for decode-shaped M <= 32.  Every weight byte is
// read exactly once, straight from HBM into MFMA operand registers with
// coalesced dwordx4 loads (no LDS hop), and multiplied against all M rows at
// once on v_mfma_i32_32x32x32_i8, whose internal reduction replaces the
// cross-lane dot-product reduce.  The GPU counterpart of the reference's
// single-row route vx_packed_linear_single_row_range
// (native/src/kernels/packed_linear_ops.inc:1471-1535) and of its M=1 QLinear
// route (native/src/kernels/qlinear_vnni_kernel.inc:41-127).
//
// Work split: one workgroup per panel of 32 output channels, split-K over its
// wavefronts.  A wavefront owns a contiguous run of the panel's 1 KiB blocks
// (the packed layout of common.h makes a panel's k-steps contiguous), requests
// up to kDepth of them at once with non-temporal loads -- a plain read of the
// same bytes is fastest in exactly this shape, 4-8 KiB per wave in flight -- and
// feeds each block unchanged to the MFMA as the weight operand; the activation
// operand (row min(l%32, M-1), k-chunk l/32) comes from the L2-resident
// activation rows.
//
// Split-K reduction: the streaming phase is integer only.  Partial dots add
// exactly; for the dequantizing epilogue the exact int32 dot of every storage
// group is parked in LDS and one thread per output then applies the scales and
// sums in ascending group order, which keeps the result bit-identical to the
// serial order the reference uses (packed_linear_ops.inc:1498-1504).
#include "common.h"
#include "device_math.h"
#include "epilogue.h"
#include "row_math.h"
#include "wave_ops.h"

#include <stdio.h>
#include <string.h>

#include <type_traits>


namespace vxhip {

namespace {

// While set on the calling thread the launchers of this file decide as always but launch nothing: what
// launch_gemv_stream then returns tells whether (and as which variant) a call would run.
thread_local bool gemv_dry_run = false;

extern __shared__ __attribute__((aligned(16))) char gemv_lds[];

constexpr int kDepth = 4;  // 1 KiB blocks in flight per wave
constexpr int kPrepPerThread = 8;  // f32 elements of a row that a thread of a preparing kernel holds
constexpr uint32_t kFitLdsRows = 8;  // the exact-fit kernel keeps the activation rows in LDS up to this many rows

__device__ __forceinline__ v4i load_stream(const int8_t* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const v4i*>(p));
}

// MODE: Epilogue.  GK: k-steps of 32 per scale group (1, 2, 4 or 8).  WAVES:
// wavefronts of the workgroup, all sharing one panel.  W4: four-bit weights, a 1 KiB block
// then carries two k-steps and is split into their operands in registers (three VALU
// operations per dword), so the stream is half as long for the same K.
//
// SPLIT (1, 2 or 4): workgroups per panel.  A matrix of few panels (N = 1024 is 32 of them) leaves
// most compute units without a workgroup; then SPLIT workgroups share a panel, each taking
// CH = 32 / SPLIT of its channels.  A workgroup reads only the bytes of a block that hold its
// channels (whole 128-byte lines: eight channels are lanes 8q..8q+7 and 32+8q..32+8q+7): the other
// lanes are pointed at the same lines, so nothing in the stream becomes conditional, the MFMA runs
// on a full operand whose other rows repeat the workgroup's own, and only the accumulator quads of
// the workgroup's channels are parked, folded and stored.
//
// PREP: the activations arrive as f32 rows (a.x_f32, at most kMaxPrepRows of them) and the workgroup
// prepares them itself, exactly as prepare_i8_kernel does (boundary.hip): per row scale = max|x| / 127
// with a true division, floored at 2^-126, 1 for a zero row; codes = ties-to-even(x / scale) clamped to
// +-127; a row holding NaN or Inf gets zero codes and a NaN scale.  The codes live in LDS, where the
// MFMA's activation operand is then read from.  Every workgroup repeats this for all rows -- a few
// 16 KiB reads that hit L2, issued behind the first weight requests -- and the linear is one launch
// instead of two: the single-row route of the reference (packed_linear_ops.inc:1471-1535) also
// quantizes the row and multiplies in one call.
constexpr int kRowsPrepared = 0, kRowsF32 = 1, kRowsNorm = 2, kRowsSwiglu = 3;

template <int MODE, int GK, int WAVES, bool W4, int SPLIT, int ROWOP>
__global__ __launch_bounds__(WAVES * 64, (ROWOP == 2 && WAVES == 8) ? 4 : 1) void gemv_panel_kernel(const LinearArgs a) {
    constexpr bool F = MODE == (int)Epilogue::DequantF32;
    // ROWOP: kRowsPrepared (0) int8 rows; kRowsF32 f32 rows prepared here; kRowsNorm, kRowsSwiglu: with
    // RMSNorm or SwiGLU in front of the preparation
    constexpr bool PREP = ROWOP != kRowsPrepared, NORM = ROWOP == kRowsNorm, SWIGLU = ROWOP == kRowsSwiglu;
    static_assert(F || !(NORM || SWIGLU), "row operations ride in front of the dynamic preparation only");
    static_assert(MODE != (int)Epilogue::RequantRow || !PREP, "f32 activations: PackedLinear, or QLinear behind a QuantizeLinear");
    constexpr int CH = 32 / SPLIT;     // channels of this workgroup
    constexpr int QUADS = 4 / SPLIT;   // accumulator quads (8 channels each) of this workgroup
    static_assert(F || !W4, "four-bit weights exist for the dequantizing epilogue only");
    constexpr int SPB = W4 ? 2 : 1;              // k-steps per 1 KiB block
    constexpr int UNIT = GK > SPB ? GK : SPB;    // a wave's run is a whole number of these
    const int lane = threadIdx.x & 63;
    // wave-uniform, and known to the compiler as such: the bounds of the wave's run and every
    // branch on them are then scalar.  (That is needed, not only cheaper: an MFMA is not
    // predicated by the EXEC mask, so a guard the compiler took for divergent and turned into
    // EXEC masking around a lone MFMA would not guard it.)
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t panel = blockIdx.x / SPLIT, sub = blockIdx.x % SPLIT;
    const uint32_t rows = a.rows;
    const uint32_t ch0 = panel * 32u + sub * CH;  // first channel of this workgroup
    // the lane whose 16 bytes of a block this lane loads: itself when its channel is the
    // workgroup's, else the lane that holds the workgroup's channel at the same offset
    const uint32_t src_lane = SPLIT == 1 ? (uint32_t)lane : ((lane & 32) | (sub * CH + (lane & (CH - 1))));

    // this wave's run of k-steps, aligned to whole groups
    const uint32_t steps = (a.k + 31u) / 32u;
    const uint32_t chunks = (steps + UNIT - 1) / UNIT;
    const uint32_t per = (chunks + WAVES - 1) / WAVES;
    const uint32_t t0 = min((uint32_t)wave * per * UNIT, steps);
    const uint32_t t1 = min((uint32_t)(wave + 1) * per * UNIT, steps);

    const int8_t* wp = a.w + (size_t)panel * a.ksteps * 1024u + src_lane * 16u;
    const uint32_t m = min((uint32_t)(lane & 31), rows - 1u);
    // row-major rows, or operand order: the row's 16-byte chunks 512 bytes apart (see
    // ActivationLayout), which makes the 64 lanes' loads of a k-step one contiguous KiB
    const int8_t* xp = PREP ? nullptr : a.x + (size_t)m * (a.x_operand_order ? 16u : a.ldx);
    const uint32_t x_chunk_pitch = a.x_operand_order ? 16u * kOperandOrderRows : 16u;
    const uint32_t half = lane >> 5;
    const uint32_t last_chunk = (a.k - 1u) / 16u;

    // LDS: F: dots[group][row][CH] exact int32 group dots   R: parts[wave][row][CH]
    int32_t* parts = reinterpret_cast<int32_t*>(gemv_lds);
    const bool row_live = (uint32_t)(lane & 31) < rows;

    // slot <- the block that starts at k-step t (t even for four-bit weights) and the
    // activation chunks of its steps
    v4i wbuf[kDepth], xbuf[kDepth][SPB];
    auto issue = [&](int slot, uint32_t t) {
        wbuf[slot] = load_stream(wp + (size_t)(t / SPB) * 1024u);
        if constexpr (!PREP) {
#pragma unroll
            for (int h = 0; h < SPB; h++) {
                const uint32_t chunk = min((t + h) * 2u + half, last_chunk);
                xbuf[slot][h] = *reinterpret_cast<const v4i*>(xp + (size_t)chunk * x_chunk_pitch);
            }
        }
    };

    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;

    // PREP: the f32 rows are requested first of all (loads return in order: behind the weight stream
    // they would arrive with it, in front of it they are L2 hits whose preparation then runs while the
    // first weight blocks are on their way) and stay in registers for the two passes.
    constexpr int PREP_ROWS = PREP ? (int)kMaxPrepRows : 1, PREP_KEPT = PREP ? kPrepPerThread : 1;
    // A row operation of the decoder may ride in front of the preparation (F only): RMSNorm with
    // a.row_gain, or SwiGLU over rows that hold [gate | up]; its other operands travel with the rows.
    constexpr bool ROWOPS = PREP && F;
    // pass i of row r holds elements (whole 16-byte chunks of codes are written, so up to the padded end)
    const uint32_t prep_end = (a.k + 15u) / 16u * 16u;
    auto live = [&](int r, int i) { return (uint32_t)r < rows && (uint32_t)(i * WAVES * 64) < prep_end; };
    float xrows[PREP_ROWS][PREP_KEPT];
    float xup[SWIGLU ? PREP_ROWS : 1][SWIGLU ? PREP_KEPT : 1];
    float xgain[NORM ? PREP_KEPT : 1];
    if constexpr (PREP) {
#pragma unroll
        for (int r = 0; r < PREP_ROWS; r++) {
            const float* src = a.x_f32 + (size_t)min((uint32_t)r, rows - 1u) * a.ldx;
#pragma unroll
            for (int i = 0; i < PREP_KEPT; i++) {
                const uint32_t j = threadIdx.x + i * WAVES * 64;
                xrows[r][i] = 0.0f;
                if constexpr (SWIGLU) xup[r][i] = 0.0f;
                if (live(r, i)) {  // (scalar: whole passes past the row end, and rows not given, cost nothing)
                    xrows[r][i] = j < a.k ? src[j] : 0.0f;
                    if constexpr (SWIGLU) xup[r][i] = j < a.k ? src[a.k + j] : 0.0f;
                }
            }
        }
        if constexpr (NORM) {
#pragma unroll
            for (int i = 0; i < PREP_KEPT; i++) {
                const uint32_t j = threadIdx.x + i * WAVES * 64;
                xgain[i] = 0.0f;
                if (live(0, i)) xgain[i] = j < a.k ? a.row_gain[j] : 0.0f;
            }
        }
    }

    // The tail's per-output operands (activation scale, bias) are requested now, so that their
    // latency hides behind the stream instead of following it.
    constexpr int TAIL_ITERS = ((int)(PREP ? kMaxPrepRows : kMaxGemvRows) * CH + WAVES * 64 - 1) / (WAVES * 64);
    float tail_rs[F ? TAIL_ITERS : 1], tail_bias[F ? TAIL_ITERS : 1], tail_add[ROWOPS ? TAIL_ITERS : 1];
    if constexpr (F) {
#pragma unroll
        for (int it = 0; it < TAIL_ITERS; it++) {
            const uint32_t o = threadIdx.x + it * WAVES * 64;
            tail_rs[it] = PREP ? 0.0f : a.row_scale[min(o / CH, rows - 1u)];
            tail_bias[it] = a.bias_f32[ch0 + o % CH];  // padded to whole panels
            if constexpr (ROWOPS) {
                // the residual the output is added to: this thread's element, read before anything writes it
                const uint32_t om = o / CH, on = ch0 + o % CH;
                tail_add[it] = (a.add_to && om < rows && on < a.n) ? a.add_to[(size_t)om * a.n + on] : 0.0f;
            }
        }
    }

    // F: the panel's group scales [group][32] are fetched first (they are L2 hits and return
    // ahead of the HBM stream) and kept in LDS for the tail.
    constexpr int SCALE_SLOTS = 4;  // per thread; covers groups * 32 <= SCALE_SLOTS * threads
    float* lds_scales = reinterpret_cast<float*>(gemv_lds) + (size_t)a.groups * rows * CH;
    float sc[F ? SCALE_SLOTS : 1];
    uint32_t sc_base = 0;
    if constexpr (F) {
        const uint32_t total = a.groups * CH;
        auto fetch = [&](uint32_t e) {
            return e < total ? a.scales_t[(size_t)(e / CH) * a.n_pad + ch0 + e % CH] : 0.0f;
        };
        // many groups on few waves: copy all but the last pass before the stream starts
        while (total - sc_base > (uint32_t)(SCALE_SLOTS * WAVES * 64)) {
#pragma unroll
            for (int u = 0; u < SCALE_SLOTS; u++) {
                const uint32_t e = sc_base + threadIdx.x + u * WAVES * 64;
                lds_scales[e] = fetch(e);
            }
            sc_base += SCALE_SLOTS * WAVES * 64;
        }
#pragma unroll
        for (int u = 0; u < SCALE_SLOTS; u++) sc[u] = fetch(sc_base + threadIdx.x + u * WAVES * 64);
    }

    // The streaming phase is integer only and the same for every epilogue: the exact dot of
    // each closed group (F) or of the wave's whole run (R) is parked in LDS.
    auto park = [&](uint32_t slab) {
        if (row_live) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                // quad q holds channels 8q..8q+7 of the panel; the test is scalar
                if (SPLIT > 1 && (uint32_t)(q / QUADS) != sub) continue;
                // four-bit operands carry a factor 16, which the exact dot sheds here
                *reinterpret_cast<v4i*>(parts + ((size_t)slab * rows + (lane & 31)) * CH + (q % QUADS) * 8 +
                                        half * 4) =
                    v4i{acc[q * 4] >> (W4 ? 4 : 0), acc[q * 4 + 1] >> (W4 ? 4 : 0),
                        acc[q * 4 + 2] >> (W4 ? 4 : 0), acc[q * 4 + 3] >> (W4 ? 4 : 0)};
            }
        }
    };

    // PREP: the rows' codes [rows][ldk] and scales [rows] behind the group dots and group scales
    __shared__ float slot_max[PREP_ROWS][WAVES];
    __shared__ uint32_t slot_bad[PREP_ROWS][WAVES];
    const uint32_t ldk = (a.k + 15u) / 16u * 16u;
    int8_t* prep_codes = reinterpret_cast<int8_t*>(gemv_lds) +
                         (F ? (size_t)a.groups * (rows + 1u) * CH * 4u : (size_t)WAVES * rows * CH * 4u);
    float* prep_scale = reinterpret_cast<float*>(prep_codes + (size_t)rows * ldk);
    // (NR, the number of rows, is a template tag: without a branch between the rows their chains of
    // reductions interleave)
    auto prepare_rows_of = [&](auto rows_tag) __attribute__((always_inline)) {
        constexpr int NR = decltype(rows_tag)::value;
        auto pass = [&](int i) { return (uint32_t)(i * WAVES * 64) < prep_end; };
        if constexpr (PREP && !F) {
            // QuantizeLinear in front of a QLinear: q = saturate(ties-to-even(f32(x / s) + f32(zp))), NaN -> zp
            // (native/src/kernels/quantize_linear_ops.inc:156-169), stored as the signed byte the MFMA takes
            // (an unsigned type's bytes have their top bit flipped, as input_zp already is)
            const int32_t shift = a.x_f32_unsigned ? 128 : 0;
            const float zp_f = (float)(a.input_zp + shift), lo_f = (float)(a.x_f32_unsigned ? 0 : -128),
                        hi_f = (float)(a.x_f32_unsigned ? 255 : 127);
#pragma unroll
            for (int r = 0; r < NR; r++) {
#pragma unroll
                for (int i = 0; i < PREP_KEPT; i++) {
                    if (!pass(i)) continue;
                    const uint32_t j = threadIdx.x + i * WAVES * 64;
                    const float v = xrows[r][i];
                    int32_t q = a.input_zp + shift;
                    if (v == v) {
                        const float t = __fadd_rn(__fdiv_rn(v, a.input_scale), zp_f);
                        q = t <= lo_f ? (int32_t)lo_f : t >= hi_f ? (int32_t)hi_f : (int32_t)__builtin_rintf(t);
                    }
                    if (j < ldk) prep_codes[(size_t)r * ldk + j] = (int8_t)(q - shift);
                }
            }
            __syncthreads();  // every wave reads every row's codes
        }
        if constexpr (SWIGLU) {
#pragma unroll
            for (int r = 0; r < NR; r++)
#pragma unroll
                for (int i = 0; i < PREP_KEPT; i++)
                    if (pass(i)) xrows[r][i] = swiglu_value(xrows[r][i], xup[r][i]);
        }
        if constexpr (NORM) {
            {
                // The row's sum of squares in the order of rmsnorm_prepare_kernel's 1024 threads: this
                // thread stands for VT of them (elements 1024 apart belong to the same one).
                constexpr int VT = (int)kNormThreads / (WAVES * 64);
                static_assert(VT >= 1 && PREP_KEPT % VT == 0, "a thread holds whole virtual threads");
                __shared__ double norm_slots[PREP_ROWS][kNormThreads / 64];
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    double vs[VT];
#pragma unroll
                    for (int v = 0; v < VT; v++) vs[v] = 0.0;
#pragma unroll
                    for (int i = 0; i < PREP_KEPT; i++)
                        if (pass(i)) vs[i % VT] += (double)xrows[r][i] * (double)xrows[r][i];
#pragma unroll
                    for (int v = 0; v < VT; v++) {
                        const double part = wave_sum_to_lane0(vs[v]);
                        if (lane == 0) norm_slots[r][wave + v * WAVES] = part;
                    }
                }
                __syncthreads();
#pragma unroll
                for (int r = 0; r < NR; r++) {
                    double total = 0.0;
#pragma unroll
                    for (uint32_t w = 0; w < kNormThreads / 64u; w++) total += norm_slots[r][w];
                    const double inv_std = rms_inverse(total, a.k, a.row_eps);
#pragma unroll
                    for (int i = 0; i < PREP_KEPT; i++)
                        if (pass(i)) xrows[r][i] = rms_scaled(xrows[r][i], inv_std, xgain[i]);
                }
            }
        }
        if constexpr (PREP && F) {
#pragma unroll
            for (int r = 0; r < NR; r++) {
                float maximum = 0.0f;
                uint32_t bad = 0u;
#pragma unroll
                for (int i = 0; i < PREP_KEPT; i++) {
                    if (!pass(i)) continue;
                    bad |= finite_f32(xrows[r][i]) ? 0u : 1u;
                    maximum = fmaxf(maximum, fabsf(xrows[r][i]));  // fmaxf ignores a NaN operand; `bad` records it
                }
                maximum = wave_max(maximum);
                bad = __builtin_amdgcn_ballot_w64(bad != 0u) != 0ull ? 1u : 0u;
                if (lane == 0) {
                    slot_max[r][wave] = maximum;
                    slot_bad[r][wave] = bad;
                }
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < NR; r++) {
                float maximum = slot_max[r][0];
                uint32_t bad = slot_bad[r][0];
#pragma unroll
                for (int w = 1; w < WAVES; w++) {
                    maximum = fmaxf(maximum, slot_max[r][w]);
                    bad |= slot_bad[r][w];
                }
                float scale = maximum == 0.0f ? 1.0f : __fdiv_rn(maximum, 127.0f);
                if (scale < 0x1p-126f) scale = 0x1p-126f;
#pragma unroll
                for (int i = 0; i < PREP_KEPT; i++) {
                    if (!pass(i)) continue;
                    const uint32_t j = threadIdx.x + i * WAVES * 64;
                    // (elements past k were loaded as zeros: the padding of the last 16-byte chunk)
                    if (j < ldk) prep_codes[(size_t)r * ldk + j] = (int8_t)(bad ? 0 : packed_round_i8(__fdiv_rn(xrows[r][i], scale)));
                }
                if (threadIdx.x == 0) prep_scale[r] = bad ? __builtin_nanf("") : scale;
            }
            __syncthreads();  // every wave reads every row's codes
        }
    };
    auto prepare_rows = [&]() __attribute__((always_inline)) {
        if constexpr (PREP) {
            if (rows >= 2u) prepare_rows_of(std::integral_constant<int, PREP_ROWS>{});
            else prepare_rows_of(std::integral_constant<int, 1>{});
        }
    };

    auto stash_scales = [&]() {
        if constexpr (F) {
#pragma unroll
            for (int u = 0; u < SCALE_SLOTS; u++) {
                const uint32_t e = sc_base + threadIdx.x + u * WAVES * 64;
                if (e < a.groups * CH) lds_scales[e] = sc[u];
            }
        }
    };
    // One round: the MFMAs of the kDepth blocks that start at k-step t, each slot refilled with
    // the block kDepth further on as soon as it has been consumed.  STEADY rounds lie wholly
    // inside the run and so does the round after them: nothing in them is conditional, which
    // lets the wait before each MFMA name exactly the loads it needs (a refill under a branch
    // makes the count of outstanding loads unknown and every wait a full drain of the queue).
    auto round = [&](uint32_t t, auto steady_tag) {
        constexpr bool STEADY = decltype(steady_tag)::value;
#pragma unroll
        for (int i = 0; i < kDepth; i++) {
#pragma unroll
            for (int h = 0; h < SPB; h++) {
                const uint32_t tt = t + i * SPB + h;
                if (STEADY || tt < t1) {
                    v4i wop = wbuf[i];
                    if constexpr (W4) {
#pragma unroll
                        for (int d = 0; d < 4; d++)
                            wop[d] = (h == 0 ? wbuf[i][d] << 4 : wbuf[i][d]) & (int)0xf0f0f0f0u;
                    }
                    v4i xop;
                    if constexpr (PREP) {
                        const uint32_t chunk = min(tt * 2u + half, last_chunk);
                        xop = *reinterpret_cast<const v4i*>(prep_codes + (size_t)m * ldk + chunk * 16u);
                    } else {
                        // (unsigned activation bytes become the signed operand here: one XOR per dword, in a
                        // kernel that waits for memory)
                        xop = xbuf[i][h] ^ (int)a.x_flip_mask;
                    }
                    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wop, xop, acc, 0, 0, 0);
                    if constexpr (F) {
                        // a group closes after GK steps (t0 is group aligned) or at the row end
                        if ((tt + 1) % GK == 0 || (!STEADY && tt + 1 == t1)) {
                            park(tt / GK);
#pragma unroll
                            for (int r = 0; r < 16; r++) acc[r] = 0;
                        }
                    }
                }
            }
            if (STEADY || t + (i + kDepth) * SPB < t1) issue(i, t + (i + kDepth) * SPB);
        }
    };
    constexpr uint32_t ROUND = kDepth * SPB;  // k-steps per round
    uint32_t t = t0;
    if (t1 - t0 >= 2 * ROUND) {
#pragma unroll
        for (int i = 0; i < kDepth; i++) issue(i, t0 + i * SPB);
        stash_scales();
        prepare_rows();
        for (; t + 2 * ROUND <= t1; t += ROUND) round(t, std::true_type{});
    } else {
#pragma unroll
        for (int i = 0; i < kDepth; i++)
            if (t0 + i * SPB < t1) issue(i, t0 + i * SPB);
        stash_scales();
        prepare_rows();
    }
    for (; t < t1; t += ROUND) round(t, std::false_type{});
    if constexpr (!F) park(wave);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();

    // Tail: one thread per output, index o = row * CH + channel.  F: sum += f32(dot_g) *
    // (s_a * s_w[n][g]) in ascending group order with separate roundings
    // (packed_linear_ops.inc:1498-1504); eight groups' operands are requested before the
    // first add needs one.
    const size_t slab = (size_t)rows * CH;
    if constexpr (F) {
#pragma unroll
        for (int it = 0; it < TAIL_ITERS; it++) {
            const uint32_t o = threadIdx.x + it * WAVES * 64;
            if (o >= rows * CH) break;
            const uint32_t om = o / CH, on = ch0 + o % CH;
            const float rs = PREP ? prep_scale[om] : tail_rs[it];
            float sum = 0.0f;
            const int32_t* dp = parts + o;
            const float* sp = lds_scales + o % CH;
            uint32_t g = 0;
            for (; g + 8u <= a.groups; g += 8u) {
                int32_t d[8];
                float sw[8];
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    d[u] = dp[(size_t)(g + u) * slab];
                    sw[u] = sp[(g + u) * CH];
                }
#pragma unroll
                for (int u = 0; u < 8; u++)
                    sum = __fadd_rn(sum, __fmul_rn((float)d[u], __fmul_rn(rs, sw[u])));
            }
            for (; g < a.groups; g++)
                sum = __fadd_rn(sum, __fmul_rn((float)dp[(size_t)g * slab], __fmul_rn(rs, sp[g * CH])));
            float out = __fadd_rn(sum, tail_bias[it]);
            if constexpr (ROWOPS)
                if (a.add_to) out = __fadd_rn(tail_add[it], out);
            if (on < a.n) ((float*)a.y)[(size_t)om * a.n + on] = out;
        }
    } else {
        for (uint32_t o = threadIdx.x; o < rows * CH; o += WAVES * 64) {
            const uint32_t om = o / CH, on = ch0 + o % CH;
            float rs = 0.0f;
            if constexpr (MODE == (int)Epilogue::RequantRow) rs = a.row_scale[om];
            int32_t dot = 0;
#pragma unroll
            for (int w = 0; w < WAVES; w++) dot += parts[(size_t)w * slab + o];
            store_element<MODE>(a, om, on, dot, 0.0f, rs);
        }
    }
}

// The exact-fit form of the dequantizing kernel: a panel's blocks divide evenly into WAVES runs of BPW
// blocks, each a whole number of scale groups, so the whole stream is straight-line code -- the same
// split of K over the wavefronts, the same integer group dots, the same ascending f32 sum, with
// everything that is not the stream moved out of its way:
//   * the first weight blocks are requested before anything else is looked at;
//   * XLDS (few rows): a wave copies its own slice of the activation rows (32 bytes per block and row)
//     into LDS once and reads the MFMA's activation operand from there, so the weight blocks are the
//     only vector loads of the loop;
//   * the wave that closes a group turns its dots into the products f32(dot) * (s_a * s_w[n][g])
//     itself, lane-parallel over its own groups (its scales were requested mid-stream and wait in
//     registers or in the wave's own LDS corner), so that behind the one barrier a thread per output
//     only adds GROUPS products in ascending order -- the sum the reference forms
//     (packed_linear_ops.inc:1498-1504), bit for bit.
// Measured at M=1, K=4096, N=14336 (sixteen waves of eight blocks): 10.3 us against 12.5 us for the
// general kernel, with a plain read of the same bytes at 9.3-9.6 us.
// PREP: one or two f32 rows (a.x_f32) which the workgroup prepares itself, by prepare_i8_kernel's rule to the
// letter, as the reference's single-row route quantizes the row and multiplies in one call
// (packed_linear_ops.inc:1471-1535).  A wave's 64 lanes hold exactly the elements of the wave's own K-slice
// (BPW / 2 consecutive ones per lane), so only the row maximum crosses the waves; the codes go straight into
// the wave's LDS slice, where the MFMA's activation operand is read from.
// W4: four-bit weights; a 1 KiB block then carries two k-steps (low nibbles, then high nibbles, each moved to
// the top of its byte: operands with a factor 16, which the exact dot sheds with a shift when it is parked).
template <int GK, int WAVES, int BPW, bool XLDS, bool PREP = false, bool RPROD = false, bool W4 = false, int SPLIT = 1>
__global__ __launch_bounds__(WAVES * 64, 8) void gemv_fit_kernel(const LinearArgs a) {
    constexpr int SPB = W4 ? 2 : 1, STEPS = BPW * SPB;  // k-steps per block, per wave
    static_assert(STEPS % GK == 0 && BPW >= kDepth, "a wave's run is whole groups and at least one round");
    static_assert(!PREP || (XLDS && STEPS % 4 == 0), "prepared rows live in the LDS slices; a lane loads pairs of elements");
    static_assert(!(PREP && RPROD), "one or two rows form their products lane-parallel");
    static_assert(SPLIT == 1 || SPLIT == 2 || SPLIT == 4, "workgroups per panel");
    constexpr int GPW = STEPS / GK, GROUPS = WAVES * GPW;  // groups per wave, per panel
    // SPLIT workgroups share a panel, each taking CH of its channels, as in gemv_panel_kernel: a lane whose
    // channel is another workgroup's loads the bytes of the lane that holds this workgroup's channel at the
    // same offset, and only the accumulator quads of the workgroup's channels are parked
    constexpr int CH = 32 / SPLIT, QUADS = 4 / SPLIT;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t panel = blockIdx.x / SPLIT, sub = blockIdx.x % SPLIT, rows = a.rows;
    const uint32_t ch0 = panel * 32u + sub * CH;
    const uint32_t src_lane = SPLIT == 1 ? (uint32_t)lane : ((lane & 32) | (sub * CH + (lane & (CH - 1))));
    const uint32_t t0 = (uint32_t)wave * STEPS, g0 = (uint32_t)wave * GPW;  // first k-step, first group
    const uint32_t half = lane >> 5;
    const uint32_t m = min((uint32_t)(lane & 31), rows - 1u);
    const uint32_t last_chunk = (a.k - 1u) / 16u;
    const int8_t* wp = a.w + ((size_t)panel * a.ksteps + (uint32_t)wave * BPW) * 1024u + src_lane * 16u;

    // LDS: products [GROUPS][rows][CH] (int32 dots first) | per wave: scales [GPW][CH], row scales [32] |
    // per wave (XLDS): activation slice [2 * STEPS chunks][rows] of 16 bytes
    int32_t* dots = reinterpret_cast<int32_t*>(gemv_lds);
    float* wave_scales = reinterpret_cast<float*>(gemv_lds) + (size_t)GROUPS * rows * CH + (size_t)wave * (GPW * CH + 32);
    float* wave_rs = wave_scales + GPW * CH;
    char* xslice = gemv_lds + ((size_t)GROUPS * rows * CH + (size_t)WAVES * (GPW * CH + 32)) * 4u +
                   (size_t)wave * (2 * STEPS) * rows * 16u;

    // (XLDS) this wave's activation chunks are requested first: they are cache hits and return ahead
    // of the weight stream
    constexpr int XPL = XLDS && !PREP ? (2 * STEPS * (int)kFitLdsRows + 63) / 64 : 1;  // chunks per lane
    v4i xstage[XPL];
    constexpr int EPL = STEPS / 2;  // PREP: f32 elements of a row per lane
    float xf[PREP ? (int)kMaxPrepRows : 1][PREP ? EPL : 1];
    if constexpr (PREP) {
#pragma unroll
        for (int r = 0; r < (int)kMaxPrepRows; r++) {
            const float* src = a.x_f32 + (size_t)min((uint32_t)r, rows - 1u) * a.ldx + (size_t)t0 * 32u + (uint32_t)lane * EPL;
#pragma unroll
            for (int i = 0; i < EPL; i += 2) {
                const float2 v = *reinterpret_cast<const float2*>(src + i);
                xf[r][i] = v.x;
                xf[r][i + 1] = v.y;
            }
        }
    } else if constexpr (XLDS) {
#pragma unroll
        for (int j = 0; j < XPL; j++) {
            const uint32_t e = min((uint32_t)lane + 64u * j, 2u * STEPS * rows - 1u);
            const uint32_t c = min(t0 * 2u + e / rows, last_chunk), r = e % rows;
            xstage[j] = *reinterpret_cast<const v4i*>(
                a.x + (a.x_operand_order ? ((size_t)c * kOperandOrderRows + r) * 16u : (size_t)r * a.ldx + (size_t)c * 16u));
        }
    }
    // (the order is kept by hand: loads come back in the order of their issue, and left to itself the
    // scheduler puts the weight requests first, so that the wait for these few bytes becomes a wait for
    // the first four blocks and the next four go out a memory round trip late)
    __builtin_amdgcn_sched_barrier(0);
    const int8_t* xp = a.x + (size_t)m * (a.x_operand_order ? 16u : a.ldx);
    const uint32_t x_chunk_pitch = a.x_operand_order ? 16u * kOperandOrderRows : 16u;
    v4i wbuf[kDepth], xbuf[XLDS ? 1 : kDepth][SPB];
    auto issue = [&](int slot, uint32_t b) {
        wbuf[slot] = load_stream(wp + (size_t)b * 1024u);
        if constexpr (!XLDS) {
#pragma unroll
            for (int h = 0; h < SPB; h++) {
                const uint32_t chunk = min((t0 + b * SPB + h) * 2u + half, last_chunk);
                xbuf[slot][h] = *reinterpret_cast<const v4i*>(xp + (size_t)chunk * x_chunk_pitch);
            }
        }
    };
#pragma unroll
    for (int i = 0; i < kDepth; i++) issue(i, i);
    __builtin_amdgcn_sched_barrier(0);

    // what the tail needs, requested behind the first blocks: the wave's group scales, lane e <-> (group
    // g0 + e / CH, channel e % CH); the row scales; the bias of this thread's outputs
    constexpr int SPL = (GPW * CH + 63) / 64;
    float sreg[SPL];
#pragma unroll
    for (int u = 0; u < SPL; u++) {
        const uint32_t e = min((uint32_t)lane + 64u * u, (uint32_t)(GPW * CH) - 1u);
        sreg[u] = a.scales_t[(size_t)(g0 + e / CH) * a.n_pad + ch0 + e % CH];
    }
    // (RPROD: the scale of the row whose dots the lane holds in its accumulators; else lane r carries row r's)
    float rs_lane = 0.0f;
    if constexpr (!PREP) rs_lane = a.row_scale[RPROD ? m : min((uint32_t)lane, rows - 1u)];
    constexpr int OPT_ = ((int)kMaxGemvRows * CH + WAVES * 64 - 1) / (WAVES * 64);  // outputs per thread
    float bias_t[OPT_];
#pragma unroll
    for (int it = 0; it < OPT_; it++) bias_t[it] = a.bias_f32[ch0 + (threadIdx.x + it * WAVES * 64) % CH];

    if constexpr (PREP) {
        // per row: scale = max|x| / 127 (true division; 1 for a zero row; floored at 2^-126), codes =
        // ties-to-even(x / scale) clamped to +-127; a row that is not finite gets zero codes and a NaN scale
        __shared__ float slot_max[kMaxPrepRows][WAVES];
        __shared__ uint32_t slot_bad[kMaxPrepRows][WAVES];
#pragma unroll
        for (int r = 0; r < (int)kMaxPrepRows; r++) {
            float maximum = 0.0f;
            uint32_t bad = 0u;
#pragma unroll
            for (int i = 0; i < EPL; i++) {
                bad |= finite_f32(xf[r][i]) ? 0u : 1u;
                maximum = fmaxf(maximum, fabsf(xf[r][i]));
            }
            maximum = wave_max(maximum);
            bad = __builtin_amdgcn_ballot_w64(bad != 0u) != 0ull ? 1u : 0u;
            if (lane == 0) {
                slot_max[r][wave] = maximum;
                slot_bad[r][wave] = bad;
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < (int)kMaxPrepRows; r++) {
            float maximum = slot_max[r][0];
            uint32_t bad = slot_bad[r][0];
#pragma unroll
            for (int w = 1; w < WAVES; w++) {
                maximum = fmaxf(maximum, slot_max[r][w]);
                bad |= slot_bad[r][w];
            }
            float scale = maximum == 0.0f ? 1.0f : __fdiv_rn(maximum, 127.0f);
            if (scale < 0x1p-126f) scale = 0x1p-126f;
            if ((uint32_t)r < rows) {
                // element j = lane * EPL + i of the slice lives in chunk j / 16 at byte j % 16: [chunk][row] of 16 bytes
#pragma unroll
                for (int i = 0; i < EPL; i += 2) {
                    const uint32_t j = (uint32_t)lane * EPL + i;
                    const int32_t q0 = bad ? 0 : packed_round_i8(__fdiv_rn(xf[r][i], scale));
                    const int32_t q1 = bad ? 0 : packed_round_i8(__fdiv_rn(xf[r][i + 1], scale));
                    *reinterpret_cast<uint16_t*>(xslice + ((size_t)(j / 16u) * rows + r) * 16u + j % 16u) =
                        (uint16_t)((uint32_t)(q0 & 0xff) | ((uint32_t)(q1 & 0xff) << 8));
                }
            }
            const float row_scale = bad ? __builtin_nanf("") : scale;
            if (min((uint32_t)lane, rows - 1u) == (uint32_t)r) rs_lane = row_scale;  // (as the loaded scales: lane r carries row r's)
        }
    } else if constexpr (XLDS) {
#pragma unroll
        for (int j = 0; j < XPL; j++) {
            const uint32_t e = (uint32_t)lane + 64u * j;
            if (e < 2u * STEPS * rows) *reinterpret_cast<v4i*>(xslice + (size_t)e * 16u) = xstage[j];
        }
    }

    v16i acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0;
    const bool row_live = (uint32_t)(lane & 31) < rows;
#pragma unroll
    for (int b = 0; b < BPW; b++) {
        const int slot = b % kDepth;
#pragma unroll
        for (int h = 0; h < SPB; h++) {
            const int t = b * SPB + h;  // the wave's k-step
            v4i xop, wop = wbuf[slot];
            if constexpr (XLDS) xop = *reinterpret_cast<const v4i*>(xslice + ((size_t)(2 * t + half) * rows + m) * 16u);
            else xop = xbuf[slot][h];
            if constexpr (W4) {
#pragma unroll
                for (int d = 0; d < 4; d++) wop[d] = (h == 0 ? wbuf[slot][d] << 4 : wbuf[slot][d]) & (int)0xf0f0f0f0u;
            }
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wop, xop, acc, 0, 0, 0);
            if (h == SPB - 1 && b + kDepth < BPW) issue(slot, b + kDepth);
            if constexpr (RPROD) {
                // the wave's group scales go to its LDS strip once they are here (they were requested behind
                // the first kDepth blocks), in time for the first group that closes
                if (t == (GK > kDepth * SPB ? kDepth * SPB : GK) - 1) {
#pragma unroll
                    for (int u = 0; u < SPL; u++) {
                        const uint32_t e = (uint32_t)lane + 64u * u;
                        if (e < (uint32_t)(GPW * CH)) wave_scales[e] = sreg[u];
                    }
                }
            }
            if ((t + 1) % GK == 0) {
                if (row_live) {
                    int32_t* dp = dots + ((size_t)(g0 + t / GK) * rows + (lane & 31)) * CH + half * 4u;
                    if constexpr (RPROD) {
                        // many rows: the products are formed here, in the accumulators' own layout (a lane holds
                        // its row's dots of sixteen channels), and parked as floats
                        const float* sw = wave_scales + (t / GK) * CH + half * 4u;
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            // quad q holds channels 8q..8q+7 of the panel; the test is scalar
                            if (SPLIT > 1 && (uint32_t)(q / QUADS) != sub) continue;
                            const v4f s4 = *reinterpret_cast<const v4f*>(sw + (q % QUADS) * 8);
                            v4f p;
#pragma unroll
                            for (int i = 0; i < 4; i++)
                                p[i] = __fmul_rn((float)(acc[q * 4 + i] >> (W4 ? 4 : 0)), __fmul_rn(rs_lane, s4[i]));
                            *reinterpret_cast<v4f*>(reinterpret_cast<float*>(dp) + (q % QUADS) * 8) = p;
                        }
                    } else {
#pragma unroll
                        for (int q = 0; q < 4; q++) {
                            if (SPLIT > 1 && (uint32_t)(q / QUADS) != sub) continue;
                            *reinterpret_cast<v4i*>(dp + (q % QUADS) * 8) =
                                v4i{acc[q * 4] >> (W4 ? 4 : 0), acc[q * 4 + 1] >> (W4 ? 4 : 0), acc[q * 4 + 2] >> (W4 ? 4 : 0),
                                    acc[q * 4 + 3] >> (W4 ? 4 : 0)};
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; r++) acc[r] = 0;
            }
        }
    }

    // products of this wave's groups, in place: element e of its region is (group g0 + e / (rows * CH),
    // row (e / CH) % rows, channel e % CH)
    float* prod = reinterpret_cast<float*>(dots) + (size_t)g0 * rows * CH;
    if constexpr (RPROD) {
        (void)prod;
    } else if (rows == 1u) {
#pragma unroll
        for (int u = 0; u < SPL; u++) {
            const uint32_t e = (uint32_t)lane + 64u * u;
            if (e < (uint32_t)(GPW * CH))
                prod[e] = __fmul_rn((float)reinterpret_cast<const int32_t*>(prod)[e], __fmul_rn(rs_lane, sreg[u]));
        }
    } else {
#pragma unroll
        for (int u = 0; u < SPL; u++) {
            const uint32_t e = (uint32_t)lane + 64u * u;
            if (e < (uint32_t)(GPW * CH)) wave_scales[e] = sreg[u];
        }
        if ((uint32_t)lane < rows) wave_rs[lane] = rs_lane;
        const uint32_t per_group = rows * CH;
        for (uint32_t e = lane; e < GPW * per_group; e += 64u) {
            const float sw = wave_scales[(e / per_group) * CH + e % CH];
            const float rs = wave_rs[(e / CH) % rows];
            prod[e] = __fmul_rn((float)reinterpret_cast<const int32_t*>(prod)[e], __fmul_rn(rs, sw));
        }
    }
    __syncthreads();
    const float* products = reinterpret_cast<const float*>(dots);
#pragma unroll
    for (int it = 0; it < OPT_; it++) {
        const uint32_t o = threadIdx.x + it * WAVES * 64;
        if (o >= rows * CH) break;
        // (sixteen products are requested before the first add needs one)
        constexpr int BATCH = GROUPS % 16 == 0 ? 16 : GROUPS % 8 == 0 ? 8 : GROUPS % 4 == 0 ? 4 : 1;
        static_assert(GROUPS % BATCH == 0, "the groups of a panel come in whole batches");
        float sum = 0.0f;
#pragma unroll
        for (int gb = 0; gb < GROUPS; gb += BATCH) {
            float p[BATCH];
#pragma unroll
            for (int g = 0; g < BATCH; g++) p[g] = products[(size_t)(gb + g) * rows * CH + o];
#pragma unroll
            for (int g = 0; g < BATCH; g++) sum = __fadd_rn(sum, p[g]);
        }
        const uint32_t on = ch0 + o % CH;
        if (on < a.n) ((float*)a.y)[(size_t)(o / CH) * a.n + on] = __fadd_rn(sum, bias_t[it]);
    }
}

template <int GK, int WAVES, int BPW, bool W4, int SPLIT = 1>
bool launch_fit(hipStream_t s, const LinearArgs& a, size_t lds, bool xlds, bool rprod) {
    auto kern = xlds ? gemv_fit_kernel<GK, WAVES, BPW, true, false, false, W4, SPLIT> : gemv_fit_kernel<GK, WAVES, BPW, false, false, false, W4, SPLIT>;
    if (rprod)
        kern = xlds ? gemv_fit_kernel<GK, WAVES, BPW, true, false, true, W4, SPLIT> : gemv_fit_kernel<GK, WAVES, BPW, false, false, true, W4, SPLIT>;
    if constexpr (SPLIT == 1 && (BPW * (W4 ? 2 : 1)) % 4 == 0) {
        if (a.x_f32) kern = gemv_fit_kernel<GK, WAVES, BPW, true, true, false, W4>;
    }
    if (gemv_dry_run) return true;
    if (lds > 64u * 1024u) {
        static std::atomic<uint64_t> configured[5] = {{0}, {0}, {0}, {0}, {0}};
        if (!raise_lds_limit((const void*)kern, 160 * 1024, configured[a.x_f32 ? 4 : (rprod ? 2 : 0) + (xlds ? 1 : 0)])) return false;
    }
    hipLaunchKernelGGL(kern, dim3((a.n + 31u) / 32u * SPLIT), dim3(WAVES * 64), lds, s, a);
    return hipGetLastError() == hipSuccess;
}

// The exact-fit kernel takes: the dequantizing epilogue on prepared int8 rows (or one or two f32 rows), eight- or
// four-bit weights, and a K whose blocks are WAVES x BPW of an instance with whole groups in every run; with few
// panels (eight-bit weights, prepared rows, K up to 4096) two or four workgroups share a panel's channels, as in
// the general kernel.  Returns the variant suffix, or null when the general kernel has to run.
template <int GK, bool W4>
const char* launch_fit_mode(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    constexpr uint32_t SPB = W4 ? 2u : 1u;
    if (force && (strstr(force, "nofit") || strstr(force, "wv"))) return nullptr;  // (wv..: a general-kernel name)
    if (a.row_gain || a.row_swiglu || a.add_to || a.weight_bits != (W4 ? 4u : 8u) || a.x_flip_mask) return nullptr;
    // f32 rows (prepared in the kernel): one or two whole rows of exactly the stream's length, pairs of elements aligned
    const bool prep = a.x_f32 != nullptr;
    if (prep && (a.rows > kMaxPrepRows || a.k != a.ksteps * 32u * SPB || (a.ldx % 2u) != 0u || ((uintptr_t)a.x_f32 % 8u) != 0u))
        return nullptr;
    const uint32_t panels = (a.n + 31u) / 32u;
    const bool forced = force && strstr(force, "fit");
    // workgroups per panel: the general kernel's rule (and its names: c8, c16 for the channels of a workgroup)
    uint32_t split = 1;
    if (!W4 && !prep && a.ksteps <= 128u) {
        split = panels * 4u <= (uint32_t)cu_count ? 4u : panels * 2u <= (uint32_t)cu_count ? 2u : 1u;
        if (force && strstr(force, "c8")) split = 4;
        else if (force && strstr(force, "c16")) split = 2;
        else if (force && strstr(force, "c32")) split = 1;
    }
    // (one workgroup per panel and panels for fewer than three quarters of the compute units: the general kernel)
    if (split == 1u && panels * 4u < (uint32_t)cu_count * 3u && !forced) return nullptr;
    // (four-bit weights with more rows than the LDS copy takes: the stream is half as long and the activation loads
    // per block weigh twice as much -- 16 rows 12.1 us here against 12.0 in the general kernel, 32 rows 17.5 against 17.7)
    if (W4 && a.rows > kFitLdsRows && !forced) return nullptr;
    if (a.groups * GK != a.ksteps * SPB) return nullptr;  // (no padding group: every group of the stream has its scales)
    const size_t ch = 32u / split;
    auto lds_for = [&](uint32_t waves, uint32_t steps, bool xlds) {
        const size_t groups = (size_t)waves * steps / GK;
        return groups * a.rows * ch * 4u + (size_t)waves * (steps / GK * ch + 32u) * 4u +
               (xlds ? (size_t)waves * 2u * steps * a.rows * 16u : 0u);
    };
    // where the products are formed: lane-parallel over the parked dots (one row), or by the parking wave
    // in its accumulators' layout (more rows)
    // (measured at K=4096, N=14336: one row 10.8 us either way, 2 / 4 / 8 / 16 / 32 rows 10.8 / 10.9 / 11.0 / 11.9 / 16.3 us
    // against 11.1 / 11.3 / 12.9 / 15.9 / 27.9 lane-parallel and 12.5 / 12.6 / 12.8 / 13.5 / 18.4 in the general kernel)
    const bool rprod = !prep && (force && strstr(force, "rprod") ? true : force && strstr(force, "lprod") ? false : a.rows > 1u);
    static thread_local char name[24];
    bool taken = false, ok = false;
    auto run = [&](auto waves_tag, auto bpw_tag, auto splits_tag) {
        constexpr int W = decltype(waves_tag)::value, B = decltype(bpw_tag)::value, STEPS = B * (int)SPB;
        constexpr bool SPLITS = decltype(splits_tag)::value;  // the instance is built for shared panels too
        if constexpr (STEPS % GK == 0) {
            if (taken || a.ksteps != (uint32_t)(W * B)) return;
            // (an instance named in full, "fit12x8", rules the others out)
            char id[16];
            snprintf(id, sizeof id, "fit%dx%d", W, B);
            if (const char* named = force ? strstr(force, "fit") : nullptr)
                if (named[3] >= '0' && named[3] <= '9' && strncmp(named, id, strlen(id)) != 0) return;
            // the activation rows go through LDS while two workgroups still fit a compute unit that way
            bool xlds = a.rows <= kFitLdsRows;
            size_t lds = lds_for(W, STEPS, xlds);
            if (xlds && lds > 80u * 1024u && !prep) {
                xlds = false;
                lds = lds_for(W, STEPS, false);
            }
            if (lds > 156u * 1024u || (prep && STEPS % 4 != 0)) return;
            if constexpr (SPLITS) {
                if (split == 4u) ok = launch_fit<GK, W, B, W4, 4>(s, a, lds, xlds, rprod);
                else if (split == 2u) ok = launch_fit<GK, W, B, W4, 2>(s, a, lds, xlds, rprod);
                else ok = launch_fit<GK, W, B, W4>(s, a, lds, xlds, rprod);
            } else {
                if (split != 1u) return;
                ok = launch_fit<GK, W, B, W4>(s, a, lds, xlds, rprod);
            }
            taken = true;
            snprintf(name, sizeof name, "fit%dx%d%s%s", W, B, split == 4u ? "c8" : split == 2u ? "c16" : "", prep ? "-prep" : "");
        }
    };
    using std::integral_constant;
    using std::true_type;
    using std::false_type;
    if constexpr (W4) {  // K = 1024, 2048, 3072, 4096, 8192, 14336
        run(integral_constant<int, 4>{}, integral_constant<int, 4>{}, false_type{});
        run(integral_constant<int, 8>{}, integral_constant<int, 4>{}, false_type{});
        run(integral_constant<int, 8>{}, integral_constant<int, 6>{}, false_type{});
        run(integral_constant<int, 16>{}, integral_constant<int, 4>{}, false_type{});
        run(integral_constant<int, 16>{}, integral_constant<int, 8>{}, false_type{});
        run(integral_constant<int, 16>{}, integral_constant<int, 14>{}, false_type{});
    } else {  // K = 2048, 4096, 8192, 14336, 1024, 3072
        run(integral_constant<int, 16>{}, integral_constant<int, 4>{}, true_type{});
        run(integral_constant<int, 16>{}, integral_constant<int, 8>{}, true_type{});
        run(integral_constant<int, 16>{}, integral_constant<int, 16>{}, false_type{});
        run(integral_constant<int, 16>{}, integral_constant<int, 28>{}, false_type{});
        run(integral_constant<int, 8>{}, integral_constant<int, 4>{}, true_type{});
        // K = 3072, measured at N = 1024 (four workgroups a panel) and N = 6144: twelve waves of eight blocks are
        // faster with shared panels (1 / 32 rows: 3.75 / 5.0 us against 4.1 / 5.9) and with many rows (32 rows at
        // N = 6144: 7.2 against 10.2 us); eight waves of twelve by 0.1 us with up to eight rows on whole panels
        if (split == 1u && a.rows <= kFitLdsRows) run(integral_constant<int, 8>{}, integral_constant<int, 12>{}, true_type{});
        run(integral_constant<int, 12>{}, integral_constant<int, 8>{}, true_type{});
        run(integral_constant<int, 8>{}, integral_constant<int, 12>{}, true_type{});
    }
    return ok ? name : nullptr;
}

template <int MODE, int GK, int WAVES, bool W4, int SPLIT = 1, int ROWOP = kRowsPrepared>
bool launch_panel(hipStream_t s, const LinearArgs& a, size_t lds) {
    auto kern = gemv_panel_kernel<MODE, GK, WAVES, W4, SPLIT, ROWOP>;
    if (gemv_dry_run) return true;
    if (lds > 64u * 1024u) {
        static std::atomic<uint64_t> configured{0};
        if (!raise_lds_limit((const void*)kern, 160 * 1024, configured)) return false;
    }
    hipLaunchKernelGGL(kern, dim3((a.n + 31u) / 32u * SPLIT), dim3(WAVES * 64), lds, s, a);
    return hipGetLastError() == hipSuccess;
}

template <int MODE, int GK, int WAVES, bool W4, int ROWOP = kRowsPrepared>
bool launch_split(hipStream_t s, const LinearArgs& a, size_t lds, int split) {
    if (split == 4) return launch_panel<MODE, GK, WAVES, W4, 4, ROWOP>(s, a, lds);
    if (split == 2) return launch_panel<MODE, GK, WAVES, W4, 2, ROWOP>(s, a, lds);
    return launch_panel<MODE, GK, WAVES, W4, 1, ROWOP>(s, a, lds);
}

template <int MODE, int GK, bool W4 = false>
const char* launch_mode(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    if constexpr (MODE == (int)Epilogue::DequantF32) {
        if (const char* fit = launch_fit_mode<GK, W4>(s, a, cu_count, force)) return fit;
    }
    // blocks of the stream per panel, and the units a wave's run is made of
    constexpr uint32_t SPB = W4 ? 2 : 1, UNIT = GK > SPB ? GK : SPB;
    const uint32_t steps = ((a.k + 31u) / 32u + SPB - 1u) / SPB;  // 1 KiB blocks per panel
    // Measured at K=4096, N=14336: 4 blocks in flight per wave and 16 blocks per wave (two
    // workgroups of 8 waves resident per CU) stream fastest; more waves or deeper queues cost
    // occupancy, fewer leave the memory system short of requests.
    int waves = steps >= 16u * 16u ? 16 : steps >= 8u * 16u ? 8 : steps >= 4u * 16u ? 4 : 2;
    // Few panels (small N) leave most of the device idle and every wave latency bound on its
    // own short run: then split K further, down to one scale group per wave, until about 4096
    // waves are in flight.
    const uint32_t panels = (a.n + 31u) / 32u, chunks = ((a.k + 31u) / 32u + UNIT - 1) / UNIT;
    for (int more = waves * 2; more <= 16 && (uint32_t)more <= chunks && panels * (uint32_t)more <= 4096u; more *= 2)
        waves = more;
    if (force && strstr(force, "wv16")) waves = 16;
    else if (force && strstr(force, "wv8")) waves = 8;
    else if (force && strstr(force, "wv4")) waves = 4;
    else if (force && strstr(force, "wv2")) waves = 2;
    // f32 rows are prepared by workgroups of eight waves or more (waves past the end of a short row idle)
    if (a.x_f32 && waves < 8) waves = 8;
    // Fewer panels than half the compute units: two or four workgroups share each panel's
    // channels (only the 8- and 16-wave kernels are built that way; such shapes have them
    // unless K is tiny).
    int split = 1;
    if (waves >= 8) {
        split = panels * 4u <= (uint32_t)cu_count ? 4 : panels * 2u <= (uint32_t)cu_count ? 2 : 1;
        if (force && strstr(force, "c8")) split = 4;
        else if (force && strstr(force, "c16")) split = 2;
        else if (force && strstr(force, "c32")) split = 1;
    }
    const size_t ch_bytes = 128u / (size_t)split;  // one row of the workgroup's channels, int32 or f32
    size_t lds = MODE == (int)Epilogue::DequantF32 ? (size_t)a.groups * (a.rows + 1u) * ch_bytes
                                                    : (size_t)waves * a.rows * ch_bytes;
    // f32 activations: the kernel prepares them itself (codes and scales in LDS behind the rest)
    const bool prep = a.x_f32 != nullptr;
    if (prep) {
        // (a thread keeps kPrepPerThread elements of every row in registers between the two passes)
        if (MODE == (int)Epilogue::RequantRow || a.rows > kMaxPrepRows || waves < 8 ||
            a.k > (uint32_t)kPrepPerThread * (uint32_t)waves * 64u || (MODE != (int)Epilogue::DequantF32 && a.zw))
            return nullptr;
        lds += (size_t)a.rows * ((a.k + 15u) / 16u * 16u) + (size_t)a.rows * 4u + 16u;
        // RMSNorm in front: the sum of squares follows the 1024-thread row kernel, which rows of 1024
        // elements and more get
        if (a.row_gain && a.k < kNormThreads) return nullptr;
        // (that form is built for eight waves only: its double arithmetic does not fit the registers of sixteen)
        if (a.row_gain) {
            if (a.k > (uint32_t)kPrepPerThread * 8u * 64u) return nullptr;
            waves = 8;
        }
    }
    // the MFMA GEMM takes shapes whose group dots or scales do not fit
    if (lds > 156u * 1024u) return nullptr;
    bool ok = false;
    if constexpr (MODE != (int)Epilogue::RequantRow) {
        if (prep) {
            if constexpr (MODE == (int)Epilogue::DequantF32) {
                if (a.row_gain)
                    ok = launch_split<MODE, GK, 8, W4, kRowsNorm>(s, a, lds, split);
                else if (a.row_swiglu)
                    ok = waves == 16 ? launch_split<MODE, GK, 16, W4, kRowsSwiglu>(s, a, lds, split)
                                     : launch_split<MODE, GK, 8, W4, kRowsSwiglu>(s, a, lds, split);
                else
                    ok = waves == 16 ? launch_split<MODE, GK, 16, W4, kRowsF32>(s, a, lds, split)
                                     : launch_split<MODE, GK, 8, W4, kRowsF32>(s, a, lds, split);
            } else {
                ok = waves == 16 ? launch_split<MODE, GK, 16, W4, kRowsF32>(s, a, lds, split)
                                 : launch_split<MODE, GK, 8, W4, kRowsF32>(s, a, lds, split);
            }
            if (!ok) return nullptr;
            static const char* const prep_names[3][2] = {{"wv8-prep", "wv16-prep"},
                                                         {"wv8c16-prep", "wv16c16-prep"},
                                                         {"wv8c8-prep", "wv16c8-prep"}};
            return prep_names[split == 4 ? 2 : split == 2 ? 1 : 0][waves == 16 ? 1 : 0];
        }
    }
    if (waves == 16) ok = launch_split<MODE, GK, 16, W4>(s, a, lds, split);
    else if (waves == 8) ok = launch_split<MODE, GK, 8, W4>(s, a, lds, split);
    else if (waves == 4) ok = launch_panel<MODE, GK, 4, W4>(s, a, lds);
    else ok = launch_panel<MODE, GK, 2, W4>(s, a, lds);
    if (!ok) return nullptr;
    static const char* const names[3][4] = {{"wv2", "wv4", "wv8", "wv16"},
                                            {"wv2", "wv4", "wv8c16", "wv16c16"},
                                            {"wv2", "wv4", "wv8c8", "wv16c8"}};
    return names[split == 4 ? 2 : split == 2 ? 1 : 0][waves == 16 ? 3 : waves == 8 ? 2 : waves == 4 ? 1 : 0];
}

}  // namespace

void set_gemv_dry_run(bool on) { gemv_dry_run = on; }

const char* launch_gemv_stream(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    if (cu_count <= 0) cu_count = 256;
    if (a.rows == 0u || a.rows > kMaxGemvRows) return nullptr;
    const bool row_ops = a.row_gain || a.row_swiglu || a.add_to;
    if (row_ops && (!a.x_f32 || a.mode != Epilogue::DequantF32 || (a.row_gain && a.row_swiglu))) return nullptr;
    if (a.x_f32) {
        if (a.ldx < a.k) return nullptr;  // f32 rows of ldx elements
        if (a.row_swiglu && a.ldx < 2u * a.k) return nullptr;  // [gate | up]
    } else {
        if (((uintptr_t)a.x % 16u) != 0u) return nullptr;
        if (!a.x_operand_order && (a.ldx < 16u || (a.ldx % 16u) != 0u)) return nullptr;
    }
    static_assert(kMaxGemvRows <= kOperandOrderRows, "an operand-order buffer holds every row of a GEMV");
    if (a.weight_bits != 8u && !(a.weight_bits == 4u && a.mode == Epilogue::DequantF32)) return nullptr;
    const char* kind = nullptr;
    const char* family = nullptr;
    switch (a.mode) {
        case Epilogue::RequantTensor:
            family = "hip.qlinear.gemv-mfma";
            kind = launch_mode<(int)Epilogue::RequantTensor, 1>(s, a, cu_count, force);
            break;
        case Epilogue::RequantRow:
            family = "hip.qlinear.gemv-mfma-rowscale";
            kind = launch_mode<(int)Epilogue::RequantRow, 1>(s, a, cu_count, force);
            break;
        case Epilogue::DequantF32:
            if (a.weight_bits == 4u) {
                family = "hip.packed-linear.w4a8-gemv-mfma";
                switch (a.group_size) {
                    case 32: kind = launch_mode<(int)Epilogue::DequantF32, 1, true>(s, a, cu_count, force); break;
                    case 64: kind = launch_mode<(int)Epilogue::DequantF32, 2, true>(s, a, cu_count, force); break;
                    case 128: kind = launch_mode<(int)Epilogue::DequantF32, 4, true>(s, a, cu_count, force); break;
                    case 256: kind = launch_mode<(int)Epilogue::DequantF32, 8, true>(s, a, cu_count, force); break;
                    default: return nullptr;
                }
                break;
            }
            family = "hip.packed-linear.a8-gemv-mfma";
            switch (a.group_size) {
                case 32: kind = launch_mode<(int)Epilogue::DequantF32, 1>(s, a, cu_count, force); break;
                case 64: kind = launch_mode<(int)Epilogue::DequantF32, 2>(s, a, cu_count, force); break;
                case 128: kind = launch_mode<(int)Epilogue::DequantF32, 4>(s, a, cu_count, force); break;
                case 256: kind = launch_mode<(int)Epilogue::DequantF32, 8>(s, a, cu_count, force); break;
                default: return nullptr;
            }
            break;
    }
    if (!kind) return nullptr;
    static thread_local char name[96];
    snprintf(name, sizeof name, "%s.%s%s%s", family, kind, a.row_gain ? "-rmsnorm" : a.row_swiglu ? "-swiglu" : "",
             a.add_to ? "-add" : "");
    return name;
}

}  // namespace vxhip
