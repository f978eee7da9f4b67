// int8 MFMA GEMM for large prefill shapes on v_mfma_i32_16x16x64_i8: the requantizing epilogues
// of gemm_mfma.hip (same bytes), the same LDS stages and prepacked weights, but the matrix
// instruction with the long inner dimension.  Fed with random 8-bit operands the device is
// power limited and lowers its clock until the matrix pipes fit the budget; per delivered
// operation the 16x16x64 form moves a quarter of the accumulator registers of the 32x32x32
// form and sustains about 1.16 times its rate (3.7 against 3.2 POP/s in a register-only loop).
// Replaces, on gfx950, what the reference does on the CPU in vx_qgemm_w8a8_avx2
// (native/src/kernels/packed_quant_gemm.c:2411-2600).
//
// Operand roles as in gemm_mfma.hip: weights are the MFMA "A" operand (16 output channels x 64
// k), activations the "B" operand (64 k x 16 rows).  Lane l of an operand holds 16 consecutive
// k-bytes, chunk l/16 of the 64, of channel or row l%16; lane l of a result tile holds row
// l%16 and the four consecutive channels 4*(l/16) .. +3.
//
// One A operand is half of two adjacent 1 KiB blocks of the prepacked weight (common.h): lanes
// 0..31 read block 2t, lanes 32..63 block 2t+1, each its channel's two 16-byte slots.  The B
// operand comes from the row-major, XOR-swizzled activation image gemm_mfma.hip describes.
#include "common.h"
#include "device_math.h"
#include "epilogue.h"
#include "gemm_tile.h"

#include <stdio.h>
#include <string.h>

namespace vxhip {

namespace {

extern __shared__ __attribute__((aligned(1024))) char lds_raw[];

// WN x WM wavefronts, each owning TN x TM result tiles of 16 channels x 16 rows.  MODE is the
// requantizing Epilogue.  Two LDS stages of 128 k-bytes, i.e. two 64-wide MFMA steps each.
// FLIP: the activation bytes are unsigned; each activation fragment has its top bits flipped (one XOR per
// dword) in front of the first MFMA row of the step that uses it, so that a U8 input needs no pass of its own.
// DQ: the DequantizeLinear behind the QLinear rides in the epilogue -- each byte's value goes out as
// f32((q - dq_zp) * dq_scale) (a.dq_out, 16 bytes a lane and tile), the bytes themselves only if a.y is set.
template <int WN, int WM, int TN, int TM, int MODE, bool FLIP = false, bool DQ = false>
__global__ __launch_bounds__(WN* WM * 64) void gemm_k64_kernel(const GemmParams p) {
    static_assert(MODE != (int)Epilogue::DequantF32, "requantizing epilogues only");
    static_assert(TN % 4 == 0, "the epilogue transposes four channel tiles at a time");
    constexpr int NWAVES = WN * WM;
    constexpr int BN = WN * TN * 16, BM = WM * TM * 16;
    constexpr int KS = 4;  // 32-byte k-steps per stage (the unit of the weight blocks)
    constexpr int WBLK = (BN / 32) * KS, XBLK = BM / 8;  // 1 KiB blocks per stage
    static_assert(WBLK % NWAVES == 0 && XBLK % NWAVES == 0, "blocks must divide over waves");
    constexpr int WLOADS = WBLK / NWAVES, XLOADS = XBLK / NWAVES, NLOADS = WLOADS + XLOADS;
    constexpr int STAGE_BYTES = (WBLK + XBLK) * 1024;
    const LinearArgs& a = p.a;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wave_n = wave % WN, wave_m = wave / WN;

    uint32_t m0, n0;
    {
        const TileOrigin t = tile_of_workgroup<BN, BM>(p);
        if (!t.valid) return;
        m0 = t.m0;
        n0 = t.n0;
    }

    // ---- operand loads (global -> LDS), as in gemm_mfma.hip ------------------------------
    const uint32_t w_lane = lane * 16u;
    const uint32_t panel_bytes = a.ksteps * 1024u;
    const int8_t* const w_tile = a.w + (size_t)(n0 / 32u) * panel_bytes;
    const uint32_t last_chunk = (a.k - 1u) / 16u;
    const uint32_t my_chunk = (lane & 7) ^ ((lane >> 3) & 7);
    uint32_t xrow[XLOADS];
#pragma unroll
    for (int i = 0; i < XLOADS; i++) {
        const int b = wave + i * NWAVES;
        uint32_t row = m0 + b * 8 + (lane >> 3);
        row = min(row, a.rows - 1u);
        xrow[i] = row * a.ldx;
    }
    const uint32_t ksteps_real = (a.k + 31u) / 32u;
    const uint32_t nkb = (ksteps_real + KS - 1) / KS;
    auto issue_one = [&](auto t_tag, uint32_t kb, int stage) {
        constexpr int t = decltype(t_tag)::value;
        kb = min(kb, nkb - 1u);  // a block past the end refills a stage nobody reads
        char* base = lds_raw + stage * STAGE_BYTES;
        if constexpr (t < WLOADS) {
            const uint32_t b = wave + t * NWAVES;
            const int8_t* src = w_tile + (size_t)(b / KS) * panel_bytes + (size_t)(kb * KS + b % KS) * 1024u;
            load_to_lds16(src + w_lane, base + b * 1024);
        } else {
            const uint32_t chunk16 = min(kb * 8u + my_chunk, last_chunk) * 16u;
            const uint32_t b = wave + (t - WLOADS) * NWAVES;
            load_to_lds16(a.x + (xrow[t - WLOADS] + chunk16), base + (WBLK + b) * 1024);
        }
    };

    v4i acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++) acc[i][j] = v4i{0, 0, 0, 0};

    float row_scale[TM];
    if constexpr (MODE == (int)Epilogue::RequantRow) {
#pragma unroll
        for (int j = 0; j < TM; j++) {
            const uint32_t m = min(m0 + (wave_m * TM + j) * 16 + (lane & 15), a.rows - 1u);
            row_scale[j] = a.row_scale[m];
        }
    }

    // ---- fragment addressing -----------------------------------------------------------
    // weights: tile i of the wave is half (i%2) of panel wave_n*TN/2 + i/2; MFMA step s of the stage
    // is the block pair (2s, 2s+1).  Lane l reads block 2s + l/32, slot 16*(i%2) + l%16 + 32*((l/16)%2).
    const uint32_t a_frag = (uint32_t)(wave_n * (TN / 2) * KS) * 1024u + (uint32_t)(lane >> 5) * 1024u +
                            (uint32_t)((lane & 15) + 32 * ((lane >> 4) & 1)) * 16u;
    // activations: row (wave_m*TM + j)*16 + l%16 of 128 bytes, chunk 4s + l/16 at slot chunk ^ (row%8)
    const uint32_t x_row = WBLK * 1024u + ((uint32_t)(wave_m * TM * 16) + (lane & 15)) * 128u;
    uint32_t x_slot[2];
#pragma unroll
    for (int s = 0; s < 2; s++) x_slot[s] = (((4u * s + (lane >> 4)) ^ (lane & 7u)) << 4);

    v4i af[TN], bf[2][TM];
    auto read_a = [&](auto i_tag, const char* stage, auto s_tag) {
        constexpr int i = decltype(i_tag)::value, s = decltype(s_tag)::value;
        af[i] = *reinterpret_cast<const v4i*>(stage + a_frag + ((i / 2) * KS + 2 * s) * 1024 + (i & 1) * 256);
    };
    auto read_b = [&](auto j_tag, const char* stage, auto s_tag) {
        constexpr int j = decltype(j_tag)::value, s = decltype(s_tag)::value;
        bf[s][j] = *reinterpret_cast<const v4i*>(stage + x_row + j * 16 * 128 + x_slot[s]);
    };

    // ---- main loop -------------------------------------------------------------------------
    // A k-block is two MFMA steps of TN rows of TM MFMAs (row i: channel tile i against every row
    // tile).  The weight fragment of a row is replaced as soon as the row has issued, by the same
    // row's fragment of the following step; the activation fragments are double buffered by step
    // parity.  Step 0 reads step 1's fragments from the same stage.  Step 1 runs its first RB rows,
    // then waits for its own LDS reads and its loads of the next k-block, passes the barrier,
    // and from there on reads the next stage's step 0 and refills the current stage for k-block
    // kb+2, every request placed behind a fixed MFMA so that LDS reads, global loads and MFMAs
    // issue evenly mixed.
    constexpr int RB = 1;
    static_assert(TN - RB >= TM && TN >= TM, "every activation fragment needs a row to be re-read behind");
    // both stages are requested at once: the second k-block's latency then runs beside the first's
    static_for<NLOADS>([&](auto t) { issue_one(t, 0u, 0); });
    static_for<NLOADS>([&](auto t) { issue_one(t, 1u, 1); });

    float* lds_f0 = reinterpret_cast<float*>(lds_raw + 2 * STAGE_BYTES);
    int32_t* lds_cb = reinterpret_cast<int32_t*>(lds_f0 + BN);
    float* lds_bo = reinterpret_cast<float*>(lds_cb + BN);
    int32_t* lds_zw = reinterpret_cast<int32_t*>(lds_bo + BN);
    for (int t = threadIdx.x; t < BN; t += NWAVES * 64) {
        const ChannelConsts c = channel_consts<MODE>(a, n0 + t);
        lds_f0[t] = c.f0;
        lds_cb[t] = c.cb;
        lds_bo[t] = c.bo;
        lds_zw[t] = c.zw;
    }

    auto mfma_row = [&](auto i_tag, auto s_tag, auto&& after) {
        constexpr int i = decltype(i_tag)::value, s = decltype(s_tag)::value;
        static_for<TM>([&](auto j_tag) {
            constexpr int j = decltype(j_tag)::value;
            if constexpr (FLIP && i == 0) bf[s][j] ^= (int)0x80808080u;
            acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[i], bf[s][j], acc[i][j], 0, 0, 0);
            after(j_tag);
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    wait_vmcnt<0>();
    wg_barrier();
    static_for<TM>([&](auto j) { read_b(j, lds_raw, IC<0>{}); });
    static_for<TN>([&](auto i) { read_a(i, lds_raw, IC<0>{}); });

    auto k_block = [&](uint32_t kb, auto last_tag) {
        constexpr bool LAST = decltype(last_tag)::value;
        const int cur = kb & 1;
        const char* stage = lds_raw + cur * STAGE_BYTES;
        const char* next = lds_raw + (cur ^ 1) * STAGE_BYTES;
        // step 0: behind row i, the same row's weight fragment of step 1; the activation fragments of
        // step 1 go out behind the first MFMAs of rows 0 .. TM-1
        static_for<TN>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            mfma_row(i_tag, IC<0>{}, [&](auto j_tag) {
                constexpr int j = decltype(j_tag)::value;
                if constexpr (j == 0 && i < TM) read_b(IC<(i < TM ? i : 0)>{}, stage, IC<1>{});
                if constexpr (j == TM - 1) read_a(i_tag, stage, IC<1>{});
            });
        });
        if constexpr (LAST) {
            static_for<TN>([&](auto i_tag) { mfma_row(i_tag, IC<1>{}, [&](auto) {}); });
        } else {
            static_for<RB>([&](auto i_tag) { mfma_row(i_tag, IC<1>{}, [&](auto) {}); });
            wait_lgkm0();     // my reads of this stage have landed in registers
            wait_vmcnt<0>();  // my loads of the next k-block have landed
            wg_barrier();
            static_for<RB>([&](auto i_tag) { read_a(i_tag, next, IC<0>{}); });
            // (TN - RB) * TM MFMAs carry the NLOADS loads of k-block kb+2 and TM activation reads
            constexpr int REST = (TN - RB) * TM;
            static_for<TN - RB>([&](auto r_tag) {
                constexpr int i = RB + decltype(r_tag)::value;
                mfma_row(IC<i>{}, IC<1>{}, [&](auto j_tag) {
                    constexpr int j = decltype(j_tag)::value;
                    constexpr int m = (i - RB) * TM + j;
                    if constexpr (j == 0 && i - RB < TM) read_b(IC<(i - RB < TM ? i - RB : 0)>{}, next, IC<0>{});
                    if constexpr (j == TM - 1) read_a(IC<i>{}, next, IC<0>{});
                    static_for<NLOADS>([&](auto l_tag) {
                        constexpr int l = decltype(l_tag)::value;
                        if constexpr ((l * REST) / NLOADS == m) issue_one(l_tag, kb + 2u, cur);
                    });
                });
            });
        }
    };
    for (uint32_t kb = 0; kb + 1 < nkb; kb++) k_block(kb, std::false_type{});
    k_block(nkb - 1u, std::true_type{});
    wait_vmcnt<0>();  // nothing of this workgroup may still be writing LDS when the epilogue runs

    // ---- epilogue: requantize, pack, transpose across the four lane groups, 16-byte stores ----
    const float zp_f = (float)a.out_zp, lo_f = (float)a.out_lo, hi_f = (float)a.out_hi;
    const float so = a.output_scale, sr = a.output_scale_recip;
    [[maybe_unused]] const float dq_zp_f = (float)a.dq_zp;
    uint32_t mrow[TM];
    int32_t rsum[TM];
    uint32_t miss1 = 1, miss2 = 1;
    if (MODE == (int)Epilogue::RequantRow && a.div_proof) {
        miss1 = a.div_proof[0];
        miss2 = a.div_proof[1];
    }
    bool lean = a.zw == nullptr;
    if constexpr (MODE == (int)Epilogue::RequantRow) lean = lean && fast_div_in_range(so) && miss2 == 0;
    const bool no_int_terms = a.int_bias_zero && (MODE == (int)Epilogue::RequantRow || a.input_zp == 0);
    const bool bare_ok = no_int_terms && a.out_zp == 0 && (MODE != (int)Epilogue::RequantRow || miss1 == 0);
    bool bad = false;
#pragma unroll
    for (int j = 0; j < TM; j++) {
        mrow[j] = m0 + (wave_m * TM + j) * 16 + (lane & 15);
        rsum[j] = (a.zw && mrow[j] < a.rows) ? a.rowsum[mrow[j]] : 0;
        if constexpr (MODE == (int)Epilogue::RequantRow) {
            const float plo = __fmul_rn(row_scale[j], a.wscale_min), phi = __fmul_rn(row_scale[j], a.wscale_max);
            if (mrow[j] < a.rows) {
                bad |= !scale_valid(__fdiv_rn(plo, so)) || !scale_valid(__fdiv_rn(phi, so));
                lean &= fast_div_in_range(plo) && fast_div_in_range(phi);
            }
        }
    }
    if (bad) atomicOr(a.fault, (uint32_t)kFaultBadMultiplier);
    const bool wave_lean = __builtin_amdgcn_ballot_w64(!lean) == 0ull;
    // LEVEL 0: general.  1: no weight zero points, every quotient in the range of the proved short
    // division.  2: in addition nothing to add to the accumulator or the product (gemm_mfma.hip).
    auto run = [&](auto level_tag, auto streamed_tag) {
        constexpr int LEVEL = decltype(level_tag)::value;
        constexpr bool STREAMED = decltype(streamed_tag)::value;
        constexpr bool LEAN = LEVEL >= 1, BARE = LEVEL == 2;
#pragma unroll
        for (int h = 0; h < TN / 4; h++) {
            v4f f0[4], bo[4];
            v4i cb[4], zw[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int c0 = (wave_n * TN + h * 4 + t) * 16 + (lane >> 4) * 4;
                f0[t] = *reinterpret_cast<const v4f*>(lds_f0 + c0);
                cb[t] = *reinterpret_cast<const v4i*>(lds_cb + c0);
                bo[t] = v4f{0.f, 0.f, 0.f, 0.f};
                zw[t] = v4i{0, 0, 0, 0};
                if (MODE == (int)Epilogue::RequantRow && (BARE || a.bias_row)) bo[t] = *reinterpret_cast<const v4f*>(lds_bo + c0);
                if (!LEAN && a.zw) zw[t] = *reinterpret_cast<const v4i*>(lds_zw + c0);
            }
#pragma unroll
            for (int j = 0; j < TM; j++) {
                uint32_t pk[4];
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    uint32_t u[4];
                    v4f dq;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        uint32_t total = (uint32_t)acc[h * 4 + t][j][e];
                        if (!BARE) total += (uint32_t)cb[t][e];
                        if (!LEAN) total -= (uint32_t)zw[t][e] * (uint32_t)rsum[j];
                        float mu = f0[t][e];
                        if constexpr (MODE == (int)Epilogue::RequantRow) {
                            const float prod = __fmul_rn(row_scale[j], f0[t][e]);
                            mu = BARE   ? div_by_uniform_once(prod, so, sr)
                                 : LEAN ? div_by_uniform(prod, so, sr)
                                        : __fdiv_rn(prod, so);
                        }
                        float v = __fmul_rn((float)(int32_t)total, mu);
                        if (!BARE) v = __fadd_rn(v, zp_f);
                        if (MODE == (int)Epilogue::RequantRow && (BARE || a.bias_row)) v = __fadd_rn(v, bo[t][e]);
                        // clamp, then ties-to-even by adding 1.5 * 2^23: the low mantissa bits are the integer
                        v = __builtin_amdgcn_fmed3f(v, lo_f, hi_f);
                        const float rounded = __fadd_rn(v, 12582912.0f);
                        u[e] = __float_as_uint(rounded);
                        if constexpr (DQ) {
                            // the byte's value as a float (exact), then the DequantizeLinear's one rounding
                            const float qf = __fsub_rn(rounded, 12582912.0f);
                            dq[e] = __fmul_rn(__fsub_rn(qf, dq_zp_f), a.dq_scale);
                        }
                    }
                    if constexpr (DQ) {
                        const uint32_t nq = n0 + (wave_n * TN + h * 4 + t) * 16 + (lane >> 4) * 4;
                        if (mrow[j] < a.rows && nq < a.n) *reinterpret_cast<v4f*>(a.dq_out + (size_t)mrow[j] * a.n + nq) = dq;
                    }
                    const uint32_t p01 = __builtin_amdgcn_perm(u[1], u[0], 0x0c0c0400u);
                    const uint32_t p23 = __builtin_amdgcn_perm(u[3], u[2], 0x0c0c0400u);
                    pk[t] = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
                }
                // pk[t] in lane group g = channels 4g..4g+3 of tile t.  Transpose the 4 x 4 of (tile, lane
                // group): afterwards lane group g holds the four dwords of tile g, 16 consecutive bytes.
                const auto s02 = __builtin_amdgcn_permlane32_swap(pk[0], pk[2], false, false);
                const auto s13 = __builtin_amdgcn_permlane32_swap(pk[1], pk[3], false, false);
                const auto r01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
                const auto r23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
                const uint32_t n16 = n0 + (wave_n * TN + h * 4 + (lane >> 4)) * 16;
                if ((!DQ || a.y) && mrow[j] < a.rows && n16 < a.n) {
                    const v4i v = v4i{(int)r01[0], (int)r01[1], (int)r23[0], (int)r23[1]};
                    store_stream<STREAMED>(reinterpret_cast<v4i*>((uint8_t*)a.y + (size_t)mrow[j] * a.n + n16), v);
                }
            }
        }
    };
    // (the two straight-line levels come in a streamed copy as well; the general one stores plainly)
    const bool streamed = !DQ && a.stream_out != 0u;  // (the dequantizing form's f32 stores are never streamed)
    if (wave_lean && bare_ok) {
        if (streamed) run(IC<2>{}, std::true_type{});
        else run(IC<2>{}, std::false_type{});
    } else if (wave_lean) {
        if (streamed) run(IC<1>{}, std::true_type{});
        else run(IC<1>{}, std::false_type{});
    } else {
        run(IC<0>{}, std::false_type{});
    }
}

// ---- the dequantizing form (PackedLinear under DYNAMIC_I8) ----------------------------------------
// sum += f32(dot_g) * (s_a * s_w[n][g]) in ascending group order with every product and sum rounded
// on its own (packed_linear_ops.inc:1498-1504): four VALU operations per output and group against
// 2 * group_size matrix operations, so the kernel is bound by the vector pipe, not by the MFMAs.
// It therefore runs small wave tiles (64 channels x 32 rows) at four waves per SIMD and leaves the
// overlap of one wave's fold with the other waves' MFMAs to the hardware: two workgroups of
// 128 x 128 per compute unit, each with its own barrier.  GK: 64-wide MFMA steps per scale group
// (1, 2 or 4).  W4: four-bit weights; a 1 KiB block then holds the block pair of one MFMA step, low
// nibbles for its first 32 k, high nibbles for the rest, and a lane shifts its half into place.
// The scales of the groups that end in a k-block travel as the tail of that k-block's LDS stage.
// UNI: every channel has one scale for all its groups (a per-channel scale replicated, which is what
// per-channel quantization exports); s_a * s_w is then formed once per output instead of once per
// output and group -- the same products, so the same bits -- and the fold is three operations.
template <int GK, bool W4, int WM, int NS, bool UNI>
__global__ __launch_bounds__(WM * 128, 4) void gemm_k64_f32_kernel(const GemmParams p) {
    constexpr int WN = 2, TN = 4, TM = 2, NWAVES = WN * WM;
    constexpr int BN = WN * TN * 16, BM = WM * TM * 16;  // 128 channels x 128 or 256 rows
    constexpr int KS = 4, KB = W4 ? 2 : 4;  // 32-byte k-steps and 1 KiB weight blocks per panel and stage
    constexpr int WBLK = (BN / 32) * KB, XBLK = BM / 8;
    constexpr int WLOADS = WBLK / NWAVES, XLOADS = XBLK / NWAVES;
    static_assert(WBLK % NWAVES == 0 && XBLK % NWAVES == 0, "blocks must divide over waves");
    constexpr int GPB = GK == 1 ? 2 : 1;  // scale groups that end in a k-block (GK == 4: every second block)
    constexpr int SCALE_OFF = (WBLK + XBLK) * 1024;
    constexpr int STAGE_BYTES = SCALE_OFF + GPB * BN * 4;
    constexpr int NLOADS = WLOADS + XLOADS;
    const LinearArgs& a = p.a;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wave_n = wave % WN, wave_m = wave / WN;
    uint32_t m0, n0;
    {
        const TileOrigin t = tile_of_workgroup<BN, BM, 8>(p);
        if (!t.valid) return;
        m0 = t.m0;
        n0 = t.n0;
    }

    const uint32_t w_lane = lane * 16u;
    const uint32_t panel_bytes = a.ksteps * 1024u;
    const int8_t* const w_tile = a.w + (size_t)(n0 / 32u) * panel_bytes;
    const uint32_t last_chunk = (a.k - 1u) / 16u;
    const uint32_t my_chunk = (lane & 7) ^ ((lane >> 3) & 7);
    uint32_t xrow[XLOADS];
#pragma unroll
    for (int i = 0; i < XLOADS; i++) {
        const int b = wave + i * NWAVES;
        uint32_t row = m0 + b * 8 + (lane >> 3);
        row = min(row, a.rows - 1u);
        xrow[i] = row * a.ldx;
    }
    const uint32_t ksteps_real = (a.k + 31u) / 32u;
    const uint32_t nkb = (ksteps_real + KS - 1) / KS;
    auto issue_block = [&](uint32_t kb, int stage) {
        char* base = lds_raw + stage * STAGE_BYTES;
        // the scales of the groups that end in this k-block: 64 channels per wavefront, 4 bytes per lane
        if (!UNI && wave < GPB * (BN / 64)) {
            const uint32_t slot = wave / (BN / 64), half = wave % (BN / 64);
            const uint32_t g = min(GK == 1 ? kb * 2u + slot : GK == 2 ? kb : kb / 2u, a.groups - 1u);
            load_to_lds4(a.scales_t + (size_t)g * a.n_pad + n0 + half * 64 + lane,
                         base + SCALE_OFF + (slot * BN + half * 64) * 4);
        }
        static_for<NLOADS>([&](auto t_tag) {
            constexpr int t = decltype(t_tag)::value;
            if constexpr (t < WLOADS) {
                const uint32_t b = wave + t * NWAVES;
                const int8_t* src = w_tile + (size_t)(b / KB) * panel_bytes + (size_t)(kb * KB + b % KB) * 1024u;
                load_to_lds16(src + w_lane, base + b * 1024);
            } else {
                const uint32_t chunk16 = min(kb * 8u + my_chunk, last_chunk) * 16u;
                const uint32_t b = wave + (t - WLOADS) * NWAVES;
                load_to_lds16(a.x + (xrow[t - WLOADS] + chunk16), base + (WBLK + b) * 1024);
            }
        });
    };

    v4i acc[TN][TM];
    v4f fsum[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++) {
            acc[i][j] = v4i{0, 0, 0, 0};
            fsum[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
        }
    float row_scale[TM];
#pragma unroll
    for (int j = 0; j < TM; j++) {
        const uint32_t m = min(m0 + (wave_m * TM + j) * 16 + (lane & 15), a.rows - 1u);
        row_scale[j] = a.row_scale[m];
    }

    // fragment addressing (see the requantizing kernel); four-bit weights: one block per MFMA step,
    // the lane's 16-byte slot is the same for both halves of the step
    const uint32_t a_frag = W4 ? (uint32_t)(wave_n * (TN / 2) * KB) * 1024u + (uint32_t)((lane & 15) + 32 * ((lane >> 4) & 1)) * 16u
                               : (uint32_t)(wave_n * (TN / 2) * KB) * 1024u + (uint32_t)(lane >> 5) * 1024u +
                                     (uint32_t)((lane & 15) + 32 * ((lane >> 4) & 1)) * 16u;
    const uint32_t nib_shift = lane < 32 ? 4u : 0u;
    const uint32_t x_row = WBLK * 1024u + ((uint32_t)(wave_m * TM * 16) + (lane & 15)) * 128u;
    uint32_t x_slot[2];
#pragma unroll
    for (int s = 0; s < 2; s++) x_slot[s] = (((4u * s + (lane >> 4)) ^ (lane & 7u)) << 4);
    const uint32_t sw_lane = SCALE_OFF + (uint32_t)(wave_n * TN * 16 + (lane >> 4) * 4) * 4u;

    // UNI: the products s_a * s_w of the lane's outputs
    float gs_all[UNI ? TN : 1][UNI ? TM : 1][4];
    if constexpr (UNI) {
#pragma unroll
        for (int i = 0; i < TN; i++) {
            const v4f sw = *reinterpret_cast<const v4f*>(a.scales_t + n0 + (wave_n * TN + i) * 16 + (lane >> 4) * 4);
#pragma unroll
            for (int j = 0; j < TM; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) gs_all[i][j][e] = __fmul_rn(row_scale[j], sw[e]);
        }
    }
    // fold of scale-group slot `slot` of the stage: every tile of the wave
    auto fold = [&](const char* stage, int slot) {
#pragma unroll
        for (int i = 0; i < TN; i++) {
            v4f sw = {0.f, 0.f, 0.f, 0.f};
            if constexpr (!UNI) sw = *reinterpret_cast<const v4f*>(stage + sw_lane + (slot * BN + i * 16) * 4);
#pragma unroll
            for (int j = 0; j < TM; j++) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float gs = UNI ? gs_all[UNI ? i : 0][UNI ? j : 0][e] : __fmul_rn(row_scale[j], sw[e]);
                    // four-bit operands carry a factor 16; the dot is exact, so is the shift
                    const float term = __fmul_rn((float)(acc[i][j][e] >> (W4 ? 4 : 0)), gs);
                    fsum[i][j][e] = __fadd_rn(fsum[i][j][e], term);
                }
            }
        }
    };

    // NS stages: k-blocks kb+1 .. kb+NS-1 are in flight while k-block kb is consumed.  One barrier per
    // k-block, at its top: behind it every wave's loads of the block have landed and every wave is done
    // with the previous block, whose stage is refilled at once.  (Blocks past the end are clamped to the
    // last one, so the count of loads in flight is the same in every iteration.)
    static_for<NS - 1>([&](auto b_tag) { issue_block(min((uint32_t)decltype(b_tag)::value, nkb - 1u), decltype(b_tag)::value); });
    int cur = 0, refill = NS - 1;
    for (uint32_t kb = 0; kb < nkb; kb++) {
        wait_vmcnt<(NS - 2) * NLOADS>();  // (waves that also carry a scale load wait for one load more than they must)
        wg_barrier();
        issue_block(min(kb + NS - 1u, nkb - 1u), refill);
        const char* stage = lds_raw + cur * STAGE_BYTES;
#pragma unroll
        for (int s = 0; s < 2; s++) {
            v4i af[TN], bf[TM];
#pragma unroll
            for (int j = 0; j < TM; j++) bf[j] = *reinterpret_cast<const v4i*>(stage + x_row + j * 16 * 128 + x_slot[s]);
#pragma unroll
            for (int i = 0; i < TN; i++) {
                if constexpr (W4) {
                    const v4i raw = *reinterpret_cast<const v4i*>(stage + a_frag + ((i / 2) * KB + s) * 1024 + (i & 1) * 256);
#pragma unroll
                    for (int d = 0; d < 4; d++) af[i][d] = (raw[d] << nib_shift) & (int)0xf0f0f0f0u;
                } else {
                    af[i] = *reinterpret_cast<const v4i*>(stage + a_frag + ((i / 2) * KB + 2 * s) * 1024 + (i & 1) * 256);
                }
            }
            // first MFMA step of a scale group: accumulate onto zero instead of clearing registers
            const bool fresh = GK == 1 || (GK == 2 && s == 0) || (GK == 4 && s == 0 && (kb & 1u) == 0u);
            const v4i zero = {0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < TN; i++)
#pragma unroll
                for (int j = 0; j < TM; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[i], bf[j], fresh ? zero : acc[i][j], 0, 0, 0);
            // last MFMA step of a scale group (or of the row): fold it.  A group that starts past the
            // end of k does not exist (its dot would be zero, but adding +0.0 can flip a -0.0 sum).
            if constexpr (GK == 1) {
                if (kb * 2u + s < a.groups) fold(stage, s);
            } else if constexpr (GK == 2) {
                if (s == 1) fold(stage, 0);
            } else {
                if (s == 1 && ((kb & 1u) == 1u || kb + 1u == nkb)) fold(stage, 0);
            }
        }
        refill = cur;
        cur = cur + 1 == NS ? 0 : cur + 1;
    }
    wait_vmcnt<0>();

    // ---- epilogue: + bias, 16-byte stores (a lane owns row l%16 and four consecutive channels) ----
    // (streamed stores, as in the requantizing kernel, were measured here too: config 5's 32 MiB of f32 output
    // 0.7 % faster, the second copy of the epilogue 1.3 % slower where it is not used; left out)
    const bool vec_ok = (a.n % 4u) == 0u;
#pragma unroll
    for (int j = 0; j < TM; j++) {
        const uint32_t m = m0 + (wave_m * TM + j) * 16 + (lane & 15);
        if (m >= a.rows) continue;
#pragma unroll
        for (int i = 0; i < TN; i++) {
            const uint32_t n = n0 + (wave_n * TN + i) * 16 + (lane >> 4) * 4;
            if (n >= a.n) continue;
            const v4f b = *reinterpret_cast<const v4f*>(a.bias_f32 + n);
            v4f out;
#pragma unroll
            for (int e = 0; e < 4; e++) out[e] = __fadd_rn(fsum[i][j][e], b[e]);
            float* y = (float*)a.y + (size_t)m * a.n + n;
            if (vec_ok) {
                *reinterpret_cast<v4f*>(y) = out;
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < a.n) y[e] = out[e];
            }
        }
    }
}

template <int GK, bool W4, int WM, int NS, bool UNI>
bool launch_f32_as(hipStream_t s, const LinearArgs& a);

template <int GK, bool W4, int WM, int NS>
bool launch_f32(hipStream_t s, const LinearArgs& a) {
    // (the instances listed keep the products in registers without spilling at four waves per SIMD;
    // the others would lose more to scratch traffic than the fourth operation costs)
    constexpr bool kUniformFits = GK == 1 || (GK == 2 && (W4 || WM == 8));
    if constexpr (kUniformFits) {
        if (a.uniform_group_scales) return launch_f32_as<GK, W4, WM, NS, true>(s, a);
    }
    return launch_f32_as<GK, W4, WM, NS, false>(s, a);
}

template <int GK, bool W4, int WM, int NS, bool UNI>
bool launch_f32_as(hipStream_t s, const LinearArgs& a) {
    constexpr int BN = 128, BM = WM * 32;
    constexpr int LDS = NS * (((BN / 32) * (W4 ? 2 : 4) + BM / 8) * 1024 + (GK == 1 ? 2 : 1) * BN * 4);
    static_assert(LDS <= 160 * 1024, "stages do not fit the LDS");
    static std::atomic<uint64_t> configured{0};
    auto kern = gemm_k64_f32_kernel<GK, W4, WM, NS, UNI>;
    if (!raise_lds_limit((const void*)kern, LDS, configured)) return false;
    GemmParams p;
    p.a = a;
    p.tiles_n = (a.n + BN - 1) / BN;
    p.tiles_m = (a.rows + BM - 1) / BM;
    const uint32_t total = p.tiles_n * p.tiles_m;
    const uint32_t grid = ((total + 7u) / 8u) * 8u;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WM * 128), LDS, s, p);
    return hipGetLastError() == hipSuccess;
}

template <int WN, int WM, int TN, int TM, int MODE, bool FLIP = false, bool DQ = false>
bool launch_one(hipStream_t s, const LinearArgs& a) {
    constexpr int BN = WN * TN * 16, BM = WM * TM * 16;
    constexpr int LDS = 2 * ((BN / 32) * 4 + BM / 8) * 1024 + BN * 16;
    static_assert(LDS <= 160 * 1024, "stages do not fit the LDS");
    static std::atomic<uint64_t> configured{0};
    auto kern = gemm_k64_kernel<WN, WM, TN, TM, MODE, FLIP, DQ>;
    if (!raise_lds_limit((const void*)kern, LDS, configured)) return false;
    GemmParams p;
    p.a = a;
    p.a.stream_out = (size_t)a.rows * a.n >= (12u << 20) ? 1u : 0u;  // (see store_stream: the byte output only)
    p.tiles_n = (a.n + BN - 1) / BN;
    p.tiles_m = (a.rows + BM - 1) / BM;
    const uint32_t total = p.tiles_n * p.tiles_m;
    const uint32_t grid = ((total + 7u) / 8u) * 8u;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WN * WM * 64), LDS, s, p);
    return hipGetLastError() == hipSuccess;
}

}  // namespace

// The requantizing GEMM on 16x16x64 MFMAs.  tile 0: 256 channels x 256 rows per workgroup; 1: 256 x
// 128.  The caller has checked what the straight-line epilogue needs (n % 16 == 0, a 16-byte
// aligned byte output, no accumulator dump).  Returns the tile's name, or null if nothing ran.
const char* launch_gemm_k64(hipStream_t s, const LinearArgs& a, int tile) {
    const bool row = a.mode == Epilogue::RequantRow;
    if (a.mode == Epilogue::DequantF32) return nullptr;
    constexpr int T = (int)Epilogue::RequantTensor, R = (int)Epilogue::RequantRow;
    const bool dq = a.dq_out != nullptr;
    bool ok = false;
    if (a.x_flip_mask) {
        // unsigned activation bytes, flipped in the kernel (the per-tensor form only: per-token scales come with I8 rows)
        if (row) return nullptr;
        if (tile == 0) ok = dq ? launch_one<2, 4, 8, 4, T, true, true>(s, a) : launch_one<2, 4, 8, 4, T, true>(s, a);
        else ok = dq ? launch_one<2, 4, 8, 2, T, true, true>(s, a) : launch_one<2, 4, 8, 2, T, true>(s, a);
    } else if (tile == 0) {
        ok = row ? (dq ? launch_one<2, 4, 8, 4, R, false, true>(s, a) : launch_one<2, 4, 8, 4, R>(s, a))
                 : (dq ? launch_one<2, 4, 8, 4, T, false, true>(s, a) : launch_one<2, 4, 8, 4, T>(s, a));
    } else {
        ok = row ? (dq ? launch_one<2, 4, 8, 2, R, false, true>(s, a) : launch_one<2, 4, 8, 2, R>(s, a))
                 : (dq ? launch_one<2, 4, 8, 2, T, false, true>(s, a) : launch_one<2, 4, 8, 2, T>(s, a));
    }
    if (!ok) return nullptr;
    return tile == 0 ? (dq ? "t256x256k64-dq" : "t256x256k64") : (dq ? "t256x128k64-dq" : "t256x128k64");
}

// The dequantizing GEMM on 16x16x64 MFMAs; group sizes 64, 128 and 256.  deep: one workgroup of
// sixteen waves per compute unit on a 128 x 256 tile with three LDS stages (eight-bit weights only),
// else two workgroups of eight waves on 128 x 128 tiles with two stages each.
const char* launch_gemm_k64_f32(hipStream_t s, const LinearArgs& a, bool deep) {
    if (a.mode != Epilogue::DequantF32 || a.acc_out || !a.y) return nullptr;
    bool ok = false;
    if (a.weight_bits == 4u) {
        deep = false;
        switch (a.group_size) {
            case 64: ok = launch_f32<1, true, 4, 2>(s, a); break;
            case 128: ok = launch_f32<2, true, 4, 2>(s, a); break;
            case 256: ok = launch_f32<4, true, 4, 2>(s, a); break;
            default: return nullptr;
        }
    } else if (deep) {
        switch (a.group_size) {
            case 64: ok = launch_f32<1, false, 8, 3>(s, a); break;
            case 128: ok = launch_f32<2, false, 8, 3>(s, a); break;
            case 256: ok = launch_f32<4, false, 8, 3>(s, a); break;
            default: return nullptr;
        }
    } else {
        switch (a.group_size) {
            case 64: ok = launch_f32<1, false, 4, 2>(s, a); break;
            case 128: ok = launch_f32<2, false, 4, 2>(s, a); break;
            case 256: ok = launch_f32<4, false, 4, 2>(s, a); break;
            default: return nullptr;
        }
    }
    return !ok ? nullptr : deep ? "t128x256k64s3" : "t128x128k64";
}

}  // namespace vxhip
