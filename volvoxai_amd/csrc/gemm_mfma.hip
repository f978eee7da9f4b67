// int8 MFMA GEMM for prefill-shaped M: D[n][m] = sum_k W[n][k] * X[m][k] with
// exact int32 accumulation on v_mfma_i32_32x32x32_i8, LDS-staged double
// buffered operand tiles, and the requantizing or dequantizing epilogue fused
// in.  Replaces, on gfx950, what the reference does on the CPU in
// vx_qgemm_w8a8_avx2 (native/src/kernels/packed_quant_gemm.c:2411-2600) and
// vx_packed_linear_i8_rows4 (native/src/kernels/packed_linear_ops.inc:660-853).
//
// Operand roles: the weights are the MFMA "A" operand (32 output channels x 32
// k) and the activations the "B" operand (32 k x 32 rows), so a lane ends up
// holding one activation row m and runs of four consecutive channels n -- four
// output bytes that are contiguous in y[m][n].
//
// Data movement: both operands go global -> LDS with global_load_lds_dwordx4
// (no VGPR staging); one such instruction fills 1 KiB of LDS, lane l writing
// bytes 16*l.. of it.
//  * Weights are prepacked in operand order (common.h), so a stage's weight
//    tile is a linear copy and a fragment read is ds_read_b128 at 16*lane.
//  * Activations are row-major.  One instruction fetches 8 rows x 128 bytes --
//    whole cache lines; fetching 32 rows x 32 bytes instead runs the texture
//    path three times slower -- so the LDS image is row-major with 128-byte
//    rows.  Lane l of a load picks the 16-byte chunk (l%8) ^ (row%8) of its row,
//    i.e. chunk c of row r lives at slot c ^ (r%8); a fragment read (32 rows, one
//    chunk column) then touches 8 different slots in every 8 consecutive rows
//    and stays free of bank conflicts.
#include "common.h"
#include "device_math.h"
#include "epilogue.h"
#include "gemm_tile.h"

#include <stdio.h>
#include <string.h>

namespace vxhip {

namespace {

extern __shared__ __attribute__((aligned(1024))) char lds_raw[];

constexpr int KS = 4;  // k-steps of 32 per stage: 128 bytes of k, one cache line per activation row

// WN x WM wavefronts, each owning TN x TM MFMA tiles of 32x32.  MODE is the
// Epilogue; GK = k-steps per scale group (DequantF32).  FAST selects the
// straight-line requantizing epilogue (needs n % 16 == 0, a byte output and no
// accumulator dump); otherwise the guarded per-quad epilogue runs.  W4: four-bit weights
// (DequantF32 only); a 1 KiB weight block then holds two k-steps, travels through LDS packed
// and is split into the two MFMA operands in registers.  NS: LDS stages (a power of two).  Two
// are all that fits beside a 256x256 tile; a launch of few small tiles is bound by the latency
// of one k-block's loads per iteration instead, and with four stages three k-blocks are in
// flight while one is consumed.
template <int WN, int WM, int TN, int TM, int MODE, int GK, bool FAST, bool W4, int NS>
__global__ __launch_bounds__(WN* WM * 64) void gemm_mfma_kernel(const GemmParams p) {
    static_assert(NS >= 2 && (NS & (NS - 1)) == 0, "stage count must be a power of two");
    // (the dequantizing epilogue loads group scales inside the loop; the compiler's wait for them
    // would, with loads completing in order, pull in every k-block requested before them)
    static_assert(NS == 2 || MODE != (int)Epilogue::DequantF32, "deep staging is for the requantizing modes");
    constexpr int NWAVES = WN * WM;
    constexpr int BN = WN * TN * 32, BM = WM * TM * 32;
    constexpr int SPB = W4 ? 2 : 1;   // k-steps per weight block
    constexpr int KB = KS / SPB;      // weight blocks per panel and stage
    constexpr int WBLK = (BN / 32) * KB, XBLK = BM / 8;  // 1 KiB blocks per stage
    static_assert(!W4 || MODE == (int)Epilogue::DequantF32, "four-bit weights dequantize only");
    static_assert(WBLK % NWAVES == 0 && XBLK % NWAVES == 0, "blocks must divide over waves");
    constexpr int WLOADS = WBLK / NWAVES, XLOADS = XBLK / NWAVES;
    constexpr bool F32OUT = MODE == (int)Epilogue::DequantF32;
    // PIPE (dequantizing epilogue, one scale group per k-block, wave tiles of at most two MFMA
    // tiles): two sets of tile accumulators by k-block parity.  While the MFMAs of k-block kb fill
    // one set, the fold of group kb-1 (four VALU operations per output) drains the other in the
    // MFMAs' shadow, four outputs after each MFMA, instead of following them.  The group's BN
    // weight scales travel with the operands, as the tail of the stage of the k-block that folds
    // them: a vector load in the loop would be waited for by the compiler, together with every
    // operand load requested before it.  (Larger wave tiles do not fit two accumulator sets in
    // the 256 VGPRs of a two-waves-per-SIMD kernel, and with AGPRs in play the compiler copies
    // accumulators back and forth wholesale, which measured slower than not overlapping.)
    constexpr bool PIPE = F32OUT && GK == KS && TN * TM <= 2;
    constexpr int SCALE_OFF = (WBLK + XBLK) * 1024;
    constexpr int STAGE_BYTES = SCALE_OFF + (PIPE ? BN * 4 : 0);
    const LinearArgs& a = p.a;

    const int lane = threadIdx.x & 63;
    // wave-uniform, and known to the compiler as such: everything derived from it is scalar
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int wave_n = wave % WN, wave_m = wave / WN;

    uint32_t m0, n0;
    {
        const TileOrigin t = tile_of_workgroup<BN, BM>(p);
        if (!t.valid) return;
        m0 = t.m0;
        n0 = t.n0;
    }

    // ---- per-lane load sources ---------------------------------------------
    // Weights: block b = wave + t*NWAVES of the stage is (panel b/KB, block b%KB); its address is
    // a uniform base plus the lane's 16*lane.  Activations: a per-lane row offset plus a chunk
    // offset that is the same for all of a lane's loads of one k-block.
    const uint32_t w_lane = lane * 16u;
    const uint32_t panel_bytes = a.ksteps * 1024u;
    const int8_t* const w_tile = a.w + (size_t)(n0 / 32u) * panel_bytes;
    const uint32_t last_chunk = (a.k - 1u) / 16u;  // rows are readable up to here
    const uint32_t my_chunk = (lane & 7) ^ ((lane >> 3) & 7);  // slot l%8 of row l/8 holds this chunk
    uint32_t xrow[XLOADS];
#pragma unroll
    for (int i = 0; i < XLOADS; i++) {
        const int b = wave + i * NWAVES;  // rows 8b .. 8b+7 of the tile
        uint32_t row = m0 + b * 8 + (lane >> 3);
        row = min(row, a.rows - 1u);  // rows past the end compute values nobody stores
        xrow[i] = row * a.ldx;
    }
    const uint32_t ksteps_real = (a.k + 31u) / 32u;
    const uint32_t nkb = (ksteps_real + KS - 1) / KS;

    // Load t of the NLOADS that make up this wave's share of a stage (weights first).
    // Blocks past the end are clamped to the last one: such a load refills a stage nobody reads.
    constexpr int NLOADS = WLOADS + XLOADS;
    auto issue_one = [&](auto t_tag, uint32_t kb, int stage) {
        constexpr int t = decltype(t_tag)::value;
        if constexpr (PIPE && t == 0) {
            // stage of k-block kb: the scales of group kb-1, which that k-block folds (kb = 0
            // folds zeros; any finite scales do).  64 channels per wavefront, 4 bytes per lane.
            if (wave < BN / 64) {
                const uint32_t g = min(max(kb, 1u) - 1u, a.groups - 1u);
                load_to_lds4(a.scales_t + (size_t)g * a.n_pad + n0 + wave * 64 + lane,
                             lds_raw + stage * STAGE_BYTES + SCALE_OFF + wave * 256);
            }
        }
        kb = min(kb, nkb - 1u);
        char* base = lds_raw + stage * STAGE_BYTES;
        if constexpr (t < WLOADS) {
            const uint32_t b = wave + t * NWAVES;
            const int8_t* src = w_tile + (size_t)(b / KB) * panel_bytes + (size_t)(kb * KB + b % KB) * 1024u;
            load_to_lds16(src + w_lane, base + b * 1024);
        } else {
            // k-chunks past the row end pair with zero weights: clamp the address
            const uint32_t chunk16 = min(kb * 8u + my_chunk, last_chunk) * 16u;
            const uint32_t b = wave + (t - WLOADS) * NWAVES;
            load_to_lds16(a.x + (xrow[t - WLOADS] + chunk16), base + (WBLK + b) * 1024);
        }
    };
    // ---- accumulators --------------------------------------------------------
    v16i acc[TN][TM];
    v16i acc_odd[PIPE ? TN : 1][PIPE ? TM : 1];  // PIPE: accumulators of the odd k-blocks
    v16i fsum[F32OUT ? TN : 1][F32OUT ? TM : 1];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                acc[i][j][r] = 0;
                if constexpr (PIPE) acc_odd[i][j][r] = 0;
            }
    if constexpr (F32OUT) {
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int j = 0; j < TM; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) fsum[i][j][r] = 0;  // bit pattern of +0.0f
    }

    // activation scale of the lane's row in each of its TM tiles
    float row_scale[TM];
    if constexpr (MODE != (int)Epilogue::RequantTensor) {
#pragma unroll
        for (int j = 0; j < TM; j++) {
            const uint32_t m = min(m0 + (wave_m * TM + j) * 32 + (lane & 31), a.rows - 1u);
            row_scale[j] = a.row_scale[m];
        }
    }
    // first channel of the lane's quad q in tile i: n0 + (wave_n*TN+i)*32 + q*8 + (lane>>5)*4
    const uint32_t nbase = n0 + wave_n * TN * 32 + (lane >> 5) * 4;

    // Per-group scale-accumulate of PackedLinear/DYNAMIC_I8: complete the exact
    // int32 dot of one storage group, then sum += f32(dot) * (s_a * s_w[n][g]) in
    // ascending group order (packed_linear_ops.inc:1498-1504).
    // The group's weight scales are requested one group ahead (right after the previous fold),
    // so the fold never waits on their L2 latency (that wait was 15 % of the large-K GEMM).
    v4f sw_next[F32OUT ? TN : 1][4];
    auto load_scales = [&](uint32_t g) {
        if constexpr (F32OUT) {
            const float* srow = a.scales_t + (size_t)min(g, a.groups - 1u) * a.n_pad;
#pragma unroll
            for (int i = 0; i < TN; i++)
#pragma unroll
                for (int q = 0; q < 4; q++)
                    sw_next[i][q] = *reinterpret_cast<const v4f*>(srow + nbase + i * 32 + q * 8);
        }
    };
    if constexpr (!PIPE) load_scales(0);
    auto fold_group = [&](uint32_t g) {
        if constexpr (F32OUT) {
#pragma unroll
            for (int i = 0; i < TN; i++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const v4f sw = sw_next[i][q];
#pragma unroll
                    for (int j = 0; j < TM; j++) {
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const int r = q * 4 + e;
                            const float gs = __fmul_rn(row_scale[j], sw[e]);
                            // four-bit operands carry a factor 16; the dot is exact, so is the shift
                            const float term = __fmul_rn((float)(acc[i][j][r] >> (W4 ? 4 : 0)), gs);
                            fsum[i][j][r] = __float_as_int(
                                __fadd_rn(__int_as_float(fsum[i][j][r]), term));
                            // groups that end inside a k-block restart from the MFMA's zero C operand
                            if constexpr (GK > KS) acc[i][j][r] = 0;
                        }
                    }
                }
            }
            load_scales(g + 1u);
        }
    };

    // PIPE: the fold of the accumulator set of parity P, four outputs (one quad of one tile) per
    // slot.  Slots are ordered (tile column i, quad q, tile row j), so a unit u = (i, q) of four
    // channel scales serves TM consecutive slots; it is read from the stage AHEAD units ahead, the
    // first units of the next k-block from that block's stage (which has landed in the step after
    // the barrier; AHEAD is chosen so that no earlier step reaches for it).  Two ahead lets the
    // wait before a fold name the one read it needs instead of draining the LDS queue.
    constexpr int UNITS = TN * 4;
    constexpr int AHEAD = UNITS / KS >= 2 ? 2 : 1;
    v4f sw_ring[PIPE ? 4 : 1];
    const uint32_t sw_lane = (uint32_t)(wave_n * TN * 32 + (lane >> 5) * 4) * 4u + SCALE_OFF;
    auto read_scale_unit = [&](auto unit_tag, const char* stage) {
        constexpr int u = decltype(unit_tag)::value;
        sw_ring[u & 3] = *reinterpret_cast<const v4f*>(stage + sw_lane + ((u / 4) * 32 + (u % 4) * 8) * 4);
    };
    auto fold_slot = [&](auto parity_tag, auto idx_tag, const char* stage, const char* next_stage, auto more_tag) {
        constexpr int P = decltype(parity_tag)::value, IDX = decltype(idx_tag)::value;
        constexpr int u = IDX / TM, j = IDX % TM, i = u / 4, q = u % 4;
        if constexpr (j == 0) {
            if constexpr (u + AHEAD < UNITS) read_scale_unit(IC<u + AHEAD>{}, stage);
            else if constexpr (decltype(more_tag)::value) read_scale_unit(IC<u + AHEAD - UNITS>{}, next_stage);
        }
        const v4f sw = sw_ring[u & 3];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int r = q * 4 + e;
            const int32_t dot = (P == 0 ? acc[i][j][r] : acc_odd[i][j][r]) >> (W4 ? 4 : 0);
            const float gs = __fmul_rn(row_scale[j], sw[e]);
            float sum = __fadd_rn(__int_as_float(fsum[i][j][r]), __fmul_rn((float)dot, gs));
            // the sum is needed only after the loop, and left to itself the optimizer collects all
            // folds of a k-block behind its MFMAs; this pins each where it is written
            asm volatile("" : "+v"(sum));
            fsum[i][j][r] = __float_as_int(sum);
        }
    };

    // ---- fragment addressing ---------------------------------------------------
    // weights: block (panel, step) at 1 KiB granularity, lane slot 16*lane
    // activations: row (wave_m*TM+j)*32 + lane%32 of 128 bytes, chunk 2s + lane/32 at slot chunk ^ (row%8)
    const uint32_t w_frag = (uint32_t)(wave_n * TN * KB) * 1024u + lane * 16u;
    const uint32_t x_row = WBLK * 1024u + ((uint32_t)(wave_m * TM * 32) + (lane & 31)) * 128u;
    uint32_t x_slot[KS];
#pragma unroll
    for (int s = 0; s < KS; s++) x_slot[s] = (((2u * s + (lane >> 5)) ^ (lane & 7u)) << 4);

    // fragment r of a k-step, in the order the MFMAs want them: w0, x0 .. x(TM-1), w1 .. w(TN-1)
    constexpr int READS = TN + TM, MF = TN * TM;
    // Four-bit weights: the packed block of steps (s, s+1) is read at even s into wraw and split
    // by the step that first uses it; odd s has no weight read.
    v4i wraw[W4 ? TN : 1];
    auto read_one = [&](auto r_tag, const char* stage, auto s_tag, v4i (&wf)[TN], v4i (&xf)[TM]) {
        constexpr int r = decltype(r_tag)::value;
        constexpr int s = decltype(s_tag)::value;
        if constexpr (r == 0 || r > TM) {
            constexpr int i = r == 0 ? 0 : r - TM;
            if constexpr (!W4) {
                wf[i] = *reinterpret_cast<const v4i*>(stage + w_frag + (i * KS + s) * 1024);
            } else if constexpr ((s & 1) == 0) {
                wraw[i] = *reinterpret_cast<const v4i*>(stage + w_frag + (i * KB + s / 2) * 1024);
            }
        } else {
            constexpr int j = r - 1;
            xf[j] = *reinterpret_cast<const v4i*>(stage + x_row + j * 32 * 128 + x_slot[s]);
        }
    };

    // ---- main loop -------------------------------------------------------------
    // Two LDS stages.  One barrier per k-block, placed before the block's last k-step: by
    // then a wave has issued all its reads of the current stage (fragments are requested one
    // step ahead of the MFMAs that use them), so after the barrier the stage can be refilled
    // for block kb+2 and the first fragments of block kb+1 can be requested while the last
    // MFMAs of block kb still run.  MFMA issue therefore never waits on LDS latency.
    //
    // The instruction order inside a k-step is written out and fenced (sched_barrier) rather
    // than left to the scheduler: MFMA m is preceded by the fragment reads and operand loads
    // whose turn it is, so LDS reads, global->LDS loads and MFMAs issue evenly mixed.
    static_for<NS - 1>([&](auto b_tag) {
        static_for<NLOADS>([&](auto t) { issue_one(t, decltype(b_tag)::value, decltype(b_tag)::value); });
    });
    // per-channel epilogue constants of this tile (structure of arrays, so a lane's four
    // consecutive channels are one ds_read_b128 each), computed while the first stage is in flight
    float* lds_f0 = reinterpret_cast<float*>(lds_raw + NS * STAGE_BYTES);
    int32_t* lds_cb = reinterpret_cast<int32_t*>(lds_f0 + BN);
    float* lds_bo = reinterpret_cast<float*>(lds_cb + BN);
    int32_t* lds_zw = reinterpret_cast<int32_t*>(lds_bo + BN);
    if constexpr (!F32OUT) {
        for (int t = threadIdx.x; t < BN; t += NWAVES * 64) {
            const ChannelConsts c = channel_consts<MODE>(a, n0 + t);
            lds_f0[t] = c.f0;
            lds_cb[t] = c.cb;
            lds_bo[t] = c.bo;
            lds_zw[t] = c.zw;
        }
    }

    v4i wf[2][TN], xf[2][TM];
    // One k-step: the MFMAs on fragment buffer S%2; mixed in, the reads of step RS of `rstage`
    // into the other buffer (if READ) and the first NL operand loads of block load_kb into
    // load_stage.  (All of a stage's loads go out in the step after the barrier: issuing part
    // of them a step or two later measured slower, they then land too late.)
    auto step = [&](auto s_tag, auto read_tag, auto rs_tag, const char* rstage, auto nl_tag, uint32_t load_kb,
                    int load_stage, uint32_t kb, auto parity_tag, const char* cstage) {
        constexpr int S = decltype(s_tag)::value;
        constexpr int P = decltype(parity_tag)::value;  // k-block parity (PIPE)
        constexpr bool READ = decltype(read_tag)::value;
        constexpr int NL = decltype(nl_tag)::value;
        constexpr int CB = S & 1, NB = CB ^ 1;
        static_for<MF>([&](auto m_tag) {
            constexpr int m = decltype(m_tag)::value;
            constexpr int i = m / TM, j = m % TM;
            if constexpr (W4 && (S & 1) == 0 && j == 0) {
                // low nibbles: this step's operand; high nibbles: the next step's (fragment
                // buffer 1, whose last readers were issued in the previous step)
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    wf[0][i][d] = (wraw[i][d] << 4) & (int)0xf0f0f0f0u;
                    wf[1][i][d] = wraw[i][d] & (int)0xf0f0f0f0u;
                }
            }
            // first k-step of a scale group: accumulate onto zero instead of clearing registers
            constexpr bool FRESH = F32OUT && GK <= KS && (S % GK) == 0;
            const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            if constexpr (PIPE && P == 1)
                acc_odd[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[CB][i], xf[CB][j],
                                                                      FRESH ? zero : acc_odd[i][j], 0, 0, 0);
            else
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[CB][i], xf[CB][j], FRESH ? zero : acc[i][j], 0, 0, 0);
            // PIPE: one slot (four outputs) of the other set's fold rides behind every MFMA
            if constexpr (PIPE) fold_slot(IC<P ^ 1>{}, IC<S * MF + m>{}, cstage, rstage, read_tag);
            // after MFMA m: the reads and loads whose slot it is.  Reads keep clear of the
            // step's last MFMAs, which cover the latency of the final read.
            if constexpr (READ) {
                static_for<READS>([&](auto r_tag) {
                    constexpr int r = decltype(r_tag)::value;
                    if constexpr ((r * (MF - 1)) / READS == m) read_one(r_tag, rstage, rs_tag, wf[NB], xf[NB]);
                });
            }
            if constexpr (NL > 0) {
                static_for<NL>([&](auto l_tag) {
                    constexpr int l = decltype(l_tag)::value;
                    if constexpr ((l * MF) / NL == m) issue_one(l_tag, load_kb, load_stage);
                });
            }
            if constexpr (!F32OUT || PIPE) __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (F32OUT && !PIPE) {
            if constexpr (GK <= KS) {
                if ((S + 1) % GK == 0) fold_group((kb * KS + S) / GK);
            }
        }
    };

    // k-block 0 has landed; the NS-2 younger ones may still be on their way
    wait_vmcnt<(NS - 2) * NLOADS>();
    wg_barrier();
    // (unconditional: a block past the end is clamped to the last one, and the waits below
    // count on every block having been requested)
    static_for<NLOADS>([&](auto t) { issue_one(t, NS - 1, NS - 1); });
    static_for<READS>([&](auto r) { read_one(r, lds_raw, IC<0>{}, wf[0], xf[0]); });
    if constexpr (PIPE) static_for<AHEAD>([&](auto u_tag) { read_scale_unit(u_tag, lds_raw); });
    auto k_block = [&](uint32_t kb, auto last_tag, auto parity_tag) {
        constexpr bool LAST = decltype(last_tag)::value;
        const int cur = kb & (NS - 1);
        const char* stage = lds_raw + cur * STAGE_BYTES;
        static_for<KS - 1>([&](auto s_tag) {
            constexpr int S = decltype(s_tag)::value;
            step(s_tag, std::true_type{}, IC<S + 1>{}, stage, IC<0>{}, 0u, 0, kb, parity_tag, stage);
        });
        if constexpr (!LAST) {
            wait_lgkm0();     // my reads of this stage have landed in registers
            // my loads of the next k-block have landed (the NS-2 blocks after it need not have)
            wait_vmcnt<(NS - 2) * NLOADS>();
            wg_barrier();
            step(IC<KS - 1>{}, std::true_type{}, IC<0>{}, lds_raw + ((cur + 1) & (NS - 1)) * STAGE_BYTES,
                 IC<NLOADS>{}, kb + NS, cur, kb, parity_tag, stage);
        } else {
            step(IC<KS - 1>{}, std::false_type{}, IC<0>{}, stage, IC<0>{}, 0u, 0, kb, parity_tag, stage);
        }
        if constexpr (F32OUT && (GK > KS)) {
            if (((kb + 1) * KS) % GK == 0 || kb + 1 == nkb) fold_group((kb * KS) / GK);
        }
    };
    if constexpr (PIPE) {
        // pairs of k-blocks, so that the parity of a block is a compile-time fact; then the one or
        // two blocks that are left, and the fold of the last group, which has no MFMAs to hide in
        uint32_t kb = 0;
        for (; kb + 2 < nkb; kb += 2) {
            k_block(kb, std::false_type{}, IC<0>{});
            k_block(kb + 1, std::false_type{}, IC<1>{});
        }
        if (kb + 2 == nkb) {
            k_block(kb, std::false_type{}, IC<0>{});
            k_block(kb + 1, std::true_type{}, IC<1>{});
        } else {
            k_block(kb, std::true_type{}, IC<0>{});
        }
        // the last group's scales are the tail of the stage requested as k-block nkb
        wait_vmcnt<0>();
        wg_barrier();
        const char* last_stage = lds_raw + (nkb & (NS - 1)) * STAGE_BYTES;
        static_for<AHEAD>([&](auto u_tag) { read_scale_unit(u_tag, last_stage); });
        if (nkb & 1u)
            static_for<TN * TM * 4>([&](auto idx) { fold_slot(IC<0>{}, idx, last_stage, last_stage, std::false_type{}); });
        else
            static_for<TN * TM * 4>([&](auto idx) { fold_slot(IC<1>{}, idx, last_stage, last_stage, std::false_type{}); });
    } else {
        for (uint32_t kb = 0; kb + 1 < nkb; kb++) k_block(kb, std::false_type{}, IC<0>{});
        k_block(nkb - 1u, std::true_type{}, IC<0>{});
    }
    wait_vmcnt<0>();  // nothing of this workgroup may still be writing LDS when the epilogue reuses it

    // ---- epilogue ----------------------------------------------------------------
    if constexpr (FAST && !F32OUT) {
        // Straight-line requantization.  A lane owns row m (per j) and, per 32-wide tile i,
        // the quads q*8 + (lane>>5)*4 + 0..3.  After packing each quad to one dword, lanes l
        // and l+32 exchange two dwords (v_permlane32_swap), which leaves each lane with 16
        // consecutive output bytes: one dwordx4 store per tile and row.
        const float zp_f = (float)a.out_zp, lo_f = (float)a.out_lo, hi_f = (float)a.out_hi;
        const float so = a.output_scale, sr = a.output_scale_recip;
        uint32_t mrow[TM];
        int32_t rsum[TM];
        // mismatch counts of the one- and two-correction division by the output scale
        uint32_t miss1 = 1, miss2 = 1;
        if (MODE == (int)Epilogue::RequantRow && a.div_proof) {
            miss1 = a.div_proof[0];
            miss2 = a.div_proof[1];
        }
        bool lean = a.zw == nullptr;
        if constexpr (MODE == (int)Epilogue::RequantRow) lean = lean && fast_div_in_range(so) && miss2 == 0;
        // BARE on top of LEAN: nothing to add to the accumulator or to the product (an output zero
        // point of 0 adds +0.0, which changes no value that is rounded afterwards), and for
        // per-row scales the one-correction division is proved as well
        const bool no_int_terms = a.int_bias_zero && (MODE == (int)Epilogue::RequantRow || a.input_zp == 0);
        const bool bare_ok = no_int_terms && a.out_zp == 0 && (MODE != (int)Epilogue::RequantRow || miss1 == 0);
        bool bad = false;
#pragma unroll
        for (int j = 0; j < TM; j++) {
            mrow[j] = m0 + (wave_m * TM + j) * 32 + (lane & 31);
            rsum[j] = (a.zw && mrow[j] < a.rows) ? a.rowsum[mrow[j]] : 0;
            if constexpr (MODE == (int)Epilogue::RequantRow) {
                // the multiplier is monotone in the weight scale: its extremes decide validity
                // and whether every product stays in the range of the short division
                const float plo = __fmul_rn(row_scale[j], a.wscale_min), phi = __fmul_rn(row_scale[j], a.wscale_max);
                if (mrow[j] < a.rows) {
                    bad |= !scale_valid(__fdiv_rn(plo, so)) || !scale_valid(__fdiv_rn(phi, so));
                    lean &= fast_div_in_range(plo) && fast_div_in_range(phi);
                }
            }
        }
        if (bad) atomicOr(a.fault, (uint32_t)kFaultBadMultiplier);
        const bool wave_lean = __builtin_amdgcn_ballot_w64(!lean) == 0ull;
        // LEVEL 0: general.  1 (LEAN): no weight zero points, every quotient in the range of the
        // proved short division.  2 (BARE): see above.
        auto run = [&](auto level_tag) {
            constexpr int LEVEL = decltype(level_tag)::value;
            constexpr bool LEAN = LEVEL >= 1, BARE = LEVEL == 2;
#pragma unroll
            for (int i = 0; i < TN; i++) {
                uint32_t packed[TM][4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int c0 = (wave_n * TN + i) * 32 + q * 8 + (lane >> 5) * 4;
                    const v4f f0 = *reinterpret_cast<const v4f*>(lds_f0 + c0);
                    const v4i cb = *reinterpret_cast<const v4i*>(lds_cb + c0);
                    v4f bo = {0.f, 0.f, 0.f, 0.f};
                    v4i zw = {0, 0, 0, 0};
                    if (MODE == (int)Epilogue::RequantRow && (BARE || a.bias_row)) bo = *reinterpret_cast<const v4f*>(lds_bo + c0);
                    if (!LEAN && a.zw) zw = *reinterpret_cast<const v4i*>(lds_zw + c0);
#pragma unroll
                    for (int j = 0; j < TM; j++) {
                        uint32_t u[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            uint32_t total = (uint32_t)acc[i][j][q * 4 + e];
                            if (!BARE) total += (uint32_t)cb[e];
                            if (!LEAN) total -= (uint32_t)zw[e] * (uint32_t)rsum[j];
                            float mu = f0[e];
                            if constexpr (MODE == (int)Epilogue::RequantRow) {
                                const float prod = __fmul_rn(row_scale[j], f0[e]);
                                mu = BARE   ? div_by_uniform_once(prod, so, sr)
                                     : LEAN ? div_by_uniform(prod, so, sr)
                                            : __fdiv_rn(prod, so);
                            }
                            float t = __fmul_rn((float)(int32_t)total, mu);
                            if (!BARE) t = __fadd_rn(t, zp_f);
                            // BARE adds the bias term unconditionally: it is +0.0 when there is none
                            if (MODE == (int)Epilogue::RequantRow && (BARE || a.bias_row)) t = __fadd_rn(t, bo[e]);
                            // A valid multiplier cannot produce NaN here and an invalid one was flagged
                            // above.  Clamp, then round to nearest even by adding 1.5 * 2^23: the sum's
                            // low mantissa bits are the two's-complement integer.
                            t = __builtin_amdgcn_fmed3f(t, lo_f, hi_f);
                            u[e] = __float_as_uint(__fadd_rn(t, 12582912.0f));
                        }
                        // byte 0 of each of the four words
                        const uint32_t p01 = __builtin_amdgcn_perm(u[1], u[0], 0x0c0c0400u);
                        const uint32_t p23 = __builtin_amdgcn_perm(u[3], u[2], 0x0c0c0400u);
                        packed[j][q] = __builtin_amdgcn_perm(p23, p01, 0x05040100u);
                    }
                }
                const uint32_t n16 = n0 + (wave_n * TN + i) * 32 + (lane >> 5) * 16;
#pragma unroll
                for (int j = 0; j < TM; j++) {
                    // lanes 0-31 keep quads 0,1 and receive the partner's; lanes 32-63 end with quads 2,3
                    const auto s02 = __builtin_amdgcn_permlane32_swap(packed[j][0], packed[j][2], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(packed[j][1], packed[j][3], false, false);
                    if (mrow[j] < a.rows && n16 < a.n) {
                        const uint4 v = make_uint4(s02[0], s02[1], s13[0], s13[1]);
                        *reinterpret_cast<uint4*>((uint8_t*)a.y + (size_t)mrow[j] * a.n + n16) = v;
                    }
                }
            }
        };
        if (wave_lean && bare_ok) run(IC<2>{});
        else if (wave_lean) run(IC<1>{});
        else run(IC<0>{});
    } else {
#pragma unroll
        for (int j = 0; j < TM; j++) {
            const uint32_t m = m0 + (wave_m * TM + j) * 32 + (lane & 31);
            int32_t rsum = 0;
            if constexpr (!F32OUT) {
                if (a.zw && m < a.rows) rsum = a.rowsum[m];
            }
            float rs = 0.0f;
            if constexpr (MODE != (int)Epilogue::RequantTensor) rs = row_scale[j];
#pragma unroll
            for (int i = 0; i < TN; i++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    int32_t dot[4];
                    float fs[4];
                    ChannelConsts cc[4];
                    const uint32_t n = nbase + i * 32 + q * 8;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        dot[e] = acc[i][j][q * 4 + e];
                        fs[e] = 0.0f;
                        if constexpr (F32OUT) {
                            fs[e] = __int_as_float(fsum[i][j][q * 4 + e]);
                        } else {
                            const int c = n - n0 + e;
                            cc[e] = ChannelConsts{lds_f0[c], lds_cb[c], lds_bo[c], lds_zw[c]};
                        }
                    }
                    store_quad<MODE>(a, m, n, dot, fs, rs, rsum, cc);
                }
            }
        }
    }
}

template <int WN, int WM, int TN, int TM, int MODE, int GK, bool FAST, bool W4, int NS>
bool launch_one(hipStream_t s, const LinearArgs& a) {
    constexpr int BN = WN * TN * 32, BM = WM * TM * 32;
    // the stages and, behind them, the per-channel epilogue constants
    constexpr bool PIPE = MODE == (int)Epilogue::DequantF32 && GK == KS && TN * TM <= 2;  // as in the kernel
    constexpr int LDS = NS * (((BN / 32) * KS / (W4 ? 2 : 1) + BM / 8) * 1024 + (PIPE ? BN * 4 : 0)) + BN * 16;
    static_assert(LDS <= 160 * 1024, "stages do not fit the LDS");
    static std::atomic<uint64_t> configured{0};
    auto kern = gemm_mfma_kernel<WN, WM, TN, TM, MODE, GK, FAST, W4, NS>;
    if (!raise_lds_limit((const void*)kern, LDS, configured)) return false;
    GemmParams p;
    p.a = a;
    p.tiles_n = (a.n + BN - 1) / BN;
    p.tiles_m = (a.rows + BM - 1) / BM;
    const uint32_t total = p.tiles_n * p.tiles_m;
    const uint32_t grid = ((total + 7u) / 8u) * 8u;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WN * WM * 64), LDS, s, p);
    return hipGetLastError() == hipSuccess;
}

template <int WN, int WM, int TN, int TM, int MODE, int GK, bool W4 = false, int NS = 2>
bool launch_cfg(hipStream_t s, const LinearArgs& a) {
    if constexpr (MODE != (int)Epilogue::DequantF32) {
        if ((a.n % 16u) == 0u && a.y && !a.acc_out && !a.dq_out && ((uintptr_t)a.y % 16u) == 0u)
            return launch_one<WN, WM, TN, TM, MODE, GK, true, false, NS>(s, a);
    }
    return launch_one<WN, WM, TN, TM, MODE, GK, false, W4, NS>(s, a);
}

template <int MODE, int GK, bool W4 = false>
const char* dispatch_tile(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    auto forced = [&](const char* tag) { return force && strstr(force, tag) != nullptr; };
    if constexpr (MODE == (int)Epilogue::DequantF32) {
        // int32 tile accumulators plus f32 running sums: the wave tile is at most 64x64, and with
        // a scale group per k-step the eight-wave tile runs out of registers.  A wave folds a
        // group (four VALU operations per output) strictly after that group's MFMAs, so its time
        // per k-block grows with its tile: few rows or few channels take narrower tiles, which
        // also puts more workgroups on the device.
        const auto tiles = [&](uint32_t bn, uint32_t bm) {
            return (uint64_t)((a.n + bn - 1) / bn) * ((a.rows + bm - 1) / bm);
        };
        const uint64_t enough = (uint64_t)cu_count * 3 / 4;
        int pick = a.rows <= 64u ? 3 : tiles(128, 256) >= enough && GK > 1 ? 0 : tiles(128, 128) >= enough ? 1
                   : tiles(64, 128) >= enough ? 2 : 3;
        // Enough 128 x 128 tiles for every compute unit to hold its two workgroups, or most of them: the
        // 16x16x64 kernel of gemm_k64.hip (group sizes of 64 and more), unless a tile of this file is named.
        const bool named = forced("t256x") || forced("t128x") || forced("t64x");
        if (a.group_size >= 64u && (forced("k64") || (!named && tiles(128, 128) >= enough))) {
            // long rows with one scale per channel: sixteen waves on a 128 x 256 tile, three stages
            // (K = 14336, N = 4096, 2048 rows: 211 against 232 us; short rows favour the small tile)
            const bool deep = forced("t128x256k64") || (!forced("k64") && a.uniform_group_scales && a.weight_bits == 8u &&
                                                        a.group_size <= 128u && a.k >= 4096u && tiles(128, 256) >= enough);
            const char* t = launch_gemm_k64_f32(s, a, deep);
            if (t) return t;
        }
        if (forced("t256x256")) pick = GK > 1 ? 0 : 1;
        if (forced("t128x128")) pick = 1;
        if (forced("t64x128")) pick = 2;
        if (forced("t64x64")) pick = 3;
        if constexpr (GK == KS) {
            // one group per k-block: eight waves of 64x32 fold in the shadow of their MFMAs.  Measured
            // against the plain 128x128 tile: 30 against 42 us at 4096x3072 -> 1024, 36 against 50 us
            // at 256x4096 -> 14336; the 128x256 tile stays ahead where there is work for it.
            if ((pick == 1 && !forced("t128x128")) || forced("t128x128p"))
                return launch_cfg<2, 4, 2, 1, MODE, GK, W4>(s, a) ? "t128x128p" : nullptr;
        }
        if (pick == 0) return launch_cfg<2, 4, 2, 2, MODE, GK, W4>(s, a) ? "t128x256" : nullptr;
        if (pick == 1) return launch_cfg<2, 2, 2, 2, MODE, GK, W4>(s, a) ? "t128x128" : nullptr;
        if (pick == 2) return launch_cfg<2, 2, 1, 2, MODE, GK, W4>(s, a) ? "t64x128" : nullptr;
        return launch_cfg<2, 2, 1, 1, MODE, GK, W4>(s, a) ? "t64x64" : nullptr;
    } else {
        // Largest tile (channels x rows) that still gives every compute unit work; names are BNxBM.
        const auto tiles = [&](uint32_t bn, uint32_t bm) {
            return (uint64_t)((a.n + bn - 1) / bn) * ((a.rows + bm - 1) / bm);
        };
        const uint64_t enough = (uint64_t)cu_count * 3 / 4;
        int pick = tiles(256, 256) >= enough ? 0 : tiles(256, 128) >= enough ? 1 : tiles(128, 128) >= enough ? 2
                   : tiles(128, 64) >= enough ? 3 : 4;
        if (forced("t256x256")) pick = 0;
        if (forced("t256x128")) pick = 1;
        if (forced("t128x128")) pick = 2;
        if (forced("t128x64")) pick = 3;
        if (forced("t64x64")) pick = 4;
        // The two large tiles run on the 16x16x64 MFMA (gemm_k64.hip) when the straight-line epilogue
        // applies; a forced tile name without "k64" keeps the 32x32x32 kernel of this file.
        // (with a.dq_out the dequantized values go out as well, or alone)
        const bool fast_ok = (a.n % 16u) == 0u && (a.y || a.dq_out) && !a.acc_out && ((uintptr_t)a.y % 16u) == 0u &&
                             ((uintptr_t)a.dq_out % 16u) == 0u;
        const bool named = forced("t256x") || forced("t128x") || forced("t64x");
        if (pick <= 1 && fast_ok && (forced("k64") || !named)) return launch_gemm_k64(s, a, pick);
        if (a.x_flip_mask) return nullptr;  // only those kernels flip unsigned bytes themselves: the caller stages them
        if (pick == 0 && forced("wv4")) return launch_cfg<2, 2, 4, 4, MODE, GK>(s, a) ? "t256x256wv4" : nullptr;
        if (pick == 0) return launch_cfg<2, 4, 4, 2, MODE, GK>(s, a) ? "t256x256" : nullptr;
        if (pick == 1 && forced("wv4")) return launch_cfg<2, 2, 4, 2, MODE, GK>(s, a) ? "t256x128wv4" : nullptr;
        if (pick == 1) return launch_cfg<2, 4, 4, 1, MODE, GK>(s, a) ? "t256x128" : nullptr;
        // one round of tiles or less: the k loop waits on each k-block's loads in turn; four
        // stages keep three k-blocks in flight (the small tiles leave the LDS for them)
        const bool deep = forced("s4") || (!forced("s2") && tiles(128, pick == 2 ? 128 : 64) <= (uint64_t)cu_count * 3 / 2);
        if (pick == 4) return launch_cfg<2, 2, 1, 1, MODE, GK, false, 4>(s, a) ? "t64x64s4" : nullptr;
        if (pick == 2 && deep) return launch_cfg<2, 2, 2, 2, MODE, GK, false, 4>(s, a) ? "t128x128s4" : nullptr;
        if (pick == 2) return launch_cfg<2, 2, 2, 2, MODE, GK>(s, a) ? "t128x128" : nullptr;
        // (eight waves of 32 x 32 instead of four of 64 x 32: the loop is bound by the operand loads either way, the
        // epilogue is spread over twice the waves -- M=512, K=N=4096: 15.6 -> 14.9 us; four waves when named)
        if (deep && !forced("wv4")) return launch_cfg<4, 2, 1, 1, MODE, GK, false, 4>(s, a) ? "t128x64s4w8" : nullptr;
        if (deep) return launch_cfg<2, 2, 2, 1, MODE, GK, false, 4>(s, a) ? "t128x64s4" : nullptr;
        return launch_cfg<2, 2, 2, 1, MODE, GK>(s, a) ? "t128x64" : nullptr;
    }
}

}  // namespace

const char* launch_gemm_mfma(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    if (a.x_operand_order) return nullptr;  // the tiles are staged from row-major activations
    if (a.ldx < 16u || (a.ldx % 16u) != 0u || ((uintptr_t)a.x % 16u) != 0u) return nullptr;
    if ((uint64_t)a.rows * a.ldx > 0xffffffffull) return nullptr;  // 32-bit activation offsets
    if (a.weight_bits != 8u && !(a.weight_bits == 4u && a.mode == Epilogue::DequantF32)) return nullptr;
    const char* tile = nullptr;
    static thread_local char name[96];
    const char* family = nullptr;
    switch (a.mode) {
        case Epilogue::RequantTensor:
            tile = dispatch_tile<(int)Epilogue::RequantTensor, 1>(s, a, cu_count, force);
            family = "hip.qlinear.mfma-i8";
            break;
        case Epilogue::RequantRow:
            tile = dispatch_tile<(int)Epilogue::RequantRow, 1>(s, a, cu_count, force);
            family = "hip.qlinear.mfma-i8-rowscale";
            break;
        case Epilogue::DequantF32:
            if (a.weight_bits == 4u) {
                family = "hip.packed-linear.w4a8-mfma";
                switch (a.group_size) {
                    case 32: tile = dispatch_tile<(int)Epilogue::DequantF32, 1, true>(s, a, cu_count, force); break;
                    case 64: tile = dispatch_tile<(int)Epilogue::DequantF32, 2, true>(s, a, cu_count, force); break;
                    case 128: tile = dispatch_tile<(int)Epilogue::DequantF32, 4, true>(s, a, cu_count, force); break;
                    case 256: tile = dispatch_tile<(int)Epilogue::DequantF32, 8, true>(s, a, cu_count, force); break;
                    default: return nullptr;
                }
                break;
            }
            family = "hip.packed-linear.a8-mfma";
            switch (a.group_size) {
                case 32: tile = dispatch_tile<(int)Epilogue::DequantF32, 1>(s, a, cu_count, force); break;
                case 64: tile = dispatch_tile<(int)Epilogue::DequantF32, 2>(s, a, cu_count, force); break;
                case 128: tile = dispatch_tile<(int)Epilogue::DequantF32, 4>(s, a, cu_count, force); break;
                case 256: tile = dispatch_tile<(int)Epilogue::DequantF32, 8>(s, a, cu_count, force); break;
                default: return nullptr;
            }
            break;
    }
    if (!tile) return nullptr;
    snprintf(name, sizeof name, "%s.%s", family, tile);
    return name;
}

}  // namespace vxhip
