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

#include <stdio.h>
#include <string.h>

#include <type_traits>

// Compile-time probes used only when tuning (all off in the shipped build):
// leave out one ingredient of the main loop to see what bounds it.
#ifndef VXHIP_PROBE_NO_LOADS
#define VXHIP_PROBE_NO_LOADS 0
#endif
#ifndef VXHIP_PROBE_NO_MFMA
#define VXHIP_PROBE_NO_MFMA 0
#endif
#ifndef VXHIP_PROBE_NO_EPILOGUE
#define VXHIP_PROBE_NO_EPILOGUE 0
#endif
// The L2 prefetch of later k-blocks measured slower than leaving it out (the extra
// requests compete with the real loads), so it is compiled out unless asked for.
#ifndef VXHIP_PROBE_NO_PREFETCH
#define VXHIP_PROBE_NO_PREFETCH 1
#endif

namespace vxhip {

namespace {

extern __shared__ __attribute__((aligned(1024))) char lds_raw[];

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lgkm0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void wg_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ void load_to_lds16(const void* gptr, void* lptr) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gptr,
                                     (__attribute__((address_space(3))) void*)lptr, 16, 0, 0);
}

struct GemmParams {
    LinearArgs a;
    uint32_t tiles_n, tiles_m;
};

constexpr int KS = 4;  // k-steps of 32 per stage: 128 bytes of k, one cache line per activation row

// WN x WM wavefronts, each owning TN x TM MFMA tiles of 32x32.  MODE is the
// Epilogue; GK = k-steps per scale group (DequantF32).  FAST selects the
// straight-line requantizing epilogue (needs n % 16 == 0, a byte output and no
// accumulator dump); otherwise the guarded per-quad epilogue runs.
template <int WN, int WM, int TN, int TM, int MODE, int GK, bool FAST>
__global__ __launch_bounds__(WN* WM * 64) void gemm_mfma_kernel(const GemmParams p) {
    constexpr int NWAVES = WN * WM;
    constexpr int BN = WN * TN * 32, BM = WM * TM * 32;
    constexpr int WBLK = (BN / 32) * KS, XBLK = BM / 8;  // 1 KiB blocks per stage
    static_assert(WBLK % NWAVES == 0 && XBLK % NWAVES == 0, "blocks must divide over waves");
    constexpr int WLOADS = WBLK / NWAVES, XLOADS = XBLK / NWAVES;
    constexpr int STAGE_BYTES = (WBLK + XBLK) * 1024;
    constexpr bool F32OUT = MODE == (int)Epilogue::DequantF32;
    const LinearArgs& a = p.a;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wave_n = wave % WN, wave_m = wave / WN;

    // ---- workgroup -> tile, XCD aware ------------------------------------
    // Consecutive workgroup ids land on different XCDs (8 of them, each with
    // its own L2).  Give XCD x the x-th contiguous run of tiles, and order
    // tiles so a run is a compact block of the output: that block's operand
    // slices are then shared through one L2 instead of being fetched by all.
    const uint32_t total = p.tiles_n * p.tiles_m;
    const uint32_t per_xcd = (total + 7u) / 8u;
    const uint32_t lin = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if (lin >= total) return;
    constexpr uint32_t GROUP_M = 4;
    const uint32_t band = lin / (GROUP_M * p.tiles_n);
    const uint32_t band_first = band * GROUP_M;
    const uint32_t band_rows = min(GROUP_M, p.tiles_m - band_first);
    const uint32_t in_band = lin - band * GROUP_M * p.tiles_n;
    const uint32_t tile_m = band_first + in_band % band_rows;
    const uint32_t tile_n = in_band / band_rows;
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    // ---- per-lane load sources ---------------------------------------------
    const int8_t* wsrc[WLOADS];
    uint32_t xoff[XLOADS];
#pragma unroll
    for (int i = 0; i < WLOADS; i++) {
        const int b = wave + i * NWAVES;  // block index inside the weight part: panel-major
        const int pn = b / KS, s = b % KS;
        wsrc[i] = a.w + ((size_t)(n0 / 32 + pn) * a.ksteps + s) * 1024u + lane * 16;
    }
    const uint32_t last_chunk = (a.k - 1u) / 16u;  // rows are readable up to here
    const uint32_t my_chunk = (lane & 7) ^ ((lane >> 3) & 7);  // slot l%8 of row l/8 holds this chunk
#pragma unroll
    for (int i = 0; i < XLOADS; i++) {
        const int b = wave + i * NWAVES;  // rows 8b .. 8b+7 of the tile
        uint32_t row = m0 + b * 8 + (lane >> 3);
        row = min(row, a.rows - 1u);  // rows past the end compute values nobody stores
        xoff[i] = row * a.ldx;
    }
    const uint32_t ksteps_real = (a.k + 31u) / 32u;
    const uint32_t nkb = (ksteps_real + KS - 1) / KS;

    auto issue_stage = [&](uint32_t kb, int stage) {
        if (VXHIP_PROBE_NO_LOADS && kb > 0) return;
        char* base = lds_raw + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < WLOADS; i++) {
            const int b = wave + i * NWAVES;
            load_to_lds16(wsrc[i] + (size_t)kb * KS * 1024u, base + b * 1024);
        }
        // k-chunks past the row end pair with zero weights: clamp the address
        const uint32_t chunk = min(kb * 8u + my_chunk, last_chunk);
#pragma unroll
        for (int i = 0; i < XLOADS; i++) {
            const int b = wave + i * NWAVES;
            load_to_lds16(a.x + xoff[i] + chunk * 16u, base + (WBLK + b) * 1024);
        }
    };

    // ---- accumulators --------------------------------------------------------
    v16i acc[TN][TM];
    v16i fsum[F32OUT ? TN : 1][F32OUT ? TM : 1];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
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
    auto fold_group = [&](uint32_t g) {
        if constexpr (F32OUT) {
            const float* srow = a.scales_t + (size_t)min(g, a.groups - 1u) * a.n_pad;
#pragma unroll
            for (int i = 0; i < TN; i++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const v4f sw = *reinterpret_cast<const v4f*>(srow + nbase + i * 32 + q * 8);
#pragma unroll
                    for (int j = 0; j < TM; j++) {
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const int r = q * 4 + e;
                            const float gs = __fmul_rn(row_scale[j], sw[e]);
                            const float term = __fmul_rn((float)acc[i][j][r], gs);
                            fsum[i][j][r] = __float_as_int(
                                __fadd_rn(__int_as_float(fsum[i][j][r]), term));
                            acc[i][j][r] = 0;
                        }
                    }
                }
            }
        }
    };

    // ---- fragment addressing ---------------------------------------------------
    // weights: block (panel, step) at 1 KiB granularity, lane slot 16*lane
    // activations: row (wave_m*TM+j)*32 + lane%32 of 128 bytes, chunk 2s + lane/32 at slot chunk ^ (row%8)
    const uint32_t w_frag = (uint32_t)(wave_n * TN * KS) * 1024u + lane * 16u;
    const uint32_t x_row = WBLK * 1024u + ((uint32_t)(wave_m * TM * 32) + (lane & 31)) * 128u;
    uint32_t x_slot[KS];
#pragma unroll
    for (int s = 0; s < KS; s++) x_slot[s] = (((2u * s + (lane >> 5)) ^ (lane & 7u)) << 4);

    auto read_frags = [&](const char* stage, int s, v4i (&wf)[TN], v4i (&xf)[TM]) {
#pragma unroll
        for (int i = 0; i < TN; i++)
            wf[i] = *reinterpret_cast<const v4i*>(stage + w_frag + (i * KS + s) * 1024);
#pragma unroll
        for (int j = 0; j < TM; j++)
            xf[j] = *reinterpret_cast<const v4i*>(stage + x_row + j * 32 * 128 + x_slot[s]);
    };

    // ---- main loop -------------------------------------------------------------
    // Two LDS stages.  One barrier per k-block, placed before the block's last k-step: by
    // then a wave has issued all its reads of the current stage (fragments are requested one
    // step ahead of the MFMAs that use them), so after the barrier the stage can be refilled
    // for block kb+2 and the first fragments of block kb+1 can be requested while the last
    // MFMAs of block kb still run.  MFMA issue therefore never waits on LDS latency.
    issue_stage(0, 0);
    // per-channel epilogue constants of this tile (structure of arrays, so a lane's four
    // consecutive channels are one ds_read_b128 each), computed while the first stage is in flight
    float* lds_f0 = reinterpret_cast<float*>(lds_raw + 2 * STAGE_BYTES);
    int32_t* lds_cb = reinterpret_cast<int32_t*>(lds_f0 + BN);
    float* lds_bo = reinterpret_cast<float*>(lds_cb + BN);
    int32_t* lds_zw = reinterpret_cast<int32_t*>(lds_bo + BN);
    char* lds_sink = reinterpret_cast<char*>(lds_zw + BN);  // 1 KiB landing pad of the L2 prefetches
    if constexpr (!F32OUT) {
        for (int t = threadIdx.x; t < BN; t += NWAVES * 64) {
            const ChannelConsts c = channel_consts<MODE>(a, n0 + t);
            lds_f0[t] = c.f0;
            lds_cb[t] = c.cb;
            lds_bo[t] = c.bo;
            lds_zw[t] = c.zw;
        }
    }
    // L2 prefetch: the operand slices of a k-block are shared by the workgroups of an XCD, but
    // the first one to touch a line waits for the fabric.  Touch the lines of block kb+PF_AHEAD
    // early (one 16-byte piece per 128-byte line, dumped into a scratch pad) so that the real
    // loads, issued two blocks later, hit in L2.
    constexpr uint32_t PF_AHEAD = 3;
    constexpr int PF_LINES = (WBLK * 8 + BM);           // 128-byte lines per stage
    constexpr int PF_LOADS = (PF_LINES + NWAVES * 64 - 1) / (NWAVES * 64);  // per wave
    auto prefetch_l2 = [&](uint32_t kb) {
        if (VXHIP_PROBE_NO_LOADS || VXHIP_PROBE_NO_PREFETCH) return;
        kb = min(kb, nkb - 1u);
#pragma unroll
        for (int i = 0; i < PF_LOADS; i++) {
            const uint32_t line = min((uint32_t)(i * NWAVES + wave) * 64u + lane, (uint32_t)PF_LINES - 1u);
            const int8_t* src;
            if (line < (uint32_t)WBLK * 8u) {  // weight lines: panel-major blocks of 8 lines
                const uint32_t blk = line >> 3, pn = blk / KS, st = blk % KS;
                src = a.w + ((size_t)(n0 / 32 + pn) * a.ksteps + kb * KS + st) * 1024u + (line & 7u) * 128u;
            } else {
                const uint32_t row = min(m0 + (line - WBLK * 8u), a.rows - 1u);
                src = a.x + (size_t)row * a.ldx + min(kb * 8u, last_chunk) * 16u;
            }
            load_to_lds16(src, lds_sink);
        }
    };
    auto mfma_step = [&](int s, uint32_t kb, v4i (&wf)[TN], v4i (&xf)[TM]) {
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int j = 0; j < TM; j++) {
                if (VXHIP_PROBE_NO_MFMA) {
                    acc[i][j][0] += wf[i][0] ^ xf[j][1];
                    continue;
                }
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i], xf[j], acc[i][j], 0, 0, 0);
            }
        if constexpr (F32OUT) {
            if constexpr (GK <= KS) {
                if ((s + 1) % GK == 0) fold_group((kb * KS + s) / GK);
            }
        }
    };
    // interleave the next step's fragment reads with this step's MFMAs
    auto interleave = [&]() {
        constexpr int READS = TN + TM, MF = TN * TM, PER = MF / READS;
#pragma unroll
        for (int r = 0; r < READS; r++) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // one LDS read
            __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);  // PER MFMAs
        }
        if constexpr (MF - PER * READS > 0) __builtin_amdgcn_sched_group_barrier(0x008, MF - PER * READS, 0);
    };

    prefetch_l2(1);
    prefetch_l2(2);
    wait_vmcnt<0>();
    wg_barrier();
    if (nkb > 1) issue_stage(1, 1);
    prefetch_l2(PF_AHEAD);
    v4i wf[2][TN], xf[2][TM];
    read_frags(lds_raw, 0, wf[0], xf[0]);
    for (uint32_t kb = 0; kb < nkb; kb++) {
        const int cur = kb & 1;
        const char* stage = lds_raw + cur * STAGE_BYTES;
#pragma unroll
        for (int s = 0; s < KS - 1; s++) {
            read_frags(stage, s + 1, wf[(s + 1) & 1], xf[(s + 1) & 1]);
            mfma_step(s, kb, wf[s & 1], xf[s & 1]);
            if constexpr (!F32OUT) interleave();
        }
        if (kb + 1 < nkb) {
            wait_lgkm0();  // my reads of this stage have landed in registers
            // my loads of the next stage have landed (the prefetches issued after them may still fly)
            if (VXHIP_PROBE_NO_LOADS || VXHIP_PROBE_NO_PREFETCH) wait_vmcnt<0>(); else wait_vmcnt<PF_LOADS>();
            wg_barrier();
            if (kb + 2 < nkb) issue_stage(kb + 2, cur);
            prefetch_l2(kb + 1 + PF_AHEAD);
            read_frags(lds_raw + (cur ^ 1) * STAGE_BYTES, 0, wf[0], xf[0]);
        }
        mfma_step(KS - 1, kb, wf[(KS - 1) & 1], xf[(KS - 1) & 1]);
        if constexpr (!F32OUT) interleave();
        if constexpr (F32OUT && (GK > KS)) {
            if (((kb + 1) * KS) % GK == 0 || kb + 1 == nkb) fold_group((kb * KS) / GK);
        }
    }
    wait_vmcnt<0>();  // nothing of this workgroup may still be writing LDS when the epilogue reuses it
    if (VXHIP_PROBE_NO_EPILOGUE) {
        int fold = 0;
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int j = 0; j < TM; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) fold ^= acc[i][j][r];
        if (fold == 0x7fffffff) ((int*)a.y)[0] = 1;
        return;
    }

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
        bool lean = fast_div_in_range(so) && a.zw == nullptr;
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
        // LEAN: no weight zero points and every quotient in the range of div_by_uniform
        auto run = [&](auto lean_tag) {
            constexpr bool LEAN = decltype(lean_tag)::value;
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
                    if (MODE == (int)Epilogue::RequantRow && a.bias_row) bo = *reinterpret_cast<const v4f*>(lds_bo + c0);
                    if (!LEAN && a.zw) zw = *reinterpret_cast<const v4i*>(lds_zw + c0);
#pragma unroll
                    for (int j = 0; j < TM; j++) {
                        uint32_t u[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            uint32_t total = (uint32_t)acc[i][j][q * 4 + e] + (uint32_t)cb[e];
                            if (!LEAN) total -= (uint32_t)zw[e] * (uint32_t)rsum[j];
                            float mu = f0[e];
                            if constexpr (MODE == (int)Epilogue::RequantRow) {
                                const float prod = __fmul_rn(row_scale[j], f0[e]);
                                mu = LEAN ? div_by_uniform(prod, so, sr) : __fdiv_rn(prod, so);
                            }
                            float t = __fadd_rn(__fmul_rn((float)(int32_t)total, mu), zp_f);
                            if (MODE == (int)Epilogue::RequantRow && a.bias_row) t = __fadd_rn(t, bo[e]);
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
        if (wave_lean) run(std::true_type{}); else run(std::false_type{});
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

template <int WN, int WM, int TN, int TM, int MODE, int GK, bool FAST>
bool launch_one(hipStream_t s, const LinearArgs& a) {
    constexpr int BN = WN * TN * 32, BM = WM * TM * 32;
    constexpr int LDS = 2 * ((BN / 32) * KS + BM / 8) * 1024 + BN * 16 + 1024;
    static bool configured = false;
    auto kern = gemm_mfma_kernel<WN, WM, TN, TM, MODE, GK, FAST>;
    if (!configured) {
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS) !=
            hipSuccess)
            return false;
        configured = true;
    }
    GemmParams p;
    p.a = a;
    p.tiles_n = (a.n + BN - 1) / BN;
    p.tiles_m = (a.rows + BM - 1) / BM;
    const uint32_t total = p.tiles_n * p.tiles_m;
    const uint32_t grid = ((total + 7u) / 8u) * 8u;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WN * WM * 64), LDS, s, p);
    return hipGetLastError() == hipSuccess;
}

template <int WN, int WM, int TN, int TM, int MODE, int GK>
bool launch_cfg(hipStream_t s, const LinearArgs& a) {
    if constexpr (MODE != (int)Epilogue::DequantF32) {
        if ((a.n % 16u) == 0u && a.y && !a.acc_out && ((uintptr_t)a.y % 16u) == 0u)
            return launch_one<WN, WM, TN, TM, MODE, GK, true>(s, a);
    }
    return launch_one<WN, WM, TN, TM, MODE, GK, false>(s, a);
}

template <int MODE, int GK>
const char* dispatch_tile(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    auto forced = [&](const char* tag) { return force && strstr(force, tag) != nullptr; };
    const uint64_t big_tiles = (uint64_t)((a.n + 255) / 256) * ((a.rows + 255) / 256);
    bool big = big_tiles >= (uint64_t)cu_count * 3 / 4;
    if (forced("t256x256")) big = true;
    if (forced("t128x128")) big = false;
    if constexpr (MODE == (int)Epilogue::DequantF32) {
        // int32 tile accumulators plus f32 running sums: keep the wave tile at 64x64
        if (big) return launch_cfg<2, 4, 2, 2, MODE, GK>(s, a) ? "t128x256" : nullptr;
        return launch_cfg<2, 2, 2, 2, MODE, GK>(s, a) ? "t128x128" : nullptr;
    } else {
        if (big && forced("w4")) return launch_cfg<2, 2, 4, 4, MODE, GK>(s, a) ? "t256x256w4" : nullptr;
        if (big) return launch_cfg<2, 4, 4, 2, MODE, GK>(s, a) ? "t256x256" : nullptr;
        return launch_cfg<2, 2, 2, 2, MODE, GK>(s, a) ? "t128x128" : nullptr;
    }
}

}  // namespace

const char* launch_gemm_mfma(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    if (a.ldx < 16u || (a.ldx % 16u) != 0u || ((uintptr_t)a.x % 16u) != 0u) return nullptr;
    if ((uint64_t)a.rows * a.ldx > 0xffffffffull) return nullptr;  // 32-bit activation offsets
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
