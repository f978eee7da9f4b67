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
// (no VGPR staging).  Weights are already in operand order (see common.h), so
// their tile is a linear copy.  Activations are row-major; lane l of a load
// fetches the 16 bytes X[m0 + l%32][k0 + 16*(l/32) ..], which lands them in
// LDS in operand order as well.  Every fragment read is then one conflict-free
// ds_read_b128 at lane*16.
#include "common.h"
#include "device_math.h"
#include "epilogue.h"

#include <stdio.h>
#include <string.h>

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

// WN x WM wavefronts, each owning TN x TM MFMA tiles of 32x32; KS k-steps of
// 32 per stage.  MODE is the Epilogue; GK = k-steps per scale group (DequantF32).
template <int WN, int WM, int TN, int TM, int KS, int MODE, int GK>
__global__ __launch_bounds__(WN* WM * 64) void gemm_mfma_kernel(const GemmParams p) {
    constexpr int NWAVES = WN * WM;
    constexpr int BN = WN * TN * 32, BM = WM * TM * 32;
    constexpr int WBLK = (BN / 32) * KS, XBLK = (BM / 32) * KS;  // 1 KiB blocks per stage
    constexpr int NBLK = WBLK + XBLK;
    static_assert(WBLK % NWAVES == 0 && XBLK % NWAVES == 0, "blocks must divide over waves");
    constexpr int WLOADS = WBLK / NWAVES, XLOADS = XBLK / NWAVES, LOADS = WLOADS + XLOADS;
    constexpr int STAGE_BYTES = NBLK * 1024;
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
        const int b = wave + i * NWAVES;  // block index inside the weight part
        const int pn = b / KS, s = b % KS;
        wsrc[i] = a.w + ((size_t)(n0 / 32 + pn) * a.ksteps + s) * 1024u + lane * 16;
    }
    const uint32_t last_chunk = (a.k - 1u) / 16u;  // rows are readable up to here
#pragma unroll
    for (int i = 0; i < XLOADS; i++) {
        const int b = wave + i * NWAVES;
        const int pm = b / KS;
        uint32_t row = m0 + pm * 32 + (lane & 31);
        row = min(row, a.rows - 1u);  // rows past the end compute values nobody stores
        xoff[i] = row * a.ldx;
    }
    const uint32_t ksteps_real = (a.k + 31u) / 32u;
    const uint32_t nkb = (ksteps_real + KS - 1) / KS;

    auto issue_stage = [&](uint32_t kb, int stage) {
        char* base = lds_raw + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < WLOADS; i++) {
            const int b = wave + i * NWAVES;
            load_to_lds16(wsrc[i] + (size_t)kb * KS * 1024u, base + b * 1024);
        }
#pragma unroll
        for (int i = 0; i < XLOADS; i++) {
            const int b = wave + i * NWAVES;
            const int s = b % KS;
            // k-chunks past the row end pair with zero weights: clamp the address
            const uint32_t chunk = min((kb * KS + s) * 2u + (lane >> 5), last_chunk);
            load_to_lds16(a.x + xoff[i] + chunk * 16u, base + (WBLK + b) * 1024);
        }
    };

    // ---- accumulators --------------------------------------------------------
    v16i acc[TN][TM];
    v16i fsum[MODE == (int)Epilogue::DequantF32 ? TN : 1][MODE == (int)Epilogue::DequantF32 ? TM : 1];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    if constexpr (MODE == (int)Epilogue::DequantF32) {
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
        if constexpr (MODE == (int)Epilogue::DequantF32) {
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

    // ---- main loop -------------------------------------------------------------
    issue_stage(0, 0);
    // per-channel epilogue constants of this tile, computed while the first stage is in flight
    ChannelConsts* lds_cc = reinterpret_cast<ChannelConsts*>(lds_raw + 2 * STAGE_BYTES);
    if constexpr (MODE != (int)Epilogue::DequantF32) {
        for (int t = threadIdx.x; t < BN; t += NWAVES * 64) lds_cc[t] = channel_consts<MODE>(a, n0 + t);
    }
    for (uint32_t kb = 0; kb < nkb; kb++) {
        const int cur = kb & 1;
        if (kb + 1 < nkb) {
            issue_stage(kb + 1, cur ^ 1);
            wait_vmcnt<LOADS>();
        } else {
            wait_vmcnt<0>();
        }
        wg_barrier();
        const char* wl = lds_raw + cur * STAGE_BYTES + lane * 16;
        const char* xl = wl + WBLK * 1024;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            v4i wf[TN], xf[TM];
#pragma unroll
            for (int i = 0; i < TN; i++)
                wf[i] = *reinterpret_cast<const v4i*>(wl + ((wave_n * TN + i) * KS + s) * 1024);
#pragma unroll
            for (int j = 0; j < TM; j++)
                xf[j] = *reinterpret_cast<const v4i*>(xl + ((wave_m * TM + j) * KS + s) * 1024);
#pragma unroll
            for (int i = 0; i < TN; i++)
#pragma unroll
                for (int j = 0; j < TM; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[i], xf[j], acc[i][j], 0, 0, 0);
            if constexpr (MODE == (int)Epilogue::DequantF32) {
                if constexpr (GK <= KS) {
                    if ((s + 1) % GK == 0) fold_group((kb * KS + s) / GK);
                }
            }
        }
        if constexpr (MODE == (int)Epilogue::DequantF32 && (GK > KS)) {
            if (((kb + 1) * KS) % GK == 0 || kb + 1 == nkb) fold_group((kb * KS) / GK);
        }
        wait_lgkm0();
        wg_barrier();
    }

    // ---- epilogue ----------------------------------------------------------------
#pragma unroll
    for (int j = 0; j < TM; j++) {
        const uint32_t m = m0 + (wave_m * TM + j) * 32 + (lane & 31);
        int32_t rsum = 0;
        if constexpr (MODE != (int)Epilogue::DequantF32) {
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
                    if constexpr (MODE == (int)Epilogue::DequantF32)
                        fs[e] = __int_as_float(fsum[i][j][q * 4 + e]);
                    else
                        cc[e] = lds_cc[n - n0 + e];
                }
                store_quad<MODE>(a, m, n, dot, fs, rs, rsum, cc);
            }
        }
    }
}

template <int WN, int WM, int TN, int TM, int KS, int MODE, int GK>
bool launch_cfg(hipStream_t s, const LinearArgs& a) {
    constexpr int BN = WN * TN * 32, BM = WM * TM * 32;
    constexpr int LDS = 2 * ((BN / 32) + (BM / 32)) * KS * 1024 + BN * (int)sizeof(ChannelConsts);
    static bool configured = false;
    auto kern = gemm_mfma_kernel<WN, WM, TN, TM, KS, MODE, GK>;
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

template <int MODE, int GK>
const char* dispatch_tile(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    const bool want_big = force ? strstr(force, "t256x256") != nullptr : false;
    const bool want_small = force ? strstr(force, "t128x128") != nullptr : false;
    const uint64_t big_tiles = (uint64_t)((a.n + 255) / 256) * ((a.rows + 255) / 256);
    bool big = big_tiles >= (uint64_t)cu_count * 3 / 4;
    if (want_big) big = true;
    if (want_small) big = false;
    if constexpr (MODE == (int)Epilogue::DequantF32) {
        // int32 tile accumulators plus f32 running sums: keep the wave tile at 64x64
        if (big) return launch_cfg<2, 4, 2, 2, 4, MODE, GK>(s, a) ? "t128x256" : nullptr;
        return launch_cfg<2, 2, 2, 2, 4, MODE, GK>(s, a) ? "t128x128" : nullptr;
    } else {
        if (big) return launch_cfg<2, 2, 4, 4, 4, MODE, GK>(s, a) ? "t256x256" : nullptr;
        return launch_cfg<2, 2, 2, 2, 4, MODE, GK>(s, a) ? "t128x128" : nullptr;
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
