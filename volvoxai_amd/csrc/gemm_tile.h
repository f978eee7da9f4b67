// Pieces shared by the LDS-tiled GEMM kernels (gemm_mfma.hip, gemm_k64.hip): waits and barriers
// spelled out, the global -> LDS load, compile-time loops, and the workgroup -> tile mapping.
#pragma once

#include "common.h"

#include <type_traits>
#include <utility>

namespace vxhip {

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

// one instruction fills 1 KiB (or 256 bytes) of LDS, lane l writing bytes 16*l (4*l) of it
__device__ __forceinline__ void load_to_lds16(const void* gptr, void* lptr) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gptr,
                                     (__attribute__((address_space(3))) void*)lptr, 16, 0, 0);
}
__device__ __forceinline__ void load_to_lds4(const void* gptr, void* lptr) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gptr,
                                     (__attribute__((address_space(3))) void*)lptr, 4, 0, 0);
}

struct GemmParams {
    LinearArgs a;
    uint32_t tiles_n, tiles_m;
};

template <int V>
using IC = std::integral_constant<int, V>;
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(IC<I>{}), ...);
}
// f(IC<0>{}), f(IC<1>{}), ... f(IC<N-1>{}): a loop whose index is a compile-time constant
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// Workgroup -> tile, XCD aware.  Consecutive workgroup ids land on different XCDs (8 of them,
// each with its own L2).  XCD x is given the x-th contiguous run of tiles, and tiles are ordered
// in bands of GROUP_M tile rows so that a run is a compact block of the output: that block's
// operand slices are then shared through one L2 instead of being fetched by all.
struct TileOrigin {
    uint32_t m0, n0;
    bool valid;
};
template <int BN, int BM, uint32_t GROUP_M = 4>
__device__ __forceinline__ TileOrigin tile_of_workgroup(const GemmParams& p) {
    const uint32_t total = p.tiles_n * p.tiles_m;
    const uint32_t per_xcd = (total + 7u) / 8u;
    const uint32_t lin = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if (lin >= total) return TileOrigin{0u, 0u, false};
    const uint32_t band = lin / (GROUP_M * p.tiles_n);
    const uint32_t band_first = band * GROUP_M;
    const uint32_t band_rows = min(GROUP_M, p.tiles_m - band_first);
    const uint32_t in_band = lin - band * GROUP_M * p.tiles_n;
    const uint32_t tile_m = band_first + in_band % band_rows;
    const uint32_t tile_n = in_band / band_rows;
    return TileOrigin{tile_m * (uint32_t)BM, tile_n * (uint32_t)BN, true};
}

// gemm_k64.hip
const char* launch_gemm_k64(hipStream_t s, const LinearArgs& a, int tile);
const char* launch_gemm_k64_f32(hipStream_t s, const LinearArgs& a, bool deep);

}  // namespace vxhip
