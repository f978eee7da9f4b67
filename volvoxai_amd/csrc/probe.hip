// Hardware-ceiling probe for the MFMA roofline: how fast do the matrix pipes run when they
// are fed without a single stall?  Every wave keeps 16 independent 32x32 accumulators in
// registers and issues v_mfma_i32_32x32x32_i8 back to back -- no memory, no LDS, no barrier --
// or, in the second form, two waves per SIMD with 16 independent 16x16 accumulators each and
// v_mfma_i32_16x16x64_i8 (the same operations per round and SIMD), which is the instruction and the
// occupancy of the large GEMM tiles.
// With constant operands the device holds its clock; with random 8-bit operands (what a GEMM
// on uniform +-127 data feeds them) the datapath toggles fully and the power manager lowers
// the shader clock, which bounds what any int8 GEMM can reach on such data.
#include "common.h"

#include <type_traits>
#include <vector>

namespace vxhip {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kAccumulators = 16;

template <bool K64>
__global__ __launch_bounds__(K64 ? 512 : 256) void mfma_rate_kernel(const v4i* __restrict__ operands, uint32_t rounds,
                                                        uint64_t* __restrict__ clocks, int* sink) {
    // 16 tiles per wave either way; the 16x16x64 form runs two waves per SIMD (as the GEMM does), so
    // a round is the same number of operations per SIMD in both forms
    constexpr int kTiles = kAccumulators;
    using Tile = typename std::conditional<K64, v4i, v16i>::type;
    Tile acc[kTiles];
#pragma unroll
    for (int i = 0; i < kTiles; i++)
#pragma unroll
        for (int r = 0; r < (K64 ? 4 : 16); r++) acc[i][r] = 0;
    v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a[i] = operands[i * 256 + (threadIdx.x & 255u)];
        b[i] = operands[(i + 4) * 256 + (threadIdx.x & 255u)];
    }
    const uint64_t c0 = __builtin_readcyclecounter(), t0 = __builtin_amdgcn_s_memrealtime();
    for (uint32_t it = 0; it < rounds; it++) {
#pragma unroll
        for (int i = 0; i < kTiles; i++) {
            if constexpr (K64)
                acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[(i >> 2) & 3], b[i & 3], acc[i], 0, 0, 0);
            else
                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 3], b[(i >> 2) & 3], acc[i], 0, 0, 0);
        }
    }
    int fold = 0;
#pragma unroll
    for (int i = 0; i < kTiles; i++)
#pragma unroll
        for (int r = 0; r < (K64 ? 4 : 16); r++) fold ^= acc[i][r];
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clocks[0] = __builtin_readcyclecounter() - c0;       // shader cycles
        clocks[1] = __builtin_amdgcn_s_memrealtime() - t0;   // 100 MHz ticks
    }
    if (fold == 0x12345) sink[0] = fold;  // keeps the accumulators alive
}

// The HBM counterpart: the same bytes a GEMV streams, read and folded into a word that is never
// stored -- no MFMA, no LDS, no tail.  What this reaches is what the memory system gives a
// kernel of that size, launch ramp and drain included.
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ data, size_t count,
                                                          uint32_t* sink) {
    const size_t stride = (size_t)gridDim.x * 256u;
    size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    uint32_t fold = 0u;
    for (; i + 3u * stride < count; i += 4u * stride) {  // four loads in flight per thread
        const uint4 a = data[i], b = data[i + stride], c = data[i + 2u * stride], d = data[i + 3u * stride];
        fold ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    for (; i < count; i += stride) {
        const uint4 a = data[i];
        fold ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (fold == 0x9e3779b9u) sink[0] = fold;  // keeps the loads alive; practically never true
}

// Do matrix and vector instructions of a SIMD run beside each other?  Four waves per SIMD, random 8-bit
// operands.  A round of a wave is what a 64 x 32 wave tile of the dequantizing GEMM does per scale group of
// 128: sixteen v_mfma_i32_16x16x64_i8 (two per result tile) and the fold of 32 accumulator registers,
// sum += f32(dot) * c with each operation rounded on its own (three vector instructions per register; the
// vector-only form needs a fourth, an integer add, to keep the conversion in the loop).
// MODE 0: the MFMAs alone.  1: the folds alone.  2: both in every wave, the fold of a tile behind the MFMAs
// of the next.  3: even waves run the MFMAs, odd waves the folds (half of each kind of work).
template <int MODE>
__global__ __launch_bounds__(1024) void mfma_valu_overlap_kernel(const v4i* __restrict__ operands, uint32_t rounds,
                                                                uint64_t* __restrict__ clocks, float* sink) {
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    v4i a[2], b[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        a[i] = operands[(threadIdx.x & 255u) + 256 * i];
        b[i] = operands[(threadIdx.x & 255u) + 256 * (i + 2)];
    }
    v4i acc[8];
    float sum[32];
#pragma unroll
    for (int i = 0; i < 8; i++) acc[i] = v4i{(int)threadIdx.x, i, 3, 4};
#pragma unroll
    for (int i = 0; i < 32; i++) sum[i] = 0.f;
    const float c = __int_as_float(0x3a83126f + (int)(threadIdx.x & 7u));
    auto mfmas = [&](int i) {
        acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[0], b[i & 1], acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[1], b[(i + 1) & 1], acc[i], 0, 0, 0);
    };
    auto fold = [&](int j, bool alone) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            sum[j * 4 + e] = __fadd_rn(sum[j * 4 + e], __fmul_rn((float)acc[j][e], c));
            if (alone) acc[j][e] += 0x01010101;
        }
    };
    const uint64_t c0 = __builtin_readcyclecounter(), t0 = __builtin_amdgcn_s_memrealtime();
    const bool folds_only = MODE == 1 || (MODE == 3 && (wave & 1));
    if (folds_only) {
        for (uint32_t r = 0; r < rounds; r++)
#pragma unroll
            for (int i = 0; i < 8; i++) fold(i, true);
    } else {
        for (uint32_t r = 0; r < rounds; r++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                mfmas(i);
                if constexpr (MODE == 2) fold((i + 7) & 7, false);
            }
    }
    float f = 0.f;
#pragma unroll
    for (int i = 0; i < 32; i++) f += sum[i];
#pragma unroll
    for (int i = 0; i < 8; i++) f += (float)(acc[i][0] ^ acc[i][1] ^ acc[i][2] ^ acc[i][3]);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clocks[0] = __builtin_readcyclecounter() - c0;
        clocks[1] = __builtin_amdgcn_s_memrealtime() - t0;
    }
    if (f == 1.2345f) sink[0] = f;
}

}  // namespace
}  // namespace vxhip

using namespace vxhip;

extern "C" VxHipStatus vxhip_probe_mfma_valu_overlap(VxHipContext* ctx, uint32_t rounds, uint32_t constant_operands,
                                                     double* microseconds, double* shader_mhz) {
    if (!ctx || !rounds || !microseconds) {
        set_error("probe_mfma_valu_overlap: null context/result or zero rounds");
        return VXHIP_INVALID_ARGUMENT;
    }
    VXHIP_TRY(hipSetDevice(ctx->device));
    std::vector<uint32_t> host(4 * 256 * 4);
    uint32_t lcg = 12345u;
    for (auto& v : host) {
        lcg = lcg * 1664525u + 1013904223u;
        const uint32_t hi = lcg;
        lcg = lcg * 1664525u + 1013904223u;
        v = constant_operands ? 0x01010101u : (hi & 0xffff0000u) | (lcg >> 16);
    }
    v4i* operands = nullptr;
    uint64_t* clocks = nullptr;
    float* sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    VxHipStatus st = VXHIP_OK;
    auto check = [&](hipError_t e, const char* what) {
        if (st == VXHIP_OK && e != hipSuccess) st = hip_status(e, what);
    };
    check(hipMalloc((void**)&operands, host.size() * 4), "hipMalloc");
    check(hipMalloc((void**)&clocks, 16), "hipMalloc");
    check(hipMalloc((void**)&sink, 64), "hipMalloc");
    check(hipEventCreate(&e0), "hipEventCreate");
    check(hipEventCreate(&e1), "hipEventCreate");
    if (st == VXHIP_OK) {
        check(hipMemcpyAsync(operands, host.data(), host.size() * 4, hipMemcpyHostToDevice, ctx->stream), "copy");
        check(hipStreamSynchronize(ctx->stream), "sync");
    }
    const int groups = ctx->cu_count > 0 ? ctx->cu_count : 256;
    void (*const kernels[4])(const v4i*, uint32_t, uint64_t*, float*) = {
        mfma_valu_overlap_kernel<0>, mfma_valu_overlap_kernel<1>, mfma_valu_overlap_kernel<2>, mfma_valu_overlap_kernel<3>};
    for (int mode = 0; mode < 4 && st == VXHIP_OK; mode++) {
        float ms = 0.0f;
        // one launch to settle the clock, then the timed one
        hipLaunchKernelGGL(kernels[mode], dim3(groups), dim3(1024), 0, ctx->stream, operands, rounds, clocks, sink);
        check(hipEventRecord(e0, ctx->stream), "record");
        hipLaunchKernelGGL(kernels[mode], dim3(groups), dim3(1024), 0, ctx->stream, operands, rounds, clocks, sink);
        check(hipGetLastError(), "launch");
        check(hipEventRecord(e1, ctx->stream), "record");
        check(hipEventSynchronize(e1), "sync");
        check(hipEventElapsedTime(&ms, e0, e1), "elapsed");
        uint64_t c[2] = {0, 0};
        check(hipMemcpy(c, clocks, sizeof c, hipMemcpyDeviceToHost), "read clocks");
        microseconds[mode] = ms * 1e3;
        if (shader_mhz) shader_mhz[mode] = c[1] ? (double)c[0] / ((double)c[1] / 100.0) : 0.0;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(operands);
    (void)hipFree(clocks);
    (void)hipFree(sink);
    return st;
}

extern "C" VxHipStatus vxhip_probe_stream_read(VxHipContext* ctx, const void* const* buffers_dev,
                                               uint32_t buffer_count, size_t bytes_each, uint32_t launches,
                                               double* gigabytes_per_second, double* microseconds) {
    if (!ctx || !buffers_dev || !buffer_count || bytes_each < 16u || !launches || !gigabytes_per_second) {
        set_error("probe_stream_read: null argument, no buffer or no launch");
        return VXHIP_INVALID_ARGUMENT;
    }
    for (uint32_t i = 0; i < buffer_count; i++) {
        if (!buffers_dev[i] || ((uintptr_t)buffers_dev[i] % 16u) != 0u) {
            set_error("probe_stream_read: buffer %u is null or not 16-byte aligned", i);
            return VXHIP_INVALID_ARGUMENT;
        }
    }
    VXHIP_TRY(hipSetDevice(ctx->device));
    uint32_t* sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    VxHipStatus st = VXHIP_OK;
    auto check = [&](hipError_t e, const char* what) {
        if (st == VXHIP_OK && e != hipSuccess) st = hip_status(e, what);
    };
    check(hipMalloc((void**)&sink, 64), "hipMalloc");
    check(hipEventCreate(&e0), "hipEventCreate");
    check(hipEventCreate(&e1), "hipEventCreate");
    const size_t count = bytes_each / 16u;
    const int groups = 16 * (ctx->cu_count > 0 ? ctx->cu_count : 256);  // measured best among 4, 8, 16 per CU
    float ms = 0.0f;
    if (st == VXHIP_OK) {
        for (uint32_t i = 0; i < buffer_count; i++)  // warm-up, one pass over every buffer
            hipLaunchKernelGGL(stream_read_kernel, dim3(groups), dim3(256), 0, ctx->stream,
                               (const uint4*)buffers_dev[i], count, sink);
        check(hipStreamSynchronize(ctx->stream), "warm-up launches");
        check(hipEventRecord(e0, ctx->stream), "record");
        for (uint32_t i = 0; i < launches; i++)
            hipLaunchKernelGGL(stream_read_kernel, dim3(groups), dim3(256), 0, ctx->stream,
                               (const uint4*)buffers_dev[i % buffer_count], count, sink);
        check(hipGetLastError(), "launch");
        check(hipEventRecord(e1, ctx->stream), "record");
        check(hipEventSynchronize(e1), "sync");
        check(hipEventElapsedTime(&ms, e0, e1), "elapsed");
    }
    if (st == VXHIP_OK) {
        const double us = (double)ms * 1e3 / launches;
        *gigabytes_per_second = (double)(count * 16u) / us / 1e3;
        if (microseconds) *microseconds = us;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    return st;
}

extern "C" VxHipStatus vxhip_probe_mfma_rate(VxHipContext* ctx, uint32_t rounds, uint32_t flags,
                                             double* tops, double* shader_mhz, double* microseconds) {
    const bool random_operands = (flags & 1u) != 0u, k64 = (flags & 2u) != 0u;
    if (!ctx || !rounds || !tops) {
        set_error("probe_mfma_rate: null context/result or zero rounds");
        return VXHIP_INVALID_ARGUMENT;
    }
    VXHIP_TRY(hipSetDevice(ctx->device));
    std::vector<uint32_t> host(8 * 256 * 4);
    uint32_t lcg = 12345u;
    for (auto& v : host) {
        lcg = lcg * 1664525u + 1013904223u;
        uint32_t hi = lcg;
        lcg = lcg * 1664525u + 1013904223u;
        v = random_operands ? ((hi & 0xffff0000u) | (lcg >> 16)) : 0x01010101u;
    }
    v4i* operands = nullptr;
    uint64_t* clocks = nullptr;
    int* sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    VxHipStatus st = VXHIP_OK;
    auto check = [&](hipError_t e, const char* what) {
        if (st == VXHIP_OK && e != hipSuccess) st = hip_status(e, what);
    };
    check(hipMalloc((void**)&operands, host.size() * 4), "hipMalloc");
    check(hipMalloc((void**)&clocks, 16), "hipMalloc");
    check(hipMalloc((void**)&sink, 64), "hipMalloc");
    check(hipEventCreate(&e0), "hipEventCreate");
    check(hipEventCreate(&e1), "hipEventCreate");
    if (st == VXHIP_OK) {
        check(hipMemcpyAsync(operands, host.data(), host.size() * 4, hipMemcpyHostToDevice, ctx->stream), "copy");
        check(hipStreamSynchronize(ctx->stream), "sync");
    }
    // one workgroup per compute unit: one wave on every SIMD (two in the 16x16x64 form)
    const int groups = ctx->cu_count > 0 ? ctx->cu_count : 256;
    float ms = 0.0f;
    if (st == VXHIP_OK) {
        auto kern = k64 ? mfma_rate_kernel<true> : mfma_rate_kernel<false>;
        const int threads = k64 ? 512 : 256;
        hipLaunchKernelGGL(kern, dim3(groups), dim3(threads), 0, ctx->stream, operands, rounds, clocks, sink);
        check(hipStreamSynchronize(ctx->stream), "warm-up launch");
        check(hipEventRecord(e0, ctx->stream), "record");
        hipLaunchKernelGGL(kern, dim3(groups), dim3(threads), 0, ctx->stream, operands, rounds, clocks, sink);
        check(hipGetLastError(), "launch");
        check(hipEventRecord(e1, ctx->stream), "record");
        check(hipEventSynchronize(e1), "sync");
        check(hipEventElapsedTime(&ms, e0, e1), "elapsed");
    }
    uint64_t c[2] = {0, 0};
    if (st == VXHIP_OK) check(hipMemcpy(c, clocks, sizeof c, hipMemcpyDeviceToHost), "read clocks");
    if (st == VXHIP_OK) {
        const double ops = (double)groups * 4.0 * rounds * kAccumulators * 65536.0;
        *tops = ops / 1e12 / (ms * 1e-3);
        if (shader_mhz) *shader_mhz = c[1] ? (double)c[0] / ((double)c[1] / 100.0) : 0.0;
        if (microseconds) *microseconds = ms * 1e3;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(operands);
    (void)hipFree(clocks);
    (void)hipFree(sink);
    return st;
}
