// Hardware-ceiling probe for the MFMA roofline: how fast do the matrix pipes run when they
// are fed without a single stall?  Every wave keeps 16 independent 32x32 accumulators in
// registers and issues v_mfma_i32_32x32x32_i8 back to back -- no memory, no LDS, no barrier.
// With constant operands the device holds its clock; with random 8-bit operands (what a GEMM
// on uniform +-127 data feeds them) the datapath toggles fully and the power manager lowers
// the shader clock, which bounds what any int8 GEMM can reach on such data.
#include "common.h"

#include <vector>

namespace vxhip {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kAccumulators = 16;

__global__ __launch_bounds__(256) void mfma_rate_kernel(const v4i* __restrict__ operands, uint32_t rounds,
                                                        uint64_t* __restrict__ clocks, int* sink) {
    v16i acc[kAccumulators];
#pragma unroll
    for (int i = 0; i < kAccumulators; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
    v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a[i] = operands[i * 256 + threadIdx.x];
        b[i] = operands[(i + 4) * 256 + threadIdx.x];
    }
    const uint64_t c0 = __builtin_readcyclecounter(), t0 = __builtin_amdgcn_s_memrealtime();
    for (uint32_t it = 0; it < rounds; it++) {
#pragma unroll
        for (int i = 0; i < kAccumulators; i++)
            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 3], b[(i >> 2) & 3], acc[i], 0, 0, 0);
    }
    int fold = 0;
#pragma unroll
    for (int i = 0; i < kAccumulators; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) fold ^= acc[i][r];
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clocks[0] = __builtin_readcyclecounter() - c0;       // shader cycles
        clocks[1] = __builtin_amdgcn_s_memrealtime() - t0;   // 100 MHz ticks
    }
    if (fold == 0x12345) sink[0] = fold;  // keeps the accumulators alive
}

}  // namespace
}  // namespace vxhip

using namespace vxhip;

extern "C" VxHipStatus vxhip_probe_mfma_rate(VxHipContext* ctx, uint32_t rounds, uint32_t random_operands,
                                             double* tops, double* shader_mhz, double* microseconds) {
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
    // one workgroup of four waves per compute unit: one wave on every SIMD
    const int groups = ctx->cu_count > 0 ? ctx->cu_count : 256;
    float ms = 0.0f;
    if (st == VXHIP_OK) {
        hipLaunchKernelGGL(mfma_rate_kernel, dim3(groups), dim3(256), 0, ctx->stream, operands, rounds, clocks, sink);
        check(hipStreamSynchronize(ctx->stream), "warm-up launch");
        check(hipEventRecord(e0, ctx->stream), "record");
        hipLaunchKernelGGL(mfma_rate_kernel, dim3(groups), dim3(256), 0, ctx->stream, operands, rounds, clocks, sink);
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
