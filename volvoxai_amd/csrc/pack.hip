// Weight prepacking for gfx950 int8 MFMA: the counterpart of the reference's
// vx_pack_q8_weight step (native/src/kernels/packed_quant_gemm.c:237-392),
// which lays weights out for its AVX microkernels and stores per-column weight
// sums for the zero-point fold.  Here the layout is the MFMA operand order
// described in common.h and the sums are of the signed bytes.
#include "common.h"

namespace vxhip {

// One thread produces one 16-byte lane slot of one 1 KiB block.
__global__ __launch_bounds__(256) void pack_weight_kernel(
        const uint8_t* __restrict__ raw, size_t row_stride, uint32_t n, uint32_t k,
        uint32_t flip, uint32_t panels, uint32_t ksteps, uint8_t* __restrict__ out) {
    const size_t slot = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)panels * ksteps * 64u;
    if (slot >= total) return;
    const uint32_t lane = (uint32_t)(slot & 63u);
    const size_t block = slot >> 6;
    const uint32_t step = (uint32_t)(block % ksteps);
    const uint32_t panel = (uint32_t)(block / ksteps);
    const uint32_t row = panel * 32u + (lane & 31u);
    const uint32_t k0 = step * 32u + (lane >> 5) * 16u;
    uint32_t words[4] = {0u, 0u, 0u, 0u};
    if (row < n) {
        const uint8_t* src = raw + (size_t)row * row_stride;
        const uint32_t x = flip ? 0x80u : 0u;
        for (uint32_t j = 0; j < 16u; j++) {
            const uint32_t kk = k0 + j;
            // padding is the value zero in the signed domain
            const uint32_t b = kk < k ? ((uint32_t)src[kk] ^ x) : 0u;
            words[j >> 2] |= b << ((j & 3u) * 8u);
        }
    }
    uint4 v = make_uint4(words[0], words[1], words[2], words[3]);
    *reinterpret_cast<uint4*>(out + slot * 16u) = v;
}

// Four-bit form: one thread produces one 16-byte lane slot, i.e. 16 weights of each of the
// block's two steps.  Source codes of `bits` = 2, 3 or 4 bits are offset by half their range
// (packed_linear_ops.inc:472-477; three-bit codes are a dense bitstream over the row, :249-254);
// every such value fits a 4-bit two's complement number, which is what the block stores, so
// the narrower widths run on the four-bit kernels unchanged.
__global__ __launch_bounds__(256) void pack_nibble_kernel(
        const uint32_t* __restrict__ raw, uint32_t row_words, uint32_t n, uint32_t k, uint32_t bits,
        uint32_t panels, uint32_t kblocks, uint8_t* __restrict__ out) {
    const size_t slot = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t total = (size_t)panels * kblocks * 64u;
    if (slot >= total) return;
    const uint32_t lane = (uint32_t)(slot & 63u);
    const size_t block = slot >> 6;
    const uint32_t pair = (uint32_t)(block % kblocks);
    const uint32_t panel = (uint32_t)(block / kblocks);
    const uint32_t row = panel * 32u + (lane & 31u);
    const uint32_t k0 = pair * 64u + (lane >> 5) * 16u;
    uint32_t words[4] = {0u, 0u, 0u, 0u};
    if (row < n) {
        const uint32_t* src = raw + (size_t)row * row_words;
        auto value = [&](uint32_t kk) -> uint32_t {
            if (kk >= k) return 0u;  // padding is the value zero
            const uint64_t bit = (uint64_t)kk * bits;
            const uint32_t shift = (uint32_t)(bit & 31u);
            uint32_t code = src[bit >> 5] >> shift;
            if (shift + bits > 32u) code |= src[(bit >> 5) + 1u] << (32u - shift);
            code &= (1u << bits) - 1u;
            return (code - (1u << (bits - 1u))) & 15u;
        };
        for (uint32_t j = 0; j < 16u; j++) {
            const uint32_t b = value(k0 + j) | (value(k0 + 32u + j) << 4);
            words[j >> 2] |= b << ((j & 3u) * 8u);
        }
    }
    *reinterpret_cast<uint4*>(out + slot * 16u) = make_uint4(words[0], words[1], words[2], words[3]);
}

// One wavefront per output channel: sum of signed bytes and max |w - zp|.
__global__ __launch_bounds__(256) void weight_row_stats_kernel(
        const uint8_t* __restrict__ raw, size_t row_stride, uint32_t n, uint32_t k, uint32_t flip,
        const int32_t* __restrict__ zps, int32_t* __restrict__ sums, int32_t* __restrict__ absmax) {
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    if (row >= n) return;
    const uint8_t* src = raw + (size_t)row * row_stride;
    const int32_t zp = zps ? zps[row] : 0;
    int32_t sum = 0, amax = 0;
    for (uint32_t kk = lane; kk < k; kk += 64u) {
        const int32_t v = (int32_t)(int8_t)(src[kk] ^ (flip ? 0x80u : 0u));
        sum += v;
        const int32_t d = v - zp;
        amax = max(amax, d < 0 ? -d : d);
    }
    for (int off = 32; off > 0; off >>= 1) {
        sum += __shfl_down(sum, off, 64);
        amax = max(amax, __shfl_down(amax, off, 64));
    }
    if (lane == 0) {
        sums[row] = sum;
        atomicMax(absmax, amax);
    }
}

VxHipStatus pack_weight(hipStream_t stream, const uint8_t* raw_dev, size_t row_stride, uint32_t n,
                        uint32_t k, bool flip, PackedWeight* out) {
    out->n = n;
    out->k = k;
    out->panels = ((n + kPanelRows - 1) / kPanelRows + kPanelPad - 1) / kPanelPad * kPanelPad;
    out->ksteps = ((k + kStepK - 1) / kStepK + kStepPad - 1) / kStepPad * kStepPad;
    VXHIP_TRY(hipMalloc((void**)&out->data, out->bytes()));
    const size_t slots = (size_t)out->panels * out->ksteps * 64u;
    const unsigned blocks = (unsigned)((slots + 255u) / 256u);
    hipLaunchKernelGGL(pack_weight_kernel, dim3(blocks), dim3(256), 0, stream, raw_dev, row_stride,
                       n, k, flip ? 1u : 0u, out->panels, out->ksteps, (uint8_t*)out->data);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus pack_weight_nibbles(hipStream_t stream, const uint32_t* raw_dev, uint32_t row_words,
                                uint32_t n, uint32_t k, uint32_t bits, PackedWeight* out) {
    out->n = n;
    out->k = k;
    out->bits = 4;
    out->panels = ((n + kPanelRows - 1) / kPanelRows + kPanelPad - 1) / kPanelPad * kPanelPad;
    const uint32_t steps = ((k + kStepK - 1) / kStepK + kStepPad - 1) / kStepPad * kStepPad;
    out->ksteps = steps / 2u;
    VXHIP_TRY(hipMalloc((void**)&out->data, out->bytes()));
    const size_t slots = (size_t)out->panels * out->ksteps * 64u;
    hipLaunchKernelGGL(pack_nibble_kernel, dim3((unsigned)((slots + 255u) / 256u)), dim3(256), 0, stream,
                       raw_dev, row_words, n, k, bits, out->panels, out->ksteps, (uint8_t*)out->data);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus weight_row_stats(hipStream_t stream, const uint8_t* raw_dev, size_t row_stride,
                             uint32_t n, uint32_t k, bool flip, const int32_t* zps,
                             int32_t* sums_dev, int32_t* absmax_dev) {
    VXHIP_TRY(hipMemsetAsync(absmax_dev, 0, sizeof(int32_t), stream));
    hipLaunchKernelGGL(weight_row_stats_kernel, dim3((n + 3u) / 4u), dim3(256), 0, stream, raw_dev,
                       row_stride, n, k, flip ? 1u : 0u, zps, sums_dev, absmax_dev);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

}  // namespace vxhip
