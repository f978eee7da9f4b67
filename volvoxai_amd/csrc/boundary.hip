// Kernels on either side of the linear: activation staging, PackedLinear's
// dynamic activation quantization
// and the QuantizeLinear / DequantizeLinear boundaries.  All HBM-bound
// elementwise or per-row work.
#include "common.h"
#include "device_math.h"
#include "wave_ops.h"

namespace vxhip {

// ---- activation staging -----------------------------------------------------
// Copies raw I8/U8 rows into a 16-byte aligned, zero padded signed buffer and
// writes each row's sum of signed bytes (the operand-sum term of the
// zero-point fold, cf. native/src/kernels/qlinear_vnni_kernel.inc:113-116).
// One wavefront per row.
__global__ __launch_bounds__(256) void stage_activations_kernel(
        const uint8_t* __restrict__ x, uint32_t rows, uint32_t k, uint32_t flip,
        int8_t* __restrict__ staged, uint32_t ld, int32_t* __restrict__ rowsum) {
    const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63u;
    if (row >= rows) return;
    const uint8_t* src = x + (size_t)row * k;
    int32_t sum = 0;
    for (uint32_t kk = lane; kk < ld; kk += 64u) {
        int8_t v = 0;
        if (kk < k) v = (int8_t)(src[kk] ^ (flip ? 0x80u : 0u));
        sum += v;
        if (staged) staged[(size_t)row * ld + kk] = v;
    }
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_down(sum, off, 64);
    if (lane == 0 && rowsum) rowsum[row] = sum;
}

VxHipStatus launch_stage_activations(hipStream_t s, const void* x, uint32_t rows, uint32_t k,
                                     bool flip, int8_t* staged, uint32_t ld, int32_t* rowsum) {
    hipLaunchKernelGGL(stage_activations_kernel, dim3((rows + 3u) / 4u), dim3(256), 0, s,
                       (const uint8_t*)x, rows, k, flip ? 1u : 0u, staged, ld, rowsum);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

// ---- PackedLinear activation preparation ------------------------------------
// One workgroup per row (native/src/kernels/packed_linear_ops.inc:1574-1597):
//   scale = max|x| / 127 (1.0 for an all-zero row, floored at 2^-126),
//   code  = ties-to-even(x / scale) clamped to +-127, with a true f32 divide
//   (multiplying by a reciprocal moves half-way values, ibid. :34-36).
// A row holding NaN or Inf gets zero codes and a NaN scale, which makes every
// output of that row NaN downstream as the reference requires (:1495).
__global__ __launch_bounds__(1024) void prepare_i8_kernel(
        const float* __restrict__ x, uint32_t k, int8_t* __restrict__ prepared, const ActivationLayout layout,
        float* __restrict__ scales) {
    const uint32_t ld = layout.ld;
    __shared__ float slot_max[16];
    __shared__ uint32_t slot_bad[16];
    const uint32_t row = blockIdx.x;
    const float* src = x + (size_t)row * k;
    float maximum = 0.0f;
    uint32_t bad = 0u;
    // a thread's first elements stay in registers for the second pass (rows of up to 4096 at
    // 1024 threads are then read once)
    constexpr int kKept = 4;
    float kept[kKept];
#pragma unroll
    for (int i = 0; i < kKept; i++) {
        const uint32_t j = threadIdx.x + i * blockDim.x;
        kept[i] = j < k ? src[j] : 0.0f;
        bad |= finite_f32(kept[i]) ? 0u : 1u;
        maximum = fmaxf(maximum, fabsf(kept[i]));  // fmaxf ignores a NaN operand; `bad` records it
    }
    for (uint32_t j = threadIdx.x + kKept * blockDim.x; j < k; j += blockDim.x) {
        const float v = src[j];
        bad |= finite_f32(v) ? 0u : 1u;
        maximum = fmaxf(maximum, fabsf(v));
    }
    maximum = wave_max(maximum);
    bad = __builtin_amdgcn_ballot_w64(bad != 0u) != 0ull ? 1u : 0u;
    if ((threadIdx.x & 63u) == 0u) {
        slot_max[threadIdx.x >> 6] = maximum;
        slot_bad[threadIdx.x >> 6] = bad;
    }
    __syncthreads();
    maximum = slot_max[0];
    bad = slot_bad[0];
    for (uint32_t w = 1; w < blockDim.x / 64u; w++) {
        maximum = fmaxf(maximum, slot_max[w]);
        bad |= slot_bad[w];
    }
    float scale = maximum == 0.0f ? 1.0f : __fdiv_rn(maximum, 127.0f);
    if (scale < 0x1p-126f) scale = 0x1p-126f;
#pragma unroll
    for (int i = 0; i < kKept; i++) {
        const uint32_t j = threadIdx.x + i * blockDim.x;
        if (j < ld)
            prepared[activation_offset(layout, row, j)] =
                (int8_t)(!bad && j < k ? packed_round_i8(__fdiv_rn(kept[i], scale)) : 0);
    }
    for (uint32_t j = threadIdx.x + kKept * blockDim.x; j < ld; j += blockDim.x) {
        int32_t q = 0;
        if (!bad && j < k) q = packed_round_i8(__fdiv_rn(src[j], scale));
        prepared[activation_offset(layout, row, j)] = (int8_t)q;
    }
    if (threadIdx.x == 0) scales[row] = bad ? __builtin_nanf("") : scale;
}

// The same rule for many rows in row-major layout (k % 4 == 0, 16-byte aligned rows): a workgroup
// per row, 16 bytes per lane and load, four codes per store, and the whole row kept in registers
// between the two passes when it has at most 256 * 4 * kKeptChunks elements -- the row is then read
// from HBM once and the kernel runs at the speed of that read.
template <int kKeptChunks>
__global__ __launch_bounds__(256) void prepare_i8_rows_kernel(const float* __restrict__ x, uint32_t k,
                                                              int8_t* __restrict__ prepared, uint32_t ld,
                                                              float* __restrict__ scales) {
    __shared__ float slot_max[4];
    __shared__ uint32_t slot_bad[4];
    const uint32_t row = blockIdx.x;
    const v4f* src = reinterpret_cast<const v4f*>(x + (size_t)row * k);
    const uint32_t chunks = k / 4u;
    float maximum = 0.0f;
    uint32_t bad = 0u;
    v4f kept[kKeptChunks];
#pragma unroll
    for (int i = 0; i < kKeptChunks; i++) {
        const uint32_t c = threadIdx.x + i * 256u;
        kept[i] = c < chunks ? __builtin_nontemporal_load(src + c) : v4f{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < kKeptChunks; i++) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            bad |= finite_f32(kept[i][e]) ? 0u : 1u;
            maximum = fmaxf(maximum, fabsf(kept[i][e]));  // fmaxf ignores a NaN operand; `bad` records it
        }
    }
    for (uint32_t c = threadIdx.x + kKeptChunks * 256u; c < chunks; c += 256u) {
        const v4f v = src[c];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            bad |= finite_f32(v[e]) ? 0u : 1u;
            maximum = fmaxf(maximum, fabsf(v[e]));
        }
    }
    maximum = wave_max(maximum);
    bad = __builtin_amdgcn_ballot_w64(bad != 0u) != 0ull ? 1u : 0u;
    if ((threadIdx.x & 63u) == 0u) {
        slot_max[threadIdx.x >> 6] = maximum;
        slot_bad[threadIdx.x >> 6] = bad;
    }
    __syncthreads();
    maximum = fmaxf(fmaxf(slot_max[0], slot_max[1]), fmaxf(slot_max[2], slot_max[3]));
    bad = slot_bad[0] | slot_bad[1] | slot_bad[2] | slot_bad[3];
    float scale = maximum == 0.0f ? 1.0f : __fdiv_rn(maximum, 127.0f);
    if (scale < 0x1p-126f) scale = 0x1p-126f;
    uint32_t* dst = reinterpret_cast<uint32_t*>(prepared + (size_t)row * ld);
    auto codes = [&](const v4f v) {
        if (bad) return 0u;
        return pack4_bytes(packed_round_i8(__fdiv_rn(v[0], scale)), packed_round_i8(__fdiv_rn(v[1], scale)),
                           packed_round_i8(__fdiv_rn(v[2], scale)), packed_round_i8(__fdiv_rn(v[3], scale)));
    };
#pragma unroll
    for (int i = 0; i < kKeptChunks; i++) {
        const uint32_t c = threadIdx.x + i * 256u;
        if (c < chunks) dst[c] = codes(kept[i]);
    }
    for (uint32_t c = threadIdx.x + kKeptChunks * 256u; c < chunks; c += 256u) dst[c] = codes(src[c]);
    for (uint32_t c = chunks + threadIdx.x; c < ld / 4u; c += 256u) dst[c] = 0u;  // the padding of the row
    if (threadIdx.x == 0) scales[row] = bad ? __builtin_nanf("") : scale;
}

VxHipStatus launch_prepare_i8(hipStream_t s, const float* x, uint32_t rows, uint32_t k,
                              int8_t* prepared, ActivationLayout layout, float* scales) {
    // (operand order has room for 32 rows, and its rows are whole 16-byte chunks)
    if (layout.operand_order && (rows > kOperandOrderRows || layout.ld != (k + 15u) / 16u * 16u))
        return VXHIP_INVALID_ARGUMENT;
    // many rows: the vectorized kernel (rows that fit its registers are read once)
    if (!layout.operand_order && rows > 64u && (k % 4u) == 0u && (layout.ld % 4u) == 0u && ((uintptr_t)x % 16u) == 0u &&
        ((uintptr_t)prepared % 4u) == 0u) {
        if (k <= 4096u)
            hipLaunchKernelGGL(prepare_i8_rows_kernel<4>, dim3(rows), dim3(256), 0, s, x, k, prepared, layout.ld, scales);
        else
            hipLaunchKernelGGL(prepare_i8_rows_kernel<14>, dim3(rows), dim3(256), 0, s, x, k, prepared, layout.ld, scales);
        VXHIP_TRY(hipGetLastError());
        return VXHIP_OK;
    }
    // few long rows: latency bound, give each row a full workgroup
    const uint32_t block = rows <= 256u && k >= 1024u ? 1024u : 256u;
    hipLaunchKernelGGL(prepare_i8_kernel, dim3(rows), dim3(block), 0, s, x, k, prepared, layout, scales);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

// one thread per 16-byte chunk of a row
__global__ __launch_bounds__(256) void unblock_activations_kernel(const int8_t* __restrict__ blocked,
                                                                  uint32_t rows, uint32_t chunks,
                                                                  int8_t* __restrict__ row_major, uint32_t ld) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= rows * chunks) return;
    const uint32_t row = i / chunks, chunk = i % chunks;
    *reinterpret_cast<uint4*>(row_major + (size_t)row * ld + chunk * 16u) =
        *reinterpret_cast<const uint4*>(blocked + ((size_t)chunk * kOperandOrderRows + row) * 16u);
}

VxHipStatus launch_unblock_activations(hipStream_t s, const int8_t* blocked, uint32_t rows, uint32_t k,
                                       int8_t* row_major, uint32_t ld) {
    const uint32_t chunks = (k + 15u) / 16u;
    if (rows > kOperandOrderRows || ld < chunks * 16u || (ld % 16u) != 0u || ((uintptr_t)blocked % 16u) != 0u ||
        ((uintptr_t)row_major % 16u) != 0u)
        return VXHIP_INVALID_ARGUMENT;
    if (!rows) return VXHIP_OK;
    hipLaunchKernelGGL(unblock_activations_kernel, dim3((rows * chunks + 255u) / 256u), dim3(256), 0, s, blocked,
                       rows, chunks, row_major, ld);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* p, uint32_t count, uint32_t value) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] = value;
}

VxHipStatus launch_fill_u32(hipStream_t s, uint32_t* p, uint32_t count, uint32_t value) {
    if (!count) return VXHIP_OK;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((count + 255u) / 256u), dim3(256), 0, s, p, count, value);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

// ---- exactness proof of the short division ------------------------------------
// Division by a fixed divisor scales exactly with the dividend's exponent (as long as nothing
// leaves the normal range), so trying all 2^23 mantissas at one exponent decides it for every
// dividend.  Thread t checks mantissas 4t .. 4t+3.
__global__ __launch_bounds__(256) void division_proof_kernel(float s, float r, uint32_t* counters) {
    const uint32_t t = blockIdx.x * 256u + threadIdx.x;
    uint32_t bad1 = 0, bad2 = 0;
#pragma unroll
    for (uint32_t i = 0; i < 4; i++) {
        const float p = __uint_as_float(0x3f800000u | (t * 4u + i));
        const float want = __fdiv_rn(p, s);
        bad1 += div_by_uniform_once(p, s, r) != want;
        bad2 += div_by_uniform(p, s, r) != want;
    }
    if (bad1) atomicAdd(counters, bad1);
    if (bad2) atomicAdd(counters + 1, bad2);
}

VxHipStatus launch_division_proof(hipStream_t s, float divisor, float recip, uint32_t* counters) {
    VxHipStatus st = launch_fill_u32(s, counters, 2, 0);
    if (st != VXHIP_OK) return st;
    hipLaunchKernelGGL(division_proof_kernel, dim3((1u << 23) / 4u / 256u), dim3(256), 0, s, divisor, recip,
                       counters);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

// ---- QuantizeLinear / DequantizeLinear --------------------------------------
// q = saturate(ties-to-even(f32(x / s) + f32(zp))); NaN -> zp; +-Inf saturate
// (native/src/kernels/quantize_linear_ops.inc:156-169).
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ x, uint32_t n,
                                                       uint8_t* __restrict__ y, float scale,
                                                       int32_t zp, int32_t lo, int32_t hi) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    int32_t q;
    if (v != v) {
        q = zp;
    } else {
        const float t = __fadd_rn(__fdiv_rn(v, scale), (float)zp);
        if (t <= (float)lo) q = lo;
        else if (t >= (float)hi) q = hi;
        else q = (int32_t)__builtin_rintf(t);
    }
    y[i] = (uint8_t)q;
}

// y = f32((double)(q - zp) * (double)s)   (quantize_linear_ops.inc:9-16)
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ x, uint32_t n,
                                                         float scale, int32_t zp, uint32_t is_i8,
                                                         float* __restrict__ y) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int32_t q = is_i8 ? (int32_t)(int8_t)x[i] : (int32_t)x[i];
    y[i] = (float)((double)(q - zp) * (double)scale);
}

// RequantizeLinear: q' = saturate(ties-to-even(f32(f32(f32(q - zp_in) * m) + f32(zp_out)))), m = f32(s_in / s_out)
// formed by the host (native/src/kernels/portable_inference_kernels.inc:2437-2463); 16 bytes per thread
// where the tensors allow it.
__device__ __forceinline__ uint32_t requantize_byte(uint32_t byte, uint32_t in_i8, int32_t zp_in, float m, float zp_out_f,
                                                    float lo_f, float hi_f) {
    const int32_t q = in_i8 ? (int32_t)(int8_t)byte : (int32_t)byte;
    const float t = __fadd_rn(__fmul_rn((float)(q - zp_in), m), zp_out_f);
    // (t is finite: a byte difference times a finite multiplier plus a byte)
    return (uint32_t)(int32_t)__builtin_rintf(fminf(fmaxf(t, lo_f), hi_f)) & 255u;
}
__global__ __launch_bounds__(256) void requantize_kernel(const uint8_t* __restrict__ x, uint32_t n, uint8_t* __restrict__ y,
                                                         float m, int32_t zp_in, int32_t zp_out, uint32_t in_i8,
                                                         uint32_t out_i8, uint32_t vectors) {
    const float zp_out_f = (float)zp_out, lo_f = out_i8 ? -128.0f : 0.0f, hi_f = out_i8 ? 127.0f : 255.0f;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < vectors) {
        const uint4 v = reinterpret_cast<const uint4*>(x)[i];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        uint32_t o[4];
#pragma unroll
        for (int d = 0; d < 4; d++) {
            o[d] = 0u;
#pragma unroll
            for (int b = 0; b < 4; b++)
                o[d] |= requantize_byte((w[d] >> (8 * b)) & 255u, in_i8, zp_in, m, zp_out_f, lo_f, hi_f) << (8 * b);
        }
        reinterpret_cast<uint4*>(y)[i] = make_uint4(o[0], o[1], o[2], o[3]);
    } else {
        const uint32_t e = vectors * 16u + (i - vectors);  // the tail (or everything, for unaligned tensors) byte by byte
        if (e < n) y[e] = (uint8_t)requantize_byte(x[e], in_i8, zp_in, m, zp_out_f, lo_f, hi_f);
    }
}

VxHipStatus launch_requantize(hipStream_t s, const void* x, uint32_t n, void* y, float multiplier, int32_t zp_in,
                              int32_t zp_out, bool in_i8, bool out_i8) {
    if (!n) return VXHIP_OK;
    const bool aligned = ((uintptr_t)x % 16u) == 0u && ((uintptr_t)y % 16u) == 0u;
    const uint32_t vectors = aligned ? n / 16u : 0u;
    const uint32_t threads = vectors + (n - vectors * 16u);
    hipLaunchKernelGGL(requantize_kernel, dim3((threads + 255u) / 256u), dim3(256), 0, s, (const uint8_t*)x, n,
                       (uint8_t*)y, multiplier, zp_in, zp_out, in_i8 ? 1u : 0u, out_i8 ? 1u : 0u, vectors);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus launch_quantize(hipStream_t s, const float* x, uint32_t n, void* y, float scale,
                            int32_t zp, bool is_i8) {
    if (!n) return VXHIP_OK;
    hipLaunchKernelGGL(quantize_kernel, dim3((n + 255u) / 256u), dim3(256), 0, s, x, n,
                       (uint8_t*)y, scale, zp, is_i8 ? -128 : 0, is_i8 ? 127 : 255);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus launch_dequantize(hipStream_t s, const void* x, uint32_t n, float scale, int32_t zp,
                              bool is_i8, float* y) {
    if (!n) return VXHIP_OK;
    hipLaunchKernelGGL(dequantize_kernel, dim3((n + 255u) / 256u), dim3(256), 0, s,
                       (const uint8_t*)x, n, scale, zp, is_i8 ? 1u : 0u, y);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

}  // namespace vxhip
