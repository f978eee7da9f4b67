// Fused epilogues shared by the MFMA GEMM and the streaming GEMV.
//
//  RequantTensor  canonical QLinear: one input scale / zero point per call
//                 (native/src/kernels/portable_inference_kernels.inc:1006-1028)
//  RequantRow     the same rule with one input scale per activation row
//  DequantF32     PackedLinear/DYNAMIC_I8 final step: running group sum + bias
//                 (native/src/kernels/packed_linear_ops.inc:1533)
#pragma once

#include "common.h"
#include "device_math.h"

namespace vxhip {

// Per-channel constants of the requantizing epilogue, derived inside the
// kernel from the compiled weight and the call's scalars (no helper launch):
//   f0    RequantTensor: mult[n] = f32(f32(s_in * s_w[n]) / s_out)
//         RequantRow:    s_w[n]
//   cb    bias[n] - zx * sum_k(ws[n][k]) + K * zx * zw[n]   (signed-byte domain)
//   bo    RequantRow: f32(bias_f32[n] / s_out), else 0
//   zw    weight zero point in the signed-byte domain
// so that  acc = dot(xs, ws) + cb - zw * sum_k(xs[m][k])  equals the reference's
// bias + sum (x - zx)(w - zw)  (portable_inference_kernels.inc:1010-1020).
// Integer arithmetic is modulo 2^32; the host has proved the true value fits.
struct ChannelConsts {
    float f0;
    int32_t cb;
    float bo;
    int32_t zw;
};

template <int MODE>
__device__ __forceinline__ ChannelConsts channel_consts(const LinearArgs& a, uint32_t n) {
    ChannelConsts c;
    const float sw = a.wscale[n];
    const int32_t zw = a.zw ? a.zw[n] : 0;
    c.zw = zw;
    c.bo = 0.0f;
    if constexpr (MODE == (int)Epilogue::RequantTensor) {
        c.f0 = requant_multiplier(a.input_scale, sw, a.output_scale);
        if (!scale_valid(c.f0) && n < a.n) atomicOr(a.fault, (uint32_t)kFaultBadMultiplier);
        const uint32_t t = (uint32_t)a.k * (uint32_t)zw - (uint32_t)a.wsum[n];
        c.cb = (int32_t)((uint32_t)a.bias_i32[n] + (uint32_t)a.input_zp * t);
    } else {
        c.f0 = sw;
        c.cb = a.bias_i32[n];
        if (a.bias_row && n < a.n) {
            const float b = a.bias_row[n];
            // a bias that is not finite is a bad descriptor (the CPU rule declines the call)
            if (!(fabsf(b) <= 3.402823466e38f)) atomicOr(a.fault, (uint32_t)kFaultBadBias);
            c.bo = __fdiv_rn(b, a.output_scale);
        }
    }
    return c;
}

// One requantized output element.
template <int MODE>
__device__ __forceinline__ int32_t requant_one(const LinearArgs& a, int32_t dot, const ChannelConsts& c,
                                               float row_scale, int32_t rsum, int32_t* total_out) {
    const int32_t total = (int32_t)((uint32_t)dot + (uint32_t)c.cb - (uint32_t)c.zw * (uint32_t)rsum);
    *total_out = total;
    float mu = c.f0;
    if constexpr (MODE == (int)Epilogue::RequantRow) {
        mu = requant_multiplier(row_scale, c.f0, a.output_scale);
        if (!scale_valid(mu)) atomicOr(a.fault, (uint32_t)kFaultBadMultiplier);
    }
    float t = transform_accumulator(total, mu, (float)a.out_zp);
    if constexpr (MODE == (int)Epilogue::RequantRow) {
        if (a.bias_row) t = __fadd_rn(t, c.bo);
    }
    return requantize(t, (float)a.out_lo, (float)a.out_hi, a.out_zp);
}

// The DequantizeLinear that reads a requantized value, applied where the value is made:
// f32((double)(q - zp) * (double)s) (native/src/kernels/quantize_linear_ops.inc:9-16).  q - zp has at
// most nine bits, so its product with an f32 is exact in double and rounds once: the single f32
// multiplication below gives the same bits.
__device__ __forceinline__ float dequantized(const LinearArgs& a, int32_t q) {
    return __fmul_rn((float)(q - a.dq_zp), a.dq_scale);
}

// One output element (split-K tail, where a thread owns one element).
template <int MODE>
__device__ __forceinline__ void store_element(const LinearArgs& a, uint32_t m, uint32_t n,
                                              int32_t dot, float fsum, float row_scale) {
    if (m >= a.rows || n >= a.n) return;
    if constexpr (MODE == (int)Epilogue::DequantF32) {
        ((float*)a.y)[(size_t)m * a.n + n] = __fadd_rn(fsum, a.bias_f32[n]);
    } else {
        const int32_t rsum = a.zw ? a.rowsum[m] : 0;
        const ChannelConsts c = channel_consts<MODE>(a, n);
        int32_t total;
        const int32_t q = requant_one<MODE>(a, dot, c, row_scale, rsum, &total);
        if (a.y) ((uint8_t*)a.y)[(size_t)m * a.n + n] = (uint8_t)q;
        if (a.acc_out) a.acc_out[(size_t)m * a.n + n] = total;
        if (a.dq_out) a.dq_out[(size_t)m * a.n + n] = dequantized(a, q);
    }
}

// Four consecutive channels n..n+3 of row m (the MFMA output quad of a lane);
// n is a multiple of 4.  Only the stores are guarded.
template <int MODE>
__device__ __forceinline__ void store_quad(const LinearArgs& a, uint32_t m, uint32_t n,
                                           const int32_t (&dot)[4], const float (&fsum)[4],
                                           float row_scale, int32_t rsum, const ChannelConsts (&cc)[4]) {
    if (m >= a.rows || n >= a.n) return;
    const bool vec_ok = (a.n % 4u) == 0u;  // then n..n+3 < a.n and the row start is aligned
    if constexpr (MODE == (int)Epilogue::DequantF32) {
        const v4f b = *reinterpret_cast<const v4f*>(a.bias_f32 + n);
        v4f out;
#pragma unroll
        for (int e = 0; e < 4; e++) out[e] = __fadd_rn(fsum[e], b[e]);
        float* y = (float*)a.y + (size_t)m * a.n + n;
        if (vec_ok) {
            *reinterpret_cast<v4f*>(y) = out;
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n + e < a.n) y[e] = out[e];
        }
    } else {
        int32_t total[4], q[4];
#pragma unroll
        for (int e = 0; e < 4; e++) q[e] = requant_one<MODE>(a, dot[e], cc[e], row_scale, rsum, &total[e]);
        if (a.y) {
            uint8_t* y = (uint8_t*)a.y + (size_t)m * a.n + n;
            if (vec_ok) {
                *reinterpret_cast<uint32_t*>(y) = pack4_bytes(q[0], q[1], q[2], q[3]);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < a.n) y[e] = (uint8_t)q[e];
            }
        }
        if (a.acc_out) {
            int32_t* ao = a.acc_out + (size_t)m * a.n + n;
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (n + e < a.n) ao[e] = total[e];
        }
        if (a.dq_out) {
            float* dq = a.dq_out + (size_t)m * a.n + n;
            if (vec_ok) {
                *reinterpret_cast<v4f*>(dq) = v4f{dequantized(a, q[0]), dequantized(a, q[1]), dequantized(a, q[2]),
                                                  dequantized(a, q[3])};
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (n + e < a.n) dq[e] = dequantized(a, q[e]);
            }
        }
    }
}

}  // namespace vxhip
