// Bandwidth-bound W8A8 linear for decode-shaped M <= 16.  Every weight byte is
// read exactly once, straight from HBM into MFMA operand registers with
// coalesced dwordx4 loads (no LDS hop), and multiplied against all M rows at
// once on v_mfma_i32_16x16x64_i8, whose internal reduction replaces the
// cross-lane dot-product reduce.  The GPU counterpart of the reference's
// single-row route vx_packed_linear_single_row_range
// (native/src/kernels/packed_linear_ops.inc:1471-1535) and of its M=1 QLinear
// route (native/src/kernels/qlinear_vnni_kernel.inc:41-127).
//
// Work unit: 16 output channels.  A wavefront streams a unit's weights over a
// K range in steps of 64: lane l supplies the weight operand row l%16, k-chunk
// l/16 (one dwordx4 from the packed layout) and the activation operand row
// min(l%16, M-1), same k-chunk (one dwordx4 from the row-major activations,
// L2-resident).  After a step the lane holds the partial dots of channels
// 4*(l/16)+0..3 for row l%16.
//
// Split-K: with few units (small N) the waves of a workgroup share one unit
// and split K.  Integer partials add exactly; the f32 group terms of the
// dequantizing epilogue are parked in LDS and summed in ascending group order
// by one thread per output, which keeps the result bit-identical to the serial
// order the reference uses (packed_linear_ops.inc:1498-1504).
#include "common.h"
#include "device_math.h"
#include "epilogue.h"

#include <stdio.h>
#include <string.h>

namespace vxhip {

namespace {

extern __shared__ __attribute__((aligned(16))) char gemv_lds[];

constexpr int kDepth = 8;  // k64 steps in flight per wave (8 KiB of weights)

// MODE: Epilogue.  GK: k64 steps per scale group (1, 2, 4) or 0 for G=32 (two
// groups per step).  SK: waves of the workgroup sharing one unit (1 or 4).
template <int MODE, int GK, int SK>
__global__ __launch_bounds__(256) void gemv_stream_kernel(const LinearArgs a) {
    constexpr bool F = MODE == (int)Epilogue::DequantF32;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const uint32_t units = (a.n + 15u) / 16u;
    const uint32_t unit = SK == 1 ? blockIdx.x * 4u + wave : blockIdx.x;
    const bool active = unit < units;  // inactive waves still reach every barrier

    const uint32_t steps = (a.k + 63u) / 64u;  // k64 steps that hold real k
    // K range of this wave, aligned to whole groups
    uint32_t t0 = 0, t1 = steps;
    if constexpr (SK > 1) {
        constexpr uint32_t align = GK > 0 ? GK : 1;
        const uint32_t chunks = (steps + align - 1) / align;
        const uint32_t per = (chunks + SK - 1) / SK;
        t0 = min(wave * per * align, steps);
        t1 = min((wave + 1) * per * align, steps);
    }
    if (!active) t1 = t0;

    const uint32_t r16 = lane & 15, c = lane >> 4;
    const uint32_t panel = unit >> 1, half = unit & 1u;
    // weight operand: 32-row panel blocks of 1 KiB per 32 k; this lane's slot
    const int8_t* wp = a.w + ((size_t)panel * a.ksteps + (c >> 1)) * 1024u +
                       (half * 16u + r16 + 32u * (c & 1u)) * 16u;
    const uint32_t m = min(r16, a.rows - 1u);
    const int8_t* xp = a.x + (size_t)m * a.ldx;
    const uint32_t last_chunk = (a.k - 1u) / 16u;
    const uint32_t nq = unit * 16u + c * 4u;  // first of the lane's four channels

    float row_scale = 0.0f;
    if constexpr (MODE != (int)Epilogue::RequantTensor) row_scale = a.row_scale[m];

    v4i wbuf[kDepth], xbuf[kDepth];
    v4f sbuf[kDepth][GK == 0 ? 2 : 1];
    auto issue = [&](int slot, uint32_t t) {
        wbuf[slot] = *reinterpret_cast<const v4i*>(wp + (size_t)t * 2048u);
        const uint32_t chunk = min(t * 4u + c, last_chunk);
        xbuf[slot] = *reinterpret_cast<const v4i*>(xp + chunk * 16u);
        if constexpr (F) {
            if constexpr (GK == 0) {
                const uint32_t g = min(t * 2u, a.groups - 1u), g1 = min(t * 2u + 1u, a.groups - 1u);
                sbuf[slot][0] = *reinterpret_cast<const v4f*>(a.scales_t + (size_t)g * a.n_pad + nq);
                sbuf[slot][1] = *reinterpret_cast<const v4f*>(a.scales_t + (size_t)g1 * a.n_pad + nq);
            } else if (slot % GK == GK - 1 || t + 1 == t1) {
                // the scale rides in the slot of the step that closes the group, which is
                // not refilled until that step's fold has read it
                const uint32_t g = min(t / GK, a.groups - 1u);
                sbuf[slot][0] = *reinterpret_cast<const v4f*>(a.scales_t + (size_t)g * a.n_pad + nq);
            }
        }
    };

    v4i acc = {0, 0, 0, 0};
    float fsum[4] = {0.f, 0.f, 0.f, 0.f};
    float* terms = reinterpret_cast<float*>(gemv_lds);  // [groups][256], split-K dequant only

    // sum += f32(dot) * (s_a * s_w[n][g])  -- or park the term for the ordered tail
    auto fold = [&](const v4i& dots, const v4f& sw, uint32_t g) {
        if constexpr (F) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float term = __fmul_rn((float)dots[e], __fmul_rn(row_scale, sw[e]));
                if constexpr (SK == 1) fsum[e] = __fadd_rn(fsum[e], term);
                else if (g < a.groups) terms[(size_t)g * 256u + lane * 4 + e] = term;
            }
        }
    };

#pragma unroll
    for (int i = 0; i < kDepth; i++)
        if (t0 + i < t1) issue(i, t0 + i);

    for (uint32_t t = t0; t < t1; t += kDepth) {
#pragma unroll
        for (int i = 0; i < kDepth; i++) {
            if (t + i < t1) {
                if constexpr (F && GK == 0) {
                    // two 32-wide groups per step: mask the other half of k
                    v4i lo = xbuf[i], hi = xbuf[i];
                    if (c >= 2) lo = v4i{0, 0, 0, 0}; else hi = v4i{0, 0, 0, 0};
                    const v4i z = {0, 0, 0, 0};
                    v4i d0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wbuf[i], lo, z, 0, 0, 0);
                    v4i d1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(wbuf[i], hi, z, 0, 0, 0);
                    fold(d0, sbuf[i][0], (t + i) * 2u);
                    fold(d1, sbuf[i][1], (t + i) * 2u + 1u);
                } else {
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wbuf[i], xbuf[i], acc, 0, 0, 0);
                    if constexpr (F) {
                        // group closes after GK steps (t0 is group aligned) or at the row end
                        if ((i + 1) % GK == 0 || t + i + 1 == t1) {
                            fold(acc, sbuf[i][0], (t + i) / GK);
                            acc = v4i{0, 0, 0, 0};
                        }
                    }
                }
                if (t + i + kDepth < t1) issue(i, t + i + kDepth);
            }
        }
    }

    if constexpr (SK == 1) {
        if (!active) return;
        int32_t dot[4] = {acc[0], acc[1], acc[2], acc[3]};
        int32_t rsum = 0;
        if constexpr (MODE != (int)Epilogue::DequantF32) {
            if (a.zw) rsum = a.rowsum[m];
        }
        ChannelConsts cc[4];
        if constexpr (!F) {
#pragma unroll
            for (int e = 0; e < 4; e++) cc[e] = channel_consts<MODE>(a, nq + e);
        }
        if (r16 < a.rows) store_quad<MODE>(a, r16, nq, dot, fsum, row_scale, rsum, cc);
    } else {
        // element e of lane l sits at index 4*l+e; thread tid finishes index tid
        int32_t* parts = reinterpret_cast<int32_t*>(gemv_lds);  // [SK][256], requant only
        if constexpr (!F) {
#pragma unroll
            for (int e = 0; e < 4; e++) parts[wave * 256 + lane * 4 + e] = acc[e];
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __syncthreads();
        if (!active) return;
        const uint32_t tid = threadIdx.x;
        const uint32_t l = tid >> 2, e = tid & 3u;
        const uint32_t om = l & 15u, on = unit * 16u + (l >> 4) * 4u + e;
        float rs = 0.0f;
        if constexpr (MODE != (int)Epilogue::RequantTensor) rs = a.row_scale[min(om, a.rows - 1u)];
        if constexpr (F) {
            float sum = 0.0f;
            for (uint32_t g = 0; g < a.groups; g++) sum = __fadd_rn(sum, terms[(size_t)g * 256u + tid]);
            store_element<MODE>(a, om, on, 0, sum, rs);
        } else {
            int32_t dot = 0;
#pragma unroll
            for (int w = 0; w < SK; w++) dot += parts[w * 256 + tid];
            store_element<MODE>(a, om, on, dot, 0.0f, rs);
        }
    }
}

template <int MODE, int GK>
const char* launch_mode(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    const uint32_t units = (a.n + 15u) / 16u;
    bool split = units < (uint32_t)cu_count * 4u;  // fewer than four waves per CU otherwise
    if (force && strstr(force, "splitk")) split = true;
    if (force && strstr(force, "stream")) split = false;
    size_t lds = 0;
    if (split) {
        lds = MODE == (int)Epilogue::DequantF32 ? (size_t)a.groups * 1024u : 4u * 1024u;
        if (lds > 64u * 1024u) split = false;
    }
    if (split) {
        hipLaunchKernelGGL((gemv_stream_kernel<MODE, GK, 4>), dim3(units), dim3(256), lds, s, a);
        return hipGetLastError() == hipSuccess ? "splitk4" : nullptr;
    }
    hipLaunchKernelGGL((gemv_stream_kernel<MODE, GK, 1>), dim3((units + 3u) / 4u), dim3(256), 0, s, a);
    return hipGetLastError() == hipSuccess ? "stream" : nullptr;
}

}  // namespace

const char* launch_gemv_stream(hipStream_t s, const LinearArgs& a, int cu_count, const char* force) {
    if (a.rows == 0u || a.rows > kMaxGemvRows || a.ldx < 16u || (a.ldx % 16u) != 0u ||
        ((uintptr_t)a.x % 16u) != 0u)
        return nullptr;
    const char* kind = nullptr;
    const char* family = nullptr;
    switch (a.mode) {
        case Epilogue::RequantTensor:
            family = "hip.qlinear.gemv-mfma16";
            kind = launch_mode<(int)Epilogue::RequantTensor, 1>(s, a, cu_count, force);
            break;
        case Epilogue::RequantRow:
            family = "hip.qlinear.gemv-mfma16-rowscale";
            kind = launch_mode<(int)Epilogue::RequantRow, 1>(s, a, cu_count, force);
            break;
        case Epilogue::DequantF32:
            family = "hip.packed-linear.a8-gemv-mfma16";
            switch (a.group_size) {
                case 32: kind = launch_mode<(int)Epilogue::DequantF32, 0>(s, a, cu_count, force); break;
                case 64: kind = launch_mode<(int)Epilogue::DequantF32, 1>(s, a, cu_count, force); break;
                case 128: kind = launch_mode<(int)Epilogue::DequantF32, 2>(s, a, cu_count, force); break;
                case 256: kind = launch_mode<(int)Epilogue::DequantF32, 4>(s, a, cu_count, force); break;
                default: return nullptr;
            }
            break;
    }
    if (!kind) return nullptr;
    static thread_local char name[96];
    snprintf(name, sizeof name, "%s.%s", family, kind);
    return name;
}

}  // namespace vxhip
