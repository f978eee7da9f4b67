// The element rules of the row operations in front of a decoder's linears, shared by the row kernels
// (decoder_glue.hip) and by the streaming linear when it carries such an operation in its own
// prologue (gemv_stream.hip), so that both give the same bits.
#ifndef VXHIP_ROW_MATH_H
#define VXHIP_ROW_MATH_H

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

namespace vxhip {

// RMSNorm in double, rounded to f32 once per element: y = f32(x * (1 / sqrt(mean(x^2) + eps)) * gain).
// `total` is the row's sum of squares in the order of rmsnorm_prepare_kernel: a thread of a 1024-thread
// workgroup adds its elements in ascending order, a wavefront its 64 lanes as a shuffle-down tree, the
// workgroup its wavefronts in ascending order.
constexpr uint32_t kNormThreads = 1024;
__device__ __forceinline__ double rms_inverse(double total, uint32_t d, double eps) {
    const double var = total / (double)d;
    return 1.0 / sqrt(var + eps);
}
__device__ __forceinline__ float rms_scaled(float v, double inv_std, float gain) {
    return (float)((double)v * inv_std * (double)gain);
}

// SwiGLU: silu(gate) * up with silu(g) = g / (1 + exp(-g)), every step rounded to f32.
__device__ __forceinline__ float swiglu_value(float gate, float up) {
    const float s = __fdiv_rn(gate, __fadd_rn(1.0f, expf(-gate)));
    return __fmul_rn(s, up);
}

}  // namespace vxhip
#endif
