// Device-side scalar rules of the W8A8 contract.  Every f32 operation that the
// reference rounds separately is written with an explicit round-to-nearest
// intrinsic, so the compiler can neither contract a multiply-add into an FMA
// nor reassociate: a fused value can cross a ties-to-even boundary and change
// the output byte (reference: native/src/kernels/w8a8_affine.h:133-144).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vxhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// A store of output that nothing in the launch reads again, for launches whose whole output would
// otherwise sit dirty in the L2s until the kernel ends and leave in one burst behind the last wave
// (`streamed`, uniform over the launch): it then goes out while the kernel still runs.  Measured on the
// 256 x 256 requantizing tile at K=N=4096: 3072 / 4096 / 6144 / 8192 rows 0.5-1.3 us faster, 16384 rows the
// same, 2048 rows and fewer 0.4 us slower (their stores cover half lines, which the L2 otherwise merges).
// (STREAMED is a compile-time tag: under a run-time condition the compiler folds the two stores into a plain one)
template <bool STREAMED, class T>
__device__ __forceinline__ void store_stream(T* p, const T& v) {
    if constexpr (STREAMED) __builtin_nontemporal_store(v, p);
    else *p = v;
}

__device__ __forceinline__ bool scale_valid(float v) {
    // finite and strictly positive (w8a8_affine.h:63-65)
    return v > 0.0f && v < __builtin_inff();
}

// multiplier = f32(f32(s_in * s_w) / s_out)   (w8a8_affine.h:155-181)
__device__ __forceinline__ float requant_multiplier(float s_in, float s_w, float s_out) {
    return __fdiv_rn(__fmul_rn(s_in, s_w), s_out);
}

// p / s for a divisor that is the same for the whole launch, given r = RN(1/s)
// from the host.  Two Newton corrections with exact FMA residuals: after the
// first the quotient is faithful, and Markstein's theorem then makes the second
// the correctly rounded quotient, i.e. the same bits as an IEEE division -- as
// long as nothing under- or overflows, which fast_div_in_range() guarantees.
// Five full-rate operations instead of the ~11 of the generic divide sequence.
__device__ __forceinline__ float div_by_uniform(float p, float s, float r) {
    float q = __fmul_rn(p, r);
    float e = __fmaf_rn(-q, s, p);
    q = __fmaf_rn(e, r, q);
    e = __fmaf_rn(-q, s, p);
    return __fmaf_rn(e, r, q);
}

// The same with one correction.  Markstein's theorem makes it exact whenever the first product
// is already faithful; callers use it only for divisors where launch_division_proof counted no
// mismatch over all dividend mantissas.
__device__ __forceinline__ float div_by_uniform_once(float p, float s, float r) {
    const float q = __fmul_rn(p, r);
    const float e = __fmaf_rn(-q, s, p);
    return __fmaf_rn(e, r, q);
}

// Operands between 2^-60 and 2^60 keep every intermediate of div_by_uniform a
// normal number (quotient within 2^+-120, residuals 2^-24 below the operands).
__device__ __forceinline__ bool fast_div_in_range(float v) {
    return v >= 0x1p-60f && v <= 0x1p60f;
}

// t = f32(f32(acc) * mult) + f32(zp)          (w8a8_affine.h:139-144)
__device__ __forceinline__ float transform_accumulator(int32_t acc, float mult, float zp_f) {
    return __fadd_rn(__fmul_rn((float)acc, mult), zp_f);
}

// Saturating ties-to-even round into [lo, hi]; NaN maps to the zero point
// (w8a8_affine.h:114-131).  v_rndne_f32 is ties-to-even and equals the
// reference's floor-based rule for every value strictly inside the range.
__device__ __forceinline__ int32_t requantize(float t, float lo_f, float hi_f, int32_t zp) {
    if (t != t) return zp;
    float c = fminf(fmaxf(t, lo_f), hi_f);
    return (int32_t)__builtin_rintf(c);
}

// PackedLinear activation code: ties-to-even, clamped to +-127
// (packed_linear.h:108-116).
__device__ __forceinline__ int32_t packed_round_i8(float v) {
    float c = fminf(fmaxf(v, -127.0f), 127.0f);
    return (int32_t)__builtin_rintf(c);
}

__device__ __forceinline__ bool finite_f32(float v) {
    return (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u;
}

__device__ __forceinline__ uint32_t pack4_bytes(int32_t a, int32_t b, int32_t c, int32_t d) {
    return (uint32_t)(a & 255) | ((uint32_t)(b & 255) << 8) | ((uint32_t)(c & 255) << 16) |
           ((uint32_t)(d & 255) << 24);
}

}  // namespace vxhip
