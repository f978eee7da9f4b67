// Wavefront reductions whose lane exchanges stay in the register file.
//
// A shuffle (`__shfl_*`) goes through the LDS crossbar: a round trip of ~100 cycles, and the six of
// a 64-lane tree depend on each other.  Inside a row of 16 lanes a data-parallel-primitive (DPP)
// move does the same exchange in the vector ALU.  The row-sized kernels of a decoder layer are
// latency bound and hold one or two such trees each.
//
// Every lane of the wavefront must be active when these are called.
#ifndef VXHIP_WAVE_OPS_H
#define VXHIP_WAVE_OPS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vxhip {

// DPP controls: quad permutes [1,0,3,2] and [2,3,0,1] (lane^1, lane^2), the mirror of each eight
// and of each sixteen lanes, and row_shl:n (lane i takes lane i+n of its row, 0 past the row end).
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140;
constexpr int kDppRowShl = 0x100;

template <int CTRL>
__device__ __forceinline__ int lane_exchange(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float lane_exchange(float v) {
    return __builtin_bit_cast(float, lane_exchange<CTRL>(__builtin_bit_cast(int, v)));
}
template <int CTRL>
__device__ __forceinline__ double lane_exchange(double v) {
    const uint64_t bits = __builtin_bit_cast(uint64_t, v);
    const uint32_t lo = (uint32_t)lane_exchange<CTRL>((int)(uint32_t)bits);
    const uint32_t hi = (uint32_t)lane_exchange<CTRL>((int)(uint32_t)(bits >> 32));
    return __builtin_bit_cast(double, ((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// fmaxf over the 64 lanes, in every lane (the order of a maximum does not matter).
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, lane_exchange<kDppXor1>(v));
    v = fmaxf(v, lane_exchange<kDppXor2>(v));
    v = fmaxf(v, lane_exchange<kDppHalfMirror>(v));
    v = fmaxf(v, lane_exchange<kDppMirror>(v));  // every lane: the maximum of its row of 16
    return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

// The sum over the 64 lanes, in every lane, as a butterfly (pairs, quads, eights, rows, then the
// four rows): for callers that need no particular order.
__device__ __forceinline__ float wave_sum(float v) {
    v += lane_exchange<kDppXor1>(v);
    v += lane_exchange<kDppXor2>(v);
    v += lane_exchange<kDppHalfMirror>(v);
    v += lane_exchange<kDppMirror>(v);
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}

// Lane i takes lane i + 32 (valid in lanes 0..31) or lane i + 16 (valid in lanes 0..15): the two
// row-crossing steps of a shuffle-down tree as lane-permute swaps in the vector ALU.  A swap of a
// register with a copy of itself leaves the upper half (the odd rows) of the copy in its lower half
// (its even rows).
__device__ __forceinline__ uint32_t lane_down32(uint32_t v) {
    return __builtin_amdgcn_permlane32_swap(v, v, false, false)[1];
}
__device__ __forceinline__ uint32_t lane_down16(uint32_t v) {
    return __builtin_amdgcn_permlane16_swap(v, v, false, false)[1];
}
__device__ __forceinline__ float lane_down32(float v) {
    return __builtin_bit_cast(float, lane_down32(__builtin_bit_cast(uint32_t, v)));
}
__device__ __forceinline__ float lane_down16(float v) {
    return __builtin_bit_cast(float, lane_down16(__builtin_bit_cast(uint32_t, v)));
}
__device__ __forceinline__ double lane_down32(double v) {
    const uint64_t bits = __builtin_bit_cast(uint64_t, v);
    return __builtin_bit_cast(double, ((uint64_t)lane_down32((uint32_t)(bits >> 32)) << 32) | lane_down32((uint32_t)bits));
}
__device__ __forceinline__ double lane_down16(double v) {
    const uint64_t bits = __builtin_bit_cast(uint64_t, v);
    return __builtin_bit_cast(double, ((uint64_t)lane_down16((uint32_t)(bits >> 32)) << 32) | lane_down16((uint32_t)bits));
}

// The sum over the 64 lanes in the order of a shuffle-down tree with offsets 32, 16, 8, 4, 2, 1
// (bit for bit what that tree gives), valid in lane 0 only.  No step goes through LDS: the two
// that cross rows are lane-permute swaps, the four inside the row DPP moves.
template <typename T>
__device__ __forceinline__ T wave_sum_to_lane0(T v) {
    v += lane_down32(v);
    v += lane_down16(v);
    v += lane_exchange<kDppRowShl + 8>(v);
    v += lane_exchange<kDppRowShl + 4>(v);
    v += lane_exchange<kDppRowShl + 2>(v);
    v += lane_exchange<kDppRowShl + 1>(v);
    return v;
}

}  // namespace vxhip
#endif
