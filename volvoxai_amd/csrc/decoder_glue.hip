// The steps either side of the W8A8 linears in a decoder layer, fused so that a decode step
// is a dozen launches per layer instead of several dozen elementwise ones:
//
//   rmsnorm_prepare   RMSNorm (native/src/kernels/softmax_rmsnorm.inc:3-17: double accumulation,
//                     x * inv_std * gain in double, one rounding to f32) followed by the
//                     PackedLinear activation preparation of that row
//                     (native/src/kernels/packed_linear_ops.inc:97-217)
//   swiglu_prepare    silu(gate) * up, then the same preparation
//   rope_append       non-interleaved rotary embedding of q and k
//                     (native/src/kernels/llm_math.h:256-274) and the KV-cache append
//   gqa_attention     grouped-query attention of the new tokens over the cache: f32 scores
//                     scaled by 1/sqrt(d), causal visibility slot <= position, softmax, P.V
//
// All are row-sized, latency-bound kernels; none of them is on the int8 roofline.
#include "common.h"
#include "device_math.h"
#include "row_math.h"
#include "wave_ops.h"

#include <math.h>

namespace vxhip {
namespace {

extern __shared__ __attribute__((aligned(16))) char glue_lds[];

// LAST: nothing writes `slots` again before the kernel ends, so no second barrier is needed.
template <bool LAST = false>
__device__ __forceinline__ float block_max(float v, float* slots) {
    v = wave_max(v);
    if ((threadIdx.x & 63u) == 0u) slots[threadIdx.x >> 6] = v;
    __syncthreads();
    float m = slots[0];
    for (uint32_t w = 1; w < blockDim.x / 64u; w++) m = fmaxf(m, slots[w]);
    if constexpr (!LAST) __syncthreads();
    return m;
}

// Shared tail of the two *_prepare kernels: the row's f32 values are in `vals` (LDS), element j
// written by thread j % blockDim.x, which is also the thread that reads it here.
// scale = max|v| / 127 (1.0 for an all-zero row, floored at 2^-126), code = ties-to-even(v / scale)
// clamped to +-127 with a true f32 divide; a non-finite row gets zero codes and a NaN scale.
// The codes of row `row` go where `layout` puts them (row-major rows of d bytes, or operand order,
// whose last 16-byte chunk is filled up with zeros).
__device__ __forceinline__ void prepare_row(const float* vals, uint32_t d, int8_t* codes, ActivationLayout layout,
                                            uint32_t row, float* scale_out, float* slots) {
    // one reduction for both questions: a non-finite element counts as +inf, which no finite
    // maximum can be
    float maximum = 0.0f;
    for (uint32_t j = threadIdx.x; j < d; j += blockDim.x) {
        const float v = vals[j];
        maximum = fmaxf(maximum, finite_f32(v) ? fabsf(v) : __builtin_inff());
    }
    maximum = block_max<true>(maximum, slots);
    const float bad = maximum == __builtin_inff() ? 1.0f : 0.0f;
    float scale = maximum == 0.0f || bad != 0.0f ? 1.0f : __fdiv_rn(maximum, 127.0f);
    if (scale < 0x1p-126f) scale = 0x1p-126f;
    for (uint32_t j = threadIdx.x; j < d; j += blockDim.x)
        codes[activation_offset(layout, row, j)] =
            bad != 0.0f ? (int8_t)0 : (int8_t)packed_round_i8(__fdiv_rn(vals[j], scale));
    if (layout.operand_order)
        for (uint32_t j = d + threadIdx.x; j < layout.ld; j += blockDim.x) codes[activation_offset(layout, row, j)] = 0;
    if (threadIdx.x == 0) *scale_out = bad != 0.0f ? __builtin_nanf("") : scale;
}

// delta (may be null): the row is first updated in place, x += delta (the residual add), and the
// updated row is what gets normalized.
__global__ __launch_bounds__(1024) void rmsnorm_prepare_kernel(float* __restrict__ x, const float* __restrict__ delta,
                                                              const float* __restrict__ gain, uint32_t d, double eps,
                                                              int8_t* __restrict__ prepared,
                                                              const ActivationLayout layout,
                                                              float* __restrict__ row_scales,
                                                              float* __restrict__ normalized) {
    float* vals = reinterpret_cast<float*>(glue_lds);
    __shared__ double dslots[16];
    __shared__ float slots[16];
    const uint32_t row = blockIdx.x;
    float* src = x + (size_t)row * d;
    double sum = 0.0;
    // the first pass's gain is requested with the row, not after the reduction
    const float gain_first = threadIdx.x < d ? gain[threadIdx.x] : 0.0f;
    for (uint32_t j = threadIdx.x; j < d; j += blockDim.x) {
        float v = src[j];
        if (delta) {
            v = __fadd_rn(v, delta[(size_t)row * d + j]);
            src[j] = v;
        }
        vals[j] = v;
        sum += (double)v * (double)v;
    }
    sum = wave_sum_to_lane0(sum);
    if ((threadIdx.x & 63u) == 0u) dslots[threadIdx.x >> 6] = sum;
    __syncthreads();
    double total = 0.0;
    for (uint32_t w = 0; w < blockDim.x / 64u; w++) total += dslots[w];
    const double inv_std = rms_inverse(total, d, eps);
    for (uint32_t j = threadIdx.x; j < d; j += blockDim.x) {
        const float gj = j == threadIdx.x ? gain_first : gain[j];
        const float y = rms_scaled(vals[j], inv_std, gj);
        vals[j] = y;
        if (normalized) normalized[(size_t)row * d + j] = y;
    }
    // (no barrier: prepare_row walks the row with the same stride, a thread reads its own writes)
    prepare_row(vals, d, prepared, layout, row, row_scales + row, slots);
}

__global__ __launch_bounds__(1024) void swiglu_prepare_kernel(const float* __restrict__ gate_up, uint32_t inter,
                                                             int8_t* __restrict__ prepared,
                                                             const ActivationLayout layout,
                                                             float* __restrict__ row_scales,
                                                             float* __restrict__ activated) {
    float* vals = reinterpret_cast<float*>(glue_lds);
    __shared__ float slots[16];
    const uint32_t row = blockIdx.x;
    const float* gate = gate_up + (size_t)row * 2u * inter;
    const float* up = gate + inter;
    for (uint32_t j = threadIdx.x; j < inter; j += blockDim.x) {
        const float y = swiglu_value(gate[j], up[j]);
        vals[j] = y;
        if (activated) activated[(size_t)row * inter + j] = y;
    }
    // (no barrier: prepare_row walks the row with the same stride, a thread reads its own writes)
    prepare_row(vals, inter, prepared, layout, row, row_scales + row, slots);
}

// grid rows * t, one workgroup per token walking the elements of all its heads (a workgroup per head
// is a launch of a hundred thousand workgroups that move 512 bytes each).  Token (row, i) sits at cache
// slot positions[i]; cos/sin are [max_seq][head_dim] tables indexed by that slot.
__global__ __launch_bounds__(256) void rope_append_kernel(const float* __restrict__ qkv, const float* __restrict__ cos_table,
                                                          const float* __restrict__ sin_table,
                                                          const int64_t* __restrict__ positions, uint32_t t, uint32_t q_heads,
                                                          uint32_t kv_heads, uint32_t head_dim, uint32_t max_seq,
                                                          float* __restrict__ q_out, float* __restrict__ k_cache,
                                                          float* __restrict__ v_cache, uint32_t* __restrict__ fault) {
    const uint32_t token = blockIdx.x;
    const uint32_t row = token / t, i = token % t;
    const uint32_t width = (q_heads + 2u * kv_heads) * head_dim;
    const uint64_t named = (uint64_t)positions[i];
    if (named >= max_seq) {  // outside the caches and the tables: touch nothing, say so
        if (threadIdx.x == 0) atomicOr(fault, (uint32_t)kFaultBadPosition);
        return;
    }
    const uint32_t slot = (uint32_t)named;
    const uint32_t half = head_dim / 2u;
    for (uint32_t j = threadIdx.x; j < width; j += blockDim.x) {
        const uint32_t head = j / head_dim, dd = j % head_dim;
        const float* src = qkv + (size_t)token * width + (size_t)head * head_dim;
        const float v = src[dd];
        if (head >= q_heads + kv_heads) {  // value head: plain append
            const uint32_t h = head - q_heads - kv_heads;
            v_cache[(((size_t)row * kv_heads + h) * max_seq + slot) * head_dim + dd] = v;
            continue;
        }
        const float partner = dd < half ? -src[dd + half] : src[dd - half];
        const float c = cos_table[(size_t)slot * head_dim + dd], s = sin_table[(size_t)slot * head_dim + dd];
        const float y = __fadd_rn(__fmul_rn(v, c), __fmul_rn(partner, s));
        if (head < q_heads) q_out[((size_t)token * q_heads + head) * head_dim + dd] = y;
        else k_cache[(((size_t)row * kv_heads + (head - q_heads)) * max_seq + slot) * head_dim + dd] = y;
    }
}

// grid (rows * t, q_heads / REP), block 256: a workgroup takes REP query heads that share one KV
// head, so every K and V row is read once for all of them.  LDS per head: q[head_dim] +
// scores[max_seq] + partial[8][head_dim] floats.  Scores: one thread per visible slot (its whole
// dot products, 16-byte loads, all independent); P.V: the slots split over eight groups of
// 32 threads, a thread four channels.
//
// FUSED (decode, t = 1): q is the qkv row as the linear wrote it.  The workgroup rotates its own
// query heads and the new key of its KV head itself (the arithmetic of rope_append_kernel), uses
// that key and the new value from LDS for the slot being appended, and the first workgroup of
// each KV group also stores them in the caches for later steps; slots before the new one come
// from the caches, so workgroups do not depend on each other.  Every slot is still handled by
// the thread, and in the order, that the unfused kernel gives it: the results are the same bits.
//
// Scores, NC = head_dim / 32 in {1, 2, 4, 8}: eight lanes share a key row, each loading the 16-byte
// chunks c = lane%8 + 8*i, so one load instruction of a wavefront covers eight rows with whole
// 128-byte lines (a thread per row touches 64 lines with every load and refetches each of them
// eight times once the rows outgrow the L1); the eight partial dots meet in three xor-shuffles.
// Rows of four passes (128 slots) are requested before the first is used.  NC = 0 keeps the
// thread-per-row loop for other head sizes.
template <int REP, bool FUSED, int NC>
__global__ __launch_bounds__(256) void gqa_attention_kernel(const float* __restrict__ q,
                                                            float* __restrict__ k_cache,
                                                            float* __restrict__ v_cache,
                                                            const int64_t* __restrict__ positions, uint32_t t,
                                                            uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                                                            uint32_t max_seq, float scale, float* __restrict__ out,
                                                            const float* __restrict__ cos_table,
                                                            const float* __restrict__ sin_table,
                                                            uint32_t* __restrict__ fault) {
    const uint32_t per_head = 9u * head_dim + max_seq;
    float* lds = reinterpret_cast<float*>(glue_lds);
    float* k_new = lds + REP * per_head;  // FUSED: the appended key and value, head_dim floats each
    float* v_new = k_new + head_dim;
    const uint32_t token = blockIdx.x;
    const uint32_t head0 = blockIdx.y * REP;
    const uint32_t row = token / t, i = token % t;
    const uint32_t kvh = head0 / (q_heads / kv_heads);
    const uint64_t named = (uint64_t)positions[i];
    if (named >= max_seq) {  // (the whole workgroup) outside the caches: touch nothing, say so
        if (threadIdx.x == 0) atomicOr(fault, (uint32_t)kFaultBadPosition);
        return;
    }
    const uint32_t position = (uint32_t)named;
    const uint32_t visible = position + 1u;  // slots 0 .. position
    // slots read from the caches: all visible ones, or all before the one being appended
    const uint32_t cached = FUSED ? position : visible;
    float* kbase = k_cache + ((size_t)row * kv_heads + kvh) * max_seq * head_dim;
    float* vbase = v_cache + ((size_t)row * kv_heads + kvh) * max_seq * head_dim;
    // Cached rows arrive in blocks that are requested two blocks ahead of their use, the first
    // two before the query is ready: every workgroup of the launch is resident at once and in the
    // same phase, each dependent request costs all of them a round trip to a loaded memory
    // (2-3 us), and up to 256 slots this way cost one for the keys and one for the values.  A
    // request never depends on a branch: rows past the end are clamped to the last cached one
    // (row 0 of the cache when there is none), so they cost no memory traffic and the waits
    // stay exact.
    // rows of PASSES passes of 32 are in a block (fewer at head size 256, whose rows are twice as
    // long: the two blocks must leave room for three wavefronts per SIMD where they can)
    constexpr int PASSES = NC > 4 ? 2 : 4, KC = NC > 0 ? NC : 1;
    const uint32_t last_cached = max(cached, 1u) - 1u;
    const uint32_t lane8 = threadIdx.x & 7u, rowg = threadIdx.x >> 3;
    float4 kv_a[PASSES][KC], kv_b[PASSES][KC];
    auto request_keys = [&](float4 (&buf)[PASSES][KC], uint32_t s0) {
#pragma unroll
        for (int u = 0; u < PASSES; u++) {
            const uint32_t srow = min(s0 + u * 32u + rowg, last_cached);
            const float4* kr = reinterpret_cast<const float4*>(kbase + (size_t)srow * head_dim);
#pragma unroll
            for (int c = 0; c < KC; c++) buf[u][c] = kr[lane8 + 8u * c];
        }
    };
    if constexpr (FUSED && NC > 0) {
        // (head sizes up to 256: a thread rotates at most one channel)  The operands of the rotation
        // are requested before the keys: loads return in order, so requested after them they
        // would hold the query back until every key of both blocks had arrived.
        const uint32_t width = (q_heads + 2u * kv_heads) * head_dim, half = head_dim / 2u;
        const float* src = q + (size_t)token * width;
        const bool writer = head0 % (q_heads / kv_heads) == 0u;
        const uint32_t dd = threadIdx.x, mate = dd < half ? dd + half : dd - half;
        const bool rotates = dd < head_dim;
        float in_q[REP], in_q_mate[REP], in_k = 0.0f, in_k_mate = 0.0f, in_v = 0.0f, in_cos = 0.0f, in_sin = 0.0f;
#pragma unroll
        for (int h = 0; h < REP; h++) in_q[h] = in_q_mate[h] = 0.0f;
        if (rotates) {
#pragma unroll
            for (int h = 0; h < REP; h++) {
                in_q[h] = src[(size_t)(head0 + h) * head_dim + dd];
                in_q_mate[h] = src[(size_t)(head0 + h) * head_dim + mate];
            }
            in_k = src[(size_t)(q_heads + kvh) * head_dim + dd];
            in_k_mate = src[(size_t)(q_heads + kvh) * head_dim + mate];
            in_v = src[(size_t)(q_heads + kv_heads + kvh) * head_dim + dd];
            in_cos = cos_table[(size_t)position * head_dim + dd];
            in_sin = sin_table[(size_t)position * head_dim + dd];
        }
        request_keys(kv_a, 0u);
        request_keys(kv_b, 32u * PASSES);
        if (rotates) {
            auto rotated = [&](float own, float other) {  // the arithmetic of rope_append_kernel
                return __fadd_rn(__fmul_rn(own, in_cos), __fmul_rn(dd < half ? -other : other, in_sin));
            };
#pragma unroll
            for (int h = 0; h < REP; h++) lds[h * per_head + dd] = rotated(in_q[h], in_q_mate[h]);
            const float kn = rotated(in_k, in_k_mate);
            k_new[dd] = kn;
            v_new[dd] = in_v;
            if (writer) {
                kbase[(size_t)position * head_dim + dd] = kn;
                vbase[(size_t)position * head_dim + dd] = in_v;
            }
        }
    } else if constexpr (FUSED) {
        const uint32_t width = (q_heads + 2u * kv_heads) * head_dim, half = head_dim / 2u;
        const float* src = q + (size_t)token * width;
        const bool writer = head0 % (q_heads / kv_heads) == 0u;
        auto rotated = [&](const float* head, uint32_t dd) {
            const float partner = dd < half ? -head[dd + half] : head[dd - half];
            const float c = cos_table[(size_t)position * head_dim + dd], sn = sin_table[(size_t)position * head_dim + dd];
            return __fadd_rn(__fmul_rn(head[dd], c), __fmul_rn(partner, sn));
        };
        for (uint32_t dd = threadIdx.x; dd < head_dim; dd += 256u) {
#pragma unroll
            for (int h = 0; h < REP; h++) lds[h * per_head + dd] = rotated(src + (size_t)(head0 + h) * head_dim, dd);
            const float kn = rotated(src + (size_t)(q_heads + kvh) * head_dim, dd);
            const float vn = src[(size_t)(q_heads + kv_heads + kvh) * head_dim + dd];
            k_new[dd] = kn;
            v_new[dd] = vn;
            if (writer) {
                kbase[(size_t)position * head_dim + dd] = kn;
                vbase[(size_t)position * head_dim + dd] = vn;
            }
        }
    } else {
        float in_q[REP];
#pragma unroll
        for (int h = 0; h < REP; h++)
            in_q[h] = threadIdx.x < head_dim ? q[((size_t)token * q_heads + head0 + h) * head_dim + threadIdx.x] : 0.0f;
        if constexpr (NC > 0) {
            request_keys(kv_a, 0u);
            request_keys(kv_b, 32u * PASSES);
        }
#pragma unroll
        for (int h = 0; h < REP; h++) {
            if (threadIdx.x < head_dim) lds[h * per_head + threadIdx.x] = in_q[h];
            for (uint32_t dd = threadIdx.x + 256u; dd < head_dim; dd += 256u)
                lds[h * per_head + dd] = q[((size_t)token * q_heads + head0 + h) * head_dim + dd];
        }
    }
    __syncthreads();
    // P.V: group g of 32 threads takes slots g, g + 8, ..., a thread four channels of each; the
    // values come in batches of eight rows, requested two batches ahead like the keys, the first
    // two before the softmax.  (Requesting them while key blocks are still alive takes more than
    // 256 registers, which halves the workgroups a compute unit holds and was slower.)
    const uint32_t group = threadIdx.x >> 5, chunk = threadIdx.x & 31u;
    constexpr int VROWS = 8;
    float4 vv_a[VROWS], vv_b[VROWS];
    auto request_values = [&](float4 (&buf)[VROWS], uint32_t s0, uint32_t c4) {
#pragma unroll
        for (int u = 0; u < VROWS; u++) {
            const uint32_t s = min(s0 + group + 8u * u, last_cached);
            buf[u] = *reinterpret_cast<const float4*>(vbase + (size_t)s * head_dim + min(c4, head_dim - 4u));
        }
    };
    constexpr uint32_t BATCH = 8u * VROWS;  // slots per batch over the eight groups
    float m[REP];
#pragma unroll
    for (int h = 0; h < REP; h++) m[h] = -INFINITY;
    if constexpr (NC > 0) {
        // this lane's share of a row's dot with each query head, then the sum over the eight lanes
        auto finish = [&](float (&dot)[REP], uint32_t slot) {
#pragma unroll
            for (int h = 0; h < REP; h++) {
                float d = dot[h];
                // the eight lanes' sum as a butterfly of lane exchanges inside the register file
                // (an exchange through the LDS crossbar costs a round trip, and the three of a
                // row depend on each other): partners lane^1, lane^2, then the mirrored lane of
                // the other quad, whose four lanes all hold that quad's sum by then
                d += lane_exchange<kDppXor1>(d);
                d += lane_exchange<kDppXor2>(d);
                d += lane_exchange<kDppHalfMirror>(d);
                d = __fmul_rn(d, scale);
                if (lane8 == 0u) lds[h * per_head + head_dim + slot] = d;
                m[h] = fmaxf(m[h], d);
            }
        };
        // this lane's chunks of the query heads: registers when they are few (a read from LDS
        // cannot be hoisted over the score writes by the compiler and would repeat per row)
        constexpr bool Q_HELD = REP * KC <= 8;
        float4 q_held[Q_HELD ? REP : 1][Q_HELD ? KC : 1];
        if constexpr (Q_HELD) {
#pragma unroll
            for (int h = 0; h < REP; h++)
#pragma unroll
                for (int c = 0; c < KC; c++)
                    q_held[h][c] = *reinterpret_cast<const float4*>(lds + h * per_head + 4u * (lane8 + 8u * c));
        }
        auto accumulate = [&](float (&dot)[REP], const float4& kv, int c) {
#pragma unroll
            for (int h = 0; h < REP; h++) {
                float4 qv;
                if constexpr (Q_HELD) qv = q_held[h][c];
                else qv = *reinterpret_cast<const float4*>(lds + h * per_head + 4u * (lane8 + 8u * c));
                // fused multiply-adds: the score phase is bound by vector instruction issue (two
                // wavefronts per SIMD, each a few hundred instructions), and this halves it
                dot[h] = __builtin_fmaf(qv.x, kv.x, dot[h]);
                dot[h] = __builtin_fmaf(qv.y, kv.y, dot[h]);
                dot[h] = __builtin_fmaf(qv.z, kv.z, dot[h]);
                dot[h] = __builtin_fmaf(qv.w, kv.w, dot[h]);
            }
        };
        constexpr uint32_t BLOCK = 32u * PASSES;  // slots per block
        auto score_block = [&](float4 (&buf)[PASSES][KC], uint32_t s0) {
#pragma unroll
            for (int u = 0; u < PASSES; u++) {
                const uint32_t srow = s0 + u * 32u + rowg;
                float dot[REP];
#pragma unroll
                for (int h = 0; h < REP; h++) dot[h] = 0.0f;
#pragma unroll
                for (int c = 0; c < NC; c++) accumulate(dot, buf[u][c], c);
                // (all 64 lanes take part in the shuffles; a row past the end repeats the last
                // cached one, rewrites its score with the same value and is dropped from the
                // maximum here)
                float keep[REP];
#pragma unroll
                for (int h = 0; h < REP; h++) keep[h] = m[h];
                finish(dot, min(srow, last_cached));
                if (srow >= cached) {
#pragma unroll
                    for (int h = 0; h < REP; h++) m[h] = keep[h];
                }
            }
        };
        for (uint32_t s0 = 0; s0 < cached; s0 += 2u * BLOCK) {
            score_block(kv_a, s0);
            request_keys(kv_a, s0 + 2u * BLOCK);
            if (s0 + BLOCK < cached) score_block(kv_b, s0 + BLOCK);  // (a scalar branch)
            request_keys(kv_b, s0 + 3u * BLOCK);
        }
        if constexpr (FUSED) {
            // the appended slot, from LDS, by the eight lanes that own it in the unfused kernel and in
            // the same order of operations
            if (rowg == position % 32u) {
                float dot[REP];
#pragma unroll
                for (int h = 0; h < REP; h++) dot[h] = 0.0f;
#pragma unroll
                for (int c = 0; c < NC; c++)
                    accumulate(dot, *reinterpret_cast<const float4*>(k_new + 4u * (lane8 + 8u * c)), c);
                finish(dot, position);
            }
        }
    } else {
        if constexpr (FUSED) {
            // the appended slot, from LDS; it is the last slot of the thread that owns it
            if (threadIdx.x == position % 256u) {
                float dot[REP];
#pragma unroll
                for (int h = 0; h < REP; h++) dot[h] = 0.0f;
                for (uint32_t c = 0; c < head_dim / 4u; c++) {
#pragma unroll
                    for (int h = 0; h < REP; h++) {
                        const float* qs = lds + h * per_head;
                        dot[h] += qs[4 * c] * k_new[4 * c] + qs[4 * c + 1] * k_new[4 * c + 1] +
                                  qs[4 * c + 2] * k_new[4 * c + 2] + qs[4 * c + 3] * k_new[4 * c + 3];
                    }
                }
#pragma unroll
                for (int h = 0; h < REP; h++) {
                    dot[h] = __fmul_rn(dot[h], scale);
                    lds[h * per_head + head_dim + position] = dot[h];
                    m[h] = fmaxf(m[h], dot[h]);
                }
            }
        }
        for (uint32_t s = threadIdx.x; s < cached; s += 256u) {
            const float4* kr = reinterpret_cast<const float4*>(kbase + (size_t)s * head_dim);
            float dot[REP];
#pragma unroll
            for (int h = 0; h < REP; h++) dot[h] = 0.0f;
#pragma unroll 8
            for (uint32_t c = 0; c < head_dim / 4u; c++) {
                const float4 kv = kr[c];
#pragma unroll
                for (int h = 0; h < REP; h++) {
                    const float* qs = lds + h * per_head;
                    dot[h] += qs[4 * c] * kv.x + qs[4 * c + 1] * kv.y + qs[4 * c + 2] * kv.z + qs[4 * c + 3] * kv.w;
                }
            }
#pragma unroll
            for (int h = 0; h < REP; h++) {
                dot[h] = __fmul_rn(dot[h], scale);
                lds[h * per_head + head_dim + s] = dot[h];
                m[h] = fmaxf(m[h], dot[h]);
            }
        }
    }
    if constexpr (NC > 0) {
        request_values(vv_a, 0u, chunk * 4u);
        request_values(vv_b, BATCH, chunk * 4u);
    }
    // Softmax.  The heads' maxima cross the workgroup in one exchange (every thread scored slots
    // of every head); after that the 4 / REP wavefronts of a group own one head each, so the heads'
    // exponentials, sums and divisions run side by side instead of one head after the other.
    {
        constexpr uint32_t GROUP = 256u / REP, GROUP_WAVES = 4u / REP;
        __shared__ float wave_maxima[4 * REP], wave_sums[4];
        const uint32_t wave = threadIdx.x >> 6, own = threadIdx.x / GROUP, at = threadIdx.x % GROUP;
#pragma unroll
        for (int h = 0; h < REP; h++) {
            const float mw = wave_max(m[h]);
            if ((threadIdx.x & 63u) == 0u) wave_maxima[wave * REP + h] = mw;
        }
        __syncthreads();  // (also: the scores of a slot are read below by other threads than wrote them)
        float mh = wave_maxima[own];
#pragma unroll
        for (uint32_t w = 1; w < 4u; w++) mh = fmaxf(mh, wave_maxima[w * REP + own]);
        float* scores = lds + own * per_head + head_dim;
        float sum = 0.0f;
        for (uint32_t s = at; s < visible; s += GROUP) {
            const float e = expf(scores[s] - mh);
            scores[s] = e;
            sum += e;
        }
        sum = wave_sum_to_lane0(sum);
        if ((threadIdx.x & 63u) == 0u) wave_sums[wave] = sum;
        __syncthreads();
        float total = wave_sums[own * GROUP_WAVES];
#pragma unroll
        for (uint32_t w = 1; w < GROUP_WAVES; w++) total += wave_sums[own * GROUP_WAVES + w];
        for (uint32_t s = at; s < visible; s += GROUP) scores[s] = __fdiv_rn(scores[s], total);
    }
    __syncthreads();
    for (uint32_t c4 = chunk * 4u; c4 < head_dim; c4 += 128u) {
        float4 acc[REP];
#pragma unroll
        for (int h = 0; h < REP; h++) acc[h] = make_float4(0.f, 0.f, 0.f, 0.f);
        auto weigh = [&](const float4& vv, uint32_t s) {
#pragma unroll
            for (int h = 0; h < REP; h++) {
                const float p = lds[h * per_head + head_dim + s];
                acc[h].x = __builtin_fmaf(p, vv.x, acc[h].x);
                acc[h].y = __builtin_fmaf(p, vv.y, acc[h].y);
                acc[h].z = __builtin_fmaf(p, vv.z, acc[h].z);
                acc[h].w = __builtin_fmaf(p, vv.w, acc[h].w);
            }
        };
        if constexpr (NC > 0) {
            auto weigh_batch = [&](float4 (&buf)[VROWS], uint32_t s0) {
#pragma unroll
                for (int u = 0; u < VROWS; u++) {
                    const uint32_t s = s0 + group + 8u * u;
                    if (s < cached) weigh(buf[u], s);
                }
            };
            if (c4 != chunk * 4u) {  // head sizes above 128: a later pass
                request_values(vv_a, 0u, c4);
                request_values(vv_b, BATCH, c4);
            }
            for (uint32_t s0 = 0; s0 < cached; s0 += 2u * BATCH) {
                weigh_batch(vv_a, s0);
                request_values(vv_a, s0 + 2u * BATCH, c4);
                if (s0 + BATCH < cached) weigh_batch(vv_b, s0 + BATCH);
                request_values(vv_b, s0 + 3u * BATCH, c4);
            }
        } else {
#pragma unroll 8
            for (uint32_t s = group; s < cached; s += 8u)
                weigh(*reinterpret_cast<const float4*>(vbase + (size_t)s * head_dim + c4), s);
        }
        if constexpr (FUSED) {
            if (group == position % 8u) {  // the appended slot closes its group's sum
                const float4 vv = *reinterpret_cast<const float4*>(v_new + c4);
#pragma unroll
                for (int h = 0; h < REP; h++) {
                    const float p = lds[h * per_head + head_dim + position];
                    acc[h].x = __builtin_fmaf(p, vv.x, acc[h].x);
                    acc[h].y = __builtin_fmaf(p, vv.y, acc[h].y);
                    acc[h].z = __builtin_fmaf(p, vv.z, acc[h].z);
                    acc[h].w = __builtin_fmaf(p, vv.w, acc[h].w);
                }
            }
        }
#pragma unroll
        for (int h = 0; h < REP; h++)
            *reinterpret_cast<float4*>(lds + h * per_head + head_dim + max_seq + group * head_dim + c4) = acc[h];
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < REP; h++) {
        const float* partial = lds + h * per_head + head_dim + max_seq;
        for (uint32_t dd = threadIdx.x; dd < head_dim; dd += 256u) {
            float total = 0.0f;
#pragma unroll
            for (uint32_t g = 0; g < 8u; g++) total += partial[g * head_dim + dd];
            out[((size_t)token * q_heads + head0 + h) * head_dim + dd] = total;
        }
    }
}

// Prompt attention (t > 1 tokens per row).  The kernel above gives every (token, head) its own
// workgroup, so a prompt of t tokens reads each key and value row t times.  Here a workgroup takes
// `tq` consecutive tokens of one row and the `rep` query heads of one KV head, qw = tq * rep <= 32
// queries, and walks that KV head's rows once for all of them, 64 slots at a time through LDS:
//   scores   thread (slot = tid % 64, wavefront) holds eight queries' dots with one staged key row;
//            the eight queries are the same for the whole wavefront, so they are read through the
//            scalar cache straight from global memory and cost no LDS bandwidth (as LDS broadcast
//            reads they took nine tenths of it and bounded the kernel)
//   softmax  a wavefront per query, over the slots that query may see (slot <= its position)
//   P.V      thread (four channels, tid / 32) holds four queries' sums over the staged value rows
// The arithmetic is that of the kernel above (f32, scores scaled after the dot, exp(x - max),
// a true division by the sum) with fused multiply-adds and its own summation order.
// grid (rows * ceil(t / tq), kv_heads), block 256.
// LDS: scores [qw][max_seq rounded up to 64], staged rows [64][head_dim + 4].
constexpr uint32_t kPrefillQueries = 32u, kPrefillSlots = 64u;

__global__ __launch_bounds__(256) void gqa_prefill_kernel(const float* __restrict__ q,
                                                          const float* __restrict__ k_cache,
                                                          const float* __restrict__ v_cache,
                                                          const int64_t* __restrict__ positions, uint32_t t,
                                                          uint32_t tq, uint32_t q_heads, uint32_t kv_heads,
                                                          uint32_t head_dim, uint32_t max_seq, float scale,
                                                          float* __restrict__ out, uint32_t* __restrict__ fault) {
    __shared__ uint32_t visible[kPrefillQueries];  // slots query i may see; 0: no such query
    const uint32_t rep = q_heads / kv_heads, qw = tq * rep;
    const uint32_t blocks = (t + tq - 1u) / tq;
    const uint32_t row = blockIdx.x / blocks, i0 = (blockIdx.x % blocks) * tq, kvh = blockIdx.y;
    // (a score row is a whole number of 64-slot blocks, so that P.V never has to guard a slot)
    const uint32_t hd4 = head_dim / 4u, pitch = head_dim + 4u, score_pitch = (max_seq + 63u) & ~63u;
    float* sc = reinterpret_cast<float*>(glue_lds);
    float* stage = sc + (size_t)qw * score_pitch;
    const float* kbase = k_cache + ((size_t)row * kv_heads + kvh) * max_seq * head_dim;
    const float* vbase = v_cache + ((size_t)row * kv_heads + kvh) * max_seq * head_dim;
    auto token_of = [&](uint32_t qi) { return i0 + qi / rep; };
    auto head_of = [&](uint32_t qi) { return kvh * rep + qi % rep; };

    if (threadIdx.x < kPrefillQueries) {
        const uint32_t qi = threadIdx.x;
        uint32_t v = 0u;
        if (qi < qw && token_of(qi) < t) {
            const uint64_t named = (uint64_t)positions[token_of(qi)];
            if (named >= max_seq) atomicOr(fault, (uint32_t)kFaultBadPosition);  // (its output row is left as it is)
            else v = (uint32_t)named + 1u;
        }
        visible[qi] = v;
    }
    __syncthreads();
    uint32_t span = 0u;  // slots any query of the workgroup sees
    for (uint32_t qi = 0; qi < qw; qi++) span = max(span, visible[qi]);

    // Rows s0 .. s0+63 of a cache (zeros past the span) go to the stage in two steps: requested
    // into registers, stored to LDS a block later -- the request of the next block is in flight
    // while this one is being used.
    constexpr int kStageRegs = 16;  // 64 rows x 256 floats over 256 threads, as 16-byte words
    const uint32_t stage_words = kPrefillSlots * hd4;
    auto fetch_rows = [&](const float* base, uint32_t s0, float4 (&v)[kStageRegs]) {
#pragma unroll
        for (int u = 0; u < kStageRegs; u++) {
            const uint32_t e = threadIdx.x + u * 256u, srow = s0 + e / hd4;
            v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e < stage_words && srow < span)
                v[u] = *reinterpret_cast<const float4*>(base + (size_t)srow * head_dim + 4u * (e % hd4));
        }
    };
    auto commit_rows = [&](const float4 (&v)[kStageRegs]) {
#pragma unroll
        for (int u = 0; u < kStageRegs; u++) {
            const uint32_t e = threadIdx.x + u * 256u;
            if (e < stage_words) *reinterpret_cast<float4*>(stage + (size_t)(e / hd4) * pitch + 4u * (e % hd4)) = v[u];
        }
    };
    float4 ahead[kStageRegs];
    fetch_rows(kbase, 0u, ahead);

    {   // scores
        const uint32_t slot = threadIdx.x & 63u;
        const uint32_t first = __builtin_amdgcn_readfirstlane((threadIdx.x >> 6) * 8u);  // wave-uniform
        // (queries past qw, or of tokens past t, repeat a valid one; their dots are dropped below)
        const float* qrow[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t qi = min(first + j, qw - 1u);
            qrow[j] = q + ((size_t)(row * t + min(token_of(qi), t - 1u)) * q_heads + head_of(qi)) * head_dim;
        }
        for (uint32_t s0 = 0; s0 < span; s0 += kPrefillSlots) {
            commit_rows(ahead);
            __syncthreads();
            // the next block of keys, or after the last one the first block of values
            if (s0 + kPrefillSlots < span) fetch_rows(kbase, s0 + kPrefillSlots, ahead);
            else fetch_rows(vbase, 0u, ahead);
            float dot[8];
#pragma unroll
            for (int j = 0; j < 8; j++) dot[j] = 0.0f;
            const float* krow = stage + (size_t)slot * pitch;
#pragma unroll 4
            for (uint32_t c = 0; c < hd4; c++) {  // (unrolled: the loads of four steps go out together)
                const float4 kv = *reinterpret_cast<const float4*>(krow + 4u * c);
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float4 qv = *reinterpret_cast<const float4*>(qrow[j] + 4u * c);
                    dot[j] = __builtin_fmaf(qv.x, kv.x, dot[j]);
                    dot[j] = __builtin_fmaf(qv.y, kv.y, dot[j]);
                    dot[j] = __builtin_fmaf(qv.z, kv.z, dot[j]);
                    dot[j] = __builtin_fmaf(qv.w, kv.w, dot[j]);
                }
            }
            const uint32_t s = s0 + slot;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t qi = first + j;
                if (qi < qw && s < visible[qi]) sc[(size_t)qi * score_pitch + s] = __fmul_rn(dot[j], scale);
            }
            __syncthreads();
        }
    }
    {   // softmax: probabilities over the visible slots, zeros from there to the span
        const uint32_t lane = threadIdx.x & 63u;
        for (uint32_t qi = threadIdx.x >> 6; qi < qw; qi += 4u) {  // (uniform per wavefront)
            float* mine = sc + (size_t)qi * score_pitch;
            const uint32_t seen = visible[qi];
            if (seen != 0u) {
                float m = -INFINITY;
                for (uint32_t s = lane; s < seen; s += 64u) m = fmaxf(m, mine[s]);
                m = wave_max(m);
                float sum = 0.0f;
                for (uint32_t s = lane; s < seen; s += 64u) {
                    const float e = expf(mine[s] - m);
                    mine[s] = e;
                    sum += e;
                }
                sum = wave_sum(sum);
                for (uint32_t s = lane; s < seen; s += 64u) mine[s] = __fdiv_rn(mine[s], sum);
            }
            const uint32_t span_blocks = (span + kPrefillSlots - 1u) / kPrefillSlots * kPrefillSlots;
            for (uint32_t s = seen + lane; s < span_blocks; s += 64u) mine[s] = 0.0f;
        }
    }
    __syncthreads();
    {   // P.V
        const uint32_t c4 = (threadIdx.x & 31u) * 4u, first = (threadIdx.x >> 5) * 4u;
        float4 acc[2][4];  // channel passes c4 and c4 + 128 (head sizes up to 256) x four queries
#pragma unroll
        for (int pass = 0; pass < 2; pass++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[pass][j] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (uint32_t s0 = 0; s0 < span; s0 += kPrefillSlots) {
            commit_rows(ahead);
            __syncthreads();
            if (s0 + kPrefillSlots < span) fetch_rows(vbase, s0 + kPrefillSlots, ahead);
            // (every row of the block: the staged rows past the span are zeros and so are their
            // probabilities, and a fixed count lets the reads of eight rows go out together)
#pragma unroll 8
            for (uint32_t r = 0; r < kPrefillSlots; r++) {
                float p[4];
#pragma unroll
                for (int j = 0; j < 4; j++) p[j] = sc[(size_t)min(first + j, qw - 1u) * score_pitch + s0 + r];
#pragma unroll
                for (int pass = 0; pass < 2; pass++) {
                    const uint32_t cc = c4 + pass * 128u;
                    if (cc < head_dim) {
                        const float4 vv = *reinterpret_cast<const float4*>(stage + (size_t)r * pitch + cc);
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            acc[pass][j].x = __builtin_fmaf(p[j], vv.x, acc[pass][j].x);
                            acc[pass][j].y = __builtin_fmaf(p[j], vv.y, acc[pass][j].y);
                            acc[pass][j].z = __builtin_fmaf(p[j], vv.z, acc[pass][j].z);
                            acc[pass][j].w = __builtin_fmaf(p[j], vv.w, acc[pass][j].w);
                        }
                    }
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t qi = first + j;
            if (qi >= qw || token_of(qi) >= t || visible[qi] == 0u) continue;
            float* dst = out + ((size_t)(row * t + token_of(qi)) * q_heads + head_of(qi)) * head_dim;
#pragma unroll
            for (int pass = 0; pass < 2; pass++) {
                const uint32_t cc = c4 + pass * 128u;
                if (cc < head_dim) *reinterpret_cast<float4*>(dst + cc) = acc[pass][j];
            }
        }
    }
}

// The same prompt attention for head size 128 on the f32 matrix pipes (v_mfma_f32_32x32x2f32: full
// f32 products and sums, not a reduced-precision format).  The queries of a workgroup are the 32
// rows of the A operand and stay in registers for the whole kernel: lane l holds query l % 32 and,
// for the scores, 32 of its 128 channels.  Per 64-slot block:
//   scores  wavefront w takes slots 32 * (w & 1) .. +31 and channels 64 * (w >> 1) .. +63: 32 MFMAs,
//           each adding the channel pair (c, c + 32) of the lane halves; the two channel halves of
//           a slot tile are added through the score rows in LDS (one stores, one adds and scales)
//   P.V     wavefront w takes output channels 32 * w .. +31: 32 MFMAs, each adding the slot pair
//           (s, s + 32); the sums stay in 16 accumulator registers across the blocks
// Softmax and staging are those of the kernel above.  A workgroup's score rows are always 32.
// (The kernel above reads its queries through the scalar cache, which two workgroups per compute
// unit overflow: 189 us per launch of a 32-row, 128-token prompt against 102 us here.)
typedef float v16f __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void gqa_prefill_mfma_kernel(const float* __restrict__ q,
                                                               const float* __restrict__ k_cache,
                                                               const float* __restrict__ v_cache,
                                                               const int64_t* __restrict__ positions, uint32_t t,
                                                               uint32_t tq, uint32_t q_heads, uint32_t kv_heads,
                                                               uint32_t max_seq, float scale, float* __restrict__ out,
                                                               uint32_t* __restrict__ fault) {
    constexpr uint32_t HD = 128u, HD4 = HD / 4u, PITCH = HD + 4u;
    __shared__ uint32_t visible[kPrefillQueries];
    const uint32_t rep = q_heads / kv_heads, qw = tq * rep;
    const uint32_t blocks = (t + tq - 1u) / tq;
    const uint32_t row = blockIdx.x / blocks, i0 = (blockIdx.x % blocks) * tq, kvh = blockIdx.y;
    const uint32_t score_pitch = (max_seq + 63u) & ~63u;
    float* sc = reinterpret_cast<float*>(glue_lds);             // [32][score_pitch]
    float* stage = sc + (size_t)kPrefillQueries * score_pitch;  // [64][PITCH]
    const float* kbase = k_cache + ((size_t)row * kv_heads + kvh) * max_seq * HD;
    const float* vbase = v_cache + ((size_t)row * kv_heads + kvh) * max_seq * HD;
    const uint32_t lane = threadIdx.x & 63u, r = lane & 31u, h = lane >> 5;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    auto token_of = [&](uint32_t qi) { return i0 + qi / rep; };
    auto head_of = [&](uint32_t qi) { return kvh * rep + qi % rep; };

    if (threadIdx.x < kPrefillQueries) {
        const uint32_t qi = threadIdx.x;
        uint32_t v = 0u;
        if (qi < qw && token_of(qi) < t) {
            const uint64_t named = (uint64_t)positions[token_of(qi)];
            if (named >= max_seq) atomicOr(fault, (uint32_t)kFaultBadPosition);  // (its output row is left as it is)
            else v = (uint32_t)named + 1u;
        }
        visible[qi] = v;
    }
    // this lane's 32 channels of query r for the scores (zeros for a query that does not exist)
    const uint32_t score_channel = 64u * (wave >> 1) + 32u * h;
    float qreg[32];
    {
        const bool exists = r < qw && token_of(r) < t;
        const float* src = q + ((size_t)(row * t + (exists ? token_of(r) : 0u)) * q_heads + head_of(exists ? r : 0u)) * HD +
                           score_channel;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float4 v = exists ? *reinterpret_cast<const float4*>(src + 4 * j) : make_float4(0.f, 0.f, 0.f, 0.f);
            qreg[4 * j] = v.x, qreg[4 * j + 1] = v.y, qreg[4 * j + 2] = v.z, qreg[4 * j + 3] = v.w;
        }
    }
    __syncthreads();
    uint32_t span = 0u;
    for (uint32_t qi = 0; qi < qw; qi++) span = max(span, visible[qi]);
    const uint32_t span_blocks = (span + kPrefillSlots - 1u) / kPrefillSlots * kPrefillSlots;

    constexpr int kStageRegs = 8;  // 64 rows x 128 floats over 256 threads, as 16-byte words
    auto fetch_rows = [&](const float* base, uint32_t s0, float4 (&v)[kStageRegs]) {
#pragma unroll
        for (int u = 0; u < kStageRegs; u++) {
            const uint32_t e = threadIdx.x + u * 256u, srow = s0 + e / HD4;
            v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (srow < span) v[u] = *reinterpret_cast<const float4*>(base + (size_t)srow * HD + 4u * (e % HD4));
        }
    };
    auto commit_rows = [&](const float4 (&v)[kStageRegs]) {
#pragma unroll
        for (int u = 0; u < kStageRegs; u++) {
            const uint32_t e = threadIdx.x + u * 256u;
            *reinterpret_cast<float4*>(stage + (size_t)(e / HD4) * PITCH + 4u * (e % HD4)) = v[u];
        }
    };
    float4 ahead[kStageRegs];
    fetch_rows(kbase, 0u, ahead);

    // The 16 accumulator registers of a lane are rows 8 * (v / 4) + 4 * h + v % 4 of column r.
    auto tile_row = [&](int v) { return 8u * (uint32_t)(v / 4) + 4u * h + (uint32_t)(v % 4); };

    for (uint32_t s0 = 0; s0 < span; s0 += kPrefillSlots) {  // scores
        commit_rows(ahead);
        __syncthreads();
        if (s0 + kPrefillSlots < span) fetch_rows(kbase, s0 + kPrefillSlots, ahead);
        else fetch_rows(vbase, 0u, ahead);
        const uint32_t slot_tile = 32u * (wave & 1u);
        const float* krow = stage + (size_t)(slot_tile + r) * PITCH + score_channel;
        v16f acc;
#pragma unroll
        for (int v = 0; v < 16; v++) acc[v] = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float4 kv = *reinterpret_cast<const float4*>(krow + 4 * j);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[4 * j], kv.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[4 * j + 1], kv.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[4 * j + 2], kv.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[4 * j + 3], kv.w, acc, 0, 0, 0);
        }
        float* tile = sc + s0 + slot_tile + r;  // + query * score_pitch
        if ((wave >> 1) == 0u) {
#pragma unroll
            for (int v = 0; v < 16; v++) tile[(size_t)tile_row(v) * score_pitch] = acc[v];
        }
        __syncthreads();
        if ((wave >> 1) == 1u) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float* at = tile + (size_t)tile_row(v) * score_pitch;
                *at = __fmul_rn(__fadd_rn(*at, acc[v]), scale);
            }
        }
        __syncthreads();
    }
    {   // softmax: probabilities over the visible slots, zeros from there to the end of the last block
        for (uint32_t qi = wave; qi < kPrefillQueries; qi += 4u) {
            float* mine = sc + (size_t)qi * score_pitch;
            const uint32_t seen = qi < qw ? visible[qi] : 0u;
            if (seen != 0u) {
                float m = -INFINITY;
                for (uint32_t s = lane; s < seen; s += 64u) m = fmaxf(m, mine[s]);
                m = wave_max(m);
                float sum = 0.0f;
                for (uint32_t s = lane; s < seen; s += 64u) {
                    const float e = expf(mine[s] - m);
                    mine[s] = e;
                    sum += e;
                }
                sum = wave_sum(sum);
                for (uint32_t s = lane; s < seen; s += 64u) mine[s] = __fdiv_rn(mine[s], sum);
            }
            for (uint32_t s = seen + lane; s < span_blocks; s += 64u) mine[s] = 0.0f;
        }
    }
    __syncthreads();
    v16f o;
#pragma unroll
    for (int v = 0; v < 16; v++) o[v] = 0.0f;
    for (uint32_t s0 = 0; s0 < span; s0 += kPrefillSlots) {  // P.V
        commit_rows(ahead);
        __syncthreads();
        if (s0 + kPrefillSlots < span) fetch_rows(vbase, s0 + kPrefillSlots, ahead);
        const float* prow = sc + (size_t)r * score_pitch + s0 + 32u * h;      // probabilities of query r
        const float* vcol = stage + (size_t)(32u * h) * PITCH + 32u * wave + r;  // channel 32 * wave + r
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float4 pv = *reinterpret_cast<const float4*>(prow + 4 * j);
            o = __builtin_amdgcn_mfma_f32_32x32x2f32(pv.x, vcol[(size_t)(4 * j) * PITCH], o, 0, 0, 0);
            o = __builtin_amdgcn_mfma_f32_32x32x2f32(pv.y, vcol[(size_t)(4 * j + 1) * PITCH], o, 0, 0, 0);
            o = __builtin_amdgcn_mfma_f32_32x32x2f32(pv.z, vcol[(size_t)(4 * j + 2) * PITCH], o, 0, 0, 0);
            o = __builtin_amdgcn_mfma_f32_32x32x2f32(pv.w, vcol[(size_t)(4 * j + 3) * PITCH], o, 0, 0, 0);
        }
        __syncthreads();
    }
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const uint32_t qi = tile_row(v);
        if (qi >= qw || token_of(qi) >= t || visible[qi] == 0u) continue;
        out[((size_t)(row * t + token_of(qi)) * q_heads + head_of(qi)) * HD + 32u * wave + r] = o[v];
    }
}

// Few rows leave most of the device idle and the kernel latency bound: then a row gets a full
// 1024-thread workgroup; with many rows 256 threads per row keep more rows resident.
uint32_t row_block(uint32_t rows, uint32_t d) {
    return rows <= 256u && d >= 1024u ? 1024u : 256u;
}

// Query heads that share a workgroup (and with it every key and value row of their KV head):
// four for wide groups, two for any even group, else one.  With the key and value rows requested
// ahead of their use the kernel is bound by those reads, and two heads per workgroup (half the
// requests, half the workgroups) run a 32-row decode step of 16 heads 3 % faster than one; before
// that rewrite the kernel was latency bound and one head per workgroup was the faster choice.
// Few rows: while one head per workgroup still leaves no compute unit with two workgroups the launch
// is latency bound again, and the heads are faster apart (28 layers of 16 query / 8 KV heads of 128,
// per decode step: 1 row 1.13 -> 1.10 ms, 16 rows 1.385 -> 1.348; 32 rows 1.49 with two heads
// together, 1.55 apart).
uint32_t heads_per_workgroup(uint32_t rep, uint32_t query_heads_in_launch, int compute_units) {
    if (query_heads_in_launch <= (uint32_t)(compute_units > 0 ? compute_units : 256)) return 1u;
    return rep >= 8u && rep % 4u == 0u ? 4u : rep % 2u == 0u ? 2u : 1u;
}

bool device_ready(VxHipContext* ctx) {
    return ctx && hipSetDevice(ctx->device) == hipSuccess;
}

// What a prepare entry point writes: row-major rows of d codes, or, on a context set to
// VXHIP_ACTIVATIONS_OPERAND32 and for at most 32 rows, operand order.
ActivationLayout prepared_layout(const VxHipContext* ctx, uint32_t rows, uint32_t d) {
    if (ctx->activation_layout == VXHIP_ACTIVATIONS_OPERAND32 && rows <= kOperandOrderRows)
        return ActivationLayout{(d + 15u) / 16u * 16u, 1u};
    return ActivationLayout{d, 0u};
}

// Picks the instance for the query heads per workgroup (4 or 1) and the head size.
template <bool FUSED>
void launch_attention(hipStream_t stream, uint32_t together, dim3 grid, size_t lds, const float* q, float* k_cache,
                      float* v_cache, const int64_t* positions, uint32_t t, uint32_t q_heads, uint32_t kv_heads,
                      uint32_t head_dim, uint32_t max_seq, float scale, float* out, const float* cos_table,
                      const float* sin_table, uint32_t* fault) {
#define VXHIP_ATTENTION(R, NC)                                                                                  \
    hipLaunchKernelGGL((gqa_attention_kernel<R, FUSED, NC>), grid, dim3(256), lds, stream, q, k_cache, v_cache, \
                       positions, t, q_heads, kv_heads, head_dim, max_seq, scale, out, cos_table, sin_table, fault)
#define VXHIP_ATTENTION_HEADS(NC)     \
    do {                              \
        if (together == 4u) VXHIP_ATTENTION(4, NC); \
        else if (together == 2u) VXHIP_ATTENTION(2, NC); \
        else VXHIP_ATTENTION(1, NC);  \
    } while (0)
    switch (head_dim) {
        case 32: VXHIP_ATTENTION_HEADS(1); break;
        case 64: VXHIP_ATTENTION_HEADS(2); break;
        case 128: VXHIP_ATTENTION_HEADS(4); break;
        case 256: VXHIP_ATTENTION_HEADS(8); break;
        default: VXHIP_ATTENTION_HEADS(0); break;
    }
#undef VXHIP_ATTENTION_HEADS
#undef VXHIP_ATTENTION
}

// Embedding lookup (embedding.inc:5-16): out[i] = table[tokens[i]], one workgroup per token.
// The reference reads whatever an id outside the table points at; here such a row is zeros and
// a fault bit is raised.
__global__ __launch_bounds__(256) void embedding_gather_kernel(const int32_t* __restrict__ tokens,
                                                               const float* __restrict__ table,
                                                               float* __restrict__ out, uint32_t d, uint32_t vocab,
                                                               uint32_t* fault) {
    const int32_t id = tokens[blockIdx.x];
    const bool ok = id >= 0 && (uint32_t)id < vocab;
    const float* src = table + (size_t)(ok ? id : 0) * d;
    float* dst = out + (size_t)blockIdx.x * d;
    if (!ok && threadIdx.x == 0) atomicOr(fault, (uint32_t)kFaultBadToken);
    if ((d & 3u) == 0u) {
        for (uint32_t j = threadIdx.x * 4u; j < d; j += blockDim.x * 4u) {
            const float4 v = ok ? *reinterpret_cast<const float4*>(src + j) : make_float4(0.f, 0.f, 0.f, 0.f);
            *reinterpret_cast<float4*>(dst + j) = v;
        }
    } else {
        for (uint32_t j = threadIdx.x; j < d; j += blockDim.x) dst[j] = ok ? src[j] : 0.0f;
    }
}

// ArgMax over the last axis (reduction_argmax.inc:211-235): a scan in index order that replaces
// the best only on a strictly greater value, so ties keep the first index, a NaN is never
// chosen, and a NaN in element 0 wins the row (nothing compares greater than it).  A candidate
// (v, i) beats (bv, bi) if v > bv, or v == bv and i < bi, which gives the same answer in any
// evaluation order.  One workgroup per row; `advance` (optional) are counters the first
// workgroup increments, e.g. the decode position.
__global__ __launch_bounds__(1024) void argmax_rows_kernel(const float* __restrict__ x, uint32_t n,
                                                           int32_t* __restrict__ out, int64_t* advance,
                                                           uint32_t advance_count) {
    const float* row = x + (size_t)blockIdx.x * n;
    const float first = row[0];  // (requested with the row, not after the reduction)
    float bv = -INFINITY;
    uint32_t bi = 0xffffffffu;
    auto offer = [&](float v, uint32_t i) {
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    };
    if ((n & 3u) == 0u && ((uintptr_t)row & 15u) == 0u) {
        // eight loads go out together: one round trip for 32 elements a thread instead of eight (the
        // branches of `offer` keep the compiler from overlapping the loads of a plain loop)
        constexpr uint32_t U = 8;
        const uint32_t pitch = blockDim.x * 4u;
        for (uint32_t j0 = threadIdx.x * 4u; j0 < n; j0 += pitch * U) {
            float4 v[U];
#pragma unroll
            for (uint32_t u = 0; u < U; u++) {
                const uint32_t j = j0 + u * pitch;
                v[u] = j < n ? *reinterpret_cast<const float4*>(row + j) : float4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (uint32_t u = 0; u < U; u++) {
                const uint32_t j = j0 + u * pitch;
                if (j < n) {
                    offer(v[u].x, j);
                    offer(v[u].y, j + 1u);
                    offer(v[u].z, j + 2u);
                    offer(v[u].w, j + 3u);
                }
            }
        }
    } else {
        for (uint32_t j = threadIdx.x; j < n; j += blockDim.x) offer(row[j], j);
    }
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_down(bv, off, 64);
        const uint32_t oi = __shfl_down(bi, off, 64);
        offer(ov, oi);
    }
    __shared__ float wave_v[16];
    __shared__ uint32_t wave_i[16];
    const uint32_t wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    if ((threadIdx.x & 63u) == 0u) {
        wave_v[wave] = bv;
        wave_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < waves; w++) offer(wave_v[w], wave_i[w]);
        out[blockIdx.x] = (first != first || bi == 0xffffffffu) ? 0 : (int32_t)bi;
    }
    if (blockIdx.x == 0 && advance && threadIdx.x < advance_count) advance[threadIdx.x] += 1;
}

}  // namespace
}  // namespace vxhip

using namespace vxhip;

extern "C" {

VxHipStatus vxhip_rmsnorm_prepare_i8(VxHipContext* ctx, const float* input_dev, const float* gain_dev, uint32_t rows,
                                     uint32_t d, double eps, int8_t* prepared_dev, float* row_scales_dev,
                                     float* normalized_dev) {
    if (!ctx || !input_dev || !gain_dev || !prepared_dev || !row_scales_dev || !d || d > 15360u) {
        set_error("rmsnorm_prepare_i8: null argument or row length outside 1..15360");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!rows) return VXHIP_OK;
    if (!device_ready(ctx)) return VXHIP_BACKEND_UNAVAILABLE;
    hipLaunchKernelGGL(rmsnorm_prepare_kernel, dim3(rows), dim3(row_block(rows, d)), d * sizeof(float), ctx->stream,
                       const_cast<float*>(input_dev), (const float*)nullptr, gain_dev, d, eps, prepared_dev,
                       prepared_layout(ctx, rows, d), row_scales_dev, normalized_dev);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus vxhip_add_rmsnorm_prepare_i8(VxHipContext* ctx, float* residual_dev, const float* delta_dev,
                                         const float* gain_dev, uint32_t rows, uint32_t d, double eps,
                                         int8_t* prepared_dev, float* row_scales_dev) {
    if (!ctx || !residual_dev || !delta_dev || !gain_dev || !prepared_dev || !row_scales_dev || !d || d > 15360u) {
        set_error("add_rmsnorm_prepare_i8: null argument or row length outside 1..15360");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!rows) return VXHIP_OK;
    if (!device_ready(ctx)) return VXHIP_BACKEND_UNAVAILABLE;
    hipLaunchKernelGGL(rmsnorm_prepare_kernel, dim3(rows), dim3(row_block(rows, d)), d * sizeof(float), ctx->stream,
                       residual_dev, delta_dev, gain_dev, d, eps, prepared_dev, prepared_layout(ctx, rows, d),
                       row_scales_dev, (float*)nullptr);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus vxhip_swiglu_prepare_i8(VxHipContext* ctx, const float* gate_up_dev, uint32_t rows, uint32_t inter,
                                    int8_t* prepared_dev, float* row_scales_dev, float* activated_dev) {
    if (!ctx || !gate_up_dev || !prepared_dev || !row_scales_dev || !inter || inter > 15360u) {
        set_error("swiglu_prepare_i8: null argument or row length outside 1..15360");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!rows) return VXHIP_OK;
    if (!device_ready(ctx)) return VXHIP_BACKEND_UNAVAILABLE;
    hipLaunchKernelGGL(swiglu_prepare_kernel, dim3(rows), dim3(row_block(rows, inter)), inter * sizeof(float),
                       ctx->stream, gate_up_dev, inter, prepared_dev, prepared_layout(ctx, rows, inter), row_scales_dev,
                       activated_dev);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus vxhip_rope_append_kv(VxHipContext* ctx, const float* qkv_dev, const float* cos_dev, const float* sin_dev,
                                 const int64_t* positions_dev, uint32_t rows, uint32_t t, uint32_t q_heads,
                                 uint32_t kv_heads, uint32_t head_dim, uint32_t max_seq, float* q_out_dev,
                                 float* k_cache_dev, float* v_cache_dev) {
    if (!ctx || !qkv_dev || !cos_dev || !sin_dev || !positions_dev || !q_out_dev || !k_cache_dev || !v_cache_dev ||
        !q_heads || !kv_heads || q_heads % kv_heads || !head_dim || head_dim % 2u || head_dim > 1024u || !max_seq) {
        set_error("rope_append_kv: null argument or unsupported head geometry");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!rows || !t) return VXHIP_OK;
    if (!device_ready(ctx)) return VXHIP_BACKEND_UNAVAILABLE;
    hipLaunchKernelGGL(rope_append_kernel, dim3(rows * t), dim3(256), 0, ctx->stream,
                       qkv_dev, cos_dev, sin_dev, positions_dev, t, q_heads, kv_heads, head_dim, max_seq, q_out_dev,
                       k_cache_dev, v_cache_dev, ctx->fault_dev);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus vxhip_gqa_attention(VxHipContext* ctx, const float* q_dev, const float* k_cache_dev,
                                const float* v_cache_dev, const int64_t* positions_dev, uint32_t rows, uint32_t t,
                                uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim, uint32_t max_seq,
                                float* out_dev) {
    if (!ctx || !q_dev || !k_cache_dev || !v_cache_dev || !positions_dev || !out_dev || !q_heads || !kv_heads ||
        q_heads % kv_heads || !head_dim || head_dim % 4u || !max_seq) {
        set_error("gqa_attention: null argument or unsupported geometry");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!rows || !t) return VXHIP_OK;
    if (!device_ready(ctx)) return VXHIP_BACKEND_UNAVAILABLE;
    const float scale = (float)(1.0 / sqrt((double)head_dim));
    const uint32_t rep = q_heads / kv_heads;
    if (t >= 8u && rep <= kPrefillQueries && head_dim == 128u) {
        // a prompt at head size 128: the matrix-pipe kernel, if its 32 score rows fit
        const size_t lds = ((size_t)kPrefillQueries * ((max_seq + 63u) & ~63u) + (size_t)kPrefillSlots * (128u + 4u)) *
                           sizeof(float);
        if (lds <= 150u * 1024u) {
            static std::atomic<uint64_t> configured{0};
            if (!raise_lds_limit((const void*)gqa_prefill_mfma_kernel, 152 * 1024, configured)) {
                set_error("gqa_attention: the prompt kernel's LDS limit could not be raised");
                return VXHIP_EXECUTION_FAILED;
            }
            const uint32_t tq = kPrefillQueries / rep;
            const dim3 grid(rows * ((t + tq - 1u) / tq), kv_heads);
            hipLaunchKernelGGL(gqa_prefill_mfma_kernel, grid, dim3(256), lds, ctx->stream, q_dev, k_cache_dev,
                               v_cache_dev, positions_dev, t, tq, q_heads, kv_heads, max_seq, scale, out_dev,
                               ctx->fault_dev);
            VXHIP_TRY(hipGetLastError());
            return VXHIP_OK;
        }
    }
    if (t >= 8u && rep <= kPrefillQueries && head_dim <= 256u) {
        // a prompt: tokens share the walk over the cache, as many per workgroup as the LDS holds
        uint32_t tq = kPrefillQueries / rep;
        auto lds_for = [&](uint32_t tokens) {
            const size_t qw = (size_t)tokens * rep;
            return (qw * ((max_seq + 63u) & ~63u) + (size_t)kPrefillSlots * (head_dim + 4u)) * sizeof(float);
        };
        while (tq > 1u && lds_for(tq) > 150u * 1024u) tq /= 2u;
        // two workgroups per compute unit hide each other's staging, if four tokens or more still
        // share a walk then
        if (lds_for(tq) > 78u * 1024u) {
            uint32_t fewer = tq;
            while (fewer > 4u && lds_for(fewer) > 78u * 1024u) fewer /= 2u;
            if (lds_for(fewer) <= 78u * 1024u) tq = fewer;
        }
        if (lds_for(tq) <= 150u * 1024u) {
            static std::atomic<uint64_t> configured{0};
            if (!raise_lds_limit((const void*)gqa_prefill_kernel, 152 * 1024, configured)) {  // (plus its static 128 bytes)
                set_error("gqa_attention: the prompt kernel's LDS limit could not be raised");
                return VXHIP_EXECUTION_FAILED;
            }
            const dim3 grid(rows * ((t + tq - 1u) / tq), kv_heads);
            hipLaunchKernelGGL(gqa_prefill_kernel, grid, dim3(256), lds_for(tq), ctx->stream, q_dev, k_cache_dev,
                               v_cache_dev, positions_dev, t, tq, q_heads, kv_heads, head_dim, max_seq, scale, out_dev,
                               ctx->fault_dev);
            VXHIP_TRY(hipGetLastError());
            return VXHIP_OK;
        }
    }
    const uint32_t together = heads_per_workgroup(rep, rows * t * q_heads, ctx->cu_count);
    const size_t lds = (size_t)together * (9u * head_dim + max_seq) * sizeof(float);
    if (lds > 60u * 1024u) {
        set_error("gqa_attention: head_dim/max_seq too large for the score buffer");
        return VXHIP_INVALID_ARGUMENT;
    }
    const dim3 grid(rows * t, q_heads / together);
    launch_attention<false>(ctx->stream, together, grid, lds, q_dev, const_cast<float*>(k_cache_dev),
                            const_cast<float*>(v_cache_dev), positions_dev, t, q_heads, kv_heads, head_dim, max_seq,
                            scale, out_dev, nullptr, nullptr, ctx->fault_dev);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus vxhip_rope_gqa_attention_decode(VxHipContext* ctx, const float* qkv_dev, const float* cos_dev,
                                            const float* sin_dev, const int64_t* position_dev, uint32_t rows,
                                            uint32_t q_heads, uint32_t kv_heads, uint32_t head_dim,
                                            uint32_t max_seq, float* k_cache_dev, float* v_cache_dev,
                                            float* out_dev) {
    if (!ctx || !qkv_dev || !cos_dev || !sin_dev || !position_dev || !k_cache_dev || !v_cache_dev || !out_dev ||
        !q_heads || !kv_heads || q_heads % kv_heads || !head_dim || head_dim % 4u || head_dim > 1024u || !max_seq) {
        set_error("rope_gqa_attention_decode: null argument or unsupported geometry");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!rows) return VXHIP_OK;
    if (!device_ready(ctx)) return VXHIP_BACKEND_UNAVAILABLE;
    const float scale = (float)(1.0 / sqrt((double)head_dim));
    const uint32_t rep = q_heads / kv_heads;
    const uint32_t together = heads_per_workgroup(rep, rows * q_heads, ctx->cu_count);
    const size_t lds = ((size_t)together * (9u * head_dim + max_seq) + 2u * head_dim) * sizeof(float);
    if (lds > 60u * 1024u) {
        set_error("rope_gqa_attention_decode: head_dim/max_seq too large for the score buffer");
        return VXHIP_INVALID_ARGUMENT;
    }
    const dim3 grid(rows, q_heads / together);
    launch_attention<true>(ctx->stream, together, grid, lds, qkv_dev, k_cache_dev, v_cache_dev, position_dev, 1u,
                           q_heads, kv_heads, head_dim, max_seq, scale, out_dev, cos_dev, sin_dev, ctx->fault_dev);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus vxhip_embedding_gather_f32(VxHipContext* ctx, const int32_t* tokens_dev, const float* table_dev,
                                       uint32_t count, uint32_t d_model, uint32_t vocab, float* out_dev) {
    if (!ctx || !tokens_dev || !table_dev || !out_dev || !d_model || !vocab) {
        set_error("embedding_gather_f32: null argument or empty table");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!count) return VXHIP_OK;
    if (!device_ready(ctx)) return VXHIP_BACKEND_UNAVAILABLE;
    hipLaunchKernelGGL(embedding_gather_kernel, dim3(count), dim3(256), 0, ctx->stream, tokens_dev, table_dev,
                       out_dev, d_model, vocab, ctx->fault_dev);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

VxHipStatus vxhip_argmax_rows_f32(VxHipContext* ctx, const float* input_dev, uint32_t rows, uint32_t n,
                                  int32_t* indices_dev, int64_t* advance_dev, uint32_t advance_count) {
    if (!ctx || !input_dev || !indices_dev || !n || (advance_count && !advance_dev) || advance_count > 64u) {
        set_error("argmax_rows_f32: null argument, empty axis or more than 64 counters");
        return VXHIP_INVALID_ARGUMENT;
    }
    if (!rows) return VXHIP_OK;
    if (!device_ready(ctx)) return VXHIP_BACKEND_UNAVAILABLE;
    const uint32_t block = n >= 4096u ? 1024u : n >= 1024u ? 256u : 64u;
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(rows), dim3(block), 0, ctx->stream, input_dev, n, indices_dev,
                       advance_dev, advance_count);
    VXHIP_TRY(hipGetLastError());
    return VXHIP_OK;
}

}  // extern "C"
