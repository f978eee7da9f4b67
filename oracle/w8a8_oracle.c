/*
 * CPU restatement of the reference's W8A8 linear arithmetic -- TEST
 * INFRASTRUCTURE ONLY (see w8a8_oracle.h).  Plain scalar C, written to be
 * obviously equal to the cited reference rule rather than fast.  Build with
 * -ffp-contract=off: every f32 operation below is one IEEE rounding.
 */
#include "w8a8_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---- shared scalar helpers ------------------------------------------- */

static int finite_f32(float v) {
    uint32_t bits;
    memcpy(&bits, &v, sizeof bits);
    return ((bits >> 23) & 0xffu) != 0xffu;
}

static int scale_ok(float v) { return finite_f32(v) && v > 0.0f; }

static int byte_dtype(uint32_t dtype) {
    return dtype == VXO_DTYPE_I8 || dtype == VXO_DTYPE_U8;
}

static int zero_point_ok(int32_t zp, uint32_t dtype) {
    if (dtype == VXO_DTYPE_I8) return zp >= -128 && zp <= 127;
    if (dtype == VXO_DTYPE_U8) return zp >= 0 && zp <= 255;
    return 0;
}

static int32_t load_byte(const void* p, uint32_t dtype, size_t i) {
    return dtype == VXO_DTYPE_I8 ? (int32_t)((const int8_t*)p)[i]
                                 : (int32_t)((const uint8_t*)p)[i];
}

static void store_byte(void* p, uint32_t dtype, size_t i, int32_t v) {
    if (dtype == VXO_DTYPE_I8) ((int8_t*)p)[i] = (int8_t)v;
    else ((uint8_t*)p)[i] = (uint8_t)v;
}

/* ---- w8a8_affine.h ---------------------------------------------------- */

int32_t vxo_round_ties_even(float value) {
    /* floor, then decide on the fractional part; exact ties go to even */
    const float fl = floorf(value);
    const int32_t lo = (int32_t)fl;
    const float frac = value - (float)lo;
    if (frac < 0.5f) return lo;
    if (frac > 0.5f) return lo + 1;
    return (lo % 2 == 0) ? lo : lo + 1;
}

int32_t vxo_requantize(float t, int32_t minimum, int32_t maximum,
                       int32_t nan_value) {
    if (t != t) return nan_value;
    if (t <= (float)minimum) return minimum;
    if (t >= (float)maximum) return maximum;
    return vxo_round_ties_even(t);
}

float vxo_transform_accumulator(int64_t accumulator, float multiplier,
                                int32_t output_zero_point) {
    volatile float scaled = (float)accumulator * multiplier; /* rounding 1 */
    volatile float shifted = scaled + (float)output_zero_point; /* rounding 2 */
    return shifted;
}

int vxo_multiplier(float input_scale, float weight_scale, float output_scale,
                   float* multiplier_out) {
    volatile float product, multiplier;
    if (!multiplier_out || !scale_ok(input_scale) || !scale_ok(weight_scale) ||
        !scale_ok(output_scale))
        return 0;
    product = input_scale * weight_scale;   /* f32(s_x * s_w) */
    multiplier = product / output_scale;    /* f32(. / s_y)   */
    if (!scale_ok(multiplier)) return 0;
    *multiplier_out = multiplier;
    return 1;
}

/* ---- QLinear (requantizing epilogue) ---------------------------------- */

int vxo_qlinear_i8u8(const void* input, const void* weight,
                     const int32_t* bias, const float* weight_scales,
                     const int32_t* weight_zero_points, void* output,
                     int32_t* accumulators, uint32_t rows, uint32_t d_in,
                     uint32_t d_out, float input_scale,
                     int32_t input_zero_point, float output_scale,
                     int32_t output_zero_point, uint32_t input_dtype,
                     uint32_t weight_dtype, uint32_t output_dtype) {
    if (!input || !weight || !bias || !weight_scales || !weight_zero_points ||
        !output || !rows || !d_in || !d_out || !byte_dtype(input_dtype) ||
        !byte_dtype(weight_dtype) || !byte_dtype(output_dtype) ||
        !scale_ok(input_scale) || !scale_ok(output_scale) ||
        !zero_point_ok(input_zero_point, input_dtype) ||
        !zero_point_ok(output_zero_point, output_dtype))
        return 0;
    const int32_t lo = output_dtype == VXO_DTYPE_I8 ? -128 : 0;
    const int32_t hi = output_dtype == VXO_DTYPE_I8 ? 127 : 255;
    /* whole descriptor is validated before the first output byte */
    for (uint32_t n = 0; n < d_out; n++) {
        float m;
        if (!zero_point_ok(weight_zero_points[n], weight_dtype) ||
            !vxo_multiplier(input_scale, weight_scales[n], output_scale, &m))
            return 0;
    }
    for (uint32_t r = 0; r < rows; r++) {
        for (uint32_t n = 0; n < d_out; n++) {
            int64_t acc = bias[n];
            float mult;
            vxo_multiplier(input_scale, weight_scales[n], output_scale, &mult);
            for (uint32_t k = 0; k < d_in; k++) {
                const int32_t x =
                    load_byte(input, input_dtype, (size_t)r * d_in + k) -
                    input_zero_point;
                const int32_t w =
                    load_byte(weight, weight_dtype, (size_t)n * d_in + k) -
                    weight_zero_points[n];
                acc += (int64_t)x * (int64_t)w;
                /* every prefix must stay inside int32 */
                if (acc < INT32_MIN || acc > INT32_MAX) return 0;
            }
            if (accumulators) accumulators[(size_t)r * d_out + n] = (int32_t)acc;
            const float t =
                vxo_transform_accumulator(acc, mult, output_zero_point);
            store_byte(output, output_dtype, (size_t)r * d_out + n,
                       vxo_requantize(t, lo, hi, output_zero_point));
        }
    }
    return 1;
}

int vxo_qlinear_rowscale_i8u8(const int8_t* input, const void* weight,
                              const int32_t* bias_i32, const float* bias_f32,
                              const float* weight_scales,
                              const int32_t* weight_zero_points, void* output,
                              int32_t* accumulators, uint32_t rows,
                              uint32_t d_in, uint32_t d_out,
                              const float* row_scales, float output_scale,
                              int32_t output_zero_point, uint32_t weight_dtype,
                              uint32_t output_dtype) {
    if (!input || !weight || !weight_scales || !weight_zero_points ||
        !row_scales || !output || !rows || !d_in || !d_out ||
        !byte_dtype(weight_dtype) || !byte_dtype(output_dtype) ||
        !scale_ok(output_scale) ||
        !zero_point_ok(output_zero_point, output_dtype))
        return 0;
    const int32_t lo = output_dtype == VXO_DTYPE_I8 ? -128 : 0;
    const int32_t hi = output_dtype == VXO_DTYPE_I8 ? 127 : 255;
    for (uint32_t r = 0; r < rows; r++)
        for (uint32_t n = 0; n < d_out; n++) {
            float m;
            if (!zero_point_ok(weight_zero_points[n], weight_dtype) ||
                !vxo_multiplier(row_scales[r], weight_scales[n], output_scale, &m))
                return 0;
        }
    /* the real-valued bias is part of the descriptor: a value that is not finite declines the call */
    if (bias_f32)
        for (uint32_t n = 0; n < d_out; n++)
            if (!finite_f32(bias_f32[n])) return 0;
    for (uint32_t r = 0; r < rows; r++) {
        for (uint32_t n = 0; n < d_out; n++) {
            /* the reference loop with rows = 1 and input_scale = row_scales[r] */
            int64_t acc = bias_i32 ? bias_i32[n] : 0;
            float mult;
            vxo_multiplier(row_scales[r], weight_scales[n], output_scale, &mult);
            for (uint32_t k = 0; k < d_in; k++) {
                const int32_t x = input[(size_t)r * d_in + k];
                const int32_t w =
                    load_byte(weight, weight_dtype, (size_t)n * d_in + k) -
                    weight_zero_points[n];
                acc += (int64_t)x * (int64_t)w;
                if (acc < INT32_MIN || acc > INT32_MAX) return 0;
            }
            if (accumulators) accumulators[(size_t)r * d_out + n] = (int32_t)acc;
            float t = vxo_transform_accumulator(acc, mult, output_zero_point);
            if (bias_f32) {
                /* extension (no reference counterpart): the real-valued bias in
                 * output units, added as one more separately rounded f32 term */
                volatile float in_output_units = bias_f32[n] / output_scale;
                volatile float shifted = t + in_output_units;
                t = shifted;
            }
            store_byte(output, output_dtype, (size_t)r * d_out + n,
                       vxo_requantize(t, lo, hi, output_zero_point));
        }
    }
    return 1;
}

/* ---- PackedLinear W8 under DYNAMIC_I8 --------------------------------- */

int32_t vxo_packed_round_i8(float value) {
    if (value >= 127.0f) return 127;
    if (value <= -127.0f) return -127;
    int32_t q = (int32_t)value; /* toward zero */
    const float rem = value - (float)q;
    if (rem > 0.5f || (rem == 0.5f && (q & 1))) q++;
    if (rem < -0.5f || (rem == -0.5f && (q & 1))) q--;
    return q;
}

int vxo_packed_prepare_i8(const float* input, uint32_t k, int8_t* prepared,
                          float* scale) {
    float maximum = 0.0f;
    int finite = 1;
    for (uint32_t j = 0; j < k; j++) {
        const float v = input[j];
        if (!finite_f32(v)) { finite = 0; break; }
        const float a = v < 0.0f ? -v : v;
        if (a > maximum) maximum = a;
    }
    float s = maximum == 0.0f ? 1.0f : maximum / 127.0f;
    if (s < 0x1p-126f) s = 0x1p-126f;
    *scale = s;
    if (!finite) {
        memset(prepared, 0, k);
        return 0;
    }
    for (uint32_t j = 0; j < k; j++) {
        const float ratio = input[j] / s; /* true f32 division */
        prepared[j] = (int8_t)vxo_packed_round_i8(ratio);
    }
    return 1;
}

static int group_size_ok(uint32_t g) {
    return g == 32u || g == 64u || g == 128u || g == 256u;
}

/* src/kernels/packed_linear_ops.inc:472-480: codes are offset by half their
 * range (W8 128, W4 8, W2 2), little-endian within their I32 word; W3 is a
 * dense bitstream over the row (:249-254), offset 4. */
static int32_t packed_code(const uint32_t* row_words, uint32_t k, uint32_t bits) {
    if (bits == 4u)
        return (int32_t)((row_words[k / 8u] >> ((k % 8u) * 4u)) & 15u) - 8;
    if (bits == 2u)
        return (int32_t)((row_words[k / 16u] >> ((k % 16u) * 2u)) & 3u) - 2;
    if (bits == 3u) {
        const uint64_t bit = (uint64_t)k * 3u;
        const uint32_t shift = (uint32_t)(bit % 32u);
        uint32_t value = row_words[bit / 32u] >> shift;
        if (shift > 29u) value |= row_words[bit / 32u + 1u] << (32u - shift);
        return (int32_t)(value & 7u) - 4;
    }
    return (int32_t)((row_words[k / 4u] >> ((k % 4u) * 8u)) & 255u) - 128;
}

/* src/kernels/packed_linear_ops.inc:246-248 */
static uint32_t packed_words(uint32_t k, uint32_t bits) {
    return (k / 32u) * bits + ((k % 32u) * bits + 31u) / 32u;
}

int vxo_packed_linear_a8_bits(const int8_t* activation, const float* row_scales,
                              const uint8_t* row_finite, const uint32_t* packed,
                              const float* scales, const float* bias,
                              float* output, int32_t* accumulators,
                              uint64_t rows, uint32_t k, uint32_t n,
                              uint32_t group_size, uint32_t weight_bits) {
    if (!activation || !row_scales || !packed || !scales || !output || !k ||
        !n || !group_size_ok(group_size) ||
        (weight_bits != 2u && weight_bits != 3u && weight_bits != 4u && weight_bits != 8u))
        return -1;
    const uint32_t words = packed_words(k, weight_bits);
    const uint32_t groups = (k + group_size - 1u) / group_size;
    for (uint64_t r = 0; r < rows; r++) {
        const int8_t* a = activation + r * k;
        const float as = row_scales[r];
        for (uint32_t o = 0; o < n; o++) {
            if (row_finite && !row_finite[r]) {
                output[r * n + o] = nanf("");
                if (accumulators) accumulators[r * n + o] = 0;
                continue;
            }
            const uint32_t* w = packed + (uint64_t)o * words;
            float sum = 0.0f;
            int64_t total = 0;
            for (uint32_t g = 0; g < groups; g++) {
                const uint32_t begin = g * group_size;
                const uint32_t end = begin + group_size < k ? begin + group_size : k;
                int32_t dot = 0;
                for (uint32_t j = begin; j < end; j++)
                    dot += (int32_t)a[j] * packed_code(w, j, weight_bits);
                total += dot;
                const float group_scale = as * scales[(uint64_t)o * groups + g];
                const float term = (float)dot * group_scale;
                sum = sum + term; /* ascending group order */
            }
            if (accumulators) accumulators[r * n + o] = (int32_t)total;
            output[r * n + o] = sum + (bias ? bias[o] : 0.0f);
        }
    }
    return 0;
}

int vxo_packed_linear_a8(const int8_t* activation, const float* row_scales,
                         const uint8_t* row_finite, const uint32_t* packed,
                         const float* scales, const float* bias, float* output,
                         int32_t* accumulators, uint64_t rows, uint32_t k,
                         uint32_t n, uint32_t group_size) {
    return vxo_packed_linear_a8_bits(activation, row_scales, row_finite, packed,
                                     scales, bias, output, accumulators, rows,
                                     k, n, group_size, 8u);
}

int vxo_packed_linear_forward_bits(const float* input, const uint32_t* packed,
                                   const float* scales, const float* bias,
                                   float* output, uint64_t rows, uint32_t k,
                                   uint32_t n, uint32_t group_size,
                                   uint32_t weight_bits) {
    if (!input || !k || !n || !group_size_ok(group_size)) return -1;
    int8_t* prepared = (int8_t*)malloc(k);
    if (!prepared) return -1;
    int status = 0;
    for (uint64_t r = 0; r < rows && status == 0; r++) {
        float as;
        const uint8_t finite =
            (uint8_t)vxo_packed_prepare_i8(input + r * k, k, prepared, &as);
        status = vxo_packed_linear_a8_bits(prepared, &as, &finite, packed,
                                           scales, bias, output + r * n, NULL,
                                           1u, k, n, group_size, weight_bits);
    }
    free(prepared);
    return status;
}

/* vx_packed_linear_forward with its output window (packed_linear_ops.inc:1550-1553:
 * units are elements of the row-major output; unit_count 0 = rows * n; a window
 * past the end is refused; :1555 the rows first / n .. ceil((first + units) / n);
 * :1593-1596 per row the columns [begin, end) that lie inside the window).  Every
 * element outside the window keeps its value. */
int vxo_packed_linear_forward_window(const float* input, const uint32_t* packed,
                                     const float* scales, const float* bias,
                                     float* output, uint64_t rows, uint32_t k,
                                     uint32_t n, uint32_t group_size,
                                     uint32_t weight_bits, uint64_t first_unit,
                                     uint64_t unit_count) {
    if (!input || !k || !n || !group_size_ok(group_size)) return -1;
    const uint64_t first = first_unit;
    const uint64_t units = unit_count ? unit_count : rows * n;
    if (first > rows * n || units > rows * n - first) return -1;
    int8_t* prepared = (int8_t*)malloc(k);
    float* whole = (float*)malloc((size_t)n * sizeof(float));
    if (!prepared || !whole) {
        free(prepared);
        free(whole);
        return -1;
    }
    int status = 0;
    for (uint64_t row = first / n; row < (first + units + n - 1u) / n && status == 0; row++) {
        float as;
        const uint8_t finite =
            (uint8_t)vxo_packed_prepare_i8(input + row * k, k, prepared, &as);
        status = vxo_packed_linear_a8_bits(prepared, &as, &finite, packed, scales,
                                           bias, whole, NULL, 1u, k, n,
                                           group_size, weight_bits);
        const uint32_t begin = first > row * n ? (uint32_t)(first - row * n) : 0u;
        const uint32_t end = first + units < (row + 1u) * n
                                 ? (uint32_t)(first + units - row * n) : n;
        for (uint32_t c = begin; c < end && status == 0; c++)
            output[row * n + c] = whole[c];
    }
    free(prepared);
    free(whole);
    return status;
}

int vxo_packed_linear_forward(const float* input, const uint32_t* packed,
                              const float* scales, const float* bias,
                              float* output, uint64_t rows, uint32_t k,
                              uint32_t n, uint32_t group_size) {
    return vxo_packed_linear_forward_bits(input, packed, scales, bias, output,
                                          rows, k, n, group_size, 8u);
}

/* ---- Quantize / Dequantize boundaries --------------------------------- */

int vxo_quantize_linear(const float* input, uint32_t elements, void* output,
                        float scale, int32_t zero_point, uint32_t dtype) {
    if (!input || !output || !byte_dtype(dtype) || !scale_ok(scale) ||
        !zero_point_ok(zero_point, dtype))
        return 0;
    const int32_t lo = dtype == VXO_DTYPE_I8 ? -128 : 0;
    const int32_t hi = dtype == VXO_DTYPE_I8 ? 127 : 255;
    for (uint32_t i = 0; i < elements; i++) {
        float v = input[i];
        int32_t q;
        if (v != v) {
            q = zero_point;
        } else {
            const float ratio = v / scale;
            v = ratio + (float)zero_point;
            if (v <= (float)lo) q = lo;
            else if (v >= (float)hi) q = hi;
            else if (!finite_f32(v)) q = v < 0.0f ? lo : hi;
            else q = vxo_round_ties_even(v);
        }
        store_byte(output, dtype, i, q);
    }
    return 1;
}

int vxo_dequantize_linear(const void* input, uint32_t elements, float scale,
                          int32_t zero_point, uint32_t dtype, float* output) {
    if (!input || !output || !byte_dtype(dtype)) return 0;
    for (uint32_t i = 0; i < elements; i++) {
        const double centered = (double)load_byte(input, dtype, i) - (double)zero_point;
        output[i] = (float)(centered * (double)scale);
    }
    return 1;
}

/* RequantizeLinear: a byte tensor moved from one per-tensor descriptor to another
 * (native/src/kernels/portable_inference_kernels.inc:2437-2463).  multiplier = f32(s_in / s_out);
 * q' = saturate(ties-to-even(f32(f32(f32(q - zp_in) * multiplier) + f32(zp_out)))): the product and
 * the sum are rounded separately.  Declines a scale that is not finite and positive, a zero point
 * outside its type, and a multiplier that is not finite and positive. */
int vxo_requantize_linear(const void* input, uint32_t elements, float input_scale,
                          int32_t input_zero_point, float output_scale, int32_t output_zero_point,
                          uint32_t input_dtype, uint32_t output_dtype, void* output) {
    if (!input || !output || !elements || !byte_dtype(input_dtype) || !byte_dtype(output_dtype) ||
        !scale_ok(input_scale) || !scale_ok(output_scale) || !zero_point_ok(input_zero_point, input_dtype) ||
        !zero_point_ok(output_zero_point, output_dtype))
        return 0;
    const volatile float multiplier = input_scale / output_scale;
    if (!scale_ok(multiplier)) return 0;
    const int32_t lo = output_dtype == VXO_DTYPE_I8 ? -128 : 0;
    const int32_t hi = output_dtype == VXO_DTYPE_I8 ? 127 : 255;
    for (uint32_t i = 0; i < elements; i++) {
        const float centered = (float)(load_byte(input, input_dtype, i) - input_zero_point);
        const volatile float scaled = centered * multiplier;
        const volatile float transformed = scaled + (float)output_zero_point;
        store_byte(output, output_dtype, i, vxo_requantize(transformed, lo, hi, output_zero_point));
    }
    return 1;
}

/* ---- PTQ rules used to synthesise inputs ------------------------------ */

static double round_ties_even_f64(double v) {
    const double lo = floor(v);
    const double frac = v - lo;
    if (frac < 0.5) return lo;
    if (frac > 0.5) return lo + 1.0;
    return ((int64_t)lo % 2 == 0) ? lo : lo + 1.0;
}

int vxo_ptq_symmetric_scale(const float* values, int64_t count, float* scale) {
    if (!values || count <= 0 || !scale) return -1;
    double magnitude = 0.0;
    for (int64_t i = 0; i < count; i++) {
        if (!finite_f32(values[i])) return -1;
        const double a = fabs((double)values[i]);
        if (a > magnitude) magnitude = a;
    }
    const float s = (float)(magnitude == 0.0 ? 1.0 : magnitude / 127.0);
    if (finite_f32(s) && s > 0.0f) { *scale = s; return 0; }
    if (s == 0.0f) { *scale = 0x1p-126f; return 0; }
    return -1;
}

int vxo_ptq_quantize_i8(const float* values, int64_t count, float scale,
                        int32_t zero_point, int8_t* output) {
    if (!values || !output || !scale_ok(scale) || zero_point < -128 ||
        zero_point > 127)
        return -1;
    for (int64_t i = 0; i < count; i++) {
        if (!finite_f32(values[i])) return -1;
        double q = round_ties_even_f64((double)values[i] / (double)scale +
                                       (double)zero_point);
        if (q < -128.0) q = -128.0;
        if (q > 127.0) q = 127.0;
        output[i] = (int8_t)q;
    }
    return 0;
}

int vxo_ptq_pack_bias_i32(const float* values, int32_t count,
                          float input_scale, const float* weight_scales,
                          int32_t* output) {
    if (count < 0 || (count > 0 && (!values || !weight_scales || !output)) ||
        !scale_ok(input_scale))
        return -1;
    for (int pass = 0; pass < 2; pass++) {
        for (int32_t i = 0; i < count; i++) {
            if (!finite_f32(values[i]) || !scale_ok(weight_scales[i])) return -1;
            const float acc_scale = input_scale * weight_scales[i];
            if (!scale_ok(acc_scale)) return -1;
            const float ratio = values[i] / acc_scale;
            if (!finite_f32(ratio)) return -1;
            const double q = round_ties_even_f64((double)ratio);
            if (q < (double)INT32_MIN || q > (double)INT32_MAX) return -1;
            if (pass) output[i] = (int32_t)q; /* nothing is written on failure */
        }
    }
    return 0;
}

void vxo_pack_w8_words(const int8_t* weight, uint32_t n, uint32_t k,
                       uint32_t* packed) {
    const uint32_t words = (k + 3u) / 4u;
    for (uint32_t o = 0; o < n; o++) {
        for (uint32_t w = 0; w < words; w++) {
            uint32_t word = 0;
            for (uint32_t b = 0; b < 4u; b++) {
                const uint32_t j = w * 4u + b;
                /* a code of 128 is the value zero, which pads the tail */
                const uint32_t code =
                    j < k ? (uint32_t)((int32_t)weight[(uint64_t)o * k + j] + 128) : 128u;
                word |= code << (8u * b);
            }
            packed[(uint64_t)o * words + w] = word;
        }
    }
}

void vxo_pack_w4_words(const int8_t* weight, uint32_t n, uint32_t k,
                       uint32_t* packed) {
    const uint32_t words = packed_words(k, 4u);
    for (uint32_t o = 0; o < n; o++) {
        for (uint32_t w = 0; w < words; w++) {
            uint32_t word = 0;
            for (uint32_t b = 0; b < 8u; b++) {
                const uint32_t j = w * 8u + b;
                /* a code of 8 is the value zero, which pads the tail */
                const uint32_t code =
                    j < k ? (uint32_t)((int32_t)weight[(uint64_t)o * k + j] + 8) & 15u : 8u;
                word |= code << (4u * b);
            }
            packed[(uint64_t)o * words + w] = word;
        }
    }
}

/* ---- decoder glue either side of the linears --------------------------- */

void vxo_embedding_f32(const int32_t* tokens, const float* table, float* out,
                       uint32_t count, uint32_t d_model) {
    for (uint32_t i = 0; i < count; i++)
        memcpy(out + (uint64_t)i * d_model,
               table + (uint64_t)tokens[i] * d_model, sizeof(float) * d_model);
}

void vxo_argmax_rows_f32(const float* input, uint32_t rows, uint32_t n,
                         int32_t* indices) {
    for (uint32_t r = 0; r < rows; r++) {
        const float* x = input + (uint64_t)r * n;
        double best = x[0];
        int32_t best_index = 0;
        for (uint32_t i = 1; i < n; i++) {
            const double v = x[i];
            if (v > best) { /* strict: first index on ties, NaN never greater */
                best = v;
                best_index = (int32_t)i;
            }
        }
        indices[r] = best_index;
    }
}

void vxo_pack_low_bit_words(const int8_t* weight, uint32_t n, uint32_t k,
                            uint32_t bits, uint32_t* packed) {
    const uint32_t words = packed_words(k, bits);
    const uint32_t offset = 1u << (bits - 1u), mask = (1u << bits) - 1u;
    for (uint32_t o = 0; o < n; o++) {
        uint32_t* row = packed + (uint64_t)o * words;
        for (uint32_t w = 0; w < words; w++) row[w] = 0;
        /* every code slot of the row's words, absent elements as the code of zero */
        const uint32_t slots = (uint32_t)(((uint64_t)words * 32u) / bits);
        for (uint32_t j = 0; j < slots; j++) {
            const uint32_t code =
                (j < k ? (uint32_t)((int32_t)weight[(uint64_t)o * k + j] + (int32_t)offset) : offset) & mask;
            const uint64_t bit = (uint64_t)j * bits;
            const uint32_t shift = (uint32_t)(bit % 32u);
            row[bit / 32u] |= code << shift;
            if (shift + bits > 32u) row[bit / 32u + 1u] |= code >> (32u - shift);
        }
    }
}
