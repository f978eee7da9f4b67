"""Seeded input generators shared by the fixture script and the tests.

The byte streams follow the reference's own test generators so its shapes and
seeds can be replayed: the LCG of native/tests/test_native_isa_parity.c:25-43
and the index formulas of native/tests/test_packed_quant_gemm.c:87-111.
"""
from __future__ import annotations

import numpy as np

DTYPE_U8 = 5
DTYPE_I8 = 6


def np_dtype(code):
    return np.int8 if code == DTYPE_I8 else np.uint8


class LCG:
    """state = state * 1664525 + 1013904223 (mod 2^32)."""

    def __init__(self, seed):
        self.state = np.uint32(seed)

    def words(self, count):
        out = np.empty(count, dtype=np.uint32)
        s = int(self.state)
        for i in range(count):
            s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
            out[i] = s
        self.state = np.uint32(s)
        return out

    def bytes(self, count):
        return (self.words(count) >> np.uint32(24)).astype(np.uint8)


def lcg_bytes_fast(seed, count):
    """Vectorised LCG byte stream (same values as LCG.bytes) for big tensors."""
    # x_{i} = a^i x0 + c (a^i - 1)/(a - 1): build by doubling blocks
    a, c = 1664525, 1013904223
    out = np.empty(count, dtype=np.uint64)
    # sequential over blocks of 4096 with vectorised inner jump table
    block = 4096
    mult = np.empty(block, dtype=np.uint64)
    add = np.empty(block, dtype=np.uint64)
    m, d = 1, 0
    for i in range(block):
        m = (m * a) & 0xFFFFFFFF
        d = (d * a + c) & 0xFFFFFFFF
        mult[i], add[i] = m, d
    s = seed & 0xFFFFFFFF
    pos = 0
    while pos < count:
        nb = min(block, count - pos)
        vals = (mult[:nb] * np.uint64(s) + add[:nb]) & np.uint64(0xFFFFFFFF)
        out[pos:pos + nb] = vals
        s = int(vals[nb - 1])
        pos += nb
    return (out >> np.uint64(24)).astype(np.uint8), s


def isa_parity_case(rows, d_in, d_out, input_dtype, weight_dtype, output_dtype, seed):
    """Inputs of qlinear_case (native/tests/test_native_isa_parity.c:45-91)."""
    g = LCG(seed)
    x = g.bytes(rows * d_in).reshape(rows, d_in).view(np_dtype(input_dtype))
    w = g.bytes(d_out * d_in).reshape(d_out, d_in).view(np_dtype(weight_dtype))
    bias = np.empty(d_out, dtype=np.int32)
    for c in range(d_out):
        bias[c] = int(g.words(1)[0] % 2001) - 1000
    scales = ((1 + np.arange(d_out) % 11) / 1024.0).astype(np.float32)
    zps = np.full(d_out, 0 if weight_dtype == DTYPE_I8 else 131, dtype=np.int32)
    return dict(x=x, w=w, bias=bias, scales=scales, zps=zps, s_in=1.0 / 64.0,
                zp_in=-17 if input_dtype == DTYPE_I8 else 137, s_out=1.0 / 8.0,
                zp_out=-9 if output_dtype == DTYPE_I8 else 129, in_dtype=input_dtype,
                w_dtype=weight_dtype, out_dtype=output_dtype)


def quant_gemm_case(weight_case, input_dtype, weight_dtype, output_dtype, rows, d_in, d_out):
    """Inputs of test_byte_exact_case (native/tests/test_packed_quant_gemm.c:68-131).
    weight_case: 0 bounded (|w|<=64), 1 signed (no -128), 2 full range."""
    idx = np.arange(rows * d_in, dtype=np.uint64)
    x = ((idx * 197 + idx // 3 + 251) & 0xFF).astype(np.uint8).reshape(rows, d_in)
    widx = np.arange(d_out * d_in, dtype=np.uint64)
    if weight_dtype == DTYPE_U8:
        w = ((widx * 89 + 17) & 0xFF).astype(np.uint8)
    elif weight_case == 0:
        w = ((widx * 67 % 129).astype(np.int64) - 64).astype(np.int8).view(np.uint8)
    else:
        w = ((widx * 89 % 255).astype(np.int64) - 127).astype(np.int8).view(np.uint8)
    w = w.copy()
    if weight_dtype == DTYPE_I8:
        w[0] = np.uint8(np.int8(-128 if weight_case == 2 else (-64 if weight_case == 0 else -127)).view(np.uint8))
        w[1] = np.uint8(64 if weight_case == 0 else 127)
    w = w.reshape(d_out, d_in)
    col = np.arange(d_out)
    return dict(x=x.view(np_dtype(input_dtype)), w=w.view(np_dtype(weight_dtype)),
                bias=(col * 31 - 997).astype(np.int32),
                scales=((1 + col % 7) / 512.0).astype(np.float32),
                zps=np.full(d_out, 0 if weight_dtype == DTYPE_I8 else 131, dtype=np.int32),
                s_in=1.0 / 64.0, zp_in=-13 if input_dtype == DTYPE_I8 else 137, s_out=1.0,
                zp_out=-3 if output_dtype == DTYPE_I8 else 129, in_dtype=input_dtype,
                w_dtype=weight_dtype, out_dtype=output_dtype)


def qlinear_random_case(rows, d_in, d_out, seed, input_dtype=DTYPE_I8, weight_dtype=DTYPE_I8,
                        output_dtype=DTYPE_I8, zero_weight_zp=True, s_out=0.05):
    """Benchmark-style QLinear inputs: weights uniform in [-127,127], per-channel
    scales ~U(0.005,0.02), activations clip(round(N(0,30)))."""
    rng = np.random.default_rng(seed)
    if input_dtype == DTYPE_I8:
        x = np.clip(np.rint(rng.normal(0, 30, (rows, d_in))), -127, 127).astype(np.int8)
        zp_in = 0
    else:
        x = rng.integers(0, 256, (rows, d_in)).astype(np.uint8)
        zp_in = 121
    if weight_dtype == DTYPE_I8:
        w = rng.integers(-127, 128, (d_out, d_in)).astype(np.int8)
        zps = np.zeros(d_out, np.int32) if zero_weight_zp else rng.integers(-9, 10, d_out).astype(np.int32)
    else:
        w = rng.integers(0, 256, (d_out, d_in)).astype(np.uint8)
        zps = rng.integers(120, 136, d_out).astype(np.int32)
    scales = rng.uniform(0.005, 0.02, d_out).astype(np.float32)
    bias = rng.integers(-2000, 2001, d_out).astype(np.int32)
    return dict(x=x, w=w, bias=bias, scales=scales, zps=zps, s_in=np.float32(0.02), zp_in=zp_in,
                s_out=np.float32(s_out), zp_out=0 if output_dtype == DTYPE_I8 else 128,
                in_dtype=input_dtype, w_dtype=weight_dtype, out_dtype=output_dtype)


def rowscale_case(rows, d_in, d_out, seed, with_bias=True):
    """Prefill benchmark inputs: A, B uniform in [-127,127], per-token scales
    ~U(0.01,0.05), per-channel ~U(0.002,0.01), output scale 0.05."""
    rng = np.random.default_rng(seed)
    x = rng.integers(-127, 128, (rows, d_in)).astype(np.int8)
    w = rng.integers(-127, 128, (d_out, d_in)).astype(np.int8)
    row_scales = rng.uniform(0.01, 0.05, rows).astype(np.float32)
    # keep outputs inside the byte range so the rounding path is exercised, not just saturation
    scales = (rng.uniform(0.002, 0.01, d_out) / np.sqrt(d_in) * 4).astype(np.float32)
    bias = rng.normal(0, 0.1, d_out).astype(np.float32) if with_bias else None
    return dict(x=x, w=w, row_scales=row_scales, scales=scales, zps=np.zeros(d_out, np.int32),
                bias_f32=bias, s_out=np.float32(0.05), zp_out=0)


def requantize_case(elements, seed, input_dtype=DTYPE_I8, output_dtype=DTYPE_I8):
    """RequantizeLinear inputs: every byte value in random order, two descriptors whose ratio puts a
    good part of the outputs into saturation."""
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, elements).astype(np.uint8).view(np.int8 if input_dtype == DTYPE_I8 else np.uint8)
    s_in, s_out = np.float32(rng.uniform(0.005, 0.08)), np.float32(rng.uniform(0.005, 0.08))
    zp_in = int(rng.integers(-40, 40)) if input_dtype == DTYPE_I8 else int(rng.integers(90, 170))
    zp_out = int(rng.integers(-40, 40)) if output_dtype == DTYPE_I8 else int(rng.integers(90, 170))
    return dict(x=x, s_in=s_in, zp_in=zp_in, s_out=s_out, zp_out=zp_out, in_dtype=input_dtype, out_dtype=output_dtype)


def packed_case(rows, k, n, group, seed, with_bias=True, special_rows=False):
    """PackedLinear inputs: f32 activations, W8 codes, group scales."""
    rng = np.random.default_rng(seed)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    if special_rows and rows >= 5:
        x[1] = 0.0
        x[2] = ((np.arange(k) % 9) - 4).astype(np.float32) * np.float32(2.0 ** -140)
        x[3] = ((np.arange(k) % 255) - 127).astype(np.float32) * np.float32(2.0 ** 120)
        x[4] = np.where(np.arange(k) == 0, 127.0, (np.arange(k) % 19) - 9.5).astype(np.float32)
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    groups = (k + group - 1) // group
    scales = rng.uniform(0.002, 0.01, (n, groups)).astype(np.float32)
    bias = rng.normal(0, 0.1, n).astype(np.float32) if with_bias else None
    return dict(x=x, w=w, scales=scales, bias=bias, group=group, k=k, n=n)


def low_bit(w, bits):
    """int8 weights reduced to the value range of a `bits`-wide code, -2^(bits-1) .. 2^(bits-1)-1
    (arithmetic shift, so signs and the rough distribution are kept)."""
    return (w.astype(np.int8) >> (8 - bits)).astype(np.int8)


def four_bit(w):
    return low_bit(w, 4)


def decode_case(rows, k, n, group, seed):
    """Decode benchmark inputs: int8 activations clip(round(N(0,30))), per-token scales
    ~U(0.01,0.05), weights uniform +-127, per-channel scales ~U(0.002,0.01)
    replicated over the K/G groups (PackedLinear has no whole-row group)."""
    rng = np.random.default_rng(seed)
    a8 = np.clip(np.rint(rng.normal(0, 30, (rows, k))), -127, 127).astype(np.int8)
    row_scales = rng.uniform(0.01, 0.05, rows).astype(np.float32)
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    groups = (k + group - 1) // group
    chan = rng.uniform(0.002, 0.01, n).astype(np.float32)
    scales = np.repeat(chan[:, None], groups, axis=1).copy()
    bias = rng.normal(0, 0.1, n).astype(np.float32)
    return dict(a8=a8, row_scales=row_scales, w=w, scales=scales, bias=bias, group=group, k=k, n=n)
