"""Writes tests/golden/reference_vectors.json from the reference's own C kernels.

Run in a container that has the reference tree:  the kernels are compiled from
their sources by `make -C oracle ref` into oracle/_ref/libvxref.so, and every
expected value below is an output of those kernels (qlinear_i8u8,
vx_qlinear_i8u8_native, vx_qlinear_i8u8_packed, vx_llm_forward_f32,
volvoxai_ptq_pack_bias_i32, requantize_linear_i8u8; for the decoder glue rmsnorm_f32, silu_f32, mul_f32,
cross_sdpa_gqa_f32 and the RotaryEmbedding operator) on the seeded inputs of tests/_cases.py and tests/_glue_defs.py.  Large
outputs are stored as a SHA-256 plus a leading slice; small ones whole.

    python tests/golden/make_reference_vectors.py
"""
from __future__ import annotations

import hashlib
import json
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import _cases as cases  # noqa: E402
import _glue_defs as glue  # noqa: E402
from oracle.pyoracle import Oracle, Reference  # noqa: E402

I8, U8 = cases.DTYPE_I8, cases.DTYPE_U8


def digest(a: np.ndarray) -> dict:
    a = np.ascontiguousarray(a)
    head = a.reshape(-1)[:32]
    if a.dtype == np.float32:
        head_list = [int(v) for v in head.view(np.uint32)]
    else:
        head_list = [int(v) for v in head]
    return {"sha256": hashlib.sha256(a.tobytes()).hexdigest(), "shape": list(a.shape),
            "dtype": str(a.dtype), "head": head_list}


QLINEAR_CASES = (
    [("isa_parity", dict(rows=5, d_in=192, d_out=33, input_dtype=i, weight_dtype=w, output_dtype=o,
                         seed=100 + ii * 17 + wi * 7 + oi))
     for ii, i in enumerate((I8, U8)) for wi, w in enumerate((I8, U8)) for oi, o in enumerate((I8, U8))]
    + [("isa_parity", dict(rows=3, d_in=65, d_out=17, input_dtype=U8, weight_dtype=I8, output_dtype=I8, seed=911))]
    + [("quant_gemm", dict(weight_case=2, input_dtype=i, weight_dtype=w, output_dtype=o, rows=113, d_in=37, d_out=257))
       for i in (I8, U8) for w in (I8, U8) for o in (I8, U8)]
    + [("quant_gemm", dict(weight_case=c, input_dtype=U8, weight_dtype=I8, output_dtype=I8, rows=113, d_in=37, d_out=257))
       for c in (0, 1)]
    + [("random", dict(rows=r, d_in=k, d_out=n, seed=s, input_dtype=i, weight_dtype=w, output_dtype=o,
                       zero_weight_zp=z))
       for (r, k, n, s, i, w, o, z) in [
           (8, 256, 256, 1, I8, I8, I8, True),       # the CPU-runnable benchmark shape
           (1, 4096, 512, 2, I8, I8, I8, True),      # decode shaped
           (16, 4096, 256, 3, I8, I8, I8, True),
           (16, 1000, 130, 4, U8, U8, U8, False),
           (40, 512, 384, 5, I8, I8, I8, True),      # GEMM path, 128x128 tiles
           (300, 640, 520, 6, I8, I8, U8, False),    # GEMM with weight zero points
           (257, 136, 72, 7, U8, I8, I8, True),
           (64, 48, 40, 8, I8, U8, I8, False),
       ]]
)

ROWSCALE_CASES = [dict(rows=r, d_in=k, d_out=n, seed=s, with_bias=b) for (r, k, n, s, b) in [
    (4, 256, 64, 21, True), (16, 1024, 96, 22, False), (48, 512, 256, 23, True), (130, 384, 200, 24, True)]]

PACKED_CASES = [dict(rows=r, k=k, n=n, group=g, seed=s, with_bias=b, special_rows=sp)
                for (r, k, n, g, s, b, sp) in [
    (3, 96, 5, 32, 31, True, False), (11, 1283, 19, 128, 32, True, True), (11, 257, 13, 64, 33, False, True),
    (8, 256, 256, 32, 34, True, False), (8, 256, 256, 64, 35, True, False),
    (8, 256, 256, 128, 36, True, False), (8, 256, 256, 256, 37, True, False),
    (1, 4096, 256, 128, 38, True, False), (16, 4096, 128, 128, 39, True, False),
    (5, 1024, 64, 256, 40, True, True), (40, 512, 160, 128, 41, True, True),
    (70, 320, 96, 32, 42, True, False), (33, 1280, 48, 64, 43, False, False),
    (200, 768, 136, 256, 44, True, True)]]


# Output windows (VxLLMOpArgs.first_unit / unit_count): the reference's own window list for 11 rows of n
# (native/tests/test_packed_linear_i8.c:263-265) and its small case (:186-187), on seeded inputs; the whole
# output array, pre-filled with the guard value 12345, is what gets digested.
WINDOW_GUARD = 12345.0
PACKED_WINDOW_CASES = [dict(rows=11, k=k, n=n, group=g, seed=s, bits=b) for (k, n, g, s, b) in [
    (257, 19, 64, 61, 8), (1283, 5, 128, 62, 8), (320, 13, 32, 63, 4), (96, 1, 32, 64, 8)]]


def window_list(rows, n):
    firsts = [0, 1, n - 1, n + 2, n, 3]
    counts = [0, rows * n - 2, 4 * n + 2, 3 * n - 2, 8 * n, 14]
    return [(f, c) for f, c in zip(firsts, counts) if f <= rows * n and (c or rows * n) <= rows * n - f]


REQUANTIZE_CASES = [dict(elements=e, seed=s, input_dtype=i, output_dtype=o) for (e, s, i, o) in [
    (4096, 51, I8, I8), (4096, 52, I8, U8), (4096, 53, U8, I8), (4096, 54, U8, U8), (100003, 55, I8, I8), (7, 56, U8, I8)]]


def build_case(kind, params):
    if kind == "isa_parity":
        return cases.isa_parity_case(**params)
    if kind == "quant_gemm":
        return cases.quant_gemm_case(**params)
    return cases.qlinear_random_case(**params)


def main():
    ref = Reference()
    orc = Oracle()
    out = {"_comment": "Outputs of the reference's C kernels on the seeded inputs of tests/_cases.py; "
                       "written by tests/golden/make_reference_vectors.py.",
           "qlinear": [], "rowscale": [], "packed": [], "packed_w4": [], "packed_w3": [], "packed_w2": [],
           "requantize": [], "packed_window": [], "glue": {}}
    for kind, params in QLINEAR_CASES:
        c = build_case(kind, params)
        args = (c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"],
                c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"])
        ok, y = ref.qlinear_portable(*args)
        ok2, y2 = ref.qlinear_native(*args)
        assert ok == ok2 == 1 and (y == y2).all(), (kind, params)
        packed = ref.pack_q8(c["w"], c["w_dtype"])
        ok3, y3 = ref.qlinear_packed(c["x"], packed, c["bias"], c["scales"], c["zps"], *args[5:])
        assert ok3 == 1 and (y == y3).all(), (kind, params)
        out["qlinear"].append({"kind": kind, "params": params, "expected": digest(y)})
    for params in ROWSCALE_CASES:
        c = cases.rowscale_case(**params)
        rows = c["x"].shape[0]
        ys = []
        for r in range(rows):  # the reference has only the per-tensor form: one call per row
            bias_row = np.zeros(c["w"].shape[0], np.int32)
            ok, y = ref.qlinear_portable(c["x"][r:r + 1], c["w"], bias_row, c["scales"], c["zps"],
                                         c["row_scales"][r], 0, c["s_out"], c["zp_out"], I8, I8, I8)
            assert ok == 1
            ys.append(y)
        out["rowscale"].append({"params": params, "expected_without_bias": digest(np.concatenate(ys))})
    for params in PACKED_CASES:
        c = cases.packed_case(**params)
        words = orc.pack_w8_words(c["w"])
        st, y = ref.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"])
        assert st == 0
        out["packed"].append({"params": params, "expected": digest(y)})
    for params in PACKED_CASES:  # the same inputs with the weights reduced to four bits
        c = cases.packed_case(**params)
        words = orc.pack_w4_words(cases.four_bit(c["w"]))
        st, y = ref.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=4)
        assert st == 0
        out["packed_w4"].append({"params": params, "expected": digest(y)})
        for bits in (3, 2):
            words = orc.pack_low_bit_words(cases.low_bit(c["w"], bits), bits)
            st, y = ref.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=bits)
            assert st == 0
            out[f"packed_w{bits}"].append({"params": params, "expected": digest(y)})
    for params in PACKED_WINDOW_CASES:
        bits = params["bits"]
        c = cases.packed_case(**{k: v for k, v in params.items() if k != "bits"}, special_rows=True)
        words = orc.pack_w8_words(c["w"]) if bits == 8 else orc.pack_w4_words(cases.four_bit(c["w"]))
        for first, count in window_list(params["rows"], params["n"]):
            y = np.full((params["rows"], params["n"]), WINDOW_GUARD, np.float32)
            st, _ = ref.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=bits,
                                      first_unit=first, unit_count=count, out=y)
            assert st == 0
            out["packed_window"].append({"params": params, "first_unit": first, "unit_count": count, "expected": digest(y)})
        # a window that does not fit is refused and nothing is written
        y = np.full((params["rows"], params["n"]), WINDOW_GUARD, np.float32)
        st, _ = ref.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=bits,
                                  first_unit=2, unit_count=params["rows"] * params["n"] - 1, out=y)
        assert st == -1 and (y == WINDOW_GUARD).all()
    for params in REQUANTIZE_CASES:
        c = cases.requantize_case(**params)
        ok, y = ref.requantize_linear(c["x"], c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], c["in_dtype"], c["out_dtype"])
        assert ok == 1
        out["requantize"].append({"params": params, "expected": digest(y)})
    # The decoder glue: rmsnorm_f32, silu_f32 + mul_f32, the RotaryEmbedding operator of vx_llm_forward_f32 and
    # cross_sdpa_gqa_f32 on the seeded inputs of tests/_glue_defs.py.  Outputs that a kernel is held to bit for
    # bit are digested; those compared under a tolerance are stored whole (as their f32 bit patterns).
    def bits(a):
        return [int(v) for v in np.ascontiguousarray(a).reshape(-1).view(np.uint32)]

    g = out["glue"]
    g["rmsnorm"] = []
    for params in glue.RMSNORM_CASES:
        x, gain = glue.rmsnorm_case(**params)
        g["rmsnorm"].append({"params": params, "eps": glue.EPS, "expected": digest(ref.rmsnorm(x, gain, glue.EPS))})
    gu = glue.silu_mul_case()
    half = gu.shape[1] // 2
    g["silu_mul"] = {"shape": [gu.shape[0], half], "expected_bits": bits(ref.silu_mul(gu[:, :half], gu[:, half:]))}
    x, cos, sin = glue.rotary_case()
    st, y = ref.rotary(x, cos, sin)
    assert st == 0
    g["rotary"] = {"expected": digest(y)}
    g["attention"] = []
    for params in glue.ATTENTION_CASES:
        q, k, v = glue.attention_case(**params)
        y = ref.attention(q, k, v, params["q_heads"], params["kv_heads"], params["head_dim"], params["causal"])
        g["attention"].append({"params": params, "shape": list(y.shape), "expected_bits": bits(y)})
    path = Path(__file__).with_name("reference_vectors.json")
    path.write_text(json.dumps(out, indent=1) + "\n")
    print("wrote", path, path.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
