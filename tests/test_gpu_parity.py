"""Parity of the HIP path, called through the C ABI, with the CPU oracle and
with the committed outputs of the reference's C kernels.  Integer, byte and
f32 results are all held bit-exact (the f32 epilogue reproduces the
reference's operation order, so no tolerance is needed; the north-star
tolerance of 1e-5 rel / 1e-6 abs is therefore met with margin zero)."""
import ctypes as C
import hashlib
import json
from pathlib import Path

import numpy as np
import pytest

import _cases as cases

pytestmark = pytest.mark.gpu

GOLDEN = Path(__file__).parent / "golden"
KATS = json.loads((GOLDEN / "reference_kats.json").read_text())
VECTORS = json.loads((GOLDEN / "reference_vectors.json").read_text())
I8, U8 = cases.DTYPE_I8, cases.DTYPE_U8
DT = {"int8": I8, "uint8": U8}


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def same_f32(a, b):
    """Bitwise equal, with any NaN matching any NaN (the reference stores a
    default quiet NaN; payloads are not part of its contract)."""
    na, nb = np.isnan(a), np.isnan(b)
    return bool((na == nb).all() and (a.view(np.uint32)[~na] == b.view(np.uint32)[~nb]).all())


def build_qcase(entry):
    kind, p = entry["kind"], entry["params"]
    if kind == "isa_parity":
        return cases.isa_parity_case(**p)
    if kind == "quant_gemm":
        return cases.quant_gemm_case(**p)
    return cases.qlinear_random_case(**p)


def run_resident_qlinear(vx, ctx, c, want_acc=False):
    lin = vx.QLinear(c["w"], c["scales"], c["zps"], c["bias"], c["w_dtype"])
    res = lin.forward(ctx, dev(c["x"]), c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], c["in_dtype"],
                      c["out_dtype"], want_accumulators=want_acc)
    ctx.synchronize()
    variant = ctx.last_variant
    out = [res[0], host(res[1])] + ([host(res[2])] if want_acc else [])
    lin.close()
    return out, variant


# ---- known-answer vectors through the drop-in entry point ----------------------------

def test_kat_literal_and_halfway_through_drop_in():
    import volvoxai_amd as vx
    k = KATS["qlinear_literal"]
    ok, y = vx.qlinear_i8u8(np.array(k["input"], np.int8), np.array(k["weight"], np.int8),
                            np.array(k["weight_scales"], np.float32), np.array(k["weight_zero_points"], np.int32),
                            np.array(k["bias"], np.int32), 2, 3, 4, k["input_scale"], k["input_zero_point"],
                            k["output_scale"], k["output_zero_point"], I8, I8, I8)
    assert ok == 1 and y.tolist() == k["expected"]
    h = KATS["affine_halfway"]
    x = np.zeros((h["rows"], h["channels"]), np.uint8)
    x[:, :h["input_run"]["count"]] = h["input_run"]["value"]
    x[:, h["input_run"]["count"]] = h["input_run"]["then"]
    for wd in h["weight_dtypes"]:
        w = np.full((h["outputs"], h["channels"]), h["weight_value"], np.int8 if wd == "int8" else np.uint8)
        ok, y = vx.qlinear_i8u8(x, w, np.full(h["outputs"], h["weight_scale"], np.float32),
                                np.zeros(h["outputs"], np.int32), np.zeros(h["outputs"], np.int32),
                                h["rows"], h["channels"], h["outputs"], h["input_scale"], h["input_zero_point"],
                                h["output_scale"], h["output_zero_point"], U8, DT[wd], I8)
        assert ok == 1 and (y == h["expected_all"]).all(), "an FMA crept into the requantization epilogue"


def test_kat_packed_near_tie(oracle):
    import volvoxai_amd as vx
    k = KATS["packed_near_tie_logits"]
    x = np.zeros((1, k["k"]), np.float32)
    for idx, v in k["x_nonzero"].items():
        x[0, int(idx)] = v
    w = np.zeros((k["n"], k["k"]), np.int8)
    for row, col in k["weight_plus_one_at"]:
        w[row, col] = 1
    words = oracle.pack_w8_words(w)
    st, y = vx.packed_linear_f32(x, words, np.array(k["scales"], np.float32), np.array(k["bias"], np.float32),
                                 k["k"], k["n"], k["group_size"])
    _, want = oracle.packed_linear(x, words, np.array(k["scales"], np.float32), np.array(k["bias"], np.float32),
                                   k["n"], k["group_size"])
    assert st == 0 and int(np.argmax(y[0])) == k["expected_argmax"] and same_f32(y, want)


# ---- committed outputs of the reference's C kernels -----------------------------------

@pytest.mark.parametrize("entry", VECTORS["qlinear"], ids=lambda e: f"{e['kind']}-{'-'.join(str(v) for v in e['params'].values())}")
def test_qlinear_reference_vectors(ctx, oracle, entry):
    import volvoxai_amd as vx
    c = build_qcase(entry)
    (ok, y, acc), variant = run_resident_qlinear(vx, ctx, c, want_acc=True)
    assert ok == 1, vx.library().vxhip_last_error()
    assert sha(y) == entry["expected"]["sha256"], f"bytes differ from the reference ({variant})"
    _, _, want_acc = oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"],
                                    c["s_out"], c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"], want_acc=True)
    assert (acc == want_acc).all()
    # the host-pointer drop-in gives the same bytes
    ok2, y2 = vx.qlinear_i8u8(c["x"], c["w"], c["scales"], c["zps"], c["bias"], *c["x"].shape, c["w"].shape[0],
                              c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"])
    assert ok2 == 1 and (y2 == y).all()


@pytest.mark.parametrize("entry", VECTORS["rowscale"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_rowscale_reference_vectors(ctx, oracle, entry):
    import volvoxai_amd as vx
    c = cases.rowscale_case(**entry["params"])
    lin = vx.QLinear(c["w"], c["scales"], c["zps"], None, I8)
    xd, rs = dev(c["x"]), dev(c["row_scales"])
    ok, y, acc = lin.forward_rowscale(ctx, xd, rs, c["s_out"], c["zp_out"], want_accumulators=True)
    ctx.synchronize()
    assert ok == 1 and sha(host(y)) == entry["expected_without_bias"]["sha256"], ctx.last_variant
    assert (host(acc) == c["x"].astype(np.int64) @ c["w"].astype(np.int64).T).all()
    if c["bias_f32"] is not None:  # extension: checked against the oracle only
        ok, yb = lin.forward_rowscale(ctx, xd, rs, c["s_out"], c["zp_out"], bias_f32=dev(c["bias_f32"]))
        ctx.synchronize()
        ok2, want, _ = oracle.qlinear_rowscale(c["x"], c["w"], c["scales"], c["zps"], c["row_scales"], c["s_out"],
                                               c["zp_out"], bias_f32=c["bias_f32"])
        assert ok == ok2 == 1 and (host(yb) == want).all()
    assert ctx.fault_flags() == 0
    lin.close()


@pytest.mark.parametrize("entry", VECTORS["packed"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_packed_reference_vectors(ctx, oracle, entry):
    import volvoxai_amd as vx
    c = cases.packed_case(**entry["params"])
    words = oracle.pack_w8_words(c["w"])
    pl = vx.PackedLinear(words, c["scales"], c["bias"], c["k"], c["n"], c["group"])
    st, y = pl.forward_f32(ctx, dev(c["x"]))
    ctx.synchronize()
    y = host(y)
    assert st == 0
    if not np.isnan(y).any():
        assert sha(y) == entry["expected"]["sha256"], f"f32 bits differ from the reference ({ctx.last_variant})"
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"])
    assert same_f32(y, want), ctx.last_variant
    pl.close()


# ---- both kernel families give the same bits ------------------------------------------

@pytest.mark.parametrize("rows,k,n", [(1, 256, 64), (7, 640, 100), (16, 4096, 96), (16, 48, 40), (32, 1024, 72),
                                      (23, 300, 33)])
def test_gemv_and_gemm_agree_qlinear(ctx, oracle, rows, k, n):
    import volvoxai_amd as vx
    c = cases.qlinear_random_case(rows, k, n, 77, I8, U8, I8, False)
    _, want = oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"],
                             c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"])
    seen = set()
    try:
        for force in ("gemv.wv2", "gemv.wv8c32", "gemv.wv8c8", "gemv.wv16c16", "mfma-i8.t128x128s2", "mfma-i8.t256x256", "mfma-i8.t256x128",
                      "mfma-i8.t128x64s2", "mfma-i8.t256x128wv4", "mfma-i8.t128x128s4", "mfma-i8.t128x64s4", "mfma-i8.t128x64s4wv4",
                      "mfma-i8.t64x64", "mfma-i8.t256x256k64", "mfma-i8.t256x128k64"):
            vx.force_variant(force)
            (ok, y), variant = run_resident_qlinear(vx, ctx, c)
            assert ok == 1 and (y == want).all(), variant
            seen.add(variant)
    finally:
        vx.force_variant(None)
    # (the 16x16x64 tiles need n % 16 == 0: elsewhere their names fall back to the 32x32x32 tiles)
    assert len(seen) == (15 if n % 16 == 0 else 13), seen


@pytest.mark.parametrize("rows,k,n", [(1, 256, 64), (9, 4096, 96), (32, 1000, 48), (40, 512, 64), (300, 1040, 272), (129, 777, 80)])
def test_unsigned_activation_bytes_flipped_in_the_kernels(ctx, oracle, rows, k, n):
    """U8 activations: the streaming kernel and the 16x16x64 tiles flip the bytes' top bits themselves
    when the rows are whole aligned 16-byte chunks; other row lengths and other tiles get them staged
    first.  The bytes are the oracle's on every route, with and without weight zero points."""
    import volvoxai_amd as vx
    for zero_weight_zp in (True, False):
        c = cases.qlinear_random_case(rows, k, n, 6100 + rows, U8, I8, U8, zero_weight_zp=zero_weight_zp)
        ok, want = oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"],
                                  c["zp_out"], U8, I8, U8)
        assert ok == 1
        try:
            for force in (None, "gemv", "mfma-i8.t256x256k64", "mfma-i8.t256x128k64", "mfma-i8.t128x128s4"):
                if force == "gemv" and rows > 32:
                    continue
                vx.force_variant(force)
                (ok, y), variant = run_resident_qlinear(vx, ctx, c)
                assert ok == 1 and (y == want).all(), (variant, zero_weight_zp)
        finally:
            vx.force_variant(None)
    assert ctx.fault_flags() == 0


@pytest.mark.parametrize("group", [32, 64, 128, 256])
@pytest.mark.parametrize("rows,k,n", [(1, 4096, 48), (5, 1000, 36), (16, 1536, 130), (32, 1024, 40), (27, 1024, 96)])
def test_gemv_and_gemm_agree_packed(ctx, oracle, rows, k, n, group):
    import volvoxai_amd as vx
    c = cases.packed_case(rows, k, n, group, 5 + group, True, special_rows=(rows >= 5))
    words = oracle.pack_w8_words(c["w"])
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group)
    pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group)
    xd = dev(c["x"])
    seen = set()
    try:
        for force in ("gemv.wv2", "gemv.wv16c32", "gemv.wv16c8", "gemv.wv8c16", "a8-mfma.t128x128", "a8-mfma.t256x256", "a8-mfma.t64x128",
                      "a8-mfma.t64x64", "a8-mfma.t128x128p", "a8-mfma.t128x128k64", "a8-mfma.t128x256k64s3"):
            vx.force_variant(force)
            st, y = pl.forward_f32(ctx, xd)
            ctx.synchronize()
            assert st == 0 and same_f32(host(y), want), ctx.last_variant
            seen.add(ctx.last_variant)
    finally:
        vx.force_variant(None)
    # one scale group per k-step has no eight-wave tile: that request runs the four-wave one
    # (the pipelined 128x128 tile exists for one group per k-block only, i.e. G = 128)
    assert len(seen) == (7 if group == 32 else 11 if group == 128 else 10), seen
    pl.close()


# ---- four-bit weights ---------------------------------------------------------------------

@pytest.mark.parametrize("entry", VECTORS["packed_w4"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_packed_w4_reference_vectors(ctx, oracle, entry):
    import volvoxai_amd as vx
    c = cases.packed_case(**entry["params"])
    words = oracle.pack_w4_words(cases.four_bit(c["w"]))
    pl = vx.PackedLinear(words, c["scales"], c["bias"], c["k"], c["n"], c["group"], weight_bits=4)
    st, y = pl.forward_f32(ctx, dev(c["x"]))
    ctx.synchronize()
    y = host(y)
    assert st == 0 and "w4a8" in ctx.last_variant
    family = ctx.last_variant.rsplit(".", 1)[0]  # the id without the tile or wave suffix
    assert family in {r["id"] for r in vx.kernel_variants()}, ctx.last_variant
    if not np.isnan(y).any():
        assert sha(y) == entry["expected"]["sha256"], f"f32 bits differ from the reference ({ctx.last_variant})"
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=4)
    assert same_f32(y, want), ctx.last_variant
    pl.close()


@pytest.mark.parametrize("bits", [3, 2])
def test_packed_low_bit_reference_vectors(ctx, oracle, bits):
    """Two- and three-bit codes are widened to four bits when the weights are prepacked and run on
    the four-bit kernels; outputs are the reference's bits."""
    import volvoxai_amd as vx
    for entry in VECTORS[f"packed_w{bits}"]:
        c = cases.packed_case(**entry["params"])
        words = oracle.pack_low_bit_words(cases.low_bit(c["w"], bits), bits)
        pl = vx.PackedLinear(words, c["scales"], c["bias"], c["k"], c["n"], c["group"], weight_bits=bits)
        st, y = pl.forward_f32(ctx, dev(c["x"]))
        ctx.synchronize()
        y = host(y)
        assert st == 0 and "w4a8" in ctx.last_variant
        if not np.isnan(y).any():
            assert sha(y) == entry["expected"]["sha256"], (entry["params"], ctx.last_variant)
        _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=bits)
        assert same_f32(y, want), (entry["params"], ctx.last_variant)
        pl.close()


@pytest.mark.parametrize("group", [32, 64, 128, 256])
@pytest.mark.parametrize("rows,k,n", [(1, 4096, 48), (5, 1000, 36), (16, 1536, 130), (32, 1024, 40), (27, 1056, 96),
                                      (3, 40, 7)])
def test_gemv_and_gemm_agree_packed_w4(ctx, oracle, rows, k, n, group):
    import volvoxai_amd as vx
    c = cases.packed_case(rows, k, n, group, 9 + group, True, special_rows=(rows >= 5))
    words = oracle.pack_w4_words(cases.four_bit(c["w"]))
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group, bits=4)
    pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group, weight_bits=4)
    xd = dev(c["x"])
    seen = set()
    try:
        for force in ("gemv.wv2", "gemv.wv16c32", "gemv.wv16c8", "gemv.wv8c16", "a8-mfma.t128x128", "a8-mfma.t256x256", "a8-mfma.t64x128",
                      "a8-mfma.t64x64", "a8-mfma.t128x128p", "a8-mfma.t128x128k64", "a8-mfma.t128x256k64s3"):
            vx.force_variant(force)
            st, y = pl.forward_f32(ctx, xd)
            ctx.synchronize()
            assert st == 0 and same_f32(host(y), want), ctx.last_variant
            seen.add(ctx.last_variant)
    finally:
        vx.force_variant(None)
    assert all("w4a8" in v for v in seen) and len(seen) == (7 if group == 32 else 10 if group == 128 else 9), seen
    pl.close()


def test_packed_w4_one_shot_entry(oracle):
    """The vx_llm_forward_f32-shaped HOST entry with groups=4, and groups=0, which the reference
    reads as 4 (packed_linear_ops.inc:1547); widths it does not run are declined."""
    import volvoxai_amd as vx
    c = cases.packed_case(6, 200, 9, 64, 21, special_rows=True)
    words = oracle.pack_w4_words(cases.four_bit(c["w"]))
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], 9, 64, bits=4)
    for groups in (4, 0):
        st, y = vx.packed_linear_f32(c["x"], words, c["scales"], c["bias"], 200, 9, 64, groups=groups)
        assert st == 0 and same_f32(y, want)
    assert vx.packed_linear_f32(c["x"], words, c["scales"], c["bias"], 200, 9, 64, groups=5)[0] == -1


def test_random_shape_sweep_packed_w4(ctx, oracle):
    """Thirty seeded W4 shapes: ragged K (partial last word, block and group), every group size,
    rows on both sides of the GEMV/GEMM boundary."""
    import volvoxai_amd as vx
    rng = np.random.default_rng(78)
    for trial in range(30):
        rows = int(rng.choice([1, 2, 5, 16, 31, 32, 33, 40, 130, 300]))
        k = int(rng.choice([1, 7, 32, 33, 64, 95, 128, 130, 257, 512, 1000]))
        n = int(rng.choice([1, 2, 31, 32, 33, 70, 129, 264]))
        group = int(rng.choice([32, 64, 128, 256]))
        c = cases.packed_case(rows, k, n, group, 700 + trial, with_bias=bool(trial % 2), special_rows=(trial % 5 == 0))
        words = oracle.pack_w4_words(cases.four_bit(c["w"]))
        _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group, bits=4)
        pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group, weight_bits=4)
        for force in (None, "a8-mfma" if rows <= 32 else None):
            vx.force_variant(force)
            try:
                st, y = pl.forward_f32(ctx, dev(c["x"]))
                ctx.synchronize()
            finally:
                vx.force_variant(None)
            assert st == 0 and same_f32(host(y), want), (trial, rows, k, n, group, ctx.last_variant)
        pl.close()


def test_packed_w4_large_shapes_against_w8(ctx, oracle):
    """Full-size shapes, too big for the CPU oracle in a test: four-bit weights must give exactly
    what the same values stored as eight-bit codes give (already pinned), at M=1 (streaming kernel)
    and M=512 (MFMA GEMM)."""
    import volvoxai_amd as vx
    k, n, group = 4096, 14336, 128
    rng = np.random.default_rng(4)
    w = rng.integers(-8, 8, (n, k)).astype(np.int8)
    scales = rng.uniform(0.002, 0.01, (n, k // group)).astype(np.float32)
    bias = rng.normal(0, 0.1, n).astype(np.float32)
    p4 = vx.PackedLinear(oracle.pack_w4_words(w), scales, bias, k, n, group, weight_bits=4)
    p8 = vx.PackedLinear(oracle.pack_w8_words(w), scales, bias, k, n, group)
    assert p4.resident_bytes < 0.56 * p8.resident_bytes
    for rows in (1, 512):
        x = dev(rng.normal(0, 1, (rows, k)).astype(np.float32))
        st4, y4 = p4.forward_f32(ctx, x)
        v4 = ctx.last_variant
        st8, y8 = p8.forward_f32(ctx, x)
        ctx.synchronize()
        assert st4 == st8 == 0 and "w4a8" in v4
        assert same_f32(host(y4), host(y8)), (rows, v4)
    p4.close(); p8.close()


# ---- benchmark shapes ---------------------------------------------------------------------

@pytest.mark.parametrize("rows", [1, 4, 16])
def test_decode_shape_config2(ctx, oracle, rows):
    """M in {1,4,16}, K=4096, N=14336, prepared int8 activations, dequant+bias f32."""
    import volvoxai_amd as vx
    c = cases.decode_case(rows, 4096, 14336, 128, 1000 + rows)
    words = oracle.pack_w8_words(c["w"])
    pl = vx.PackedLinear(words, c["scales"], c["bias"], 4096, 14336, 128)
    st, y, acc = pl.forward_a8(ctx, dev(c["a8"]), dev(c["row_scales"]), want_accumulators=True)
    ctx.synchronize()
    assert st == 0 and "gemv" in ctx.last_variant
    st2, want, want_acc = oracle.packed_linear_a8(c["a8"], c["row_scales"], words, c["scales"], c["bias"], 14336, 128)
    y, acc = host(y), host(acc)
    assert (acc == want_acc).all()
    assert same_f32(y, want)
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-6)  # the stated tolerance, met exactly
    pl.close()


def test_config1_cpu_route_shape(ctx, oracle):
    """8x256x256: f32 activations quantized per tensor the PTQ way, QLinear, DQ."""
    import volvoxai_amd as vx
    rng = np.random.default_rng(1)
    xf = rng.normal(0, 1, (8, 256)).astype(np.float32)
    w = rng.integers(-127, 128, (256, 256)).astype(np.int8)
    sw = rng.uniform(0.005, 0.02, 256).astype(np.float32)
    bf = rng.normal(0, 0.1, 256).astype(np.float32)
    s_x = oracle.ptq_symmetric_scale(xf)
    xq = oracle.ptq_quantize_i8(xf, s_x)
    ok_q, xq_gpu = vx.quantize_typed_f32_i8u8(xf, s_x, 0, I8)
    st, bq = oracle.ptq_pack_bias(bf, s_x, sw)
    assert st == 0 and ok_q == 1
    _, xq_rule = oracle.quantize(xf, s_x, 0, I8)
    assert (xq_gpu == xq_rule).all()
    zps = np.zeros(256, np.int32)
    ok, y = vx.qlinear_i8u8(xq, w, sw, zps, bq, 8, 256, 256, s_x, 0, 0.25, 0, I8, I8, I8)
    ok2, want = oracle.qlinear(xq, w, bq, sw, zps, s_x, 0, 0.25, 0, I8, I8, I8)
    assert ok == ok2 == 1 and (y == want).all()
    ok3, deq = vx.dequantize_typed_i8u8_f32(y, 0.25, 0, I8)
    _, want_deq = oracle.dequantize(want, 0.25, 0, I8)
    assert ok3 == 1 and same_f32(deq, want_deq)


@pytest.mark.parametrize("rows", [512, 2048, 4096])
def test_prefill_shape_config3_subblocks(ctx, oracle, rows):
    """M in {512,2048,4096}, K=N=4096, per-token x per-channel scale, requant to int8
    at output scale 0.05.  An output sub-block depends only on its own rows of A
    and B, so the oracle checks random sub-blocks at full problem size; the
    int32 accumulators of the whole output are checked against an f64 GEMM."""
    import torch
    import volvoxai_amd as vx
    c = cases.rowscale_case(rows, 4096, 4096, 3000 + rows)
    lin = vx.QLinear(c["w"], c["scales"], c["zps"], None, I8)
    xd = dev(c["x"])
    ok, y, acc = lin.forward_rowscale(ctx, xd, dev(c["row_scales"]), c["s_out"], 0, bias_f32=dev(c["bias_f32"]),
                                      want_accumulators=True)
    ctx.synchronize()
    assert ok == 1 and "mfma-i8-rowscale" in ctx.last_variant and ctx.fault_flags() == 0
    exact = xd.double() @ dev(c["w"]).double().T  # |sum| < 2^53: exact in f64
    assert torch.equal(acc.double(), exact)
    y = host(y)
    rng = np.random.default_rng(rows)
    for _ in range(3):
        rs = np.sort(rng.choice(rows, 24, replace=False))
        cs = np.sort(rng.choice(4096, 40, replace=False))
        ok2, want, _ = oracle.qlinear_rowscale(c["x"][rs], c["w"][cs], c["scales"][cs], c["zps"][cs],
                                               c["row_scales"][rs], c["s_out"], 0, bias_f32=c["bias_f32"][cs])
        assert ok2 == 1 and (y[np.ix_(rs, cs)] == want).all()
    saturated = ((y == 127) | (y == -128)).mean()
    assert saturated < 0.5, "inputs should exercise the rounding path, not only saturation"
    lin.close()


@pytest.mark.parametrize("s_out_bits", [0x3D4CCCCD,   # 0.05
                                        0x3FFFFFFF,   # mantissa all ones
                                        0x3F800001,   # one ulp above 1
                                        0x40400000,   # 3.0
                                        0x3C49BA5E,   # 0.0123
                                        0x3DE38E39])  # ~1/9
@pytest.mark.parametrize("zp_out,int_bias", [(0, False), (0, True), (-3, False)])
def test_rowscale_epilogue_levels_and_divisors(ctx, oracle, s_out_bits, zp_out, int_bias):
    """The MFMA GEMM picks its requantizing epilogue from the call: no integer terms and a
    zero output zero point take the shortest one (one-correction division, proved per divisor
    on the device), otherwise the two-correction or the general one.  Every pick must give the
    oracle's bytes, for divisors whose reciprocal rounds awkwardly too."""
    import volvoxai_amd as vx
    rows, k, n = 160, 384, 256
    s_out = np.array([s_out_bits], np.uint32).view(np.float32)[0]
    c = cases.rowscale_case(rows, k, n, 77)
    # land the outputs inside the byte range whatever the divisor
    scales = (c["scales"] * (s_out / np.float32(0.05))).astype(np.float32)
    bias_f32 = (c["bias_f32"] * (s_out / np.float32(0.05))).astype(np.float32)
    bias_i32 = np.random.default_rng(5).integers(-5000, 5000, n).astype(np.int32) if int_bias else None
    lin = vx.QLinear(c["w"], scales, c["zps"], bias_i32, I8)
    ok2, want, _ = oracle.qlinear_rowscale(c["x"], c["w"], scales, c["zps"], c["row_scales"], s_out, zp_out,
                                           bias_i32=bias_i32, bias_f32=bias_f32)
    # the 32x32x32 tile the shape picks by itself, and both 16x16x64 tiles (their own epilogue code)
    for force in ("mfma-i8", "mfma-i8-rowscale.t256x256k64", "mfma-i8-rowscale.t256x128k64"):
        vx.force_variant(force)
        try:
            ok, y = lin.forward_rowscale(ctx, dev(c["x"]), dev(c["row_scales"]), s_out, zp_out, bias_f32=dev(bias_f32))
            ctx.synchronize()
        finally:
            vx.force_variant(None)
        assert ok == ok2 == 1 and "mfma-i8-rowscale" in ctx.last_variant and ("k64" in force) == ("k64" in ctx.last_variant)
        y = host(y)
        assert (y == want).all(), ctx.last_variant
        assert ((y == 127) | (y == -128)).mean() < 0.5
    assert ctx.fault_flags() == 0
    lin.close()


@pytest.mark.parametrize("zp_out,int_bias", [(0, False), (3, True)])
def test_streamed_output_stores(ctx, oracle, zp_out, int_bias):
    """Byte outputs of 12 MiB and more leave the large 16x16x64 tiles through streamed stores, a copy of
    the straight-line epilogue of its own (both of its levels here): 3072 rows x 4096 channels, exactly the
    size at which they start, must equal the small tile's plainly stored output everywhere and the
    oracle's bytes on random sub-blocks."""
    import volvoxai_amd as vx
    rows, k, n = 3072, 256, 4096
    c = cases.rowscale_case(rows, k, n, 91)
    bias_i32 = np.random.default_rng(6).integers(-3000, 3000, n).astype(np.int32) if int_bias else None
    lin = vx.QLinear(c["w"], c["scales"], c["zps"], bias_i32, I8)
    xd, sd, bd = dev(c["x"]), dev(c["row_scales"]), dev(c["bias_f32"])
    got = {}
    for force in ("mfma-i8-rowscale.t256x256k64", "mfma-i8-rowscale.t256x128k64", "mfma-i8-rowscale.t128x64"):
        vx.force_variant(force)
        try:
            ok, y = lin.forward_rowscale(ctx, xd, sd, c["s_out"], zp_out, bias_f32=bd)
            ctx.synchronize()
        finally:
            vx.force_variant(None)
        assert ok == 1 and ("k64" in force) == ("k64" in ctx.last_variant), ctx.last_variant
        got[force] = host(y)
    plain = got["mfma-i8-rowscale.t128x64"]
    assert (got["mfma-i8-rowscale.t256x256k64"] == plain).all() and (got["mfma-i8-rowscale.t256x128k64"] == plain).all()
    rng = np.random.default_rng(12)
    for _ in range(3):
        rs = np.sort(rng.choice(rows, 24, replace=False))
        cs = np.sort(rng.choice(n, 40, replace=False))
        ok2, want, _ = oracle.qlinear_rowscale(c["x"][rs], c["w"][cs], c["scales"][cs], c["zps"][cs], c["row_scales"][rs],
                                               c["s_out"], zp_out, bias_i32=None if bias_i32 is None else bias_i32[cs],
                                               bias_f32=c["bias_f32"][cs])
        assert ok2 == 1 and (plain[np.ix_(rs, cs)] == want).all()
    assert ((plain == 127) | (plain == -128)).mean() < 0.5 and ctx.fault_flags() == 0
    lin.close()


def test_outlier_large_k_config5_reduced_rows(ctx, oracle):
    """K=14336, N=4096 with 1% outlier channels scaled x20 before the dynamic
    per-row quantization; 96 rows here (the oracle is scalar), full K and N."""
    import volvoxai_amd as vx
    rows, k, n, g = 96, 14336, 4096, 128
    rng = np.random.default_rng(55)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    x[:, rng.choice(k, k // 100, replace=False)] *= 20.0
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    chan = rng.uniform(0.002, 0.01, n).astype(np.float32)
    scales = np.repeat(chan[:, None], k // g, axis=1).copy()
    bias = rng.normal(0, 0.1, n).astype(np.float32)
    words = oracle.pack_w8_words(w)
    pl = vx.PackedLinear(words, scales, bias, k, n, g)
    st, y = pl.forward_f32(ctx, dev(x))
    ctx.synchronize()
    assert st == 0 and "a8-mfma" in ctx.last_variant
    cs = np.sort(rng.choice(n, 160, replace=False))
    _, want = oracle.packed_linear(x, np.ascontiguousarray(words[cs]), np.ascontiguousarray(scales[cs]),
                                   np.ascontiguousarray(bias[cs]), len(cs), g)
    assert same_f32(host(y)[:, cs], want)
    pl.close()


def test_outlier_large_k_config5_full_size(ctx, oracle):
    """The whole shape, M=2048, K=14336, N=4096, f32 rows with 1% outlier channels: the prepared
    codes and scales against the oracle on sampled rows, the full-K int32 sums of the whole output
    against an f64 GEMM, and the f32 outputs against the oracle on random sub-blocks (an output
    depends only on its own row of activations and its own weight row)."""
    import torch
    import volvoxai_amd as vx
    from volvoxai_amd.w8a8 import packed_prepare_i8
    rows, k, n, g = 2048, 14336, 4096, 128
    rng = np.random.default_rng(55)
    x = rng.normal(0, 1, (rows, k)).astype(np.float32)
    x[:, rng.choice(k, k // 100, replace=False)] *= 20.0
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    chan = rng.uniform(0.002, 0.01, n).astype(np.float32)
    scales = np.repeat(chan[:, None], k // g, axis=1).copy()
    bias = rng.normal(0, 0.1, n).astype(np.float32)
    words = oracle.pack_w8_words(w)
    pl = vx.PackedLinear(words, scales, bias, k, n, g)
    xd = dev(x)
    st, y = pl.forward_f32(ctx, xd)
    ctx.synchronize()
    variant = ctx.last_variant
    assert st == 0 and "a8-mfma" in variant
    a8, sc = packed_prepare_i8(ctx, xd)
    st, y2, acc = pl.forward_a8(ctx, a8, sc, want_accumulators=True)
    ctx.synchronize()
    assert st == 0 and torch.equal(y.view(torch.int32), y2.view(torch.int32))
    exact = a8.double() @ dev(w).double().T  # |sum| <= 14336 * 127 * 127 < 2^53: exact in f64
    assert torch.equal(acc.double(), exact)
    del exact
    y, a8, sc = host(y), host(a8), host(sc)
    rs = np.sort(rng.choice(rows, 48, replace=False))
    want_a, want_s, fin = oracle.packed_prepare(x[rs])
    assert fin.all() and (a8[rs] == want_a).all() and (sc[rs].view(np.uint32) == want_s.view(np.uint32)).all()
    for _ in range(3):
        rs = np.sort(rng.choice(rows, 24, replace=False))
        cs = np.sort(rng.choice(n, 40, replace=False))
        _, want = oracle.packed_linear(np.ascontiguousarray(x[rs]), np.ascontiguousarray(words[cs]),
                                       np.ascontiguousarray(scales[cs]), np.ascontiguousarray(bias[cs]), len(cs), g)
        assert same_f32(y[np.ix_(rs, cs)], want), variant
    pl.close()


# ---- values only the device can check -------------------------------------------------------

def test_device_side_faults_are_raised_and_cleared(oracle):
    """Row scales and the real-valued bias of the per-token form live in device memory, so the host
    admission cannot see them.  Where the CPU rule declines the call, the kernels raise a sticky
    fault bit (1: a multiplier is not finite and positive; 8: a bias is not finite), in both kernel
    families; clearing the word is ordered on the stream."""
    import torch
    import volvoxai_amd as vx
    own = vx.Context(0, torch.cuda.current_stream())  # fault bits are sticky: not the shared context
    # the streaming GEMV, the 32x32x32 GEMM and (named) the 16x16x64 GEMM
    for rows, bad_row, force in ((8, 3, None), (160, 77, None), (160, 77, "mfma-i8-rowscale.t256x128k64")):
        vx.force_variant(force)
        c = cases.rowscale_case(rows, 256, 64, 5)
        lin = vx.QLinear(c["w"], c["scales"], c["zps"], None, I8)
        xd, bd = dev(c["x"]), dev(c["bias_f32"])
        ok, _ = lin.forward_rowscale(own, xd, dev(c["row_scales"]), c["s_out"], 0, bias_f32=bd)
        assert ok == 1 and own.fault_flags() == 0
        for value in (0.0, -1.0, np.nan, np.inf):
            rs = c["row_scales"].copy()
            rs[bad_row] = value
            assert oracle.qlinear_rowscale(c["x"], c["w"], c["scales"], c["zps"], rs, c["s_out"], 0)[0] == 0
            ok, _ = lin.forward_rowscale(own, xd, dev(rs), c["s_out"], 0, bias_f32=bd)
            assert ok == 1 and own.fault_flags() == 1, (rows, value, own.last_variant)  # provisional 1, then the bit
            own.clear_fault_flags()
            assert own.fault_flags() == 0
        for value in (np.nan, -np.inf):
            b = c["bias_f32"].copy()
            b[9] = value
            assert oracle.qlinear_rowscale(c["x"], c["w"], c["scales"], c["zps"], c["row_scales"], c["s_out"], 0,
                                           bias_f32=b)[0] == 0
            ok, _ = lin.forward_rowscale(own, xd, dev(c["row_scales"]), c["s_out"], 0, bias_f32=dev(b))
            assert ok == 1 and own.fault_flags() == 8, (rows, value, own.last_variant)
            own.clear_fault_flags()
        # the word is clean again and a good call stays clean
        ok, y = lin.forward_rowscale(own, xd, dev(c["row_scales"]), c["s_out"], 0, bias_f32=bd)
        _, want, _ = oracle.qlinear_rowscale(c["x"], c["w"], c["scales"], c["zps"], c["row_scales"], c["s_out"], 0,
                                             bias_f32=c["bias_f32"])
        assert ok == 1 and own.fault_flags() == 0 and (host(y) == want).all()
        assert force is None or "k64" in own.last_variant
        lin.close()
    vx.force_variant(None)
    own.close()


def test_two_contexts_keep_their_own_variant_ids(ctx):
    """The id of the kernel that ran is held per context, not per thread."""
    import torch
    import volvoxai_amd as vx
    other = vx.Context(0, torch.cuda.current_stream())
    small = cases.qlinear_random_case(4, 256, 64, 2)
    big = cases.qlinear_random_case(64, 256, 128, 2)
    (ok1, _), v1 = run_resident_qlinear(vx, ctx, big)
    (ok2, _), v2 = run_resident_qlinear(vx, other, small)
    assert ok1 == ok2 == 1 and "gemv" in v2 and "mfma-i8" in v1
    assert ctx.last_variant == v1 and other.last_variant == v2  # the second launch did not overwrite the first
    other.close()


# ---- boundaries and edge cases ------------------------------------------------------------

def test_prepare_matches_oracle(ctx, oracle):
    import volvoxai_amd as vx
    from volvoxai_amd.w8a8 import packed_prepare_i8
    c = cases.packed_case(9, 1283, 4, 128, 3, special_rows=True)
    x = c["x"].copy()
    x[7, 5] = np.nan
    x[8, 0] = -np.inf
    a8, s = packed_prepare_i8(ctx, dev(x))
    ctx.synchronize()
    want_a, want_s, fin = oracle.packed_prepare(x)
    a8, s = host(a8), host(s)
    assert (np.isnan(s) == (fin == 0)).all()
    good = fin == 1
    assert (s[good].view(np.uint32) == want_s[good].view(np.uint32)).all()
    assert (a8[good] == want_a[good]).all() and not a8[~good].any()


def test_quantize_dequantize_match_oracle(oracle):
    import volvoxai_amd as vx
    rng = np.random.default_rng(8)
    x = np.concatenate([rng.normal(0, 40, 5000), np.arange(-6, 6) + 0.5,
                        [np.nan, np.inf, -np.inf, 1e30, -1e30, 0.0, -0.0]]).astype(np.float32)
    for dt, zp in ((I8, -7), (U8, 131), (I8, 0)):
        ok, q = vx.quantize_typed_f32_i8u8(x, 0.37, zp, dt)
        ok2, want = oracle.quantize(x, 0.37, zp, dt)
        assert ok == ok2 == 1 and (q == want).all()
        ok, d = vx.dequantize_typed_i8u8_f32(want, 0.37, zp, dt)
        _, wd = oracle.dequantize(want, 0.37, zp, dt)
        assert ok == 1 and same_f32(d, wd)


@pytest.mark.parametrize("rows,k,n", [(1, 96, 40), (17, 4096, 300), (32, 1024, 1024), (33, 200, 72), (200, 777, 130),
                                      (600, 1024, 512), (2048, 192, 4096), (4000, 128, 4096)])  # the last two: the large tiles
@pytest.mark.parametrize("idt,odt", [(I8, I8), (U8, U8), (I8, U8)])
def test_qlinear_dequantized_equals_the_two_nodes(ctx, oracle, rows, k, n, idt, odt):
    """QLinear with the DequantizeLinear behind it folded into its epilogue
    (native/src/kernels/quantize_linear_ops.inc:9-16 applied to each byte where it is made): the f32
    values are those of the two operators one after the other, the bytes (asked for as well) too;
    dequantization parameters other than the output's own are honoured; a bad one declines."""
    import volvoxai_amd as vx
    c = cases.qlinear_random_case(rows, k, n, 4100 + rows + n, idt, I8, odt, zero_weight_zp=(rows % 2 == 0))
    ok, q = oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"], c["zp_out"],
                           idt, I8, odt)
    assert ok == 1
    lin = vx.QLinear(c["w"], c["scales"], c["zps"], c["bias"], I8)
    xd = dev(c["x"])
    for dq_scale, dq_zp in ((None, None), (np.float32(0.37), 3)):
        s, z = (c["s_out"], c["zp_out"]) if dq_scale is None else (dq_scale, dq_zp)
        _, want = oracle.dequantize(q, s, z, odt)
        got = lin.forward_dequantized(ctx, xd, c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], idt, odt, dequant_scale=dq_scale,
                                      dequant_zero_point=dq_zp, want_bytes=True)
        assert got[0] == 1 and same_f32(got[1].cpu().numpy(), want) and (got[2].cpu().numpy() == q).all(), ctx.last_variant
        if rows >= 2048 and rows % 2 == 0:   # no weight zero points: the 16x16x64 tiles, dequantizing in their own epilogue
            assert ctx.last_variant.endswith("k64-dq"), ctx.last_variant
        ok2, only = lin.forward_dequantized(ctx, xd, c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], idt, odt,
                                            dequant_scale=dq_scale, dequant_zero_point=dq_zp)
        assert ok2 == 1 and same_f32(only.cpu().numpy(), want)
    for bad_scale, bad_zp in ((0.0, 0), (float("nan"), 0), (0.1, 300), (0.1, -129 if odt == I8 else -1)):
        assert lin.forward_dequantized(ctx, xd, c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], idt, odt,
                                       dequant_scale=bad_scale, dequant_zero_point=bad_zp)[0] == 0
    assert ctx.fault_flags() == 0
    lin.close()


@pytest.mark.parametrize("rows", [1, 2, 3, 4])
@pytest.mark.parametrize("k,n,group,bits", [(4096, 14336, 128, 8), (1000, 200, 32, 8), (129, 40, 64, 8), (4096, 1024, 128, 4),
                                            (2048, 4096, 256, 8), (1024, 6144, 128, 3), (3072, 1024, 64, 2)])
def test_few_f32_rows_are_prepared_inside_the_gemv(ctx, oracle, rows, k, n, group, bits):
    """PackedLinear on one or two f32 rows is one launch: the streaming kernel quantizes the rows itself
    (the reference's single-row route does both in one call, packed_linear_ops.inc:1471-1535).  Same
    bits as the oracle and as the two launches, special rows included (all zero, denormal, huge, NaN)."""
    import volvoxai_amd as vx
    c = cases.packed_case(max(rows, 5), k, n, group, 8800 + rows + n, special_rows=True)
    x = c["x"][[0, 3, 1, 2][:rows]] if rows > 1 else c["x"][:1]
    x = np.ascontiguousarray(x)
    if rows % 2 == 0:
        x[rows - 1, k // 2] = np.nan   # a row that holds a NaN: every output of the row is NaN
    w = c["w"] if bits == 8 else cases.low_bit(c["w"], bits)
    words = oracle.pack_w8_words(w) if bits == 8 else oracle.pack_low_bit_words(w, bits)
    _, want = oracle.packed_linear(x, words, c["scales"], c["bias"], n, group, bits=bits)
    pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group, weight_bits=bits)
    st, y = pl.forward_f32(ctx, dev(x))
    ctx.synchronize()
    # (more rows keep the two launches)
    assert st == 0 and ctx.last_variant.endswith("-prep") == (rows <= 2) and "gemv-mfma" in ctx.last_variant, ctx.last_variant
    assert same_f32(y.cpu().numpy(), want)
    vx.force_variant("gemv.noprep")
    try:
        st2, y2 = pl.forward_f32(ctx, dev(x))
        ctx.synchronize()
        assert st2 == 0 and not ctx.last_variant.endswith("-prep")
    finally:
        vx.force_variant(None)
    assert same_f32(y2.cpu().numpy(), want)
    assert ctx.fault_flags() == 0
    pl.close()


@pytest.mark.parametrize("rows,k,n", [(1, 4096, 4096), (2, 1024, 300), (1, 1000, 72), (2, 96, 40), (3, 4096, 512), (40, 777, 130),
                                      (300, 256, 64)])
@pytest.mark.parametrize("idt,odt", [(I8, I8), (U8, U8), (U8, I8)])
def test_qlinear_on_f32_rows_equals_the_three_nodes(ctx, oracle, rows, k, n, idt, odt):
    """QuantizeLinear -> QLinear -> DequantizeLinear through one entry point: one launch for one or two
    rows (the streaming kernel quantizes the rows itself), the quantization as a launch of its own
    otherwise; bytes and f32 are those of the three operators in turn, NaN, infinities and
    half-way values in the input included; weight zero points keep the separate launches."""
    import volvoxai_amd as vx
    for zero_weight_zp in (True, False):
        c = cases.qlinear_random_case(rows, k, n, 5200 + rows + n, idt, I8, odt, zero_weight_zp=zero_weight_zp)
        rng = np.random.default_rng(rows * 7 + n)
        x = rng.normal(0, 40 * c["s_in"], (rows, k)).astype(np.float32)
        x[0, :6] = [np.nan, np.inf, -np.inf, 0.5 * c["s_in"], 1.5 * c["s_in"], -2.5 * c["s_in"]]
        ok, xq = oracle.quantize(x, c["s_in"], c["zp_in"], idt)
        ok1, q = oracle.qlinear(xq, c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"], c["zp_out"],
                                idt, I8, odt)
        assert ok == 1 and ok1 == 1
        _, want = oracle.dequantize(q, c["s_out"], c["zp_out"], odt)
        lin = vx.QLinear(c["w"], c["scales"], c["zps"], c["bias"], I8)
        got = lin.forward_f32(ctx, dev(x), c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], idt, odt, want_bytes=True)
        assert got[0] == 1 and (got[2].cpu().numpy() == q).all() and same_f32(got[1].cpu().numpy(), want), ctx.last_variant
        inside = rows <= 2 and zero_weight_zp
        assert ctx.last_variant.endswith("-prep") == inside, ctx.last_variant
        ok2, only_bytes = lin.forward_f32(ctx, dev(x), c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], idt, odt, want_f32=False,
                                          want_bytes=True)[::2]
        assert ok2 == 1 and (only_bytes.cpu().numpy() == q).all()
        lin.close()
    assert ctx.fault_flags() == 0


@pytest.mark.parametrize("entry", VECTORS["requantize"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_requantize_reference_vectors(ctx, oracle, entry):
    """RequantizeLinear: the bytes of the reference's own kernel (committed digests), through the host-pointer
    drop-in and the resident entry, on aligned and on unaligned tensors."""
    import volvoxai_amd as vx
    c = cases.requantize_case(**entry["params"])
    args = (c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], c["in_dtype"], c["out_dtype"])
    ok, y = vx.requantize_linear_i8u8(c["x"], *args)
    assert ok == 1 and sha(y) == entry["expected"]["sha256"]
    ok2, want = oracle.requantize_linear(c["x"], *args)
    assert ok2 == 1 and (y == want).all()
    xd = dev(np.concatenate([np.zeros(3, c["x"].dtype), c["x"]]))[3:]   # three bytes off a 16-byte boundary
    ok3, yd = vx.requantize_forward(ctx, xd.contiguous() if False else xd, *args)
    ctx.synchronize()
    assert ok3 == 1 and (host(yd) == want).all() and ctx.last_variant == "hip.requantize-linear.elementwise"
    ok4, ya = vx.requantize_forward(ctx, dev(c["x"]), *args)
    ctx.synchronize()
    assert ok4 == 1 and (host(ya) == want).all()


def test_requantize_declines(oracle):
    import volvoxai_amd as vx
    x = np.arange(-8, 8).astype(np.int8)
    for args in ((0.0, 0, 1.0, 0, I8, I8), (1.0, 0, float("nan"), 0, I8, I8), (1.0, 128, 1.0, 0, I8, I8),
                 (1.0, 0, 1.0, -1, I8, U8), (3e38, 0, 1e-38, 0, I8, I8), (1e-38, 0, 3e38, 0, I8, I8), (1.0, 0, 1.0, 0, 3, I8)):
        assert oracle.requantize_linear(x, *args)[0] == 0
        ok, y = vx.requantize_linear_i8u8(x, *args)
        assert ok == 0 and not y.any(), args   # declined, output untouched
    # unequal counts and overlapping buffers, as the reference's device forms refuse them
    lib = vx.library()
    buf = np.zeros(64, np.int8)
    p = buf.ctypes.data
    import ctypes as C
    call = lambda a, na, b, nb: lib.vxhip_requantize_linear_i8u8(C.c_void_p(a), na, C.c_void_p(b), nb, 1.0, 0, 0.5, 0, I8, I8)
    assert call(p, 16, p + 32, 8) == 0 and call(p, 16, p + 8, 16) == 0 and call(p, 16, p + 16, 16) == 1


def test_host_pointer_entry_points_keep_weights_resident(oracle):
    """vxhip_qlinear_i8u8 / vxhip_packed_linear_f32 pack a weight once per (pointers, shape, type,
    fingerprint) and reuse it: the second call adds nothing to the resident set, refilling the
    buffer in place is noticed (the bytes are the new weight's), clearing empties the set."""
    import volvoxai_amd as vx
    lib = vx.library()
    lib.vxhip_resident_weights_clear()
    c = cases.qlinear_random_case(9, 512, 160, 91, I8, I8, I8, False)
    w = np.ascontiguousarray(c["w"])
    args = lambda: (c["x"], w, c["scales"], c["zps"], c["bias"], 9, 512, 160, c["s_in"], c["zp_in"], c["s_out"], c["zp_out"],
                    I8, I8, I8)
    ok, y = vx.qlinear_i8u8(*args())
    _, want = oracle.qlinear(c["x"], w, c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], I8, I8, I8)
    held = lib.vxhip_resident_weights_bytes()
    assert ok == 1 and (y == want).all() and held > 0
    ok, y = vx.qlinear_i8u8(*args())
    assert ok == 1 and (y == want).all() and lib.vxhip_resident_weights_bytes() == held      # reused
    w[:] = np.roll(w, 1, axis=0)                                                              # same buffer, new weight
    _, want2 = oracle.qlinear(c["x"], w, c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], I8, I8, I8)
    ok, y = vx.qlinear_i8u8(*args())
    assert ok == 1 and (y == want2).all() and not (want2 == want).all()
    assert lib.vxhip_resident_weights_bytes() == 2 * held                                     # packed again, beside the old entry
    p = cases.packed_case(3, 256, 40, 64, 92)
    words = oracle.pack_w8_words(p["w"])
    st, z = vx.packed_linear_f32(p["x"], words, p["scales"], p["bias"], 256, 40, 64)
    _, zwant = oracle.packed_linear(p["x"], words, p["scales"], p["bias"], 40, 64)
    grown = lib.vxhip_resident_weights_bytes()
    assert st == 0 and same_f32(z, zwant) and grown > 2 * held
    st, z = vx.packed_linear_f32(p["x"], words, p["scales"], p["bias"], 256, 40, 64)
    assert st == 0 and same_f32(z, zwant) and lib.vxhip_resident_weights_bytes() == grown
    lib.vxhip_resident_weights_clear()
    assert lib.vxhip_resident_weights_bytes() == 0
    # a byte limit: the least recently used weight leaves, a weight above the limit is not kept at all
    import os
    os.environ["VXHIP_RESIDENT_WEIGHT_BYTES"] = str(held + held // 2)
    try:
        vx.qlinear_i8u8(*args())
        other = np.ascontiguousarray(np.roll(w, 3, axis=1))
        _, want3 = oracle.qlinear(c["x"], other, c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], I8, I8, I8)
        ok, y = vx.qlinear_i8u8(c["x"], other, c["scales"], c["zps"], c["bias"], 9, 512, 160, c["s_in"], c["zp_in"], c["s_out"],
                                c["zp_out"], I8, I8, I8)
        assert ok == 1 and (y == want3).all() and lib.vxhip_resident_weights_bytes() == held
        os.environ["VXHIP_RESIDENT_WEIGHT_BYTES"] = "1024"
        lib.vxhip_resident_weights_clear()
        ok, y = vx.qlinear_i8u8(*args())
        assert ok == 1 and (y == want2).all() and lib.vxhip_resident_weights_bytes() == 0
    finally:
        del os.environ["VXHIP_RESIDENT_WEIGHT_BYTES"]
        lib.vxhip_resident_weights_clear()


def test_recorded_launches_replay_on_new_values(oracle):
    """A context records the launches of its entry points and replays them: a PackedLinear on two prepared rows and a
    QLinear behind it, recorded once, replayed on three sets of activations written into the same device buffers;
    every replay equals the oracle.  A recording that would have to grow the context's scratch is refused."""
    import torch
    import volvoxai_amd as vx
    c = cases.decode_case(2, 512, 96, 128, 77)
    words = oracle.pack_w8_words(c["w"])
    pl = vx.PackedLinear(words, c["scales"], c["bias"], 512, 96, 128)
    q = cases.qlinear_random_case(5, 256, 64, 31, I8, I8, I8, False)
    lin = vx.QLinear(q["w"], q["scales"], q["zps"], q["bias"], I8)
    stream = torch.cuda.Stream()
    ctx = vx.Context(0, stream)
    try:
        a8, rs = dev(c["a8"]), dev(c["row_scales"])
        xq = dev(q["x"])
        y = torch.empty((2, 96), dtype=torch.float32, device="cuda")
        yq = torch.empty((5, 64), dtype=torch.int8, device="cuda")

        def calls():
            st, _ = pl.forward_a8(ctx, a8, rs, out=y)
            ok = lin.forward(ctx, xq, q["s_in"], q["zp_in"], q["s_out"], q["zp_out"], I8, I8, out=yq)[0]
            assert st == 0 and ok == 1

        # unwarmed: the QLinear's first call needs scratch, which a recording may not allocate
        fresh = vx.Context(0, stream)
        fresh.begin_recording()
        big = cases.qlinear_random_case(300, 256, 64, 32, I8, I8, I8, False)
        refused = lin.forward(fresh, dev(big["x"]), big["s_in"], big["zp_in"], big["s_out"], big["zp_out"], I8, I8)[0]
        abandoned = vx.library().vxhip_context_end_recording(fresh._h, None)
        assert refused == 0 and abandoned == 0 and "recorded" in vx.library().vxhip_last_error().decode()
        fresh.close()

        calls()                      # the unrecorded run sizes the scratch
        ctx.synchronize()
        ctx.begin_recording()
        calls()
        # waits and host copies cannot be recorded: refused, the recording stays open
        flags = C.c_uint32(0)
        assert vx.library().vxhip_context_synchronize(ctx._h) != 0
        assert vx.library().vxhip_context_fault_flags(ctx._h, C.byref(flags)) != 0
        assert "recording" in vx.library().vxhip_last_error().decode()
        replay = ctx.end_recording()
        rng = np.random.default_rng(5)
        for trial in range(3):
            na8 = rng.integers(-127, 128, c["a8"].shape).astype(np.int8)
            nrs = rng.uniform(0.01, 0.05, 2).astype(np.float32)
            nx = rng.integers(-127, 128, q["x"].shape).astype(np.int8)
            with torch.cuda.stream(stream):
                a8.copy_(torch.from_numpy(na8)); rs.copy_(torch.from_numpy(nrs)); xq.copy_(torch.from_numpy(nx))
                y.zero_(); yq.zero_()
            replay.launch(ctx)
            ctx.synchronize()
            _, want, _ = oracle.packed_linear_a8(na8, nrs, words, c["scales"], c["bias"], 96, 128)
            _, wantq = oracle.qlinear(nx, q["w"], q["bias"], q["scales"], q["zps"], q["s_in"], q["zp_in"], q["s_out"], q["zp_out"],
                                      I8, I8, I8)
            assert same_f32(y.cpu().numpy(), want) and (yq.cpu().numpy() == wantq).all(), trial
        replay.close()
    finally:
        ctx.close()
        pl.close()
        lin.close()


def test_host_pointer_entry_point_from_several_threads(oracle):
    """Four threads call vxhip_qlinear_i8u8 at once, two weights among them: every thread has its own context and
    stream, the resident set is shared, and every call returns the oracle's bytes."""
    import threading
    import volvoxai_amd as vx
    lib = vx.library()
    lib.vxhip_resident_weights_clear()
    weights = [cases.qlinear_random_case(5, 384, 64, 700 + i, I8, I8, I8, False) for i in range(2)]
    wants = [oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"], c["zp_out"],
                            I8, I8, I8)[1] for c in weights]
    failures = []

    def worker(index):
        for call in range(12):
            c, want = weights[(index + call) % 2], wants[(index + call) % 2]
            ok, y = vx.qlinear_i8u8(c["x"], c["w"], c["scales"], c["zps"], c["bias"], 5, 384, 64, c["s_in"], c["zp_in"], c["s_out"],
                                    c["zp_out"], I8, I8, I8)
            if ok != 1 or not (y == want).all():
                failures.append((index, call))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
    assert not failures and not any(t.is_alive() for t in threads)
    one = lib.vxhip_resident_weights_bytes()
    assert one > 0
    lib.vxhip_resident_weights_clear()


def test_declines_leave_output_untouched():
    import volvoxai_amd as vx
    c = cases.qlinear_random_case(2, 16, 4, 3)
    base = dict(input=c["x"], weight=c["w"], weight_scales=c["scales"], weight_zero_points=c["zps"], bias=c["bias"],
                rows=2, d_in=16, d_out=4, input_scale=c["s_in"], input_zero_point=0, output_scale=c["s_out"],
                output_zero_point=0, input_dtype=I8, weight_dtype=I8, output_dtype=I8)
    for patch in (dict(input_scale=0.0), dict(input_zero_point=300), dict(output_scale=float("inf")),
                  dict(input_scale=1e-30, weight_scales=np.full(4, 1e-30, np.float32)),
                  dict(bias=np.full(4, 2**31 - 1, np.int32)), dict(input_dtype=18)):
        ok, y = vx.qlinear_i8u8(**{**base, **patch})
        assert ok == 0 and not y.any(), patch
    # K beyond the int32 proof (K * max|x-zx| * max|w-zw| > INT32_MAX): declined before launch
    big = cases.qlinear_random_case(1, 140000, 4, 4, U8, U8, I8, False)
    ok, _ = vx.qlinear_i8u8(big["x"], big["w"], big["scales"], big["zps"], big["bias"], 1, 140000, 4, big["s_in"],
                            big["zp_in"], big["s_out"], big["zp_out"], U8, U8, I8)
    assert ok == 0 and b"int32" in vx.library().vxhip_last_error()


def test_context_reports_variant_and_clean_fault_word(ctx):
    import volvoxai_amd as vx
    c = cases.qlinear_random_case(64, 256, 128, 2)
    (ok, _), variant = run_resident_qlinear(vx, ctx, c)
    assert ok == 1 and variant.startswith("hip.qlinear.mfma-i8")
    assert variant.split(".t")[0] in {r["id"] for r in vx.kernel_variants()}
    assert ctx.fault_flags() == 0


# ---- seeded sweep over ragged shapes ----------------------------------------------------------

def test_random_shape_sweep_qlinear(ctx, oracle):
    """Forty seeded shapes with ragged rows/K/N, every byte-dtype combination, weight zero points
    and both output scales' regimes; each through the default dispatch and the other kernel family."""
    import volvoxai_amd as vx
    rng = np.random.default_rng(2025)
    for trial in range(40):
        rows = int(rng.choice([1, 2, 3, 7, 16, 17, 31, 32, 33, 64, 100, 257]))
        k = int(rng.choice([1, 5, 16, 31, 32, 33, 100, 127, 128, 129, 255, 640, 1000]))
        n = int(rng.choice([1, 3, 16, 31, 32, 33, 48, 100, 255, 256, 300]))
        in_dt, w_dt, out_dt = (int(rng.choice([I8, U8])) for _ in range(3))
        c = cases.qlinear_random_case(rows, k, n, 9000 + trial, in_dt, w_dt, out_dt, zero_weight_zp=bool(trial % 2),
                                      s_out=float(rng.choice([0.05, 0.5, 3.0])))
        ok_w, want = oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"],
                                    c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"])
        assert ok_w == 1
        for force in (None, "mfma-i8" if rows <= 32 else None):
            if force is None and rows > 32 and trial % 3 == 0:
                force = "mfma-i8.t128x64"
            vx.force_variant(force)
            try:
                (ok, y), variant = run_resident_qlinear(vx, ctx, c)
            finally:
                vx.force_variant(None)
            assert ok == 1 and (y == want).all(), (trial, rows, k, n, in_dt, w_dt, out_dt, variant)
    assert ctx.fault_flags() == 0


def test_random_shape_sweep_packed(ctx, oracle):
    """Thirty seeded PackedLinear shapes: ragged K (partial last group and word), every group size,
    with and without bias, rows on both sides of the GEMV/GEMM boundary."""
    import volvoxai_amd as vx
    rng = np.random.default_rng(77)
    for trial in range(30):
        rows = int(rng.choice([1, 2, 5, 16, 31, 32, 33, 40, 130]))
        k = int(rng.choice([1, 7, 32, 33, 95, 128, 130, 257, 512, 1000]))
        n = int(rng.choice([1, 2, 31, 32, 33, 70, 129, 264]))
        group = int(rng.choice([32, 64, 128, 256]))
        c = cases.packed_case(rows, k, n, group, 500 + trial, with_bias=bool(trial % 2), special_rows=(trial % 5 == 0))
        words = oracle.pack_w8_words(c["w"])
        _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group)
        pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group)
        for force in (None, "a8-mfma" if rows <= 32 else None):
            vx.force_variant(force)
            try:
                st, y = pl.forward_f32(ctx, dev(c["x"]))
                ctx.synchronize()
            finally:
                vx.force_variant(None)
            assert st == 0 and same_f32(host(y), want), (trial, rows, k, n, group, ctx.last_variant)
        pl.close()


def test_every_tile_and_stage_variant_on_ragged_shapes(ctx, oracle):
    """Seeded ragged shapes through every forced GEMM tile, stage count and the pipelined tile, for
    both epilogue families and every packed width: each must give the oracle's bits."""
    import volvoxai_amd as vx
    rng = np.random.default_rng(31)
    packed_variants = ("a8-mfma.t128x128", "a8-mfma.t256x256", "a8-mfma.t64x128", "a8-mfma.t64x64",
                       "a8-mfma.t128x128p", "a8-mfma.t128x128k64", "a8-mfma.t128x256k64s3")
    for trial in range(24):
        rows = int(rng.choice([3, 33, 65, 128, 200, 257]))
        k = int(rng.choice([31, 64, 129, 384, 640, 1153]))
        n = int(rng.choice([5, 33, 64, 129, 256, 300]))
        group = int(rng.choice([32, 64, 128, 128, 256]))
        bits = int(rng.choice([8, 4, 3, 2]))
        c = cases.packed_case(rows, k, n, group, 4000 + trial, with_bias=bool(trial % 2), special_rows=(trial % 5 == 0))
        w = c["w"] if bits == 8 else cases.low_bit(c["w"], bits)
        words = oracle.pack_w8_words(w) if bits == 8 else oracle.pack_low_bit_words(w, bits)
        _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group, bits=bits)
        pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group, weight_bits=bits)
        xd = dev(c["x"])
        try:
            for force in packed_variants:
                vx.force_variant(force)
                st, y = pl.forward_f32(ctx, xd)
                ctx.synchronize()
                assert st == 0 and same_f32(host(y), want), (trial, rows, k, n, group, bits, ctx.last_variant)
        finally:
            vx.force_variant(None)
        pl.close()
    q_variants = ("mfma-i8.t128x128s2", "mfma-i8.t128x128s4", "mfma-i8.t128x64s2", "mfma-i8.t128x64s4", "mfma-i8.t128x64s4wv4",
                  "mfma-i8.t64x64", "mfma-i8.t256x128", "mfma-i8.t256x256", "mfma-i8.t256x128k64",
                  "mfma-i8.t256x256k64")
    for trial in range(24):
        rows = int(rng.choice([2, 33, 64, 129, 300]))
        k = int(rng.choice([15, 64, 127, 385, 777, 1024]))
        n = int(rng.choice([7, 16, 48, 100, 144, 272]))
        in_dt, w_dt, out_dt = (int(rng.choice([I8, U8])) for _ in range(3))
        c = cases.qlinear_random_case(rows, k, n, 5000 + trial, in_dt, w_dt, out_dt, bool(trial % 3 == 0))
        ok_w, want = oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"],
                                    c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"])
        assert ok_w == 1
        try:
            for force in q_variants:
                vx.force_variant(force)
                (ok, y), variant = run_resident_qlinear(vx, ctx, c)
                assert ok == 1 and (y == want).all(), (trial, rows, k, n, in_dt, w_dt, out_dt, variant)
        finally:
            vx.force_variant(None)
    assert ctx.fault_flags() == 0


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("group", [64, 128, 256])
def test_uniform_group_scales_take_the_hoisted_fold(ctx, oracle, group, bits):
    """One scale per channel replicated over the groups (what per-channel quantization exports): the
    16x16x64 tiles then form s_a * s_w once per output.  Same products, so the oracle's bits, on
    ragged shapes, special rows included; the general kernels on the same package agree."""
    import volvoxai_amd as vx
    for trial, (rows, k, n) in enumerate([(130, 1000, 144), (257, 4608, 72), (300, 384, 300), (65, 4096 + 64, 130)]):
        c = cases.packed_case(rows, k, n, group, 700 + trial, with_bias=bool(trial % 2), special_rows=True)
        scales = np.repeat(c["scales"][:, :1], c["scales"].shape[1], axis=1).copy()
        w = c["w"] if bits == 8 else cases.four_bit(c["w"])
        words = oracle.pack_w8_words(w) if bits == 8 else oracle.pack_w4_words(w)
        _, want = oracle.packed_linear(c["x"], words, scales, c["bias"], n, group, bits=bits)
        pl = vx.PackedLinear(words, scales, c["bias"], k, n, group, weight_bits=bits)
        xd = dev(c["x"])
        fam = "a8-mfma" if bits == 8 else "w4a8-mfma"
        try:
            for force in (f"{fam}.t128x128k64", f"{fam}.t128x256k64s3", f"{fam}.t128x128", None):
                vx.force_variant(force)
                st, y = pl.forward_f32(ctx, xd)
                ctx.synchronize()
                assert st == 0 and same_f32(host(y), want), (rows, k, n, group, bits, ctx.last_variant)
        finally:
            vx.force_variant(None)
        pl.close()


def test_ceiling_probes_report_rates(ctx):
    """The two measurement aids: a register-only MFMA loop and a read-only kernel.  Rates are
    machine facts, so only their sanity is checked, and that bad arguments are refused."""
    import torch
    import volvoxai_amd as vx
    from volvoxai_amd.w8a8 import VxHipError
    m = ctx.probe_mfma_rate(32, True)
    assert 100.0 < m["tops"] < 6000.0 and 300.0 < m["shader_mhz"] < 3500.0
    m = ctx.probe_mfma_rate(32, True, k64=True)
    assert 100.0 < m["tops"] < 6000.0 and 300.0 < m["shader_mhz"] < 3500.0
    bufs = [torch.zeros((1 << 20) + 48, dtype=torch.uint8, device="cuda") for _ in range(3)]
    r = ctx.probe_stream_read(bufs, launches=9)
    assert r["bytes"] == (1 << 20) + 48 and r["GBs"] > 1.0 and r["microseconds"] > 0.0
    with pytest.raises(VxHipError):
        ctx.probe_stream_read([bufs[0][1:17]], launches=1)  # not 16-byte aligned
    with pytest.raises(VxHipError):
        ctx.probe_stream_read([bufs[0][:8]], launches=1)    # less than one 16-byte word
    assert vx is not None



@pytest.mark.parametrize("rows,k,n,group", [(1, 4096, 96, 128), (5, 1000, 36, 32), (16, 1537, 130, 64),
                                            (32, 1024, 1056, 128), (27, 24, 40, 256), (32, 5000, 300, 32)])
def test_operand_order_activations(oracle, rows, k, n, group):
    """A context set to exchange prepared activations in the GEMV's operand order: the prepared
    bytes are the row-major codes re-ordered, the linear gives the oracle's bits from them (also
    where no GEMV takes the shape and the rows are copied back out for the GEMM, the last case),
    and calls with more than 32 rows stay row major."""
    import torch
    import volvoxai_amd as vx
    from volvoxai_amd.w8a8 import packed_prepare_i8
    c = cases.packed_case(rows, k, n, group, 900 + rows, True, special_rows=(rows >= 5))
    words = oracle.pack_w8_words(c["w"])
    _, want = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], n, group)
    plain, blocked = vx.Context(0, None), vx.Context(0, None)
    blocked.set_activation_layout(True)
    xd = dev(c["x"])
    codes, scales = packed_prepare_i8(plain, xd)
    bcodes, bscales = packed_prepare_i8(blocked, xd)
    plain.synchronize(), blocked.synchronize()
    chunks = (k + 15) // 16
    assert bcodes.numel() == 32 * chunks * 16
    padded = np.zeros((rows, chunks * 16), np.int8)
    padded[:, :k] = host(codes)
    got = host(bcodes).reshape(chunks, 32, 16)[:, :rows].transpose(1, 0, 2).reshape(rows, chunks * 16)
    assert (got == padded).all() and same_f32(host(bscales), host(scales))
    pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group)
    st, y = pl.forward_a8(blocked, bcodes, bscales)
    blocked.synchronize()
    assert st == 0 and same_f32(host(y), want), blocked.last_variant
    assert ("gemv" in blocked.last_variant) == (k != 5000)
    if k == 1000:  # more than 32 rows on the same context: row major, through the GEMM
        big = cases.packed_case(40, k, n, group, 77, True)
        _, want_big = oracle.packed_linear(big["x"], words, c["scales"], c["bias"], n, group)
        a8, sc = packed_prepare_i8(blocked, dev(big["x"]))
        assert tuple(a8.shape) == (40, k)
        st, y = pl.forward_a8(blocked, a8, sc)
        blocked.synchronize()
        assert st == 0 and same_f32(host(y), want_big)
    pl.close(), plain.close(), blocked.close()


@pytest.mark.parametrize("k,group,instance,bits",
                         [(1024, 128, "fit8x4", 8), (2048, 64, "fit16x4", 8), (2048, 32, "fit16x4", 8), (3072, 128, "fit8x12", 8),
                          (4096, 128, "fit16x8", 8), (4096, 256, "fit16x8", 8), (4090, 64, "fit16x8", 8), (8192, 128, "fit16x16", 8),
                          (14336, 128, "fit16x28", 8),
                          (1024, 128, "fit4x4", 4), (2048, 64, "fit8x4", 4), (3072, 128, "fit8x6", 4), (4096, 128, "fit16x4", 4),
                          (4096, 32, "fit16x4", 4), (4070, 256, "fit16x4", 4), (8192, 128, "fit16x8", 4), (14336, 128, "fit16x14", 4)])
def test_exact_fit_gemv(oracle, k, group, instance, bits):
    """The straight-line streaming kernel for a K whose blocks divide evenly over the waves: every
    instance for eight- and four-bit weights, rows on both sides of its LDS-copy limit, both places where the products are formed
    (lane-parallel over the parked dots, or by the parking wave in its accumulators), both activation
    layouts, a row whose scale is NaN, an n that ends inside a panel -- the oracle's bits each time;
    and the general kernel still gives them when the exact-fit one is ruled out by name."""
    import volvoxai_amd as vx
    from volvoxai_amd.w8a8 import packed_prepare_i8
    n = 6150 if k <= 4096 else 70  # 193 panels: taken without being named; the long rows only by name
    plain, blocked = vx.Context(0, None), vx.Context(0, None)
    blocked.set_activation_layout(True)
    c = cases.packed_case(32, k, n, group, 4000 + k + group, True, special_rows=True)
    words = oracle.pack_w8_words(c["w"]) if bits == 8 else oracle.pack_w4_words(cases.four_bit(c["w"]))
    pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group, weight_bits=bits)
    waves, bpw = (int(v) for v in instance[3:].split("x"))
    groups = (k + group - 1) // group
    try:
        for rows in (1, 2, 4, 5, 8, 9, 16, 32):
            if k == 3072 and bits == 8:  # two instances: eight waves of twelve blocks up to eight rows, then twelve of eight
                instance = "fit8x12" if rows <= 8 else "fit12x8"
                waves = int(instance[3:].split("x")[0])
            # (the products of every group, the waves' scales and, for few rows, their activation slices share LDS)
            fixed = groups * rows * 128 + waves * (groups // waves * 32 + 32) * 4
            if fixed > 156 * 1024:  # (with the activation slices on top, while that stays within 80 KiB)
                continue
            x = c["x"][:rows].copy()
            if rows >= 2:
                x[-1, 7 % k] = np.nan  # a row that is not finite: a NaN scale, a NaN output row
            _, want = oracle.packed_linear(x, words, c["scales"], c["bias"], n, group, bits=bits)
            for ctx in (plain, blocked):
                codes, scales = packed_prepare_i8(ctx, dev(x))
                if k == 3072 and bits == 8:  # either instance, named in full
                    for named_instance in ("fit8x12", "fit12x8"):
                        vx.force_variant("gemv." + named_instance)
                        st, y = pl.forward_a8(ctx, codes, scales)
                        ctx.synchronize()
                        assert st == 0 and same_f32(host(y), want) and ctx.last_variant.endswith(named_instance), (rows, ctx.last_variant)
                for force in (None, "gemv.fit.lprod", "gemv.fit.rprod", "gemv.nofit"):
                    vx.force_variant(force)
                    st, y = pl.forward_a8(ctx, codes, scales)
                    ctx.synchronize()
                    assert st == 0 and same_f32(host(y), want), (rows, force, ctx.last_variant)
                    # (unnamed it takes enough panels to fill the device, and four-bit weights only while the rows fit LDS)
                    named = force in ("gemv.fit.lprod", "gemv.fit.rprod") or (force is None and n >= 6144 and (bits == 8 or rows <= 8))
                    assert ctx.last_variant.endswith(instance) == named, (rows, force, ctx.last_variant)
        # one and two f32 rows: the kernel prepares them itself (the reference's single-row route in one launch);
        # a zero row, a row with an infinity, a plain one
        for rows, special in ((1, None), (1, "zero"), (2, "inf"), (2, None)):
            x = c["x"][5:5 + rows].copy()
            if special == "zero":
                x[0] = 0.0
            if special == "inf":
                x[1, k // 3] = np.inf
            _, want = oracle.packed_linear(x, words, c["scales"], c["bias"], n, group, bits=bits)
            for force in (None, "gemv.nofit"):
                vx.force_variant(force)
                st, y = pl.forward_f32(plain, dev(x))
                plain.synchronize()
                assert st == 0 and same_f32(host(y), want), (rows, special, force, plain.last_variant)
                prepared_here = force is None and n >= 6144 and k % (32 if bits == 8 else 64) == 0
                if k == 3072 and bits == 8:
                    instance = "fit8x12"
                assert plain.last_variant.endswith(instance + "-prep") == prepared_here, (rows, force, plain.last_variant)
    finally:
        vx.force_variant(None)
        pl.close(), plain.close(), blocked.close()


@pytest.mark.parametrize("k,group,instance", [(1024, 128, "fit8x4"), (1024, 32, "fit8x4"), (2048, 64, "fit16x4"), (2048, 32, "fit16x4"),
                                              (3072, 128, "fit12x8"), (3072, 256, "fit12x8"), (4096, 128, "fit16x8"), (4096, 256, "fit16x8"),
                                              (4090, 32, "fit16x8")])
def test_exact_fit_gemv_shared_panels(oracle, k, group, instance):
    """Few panels: four (N = 1000) or two (N = 4090) workgroups of the straight-line kernel share a panel's
    channels -- the decoder's projections at 32 rows.  Rows on both sides of the LDS-copy limit, both places
    where the products are formed, both activation layouts, a NaN row: the oracle's bits each time."""
    import volvoxai_amd as vx
    from volvoxai_amd.w8a8 import packed_prepare_i8
    plain, blocked = vx.Context(0, None), vx.Context(0, None)
    blocked.set_activation_layout(True)
    try:
        for n, suffix in ((1000, "c8"), (4090, "c16")):
            c = cases.packed_case(32, k, n, group, 4200 + k + n, True, special_rows=True)
            words = oracle.pack_w8_words(c["w"])
            pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group)
            waves = int(instance[3:].split("x")[0])
            groups, ch = (k + group - 1) // group, 32 // (4 if suffix == "c8" else 2)
            for rows in (1, 3, 8, 9, 32):
                if groups * rows * ch * 4 + waves * (groups // waves * ch + 32) * 4 > 156 * 1024:
                    continue  # (the products of every group do not fit the LDS: not a shape of the streaming kernels)
                x = c["x"][:rows].copy()
                if rows >= 2:
                    x[-1, 11 % k] = np.nan
                _, want = oracle.packed_linear(x, words, c["scales"], c["bias"], n, group)
                for ctx in (plain, blocked):
                    codes, scales = packed_prepare_i8(ctx, dev(x))
                    for force in (None, "gemv.fit.lprod", "gemv.fit.rprod", "gemv.nofit"):
                        vx.force_variant(force)
                        st, y = pl.forward_a8(ctx, codes, scales)
                        ctx.synchronize()
                        assert st == 0 and same_f32(host(y), want), (n, rows, force, ctx.last_variant)
                        assert ctx.last_variant.endswith(instance + suffix) == (force != "gemv.nofit"), (n, rows, force, ctx.last_variant)
            pl.close()
    finally:
        vx.force_variant(None)
        plain.close(), blocked.close()


def test_packed_output_window(ctx, oracle):
    """first_unit / unit_count of the PackedLinear descriptor (llm_ops.h:48-52) on both entry points: the
    reference's window list on 11 rows (test_packed_linear_i8.c:263-265), the whole output array --
    guard values included -- against the oracle's; a window that does not fit is refused untouched."""
    import torch
    import volvoxai_amd as vx
    for k, n, group, bits in [(257, 19, 64, 8), (1283, 5, 128, 8), (320, 13, 32, 4), (4096, 6150, 128, 8)]:
        rows = 11 if n < 100 else 3
        c = cases.packed_case(rows, k, n, group, 4100 + k, True, special_rows=rows >= 5)
        words = oracle.pack_w8_words(c["w"]) if bits == 8 else oracle.pack_w4_words(cases.four_bit(c["w"]))
        pl = vx.PackedLinear(words, c["scales"], c["bias"], k, n, group, weight_bits=bits)
        xd = dev(c["x"])
        windows = [(0, 0), (1, rows * n - 2), (n - 1, 4 * n + 2), (n + 2, 3 * n - 2), (n, 8 * n), (3, 14), (2 * n, n), (0, 1)]
        for first, count in windows:
            if first > rows * n or (count or rows * n) > rows * n - first:
                continue
            want = np.full((rows, n), 12345.0, np.float32)
            assert oracle.packed_linear_window(c["x"], words, c["scales"], c["bias"], want, group, first, count, bits=bits) == 0
            got = np.full((rows, n), 12345.0, np.float32)
            st, _ = vx.packed_linear_f32(c["x"], words, c["scales"], c["bias"], k, n, group, groups=bits,
                                         first_unit=first, unit_count=count, out=got)
            assert st == 0 and (got.view(np.uint32) == want.view(np.uint32)).all(), (k, n, first, count)
            yd = torch.full((rows, n), 12345.0, dtype=torch.float32, device="cuda")
            st = pl.forward_f32_window(ctx, xd, yd, first, count)
            ctx.synchronize()
            assert st == 0 and (host(yd).view(np.uint32) == want.view(np.uint32)).all(), (k, n, first, count, ctx.last_variant)
        for first, count in [(rows * n + 1, 0), (2, rows * n - 1), (rows * n, 0)]:
            got = np.full((rows, n), 12345.0, np.float32)
            st, _ = vx.packed_linear_f32(c["x"], words, c["scales"], c["bias"], k, n, group, groups=bits,
                                         first_unit=first, unit_count=count, out=got)
            assert st == -1 and (got == 12345.0).all()
            yd = torch.full((rows, n), 12345.0, dtype=torch.float32, device="cuda")
            assert pl.forward_f32_window(ctx, xd, yd, first, count) == -1
            ctx.synchronize()
            assert (host(yd) == 12345.0).all()
        pl.close()
    vx.library().vxhip_resident_weights_clear()
