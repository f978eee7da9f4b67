"""Pins the CPU oracle: against the reference's own known-answer vectors,
against outputs of the reference's C kernels (committed digests, and live when
oracle/_ref is built), and against closed forms / brute force that a dropped
term, wrong sign or transposed operand would break."""
import hashlib
import json
from pathlib import Path

import numpy as np
import pytest

import _cases as cases

GOLDEN = Path(__file__).parent / "golden"
KATS = json.loads((GOLDEN / "reference_kats.json").read_text())
VECTORS = json.loads((GOLDEN / "reference_vectors.json").read_text())
I8, U8 = cases.DTYPE_I8, cases.DTYPE_U8
DT = {"int8": I8, "uint8": U8}


def fval(v):
    if isinstance(v, str):
        return float.fromhex(v) if v.startswith("0x") else float(v)
    return float(v)


def check_digest(arr, expected):
    arr = np.ascontiguousarray(arr)
    assert list(arr.shape) == expected["shape"] and str(arr.dtype) == expected["dtype"]
    head = arr.reshape(-1)[:32]
    head = head.view(np.uint32) if arr.dtype == np.float32 else head
    assert [int(v) for v in head] == expected["head"]
    assert hashlib.sha256(arr.tobytes()).hexdigest() == expected["sha256"]


# ---- known-answer vectors held by the reference's tests -------------------------

def test_qlinear_literal_kat(oracle):
    k = KATS["qlinear_literal"]
    ok, y = oracle.qlinear(np.array(k["input"], np.int8), np.array(k["weight"], np.int8),
                           np.array(k["bias"], np.int32), np.array(k["weight_scales"], np.float32),
                           np.array(k["weight_zero_points"], np.int32), k["input_scale"],
                           k["input_zero_point"], k["output_scale"], k["output_zero_point"], I8, I8, I8)
    assert ok == 1 and y.tolist() == k["expected"]


def test_round_and_requantize_kats(oracle):
    for value, expected in KATS["round_ties_even"]["cases"]:
        assert oracle.round_ties_even(value) == expected
    for c in KATS["requantize"]["cases"]:
        assert oracle.requantize(fval(c["value"]), c["min"], c["max"], c["nan_value"]) == c["expected"]
    for value, expected in KATS["packed_round_i8"]["cases"]:
        assert oracle.packed_round_i8(value) == expected


def test_multiplier_contract(oracle):
    grid = [np.float32(fval(v)) for v in KATS["multiplier"]["scale_grid_hex"]]
    for a in grid:
        for b in grid:
            for c in grid:
                ok, m = oracle.multiplier(a, b, c)
                want = np.float32(np.float32(a * b) / c)  # f32(f32(a*b)/c), numpy keeps f32
                assert ok and m.view(np.uint32) == want.view(np.uint32)
                # the other association differs for some triples; the oracle must not use it
    for a, b, c in KATS["multiplier"]["invalid"]:
        ok, _ = oracle.multiplier(fval(a), fval(b), fval(c))
        assert not ok


def halfway_inputs(k):
    x = np.zeros((k["rows"], k["channels"]), np.uint8)
    run = k["input_run"]
    x[:, :run["count"]] = run["value"]
    x[:, run["count"]] = run["then"]
    return x


def test_affine_halfway_kat(oracle):
    k = KATS["affine_halfway"]
    x = halfway_inputs(k)
    for wd in k["weight_dtypes"]:
        w = np.full((k["outputs"], k["channels"]), k["weight_value"], np.int8 if wd == "int8" else np.uint8)
        ok, y = oracle.qlinear(x, w, np.zeros(k["outputs"], np.int32),
                               np.full(k["outputs"], k["weight_scale"], np.float32),
                               np.zeros(k["outputs"], np.int32), k["input_scale"], k["input_zero_point"],
                               k["output_scale"], k["output_zero_point"], U8, DT[wd], I8)
        assert ok == 1 and (y == k["expected_all"]).all()
    # the fused form really is different here, so the KAT does discriminate
    acc, mult = 17 * 255 + 40, np.float32(np.float32(np.float32(0.015) * np.float32(0.008)) / np.float32(0.03))
    fused = np.float64(acc) * np.float64(mult) - 17.0
    assert round(float(np.float32(fused))) == 1


def near_tie_case():
    k = KATS["packed_near_tie_logits"]
    x = np.zeros((1, k["k"]), np.float32)
    for idx, v in k["x_nonzero"].items():
        x[0, int(idx)] = v
    w = np.zeros((k["n"], k["k"]), np.int8)
    for row, col in k["weight_plus_one_at"]:
        w[row, col] = 1
    return k, x, w


def test_packed_near_tie_kat(oracle):
    k, x, w = near_tie_case()
    words = oracle.pack_w8_words(w)
    assert words[0, 1] == 0x80808080  # the reference's W8 zero word
    st, y = oracle.packed_linear(x, words, np.array(k["scales"], np.float32),
                                 np.array(k["bias"], np.float32), k["n"], k["group_size"])
    assert st == 0 and int(np.argmax(y[0])) == k["expected_argmax"]
    s_a = np.float32(np.float32(1.0003) / np.float32(127.0))
    term = np.float32(np.float32(127.0) * np.float32(s_a * np.float32(1.0)))
    assert y[0, 1].view(np.uint32) == np.float32(term + np.float32(0.0)).view(np.uint32)
    assert y[0, 0].view(np.uint32) == np.float32(term + np.float32(-0.0002)).view(np.uint32)


# ---- outputs of the reference's C kernels (committed digests) -------------------

def build_qcase(entry):
    kind, p = entry["kind"], entry["params"]
    if kind == "isa_parity":
        return cases.isa_parity_case(**p)
    if kind == "quant_gemm":
        return cases.quant_gemm_case(**p)
    return cases.qlinear_random_case(**p)


@pytest.mark.parametrize("entry", VECTORS["qlinear"], ids=lambda e: f"{e['kind']}-{'-'.join(str(v) for v in e['params'].values())}")
def test_qlinear_matches_reference_vectors(oracle, entry):
    c = build_qcase(entry)
    ok, y = oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"],
                           c["s_out"], c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"])
    assert ok == 1
    check_digest(y, entry["expected"])


@pytest.mark.parametrize("entry", VECTORS["rowscale"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_rowscale_matches_reference_vectors(oracle, entry):
    c = cases.rowscale_case(**entry["params"])
    ok, y, acc = oracle.qlinear_rowscale(c["x"], c["w"], c["scales"], c["zps"], c["row_scales"],
                                         c["s_out"], c["zp_out"])
    assert ok == 1
    check_digest(y, entry["expected_without_bias"])
    brute = c["x"].astype(np.int64) @ c["w"].astype(np.int64).T
    assert (acc == brute).all()


@pytest.mark.parametrize("entry", VECTORS["requantize"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_requantize_matches_reference_vectors(oracle, entry):
    c = cases.requantize_case(**entry["params"])
    ok, y = oracle.requantize_linear(c["x"], c["s_in"], c["zp_in"], c["s_out"], c["zp_out"], c["in_dtype"], c["out_dtype"])
    assert ok == 1
    check_digest(y, entry["expected"])


@pytest.mark.parametrize("entry", VECTORS["packed"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_packed_matches_reference_vectors(oracle, entry):
    c = cases.packed_case(**entry["params"])
    st, y = oracle.packed_linear(c["x"], oracle.pack_w8_words(c["w"]), c["scales"], c["bias"], c["n"], c["group"])
    assert st == 0
    check_digest(y, entry["expected"])


@pytest.mark.parametrize("entry", VECTORS["packed_w4"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_packed_w4_matches_reference_vectors(oracle, entry):
    c = cases.packed_case(**entry["params"])
    words = oracle.pack_w4_words(cases.four_bit(c["w"]))
    st, y = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=4)
    assert st == 0
    check_digest(y, entry["expected"])


def window_case(entry, oracle):
    params = entry["params"]
    c = cases.packed_case(**{k: v for k, v in params.items() if k != "bits"}, special_rows=True)
    words = oracle.pack_w8_words(c["w"]) if params["bits"] == 8 else oracle.pack_w4_words(cases.four_bit(c["w"]))
    return c, words


@pytest.mark.parametrize("entry", VECTORS["packed_window"],
                         ids=lambda e: f"{'x'.join(str(v) for v in e['params'].values())}-{e['first_unit']}+{e['unit_count']}")
def test_packed_output_window_matches_reference_vectors(oracle, entry):
    """first_unit / unit_count: the window's elements are the full call's, everything else keeps the
    guard value -- the whole array against what the reference's kernel left in it."""
    c, words = window_case(entry, oracle)
    y = np.full((entry["params"]["rows"], c["n"]), 12345.0, np.float32)
    st = oracle.packed_linear_window(c["x"], words, c["scales"], c["bias"], y, c["group"], entry["first_unit"],
                                     entry["unit_count"], bits=entry["params"]["bits"])
    assert st == 0
    check_digest(y, entry["expected"])
    # and what the rule fixes without any reference: window = slice of the full output, rest = guard
    _, full = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=entry["params"]["bits"])
    first, count = entry["first_unit"], entry["unit_count"] or full.size
    flat, want = y.reshape(-1), full.reshape(-1)
    inside = np.zeros(full.size, bool)
    inside[first:first + count] = True
    assert (flat[~inside] == 12345.0).all()
    nan = np.isnan(want)
    assert (np.isnan(flat[inside]) == nan[inside]).all()
    assert (flat.view(np.uint32)[inside & ~nan] == want.view(np.uint32)[inside & ~nan]).all()


def test_packed_output_window_refusals(oracle):
    c = cases.packed_case(4, 64, 6, 32, 5)
    words = oracle.pack_w8_words(c["w"])
    for first, count in [(25, 0), (0, 25), (2, 23), (24, 1)]:  # 24 units in all
        y = np.full((4, 6), 12345.0, np.float32)
        assert oracle.packed_linear_window(c["x"], words, c["scales"], c["bias"], y, 32, first, count) == -1
        assert (y == 12345.0).all()
    y = np.full((4, 6), 12345.0, np.float32)
    assert oracle.packed_linear_window(c["x"], words, c["scales"], c["bias"], y, 32, 24, 0) == -1  # 0 units = all 24: past the end
    assert oracle.packed_linear_window(c["x"], words, c["scales"], c["bias"], y, 32, 23, 1) == 0
    assert (y.reshape(-1)[:23] == 12345.0).all() and y[3, 5] != 12345.0


def test_live_reference_packed_output_window(oracle, reference):
    rng = np.random.default_rng(77)
    for trial in range(40):
        rows, k, n = int(rng.integers(1, 9)), int(rng.choice([31, 64, 200])), int(rng.integers(1, 12))
        group = int(rng.choice([32, 64, 128, 256]))
        c = cases.packed_case(rows, k, n, group, 300 + trial, with_bias=bool(trial % 2), special_rows=True)
        words = oracle.pack_w8_words(c["w"])
        first = int(rng.integers(0, rows * n + 2))
        count = int(rng.integers(0, rows * n + 2))
        a = np.full((rows, n), 12345.0, np.float32)
        b = a.copy()
        sa = oracle.packed_linear_window(c["x"], words, c["scales"], c["bias"], a, group, first, count)
        sb, _ = reference.packed_linear(c["x"], words, c["scales"], c["bias"], n, group, first_unit=first, unit_count=count, out=b)
        assert sa == sb, (trial, first, count)
        assert (a.view(np.uint32) == b.view(np.uint32)).all(), (trial, first, count)


@pytest.mark.parametrize("bits", [3, 2])
def test_packed_low_bit_matches_reference_vectors(oracle, bits):
    for entry in VECTORS[f"packed_w{bits}"]:
        c = cases.packed_case(**entry["params"])
        words = oracle.pack_low_bit_words(cases.low_bit(c["w"], bits), bits)
        st, y = oracle.packed_linear(c["x"], words, c["scales"], c["bias"], c["n"], c["group"], bits=bits)
        assert st == 0
        check_digest(y, entry["expected"])


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_packed_low_bit_codes_read_back(oracle, bits):
    """Code j of a row sits at bit j*bits of the row's words (a three-bit code may straddle two
    words); a one-hot activation reads exactly that weight back."""
    k, n = 75, 2
    rng = np.random.default_rng(bits)
    w = rng.integers(-(1 << (bits - 1)), 1 << (bits - 1), (n, k)).astype(np.int8)
    words = oracle.pack_low_bit_words(w, bits)
    assert words.shape == (n, (k // 32) * bits + ((k % 32) * bits + 31) // 32)
    stream = int.from_bytes(words[1].tobytes(), "little")
    for j in (0, 9, 10, 20, 21, 31, 32, 74):
        assert ((stream >> (j * bits)) & ((1 << bits) - 1)) - (1 << (bits - 1)) == int(w[1, j])
    scales = np.ones((n, 3), np.float32)
    for j in (0, 10, 21, 42, 74):
        a8 = np.zeros((1, k), np.int8); a8[0, j] = 1
        st, y, _ = oracle.packed_linear_a8(a8, np.ones(1, np.float32), words, scales, None, n, 32, bits=bits)
        assert st == 0 and y[0].tolist() == w[:, j].astype(np.float32).tolist()


def test_packed_w4_codes_and_group_dots(oracle):
    """Nibble j of word j//8 holds value+8, lowest nibble first; a one-hot activation reads one
    weight back, and the group dots are the plain integer products."""
    k, n, g = 75, 3, 32
    rng = np.random.default_rng(3)
    w = rng.integers(-8, 8, (n, k)).astype(np.int8)
    words = oracle.pack_w4_words(w)
    assert words.shape == (n, 10)  # (75 // 32) * 4 + ceil(11 * 4 / 32)
    for j in (0, 7, 8, 31, 32, 74):
        assert int((words[1, j // 8] >> (4 * (j % 8))) & 15) - 8 == int(w[1, j])
    assert int(words[0, 9] >> 12) == 0x88888  # the unused tail holds the code of zero
    scales = np.ones((n, 3), np.float32)
    for j in (0, 33, 74):
        a8 = np.zeros((1, k), np.int8); a8[0, j] = 1
        st, y, _ = oracle.packed_linear_a8(a8, np.ones(1, np.float32), words, scales, None, n, g, bits=4)
        assert st == 0 and y[0].tolist() == w[:, j].astype(np.float32).tolist()
    a8 = rng.integers(-127, 128, (4, k)).astype(np.int8)
    st, y, acc = oracle.packed_linear_a8(a8, np.ones(4, np.float32), words, scales, None, n, g, bits=4)
    assert st == 0 and (acc == a8.astype(np.int64) @ w.astype(np.int64).T).all()
    assert (y == acc.astype(np.float32)).all()  # sums of three small integers are exact in f32


# ---- live comparison with the reference build ------------------------------------

def test_live_reference_qlinear(oracle, reference):
    rng = np.random.default_rng(5)
    for (m, k, n) in [(7, 129, 31), (2, 33, 36), (33, 64, 64)]:
        for idt in (I8, U8):
            for wdt in (I8, U8):
                c = cases.qlinear_random_case(m, k, n, int(rng.integers(1 << 30)), idt, wdt, U8, False)
                args = (c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"],
                        c["s_out"], c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"])
                a = oracle.qlinear(*args)
                b = reference.qlinear_portable(*args)
                d = reference.qlinear_native(*args)
                assert a[0] == b[0] == d[0] == 1
                assert (a[1] == b[1]).all() and (a[1] == d[1]).all()


def test_live_reference_declines_like_oracle(oracle, reference):
    c = cases.qlinear_random_case(2, 16, 4, 3)
    base = [c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"], c["s_out"],
            c["zp_out"], c["in_dtype"], c["w_dtype"], c["out_dtype"]]
    bad_scale = list(base); bad_scale[5] = 0.0
    bad_zp = list(base); bad_zp[6] = 300
    tiny = list(base); tiny[5] = 1e-30; tiny[3] = np.full(4, 1e-30, np.float32)  # product underflows to 0
    huge_bias = list(base); huge_bias[2] = np.full(4, 2**31 - 1, np.int32)       # first add overflows
    for args in (bad_scale, bad_zp, tiny, huge_bias):
        assert oracle.qlinear(*args)[0] == reference.qlinear_portable(*args)[0] == 0


def test_live_reference_packed_and_bias_rule(oracle, reference):
    for p in [dict(rows=6, k=200, n=9, group=64, seed=1, special_rows=True),
              dict(rows=5, k=31, n=3, group=32, seed=2, with_bias=False)]:
        c = cases.packed_case(**p)
        words = oracle.pack_w8_words(c["w"])
        x = c["x"].copy()
        if p["rows"] > 5:
            x[5, 3] = np.inf
        a = oracle.packed_linear(x, words, c["scales"], c["bias"], c["n"], c["group"])
        b = reference.packed_linear(x, words, c["scales"], c["bias"], c["n"], c["group"])
        assert a[0] == b[0] == 0
        nan = np.isnan(b[1])
        assert (np.isnan(a[1]) == nan).all()
        assert (a[1].view(np.uint32)[~nan] == b[1].view(np.uint32)[~nan]).all()
        for bits in (4, 3, 2):
            lw = oracle.pack_low_bit_words(cases.low_bit(c["w"], bits), bits)
            a = oracle.packed_linear(x, lw, c["scales"], c["bias"], c["n"], c["group"], bits=bits)
            b = reference.packed_linear(x, lw, c["scales"], c["bias"], c["n"], c["group"], bits=bits)
            assert a[0] == b[0] == 0
            nan = np.isnan(b[1])
            assert (np.isnan(a[1]) == nan).all()
            assert (a[1].view(np.uint32)[~nan] == b[1].view(np.uint32)[~nan]).all()
    rng = np.random.default_rng(9)
    b = rng.normal(0, 0.3, 64).astype(np.float32)
    sw = rng.uniform(0.002, 0.02, 64).astype(np.float32)
    st1, q1 = oracle.ptq_pack_bias(b, 0.0173, sw)
    st2, q2 = reference.ptq_pack_bias(b, 0.0173, sw)
    assert st1 == st2 == 0 and (q1 == q2).all()


def glue_argmax_rows():
    """Rows that separate the scan's rules: ties, a NaN at the front, in the middle, infinities."""
    rng = np.random.default_rng(12)
    x = rng.normal(0, 1, (12, 37)).astype(np.float32)
    x[1, :] = 0.5                              # all equal -> 0
    x[2, 5] = x[2, 20] = 9.0                   # tie -> first
    x[3, 0] = np.nan                           # NaN in element 0 keeps 0
    x[4, 7] = np.nan; x[4, 30] = 8.0           # NaN elsewhere is skipped
    x[5, :] = -np.inf                          # all -inf -> 0
    x[6, 3] = np.inf; x[6, 4] = np.inf
    x[7, :] = np.nan
    x[8, 0] = -0.0; x[8, 1:] = -1.0; x[8, 9] = 0.0   # +0 does not beat -0
    x[9, 36] = 50.0                            # last element
    return x


def test_live_reference_embedding_and_argmax(oracle, reference):
    x = glue_argmax_rows()
    got = oracle.argmax_rows(x)
    assert (got == reference.argmax_rows(x)).all()
    assert got[:10].tolist() == [int(np.argmax(x[0])), 0, 5, 0, 30, 0, 3, 0, 0, 36]
    big = np.random.default_rng(2).normal(0, 1, (3, 32000)).astype(np.float32)
    assert (oracle.argmax_rows(big) == np.argmax(big, axis=1)).all()
    table = np.random.default_rng(3).normal(0, 1, (50, 24)).astype(np.float32)
    tokens = np.array([0, 49, 7, 7, 13], np.int32)
    e = oracle.embedding(tokens, table)
    assert (e == reference.embedding(tokens, table)).all() and (e == table[tokens]).all()


# ---- what the mathematics fixes ---------------------------------------------------

def test_accumulator_is_the_integer_gemm(oracle):
    c = cases.qlinear_random_case(9, 77, 21, 11, U8, U8, I8, False)
    ok, y, acc = oracle.qlinear(c["x"], c["w"], c["bias"], c["scales"], c["zps"], c["s_in"], c["zp_in"],
                                c["s_out"], c["zp_out"], U8, U8, I8, want_acc=True)
    xs = c["x"].astype(np.int64) - c["zp_in"]
    ws = c["w"].astype(np.int64) - c["zps"][:, None]
    assert ok == 1 and (acc == xs @ ws.T + c["bias"]).all()


def test_packed_prepare_closed_form(oracle):
    x = np.array([[0.0, -2.0, 1.0, 0.5, 127.0 / 254.0 * 2.0]], np.float32)  # max 2 -> scale 2/127
    a, s, fin = oracle.packed_prepare(x)
    assert fin[0] == 1 and s[0].view(np.uint32) == np.float32(np.float32(2.0) / np.float32(127.0)).view(np.uint32)
    assert a[0].tolist() == [0, -127, 64, 32, 64]  # 63.5 -> 64 (even), 31.75 -> 32
    z, sz, _ = oracle.packed_prepare(np.zeros((1, 8), np.float32))
    assert sz[0] == 1.0 and not z.any()
    _, s_tiny, _ = oracle.packed_prepare(np.full((1, 4), 2.0 ** -140, np.float32))
    assert s_tiny[0] == np.float32(2.0 ** -126)
    _, _, bad = oracle.packed_prepare(np.array([[1.0, np.nan]], np.float32))
    assert bad[0] == 0


def test_packed_group_order_matters_and_is_ascending(oracle):
    # terms of very different magnitude: ascending order rounds differently from descending
    k, g = 64, 32
    a8 = np.zeros((1, k), np.int8); a8[0, 0] = 127; a8[0, 32] = 1
    w = np.zeros((1, k), np.int8); w[0, 0] = 127; w[0, 32] = 1
    scales = np.array([[1.0, 2.0 ** -20]], np.float32)
    st, y, acc = oracle.packed_linear_a8(a8, np.ones(1, np.float32), oracle.pack_w8_words(w), scales, None, 1, g)
    want = np.float32(np.float32(0.0 + np.float32(16129.0)) + np.float32(np.float32(1.0) * np.float32(2.0 ** -20)))
    assert st == 0 and y[0, 0].view(np.uint32) == want.view(np.uint32) and acc[0, 0] == 16130


def test_quantize_dequantize_rules(oracle):
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, np.nan, np.inf, -np.inf, 1000.0, -1000.0, 0.3], np.float32)
    ok, q = oracle.quantize(x, 1.0, 0, I8)
    assert ok == 1 and q.tolist() == [0, 2, 2, 0, -2, 0, 127, -128, 127, -128, 0]
    ok, q = oracle.quantize(x, 1.0, 7, U8)
    assert q.tolist()[:6] == [8, 8, 10, 6, 6, 7]  # 7.5->8, 8.5->8, 9.5->10, 6.5->6, 5.5->6, NaN->zp
    ok, d = oracle.dequantize(np.array([-128, 0, 127], np.int8), 0.1, -3, I8)
    want = [np.float32((v + 3) * float(np.float32(0.1))) for v in (-128, 0, 127)]
    assert [v.view(np.uint32) for v in d] == [w.view(np.uint32) for w in want]


def test_requantize_linear_rules(oracle):
    """RequantizeLinear (portable_inference_kernels.inc:2437-2463) against what its definition fixes: the
    identity between equal descriptors; the I8 <-> U8 change of representation (zero points 128 apart:
    the byte with its top bit flipped); ties to even and saturation on exact halves; the association
    f32(s_in / s_out) first, then a rounded product and a rounded sum (a case where multiplying by s_in
    and dividing by s_out, or a fused multiply-add, gives another byte); the declines."""
    every = np.arange(-128, 128).astype(np.int8)
    ok, q = oracle.requantize_linear(every, 0.37, -5, 0.37, -5, I8, I8)
    assert ok == 1 and (q == every).all()
    ok, q = oracle.requantize_linear(every, 0.02, -3, 0.02, 125, I8, U8)
    assert ok == 1 and (q == (every.view(np.uint8) ^ 0x80)).all()
    ok, q = oracle.requantize_linear(every.view(np.uint8), 0.02, 125, 0.02, -3, U8, I8)
    assert ok == 1 and (q == (every.view(np.uint8) ^ 0x80).view(np.int8)).all()
    # multiplier 0.5 exactly: halves tie to even, zero point added after the product
    ok, q = oracle.requantize_linear(np.array([1, 3, 5, -1, -3, 127, -128], np.int8), 1.0, 0, 2.0, 0, I8, I8)
    assert q.tolist() == [0, 2, 2, 0, -2, 64, -64]
    ok, q = oracle.requantize_linear(np.array([1, 3, 5, -1, -3], np.int8), 1.0, 0, 2.0, 10, I8, U8)
    assert q.tolist() == [10, 12, 12, 10, 8]      # 10.5 -> 10, 11.5 -> 12, 12.5 -> 12, 9.5 -> 10, 8.5 -> 8
    # saturation at both ends of either type
    ok, q = oracle.requantize_linear(np.array([-128, 127], np.int8), 4.0, 0, 1.0, 0, I8, I8)
    assert q.tolist() == [-128, 127]
    ok, q = oracle.requantize_linear(np.array([-128, 127], np.int8), 4.0, 0, 1.0, 3, I8, U8)
    assert q.tolist() == [0, 255]
    # the association: descriptor pairs where the alternatives give another byte (found by search over
    # seeded candidates, all in f32 numpy arithmetic), then the oracle's byte against the defined one
    rng = np.random.default_rng(17)
    n = 4_000_000
    s_in = rng.uniform(0.01, 0.1, n).astype(np.float32)
    s_out = rng.uniform(0.01, 0.1, n).astype(np.float32)
    c = rng.integers(-128, 128, n).astype(np.float32)          # q - zp_in with zp_in = 0
    zp_out = rng.integers(-20, 20, n).astype(np.float32)
    m = s_in / s_out                                            # f32
    defined = np.clip(np.rint((c * m) + zp_out), -128, 127)     # each operation rounded to f32
    other = np.clip(np.rint((c * s_in) / s_out + zp_out), -128, 127)
    fused = np.clip(np.rint((c.astype(np.float64) * m.astype(np.float64) + zp_out).astype(np.float32)), -128, 127)
    differ = np.flatnonzero((defined != other) | (defined != fused))
    assert differ.size > 0   # (rare: a handful in four million -- the live comparison below carries the rest)
    for i in differ[:50]:
        ok, q = oracle.requantize_linear(np.array([int(c[i])], np.int8), s_in[i], 0, s_out[i], int(zp_out[i]), I8, I8)
        assert ok == 1 and int(q[0]) == int(defined[i]), (s_in[i], s_out[i], c[i], zp_out[i])
    # declines: scales, zero points, a multiplier that leaves f32
    x = np.array([1], np.int8)
    assert oracle.requantize_linear(x, 0.0, 0, 1.0, 0, I8, I8)[0] == 0
    assert oracle.requantize_linear(x, 1.0, 0, float("inf"), 0, I8, I8)[0] == 0
    assert oracle.requantize_linear(x, 1.0, 200, 1.0, 0, I8, I8)[0] == 0
    assert oracle.requantize_linear(x, 1.0, 0, 1.0, -1, I8, U8)[0] == 0
    assert oracle.requantize_linear(x, 3e38, 0, 1e-38, 0, I8, I8)[0] == 0     # s_in / s_out overflows
    assert oracle.requantize_linear(x, 1e-38, 0, 3e38, 0, I8, I8)[0] == 0     # ... or underflows to zero


def test_live_reference_requantize_linear(oracle, reference):
    """The reference's own requantize_linear_i8u8, compiled from its sources: every byte of either type
    through random descriptor pairs, and the same declines."""
    rng = np.random.default_rng(23)
    for trial in range(300):
        idt, odt = (I8, U8)[trial % 2], (I8, U8)[(trial // 2) % 2]
        x = np.arange(256).astype(np.uint8).view(np.int8 if idt == I8 else np.uint8)
        s_in, s_out = np.float32(rng.uniform(0.001, 0.2)), np.float32(rng.uniform(0.001, 0.2))
        zp_in = int(rng.integers(-128, 128) if idt == I8 else rng.integers(0, 256))
        zp_out = int(rng.integers(-128, 128) if odt == I8 else rng.integers(0, 256))
        a = oracle.requantize_linear(x, s_in, zp_in, s_out, zp_out, idt, odt)
        b = reference.requantize_linear(x, s_in, zp_in, s_out, zp_out, idt, odt)
        assert a[0] == b[0] == 1 and (a[1] == b[1]).all(), (trial, s_in, s_out, zp_in, zp_out)
    x = np.array([1, 2], np.int8)
    for args in ((0.0, 0, 1.0, 0, I8, I8), (1.0, 0, -1.0, 0, I8, I8), (1.0, 128, 1.0, 0, I8, I8), (1.0, 0, 1.0, 256, I8, U8),
                 (3e38, 0, 1e-38, 0, I8, I8), (1e-38, 0, 3e38, 0, I8, I8), (1.0, 0, 1.0, 0, 3, I8)):
        assert oracle.requantize_linear(x, *args)[0] == reference.requantize_linear(x, *args)[0] == 0, args


def test_ptq_rules(oracle):
    x = np.array([0.0, -3.0, 1.27], np.float32)
    s = oracle.ptq_symmetric_scale(x)
    assert s.view(np.uint32) == np.float32(3.0 / 127.0).view(np.uint32)
    q = oracle.ptq_quantize_i8(x, s)
    assert q.tolist() == [0, -127, 54]
    st, b = oracle.ptq_pack_bias(np.array([0.25, -0.75], np.float32), 0.5, np.array([0.5, 0.25], np.float32))
    assert st == 0 and b.tolist() == [1, -6]


# ---- the real-valued bias of the per-token requantizing form (no reference counterpart) ------

def _rn32(q):
    """Round an exact rational to the nearest binary32 value, ties to even, by integer arithmetic
    alone (normal range only): the definition of one IEEE rounding, independent of the host FPU."""
    from fractions import Fraction
    q = Fraction(q)
    if q == 0:
        return Fraction(0)
    sign, mag = (-1 if q < 0 else 1), abs(q)
    e = 0
    while mag >= 2:
        mag /= 2; e += 1
    while mag < 1:
        mag *= 2; e -= 1
    assert -126 <= e <= 127
    scaled = mag * (1 << 23)              # in [2^23, 2^24)
    lo = scaled.numerator // scaled.denominator
    rem = scaled - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (lo & 1)):
        lo += 1
    return sign * Fraction(lo, 1 << 23) * Fraction(2) ** e


def _round_half_even(q):
    from fractions import Fraction
    lo = q.numerator // q.denominator
    rem = q - lo
    return lo + 1 if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (lo & 1)) else lo


def _bias_rule(acc, s_row, s_w, s_y, zp, bias, lo=-128, hi=127):
    """The extension's definition, in exact rationals with one explicit rounding per step:
    y = sat_rne( rn( rn( rn(rn(acc) * rn(rn(s_row*s_w)/s_y)) + zp ) + rn(bias/s_y) ) )."""
    from fractions import Fraction as Fr
    mult = _rn32(_rn32(Fr(s_row) * Fr(s_w)) / Fr(s_y))
    t1 = _rn32(_rn32(Fr(acc)) * mult)
    t2 = _rn32(t1 + zp)
    t = _rn32(t2 + _rn32(Fr(bias) / Fr(s_y)))
    return max(lo, min(hi, _round_half_even(t)))


def _one(oracle, x, w, s_row, s_w, s_y, zp, bias, out_dtype=I8):
    ok, y, acc = oracle.qlinear_rowscale(
        np.array([[x]], np.int8), np.array([[w]], np.int8), np.array([s_w], np.float32), np.zeros(1, np.int32),
        np.array([s_row], np.float32), s_y, zp, out_dtype=out_dtype, bias_f32=np.array([bias], np.float32))
    return ok, int(y[0, 0]), int(acc[0, 0])


def test_rowscale_f32_bias_order_and_roundings(oracle):
    """t = f32(f32(f32(acc)*mult) + zp), then t + f32(bias/s_y) as one more rounding, then the
    saturating ties-even round.  Inputs where a plausible other form gives another byte."""
    # (a) zero point first, then bias.  acc = 1, mult = 0.5 + 2^-24 (one ulp above a half), zp = 1,
    # bias = -1: 1.5 + 2^-24 is a tie between 1.5 and 1.5 + 2^-23 and goes to the even 1.5; minus 1
    # is the tie 0.5 -> 0.  Bias first (exact -0.5 + 2^-24, then + 1 = 0.5 + 2^-24 -> 1) and a single
    # rounding of the exact sum (0.5 + 2^-24 -> 1) both give 1.
    m = float.fromhex("0x1.000002p-1")
    assert _one(oracle, 1, 1, m, 1.0, 1.0, 1, -1.0) == (1, 0, 1)
    assert _bias_rule(1, m, 1.0, 1.0, 1, -1.0) == 0
    # (b) bias / s_y is a true division, rounded once.  s_y = 0.05f, bias = 0x1.a00002p+0: the
    # quotient lies within half an ulp (2^-19) of 32.5, so the term is the tie 32.5 -> 32; a product
    # with the rounded reciprocal of 0.05f lands one ulp above and would give 33.
    from fractions import Fraction as Fr
    s_y, bias = float(np.float32(0.05)), float.fromhex("0x1.a00002p+0")
    assert abs(Fr(bias) / Fr(s_y) - Fr(65, 2)) < Fr(1, 1 << 19)
    assert float(np.float32(np.float32(bias) * np.float32(np.float32(1.0) / np.float32(0.05)))) > 32.5
    assert _one(oracle, 0, 1, 1.0, 1.0, s_y, 0, bias) == (1, 32, 0)
    # (c) the bias is in real units, not in output units and not in accumulator units
    assert _one(oracle, 3, 1, 0.5, 0.5, 0.25, 0, 1.0) == (1, 7, 3)      # 3 * (0.25/0.25) + 1/0.25
    # (d) ties to even after the bias, both directions, and a negative tie
    assert _one(oracle, 2, 1, 1.0, 1.0, 1.0, 0, 0.5)[1] == 2            # 2.5 -> 2
    assert _one(oracle, 3, 1, 1.0, 1.0, 1.0, 0, 0.5)[1] == 4            # 3.5 -> 4
    assert _one(oracle, -2, 1, 1.0, 1.0, 1.0, 0, -0.5)[1] == -2         # -2.5 -> -2
    # (e) saturation is applied after the bias, in both byte domains
    assert _one(oracle, 120, 1, 1.0, 1.0, 1.0, 0, 10.0)[1] == 127
    assert _one(oracle, -120, 1, 1.0, 1.0, 1.0, 0, -300.0)[1] == -128
    assert _one(oracle, 100, 1, 1.0, 1.0, 1.0, 7, 200.0, out_dtype=U8)[1] == 255
    assert _one(oracle, -100, 1, 1.0, 1.0, 1.0, 7, 0.25, out_dtype=U8)[1] == 0
    # (f) a bias that is not finite is a bad descriptor: the whole call is declined
    for bad in (np.nan, np.inf, -np.inf):
        assert _one(oracle, 1, 1, 1.0, 1.0, 1.0, 0, bad)[0] == 0


def test_rowscale_f32_bias_against_exact_rationals(oracle):
    """Seeded small cases: every output byte equals the rule evaluated in exact rationals with
    explicit roundings (no host floating point on the checking side)."""
    rng = np.random.default_rng(314)
    rows, k, n = 5, 9, 6
    x = rng.integers(-127, 128, (rows, k)).astype(np.int8)
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    s_w = rng.uniform(0.002, 0.01, n).astype(np.float32)
    s_row = rng.uniform(0.01, 0.05, rows).astype(np.float32)
    bias = rng.normal(0, 0.4, n).astype(np.float32)
    for s_y, zp in ((np.float32(0.05), 0), (np.float32(0.0123), -3)):
        ok, y, acc = oracle.qlinear_rowscale(x, w, s_w, np.zeros(n, np.int32), s_row, s_y, zp, bias_f32=bias)
        assert ok == 1 and (acc == x.astype(np.int64) @ w.astype(np.int64).T).all()
        for r in range(rows):
            for c in range(n):
                assert int(y[r, c]) == _bias_rule(int(acc[r, c]), float(s_row[r]), float(s_w[c]), float(s_y), zp,
                                                  float(bias[c])), (r, c)
        assert len(np.unique(y)) > 8  # not all saturated


def test_blocked_packed_linear_equals_the_scalar_restatement(oracle):
    """The vectorised form used for full-size shapes gives the scalar restatement's bits (which the
    reference digests pin), ragged K and partial groups included, and a NaN scale marks its row."""
    from oracle.pyoracle import packed_linear_a8_blocked
    for entry in VECTORS["packed"][:6]:
        c = cases.packed_case(**entry["params"])
        a8, s, fin = oracle.packed_prepare(c["x"])
        s = np.where(fin == 1, s, np.nan).astype(np.float32)
        got, acc = packed_linear_a8_blocked(a8, s, c["w"], c["scales"], c["bias"], c["group"])
        _, want = oracle.packed_linear(c["x"], oracle.pack_w8_words(c["w"]), c["scales"], c["bias"], c["n"], c["group"])
        nan = np.isnan(want)
        assert (np.isnan(got) == nan).all() and (got.view(np.uint32)[~nan] == want.view(np.uint32)[~nan]).all()
        if not nan.any():
            check_digest(got, entry["expected"])
            assert (acc == a8.astype(np.int64) @ c["w"].astype(np.int64).T).all()
    rng = np.random.default_rng(6)
    for rows, k, n, g in [(3, 300, 17, 64), (2, 4096, 9, 128), (5, 95, 4, 32)]:
        a8 = rng.integers(-127, 128, (rows, k)).astype(np.int8)
        w = rng.integers(-128, 128, (n, k)).astype(np.int8)
        rs = rng.uniform(0.01, 0.05, rows).astype(np.float32)
        sc = rng.uniform(0.002, 0.01, (n, (k + g - 1) // g)).astype(np.float32)
        b = rng.normal(0, 0.1, n).astype(np.float32)
        got, _ = packed_linear_a8_blocked(a8, rs, w, sc, b, g)
        _, want, _ = oracle.packed_linear_a8(a8, rs, oracle.pack_w8_words(w), sc, b, n, g)
        assert (got.view(np.uint32) == want.view(np.uint32)).all()
