"""The decoder glue pinned to the reference's own C functions: rmsnorm_f32
(native/src/kernels/softmax_rmsnorm.inc:3-17), silu_f32 and mul_f32 (native/src/kernels/elementwise_f32.inc:153),
the RotaryEmbedding operator (native/src/kernels/llm_math.h:256-274) and cross_sdpa_gqa_f32
(native/src/kernels/cross_sdpa.inc:53).  tests/golden/reference_vectors.json ("glue") holds their outputs on
the seeded inputs of tests/_glue_defs.py.  Here: the numpy statements the other tests use as their yardstick
against those vectors (RMSNorm and the rotary embedding bit for bit), the live reference build against the
vectors, and the HIP kernels against the vectors."""
import json
from pathlib import Path

import numpy as np
import pytest

import _glue_defs as glue
from test_oracle import check_digest

VECTORS = json.loads((Path(__file__).parent / "golden" / "reference_vectors.json").read_text())["glue"]


def from_bits(bits, shape):
    return np.array(bits, dtype=np.uint32).view(np.float32).reshape(shape)


# the reference's SiLU runs on its own f32 exponential, its attention is an online softmax in f32: what a
# double-precision statement of the definition, or another f32 order, may differ by
SILU_RTOL, ATTENTION_ATOL = 4e-6, 4e-6


def close_silu(got, want):
    return bool((np.abs(got.astype(np.float64) - want) <= SILU_RTOL * np.abs(want) + 1e-37).all())


@pytest.mark.parametrize("entry", VECTORS["rmsnorm"], ids=lambda e: "x".join(str(v) for v in e["params"].values()))
def test_rmsnorm_definition_is_the_references(entry):
    x, gain = glue.rmsnorm_case(**entry["params"])
    check_digest(glue.rmsnorm(x, gain, entry["eps"]), entry["expected"])


def test_rotary_definition_is_the_references():
    x, cos, sin = glue.rotary_case()
    check_digest(glue.rotary(x, cos, sin), VECTORS["rotary"]["expected"])
    # a dropped sign or a swapped half gives other bits
    half = x.shape[-1] // 2
    wrong = (x * cos[:, None, :] + np.concatenate([x[..., half:], x[..., :half]], -1) * sin[:, None, :]).astype(np.float32)
    assert (wrong != glue.rotary(x, cos, sin)).any()


def test_silu_mul_and_attention_definitions_agree_with_the_reference():
    gu = glue.silu_mul_case()
    half = gu.shape[1] // 2
    want = from_bits(VECTORS["silu_mul"]["expected_bits"], VECTORS["silu_mul"]["shape"])
    assert close_silu(want, glue.silu_mul(gu[:, :half], gu[:, half:]))
    for entry in VECTORS["attention"]:
        p = entry["params"]
        q, k, v = glue.attention_case(**p)
        want = from_bits(entry["expected_bits"], entry["shape"])
        got = glue.attention(q, k, v, p["q_heads"], p["kv_heads"], p["head_dim"], p["causal"])
        assert np.abs(got - want).max() <= ATTENTION_ATOL, p
        # causality matters: the same call without it is elsewhere
        if p["causal"] and p["tq"] > 1:
            assert np.abs(glue.attention(q, k, v, p["q_heads"], p["kv_heads"], p["head_dim"], 0) - want).max() > 1e-3


def test_live_reference_glue(reference):
    for entry in VECTORS["rmsnorm"]:
        x, gain = glue.rmsnorm_case(**entry["params"])
        check_digest(reference.rmsnorm(x, gain, entry["eps"]), entry["expected"])
    x, cos, sin = glue.rotary_case()
    st, y = reference.rotary(x, cos, sin)
    assert st == 0
    check_digest(y, VECTORS["rotary"]["expected"])
    gu = glue.silu_mul_case()
    half = gu.shape[1] // 2
    assert [int(v) for v in reference.silu_mul(gu[:, :half], gu[:, half:]).reshape(-1).view(np.uint32)] == \
        VECTORS["silu_mul"]["expected_bits"]
    for entry in VECTORS["attention"]:
        p = entry["params"]
        q, k, v = glue.attention_case(**p)
        y = reference.attention(q, k, v, p["q_heads"], p["kv_heads"], p["head_dim"], p["causal"])
        assert [int(b) for b in y.reshape(-1).view(np.uint32)] == entry["expected_bits"]


# ---- the HIP kernels against the same vectors -----------------------------------------------------

def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.gpu
def test_rmsnorm_kernel_against_the_reference_vectors(ctx):
    """The kernel sums the squares as a tree over its threads, the reference in index order: both in
    double, so the sums differ by a few units of 2^-53 and the f32 result can differ only where the exact
    value lies that close to a rounding boundary -- about one element in 10^7.  Counted here over 140,000
    elements: none may differ by more than one unit in the last place, and at most two at all."""
    import volvoxai_amd.w8a8 as vx
    differing = total = 0
    for entry in VECTORS["rmsnorm"]:
        x, gain = glue.rmsnorm_case(**entry["params"])
        want = glue.rmsnorm(x, gain, entry["eps"])  # == the reference's bits (test above)
        _, _, normalized = vx.rmsnorm_prepare_i8(ctx, _dev(x), _dev(gain), entry["eps"], want_normalized=True)
        ctx.synchronize()
        got = normalized.cpu().numpy()
        off = got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64)
        assert np.abs(off).max() <= 1, entry["params"]
        differing += int((off != 0).sum())
        total += off.size
    print(f"RMSNorm: {differing} of {total} outputs differ from rmsnorm_f32 in the last bit")
    assert differing <= 2


@pytest.mark.gpu
def test_rotary_and_attention_kernels_against_the_reference_vectors(ctx):
    """rope_append_kernel on the rotary case: the rotated rows are the RotaryEmbedding operator's bits.
    gqa_attention / the fused decode kernel on the attention cases: within the f32 noise of two different
    summation orders of cross_sdpa_gqa_f32's result."""
    import torch
    import volvoxai_amd.w8a8 as vx
    from volvoxai_amd.decoder import DecoderConfig, rope_tables
    # rotary: 2 rows x 3 tokens at slots 7..9; the q part of a qkv row carries the case's four heads
    x, cos_t, sin_t = glue.rotary_case()
    cfg = DecoderConfig(layers=1, hidden=64, q_heads=4, kv_heads=2, head_dim=32, inter=64, vocab=10, max_seq=16)
    cos, sin = rope_tables(cfg)
    qkv = np.zeros((2, 3, cfg.q_dim + 2 * cfg.kv_dim), np.float32)
    qkv[..., :cfg.q_dim] = x.reshape(2, 3, cfg.q_dim)
    kd = torch.zeros((2, cfg.kv_heads, cfg.max_seq, cfg.head_dim), dtype=torch.float32, device="cuda")
    vd = torch.zeros_like(kd)
    q = vx.rope_append_kv(ctx, _dev(qkv), _dev(cos), _dev(sin), _dev(np.arange(7, 10, dtype=np.int64)), cfg.q_heads,
                          cfg.kv_heads, cfg.head_dim, kd, vd)
    ctx.synchronize()
    check_digest(q.cpu().numpy().reshape(6, 4, 32), VECTORS["rotary"]["expected"])
    # attention: one sequence (row), keys and values placed in the cache, queries as already rotated rows
    for entry in VECTORS["attention"]:
        p = entry["params"]
        qh, kvh, d, tq, tk = p["q_heads"], p["kv_heads"], p["head_dim"], p["tq"], p["tk"]
        qa, ka, va = glue.attention_case(**p)
        want = from_bits(entry["expected_bits"], entry["shape"])
        max_seq = tk + 3
        kc = np.zeros((1, kvh, max_seq, d), np.float32)
        vc = np.zeros_like(kc)
        kc[0, :, :tk] = ka.reshape(tk, kvh, d).transpose(1, 0, 2)
        vc[0, :, :tk] = va.reshape(tk, kvh, d).transpose(1, 0, 2)
        # query i sees slots 0..positions[i]: the prompt's causal rule, or everything for the one decode row
        positions = np.arange(tq, dtype=np.int64) if p["causal"] else np.full(tq, tk - 1, np.int64)
        out = vx.gqa_attention(ctx, _dev(qa.reshape(1, tq, qh, d)), _dev(kc), _dev(vc), _dev(positions))
        ctx.synchronize()
        assert np.abs(out.cpu().numpy().reshape(tq, qh * d) - want).max() <= ATTENTION_ATOL, p


@pytest.mark.gpu
def test_swiglu_kernel_against_the_reference_vectors(ctx):
    import volvoxai_amd.w8a8 as vx
    gu = glue.silu_mul_case()
    want = from_bits(VECTORS["silu_mul"]["expected_bits"], VECTORS["silu_mul"]["shape"])
    _, _, act = vx.swiglu_prepare_i8(ctx, _dev(gu), want_activated=True)
    ctx.synchronize()
    assert close_silu(act.cpu().numpy(), want.astype(np.float64))
