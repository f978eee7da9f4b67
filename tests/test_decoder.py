"""Decoder glue: the decoder built on the W8A8 linears against its CPU restatement."""
import numpy as np
import pytest

from _decoder_ref import DecoderRef


def small_config():
    from volvoxai_amd.decoder import DecoderConfig
    return DecoderConfig(layers=2, hidden=256, q_heads=4, kv_heads=2, head_dim=64, inter=512, vocab=1000, group=128,
                         max_seq=32)


def test_w4_word_packing_matches_the_oracle(oracle):
    from volvoxai_amd.decoder import pack_w4_words
    rng = np.random.default_rng(0)
    for n, k in [(3, 75), (5, 64), (2, 1), (4, 1000)]:
        w = rng.integers(-8, 8, (n, k)).astype(np.int8)
        assert (pack_w4_words(w) == oracle.pack_w4_words(w)).all()


def test_word_packing_matches_the_oracle(oracle):
    from volvoxai_amd.decoder import pack_w8_words
    rng = np.random.default_rng(3)
    for n, k in ((5, 96), (3, 130), (1, 7)):
        w = rng.integers(-128, 128, (n, k)).astype(np.int8)
        assert (pack_w8_words(w) == oracle.pack_w8_words(w)).all()


def test_rope_tables_are_rotations():
    from volvoxai_amd.decoder import rope_tables
    cfg = small_config()
    cos, sin = rope_tables(cfg)
    assert cos.shape == (cfg.max_seq, cfg.head_dim)
    assert np.allclose(cos * cos + sin * sin, 1.0, atol=1e-6)
    assert (cos[0] == 1).all() and (sin[0] == 0).all()
    assert (cos[:, :cfg.head_dim // 2] == cos[:, cfg.head_dim // 2:]).all()


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,d", [(1, 64), (5, 1024), (33, 3000)])
def test_rmsnorm_prepare_kernel(ctx, oracle, rows, d):
    """Normalized rows against the double-precision definition; codes and scales must be exactly
    what the oracle's preparation makes of the kernel's own normalized rows."""
    import volvoxai_amd.w8a8 as vx
    rng = np.random.default_rng(d)
    x = (rng.normal(0, 3, (rows, d)) * rng.uniform(0.01, 100, (rows, 1))).astype(np.float32)
    if rows >= 5:
        x[1] = 0.0
        x[2, 3] = np.inf
    gain = rng.uniform(0.5, 1.5, d).astype(np.float32)
    a8, sc, normalized = vx.rmsnorm_prepare_i8(ctx, _dev(x), _dev(gain), 1e-6, want_normalized=True)
    ctx.synchronize()
    a8, sc, normalized = a8.cpu().numpy(), sc.cpu().numpy(), normalized.cpu().numpy()
    xd = x.astype(np.float64)
    with np.errstate(all="ignore"):
        want = (xd * (1.0 / np.sqrt((xd * xd).mean(-1, keepdims=True) + 1e-6)) * gain.astype(np.float64)).astype(np.float32)
    finite = np.isfinite(want).all(-1)
    assert np.allclose(normalized[finite], want[finite], rtol=3e-7, atol=0)
    want_codes, want_scales, fin = oracle.packed_prepare(normalized)
    good = fin == 1
    assert (np.isnan(sc) == ~good).all() and (good == finite).all() and not a8[~good].any()
    assert (a8[good] == want_codes[good]).all() and (sc[good].view(np.uint32) == want_scales[good].view(np.uint32)).all()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,inter", [(1, 32), (7, 3072), (32, 1000)])
def test_swiglu_prepare_kernel(ctx, oracle, rows, inter):
    import volvoxai_amd.w8a8 as vx
    rng = np.random.default_rng(inter)
    gu = rng.normal(0, 4, (rows, 2 * inter)).astype(np.float32)
    a8, sc, act = vx.swiglu_prepare_i8(ctx, _dev(gu), want_activated=True)
    ctx.synchronize()
    a8, sc, act = a8.cpu().numpy(), sc.cpu().numpy(), act.cpu().numpy()
    gate, up = gu[:, :inter].astype(np.float64), gu[:, inter:].astype(np.float64)
    want = gate / (1.0 + np.exp(-gate)) * up
    assert np.allclose(act, want, rtol=1e-6, atol=1e-30)
    want_codes, want_scales, fin = oracle.packed_prepare(act)
    assert fin.all() and (a8 == want_codes).all() and (sc.view(np.uint32) == want_scales.view(np.uint32)).all()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,t,start", [(2, 1, 7), (3, 5, 0)])
def test_rope_append_and_attention_kernels(ctx, rows, t, start):
    import torch
    import volvoxai_amd.w8a8 as vx
    from volvoxai_amd.decoder import DecoderConfig, rope_tables
    cfg = DecoderConfig(layers=1, hidden=64, q_heads=4, kv_heads=2, head_dim=32, inter=64, vocab=10, max_seq=16)
    rng = np.random.default_rng(rows * 10 + t)
    cos, sin = rope_tables(cfg)
    width = cfg.q_dim + 2 * cfg.kv_dim
    qkv = rng.normal(0, 1, (rows, t, width)).astype(np.float32)
    k_cache = rng.normal(0, 1, (rows, cfg.kv_heads, cfg.max_seq, cfg.head_dim)).astype(np.float32)
    v_cache = rng.normal(0, 1, (rows, cfg.kv_heads, cfg.max_seq, cfg.head_dim)).astype(np.float32)
    positions = np.arange(start, start + t, dtype=np.int64)
    kd, vd = _dev(k_cache), _dev(v_cache)
    q = vx.rope_append_kv(ctx, _dev(qkv), _dev(cos), _dev(sin), _dev(positions), cfg.q_heads, cfg.kv_heads,
                          cfg.head_dim, kd, vd)
    out = vx.gqa_attention(ctx, q, kd, vd, _dev(positions))
    ctx.synchronize()
    half = cfg.head_dim // 2

    def rope(x):  # [rows, t, heads, d]
        partner = np.concatenate([-x[..., half:], x[..., :half]], axis=-1)
        c, s = cos[positions][None, :, None, :], sin[positions][None, :, None, :]
        return (x * c + partner * s).astype(np.float32)

    wq = rope(qkv[..., :cfg.q_dim].reshape(rows, t, cfg.q_heads, cfg.head_dim))
    wk = rope(qkv[..., cfg.q_dim:cfg.q_dim + cfg.kv_dim].reshape(rows, t, cfg.kv_heads, cfg.head_dim))
    wv = qkv[..., cfg.q_dim + cfg.kv_dim:].reshape(rows, t, cfg.kv_heads, cfg.head_dim)
    k_cache[:, :, positions] = wk.transpose(0, 2, 1, 3)
    v_cache[:, :, positions] = wv.transpose(0, 2, 1, 3)
    assert (q.cpu().numpy() == wq).all()                 # two products and one sum: same bits
    assert (kd.cpu().numpy() == k_cache).all() and (vd.cpu().numpy() == v_cache).all()
    rep = cfg.q_heads // cfg.kv_heads
    want = np.zeros((rows, t, cfg.q_heads, cfg.head_dim))
    for h in range(cfg.q_heads):
        for i in range(t):
            vis = positions[i] + 1
            kk, vv = k_cache[:, h // rep, :vis].astype(np.float64), v_cache[:, h // rep, :vis].astype(np.float64)
            sc = np.einsum("bd,bsd->bs", wq[:, i, h].astype(np.float64), kk) / np.sqrt(cfg.head_dim)
            p = np.exp(sc - sc.max(-1, keepdims=True))
            p /= p.sum(-1, keepdims=True)
            want[:, i, h] = np.einsum("bs,bsd->bd", p, vv)
    assert np.allclose(out.cpu().numpy().reshape(want.shape), want, rtol=2e-5, atol=2e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,t,start,q_heads,kv_heads,head_dim,max_seq", [
    (2, 128, 0, 16, 8, 128, 256),   # the benchmark's prompt (head size 128: the matrix-pipe kernel)
    (1, 70, 5, 8, 2, 128, 200),     # the same kernel with ragged blocks, four query heads per KV head
    (3, 9, 0, 3, 1, 128, 64),       # and with query rows left empty (27 of 32 used)
    (1, 16, 0, 2, 2, 128, 9000),    # head size 128 with a cache too long for its 32 score rows
    (1, 40, 13, 8, 1, 64, 70),      # eight query heads per KV head, a prompt continued at slot 13
    (2, 9, 100, 4, 4, 256, 131),    # one head per KV head, the largest head size, an odd cache length
    (1, 200, 0, 2, 1, 32, 1000),    # a long cache: fewer tokens share a workgroup
    (3, 5, 2, 4, 2, 64, 32),        # too few tokens for the prompt kernel: the per-token one
])
def test_prompt_attention(ctx, rows, t, start, q_heads, kv_heads, head_dim, max_seq):
    """Causal grouped-query attention of t prompt tokens per row over the caches, against a float64
    statement of its definition (every token sees the slots up to its own)."""
    import volvoxai_amd.w8a8 as vx
    rng = np.random.default_rng(t * 7 + head_dim)
    q = rng.normal(0, 1, (rows, t, q_heads, head_dim)).astype(np.float32)
    k_cache = rng.normal(0, 1, (rows, kv_heads, max_seq, head_dim)).astype(np.float32)
    v_cache = rng.normal(0, 1, (rows, kv_heads, max_seq, head_dim)).astype(np.float32)
    positions = np.arange(start, start + t, dtype=np.int64)
    out = vx.gqa_attention(ctx, _dev(q), _dev(k_cache), _dev(v_cache), _dev(positions))
    ctx.synchronize()
    got = out.cpu().numpy().reshape(rows, t, q_heads, head_dim)
    rep = q_heads // kv_heads
    for h in range(q_heads):
        kk, vv = k_cache[:, h // rep].astype(np.float64), v_cache[:, h // rep].astype(np.float64)
        sc = np.einsum("btd,bsd->bts", q[:, :, h].astype(np.float64), kk) / np.sqrt(head_dim)
        sc[:, np.arange(max_seq)[None, :] > positions[:, None]] = -np.inf
        p = np.exp(sc - sc.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        want = np.einsum("bts,bsd->btd", p, vv)
        assert np.allclose(got[:, :, h], want, rtol=2e-5, atol=2e-6), h


@pytest.mark.gpu
@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("use_graph", [False, True])
def test_decoder_tokens_agree_with_cpu_restatement(oracle, use_graph, fused):
    import torch
    from volvoxai_amd.decoder import W8A8Decoder, init_weights, rope_tables
    cfg = small_config()
    weights = init_weights(cfg, 11)
    rows, prompt_len, new = 3, 5, 6
    prompt = np.random.default_rng(2).integers(0, cfg.vocab, (rows, prompt_len))
    want_tokens, want_logits = DecoderRef(cfg, weights, oracle, rope_tables).generate(prompt, new)

    from _decoder_torch import TorchGlueDecoder
    dec = (W8A8Decoder if fused else TorchGlueDecoder)(cfg, weights, rows)
    pd = torch.from_numpy(prompt).cuda()
    torch.cuda.synchronize()
    dec.prefill(pd)
    first_logits = dec.last_logits.cpu().numpy()
    if use_graph:
        dec.capture()
    got = dec.decode(new - 1).cpu().numpy()
    variant = dec.ctx.last_variant
    dec.close()
    # f32 glue sums in another order than numpy: logits agree to rounding noise, tokens exactly
    scale = np.abs(want_logits[0]).max()
    assert np.abs(first_logits - want_logits[0]).max() <= 2e-4 * scale
    assert (got == want_tokens).all(), (got, want_tokens)
    assert "a8-" in variant


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [1, 2])
@pytest.mark.parametrize("use_graph", [False, True])
def test_decode_of_one_or_two_rows_takes_the_fused_linears(oracle, rows, use_graph):
    """One row (two on request) decodes through the fused single-row linears (five launches per layer): the logits are
    bit for bit those of the nine-launch layer, the tokens those of the CPU restatement."""
    import torch
    from volvoxai_amd.decoder import DecoderConfig, W8A8Decoder, init_weights, rope_tables
    cfg = DecoderConfig(layers=2, hidden=1024, q_heads=8, kv_heads=4, head_dim=64, inter=1536, vocab=2000, group=128,
                        max_seq=32)
    weights = init_weights(cfg, 5)
    prompt_len, new = 4, 6
    prompt = np.random.default_rng(8).integers(0, cfg.vocab, (rows, prompt_len))
    want_tokens, _ = DecoderRef(cfg, weights, oracle, rope_tables).generate(prompt, new)
    pd = torch.from_numpy(prompt).cuda()
    results = []
    by_default = W8A8Decoder(cfg, weights, rows)
    assert by_default.rows_fused == (rows == 1)   # two rows run the fused forms no faster: on request only
    by_default.close()
    for fuse in (True, False):
        dec = W8A8Decoder(cfg, weights, rows, fuse_rows=fuse)
        assert dec.rows_fused == fuse
        torch.cuda.synchronize()
        dec.prefill(pd)
        if use_graph:
            dec.capture()
        got = dec.decode(new - 1).cpu().numpy()
        results.append((got, dec.last_logits.cpu().numpy(), dec.ctx.last_variant))
        dec.close()
    (fused_tokens, fused_logits, fused_route), (plain_tokens, plain_logits, _) = results
    assert (fused_tokens == want_tokens).all() and (plain_tokens == want_tokens).all()
    assert (fused_logits.view(np.uint32) == plain_logits.view(np.uint32)).all()
    assert "-rmsnorm" in fused_route or "a8-" in fused_route


@pytest.mark.gpu
def test_decoder_stages_at_benchmark_dimensions(oracle):
    """Two layers of the benchmark decoder at its own dimensions (hidden 1024, 16 query / 8 KV heads
    of 128, SwiGLU 3072, vocabulary 32000), 32 rows, 128-token prompts: every stage of the prompt
    pass, then of one decode step behind it (cache length 129, the fused decode attention, the
    32-row streaming linears) through the final norm, the lm_head and the argmax, each fed with the
    CPU restatement's own intermediate tensors.  With identical inputs the integer
    work is exact (codes, scales, linears: same bits) and the f32 glue is within rounding noise.
    The stages are chained through the restatement's tensors because the assembled pipeline is
    chaotic in the last bit: a 1e-6 difference after attention moves an activation across a
    rounding boundary of its int8 code now and then, and with random weights the softmax is so
    sharp that such a flip can select another key two stages later."""
    import torch
    import volvoxai_amd as vx
    from volvoxai_amd import w8a8
    from volvoxai_amd.decoder import DecoderConfig, init_weights, pack_w8_words, rope_tables
    cfg = DecoderConfig(layers=2)
    assert (cfg.hidden, cfg.q_heads, cfg.kv_heads, cfg.head_dim, cfg.inter, cfg.vocab) == (1024, 16, 8, 128, 3072, 32000)
    weights = init_weights(cfg, 5)
    rows, t = 32, 128
    prompt = np.random.default_rng(1).integers(0, cfg.vocab, (rows, t))
    ref = DecoderRef(cfg, weights, oracle, rope_tables, blocked=True)
    kc = [np.zeros((rows, cfg.kv_heads, 0, cfg.head_dim), np.float32) for _ in range(cfg.layers)]
    vc = [np.zeros((rows, cfg.kv_heads, 0, cfg.head_dim), np.float32) for _ in range(cfg.layers)]
    trace = []
    prompt_logits = ref.forward(prompt, 0, kc, vc, trace)
    rep = cfg.q_heads // cfg.kv_heads
    ctx = vx.Context(0, torch.cuda.current_stream())
    cos, sin = (_dev(a) for a in rope_tables(cfg))
    positions = torch.arange(t, dtype=torch.int64, device="cuda")
    bits = lambda a: np.ascontiguousarray(a).view(np.uint32)

    def linear(lin, a8, sc):
        pl = vx.PackedLinear(pack_w8_words(lin["w"]), lin["scales"], None, lin["w"].shape[1], lin["w"].shape[0], cfg.group)
        st, y = pl.forward_a8(ctx, a8, sc)
        ctx.synchronize()
        pl.close()
        assert st == 0
        return y.cpu().numpy()

    def codes_of(rows_f32):
        a8, s, fin = oracle.packed_prepare(np.ascontiguousarray(rows_f32, np.float32))
        assert fin.all()
        return a8, s

    for li, (L, tr) in enumerate(zip(weights["layers"], trace)):
        x_in = tr["x_in"].reshape(rows * t, cfg.hidden)
        # RMSNorm + preparation: the codes the restatement's pipeline feeds its QKV linear
        a8, sc = w8a8.rmsnorm_prepare_i8(ctx, _dev(x_in), _dev(L["norm1"]), cfg.eps)
        want_a8, want_s = codes_of(ref.rmsnorm(x_in, L["norm1"]))
        assert (a8.cpu().numpy() == want_a8).all() and (bits(sc.cpu().numpy()) == bits(want_s)).all(), li
        qkv = linear(L["qkv"], a8, sc)
        assert (bits(qkv) == bits(tr["qkv"].reshape(rows * t, -1))).all(), li
        # rotary embedding + cache append + prompt attention on the restatement's QKV
        kd = torch.zeros((rows, cfg.kv_heads, cfg.max_seq, cfg.head_dim), dtype=torch.float32, device="cuda")
        vd = torch.zeros_like(kd)
        q = w8a8.rope_append_kv(ctx, _dev(tr["qkv"]), cos, sin, positions, cfg.q_heads, cfg.kv_heads, cfg.head_dim, kd, vd)
        attn = w8a8.gqa_attention(ctx, q, kd, vd, positions)
        ctx.synchronize()
        assert (bits(kd[:, :, :t].cpu().numpy()) == bits(kc[li])).all() and (bits(vd[:, :, :t].cpu().numpy()) == bits(vc[li])).all()
        # against the definition in float64; with random weights the scores reach the thousands, so
        # f32 score rounding alone moves a probability by about eps * |score| (the restatement's own
        # f32 attention is no closer to the float64 value than the kernel is)
        got = attn.cpu().numpy().reshape(rows, t, cfg.q_heads, cfg.head_dim)
        q64, k64, v64 = q.cpu().numpy().astype(np.float64), kc[li].astype(np.float64), vc[li].astype(np.float64)
        truth, score_max = np.zeros(got.shape), 0.0
        for h in range(cfg.q_heads):
            sc64 = np.einsum("btd,bsd->bts", q64[:, :, h], k64[:, h // rep]) * float(np.float32(1.0 / np.sqrt(cfg.head_dim)))
            score_max = max(score_max, float(np.abs(sc64).max()))
            sc64[:, np.arange(t)[None, :] > np.arange(t)[:, None]] = -np.inf
            p64 = np.exp(sc64 - sc64.max(-1, keepdims=True))
            p64 /= p64.sum(-1, keepdims=True)
            truth[:, :, h] = np.einsum("bts,bsd->btd", p64, v64[:, h // rep])
        bound = 4.0 * 2.0 ** -24 * max(score_max, 16.0) * np.abs(truth).max()
        assert np.abs(got - truth).max() <= bound, (li, np.abs(got - truth).max(), bound)
        assert np.abs(tr["attn"].reshape(got.shape) - truth).max() <= bound  # the restatement, same yardstick
        # output projection of the restatement's attention rows: preparation inside the call
        plo = vx.PackedLinear(pack_w8_words(L["o"]["w"]), L["o"]["scales"], None, cfg.q_dim, cfg.hidden, cfg.group)
        st, o = plo.forward_f32(ctx, _dev(tr["attn"]))
        ctx.synchronize()
        plo.close()
        assert st == 0 and (bits(o.cpu().numpy()) == bits(tr["o"])).all(), li
        # residual add + RMSNorm + preparation, gate/up, SwiGLU + preparation, down
        resid = _dev(x_in)
        a8, sc = w8a8.add_rmsnorm_prepare_i8(ctx, resid, _dev(tr["o"]), _dev(L["norm2"]), cfg.eps)
        x_mid = tr["x_mid"].reshape(rows * t, cfg.hidden)
        assert (bits(resid.cpu().numpy()) == bits(x_mid)).all(), li
        want_a8, want_s = codes_of(ref.rmsnorm(x_mid, L["norm2"]))
        assert (a8.cpu().numpy() == want_a8).all() and (bits(sc.cpu().numpy()) == bits(want_s)).all(), li
        gu = linear(L["gate_up"], a8, sc)
        assert (bits(gu) == bits(tr["gu"])).all(), li
        a8, sc, act = w8a8.swiglu_prepare_i8(ctx, _dev(tr["gu"]), want_activated=True)
        ctx.synchronize()
        act = act.cpu().numpy()
        assert np.allclose(act, tr["act"], rtol=1e-6, atol=1e-30), li
        # the kernel's own activated rows fix its codes; against the restatement's rows a code may
        # differ by one where the two exponentials differ in the last bit
        own_a8, own_s = codes_of(act)
        assert (a8.cpu().numpy() == own_a8).all() and (bits(sc.cpu().numpy()) == bits(own_s)).all(), li
        ref_a8, ref_s = codes_of(tr["act"])
        off = a8.cpu().numpy().astype(np.int32) - ref_a8
        assert np.abs(off).max() <= 1 and (off != 0).mean() < 1e-3, li
        down = linear(L["down"], _dev(ref_a8), _dev(ref_s))
        assert (bits(down) == bits(tr["down"])).all(), li

    # ---- one decode step behind the prompt (cache length 129), stage by stage, through the head -----
    first = prompt_logits.argmax(-1)
    step = []
    step_logits = ref.forward(first[:, None], t, kc, vc, step)
    position = torch.full((1,), t, dtype=torch.int64, device="cuda")
    for li, (L, tr) in enumerate(zip(weights["layers"], step)):
        x_in = tr["x_in"].reshape(rows, cfg.hidden)
        a8, sc = w8a8.rmsnorm_prepare_i8(ctx, _dev(x_in), _dev(L["norm1"]), cfg.eps)
        want_a8, want_s = codes_of(ref.rmsnorm(x_in, L["norm1"]))
        assert (a8.cpu().numpy() == want_a8).all() and (bits(sc.cpu().numpy()) == bits(want_s)).all(), li
        qkv = linear(L["qkv"], a8, sc)   # 32 rows: the streaming kernel
        assert (bits(qkv) == bits(tr["qkv"].reshape(rows, -1))).all(), li
        # rotary embedding, append at slot 128 and attention over 129 slots in the one decode launch
        kd = torch.zeros((rows, cfg.kv_heads, cfg.max_seq, cfg.head_dim), dtype=torch.float32, device="cuda")
        vd = torch.zeros_like(kd)
        kd[:, :, :t] = _dev(kc[li][:, :, :t])
        vd[:, :, :t] = _dev(vc[li][:, :, :t])
        attn = w8a8.rope_gqa_attention_decode(ctx, _dev(tr["qkv"].reshape(rows, -1)), cos, sin, position, cfg.q_heads,
                                              cfg.kv_heads, cfg.head_dim, kd, vd)
        ctx.synchronize()
        assert (bits(kd[:, :, :t + 1].cpu().numpy()) == bits(kc[li])).all() and (bits(vd[:, :, :t + 1].cpu().numpy()) == bits(vc[li])).all()
        got = attn.cpu().numpy().reshape(rows, cfg.q_heads, cfg.head_dim)
        qr = ref.rope(tr["qkv"].reshape(rows, 1, -1)[..., :cfg.q_dim].reshape(rows, 1, cfg.q_heads, cfg.head_dim),
                      ref.cos[t:t + 1], ref.sin[t:t + 1])[:, 0].astype(np.float64)
        k64, v64 = kc[li].astype(np.float64), vc[li].astype(np.float64)
        truth, score_max = np.zeros(got.shape), 0.0
        for h in range(cfg.q_heads):
            sc64 = np.einsum("bd,bsd->bs", qr[:, h], k64[:, h // rep]) * float(np.float32(1.0 / np.sqrt(cfg.head_dim)))
            score_max = max(score_max, float(np.abs(sc64).max()))
            p64 = np.exp(sc64 - sc64.max(-1, keepdims=True))
            p64 /= p64.sum(-1, keepdims=True)
            truth[:, h] = np.einsum("bs,bsd->bd", p64, v64[:, h // rep])
        bound = 4.0 * 2.0 ** -24 * max(score_max, 16.0) * np.abs(truth).max()
        assert np.abs(got - truth).max() <= bound, (li, np.abs(got - truth).max(), bound)
        plo = vx.PackedLinear(pack_w8_words(L["o"]["w"]), L["o"]["scales"], None, cfg.q_dim, cfg.hidden, cfg.group)
        st, o = plo.forward_f32(ctx, _dev(tr["attn"]))
        ctx.synchronize()
        plo.close()
        assert st == 0 and (bits(o.cpu().numpy()) == bits(tr["o"])).all(), li
        resid = _dev(x_in)
        a8, sc = w8a8.add_rmsnorm_prepare_i8(ctx, resid, _dev(tr["o"]), _dev(L["norm2"]), cfg.eps)
        x_mid = tr["x_mid"].reshape(rows, cfg.hidden)
        assert (bits(resid.cpu().numpy()) == bits(x_mid)).all(), li
        want_a8, want_s = codes_of(ref.rmsnorm(x_mid, L["norm2"]))
        assert (a8.cpu().numpy() == want_a8).all() and (bits(sc.cpu().numpy()) == bits(want_s)).all(), li
        gu = linear(L["gate_up"], a8, sc)
        assert (bits(gu) == bits(tr["gu"])).all(), li
        a8, sc, act = w8a8.swiglu_prepare_i8(ctx, _dev(tr["gu"]), want_activated=True)
        ctx.synchronize()
        assert np.allclose(act.cpu().numpy(), tr["act"], rtol=1e-6, atol=1e-30), li
        ref_a8, ref_s = codes_of(tr["act"])
        down = linear(L["down"], _dev(ref_a8), _dev(ref_s))
        assert (bits(down) == bits(tr["down"])).all(), li
    # the head: last residual add + final RMSNorm + preparation, lm_head (32 rows x 32000 channels), argmax
    last = step[-1]
    resid = _dev(last["x_mid"].reshape(rows, cfg.hidden))
    a8, sc = w8a8.add_rmsnorm_prepare_i8(ctx, resid, _dev(last["down"]), _dev(weights["norm_f"]), cfg.eps)
    x_out = last["x_mid"].reshape(rows, cfg.hidden) + last["down"]
    assert (bits(resid.cpu().numpy()) == bits(x_out)).all()
    want_a8, want_s = codes_of(ref.rmsnorm(x_out, weights["norm_f"]))
    assert (a8.cpu().numpy() == want_a8).all() and (bits(sc.cpu().numpy()) == bits(want_s)).all()
    logits = linear(weights["lm_head"], a8, sc)
    assert (bits(logits) == bits(step_logits)).all()
    ids = w8a8.argmax_rows(ctx, _dev(step_logits))
    ctx.synchronize()
    assert (ids.cpu().numpy() == step_logits.argmax(-1)).all()
    ctx.close()


@pytest.mark.gpu
def test_decoder_at_benchmark_dimensions_end_to_end(oracle):
    """The assembled decoder at the benchmark's dimensions (two layers, 32 rows, 128-token prompts):
    the HIP graph replays what the eager loop computes, token for token, and the first tokens and
    logits agree with the CPU restatement wherever the pipeline did not cross a rounding boundary
    on the way (see the stage test above for why some rows do): most rows to rounding noise, every
    row's logits to a few per cent."""
    import torch
    from volvoxai_amd.decoder import DecoderConfig, W8A8Decoder, init_weights, rope_tables
    cfg = DecoderConfig(layers=2)
    weights = init_weights(cfg, 5)
    rows, prompt_len, new = 32, 128, 4
    prompt = np.random.default_rng(1).integers(0, cfg.vocab, (rows, prompt_len))
    want_tokens, want_logits = DecoderRef(cfg, weights, oracle, rope_tables, blocked=True).generate(prompt, 1)
    dec = W8A8Decoder(cfg, weights, rows)
    pd = torch.from_numpy(prompt).cuda()
    dec.prefill(pd)
    first_logits = dec.last_logits.cpu().numpy()
    eager = dec.decode(new - 1).cpu().numpy()
    dec.prefill(pd)
    dec.capture()
    replayed = dec.decode(new - 1).cpu().numpy()
    variant = dec.ctx.last_variant
    dec.close()
    assert (eager == replayed).all() and "a8-" in variant
    scale = np.abs(want_logits[0]).max()
    row_err = np.abs(first_logits - want_logits[0]).max(axis=1)
    err = row_err / scale
    assert err.max() < 0.1 and (err < 2e-4).mean() >= 0.5, np.sort(err)
    # Row by row: the token is the restatement's, or the restatement's own logits put the chosen token
    # within twice this row's measured logit error of its maximum -- a flip that the row's rounding
    # noise explains.  Anything else is a real disagreement.
    for r in range(rows):
        if eager[0][r] != want_tokens[0][r]:
            gap = want_logits[0][r].max() - want_logits[0][r][eager[0][r]]
            assert gap <= 2.0 * row_err[r], (r, int(eager[0][r]), int(want_tokens[0][r]), float(gap), float(row_err[r]))
    # rows whose logits agree to rounding noise must agree on the token unless the top two are that close
    quiet = err < 2e-4
    flips = quiet & (eager[0] != want_tokens[0])
    assert flips.sum() <= 1, np.nonzero(flips)


@pytest.mark.gpu
def test_longer_prompt_after_capture_keeps_the_graph_valid(oracle):
    """A HIP graph of a decode step holds the addresses of the context's scratch.  A later prefill
    with a longer prompt outgrows that scratch; the library keeps the old block alive, so replaying
    the graph afterwards gives exactly the tokens of an eager run."""
    import torch
    from volvoxai_amd.decoder import W8A8Decoder, init_weights
    from volvoxai_amd.decoder import DecoderConfig
    cfg = DecoderConfig(layers=2, hidden=256, q_heads=4, kv_heads=2, head_dim=64, inter=512, vocab=1000, group=128,
                        max_seq=2100)
    weights = init_weights(cfg, 3)
    rows = 3
    rng = np.random.default_rng(9)
    short, long = rng.integers(0, cfg.vocab, (rows, 2)), rng.integers(0, cfg.vocab, (rows, 2048))
    dec = W8A8Decoder(cfg, weights, rows)
    dec.prefill(torch.from_numpy(short).cuda())
    dec.capture()                                   # scratch sized for 3 x 2 tokens (1 MiB) is baked into the graph
    dec.prefill(torch.from_numpy(long).cuda())      # 3 x 2048 prepared rows of 256 bytes: the scratch grows
    replayed = dec.decode(5).cpu().numpy()
    dec.graph = None
    dec.prefill(torch.from_numpy(long).cuda())
    eager = dec.decode(5).cpu().numpy()
    dec.close()
    assert (replayed == eager).all()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,start,q_heads,kv_heads,head_dim", [(3, 0, 4, 2, 64), (2, 7, 16, 8, 128), (5, 255, 4, 4, 32),
                                                                   (2, 300, 8, 1, 64)])
def test_fused_decode_attention_equals_the_two_kernels(ctx, rows, start, q_heads, kv_heads, head_dim):
    """One launch (rotary + cache append + attention) against rope_append_kv followed by gqa_attention
    on the same inputs: the same output bits and the same caches, at the first slot, in the middle,
    past 256 slots (a thread then owns two slots) and for a group of eight query heads."""
    import torch
    from volvoxai_amd import w8a8
    rng = np.random.default_rng(rows + start)
    max_seq = 384
    width = (q_heads + 2 * kv_heads) * head_dim
    qkv = torch.from_numpy(rng.normal(0, 1, (rows, 1, width)).astype(np.float32)).cuda()
    angle = rng.uniform(0, 6.28, (max_seq, head_dim)).astype(np.float32)
    cos, sin = torch.from_numpy(np.cos(angle)).cuda(), torch.from_numpy(np.sin(angle)).cuda()
    cache = rng.normal(0, 1, (2, rows, kv_heads, max_seq, head_dim)).astype(np.float32)
    k1, v1 = torch.from_numpy(cache[0]).cuda(), torch.from_numpy(cache[1]).cuda()
    k2, v2 = k1.clone(), v1.clone()
    pos = torch.tensor([start], dtype=torch.int64, device="cuda")
    q = w8a8.rope_append_kv(ctx, qkv, cos, sin, pos, q_heads, kv_heads, head_dim, k1, v1)
    want = w8a8.gqa_attention(ctx, q, k1, v1, pos).reshape(rows, -1)
    got = w8a8.rope_gqa_attention_decode(ctx, qkv.reshape(rows, -1), cos, sin, pos, q_heads, kv_heads, head_dim, k2, v2)
    ctx.synchronize()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    assert torch.equal(k1, k2) and torch.equal(v1, v2)


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [1, 2])
@pytest.mark.parametrize("op,k,n,group,bits,add", [
    ("rmsnorm", 1024, 4096, 128, 8, False),    # the decoder's q/k/v and gate/up shapes
    ("rmsnorm", 1024, 6144, 128, 8, False),
    ("rmsnorm", 4096, 1056, 64, 8, True),
    ("rmsnorm", 2048, 512, 32, 4, False),
    ("rmsnorm", 1100, 200, 256, 8, False),     # ragged k and n
    ("swiglu", 3072, 1024, 128, 8, True),      # the decoder's down projection
    ("swiglu", 1000, 300, 64, 4, True),
    ("swiglu", 4096, 4096, 128, 8, False),
    ("none", 2048, 1024, 128, 8, True),        # the decoder's output projection
    ("none", 520, 96, 32, 8, True),
])
def test_fused_decode_linears_equal_the_separate_launches(ctx, oracle, rows, op, k, n, group, bits, add):
    """[RMSNorm | SwiGLU] -> preparation -> PackedLinear [-> residual add] as one launch
    (vxhip_packed_linear_forward_fused) gives the bits of the row kernel, the linear and the add run one
    after the other."""
    import torch
    import volvoxai_amd as vxa
    import volvoxai_amd.w8a8 as vx
    rng = np.random.default_rng(k * 7 + n + rows)
    w = rng.integers(-8, 8, (n, k)).astype(np.int8) if bits == 4 else rng.integers(-128, 128, (n, k)).astype(np.int8)
    words = oracle.pack_w4_words(w) if bits == 4 else oracle.pack_w8_words(w)
    groups = (k + group - 1) // group
    scales = rng.uniform(0.002, 0.01, (n, groups)).astype(np.float32)
    bias = rng.normal(0, 0.1, n).astype(np.float32)
    pl = vxa.PackedLinear(words, scales, bias, k, n, group, weight_bits=bits)
    try:
        width = 2 * k if op == "swiglu" else k
        x = _dev((rng.normal(0, 2, (rows, width)) * rng.uniform(0.1, 30, (rows, 1))).astype(np.float32))
        gain = _dev(rng.uniform(0.5, 1.5, k).astype(np.float32))
        resid = _dev(rng.normal(0, 1, (rows, n)).astype(np.float32))
        if op == "rmsnorm":
            a8, sc = vx.rmsnorm_prepare_i8(ctx, x.clone(), gain, 1e-6)
        elif op == "swiglu":
            a8, sc = vx.swiglu_prepare_i8(ctx, x)
        else:
            a8, sc = None, None
        if a8 is None:
            st, want = pl.forward_f32(ctx, x)
        else:
            st, want = pl.forward_a8(ctx, a8, sc)
        assert st == 0
        if add:
            want = resid + want
        code = {"none": vxa.ROW_OP_NONE, "rmsnorm": vxa.ROW_OP_RMSNORM, "swiglu": vxa.ROW_OP_SWIGLU}[op]
        out = resid.clone() if add else None
        handled, got = pl.forward_fused(ctx, x, code, gain=gain, eps=1e-6, add_to=out, out=out)   # in place when adding
        ctx.synchronize()
        assert handled == 1, vx.library().vxhip_last_error()
        route = ctx.last_variant
        assert "-prep" in route and (op == "none" or f"-{op}" in route) and route.endswith("-add") == add
        assert (got.cpu().numpy().view(np.uint32) == want.cpu().numpy().view(np.uint32)).all(), route
        if add:  # and into a buffer of its own
            handled, apart = pl.forward_fused(ctx, x, code, gain=gain, eps=1e-6, add_to=resid)
            ctx.synchronize()
            assert handled == 1 and (apart.cpu().numpy().view(np.uint32) == want.cpu().numpy().view(np.uint32)).all()
        # a row that is not finite: NaN outputs from both
        x2 = x.clone()
        x2[0, 5] = float("inf")
        if op == "rmsnorm":
            a8, sc = vx.rmsnorm_prepare_i8(ctx, x2.clone(), gain, 1e-6)
            _, want2 = pl.forward_a8(ctx, a8, sc)
        elif op == "swiglu":
            a8, sc = vx.swiglu_prepare_i8(ctx, x2)
            _, want2 = pl.forward_a8(ctx, a8, sc)
        else:
            _, want2 = pl.forward_f32(ctx, x2)
        handled, got2 = pl.forward_fused(ctx, x2, code, gain=gain, eps=1e-6)
        ctx.synchronize()
        g2, w2 = got2.cpu().numpy(), want2.cpu().numpy()
        assert handled == 1 and (np.isnan(g2) == np.isnan(w2)).all() and np.isnan(g2[0]).all()
        assert (g2[~np.isnan(g2)].view(np.uint32) == w2[~np.isnan(w2)].view(np.uint32)).all()
    finally:
        pl.close()


@pytest.mark.gpu
def test_fused_decode_linears_random_shapes(ctx, oracle):
    """Sixty random shapes (ragged k and n, every group size, 8- and 4-bit weights, one and two rows, with and
    without bias and residual) through the fused forms and through the separate launches: the same bits."""
    import volvoxai_amd as vxa
    import volvoxai_amd.w8a8 as vx
    rng = np.random.default_rng(20240)
    for case in range(60):
        op = ("none", "rmsnorm", "swiglu")[case % 3]
        rows, group, bits = int(rng.integers(1, 3)), int(rng.choice([32, 64, 128, 256])), int(rng.choice([8, 8, 4]))
        k = int(rng.integers(1024, 4097)) if op == "rmsnorm" else int(rng.integers(16, 8193))
        n, add = int(rng.integers(1, 2500)), bool(rng.integers(0, 2))
        w = rng.integers(-8, 8, (n, k)).astype(np.int8) if bits == 4 else rng.integers(-128, 128, (n, k)).astype(np.int8)
        words = oracle.pack_w4_words(w) if bits == 4 else oracle.pack_w8_words(w)
        scales = rng.uniform(0.002, 0.01, (n, (k + group - 1) // group)).astype(np.float32)
        bias = rng.normal(0, 0.1, n).astype(np.float32) if rng.integers(0, 2) else None
        pl = vxa.PackedLinear(words, scales, bias, k, n, group, weight_bits=bits)
        x = _dev((rng.normal(0, 2, (rows, 2 * k if op == "swiglu" else k)) * rng.uniform(0.01, 50, (rows, 1))).astype(np.float32))
        gain = _dev(rng.uniform(0.5, 1.5, k).astype(np.float32))
        resid = _dev(rng.normal(0, 1, (rows, n)).astype(np.float32))
        if op == "rmsnorm":
            a8, sc = vx.rmsnorm_prepare_i8(ctx, x.clone(), gain, 1e-5)
            st, want = pl.forward_a8(ctx, a8, sc)
        elif op == "swiglu":
            a8, sc = vx.swiglu_prepare_i8(ctx, x)
            st, want = pl.forward_a8(ctx, a8, sc)
        else:
            st, want = pl.forward_f32(ctx, x)
        assert st == 0
        if add:
            want = resid + want
        out = resid.clone() if add else None
        handled, got = pl.forward_fused(ctx, x, {"none": vxa.ROW_OP_NONE, "rmsnorm": vxa.ROW_OP_RMSNORM, "swiglu": vxa.ROW_OP_SWIGLU}[op],
                                        gain=gain, eps=1e-5, add_to=out, out=out)
        ctx.synchronize()
        assert handled == 1, (op, rows, k, n, group, bits)
        assert (got.cpu().numpy().view(np.uint32) == want.cpu().numpy().view(np.uint32)).all(), (op, rows, k, n, group, bits, add,
                                                                                                  ctx.last_variant)
        pl.close()
    assert ctx.fault_flags() == 0


@pytest.mark.gpu
def test_fused_decode_linear_declines_what_it_does_not_take(ctx, oracle):
    import volvoxai_amd as vxa
    rng = np.random.default_rng(1)
    k, n = 512, 64
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    pl = vxa.PackedLinear(oracle.pack_w8_words(w), rng.uniform(0.002, 0.01, (n, k // 128)).astype(np.float32), None, k, n, 128)
    try:
        gain = _dev(np.ones(k, np.float32))
        out = _dev(np.full((3, n), 7.0, np.float32))
        handled, _ = pl.forward_fused(ctx, _dev(np.ones((3, k), np.float32)), vxa.ROW_OP_NONE, out=out)   # three rows
        assert handled == 0
        handled, _ = pl.forward_fused(ctx, _dev(np.ones((1, k), np.float32)), vxa.ROW_OP_RMSNORM, gain=gain, eps=1e-6,
                                      out=out[:1])                                                       # k < 1024
        ctx.synchronize()
        assert handled == 0 and (out.cpu().numpy() == 7.0).all()
        with pytest.raises(ValueError):
            pl.forward_fused(ctx, _dev(np.ones((1, k), np.float32)), vxa.ROW_OP_SWIGLU)                  # needs [gate | up]
        with pytest.raises(ValueError):
            pl.forward_fused(ctx, _dev(np.ones((1, k), np.float32)), vxa.ROW_OP_RMSNORM)                 # no gain
    finally:
        pl.close()


@pytest.mark.gpu
def test_a_position_outside_the_cache_is_refused_on_the_device():
    """A cache slot at or past max_seq reaches the kernels only as a value in device memory: they
    leave the caches and that token's output alone and raise fault bit 4."""
    import torch
    import volvoxai_amd as vx
    from volvoxai_amd import w8a8
    own = vx.Context(0, None)  # fault bits are sticky: not the shared context
    rng = np.random.default_rng(5)
    rows, q_heads, kv_heads, head_dim, max_seq = 2, 4, 2, 64, 48
    width = (q_heads + 2 * kv_heads) * head_dim
    angle = rng.uniform(0, 6.28, (max_seq, head_dim)).astype(np.float32)
    cos, sin = torch.from_numpy(np.cos(angle)).cuda(), torch.from_numpy(np.sin(angle)).cuda()
    cache = rng.normal(0, 1, (2, rows, kv_heads, max_seq, head_dim)).astype(np.float32)
    k, v = torch.from_numpy(cache[0]).cuda(), torch.from_numpy(cache[1]).cuda()
    k0, v0 = k.clone(), v.clone()
    qkv = torch.from_numpy(rng.normal(0, 1, (rows, width)).astype(np.float32)).cuda()
    bad = torch.tensor([max_seq], dtype=torch.int64, device="cuda")
    w8a8.rope_gqa_attention_decode(own, qkv, cos, sin, bad, q_heads, kv_heads, head_dim, k, v)
    assert own.fault_flags() == 4 and torch.equal(k, k0) and torch.equal(v, v0)
    w8a8.rope_append_kv(own, qkv.reshape(rows, 1, width), cos, sin, bad, q_heads, kv_heads, head_dim, k, v)
    # a prompt whose last tokens run past the cache: the tokens inside are attended as usual
    t = 12
    positions = torch.arange(max_seq - 8, max_seq - 8 + t, dtype=torch.int64, device="cuda")
    q = torch.from_numpy(rng.normal(0, 1, (rows, t, q_heads, head_dim)).astype(np.float32)).cuda()
    out = w8a8.gqa_attention(own, q, k, v, positions)
    inside = w8a8.gqa_attention(own, q[:, :8].contiguous(), k, v, positions[:8])
    own.synchronize()
    assert own.fault_flags() == 4 and torch.equal(k, k0) and torch.equal(v, v0)
    assert torch.allclose(out[:, :8], inside, rtol=2e-5, atol=2e-6)
    own.close()


@pytest.mark.gpu
def test_embedding_gather_and_argmax_kernels(ctx, oracle):
    import torch
    from volvoxai_amd import w8a8
    from test_oracle import glue_argmax_rows
    rng = np.random.default_rng(4)
    for rows, n in [(12, 37), (32, 32000), (5, 4096), (3, 1023), (2, 1)]:
        x = glue_argmax_rows() if n == 37 else rng.normal(0, 1, (rows, n)).astype(np.float32)
        if n == 32000:
            x[4, 31999] = x[4, 17] = 40.0      # tie across threads and waves -> first
            x[5, 0] = np.nan
        counters = torch.tensor([7, 100], dtype=torch.int64, device="cuda")
        got = w8a8.argmax_rows(ctx, torch.from_numpy(x).cuda(), advance=counters)
        ctx.synchronize()
        assert (got.cpu().numpy() == oracle.argmax_rows(x)).all(), (rows, n)
        assert counters.tolist() == [8, 101]
    for d in (24, 1024, 7):
        table = rng.normal(0, 1, (50, d)).astype(np.float32)
        tokens = np.array([[0, 49], [7, 7], [13, 2]], np.int32)
        out = w8a8.embedding_gather(ctx, torch.from_numpy(tokens).cuda(), torch.from_numpy(table).cuda())
        ctx.synchronize()
        assert (out.cpu().numpy() == oracle.embedding(tokens.reshape(-1), table)).all()
    assert ctx.fault_flags() == 0
    # ids outside the table: zero rows and a sticky fault bit (on a context of its own)
    import volvoxai_amd as vx
    own = vx.Context(0, torch.cuda.current_stream())
    bad = w8a8.embedding_gather(own, torch.tensor([3, 50, -1], dtype=torch.int32, device="cuda"),
                                torch.from_numpy(table).cuda())
    own.synchronize()
    bad = bad.cpu().numpy()
    assert (bad[0] == table[3]).all() and not bad[1:].any() and own.fault_flags() & 2
    own.close()
