"""BASELINE config 4 glue: the decoder built on the W8A8 linears against its CPU restatement."""
import numpy as np
import pytest

from _decoder_ref import DecoderRef


def small_config():
    from volvoxai_amd.decoder import DecoderConfig
    return DecoderConfig(layers=2, hidden=256, q_heads=4, kv_heads=2, head_dim=64, inter=512, vocab=1000, group=128,
                         max_seq=32)


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


@pytest.mark.gpu
@pytest.mark.parametrize("use_graph", [False, True])
def test_decoder_tokens_agree_with_cpu_restatement(oracle, use_graph):
    import torch
    from volvoxai_amd.decoder import W8A8Decoder, init_weights, rope_tables
    cfg = small_config()
    weights = init_weights(cfg, 11)
    rows, prompt_len, new = 3, 5, 6
    prompt = np.random.default_rng(2).integers(0, cfg.vocab, (rows, prompt_len))
    want_tokens, want_logits = DecoderRef(cfg, weights, oracle, rope_tables).generate(prompt, new)

    dec = W8A8Decoder(cfg, weights, rows)
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
