"""The decoder glue's definitions, stated in numpy in the reference's own operation order, and the seeded
inputs they are pinned on.  tests/golden/reference_vectors.json ("glue") holds what the reference's C
functions give on these inputs; the GPU tests compare the kernels with the same vectors."""
import numpy as np


def rmsnorm(x, gain, eps):
    """rmsnorm_f32 (src/kernels/softmax_rmsnorm.inc:3-17): the squares summed in double in index order,
    inv_std = 1 / sqrt(sum / d + eps), output = f32((x * inv_std) * gain) in double."""
    xd = x.astype(np.float64)
    with np.errstate(all="ignore"):
        var = np.cumsum(xd * xd, axis=-1)[:, -1:] / x.shape[1]   # cumsum adds in index order, as the loop does
        inv_std = 1.0 / np.sqrt(var + eps)
        return ((xd * inv_std) * gain.astype(np.float64)).astype(np.float32)


def silu_mul(gate, up):
    """SiLU then Mul (src/kernels/elementwise_f32.inc:153-165): f32(x * f32(1 / (1 + exp(-x)))) * up, here
    in double (the reference's exponential is its own f32 routine: compared under a tolerance)."""
    g = gate.astype(np.float64)
    return g / (1.0 + np.exp(-g)) * up.astype(np.float64)


def rotary(x, cos, sin):
    """RotaryEmbedding, half-split pairs (src/kernels/llm_math.h:256-274): x [tokens, heads, d], tables
    [tokens, d]; y = f32(f32(x * cos) + f32(f32(sign * partner) * sin)), sign -1 for the first half."""
    half = x.shape[-1] // 2
    partner = np.concatenate([-x[..., half:], x[..., :half]], axis=-1)
    c, s = cos[:, None, :], sin[:, None, :]
    return ((x * c).astype(np.float32) + (partner * s).astype(np.float32)).astype(np.float32)


def attention(q, k, v, q_heads, kv_heads, head_dim, causal):
    """cross_sdpa_gqa_f32 (src/kernels/cross_sdpa.inc:53): q [tq, q_heads*d], k and v [tk, kv_heads*d], scores
    scaled by f32(1/sqrt(d)), query i sees keys 0..i when causal, softmax, P.V -- in double."""
    tq, tk = q.shape[0], k.shape[0]
    rep = q_heads // kv_heads
    scale = np.float64(np.float32(1.0 / np.sqrt(head_dim)))
    out = np.zeros((tq, q_heads * head_dim))
    for h in range(q_heads):
        qs = q[:, h * head_dim:(h + 1) * head_dim].astype(np.float64)
        ks = k[:, (h // rep) * head_dim:(h // rep + 1) * head_dim].astype(np.float64)
        vs = v[:, (h // rep) * head_dim:(h // rep + 1) * head_dim].astype(np.float64)
        sc = qs @ ks.T * scale
        if causal:
            sc = np.where(np.arange(tk)[None, :] <= np.arange(tq)[:, None], sc, -np.inf)
        p = np.exp(sc - sc.max(-1, keepdims=True))
        out[:, h * head_dim:(h + 1) * head_dim] = (p / p.sum(-1, keepdims=True)) @ vs
    return out


# ---- seeded inputs -------------------------------------------------------------------------------

RMSNORM_CASES = [dict(rows=5, d=1024, seed=71), dict(rows=33, d=3000, seed=72), dict(rows=32, d=1024, seed=73),
                 dict(rows=3, d=64, seed=74)]
EPS = 1e-6


def rmsnorm_case(rows, d, seed):
    rng = np.random.default_rng(seed)
    x = (rng.normal(0, 3, (rows, d)) * rng.uniform(0.01, 100, (rows, 1))).astype(np.float32)
    if rows >= 5:
        x[1] = 0.0
    gain = rng.uniform(0.5, 1.5, d).astype(np.float32)
    return x, gain


def silu_mul_case():
    rng = np.random.default_rng(75)
    gu = rng.normal(0, 4, (3, 2 * 512)).astype(np.float32)
    gu[0, :8] = [0.0, -0.0, 30.0, -30.0, 88.0, -88.0, 1e-20, -1e-20]
    return gu


def rotary_case():
    """rows=2 sequences of t=3 tokens at cache slots 7..9, four heads of 32: x [6, 4, 32], tables [6, 32]."""
    from volvoxai_amd.decoder import DecoderConfig, rope_tables
    cfg = DecoderConfig(layers=1, hidden=64, q_heads=4, kv_heads=2, head_dim=32, inter=64, vocab=10, max_seq=16)
    cos, sin = rope_tables(cfg)
    rng = np.random.default_rng(76)
    x = rng.normal(0, 1, (6, 4, 32)).astype(np.float32)
    positions = np.array([7, 8, 9, 7, 8, 9])
    return x, np.ascontiguousarray(cos[positions]), np.ascontiguousarray(sin[positions])


ATTENTION_CASES = [dict(tq=1, tk=11, q_heads=4, kv_heads=2, head_dim=32, causal=0, seed=77),    # a decode step
                   dict(tq=5, tk=5, q_heads=4, kv_heads=2, head_dim=32, causal=1, seed=78),     # a prompt
                   dict(tq=1, tk=130, q_heads=8, kv_heads=2, head_dim=128, causal=0, seed=79),  # past the 48-key tiles
                   dict(tq=60, tk=60, q_heads=2, kv_heads=1, head_dim=64, causal=1, seed=80)]


def attention_case(tq, tk, q_heads, kv_heads, head_dim, causal, seed):
    rng = np.random.default_rng(seed)
    q = rng.normal(0, 1, (tq, q_heads * head_dim)).astype(np.float32)
    k = rng.normal(0, 1, (tk, kv_heads * head_dim)).astype(np.float32)
    v = rng.normal(0, 1, (tk, kv_heads * head_dim)).astype(np.float32)
    return q, k, v
