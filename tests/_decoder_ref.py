"""CPU restatement of the config-4 decoder for the parity test: the oracle's PackedLinear
(DYNAMIC_I8) for every linear, numpy for the glue, same definitions as
volvoxai_amd/decoder.py (RMSNorm in double: native/src/kernels/softmax_rmsnorm.inc:3-17;
non-interleaved rotary embedding: native/src/kernels/llm_math.h:256-274).  Test
infrastructure only."""
import numpy as np


class DecoderRef:
    def __init__(self, cfg, weights, oracle, rope_tables, blocked=False):
        """blocked=True runs the linears through the oracle's vectorised PackedLinear (same bits as
        the scalar one, pinned in tests/test_oracle.py): the benchmark's dimensions in seconds."""
        self.cfg, self.w, self.orc, self.blocked = cfg, weights, oracle, blocked
        self.cos, self.sin = rope_tables(cfg)
        self.packed = {}

    def linear(self, key, lin, x2d):
        if self.blocked:
            from oracle.pyoracle import packed_linear_a8_blocked
            a8, s, fin = self.orc.packed_prepare(np.ascontiguousarray(x2d, np.float32))
            s = np.where(fin == 1, s, np.nan).astype(np.float32)
            return packed_linear_a8_blocked(a8, s, lin["w"], lin["scales"], None, self.cfg.group)[0]
        if key not in self.packed:
            self.packed[key] = self.orc.pack_w8_words(lin["w"])
        _, y = self.orc.packed_linear(np.ascontiguousarray(x2d, np.float32), self.packed[key], lin["scales"], None,
                                      lin["w"].shape[0], self.cfg.group)
        return y

    def rmsnorm(self, x, gain):
        # the reference's own order of operations, pinned to rmsnorm_f32 bit for bit (tests/_glue_defs.py)
        from _glue_defs import rmsnorm
        return rmsnorm(x.reshape(-1, x.shape[-1]), gain, self.cfg.eps).reshape(x.shape)

    def rope(self, x, cos, sin):
        # x [rows, t, heads, d], tables [t, d]: the RotaryEmbedding operator's arithmetic, pinned the same way
        from _glue_defs import rotary
        rows, t = x.shape[:2]
        y = rotary(x.reshape(rows * t, x.shape[2], x.shape[3]), np.tile(cos, (rows, 1)), np.tile(sin, (rows, 1)))
        return y.reshape(x.shape)

    def forward(self, tokens, start, k_cache, v_cache, trace=None):
        """tokens [rows, t] at positions start..start+t-1; caches [layers][rows, kvh, seq, d] lists
        grown in place.  Returns the logits of the last position.  `trace` (a list) receives one
        dict per layer with every intermediate tensor, for stage-by-stage comparisons."""
        cfg = self.cfg
        rows, t = tokens.shape
        x = self.w["embedding"][tokens]
        cos, sin = self.cos[start:start + t], self.sin[start:start + t]
        rep = cfg.q_heads // cfg.kv_heads
        for li, L in enumerate(self.w["layers"]):
            x_in = x
            h = self.rmsnorm(x, L["norm1"])
            qkv = self.linear((li, "qkv"), L["qkv"], h.reshape(rows * t, -1)).reshape(rows, t, -1)
            q = self.rope(qkv[..., :cfg.q_dim].reshape(rows, t, cfg.q_heads, cfg.head_dim), cos, sin)
            k = self.rope(qkv[..., cfg.q_dim:cfg.q_dim + cfg.kv_dim].reshape(rows, t, cfg.kv_heads, cfg.head_dim), cos, sin)
            v = qkv[..., cfg.q_dim + cfg.kv_dim:].reshape(rows, t, cfg.kv_heads, cfg.head_dim)
            k_cache[li] = np.concatenate([k_cache[li], k.transpose(0, 2, 1, 3)], axis=2)
            v_cache[li] = np.concatenate([v_cache[li], v.transpose(0, 2, 1, 3)], axis=2)
            seq = k_cache[li].shape[2]
            qg = q.transpose(0, 2, 1, 3).reshape(rows, cfg.kv_heads, rep, t, cfg.head_dim)
            if self.blocked:  # the same f32 products through BLAS: the benchmark's prompt in seconds
                scores = np.matmul(qg.reshape(rows, cfg.kv_heads, rep * t, cfg.head_dim),
                                   k_cache[li].transpose(0, 1, 3, 2)).reshape(rows, cfg.kv_heads, rep, t, seq)
            else:
                scores = np.einsum("bgrtd,bgsd->bgrts", qg, k_cache[li]).astype(np.float32)
            scores = scores * np.float32(1.0 / np.sqrt(cfg.head_dim))
            visible = np.arange(seq)[None, :] <= (start + np.arange(t))[:, None]
            scores = np.where(visible[None, None, None], scores, -np.inf)
            scores = scores - scores.max(-1, keepdims=True)
            p = np.exp(scores).astype(np.float32)
            p = p / p.sum(-1, keepdims=True)
            if self.blocked:
                ctxv = np.matmul(p.reshape(rows, cfg.kv_heads, rep * t, seq), v_cache[li])
            else:
                ctxv = np.einsum("bgrts,bgsd->bgrtd", p, v_cache[li]).astype(np.float32)
            attn = ctxv.reshape(rows, cfg.q_heads, t, cfg.head_dim).transpose(0, 2, 1, 3).reshape(rows * t, cfg.q_dim)
            o = self.linear((li, "o"), L["o"], attn)
            x = x + o.reshape(rows, t, -1)
            h = self.rmsnorm(x, L["norm2"])
            gu = self.linear((li, "gu"), L["gate_up"], h.reshape(rows * t, -1))
            gate, up = gu[:, :cfg.inter], gu[:, cfg.inter:]
            act = (gate / (1.0 + np.exp(-gate.astype(np.float64)))).astype(np.float32) * up
            down = self.linear((li, "down"), L["down"], act)
            if trace is not None:
                trace.append(dict(x_in=x_in, qkv=qkv, attn=attn, o=o, x_mid=x, gu=gu, act=act, down=down))
            x = x + down.reshape(rows, t, -1)
        return self.linear("head", self.w["lm_head"], self.rmsnorm(x[:, -1, :], self.w["norm_f"]))

    def generate(self, prompt, new_tokens):
        cfg = self.cfg
        rows = prompt.shape[0]
        kc = [np.zeros((rows, cfg.kv_heads, 0, cfg.head_dim), np.float32) for _ in range(cfg.layers)]
        vc = [np.zeros((rows, cfg.kv_heads, 0, cfg.head_dim), np.float32) for _ in range(cfg.layers)]
        logits = [self.forward(prompt, 0, kc, vc)]
        out = [logits[-1].argmax(-1)]
        for i in range(new_tokens - 1):
            logits.append(self.forward(out[-1][:, None], prompt.shape[1] + i, kc, vc))
            out.append(logits[-1].argmax(-1))
        return np.stack(out), logits
