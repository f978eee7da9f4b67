"""The decoder with its glue written as PyTorch ops -- a CHECKER for tests only.

The shipped decoder (volvoxai_amd/decoder.py) runs everything between the linears as HIP kernels of
the library.  This subclass keeps the library's linears (vxhip_packed_linear_forward_f32) and
replaces the glue by plain PyTorch f32/f64 ops that follow the same definitions, so a test can
compare the two token for token on the device."""
import numpy as np

from volvoxai_amd.decoder import W8A8Decoder


class TorchGlueDecoder(W8A8Decoder):
    def __init__(self, cfg, weights, rows, stream=None):
        super().__init__(cfg, weights, rows, stream)
        torch = self.torch
        for L, lw in zip(self.layers, weights["layers"]):
            L["norm1"] = torch.from_numpy(lw["norm1"]).cuda().double()
            L["norm2"] = torch.from_numpy(lw["norm2"]).cuda().double()
        self.norm_f = torch.from_numpy(weights["norm_f"]).cuda().double()
        self.tokens = torch.zeros(rows, dtype=torch.int64, device="cuda")

    def _rmsnorm(self, x, gain):
        xd = x.double()
        inv = 1.0 / self.torch.sqrt((xd * xd).mean(-1, keepdim=True) + self.cfg.eps)
        return (xd * inv * gain).float()

    def _rope(self, x, cos, sin):
        # x [rows, t, heads, d]; cos/sin [t, d]
        half = self.cfg.head_dim // 2
        partner = self.torch.cat([-x[..., half:], x[..., :half]], dim=-1)
        return x * cos[None, :, None, :] + partner * sin[None, :, None, :]

    def _torch_layer(self, li, x, cos, sin, write_slots, visible):
        """x [rows, t, hidden]; write_slots [t] cache positions of these tokens; visible
        [t, max_seq] bool: which cache slots each of them may attend to."""
        torch, cfg, L = self.torch, self.cfg, self.layers[li]
        rows, t, _ = x.shape
        h = self._rmsnorm(x, L["norm1"])
        qkv = self._linear(L["qkv"], h.reshape(rows * t, cfg.hidden)).reshape(rows, t, -1)
        q = qkv[..., :cfg.q_dim].reshape(rows, t, cfg.q_heads, cfg.head_dim)
        k = qkv[..., cfg.q_dim:cfg.q_dim + cfg.kv_dim].reshape(rows, t, cfg.kv_heads, cfg.head_dim)
        v = qkv[..., cfg.q_dim + cfg.kv_dim:].reshape(rows, t, cfg.kv_heads, cfg.head_dim)
        q, k = self._rope(q, cos, sin), self._rope(k, cos, sin)
        self.k_cache[li].index_copy_(2, write_slots, k.permute(0, 2, 1, 3))
        self.v_cache[li].index_copy_(2, write_slots, v.permute(0, 2, 1, 3))
        rep = cfg.q_heads // cfg.kv_heads
        qg = q.permute(0, 2, 1, 3).reshape(rows, cfg.kv_heads, rep * t, cfg.head_dim)
        scores = torch.matmul(qg, self.k_cache[li].transpose(-1, -2)) * (1.0 / np.sqrt(cfg.head_dim))
        scores = scores.reshape(rows, cfg.kv_heads, rep, t, cfg.max_seq)
        scores = scores.masked_fill(~visible[None, None, None], float("-inf"))
        probs = torch.softmax(scores, dim=-1).reshape(rows, cfg.kv_heads, rep * t, cfg.max_seq)
        ctxv = torch.matmul(probs, self.v_cache[li]).reshape(rows, cfg.q_heads, t, cfg.head_dim)
        attn = ctxv.permute(0, 2, 1, 3).reshape(rows * t, cfg.q_dim)
        x = x + self._linear(L["o"], attn).reshape(rows, t, cfg.hidden)
        h = self._rmsnorm(x, L["norm2"])
        gu = self._linear(L["gate_up"], h.reshape(rows * t, cfg.hidden))
        act = torch.nn.functional.silu(gu[:, :cfg.inter]) * gu[:, cfg.inter:]
        return x + self._linear(L["down"], act).reshape(rows, t, cfg.hidden)

    def _head(self, x_last):
        logits = self._linear(self.lm_head, self._rmsnorm(x_last, self.norm_f))
        return logits, logits.argmax(dim=-1)

    def prefill(self, prompt):
        torch, cfg = self.torch, self.cfg
        with torch.cuda.stream(self.stream):
            t = prompt.shape[1]
            slots = self.slots[:t]
            visible = self.slots[None, :] <= slots[:, None]
            x = self.embedding[prompt]
            for li in range(cfg.layers):
                x = self._torch_layer(li, x, self.cos[:t], self.sin[:t], slots, visible)
            self.last_logits, nxt = self._head(x[:, -1, :])
            self.tokens.copy_(nxt)
            self.position.fill_(t)
            self.history.zero_()
            self.history[0].copy_(nxt)
            self.emitted = 1
        return nxt

    def _step(self):
        cfg, pos = self.cfg, self.position
        visible = self.slots[None, :] <= pos[:, None]
        cos, sin = self.cos.index_select(0, pos), self.sin.index_select(0, pos)
        x = self.embedding[self.tokens][:, None, :]
        for li in range(cfg.layers):
            x = self._torch_layer(li, x, cos, sin, pos, visible)
        self.last_logits, nxt = self._head(x[:, 0, :])
        self.tokens.copy_(nxt)
        self.position.add_(1)
        return nxt
