"""Decoder-only transformer with every linear routed to the W8A8 PackedLinear
kernels (28 layers, hidden 1024, 16 query / 8 KV heads of 128, SwiGLU 3072 by
default).  Everything between the linears -- embedding gather, residual add +
RMSNorm + activation preparation, rotary embedding + KV-cache append,
grouped-query attention, SwiGLU + preparation, greedy selection -- runs as HIP
kernels of the same library (vxhip_*_prepare_i8, vxhip_rope_*, vxhip_gqa_*,
vxhip_embedding_gather_f32, vxhip_argmax_rows_f32); the linears are
`vxhip_packed_linear_forward_a8` / `_f32` (DYNAMIC_I8: per-row activation
quantization, int8 x int8 MFMA, dequant to f32).  PyTorch supplies device
memory, the stream and the HIP graph, no arithmetic.

The glue follows the reference's definitions: RMSNorm accumulates and scales in
double (native/src/kernels/softmax_rmsnorm.inc:3-17); the rotary embedding is the
non-interleaved form y[d] = x[d]*cos + sign*x[partner]*sin with partner d +- width/2
(native/src/kernels/llm_math.h:256-274).

A decode step has fixed shapes (position and tokens live on the device), so it can
be captured once in a HIP graph and replayed; the launches of the linears are
captured with it because the context runs on the capture stream.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from . import w8a8 as vx
from ._lib import library as _library


@dataclass(frozen=True)
class DecoderConfig:
    layers: int = 28
    hidden: int = 1024
    q_heads: int = 16
    kv_heads: int = 8
    head_dim: int = 128
    inter: int = 3072
    vocab: int = 32000
    group: int = 128
    rope_theta: float = 10000.0
    eps: float = 1e-6
    max_seq: int = 256

    @property
    def q_dim(self):
        return self.q_heads * self.head_dim

    @property
    def kv_dim(self):
        return self.kv_heads * self.head_dim


def pack_w8_words(w: np.ndarray) -> np.ndarray:
    """int8 [n, k] -> offset-binary W8 words [n, ceil(k/4)]: code = w + 128, element 4i+j in
    byte j of word i, absent elements as the zero code 0x80 (docs/packed-linear-design.md:24-32)."""
    n, k = w.shape
    words = (k + 3) // 4
    codes = np.full((n, words * 4), 0x80, np.uint8)
    codes[:, :k] = (w.astype(np.int16) + 128).astype(np.uint8)
    return codes.view("<u4").reshape(n, words)


def pack_w4_words(w: np.ndarray) -> np.ndarray:
    """int8 [n, k] with values -8..7 -> W4 words [n, vx_packed_words(k, 4)]: code = w + 8,
    element 8i+j in nibble j of word i, absent elements as the zero code 8
    (native/src/kernels/packed_linear_ops.inc:246-248, 476-477)."""
    n, k = w.shape
    words = (k // 32) * 4 + ((k % 32) * 4 + 31) // 32
    codes = np.full((n, words * 8), 8, np.uint8)
    codes[:, :k] = (w.astype(np.int16) + 8).astype(np.uint8) & 15
    pairs = codes[:, 0::2] | (codes[:, 1::2] << 4)
    return np.ascontiguousarray(pairs).view("<u4").reshape(n, words)


def init_weights(cfg: DecoderConfig, seed: int) -> dict:
    """Random-init weights of the architecture: int8 uniform +-127 with per-channel scales
    ~U(0.002, 0.01) for every linear, f32 embedding and norm gains."""
    rng = np.random.default_rng(seed)

    def linear(n, k):
        w = rng.integers(-127, 128, (n, k)).astype(np.int8)
        chan = rng.uniform(0.002, 0.01, n).astype(np.float32)
        groups = (k + cfg.group - 1) // cfg.group
        return {"w": w, "scales": np.repeat(chan[:, None], groups, axis=1).copy()}

    layers = []
    for _ in range(cfg.layers):
        layers.append({
            "norm1": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32),
            "qkv": linear(cfg.q_dim + 2 * cfg.kv_dim, cfg.hidden),
            "o": linear(cfg.hidden, cfg.q_dim),
            "norm2": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32),
            "gate_up": linear(2 * cfg.inter, cfg.hidden),
            "down": linear(cfg.hidden, cfg.inter),
        })
    return {"embedding": rng.normal(0, 1, (cfg.vocab, cfg.hidden)).astype(np.float32),
            "layers": layers,
            "norm_f": rng.uniform(0.5, 1.5, cfg.hidden).astype(np.float32),
            "lm_head": linear(cfg.vocab, cfg.hidden)}


def rope_tables(cfg: DecoderConfig):
    """cos/sin [max_seq, head_dim]: entry d and d + head_dim/2 share frequency d % (head_dim/2)."""
    half = cfg.head_dim // 2
    inv = cfg.rope_theta ** (-np.arange(half, dtype=np.float64) * 2.0 / cfg.head_dim)
    angle = np.arange(cfg.max_seq, dtype=np.float64)[:, None] * inv[None, :]
    angle = np.concatenate([angle, angle], axis=1)
    return np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)


class W8A8Decoder:
    def __init__(self, cfg: DecoderConfig, weights: dict, rows: int, stream=None, fuse_rows=None):
        import torch
        self.torch, self.cfg, self.rows = torch, cfg, rows
        # One row: a decode step runs the fused single-row forms (five launches per layer instead of nine)
        # where the library takes every linear of a layer that way.  They take two rows as well, at the
        # speed of the separate launches (fuse_rows=True asks for them; None decides by the row count).
        wanted = rows == 1 if fuse_rows is None else bool(fuse_rows)
        self.rows_fused = False  # settled below, once the linears exist: the library is asked about each one
        self.stream = stream if stream is not None else torch.cuda.Stream()
        self.ctx = vx.Context(0, self.stream)
        # prepared activations of up to 32 rows travel between the glue kernels and the GEMVs in
        # the GEMV's operand order
        self.ctx.set_activation_layout(True)
        dev = "cuda"

        def make(lin):
            k = lin["w"].shape[1]
            return vx.PackedLinear(pack_w8_words(lin["w"]), lin["scales"], None, k, lin["w"].shape[0], cfg.group)

        self.embedding = torch.from_numpy(weights["embedding"]).to(dev)
        self.layers = []
        for lw in weights["layers"]:
            self.layers.append({"gain1": torch.from_numpy(lw["norm1"]).to(dev),
                                "gain2": torch.from_numpy(lw["norm2"]).to(dev),
                                "qkv": make(lw["qkv"]), "o": make(lw["o"]),
                                "gate_up": make(lw["gate_up"]), "down": make(lw["down"])})
        self.gain_f = torch.from_numpy(weights["norm_f"]).to(dev)
        self.lm_head = make(weights["lm_head"])
        if wanted and rows <= 2:
            # the residual stream is updated in place by the first fused launch of a layer, so every
            # linear of every layer has to be taken that way, or none is
            self.rows_fused = all(
                L["qkv"].fused_takes(self.ctx, rows, vx.ROW_OP_RMSNORM, False) and L["o"].fused_takes(self.ctx, rows, vx.ROW_OP_NONE, True)
                and L["gate_up"].fused_takes(self.ctx, rows, vx.ROW_OP_RMSNORM, False)
                and L["down"].fused_takes(self.ctx, rows, vx.ROW_OP_SWIGLU, True) for L in self.layers)
        cos, sin = rope_tables(cfg)
        self.cos, self.sin = torch.from_numpy(cos).to(dev), torch.from_numpy(sin).to(dev)
        shape = (cfg.layers, rows, cfg.kv_heads, cfg.max_seq, cfg.head_dim)
        self.k_cache = torch.zeros(shape, dtype=torch.float32, device=dev)
        self.v_cache = torch.zeros(shape, dtype=torch.float32, device=dev)
        # state of the decode loop, on the device so a captured step advances by itself
        # (int32 ids, as the reference's embedding takes them)
        self.tokens = torch.zeros(rows, dtype=torch.int32, device=dev)
        self.position = torch.zeros(1, dtype=torch.int64, device=dev)
        self.history = torch.zeros((cfg.max_seq, rows), dtype=torch.int64, device=dev)
        self.slots = torch.arange(cfg.max_seq, device=dev)
        self.graph = None

    # ---- pieces ---------------------------------------------------------------------------
    def _linear(self, pl, x2d):
        torch = self.torch
        x2d = x2d.contiguous()
        out = torch.empty((x2d.shape[0], pl.n), dtype=torch.float32, device=x2d.device)
        st, _ = pl.forward_f32(self.ctx, x2d, out=out)
        if st != 0:
            raise RuntimeError(_library().vxhip_last_error().decode())
        return out

    def _linear_a8(self, pl, a8, scales):
        torch = self.torch
        out = torch.empty((scales.shape[0], pl.n), dtype=torch.float32, device=a8.device)
        st, _ = pl.forward_a8(self.ctx, a8, scales, out=out)
        if st != 0:
            raise RuntimeError(_library().vxhip_last_error().decode())
        return out

    def _layer(self, li, x2, delta, positions, rows, t):
        """One layer.  x2 [rows*t, hidden] is the residual
        stream, updated in place; delta is the previous layer's MLP output still to be added to it
        (the add rides in the next RMSNorm kernel).  Returns this layer's pending delta."""
        cfg, L = self.cfg, self.layers[li]
        if delta is None:
            a8, sc = vx.rmsnorm_prepare_i8(self.ctx, x2, L["gain1"], cfg.eps)
        else:
            a8, sc = vx.add_rmsnorm_prepare_i8(self.ctx, x2, delta, L["gain1"], cfg.eps)
        qkv = self._linear_a8(L["qkv"], a8, sc).reshape(rows, t, -1)
        if t == 1:
            # a decode step: rotary, cache append and attention in one launch
            attn = vx.rope_gqa_attention_decode(self.ctx, qkv.reshape(rows, -1), self.cos, self.sin, positions,
                                                cfg.q_heads, cfg.kv_heads, cfg.head_dim, self.k_cache[li],
                                                self.v_cache[li])
            o = self._linear(L["o"], attn)
            a8, sc = vx.add_rmsnorm_prepare_i8(self.ctx, x2, o, L["gain2"], cfg.eps)
            gu = self._linear_a8(L["gate_up"], a8, sc)
            a8, sc = vx.swiglu_prepare_i8(self.ctx, gu)
            return self._linear_a8(L["down"], a8, sc)
        q = vx.rope_append_kv(self.ctx, qkv, self.cos, self.sin, positions, cfg.q_heads, cfg.kv_heads, cfg.head_dim,
                              self.k_cache[li], self.v_cache[li])
        # the prompt: every token attends to the cache slots up to its own
        attn = vx.gqa_attention(self.ctx, q, self.k_cache[li], self.v_cache[li], positions)
        o = self._linear(L["o"], attn.reshape(rows * t, cfg.q_dim))
        a8, sc = vx.add_rmsnorm_prepare_i8(self.ctx, x2, o, L["gain2"], cfg.eps)
        gu = self._linear_a8(L["gate_up"], a8, sc)
        a8, sc = vx.swiglu_prepare_i8(self.ctx, gu)
        return self._linear_a8(L["down"], a8, sc)

    def _fused(self, pl, x, row_op, gain=None, add_to=None):
        handled, out = pl.forward_fused(self.ctx, x, row_op, gain=gain, eps=self.cfg.eps, add_to=add_to, out=add_to)
        if not handled:
            raise RuntimeError(f"the fused decode linear declined k={pl.k} n={pl.n} rows={x.shape[0]}: "
                               + _library().vxhip_last_error().decode())
        return out

    def _layer_rows_fused(self, li, x2, positions, rows):
        """One layer of a decode step of one or two rows in five launches, the fused forms of the reference's
        device route (cuda_forward_gemv_pair_kernels.inc:1136,672,1424,408): RMSNorm rides in front of the
        q/k/v and gate/up linears, SwiGLU in front of the down projection, and the two residual adds
        behind the output and down projections, which update x2 in place.  Same bits as `_layer`."""
        cfg, L = self.cfg, self.layers[li]
        qkv = self._fused(L["qkv"], x2, vx.ROW_OP_RMSNORM, gain=L["gain1"])
        attn = vx.rope_gqa_attention_decode(self.ctx, qkv, self.cos, self.sin, positions, cfg.q_heads, cfg.kv_heads,
                                            cfg.head_dim, self.k_cache[li], self.v_cache[li])
        self._fused(L["o"], attn, vx.ROW_OP_NONE, add_to=x2)
        gu = self._fused(L["gate_up"], x2, vx.ROW_OP_RMSNORM, gain=L["gain2"])
        self._fused(L["down"], gu, vx.ROW_OP_SWIGLU, add_to=x2)

    def _forward(self, tokens, positions, next_tokens=None, advance=None):
        """tokens int32 [rows, t] -> logits of the last position and their argmax (int32, written
        to `next_tokens` when given; `advance` counters are incremented by the same launch)."""
        cfg = self.cfg
        rows, t = tokens.shape
        x2 = vx.embedding_gather(self.ctx, tokens.reshape(-1), self.embedding)
        if t == 1 and self.rows_fused:
            for li in range(cfg.layers):
                self._layer_rows_fused(li, x2, positions, rows)
            handled, logits = self.lm_head.forward_fused(self.ctx, x2, vx.ROW_OP_RMSNORM, gain=self.gain_f, eps=cfg.eps)
            if not handled:
                a8, sc = vx.rmsnorm_prepare_i8(self.ctx, x2, self.gain_f, cfg.eps)
                logits = self._linear_a8(self.lm_head, a8, sc)
            return logits, vx.argmax_rows(self.ctx, logits, out=next_tokens, advance=advance)
        delta = None
        for li in range(cfg.layers):
            delta = self._layer(li, x2, delta, positions, rows, t)
        if t > 1:
            x2 = x2.reshape(rows, t, cfg.hidden)[:, -1, :].contiguous()
            delta = delta.reshape(rows, t, cfg.hidden)[:, -1, :].contiguous()
        a8, sc = vx.add_rmsnorm_prepare_i8(self.ctx, x2, delta, self.gain_f, cfg.eps)
        logits = self._linear_a8(self.lm_head, a8, sc)
        return logits, vx.argmax_rows(self.ctx, logits, out=next_tokens, advance=advance)

    # ---- prefill and decode -----------------------------------------------------------------
    def prefill(self, prompt):
        """prompt int64 [rows, t] on the device; fills the cache and returns the first new tokens."""
        torch, cfg = self.torch, self.cfg
        with torch.cuda.stream(self.stream):
            t = prompt.shape[1]
            self.last_logits, nxt = self._forward(prompt.to(torch.int32).contiguous(), self.slots[:t])
            self.tokens.copy_(nxt)
            self.position.fill_(t)
            self.history.zero_()
            self.history[0].copy_(nxt)
            self.emitted = 1
        self._check_faults("prefill")
        return nxt

    def _check_faults(self, what):
        """Token ids, cache positions and row scales live in device memory, where only the kernels
        can check them: a raised fault bit means the results of this call are meaningless."""
        flags = self.ctx.fault_flags()  # synchronises the stream
        if flags:
            self.ctx.clear_fault_flags()
            raise RuntimeError(f"W8A8Decoder.{what}: device fault flags {flags:#x} "
                               "(1 bad multiplier, 2 token id outside the table, 4 position past the cache)")

    def _step(self):
        # the argmax launch writes the next ids over the current ones and advances the position
        self.last_logits, nxt = self._forward(self.tokens[:, None], self.position, next_tokens=self.tokens,
                                              advance=self.position)
        return nxt

    def capture(self):
        """Capture one decode step in a HIP graph (after a warm-up step has sized every scratch).
        The graph stays valid when a later, larger call (a longer prompt) grows the context's
        scratch: the library keeps outgrown scratch blocks alive until the context is destroyed."""
        torch = self.torch
        keep = (self.tokens.clone(), self.position.clone(), self.k_cache.clone(), self.v_cache.clone())
        with torch.cuda.stream(self.stream):
            self._step()  # warm-up: allocations and one-time kernel attributes happen here
        self.stream.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=self.stream):
            self.step_out = self._step()
        self.stream.synchronize()
        self.tokens.copy_(keep[0])
        self.position.copy_(keep[1])
        self.k_cache.copy_(keep[2])
        self.v_cache.copy_(keep[3])
        torch.cuda.synchronize()

    def decode(self, steps):
        """Greedy decode of `steps` further tokens per row; returns int64 [emitted, rows]."""
        torch = self.torch
        with torch.cuda.stream(self.stream):
            for _ in range(steps):
                if self.graph is not None:
                    self.graph.replay()
                    nxt = self.step_out
                else:
                    nxt = self._step()
                self.history[self.emitted].copy_(nxt)
                self.emitted += 1
        self._check_faults("decode")
        return self.history[:self.emitted]

    def close(self):
        for L in self.layers:
            for name in ("qkv", "o", "gate_up", "down"):
                L[name].close()
        self.lm_head.close()
        self.ctx.close()
