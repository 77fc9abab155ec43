"""Decoder scaffolding for benchmark configuration C5 (test infrastructure).

A Qwen3-0.6B-shaped random-init decoder whose every FC (Q/K/V/O/gate/up/down,
Q4_0) and lm_head (Q6_K, tied to the embedding table) goes through a pluggable
`fc(name, x)` callable, so that a CPU leg (the oracle / the reference library) and
a GPU leg (libhipq through its C ABI) share every other line: embedding lookup,
RMSNorm, per-head q/k norm, RoPE, KV cache, grouped-query causal attention,
SwiGLU, residual adds, greedy argmax. Only the quantized matmul differs.

Follows the reference application for what it computes
(Applications/CausalLM/causal_lm.cpp:190-227, 530-533, 628-706;
layers/rms_norm.cpp:38-77; qwen3_causallm.cpp:60-82; mha_core.cpp:459-533, 617-688;
swiglu.cpp:40-62: silu(in0) * in1 with in0 = ffn_up, in1 = ffn_gate). Where the
configuration leaves a value open the usual Qwen3 one is used and recorded here:
RMSNorm eps 1e-6, RoPE theta 1e6, norm gains 1 (random-init model), fp32 KV cache,
seed 4 for weights and prompt.
"""
import numpy as np

from nntrainer_amd import synth


class Config:
    def __init__(self, layers=28, hidden=1024, inter=3072, heads=16, kv_heads=8, head_dim=128,
                 vocab=151936, eps=1e-6, theta=1e6, seed=4):
        self.layers, self.hidden, self.inter = layers, hidden, inter
        self.heads, self.kv_heads, self.head_dim = heads, kv_heads, head_dim
        self.vocab, self.eps, self.theta, self.seed = vocab, eps, theta, seed

    def fc_shapes(self):
        """name -> (N, K) of every per-layer FC, in model order."""
        h, d = self.hidden, self.head_dim
        return [("q_proj", self.heads * d, h), ("k_proj", self.kv_heads * d, h),
                ("v_proj", self.kv_heads * d, h), ("o_proj", h, self.heads * d),
                ("ffn_up", self.inter, h), ("ffn_gate", self.inter, h), ("ffn_down", h, self.inter)]


def build_weights(cfg, cr):
    """Quantized weights {name: (kind, N, K, canonical blocks)} and the fp32 embedding
    table. One generator stream (cfg.seed), consumed matrix after matrix."""
    lib = cr.oracle()
    first = 0
    w = {}
    for layer in range(cfg.layers):
        for name, n, k in cfg.fc_shapes():
            w32 = synth.normal(cfg.seed, (n, k), 0.02, first=first)
            first += n * k
            w["l%d.%s" % (layer, name)] = ("q4_0", n, k, cr.quantize_weights(lib, "q4_0", w32))
    emb = synth.normal(cfg.seed, (cfg.vocab, cfg.hidden), 0.02, first=first)
    first += cfg.vocab * cfg.hidden
    # tied lm_head: the embedding table quantized to Q6_K, one row per vocabulary entry
    w["lm_head"] = ("q6_K", cfg.vocab, cfg.hidden, cr.quantize_weights(lib, "q6_K", emb))
    # the embedding lookup reads the same Q6_K rows, as the tied layer does
    # (tie_word_embedding.cpp:213-242), so both legs see one table
    emb_q = cr.dequantize(lib, "q6_K", w["lm_head"][3], cfg.vocab * cfg.hidden).reshape(cfg.vocab, cfg.hidden)
    return w, emb_q, first


def rmsnorm(x, eps):
    x = x.astype(np.float32)
    ms = np.mean(x * x, axis=-1, keepdims=True, dtype=np.float32)
    return (x * (1.0 / np.sqrt(ms + np.float32(eps))).astype(np.float32)).astype(np.float32)


def rope(x, pos, theta):
    """x [T, heads, d]; rotate pairs (i, i + d/2) by pos * theta^(-2i/d)."""
    t, _, d = x.shape
    half = d // 2
    inv = (1.0 / (theta ** (np.arange(half, dtype=np.float64) * 2.0 / d)))
    ang = pos.astype(np.float64)[:, None] * inv[None, :]
    cos = np.cos(ang).astype(np.float32)[:, None, :]
    sin = np.sin(ang).astype(np.float32)[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return np.concatenate([x1 * cos - x2 * sin, x2 * cos + x1 * sin], axis=-1).astype(np.float32)


def attention(q, kc, vc, pos0):
    """q [T, H, d]; kc, vc [S, KV, d] (cache incl. the new rows); causal; grouped heads."""
    t, h, d = q.shape
    s, kv, _ = kc.shape
    grp = h // kv
    out = np.empty((t, h, d), np.float32)
    scale = np.float32(1.0 / np.sqrt(d))
    mask = (np.arange(s)[None, :] > (pos0 + np.arange(t))[:, None])
    for head in range(h):
        kh, vh = kc[:, head // grp, :], vc[:, head // grp, :]
        sc = (q[:, head, :] @ kh.T) * scale
        sc = np.where(mask, np.float32(-np.inf), sc)
        sc = sc - sc.max(axis=-1, keepdims=True)
        p = np.exp(sc, dtype=np.float32)
        p = p / p.sum(axis=-1, keepdims=True, dtype=np.float32)
        out[:, head, :] = p @ vh
    return out


def silu(x):
    return (x / (1.0 + np.exp(-x, dtype=np.float32))).astype(np.float32)


class Decoder:
    def __init__(self, cfg, emb, fc, trace=None):
        self.cfg, self.emb, self.fc, self.trace = cfg, emb, fc, trace
        self.kcache = [np.zeros((0, cfg.kv_heads, cfg.head_dim), np.float32) for _ in range(cfg.layers)]
        self.vcache = [np.zeros((0, cfg.kv_heads, cfg.head_dim), np.float32) for _ in range(cfg.layers)]
        self.pos = 0

    def _fc(self, name, x):
        y = self.fc(name, np.ascontiguousarray(x, np.float32))
        if self.trace is not None:
            self.trace.append((name, y.copy()))
        return y

    def step(self, ids):
        """Feeds `ids` (prefill chunk or one token); returns the next greedy token."""
        c = self.cfg
        t = len(ids)
        x = self.emb[np.asarray(ids)].astype(np.float32)
        pos = np.arange(self.pos, self.pos + t)
        for layer in range(c.layers):
            p = "l%d." % layer
            h = rmsnorm(x, c.eps)
            q = self._fc(p + "q_proj", h).reshape(t, c.heads, c.head_dim)
            k = self._fc(p + "k_proj", h).reshape(t, c.kv_heads, c.head_dim)
            v = self._fc(p + "v_proj", h).reshape(t, c.kv_heads, c.head_dim)
            q = rope(rmsnorm(q, c.eps), pos, c.theta)
            k = rope(rmsnorm(k, c.eps), pos, c.theta)
            self.kcache[layer] = np.concatenate([self.kcache[layer], k], axis=0)
            self.vcache[layer] = np.concatenate([self.vcache[layer], v], axis=0)
            a = attention(q, self.kcache[layer], self.vcache[layer], self.pos)
            x = x + self._fc(p + "o_proj", a.reshape(t, c.heads * c.head_dim))
            h = rmsnorm(x, c.eps)
            up = self._fc(p + "ffn_up", h)
            gate = self._fc(p + "ffn_gate", h)
            x = x + self._fc(p + "ffn_down", silu(up) * gate)
        self.pos += t
        # lm_head takes only the last row: a GEMV even during prefill
        logits = self._fc("lm_head", rmsnorm(x[-1:], c.eps))
        return int(np.argmax(logits[0])), logits[0]


def generate(cfg, emb, fc, prompt, n_decode, trace_first=False):
    trace = [] if trace_first else None
    dec = Decoder(cfg, emb, fc, trace)
    tok, _ = dec.step(prompt)
    first_trace = trace
    dec.trace = None
    out = [tok]
    for _ in range(n_decode - 1):
        tok, _ = dec.step([tok])
        out.append(tok)
    return out, first_trace


class CpuFC:
    """FC on the CPU: the reference library where it was built, else the oracle."""

    def __init__(self, weights, cr):
        self.cr = cr
        self.lib = cr.ref() or cr.oracle()
        self.w = {name: (kind, n, cr.prepack(self.lib, kind, blocks, n, k))
                  for name, (kind, n, k, blocks) in weights.items()}

    def __call__(self, name, x):
        kind, n, packed = self.w[name]
        return self.cr.gemm_prepacked(self.lib, kind, x, packed, n)


class GpuFC:
    """FC on the GPU through the C ABI, host buffers in and out."""

    def __init__(self, weights):
        from nntrainer_amd import capi
        self.capi = capi
        self.h = {name: (capi.Weight(kind, n, k, blocks), n) for name, (kind, n, k, blocks) in weights.items()}

    def __call__(self, name, x):
        w, n = self.h[name]
        y = np.empty((x.shape[0], n), np.float32)
        self.capi.matmul(w, x, x.shape[0], y, mem=self.capi.MEM_HOST)
        return y

    def close(self):
        for w, _ in self.h.values():
            w.destroy()
