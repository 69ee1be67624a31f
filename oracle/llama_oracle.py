"""TEST INFRASTRUCTURE ONLY: float64 restatement of one Llama decode step.

The reference patches BitStackLinear modules into a Hugging Face Llama
(bitstack/utils/decompose.py:8-31 over the layers found by
bitstack/utils/scale_utils.py:212-221) and leaves everything around the linears
to that third-party model code (`transformers`, not pinned by the reference's
pyproject.toml; 5.15.0 is what this image holds).  The published algorithm is
restated here: RMSNorm, rotate-half RoPE, grouped-query softmax attention over a
KV cache, SiLU-gated MLP, residuals, final norm, lm_head.  Pinned in
tests/test_llama_oracle.py against the `transformers` Llama model itself on a
tiny random configuration (every position of a sequence, token by token here
versus one causal pass there).

Nothing here is imported by the product; only tests, the smoke test and the
benchmark's checker may use it.
"""
from __future__ import annotations

import numpy as np


def rmsnorm(x, weight, eps):
    """weight * x / sqrt(mean(x^2) + eps) over the last axis."""
    x = np.asarray(x, dtype=np.float64)
    return np.asarray(weight, dtype=np.float64) * (x / np.sqrt((x * x).mean(-1, keepdims=True) + eps))


def rope_tables(max_len, head_dim, theta):
    """cos / sin [max_len, head_dim / 2] for inverse frequencies theta^(-2i/d)."""
    inv = 1.0 / (theta ** (np.arange(0, head_dim, 2, dtype=np.float64) / head_dim))
    ang = np.arange(max_len, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang), np.sin(ang)


def rope(x, cos, sin):
    """Rotate-half convention: dimension i pairs with i + d/2.  x [..., d]; cos, sin [d/2]."""
    x = np.asarray(x, dtype=np.float64)
    h = x.shape[-1] // 2
    a, b = x[..., :h], x[..., h:]
    return np.concatenate([a * cos - b * sin, b * cos + a * sin], axis=-1)


def silu(x):
    return x / (1.0 + np.exp(-x))


def attention_decode(q, kcache, vcache, n_valid):
    """q [heads, d]; caches [kv_heads, >= n_valid, d]; head h reads kv head h // (heads / kv_heads)."""
    heads, d = q.shape
    rep = heads // kcache.shape[0]
    out = np.zeros((heads, d))
    for h in range(heads):
        k = kcache[h // rep, :n_valid]
        v = vcache[h // rep, :n_valid]
        s = k @ q[h] / np.sqrt(d)
        e = np.exp(s - s.max())
        out[h] = (e / e.sum()) @ v
    return out


class LlamaOracle:
    """Dense-weight Llama decoder, one sequence, token by token.  `weights` maps
    Hugging Face parameter names to arrays: model.embed_tokens.weight,
    model.layers.{L}.input_layernorm.weight, ...self_attn.{q,k,v,o}_proj.weight,
    ...post_attention_layernorm.weight, ...mlp.{gate,up,down}_proj.weight,
    model.norm.weight, lm_head.weight."""

    def __init__(self, weights, layers, heads, kv_heads, head_dim, rope_theta, eps, max_len):
        self.w = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
        self.layers, self.heads, self.kv, self.d, self.eps = layers, heads, kv_heads, head_dim, eps
        self.cos, self.sin = rope_tables(max_len, head_dim, rope_theta)
        self.k = np.zeros((layers, kv_heads, max_len, head_dim))
        self.v = np.zeros((layers, kv_heads, max_len, head_dim))
        self.pos = 0

    def step(self, token):
        """Feeds one token id at the current position, returns the logits."""
        w, p = self.w, self.pos
        x = w["model.embed_tokens.weight"][token]
        for L in range(self.layers):
            pre = f"model.layers.{L}."
            h = rmsnorm(x, w[pre + "input_layernorm.weight"], self.eps)
            q = (w[pre + "self_attn.q_proj.weight"] @ h).reshape(self.heads, self.d)
            k = (w[pre + "self_attn.k_proj.weight"] @ h).reshape(self.kv, self.d)
            v = (w[pre + "self_attn.v_proj.weight"] @ h).reshape(self.kv, self.d)
            q, k = rope(q, self.cos[p], self.sin[p]), rope(k, self.cos[p], self.sin[p])
            self.k[L, :, p], self.v[L, :, p] = k, v
            ctx = attention_decode(q, self.k[L], self.v[L], p + 1).reshape(-1)
            x = x + w[pre + "self_attn.o_proj.weight"] @ ctx
            h = rmsnorm(x, w[pre + "post_attention_layernorm.weight"], self.eps)
            act = silu(w[pre + "mlp.gate_proj.weight"] @ h) * (w[pre + "mlp.up_proj.weight"] @ h)
            x = x + w[pre + "mlp.down_proj.weight"] @ act
        self.pos += 1
        return w["lm_head.weight"] @ rmsnorm(x, w["model.norm.weight"], self.eps)
