"""A minimal Llama-architecture decode loop around BitStackLinear, for measuring
end-to-end decode throughput on random-init weights (no checkpoints, no tokenizer).

Every decoder linear (q, k, v, o, gate, up, down) is a BitStackLinear at
fused_level 5 with a per-layer block count taken from a compression_config in the
reference's format, {"layer.{L}.self_attn.q_proj": n_blocks, ...}
(bitstack/utils/decompose.py:14, bitstack/utils/model_utils.py:53-66); embed_tokens
and lm_head stay dense fp16, as in the reference (only the decoder layers are
walked, bitstack/utils/scale_utils.py:212-221).  Everything around the linears
(RMSNorm, RoPE, attention over a static KV cache, SiLU gate) is plain torch: the
subject of the measurement is the linear path.  One decode step has static shapes
and reads its position from a device tensor, so it can be captured in a HIP graph
and replayed.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from bitstack_amd.modules.BitStackLinear import BitStackLinear

PROJ = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
        "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")


@dataclass
class LlamaShape:
    layers: int = 32
    hidden: int = 4096
    intermediate: int = 14336
    heads: int = 32
    kv_heads: int = 8
    vocab: int = 128256
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    k: int = 16

    @property
    def head_dim(self):
        return self.hidden // self.heads

    def proj_shape(self, name):
        kv = self.kv_heads * self.head_dim
        return {"self_attn.q_proj": (self.hidden, self.hidden), "self_attn.k_proj": (kv, self.hidden),
                "self_attn.v_proj": (kv, self.hidden), "self_attn.o_proj": (self.hidden, self.hidden),
                "mlp.gate_proj": (self.intermediate, self.hidden), "mlp.up_proj": (self.intermediate, self.hidden),
                "mlp.down_proj": (self.hidden, self.intermediate)}[name]

    def block_bytes(self, name):
        m, n = self.proj_shape(name)
        return m * n // 8 + 2 * self.k * (m + n)          # BitStackLinear.memory_per_bit

    def dense_bytes(self):
        return 2 * 2 * self.vocab * self.hidden            # embed_tokens + lm_head, fp16


LLAMA_8B = LlamaShape()
LLAMA_70B = LlamaShape(layers=80, hidden=8192, intermediate=28672, heads=64, kv_heads=8)


def synthetic_compression_config(shape: LlamaShape, target_bytes: float, lo=2, hi=12, seed=0):
    """Seeded per-layer block counts in [lo, hi], nudged until the total
    (dense part + sum of blocks) is as close to `target_bytes` as one block allows."""
    g = torch.Generator().manual_seed(seed)
    names = [f"layer.{L}.{p}" for L in range(shape.layers) for p in PROJ]
    counts = torch.randint(lo, hi + 1, (len(names),), generator=g).tolist()
    cost = [shape.block_bytes(n.split(".", 2)[2]) for n in names]
    total = shape.dense_bytes() + sum(c * b for c, b in zip(counts, cost))
    order = torch.randperm(len(names), generator=g).tolist()
    changed = True
    while changed:
        changed = False
        for j in order:
            if total > target_bytes and counts[j] > lo:
                counts[j] -= 1
                total -= cost[j]
                changed = True
            elif total + cost[j] <= target_bytes and counts[j] < hi:
                counts[j] += 1
                total += cost[j]
                changed = True
    return dict(zip(names, counts)), total


def _synthetic_bitstack(m, n, blocks, k, dev, gen, name):
    mod = BitStackLinear(0, n, m, k, False, False, dev, fused_level=5)
    mod.name = name
    mod.w_bit = blocks
    # written straight into the stacked layout stack_blocks() would produce
    mod.qweight = torch.randint(0, 256, (blocks, m * n // 8), dtype=torch.uint8, device=dev, generator=gen)
    scale = (0.01 / torch.arange(1, blocks + 1, device=dev, dtype=torch.float32)).view(blocks, 1, 1)
    mod.u = (torch.randn(blocks, m, k, device=dev, generator=gen).abs() * scale).half()
    mod.vt = (torch.randn(blocks, k, n, device=dev, generator=gen).abs() * scale).half()
    return mod


class SyntheticLlamaDecoder:
    """Batch-1 greedy decode with a static KV cache of `max_len` positions."""

    def __init__(self, shape: LlamaShape, config: dict, max_len: int, device, seed=0):
        self.s, self.dev, self.max_len = shape, torch.device(device), max_len
        g = torch.Generator(device=self.dev).manual_seed(seed)
        h = shape.hidden
        self.embed = (torch.randn(shape.vocab, h, device=self.dev, generator=g) * 0.02).half()
        self.lm_head = (torch.randn(shape.vocab, h, device=self.dev, generator=g) * 0.02).half()
        self.norm_w = torch.ones(shape.layers, 2, h, device=self.dev, dtype=torch.float16)
        self.final_norm = torch.ones(h, device=self.dev, dtype=torch.float16)
        self.lin = []
        for L in range(shape.layers):
            row = {}
            for p in PROJ:
                m, n = shape.proj_shape(p)
                row[p] = _synthetic_bitstack(m, n, config[f"layer.{L}.{p}"], shape.k, self.dev, g, f"layer.{L}.{p}")
            self.lin.append(row)
        d = shape.head_dim
        self.kcache = torch.zeros(shape.layers, shape.kv_heads, max_len, d, device=self.dev, dtype=torch.float16)
        self.vcache = torch.zeros_like(self.kcache)
        inv = 1.0 / (shape.rope_theta ** (torch.arange(0, d, 2, device=self.dev, dtype=torch.float32) / d))
        ang = torch.arange(max_len, device=self.dev, dtype=torch.float32)[:, None] * inv[None, :]
        self.cos, self.sin = ang.cos().half(), ang.sin().half()            # [max_len, d/2]
        self.pos = torch.zeros(1, device=self.dev, dtype=torch.long)       # next position to write
        self.token = torch.zeros(1, device=self.dev, dtype=torch.long)
        self.span = torch.arange(max_len, device=self.dev)

    def weight_bytes(self):
        b = self.embed.numel() * 2 + self.lm_head.numel() * 2
        for row in self.lin:
            for m in row.values():
                b += m.qweight.numel() + 2 * (m.u.numel() + m.vt.numel())
        return b

    def _rms(self, x, w):
        v = x.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.s.rms_eps)).half() * w

    def _rope(self, x, cos, sin):          # x [heads, d], rotate-half convention
        d2 = x.shape[-1] // 2
        a, b = x[..., :d2], x[..., d2:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)

    @torch.no_grad()
    def step(self):
        """Consume self.token at self.pos, write the greedy next token, advance."""
        s = self.s
        x = self.embed.index_select(0, self.token)                       # [1, h]
        cos = self.cos.index_select(0, self.pos)
        sin = self.sin.index_select(0, self.pos)
        mask = (self.span <= self.pos).view(1, 1, self.max_len)
        for L in range(s.layers):
            lin = self.lin[L]
            hn = self._rms(x, self.norm_w[L, 0])
            q = lin["self_attn.q_proj"](hn).view(s.heads, s.head_dim)
            k = lin["self_attn.k_proj"](hn).view(s.kv_heads, s.head_dim)
            v = lin["self_attn.v_proj"](hn).view(s.kv_heads, s.head_dim)
            q, k = self._rope(q, cos, sin), self._rope(k, cos, sin)
            self.kcache[L].index_copy_(1, self.pos, k.unsqueeze(1))
            self.vcache[L].index_copy_(1, self.pos, v.unsqueeze(1))
            rep = s.heads // s.kv_heads
            qg = q.view(s.kv_heads, rep, s.head_dim)
            att = torch.matmul(qg, self.kcache[L].transpose(1, 2)) / math.sqrt(s.head_dim)   # [kv, rep, max_len]
            att = att.masked_fill(~mask, float("-inf")).float().softmax(-1).half()
            ctx = torch.matmul(att, self.vcache[L]).reshape(1, s.hidden)
            x = x + lin["self_attn.o_proj"](ctx)
            hn = self._rms(x, self.norm_w[L, 1])
            gate = lin["mlp.gate_proj"](hn)
            up = lin["mlp.up_proj"](hn)
            x = x + lin["mlp.down_proj"](F.silu(gate) * up)
        logits = F.linear(self._rms(x, self.final_norm), self.lm_head)
        self.token.copy_(logits.argmax(-1))
        self.pos.add_(1)

    def prefill_positions(self, prompt: torch.Tensor):
        """Feed a prompt token by token (the measurement is about decode)."""
        self.pos.zero_()
        for tkn in prompt.tolist():
            self.token.fill_(tkn)
            self.step()
