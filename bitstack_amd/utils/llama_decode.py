"""A minimal Llama-architecture decode loop around BitStackLinear, for measuring
end-to-end decode throughput on random-init weights (no checkpoints, no tokenizer).

Every decoder linear (q, k, v, o, gate, up, down) is a BitStackLinear at
fused_level 5 with a per-layer block count taken from a compression_config in the
reference's format, {"layer.{L}.self_attn.q_proj": n_blocks, ...}
(bitstack/utils/decompose.py:14, bitstack/utils/model_utils.py:53-66); embed_tokens
and lm_head stay dense fp16, as in the reference (only the decoder layers are
walked, bitstack/utils/scale_utils.py:212-221).  Everything around the linears
(RMSNorm, RoPE, attention over a static KV cache, SiLU gate) is plain torch in
step() and the library's decode-step kernels in step_fused().  One decode step has
static shapes and reads its position from a device tensor, so it can be captured in
a HIP graph and replayed.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from bitstack_amd._lib import EPI_NONE, EPI_RESIDUAL, EPI_SWIGLU
from bitstack_amd.modules.BitStackLinear import BitStackLinear
from bitstack_amd.utils.inference_utils import (MatrixGroup, argmax_hip, attention_decode_hip,
                                                bitstack_forward_group_hip, rmsnorm_hip)

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
    # Hugging Face `rope_scaling` / `rope_parameters` dictionary (None: plain RoPE); see rope_inv_freq
    rope_scaling: dict | None = None

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


def rope_inv_freq(head_dim: int, theta: float, scaling: dict | None = None) -> torch.Tensor:
    """Inverse RoPE frequencies [head_dim / 2] (float32, CPU) for a Hugging Face rope configuration.

    None / "default": theta^(-2j/d).  "linear": those divided by `factor`.  "llama3" (the released
    Llama-3.1 / 3.2 checkpoints the reference evaluates): wavelengths above
    original_max_position_embeddings / low_freq_factor are divided by `factor`, those below
    original / high_freq_factor are kept, and the band between is blended linearly in
    original / wavelength.  Any other type raises: the tables would silently be wrong."""
    import math
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    kind = (scaling or {}).get("rope_type", (scaling or {}).get("type", "default")) or "default"
    if kind == "default":
        return inv
    if kind == "linear":
        return inv / float(scaling["factor"])
    if kind != "llama3":
        raise ValueError(f"rope scaling type {kind!r} is not supported (default, linear, llama3 are)")
    factor, lo_f, hi_f = float(scaling["factor"]), float(scaling["low_freq_factor"]), float(scaling["high_freq_factor"])
    old_len = float(scaling["original_max_position_embeddings"])
    wavelen = 2 * math.pi / inv
    smooth = (old_len / wavelen - lo_f) / (hi_f - lo_f)
    blended = (1 - smooth) * inv / factor + smooth * inv
    out = torch.where(wavelen > old_len / lo_f, inv / factor, inv)
    mid = (wavelen <= old_len / lo_f) & (wavelen >= old_len / hi_f)
    return torch.where(mid, blended, out)


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
    """Greedy decode of `batch` sequences in lock step (all at the same position)
    with a static KV cache of `max_len` positions.

    step()        every op around the linears is a torch op, one BitStackLinear
                  call per projection (the structure the reference runs);
    step_fused()  four launch pairs per layer for the seven linears (q/k/v in one,
                  o with the residual add, gate/up with the SiLU product, down with
                  the residual add; the two RMSNorms ride on the q/k/v and gate/up
                  launches) and one attention kernel, all from the library."""

    def __init__(self, shape: LlamaShape, config: dict, max_len: int, device, seed=0, batch=1):
        dev = torch.device(device)
        g = torch.Generator(device=dev).manual_seed(seed)
        h = shape.hidden
        embed = (torch.randn(shape.vocab, h, device=dev, generator=g) * 0.02).half()
        lm_head = (torch.randn(shape.vocab, h, device=dev, generator=g) * 0.02).half()
        norm_w = torch.ones(shape.layers, 2, h, device=dev, dtype=torch.float16)
        final_norm = torch.ones(h, device=dev, dtype=torch.float16)
        lin = []
        for L in range(shape.layers):
            row = {}
            for p in PROJ:
                m, n = shape.proj_shape(p)
                row[p] = _synthetic_bitstack(m, n, config[f"layer.{L}.{p}"], shape.k, dev, g, f"layer.{L}.{p}")
            lin.append(row)
        self._setup(shape, lin, embed, lm_head, norm_w, final_norm, max_len, dev, batch)

    def _setup(self, shape, lin, embed, lm_head, norm_w, final_norm, max_len, dev, batch):
        self.s, self.dev, self.max_len, self.batch = shape, dev, max_len, batch
        self.lin, self.embed, self.lm_head, self.norm_w, self.final_norm = lin, embed, lm_head, norm_w, final_norm
        d = shape.head_dim
        self.kcache = torch.zeros(shape.layers, batch, shape.kv_heads, max_len, d, device=self.dev, dtype=torch.float16)
        self.vcache = torch.zeros_like(self.kcache)
        inv = rope_inv_freq(d, shape.rope_theta, shape.rope_scaling).to(self.dev)
        ang = torch.arange(max_len, device=self.dev, dtype=torch.float32)[:, None] * inv[None, :]
        self.cos, self.sin = ang.cos().half().contiguous(), ang.sin().half().contiguous()   # [max_len, d/2]
        self.pos = torch.zeros(1, device=self.dev, dtype=torch.long)       # next position to write
        self.token = torch.zeros(batch, device=self.dev, dtype=torch.long)
        self.span = torch.arange(max_len, device=self.dev)
        self.logits = None
        self._groups = None

    @classmethod
    def from_checkpoint(cls, path, max_len, device, compression_config=None, niter=None, max_memory_MB=None, batch=1):
        """A decoder over a compressed checkpoint in the reference's layout on local disk
        (bitstack_amd/utils/checkpoint.py): `config.json` supplies the Llama dimensions
        (Hugging Face keys), `compression_config.json` + max_memory_MB pick the blocks per
        layer as the reference's --max_memory_MB does (bitstack/main.py:85-91), or pass a
        compression_config / niter directly.  Token ids in, token ids out: no tokenizer."""
        import json
        import os
        from bitstack_amd.utils import checkpoint as ck
        with open(os.path.join(path, "config.json"), "r") as f:
            hf = json.load(f)
        rope_par = hf.get("rope_parameters") or {}
        rope = hf.get("rope_theta") or rope_par.get("rope_theta", 10000.0)
        scaling = hf.get("rope_scaling") or (rope_par if rope_par.get("rope_type", "default") != "default" else None)
        rope_inv_freq(2, float(rope), scaling)              # raises here, before any weight is read, if unsupported
        shape = LlamaShape(rope_scaling=scaling, layers=hf["num_hidden_layers"], hidden=hf["hidden_size"], intermediate=hf["intermediate_size"],
                           heads=hf["num_attention_heads"], kv_heads=hf.get("num_key_value_heads", hf["num_attention_heads"]),
                           vocab=hf["vocab_size"], rope_theta=float(rope), rms_eps=float(hf.get("rms_norm_eps", 1e-5)))
        if hf.get("head_dim", shape.head_dim) != shape.head_dim:
            raise ValueError("head_dim other than hidden_size / num_attention_heads is not supported")
        if max_memory_MB is not None:
            compression_config = ck.retrieve_compression_config(ck.read_compression_configs(path), max_memory_MB)
        dev = torch.device(device)
        linears, other = ck.load_bitstack_checkpoint(path, compression_config=compression_config, niter=niter,
                                                     device=dev, fused_level=5)
        lin = [{p: linears[f"layer.{L}.{p}"] for p in PROJ} for L in range(shape.layers)]
        shape.k = lin[0][PROJ[0]].k
        f16 = lambda t: t.to(dev, torch.float16).contiguous()
        norm_w = torch.stack([torch.stack([f16(other[f"model.layers.{L}.input_layernorm.weight"]),
                                           f16(other[f"model.layers.{L}.post_attention_layernorm.weight"])])
                              for L in range(shape.layers)])
        embed = f16(other["model.embed_tokens.weight"])
        lm_head = f16(other["lm_head.weight"]) if "lm_head.weight" in other else embed      # tied embeddings
        self = cls.__new__(cls)
        self._setup(shape, lin, embed, lm_head, norm_w, f16(other["model.norm.weight"]), max_len, dev, batch)
        return self

    @classmethod
    def from_dense(cls, shape: LlamaShape, weights: dict, niter: int, max_len: int, device, k=16, batch=1):
        """Compress a dense Llama: every decoder linear becomes a BitStackLinear with `niter`
        residual blocks of rank `k`, decomposed on the device one linear at a time (what
        bitstack/utils/decompose.py:8-31 does to the Hugging Face model with
        BitStackLinear.from_linear; names layer.{L}.{proj} as there).  `weights` uses the
        Hugging Face keys: model.layers.{L}.{proj}.weight, the two layer norms per layer,
        model.embed_tokens.weight, model.norm.weight and lm_head.weight (optional: tied)."""
        import dataclasses
        dev = torch.device(device)
        shape = dataclasses.replace(shape, k=k)
        f16 = lambda t: torch.as_tensor(t).to(dev, torch.float16).contiguous()
        lin = []
        for L in range(shape.layers):
            row = {}
            for p in PROJ:
                w = torch.as_tensor(weights[f"model.layers.{L}.{p}.weight"]).to(dev, torch.float32)
                m, n = shape.proj_shape(p)
                if tuple(w.shape) != (m, n):
                    raise ValueError(f"model.layers.{L}.{p}.weight is {tuple(w.shape)}, expected {(m, n)}")
                dense = torch.nn.Linear(n, m, bias=False, device=dev, dtype=torch.float16)
                with torch.no_grad():
                    dense.weight.copy_(w)
                    mod = BitStackLinear.from_linear(dense, w_bit=niter, k=k, bias=False, fused_level=5, name=f"layer.{L}.{p}")
                mod.stack_blocks()
                row[p] = mod
                del dense, w
            lin.append(row)
        norm_w = torch.stack([torch.stack([f16(weights[f"model.layers.{L}.input_layernorm.weight"]),
                                           f16(weights[f"model.layers.{L}.post_attention_layernorm.weight"])])
                              for L in range(shape.layers)])
        embed = f16(weights["model.embed_tokens.weight"])
        lm_head = f16(weights["lm_head.weight"]) if "lm_head.weight" in weights else embed
        self = cls.__new__(cls)
        self._setup(shape, lin, embed, lm_head, norm_w, f16(weights["model.norm.weight"]), max_len, dev, batch)
        return self

    def save_checkpoint(self, path, compression_configs=None, max_shard_bytes=None):
        """Writes this decoder in the same layout (config.json included)."""
        import json
        import os
        from bitstack_amd.utils import checkpoint as ck
        s = self.s
        linears = {f"layer.{L}.{p}": self.lin[L][p] for L in range(s.layers) for p in PROJ}
        other = {"model.embed_tokens.weight": self.embed, "lm_head.weight": self.lm_head, "model.norm.weight": self.final_norm}
        for L in range(s.layers):
            other[f"model.layers.{L}.input_layernorm.weight"] = self.norm_w[L, 0]
            other[f"model.layers.{L}.post_attention_layernorm.weight"] = self.norm_w[L, 1]
        ck.save_bitstack_checkpoint(path, linears, other, compression_configs, max_shard_bytes)
        with open(os.path.join(path, "config.json"), "w") as f:
            json.dump({"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": s.layers,
                       "hidden_size": s.hidden, "intermediate_size": s.intermediate, "num_attention_heads": s.heads,
                       "num_key_value_heads": s.kv_heads, "vocab_size": s.vocab, "rope_theta": s.rope_theta,
                       "rms_norm_eps": s.rms_eps, "tie_word_embeddings": False}, f)

    def weight_bytes(self):
        b = self.embed.numel() * 2 + self.lm_head.numel() * 2
        for row in self.lin:
            for m in row.values():
                b += m.qweight.numel() + 2 * (m.u.numel() + m.vt.numel())
        return b

    def set_bits(self, bits):
        """Blocks in use per linear from now on: one count for all, or {"layer.{L}.{proj}": count}
        (BitStackLinear.set_bit on each; the grouped launches' argument blocks are rebuilt)."""
        for L, row in enumerate(self.lin):
            for p, m in row.items():
                b = bits if isinstance(bits, int) else bits[f"layer.{L}.{p}"]
                if not 1 <= b <= m.u.shape[0]:
                    raise ValueError(f"layer.{L}.{p}: {b} blocks asked, {m.u.shape[0]} loaded")
                m.set_bit(b)
        self._groups = None

    def set_memory_budget(self, path, max_memory_MB=None, compression_config=None):
        """Move the loaded decoder to another size of the same checkpoint while it runs: the
        config that fits max_memory_MB (bitstack/utils/model_utils.py:179-187) or the one given;
        linears that get fewer blocks free the surplus, those that get more read only the
        missing blocks from `path` (checkpoint.apply_compression_config).  The KV cache and
        the position stay as they are.  Returns (bytes_freed, bytes_loaded)."""
        from bitstack_amd.utils import checkpoint as ck
        if compression_config is None:
            compression_config = ck.retrieve_compression_config(ck.read_compression_configs(path), max_memory_MB)
        linears = {f"layer.{L}.{p}": m for L, row in enumerate(self.lin) for p, m in row.items()}
        moved = ck.apply_compression_config(path, linears, compression_config)
        self._groups = None
        return moved

    def reset(self):
        self.pos.zero_()
        self.kcache.zero_()
        self.vcache.zero_()

    def _rms(self, x, w):
        v = x.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.s.rms_eps)).half() * w

    def _rope(self, x, cos, sin):          # x [..., d], rotate-half convention
        d2 = x.shape[-1] // 2
        a, b = x[..., :d2], x[..., d2:]
        return torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)

    @torch.no_grad()
    def step(self):
        """Consume self.token at self.pos, write the greedy next token, advance."""
        s, B = self.s, self.batch
        x = self.embed.index_select(0, self.token)                       # [B, h]
        cos = self.cos.index_select(0, self.pos)
        sin = self.sin.index_select(0, self.pos)
        mask = (self.span <= self.pos).view(1, 1, 1, self.max_len)
        rep = s.heads // s.kv_heads
        for L in range(s.layers):
            lin = self.lin[L]
            hn = self._rms(x, self.norm_w[L, 0])
            q = lin["self_attn.q_proj"](hn).view(B, s.heads, s.head_dim)
            k = lin["self_attn.k_proj"](hn).view(B, s.kv_heads, s.head_dim)
            v = lin["self_attn.v_proj"](hn).view(B, s.kv_heads, s.head_dim)
            q, k = self._rope(q, cos, sin), self._rope(k, cos, sin)
            self.kcache[L].index_copy_(2, self.pos, k.unsqueeze(2))
            self.vcache[L].index_copy_(2, self.pos, v.unsqueeze(2))
            qg = q.view(B, s.kv_heads, rep, s.head_dim)
            att = torch.matmul(qg, self.kcache[L].transpose(2, 3)) / math.sqrt(s.head_dim)   # [B, kv, rep, max_len]
            att = att.masked_fill(~mask, float("-inf")).float().softmax(-1).half()
            ctx = torch.matmul(att, self.vcache[L]).reshape(B, s.hidden)
            x = x + lin["self_attn.o_proj"](ctx)
            hn = self._rms(x, self.norm_w[L, 1])
            gate = lin["mlp.gate_proj"](hn)
            up = lin["mlp.up_proj"](hn)
            x = x + lin["mlp.down_proj"](F.silu(gate) * up)
        self.logits = F.linear(self._rms(x, self.final_norm), self.lm_head)
        self.token.copy_(self.logits.argmax(-1))
        self.pos.add_(1)

    def _build_groups(self):
        """Argument blocks of the grouped launches.  The RMSNorm weight vectors in front of
        q/k/v and gate/up are folded into copies of those matrices' vt once
        (vt_i[r, n] * weight[n]); the scalar rsqrt(mean(x^2) + eps) is applied by the
        launch itself, so the fused step has no RMSNorm kernel inside a layer."""
        s, B = self.s, self.batch
        self._groups = []

        def folded(mods, weight):
            mats = []
            for m in mods:
                q, u, vt = m._stacked()
                mats.append((q, u, (vt.float() * weight.float().view(1, 1, -1)).half(), m.bias))
            return MatrixGroup(mats)

        for L in range(s.layers):
            lin = self.lin[L]
            self._groups.append({
                "qkv": folded([lin["self_attn.q_proj"], lin["self_attn.k_proj"], lin["self_attn.v_proj"]], self.norm_w[L, 0]),
                "o": MatrixGroup.from_modules([lin["self_attn.o_proj"]]),
                "gate_up": folded([lin["mlp.gate_proj"], lin["mlp.up_proj"]], self.norm_w[L, 1]),
                "down": MatrixGroup.from_modules([lin["mlp.down_proj"]]),
            })
        f16 = dict(dtype=torch.float16, device=self.dev)
        self._hn = torch.empty(B, s.hidden, **f16)
        self._qkv = torch.empty(B, (s.heads + 2 * s.kv_heads) * s.head_dim, **f16)
        self._ctx = torch.empty(B, s.hidden, **f16)
        self._act = torch.empty(B, s.intermediate, **f16)
        self._xa = torch.empty(B, s.hidden, **f16)
        self._xb = torch.empty(B, s.hidden, **f16)

    @torch.no_grad()
    def step_fused(self):
        """Same step on the library's grouped forwards and decode-step kernels."""
        if self._groups is None:
            self._build_groups()
        s = self.s
        xa, xb = self._xa, self._xb
        torch.index_select(self.embed, 0, self.token, out=xa)
        for L in range(s.layers):
            grp = self._groups[L]
            bitstack_forward_group_hip(grp["qkv"], xa, EPI_NONE, out=self._qkv, rms_eps=s.rms_eps)
            attention_decode_hip(self._qkv, self.kcache[L], self.vcache[L], self.cos, self.sin, self.pos,
                                 s.heads, s.kv_heads, out=self._ctx)
            bitstack_forward_group_hip(grp["o"], self._ctx, EPI_RESIDUAL, residual=xa, out=xb)
            bitstack_forward_group_hip(grp["gate_up"], xb, EPI_SWIGLU, out=self._act, rms_eps=s.rms_eps)
            bitstack_forward_group_hip(grp["down"], self._act, EPI_RESIDUAL, residual=xb, out=xa)
        rmsnorm_hip(xa, self.final_norm, s.rms_eps, out=self._hn)
        self.logits = F.linear(self._hn, self.lm_head)
        argmax_hip(self.logits, out=self.token)
        self.pos.add_(1)

    @torch.no_grad()
    def prefill(self, prompt: torch.Tensor, all_logits=False, first_layer=0, hidden=None, keep=None):
        """The whole prompt [batch, len] in one pass: every linear sees batch * len tokens (the
        library's rebuild + dense path), causal attention and RoPE are torch ops, the KV cache
        is filled for positions 0 .. len - 1, and self.token becomes the greedy token after
        the prompt.  Decode continues from there with step() or step_fused().  With
        all_logits the logits of every position [batch, len, vocab] are returned (perplexity).
        `keep` (a list) receives the input of every decoder layer; `first_layer` with `hidden`
        (such a kept input) resumes from that layer - what a change confined to one layer needs
        to be evaluated (the KV cache of the earlier layers is then left as it is)."""
        s, B = self.s, self.batch
        prompt = prompt.view(1, -1).expand(B, -1) if prompt.dim() == 1 else prompt
        n = prompt.shape[1]
        if n < 1 or n > self.max_len:
            raise ValueError("prompt length must be in 1..max_len")
        d = s.head_dim
        if first_layer == 0:
            x = self.embed.index_select(0, prompt.reshape(-1))            # [B * n, h]
        else:
            if hidden is None or tuple(hidden.shape) != (B * n, s.hidden):
                raise ValueError("resuming needs the kept input of that layer")
            x = hidden
        cos, sin = self.cos[:n].view(1, 1, n, d // 2), self.sin[:n].view(1, 1, n, d // 2)
        for L in range(first_layer, s.layers):
            if keep is not None:
                keep.append(x)
            lin = self.lin[L]
            hn = rmsnorm_hip(x, self.norm_w[L, 0], s.rms_eps)
            q = lin["self_attn.q_proj"](hn).view(B, n, s.heads, d).transpose(1, 2)
            k = lin["self_attn.k_proj"](hn).view(B, n, s.kv_heads, d).transpose(1, 2)
            v = lin["self_attn.v_proj"](hn).view(B, n, s.kv_heads, d).transpose(1, 2)
            q, k = self._rope(q, cos, sin), self._rope(k, cos, sin)
            self.kcache[L][:, :, :n].copy_(k)
            self.vcache[L][:, :, :n].copy_(v)
            ctx = torch.empty(B, n, s.hidden, dtype=torch.float16, device=self.dev)
            for b in range(B):                                            # one sequence at a time bounds the scratch
                o = F.scaled_dot_product_attention(q[b:b + 1], k[b:b + 1], v[b:b + 1], is_causal=True, enable_gqa=True)
                ctx[b].copy_(o[0].transpose(0, 1).reshape(n, s.hidden))
            x = x + lin["self_attn.o_proj"](ctx.view(B * n, s.hidden))
            hn = rmsnorm_hip(x, self.norm_w[L, 1], s.rms_eps)
            act = F.silu(lin["mlp.gate_proj"](hn))
            act.mul_(lin["mlp.up_proj"](hn))
            x = x + lin["mlp.down_proj"](act)
        if all_logits:
            full = F.linear(rmsnorm_hip(x, self.final_norm, s.rms_eps), self.lm_head).view(B, n, -1)
            self.logits = full[:, -1].contiguous()
        else:
            last = x.view(B, n, s.hidden)[:, -1].contiguous()
            self.logits = F.linear(rmsnorm_hip(last, self.final_norm, s.rms_eps), self.lm_head)
        self.token.copy_(self.logits.argmax(-1))
        self.pos.fill_(n)
        return full if all_logits else None

    def prefill_positions(self, prompt: torch.Tensor, fused=False):
        """Feed a prompt token by token (the measurement is about decode).  `prompt`
        is [len] (the same for every sequence) or [batch, len]."""
        self.pos.zero_()
        prompt = prompt.view(1, -1).expand(self.batch, -1) if prompt.dim() == 1 else prompt
        for j in range(prompt.shape[1]):
            self.token.copy_(prompt[:, j])
            (self.step_fused if fused else self.step)()
