"""Read (and, for tests and tools, write) compressed checkpoints in the reference's
on-disk layout, from a local directory, without transformers or accelerate.

Layout (what the reference's save produces and `load_bitstack_model_and_tokenizer`
consumes, bitstack/utils/model_utils.py:189-205 with bitstack/utils/decompose.py:8-21):
  * safetensors, one file (`model.safetensors`) or shards listed in
    `model.safetensors.index.json` ({"weight_map": {key: file}});
  * every decoder linear `model.layers.{L}.{self_attn|mlp}.{proj}` holds per-block
    buffers `qweight_{i}` uint8[M*N/8], `u_{i}` f16[M,k], `vt_{i}` f16[k,N]
    (bitstack/modules/BitStackLinear.py:37-46) and optionally `bias`;
  * everything else (embed_tokens, norms, lm_head) is dense;
  * `compression_config.json` next to it: a list of {"memory": bytes, "layers":
    {"layer.{L}.{self_attn|mlp}.{proj}": n_blocks}} (bitstack/main.py:88-90,
    bitstack/utils/model_utils.py:54-66).
Only blocks `i < compression_config[layer]` are read (decompose.py:15-21 creates
just those buffers and the checkpoint loader skips the rest), and they are copied
straight into the stacked `[I, ...]` buffers stack_blocks() would build
(BitStackLinear.py:183-195), so peak memory is one copy of the kept blocks.
"""
from __future__ import annotations

import json
import os
import re
from collections import defaultdict

import torch
from safetensors import safe_open
from safetensors.torch import save_file

from bitstack_amd.modules.BitStackLinear import BitStackLinear

_BLOCK_KEY = re.compile(r"^(?P<prefix>.*\.)?layers\.(?P<layer>\d+)\.(?P<name>.+)\.(?P<kind>qweight|u|vt)_(?P<i>\d+)$")
_INDEX = "model.safetensors.index.json"
_SINGLE = "model.safetensors"


def retrieve_compression_config(configs, max_memory_MB):
    """Largest config that fits (bitstack/utils/model_utils.py:179-187)."""
    max_memory = max_memory_MB * 1024 ** 2
    for config in sorted(configs, key=lambda c: c["memory"], reverse=True):
        if config["memory"] <= max_memory:
            return config["layers"]
    raise ValueError(f"No config found within the memory limit {max_memory_MB} MB")


def read_compression_configs(path):
    with open(os.path.join(path, "compression_config.json"), "r") as f:
        return json.load(f)


def _weight_map(path):
    """key -> file name, for a sharded or a single-file checkpoint."""
    index = os.path.join(path, _INDEX)
    if os.path.exists(index):
        with open(index, "r") as f:
            return dict(json.load(f)["weight_map"])
    single = os.path.join(path, _SINGLE)
    if not os.path.exists(single):
        raise FileNotFoundError(f"neither {_INDEX} nor {_SINGLE} in {path}")
    with safe_open(single, framework="pt") as f:
        return {k: _SINGLE for k in f.keys()}


class _Shards:
    """Keeps each safetensors file open once while tensors are pulled out of it."""

    def __init__(self, path, weight_map):
        self.path, self.map, self.open = path, weight_map, {}

    def get(self, key):
        name = self.map[key]
        if name not in self.open:
            self.open[name] = safe_open(os.path.join(self.path, name), framework="pt")
            self.open[name].__enter__()
        return self.open[name].get_tensor(key)

    def close(self):
        for f in self.open.values():
            f.__exit__(None, None, None)
        self.open = {}


def load_bitstack_checkpoint(path, compression_config=None, niter=None, device="cuda", fused_level=5,
                             stack=True, dense=True):
    """Returns (linears, other): `linears` maps "layer.{L}.{name}" (the keys of a
    compression config, decompose.py:14) to a BitStackLinear holding the first
    `compression_config[key]` blocks (or `niter` blocks for every layer when no
    config is given; one of the two is required, model_utils.py:197); `other`
    maps the remaining checkpoint keys to tensors on `device` (skipped with
    dense=False).  With stack=True the modules come back in the stacked layout
    every fused level needs; stack=False keeps the per-block buffers (level 0)."""
    if compression_config is None and niter is None:
        raise ValueError("either compression_config or niter is required")
    wmap = _weight_map(path)
    # group the block keys by linear
    blocks = defaultdict(lambda: {"qweight": {}, "u": {}, "vt": {}})
    full_prefix = {}
    for key in wmap:
        m = _BLOCK_KEY.match(key)
        if m:
            lname = f"layer.{m['layer']}.{m['name']}"
            blocks[lname][m["kind"]][int(m["i"])] = key
            full_prefix[lname] = key[: key.rfind(".")]
    shards = _Shards(path, wmap)
    dev = torch.device(device)
    linears, used = {}, set()
    try:
        for lname in sorted(blocks, key=lambda s: (int(s.split(".")[1]), s)):
            have = blocks[lname]
            want = compression_config[lname] if compression_config is not None else niter
            if want < 1:
                raise ValueError(f"{lname}: at least one block is needed, got {want}")
            missing = [f"{kind}_{i}" for i in range(want) for kind in ("u", "vt") if i not in have[kind]]
            no_avd = len(have["qweight"]) == 0
            if not no_avd:
                missing += [f"qweight_{i}" for i in range(want) if i not in have["qweight"]]
            if missing:
                raise KeyError(f"{lname}: checkpoint lacks {missing[:4]}{'...' if len(missing) > 4 else ''}")
            u0 = shards.get(have["u"][0])
            vt0 = shards.get(have["vt"][0])
            m_out, k = u0.shape
            n_in = vt0.shape[1]
            bias_key = full_prefix[lname] + ".bias"
            mod = BitStackLinear(0, n_in, m_out, k, False, False, dev, fused_level=fused_level)
            mod.k, mod.no_avd, mod.name, mod.w_bit = k, no_avd, lname, want
            if bias_key in wmap:
                mod.bias = shards.get(bias_key).to(dev, torch.float16)
                used.add(bias_key)
            if stack:
                u = torch.empty((want, m_out, k), dtype=torch.float16, device=dev)
                vt = torch.empty((want, k, n_in), dtype=torch.float16, device=dev)
                q = None if no_avd else torch.empty((want, m_out * n_in // 8), dtype=torch.uint8, device=dev)
                for i in range(want):
                    u[i].copy_(u0 if i == 0 else shards.get(have["u"][i]))
                    vt[i].copy_(vt0 if i == 0 else shards.get(have["vt"][i]))
                    if q is not None:
                        q[i].copy_(shards.get(have["qweight"][i]))
                mod.u, mod.vt = u, vt          # plain attributes, as stack_blocks() leaves them
                if q is not None:
                    mod.qweight = q
            else:
                for i in range(want):
                    mod.register_buffer(f"u_{i}", (u0 if i == 0 else shards.get(have["u"][i])).to(dev))
                    mod.register_buffer(f"vt_{i}", (vt0 if i == 0 else shards.get(have["vt"][i])).to(dev))
                    if not no_avd:
                        mod.register_buffer(f"qweight_{i}", shards.get(have["qweight"][i]).to(dev))
            for kind in ("qweight", "u", "vt"):
                used.update(have[kind].values())          # blocks beyond `want` are deliberately left on disk
            linears[lname] = mod
        other = {}
        if dense:
            for key in wmap:
                if key not in used:
                    other[key] = shards.get(key).to(dev)
    finally:
        shards.close()
    return linears, other


def apply_compression_config(path, linears, compression_config):
    """Move already loaded modules (stacked layout) to another compression config of
    the same checkpoint: layers that get fewer blocks drop and free the surplus,
    layers that get more read just the missing blocks from disk.  What the
    reference's set_model_bits (model_utils.py:11-17) does with a counter, done
    with memory.  Returns (bytes_freed, bytes_loaded)."""
    wmap = _weight_map(path)
    shards = _Shards(path, wmap)
    freed = loaded = 0
    try:
        for lname, mod in linears.items():
            want = compression_config[lname]
            if want < 1:
                raise ValueError(f"{lname}: at least one block is needed, got {want}")
            have = mod.w_bit
            if want < have:
                mod.set_bit(want)
                freed += (have - want) * mod.memory_per_bit()
                mod.trim_blocks()
            elif want > have:
                if mod.u.shape[0] > have:          # surplus blocks still stacked from an earlier set_bit
                    mod.trim_blocks()
                _, layer, name = lname.split(".", 2)
                base = next((k[: k.rfind(".")] for k in wmap
                             if _BLOCK_KEY.match(k) and k.endswith(f"layers.{layer}.{name}.u_0")), None)
                if base is None:
                    raise KeyError(f"{lname} is not in the checkpoint")
                idx = range(have, want)
                missing = [f"{base}.{kind}_{i}" for i in idx for kind in ("u", "vt") if f"{base}.{kind}_{i}" not in wmap]
                if missing:
                    raise KeyError(f"{lname}: checkpoint lacks {missing[:4]}")
                u = torch.stack([shards.get(f"{base}.u_{i}") for i in idx])
                vt = torch.stack([shards.get(f"{base}.vt_{i}") for i in idx])
                q = None if mod.no_avd else torch.stack([shards.get(f"{base}.qweight_{i}") for i in idx])
                mod.append_blocks(q, u, vt)
                loaded += (want - have) * mod.memory_per_bit()
    finally:
        shards.close()
    return freed, loaded


def save_bitstack_checkpoint(path, linears, other=None, compression_configs=None, max_shard_bytes=None,
                             key_prefix="model.layers."):
    """Writes `linears` ({"layer.{L}.{name}": BitStackLinear}, stacked or not) and
    the dense tensors `other` in the layout described at the top.  Sharded when
    `max_shard_bytes` is given."""
    os.makedirs(path, exist_ok=True)
    tensors = {}
    for lname, mod in linears.items():
        _, layer, name = lname.split(".", 2)
        base = f"{key_prefix}{layer}.{name}"
        stacked = hasattr(mod, "u") and isinstance(getattr(mod, "u"), torch.Tensor)
        n_blocks = mod.u.shape[0] if stacked else mod.w_bit
        for i in range(n_blocks):
            tensors[f"{base}.u_{i}"] = (mod.u[i] if stacked else getattr(mod, f"u_{i}")).detach().cpu().contiguous()
            tensors[f"{base}.vt_{i}"] = (mod.vt[i] if stacked else getattr(mod, f"vt_{i}")).detach().cpu().contiguous()
            if not mod.no_avd:
                q = mod.qweight[i] if stacked else getattr(mod, f"qweight_{i}")
                tensors[f"{base}.qweight_{i}"] = q.detach().cpu().contiguous()
        if mod.bias is not None:
            tensors[f"{base}.bias"] = mod.bias.detach().cpu().contiguous()
    for key, t in (other or {}).items():
        tensors[key] = t.detach().cpu().contiguous()
    if max_shard_bytes is None:
        save_file(tensors, os.path.join(path, _SINGLE), metadata={"format": "pt"})
    else:
        shards, cur, size = [], {}, 0
        for key in sorted(tensors):
            b = tensors[key].numel() * tensors[key].element_size()
            if cur and size + b > max_shard_bytes:
                shards.append(cur)
                cur, size = {}, 0
            cur[key] = tensors[key]
            size += b
        shards.append(cur)
        wmap = {}
        for j, shard in enumerate(shards):
            fname = f"model-{j + 1:05d}-of-{len(shards):05d}.safetensors"
            save_file(shard, os.path.join(path, fname), metadata={"format": "pt"})
            wmap.update({k: fname for k in shard})
        with open(os.path.join(path, _INDEX), "w") as f:
            json.dump({"metadata": {}, "weight_map": wmap}, f)
    if compression_configs is not None:
        with open(os.path.join(path, "compression_config.json"), "w") as f:
            json.dump(compression_configs, f)
