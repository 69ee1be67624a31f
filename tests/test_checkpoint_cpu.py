"""Checkpoint reader for the reference's on-disk layout (bitstack/utils/model_utils.py:189-205,
bitstack/utils/decompose.py:8-21): files written here with safetensors directly, read back
through the loader, compared tensor by tensor and through a level-0 forward against the oracle."""
import json
import os

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from bitstack_amd.utils import checkpoint as ck
from oracle import bitstack_oracle as bo

PROJ = {"self_attn.q_proj": (32, 32), "self_attn.k_proj": (16, 32), "mlp.down_proj": (32, 64)}


def _write(tmp_path, blocks=3, shards=1, bias_on=("self_attn.q_proj",)):
    g = torch.Generator().manual_seed(5)
    tensors = {}
    for L in range(2):
        for name, (m, n) in PROJ.items():
            for i in range(blocks):
                base = f"model.layers.{L}.{name}"
                tensors[f"{base}.qweight_{i}"] = torch.randint(0, 256, (m * n // 8,), dtype=torch.uint8, generator=g)
                tensors[f"{base}.u_{i}"] = (torch.randn(m, 4, generator=g) * 0.1).half()
                tensors[f"{base}.vt_{i}"] = (torch.randn(4, n, generator=g) * 0.1).half()
            if name in bias_on:
                tensors[f"model.layers.{L}.{name}.bias"] = torch.randn(m, generator=g).half()
        tensors[f"model.layers.{L}.input_layernorm.weight"] = torch.ones(32).half()
    tensors["model.embed_tokens.weight"] = torch.randn(10, 32, generator=g).half()
    tensors["lm_head.weight"] = torch.randn(10, 32, generator=g).half()
    keys = sorted(tensors)
    if shards == 1:
        save_file(tensors, str(tmp_path / "model.safetensors"))
    else:
        wmap = {}
        for j in range(shards):
            part = {k: tensors[k] for k in keys[j::shards]}
            fname = f"model-{j + 1:05d}-of-{shards:05d}.safetensors"
            save_file(part, str(tmp_path / fname))
            wmap.update({k: fname for k in part})
        (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": wmap}))
    return tensors


@pytest.mark.parametrize("shards", [1, 3])
def test_stacked_load_keeps_only_the_configured_blocks(tmp_path, shards):
    tensors = _write(tmp_path, blocks=3, shards=shards)
    config = {f"layer.{L}.{name}": 1 + (L + j) % 3 for L in range(2) for j, name in enumerate(PROJ)}
    linears, other = ck.load_bitstack_checkpoint(str(tmp_path), compression_config=config, device="cpu")
    assert set(linears) == set(config)
    for lname, mod in linears.items():
        _, L, name = lname.split(".", 2)
        m, n = PROJ[name]
        want = config[lname]
        assert (mod.w_bit, mod.out_features, mod.in_features, mod.k, mod.name) == (want, m, n, 4, lname)
        assert mod.qweight.shape == (want, m * n // 8) and mod.u.shape == (want, m, 4) and mod.vt.shape == (want, 4, n)
        for i in range(want):
            base = f"model.layers.{L}.{name}"
            assert torch.equal(mod.qweight[i], tensors[f"{base}.qweight_{i}"])
            assert torch.equal(mod.u[i], tensors[f"{base}.u_{i}"])
            assert torch.equal(mod.vt[i], tensors[f"{base}.vt_{i}"])
        if name == "self_attn.q_proj":
            assert torch.equal(mod.bias, tensors[f"model.layers.{L}.{name}.bias"])
        else:
            assert mod.bias is None
        assert mod.memory_per_bit() == bo.memory_per_bit(m, n, 4)
    # the dense rest comes back untouched, block tensors and biases do not
    assert set(other) == {"model.embed_tokens.weight", "lm_head.weight",
                          "model.layers.0.input_layernorm.weight", "model.layers.1.input_layernorm.weight"}
    assert torch.equal(other["lm_head.weight"], tensors["lm_head.weight"])


def test_unstacked_level0_forward_matches_oracle(tmp_path):
    tensors = _write(tmp_path, blocks=2)
    linears, _ = ck.load_bitstack_checkpoint(str(tmp_path), niter=2, device="cpu", fused_level=0, stack=False, dense=False)
    mod = linears["layer.1.mlp.down_proj"]
    x = torch.randn(3, 64, generator=torch.Generator().manual_seed(1)).half()
    y = mod(x).float().numpy()
    base = "model.layers.1.mlp.down_proj"
    packed = np.stack([tensors[f"{base}.qweight_{i}"].numpy() for i in range(2)])
    u = np.stack([tensors[f"{base}.u_{i}"].numpy() for i in range(2)])
    vt = np.stack([tensors[f"{base}.vt_{i}"].numpy() for i in range(2)])
    ref = bo.forward_exact(packed, u, vt, x.numpy(), None)
    assert np.abs(y - ref).max() <= 1e-2 * max(np.abs(ref).max(), 1e-6)


def test_errors(tmp_path):
    _write(tmp_path, blocks=2)
    with pytest.raises(ValueError):
        ck.load_bitstack_checkpoint(str(tmp_path), device="cpu")
    with pytest.raises(KeyError):          # asks for a block the checkpoint does not hold
        ck.load_bitstack_checkpoint(str(tmp_path), niter=3, device="cpu")
    with pytest.raises(FileNotFoundError):
        ck.load_bitstack_checkpoint(str(tmp_path / "nowhere"), niter=1, device="cpu")


def test_compression_config_file_and_retrieval(tmp_path):
    configs = [{"memory": 3 * 1024 ** 2, "layers": {"layer.0.a": 1}},
               {"memory": 5 * 1024 ** 2, "layers": {"layer.0.a": 2}},
               {"memory": 9 * 1024 ** 2, "layers": {"layer.0.a": 3}}]
    (tmp_path / "compression_config.json").write_text(json.dumps(configs))
    read = ck.read_compression_configs(str(tmp_path))
    assert ck.retrieve_compression_config(read, 5) == {"layer.0.a": 2}       # exact fit counts
    assert ck.retrieve_compression_config(read, 8) == {"layer.0.a": 2}
    assert ck.retrieve_compression_config(read, 100) == {"layer.0.a": 3}
    with pytest.raises(ValueError):
        ck.retrieve_compression_config(read, 2)
    # same answers as the oracle's restatement on a shuffled list
    assert ck.retrieve_compression_config(read[::-1], 8) == bo.retrieve_compression_config(read, 8)


@pytest.mark.parametrize("max_shard_bytes", [None, 4096])
def test_save_then_load_round_trip(tmp_path, max_shard_bytes):
    _write(tmp_path, blocks=3)
    linears, other = ck.load_bitstack_checkpoint(str(tmp_path), niter=3, device="cpu")
    out = tmp_path / "copy"
    ck.save_bitstack_checkpoint(str(out), linears, other, compression_configs=[{"memory": 1, "layers": {}}],
                                max_shard_bytes=max_shard_bytes)
    if max_shard_bytes is not None:
        assert os.path.exists(out / "model.safetensors.index.json")
    again, other2 = ck.load_bitstack_checkpoint(str(out), niter=3, device="cpu")
    assert set(again) == set(linears) and set(other2) == set(other)
    for k in linears:
        for attr in ("qweight", "u", "vt"):
            assert torch.equal(getattr(again[k], attr), getattr(linears[k], attr))
        assert (again[k].bias is None) == (linears[k].bias is None)
    assert ck.read_compression_configs(str(out)) == [{"memory": 1, "layers": {}}]


def test_blocks_really_come_and_go(tmp_path):
    tensors = _write(tmp_path, blocks=3, shards=3)
    names = [f"layer.{L}.{n}" for L in range(2) for n in PROJ]
    linears, _ = ck.load_bitstack_checkpoint(str(tmp_path), niter=2, device="cpu", fused_level=5, dense=False)
    x = {n: torch.randn(2, linears[n].in_features, generator=torch.Generator().manual_seed(3)).half() for n in names}

    def dense_out(name, blocks):
        _, L, proj = name.split(".", 2)
        base = f"model.layers.{L}.{proj}"
        packed = np.stack([tensors[f"{base}.qweight_{i}"].numpy() for i in range(blocks)])
        u = np.stack([tensors[f"{base}.u_{i}"].numpy() for i in range(blocks)])
        vt = np.stack([tensors[f"{base}.vt_{i}"].numpy() for i in range(blocks)])
        bias = tensors.get(f"{base}.bias")
        return bo.forward_exact(packed, u, vt, x[name].numpy(), None if bias is None else bias.numpy())

    # down to one block in some layers, up to three in others
    cfg = {n: (1 if j % 2 else 3) for j, n in enumerate(names)}
    freed, loaded = ck.apply_compression_config(str(tmp_path), linears, cfg)
    assert freed == sum(linears[n].memory_per_bit() for n in names if cfg[n] == 1)
    assert loaded == sum(linears[n].memory_per_bit() for n in names if cfg[n] == 3)
    for n in names:
        mod = linears[n]
        assert mod.w_bit == cfg[n] and mod.u.shape[0] == cfg[n] and mod.qweight.shape[0] == cfg[n] and mod.vt.shape[0] == cfg[n]
        _, L, proj = n.split(".", 2)
        for i in range(cfg[n]):
            assert torch.equal(mod.qweight[i], tensors[f"model.layers.{L}.{proj}.qweight_{i}"])
            assert torch.equal(mod.u[i], tensors[f"model.layers.{L}.{proj}.u_{i}"])
    # a counter-only change (the reference's set_bit) followed by growth: surplus is dropped first
    m = linears[names[0]]
    m.set_bit(1)
    assert m.u.shape[0] == 3
    ck.apply_compression_config(str(tmp_path), linears, {**cfg, names[0]: 2})
    assert m.w_bit == 2 and m.u.shape[0] == 2 and torch.equal(m.vt[1], tensors["model.layers.0.self_attn.q_proj.vt_1"])
    with pytest.raises(KeyError):
        ck.apply_compression_config(str(tmp_path), linears, {**cfg, names[0]: 4})
    with pytest.raises(RuntimeError):
        m.set_bit(1)
        m.append_blocks(m.qweight[:1], m.u[:1], m.vt[:1])
    # values: the level-0 forward needs per-block buffers, so compare through the stacked tensors
    for n in names[:2]:
        mod = linears[n]
        mod.set_bit(mod.u.shape[0])
        w = sum(bo.compose_weight(mod.qweight[i].numpy(), mod.u[i].numpy().astype(np.float32), mod.vt[i].numpy().astype(np.float32),
                                  weight_shape=(mod.out_features, mod.in_features)) for i in range(mod.w_bit))
        y = x[n].numpy().astype(np.float64) @ w.astype(np.float64).T + (0 if mod.bias is None else mod.bias.numpy().astype(np.float64))
        ref = dense_out(n, mod.w_bit)
        assert np.abs(y - ref).max() <= 1e-3 * max(np.abs(ref).max(), 1e-6)
