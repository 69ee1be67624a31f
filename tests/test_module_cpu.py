"""Host-side logic of the module that needs no GPU: buffers, level 0 against
the oracle, bookkeeping, stack_blocks, error behaviour."""
import numpy as np
import pytest
import torch

from bitstack_amd import BitStackLinear, compose_weight, pack_sign, unpack_sign
from bitstack_amd.utils.synthetic import synthetic_layer, algorithmic_bytes
from oracle import bitstack_oracle as O


def make_module(M, N, I, k=16, bias=False, seed=0, fused_level=0):
    q, u, vt, x = synthetic_layer(M, N, I, 3, k=k, seed=seed, signed_factors=True)
    mod = BitStackLinear(w_bit=I, in_features=N, out_features=M, k=k, bias=bias, no_avd=False,
                         dev="cpu", fused_level=fused_level)
    for i in range(I):
        getattr(mod, f"qweight_{i}").copy_(q[i])
        getattr(mod, f"u_{i}").copy_(u[i] * 30)
        getattr(mod, f"vt_{i}").copy_(vt[i] * 30)
    if bias:
        mod.bias.copy_(torch.randn(M).half())
    return mod, x


def test_buffers_match_reference_layout():
    mod, _ = make_module(32, 64, 3, k=4, bias=True)
    sd = mod.state_dict()
    assert sorted(sd) == sorted([f"{n}_{i}" for i in range(3) for n in ("qweight", "u", "vt")] + ["bias"])
    assert sd["qweight_0"].dtype == torch.uint8 and tuple(sd["qweight_0"].shape) == (32 * 64 // 8,)
    assert sd["u_1"].dtype == torch.float16 and tuple(sd["u_1"].shape) == (32, 4)
    assert sd["vt_2"].dtype == torch.float16 and tuple(sd["vt_2"].shape) == (4, 64)
    assert mod.memory_per_bit() == O.memory_per_bit(32, 64, 4)
    nob = BitStackLinear(2, 64, 32, 4, False, False, "cpu")
    assert nob.bias is None


def test_pack_unpack_torch_path_matches_oracle():
    rng = np.random.default_rng(0)
    s = (rng.integers(0, 2, size=(7, 24)) * 2 - 1).astype(np.int8)
    p = pack_sign(torch.from_numpy(s))
    assert p.dtype == torch.uint8
    assert np.array_equal(p.numpy(), O.pack_sign(s))
    back = unpack_sign(p, torch.Size((7, 24)))
    assert back.dtype == torch.int8 and np.array_equal(back.numpy(), s)


def test_level0_matches_oracle_l0():
    mod, x = make_module(48, 128, 4, bias=True, seed=3)
    y = mod(x)
    q = np.stack([getattr(mod, f"qweight_{i}").numpy() for i in range(4)])
    u = np.stack([getattr(mod, f"u_{i}").numpy() for i in range(4)])
    vt = np.stack([getattr(mod, f"vt_{i}").numpy() for i in range(4)])
    want = O.forward_l0(q, u, vt, x.numpy(), mod.bias.numpy())
    got = y.numpy().astype(np.float64)
    # same rounding order; only the accumulation order inside the two matmuls may differ
    assert np.abs(got - want.astype(np.float64)).max() <= 2e-3 * np.abs(want.astype(np.float64)).max()
    exact = O.forward_exact(q, u, vt, x.numpy(), mod.bias.numpy())
    assert np.abs(got - exact).max() / np.abs(exact).max() < 1e-2


def test_level0_keeps_leading_dims_and_honours_w_bit():
    mod, x = make_module(16, 64, 3, seed=1)
    y3 = mod(x.view(1, 3, 64))
    assert tuple(y3.shape) == (1, 3, 16)
    full = mod(x)
    mod.pop_one_bit()
    assert mod.w_bit == 2
    two = mod(x)
    mod.add_one_bit()
    assert torch.equal(mod(x), full) and not torch.equal(two, full)
    mod.set_bit(1)
    q0 = getattr(mod, "qweight_0")
    w0 = compose_weight(q0, mod.u_0, mod.vt_0, False, torch.Size((16, 64)))
    assert torch.allclose(mod(x).float(), x.float() @ w0.float().T, atol=2e-3, rtol=2e-3)


def test_invalid_level_and_unstacked_errors():
    mod, x = make_module(16, 64, 2)
    mod.fused_level = 9
    with pytest.raises(ValueError, match="Invalid fused_level: 9"):
        mod(x)
    mod.fused_level = 3
    with pytest.raises(RuntimeError, match="stack_blocks"):
        mod(x)
    mod.stack_blocks()
    with pytest.raises(RuntimeError, match="HIP device"):      # CPU tensors: no silent fallback
        mod(x)


def test_stack_blocks_layout_and_memory():
    mod, _ = make_module(16, 64, 3)
    q1 = mod.qweight_1.clone()
    mod.fused_level = 1
    mod.stack_blocks()
    assert tuple(mod.qweight.shape) == (3, 16 * 64 // 8) and mod.qweight.is_contiguous()
    assert tuple(mod.u.shape) == (3, 16, 16) and tuple(mod.vt.shape) == (3, 16, 64)
    assert torch.equal(mod.qweight[1], q1)
    assert not hasattr(mod, "qweight_0") and not hasattr(mod, "u_2")
    assert mod.memory_per_bit() == O.memory_per_bit(16, 64, 16)


def test_from_linear_decompose_matches_oracle_decomposition():
    torch.manual_seed(0)
    lin = torch.nn.Linear(64, 48, bias=True)
    with torch.no_grad():
        lin.weight.mul_(0.2)
    with torch.no_grad():      # the reference's model walker runs under no_grad (decompose.py:7)
        mod = BitStackLinear.from_linear(lin, w_bit=3, k=4, bias=True, name="layer.0.mlp.up_proj")
    assert mod.name == "layer.0.mlp.up_proj" and mod.bias is lin.bias
    W = lin.weight.detach().numpy()
    q, u, vt, norms = O.decompose_weight(W, 3, 4)
    for i in range(3):
        # signs are identical; factors are pinned through their product (joint sign freedom)
        assert np.array_equal(getattr(mod, f"qweight_{i}").numpy(), q[i]), i
        got = getattr(mod, f"u_{i}").float().numpy() @ getattr(mod, f"vt_{i}").float().numpy()
        want = u[i].astype(np.float32) @ vt[i].astype(np.float32)
        assert np.abs(got - want).max() < 5e-3 * np.abs(want).max() + 1e-5
    shell = BitStackLinear.from_linear(lin, w_bit=2, k=4, bias=False, init_only=True)
    assert shell.w_bit == 2 and float(shell.u_0.abs().sum()) == 0.0


def test_no_avd_level0_and_rank():
    m = BitStackLinear(2, 64, 32, 4, False, True, "cpu")
    assert m.k == (64 * 32) // (16 * (64 + 32)) + 4
    assert not hasattr(m, "qweight_0")
    torch.manual_seed(1)
    m.u_0.copy_(torch.randn(32, m.k).half() * 0.1)
    m.vt_0.copy_(torch.randn(m.k, 64).half() * 0.1)
    x = torch.randn(2, 64).half()
    want = x.float() @ (m.u_0.float() @ m.vt_0.float()).T
    assert torch.allclose(m(x).float(), want, atol=5e-3, rtol=5e-3)


def test_algorithmic_bytes_closed_form():
    assert algorithmic_bytes(1, 4096, 4096, 1) == 2_097_152 + 262_144 + 16_384
    assert round(algorithmic_bytes(8, 4096, 4096, 1) / 1e6, 3) == 18.891
    assert round(algorithmic_bytes(16, 4096, 14336, 1) / 1e6, 3) == 126.915


def test_unpack_sign_v2_is_the_same_mapping_with_a_dtype_check():
    from bitstack_amd.utils.pack_utils import unpack_sign_v2
    rng = np.random.default_rng(3)
    packed = torch.from_numpy(rng.integers(0, 256, size=13, dtype=np.uint8))
    for shape in [(100,), (4, 26), (13, 8)]:
        got = unpack_sign_v2(packed, torch.Size(shape)).numpy()
        want = np.unpackbits(packed.numpy(), bitorder="big")[: int(np.prod(shape))].astype(np.int8).reshape(shape) * 2 - 1
        assert np.array_equal(got, want)
    with pytest.raises(ValueError):
        unpack_sign_v2(packed.to(torch.int16), torch.Size((8,)))


# ------------------------------------------------------------------ importance scores -> configs
def test_sort_layers_and_generate_configs():
    """Hand-checked: within a bit level the linear with the lowest perplexity comes first,
    levels follow one another, a NaN borrows the next level's value plus the level's maximum
    (model_utils.py:26-66)."""
    from bitstack_amd.utils import scoring as S
    data = {"original_ppl": 9.0, "reduced_ppl": [
        {"bit": 1, "ppls": [{"layer": "a", "ppl": 7.0}, {"layer": "b", "ppl": 5.0}, {"layer": "c", "ppl": 6.0}]},
        {"bit": 2, "ppls": [{"layer": "a", "ppl": 4.0}, {"layer": "b", "ppl": 4.5}, {"layer": "c", "ppl": 3.0}]}]}
    assert S.sort_layers_and_bits_average(data) == ["b", "c", "a", "c", "a", "b"]
    per_bit = {"a": 10, "b": 20, "c": 30}
    cfgs = S.generate_configs(["b", "c", "a", "c", "a", "b"], per_bit, 100)
    assert [c["memory"] for c in cfgs] == [100, 120, 150, 160, 190, 200, 220]
    assert cfgs[0]["layers"] == {"a": 1, "b": 1, "c": 1} and cfgs[-1]["layers"] == {"a": 3, "b": 3, "c": 3}
    assert cfgs[2]["layers"] == {"a": 1, "b": 2, "c": 2}
    # a NaN at level 1 sorts by the next level's perplexity, after every finite entry
    nan = {"reduced_ppl": [
        {"bit": 1, "ppls": [{"layer": "a", "ppl": float("nan")}, {"layer": "b", "ppl": 5.0}, {"layer": "c", "ppl": float("nan")}]},
        {"bit": 2, "ppls": [{"layer": "a", "ppl": 4.0}, {"layer": "b", "ppl": 4.5}, {"layer": "c", "ppl": 3.0}]}]}
    assert S.sort_layers_and_bits_average(nan)[:3] == ["c", "a", "b"]      # 3.0 + 0, 4.0 + 0, 5.0 (the reference's NaN-poisoned max is 0)
    nan2 = {"reduced_ppl": [
        {"bit": 1, "ppls": [{"layer": "a", "ppl": 6.0}, {"layer": "b", "ppl": float("nan")}, {"layer": "c", "ppl": 5.0}]},
        {"bit": 2, "ppls": [{"layer": "a", "ppl": 4.0}, {"layer": "b", "ppl": 0.5}, {"layer": "c", "ppl": 3.0}]}]}
    assert S.sort_layers_and_bits_average(nan2)[:3] == ["c", "a", "b"]     # b: 0.5 + 6.0 sorts after the finite ones
    bad = {"reduced_ppl": [{"bit": 1, "ppls": [{"layer": "a", "ppl": float("nan")}]}]}
    with pytest.raises(ValueError):
        S.sort_layers_and_bits_average(bad)
    # the list is what retrieve_compression_config reads
    from bitstack_amd.utils import checkpoint as ck
    assert ck.retrieve_compression_config(cfgs, 155 / 1024 ** 2) == cfgs[2]["layers"]
