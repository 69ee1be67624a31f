"""The committed fixtures in tests/golden/ (written by tests/golden/make_fixtures.py from the CPU
oracle): the oracle must still reproduce them on this machine, the torch host path must agree
with them, and on a GPU the HIP path is compared with the committed numbers through the C ABI —
bit for bit for sign bytes, within max|d|/max|y| <= 1e-2 and mean|d|/mean|y| <= 1e-3 for fp16
outputs (the tolerance stated for layer outputs)."""
import os

import numpy as np
import pytest
import torch

from oracle import bitstack_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LAYERS = ["layer_decode", "layer_strip", "layer_odd"]


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def rel(got, ref):
    d = np.abs(np.asarray(got, np.float64) - np.asarray(ref, np.float64))
    return d.max() / max(np.abs(ref).max(), 1e-30), d.mean() / max(np.abs(ref).mean(), 1e-30)


# ------------------------------------------------------------------ CPU: oracle and host path
def test_sign_packing_fixture_oracle():
    f = load("sign_packing")
    assert f["hand_packed"].tolist() == [0x80, 0xFF, 0x01, 0xAA]
    for key in ("hand", "ragged", "block"):
        sign, packed = f[key + "_sign"], f[key + "_packed"]
        assert np.array_equal(O.pack_sign(sign), packed)
        assert np.array_equal(O.unpack_sign(packed, sign.shape), sign)
        assert np.array_equal(packed, np.packbits((sign.reshape(-1) > 0).astype(np.uint8), bitorder="big"))
    assert f["ragged_packed"].size == 5 and f["ragged_packed"][-1] & 0x1F == 0          # 35 signs, 5 zero padding bits
    assert np.array_equal(O.unpack_sign(f["every_byte"], (256, 8)), f["every_byte_sign"])
    assert np.array_equal(f["every_byte_sign"], np.unpackbits(f["every_byte"]).reshape(256, 8).astype(np.int8) * 2 - 1)


def test_sign_packing_fixture_torch_host_path():
    from bitstack_amd.utils.pack_utils import pack_sign, unpack_sign
    f = load("sign_packing")
    for key in ("hand", "ragged", "block"):
        sign, packed = torch.from_numpy(f[key + "_sign"]), f[key + "_packed"]
        assert np.array_equal(pack_sign(sign).numpy(), packed)
        assert np.array_equal(unpack_sign(torch.from_numpy(packed), sign.shape).numpy(), f[key + "_sign"])


@pytest.mark.parametrize("name", LAYERS)
def test_layer_fixture_oracle(name):
    f = load(name)
    q, u, vt, x, b = f["qweight"], f["u"], f["vt"], f["x"], f.get("bias")
    assert np.array_equal(O.reconstruct_w(q, u, vt).view(np.uint16), f["w_f16"].view(np.uint16))
    assert np.array_equal(O.forward_l0(q, u, vt, x, b).view(np.uint16), f["y_l0"].view(np.uint16))
    y64 = O.forward_exact(q, u, vt, x, b)
    assert np.allclose(y64, f["y_f64"], rtol=1e-12, atol=1e-12)
    # the two expected outputs agree with each other within the stated tolerance, and the
    # brute-force triple loop agrees with the closed form on a few entries
    mx, mn = rel(f["y_l0"], f["y_f64"])
    assert mx <= 1e-2 and mn <= 2e-3
    brute = O.brute_force_forward(q, u, vt, x[:1])
    want = f["y_f64"][:1] - (0 if b is None else b.astype(np.float64))
    assert np.allclose(brute, want, rtol=1e-9, atol=1e-9)


@pytest.mark.parametrize("name", LAYERS)
def test_layer_fixture_module_level0_on_cpu(name):
    from bitstack_amd import BitStackLinear
    f = load(name)
    I, M, K = f["u"].shape
    N = f["vt"].shape[2]
    mod = BitStackLinear(I, N, M, K, "bias" in f, False, "cpu")
    for i in range(I):
        getattr(mod, f"qweight_{i}").copy_(torch.from_numpy(f["qweight"][i]))
        getattr(mod, f"u_{i}").copy_(torch.from_numpy(f["u"][i]))
        getattr(mod, f"vt_{i}").copy_(torch.from_numpy(f["vt"][i]))
    if "bias" in f:
        mod.bias.copy_(torch.from_numpy(f["bias"]))
    y = mod(torch.from_numpy(f["x"])).numpy()
    mx, mn = rel(y, f["y_l0"])
    assert mx <= 2e-3 and mn <= 5e-4            # torch's fp16 matmul vs the oracle's rounding of the same order
    mx, mn = rel(y, f["y_f64"])
    assert mx <= 1e-2 and mn <= 2e-3


def test_decompose_fixture_oracle():
    f = load("decompose")
    q, u, vt, norms = O.decompose_weight(f["weight"], 3, 4)
    assert np.array_equal(q, f["qweight"])
    assert np.array_equal(O.unpack_sign(q[0], (48, 64)), np.where(f["weight"] >= 0, 1, -1))      # sign(0) = +1
    for i in range(3):
        prod = u[i].astype(np.float64) @ vt[i].astype(np.float64)
        assert np.abs(prod - f["products"][i]).max() <= 1e-3 * np.abs(f["products"][i]).max()
    assert np.allclose(norms, f["residual_norms"], rtol=1e-5)
    assert f["memory_per_bit"].tolist() == [2_359_296, 688_128, 7_929_856]


# ------------------------------------------------------------------ GPU: the HIP path through the C ABI
def dev():
    return torch.device("cuda:0")


@pytest.mark.gpu
def test_sign_packing_fixture_hip():
    from bitstack_amd.utils import pack_utils as PU
    f = load("sign_packing")
    for key in ("hand", "ragged", "block"):
        sign, packed = torch.from_numpy(f[key + "_sign"]).to(dev()), torch.from_numpy(f[key + "_packed"]).to(dev())
        assert np.array_equal(PU.unpack_sign_hip(packed, sign.shape).cpu().numpy(), f[key + "_sign"])
        assert np.array_equal(PU.pack_sign_hip(sign).cpu().numpy(), f[key + "_packed"])
    got = PU.unpack_sign_hip(torch.from_numpy(f["every_byte"]).to(dev()), torch.Size([256, 8])).cpu().numpy()
    assert np.array_equal(got, f["every_byte_sign"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", LAYERS)
def test_layer_fixture_hip(name):
    from bitstack_amd.utils import inference_utils as IU
    f = load(name)
    q, u, vt, x = (torch.from_numpy(f[k]).to(dev()) for k in ("qweight", "u", "vt", "x"))
    b = torch.from_numpy(f["bias"]).to(dev()) if "bias" in f else None
    w = IU.unpack_and_reconstruct_w_hip(q, u, vt).cpu().numpy()
    want = f["w_f16"]
    ulp = np.spacing(np.abs(want)).astype(np.float64)
    assert np.all(np.abs(w.astype(np.float64) - want.astype(np.float64)) <= ulp)     # same sum, other order: one ulp at most
    for T in (1, x.shape[0]):                              # one token (decode kernels where the shape allows) and all of them
        y = IU.bitstack_forward_hip(q, u, vt, x[:T], b).cpu().numpy()
        for ref in (f["y_f64"][:T], f["y_l0"][:T]):
            mx, mn = rel(y, ref)
            assert mx <= 1e-2 and mn <= 1e-3, (name, T, mx, mn)
