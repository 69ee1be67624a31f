"""Pins the CPU oracle (oracle/) without running the reference.

The reference ships no tests or golden vectors for this path, so each oracle
function is tied to something independent of its own formula: a library
routine it must reduce to, hand-derived known answers, fp64 brute force over
the definition, or an algebraic invariant.
"""
import numpy as np
import pytest

from oracle import bitstack_oracle as O
from oracle import c_oracle as C


def rand_case(rng, I, M, N, K, T=1, positive=False):
    q = rng.integers(0, 256, size=(I, (M * N + 7) // 8), dtype=np.uint8)
    u = rng.standard_normal((I, M, K)).astype(np.float32)
    vt = rng.standard_normal((I, K, N)).astype(np.float32)
    if positive:
        u, vt = np.abs(u), np.abs(vt)
    x = rng.standard_normal((T, N)).astype(np.float16)
    return q, (u * 0.1).astype(np.float16), (vt * 0.1).astype(np.float16), x


# ----------------------------------------------------------------- pack/unpack
KATS = [
    ([+1, -1, -1, -1, -1, -1, -1, -1], [0x80]),
    ([+1] * 8, [0xFF]),
    ([-1] * 8, [0x00]),
    ([-1, -1, -1, -1, -1, -1, -1, +1], [0x01]),
    ([+1, -1, +1, -1, +1, -1, +1, -1], [0xAA]),
    ([+1, +1, -1, -1, +1, -1, -1, +1, -1, +1, +1, +1, -1, -1, -1, -1], [0xC9, 0x70]),
    ([+1, +1, +1], [0xE0]),                 # 5 padding bits are zeros (decode to -1)
    ([-1, +1, -1, +1, -1, +1, -1, +1, +1], [0x55, 0x80]),
]


@pytest.mark.parametrize("impl", [O, C])
@pytest.mark.parametrize("signs,expect", KATS)
def test_pack_known_answers(impl, signs, expect):
    got = impl.pack_sign(np.array(signs, dtype=np.int8))
    assert got.dtype == np.uint8
    assert got.tolist() == expect


@pytest.mark.parametrize("impl", [O, C])
def test_unpack_all_byte_values(impl):
    allb = np.arange(256, dtype=np.uint8)
    got = impl.unpack_sign(allb, (256, 8))
    for b in range(256):
        want = [1 if (b >> (7 - j)) & 1 else -1 for j in range(8)]
        assert got[b].tolist() == want


@pytest.mark.parametrize("impl", [O, C])
@pytest.mark.parametrize("shape", [(8,), (3, 8), (5, 7), (16, 24), (1, 1), (13,), (64, 64)])
def test_pack_matches_numpy_packbits_and_round_trips(impl, shape):
    rng = np.random.default_rng(hash(shape) & 0xFFFF)
    s = (rng.integers(0, 2, size=shape) * 2 - 1).astype(np.int8)
    packed = impl.pack_sign(s)
    assert np.array_equal(packed, np.packbits((s.reshape(-1) > 0).astype(np.uint8), bitorder="big"))
    back = impl.unpack_sign(packed, shape)
    assert back.dtype == np.int8 and back.shape == tuple(shape)
    assert np.array_equal(back, s)                  # the reference's own invariant
    n = s.size
    ref_bits = np.unpackbits(packed, bitorder="big")[:n].astype(np.int8) * 2 - 1
    assert np.array_equal(back.reshape(-1), ref_bits)


def test_padding_bits_decode_to_minus_one():
    s = np.array([1, 1, 1], dtype=np.int8)
    packed = O.pack_sign(s)
    assert O.unpack_sign(packed, (8,)).tolist() == [1, 1, 1, -1, -1, -1, -1, -1]


@pytest.mark.parametrize("impl", [O, C])
def test_pack_rejects_non_sign_entries(impl):
    with pytest.raises(AssertionError):
        impl.pack_sign(np.array([1, 0, -1, 1, 1, 1, 1, 1], dtype=np.int8))


def test_c_half_conversion_matches_numpy_everywhere():
    allh = np.arange(65536, dtype=np.uint16)
    f = C.h2f(allh)
    want = allh.view(np.float16).astype(np.float32)
    same = (f == want) | (np.isnan(f) & np.isnan(want))
    assert same.all()
    finite = np.isfinite(want)
    assert np.array_equal(C.f2h(want[finite]), allh[finite])
    # round-to-nearest-even on values between halves
    rng = np.random.default_rng(1)
    v = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10.0 ** rng.integers(-9, 5, 200000),
        np.array([65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  2.0 ** -24 * 1.5, 2.0 ** -24 * 2.5, 2.0 ** -14, 2049.0, 2051.0, 0.0, -0.0],
                 dtype=np.float32)]).astype(np.float32)
    with np.errstate(over="ignore"):
        want16 = v.astype(np.float16).view(np.uint16)
    assert np.array_equal(C.f2h(v), want16)


# ------------------------------------------------------- compose / reconstruct
def test_compose_and_forward_match_brute_force():
    rng = np.random.default_rng(7)
    for (I, M, N, K, T) in [(1, 4, 8, 2, 1), (3, 5, 16, 4, 2), (2, 8, 24, 16, 3)]:
        q, u, vt, x = rand_case(rng, I, M, N, K, T)
        want = O.brute_force_forward(q, u, vt, x)
        got = O.forward_exact(q, u, vt, x)
        np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
        gotc = C.forward_f64(q, u, vt, x)
        np.testing.assert_allclose(gotc, want, rtol=1e-12, atol=1e-12)
        # one block of compose_weight against the definition, fp32 factors
        w = O.compose_weight(q[0], u[0].astype(np.float32), vt[0].astype(np.float32), False, (M, N))
        s = np.unpackbits(q[0], bitorder="big")[:M * N].reshape(M, N).astype(np.float64) * 2 - 1
        np.testing.assert_allclose(w, s * (u[0].astype(np.float64) @ vt[0].astype(np.float64)),
                                   rtol=1e-5, atol=1e-7)
        assert w.dtype == np.float32                 # dtype follows u
        assert O.compose_weight(q[0], u[0], vt[0], False, (M, N)).dtype == np.float16


def test_exact_form_invariants():
    rng = np.random.default_rng(11)
    I, M, N, K = 3, 16, 32, 8
    q, u, vt, x = rand_case(rng, I, M, N, K, 2)
    y = O.forward_exact(q, u, vt, x)
    # linearity in x (x scaled by a power of two stays exact in fp16)
    np.testing.assert_allclose(O.forward_exact(q, u, vt, (x * 2).astype(np.float16)), 2 * y, rtol=1e-12)
    # block additivity
    parts = sum(O.forward_exact(q[i:i + 1], u[i:i + 1], vt[i:i + 1], x) for i in range(I))
    np.testing.assert_allclose(parts, y, rtol=1e-10, atol=1e-12)
    # complementing every byte of block 1 negates that block's contribution
    q2 = q.copy()
    q2[1] = ~q2[1]
    y1 = O.forward_exact(q[1:2], u[1:2], vt[1:2], x)
    np.testing.assert_allclose(O.forward_exact(q2, u, vt, x), y - 2 * y1, rtol=1e-10, atol=1e-12)
    # scaling a row of u scales that output only
    u2 = u.copy()
    u2[:, 3, :] *= np.float16(4)
    y2 = O.forward_exact(q, u2, vt, x)
    np.testing.assert_allclose(y2[:, 3], 4 * y[:, 3], rtol=1e-12)
    np.testing.assert_allclose(np.delete(y2, 3, axis=1), np.delete(y, 3, axis=1), rtol=1e-12)
    # zeroing a column of vt removes that input's influence
    vt2 = vt.copy()
    vt2[:, :, 5] = 0
    x2 = x.copy()
    x2[:, 5] = 77
    np.testing.assert_allclose(O.forward_exact(q, u, vt2, x2), O.forward_exact(q, u, vt2, x), rtol=1e-12)
    # bias is added once per output feature
    b = rng.standard_normal(M).astype(np.float16)
    np.testing.assert_allclose(O.forward_exact(q, u, vt, x, b), y + b.astype(np.float64)[None, :], rtol=1e-12)


def test_reconstruct_single_rounding_and_agreement_with_c():
    rng = np.random.default_rng(3)
    I, M, N, K = 4, 32, 64, 16
    q, u, vt, _ = rand_case(rng, I, M, N, K)
    exact = O.reconstruct_w_exact(q, u, vt)
    w = O.reconstruct_w(q, u, vt)
    assert w.dtype == np.float16 and w.shape == (M, N)
    # one rounding of an fp32 sum: within half an fp16 ulp (+ fp32 noise) of exact
    ulp = np.spacing(np.abs(exact).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(w.astype(np.float64) - exact) <= 0.5 * ulp + 1e-6)
    wc = C.reconstruct_w(q, u, vt)
    diff = np.abs(wc.astype(np.float64) - w.astype(np.float64))
    assert np.all(diff <= ulp)                       # summation order may flip a tie
    assert np.mean(diff > 0) < 1e-2


def test_forward_l0_keeps_the_fp16_running_sum():
    """2048 + 1 + 1 in fp16 stays 2048 (ties to even, twice); an fp32 sum rounded
    once gives 2050.  Level 0 must show the former (BitStackLinear.py:107-113)."""
    M, N, K, I = 1, 8, 1, 3
    q = np.full((I, 1), 0xFF, dtype=np.uint8)          # all signs +1
    u = np.array([[[2048.0]], [[1.0]], [[1.0]]], dtype=np.float16)
    vt = np.ones((I, K, N), dtype=np.float16)
    x = np.zeros((1, N), dtype=np.float16)
    x[0, 0] = 1.0
    assert float(O.forward_l0(q, u, vt, x)[0, 0]) == 2048.0
    assert float(C.forward_l0(q, u, vt, x)[0, 0]) == 2048.0
    assert float(O.reconstruct_w(q, u, vt)[0, 0]) == 2050.0
    assert float(C.reconstruct_w(q, u, vt)[0, 0]) == 2050.0
    # and the per-block product is itself rounded to fp16 before the sum:
    # (1 + 2^-10) * (1 + 2^-10) = 1 + 2^-9 + 2^-20 -> fp16 1 + 2^-9
    u1 = np.array([[[1.0 + 2.0 ** -10]]], dtype=np.float16)
    vt1 = np.full((1, 1, N), 1.0 + 2.0 ** -10, dtype=np.float16)
    x[0, 0] = 1.0
    y = O.forward_l0(q[:1], u1, vt1, x)
    assert float(y[0, 0]) == 1.0 + 2.0 ** -9
    assert float(C.forward_l0(q[:1], u1, vt1, x)[0, 0]) == 1.0 + 2.0 ** -9


def test_forward_l0_close_to_exact_and_c_agrees():
    rng = np.random.default_rng(5)
    I, M, N, K, T = 4, 64, 128, 16, 3
    q, u, vt, x = rand_case(rng, I, M, N, K, T, positive=True)
    b = rng.standard_normal(M).astype(np.float16)
    exact = O.forward_exact(q, u, vt, x, b)
    y = O.forward_l0(q, u, vt, x, b)
    assert y.dtype == np.float16 and y.shape == (T, M)
    scale = np.abs(exact).max()
    assert np.abs(y.astype(np.float64) - exact).max() / scale < 1e-2
    assert np.abs(y.astype(np.float64) - exact).mean() / np.abs(exact).mean() < 2e-3
    yc = C.forward_l0(q, u, vt, x, b)
    assert np.abs(yc.astype(np.float64) - y.astype(np.float64)).max() / scale < 2e-3
    # leading dimensions are preserved
    x3 = x.reshape(1, T, N)
    assert O.forward_l0(q, u, vt, x3).shape == (1, T, M)


# ------------------------------------------------------------------ decompose
def test_decompose_is_truncated_svd_of_abs_residual():
    rng = np.random.default_rng(0)
    M, N, k, niter = 48, 64, 4, 3
    W = (rng.standard_normal((M, N)) * 0.02).astype(np.float32)
    W[0, 0] = 0.0                                     # sign(0) must count as +1
    q, u, vt, norms = O.decompose_weight(W, niter, k)
    assert q.shape == (niter, M * N // 8) and u.shape == (niter, M, k) and vt.shape == (niter, k, N)
    assert u.dtype == np.float16 and vt.dtype == np.float16
    assert O.unpack_sign(q[0], (M, N))[0, 0] == 1
    assert np.array_equal(O.unpack_sign(q[0], (M, N)), np.where(W >= 0, 1, -1))
    # Eckart-Young: the block-0 product is the best rank-k approximation of |W|
    uu, sv, vv = np.linalg.svd(np.abs(W).astype(np.float64), full_matrices=False)
    best = (uu[:, :k] * sv[:k]) @ vv[:k]
    prod = u[0].astype(np.float64) @ vt[0].astype(np.float64)
    assert np.abs(prod - best).max() < 2e-3 * np.abs(best).max()       # fp16 factors
    # the residual after block 0 has the Frobenius norm the tail singular values give
    assert norms[1] == pytest.approx(np.sqrt((sv[k:] ** 2).sum()), rel=1e-4)
    # residual norms never grow, approximation error falls with blocks loaded
    assert all(b <= a * (1 + 1e-6) for a, b in zip(norms, norms[1:]))
    errs = [np.linalg.norm(O.reconstruct_w_exact(q[:i], u[:i], vt[:i]) - W) for i in range(1, niter + 1)]
    assert errs[0] > errs[1] > errs[2]
    assert errs[-1] == pytest.approx(norms[-1], rel=5e-2)


# ---------------------------------------------------------------- bookkeeping
def test_memory_per_bit_closed_form():
    assert O.memory_per_bit(4096, 4096, 16) == 2_359_296
    assert O.memory_per_bit(1024, 4096, 16) == 688_128
    assert O.memory_per_bit(14336, 4096, 16) == 7_929_856
    assert O.memory_per_bit(4096, 14336, 16) == 7_929_856
    assert O.memory_per_bit(4096, 4096, 16, no_avd=True) == 2 * 16 * 8192


def test_retrieve_compression_config():
    cfgs = [{"memory": 3 * 2 ** 20, "layers": {"a": 1}},
            {"memory": 5 * 2 ** 20, "layers": {"a": 2}},
            {"memory": 9 * 2 ** 20, "layers": {"a": 3}}]
    assert O.retrieve_compression_config(cfgs, 5) == {"a": 2}
    assert O.retrieve_compression_config(cfgs, 8.99) == {"a": 2}
    assert O.retrieve_compression_config(cfgs, 100) == {"a": 3}
    with pytest.raises(ValueError):
        O.retrieve_compression_config(cfgs, 2)


def test_torch_level0_restatement_matches_the_oracle():
    """oracle/torch_l0.py (what the CPU baseline of the benchmark times) against the numpy level-0
    restatement: the same unpack, the same fp16 running sum of the weight, F.linear with fp32
    accumulation - outputs equal to the last fp16 bit or its neighbour, signs bit for bit."""
    import torch
    from oracle import torch_l0
    rng = np.random.default_rng(12)
    I, M, N, K, T = 3, 48, 64, 16, 2
    q = rng.integers(0, 256, size=(I, M * N // 8), dtype=np.uint8)
    u = (np.abs(rng.standard_normal((I, M, K))) * 0.1).astype(np.float16)
    vt = (np.abs(rng.standard_normal((I, K, N))) * 0.1).astype(np.float16)
    x = rng.standard_normal((T, N)).astype(np.float16)
    bias = rng.standard_normal(M).astype(np.float16)
    s = torch_l0.unpack_sign(torch.from_numpy(q[0]), torch.Size((M, N))).numpy()
    assert np.array_equal(s, O.unpack_sign(q[0], (M, N)))
    for b in (None, bias):
        got = torch_l0.forward_l0(torch.from_numpy(q), torch.from_numpy(u), torch.from_numpy(vt), torch.from_numpy(x),
                                  None if b is None else torch.from_numpy(b)).numpy()
        want = O.forward_l0(q, u, vt, x, b)
        assert got.dtype == np.float16 and got.shape == want.shape
        ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float64)
        assert np.all(np.abs(got.astype(np.float64) - want.astype(np.float64)) <= ulp)
        exact = O.forward_exact(q, u, vt, x, b)
        assert np.abs(got - exact).max() <= 1e-2 * np.abs(exact).max()
