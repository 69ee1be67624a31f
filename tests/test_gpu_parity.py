"""Parity of the HIP path (through the C ABI) with the CPU oracle, on a real
MI355X.  Integer / byte work is compared bit for bit; floating point within

    max|d| / max|y_ref| <= 1e-2   and   mean|d| / mean|y_ref| <= 1e-3

against the fp64 closed form and against the level-0 rounding order (the
tolerance the task states for fp16 layer outputs)."""
import numpy as np
import pytest
import torch

from bitstack_amd import BitStackLinear, _lib
from bitstack_amd.utils import inference_utils as IU
from bitstack_amd.utils import pack_utils as PU
from bitstack_amd.utils.synthetic import synthetic_layer
from oracle import bitstack_oracle as O
from oracle import c_oracle as C

pytestmark = pytest.mark.gpu

MAX_REL, MEAN_REL = 1e-2, 1e-3


def dev():
    return torch.device("cuda:0")


def rel_errors(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.abs(got - ref)
    return d.max() / max(np.abs(ref).max(), 1e-30), d.mean() / max(np.abs(ref).mean(), 1e-30)


def assert_close(got, ref, what, max_rel=MAX_REL, mean_rel=MEAN_REL):
    mx, mn = rel_errors(got, ref)
    print(f"{what}: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= max_rel and mn <= mean_rel, f"{what}: max_rel={mx:.3e} mean_rel={mn:.3e}"


def test_library_is_the_hip_build():
    assert _lib.lib().bs_version() >= 100
    assert torch.cuda.get_device_properties(0).gcnArchName.startswith("gfx950")


# ------------------------------------------------------------------ integers
@pytest.mark.parametrize("n", [8, 32, 33, 1000, 4096, 64 * 72, 1 << 20, (1 << 20) + 13, 4096 * 4096])
def test_unpack_bit_exact(n):
    print(f"unpack n={n}", flush=True)
    rng = np.random.default_rng(n & 0xFFFF)
    packed = rng.integers(0, 256, size=(n + 7) // 8, dtype=np.uint8)
    got = PU.unpack_sign_hip(torch.from_numpy(packed).to(dev()), (n,)).cpu().numpy()
    want = np.unpackbits(packed, bitorder="big")[:n].astype(np.int8) * 2 - 1
    assert got.dtype == np.int8 and np.array_equal(got, want)
    if n <= 1 << 20:
        assert np.array_equal(got, O.unpack_sign(packed, (n,)))


def test_unpack_from_unaligned_views():
    rng = np.random.default_rng(5)
    base = torch.from_numpy(rng.integers(0, 256, size=5000, dtype=np.uint8)).to(dev())
    for off in (1, 2, 3, 5):
        view = base[off:off + 4000]
        got = PU.unpack_sign_hip(view, (4000 * 8,)).cpu().numpy()
        assert np.array_equal(got, O.unpack_sign(view.cpu().numpy(), (32000,)))


def test_unpack_all_blocks_shape():
    q, _, _, _ = synthetic_layer(64, 128, 3, 1, device=dev())
    s = PU.unpack_sign_triton(q.view(-1), torch.Size([3, 64, 128]))
    assert tuple(s.shape) == (3, 64, 128)
    for i in range(3):
        assert np.array_equal(s[i].cpu().numpy(), O.unpack_sign(q[i].cpu().numpy(), (64, 128)))


@pytest.mark.parametrize("shape", [(8,), (5, 7), (13,), (64, 72), (1024, 4096)])
def test_pack_bit_exact_and_round_trip(shape):
    print(f"pack shape={shape}", flush=True)
    rng = np.random.default_rng(len(shape) + shape[0])
    s = (rng.integers(0, 2, size=shape) * 2 - 1).astype(np.int8)
    st = torch.from_numpy(s).to(dev())
    p = PU.pack_sign(st)
    assert np.array_equal(p.cpu().numpy(), np.packbits((s.reshape(-1) > 0), bitorder="big"))
    assert torch.equal(PU.unpack_sign(p, torch.Size(shape)), st)


# --------------------------------------------------------------- reconstruct
RECON_CASES = [(1, 64, 128, 16), (3, 64, 256, 16), (2, 50, 128, 16), (4, 256, 512, 16),
               (2, 64, 128, 7), (1, 64, 128, 1), (2, 40, 72, 16), (3, 33, 100, 5),
               (8, 1024, 4096, 16),
               # block counts that are not multiples of the four pairs a sign load brings, many row steps per wave,
               # ragged row counts, the most blocks the tiled kernel takes
               (5, 700, 256, 16), (7, 1000, 384, 16), (1, 2048, 1024, 16), (36, 200, 128, 16), (6, 4096, 4096, 16),
               (3, 130, 128, 3), (9, 14336, 128, 16)]


@pytest.mark.parametrize("I,M,N,K", RECON_CASES)
def test_reconstruct_w_matches_oracle(I, M, N, K):
    print(f"reconstruct I={I} M={M} N={N} K={K}", flush=True)
    q, u, vt, _ = synthetic_layer(M, N, I, 1, k=K, seed=I + M, signed_factors=True)
    u, vt = (u * 20).half(), (vt * 20).half()
    want = C.reconstruct_w(q.numpy(), u.numpy(), vt.numpy())
    qd, ud, vd = q.to(dev()), u.to(dev()), vt.to(dev())
    got = IU.unpack_and_reconstruct_w_hip(qd, ud, vd).cpu().numpy()
    assert got.dtype == np.float16 and got.shape == (M, N)
    # both are one fp16 rounding of an fp32 sum; only the summation order differs
    ulp = np.spacing(np.abs(want)).astype(np.float64)
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert np.all(diff <= ulp), f"max diff {diff.max()} vs ulp"
    assert np.mean(diff > 0) < 2e-2
    assert diff.max() <= 1e-2          # the reference's own self-check bound (atol=1e-2)
    # the int8-sign entry point gives the identical weight
    # (unpacked block by block: a block whose M * N is not a multiple of 8 ends in padding bits)
    sign = torch.stack([PU.unpack_sign_hip(qd[i], torch.Size([M, N])) for i in range(I)])
    got2 = IU.reconstruct_w_hip(sign, ud, vd).cpu().numpy()
    assert np.array_equal(got2.view(np.uint16), got.view(np.uint16))


def test_reference_self_check_scenario():
    """The one numeric check the reference carries (bitstack/utils/inference_utils.py:597-626):
    M = N = 32, k = 16, one block, sign / u / vt / x drawn from N(0, 1) in fp16; the rebuilt weight
    against `(sign * matmul(u, vt)).sum(0)` within atol = 1e-2, rtol = 0 — and, from the lines it
    keeps commented out, the fused forward against `x @ W.T`."""
    g = torch.Generator().manual_seed(0)
    M = N = 32
    x = torch.randn(1, 1, N, generator=g).half()
    sign = torch.sign(torch.randn(1, M, N, generator=g).half())
    sign[sign == 0] = 1
    packed = torch.from_numpy(O.pack_sign(sign.to(torch.int8).numpy().reshape(-1))).reshape(1, -1)
    u = torch.randn(1, M, 16, generator=g).half()
    vt = torch.randn(1, 16, N, generator=g).half()
    ref_w = (sign * torch.matmul(u.float(), vt.float()).half()).sum(dim=0)           # the script's torch_output
    pd, ud, vd = packed.to(dev()), u.to(dev()), vt.to(dev())
    w = IU.unpack_and_reconstruct_w_hip(pd, ud, vd).cpu()
    assert torch.allclose(w, ref_w, atol=1e-2, rtol=0)
    w2 = IU.reconstruct_w_hip(sign.to(torch.int8).to(dev()), ud, vd).cpu()
    assert torch.equal(w2, w)
    exact_w = O.reconstruct_w_exact(packed.numpy(), u.numpy(), vt.numpy())
    assert np.all(np.abs(w.double().numpy() - exact_w) <= np.spacing(np.abs(exact_w).astype(np.float16)).astype(np.float64))
    y = IU.bitstack_forward_hip(pd, ud, vd, x.to(dev())).cpu()
    assert tuple(y.shape) == (1, 1, M)
    assert_close(y.view(1, M).numpy(), x.view(1, N).double().numpy() @ exact_w.T, "forward vs fp64")


def test_reconstruct_zero_blocks_is_zero():
    q, u, vt, _ = synthetic_layer(64, 128, 2, 1, device=dev())
    w = IU.unpack_and_reconstruct_w_hip(q[:0], u[:0], vt[:0])
    assert float(w.abs().max()) == 0.0


# ------------------------------------------------------------------- forward
def oracle_refs(q, u, vt, x, bias=None):
    qn, un, vn, xn = q.numpy(), u.numpy(), vt.numpy(), x.numpy()
    bn = None if bias is None else bias.numpy()
    return C.forward_f64(qn, un, vn, xn, bn), C.forward_l0(qn, un, vn, xn, bn)


GEMV_CASES = [(1, 64, 512, 1), (2, 256, 512, 1), (4, 1024, 1024, 1), (3, 200, 1024, 2),
              (4, 4096, 4096, 1), (2, 1024, 4096, 4), (8, 4096, 4096, 4), (1, 1024, 4096, 1),
              (2, 14336, 4096, 1), (2, 4096, 14336, 1), (3, 512, 2048, 3), (2, 512, 1024, 5),
              (2, 300, 1536, 6), (2, 256, 512, 7), (2, 512, 1024, 8), (16, 1024, 4096, 1),
              # long stacks: 16-wave workgroups in pairs (one token), 8-wave pairs (two tokens)
              (64, 2048, 4096, 1), (16, 4096, 4096, 2),
              # 16 waves with a ragged last row tile; 16 waves, odd chunk count (no pairing)
              (48, 2500, 4096, 1), (200, 1100, 1536, 1)]


@pytest.mark.parametrize("I,M,N,T", GEMV_CASES)
def test_forward_decode_matches_oracle(I, M, N, T):
    print(f"forward decode I={I} M={M} N={N} T={T}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=I * 7 + T)
    exact, l0 = oracle_refs(q, u, vt, x)
    y = IU.bitstack_forward_hip(q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev())).cpu().numpy()
    assert y.dtype == np.float16 and y.shape == (T, M)
    assert_close(y, exact, "vs fp64")
    if I <= 16:     # beyond that the level-0 order's own fp16 running sums are the larger error
        assert_close(y, l0, "vs level-0 order")


@pytest.fixture
def decode_kernel():
    """Lets a test pin the one-token decode kernel; always back to the planner's own choice afterwards."""
    L = _lib.lib()
    yield lambda mode: _lib.check(L.bs_set_decode_kernel(mode), "bs_set_decode_kernel")
    L.bs_set_decode_kernel(_lib.DECODE_AUTO)


# one and two tokens through the block-scaled fp4 x fp6 kernel: every row-tile height (128 .. 1024 rows per workgroup),
# ragged last row tiles, N a multiple of 512 but not of 1024 (a unit whose second half lies beyond N), ranks
# below 16 (whole rank quads and a partial one missing), many blocks, several units per workgroup
MX_CASES = [(1, 64, 512, 16), (1, 128, 1024, 16), (2, 256, 1536, 16), (4, 1024, 1024, 16), (3, 200, 1024, 5),
            (2, 130, 2560, 1), (3, 1000, 512, 12), (2, 2048, 2048, 9), (4, 4096, 4096, 16), (1, 1024, 4096, 16),
            (2, 14336, 4096, 16), (2, 4096, 14336, 16), (16, 1024, 4096, 16), (64, 2048, 4096, 16),
            (48, 2500, 4096, 16), (200, 1100, 1536, 16), (16, 4096, 4096, 16), (5, 8192, 3584, 16)]


@pytest.mark.parametrize("T", [1, 2])
@pytest.mark.parametrize("I,M,N,K", MX_CASES)
def test_forward_decode_block_scaled_kernel(I, M, N, K, T, decode_kernel):
    """The block-scaled kernel splits vt * x (fp16) into three fp6 terms per 32 columns, exact to under
    1e-4 of the block maximum: same tolerance as the fp16 kernel against float64, and the two kernels
    against each other."""
    print(f"forward decode (block-scaled) I={I} M={M} N={N} K={K} T={T}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, k=K, seed=I * 5 + K + T, signed_factors=(K != 16))
    bias = (torch.randn(M, generator=torch.Generator().manual_seed(K)) * 0.01).half() if (I + K) % 2 else None
    exact, l0 = oracle_refs(q, u, vt, x, bias)
    args = (q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev()), None if bias is None else bias.to(dev()))
    decode_kernel(_lib.DECODE_MX)
    assert _lib.lib().bs_decode_kernel(I, M, N, K, T) == _lib.DECODE_MX
    y = IU.bitstack_forward_hip(*args)
    assert torch.equal(IU.bitstack_forward_hip(*args), y)                   # deterministic
    decode_kernel(_lib.DECODE_F16)
    assert _lib.lib().bs_decode_kernel(I, M, N, K, T) == _lib.DECODE_F16
    y16 = IU.bitstack_forward_hip(*args)
    y = y.cpu().numpy()
    assert y.dtype == np.float16 and y.shape == (T, M)
    assert_close(y, exact, "vs fp64")
    if I <= 16:
        assert_close(y, l0, "vs level-0 order")
    assert_close(y, y16.float().cpu().numpy(), "vs the fp16 decode kernel", 2e-3, 3e-4)


@pytest.mark.parametrize("bad", [float("nan"), float("inf"), float("-inf")])
def test_non_finite_activations_stay_non_finite_on_both_decode_kernels(bad, decode_kernel):
    """F.linear on the rebuilt weight (bitstack/modules/BitStackLinear.py:114) gives a non-finite y[t, :]
    for a token whose x holds a NaN or an infinity.  fp6 has no encoding for either, so the block-scaled
    kernel carries them in the block's scale: every output of that token must come out non-finite on
    both decode kernels, and the other token of a two-token call must stay as it was."""
    I, M, N = 3, 1024, 4096
    q, u, vt, x = synthetic_layer(M, N, I, 2, seed=77, device=dev())
    clean = {}
    for T in (1, 2):
        for col in (0, 777, N - 1):
            xb = x[:T].clone()
            xb[0, col] = bad
            for mode in (_lib.DECODE_F16, _lib.DECODE_MX):
                decode_kernel(mode)
                assert _lib.lib().bs_decode_kernel(I, M, N, 16, T) == mode
                if (T, mode) not in clean:
                    clean[(T, mode)] = IU.bitstack_forward_hip(q, u, vt, x[:T].contiguous())
                y = IU.bitstack_forward_hip(q, u, vt, xb)
                assert not bool(torch.isfinite(y[0]).any()), (T, col, mode)
                if T == 2:
                    assert torch.equal(y[1], clean[(T, mode)][1]), (col, mode)
    # a non-finite weight factor: every token's outputs
    vb = vt.clone()
    vb[1, 5, 1234] = bad
    for mode in (_lib.DECODE_F16, _lib.DECODE_MX):
        decode_kernel(mode)
        y = IU.bitstack_forward_hip(q, u, vb, x)
        assert not bool(torch.isfinite(y).any()), mode


def test_block_scaled_kernel_is_declined_where_it_does_not_apply(decode_kernel):
    decode_kernel(_lib.DECODE_MX)
    L = _lib.lib()
    assert L.bs_decode_kernel(2, 256, 512, 16, 2) == _lib.DECODE_MX        # two tokens: units of 512 columns
    assert L.bs_decode_kernel(2, 256, 512, 16, 3) == _lib.DECODE_F16       # more than two tokens
    assert L.bs_decode_kernel(2, 256, 640, 16, 1) == 0                     # N not a multiple of 512: no decode kernel at all
    q, u, vt, x = synthetic_layer(256, 1024, 2, 3, seed=1)
    exact, _ = oracle_refs(q, u, vt, x)
    y = IU.bitstack_forward_hip(q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev())).cpu().numpy()
    assert_close(y, exact, "three tokens with the block-scaled kernel requested")


@pytest.mark.parametrize("I,M,N,T", [(40, 1024, 4096, 5), (40, 4096, 4096, 5), (40, 4096, 4096, 7), (40, 1024, 4096, 6)])
def test_forward_decode_two_passes_of_unequal_length(I, M, N, T):
    """Stacks too long for the strip kernel (its vt image would not fit in LDS) take the decode kernel
    in two passes (3 + 2, 3 + 3, 4 + 3 tokens); the shorter pass has a plan of its own, and every row of
    every token must come out (a tail pass run on the first pass's tile height left half of each row
    tile unwritten)."""
    print(f"forward two passes I={I} M={M} N={N} T={T}", flush=True)
    assert _lib.decode_plan(I, M, N, 16, T)[0] > 0         # the decode kernel, not the strip kernel
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=I + T)
    exact = C.forward_f64(q.numpy(), u.numpy(), vt.numpy(), x.numpy())
    qd, ud, vd, xd = q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev())
    # poison the scratch the call will use, so an unwritten partial cannot pass by luck
    ws = _lib.workspace(xd.device, _lib.lib().bs_workspace_bytes(I, M, N, 16, T))
    ws[:ws.numel() // 4 * 4].view(torch.float32).fill_(float("nan"))
    y = IU.bitstack_forward_hip(qd, ud, vd, xd).cpu().numpy()
    assert y.shape == (T, M) and np.isfinite(y).all()
    assert_close(y, exact, "vs fp64")
    # token by token through the one-token kernel: the same numbers up to fp32 summation order
    y1 = torch.cat([IU.bitstack_forward_hip(qd, ud, vd, xd[t:t + 1].contiguous()) for t in range(T)]).float().cpu().numpy()
    assert np.abs(y.astype(np.float64) - y1).max() <= 2e-3 * np.abs(y1).max()


@pytest.mark.parametrize("I,M,N,T,K", [(2, 128, 512, 1, 16), (3, 256, 1024, 2, 5), (2, 64, 512, 1, 1)])
def test_forward_decode_signed_factors_bias_and_small_rank(I, M, N, T, K):
    print(f"forward signed I={I} M={M} N={N} T={T} K={K}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, k=K, seed=11, signed_factors=True)
    bias = (torch.randn(M, generator=torch.Generator().manual_seed(1)) * 0.01).half()
    exact, l0 = oracle_refs(q, u, vt, x, bias)
    y = IU.bitstack_forward_hip(q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev()), bias.to(dev()))
    assert_close(y.cpu().numpy(), exact, "vs fp64")
    assert_close(y.cpu().numpy(), l0, "vs level-0 order")


@pytest.mark.parametrize("I,M,N,T", [(2, 40, 72, 1), (3, 33, 200, 3), (2, 64, 520, 9), (1, 16, 8, 1), (40, 64, 256, 12)])
def test_forward_odd_shapes_take_the_rebuild_path(I, M, N, T):
    print(f"forward odd I={I} M={M} N={N} T={T}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=2)
    exact, l0 = oracle_refs(q, u, vt, x)
    y = IU.bitstack_forward_hip(q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev())).cpu().numpy()
    assert_close(y, exact, "vs fp64")
    if I <= 8:      # with more blocks the level-0 order's own fp16 sums are further from fp64 than the bound
        assert_close(y, l0, "vs level-0 order")


# 5..48 tokens: weight patches rebuilt in registers and multiplied at once (N a multiple of 128)
STRIP_CASES = [(1, 16, 128, 5, 16), (3, 100, 384, 9, 16), (2, 65, 1152, 17, 7), (4, 1000, 2048, 32, 16),
               (20, 64, 256, 6, 16), (2, 4096, 4096, 32, 16), (3, 14336, 4096, 8, 16), (2, 1024, 14336, 16, 16),
               (36, 130, 128, 12, 3), (1, 4096, 1152, 8, 16), (2, 3000, 2432, 20, 16),
               (3, 1000, 1024, 33, 16), (2, 4096, 4096, 48, 16), (4, 333, 640, 41, 5)]


# 49..96 tokens: the same patches with the strips walked by a workgroup of 128 rows (4-6 token tiles): ragged rows and
# token tiles, ranks below 16, one strip and several per chunk (few blocks leave room in LDS), several chunks per
# workgroup, row counts whose workgroups do not fill the chip (few blocks: still taken), one column group and many
WIDE_CASES = [(2, 128, 128, 49, 16), (3, 1000, 1152, 64, 16), (1, 4096, 4096, 96, 16), (8, 4096, 4096, 65, 16),
              (3, 8192, 4096, 80, 16), (2, 4096, 14336, 50, 16), (5, 333, 640, 77, 5), (12, 1024, 4096, 96, 16),
              (4, 130, 2432, 81, 12), (6, 2000, 1024, 49, 1)]


@pytest.fixture
def prefill_kernel():
    """Lets a test pin the kernel of a forward of 49 tokens or more; back to the planner's choice afterwards."""
    L = _lib.lib()
    yield lambda mode: _lib.check(L.bs_set_prefill_kernel(mode), "bs_set_prefill_kernel")
    L.bs_set_prefill_kernel(_lib.PREFILL_AUTO)


@pytest.mark.parametrize("I,M,N,T,K", WIDE_CASES)
def test_forward_49_to_96_tokens_matches_oracle(I, M, N, T, K, prefill_kernel):
    print(f"forward walked strips I={I} M={M} N={N} T={T} K={K}", flush=True)
    L = _lib.lib()
    prefill_kernel(_lib.PREFILL_WALKED)          # (from six blocks on a tall shape the planner prefers the panel kernel)
    assert L.bs_forward_path(I, M, N, K, T) == _lib.PATH_WALKED
    # the path is taken: the scratch is g x ([T, M] partial sums + T sums of squares) for g column groups, not the weight
    need = int(L.bs_workspace_bytes(I, M, N, K, T))
    groups = need // (T * (M + 1) * 4)
    assert groups >= 1 and need == (groups * T * (M + 1) * 4 + 255) // 256 * 256 and need != M * N * 2
    q, u, vt, x = synthetic_layer(M, N, I, T, k=K, seed=5 * I + T, signed_factors=True)
    bias = (torch.randn(M, generator=torch.Generator().manual_seed(T)) * 0.05).half() if T % 2 else None
    exact, l0 = oracle_refs(q, u, vt, x, bias)
    qd, ud, vd, xd = q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev())
    bd = None if bias is None else bias.to(dev())
    y = IU.bitstack_forward_hip(qd, ud, vd, xd, bd)
    assert torch.equal(IU.bitstack_forward_hip(qd, ud, vd, xd, bd), y)
    y = y.cpu().numpy()
    assert y.dtype == np.float16 and y.shape == (T, M)
    assert_close(y, exact, "vs fp64")
    if I <= 8:
        assert_close(y, l0, "vs level-0 order")
    w = IU.unpack_and_reconstruct_w_hip(qd, ud, vd)
    dense = IU.linear_f16_hip(xd, w, bd).cpu().numpy()
    assert_close(y, dense, "vs rebuilt weight x dense kernel", 2e-3, 2e-4)


# up to 128 tokens: sign tiles decoded into LDS and multiplied at once (128 rows x 128 tokens per workgroup): ragged
# rows and tokens, ranks below 16, 1..8 blocks, one strip per column group and many, runs of strips that start and
# end inside a quad of strips (the 64 bytes one sign load brings), a column count that leaves the last group short
PANEL_CASES = [(2, 128, 128, 49, 16), (3, 1000, 1152, 100, 16), (1, 4096, 4096, 128, 16), (8, 4096, 4096, 127, 16),
               (3, 8192, 4096, 120, 16), (2, 4096, 14336, 128, 16), (5, 333, 640, 97, 5), (8, 1024, 4096, 128, 16),
               (4, 130, 2432, 113, 12), (6, 2000, 1024, 97, 1), (7, 700, 512, 120, 16), (8, 14336, 384, 64, 16),
               (7, 256, 4096, 128, 16), (3, 520, 1664, 77, 16)]


@pytest.mark.parametrize("I,M,N,T,K", PANEL_CASES)
def test_forward_panel_kernel_matches_oracle(I, M, N, T, K, prefill_kernel):
    print(f"forward panel kernel I={I} M={M} N={N} T={T} K={K}", flush=True)
    L = _lib.lib()
    prefill_kernel(_lib.PREFILL_PANEL)
    # the path is taken: the scratch is g x ([T, M] partial sums + T sums of squares) for g column groups, not the weight
    need = int(L.bs_workspace_bytes(I, M, N, K, T))
    groups = need // (T * (M + 1) * 4)
    assert groups >= 1 and need == (groups * T * (M + 1) * 4 + 255) // 256 * 256
    q, u, vt, x = synthetic_layer(M, N, I, T, k=K, seed=7 * I + T, signed_factors=True)
    bias = (torch.randn(M, generator=torch.Generator().manual_seed(T)) * 0.05).half() if T % 2 else None
    exact, l0 = oracle_refs(q, u, vt, x, bias)
    qd, ud, vd, xd = q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev())
    bd = None if bias is None else bias.to(dev())
    ws = _lib.workspace(xd.device, need)
    ws[:ws.numel() // 4 * 4].view(torch.float32).fill_(float("nan"))       # an unwritten partial cannot pass by luck
    y = IU.bitstack_forward_hip(qd, ud, vd, xd, bd)
    assert torch.equal(IU.bitstack_forward_hip(qd, ud, vd, xd, bd), y)
    yn = y.cpu().numpy()
    assert yn.dtype == np.float16 and yn.shape == (T, M) and np.isfinite(yn).all()
    assert_close(yn, exact, "vs fp64")
    if I <= 8:
        assert_close(yn, l0, "vs level-0 order")
    # the same rounding points as rebuilding the fp16 weight and multiplying: only the order of the fp32 sums differs
    prefill_kernel(_lib.PREFILL_REBUILD)
    assert int(L.bs_workspace_bytes(I, M, N, K, T)) >= M * N * 2
    dense = IU.bitstack_forward_hip(qd, ud, vd, xd, bd).cpu().numpy()
    assert_close(yn, dense, "vs rebuilt weight x dense kernel", 2e-3, 2e-4)


def test_prefill_kernel_hook_selects_and_rejects(prefill_kernel):
    L = _lib.lib()
    rebuilt = 4096 * 4096 * 2
    prefill_kernel(_lib.PREFILL_REBUILD)
    for T in (49, 64, 128, 256):
        assert L.bs_workspace_bytes(8, 4096, 4096, 16, T) == rebuilt
    assert L.bs_workspace_bytes(8, 4096, 4096, 16, 48) < rebuilt            # the strip kernel below 49 tokens is not affected
    prefill_kernel(_lib.PREFILL_PANEL)
    for T in (49, 64, 128):
        assert L.bs_workspace_bytes(8, 4096, 4096, 16, T) == (8 * T * 4097 * 4 + 255) // 256 * 256   # partial sums of 8 column groups
    assert L.bs_workspace_bytes(8, 4096, 4096, 16, 129) == rebuilt          # beyond its token block
    assert L.bs_workspace_bytes(9, 4096, 4096, 16, 128) == rebuilt          # more blocks than it keeps sign words for
    assert L.bs_workspace_bytes(8, 4096, 4000, 16, 128) == 4096 * 4000 * 2   # N not a multiple of 128
    prefill_kernel(_lib.PREFILL_WALKED)
    assert L.bs_workspace_bytes(8, 4096, 4096, 16, 64) < rebuilt
    assert L.bs_workspace_bytes(8, 4096, 4096, 16, 128) == rebuilt          # the walked kernel stops at 96 tokens
    assert L.bs_set_prefill_kernel(4) < 0 and L.bs_set_prefill_kernel(-1) < 0


def test_planner_picks_walked_strips_then_panel_then_rebuild(prefill_kernel):
    """49..96 tokens: the walked strip kernel where its plan expects to win, else the panel kernel, else the
    rebuilt weight; 97..128 tokens: the panel kernel or the rebuilt weight; the hook pins each."""
    L = _lib.lib()
    path = lambda I, M, N, T: L.bs_forward_path(I, M, N, 16, T)
    assert path(3, 8192, 4096, 64) == _lib.PATH_WALKED        # 512 workgroups: the walked kernel fills the chip
    assert path(8, 4096, 14336, 64) == _lib.PATH_WALKED
    assert path(8, 14336, 4096, 64) == _lib.PATH_PANEL        # 448 workgroups for 512 slots: the walked kernel declines
    assert path(8, 8192, 4096, 64) == _lib.PATH_PANEL         # both take it: six blocks and more on a tall shape go to the panel kernel
    assert path(5, 8192, 4096, 64) == _lib.PATH_WALKED
    assert path(5, 4096, 4096, 96) == _lib.PATH_PANEL and path(4, 4096, 4096, 96) == _lib.PATH_WALKED   # above 80 tokens from five blocks
    assert path(3, 14336, 4096, 64) == _lib.PATH_PANEL
    assert path(20, 4096, 4096, 64) == _lib.PATH_REBUILD      # vt of 20 blocks: no room for two walked workgroups, too many for the panel
    assert path(8, 4096, 4096, 97) == _lib.PATH_PANEL         # seven token tiles: beyond the walked kernel
    assert path(8, 4096, 4096, 128) == _lib.PATH_PANEL
    assert path(9, 4096, 4096, 128) == _lib.PATH_REBUILD
    assert path(8, 4096, 4096, 129) == _lib.PATH_REBUILD
    assert path(3, 4096, 4000, 64) == _lib.PATH_REBUILD       # N not a multiple of 128
    assert path(2, 4096, 4096, 1) == _lib.PATH_DECODE_F16 and path(16, 4096, 4096, 1) == _lib.PATH_DECODE_MX
    assert path(4, 4096, 4096, 16) == _lib.PATH_STRIP and path(4, 4096, 4104, 16) == _lib.PATH_REBUILD
    prefill_kernel(_lib.PREFILL_REBUILD)
    assert path(8, 4096, 4096, 64) == _lib.PATH_REBUILD and path(4, 4096, 4096, 16) == _lib.PATH_STRIP
    prefill_kernel(_lib.PREFILL_PANEL)
    assert path(8, 4096, 4096, 64) == _lib.PATH_PANEL
    prefill_kernel(_lib.PREFILL_WALKED)
    assert path(8, 14336, 4096, 64) == _lib.PATH_WALKED       # pinned where its own plan would decline
    assert path(8, 4096, 4096, 128) == _lib.PATH_REBUILD


@pytest.mark.parametrize("I,M,N,T,K", STRIP_CASES)
def test_forward_few_dozen_tokens_matches_oracle(I, M, N, T, K):
    print(f"forward strips I={I} M={M} N={N} T={T} K={K}", flush=True)
    assert _lib.decode_plan(I, M, N, K, T)[0] == 0        # not the decode kernel
    q, u, vt, x = synthetic_layer(M, N, I, T, k=K, seed=3 * I + T, signed_factors=True)
    bias = (torch.randn(M, generator=torch.Generator().manual_seed(T)) * 0.05).half() if T % 2 else None
    exact, l0 = oracle_refs(q, u, vt, x, bias)
    qd, ud, vd, xd = q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev())
    y = IU.bitstack_forward_hip(qd, ud, vd, xd, None if bias is None else bias.to(dev())).cpu().numpy()
    assert y.dtype == np.float16 and y.shape == (T, M)
    assert_close(y, exact, "vs fp64")
    if I <= 8:      # with more blocks the level-0 order's own fp16 sums are further from fp64 than the bound
        assert_close(y, l0, "vs level-0 order")
    # the same rounding points as rebuilding the fp16 weight and multiplying: only the order of the
    # fp32 sums differs
    w = IU.unpack_and_reconstruct_w_hip(qd, ud, vd)
    dense = IU.linear_f16_hip(xd, w, None if bias is None else bias.to(dev())).cpu().numpy()
    assert_close(y, dense, "vs rebuilt weight x dense kernel", 2e-3, 2e-4)


PREFILL_CASES = [(2, 256, 512, 16), (8, 1024, 4096, 16), (4, 1024, 1024, 128), (2, 300, 1024, 100),
                 (8, 4096, 4096, 128), (2, 512, 1024, 512)]


@pytest.mark.parametrize("I,M,N,T", PREFILL_CASES)
def test_forward_prefill_matches_oracle(I, M, N, T):
    print(f"forward prefill I={I} M={M} N={N} T={T}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=I + T)
    exact, l0 = oracle_refs(q, u, vt, x)
    y = IU.bitstack_forward_hip(q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev())).cpu().numpy()
    assert y.shape == (T, M)
    assert_close(y, exact, "vs fp64")
    assert_close(y, l0, "vs level-0 order")


def test_linear_f16_matches_torch_fp32():
    g = torch.Generator().manual_seed(0)
    for (T, M, N, b) in [(1, 64, 128, False), (130, 200, 264, True), (256, 256, 512, True), (33, 17, 40, False)]:
        x = torch.randn(T, N, generator=g).half().to(dev())
        w = (torch.randn(M, N, generator=g) * 0.05).half().to(dev())
        bias = torch.randn(M, generator=g).half().to(dev()) if b else None
        want = x.float() @ w.float().T + (bias.float() if b else 0)
        got = IU.linear_f16_hip(x, w, bias)
        assert_close(got.float().cpu().numpy(), want.cpu().numpy(), f"linear {T}x{M}x{N}", 2e-3, 5e-4)


# ------------------------------------------------- properties at full size
def test_full_size_properties_largest_decode_shape():
    """14336 x 4096 with 16 blocks: too big for the CPU oracle in seconds, so
    check what must hold whatever the values are."""
    I, M, N = 16, 14336, 4096
    q, u, vt, x = synthetic_layer(M, N, I, 1, seed=9, device=dev())
    f = IU.bitstack_forward_hip
    y = f(q, u, vt, x).float()
    # determinism
    assert torch.equal(f(q, u, vt, x).float(), y)
    # linearity in x (vt * x is rounded to fp16, so products that fall below the
    # fp16 normal range do not double exactly: compare within the output rounding)
    assert float((f(q, u, vt, x * 2).float() - 2 * y).abs().max()) <= 2e-3 * float(y.abs().max())
    # block additivity: the stack equals the sum of its halves (fp16 output rounding only)
    parts = f(q[:8], u[:8], vt[:8], x).float() + f(q[8:], u[8:], vt[8:], x).float()
    assert float((parts - y).abs().max()) <= 2e-3 * float(y.abs().max())
    # complementing the sign bytes of every block negates the output (the decode is
    # not symmetric in the bit value, so only up to fp32 summation order)
    assert float((f(~q, u, vt, x).float() + y).abs().max()) <= 1e-3 * float(y.abs().max())
    # T = 4 rows are the four T = 1 answers
    x4 = torch.cat([x, x * 0.5, -x, x * 0.25])
    y4 = f(q, u, vt, x4).float()
    assert float((y4[0] - y[0]).abs().max()) <= 1e-3 * float(y.abs().max())
    assert float((y4[2] + y[0]).abs().max()) <= 1e-3 * float(y.abs().max())
    # spot rows against the fp64 closed form
    rows = [0, 1, 4095, 7777, 14335]
    exact = O.forward_exact(np.stack([qq.cpu().numpy().reshape(M, N // 8)[rows].reshape(-1) for qq in q]),
                            u[:, rows].cpu().numpy(), vt.cpu().numpy(), x.cpu().numpy())
    assert_close(y[:, rows].cpu().numpy(), exact, "spot rows vs fp64", 1e-2, 1e-3)


@pytest.mark.parametrize("M,N", [(28672, 8192), (8192, 28672), (8192, 8192), (1024, 8192)])
def test_llama_70b_shapes_spot_rows_on_every_path(M, N):
    """The four linear shapes of the 70B configuration with 3 blocks, at 1, 4, 8 and 64 tokens (decode
    kernel, strip kernel, rebuild + dense kernel): sampled rows against the float64 closed form, and the
    paths against one another over all rows."""
    I = 3
    q, u, vt, x = synthetic_layer(M, N, I, 64, seed=31, device=dev())
    rows = [0, 1, 63, 64, M // 2 + 5, M - 2, M - 1]
    exact = O.forward_exact(np.stack([qq.cpu().numpy().reshape(M, N // 8)[rows].reshape(-1) for qq in q]),
                            u[:, rows].cpu().numpy(), vt.cpu().numpy(), x.cpu().numpy())
    f = IU.bitstack_forward_hip
    plans = {T: _lib.decode_plan(I, M, N, 16, T)[0] for T in (1, 4, 8, 64)}
    assert plans[1] > 0 and plans[4] > 0 and plans[8] == 0 and plans[64] == 0      # decode kernel up to 4 tokens only
    ys = {}
    for T in (1, 4, 8, 64):
        print(f"70B shape M={M} N={N} I={I} T={T}", flush=True)
        y = f(q, u, vt, x[:T].contiguous())
        assert tuple(y.shape) == (T, M)
        assert_close(y[:, rows].cpu().numpy(), exact[:T], f"T={T} spot rows vs fp64", 1e-2, 1e-3)
        ys[T] = y.float()
    scale = float(ys[64].abs().max())
    for T in (1, 4, 8):
        assert float((ys[T] - ys[64][:T]).abs().max()) <= 4e-3 * scale, T


# ------------------------------------------------------------ module levels
def build_module(M, N, I, bias, seed):
    q, u, vt, x = synthetic_layer(M, N, I, 3, seed=seed, signed_factors=True)
    mod = BitStackLinear(I, N, M, 16, bias, False, "cpu")
    for i in range(I):
        getattr(mod, f"qweight_{i}").copy_(q[i])
        getattr(mod, f"u_{i}").copy_(u[i] * 10)
        getattr(mod, f"vt_{i}").copy_(vt[i] * 10)
    if bias:
        mod.bias.copy_((torch.randn(M, generator=torch.Generator().manual_seed(seed)) * 0.01).half())
    return mod, x


def test_full_size_properties_strip_kernel():
    """The same for the 5..48-token path at 14336 x 4096 with 8 blocks."""
    I, M, N = 8, 14336, 4096
    q, u, vt, x = synthetic_layer(M, N, I, 16, seed=10, device=dev())
    f = IU.bitstack_forward_hip
    assert _lib.decode_plan(I, M, N, 16, 16)[0] == 0
    y = f(q, u, vt, x)
    assert torch.equal(f(q, u, vt, x), y)                                   # determinism
    # tokens do not interact: the first eight rows are the 8-token answer, bit for bit
    assert torch.equal(f(q, u, vt, x[:8].contiguous()), y[:8])
    # and a 40-token call (three token tiles) repeats them
    x40 = torch.cat([x, x, x[:8]])
    y40 = f(q, u, vt, x40)
    yf = y.float()
    scale = float(yf.abs().max())
    # (three token tiles leave room for fewer strips per workgroup, so the strips' partial sums are
    # added in other groups: the same numbers up to the fp32 summation order)
    assert torch.equal(y40[:16], y40[16:32]) and torch.equal(y40[32:], y40[:8])
    assert float((y40[:16].float() - yf).abs().max()) <= 1e-3 * scale
    assert float((f(q, u, vt, x * 2).float() - 2 * yf).abs().max()) <= 2e-3 * scale           # linearity in x
    parts = f(q[:4], u[:4], vt[:4], x).float() + f(q[4:], u[4:], vt[4:], x).float()
    assert float((parts - yf).abs().max()) <= 4e-3 * scale                                    # block additivity (w is rounded per call)
    assert float((f(~q, u, vt, x).float() + yf).abs().max()) <= 1e-3 * scale                  # complemented signs negate
    # the decode kernel gives the same numbers up to the rounding points (it never rounds w)
    y1 = torch.cat([f(q, u, vt, x[t:t + 1].contiguous()) for t in range(4)]).float()
    assert float((y1 - yf[:4]).abs().max()) <= 4e-3 * scale


@pytest.mark.parametrize("bias", [False, True])
def test_module_levels_agree_with_level0(bias):
    M, N, I = 256, 1024, 4
    mod, x = build_module(M, N, I, bias, 21)
    y0_cpu = mod(x)                                     # level 0 on the CPU
    mod = mod.to(dev())
    xd = x.to(dev())
    y0 = mod(xd)                                        # level 0 on the GPU (torch ops)
    assert_close(y0.cpu().numpy(), y0_cpu.numpy(), "level0 gpu vs cpu", 2e-3, 5e-4)
    mod.stack_blocks()
    for level in (1, 2, 3, 4, 5):
        mod.fused_level = level
        y = mod(xd)
        assert y.dtype == torch.float16 and tuple(y.shape) == (3, M)
        assert_close(y.cpu().numpy(), y0_cpu.numpy(), f"level {level} vs level 0")
        y3 = mod(xd.view(1, 3, N))
        assert tuple(y3.shape) == (1, 3, M) and torch.equal(y3.view(3, M), y)
    # any-size: fewer blocks through the same stacked buffers
    mod.fused_level = 5
    mod.set_bit(2)
    q2 = torch.stack([mod.qweight[i] for i in range(2)]).cpu()
    exact = C.forward_f64(q2.numpy(), mod.u[:2].cpu().numpy(), mod.vt[:2].cpu().numpy(), x.numpy(),
                          None if not bias else mod.bias.cpu().numpy())
    assert_close(mod(xd).cpu().numpy(), exact, "w_bit=2 vs fp64")
    mod.set_bit(9)
    with pytest.raises(RuntimeError, match="exceeds"):
        mod(xd)


@pytest.mark.parametrize("bias", [False, True])
def test_empty_and_ragged_inputs(bias):
    """No tokens, no blocks, odd leading dimensions: the shapes torch's F.linear accepts at level 0
    (BitStackLinear.py:105-114) give the same shapes and values at every level."""
    M, N, I = 96, 512, 3
    mod, x = build_module(M, N, I, bias, 23)
    mod = mod.to(dev())
    xd = x.to(dev())
    for level in (0, 1, 2, 3, 4, 5):
        mod.fused_level = level
        mod.set_bit(I)
        if level == 1:
            mod.stack_blocks()                          # level 0 reads the per-block buffers, the others the stacked ones
        for shape in ((0, N), (2, 0, N), (0, 3, N)):
            y = mod(torch.empty(shape, dtype=torch.float16, device=dev()))
            assert y.dtype == torch.float16 and tuple(y.shape) == shape[:-1] + (M,)
        # 1 x 1 x N and 5 x 1 x N: one token and five may run different kernels, same numbers up to the rounding points
        y1 = mod(xd[:1].view(1, 1, N))
        assert tuple(y1.shape) == (1, 1, M)
        y5 = mod(xd.repeat(2, 1)[:5].view(5, 1, N))
        assert tuple(y5.shape) == (5, 1, M)
        assert float((y5[0, 0].float() - y1[0, 0].float()).abs().max()) <= 4e-3 * float(y1.float().abs().max())
        # no blocks at all: w = 0, the output is the bias (or zero)
        mod.set_bit(0)
        y = mod(xd)
        want = mod.bias.expand(3, M) if bias else torch.zeros(3, M, dtype=torch.float16, device=dev())
        assert torch.equal(y, want), level


def test_non_contiguous_input_is_handled():
    q, u, vt, x = synthetic_layer(128, 512, 2, 4, seed=4, device=dev())
    wide = torch.randn(4, 1024, device=dev()).half()
    wide[:, ::2] = x
    y = IU.bitstack_forward_hip(q, u, vt, wide[:, ::2])
    assert torch.equal(y, IU.bitstack_forward_hip(q, u, vt, x))


# ------------------------------------------------------------- decomposition on the GPU
def test_decompose_on_gpu_matches_oracle():
    """from_linear on a HIP tensor (BitStackLinear.py:49-86): SVD through torch (rocSOLVER), signs
    packed by the HIP kernel.  Factors are only defined up to a joint sign per rank, so products
    are compared; the first block's signs are those of the weight itself and must match bit for bit."""
    print("decompose on gpu", flush=True)
    torch.manual_seed(0)
    lin = torch.nn.Linear(192, 256, bias=True)
    with torch.no_grad():
        lin.weight.mul_(0.5)
    lin = lin.half()                      # the reference decomposes fp16 checkpoints
    w = lin.weight.detach().float().numpy().copy()
    q_ref, u_ref, vt_ref, norms = O.decompose_weight(w, 3, 8)
    with torch.no_grad():                 # as the reference's decompose() (bitstack/utils/decompose.py:7)
        mod = BitStackLinear.from_linear(lin.to(dev()), w_bit=3, k=8, bias=True, fused_level=5, name="t")
    assert mod.qweight_0.is_cuda and mod.u_0.dtype == torch.float16
    assert np.array_equal(mod.qweight_0.cpu().numpy(), q_ref[0])
    res = w.astype(np.float64)
    for i in range(3):
        p_gpu = getattr(mod, f"u_{i}").double().cpu().numpy() @ getattr(mod, f"vt_{i}").double().cpu().numpy()
        p_ref = u_ref[i].astype(np.float64) @ vt_ref[i].astype(np.float64)
        assert np.abs(p_gpu - p_ref).max() <= 2e-3 * np.abs(p_ref).max(), i
        s = O.unpack_sign(getattr(mod, f"qweight_{i}").cpu().numpy(), w.shape).astype(np.float64)
        res = res - s * p_gpu
        # the residual shrinks like the oracle's (Eckart-Young step by step)
        assert abs(np.linalg.norm(res) - norms[i + 1]) <= 2e-2 * norms[i + 1], i
    mod.stack_blocks()
    x = torch.randn(2, 192, generator=torch.Generator().manual_seed(1)).half()
    y = mod(x.to(dev())).float().cpu().numpy()
    want = x.double().numpy() @ (w.astype(np.float64) - res).T + lin.bias.detach().double().cpu().numpy()
    assert_close(y, want, "decomposed layer forward vs fp64")


def test_single_layer_4096_decomposed_from_gaussian_weight():
    """The reference's own CPU-runnable case at full size: W 4096 x 4096 fp32 ~ N(0, 0.02^2), seed 0,
    four residual blocks of rank 16 (decomposed on the device), x 1 x 4096 fp16 ~ N(0, 1), all blocks
    loaded; every fused level against the float64 closed form and against level 0."""
    print("single layer 4096 x 4096, niter 4, k 16", flush=True)
    M = N = 4096
    g = torch.Generator().manual_seed(0)
    w = torch.randn(M, N, generator=g) * 0.02
    x = torch.randn(1, N, generator=g).half()
    lin = torch.nn.Linear(N, M, bias=False)
    with torch.no_grad():
        lin.weight.copy_(w)
        mod = BitStackLinear.from_linear(lin.to(dev()), w_bit=4, k=16, bias=False, fused_level=0, name="single")
    q = np.stack([getattr(mod, f"qweight_{i}").cpu().numpy() for i in range(4)])
    u = np.stack([getattr(mod, f"u_{i}").cpu().numpy() for i in range(4)])
    vt = np.stack([getattr(mod, f"vt_{i}").cpu().numpy() for i in range(4)])
    wn = w.numpy()
    # block 0 holds the signs of W itself, bit for bit; its product is the best rank-16 fit of |W|
    assert np.array_equal(q[0], O.pack_sign(np.where(wn >= 0, 1, -1).astype(np.int8)))
    uu, sv, vv = np.linalg.svd(np.abs(wn).astype(np.float64), full_matrices=False)
    best = (uu[:, :16] * sv[:16]) @ vv[:16]
    assert np.abs(u[0].astype(np.float64) @ vt[0].astype(np.float64) - best).max() <= 4e-3 * np.abs(best).max()
    # the approximation error falls with every block loaded
    errs = [float(np.linalg.norm(O.reconstruct_w_exact(q[:b], u[:b], vt[:b]) - wn) / np.linalg.norm(wn)) for b in (1, 2, 3, 4)]
    print("relative error of the rebuilt weight with 1..4 blocks:", [round(e, 4) for e in errs], flush=True)
    assert errs[0] > errs[1] > errs[2] > errs[3] and errs[0] < 0.65 and errs[3] < 0.2
    exact = x.double().numpy() @ O.reconstruct_w_exact(q, u, vt).T
    xd = x.to(dev())
    y0 = mod(xd)                                        # level 0: torch ops, fp16 sums
    assert_close(y0.cpu().numpy(), exact, "level 0 vs fp64")
    mod.stack_blocks()
    for level in (1, 2, 3, 4, 5):
        mod.fused_level = level
        y = mod(xd.view(1, 1, N)).view(1, M)
        assert_close(y.cpu().numpy(), exact, f"level {level} vs fp64")
        assert_close(y.cpu().numpy(), y0.cpu().numpy(), f"level {level} vs level 0")
    # and the layer does what the dense one did, to the accuracy four blocks give
    dense = x.double().numpy() @ wn.astype(np.float64).T
    mx, mn = rel_errors(y.cpu().numpy(), dense)
    print(f"level 5 vs the dense layer: max_rel={mx:.3f} mean_rel={mn:.3f}", flush=True)
    assert mn < 0.3


# ------------------------------------------------------------- seeded random shapes
def _random_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        kind = rng.integers(0, 4)
        if kind == 0:      # decode kernel shapes: N a multiple of 512, any M
            N = 512 * int(rng.integers(1, 9)); M = int(rng.integers(1, 700)); T = int(rng.integers(1, 9))
        elif kind == 1:    # tiled rebuild + GEMM: N a multiple of 128, more tokens
            N = 128 * int(rng.integers(1, 12)); M = int(rng.integers(1, 500)); T = int(rng.integers(9, 200))
        elif kind == 2:    # N only a multiple of 8: generic rebuild, k-tail GEMM / skinny
            N = 8 * int(rng.integers(1, 90)); M = int(rng.integers(1, 300)); T = int(rng.integers(1, 70))
        else:              # tall matrices through the 8-wave decode kernels
            N = 512 * int(rng.integers(1, 4)); M = 512 * int(rng.integers(1, 5)) + int(rng.integers(0, 3)) * 7; T = int(rng.integers(1, 5))
        cases.append((int(rng.integers(1, 7)), M, N, T, int(rng.choice([16, 16, 16, 8, 3]))))
    return cases


@pytest.mark.parametrize("I,M,N,T,K", _random_cases(48, 20240607))
def test_forward_random_shapes(I, M, N, T, K):
    print(f"forward random I={I} M={M} N={N} T={T} K={K}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, k=K, seed=M + N + T, signed_factors=True)
    bias = (torch.randn(M, generator=torch.Generator().manual_seed(I)) * 0.05).half() if (M + T) % 2 else None
    exact, _ = oracle_refs(q, u, vt, x, bias)
    y = IU.bitstack_forward_hip(q.to(dev()), u.to(dev()), vt.to(dev()), x.to(dev()),
                                None if bias is None else bias.to(dev())).cpu().numpy()
    assert y.shape == (T, M)
    assert_close(y, exact, "vs fp64")


# ------------------------------------------------------------- beyond 2^31 elements
def test_unpack_more_than_2_31_signs():
    """The reference splits its launches above 2^31 - 1 elements (bitstack/utils/pack_utils.py:181-194);
    here one call with 64-bit indices.  2^31 + 40 signs, compared with numpy.unpackbits on windows at the
    start, around every multiple of 2^29 elements up to and across the 2^31 boundary, and at the end."""
    n = (1 << 31) + 40
    print(f"unpack n={n}", flush=True)
    g = torch.Generator(device=dev()).manual_seed(31)
    packed = torch.randint(0, 256, ((n + 7) // 8,), dtype=torch.uint8, device=dev(), generator=g)
    out = PU.unpack_sign_hip(packed, (n,))
    assert out.dtype == torch.int8 and out.numel() == n
    span = 1 << 16                                          # bytes per window
    starts = [0] + [k * (1 << 26) - span // 2 for k in range(1, 5)] + [packed.numel() - span]
    for b0 in starts:
        want = np.unpackbits(packed[b0:b0 + span].cpu().numpy(), bitorder="big").astype(np.int8) * 2 - 1
        got = out[8 * b0:8 * (b0 + span)].cpu().numpy()
        assert np.array_equal(got, want[:got.size]), b0
    # nothing but +-1 anywhere, and as many +1 as there are set bits (a window written twice or skipped
    # would change the count); summed in slabs to bound the temporaries
    ones = 0
    for s0 in range(0, n, 1 << 28):
        sl = out[s0:s0 + (1 << 28)]
        assert bool(((sl == 1) | (sl == -1)).all())
        ones += int((sl == 1).sum())
    lut = torch.tensor([bin(v).count("1") for v in range(256)], device=dev())
    bits = 0
    for s0 in range(0, packed.numel(), 1 << 26):
        bits += int(lut[packed[s0:s0 + (1 << 26)].long()].sum())
    assert ones == bits


def test_forward_with_2_31_weights_takes_the_rebuild_path():
    """M * N = 2^31: the decode kernel keeps per-block byte offsets in 32 bits and declines; the call must
    still be right through the rebuilt weight (one block, one token and six)."""
    I, M, N = 1, 32768, 65536
    print(f"forward M*N=2^31 I={I} M={M} N={N}", flush=True)
    assert _lib.decode_plan(I, M, N, 16, 1)[0] == 0
    g = torch.Generator(device=dev()).manual_seed(7)
    q = torch.randint(0, 256, (I, M * N // 8), dtype=torch.uint8, device=dev(), generator=g)
    u = (torch.randn(I, M, 16, device=dev(), generator=g).abs() * 0.01).half()
    vt = (torch.randn(I, 16, N, device=dev(), generator=g).abs() * 0.01).half()
    x = torch.randn(6, N, device=dev(), generator=g).half()
    rows = [0, 1, 16383, 16384, 16385, M - 1]               # rows either side of byte offset 2^27 * 8 and the last one
    qs = np.stack([qq.view(M, N // 8)[rows].reshape(-1).cpu().numpy() for qq in q])
    exact = O.forward_exact(qs, u[:, rows].cpu().numpy(), vt.cpu().numpy(), x.cpu().numpy())
    for T in (1, 6):
        y = IU.bitstack_forward_hip(q, u, vt, x[:T].contiguous())
        assert tuple(y.shape) == (T, M)
        assert_close(y[:, rows].cpu().numpy(), exact[:T], f"T={T} spot rows vs fp64")
    # the last rows of the weight itself, bit for bit against the C oracle's fp32 rebuild order within one ulp
    w = IU.unpack_and_reconstruct_w_hip(q, u, vt)
    tail = C.reconstruct_w(qs[:, -N // 8:].copy(), u[:, M - 1:].cpu().numpy(), vt.cpu().numpy())
    got = w[M - 1:].cpu().numpy()
    assert np.all(np.abs(got.astype(np.float64) - tail.astype(np.float64)) <= np.spacing(np.abs(tail)).astype(np.float64))


# ------------------------------------------------------------- seeded random shapes, every kernel choice forced
def _random_forced_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        kind = rng.integers(0, 5)
        if kind == 0:      # decode kernels, many blocks (long partial-sum lists)
            N = 512 * int(rng.integers(1, 9)); M = int(rng.integers(1, 3000)); T = int(rng.integers(1, 5)); I = int(rng.integers(1, 40))
        elif kind == 1:    # one and two tokens on wide matrices (several units per workgroup), up to the widest 8B layer
            N = 512 * int(rng.integers(1, 29)); M = 64 * int(rng.integers(1, 120)); T = int(rng.integers(1, 3)); I = int(rng.integers(1, 20))
        elif kind == 2:    # strip kernel
            N = 128 * int(rng.integers(1, 40)); M = int(rng.integers(1, 2500)); T = int(rng.integers(5, 49)); I = int(rng.integers(1, 12))
        elif kind == 3:    # rebuild + dense, ragged everything
            N = 8 * int(rng.integers(1, 300)); M = int(rng.integers(1, 1500)); T = int(rng.integers(1, 700)); I = int(rng.integers(1, 6))
        else:              # either side of the token count where the vendor GEMM takes over
            N = 1024 * int(rng.integers(1, 5)); M = 512 * int(rng.integers(1, 9)); T = int(rng.choice([1, 2, 48, 49, 600, 1024])); I = int(rng.integers(1, 10))
        cases.append((I, M, N, T, int(rng.choice([16, 16, 16, 12, 5, 1])), int(rng.integers(0, 3)), int(rng.integers(0, 3))))
    return cases


@pytest.mark.parametrize("I,M,N,T,K,decode_mode,dense_mode", _random_forced_cases(72, 20250309))
def test_forward_random_shapes_forced_kernels(I, M, N, T, K, decode_mode, dense_mode, decode_kernel):
    """bs_forward with the decode kernel (planned / fp16 / block-scaled) and the dense kernel (planned / own /
    hipBLASLt) forced at random, against a float64 evaluation of the closed form on the GPU (signs through
    the bit-exact unpack kernel): deterministic, and within the stated tolerance whatever runs the shape."""
    print(f"forward random forced I={I} M={M} N={N} T={T} K={K} decode={decode_mode} dense={dense_mode}", flush=True)
    from bitstack_amd.utils import pack_utils as PU
    g = torch.Generator(device=dev()).manual_seed(I * 7 + M + N + T)
    q = torch.randint(0, 256, (I, (M * N + 7) // 8), dtype=torch.uint8, device=dev(), generator=g)
    sc = (0.02 / torch.arange(1, I + 1, device=dev()).float()).view(I, 1, 1)
    u = (torch.randn(I, M, K, device=dev(), generator=g) * sc).half()
    vt = (torch.randn(I, K, N, device=dev(), generator=g) * sc.sqrt()).half()
    x = torch.randn(T, N, device=dev(), generator=g).half()
    bias = (torch.randn(M, device=dev(), generator=g) * 0.01).half() if (M + T) % 3 == 0 else None
    decode_kernel(decode_mode)
    assert _lib.lib().bs_set_dense_kernel(dense_mode) == 0
    try:
        y = IU.bitstack_forward_hip(q, u, vt, x, bias)
        assert torch.equal(IU.bitstack_forward_hip(q, u, vt, x, bias), y)
    finally:
        _lib.lib().bs_set_dense_kernel(_lib.DENSE_AUTO)
    w = torch.zeros(M, N, device=dev(), dtype=torch.float64)
    for i in range(I):
        w += PU.unpack_sign(q[i], (M, N)).double() * (u[i].double() @ vt[i].double())
    want = x.double() @ w.T
    if bias is not None:
        want = want + bias.double()
    assert_close(y.cpu().numpy(), want.cpu().numpy(), "vs float64 on the GPU")
