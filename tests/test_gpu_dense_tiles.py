"""Parity of the large workgroup tiles of the dense kernel (256 x 256, 128 x 256, 128 x 128 and their
partial-k-step twins) and of the prefill configurations that run on them: the four Llama-3.1-8B linear
shapes at 512 and 2048 tokens with 8 blocks, and a 70B shape at 2048 x 8 = 16384 tokens.  Every case
first asserts, through bs_linear_plan, that it runs the tile it is meant to cover."""
import numpy as np
import pytest
import torch

from bitstack_amd import _lib
from bitstack_amd.utils import inference_utils as IU
from bitstack_amd.utils.synthetic import synthetic_layer
from oracle import bitstack_oracle as O

pytestmark = pytest.mark.gpu

MAX_REL, MEAN_REL = 1e-2, 1e-3


def dev():
    return torch.device("cuda:0")


@pytest.fixture(params=[_lib.DENSE_OWN, _lib.DENSE_LIBRARY], ids=["own_kernel", "hipblaslt"])
def dense_kernel(request):
    """bs_forward's large-T path with this library's dense kernel, then with hipBLASLt, behind the same rebuild."""
    assert _lib.lib().bs_set_dense_kernel(request.param) == 0
    yield request.param
    assert _lib.lib().bs_set_dense_kernel(_lib.DENSE_AUTO) == 0


def rel(got, ref):
    got, ref = got.double(), ref.double()
    d = (got - ref).abs()
    return float(d.max() / ref.abs().max()), float(d.mean() / ref.abs().mean())


def small_tile_linear(x, w, bias, t_rng, m_rng):
    """The same product for a sub-block of the output through the 64 x 64 tile (a call small enough
    that the launcher picks it), the kernel every other dense test covers."""
    (t0, t1), (m0, m1) = t_rng, m_rng
    assert _lib.linear_plan(t1 - t0, m1 - m0, x.shape[1])[:2] == (64, 64)
    return IU.linear_f16_hip(x[t0:t1].contiguous(), w[m0:m1].contiguous(), None if bias is None else bias[m0:m1].contiguous())


# (tokens, out features, in features, expected tile, partial last k-step)
TILE_CASES = [
    (2048, 14336, 4096, (256, 256), 0),
    (2047, 14335, 4096, (256, 256), 0),        # ragged tokens and features
    (1024, 14336, 4104, (256, 256), 1),        # N % 32 != 0
    (1024, 14336, 4128, (256, 256), 0),        # N % 64 != 0: k-steps of 32
    (16384, 8192, 8192, (256, 256), 0),        # the 70B prefill of 2048 tokens x 8 sequences
    (2048, 4096, 4096, (128, 256), 0),
    (512, 14336, 4096, (128, 256), 0),
    (2048, 4096, 14336, (128, 256), 0),
    (500, 14333, 4096, (128, 256), 0),         # ragged
    (1024, 8192, 4000, (128, 256), 1),         # N % 64 != 0
    (1024, 4096, 4096, (128, 128), 0),
    (1000, 4090, 4096, (128, 128), 0),         # ragged
    (1024, 4096, 4040, (128, 128), 1),         # N % 64 != 0
]


@pytest.mark.parametrize("T,M,N,tile,ktail", TILE_CASES)
def test_dense_large_tiles_match_fp32_and_the_small_tile(T, M, N, tile, ktail):
    print(f"dense tile T={T} M={M} N={N} tile={tile} ktail={ktail}", flush=True)
    plan = _lib.linear_plan(T, M, N)
    assert plan[:2] == tile and plan[3] == ktail, plan
    g = torch.Generator(device=dev()).manual_seed(T + M + N)
    x = torch.randn(T, N, device=dev(), generator=g).half()
    w = (torch.randn(M, N, device=dev(), generator=g) * 0.05).half()
    bias = torch.randn(M, device=dev(), generator=g).half() if (T + M) % 2 else None
    y = IU.linear_f16_hip(x, w, bias)
    assert y.dtype == torch.float16 and tuple(y.shape) == (T, M)
    assert torch.equal(IU.linear_f16_hip(x, w, bias), y)                    # deterministic
    # against an fp32 product of the same fp16 operands (rows in slabs to bound the fp32 copies)
    worst_max = worst_mean = 0.0
    wf = w.float()
    for t0 in range(0, T, 2048):
        want = x[t0:t0 + 2048].float() @ wf.T
        if bias is not None:
            want += bias.float()
        mx, mn = rel(y[t0:t0 + 2048], want)
        worst_max, worst_mean = max(worst_max, mx), max(worst_mean, mn)
    print(f"  vs fp32: max_rel={worst_max:.3e} mean_rel={worst_mean:.3e}", flush=True)
    assert worst_max <= 2e-3 and worst_mean <= 5e-4
    # against the 64 x 64 tile on sub-blocks that include the ragged edges: the same exact products
    # summed in fp32 in another order, then the same single rounding
    blocks = [((0, 256), (0, 512)), ((max(T - 200, 0), T), (max(M - 500, 0), M)),
              ((T // 2 - 100, T // 2 + 156), (M // 2 - 250, M // 2 + 262))]
    for t_rng, m_rng in blocks:
        small = small_tile_linear(x, w, bias, t_rng, m_rng)
        part = y[t_rng[0]:t_rng[1], m_rng[0]:m_rng[1]]
        mx, mn = rel(part, small)
        assert mx <= 1e-3 and mn <= 5e-5, (t_rng, m_rng, mx, mn)
        assert float((part != small).float().mean()) < 0.05                   # all but a few last-bit ties agree


def test_dense_rows_too_long_for_32_bit_tile_offsets_take_the_generic_kernel():
    """The tiled kernels address a tile's rows by 32-bit byte offsets from its origin (256 rows x N x 2 bytes must stay
    below 4 GiB): from 2^23 columns the one-output-per-wave kernel runs instead, with the same result."""
    T, M, N = 2, 3, (1 << 23) + 64
    assert _lib.linear_plan(T, M, N)[:2] == (0, 0) and _lib.linear_plan(T, M, (1 << 23) - 64)[:2] != (0, 0)
    g = torch.Generator(device=dev()).manual_seed(5)
    x = (torch.randn(T, N, device=dev(), generator=g) * 0.05).half()
    w = (torch.randn(M, N, device=dev(), generator=g) * 0.05).half()
    y = IU.linear_f16_hip(x, w, None)
    want = x.double() @ w.double().T
    mx, mn = rel(y, want)
    print(f"dense N={N}: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= 2e-3 and mn <= 1e-3


def spot_rows_exact(q, u, vt, x, rows, bias=None):
    M, N = u.shape[1], vt.shape[2]
    qs = np.stack([qq.cpu().numpy().reshape(M, N // 8)[rows].reshape(-1) for qq in q])
    out = O.forward_exact(qs, u[:, rows].cpu().numpy(), vt.cpu().numpy(), x.cpu().numpy())
    if bias is not None:
        out = out + bias[rows].double().cpu().numpy()
    return out


@pytest.mark.parametrize("T", [512, 2048])
@pytest.mark.parametrize("M,N", [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)])
def test_forward_prefill_8b_shapes_8_blocks(M, N, T, dense_kernel):
    """Prefill / batched contraction on the 8B shapes with 8 blocks, 512 and 2048 tokens: sampled rows
    against the float64 closed form at the stated tolerance, the whole output against the vendor GEMM on
    the same rebuilt weight, and sub-blocks against the small dense tile."""
    I = 8
    print(f"prefill 8B shape M={M} N={N} I={I} T={T} tile={_lib.linear_plan(T, M, N)}", flush=True)
    assert _lib.decode_plan(I, M, N, 16, T)[0] == 0
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=M // 7 + T, device=dev())
    y = IU.bitstack_forward_hip(q, u, vt, x)
    assert tuple(y.shape) == (T, M) and torch.equal(IU.bitstack_forward_hip(q, u, vt, x), y)
    rows = [0, 1, 127, 128, 255, 256, M // 2 + 3, M - 257, M - 2, M - 1]
    exact = spot_rows_exact(q, u, vt, x, rows)
    mx, mn = rel(y[:, rows].cpu(), torch.from_numpy(exact))
    print(f"  spot rows vs fp64: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= MAX_REL and mn <= MEAN_REL
    w = IU.unpack_and_reconstruct_w_hip(q, u, vt)
    vendor = torch.nn.functional.linear(x, w)
    mx, mn = rel(y, vendor)
    print(f"  vs F.linear on the rebuilt weight: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= 2e-3 and mn <= 2e-4
    small = small_tile_linear(x, w, None, (T - 256, T), (M - 512, M))
    mx, mn = rel(y[T - 256:, M - 512:], small)
    assert mx <= 1e-3 and mn <= 5e-5


@pytest.mark.parametrize("M,N,I", [(8192, 8192, 3), (28672, 8192, 2)])
def test_forward_prefill_70b_shape_16384_tokens(M, N, I, dense_kernel):
    """The 70B configuration's prompt pass: every linear sees 2048 x 8 = 16384 tokens at once."""
    T = 16384
    print(f"prefill 70B shape M={M} N={N} I={I} T={T} tile={_lib.linear_plan(T, M, N)}", flush=True)
    assert _lib.linear_plan(T, M, N)[:2] == (256, 256)
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=70, device=dev())
    bias = (torch.randn(M, device=dev()) * 0.01).half()
    y = IU.bitstack_forward_hip(q, u, vt, x, bias)
    rows = [0, 255, 256, M // 2 + 9, M - 1]
    tok = list(range(0, 64)) + list(range(T // 2 - 32, T // 2 + 32)) + list(range(T - 64, T))
    exact = spot_rows_exact(q, u, vt, x[tok], rows, bias)
    mx, mn = rel(y[tok][:, rows].cpu(), torch.from_numpy(exact))
    print(f"  spot rows vs fp64: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= MAX_REL and mn <= MEAN_REL
    w = IU.unpack_and_reconstruct_w_hip(q, u, vt)
    vendor = torch.nn.functional.linear(x, w, bias)
    mx, mn = rel(y, vendor)
    print(f"  vs F.linear on the rebuilt weight: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= 2e-3 and mn <= 2e-4


def forward_with(mode, q, u, vt, x, bias=None):
    lib = _lib.lib()
    assert lib.bs_set_dense_kernel(mode) == 0
    try:
        return IU.bitstack_forward_hip(q, u, vt, x, bias)
    finally:
        assert lib.bs_set_dense_kernel(_lib.DENSE_AUTO) == 0


# (blocks, out features, in features, tokens, bias): ragged tokens, bias epilogue, a token count below and
# above the switch-over, out features that are no multiple of 8 (the library path declines: own kernel)
LIBRARY_CASES = [
    (3, 4096, 4096, 2047, True),
    (2, 1024, 4096, 300, False),
    (2, 14336, 4096, 769, True),
    (1, 4096, 1536, 1000, False),
    (2, 4100, 4096, 1024, True),
    (2, 4099, 4096, 1024, True),
]


@pytest.mark.parametrize("I,M,N,T,with_bias", LIBRARY_CASES)
def test_forward_library_gemm_matches_own_kernel_and_fp64(I, M, N, T, with_bias):
    """The hipBLASLt product behind the rebuild against this library's dense kernel on the same call (both
    round one fp32 sum per output to fp16: all but last-bit ties agree) and sampled rows against float64."""
    print(f"library gemm I={I} M={M} N={N} T={T} bias={with_bias}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=I + M + T, device=dev())
    bias = (torch.randn(M, device=dev()) * 0.05).half() if with_bias else None
    own = forward_with(_lib.DENSE_OWN, q, u, vt, x, bias)
    got = forward_with(_lib.DENSE_LIBRARY, q, u, vt, x, bias)
    assert got.dtype == torch.float16 and tuple(got.shape) == (T, M)
    assert torch.equal(forward_with(_lib.DENSE_LIBRARY, q, u, vt, x, bias), got)
    mx, mn = rel(got, own)
    print(f"  vs own kernel: max_rel={mx:.3e} mean_rel={mn:.3e} differing={float((got != own).float().mean()):.2e}", flush=True)
    assert mx <= 1e-3 and mn <= 5e-5 and float((got != own).float().mean()) < 0.05
    rows = [0, 1, M // 2, M - 2, M - 1]
    exact = spot_rows_exact(q, u, vt, x, rows, bias)
    mx, mn = rel(got[:, rows].cpu(), torch.from_numpy(exact))
    print(f"  spot rows vs fp64: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= MAX_REL and mn <= MEAN_REL


def test_dense_kernel_setting_moves_the_workspace_size_and_rejects_unknown_modes():
    lib = _lib.lib()
    I, M, N, K = 4, 4096, 4096, 16
    weight = M * N * 2
    try:
        assert lib.bs_set_dense_kernel(_lib.DENSE_OWN) == 0
        assert lib.bs_workspace_bytes(I, M, N, K, 2048) == weight
        assert lib.bs_set_dense_kernel(_lib.DENSE_LIBRARY) == 0
        assert lib.bs_workspace_bytes(I, M, N, K, 2048) == weight + (64 << 20)
        assert lib.bs_workspace_bytes(I, M, N, K, 200) == weight + (64 << 20)
        assert lib.bs_workspace_bytes(I, M + 1, N, K, 2048) == (M + 1) * N * 2       # M % 8 != 0: never the library
        assert lib.bs_workspace_bytes(I, M, N, K, 1) < weight                        # decode shapes do not rebuild
        assert lib.bs_set_dense_kernel(_lib.DENSE_AUTO) == 0                         # never the library by itself
        assert lib.bs_workspace_bytes(I, M, N, K, 200) == weight
        assert lib.bs_workspace_bytes(I, M, N, K, 2048) == weight
        ragged = N + 8                                                               # no strip kernel takes this width
        assert lib.bs_workspace_bytes(I, M, ragged, K, 48) == M * ragged * 2
        assert lib.bs_workspace_bytes(I, M, ragged, K, 49) == M * ragged * 2
        assert lib.bs_set_dense_kernel(3) < 0 and lib.bs_set_dense_kernel(-1) < 0
    finally:
        lib.bs_set_dense_kernel(_lib.DENSE_AUTO)


def test_forward_library_gemm_under_graph_replay():
    """A captured forward through the library GEMM replays to the eager result every time (the first, eager
    call has set the library up: the capture only records launches)."""
    I, M, N, T = 2, 4096, 4096, 1024
    lib = _lib.lib()
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=5, device=dev())
    assert lib.bs_set_dense_kernel(_lib.DENSE_LIBRARY) == 0
    try:
        need = int(lib.bs_workspace_bytes(I, M, N, 16, T))
        ws = torch.empty(need, dtype=torch.uint8, device=dev())
        y = torch.empty((T, M), dtype=torch.float16, device=dev())

        def call(stream):
            st = lib.bs_forward(_lib.ptr(q), _lib.ptr(u), _lib.ptr(vt), _lib.ptr(x), None, _lib.ptr(y), I, M, N, 16, T,
                                _lib.ptr(ws), need, stream)
            assert st == 0, st

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            call(_lib.stream_ptr(dev()))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        eager = y.clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            call(_lib.stream_ptr(dev()))
        for r in range(3):
            y.zero_()
            x2 = x * (1.0 + r)                      # eager work and a synchronisation between the replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, eager), r
            del x2
    finally:
        lib.bs_set_dense_kernel(_lib.DENSE_AUTO)


def test_library_gemm_is_not_set_up_under_stream_capture():
    """A shape the library path has never run is captured with this library's own dense kernel (setting
    hipBLASLt up may allocate, which a capture forbids); the replay equals the eager own-kernel result, and
    the eager library result for the same shape, set up afterwards, agrees with both."""
    I, M, N, T = 2, 2048, 1024, 648                      # a shape no other test sends through the library path
    lib = _lib.lib()
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=11, device=dev())
    try:
        own = forward_with(_lib.DENSE_OWN, q, u, vt, x)   # eager: the rebuild and dense kernels have run once
        assert lib.bs_set_dense_kernel(_lib.DENSE_LIBRARY) == 0
        need = int(lib.bs_workspace_bytes(I, M, N, 16, T))
        ws = torch.empty(need, dtype=torch.uint8, device=dev())
        y = torch.zeros((T, M), dtype=torch.float16, device=dev())
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            st = lib.bs_forward(_lib.ptr(q), _lib.ptr(u), _lib.ptr(vt), _lib.ptr(x), None, _lib.ptr(y), I, M, N, 16, T,
                                _lib.ptr(ws), need, _lib.stream_ptr(dev()))
            assert st == 0, st
        for r in range(2):
            y.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, own), r
        got = IU.bitstack_forward_hip(q, u, vt, x)         # eager, library mode: now the plan is made
        mx, mn = rel(got, own)
        assert mx <= 1e-3 and mn <= 5e-5
    finally:
        lib.bs_set_dense_kernel(_lib.DENSE_AUTO)
