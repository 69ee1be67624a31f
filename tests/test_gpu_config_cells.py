"""Every cell of the decode sweep and of the prefill configuration at its full size, through the C ABI.

Decode sweep: (out x in) in {4096x4096, 1024x4096, 14336x4096, 4096x14336} x blocks {1, 2, 4, 8, 16} x
tokens {1, 2, 4}, rank 16, the benchmark's synthetic recipe.  Prefill: the same shapes with 8 blocks at
{16, 128, 512, 2048} tokens.  The CPU oracle cannot run whole layers of this size in seconds, so every
cell is checked on sampled rows (first and last, both sides of every tile height the kernels use)
against the float64 closed form, with

    max|d| / max|y_ref| <= 1e-2   and   mean|d| / mean|y_ref| <= 1e-3,

and over ALL rows by running the cell on every kernel that takes it (planner's choice, fp16 decode
kernel, block-scaled decode kernel) and comparing the results with one another."""
import numpy as np
import pytest
import torch

from bitstack_amd import _lib
from bitstack_amd.utils import inference_utils as IU
from bitstack_amd.utils.synthetic import synthetic_layer
from oracle import bitstack_oracle as O

pytestmark = pytest.mark.gpu

MAX_REL, MEAN_REL = 1e-2, 1e-3
SHAPES = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)]
BLOCKS = [1, 2, 4, 8, 16]


def dev():
    return torch.device("cuda:0")


def sample_rows(M):
    """First and last rows and both sides of 16-, 128-, 512- and 1024-row tile edges, the middle, the ragged end."""
    rows = {0, 1, 15, 16, 127, 128, 511, 512, 1023, M // 2 - 1, M // 2, M - 513, M - 512, M - 129, M - 128, M - 17, M - 16, M - 2, M - 1}
    return sorted(r for r in rows if 0 <= r < M)


def exact_rows(q, u, vt, x, rows):
    """float64 closed form of y[:, rows] (the oracle on the sampled rows' sign bytes and u rows)."""
    I, M, _ = u.shape
    N = vt.shape[2]
    idx = torch.tensor(rows, device=q.device)
    qs = np.stack([qq.view(M, N // 8)[idx].reshape(-1).cpu().numpy() for qq in q])
    return O.forward_exact(qs, u[:, idx].cpu().numpy(), vt.cpu().numpy(), x.cpu().numpy())


def rel_errors(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.abs(got - ref)
    return d.max() / max(np.abs(ref).max(), 1e-30), d.mean() / max(np.abs(ref).mean(), 1e-30)


def assert_close(got, ref, what, max_rel=MAX_REL, mean_rel=MEAN_REL):
    mx, mn = rel_errors(got, ref)
    print(f"  {what}: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= max_rel and mn <= mean_rel, f"{what}: max_rel={mx:.3e} mean_rel={mn:.3e}"


@pytest.fixture
def decode_kernel():
    L = _lib.lib()
    yield lambda mode: _lib.check(L.bs_set_decode_kernel(mode), "bs_set_decode_kernel")
    L.bs_set_decode_kernel(_lib.DECODE_AUTO)


@pytest.mark.parametrize("I", BLOCKS)
@pytest.mark.parametrize("M,N", SHAPES)
def test_decode_sweep_cell(M, N, I, decode_kernel):
    """One (shape, blocks) layer of the sweep at 1, 2 and 4 tokens."""
    print(f"decode sweep cell M={M} N={N} I={I}", flush=True)
    L = _lib.lib()
    q, u, vt, x4 = synthetic_layer(M, N, I, 4, seed=1000 + I + M // 7 + N // 11, device=dev())
    rows = sample_rows(M)
    exact4 = exact_rows(q, u, vt, x4, rows)
    one_token = None
    for T in (1, 2, 4):
        x = x4[:T].contiguous()
        results = {}
        for mode, name in ((_lib.DECODE_AUTO, "planned"), (_lib.DECODE_F16, "fp16"), (_lib.DECODE_MX, "block-scaled")):
            decode_kernel(mode)
            kernel = L.bs_decode_kernel(I, M, N, 16, T)
            assert kernel in (_lib.DECODE_F16, _lib.DECODE_MX), (T, mode, kernel)   # every cell is a decode-kernel shape
            if mode == _lib.DECODE_MX and kernel != _lib.DECODE_MX:
                assert T > 2                                                      # the block-scaled kernel stops at two tokens
                continue
            print(f"  T={T} {name}: kernel {kernel}, plan {_lib.decode_plan(I, M, N, 16, T)}", flush=True)
            y = IU.bitstack_forward_hip(q, u, vt, x)
            assert y.dtype == torch.float16 and tuple(y.shape) == (T, M)
            assert torch.equal(IU.bitstack_forward_hip(q, u, vt, x), y)             # deterministic
            assert_close(y[:, rows].cpu().numpy(), exact4[:T], f"T={T} {name} sampled rows vs fp64")
            results[name] = y.float()
        decode_kernel(_lib.DECODE_AUTO)
        scale = float(results["planned"].abs().max())
        for name, y in results.items():
            if name != "planned":
                d = float((y - results["planned"]).abs().max())
                print(f"  T={T} {name} vs planned, all rows: max|d|/max|y| = {d / scale:.3e}", flush=True)
                assert d <= 2e-3 * scale, (T, name)
        if T == 1:
            one_token = results["planned"]
        else:
            # the first token of a longer pass is the one-token answer up to summation order
            assert float((results["planned"][0] - one_token[0]).abs().max()) <= 2e-3 * scale, T


PREFILL_T = [16, 128, 512, 2048]


@pytest.mark.parametrize("T", PREFILL_T)
@pytest.mark.parametrize("M,N", SHAPES)
def test_prefill_cell(M, N, T):
    """One layer of the prefill configuration: 8 blocks, T tokens.  Sampled rows and tokens against float64;
    all outputs against the rebuilt weight multiplied by torch (the vendor GEMM), whose rounding points the
    forward shares whichever kernel runs it (strip kernel at 16 tokens, rebuild + dense kernel above)."""
    I = 8
    print(f"prefill cell M={M} N={N} I={I} T={T}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=2000 + T + M // 7 + N // 11, device=dev())
    y = IU.bitstack_forward_hip(q, u, vt, x)
    assert y.dtype == torch.float16 and tuple(y.shape) == (T, M)
    assert torch.equal(IU.bitstack_forward_hip(q, u, vt, x), y)
    rows = sample_rows(M)
    tok = sorted(set(list(range(0, min(T, 40))) + list(range(max(T // 2 - 20, 0), min(T // 2 + 20, T))) + list(range(max(T - 40, 0), T))))
    ti = torch.tensor(tok, device=dev())
    exact = exact_rows(q, u, vt, x[ti], rows)
    assert_close(y[ti][:, rows].cpu().numpy(), exact, "sampled rows and tokens vs fp64")
    w = IU.unpack_and_reconstruct_w_hip(q, u, vt)
    ref = torch.nn.functional.linear(x, w).float()
    d = (y.float() - ref).abs()
    mx, mn = float(d.max() / ref.abs().max()), float(d.mean() / ref.abs().mean())
    print(f"  all outputs vs F.linear on the rebuilt weight: max_rel={mx:.3e} mean_rel={mn:.3e}", flush=True)
    assert mx <= 2e-3 and mn <= 2e-4
