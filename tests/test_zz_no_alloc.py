"""The forward for callers that cannot allocate (bs_forward_static): the scratch of the kernels is a
device array inside the library.  Through the C ABI, against bs_forward with a caller-owned workspace
on the same inputs: identical bits, on calls in a row that share the array (the second smaller, so
that stale contents of the first would show), on every path that needs scratch (block-scaled and
fp16 decode kernels, strip kernel, rebuilt weight + dense kernel).  Sizes beyond the array are refused;
warm calls leave the device's free memory untouched; a captured call replays onto the dirty array."""
import ctypes

import pytest
import torch

from bitstack_amd import _lib
from bitstack_amd.utils import inference_utils as IU
from bitstack_amd.utils.synthetic import synthetic_layer

pytestmark = pytest.mark.gpu


def forward_static(q, u, vt, x, bias=None):
    dev = _lib.require_gpu(q, u, vt, x, bias)
    I, M, K = u.shape
    N = vt.shape[2]
    T = x.shape[0]
    y = torch.empty((T, M), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        st = _lib.lib().bs_forward_static(_lib.ptr(q), _lib.ptr(u), _lib.ptr(vt), _lib.ptr(x), _lib.ptr(bias), _lib.ptr(y),
                                          I, M, N, K, T, _lib.stream_ptr(dev))
    return st, y


# (blocks, out, in, tokens): two calls in a row per pair, the second with a smaller input
PAIRS = [((16, 14336, 4096, 1), (2, 1024, 4096, 1)),          # block-scaled decode kernel, then the fp16 one
         ((8, 4096, 4096, 4), (3, 512, 2048, 3)),             # fp16 decode kernel, four and three tokens
         ((4, 4096, 4096, 16), (2, 1000, 1024, 6)),           # strip kernel
         ((2, 2048, 4096, 64), (2, 300, 520, 9)),             # weight rebuilt into the scratch + dense kernel
         ((2, 4096, 4096, 600), (1, 1024, 1024, 512))]        # ... at larger token counts


@pytest.mark.parametrize("first,second", PAIRS)
def test_static_scratch_forward_matches_workspace_forward(first, second):
    dev = torch.device("cuda:0")
    for n, (I, M, N, T) in enumerate((first, second)):
        print(f"static scratch forward I={I} M={M} N={N} T={T}", flush=True)
        q, u, vt, x = synthetic_layer(M, N, I, T, seed=I + T, device=dev)
        bias = (torch.randn(M, device=dev) * 0.01).half() if n else None
        want = IU.bitstack_forward_hip(q, u, vt, x, bias)
        st, got = forward_static(q, u, vt, x, bias)
        assert st == 0, _lib.error_string(st)
        assert torch.equal(got, want)
        st, again = forward_static(q, u, vt, x, bias)         # and once more on the now dirty array
        assert st == 0 and torch.equal(again, want)


# one shape per scratch-using path: block-scaled decode, fp16 decode, strip kernel, rebuilt weight + dense kernel
PATH_SHAPES = [(16, 4096, 4096, 1), (3, 1024, 4096, 4), (4, 2048, 2048, 16), (2, 2048, 4096, 200)]


def test_static_scratch_forward_allocates_nothing_once_warm():
    """After one call per shape (which looks the array's address up and raises LDS limits), further calls
    change neither the bytes the driver reports free (hipMemGetInfo) nor torch's own allocator counters."""
    dev = torch.device("cuda:0")
    L = _lib.lib()
    cases = []
    for (I, M, N, T) in PATH_SHAPES:
        q, u, vt, x = synthetic_layer(M, N, I, T, seed=I + T, device=dev)
        y = torch.empty((T, M), dtype=torch.float16, device=dev)
        cases.append((q, u, vt, x, y, I, M, N, T))
    stream = _lib.stream_ptr(dev)

    def call_all():
        for (q, u, vt, x, y, I, M, N, T) in cases:
            st = L.bs_forward_static(_lib.ptr(q), _lib.ptr(u), _lib.ptr(vt), _lib.ptr(x), None, _lib.ptr(y), I, M, N, 16, T, stream)
            assert st == 0, _lib.error_string(st)

    call_all()                                               # warm: symbol address, LDS grants, code objects
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info(dev)
    alloc0, reserved0 = torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev)
    for _ in range(3):
        call_all()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info(dev)
    assert free1 == free0, (free0, free1)
    assert torch.cuda.memory_allocated(dev) == alloc0 and torch.cuda.memory_reserved(dev) == reserved0


@pytest.mark.parametrize("I,M,N,T", PATH_SHAPES)
def test_static_scratch_forward_under_graph_replay(I, M, N, T):
    """The use the entry point is for: after one eager call, a captured bs_forward_static replays to the
    eager result every time, with another shape dirtying the shared array between the replays."""
    dev = torch.device("cuda:0")
    L = _lib.lib()
    print(f"static scratch forward under capture I={I} M={M} N={N} T={T}", flush=True)
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=3 * I + T, device=dev)
    y = torch.zeros((T, M), dtype=torch.float16, device=dev)

    def call():
        st = L.bs_forward_static(_lib.ptr(q), _lib.ptr(u), _lib.ptr(vt), _lib.ptr(x), None, _lib.ptr(y), I, M, N, 16, T,
                                 _lib.stream_ptr(dev))
        assert st == 0, _lib.error_string(st)

    call()                                                   # eager first: set-up happens outside the capture
    torch.cuda.synchronize()
    eager = y.clone()
    assert torch.equal(eager, IU.bitstack_forward_hip(q, u, vt, x))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    q2, u2, vt2, x2 = synthetic_layer(512, 1024, 2, 3, seed=9, device=dev)
    for r in range(3):
        y.fill_(float("nan"))
        st, _ = forward_static(q2, u2, vt2, x2)             # eager work on the same array between the replays
        assert st == 0
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), r


def test_static_scratch_forward_refuses_what_does_not_fit():
    dev = torch.device("cuda:0")
    L = _lib.lib()
    I, M, N, T = 2, 8192, 8192, 200                          # rebuilt weight: 128 MiB of scratch
    assert L.bs_workspace_bytes(I, M, N, 16, T) > _lib.STATIC_SCRATCH_BYTES
    q, u, vt, x = synthetic_layer(M, N, I, T, seed=1, device=dev)
    st, _ = forward_static(q, u, vt, x)
    assert st == -5 and "workspace" in _lib.error_string(st)
    # the same layer at one token fits, and an empty token dimension is a no-op
    st, y = forward_static(q, u, vt, x[:1].contiguous())
    assert st == 0 and torch.equal(y, IU.bitstack_forward_hip(q, u, vt, x[:1].contiguous()))
    st, y0 = forward_static(q, u, vt, x[:0].contiguous())
    assert st == 0 and tuple(y0.shape) == (0, M)
    nul = ctypes.c_void_p(0)
    assert L.bs_forward_static(nul, nul, nul, nul, nul, nul, 1, 64, 512, 16, 1, nul) == -1      # null pointers
    assert L.bs_forward_static(nul, nul, nul, nul, nul, nul, 1, 64, 512, 17, 1, nul) == -3      # rank
