"""CPU-side checks of the shared library: it loads, exports every symbol the
header declares, and rejects bad arguments with the documented status before
touching a device (no kernel is launched here)."""
import ctypes
import os
import re

import pytest

from bitstack_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bitstack_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bs_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build(force=False)
    return _lib.lib()


def test_header_and_binding_agree():
    assert declared_functions() == sorted(_lib.SIGNATURES)


def test_every_declared_symbol_is_exported(L):
    for name in declared_functions():
        assert hasattr(L, name), name


def test_version_and_error_strings(L):
    assert L.bs_version() >= 100
    assert _lib.error_string(0) == "ok"
    for code in (-1, -2, -3, -4, -5, -6, -7):
        assert _lib.error_string(code) not in ("ok", "unknown status")
    assert _lib.error_string(-999) == "unknown status"


def test_argument_validation_returns_status_not_crash(L):
    nul = ctypes.c_void_p(0)
    one = ctypes.c_void_p(256)       # non-null, never dereferenced on these paths
    odd = ctypes.c_void_p(257)
    # unpack / pack
    assert L.bs_unpack_sign(nul, one, 8, nul) == -1
    assert L.bs_unpack_sign(one, one, -1, nul) == -2
    assert L.bs_unpack_sign(nul, nul, 0, nul) == 0
    assert L.bs_pack_sign(one, nul, 8, nul) == -1
    # reconstruct
    assert L.bs_reconstruct_w(one, one, one, one, 1, 0, 128, 16, nul) == -2
    assert L.bs_reconstruct_w(one, one, one, one, 1, 64, 128, 17, nul) == -3
    assert L.bs_reconstruct_w(one, one, one, one, 1, 64, 128, 0, nul) == -3
    assert L.bs_reconstruct_w(nul, one, one, one, 1, 64, 128, 16, nul) == -1
    assert L.bs_reconstruct_w(one, odd, one, one, 1, 64, 128, 16, nul) == -4
    assert L.bs_reconstruct_w_from_sign(one, one, one, nul, 1, 64, 128, 16, nul) == -1
    # forward
    assert L.bs_forward(one, one, one, one, nul, one, 1, 64, 100, 16, 1, one, 1 << 30, nul) == -2   # N % 8
    assert L.bs_forward(one, one, one, one, nul, one, 1, 64, 128, 32, 1, one, 1 << 30, nul) == -3
    assert L.bs_forward(one, one, one, nul, nul, one, 1, 64, 128, 16, 1, one, 1 << 30, nul) == -1
    assert L.bs_forward(odd, one, one, one, nul, one, 1, 64, 128, 16, 1, one, 1 << 30, nul) == -4
    assert L.bs_forward(one, one, one, one, nul, one, 1, 64, 512, 16, 1, nul, 0, nul) == -5
    assert L.bs_forward(one, one, one, one, nul, one, 1, 64, 512, 16, 1, one, 16, nul) == -5
    assert L.bs_forward(one, one, one, one, nul, one, 1, 64, 512, 16, 0, nul, 0, nul) == 0        # T == 0
    # linear
    assert L.bs_linear_f16(nul, one, nul, one, 4, 64, 128, nul) == -1
    assert L.bs_linear_f16(one, one, nul, one, 4, 0, 128, nul) == -2


def test_workspace_bytes(L):
    assert L.bs_workspace_bytes(8, 4096, 4096, 16, 0) == 0
    assert L.bs_workspace_bytes(8, 4096, 4100, 16, 1) == -2
    assert L.bs_workspace_bytes(8, 4096, 4096, 20, 1) == -3
    # prefill and odd shapes rebuild the fp16 weight (the vendor GEMM and its 64 MiB only in comparator mode)
    assert L.bs_workspace_bytes(8, 4096, 4096, 16, 512) == 4096 * 4096 * 2
    assert L.bs_set_dense_kernel(_lib.DENSE_LIBRARY) == 0
    assert L.bs_workspace_bytes(8, 4096, 4096, 16, 512) == 4096 * 4096 * 2 + (64 << 20)
    assert L.bs_set_dense_kernel(_lib.DENSE_AUTO) == 0
    # 49..128 tokens: partial sums per column group of the walked / panel kernels, not the weight
    assert L.bs_workspace_bytes(8, 4096, 4096, 16, 128) == (8 * 128 * 4097 * 4 + 255) // 256 * 256
    assert L.bs_workspace_bytes(8, 4096, 4104, 16, 20) == 4096 * 4104 * 2
    assert L.bs_workspace_bytes(2, 64, 72, 16, 1) == ((64 * 72 * 2 + 255) // 256) * 256
    # decode keeps fp32 partial row sums: a multiple of T * M * 4, far below the weight
    for T in (1, 4):
        b = L.bs_workspace_bytes(8, 4096, 4096, 16, T)
        assert b > 0 and b % (T * 4096 * 4) == 0 and b < 4096 * 4096 * 2
    # 5..48 tokens: partial sums per group of strips (plus the groups' sums of squares of x)
    for T in (8, 32, 48):
        b = L.bs_workspace_bytes(8, 4096, 4096, 16, T)
        assert T * 4096 * 4 <= b <= 32 * (T * 4096 * 4 + T * 4) + 256


def test_kernel_hooks_belong_to_the_calling_thread(L):
    """A hook set on one thread moves neither the plan nor the workspace size another thread sees."""
    import threading
    seen = {}

    def other():
        seen["decode"] = L.bs_decode_kernel(4, 4096, 4096, 16, 1)
        seen["ws"] = L.bs_workspace_bytes(4, 4096, 4096, 16, 512)
        # and what this thread sets stays here
        L.bs_set_decode_kernel(_lib.DECODE_F16)

    base_decode = L.bs_decode_kernel(4, 4096, 4096, 16, 1)
    base_ws = L.bs_workspace_bytes(4, 4096, 4096, 16, 512)
    try:
        assert L.bs_set_decode_kernel(_lib.DECODE_MX) == 0 and L.bs_set_dense_kernel(_lib.DENSE_LIBRARY) == 0
        assert L.bs_decode_kernel(4, 4096, 4096, 16, 1) == _lib.DECODE_MX
        assert L.bs_workspace_bytes(4, 4096, 4096, 16, 512) == base_ws + (64 << 20)
        t = threading.Thread(target=other)
        t.start()
        t.join()
        assert seen == {"decode": base_decode, "ws": base_ws}
        assert L.bs_decode_kernel(4, 4096, 4096, 16, 1) == _lib.DECODE_MX
    finally:
        L.bs_set_decode_kernel(_lib.DECODE_AUTO)
        L.bs_set_dense_kernel(_lib.DENSE_AUTO)


def test_group_and_decode_step_validation(L):
    nul, one, odd = ctypes.c_void_p(0), ctypes.c_void_p(256), ctypes.c_void_p(257)
    mats = (_lib.bs_matrix * 2)()
    for m in mats:
        m.packed, m.u, m.vt, m.bias, m.I, m.M = 256, 256, 256, None, 2, 128
    assert L.bs_forward_group_workspace_bytes(mats, 2, 512, 16, 1) > 0
    assert L.bs_forward_group_workspace_bytes(mats, 2, 500, 16, 1) == -2          # N % 8
    assert L.bs_forward_group_workspace_bytes(mats, 2, 520, 16, 1) == -2          # not a decode-kernel shape
    assert L.bs_forward_group_workspace_bytes(mats, 5, 512, 16, 1) == -2          # more than BS_MAX_GROUP
    assert L.bs_forward_group_workspace_bytes(mats, 2, 512, 16, 9) > 0            # 9..48 tokens: the strip kernel
    assert L.bs_forward_group_workspace_bytes(mats, 2, 512, 16, 49) == -2         # more than 48 tokens
    assert L.bs_forward_group_workspace_bytes(mats, 2, 512, 17, 1) == -3
    assert L.bs_forward_group_workspace_bytes(nul, 2, 512, 16, 1) == -1
    big = 1 << 30
    assert L.bs_forward_group(mats, 2, 512, 16, nul, 1, 0, nul, one, one, big, nul) == -1       # x
    assert L.bs_forward_group(mats, 2, 512, 16, one, 1, 1, nul, one, one, big, nul) == -1       # residual epilogue, no residual
    assert L.bs_forward_group(mats, 2, 512, 16, one, 1, 7, nul, one, one, big, nul) == -2       # unknown epilogue
    assert L.bs_forward_group(mats, 2, 512, 16, one, 1, 0, nul, one, nul, 0, nul) == -5
    mats[1].vt = 257
    assert L.bs_forward_group(mats, 2, 512, 16, one, 1, 0, nul, one, one, big, nul) == -4
    mats[1].vt = 256
    mats[1].M = 64
    assert L.bs_forward_group(mats, 2, 512, 16, one, 1, 2, nul, one, one, big, nul) == -2       # SwiGLU needs equal M
    assert L.bs_forward_group_rms(mats, 2, 512, 16, nul, 1, 1e-5, 0, nul, one, one, big, nul) == -1
    assert L.bs_forward_group_rms(mats, 2, 512, 16, one, 1, -1.0, 0, nul, one, one, big, nul) == -2   # eps < 0
    assert L.bs_argmax_f16(nul, one, 1, 64, nul) == -1
    assert L.bs_argmax_f16(one, one, 1, 0, nul) == -2
    assert L.bs_argmax_f16(one, one, 2, 13, nul) == -4
    # rmsnorm / attention
    assert L.bs_rmsnorm_f16(one, one, one, 1, 100, 1e-5, nul) == -2
    assert L.bs_rmsnorm_f16(one, one, one, 1, 32768, 1e-5, nul) == -2
    assert L.bs_rmsnorm_f16(one, nul, one, 1, 512, 1e-5, nul) == -1
    assert L.bs_rmsnorm_f16(odd, one, one, 1, 512, 1e-5, nul) == -4
    assert L.bs_rmsnorm_f16(nul, nul, nul, 0, 512, 1e-5, nul) == 0
    att = lambda *a: L.bs_attention_decode_f16(*a)
    assert att(one, one, one, one, one, one, one, 1, 32, 8, 64, 128, nul) == -2                 # head_dim
    assert att(one, one, one, one, one, one, one, 1, 32, 5, 128, 128, nul) == -2                # heads % kv_heads
    assert att(one, one, one, one, one, one, one, 1, 32, 8, 128, 10000, nul) == -2              # max_len
    assert att(one, one, one, one, one, nul, one, 1, 32, 8, 128, 128, nul) == -1                # pos
    assert att(one, odd, one, one, one, one, one, 1, 32, 8, 128, 128, nul) == -4


def test_no_fallback_when_the_library_or_the_device_is_missing(tmp_path):
    """The product path fails loudly: a missing shared library is an error that names the
    build step, and the HIP entry points refuse host tensors (only fused_level 0 is torch-only)."""
    import subprocess
    import sys
    import torch
    from bitstack_amd import BitStackLinear
    from bitstack_amd.utils import inference_utils as IU
    from bitstack_amd.utils import pack_utils as PU
    code = ("import bitstack_amd._lib as L\n"
            f"L.LIB_PATH = {str(tmp_path / 'absent.so')!r}\n"
            "try:\n    L.lib()\nexcept RuntimeError as e:\n    print('RAISED', e)\n")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True,
                         cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert "RAISED" in out.stdout and "is missing" in out.stdout and "no fallback" in out.stdout, out.stdout + out.stderr
    q = torch.zeros(2, 64 * 512 // 8, dtype=torch.uint8)
    u, vt, x = torch.zeros(2, 64, 16).half(), torch.zeros(2, 16, 512).half(), torch.zeros(1, 512).half()
    for call in (lambda: IU.bitstack_forward_hip(q, u, vt, x), lambda: IU.unpack_and_reconstruct_w_hip(q, u, vt),
                 lambda: PU.unpack_sign_hip(q[0], (64, 512)), lambda: IU.linear_f16_hip(x, torch.zeros(64, 512).half())):
        with pytest.raises(RuntimeError, match="HIP device"):
            call()
    mod = BitStackLinear(2, 512, 64, 16, False, False, "cpu", fused_level=5)
    mod.stack_blocks()
    with pytest.raises(RuntimeError, match="HIP device"):
        mod(x)
