"""ctypes binding of libbitstack_hip.so (the C ABI in include/bitstack_hip.h).

There is no CPU fallback: if the shared library is missing, or a tensor is not
on a HIP device, the call raises.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
import threading

import torch

_CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(_CSRC, "libbitstack_hip.so")

# name -> (restype, argtypes); mirrors include/bitstack_hip.h one to one
_P, _I, _L = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
SIGNATURES = {
    "bs_version": (_I, []),
    "bs_error_string": (ctypes.c_char_p, [_I]),
    "bs_pack_sign": (_I, [_P, _P, _L, _P]),
    "bs_unpack_sign": (_I, [_P, _P, _L, _P]),
    "bs_reconstruct_w_from_sign": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "bs_reconstruct_w": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "bs_workspace_bytes": (_L, [_I, _I, _I, _I, _I]),
    "bs_decode_plan": (_I, [_I, _I, _I, _I, _I, _P, _P, _P, _P]),
    "bs_forward": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _L, _P]),
    "bs_forward_static": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "bs_linear_f16": (_I, [_P, _P, _P, _P, _I, _I, _I, _P]),
    "bs_linear_plan": (_I, [_I, _I, _I, _P, _P, _P, _P]),
    "bs_decode_kernel": (_I, [_I, _I, _I, _I, _I]),
    "bs_set_decode_kernel": (_I, [_I]),
    "bs_set_dense_kernel": (_I, [_I]),
    "bs_set_prefill_kernel": (_I, [_I]),
    "bs_forward_path": (_I, [_I, _I, _I, _I, _I]),
}
DECODE_AUTO, DECODE_F16, DECODE_MX = 0, 1, 2
DENSE_AUTO, DENSE_OWN, DENSE_LIBRARY = 0, 1, 2
PREFILL_AUTO, PREFILL_REBUILD, PREFILL_WALKED, PREFILL_PANEL = 0, 1, 2, 3
PATH_NAMES = {0: "rebuild + dense", 1: "gemv_kernel (fp16 MFMA)", 2: "gemv_mx_kernel (fp4 x fp6 MFMA)", 3: "strip_forward_kernel",
              4: "strip_wide_kernel", 5: "panel_forward_kernel"}
PATH_REBUILD, PATH_DECODE_F16, PATH_DECODE_MX, PATH_STRIP, PATH_WALKED, PATH_PANEL = range(6)
STATIC_SCRATCH_BYTES = 64 << 20



class bs_matrix(ctypes.Structure):
    """struct bs_matrix of include/bitstack_hip.h."""
    _fields_ = [("packed", _P), ("u", _P), ("vt", _P), ("bias", _P), ("I", ctypes.c_int32), ("M", ctypes.c_int32)]


SIGNATURES.update({
    "bs_forward_group_workspace_bytes": (_L, [_P, _I, _I, _I, _I]),
    "bs_forward_group": (_I, [_P, _I, _I, _I, _P, _I, _I, _P, _P, _P, _L, _P]),
    "bs_forward_group_rms": (_I, [_P, _I, _I, _I, _P, _I, ctypes.c_float, _I, _P, _P, _P, _L, _P]),
    "bs_argmax_f16": (_I, [_P, _P, _I, _I, _P]),
    "bs_rmsnorm_f16": (_I, [_P, _P, _P, _I, _I, ctypes.c_float, _P]),
    "bs_attention_decode_f16": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
})
EPI_NONE, EPI_RESIDUAL, EPI_SWIGLU = 0, 1, 2

_lib = None
_lock = threading.Lock()


def build(force: bool = True) -> str:
    """Compile the HIP sources for gfx950 (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-C", _CSRC, "-j8"] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        f"{LIB_PATH} is missing: build it with `make -C {_CSRC}` "
                        "(or __graft_entry__.build()); there is no fallback path")
                L = ctypes.CDLL(LIB_PATH)
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(L, name)
                    fn.restype, fn.argtypes = res, args
                _lib = L
    return _lib


def decode_plan(I, M, N, K, T):
    """(waves, row_tiles_per_wave, workgroups, partials_per_row) of the decode kernel, waves == 0 if not used."""
    vals = [ctypes.c_int(0) for _ in range(4)]
    check(lib().bs_decode_plan(I, M, N, K, T, *[ctypes.byref(v) for v in vals]), "bs_decode_plan")
    return tuple(v.value for v in vals)


def linear_plan(T, M, N):
    """(tile_tokens, tile_features, k_step, k_tail) of the dense kernel for these dimensions."""
    vals = [ctypes.c_int(0) for _ in range(4)]
    check(lib().bs_linear_plan(T, M, N, *[ctypes.byref(v) for v in vals]), "bs_linear_plan")
    return tuple(v.value for v in vals)


def error_string(status: int) -> str:
    return lib().bs_error_string(int(status)).decode()


def check(status: int, what: str) -> None:
    if status != 0:
        raise RuntimeError(f"{what} failed with status {status}: {error_string(status)}")


def require_gpu(*tensors) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("bitstack_amd HIP kernels need tensors on a HIP device; "
                               f"got a tensor on {t.device} (fused_level 0 is the torch-only path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def stream_ptr(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


_workspaces: dict = {}
_retired: list = []


def workspace(dev, nbytes: int):
    """Per-(device, stream) scratch tensor, grown on demand.  Kernels on one
    stream are ordered, so reusing it across calls on that stream is safe.

    A buffer that is outgrown is kept alive for the life of the process, never
    handed back to the allocator: a HIP graph captured while it was current has
    its address baked in, and its replays must keep writing into memory nobody
    else owns.  (A graph captured before a growth still uses the old buffer; it
    stays correct, it just does not share scratch with later eager calls.)"""
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    with _lock:
        buf = _workspaces.get(key)
        if buf is None or buf.numel() < nbytes:
            if buf is not None:
                _retired.append(buf)
            # grow geometrically so that a sequence of slowly growing requests retires few buffers
            size = max(nbytes, 1 << 20, 0 if buf is None else 2 * buf.numel())
            buf = torch.empty(size, dtype=torch.uint8, device=dev)
            _workspaces[key] = buf
    return buf
