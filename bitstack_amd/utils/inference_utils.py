"""Fused inference helpers with the reference's names and argument meanings
(bitstack/utils/inference_utils.py); every one is a thin call into the C ABI.
"""
from __future__ import annotations

import torch

from bitstack_amd import _lib


def _f16c(t):
    if t.dtype != torch.float16:
        raise TypeError(f"expected float16, got {t.dtype}")
    return t.contiguous()


def _dims(u, vt):
    if u.dim() != 3 or vt.dim() != 3 or u.shape[0] != vt.shape[0] or u.shape[2] != vt.shape[1]:
        raise ValueError(f"u {tuple(u.shape)} / vt {tuple(vt.shape)} are not [I,M,K] / [I,K,N]")
    I, M, K = u.shape
    return I, M, vt.shape[2], K


def reconstruct_w_hip(sign, u, vt):
    """(sign * u @ vt).sum(0) from unpacked int8 signs [I, M, N]
    (reconstruct_w_triton, inference_utils.py:135-156)."""
    dev = _lib.require_gpu(sign, u, vt)
    I, M, N, K = _dims(u, vt)
    if tuple(sign.shape) != (I, M, N) or sign.dtype != torch.int8:
        raise ValueError(f"sign must be int8 [{I},{M},{N}], got {sign.dtype} {tuple(sign.shape)}")
    sign, u, vt = sign.contiguous(), _f16c(u), _f16c(vt)
    w = torch.empty((M, N), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bs_reconstruct_w_from_sign(_lib.ptr(sign), _lib.ptr(u), _lib.ptr(vt),
                                                         _lib.ptr(w), I, M, N, K, _lib.stream_ptr(dev)),
                   "bs_reconstruct_w_from_sign")
    return w


def unpack_and_reconstruct_w_hip(packed_sign, u, vt):
    """(sign * u @ vt).sum(0) straight from packed signs [I, M*N/8]
    (unpack_and_reconstruct_w_triton and _v2, inference_utils.py:371-387, :465-488)."""
    dev = _lib.require_gpu(packed_sign, u, vt)
    I, M, N, K = _dims(u, vt)
    if packed_sign.dtype != torch.uint8 or packed_sign.numel() != I * ((M * N + 7) // 8):
        raise ValueError(f"packed signs must be uint8 with {I}*{(M * N + 7) // 8} bytes, got "
                         f"{packed_sign.dtype} {tuple(packed_sign.shape)}")
    packed_sign, u, vt = packed_sign.contiguous(), _f16c(u), _f16c(vt)
    w = torch.empty((M, N), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bs_reconstruct_w(_lib.ptr(packed_sign), _lib.ptr(u), _lib.ptr(vt),
                                               _lib.ptr(w), I, M, N, K, _lib.stream_ptr(dev)),
                   "bs_reconstruct_w")
    return w


def bitstack_forward_hip(packed_sign, u, vt, x, bias=None):
    """y = x @ (sum_i sign_i * u_i @ vt_i)^T (+ bias) from packed signs; x is
    [..., N] fp16 (reconstruct_and_forward_triton, inference_utils.py:252-284,
    generalised to packed input, any leading shape and an optional bias)."""
    dev = _lib.require_gpu(packed_sign, u, vt, x, bias)
    I, M, N, K = _dims(u, vt)
    if x.shape[-1] != N:
        raise ValueError(f"x has {x.shape[-1]} input features, the layer has {N}")
    if packed_sign.dtype != torch.uint8 or packed_sign.numel() != I * ((M * N + 7) // 8):
        raise ValueError("packed signs do not match u / vt")
    packed_sign, u, vt, x2 = packed_sign.contiguous(), _f16c(u), _f16c(vt), _f16c(x).view(-1, N)
    if bias is not None:
        bias = _f16c(bias)
    T = x2.shape[0]
    y = torch.empty((T, M), dtype=torch.float16, device=dev)
    L = _lib.lib()
    need = L.bs_workspace_bytes(I, M, N, K, T)
    if need < 0:
        _lib.check(int(need), "bs_workspace_bytes")
    ws = _lib.workspace(dev, int(need))
    with torch.cuda.device(dev):
        _lib.check(L.bs_forward(_lib.ptr(packed_sign), _lib.ptr(u), _lib.ptr(vt), _lib.ptr(x2),
                                _lib.ptr(bias), _lib.ptr(y), I, M, N, K, T, _lib.ptr(ws),
                                ws.numel(), _lib.stream_ptr(dev)), "bs_forward")
    return y.view(x.shape[:-1] + (M,))


def linear_f16_hip(x, w, bias=None):
    """F.linear on the library's own MFMA kernel (fp16 in, fp32 accumulate)."""
    dev = _lib.require_gpu(x, w, bias)
    M, N = w.shape
    x2, w = _f16c(x).view(-1, N), _f16c(w)
    if bias is not None:
        bias = _f16c(bias)
    T = x2.shape[0]
    y = torch.empty((T, M), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bs_linear_f16(_lib.ptr(x2), _lib.ptr(w), _lib.ptr(bias), _lib.ptr(y),
                                            T, M, N, _lib.stream_ptr(dev)), "bs_linear_f16")
    return y.view(x.shape[:-1] + (M,))


def reconstruct_and_forward_hip(sign, u, vt, x):
    """Reference signature of level 5 (unpacked int8 signs, 3-D x, no bias;
    inference_utils.py:252-284): rebuild the weight, then the MFMA linear."""
    if x.dim() != 3:
        raise ValueError("x must be [BZ, L, N]")
    return linear_f16_hip(x, reconstruct_w_hip(sign, u, vt))


# drop-in aliases for code written against the reference's names
reconstruct_w_triton = reconstruct_w_hip
unpack_and_reconstruct_w_triton = unpack_and_reconstruct_w_hip
unpack_and_reconstruct_w_triton_v2 = unpack_and_reconstruct_w_hip
unpack_and_reconstruct_w_triton_v3 = unpack_and_reconstruct_w_hip
reconstruct_and_forward_triton = reconstruct_and_forward_hip
