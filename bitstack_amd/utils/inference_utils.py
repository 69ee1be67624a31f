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


class MatrixGroup:
    """Up to four stacked BitStack matrices with the same in_features and rank that
    are always applied to the same input (q/k/v, gate/up): the argument block of
    bs_forward_group, built once.  Keeps the tensors alive."""

    def __init__(self, mats):
        # mats: sequence of (packed_sign [I, M*N/8], u [I, M, K], vt [I, K, N], bias or None)
        self.tensors = []
        self.M = []
        arr = (_lib.bs_matrix * len(mats))()
        N = K = None
        for j, (q, u, vt, bias) in enumerate(mats):
            _lib.require_gpu(q, u, vt, bias)
            I, M, n, k = _dims(u, vt)
            if N is None:
                N, K = n, k
            elif (n, k) != (N, K):
                raise ValueError("matrices of a group share in_features and rank")
            if q.dtype != torch.uint8 or q.numel() != I * ((M * n + 7) // 8):
                raise ValueError("packed signs do not match u / vt")
            q, u, vt = q.contiguous(), _f16c(u), _f16c(vt)
            bias = None if bias is None else _f16c(bias)
            self.tensors.append((q, u, vt, bias))
            arr[j].packed, arr[j].u, arr[j].vt = q.data_ptr(), u.data_ptr(), vt.data_ptr()
            arr[j].bias = None if bias is None else bias.data_ptr()
            arr[j].I, arr[j].M = I, M
            self.M.append(M)
        self.arr, self.n, self.N, self.K = arr, len(mats), N, K
        self.dev = mats[0][0].device
        self._need = {}

    @classmethod
    def from_modules(cls, modules):
        """modules: BitStackLinear objects after stack_blocks(), using their first w_bit blocks."""
        mats = []
        for m in modules:
            q, u, vt = m._stacked()
            mats.append((q, u, vt, m.bias))
        return cls(mats)

    def workspace_bytes(self, T):
        if T not in self._need:
            self._need[T] = int(_lib.lib().bs_forward_group_workspace_bytes(self.arr, self.n, self.N, self.K, T))
        return self._need[T]


def bitstack_forward_group_hip(group: MatrixGroup, x, epilogue=_lib.EPI_NONE, residual=None, out=None, rms_eps=None):
    """All matrices of `group` applied to x [T, N] (T <= 48) in one launch, with
    the outputs side by side [T, sum M] (EPI_NONE), plus `residual` (EPI_RESIDUAL),
    or silu(first) * second [T, M] (EPI_SWIGLU).  What three (two) module calls and
    the element-wise ops after them do in a decoder layer.  With rms_eps set, x is
    the un-normalised row and every output is scaled by rsqrt(mean(x^2) + rms_eps)
    (the norm's weight vector must already be folded into the group's vt)."""
    dev = _lib.require_gpu(x, residual, out)
    x2 = _f16c(x).view(-1, group.N)
    T = x2.shape[0]
    width = group.M[0] if epilogue == _lib.EPI_SWIGLU else sum(group.M)
    need = group.workspace_bytes(T)
    if need < 0:
        _lib.check(need, "bs_forward_group_workspace_bytes")
    if residual is not None:
        residual = _f16c(residual)
        if residual.numel() != T * width:
            raise ValueError("residual does not match the output")
    y = out if out is not None else torch.empty((T, width), dtype=torch.float16, device=dev)
    if y.dtype != torch.float16 or not y.is_contiguous() or y.numel() != T * width:
        raise ValueError("out must be a contiguous fp16 [T, width] tensor")
    ws = _lib.workspace(dev, need)
    with torch.cuda.device(dev):
        if rms_eps is None:
            _lib.check(_lib.lib().bs_forward_group(group.arr, group.n, group.N, group.K, _lib.ptr(x2), T, epilogue,
                                                   _lib.ptr(residual), _lib.ptr(y), _lib.ptr(ws), ws.numel(),
                                                   _lib.stream_ptr(dev)), "bs_forward_group")
        else:
            _lib.check(_lib.lib().bs_forward_group_rms(group.arr, group.n, group.N, group.K, _lib.ptr(x2), T, float(rms_eps),
                                                       epilogue, _lib.ptr(residual), _lib.ptr(y), _lib.ptr(ws), ws.numel(),
                                                       _lib.stream_ptr(dev)), "bs_forward_group_rms")
    return y


def rmsnorm_hip(x, weight, eps, out=None):
    """weight * fp16(x * rsqrt(mean(x^2) + eps)) over the last dimension."""
    dev = _lib.require_gpu(x, weight, out)
    H = x.shape[-1]
    x2, weight = _f16c(x).view(-1, H), _f16c(weight)
    y = out if out is not None else torch.empty_like(x2)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bs_rmsnorm_f16(_lib.ptr(x2), _lib.ptr(weight), _lib.ptr(y), x2.shape[0], H, float(eps),
                                             _lib.stream_ptr(dev)), "bs_rmsnorm_f16")
    return y.view(x.shape)


def attention_decode_hip(qkv, kcache, vcache, cos, sin, pos, heads, kv_heads, out=None):
    """One decode position for B sequences: RoPE on q and k of qkv [B, (heads + 2 kv) * d],
    append k, v at *pos to the caches [B, kv, max_len, d], attention over 0..*pos;
    returns [B, heads * d].  `pos` is a one-element int64 device tensor."""
    dev = _lib.require_gpu(qkv, kcache, vcache, cos, sin, pos, out)
    B = qkv.shape[0]
    d = kcache.shape[-1]
    max_len = kcache.shape[-2]
    if qkv.dtype != torch.float16 or not qkv.is_contiguous() or qkv.shape[1] != (heads + 2 * kv_heads) * d:
        raise ValueError("qkv must be contiguous fp16 [B, (heads + 2 kv_heads) * head_dim]")
    for c in (kcache, vcache):
        if c.dtype != torch.float16 or not c.is_contiguous() or c.numel() != B * kv_heads * max_len * d:
            raise ValueError("caches must be contiguous fp16 [B, kv_heads, max_len, head_dim]")
    if pos.dtype != torch.int64 or pos.numel() != 1:
        raise ValueError("pos must be a one-element int64 tensor")
    if cos.shape != (max_len, d // 2) or sin.shape != (max_len, d // 2) or not cos.is_contiguous() or not sin.is_contiguous():
        raise ValueError("cos / sin must be contiguous [max_len, head_dim / 2]")
    y = out if out is not None else torch.empty((B, heads * d), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bs_attention_decode_f16(_lib.ptr(qkv), _lib.ptr(kcache), _lib.ptr(vcache), _lib.ptr(_f16c(cos)),
                                                      _lib.ptr(_f16c(sin)), _lib.ptr(pos), _lib.ptr(y), B, heads, kv_heads,
                                                      d, max_len, _lib.stream_ptr(dev)), "bs_attention_decode_f16")
    return y


def argmax_hip(x, out=None):
    """Index of the largest value of every row of x [B, V] (fp16), int64 [B]."""
    dev = _lib.require_gpu(x, out)
    if x.dim() != 2 or x.dtype != torch.float16 or not x.is_contiguous():
        raise ValueError("x must be a contiguous fp16 [B, V] tensor")
    y = out if out is not None else torch.empty(x.shape[0], dtype=torch.int64, device=dev)
    if y.dtype != torch.int64 or y.numel() != x.shape[0] or not y.is_contiguous():
        raise ValueError("out must be a contiguous int64 [B] tensor")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bs_argmax_f16(_lib.ptr(x), _lib.ptr(y), x.shape[0], x.shape[1], _lib.stream_ptr(dev)),
                   "bs_argmax_f16")
    return y


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
