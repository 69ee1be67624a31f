"""Sign packing helpers with the reference's names and meanings
(bitstack/utils/pack_utils.py), device side in HIP.

pack_sign / unpack_sign keep the reference signatures.  On a HIP tensor they
run the gfx950 kernels; on a CPU tensor they run the same torch expressions
the reference uses (that is the reference's own CPU behaviour, needed for
compression-time code and fused_level 0).
"""
from __future__ import annotations

import torch

from bitstack_amd import _lib


def _pack_sign_torch(w_sign):
    # bitstack/utils/pack_utils.py:5-18
    assert (w_sign.abs() == 1).all()
    binary = ((w_sign + 1) // 2).view(-1)
    n = binary.numel()
    n_padding = (8 - n % 8) % 8
    if n_padding > 0:
        binary = torch.cat([binary, torch.zeros(n_padding, dtype=binary.dtype, device=binary.device)])
    binary = binary.view(-1, 8).to(torch.uint8)
    packed = torch.zeros(binary.size(0), dtype=torch.uint8, device=binary.device)
    for i in range(8):
        packed |= binary[:, i] << (7 - i)
    return packed


def _unpack_sign_torch(packed, original_shape):
    # bitstack/utils/pack_utils.py:20-26
    bit_masks = torch.tensor([128, 64, 32, 16, 8, 4, 2, 1], device=packed.device, dtype=torch.uint8)
    unpacked = ((packed.unsqueeze(-1) & bit_masks) > 0).to(torch.int8).view(-1)
    n = torch.Size(original_shape).numel()
    return unpacked[:n].view(original_shape) * 2 - 1


def pack_sign_hip(w_sign):
    """int8 +-1 tensor of any shape -> uint8[ceil(n/8)] on the same device."""
    dev = _lib.require_gpu(w_sign)
    s = w_sign.to(torch.int8).contiguous().view(-1)
    n = s.numel()
    packed = torch.empty((n + 7) // 8, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bs_pack_sign(_lib.ptr(s), _lib.ptr(packed), n, _lib.stream_ptr(dev)),
                   "bs_pack_sign")
    return packed


def unpack_sign_hip(packed, original_shape):
    """uint8 packed signs -> int8 +-1 of `original_shape`
    (the reference's unpack_sign_triton, pack_utils.py:177-204)."""
    dev = _lib.require_gpu(packed)
    shape = torch.Size(original_shape)
    n = shape.numel()
    p = packed.contiguous().view(-1)
    if p.dtype != torch.uint8:
        raise TypeError(f"packed signs must be uint8, got {p.dtype}")
    if p.numel() * 8 < n:
        raise ValueError(f"{p.numel()} packed bytes cannot hold {n} signs")
    out = torch.empty(n, dtype=torch.int8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().bs_unpack_sign(_lib.ptr(p), _lib.ptr(out), n, _lib.stream_ptr(dev)),
                   "bs_unpack_sign")
    return out.view(shape)


# drop-in alias: callers written against the reference import this name
unpack_sign_triton = unpack_sign_hip


def pack_sign(w_sign):
    if w_sign.is_cuda:
        assert (w_sign.abs() == 1).all()
        return pack_sign_hip(w_sign)
    return _pack_sign_torch(w_sign)


def unpack_sign(packed, original_shape):
    if packed.is_cuda:
        return unpack_sign_hip(packed, original_shape)
    return _unpack_sign_torch(packed, original_shape)


def unpack_sign_v2(packed, original_shape):
    """Same mapping and the same dtype check as the reference's second variant
    (bitstack/utils/pack_utils.py:50-82, a cached-mask rewrite of unpack_sign)."""
    if packed.dtype != torch.uint8:
        raise ValueError(f"Expected packed tensor of dtype torch.uint8, but got {packed.dtype}")
    return unpack_sign(packed, torch.Size(original_shape))

