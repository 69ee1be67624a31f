"""BitStackLinear for MI355X: the reference module's interface
(bitstack/modules/BitStackLinear.py) with the forwards running on hand-written
HIP kernels.

Kept from the reference: constructor and from_linear signatures, buffer names /
dtypes / shapes (`qweight_i`, `u_i`, `vt_i`, optional `bias`; stacked
`qweight`, `u`, `vt` after stack_blocks), the fused_level switch and its error,
set_bit / pop_one_bit / add_one_bit (counter only), memory_per_bit,
decompose_weight, compose_weight, ScaledActivation.

fused_level on this build:
  0  torch ops only, block by block (the reference's level 0; CPU or GPU)
  1  HIP unpack of all blocks -> torch batched matmul / mul / sum -> F.linear
  2  HIP unpack -> HIP reconstruct from int8 signs -> F.linear
  3  HIP fused unpack + reconstruct from packed signs -> F.linear
  4  as 3 (deterministic; the reference's fp16 atomics are not reproduced)
     followed by the library's own MFMA linear instead of F.linear
  5  one C-ABI call for the whole forward: packed-sign MFMA GEMV for <= 4
     tokens, weight patches rebuilt in registers for 5..48, rebuild-once +
     MFMA GEMM above.  Unlike the reference's level 5
     it takes any [..., N] input and a bias.
Levels 1-5 need the tensors on a HIP device and the built shared library;
there is no fallback.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from bitstack_amd.utils.pack_utils import pack_sign, unpack_sign, unpack_sign_hip
from bitstack_amd.utils.inference_utils import (
    bitstack_forward_hip,
    linear_f16_hip,
    reconstruct_w_hip,
    unpack_and_reconstruct_w_hip,
)


def compose_weight(weight_sign, u, vt, no_avd=False, weight_shape=None, packed_sign=True):
    """One block's contribution, in the dtype of u (BitStackLinear.py:7-15)."""
    if no_avd:
        return u @ vt
    if packed_sign:
        weight_sign = unpack_sign(weight_sign, weight_shape)
    return weight_sign.to(u.dtype) * torch.matmul(u, vt)


class ScaledActivation(nn.Module):
    """BitStackLinear.py:18-25."""

    def __init__(self, module, scales):
        super().__init__()
        self.act = module
        self.scales = nn.Parameter(scales.data)

    def forward(self, x):
        return self.act(x) / self.scales.view(1, 1, -1).to(x.device)


class BitStackLinear(nn.Module):
    def __init__(self, w_bit, in_features, out_features, k, bias, no_avd, dev, fused_level=0):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.w_bit = w_bit
        # BitStackLinear.py:33: the ablation without signs gets the sign bytes back as extra rank
        self.k = k if not no_avd else (in_features * out_features) // (16 * (in_features + out_features)) + k
        self.no_avd = no_avd
        self.fused_level = fused_level
        self.name = None
        for i in range(self.w_bit):
            if not no_avd:
                self.register_buffer(f"qweight_{i}", torch.zeros((out_features * in_features) // 8, dtype=torch.uint8))
            self.register_buffer(f"u_{i}", torch.zeros(out_features, self.k, dtype=torch.float16))
            self.register_buffer(f"vt_{i}", torch.zeros(self.k, in_features, dtype=torch.float16))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=torch.float16))
        else:
            self.bias = None

    # ------------------------------------------------------------------ build
    def decompose_weight(self, original_weight):
        """Iterative sign / rank-k SVD of |residual| (BitStackLinear.py:49-75)."""
        residual = original_weight.to(torch.float32)
        shape = residual.data.shape
        for i in range(self.w_bit):
            sign = residual.sign()
            sign[sign == 0] = 1
            target = residual if self.no_avd else residual.abs()
            uu, sv, vv = torch.linalg.svd(target, full_matrices=False)
            root = torch.sqrt(sv[: self.k])
            us_k = uu[:, : self.k] * root.unsqueeze(0)
            vt_k = root.unsqueeze(1) * vv[: self.k, :]
            packed = None
            if not self.no_avd:
                packed = pack_sign(sign.to(torch.int8))
                assert unpack_sign(packed, shape).equal(sign.to(torch.int8))
                setattr(self, f"qweight_{i}", packed)
            setattr(self, f"u_{i}", us_k.to(torch.float16).contiguous())
            setattr(self, f"vt_{i}", vt_k.to(torch.float16).contiguous())
            w_i = compose_weight(packed, us_k, vt_k, self.no_avd, shape)   # fp32 factors on purpose
            assert torch.isinf(w_i).sum() == 0
            assert torch.isnan(w_i).sum() == 0
            residual = residual - w_i

    @classmethod
    def from_linear(cls, linear, w_bit, k=1, bias=True, no_avd=False, fused_level=0, name=None, init_only=False):
        qlinear = cls(w_bit=w_bit, in_features=linear.in_features, out_features=linear.out_features,
                      bias=bias, k=k, no_avd=no_avd, dev=linear.weight.device, fused_level=fused_level)
        qlinear.name = name
        if init_only:
            return qlinear
        qlinear.decompose_weight(linear.weight)
        if bias:
            qlinear.bias = linear.bias
        return qlinear

    # ---------------------------------------------------------------- forward
    @torch.no_grad()
    def forward(self, x):
        level = self.fused_level
        if level == 0:
            return self.forward_l0(x)
        if level == 1:
            return self.forward_l1(x)
        if level == 2:
            return self.forward_l2(x)
        if level == 3:
            return self.forward_l3(x)
        if level == 4:
            return self.forward_l4(x)
        if level == 5:
            return self.forward_l5(x)
        raise ValueError(f"Invalid fused_level: {self.fused_level}")

    def _stacked(self):
        if not hasattr(self, "u") or self.u is None:
            raise RuntimeError("fused_level >= 1 reads the stacked buffers: call stack_blocks() first")
        assert not self.no_avd   # the sign-free ablation only exists at level 0
        if self.w_bit > self.u.shape[0]:
            raise RuntimeError(f"w_bit={self.w_bit} exceeds the {self.u.shape[0]} stacked blocks")
        b = self.w_bit
        return self.qweight[:b], self.u[:b], self.vt[:b]

    @torch.no_grad()
    def forward_l0(self, x):
        # BitStackLinear.py:105-114: fp16 product per block, fp16 running sum
        w = torch.zeros((self.out_features, self.in_features), dtype=torch.float16, device=x.device)
        for i in range(self.w_bit):
            q = None if self.no_avd else getattr(self, f"qweight_{i}")
            w += compose_weight(q, getattr(self, f"u_{i}"), getattr(self, f"vt_{i}"), self.no_avd, w.shape)
        return F.linear(x, w, bias=self.bias)

    @torch.no_grad()
    def forward_l1(self, x):
        q, u, vt = self._stacked()
        sign = unpack_sign_hip(q.reshape(-1), torch.Size([self.w_bit, self.out_features, self.in_features]))
        w = torch.matmul(u, vt)
        w = (w.mul_(sign)).sum(dim=0).contiguous()
        return F.linear(x, w, bias=self.bias)

    @torch.no_grad()
    def forward_l2(self, x):
        q, u, vt = self._stacked()
        sign = unpack_sign_hip(q.reshape(-1), torch.Size([self.w_bit, self.out_features, self.in_features]))
        return F.linear(x, reconstruct_w_hip(sign, u, vt), bias=self.bias)

    @torch.no_grad()
    def forward_l3(self, x):
        q, u, vt = self._stacked()
        return F.linear(x, unpack_and_reconstruct_w_hip(q, u, vt), bias=self.bias)

    @torch.no_grad()
    def forward_l4(self, x):
        q, u, vt = self._stacked()
        return linear_f16_hip(x, unpack_and_reconstruct_w_hip(q, u, vt), self.bias)

    @torch.no_grad()
    def forward_l5(self, x):
        q, u, vt = self._stacked()
        return bitstack_forward_hip(q, u, vt, x, self.bias)

    # ------------------------------------------------------------ bookkeeping
    def memory_per_bit(self):
        # BitStackLinear.py:159-171: bytes of one block
        memory = 0
        if self.fused_level == 0:
            if not self.no_avd:
                memory += self.qweight_0.numel() * self.qweight_0.element_size()
            for t in (self.u_0, self.vt_0):
                memory += t.numel() * t.element_size()
        else:
            if not self.no_avd:
                memory += self.qweight[0].numel() * self.qweight[0].element_size()
            for t in (self.u[0], self.vt[0]):
                memory += t.numel() * t.element_size()
        return memory

    def pop_one_bit(self):
        # counter only, nothing is freed (BitStackLinear.py:173-175)
        self.w_bit -= 1

    def add_one_bit(self):
        self.w_bit += 1

    def set_bit(self, bit):
        self.w_bit = bit

    def stack_blocks(self):
        """Per-block buffers -> contiguous [I, ...] tensors (BitStackLinear.py:183-195)."""
        if not self.no_avd:
            self.qweight = torch.stack([getattr(self, f"qweight_{i}") for i in range(self.w_bit)])
        self.u = torch.stack([getattr(self, f"u_{i}") for i in range(self.w_bit)])
        self.vt = torch.stack([getattr(self, f"vt_{i}") for i in range(self.w_bit)])
        for i in range(self.w_bit):
            if not self.no_avd:
                delattr(self, f"qweight_{i}")
            delattr(self, f"u_{i}")
            delattr(self, f"vt_{i}")

    # ---- beyond the reference: blocks that really come and go ----------------
    # The reference's pop_one_bit / add_one_bit only move a counter
    # (BitStackLinear.py:173-178); these two move memory, on the stacked layout.
    def trim_blocks(self):
        """Give back the memory of the stacked blocks beyond w_bit."""
        if not hasattr(self, "u") or self.u is None or self.u.shape[0] <= self.w_bit:
            return 0
        per_block = self.u[0].numel() * 2 + self.vt[0].numel() * 2 + (0 if self.no_avd else self.qweight[0].numel())
        freed = (self.u.shape[0] - self.w_bit) * per_block
        keep = self.w_bit
        self.u = self.u[:keep].clone()
        self.vt = self.vt[:keep].clone()
        if not self.no_avd:
            self.qweight = self.qweight[:keep].clone()
        return freed

    def append_blocks(self, qweight, u, vt):
        """Stack further blocks ([n, M*N/8] uint8, [n, M, k], [n, k, N] fp16) behind the
        loaded ones and count them in."""
        if not hasattr(self, "u") or self.u is None:
            raise RuntimeError("append_blocks works on the stacked layout: call stack_blocks() first")
        if self.w_bit != self.u.shape[0]:
            raise RuntimeError("blocks beyond w_bit are still stacked: trim_blocks() first")
        n = u.shape[0]
        if u.shape[1:] != self.u.shape[1:] or vt.shape[1:] != self.vt.shape[1:] or vt.shape[0] != n:
            raise ValueError("block shapes do not match the layer")
        dev = self.u.device
        self.u = torch.cat([self.u, u.to(dev, torch.float16)])
        self.vt = torch.cat([self.vt, vt.to(dev, torch.float16)])
        if not self.no_avd:
            if qweight is None or qweight.shape != (n, self.qweight.shape[1]) or qweight.dtype != torch.uint8:
                raise ValueError("packed signs do not match the layer")
            self.qweight = torch.cat([self.qweight, qweight.to(dev)])
        self.w_bit += n

