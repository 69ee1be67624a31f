"""The reference's CPU path (fused_level 0) restated with torch-CPU ops, for
timing the CPU baseline.  TEST / BENCHMARK INFRASTRUCTURE ONLY; the shipped
package never imports it.

Follows bitstack/modules/BitStackLinear.py:105-114 and :7-15 and
bitstack/utils/pack_utils.py:20-26 step by step (mask-broadcast unpack, fp16
u @ vt per block, fp16 running sum of the weight, F.linear), because the cost
of exactly those temporaries is what the reference pays on a CPU.
"""
import torch
import torch.nn.functional as F

_MASKS = torch.tensor([128, 64, 32, 16, 8, 4, 2, 1], dtype=torch.uint8)


def unpack_sign(packed, shape):
    s = ((packed.unsqueeze(-1) & _MASKS) > 0).to(torch.int8).view(-1)
    return s[: shape.numel()].view(shape) * 2 - 1


@torch.no_grad()
def forward_l0(qweight, u, vt, x, bias=None):
    """qweight uint8[I, M*N/8], u f16[I,M,K], vt f16[I,K,N], x f16[..., N] (CPU tensors)."""
    I, M, _ = u.shape
    N = vt.shape[2]
    shape = torch.Size((M, N))
    w = torch.zeros(shape, dtype=torch.float16)
    for i in range(I):
        w += unpack_sign(qweight[i], shape).to(torch.float16) * torch.matmul(u[i], vt[i])
    return F.linear(x, w, bias=bias)
