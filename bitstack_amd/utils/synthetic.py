"""Seeded synthetic BitStack layers (no checkpoints, no network).

The recipe is the benchmark's: packed signs are uniform random bytes (every
bit an independent fair coin in the storage format), u and vt are |N(0,1)|
scaled by 0.01 / block_index (block_index starts at 1) so later residual
blocks are smaller, x is N(0,1).  Everything is drawn on the CPU from one
torch.Generator in the fixed order signs, u, vt, x, so a CPU checker and the
GPU kernels see identical bits.
"""
from __future__ import annotations

import torch

# (out_features, in_features) of the Llama-3.1-8B decoder linears
LLAMA8B_SHAPES = {
    "q_proj": (4096, 4096),
    "k_proj": (1024, 4096),
    "v_proj": (1024, 4096),
    "o_proj": (4096, 4096),
    "gate_proj": (14336, 4096),
    "up_proj": (14336, 4096),
    "down_proj": (4096, 14336),
}


def synthetic_layer(M, N, I, T, k=16, seed=0, device="cpu", signed_factors=False):
    """Returns (qweight uint8[I, ceil(M*N/8)], u f16[I,M,k], vt f16[I,k,N], x f16[T,N])."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randint(0, 256, (I, (M * N + 7) // 8), dtype=torch.uint8, generator=g)
    scale = (0.01 / torch.arange(1, I + 1, dtype=torch.float32)).view(I, 1, 1)
    u = torch.randn(I, M, k, generator=g)
    vt = torch.randn(I, k, N, generator=g)
    if not signed_factors:
        u, vt = u.abs(), vt.abs()
    u, vt = (u * scale).half(), (vt * scale).half()
    x = torch.randn(T, N, generator=g).half()
    dev = torch.device(device)
    return q.to(dev), u.to(dev), vt.to(dev), x.to(dev)


def algorithmic_bytes(I, M, N, T, k=16, bias=False):
    """Bytes one forward must move: signs + u + vt once, x in, y out."""
    return I * (M * N // 8 + 2 * k * (M + N)) + 2 * T * (N + M) + (2 * M if bias else 0)
