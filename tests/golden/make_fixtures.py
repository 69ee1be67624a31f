"""Writes the golden fixtures in this directory (run from the repo root:
`python tests/golden/make_fixtures.py`).

The reference ships no golden vectors, known-answer tests or fixtures for this path, so
these are inputs together with the outputs of the CPU oracle (oracle/bitstack_oracle.py),
which is itself pinned by closed forms, brute force and textbook routines in
tests/test_oracle.py.  What the fixtures add: the exact bytes and numbers that were checked
in this container travel with the repository, so a different numpy / BLAS / torch on another
machine cannot move the oracle unnoticed, and the HIP path is compared with committed
numbers as well as with the oracle run on the spot.

Everything is stored with numpy.savez_compressed (no pickling); inputs are small and seeded.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import bitstack_oracle as O  # noqa: E402


def sign_fixture():
    """pack_sign / unpack_sign (bitstack/utils/pack_utils.py:5-26)."""
    rng = np.random.default_rng(1)
    hand = np.array([[1, -1, -1, -1, -1, -1, -1, -1],        # 0x80
                     [1, 1, 1, 1, 1, 1, 1, 1],               # 0xFF
                     [-1, -1, -1, -1, -1, -1, -1, 1],        # 0x01
                     [1, -1, 1, -1, 1, -1, 1, -1]], dtype=np.int8)   # 0xAA
    ragged = np.where(rng.integers(0, 2, size=(5, 7)) > 0, 1, -1).astype(np.int8)      # 35 signs: 5 padding bits
    block = np.where(rng.integers(0, 2, size=(64, 72)) > 0, 1, -1).astype(np.int8)
    every_byte = np.arange(256, dtype=np.uint8)
    return dict(hand_sign=hand, hand_packed=O.pack_sign(hand),
                ragged_sign=ragged, ragged_packed=O.pack_sign(ragged),
                block_sign=block, block_packed=O.pack_sign(block),
                every_byte=every_byte, every_byte_sign=O.unpack_sign(every_byte, (256, 8)))


def layer_fixture(seed, I, M, N, K, T, signed, with_bias):
    """One small layer: the rebuilt weight (one fp16 rounding of the fp32 sum,
    bitstack/utils/inference_utils.py:79-109), the forward in level-0 rounding order
    (bitstack/modules/BitStackLinear.py:105-114) and in float64."""
    rng = np.random.default_rng(seed)
    q = rng.integers(0, 256, size=(I, (M * N + 7) // 8), dtype=np.uint8)
    scale = (0.3 / np.arange(1, I + 1, dtype=np.float32)).reshape(I, 1, 1)
    u = rng.standard_normal((I, M, K)).astype(np.float32)
    vt = rng.standard_normal((I, K, N)).astype(np.float32)
    if not signed:
        u, vt = np.abs(u), np.abs(vt)
    u, vt = (u * scale).astype(np.float16), (vt * scale).astype(np.float16)
    x = rng.standard_normal((T, N)).astype(np.float16)
    bias = (rng.standard_normal(M) * 0.1).astype(np.float16) if with_bias else None
    out = dict(qweight=q, u=u, vt=vt, x=x,
               w_f16=O.reconstruct_w(q, u, vt),
               y_l0=O.forward_l0(q, u, vt, x, bias), y_f64=O.forward_exact(q, u, vt, x, bias))
    if with_bias:
        out["bias"] = bias
    return out


def decompose_fixture():
    """decompose_weight (bitstack/modules/BitStackLinear.py:49-75): signs, the products
    u_i vt_i (factors are only defined up to a joint sign per rank) and residual norms."""
    rng = np.random.default_rng(3)
    W = (rng.standard_normal((48, 64)) * 0.02).astype(np.float32)
    W[0, 0] = 0.0
    q, u, vt, norms = O.decompose_weight(W, 3, 4)
    prods = np.stack([u[i].astype(np.float64) @ vt[i].astype(np.float64) for i in range(3)])
    return dict(weight=W, qweight=q, products=prods, residual_norms=np.asarray(norms, dtype=np.float64),
                memory_per_bit=np.array([O.memory_per_bit(4096, 4096, 16), O.memory_per_bit(1024, 4096, 16),
                                         O.memory_per_bit(14336, 4096, 16)], dtype=np.int64))


def main():
    np.savez_compressed(os.path.join(HERE, "sign_packing.npz"), **sign_fixture())
    # decode-kernel shape (N a multiple of 512), strip/tiled shape with a ragged M and small rank, odd shape
    np.savez_compressed(os.path.join(HERE, "layer_decode.npz"), **layer_fixture(11, 3, 64, 512, 16, 4, False, True))
    np.savez_compressed(os.path.join(HERE, "layer_strip.npz"), **layer_fixture(12, 2, 50, 256, 7, 20, True, False))
    np.savez_compressed(os.path.join(HERE, "layer_odd.npz"), **layer_fixture(13, 2, 33, 72, 16, 5, True, True))
    np.savez_compressed(os.path.join(HERE, "decompose.npz"), **decompose_fixture())
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
