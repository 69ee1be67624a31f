"""CPU restatement (numpy) of the BitStack compressed-linear forward path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file:
it is the checker that the HIP kernels are compared against (tests, the smoke
entry, and the CPU-baseline leg of the benchmark), never the thing measured.

Every function cites the reference lines it restates (paths relative to the
reference checkout).  How each function is pinned, without running the
reference (which ships no tests, fixtures or golden vectors for this path):

  pack_sign / unpack_sign   numpy.packbits/unpackbits(bitorder='big'), hand
                            known-answer bytes, exhaustive sweep over all 256
                            byte values, round trip, padding case.
  compose_weight            fp64 triple-loop brute force on tiny shapes.
  reconstruct_w             same brute force; block additivity; byte-complement
                            negation.
  forward_exact             brute force; linearity in x; row/column scaling.
  forward_l0                hand-built case where the fp16 running sum loses
                            what an fp32 sum keeps (2048 + 1 + 1), bounded
                            against forward_exact otherwise.
  decompose_weight          Eckart-Young against numpy.linalg.svd, monotone
                            residual, sign(0) = +1, pack/unpack round trip.
  memory_per_bit,
  retrieve_compression_config   closed forms / hand cases.

Parity status: every function above has at least one such pin in
tests/test_oracle.py; none is "parity unpinned".
"""
from __future__ import annotations

import numpy as np

_BIT_MASKS = np.array([128, 64, 32, 16, 8, 4, 2, 1], dtype=np.uint8)


# --------------------------------------------------------------------------- #
# sign packing  (bitstack/utils/pack_utils.py)
# --------------------------------------------------------------------------- #
def pack_sign(w_sign: np.ndarray) -> np.ndarray:
    """pack_utils.py:5-18.  +-1 int8 of any shape -> uint8[ceil(n/8)].

    Flatten row-major, map +1 -> bit 1 and -1 -> bit 0, pad with 0 bits (which
    later decode to -1) up to a multiple of eight, first element of each group
    of eight lands in the most significant bit.
    """
    s = np.asarray(w_sign)
    if not np.all(np.abs(s) == 1):                      # pack_utils.py:6
        raise AssertionError("pack_sign expects +-1 entries")
    bits = ((s.astype(np.int16) + 1) // 2).reshape(-1).astype(np.uint8)
    pad = (8 - bits.size % 8) % 8                        # pack_utils.py:9
    if pad:
        bits = np.concatenate([bits, np.zeros(pad, dtype=np.uint8)])
    groups = bits.reshape(-1, 8)
    packed = np.zeros(groups.shape[0], dtype=np.uint8)
    for i in range(8):                                   # pack_utils.py:16-17
        packed |= (groups[:, i] << np.uint8(7 - i)).astype(np.uint8)
    return packed


def unpack_sign(packed: np.ndarray, original_shape) -> np.ndarray:
    """pack_utils.py:20-26.  uint8[...] -> int8 +-1 of `original_shape`."""
    p = np.asarray(packed, dtype=np.uint8).reshape(-1)
    n = int(np.prod(original_shape, dtype=np.int64))
    hit = (p[:, None] & _BIT_MASKS[None, :]) > 0         # pack_utils.py:21-22
    flat = hit.astype(np.int8).reshape(-1)[:n]
    return (flat * 2 - 1).astype(np.int8).reshape(original_shape)


# --------------------------------------------------------------------------- #
# weight composition  (bitstack/modules/BitStackLinear.py)
# --------------------------------------------------------------------------- #
def _matmul_like_torch(u: np.ndarray, vt: np.ndarray) -> np.ndarray:
    """torch.matmul on fp16 operands returns fp16 after a wider accumulate;
    fp32 operands stay fp32.  (BitStackLinear.py:14 takes the dtype of u.)"""
    if u.dtype == np.float16:
        return (u.astype(np.float32) @ vt.astype(np.float32)).astype(np.float16)
    return u @ vt


def compose_weight(weight_sign, u, vt, no_avd=False, weight_shape=None, packed_sign=True):
    """BitStackLinear.py:7-15.  One block: sign * (u @ vt) in the dtype of u."""
    if no_avd:
        return _matmul_like_torch(u, vt)
    if packed_sign:
        weight_sign = unpack_sign(weight_sign, weight_shape)
    return weight_sign.astype(u.dtype) * _matmul_like_torch(u, vt)


def reconstruct_w(qweight, u, vt, out_dtype=np.float16) -> np.ndarray:
    """Fused reconstruction semantics of levels 2-4
    (inference_utils.py:79-109 and :326-339): per block an fp32 product
    u_i @ vt_i, sign applied, fp32 sum over blocks, ONE rounding to fp16.

    qweight uint8[I, M*N/8], u f16[I, M, K], vt f16[I, K, N] -> f16[M, N].
    """
    I, M, _ = u.shape
    N = vt.shape[2]
    acc = np.zeros((M, N), dtype=np.float32)
    for i in range(I):
        s = unpack_sign(qweight[i], (M, N)).astype(np.float32)
        acc += s * (u[i].astype(np.float32) @ vt[i].astype(np.float32))
    return acc.astype(out_dtype)


def reconstruct_w_exact(qweight, u, vt) -> np.ndarray:
    """Same closed form in fp64 (no intermediate rounding)."""
    I, M, _ = u.shape
    N = vt.shape[2]
    acc = np.zeros((M, N), dtype=np.float64)
    for i in range(I):
        s = unpack_sign(qweight[i], (M, N)).astype(np.float64)
        acc += s * (u[i].astype(np.float64) @ vt[i].astype(np.float64))
    return acc


def forward_l0(qweight, u, vt, x, bias=None) -> np.ndarray:
    """BitStackLinear.py:105-114, the unfused forward, with its rounding order:
    w starts as fp16 zeros; each block's product is rounded to fp16, the sign
    multiply is exact, `w +=` rounds the running sum to fp16 after every block;
    F.linear then contracts x with w (wide accumulate, one rounding to fp16).

    qweight: sequence/array of I packed blocks, u: [I, M, K] f16, vt: [I, K, N]
    f16, x: [..., N] f16, bias: [M] f16 or None -> [..., M] f16.
    """
    I, M, _ = u.shape
    N = vt.shape[2]
    w = np.zeros((M, N), dtype=np.float16)
    for i in range(I):
        w = (w + compose_weight(qweight[i], u[i], vt[i], False, (M, N))).astype(np.float16)
    y = x.astype(np.float32).reshape(-1, N) @ w.astype(np.float32).T
    if bias is not None:
        y = y + bias.astype(np.float32)[None, :]
    return y.astype(np.float16).reshape(x.shape[:-1] + (M,))


def forward_exact(qweight, u, vt, x, bias=None) -> np.ndarray:
    """y = x (sum_i S_i o (U_i Vt_i))^T + b evaluated in fp64."""
    w = reconstruct_w_exact(qweight, u, vt)
    N = w.shape[1]
    y = x.astype(np.float64).reshape(-1, N) @ w.T
    if bias is not None:
        y = y + bias.astype(np.float64)[None, :]
    return y.reshape(x.shape[:-1] + (w.shape[0],))


# --------------------------------------------------------------------------- #
# decomposition  (BitStackLinear.py:49-75) - feeds the single-layer CPU config
# --------------------------------------------------------------------------- #
def decompose_weight(weight: np.ndarray, niter: int, k: int):
    """Iterative sign / rank-k SVD of |residual|.

    Returns (qweight uint8[niter, ceil(M*N/8)], u f16[niter, M, k],
    vt f16[niter, k, N], residual_norms[niter + 1]).  The stored factors are
    fp16 copies; the residual update uses the un-rounded fp32 factors
    (BitStackLinear.py:70-75).  sign(0) counts as +1 (:53-54).
    """
    r = np.asarray(weight, dtype=np.float32).copy()
    M, N = r.shape
    qs, us, vts, norms = [], [], [], [float(np.linalg.norm(r))]
    for _ in range(niter):
        s = np.sign(r).astype(np.int8)
        s[s == 0] = 1
        uu, sv, vv = np.linalg.svd(np.abs(r), full_matrices=False)   # :59
        root = np.sqrt(sv[:k]).astype(np.float32)
        us_k = (uu[:, :k] * root[None, :]).astype(np.float32)        # :61-63
        vt_k = (root[:, None] * vv[:k, :]).astype(np.float32)        # :64
        packed = pack_sign(s)
        assert np.array_equal(unpack_sign(packed, (M, N)), s)        # :68
        qs.append(packed)
        us.append(us_k.astype(np.float16))
        vts.append(vt_k.astype(np.float16))
        w_i = s.astype(np.float32) * (us_k @ vt_k)                   # :72
        assert np.isfinite(w_i).all()                                # :73-74
        r = r - w_i
        norms.append(float(np.linalg.norm(r)))
    return np.stack(qs), np.stack(us), np.stack(vts), norms


# --------------------------------------------------------------------------- #
# bookkeeping
# --------------------------------------------------------------------------- #
def memory_per_bit(out_features: int, in_features: int, k: int, no_avd: bool = False) -> int:
    """BitStackLinear.py:159-171: bytes of one residual block."""
    mem = 0 if no_avd else (out_features * in_features) // 8
    return mem + 2 * (out_features * k + k * in_features)


def retrieve_compression_config(configs, max_memory_MB):
    """model_utils.py:179-187: largest config whose memory fits the budget."""
    budget = max_memory_MB * 1024 ** 2
    for cfg in sorted(configs, key=lambda c: c["memory"], reverse=True):
        if cfg["memory"] <= budget:
            return cfg["layers"]
    raise ValueError(f"No config found within the memory limit {max_memory_MB} MB")


# --------------------------------------------------------------------------- #
# brute force (pure Python loops; tiny shapes only) - used to pin the above
# --------------------------------------------------------------------------- #
def brute_force_forward(qweight, u, vt, x):
    """Literal triple loop over the definition, fp64, bit addressing done by
    hand: element (m, n) of block i lives in byte (m*N+n)//8, bit 7-(m*N+n)%8
    (inference_utils.py:326-339)."""
    I, M, K = u.shape
    N = vt.shape[2]
    xf = x.reshape(-1, N)
    out = [[0.0] * M for _ in range(xf.shape[0])]
    for t in range(xf.shape[0]):
        for m in range(M):
            tot = 0.0
            for i in range(I):
                for n in range(N):
                    flat = m * N + n
                    bit = (int(qweight[i][flat // 8]) >> (7 - flat % 8)) & 1
                    p = 0.0
                    for r in range(K):
                        p += float(u[i, m, r]) * float(vt[i, r, n])
                    tot += (2 * bit - 1) * p * float(xf[t, n])
            out[t][m] = tot
    return np.array(out, dtype=np.float64).reshape(x.shape[:-1] + (M,))
