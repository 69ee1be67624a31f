/*
 * bitstack_hip.h - C ABI of the MI355X (gfx950) BitStack compressed-linear
 * forward path.
 *
 * Every entry point takes plain device pointers and sizes, returns an int
 * status (0 = ok, negative = error, see bs_error_string), never throws, never
 * aborts and never synchronises the host with the device: work is enqueued on
 * the HIP stream that is passed in (a hipStream_t cast to void*, NULL = the
 * default stream).  Tensors are dense and row-major exactly as the reference
 * module stores them after stack_blocks() (bitstack/modules/
 * BitStackLinear.py:183-195):
 *
 *   packed  uint8 [I, M*N/8]  signs, flat row-major over (M, N), first element
 *                             of every group of eight in the most significant
 *                             bit, bit 1 = +1, bit 0 = -1
 *                             (bitstack/utils/pack_utils.py:5-18)
 *   u       fp16  [I, M, K]
 *   vt      fp16  [I, K, N]
 *   x       fp16  [T, N]      y  fp16 [T, M]      bias fp16 [M] or NULL
 *
 * with I = blocks loaded (w_bit), M = out_features, N = in_features,
 * K = rank of a block (1..16), T = tokens.
 */
#ifndef BITSTACK_HIP_H
#define BITSTACK_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BS_OK                 0
#define BS_ERR_NULL          -1   /* a required pointer is NULL                      */
#define BS_ERR_SHAPE         -2   /* non-positive or unsupported dimension           */
#define BS_ERR_RANK          -3   /* K outside 1..16                                 */
#define BS_ERR_ALIGN         -4   /* pointer not aligned as documented               */
#define BS_ERR_WORKSPACE     -5   /* workspace missing or smaller than required      */
#define BS_ERR_NO_DEVICE     -6   /* no HIP device / wrong architecture              */
#define BS_ERR_LIBRARY       -7   /* the vendor GEMM (comparator mode only) failed   */
#define BS_ERR_HIP_BASE   -1000   /* -(1000 + hipError_t) for a failed HIP call      */

/* Library version, major * 10000 + minor * 100 + patch. */
int bs_version(void);

/* Static, human readable text for a status returned by any entry point. */
const char *bs_error_string(int status);

/*
 * Pack n_elems signs (+-1, int8) into ceil(n_elems/8) bytes; tail bits are 0.
 * Replaces pack_sign, bitstack/utils/pack_utils.py:5-18.
 * Entries other than +-1 are not diagnosed on the device: a positive entry
 * packs as +1, anything else as -1.
 */
int bs_pack_sign(const int8_t *sign, uint8_t *packed, int64_t n_elems, void *stream);

/*
 * Unpack n_elems signs from ceil(n_elems/8) bytes into int8 +-1.
 * Replaces unpack_sign / unpack_sign_triton + unpack_sign_kernel,
 * bitstack/utils/pack_utils.py:20-26, :94-138, :177-204.  Bit exact.
 */
int bs_unpack_sign(const uint8_t *packed, int8_t *out, int64_t n_elems, void *stream);

/*
 * w[M, N] (fp16) = sum_i sign_i o (u_i @ vt_i), fp32 accumulation over K and
 * over the blocks, one rounding to fp16, from ALREADY UNPACKED int8 signs
 * [I, M, N].  Replaces reconstruct_w_triton + fused_reconstruct_kernel,
 * bitstack/utils/inference_utils.py:47-115, :135-156.
 */
int bs_reconstruct_w_from_sign(const int8_t *sign, const void *u, const void *vt, void *w,
                               int I, int M, int N, int K, void *stream);

/*
 * Same result straight from the packed signs.  Replaces
 * unpack_and_reconstruct_w_triton (+ _v2) and their kernels,
 * bitstack/utils/inference_utils.py:291-387, :395-488.  Deterministic (no
 * atomics).  Any M, N (bits are addressed through the flat element index);
 * the tiled MFMA kernel runs when N % 128 == 0 and the buffers are 16-byte
 * aligned, a one-output-per-thread kernel otherwise.
 */
int bs_reconstruct_w(const uint8_t *packed, const void *u, const void *vt, void *w,
                     int I, int M, int N, int K, void *stream);

/*
 * Bytes of device scratch bs_forward needs for these dimensions (0 is a valid
 * answer); negative = error status.
 */
int64_t bs_workspace_bytes(int I, int M, int N, int K, int T);

/*
 * y[T, M] = x[T, N] @ (sum_i sign_i o (u_i @ vt_i))^T (+ bias), the whole
 * forward of the layer from packed signs.  Replaces BitStackLinear.forward at
 * fused levels 1-5 (bitstack/modules/BitStackLinear.py:116-157) including
 * reconstruct_and_forward_triton + fused_reconstruct_and_forward_kernel
 * (bitstack/utils/inference_utils.py:171-284).
 *
 * T <= 4 runs the packed-sign GEMV (signs contracted on MFMA against
 * vt_i o x, scaled by u_i, all blocks in one pass; N % 512 == 0); 5 <= T <= 48
 * the strip kernel (16 x 16 patches of the weight rebuilt in registers and
 * multiplied by x at once, the weight never stored; N % 128 == 0; when it does
 * not take the shape, T <= 8 is two GEMV passes); 49 <= T <= 96 the same
 * patches with the strips walked by workgroups of 128 rows, where that beats
 * the next paths (N % 128 == 0, vt of all blocks of a strip within 40 KB of
 * LDS, workgroups that fill the chip or at most 6 blocks); otherwise, up to
 * 128 tokens and 8 blocks (N % 128 == 0), the panel kernel: 128 x 128 tiles of
 * the weight decoded into LDS strip by strip and multiplied on the matrix
 * cores at once, the weight never stored; larger T rebuilds the weight once
 * into `workspace` and runs a dense MFMA GEMM.  Requires
 * N % 8 == 0.  `workspace` must hold bs_workspace_bytes(...) bytes, 256-byte
 * aligned; its contents on entry do not matter and it may be reused by the
 * next call on the same stream.
 */
int bs_forward(const uint8_t *packed, const void *u, const void *vt, const void *x,
               const void *bias, void *y, int I, int M, int N, int K, int T,
               void *workspace, int64_t workspace_bytes, void *stream);

/*
 * bs_forward for callers that cannot allocate device memory or pass a workspace
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  The scratch of the kernels is a
 * device array inside the library, BS_STATIC_SCRATCH_BYTES per GPU, held until
 * the process ends; the call allocates nothing and frees nothing.  Dimensions
 * whose scratch (bs_workspace_bytes in the default dense-kernel mode) exceeds
 * BS_STATIC_SCRATCH_BYTES return
 * BS_ERR_WORKSPACE: 64 MiB holds the partial sums of every 1..4-token forward of
 * the 8B and 70B linear shapes up to 36 blocks and of their 5..8-token forwards
 * up to 12 blocks; the strip kernel at several dozen tokens on the largest
 * matrices and every forward that rebuilds a weight of more than 32 Mi elements
 * (more than 128 tokens, more than 8 blocks above 96 tokens, or N not a
 * multiple of 128) need more and are refused.
 * All calls on one GPU share the one array: calls that overlap in time on the
 * same GPU (different streams, different host threads) race; calls on one
 * stream are ordered and safe.  Same results as bs_forward, bit for bit, for
 * the same arguments (the comparator mode of bs_set_dense_kernel is ignored
 * here: the vendor GEMM needs scratch of its own and allocates when it is set
 * up).  The FIRST call per device and kernel must be made outside stream
 * capture: it looks the array's address up and, for kernels with more than
 * 64 KB of LDS, raises their limit - host-side set-up that a capture does not
 * record.  The array used is that of the device current at the call, which
 * must be the device of `stream`.
 */
#define BS_STATIC_SCRATCH_BYTES (64 << 20)
int bs_forward_static(const uint8_t *packed, const void *u, const void *vt, const void *x,
                      const void *bias, void *y, int I, int M, int N, int K, int T, void *stream);

/*
 * Introspection for benchmarks and tests: which decode kernel instantiation
 * (waves per workgroup, 16-row tiles per wave), how many workgroups and how
 * many partial sums per row and block bs_forward would use for these
 * dimensions; *waves == 0 means the decode kernel does not run them (the
 * strip kernel or the dense path does: more than 4 tokens with N % 128 == 0,
 * more than 8 tokens, N not a multiple of 512).  No counterpart in the reference
 * (Triton picks its configuration by autotuning,
 * bitstack/utils/inference_utils.py:8-39).
 */
int bs_decode_plan(int I, int M, int N, int K, int T, int *waves, int *row_tiles_per_wave,
                   int *workgroups, int *partials_per_row);

/*
 * Which decode kernel bs_forward runs for these dimensions: 0 none (strip kernel
 * or dense path), BS_DECODE_F16 the fp16-MFMA kernel (1..4 tokens per pass),
 * BS_DECODE_MX the block-scaled fp4 x fp6 MFMA kernel (one or two tokens; signs
 * as the fp4 operand, vt o x as three fp6 terms).  For more than four tokens the
 * answer is that of the first pass.  Negative = error status.
 */
#define BS_DECODE_F16 1
#define BS_DECODE_MX  2
int bs_decode_kernel(int I, int M, int N, int K, int T);

/*
 * Introspection for benchmarks and tests: the kernel family bs_forward runs for
 * these dimensions under the calling thread's hook settings (for 5..8 tokens
 * on the decode kernels: that of the first pass).  Negative = error status.
 * No counterpart in the reference (its fused_level is chosen by the caller,
 * bitstack/modules/BitStackLinear.py:116-157).
 */
#define BS_PATH_REBUILD    0   /* weight rebuilt into the workspace, then the dense product */
#define BS_PATH_DECODE_F16 1   /* gemv_kernel: packed-sign GEMV on fp16 MFMA, 1..4 tokens per pass */
#define BS_PATH_DECODE_MX  2   /* gemv_mx_kernel: the same on the block-scaled fp4 x fp6 MFMA, 1..2 tokens */
#define BS_PATH_STRIP      3   /* strip_forward_kernel: 5..48 tokens, patches rebuilt in registers */
#define BS_PATH_WALKED     4   /* strip_wide_kernel: 49..96 tokens, strips walked by 128-row workgroups */
#define BS_PATH_PANEL      5   /* panel_forward_kernel: up to 128 tokens, W tiles decoded into LDS */
int bs_forward_path(int I, int M, int N, int K, int T);

/*
 * Test and benchmark hook: 0 = choose the decode kernel of one- and two-token
 * passes by shape (the default), BS_DECODE_F16 = always the fp16 kernel,
 * BS_DECODE_MX = the block-scaled kernel wherever it takes the shape
 * (N % 512 == 0, at most two tokens).  The setting belongs to the CALLING
 * THREAD (every thread starts at 0): bs_workspace_bytes, bs_decode_plan and
 * bs_forward called from one thread always agree, whatever other threads set.
 * No counterpart in the reference.
 */
int bs_set_decode_kernel(int mode);

/*
 * Test and benchmark hook: which kernel multiplies the rebuilt weight in
 * bs_forward's large-T path.  0 and BS_DENSE_OWN = this library's linear_f16
 * kernels (the default, and the only kernels bs_forward ever picks by itself),
 * BS_DENSE_LIBRARY = hipBLASLt wherever it takes the shape (M and N multiples of
 * 8, 16-byte aligned y): the comparator the own kernels are timed against; in
 * the reference this product is F.linear on the rebuilt weight
 * (bitstack/modules/BitStackLinear.py:132,140,148), which on ROCm is that
 * library.  hipBLASLt is opened at run time; where it is missing, has no kernel
 * for a shape, or the shape is first seen under stream capture (setting the
 * library up is host work that may allocate) the call runs this library's
 * kernel; a failure after the library has accepted the call is returned
 * (BS_ERR_LIBRARY or a HIP status), not papered over.  In library mode
 * bs_workspace_bytes adds 64 MiB of scratch for it behind the rebuilt weight.
 * Per calling thread, like bs_set_decode_kernel.
 */
#define BS_DENSE_OWN     1
#define BS_DENSE_LIBRARY 2
int bs_set_dense_kernel(int mode);

/*
 * Test and benchmark hook: which kernel runs a bs_forward of 49 tokens or more
 * where several take the shape.  0 = by shape (the default),
 * BS_PREFILL_REBUILD = always rebuild the weight and run the dense product,
 * BS_PREFILL_WALKED = the walked strip kernel wherever it takes the shape
 * (49..96 tokens), BS_PREFILL_PANEL = the panel kernel wherever it takes the
 * shape (up to 128 tokens, up to 8 blocks, N % 128 == 0).  bs_workspace_bytes
 * follows the setting.  Per calling thread, like bs_set_decode_kernel.  No
 * counterpart in the reference.
 */
#define BS_PREFILL_REBUILD 1
#define BS_PREFILL_WALKED  2
#define BS_PREFILL_PANEL   3
int bs_set_prefill_kernel(int mode);

/*
 * y[T, M] = x[T, N] @ w[M, N]^T (+ bias) on MFMA, fp32 accumulation: the
 * dense contraction bs_forward uses for large T, exposed for levels 2-4 where
 * the reference calls F.linear on the rebuilt weight
 * (bitstack/modules/BitStackLinear.py:132,140,148).
 */
int bs_linear_f16(const void *x, const void *w, const void *bias, void *y,
                  int T, int M, int N, void *stream);

/*
 * Introspection for benchmarks and tests: the workgroup tile (tokens x output
 * features), the k-step and whether the last k-step is partial (N not a multiple
 * of the step) of the dense kernel bs_linear_f16 - and bs_forward above 48
 * tokens - runs for these dimensions with 16-byte aligned buffers.  32 x 32
 * with *k_step == 0 is the no-LDS kernel for up to 32 tokens, 0 x 0 the
 * one-wave-per-output kernel (N % 8 != 0).  No counterpart in the reference
 * (F.linear picks a vendor kernel).
 */
int bs_linear_plan(int T, int M, int N, int *tile_tokens, int *tile_features, int *k_step, int *k_tail);

/*
 * ---- decode step: several matrices per launch, fused epilogues -----------
 * One decode forward (T <= 48 tokens; more than 8 need N % 128 == 0) of up to 4 compressed matrices that read
 * the same x, in one kernel pair: what q_proj/k_proj/v_proj (or gate_proj/
 * up_proj) of a decoder layer do with three (two) BitStackLinear.forward calls,
 * bitstack/modules/BitStackLinear.py:88-157, each as in bs_forward.  All share
 * N and K; block counts and row counts are per matrix.
 *   BS_EPI_NONE      y[T, sum M_j]: the outputs side by side, matrix j at column
 *                    offset M_0 + ... + M_{j-1}
 *   BS_EPI_RESIDUAL  the same, plus residual[T, sum M_j] (fp16 add of the fp16
 *                    result, as `x + proj(h)` in the decoder layer)
 *   BS_EPI_SWIGLU    n == 2, M_0 == M_1: y[T, M_0] = silu(first) * second
 *                    computed from the fp16-rounded results, as
 *                    `act_fn(gate_proj(h)) * up_proj(h)` in the MLP
 * Only shapes the decode kernel takes (every matrix: N % 512 == 0,
 * M * N < 2^31, alignment as bs_forward); anything else returns BS_ERR_SHAPE
 * and the caller issues bs_forward per matrix.  Workspace as bs_forward, size
 * from bs_forward_group_workspace_bytes (negative = status).
 */
#define BS_EPI_NONE      0
#define BS_EPI_RESIDUAL  1
#define BS_EPI_SWIGLU    2
#define BS_MAX_GROUP     4

typedef struct bs_matrix {
    const uint8_t *packed;   /* [I, M*N/8] */
    const void *u;           /* f16 [I, M, K] */
    const void *vt;          /* f16 [I, K, N] */
    const void *bias;        /* f16 [M] or NULL */
    int32_t I, M;
} bs_matrix;

int64_t bs_forward_group_workspace_bytes(const bs_matrix *mats, int n, int N, int K, int T);

int bs_forward_group(const bs_matrix *mats, int n, int N, int K, const void *x, int T,
                     int epilogue, const void *residual, void *y,
                     void *workspace, int64_t workspace_bytes, void *stream);

/*
 * The same with an RMSNorm in front, without a launch for it: x is the
 * UN-normalised row, every output is multiplied by rsqrt(mean(x[t, :]^2) + eps)
 * before the bias (each workgroup of the reduce kernel recomputes that scalar),
 * and the norm's weight vector is expected folded into the matrices by the
 * caller (vt_i[r, n] * weight[n], done once).  input_layernorm -> q/k/v and
 * post_attention_layernorm -> gate/up of a decoder layer then cost no kernel
 * of their own.
 */
int bs_forward_group_rms(const bs_matrix *mats, int n, int N, int K, const void *x, int T, float eps,
                         int epilogue, const void *residual, void *y,
                         void *workspace, int64_t workspace_bytes, void *stream);

/*
 * y[T, H] = weight o fp16( x * rsqrt(mean(x^2) + eps) ), statistics in fp32:
 * the RMSNorm in front of the attention and MLP linears of a decoder layer
 * (the reference leaves it to the Hugging Face model it patches,
 * bitstack/utils/scale_utils.py:212-221 walks `model.model.layers`).
 * H % 8 == 0, H <= 16384, 16-byte aligned rows.
 */
int bs_rmsnorm_f16(const void *x, const void *weight, void *y, int T, int H, float eps, void *stream);

/*
 * One decode position of grouped-query attention for B sequences that are all
 * at position *pos (device int64): rotate q and k of `qkv`
 * [B, (heads + 2 kv_heads) * head_dim] (rotate-half RoPE with cos/sin
 * [max_len, head_dim / 2]), store k and v at *pos in the caches
 * [B, kv_heads, max_len, head_dim], softmax(q k^T / sqrt(head_dim)) v over
 * positions 0..*pos, write out[B, heads * head_dim].  head_dim == 128,
 * max_len <= 8192.  The step between the q/k/v and o linears of a decoder
 * layer; no counterpart inside the reference repository (Hugging Face's
 * LlamaAttention).
 */
int bs_attention_decode_f16(const void *qkv, void *kcache, void *vcache, const void *cos, const void *sin,
                            const int64_t *pos, void *out, int B, int heads, int kv_heads, int head_dim,
                            int max_len, void *stream);

/*
 * out[b] = index of the largest of x[b, 0..V) (fp16; the lowest index among
 * equal values): the greedy token of a decode step from the logits.  Rows must
 * start 16-byte aligned (V % 8 == 0 when B > 1).  No counterpart in the
 * reference (generation is left to Hugging Face code).
 */
int bs_argmax_f16(const void *x, int64_t *out, int B, int V, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* BITSTACK_HIP_H */
