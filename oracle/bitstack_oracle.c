/*
 * CPU restatement (plain C) of the BitStack compressed-linear forward path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels at sizes where the
 * numpy restatement (bitstack_oracle.py, same directory) would take too long.
 * The shipped library never links or loads this file.
 *
 * Reference lines restated (paths relative to the reference checkout):
 *   bso_pack_sign        bitstack/utils/pack_utils.py:5-18
 *   bso_unpack_sign      bitstack/utils/pack_utils.py:20-26
 *   bso_reconstruct_w    bitstack/utils/inference_utils.py:79-109, :326-339
 *   bso_forward_l0       bitstack/modules/BitStackLinear.py:105-114 (+ :7-15)
 *   bso_forward_f64      the closed form y = x (sum_i S_i o (U_i Vt_i))^T + b
 *
 * Pinned in tests/test_oracle.py against the numpy restatement, which in turn
 * is pinned against numpy.packbits, hand known-answer vectors and fp64 brute
 * force.  fp16 <-> fp32 conversion is done by hand (round to nearest even) and
 * is itself checked against numpy over all 65536 half patterns.
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp -shared -fPIC)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* IEEE binary16 <-> binary32, round to nearest even                         */
/* ------------------------------------------------------------------------ */
static inline float h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static inline uint16_t f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) {                       /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x200u : 0));
    }
    if (absx >= 0x477FF000u) {                       /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx < 0x38800000u) {                        /* below 2^-14: subnormal half */
        if (absx < 0x33000000u) return (uint16_t)sign;   /* < 2^-25 -> 0 */
        int e = (int)(absx >> 23);
        uint32_t man = (absx & 0x7FFFFFu) | 0x800000u;
        int shift = 126 - e;                         /* 14..24 */
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((absx - 0x38000000u) >> 13);
    uint32_t rem = absx & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
    return (uint16_t)(sign | half);
}

void bso_h2f(const uint16_t *in, float *out, int64_t n)
{
    for (int64_t i = 0; i < n; i++) out[i] = h2f(in[i]);
}

void bso_f2h(const float *in, uint16_t *out, int64_t n)
{
    for (int64_t i = 0; i < n; i++) out[i] = f2h(in[i]);
}

/* ------------------------------------------------------------------------ */
/* sign packing                                                              */
/* ------------------------------------------------------------------------ */
/* pack_utils.py:5-18.  Returns -1 when an entry is not +-1 (the reference
 * asserts), otherwise the number of bytes written = ceil(n / 8). */
int64_t bso_pack_sign(const int8_t *sign, int64_t n, uint8_t *packed)
{
    int64_t nbytes = (n + 7) / 8;
    for (int64_t j = 0; j < nbytes; j++) {
        uint8_t b = 0;
        for (int i = 0; i < 8; i++) {
            int64_t e = 8 * j + i;
            if (e >= n) break;                       /* zero padding, pack_utils.py:9-12 */
            if (sign[e] != 1 && sign[e] != -1) return -1;
            if (sign[e] == 1) b |= (uint8_t)(1u << (7 - i));
        }
        packed[j] = b;
    }
    return nbytes;
}

/* pack_utils.py:20-26. */
void bso_unpack_sign(const uint8_t *packed, int64_t n, int8_t *out)
{
    for (int64_t e = 0; e < n; e++) {
        int bit = (packed[e >> 3] >> (7 - (e & 7))) & 1;
        out[e] = (int8_t)(2 * bit - 1);
    }
}

static inline float sign_at(const uint8_t *q, int64_t flat)
{
    return ((q[flat >> 3] >> (7 - (flat & 7))) & 1) ? 1.0f : -1.0f;
}

/* ------------------------------------------------------------------------ */
/* levels 2-4: fp32 product, fp32 sum over blocks, one rounding              */
/* ------------------------------------------------------------------------ */
void bso_reconstruct_w(const uint8_t *q, const uint16_t *u, const uint16_t *vt,
                       int I, int M, int N, int K, uint16_t *w_out)
{
    int64_t bytes_per_block = ((int64_t)M * N + 7) / 8;
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        float *acc = (float *)calloc((size_t)N, sizeof(float));
        float *vrow = (float *)malloc((size_t)N * sizeof(float));
        for (int i = 0; i < I; i++) {
            const uint8_t *qi = q + (int64_t)i * bytes_per_block;
            const uint16_t *ui = u + ((int64_t)i * M + m) * K;
            const uint16_t *vti = vt + (int64_t)i * K * N;
            for (int n = 0; n < N; n++) vrow[n] = 0.0f;
            for (int r = 0; r < K; r++) {
                float ur = h2f(ui[r]);
                const uint16_t *vr = vti + (int64_t)r * N;
                for (int n = 0; n < N; n++) vrow[n] += ur * h2f(vr[n]);
            }
            for (int n = 0; n < N; n++)
                acc[n] += sign_at(qi, (int64_t)m * N + n) * vrow[n];
        }
        for (int n = 0; n < N; n++) w_out[(int64_t)m * N + n] = f2h(acc[n]);
        free(acc);
        free(vrow);
    }
}

/* ------------------------------------------------------------------------ */
/* level 0: fp16 product per block, fp16 running sum, then the linear        */
/* ------------------------------------------------------------------------ */
void bso_forward_l0(const uint8_t *q, const uint16_t *u, const uint16_t *vt,
                    const uint16_t *x, const uint16_t *bias,
                    int I, int M, int N, int K, int T, uint16_t *y)
{
    int64_t bytes_per_block = ((int64_t)M * N + 7) / 8;
    float *xf = (float *)malloc((size_t)T * N * sizeof(float));
    for (int64_t j = 0; j < (int64_t)T * N; j++) xf[j] = h2f(x[j]);
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        uint16_t *w = (uint16_t *)calloc((size_t)N, sizeof(uint16_t));   /* fp16 zeros, :107 */
        float *p = (float *)malloc((size_t)N * sizeof(float));
        for (int i = 0; i < I; i++) {
            const uint8_t *qi = q + (int64_t)i * bytes_per_block;
            const uint16_t *ui = u + ((int64_t)i * M + m) * K;
            const uint16_t *vti = vt + (int64_t)i * K * N;
            for (int n = 0; n < N; n++) p[n] = 0.0f;
            for (int r = 0; r < K; r++) {
                float ur = h2f(ui[r]);
                const uint16_t *vr = vti + (int64_t)r * N;
                for (int n = 0; n < N; n++) p[n] += ur * h2f(vr[n]);
            }
            for (int n = 0; n < N; n++) {
                float prod = h2f(f2h(p[n]));                              /* matmul -> fp16, :14 */
                float wi = sign_at(qi, (int64_t)m * N + n) * prod;        /* exact */
                w[n] = f2h(h2f(w[n]) + wi);                               /* fp16 +=, :111-113 */
            }
        }
        for (int t = 0; t < T; t++) {
            float acc = 0.0f;
            const float *xt = xf + (int64_t)t * N;
            for (int n = 0; n < N; n++) acc += xt[n] * h2f(w[n]);
            if (bias) acc += h2f(bias[m]);
            y[(int64_t)t * M + m] = f2h(acc);
        }
        free(w);
        free(p);
    }
    free(xf);
}

/* ------------------------------------------------------------------------ */
/* closed form in fp64                                                       */
/* ------------------------------------------------------------------------ */
void bso_forward_f64(const uint8_t *q, const uint16_t *u, const uint16_t *vt,
                     const uint16_t *x, const uint16_t *bias,
                     int I, int M, int N, int K, int T, double *y)
{
    int64_t bytes_per_block = ((int64_t)M * N + 7) / 8;
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        double *w = (double *)calloc((size_t)N, sizeof(double));
        double *p = (double *)malloc((size_t)N * sizeof(double));
        for (int i = 0; i < I; i++) {
            const uint8_t *qi = q + (int64_t)i * bytes_per_block;
            const uint16_t *ui = u + ((int64_t)i * M + m) * K;
            const uint16_t *vti = vt + (int64_t)i * K * N;
            for (int n = 0; n < N; n++) p[n] = 0.0;
            for (int r = 0; r < K; r++) {
                double ur = (double)h2f(ui[r]);
                const uint16_t *vr = vti + (int64_t)r * N;
                for (int n = 0; n < N; n++) p[n] += ur * (double)h2f(vr[n]);
            }
            for (int n = 0; n < N; n++)
                w[n] += (double)sign_at(qi, (int64_t)m * N + n) * p[n];
        }
        for (int t = 0; t < T; t++) {
            double acc = 0.0;
            for (int n = 0; n < N; n++) acc += (double)h2f(x[(int64_t)t * N + n]) * w[n];
            if (bias) acc += (double)h2f(bias[m]);
            y[(int64_t)t * M + m] = acc;
        }
        free(w);
        free(p);
    }
}

int bso_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
