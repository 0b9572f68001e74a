/*
 * CPU oracle for the block-scaled FP8 GEMM  C[M,N] (bf16) = A . B^T.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the GPU kernels are compared
 * against and the CPU baseline that is timed beside them.  Nothing in the shipped
 * library links, loads or calls it; only tests, the smoke check and the benchmark's
 * cpu_baseline leg do.
 *
 * It restates, in plain C, the arithmetic of the reference's only executable
 * definition of the operation:
 *   - /root/reference/check.cu:30-49  (ref_kernel: indexing, per-128-K-block fp32 sum,
 *     "result += block * as * bs" evaluated left to right, final cast to bf16)
 *   - /root/reference/utils.h:65-76   (gemmCPU: the i / j / t host loop nest)
 *   - /root/reference/check.cu:17-22  (convert_float_to_fp8: fp32 -> fp8, saturating, RNE)
 *   - /root/reference/quantize.py:16-67 (1x128 and 128x128 quantisers; scale = max/amax as
 *     torch evaluates it, returned inverse scale = 1/scale), with FP8 max = 448 (OCP e4m3fn)
 *     instead of the MI300 fnuz flavour.
 *
 * Layouts (check.cu:42-48):  a byte at m + k*M, b byte at n + k*N, a_scale at m + kb*M,
 * b_scale at nb + kb*ceil(N/128), c at m*N + n.
 *
 * Pinned by tests/test_oracle_*.py:
 *   codec        - brute-force nearest-even over all finite codes, torch float8_e4m3fn,
 *                  exhaustive decode table from the OCP bit layout
 *   bf16         - closed-form RNE against torch.bfloat16 on random and tie cases
 *   ref_gemm     - exact int64 fixed-point block sums -> fp64 (oracle_ref_gemm_f64),
 *                  numpy matmul for unit scales, one-hot index pins, Fraction brute force,
 *                  the reference's own gemmCPU/genMat built from its header where available
 *   quantisers   - the reference's own outputs for fp32 and bf16 sources, bit for bit
 *                  (tests/golden/quantize_reference.npz), closed-form invariants (max code 448
 *                  per group, half-ulp error bound, zero group), layout pins
 * ref_gemm_rows (the n-vectorised loop order) is pinned bit-for-bit to ref_gemm_naive.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define KBLK 128

/* ------------------------------------------------------------------ fp8 e4m3fn / bf16 */

/* OCP e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa; no inf; 0x7F / 0xFF are NaN. */
float oracle_e4m3fn_to_f32(uint8_t v)
{
    int s = v >> 7, e = (v >> 3) & 15, m = v & 7;
    float r;
    if (e == 15 && m == 7)
        r = NAN;
    else if (e == 0)
        r = ldexpf((float)m, -9);
    else
        r = ldexpf((float)(8 + m), e - 10);
    return s ? -r : r;
}

/* fp32 -> e4m3fn, round to nearest even, saturate finite (|x| > 448 and inf -> +-448),
 * NaN -> 0x7F | sign.  Same contract as the cast in check.cu:20 on OCP hardware. */
uint8_t oracle_f32_to_e4m3fn(float x)
{
    uint32_t u;
    memcpy(&u, &x, 4);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    if (isnan(x))
        return sign | 0x7F;
    float ax = fabsf(x);
    if (ax >= 448.0f)
        return sign | 0x7E;
    if (ax < 0.015625f) { /* below the smallest normal 2^-6: fixed step 2^-9 */
        int q = (int)nearbyintf(ax * 512.0f);
        return sign | (uint8_t)q; /* q == 8 is exactly the code of 2^-6 */
    }
    int e;
    float f = frexpf(ax, &e);             /* ax = f * 2^e, f in [0.5, 1) */
    int m = (int)nearbyintf(f * 16.0f);   /* 8..16, ties to even */
    if (m == 16) {
        m = 8;
        e += 1;
    }
    int code = ((e + 6) << 3) | (m - 8);
    if (code > 0x7E)
        code = 0x7E;
    return sign | (uint8_t)code;
}

/* fp32 -> bf16, round to nearest even; NaN stays NaN (quiet). */
uint16_t oracle_f32_to_bf16(float x)
{
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u)
        return (uint16_t)((u >> 16) | 0x40);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float oracle_bf16_to_f32(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void oracle_f32_to_e4m3fn_array(const float *in, uint8_t *out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = oracle_f32_to_e4m3fn(in[i]);
}

void oracle_e4m3fn_to_f32_array(const uint8_t *in, float *out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = oracle_e4m3fn_to_f32(in[i]);
}

void oracle_f32_to_bf16_array(const float *in, uint16_t *out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = oracle_f32_to_bf16(in[i]);
}

void oracle_bf16_to_f32_array(const uint16_t *in, float *out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = oracle_bf16_to_f32(in[i]);
}

/* ------------------------------------------------------------------ the GEMM itself */

/* Literal restatement: utils.h:65-76's i / j / t nest around check.cu:36-48's body. */
void oracle_ref_gemm_naive(const uint8_t *a, const uint8_t *b, const float *as, const float *bs,
                           uint16_t *c, int m, int n, int k)
{
    float lut[256];
    for (int v = 0; v < 256; ++v)
        lut[v] = oracle_e4m3fn_to_f32((uint8_t)v);
    int sn = (n + KBLK - 1) / KBLK;
    for (int i = 0; i < m; ++i) {
        for (int j = 0; j < n; ++j) {
            float result = 0.0f;
            for (int t = 0; t < k; t += KBLK) {
                float block_result = 0.0f;
                for (int ii = 0; ii < KBLK; ++ii) {
                    float av = lut[a[(size_t)i + (size_t)(t + ii) * m]];
                    float bv = lut[b[(size_t)j + (size_t)(t + ii) * n]];
                    block_result += av * bv; /* product of two e4m3 values is exact in fp32 */
                }
                float scaled = block_result * as[i + (size_t)(t / KBLK) * m];
                scaled = scaled * bs[j / KBLK + (size_t)(t / KBLK) * sn];
                result += scaled;
            }
            c[(size_t)i * n + j] = oracle_f32_to_bf16(result);
        }
    }
}

/* Same arithmetic, same order of every floating-point operation per output element
 * (ascending ii inside a block, ascending block index outside), but the loops are
 * arranged so the compiler vectorises across n, which is the contiguous direction of b.
 * Rows are independent and spread over OpenMP threads.  out_f32 (optional, may be NULL)
 * receives the fp32 value before the bf16 cast. */
#define JT 64
/* block_dot.c: blk[j] = sum over ii (ascending) of ar[ii] * bp[ii*ldb + j], j < jw <= 64 */
void oracle_block_dot(const float *ar, const float *bp, size_t ldb, float *blk, int jw);
void oracle_ref_gemm(const uint8_t *a, const uint8_t *b, const float *as, const float *bs,
                     uint16_t *c, float *out_f32, int m, int n, int k, int nthreads)
{
    float lut[256];
    for (int v = 0; v < 256; ++v)
        lut[v] = oracle_e4m3fn_to_f32((uint8_t)v);
    int sn = (n + KBLK - 1) / KBLK;
    int nkb = k / KBLK;
    /* decode b once: bf[k][n] */
    float *bf = (float *)malloc((size_t)k * n * sizeof(float));
    if (!bf)
        return;
#ifdef _OPENMP
    if (nthreads <= 0)
        nthreads = omp_get_max_threads();
#else
    nthreads = 1;
#endif
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (long idx = 0; idx < (long)k * n; ++idx)
        bf[idx] = lut[b[idx]];

    enum { RB = 8 };
#pragma omp parallel num_threads(nthreads)
    {
        float *arow = (float *)malloc((size_t)RB * k * sizeof(float));
        float *acc = (float *)malloc((size_t)RB * JT * sizeof(float));
#pragma omp for schedule(dynamic, 1)
        for (int i0 = 0; i0 < m; i0 += RB) {
            int rb = (m - i0 < RB) ? (m - i0) : RB;
            for (int t = 0; t < k; ++t)
                for (int r = 0; r < rb; ++r)
                    arow[(size_t)r * k + t] = lut[a[(size_t)(i0 + r) + (size_t)t * m]];
            for (int j0 = 0; j0 < n; j0 += JT) {
                int jw = (n - j0 < JT) ? (n - j0) : JT;
                for (int x = 0; x < rb * JT; ++x)
                    acc[x] = 0.0f;
                for (int kb = 0; kb < nkb; ++kb) {
                    for (int r = 0; r < rb; ++r) {
                        float blk[JT];
                        const float *ar = arow + (size_t)r * k + (size_t)kb * KBLK;
                        const float *bp = bf + (size_t)kb * KBLK * n + j0;
                        float sa = as[(i0 + r) + (size_t)kb * m];
                        oracle_block_dot(ar, bp, (size_t)n, blk, jw);
                        float *ac = acc + r * JT;
                        for (int j = 0; j < jw; ++j) {
                            float scaled = blk[j] * sa;
                            scaled = scaled * bs[(j0 + j) / KBLK + (size_t)kb * sn];
                            ac[j] += scaled;
                        }
                    }
                }
                for (int r = 0; r < rb; ++r)
                    for (int j = 0; j < jw; ++j) {
                        size_t o = (size_t)(i0 + r) * n + j0 + j;
                        c[o] = oracle_f32_to_bf16(acc[r * JT + j]);
                        if (out_f32)
                            out_f32[o] = acc[r * JT + j];
                    }
            }
        }
        free(arow);
        free(acc);
    }
    free(bf);
}

/* Checker of the checker: every e4m3 value is an integer multiple of 2^-9, so a product
 * is an integer multiple of 2^-18 and a 128-term block sum fits int64 exactly.  The
 * scales are applied and the blocks summed in fp64. */
void oracle_ref_gemm_f64(const uint8_t *a, const uint8_t *b, const float *as, const float *bs,
                         double *c, int m, int n, int k)
{
    int32_t ilut[256];
    for (int v = 0; v < 256; ++v) {
        float f = oracle_e4m3fn_to_f32((uint8_t)v);
        ilut[v] = isnan(f) ? 0 : (int32_t)lrintf(ldexpf(f, 9));
    }
    int sn = (n + KBLK - 1) / KBLK;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            double result = 0.0;
            for (int t = 0; t < k; t += KBLK) {
                int64_t s = 0;
                for (int ii = 0; ii < KBLK; ++ii)
                    s += (int64_t)ilut[a[(size_t)i + (size_t)(t + ii) * m]] *
                         (int64_t)ilut[b[(size_t)j + (size_t)(t + ii) * n]];
                result += ldexp((double)s, -18) * (double)as[i + (size_t)(t / KBLK) * m] *
                          (double)bs[j / KBLK + (size_t)(t / KBLK) * sn];
            }
            c[(size_t)i * n + j] = result;
        }
}

/* ref_gemm_naive's arithmetic at a list of (row, col) points only: used to spot-check
 * full-size problems without computing all of C on the CPU. */
void oracle_ref_gemm_points(const uint8_t *a, const uint8_t *b, const float *as, const float *bs,
                            const int *rows, const int *cols, int npts, float *out_f32,
                            uint16_t *out_bf16, int m, int n, int k)
{
    float lut[256];
    for (int v = 0; v < 256; ++v)
        lut[v] = oracle_e4m3fn_to_f32((uint8_t)v);
    int sn = (n + KBLK - 1) / KBLK;
#pragma omp parallel for schedule(static)
    for (int p = 0; p < npts; ++p) {
        int i = rows[p], j = cols[p];
        float result = 0.0f;
        for (int t = 0; t < k; t += KBLK) {
            float block_result = 0.0f;
            for (int ii = 0; ii < KBLK; ++ii)
                block_result += lut[a[(size_t)i + (size_t)(t + ii) * m]] *
                                lut[b[(size_t)j + (size_t)(t + ii) * n]];
            float scaled = block_result * as[i + (size_t)(t / KBLK) * m];
            scaled = scaled * bs[j / KBLK + (size_t)(t / KBLK) * sn];
            result += scaled;
        }
        if (out_f32)
            out_f32[p] = result;
        if (out_bf16)
            out_bf16[p] = oracle_f32_to_bf16(result);
    }
}

/* ------------------------------------------------------------------ input producers */

static inline uint64_t splitmix64(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

/* Counter-based N(0,1): element idx of stream `seed`, independent of generation order. */
static inline double normal_at(uint64_t seed, uint64_t idx)
{
    uint64_t h1 = splitmix64(seed * 0xD1342543DE82EF95ull + 2 * idx);
    uint64_t h2 = splitmix64(seed * 0xD1342543DE82EF95ull + 2 * idx + 1);
    double u1 = ((double)(h1 >> 11) + 1.0) * (1.0 / 9007199254740992.0); /* (0,1] */
    double u2 = (double)(h2 >> 11) * (1.0 / 9007199254740992.0);         /* [0,1) */
    return sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
}

/* rows x cols row-major N(0,1) rounded to bf16 (returned widened to fp32).  With
 * outlier_pct > 0 a seeded Bernoulli(outlier_pct/100) mask multiplies entries by
 * outlier_mul before the bf16 rounding. */
void oracle_gen_normal_bf16(float *out, size_t rows, size_t cols, uint64_t seed,
                            double outlier_pct, double outlier_mul)
{
#pragma omp parallel for schedule(static)
    for (long r = 0; r < (long)rows; ++r)
        for (size_t cidx = 0; cidx < cols; ++cidx) {
            uint64_t idx = (uint64_t)r * cols + cidx;
            double v = normal_at(seed, idx);
            if (outlier_pct > 0.0) {
                uint64_t h = splitmix64((seed ^ 0xA5A5A5A5ull) * 0x9E3779B97F4A7C15ull + idx);
                double u = (double)(h >> 11) * (1.0 / 9007199254740992.0);
                if (u < outlier_pct * 0.01)
                    v *= outlier_mul;
            }
            out[idx] = oracle_bf16_to_f32(oracle_f32_to_bf16((float)v));
        }
}

/* The quantisers of quantize.py with FP8 max 448 (torch.float8_e4m3fn).  Per scale group:
 *     amax' = max(amax, 1e-12)
 *     scale = (1 / amax') * 448        two roundings: torch evaluates `finfo.max / tensor`
 *                                      (quantize.py:28,54) as tensor.reciprocal() * finfo.max
 *     q     = fp8_rne(clamp(x * scale, +-448))
 *     stored inverse scale = 1 / scale (quantize.py:39,65: scale.float().reciprocal())
 * bf16_arith = 0: every step in fp32 (what torch does for an fp32 tensor).
 * bf16_arith = 1: what torch does for a bf16 tensor, whose element-wise results are rounded to
 *     bf16 after every operation: 1e-12, the reciprocal, the product with 448 and x * scale are
 *     each rounded to bf16; the stored inverse scale is the fp32 reciprocal of the bf16 scale.
 * Both forms reproduce the reference's own outputs bit for bit
 * (tests/golden/quantize_reference.npz, written by importing quantize.py). */
static inline float q_round(float v, int bf16_arith)
{
    return bf16_arith ? oracle_bf16_to_f32(oracle_f32_to_bf16(v)) : v;
}

static inline float q_scale(float amax, int bf16_arith)
{
    float floor_ = q_round(1e-12f, bf16_arith);
    float r = q_round(1.0f / fmaxf(amax, floor_), bf16_arith);
    return q_round(r * 448.0f, bf16_arith);
}

static inline uint8_t q_code(float x, float scale, int bf16_arith)
{
    float v = q_round(x * scale, bf16_arith);
    v = fminf(fmaxf(v, -448.0f), 448.0f);
    return oracle_f32_to_e4m3fn(v);
}

/* quantize.py:43-67 (to_float8_rowwise_scale): one scale per row and 128-wide K group.
 * x is M x K row-major.  Outputs are written in the kernel's layouts (the transposes the
 * reference leaves to its host code, check.cu:164-167): q at m + k*M, a_scale at m + kb*M. */
void oracle_quantize_a_1x128(const float *x, uint8_t *q, float *a_scale, int m, int k, int bf16_arith)
{
    int nkb = k / KBLK;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < m; ++i)
        for (int kb = 0; kb < nkb; ++kb) {
            const float *g = x + (size_t)i * k + (size_t)kb * KBLK;
            float amax = 0.0f;
            for (int t = 0; t < KBLK; ++t)
                amax = fmaxf(amax, fabsf(g[t]));
            float scale = q_scale(amax, bf16_arith);
            for (int t = 0; t < KBLK; ++t)
                q[(size_t)i + (size_t)(kb * KBLK + t) * m] = q_code(g[t], scale, bf16_arith);
            a_scale[(size_t)i + (size_t)kb * m] = 1.0f / scale;
        }
}

/* quantize.py:16-41 (to_float8_block_scale), same arithmetic per 128 x 128 block.
 * x is N x K row-major.  N need not be a multiple of 128: the last block's amax is taken
 * over the rows that exist (equivalent to zero padding; quantize.py:23-26 drops such rows).
 * Outputs: q at n + k*N, b_scale at nb + kb*ceil(N/128). */
void oracle_quantize_b_128x128(const float *x, uint8_t *q, float *b_scale, int n, int k, int bf16_arith)
{
    int nkb = k / KBLK, sn = (n + KBLK - 1) / KBLK;
#pragma omp parallel for schedule(static) collapse(2)
    for (int nb = 0; nb < sn; ++nb)
        for (int kb = 0; kb < nkb; ++kb) {
            int r1 = (nb + 1) * KBLK < n ? (nb + 1) * KBLK : n;
            float amax = 0.0f;
            for (int r = nb * KBLK; r < r1; ++r)
                for (int t = 0; t < KBLK; ++t)
                    amax = fmaxf(amax, fabsf(x[(size_t)r * k + (size_t)kb * KBLK + t]));
            float scale = q_scale(amax, bf16_arith);
            for (int r = nb * KBLK; r < r1; ++r)
                for (int t = 0; t < KBLK; ++t)
                    q[(size_t)r + (size_t)(kb * KBLK + t) * n] =
                        q_code(x[(size_t)r * k + (size_t)kb * KBLK + t], scale, bf16_arith);
            b_scale[(size_t)nb + (size_t)kb * sn] = 1.0f / scale;
        }
}

/* Whole input set of one benchmark configuration: seeded N(0,1) -> bf16 -> quantise.
 * a: M*K bytes, b: N*K bytes, a_scale: (K/128)*M, b_scale: (K/128)*ceil(N/128). */
void oracle_make_inputs(uint8_t *a, uint8_t *b, float *a_scale, float *b_scale, int m, int n, int k,
                        uint64_t seed, double a_outlier_pct, double a_outlier_mul)
{
    float *xa = (float *)malloc((size_t)m * k * sizeof(float));
    float *xb = (float *)malloc((size_t)n * k * sizeof(float));
    oracle_gen_normal_bf16(xa, (size_t)m, (size_t)k, seed * 2 + 1, a_outlier_pct, a_outlier_mul);
    oracle_gen_normal_bf16(xb, (size_t)n, (size_t)k, seed * 2 + 2, 0.0, 1.0);
    oracle_quantize_a_1x128(xa, a, a_scale, m, k, 0);
    oracle_quantize_b_128x128(xb, b, b_scale, n, k, 0);
    free(xa);
    free(xb);
}

/* max |c - ref| and max |ref| over bf16 arrays; returns the count of positions where
 * exactly one side is NaN or the difference exceeds rtol*max|ref| + atol. */
long oracle_compare_bf16(const uint16_t *c, const uint16_t *ref, size_t count, double rtol,
                         double atol, double *max_err, double *max_ref)
{
    double mr = 0.0, me = 0.0;
    for (size_t i = 0; i < count; ++i) {
        double r = fabs((double)oracle_bf16_to_f32(ref[i]));
        if (r > mr && !isnan(r))
            mr = r;
    }
    double bound = rtol * mr + atol;
    long bad = 0;
    for (size_t i = 0; i < count; ++i) {
        float x = oracle_bf16_to_f32(c[i]), r = oracle_bf16_to_f32(ref[i]);
        if (isnan(x) || isnan(r)) {
            if (isnan(x) != isnan(r))
                ++bad;
            continue;
        }
        double e = fabs((double)x - (double)r);
        if (e > me)
            me = e;
        if (e > bound)
            ++bad;
    }
    if (max_err)
        *max_err = me;
    if (max_ref)
        *max_ref = mr;
    return bad;
}

int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
