/*
 * Inner 128-term block dot product of the CPU oracle (test infrastructure, see
 * fp8gemm_oracle.c).  Restates the ii loop of /root/reference/check.cu:39-44 for up to 64
 * adjacent output columns at once.
 *
 * This file alone is compiled with floating-point contraction allowed and with AVX2/AVX-512
 * clones: the product of two e4m3 values has at most 8 significant bits, so it is exact in
 * fp32 and a fused multiply-add rounds exactly like the separate multiply and add of the
 * reference.  Each column's additions stay in ascending ii order, so the result is
 * bit-identical to the scalar loop (pinned by tests/test_oracle_gemm.py).
 */
#include <stddef.h>

#define KBLK 128
#define JT 64

__attribute__((target_clones("arch=skylake-avx512", "arch=haswell", "default")))
void oracle_block_dot(const float *ar, const float *bp, size_t ldb, float *blk, int jw)
{
    if (jw == JT) {
        float acc[JT];
        for (int j = 0; j < JT; ++j)
            acc[j] = 0.0f;
        for (int ii = 0; ii < KBLK; ++ii) {
            float av = ar[ii];
            const float *br = bp + (size_t)ii * ldb;
#pragma omp simd
            for (int j = 0; j < JT; ++j)
                acc[j] += av * br[j];
        }
        for (int j = 0; j < JT; ++j)
            blk[j] = acc[j];
    } else {
        for (int j = 0; j < jw; ++j)
            blk[j] = 0.0f;
        for (int ii = 0; ii < KBLK; ++ii) {
            float av = ar[ii];
            const float *br = bp + (size_t)ii * ldb;
            for (int j = 0; j < jw; ++j)
                blk[j] += av * br[j];
        }
    }
}
