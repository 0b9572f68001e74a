// Host-side helpers of the C++ drivers: the counterparts of /root/reference/utils.h
// (genMat :25-33, allClose :35-47, row_to_col_major :49-55) and of the vector-based
// gemmGPU signature (/root/reference/check.cu:51-52), written against the C ABI.
#pragma once
#include "../../include/fp8_block_gemm.h"

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

namespace harness {

using bf16_bits = unsigned short;

inline float bf16_to_float(bf16_bits h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// Seeded uniform(-5, 5) values; every call restarts the same stream (utils.h:26-27).
inline std::vector<float> genMat(size_t len)
{
    std::default_random_engine engine(7);
    std::uniform_real_distribution<float> dist(-5.f, 5.f);
    std::vector<float> v(len);
    for (auto& x : v)
        x = dist(engine);
    return v;
}

// First offending index is reported, like utils.h:40-44.
inline bool allClose(const std::vector<bf16_bits>& x, const std::vector<bf16_bits>& y, float tol)
{
    if (x.size() != y.size())
        return false;
    for (size_t i = 0; i < x.size(); ++i) {
        float d = std::fabs(bf16_to_float(x[i]) - bf16_to_float(y[i]));
        if (!(d <= tol)) {
            std::printf("%zu---%g---%g\n", i, bf16_to_float(x[i]), bf16_to_float(y[i]));
            return false;
        }
    }
    return true;
}

inline void row_to_col_major(const std::vector<float>& in, std::vector<float>& out, int rows, int cols)
{
    for (int i = 0; i < rows; ++i)
        for (int j = 0; j < cols; ++j)
            out[(size_t)j * rows + i] = in[(size_t)i * cols + j];
}

// fp32 -> e4m3fn code, round to nearest even, saturating at 448 (host side, for synthetic operands)
inline uint8_t e4m3fn_from_float(float x)
{
    const uint8_t sign = std::signbit(x) ? 0x80 : 0;
    float ax = std::fabs(x);
    if (!(ax < 448.f))
        return sign | 0x7E;
    if (ax < 0.0009765625f)  // below half the smallest subnormal (2^-10): zero
        return sign;
    int e;
    (void)std::frexp(ax, &e);            // ax = f * 2^e, f in [0.5, 1)
    int exp = e - 1 < -6 ? -6 : e - 1;   // exponent of the code's binade (subnormals share -6)
    const float step = std::ldexp(1.f, exp - 3);
    const float q = std::nearbyint(ax / step);  // default rounding mode: ties to even
    const float v = q * step;
    (void)std::frexp(v, &e);
    exp = e - 1 < -6 ? -6 : e - 1;
    const int mant = (int)(v / std::ldexp(1.f, exp - 3)) - (v >= 0.015625f ? 8 : 0);
    const int biased = v >= 0.015625f ? exp + 7 : 0;
    return sign | (uint8_t)((biased << 3) | mant);
}

// Operands with the statistics of the benchmark's: standard normal values, A quantised per row and
// 128-wide K group (scale = amax / 448, /root/reference/quantize.py:43-67), B per 128 x 128 block
// (quantize.py:16-41), written in the GEMM's layouts (a: m + k*M, b: n + k*N, scales [K/128][.]).
inline void quantised_normal_operands(std::vector<uint8_t>& a, std::vector<float>& as, std::vector<uint8_t>& b,
                                      std::vector<float>& bs, size_t M, size_t N, size_t K)
{
    std::mt19937 engine(7);
    std::normal_distribution<float> dist(0.f, 1.f);
    const size_t nkb = K / 128, sn = (N + 127) / 128;
    std::vector<float> grp(128 * 128);
    for (size_t kb = 0; kb < nkb; ++kb)
        for (size_t m = 0; m < M; ++m) {
            float amax = 1e-12f;
            for (int i = 0; i < 128; ++i) {
                grp[i] = dist(engine);
                amax = std::fmax(amax, std::fabs(grp[i]));
            }
            as[kb * M + m] = amax / 448.f;
            for (int i = 0; i < 128; ++i)
                a[m + (kb * 128 + i) * M] = e4m3fn_from_float(grp[i] * (448.f / amax));
        }
    for (size_t kb = 0; kb < nkb; ++kb)
        for (size_t nb = 0; nb < sn; ++nb) {
            const size_t cols = N - nb * 128 < 128 ? N - nb * 128 : 128;
            float amax = 1e-12f;
            for (size_t i = 0; i < 128 * cols; ++i) {
                grp[i] = dist(engine);
                amax = std::fmax(amax, std::fabs(grp[i]));
            }
            bs[kb * sn + nb] = amax / 448.f;
            for (size_t kk = 0; kk < 128; ++kk)
                for (size_t c = 0; c < cols; ++c)
                    b[nb * 128 + c + (kb * 128 + kk) * N] = e4m3fn_from_float(grp[kk * cols + c] * (448.f / amax));
        }
}

// gemmGPU(C, A, B, As, Bs, M, N, K, option) with the reference's argument meaning.
inline int gemmGPU(std::vector<bf16_bits>& C, const std::vector<float>& A, const std::vector<float>& B,
                   const std::vector<float>& As, const std::vector<float>& Bs, size_t M, size_t N,
                   size_t K, int option)
{
    int rc = fp8_gemm_host(C.data(), A.data(), B.data(), As.data(), Bs.data(), M, N, K, option);
    if (rc != 0)
        std::fprintf(stderr, "gemmGPU failed: %s (%d)\n", fp8_block_gemm_error_string(rc), rc);
    return rc;
}

}  // namespace harness
