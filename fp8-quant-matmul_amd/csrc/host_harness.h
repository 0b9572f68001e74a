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
