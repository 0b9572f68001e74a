// C entry points around the reference's own host helpers, compiled from the header where
// it lies (never copied).  Test infrastructure: used to pin the CPU oracle against
//   genMat            /root/reference/utils.h:25-33  (seed-7 uniform(-5,5) stream)
//   row_to_col_major  /root/reference/utils.h:49-55
//   gemmCPU           /root/reference/utils.h:65-76  (unscaled fp32 i/j/t GEMM)
//   allClose          /root/reference/utils.h:35-47
#include "utils.h"
#include <cstring>

extern "C" {

void ref_genMat(float* out, size_t len)
{
    auto v = genMat(len);
    std::memcpy(out, v.data(), len * sizeof(float));
}

void ref_row_to_col_major(const float* in, float* out, int M, int N)
{
    std::vector<float> src(in, in + (size_t)M * N), dst((size_t)M * N);
    row_to_col_major(src, dst, M, N);
    std::memcpy(out, dst.data(), dst.size() * sizeof(float));
}

// A: M x K row-major, B: K x N row-major, C: M x N row-major (utils.h:65-76)
void ref_gemmCPU(float* C, const float* A, const float* B, size_t M, size_t N, size_t K)
{
    std::vector<float> a(A, A + M * K), b(B, B + K * N), c(M * N);
    gemmCPU(c, a, b, M, N, K);
    std::memcpy(C, c.data(), c.size() * sizeof(float));
}

// bf16 bit patterns in; returns 1 when every |a-b| <= tolerance
int ref_allClose(const unsigned short* a, const unsigned short* b, size_t len, float tolerance)
{
    std::vector<__hip_bfloat16> va(len), vb(len);
    std::memcpy(va.data(), a, len * 2);
    std::memcpy(vb.data(), b, len * 2);
    return allClose(va, vb, tolerance) ? 1 : 0;
}
}
