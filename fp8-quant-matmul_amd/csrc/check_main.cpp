// Correctness driver: the procedure of /root/reference/check.cu:132-184.  Seed-7
// uniform(-5,5) values for a, b and both scale arrays, a and a_scale transposed to column
// major, the scalar definition kernel as reference (option 2) against the dispatched kernel
// (option 0), absolute tolerance 100.  Shape from the command line (default 128 128 256).
// Unlike the reference it exits non-zero on a mismatch.
#include "host_harness.h"

#include <cstdlib>

int main(int argc, char** argv)
{
    using namespace harness;
    size_t M = argc > 1 ? std::strtoul(argv[1], nullptr, 10) : 128;
    size_t N = argc > 2 ? std::strtoul(argv[2], nullptr, 10) : 128;
    size_t K = argc > 3 ? std::strtoul(argv[3], nullptr, 10) : 256;
    float tolerance = argc > 4 ? std::strtof(argv[4], nullptr) : 100.f;

    const auto matA = genMat(M * K);
    const auto matB = genMat(K * N);
    const auto matAs = genMat(M * K / 128);
    const auto matBs = genMat((K / 128) * ((N + 127) / 128));
    std::vector<float> matA_col(M * K), matAs_col(M * K / 128);
    row_to_col_major(matA, matA_col, (int)M, (int)K);
    row_to_col_major(matAs, matAs_col, (int)M, (int)(K / 128));

    std::vector<bf16_bits> c_ref(M * N), c_my(M * N);
    if (gemmGPU(c_ref, matA_col, matB, matAs_col, matBs, M, N, K, 2) != 0)
        return 2;
    if (gemmGPU(c_my, matA_col, matB, matAs_col, matBs, M, N, K, 0) != 0)
        return 2;
    std::printf("kernel: %s\n", fp8_block_gemm_last_kernel());
    if (allClose(c_ref, c_my, tolerance)) {
        std::printf("2 matrices are equal\n");
        return 0;
    }
    return 1;
}
