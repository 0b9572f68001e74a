// The definition kernel: one thread per C element, sequential fp32 sum over each 128-wide
// K block, scales applied per block, bf16 store.  Counterpart of ref_kernel
// (/root/reference/check.cu:30-49); threads are mapped with n fastest so that the b reads
// and the c stores of a wavefront are contiguous (the reference maps m fastest).
#include "device_common.h"
#include "launchers.h"

namespace fp8gemm {

__global__ void __launch_bounds__(256) scalar_gemm_kernel(const uint8_t* __restrict__ a,
                                                          const uint8_t* __restrict__ b,
                                                          const float* __restrict__ as,
                                                          const float* __restrict__ bs,
                                                          uint16_t* __restrict__ c, int m, int n, int k)
{
    // no fused multiply-add anywhere but the explicit fmaf below: "result += block * as * bs"
    // keeps its three separately rounded operations, as in a CPU build of the same line
#pragma clang fp contract(off)
    // rows ride on grid.x, whose limit (2^31 - 1 blocks) no accepted m reaches; grid.y carries the
    // 64-column strips, of which the validation's 2^31 - 1 element bound on m*n leaves few when m is large
    int col = blockIdx.y * 64 + (threadIdx.x & 63);
    int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= m || col >= n)
        return;
    int sn = (n + KBLOCK - 1) / KBLOCK;
    float result = 0.0f;
    for (int k0 = 0; k0 < k; k0 += KBLOCK) {
        float block = 0.0f;
        for (int ii = 0; ii < KBLOCK; ++ii) {
            float av = e4m3fn_to_f32(a[(size_t)row + (size_t)(k0 + ii) * m]);
            float bv = e4m3fn_to_f32(b[(size_t)col + (size_t)(k0 + ii) * n]);
            block = fmaf(av, bv, block);  // the product is exact in fp32, so fma == mul + add
        }
        float scaled = block * as[row + (size_t)(k0 / KBLOCK) * m];
        scaled = scaled * bs[col / KBLOCK + (size_t)(k0 / KBLOCK) * sn];
        result = result + scaled;
    }
    c[(size_t)row * n + col] = f32_to_bf16_bits(result);
}

hipError_t launch_scalar(const GemmArgs& g, hipStream_t s)
{
    const unsigned strips = (unsigned)((g.n + 63) / 64);
    if (strips > 65535u)  // n beyond 4 M columns: not a shape this kernel is for
        return hipErrorInvalidConfiguration;
    dim3 grid((unsigned)((g.m + 3) / 4), strips);
    hipLaunchKernelGGL(scalar_gemm_kernel, grid, dim3(256), 0, s, g.a, g.b, g.a_scale, g.b_scale,
                       g.c, g.m, g.n, g.k);
    return hipGetLastError();
}

}  // namespace fp8gemm
