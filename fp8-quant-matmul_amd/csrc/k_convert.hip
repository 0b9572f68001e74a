// fp32 -> fp8 e4m3fn (OCP), round to nearest even, saturating at +-448, NaN kept.
// Counterpart of convert_float_to_fp8 (/root/reference/check.cu:17-22); grid-stride so
// that any element count is converted (the reference launch drops a tail, check.cu:83).
#include "device_common.h"
#include "launchers.h"

namespace fp8gemm {

__device__ __forceinline__ float clamp448(float x)
{
    // NaN passes through; +-inf and everything beyond the largest finite code saturate
    return (x != x) ? x : __builtin_amdgcn_fmed3f(x, 448.0f, -448.0f);
}

__global__ void __launch_bounds__(256) convert_kernel(const float* __restrict__ in,
                                                      uint8_t* __restrict__ out, size_t count)
{
    size_t quads = count / 4;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += stride) {
        float4 v = reinterpret_cast<const float4*>(in)[q];
        int w = 0;
        w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(v.x), clamp448(v.y), w, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(v.z), clamp448(v.w), w, true);
        reinterpret_cast<int*>(out)[q] = w;
    }
    size_t tail = quads * 4 + (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tail < count) {
        int w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp448(in[tail]), 0.0f, 0, false);
        out[tail] = (uint8_t)(w & 0xFF);
    }
}

hipError_t launch_convert(const float* in, uint8_t* out, size_t count, hipStream_t s)
{
    if (count == 0)
        return hipSuccess;
    size_t quads = count / 4;
    size_t blocks = (quads + 255) / 256;
    if (blocks < 1)
        blocks = 1;
    if (blocks > 256 * 16)
        blocks = 256 * 16;
    hipLaunchKernelGGL(convert_kernel, dim3((unsigned)blocks), dim3(256), 0, s, in, out, count);
    return hipGetLastError();
}

}  // namespace fp8gemm
