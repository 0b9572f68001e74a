// Calibration kernel for the HBM traffic counters: copies a buffer of known size so that
// FETCH_SIZE / WRITE_SIZE readings of the GEMM kernels can be scaled by what the same
// counters report for a known number of bytes.  Usage: calib_copy [MiB] [repeats]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

__global__ void __launch_bounds__(256) calib_copy_kernel(const uint4* __restrict__ src,
                                                         uint4* __restrict__ dst, size_t n16)
{
    size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
        dst[i] = src[i];
}

int main(int argc, char** argv)
{
    size_t mib = argc > 1 ? std::strtoul(argv[1], nullptr, 10) : 1024;
    int reps = argc > 2 ? std::atoi(argv[2]) : 3;
    size_t bytes = mib << 20;
    void *src, *dst;
    if (hipMalloc(&src, bytes) != hipSuccess || hipMalloc(&dst, bytes) != hipSuccess)
        return 2;
    if (hipMemset(src, 1, bytes) != hipSuccess)
        return 2;
    for (int i = 0; i < reps; ++i)
        hipLaunchKernelGGL(calib_copy_kernel, dim3(256 * 8), dim3(256), 0, nullptr,
                           static_cast<const uint4*>(src), static_cast<uint4*>(dst), bytes / 16);
    if (hipDeviceSynchronize() != hipSuccess)
        return 2;
    std::printf("copied %zu bytes (read) + %zu bytes (written) per launch, %d launches\n", bytes, bytes, reps);
    return 0;
}
