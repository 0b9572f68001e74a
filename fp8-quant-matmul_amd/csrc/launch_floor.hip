// Launch floor of the device: time per launch of kernels that do nothing, issued back to back
// into one stream (the way bench.py times the GEMM).  The figure bounds every latency-type
// number from below: the decode shape's HBM floor is 1.9 us of data movement plus this.
// Usage: launch_floor [launches]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

__global__ void empty_kernel(int* p)
{
    if (p && threadIdx.x == 0xFFFF)
        *p = 1;
}

__global__ void __launch_bounds__(512) lds_kernel(int* p)
{
    extern __shared__ int sm[];
    sm[threadIdx.x] = (int)threadIdx.x;
    __syncthreads();
    if (p && sm[(threadIdx.x + 1) & 511] == 0xFFFF)
        *p = 1;
}

int main(int argc, char** argv)
{
    const int launches = argc > 1 ? std::atoi(argv[1]) : 200;
    hipStream_t s;
    hipEvent_t e0, e1;
    if (hipStreamCreate(&s) != hipSuccess || hipEventCreate(&e0) != hipSuccess ||
        hipEventCreate(&e1) != hipSuccess)
        return 2;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(lds_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024) != hipSuccess)
        return 2;
    struct Case { const char* name; int grid, block, lds; };
    const Case cases[] = {{"empty, 1 x 64 threads", 1, 64, 0},
                          {"empty, 256 x 512 threads", 256, 512, 0},
                          {"140 KiB LDS, 256 x 512 threads", 256, 512, 140 * 1024},
                          {"140 KiB LDS, 32 x 512 threads", 32, 512, 140 * 1024}};
    for (const Case& c : cases) {
        for (int pass = 0; pass < 2; ++pass) {  // pass 0 warms up
            (void)hipEventRecord(e0, s);
            for (int i = 0; i < launches; ++i) {
                if (c.lds)
                    hipLaunchKernelGGL(lds_kernel, dim3(c.grid), dim3(c.block), c.lds, s, nullptr);
                else
                    hipLaunchKernelGGL(empty_kernel, dim3(c.grid), dim3(c.block), 0, s, nullptr);
            }
            (void)hipEventRecord(e1, s);
            if (hipEventSynchronize(e1) != hipSuccess)
                return 2;
            float ms = 0.f;
            (void)hipEventElapsedTime(&ms, e0, e1);
            if (pass == 1)
                std::printf("%-34s %.2f us per launch\n", c.name, ms * 1e3 / launches);
        }
    }
    return 0;
}
