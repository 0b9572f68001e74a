// Read bandwidth from HBM for the decode kernels' access pattern, without their arithmetic: a matrix of
// `blocks` x 2048 rows of 7168 bytes (more than the caches hold from 40 blocks on) is read in units of
// 2048 rows x P bytes, the way a strip of B is read -- P contiguous bytes of every k-row.  Three questions:
//   strided  how fast the memory system serves pieces of P bytes (plain loads, eight in flight per lane);
//   ring     the same through the kernels' copy structure (loads that write the LDS, a ring of stages, one
//            barrier per stage);
//   +write   what a thin stream of writes among the reads costs (8 KB per unit, 3 % of the bytes: a strip of C).
// Build: make -C fp8-quant-matmul_amd bin/hbm_probe.  Run: bin/hbm_probe [blocks = 64].
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>

#include "device_common.h"

#define CK(x)                                                                      \
    do {                                                                           \
        hipError_t e_ = (x);                                                       \
        if (e_ != hipSuccess) {                                                    \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            return 1;                                                              \
        }                                                                          \
    } while (0)

constexpr int ROW_BYTES = 7168, UNIT_ROWS = 2048, THREADS = 512;

// WR: 0 = reads only; 1 = 8 KB of writes per unit to memory of their own (they reach HBM); 2 = the same 8 KB of
// the workgroup every time (they stay in the caches)
template <int P, int WR>
__global__ void __launch_bounds__(THREADS) strided_kernel(const uint8_t* __restrict__ base, int* out, int strips, int units,
                                                          uint8_t* wbuf)
{
    constexpr int LPR = P / 16;        // lanes per row
    constexpr int RPI = THREADS / LPR;  // rows per instruction of the workgroup
    v4i acc = {0, 0, 0, 0};
    for (int u = blockIdx.x; u < units; u += gridDim.x) {
        const int blk = u / strips, strip = u - blk * strips;
        const uint8_t* p = base + (size_t)blk * UNIT_ROWS * ROW_BYTES + (size_t)strip * P +
                           (threadIdx.x / LPR) * (size_t)ROW_BYTES + (threadIdx.x % LPR) * 16;
        for (int r = 0; r < UNIT_ROWS; r += RPI * 8) {
            v4i v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                v[i] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(p + (size_t)(r + i * RPI) * ROW_BYTES));
#pragma unroll
            for (int i = 0; i < 8; ++i)
                acc ^= v[i];
        }
        if (WR == 1)
            *reinterpret_cast<v4i*>(wbuf + (size_t)u * 8192 + threadIdx.x * 16) = acc;
        if (WR == 2)
            *reinterpret_cast<v4i*>(wbuf + (size_t)blockIdx.x * 8192 + threadIdx.x * 16) = acc;
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678)
        out[0] = 1;
}

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// stages of 128 rows x P bytes through NS slots of the LDS; a workgroup walks its units as one stream of stages
template <int P, int NS>
__global__ void __launch_bounds__(THREADS) ring_kernel(const uint8_t* __restrict__ base, int* out, int strips, int units)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)LDS_PTR(uint8_t, smem);
    constexpr int STAGE = 128 * P;
    constexpr int LPR = P / 16, RPI = 64 / LPR;  // lanes per row, rows per instruction of a wave
    constexpr int Q = 128 / (8 * RPI);          // instructions per wave and stage
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int STAGES_PER_UNIT = UNIT_ROWS / 128;
    const int mine = (units - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    const int total = mine > 0 ? mine * STAGES_PER_UNIT : 0;
    int iu = blockIdx.x, ik = 0, islot = 0, issued = 0;
    auto issue = [&]() {
        if (issued < total) {
            const int blk = iu / strips, strip = iu - blk * strips;
            const uint8_t* p = base + (size_t)blk * UNIT_ROWS * ROW_BYTES + (size_t)ik * 128 * ROW_BYTES + (size_t)strip * P;
            const v4i r = make_rsrc_words(p, (uint32_t)(128 * ROW_BYTES));
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int row = (wave * Q + q) * RPI + lane / LPR;
                lds_dma16(r, (uint32_t)(row * ROW_BYTES + (lane % LPR) * 16), lds_base + islot * STAGE + (wave * Q + q) * 1024);
            }
            if (++ik == STAGES_PER_UNIT) {
                ik = 0;
                iu += gridDim.x;
            }
            islot = islot == NS - 1 ? 0 : islot + 1;
        }
        ++issued;
    };
#pragma unroll
    for (int p = 0; p < NS - 1; ++p)
        issue();
    for (int t = 0; t < total; ++t) {
        const int younger = total - 1 - t < NS - 2 ? total - 1 - t : NS - 2;
        switch (younger) {
        case 0: wait_vmcnt<0>(); break;
        case 1: wait_vmcnt<Q>(); break;
        case 2: wait_vmcnt<2 * Q>(); break;
        case 3: wait_vmcnt<3 * Q>(); break;
        default: wait_vmcnt<4 * Q>(); break;
        }
        __syncthreads();
        issue();
    }
    if (smem[threadIdx.x] == 0x77 && strips == 12345)
        out[0] = 1;
}

int main(int argc, char** argv)
{
    const int blocks = argc > 1 ? atoi(argv[1]) : 64;
    if (blocks < 1 || blocks > 256) {
        printf("blocks: 1 ... 256\n");
        return 1;
    }
    const size_t bytes = (size_t)blocks * UNIT_ROWS * ROW_BYTES;
    uint8_t *d, *wbuf;
    int* out;
    CK(hipMalloc(&d, bytes));
    CK(hipMalloc(&out, 4));
    CK(hipMalloc(&wbuf, (size_t)blocks * (ROW_BYTES / 128) * 8192));
    CK(hipMemset(d, 1, bytes));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const int grid = 256, reps = 10;
    printf("%zu MB, %d workgroups of %d threads\n", bytes >> 20, grid, THREADS);
    auto timed = [&](auto launch, const char* name, int P) -> int {
        for (int i = 0; i < 3; ++i)
            launch();
        CK(hipEventRecord(e0, 0));
        for (int i = 0; i < reps; ++i)
            launch();
        CK(hipEventRecord(e1, 0));
        CK(hipEventSynchronize(e1));
        CK(hipGetLastError());
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        printf("%-34s P = %4d: %6.1f us per pass, %5.0f GB/s read\n", name, P, ms * 1e3 / reps, bytes / (ms * 1e-3 / reps) * 1e-9);
        fflush(stdout);
        return 0;
    };
#define STRIDED(P, WR, name)                                                                                          \
    if (timed([&] { hipLaunchKernelGGL((strided_kernel<P, WR>), dim3(grid), dim3(THREADS), 0, 0, d, out, ROW_BYTES / P, \
                                       (ROW_BYTES / P) * blocks, wbuf); }, name, P))                                  \
        return 1;
#define RING(P, NS, name)                                                                                             \
    CK(hipFuncSetAttribute(reinterpret_cast<const void*>(ring_kernel<P, NS>), hipFuncAttributeMaxDynamicSharedMemorySize, \
                           NS * 128 * P));                                                                            \
    if (timed([&] { hipLaunchKernelGGL((ring_kernel<P, NS>), dim3(grid), dim3(THREADS), NS * 128 * P, 0, d, out,      \
                                       ROW_BYTES / P, (ROW_BYTES / P) * blocks); }, name, P))                         \
        return 1;
    STRIDED(128, 0, "strided")
    STRIDED(256, 0, "strided")
    STRIDED(512, 0, "strided")
    STRIDED(1024, 0, "strided")
    RING(128, 6, "ring, 6 stages")
    RING(128, 8, "ring, 8 stages")
    RING(256, 4, "ring, 4 stages")
    RING(256, 3, "ring, 3 stages")
    STRIDED(128, 1, "strided + 3 % writes to HBM")
    STRIDED(128, 2, "strided + 3 % writes, cached")
    return 0;
}
