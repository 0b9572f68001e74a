// What does the MI355X sustain for the instruction mix of the block-scaled GEMM, with no
// memory stalls at all?  Every wave loops over register-resident random fp8 operands and
// issues, per v_mfma_f32_32x32x64_f8f6f4: NF v_fmac_f32 on the result of an earlier MFMA (the
// scale fold needs 8) and NR ds_read_b64_tr_b8 (the 64x96 wave tile needs 3.3).  Two waves per
// SIMD, 256 workgroups, nothing else in the loop: no barrier, no wait on memory, no copy.  The
// figures bound what any schedule of that mix can reach on this part.
// Usage: mfma_mix_bench [iterations [constant]]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
#define LDS_ADDR(p) ((unsigned)(size_t)((__attribute__((address_space(3))) unsigned char*)(p)))
#define CHECK(x)                                                                   \
    do {                                                                           \
        hipError_t e_ = (x);                                                       \
        if (e_ != hipSuccess) {                                                    \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));          \
            std::exit(2);                                                          \
        }                                                                          \
    } while (0)

template <int NF, int NR>
__global__ void __launch_bounds__(512) mix_kernel(const v8i* data, float* out, int iters)
{
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    const int gid = blockIdx.x * blockDim.x + threadIdx.x, tid = threadIdx.x, lane = tid & 63;
    for (int i = tid; i < 65536 / 32; i += blockDim.x)
        reinterpret_cast<v8i*>(smem)[i] = data[(gid + i * 7) % 65536];
    __syncthreads();
    v8i x[4], y[4];
    for (int i = 0; i < 4; ++i) {
        x[i] = data[(gid * 8 + i) % 65536];
        y[i] = data[(gid * 8 + 4 + i) % 65536];
    }
    v16f acc[4], folded[4];
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 16; ++j) {
            acc[i][j] = 0.f;
            folded[i][j] = 0.f;
        }
    // conflict-free transposing-read addresses (the GEMM's 256-byte-row swizzle)
    const int g = lane >> 4, i16 = lane & 15;
    const unsigned addr = LDS_ADDR(smem) + ((8 * g + (i16 >> 1)) * 256 +
                                            ((((tid >> 6) * 2) ^ (2 * (i16 >> 1))) * 16) + (i16 & 1) * 8);
    float scale = 1.0001f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0"
                         : "+v"(acc[u])
                         : "v"(x[u]), "v"(y[u]));  // fixed registers: a run-time index would cost moves
#pragma unroll
            for (int j = 0; j < NF; ++j)
                asm volatile("v_fmac_f32 %0, %1, %2"
                             : "+v"(folded[u][j % 16])
                             : "v"(scale), "v"(acc[(u + 2) & 3][j % 16]));
            v2i r;
            if (NR >= 1) asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"((u * 8192) % 65536));
            if (NR >= 2) asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"((u * 8192 + 2048) % 65536));
            if (NR >= 3) asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"((u * 8192 + 4096) % 65536));
            if (NR >= 4) asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"((u * 8192 + 6144) % 65536));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    float s = 0.f;
    for (int i = 0; i < 4; ++i)
        for (int j = 0; j < 16; ++j)
            s += acc[i][j] + folded[i][j];
    out[gid] = s;
}

template <int NF, int NR>
void run(const v8i* data, float* out, int iters)
{
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    auto kern = mix_kernel<NF, NR>;
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    float ms = 0.f;
    // the last of five launches counts: the part needs ~30 ms of continuous load after an idle
    // gap to reach its steady clock
    for (int rep = 0; rep < 5; ++rep) {
        CHECK(hipEventRecord(e0));
        hipLaunchKernelGGL(kern, dim3(256), dim3(512), 65536, nullptr, data, out, iters);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        CHECK(hipEventElapsedTime(&ms, e0, e1));
    }
    const double flops = 256.0 * 8 * iters * 4 * 131072.0;
    std::printf("per MFMA: %2d v_fmac, %d ds_read_b64_tr_b8 : %8.2f ms  %6.0f TFLOP/s  %5.1f %% of 5033\n", NF, NR,
                ms, flops / ms * 1e-9, flops / ms * 1e-9 / 50.33);
}

int main(int argc, char** argv)
{
    const int iters = argc > 1 ? std::atoi(argv[1]) : 50000;
    std::vector<unsigned char> h(65536 * 32);
    std::srand(3);
    const bool constant = argc > 2 && std::atoi(argv[2]) != 0;  // operands that do not toggle
    for (auto& v : h) {
        v = std::rand() & 0xFF;
        if ((v & 0x78) == 0x78)
            v &= 0x3F;  // keep magnitudes moderate, no NaN codes
        if (constant)
            v = 0x38;
    }
    std::printf("operands: %s\n", constant ? "constant code 0x38" : "pseudo-random codes");
    void* data;
    float* out;
    CHECK(hipMalloc(&data, h.size()));
    CHECK(hipMemcpy(data, h.data(), h.size(), hipMemcpyHostToDevice));
    CHECK(hipMalloc(reinterpret_cast<void**>(&out), 256 * 512 * sizeof(float)));
    const v8i* d = static_cast<const v8i*>(data);
    run<0, 0>(d, out, iters);
    run<8, 0>(d, out, iters);
    run<0, 3>(d, out, iters);
    run<8, 2>(d, out, iters);
    run<8, 3>(d, out, iters);
    run<9, 2>(d, out, iters);
    run<9, 3>(d, out, iters);
    run<10, 3>(d, out, iters);
    run<10, 4>(d, out, iters);
    run<12, 4>(d, out, iters);
    return 0;
}
