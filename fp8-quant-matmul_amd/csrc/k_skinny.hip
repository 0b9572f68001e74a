// Streaming kernel for tiny M (decode shapes, M <= 32): HBM-bound, B is read exactly once.
// The reference has no kernel for this regime (its smallest tile needs M >= 64,
// /root/reference/mn_small.hip:16,121-125); the math is the same block-scaled product
// (/root/reference/check.cu:36-48).
//
// One workgroup owns 32 columns of C and a range of K blocks; its 8 waves split that K range,
// so a workgroup streams a [K_range x 32 B] strip of B and the matching strip of A.  Each wave
// copies only the rows it will multiply itself (global -> LDS, 16 bytes per lane, written to LDS
// by the load itself), waits for its own copies and goes on without any workgroup barrier.
// Operands come out of LDS through ds_read_b64_tr_b8 and feed v_mfma_f32_16x16x128_f8f6f4 with
// rows = n, columns = m, exactly as in the tile kernel.  The eight partial results are summed
// through LDS in wave order (deterministic), then stored as bf16, or as fp32 partials when
// the K range is also split across workgroups (grid.y > 1).
//
// LDS per wave: 2 K blocks x 128 rows x 32 B for B, the same for A = 16 KiB; rows are 32 bytes
// (two 16-byte chunks); chunk c of row r sits at position c ^ ((r >> 3) & 1) so that the two
// 16-lane groups served together by a transposing read hit different banks.
#include "device_common.h"
#include "launchers.h"

namespace fp8gemm {

namespace {

constexpr int SK_BN = 32;
constexpr int SK_THREADS = 512;
constexpr int SK_WAVE_LDS = 16384;
constexpr int SK_LDS = 8 * SK_WAVE_LDS;  // 128 KiB, reused for the final reduction
constexpr int SK_CHUNK_KB = 2;           // K blocks per wave per pass

template <bool SPLIT>
__global__ void __launch_bounds__(SK_THREADS)
skinny_gemm_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                   const float* __restrict__ a_scale, const float* __restrict__ b_scale,
                   uint16_t* __restrict__ c, float* __restrict__ partial, int M, int N, int K,
                   int tiles_n, int kb_per_split)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    auto lds = LDS_PTR(uint8_t, smem);
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // neighbouring column strips share 128-byte lines of B: keep them on one XCD (id % 8)
    const int pid = blockIdx.x;
    const int xcd = pid & 7, q8 = tiles_n >> 3, r8 = tiles_n & 7;
    const int tile = xcd * q8 + (xcd < r8 ? xcd : r8) + (pid >> 3);
    const int n0 = tile * SK_BN;

    const int nkb = K / KBLOCK;
    const int wg_kb0 = blockIdx.y * kb_per_split;
    const int wg_kb1 = (wg_kb0 + kb_per_split < nkb) ? (wg_kb0 + kb_per_split) : nkb;
    const int cnt = wg_kb1 - wg_kb0;
    const int per_wave = (cnt + 7) / 8;
    const int wk0 = wg_kb0 + wave * per_wave;
    const int wk1 = (wk0 + per_wave < wg_kb1) ? (wk0 + per_wave) : wg_kb1;

    const uint32_t a_bytes = (uint32_t)M * (uint32_t)K, b_bytes = (uint32_t)N * (uint32_t)K;
    const int sn = (N + KBLOCK - 1) / KBLOCK;
    const int nb = n0 >> 7;
    const uint32_t region = (uint32_t)(wave * SK_WAVE_LDS);  // B strip, then A strip at +8192

    // copy plan: one instruction moves 32 rows x 32 B; lane l -> row l/2, chunk position l&1
    const int crow = lane >> 1;
    const int cchunk = (lane & 1) ^ ((crow >> 3) & 1);
    const bool vb = n0 + 16 * cchunk < N;
    const bool va = 16 * cchunk < M;
    const uint32_t voff_b0 = vb ? (uint32_t)(crow * N + n0 + 16 * cchunk) : 0x80000000u;
    const uint32_t voff_a0 = va ? (uint32_t)(crow * M + 16 * cchunk) : 0x80000000u;

    // transposing reads: lane = 16*g + i; read t covers rows 32*t + 8*g + (i>>1)
    const int g4 = lane >> 4, i16 = lane & 15;
    const uint32_t row_off = (uint32_t)((8 * g4 + (i16 >> 1)) * 32 + (i16 & 1) * 8);
    uint32_t addr_p[2];  // patch 0 / 1 of a 32-wide strip
    addr_p[0] = region + row_off + (uint32_t)(((0 ^ (g4 & 1))) * 16);
    addr_p[1] = region + row_off + (uint32_t)(((1 ^ (g4 & 1))) * 16);

    auto read_frag = [&](uint32_t addr) -> v8i {
        v2i r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr));
        v2i r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 1024));
        v2i r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 2048));
        v2i r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 3072));
        return (v8i){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    };

    const __amdgpu_buffer_rsrc_t ras = make_rsrc(a_scale, (uint32_t)nkb * (uint32_t)M * 4u);
    const int m_lane = lane & 15;

    v4f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
            acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};

    for (int kc = wk0; kc < wk1; kc += SK_CHUNK_KB) {
        const int nk = (wk1 - kc < SK_CHUNK_KB) ? (wk1 - kc) : SK_CHUNK_KB;
        const uint32_t skip_a = (uint32_t)kc * KBLOCK * (uint32_t)M;
        const uint32_t skip_b = (uint32_t)kc * KBLOCK * (uint32_t)N;
        const v4i ra = make_rsrc_words(a + skip_a, a_bytes - skip_a);
        const v4i rb = make_rsrc_words(b + skip_b, b_bytes - skip_b);
        // the previous pass's LDS reads have been consumed by its MFMAs before we get here
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        for (int q = 0; q < nk * 4; ++q) {
            lds_dma16(rb, vb ? voff_b0 + (uint32_t)(q * 32 * N) : 0x80000000u,
                      lds_base + region + (uint32_t)(q * 1024));
            lds_dma16(ra, va ? voff_a0 + (uint32_t)(q * 32 * M) : 0x80000000u,
                      lds_base + region + 8192u + (uint32_t)(q * 1024));
        }
        float s[SK_CHUNK_KB][2];
#pragma unroll
        for (int kk = 0; kk < SK_CHUNK_KB; ++kk) {
            const int kb = (kc + kk < nkb) ? (kc + kk) : (nkb - 1);
            const float bsv = b_scale[(size_t)kb * sn + nb];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                float av = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               ras, (uint32_t)((kb * M + m_lane + 16 * i) * 4), 0, 0));
                s[kk][i] = av * bsv;
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's own copies have landed
#pragma unroll
        for (int kk = 0; kk < SK_CHUNK_KB; ++kk) {
            if (kk < nk) {
                const uint32_t ko = (uint32_t)(kk * 4096);
                v8i fb[2], fa[2];
                fb[0] = read_frag(addr_p[0] + ko);
                fb[1] = read_frag(addr_p[1] + ko);
                fa[0] = read_frag(addr_p[0] + 8192u + ko);
                fa[1] = read_frag(addr_p[1] + 8192u + ko);
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        v4f blk = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            fb[j], fa[i], (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                        acc[i][j] = (v4f){fmaf(s[kk][i], blk[0], acc[i][j][0]),
                                          fmaf(s[kk][i], blk[1], acc[i][j][1]),
                                          fmaf(s[kk][i], blk[2], acc[i][j][2]),
                                          fmaf(s[kk][i], blk[3], acc[i][j][3])};
                    }
            }
        }
    }

    // ---- sum the eight waves' partial results through LDS, in wave order
    __syncthreads();
    auto red = LDS_PTR(v4f, smem);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
            red[(wave * 4 + i * 2 + j) * 64 + lane] = acc[i][j];
    __syncthreads();
    if (threadIdx.x < 256) {
        const int e = threadIdx.x >> 6;  // i*2 + j
        v4f sum = red[e * 64 + lane];
#pragma unroll
        for (int w = 1; w < 8; ++w)
            sum += red[(w * 4 + e) * 64 + lane];
        const int mrow = 16 * (e >> 1) + (lane & 15);
        const int ncol = n0 + 16 * (e & 1) + 4 * (lane >> 4);
        if (mrow < M && ncol < N) {
            const size_t o = (size_t)mrow * N + ncol;
            if (SPLIT) {
                *reinterpret_cast<v4f*>(partial + (size_t)blockIdx.y * M * N + o) = sum;
            } else {
                uint2 pk;
                pk.x = pack_bf16x2(sum[0], sum[1]);
                pk.y = pack_bf16x2(sum[2], sum[3]);
                *reinterpret_cast<uint2*>(c + o) = pk;
            }
        }
    }
}

}  // namespace

bool skinny_supports(const GemmArgs& g)
{
    return g.m <= 32 && g.m % 16 == 0 && g.n % 16 == 0 &&
           (reinterpret_cast<uintptr_t>(g.a) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.b) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.c) % 8 == 0);
}

// Microseconds, fitted to measurements with M = 16 and 32, N = 1536 ... 7168, K = 1536 ... 7168 (operands in
// the caches).  A wave copies and multiplies two K blocks per pass, eight waves per workgroup: up to 16
// K blocks of a workgroup's range go in one pass, which the 4.4 us cover (launch, one pass, the LDS
// reduction, the store); every further pass, or further round of 256 workgroups, waits for its copies again
// and costs in proportion to the workgroups that pull on the memory system together; a K split over
// workgroups adds the reduction launch and the partial sums.
double skinny_cost(const GemmArgs& g, int ksplit)
{
    if (ksplit <= 0)  // the floor: one pass of one round, no K split
        return 4.4;
    const int strips = (g.n + SK_BN - 1) / SK_BN;
    const int nkb = g.k / KBLOCK;
    const int kbs = (nkb + ksplit - 1) / ksplit;
    const int passes = ((kbs + 7) / 8 + SK_CHUNK_KB - 1) / SK_CHUNK_KB;
    const long wgs = (long)strips * ksplit;
    const long rounds = (wgs + 255) / 256;
    const double together = wgs < 256 ? (double)wgs : 256.0;
    return 4.4 + (ksplit > 1 ? 2.7 : 0.0) + (double)(passes * rounds - 1) * 0.028 * together;
}

// the K split (over workgroups) with the lowest cost; every split owns at least one K block
int skinny_ksplit(const GemmArgs& g)
{
    const int nkb = g.k / KBLOCK;
    int best = 1;
    double best_cost = skinny_cost(g, 1);
    for (int ks = 2; ks <= 8 && ks <= nkb; ++ks) {
        if ((ks - 1) * ((nkb + ks - 1) / ks) >= nkb)
            continue;
        const double c = skinny_cost(g, ks);
        if (c < best_cost) {
            best_cost = c;
            best = ks;
        }
    }
    return best;
}

hipError_t launch_skinny(const GemmArgs& g, int ksplit, float* partial, hipStream_t s)
{
    const int tiles_n = (g.n + SK_BN - 1) / SK_BN;
    const int nkb = g.k / KBLOCK;
    if (ksplit < 1 || ksplit > nkb || ksplit > 65535 || (ksplit > 1 && !partial))
        return hipErrorInvalidValue;
    const int kb_per_split = (nkb + ksplit - 1) / ksplit;
    dim3 grid(tiles_n, ksplit);
    hipError_t e;
    if (ksplit > 1) {
        auto kern = skinny_gemm_kernel<true>;
        FP8GEMM_ALLOW_LDS(kern, SK_LDS);
        hipLaunchKernelGGL(kern, grid, dim3(SK_THREADS), SK_LDS, s, g.a, g.b, g.a_scale, g.b_scale,
                           g.c, partial, g.m, g.n, g.k, tiles_n, kb_per_split);
        e = hipGetLastError();
        if (e != hipSuccess)
            return e;
        return launch_splitk_reduce(g, ksplit, partial, s);
    }
    auto kern = skinny_gemm_kernel<false>;
    FP8GEMM_ALLOW_LDS(kern, SK_LDS);
    hipLaunchKernelGGL(kern, grid, dim3(SK_THREADS), SK_LDS, s, g.a, g.b, g.a_scale, g.b_scale, g.c,
                       partial, g.m, g.n, g.k, tiles_n, kb_per_split);
    return hipGetLastError();
}

}  // namespace fp8gemm
