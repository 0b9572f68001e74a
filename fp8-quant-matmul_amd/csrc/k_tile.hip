// MFMA tile kernel for gfx950: the successor of in_smem_kernel (/root/reference/mn_large.hip:11-128)
// and, with the K range split over workgroups, of k_large_kernel (/root/reference/mn_small.hip:10-137).
//
// Data path (all of it differs from the reference, which scatters single bytes into LDS):
//   * A ([K][M], m contiguous) and B ([K][N], n contiguous) tiles of 128 K-rows are copied
//     global -> LDS with 16-byte buffer loads that write LDS directly (no VGPR round trip),
//     keeping the global orientation: one LDS row per k, 256 bytes per row.  The 16-byte
//     column chunk c of row r is stored at chunk position c ^ (2 * (r & 7)), which makes the
//     transposing reads below bank-conflict free.
//   * Operands are fetched with ds_read_b64_tr_b8: 16 lanes read an 8(k) x 16(m|n) byte
//     patch and receive it transposed, i.e. lane i holds 8 consecutive k of column i.  Four
//     such reads give the 32 bytes per lane that v_mfma_f32_32x32x64_f8f6f4 consumes.
//     The k order inside the instruction is permuted identically for both operands, which
//     leaves the dot product unchanged.
//   * Two MFMAs (K = 64 each) cover a 128-wide scale block of one 32x32 patch; the block sum
//     lives in 16 registers for a moment and is folded into the running result with
//     a_scale[kb][m] * b_scale[kb][n/128] by one FMA per element (mn_large.hip:100-106,
//     mn_small.hip:85-88 do the same with a second full-size accumulator).  The 16-pass
//     32x32x64 MFMA is used rather than the 8-pass 16x16x128 because a wave can issue about
//     eight VALU instructions in the shadow of the former and none in that of the latter
//     (measured), and this kernel needs ~11 VALU instructions per MFMA for the scale fold.
//   * The MFMA computes the transposed patch (rows = n, columns = m) as mn_small.hip does,
//     so that a lane owns one m (one a_scale value) and runs of 4 consecutive n (8-byte stores).
//   * Two LDS stages: the copy of K block kb+1 is in flight while block kb is multiplied.
//
// Work decomposition: grid.x = tiles (XCD-aware order), grid.y = K splits.
#include "device_common.h"
#include "launchers.h"

namespace fp8gemm {

namespace {

constexpr int LDS_ROW = 256;                       // bytes per k-row of a stage (A or B)
constexpr int LDS_MAT = KBLOCK * LDS_ROW;          // 32 KiB: one matrix, one stage
constexpr int LDS_STAGE = 2 * LDS_MAT;             // A then B
constexpr int LDS_TOTAL = 2 * LDS_STAGE;           // two stages, 128 KiB
constexpr int NTHREADS = 512;
constexpr int GROUP_M = 8;                         // tile rows per L2 locality group

template <int BM, int BN, int WM, int WN, bool SPLIT>
__global__ void __launch_bounds__(NTHREADS)
tile_gemm_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                 const float* __restrict__ a_scale, const float* __restrict__ b_scale,
                 uint16_t* __restrict__ c, float* __restrict__ partial, int M, int N, int K,
                 int tiles_m, int tiles_n, int kb_per_split)
{
    static_assert(WM * WN == 8, "eight waves per workgroup");
    constexpr int TM = BM / WM, TN = BN / WN;      // wave tile
    constexpr int MI = TM / 32, NJ = TN / 32;      // 32x32 patches per wave
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile is made of 32x32 patches");
    static_assert(TN <= 128, "a wave's n range touches at most two 128-wide scale blocks");
    static_assert(BM <= 256 && BN <= 256, "LDS rows hold 256 bytes");

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    auto lds = LDS_PTR(uint8_t, smem);
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = wave / WM;

    // ---- which tile: consecutive workgroup ids land on different XCDs (id % 8), so give
    // each XCD a contiguous run of tile numbers, and walk tiles in groups of GROUP_M rows
    // so that the tiles an XCD works on together share A and B panels in its L2.
    const int T = tiles_m * tiles_n;
    const int pid = blockIdx.x;
    const int xcd = pid & 7, q8 = T >> 3, r8 = T & 7;
    const int logical = xcd * q8 + (xcd < r8 ? xcd : r8) + (pid >> 3);
    const int per_group = GROUP_M * tiles_n;
    const int group = logical / per_group;
    const int first_m = group * GROUP_M;
    const int gsz = (tiles_m - first_m < GROUP_M) ? (tiles_m - first_m) : GROUP_M;
    const int in_group = logical - group * per_group;
    const int m0 = (first_m + in_group % gsz) * BM;
    const int n0 = (in_group / gsz) * BN;

    const int nkb = K / KBLOCK;
    const int kb0 = blockIdx.y * kb_per_split;
    const int kb1 = (kb0 + kb_per_split < nkb) ? (kb0 + kb_per_split) : nkb;

    // ---- global -> LDS copy plan.  A stage matrix is 32 slabs of 4 rows x 256 B; one
    // 16-byte load per lane fills a slab (LDS address = slab base + lane*16).  Wave w owns
    // slabs 4w..4w+3 of A and of B.  Lane l writes chunk position p = l & 15 of row r and
    // therefore fetches column chunk p ^ (2 * (r & 7)).  Chunks outside the tile or the matrix get
    // an out-of-range offset: the buffer load then returns zeros and touches no memory.
    uint32_t voff_a[4], voff_b[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int r = 16 * wave + 4 * q + (lane >> 4);
        const int cc = (lane & 15) ^ (2 * (r & 7));
        const bool va = (16 * cc < BM) && (m0 + 16 * cc < M);
        const bool vb = (16 * cc < BN) && (n0 + 16 * cc < N);
        voff_a[q] = va ? (uint32_t)(r * M + m0 + 16 * cc) : 0x80000000u;
        voff_b[q] = vb ? (uint32_t)(r * N + n0 + 16 * cc) : 0x80000000u;
    }
    const uint32_t a_bytes = (uint32_t)M * (uint32_t)K, b_bytes = (uint32_t)N * (uint32_t)K;

    // copy step q of K block kb into `stage`: q = 0..3 are the wave's A slabs, 4..7 its B slabs
    auto issue_copy_step = [&](int stage, int kb, int q) {
        const uint32_t dst = lds_base + (uint32_t)(stage * LDS_STAGE + wave * 4096);
        if (q < 4) {
            const uint32_t skip_a = (uint32_t)kb * KBLOCK * (uint32_t)M;
            lds_dma16(make_rsrc_words(a + skip_a, a_bytes - skip_a), voff_a[q], dst + q * 1024);
        } else {
            const uint32_t skip_b = (uint32_t)kb * KBLOCK * (uint32_t)N;
            lds_dma16(make_rsrc_words(b + skip_b, b_bytes - skip_b), voff_b[q - 4],
                      dst + LDS_MAT + (q - 4) * 1024);
        }
    };
    auto issue_copy = [&](int stage, int kb) {
#pragma unroll
        for (int q = 0; q < 8; ++q)
            issue_copy_step(stage, kb, q);
    };

    // ---- transposing LDS reads.  Lane l = 16*g + i feeds MFMA row/column (l & 31) and k half
    // (l >> 5).  For K step ks (64 wide) read t of the lane covers k rows
    // 64*ks + 32*(g>>1) + 8*t + (i>>1), 8-byte half (i & 1) of 16-byte chunk (patch chunk + (g&1)).
    // (row & 7) = (i >> 1) does not depend on t or ks: one address per patch plus immediates.
    const int g4 = lane >> 4, i16 = lane & 15;
    const int swz = 2 * (i16 >> 1);
    const uint32_t lane_off = (uint32_t)((32 * (g4 >> 1) + (i16 >> 1)) * LDS_ROW + (i16 & 1) * 8);
    uint32_t addr_a[MI], addr_b[NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
        addr_a[i] = lane_off + (uint32_t)((((wm * TM) / 16 + 2 * i + (g4 & 1)) ^ swz) * 16);
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        addr_b[j] = LDS_MAT + lane_off + (uint32_t)((((wn * TN) / 16 + 2 * j + (g4 & 1)) ^ swz) * 16);

    // 32 bytes per lane of one operand for K step ks
    auto read_frag = [&](uint32_t addr, int ks) -> v8i {
        const uint32_t base = addr + (uint32_t)(ks * 64 * LDS_ROW);
        v2i r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base));
        v2i r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 8 * LDS_ROW));
        v2i r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 16 * LDS_ROW));
        v2i r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 24 * LDS_ROW));
        return (v8i){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    };

    // ---- scales.  One a_scale per lane and 32-row patch (the lane's m).  A wave's n range is at
    // most 128 wide, so it touches at most two 128-wide b_scale blocks (nb_lo, nb_hi); a 32-wide
    // patch never straddles a block boundary.
    const int m_lane = m0 + wm * TM + (lane & 31);
    const int sn = (N + KBLOCK - 1) / KBLOCK;
    const int n_wave = n0 + wn * TN;
    int nb_lo = n_wave >> 7, nb_hi = (n_wave + TN - 1) >> 7;
    nb_lo = nb_lo < sn ? nb_lo : sn - 1;
    nb_hi = nb_hi < sn ? nb_hi : sn - 1;
    bool patch_hi[NJ];  // patch j lies in the second block
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        patch_hi[j] = ((n_wave + 32 * j) >> 7) > (n_wave >> 7);
    __amdgpu_buffer_rsrc_t ras = make_rsrc(a_scale, (uint32_t)nkb * (uint32_t)M * 4u);
    // raw scale values of one K block; the a_scale * b_scale product is formed when used
    auto load_scales = [&](int kb, float (&sa)[MI], float& sb_lo, float& sb_hi) {
        sb_lo = b_scale[(size_t)kb * sn + nb_lo];
        sb_hi = b_scale[(size_t)kb * sn + nb_hi];
#pragma unroll
        for (int i = 0; i < MI; ++i)
            sa[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                  ras, (uint32_t)((kb * M + m_lane + 32 * i) * 4), 0, 0));
    };

    v16f acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;
    const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // The copy and the scale loads of K block kb+1 are issued at the top of iteration kb and
    // first needed at the top of iteration kb+1: a whole block of MFMA work hides them.
    float sa_next[MI], sb_next = 0.f, sb_next_hi = 0.f;
#pragma unroll
    for (int i = 0; i < MI; ++i)
        sa_next[i] = 0.f;
    if (kb0 < kb1) {
        issue_copy(0, kb0);
        load_scales(kb0, sa_next, sb_next, sb_next_hi);
    }

    for (int kb = kb0; kb < kb1; ++kb) {
        const int stage = (kb - kb0) & 1;
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's LDS copies have landed
        __syncthreads();                     // everyone's have, and stage^1 is no longer read
        float s[MI], s_hi[MI];
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            s[i] = sa_next[i] * sb_next;
            s_hi[i] = sa_next[i] * sb_next_hi;
        }
        const bool more = kb + 1 < kb1;
        if (more)
            load_scales(kb + 1, sa_next, sb_next, sb_next_hi);

        // The eight copy instructions of the next K block are spread over the first half of
        // this block's MFMAs: issued in one burst right after the barrier, the 64 copies of a
        // workgroup queue up in the address unit and hold every wave back from its LDS reads.
        constexpr int N_MFMA = MI * NJ * 2;
        constexpr int SLOTS = (N_MFMA / 2 < 8) ? (N_MFMA / 2 < 1 ? 1 : N_MFMA / 2) : 8;
        int slot = 0;
        auto copy_slot = [&]() {
            if (slot < SLOTS) {
                if (more) {
#pragma unroll
                    for (int q = 0; q < 8; ++q)
                        if (q >= slot * 8 / SLOTS && q < (slot + 1) * 8 / SLOTS)
                            issue_copy_step(stage ^ 1, kb + 1, q);
                }
                ++slot;
            }
        };

        const uint32_t so = (uint32_t)(stage * LDS_STAGE);
        v8i fa[MI][2];
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            fa[i][0] = read_frag(addr_a[i] + so, 0);
            fa[i][1] = read_frag(addr_a[i] + so, 1);
        }
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const v8i fb0 = read_frag(addr_b[j] + so, 0);
            const v8i fb1 = read_frag(addr_b[j] + so, 1);
            v16f blk[MI];
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                blk[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb0, fa[i][0], zero16, 0, 0, 0,
                                                                          0, 0, 0);
                copy_slot();
            }
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                blk[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb1, fa[i][1], blk[i], 0, 0, 0,
                                                                          0, 0, 0);
                copy_slot();
            }
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const float sc = patch_hi[j] ? s_hi[i] : s[i];
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[i][j][r] = fmaf(sc, blk[i][r], acc[i][j][r]);
            }
        }
    }

    // ---- epilogue: lane owns row m = .. + (lane & 31) and, per patch, four runs of 4 columns:
    // accumulator register 4*q + e is column 8*q + 4*(lane >> 5) + e of the patch
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int mrow = m_lane + 32 * i;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int ncol = n0 + wn * TN + 32 * j + 8 * q + 4 * (lane >> 5);
                if (mrow < M && ncol < N) {
                    const size_t o = (size_t)mrow * N + ncol;
                    const v4f v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                   acc[i][j][4 * q + 3]};
                    if (SPLIT) {
                        *reinterpret_cast<v4f*>(partial + (size_t)blockIdx.y * M * N + o) = v;
                    } else {
                        uint2 pk;
                        pk.x = pack_bf16x2(v[0], v[1]);
                        pk.y = pack_bf16x2(v[2], v[3]);
                        *reinterpret_cast<uint2*>(c + o) = pk;
                    }
                }
            }
        }
    }
}

// sum of the K-split partials in split order, then bf16
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ partial,
                                                            uint16_t* __restrict__ c, size_t mn,
                                                            int ksplit)
{
    size_t i4 = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i4 >= mn)
        return;
    v4f s = *reinterpret_cast<const v4f*>(partial + i4);
    for (int z = 1; z < ksplit; ++z) {
        v4f p = *reinterpret_cast<const v4f*>(partial + (size_t)z * mn + i4);
        s += p;
    }
    uint2 pk;
    pk.x = pack_bf16x2(s[0], s[1]);
    pk.y = pack_bf16x2(s[2], s[3]);
    *reinterpret_cast<uint2*>(c + i4) = pk;
}

template <int BM, int BN, int WM, int WN>
hipError_t launch_variant(const GemmArgs& g, int ksplit, float* partial, hipStream_t s)
{
    const int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    const int nkb = g.k / KBLOCK;
    const int kb_per_split = (nkb + ksplit - 1) / ksplit;
    dim3 grid(tiles_m * tiles_n, ksplit);
    hipError_t e;
    if (ksplit > 1) {
        auto kern = tile_gemm_kernel<BM, BN, WM, WN, true>;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, LDS_TOTAL);
        if (e != hipSuccess)
            return e;
        hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), LDS_TOTAL, s, g.a, g.b, g.a_scale, g.b_scale,
                           g.c, partial, g.m, g.n, g.k, tiles_m, tiles_n, kb_per_split);
    } else {
        auto kern = tile_gemm_kernel<BM, BN, WM, WN, false>;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, LDS_TOTAL);
        if (e != hipSuccess)
            return e;
        hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), LDS_TOTAL, s, g.a, g.b, g.a_scale, g.b_scale,
                           g.c, partial, g.m, g.n, g.k, tiles_m, tiles_n, kb_per_split);
    }
    return hipGetLastError();
}

}  // namespace

bool tile_supports(const GemmArgs& g)
{
    // 16-byte copies need every k-row of a and b to start 16-byte aligned
    return g.m % 16 == 0 && g.n % 16 == 0 && (reinterpret_cast<uintptr_t>(g.a) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.b) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.c) % 8 == 0);
}

const char* tile_variant_name(int variant)
{
    switch (variant) {
    case TILE_256x256: return "tile256x256";
    case TILE_256x128: return "tile256x128";
    case TILE_128x128: return "tile128x128";
    case TILE_256x192: return "tile256x192";
    case TILE_128x192: return "tile128x192";
    default: return "tile?";
    }
}

void tile_variant_dims(int variant, int* bm, int* bn)
{
    switch (variant) {
    case TILE_256x256: *bm = 256; *bn = 256; break;
    case TILE_256x128: *bm = 256; *bn = 128; break;
    case TILE_256x192: *bm = 256; *bn = 192; break;
    case TILE_128x192: *bm = 128; *bn = 192; break;
    default: *bm = 128; *bn = 128; break;
    }
}

hipError_t launch_tile(const GemmArgs& g, int variant, int ksplit, float* partial, hipStream_t s)
{
    switch (variant) {
    case TILE_256x256: return launch_variant<256, 256, 4, 2>(g, ksplit, partial, s);
    case TILE_256x128: return launch_variant<256, 128, 4, 2>(g, ksplit, partial, s);
    case TILE_128x128: return launch_variant<128, 128, 2, 4>(g, ksplit, partial, s);
    case TILE_256x192: return launch_variant<256, 192, 4, 2>(g, ksplit, partial, s);
    case TILE_128x192: return launch_variant<128, 192, 4, 2>(g, ksplit, partial, s);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_splitk_reduce(const GemmArgs& g, int ksplit, const float* partial, hipStream_t s)
{
    size_t mn = (size_t)g.m * g.n;
    unsigned blocks = (unsigned)((mn / 4 + 255) / 256);
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, partial, g.c, mn, ksplit);
    return hipGetLastError();
}

}  // namespace fp8gemm
