// Persistent form of the MFMA tile kernel for shapes with more tiles than compute units.
//
// The plain kernel (k_tile.hip) runs one tile per workgroup: with one workgroup per CU (the LDS
// ring fills the CU) every round of 256 tiles pays the launch of a new workgroup, an empty
// ring (one global round trip before the first MFMA) and an output burst during which no MFMA
// runs.  Here a workgroup walks through its tiles itself and the ring never drains: the K
// blocks of all its tiles form one stream, the copies for block g+NS-1 of the stream are
// issued while block g is multiplied, also across a tile boundary, so the first blocks of
// the next tile land while the finished tile is converted and stored.
//
// The finished tile cannot use the whole ring as its staging area (NS-1 slots hold the next
// tile's blocks): it leaves in pieces of PR rows through the one slot whose block was
// multiplied last.
//
// Data path, LDS layout, MFMA orientation and scale folding are those of k_tile.hip
// (successor of in_smem_kernel, /root/reference/mn_large.hip:11-128; the reference lists a
// persistent kernel that overlaps the epilogue with the next tile as future work,
// /root/reference/README.md:29).
#include "tile_common.h"

namespace fp8gemm {

namespace {

#include "w4_loop.inc"

// One problem of a grouped launch as the kernel sees it.
struct Problem {
    const uint8_t* a;
    const uint8_t* b;
    const float* a_scale;
    const float* b_scale;
    uint16_t* c;
    int M;
    int lda;  // elements between consecutive k-rows of a and of a_scale (>= M, a multiple of 16)
};

// GROUPED = false: one problem (`one`), tiles_m x tiles_n tiles.  GROUPED = true: the problems of
// `tab` (same N and K, own M), whose tiles are numbered one group after the other.
template <int BM, int BN, int WM, int WN, int NS, int PR, bool GROUPED>
__device__ __forceinline__ void persistent_body(const Problem& one, const GroupTable* tab, int N, int K,
                                                int tiles_m, int tiles_n)
{
    constexpr int NW = WM * WN;    // waves per workgroup; four = one wave per SIMD (k_block_w4)
    constexpr int NTH = 64 * NW;
    using S = TileShape<BM, BN, WM, WN, NS, NW>;
    static_assert(NW == 8 || NW == 4, "eight or four waves per workgroup");
    static_assert(NS >= 2 && NS <= 4, "two to four LDS stages");
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int MI = TM / 32, NJ = TN / 32;
    static_assert(TM % 32 == 0 && TN % 32 == 0 && TN <= 128 && BM <= 256 && BN <= 256, "wave tile");
    constexpr int RSA = S::RSA, RSB = S::RSB, NA = S::NA, NB = S::NB, NCOPY = S::NCOPY;
    constexpr int CROW = BN * 2 + 8;          // staging bytes per tile row (conflict-free writes)
    static_assert(PR % 32 == 0 && BM % PR == 0, "a piece is a whole number of 32-row patches");
    static_assert(PR * CROW <= S::STAGE, "a piece must fit one ring slot");
    // four waves: the finished tile is staged beside the ring, which then never pauses
    constexpr int STAGING_W4 = NS * S::STAGE;
    static_assert(NW == 8 || STAGING_W4 + PR * CROW <= 160 * 1024, "ring and staging area exceed the LDS");
    constexpr int CPR = BN / 8;               // 16-byte chunks per tile row
    // fold of a patch column under the next column's MFMAs: pays for the 2 x 3 patches of the
    // 256 x 192 tile (4 % there), not for the smaller wave tiles (0 to -2 %)
    constexpr bool PIPELINED_FOLD = MI * NJ >= 6;
    constexpr int CHUNKS = PR * CPR;

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    auto lds = LDS_PTR(uint8_t, smem);
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = wave / WM;

    // ---- this workgroup's tiles.  Workgroup ids go round the 8 XCDs (id % 8); each XCD owns
    // a contiguous run of the tile order (groups of GROUP_M tile rows, as in k_tile.hip) and
    // its workgroups take the run's tiles in turn, so that the tiles an XCD works on at any
    // moment are neighbours and share A and B panels in its L2.
    const int T = GROUPED ? tab->tile_start[tab->groups] : tiles_m * tiles_n;
    const int pid = blockIdx.x, per_xcd = gridDim.x >> 3;  // gridDim.x is a multiple of 8
    const int xcd = pid & 7, q8 = T >> 3, r8 = T & 7;
    const int run0 = xcd * q8 + (xcd < r8 ? xcd : r8);
    const int run_len = q8 + (xcd < r8 ? 1 : 0);
    const int li = pid >> 3;
    const int n_my = li < run_len ? (run_len - li + per_xcd - 1) / per_xcd : 0;
    if (n_my == 0)
        return;
    const int per_group = GROUP_M * tiles_n;
    // tile number j of this workgroup: its problem and its origin in that problem's C
    auto tile_origin = [&](int j, Problem& pr, int& m0, int& n0) __attribute__((always_inline)) {
        int logical = run0 + li + j * per_xcd;
        int tm = tiles_m;
        if (GROUPED) {
            int g = 0;
            while (g + 1 < tab->groups && logical >= tab->tile_start[g + 1])
                ++g;
            logical -= tab->tile_start[g];
            pr = Problem{tab->a[g], tab->b[g], tab->a_scale[g], tab->b_scale[g], tab->c[g], tab->m[g], tab->lda[g]};
            tm = (pr.M + BM - 1) / BM;
        } else {
            pr = one;
        }
        const int group = logical / per_group;
        const int first_m = group * GROUP_M;
        const int gsz = (tm - first_m < GROUP_M) ? (tm - first_m) : GROUP_M;
        const int in_group = logical - group * per_group;
        m0 = (first_m + in_group % gsz) * BM;
        n0 = (in_group / gsz) * BN;
    };

    const int nkb = K / KBLOCK;
    const int sn = (N + KBLOCK - 1) / KBLOCK;
    // buffer resources of the copy stream's current tile (fixed for a single problem)
    v4i rsrc_a, rsrc_b, rsrc_s, rsrc_bs;
    int f_lda = one.lda;  // leading dimension of the problem the copy stream is in
    auto set_resources = [&](const Problem& pr) __attribute__((always_inline)) {
        rsrc_a = make_rsrc_words(pr.a, (uint32_t)pr.lda * (uint32_t)K);
        rsrc_b = make_rsrc_words(pr.b, (uint32_t)N * (uint32_t)K);
        rsrc_s = make_rsrc_words(pr.a_scale, (uint32_t)nkb * (uint32_t)pr.lda * 4u);
        rsrc_bs = make_rsrc_words(pr.b_scale, (uint32_t)nkb * (uint32_t)sn * 4u);
        f_lda = pr.lda;
    };

    // ---- the copy stream: K block f_kb of this workgroup's tile number f_tile is the next one
    // to be copied.  Per-lane offsets (copy plan of k_tile.hip) belong to that tile.
    uint32_t voff_a[S::NVA], voff_b[S::NVB], voff_s, voff_sb = 0x80000000u;
    int f_tile = 0, f_kb = 0;
    int fill_left = n_my * nkb;  // blocks not yet copied
    auto fill_setup = [&](int j) __attribute__((always_inline)) {
        Problem pr;
        int m0, n0;
        tile_origin(j, pr, m0, n0);
        if (GROUPED || j == 0)
            set_resources(pr);
        const int M = pr.M, lda = pr.lda;
#pragma unroll
        for (int q = 0; q < S::NVA; ++q) {
            const int r = RSA == 256 ? (NA * wave + q) * 4 + (lane >> 4) : (NA * wave + q) * 8 + (lane >> 3);
            const int cc = (RSA == 256 ? (lane & 15) : (lane & 7)) ^ row_swizzle<RSA>(r & 7);
            const bool ok = (16 * cc < BM) && (m0 + 16 * cc < M);
            voff_a[q] = ok ? (uint32_t)(r * lda + m0 + 16 * cc) : 0x80000000u;
        }
#pragma unroll
        for (int q = 0; q < S::NVB; ++q) {
            const int r = RSB == 256 ? (NB * wave + q) * 4 + (lane >> 4) : (NB * wave + q) * 8 + (lane >> 3);
            const int cc = (RSB == 256 ? (lane & 15) : (lane & 7)) ^ row_swizzle<RSB>(r & 7);
            const bool ok = (16 * cc < BN) && (n0 + 16 * cc < N);
            voff_b[q] = ok ? (uint32_t)(r * N + n0 + 16 * cc) : 0x80000000u;
        }
        voff_s = (4 * lane < BM && m0 + 4 * lane < M) ? (uint32_t)((m0 + 4 * lane) * 4) : 0x80000000u;
        if (NW == 4)  // lanes 0..3 bring b_scale[kb][n0/128 + lane]
            voff_sb = (lane < 4 && (n0 >> 7) + lane < sn) ? (uint32_t)(((n0 >> 7) + lane) * 4) : 0x80000000u;
    };
    // copy instruction q of the stream's next block into ring slot `slot`
    auto fill_copy = [&](int slot, int q) __attribute__((always_inline)) {
        const uint32_t stage = lds_base + (uint32_t)(slot * S::STAGE);
        if (q < NA) {
            lds_dma16(rsrc_a, voff_a[S::template voff_index<RSA>(q)], stage + (uint32_t)((NA * wave + q) * 1024),
                      (uint32_t)(f_kb * KBLOCK + S::template extra_rows<RSA>(q)) * (uint32_t)f_lda);
        } else if (q < NA + NB) {
            lds_dma16(rsrc_b, voff_b[S::template voff_index<RSB>(q - NA)],
                      stage + S::MAT_A + (uint32_t)((NB * wave + (q - NA)) * 1024),
                      (uint32_t)(f_kb * KBLOCK + S::template extra_rows<RSB>(q - NA)) * (uint32_t)N);
        } else if (wave == 0) {
            lds_dma16(rsrc_s, voff_s, stage + S::SCALE_OFF, (uint32_t)f_kb * (uint32_t)f_lda * 4u);
        } else if (NW == 4 && wave == 1) {
            lds_dma4(rsrc_bs, voff_sb, stage + S::SB_OFF, (uint32_t)f_kb * (uint32_t)sn * 4u);
        }
    };
    auto fill_advance = [&]() __attribute__((always_inline)) {
        --fill_left;
        if (++f_kb == nkb) {
            f_kb = 0;
            ++f_tile;
            if (fill_left > 0)
                fill_setup(f_tile);
        }
    };

    // ---- LDS read addresses (k_tile.hip): they do not depend on the tile
    const int g4 = lane >> 4, i16 = lane & 15;
    uint32_t addr_a[MI], addr_b[NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
        addr_a[i] = (uint32_t)((32 * (g4 >> 1) + (i16 >> 1)) * RSA + (i16 & 1) * 8 +
                               ((((wm * TM) / 16 + 2 * i + (g4 & 1)) ^ row_swizzle<RSA>(i16 >> 1)) * 16));
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        addr_b[j] = (uint32_t)(S::MAT_A + (32 * (g4 >> 1) + (i16 >> 1)) * RSB + (i16 & 1) * 8 +
                               ((((wn * TN) / 16 + 2 * j + (g4 & 1)) ^ row_swizzle<RSB>(i16 >> 1)) * 16));
    const uint32_t addr_s = S::SCALE_OFF + (uint32_t)((wm * TM + (lane & 31)) * 4);
    auto read_frag = [&](uint32_t addr, int ks, int rs) __attribute__((always_inline)) -> v8i {
        const uint32_t base = addr + (uint32_t)(ks * 64 * rs);
        v2i r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base));
        v2i r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 8 * rs));
        v2i r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 16 * rs));
        v2i r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 24 * rs));
        return (v8i){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    };
    const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // ---- a finished tile: bf16, in pieces of PR rows through `staging` (LDS bytes that nobody
    // else touches meanwhile), 16 bytes per lane along whole tile rows.  A lane owns row
    // m = .. + (lane & 31) and, per patch, four runs of 4 columns: stored straight from the
    // registers that would be 8-byte pieces of 32 different rows per instruction.
    // sum(i, jj, r) = running sum r of patch (i, jj)
    auto store_tile = [&](auto sum, uint32_t staging, int m0, int n0, int M,
                          uint16_t* __restrict__ c) __attribute__((always_inline)) {
        // opaque copy of the thread id: keeps the address arithmetic below inside the tile loop
        // (hoisted, it would sit in registers the K loop needs and be spilled)
        int tid = (int)threadIdx.x;
        asm volatile("" : "+v"(tid));
        const int lane_e = tid & 63;
#pragma unroll
        for (int p = 0; p < BM / PR; ++p) {
            if (p > 0)
                __syncthreads();  // the previous piece has been read out
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int prow = wm * TM + 32 * i;
                if (prow / PR == p) {
                    const uint32_t rbase = staging + (uint32_t)((prow - p * PR + (lane_e & 31)) * CROW);
#pragma unroll
                    for (int jj = 0; jj < NJ; ++jj)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int col = wn * TN + 32 * jj + 8 * q + 4 * (lane_e >> 5);
                            v2i pk = {(int)pack_bf16x2(sum(i, jj, 4 * q), sum(i, jj, 4 * q + 1)),
                                      (int)pack_bf16x2(sum(i, jj, 4 * q + 2), sum(i, jj, 4 * q + 3))};
                            *LDS_PTR(v2i, lds + rbase + col * 2) = pk;
                        }
                }
            }
            __syncthreads();
#pragma unroll
            for (int it = 0; it < (CHUNKS + NTH - 1) / NTH; ++it) {
                const int idx = it * NTH + tid;
                const int row = idx / CPR, ch = idx - row * CPR;
                const int mrow = m0 + p * PR + row;
                const int ncol = n0 + ch * 8;
                if (idx < CHUNKS && mrow < M && ncol < N) {
                    const v2i lo = *LDS_PTR(v2i, lds + staging + row * CROW + ch * 16);
                    const v2i hi = *LDS_PTR(v2i, lds + staging + row * CROW + ch * 16 + 8);
                    *reinterpret_cast<v4i*>(c + (size_t)mrow * N + ncol) = (v4i){lo.x, lo.y, hi.x, hi.y};
                }
            }
        }
    };

    if constexpr (NW == 4) {
        // ================= one wave per SIMD =================
        // A wave owns a 128 x 96 patch grid (2.33 transposing reads per MFMA instead of the 3.33 of
        // a 64 x 96 wave tile) and all 512 registers of its SIMD lane.  Nobody else issues on the
        // SIMD, so the K blocks run as one assembly loop with every instruction placed by hand
        // (w4_loop.inc; schedule, register map and wait counts: gen_w4_loop.py).  What that loop
        // does differently from the eight-wave schedule below:
        //   * the barrier of a K block sits before its LAST patch column: by then all fragments of
        //     the block are in registers, so the slot is free for the block after next right away,
        //     and the fragments of the next block (landed a whole block ago) are read while the
        //     last column is multiplied -- no MFMA waits for an LDS round trip behind a barrier;
        //   * the fold of a block's last patch rides on the first MFMAs of the next block;
        //   * b_scale rides in the stage like a_scale (a scalar load in flight would turn the
        //     counted LDS waits into full ones);
        //   * the finished tile is staged beside the two ring slots: the copy stream never pauses.
        // This part only walks the tiles, keeps the copy stream's bookkeeping and stores the tiles.
        static_assert(BM == 256 && BN == 192 && WM == 2 && WN == 2 && NS == 2 && !GROUPED,
                      "the assembly loop is written for this shape");
        static_assert(S::STAGE == 66816 && NA == 8 && NB == 8, "ring geometry the assembly loop assumes");
        const uint32_t scale_kind = wave < 2 ? (uint32_t)wave : 2u;
        const uint32_t lds_wave = lds_base + (uint32_t)(NA * wave * 1024);
        const uint32_t lds_scale = lds_base + (wave == 0 ? S::SCALE_OFF : S::SB_OFF);
        const uint32_t vbase_a0 = lds_base + addr_a[0], vbase_a1 = lds_base + addr_a[1];
        const uint32_t vbase_a2 = lds_base + addr_a[2], vbase_a3 = lds_base + addr_a[3];
        const uint32_t vbase_b0 = lds_base + addr_b[0], vbase_b1 = lds_base + addr_b[1], vbase_b2 = lds_base + addr_b[2];
        const uint32_t vaddr_s = lds_base + addr_s;

        v32f sums[6], blk;
        v32i frag0 = {}, frag1 = {}, frag2 = {};
        v16i frag3 = {};
        float scale_carry = 0.f;
#pragma unroll
        for (int r = 0; r < 32; ++r)
            blk[r] = 0.f;

        // once the stream has run dry its copy instructions stay in the loop with offsets outside
        // their buffers: they fetch nothing and write zeros into the slot nobody reads
        auto stream_dry = [&]() __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < S::NVA; ++q)
                voff_a[q] = 0x80000000u;
#pragma unroll
            for (int q = 0; q < S::NVB; ++q)
                voff_b[q] = 0x80000000u;
            voff_s = voff_sb = 0x80000000u;
        };
        fill_setup(0);
#pragma unroll
        for (int q = 0; q < NCOPY; ++q)
            fill_copy(0, q);
        fill_advance();
        if (fill_left > 0) {
#pragma unroll
            for (int q = 0; q < NCOPY; ++q)
                fill_copy(1, q);
            fill_advance();
            wait_vmcnt<NCOPY - 1>();  // block 0 landed (waves 0 and 1: and their first copy of block 1)
        } else {
            wait_vmcnt<0>();
        }
        if (fill_left == 0)
            stream_dry();
        __syncthreads();
        w4_first_reads(frag0, frag1, frag2, frag3, vbase_a0, vbase_a1, vbase_a2, vbase_a3, vbase_b0);

        uint32_t slot_off = 0;  // LDS offset of the ring slot of the block multiplied next
        for (int j = 0; j < n_my; ++j) {
            Problem pr;
            int m0, n0;
            tile_origin(j, pr, m0, n0);
            const int n_wave = n0 + wn * TN;
            // the stage holds b_scale[kb][n0/128 + 0..3]; a wave's n range touches at most two of them
            const uint32_t lds_sb_lo = lds_base + S::SB_OFF + 4u * (uint32_t)((n_wave >> 7) - (n0 >> 7));
            const uint32_t lds_sb_hi = lds_base + S::SB_OFF + 4u * (uint32_t)(((n_wave + TN - 1) >> 7) - (n0 >> 7));
            uint32_t hi_mask[NJ];  // all ones when patch column jj lies in the wave's second b_scale block
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj)
                hi_mask[jj] = (uint32_t)-(int)(((n_wave + 32 * jj) >> 7) > (n_wave >> 7));
#pragma unroll
            for (int t = 0; t < 6; ++t)
#pragma unroll
                for (int r = 0; r < 32; ++r)
                    sums[t][r] = 0.f;

            int kb = 0;
            while (kb < nkb) {
                // as many blocks as the copy stream can take without leaving its tile
                int cnt = nkb - kb;
                if (fill_left > 0 && nkb - f_kb < cnt)
                    cnt = nkb - f_kb;
                uint32_t count = (uint32_t)cnt;
                const uint32_t str_a = (uint32_t)(KBLOCK * f_lda), str_b = (uint32_t)(KBLOCK * N);
                const uint32_t str_sc = wave == 0 ? (uint32_t)f_lda * 4u : (uint32_t)sn * 4u;
                uint32_t off_a = (uint32_t)f_kb * str_a, off_b = (uint32_t)f_kb * str_b, off_sc = (uint32_t)f_kb * str_sc;
                // wave-uniform operands of the loop must sit in scalar registers
                auto sgpr = [](uint32_t x) __attribute__((always_inline)) {
                    return (uint32_t)__builtin_amdgcn_readfirstlane((int)x);
                };
                off_a = sgpr(off_a), off_b = sgpr(off_b), off_sc = sgpr(off_sc), count = sgpr(count);
                slot_off = sgpr(slot_off);
                w4_k_blocks(sums[0], sums[1], sums[2], sums[3], sums[4], sums[5], blk, frag0, frag1, frag2, frag3,
                            scale_carry, vbase_a0, vbase_a1, vbase_a2, vbase_a3, vbase_b0, vbase_b1, vbase_b2,
                            vaddr_s, voff_a[0], voff_a[1], voff_b[0], voff_b[1], wave == 0 ? voff_s : voff_sb,
                            rsrc_a, rsrc_b, wave == 0 ? rsrc_s : rsrc_bs, off_a, off_b, off_sc, sgpr(str_a),
                            sgpr(str_b), sgpr(str_sc), sgpr((uint32_t)(8 * f_lda)), sgpr((uint32_t)(8 * N)), slot_off,
                            sgpr(lds_wave), sgpr(lds_scale), sgpr(scale_kind), sgpr(lds_sb_lo), sgpr(lds_sb_hi),
                            sgpr(hi_mask[0]), sgpr(hi_mask[1]), sgpr(hi_mask[2]), count);
                kb += cnt;
                if (fill_left > 0) {
                    fill_left -= cnt;
                    f_kb += cnt;
                    if (f_kb == nkb) {
                        f_kb = 0;
                        ++f_tile;
                        if (fill_left > 0)
                            fill_setup(f_tile);
                        else
                            stream_dry();
                    }
                }
            }
            // the last patch's fold, then the tile leaves through the staging area
            w4_last_fold(sums[5], blk, scale_carry);
            scale_carry = 0.f;
#pragma unroll
            for (int r = 16; r < 32; ++r)
                blk[r] = 0.f;
            store_tile([&](int i, int jj, int r) __attribute__((always_inline)) {
                           const int q = jj * MI + i;
                           return sums[q / 2][(q % 2) * 16 + r];
                       },
                       (uint32_t)STAGING_W4, m0, n0, pr.M, pr.c);
        }
        return;
    }

    // ---- fill the ring: the first NS-1 blocks of the stream
    fill_setup(0);
#pragma unroll
    for (int p = 0; p < NS - 1; ++p)
        if (fill_left > 0) {
#pragma unroll
            for (int q = 0; q < NCOPY; ++q)
                fill_copy(p, q);
            fill_advance();
        }
    int slot = 0;            // ring slot of the block being multiplied
    int slot_fill = NS - 1;  // ring slot the stream's next block goes into

    for (int j = 0; j < n_my; ++j) {
        Problem pr;
        int m0, n0;
        tile_origin(j, pr, m0, n0);
        const float* __restrict__ b_scale = pr.b_scale;
        uint16_t* __restrict__ c = pr.c;
        const int M = pr.M;
        const int n_wave = n0 + wn * TN;
        int nb_lo = n_wave >> 7, nb_hi = (n_wave + TN - 1) >> 7;
        nb_lo = nb_lo < sn ? nb_lo : sn - 1;
        nb_hi = nb_hi < sn ? nb_hi : sn - 1;
        uint32_t hi_mask[NJ];  // all ones when patch jj lies in the wave's second b_scale block
#pragma unroll
        for (int jj = 0; jj < NJ; ++jj)
            hi_mask[jj] = (uint32_t)-(int)(((n_wave + 32 * jj) >> 7) > (n_wave >> 7));

        v16f acc[MI][NJ];
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[i][jj][r] = 0.f;

        // One K block.  MORE = the stream has a block left to copy (always, except for the last
        // NS-1 blocks of the last tile).
        auto k_block = [&](auto more_tag, int kb) __attribute__((always_inline)) {
            constexpr bool more = decltype(more_tag)::value;
            // The first NS-1 blocks of a later tile were copied before the previous tile's
            // epilogue, which waited for them: no wait here, and none that would drag in that
            // epilogue's stores.  Otherwise at most the younger blocks may be outstanding.
            const bool landed = j > 0 && kb < NS - 1;
            if (!landed) {
                if (more) {
                    wait_vmcnt<(NS - 2) * (NCOPY - 1)>();
                } else {
                    const int younger = (nkb - 1 - kb < NS - 2) ? (nkb - 1 - kb) : (NS - 2);
                    if (NS >= 4 && younger >= 2)
                        wait_vmcnt<2 * (NCOPY - 1)>();
                    else if (NS >= 3 && younger >= 1)
                        wait_vmcnt<NCOPY - 1>();
                    else
                        wait_vmcnt<0>();
                }
            }
            __syncthreads();  // block landed for everyone; slot_fill is no longer read
            const uint32_t so = (uint32_t)(slot * S::STAGE);
            float sa[MI];
#pragma unroll
            for (int i = 0; i < MI; ++i)
                sa[i] = *LDS_PTR(float, lds + so + addr_s + 128 * i);
            const float sb_lo = b_scale[__builtin_amdgcn_readfirstlane(kb * sn + nb_lo)];
            const float sb_hi = b_scale[__builtin_amdgcn_readfirstlane(kb * sn + nb_hi)];

            v8i fa[MI][2];
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                fa[i][0] = read_frag(addr_a[i] + so, 0, RSA);
                fa[i][1] = read_frag(addr_a[i] + so, 1, RSA);
            }
            constexpr int N_MFMA = MI * NJ * 2;
            constexpr int PER_MFMA = (NCOPY + N_MFMA - 1) / N_MFMA;
            int cq = 0;
            auto copy_slot = [&](int n) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < NCOPY; ++u)
                    if (u < n && cq < NCOPY) {
                        if (more)
                            fill_copy(slot_fill, cq);
                        ++cq;
                    }
            };
            if (PIPELINED_FOLD) {
                // Column jj's MFMAs write the block sums that column jj-1's fold has just read: the
                // fold of patch (i, jj-1) sits in program order right before the first MFMA of
                // patch (i, jj), pinned there (an empty asm statement that both the folded
                // accumulator and the MFMA's B fragment pass through), so that its 16 FMAs issue
                // while the MFMAs before it are still in the pipe.  Left alone, the compiler issues
                // all MFMAs of a K block first and all folds after them, the matrix pipe idle
                // meanwhile (both waves of a SIMD reach that phase together, after the barrier).
                v16f blk[MI];
                float sc_prev[MI];
#pragma unroll
                for (int jj = 0; jj <= NJ; ++jj) {
                    v8i fb0, fb1;
                    if (jj < NJ) {
                        fb0 = read_frag(addr_b[jj] + so, 0, RSB);
                        fb1 = read_frag(addr_b[jj] + so, 1, RSB);
                    }
#pragma unroll
                    for (int i = 0; i < MI; ++i) {
                        if (jj > 0) {
#pragma unroll
                            for (int r = 0; r < 16; ++r)
                                acc[i][jj - 1][r] = fmaf(sc_prev[i], blk[i][r], acc[i][jj - 1][r]);
                            if (jj < NJ)
                                asm volatile("" : "+v"(acc[i][jj - 1]), "+v"(fb0));
                        }
                        if (jj < NJ) {
                            blk[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb0, fa[i][0], zero16, 0, 0,
                                                                                      0, 0, 0, 0);
                            copy_slot(PER_MFMA);
                        }
                    }
                    if (jj < NJ) {
#pragma unroll
                        for (int i = 0; i < MI; ++i) {
                            blk[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb1, fa[i][1], blk[i], 0, 0,
                                                                                      0, 0, 0, 0);
                            copy_slot(PER_MFMA);
                        }
                        // wave-uniform choice of the b_scale value on the scalar unit (bit select),
                        // then one product per patch
                        const float sbj = __uint_as_float((__float_as_uint(sb_hi) & hi_mask[jj]) |
                                                          (__float_as_uint(sb_lo) & ~hi_mask[jj]));
#pragma unroll
                        for (int i = 0; i < MI; ++i)
                            sc_prev[i] = sa[i] * sbj;
                    }
                }
            } else {
#pragma unroll
                for (int jj = 0; jj < NJ; ++jj) {
                    const v8i fb0 = read_frag(addr_b[jj] + so, 0, RSB);
                    const v8i fb1 = read_frag(addr_b[jj] + so, 1, RSB);
                    v16f blk[MI];
#pragma unroll
                    for (int i = 0; i < MI; ++i) {
                        blk[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb0, fa[i][0], zero16, 0, 0, 0,
                                                                                  0, 0, 0);
                        copy_slot(PER_MFMA);
                    }
#pragma unroll
                    for (int i = 0; i < MI; ++i) {
                        blk[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb1, fa[i][1], blk[i], 0, 0, 0,
                                                                                  0, 0, 0);
                        copy_slot(PER_MFMA);
                    }
#pragma unroll
                    for (int i = 0; i < MI; ++i) {
                        // wave-uniform choice of the b_scale value on the scalar unit (bit select), then one
                        // product per patch
                        const float sbj = __uint_as_float((__float_as_uint(sb_hi) & hi_mask[jj]) |
                                                          (__float_as_uint(sb_lo) & ~hi_mask[jj]));
                        const float sc = sa[i] * sbj;
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            acc[i][jj][r] = fmaf(sc, blk[i][r], acc[i][jj][r]);
                    }
                }
            }
            copy_slot(NCOPY);
            if (more)
                fill_advance();
            slot_fill = slot;
            slot = (slot + 1 == NS) ? 0 : slot + 1;
        };

        // the host launches this kernel only for nkb >= NS-1: the stream then runs dry in the
        // last NS-1 blocks of the last tile and nowhere else
        const int tail = (j + 1 < n_my) ? 0 : NS - 1;
        int kb = 0;
        for (; kb < nkb - tail; ++kb)
            k_block(std::true_type{}, kb);
        for (; kb < nkb; ++kb)
            k_block(std::false_type{}, kb);

        // ---- epilogue: bf16, in pieces of PR rows through the ring slot of the block multiplied
        // last (slot_fill by now; the stream's next copy goes there, but not before the next
        // K block's barrier).  Every copy of the stream issued so far has to have landed before
        // the first store goes out: the next tile's first blocks are then known to be there
        // without a wait that would also cover these stores.
        wait_vmcnt<0>();
        __syncthreads();  // every wave has finished reading that slot
        // (the same steps as store_tile, written out: handed to that lambda through an accessor, the
        // running sums cost the K loop 9 more registers and the kernel 1-2 % on the headline shape)
        {
            const uint32_t staging = (uint32_t)(slot_fill * S::STAGE);
            int tid = (int)threadIdx.x;
            asm volatile("" : "+v"(tid));
            const int lane_e = tid & 63;
#pragma unroll
            for (int p = 0; p < BM / PR; ++p) {
                if (p > 0)
                    __syncthreads();  // the previous piece has been read out
#pragma unroll
                for (int i = 0; i < MI; ++i) {
                    const int prow = wm * TM + 32 * i;
                    if (prow / PR == p) {
                        const uint32_t rbase = staging + (uint32_t)((prow - p * PR + (lane_e & 31)) * CROW);
#pragma unroll
                        for (int jj = 0; jj < NJ; ++jj)
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                const int col = wn * TN + 32 * jj + 8 * q + 4 * (lane_e >> 5);
                                v2i pk = {(int)pack_bf16x2(acc[i][jj][4 * q], acc[i][jj][4 * q + 1]),
                                          (int)pack_bf16x2(acc[i][jj][4 * q + 2], acc[i][jj][4 * q + 3])};
                                *LDS_PTR(v2i, lds + rbase + col * 2) = pk;
                            }
                    }
                }
                __syncthreads();
#pragma unroll
                for (int it = 0; it < (CHUNKS + NTH - 1) / NTH; ++it) {
                    const int idx = it * NTH + tid;
                    const int row = idx / CPR, ch = idx - row * CPR;
                    const int mrow = m0 + p * PR + row;
                    const int ncol = n0 + ch * 8;
                    if (idx < CHUNKS && mrow < M && ncol < N) {
                        const v2i lo = *LDS_PTR(v2i, lds + staging + row * CROW + ch * 16);
                        const v2i hi = *LDS_PTR(v2i, lds + staging + row * CROW + ch * 16 + 8);
                        *reinterpret_cast<v4i*>(c + (size_t)mrow * N + ncol) = (v4i){lo.x, lo.y, hi.x, hi.y};
                    }
                }
            }
        }
        // the next tile's first K block begins with a barrier: the slot is not written again
        // before every lane has read its chunks of the last piece
    }
}

template <int BM, int BN, int WM, int WN, int NS, int PR>
__global__ void __launch_bounds__(64 * WM * WN)
tile_gemm_persistent_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                            const float* __restrict__ a_scale, const float* __restrict__ b_scale,
                            uint16_t* __restrict__ c, int M, int lda, int N, int K, int tiles_m, int tiles_n)
{
    const Problem one{a, b, a_scale, b_scale, c, M, lda};
    persistent_body<BM, BN, WM, WN, NS, PR, false>(one, nullptr, N, K, tiles_m, tiles_n);
}

template <int BM, int BN, int WM, int WN, int NS, int PR>
__global__ void __launch_bounds__(64 * WM * WN)
tile_gemm_grouped_kernel(const GroupTable tab, int N, int K, int tiles_n)
{
    const Problem none{nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0};
    persistent_body<BM, BN, WM, WN, NS, PR, true>(none, &tab, N, K, 0, tiles_n);
}

template <int BM, int BN, int WM, int WN, int NS, int PR>
hipError_t launch_persistent_variant(const GemmArgs& g, int workgroups, hipStream_t s)
{
    using S = TileShape<BM, BN, WM, WN, NS, WM * WN>;
    // four waves stage the finished tile beside the ring
    constexpr int LDS_TOTAL = S::LDS_BYTES + (WM * WN == 4 ? PR * (BN * 2 + 8) : 0);
    const int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    auto kern = tile_gemm_persistent_kernel<BM, BN, WM, WN, NS, PR>;
    FP8GEMM_ALLOW_LDS(kern, LDS_TOTAL);
    hipLaunchKernelGGL(kern, dim3(workgroups), dim3(64 * WM * WN), LDS_TOTAL, s, g.a, g.b, g.a_scale,
                       g.b_scale, g.c, g.m, leading_dim(g), g.n, g.k, tiles_m, tiles_n);
    return hipGetLastError();
}

template <int BM, int BN, int WM, int WN, int NS, int PR>
hipError_t launch_grouped_variant(GroupTable& tab, int n, int k, int workgroups, hipStream_t s)
{
    using S = TileShape<BM, BN, WM, WN, NS>;
    constexpr int LDS_TOTAL = S::LDS_BYTES;
    const int tiles_n = (n + BN - 1) / BN;
    tab.tile_start[0] = 0;
    for (int g = 0; g < tab.groups; ++g)
        tab.tile_start[g + 1] = tab.tile_start[g] + ((tab.m[g] + BM - 1) / BM) * tiles_n;
    auto kern = tile_gemm_grouped_kernel<BM, BN, WM, WN, NS, PR>;
    FP8GEMM_ALLOW_LDS(kern, LDS_TOTAL);
    hipLaunchKernelGGL(kern, dim3(workgroups), dim3(NTHREADS), LDS_TOTAL, s, tab, n, k, tiles_n);
    return hipGetLastError();
}

int persistent_stages(int variant)
{
    switch (variant) {
    case TILE_256x192: return 2;
    case TILE_256x128: return 3;
    case TILE_128x192: return 3;
    case TILE_128x128: return 4;
    case TILE_256x192_W4: return 2;
    case TILE_256x256: return 2;
    default: return 0;
    }
}

}  // namespace

bool tile_persistent_supports(const GemmArgs& g, int variant)
{
    const int stages = persistent_stages(variant);
    return stages > 0 && tile_supports(g) && g.k / KBLOCK >= stages - 1;
}

hipError_t launch_tile_persistent(const GemmArgs& g, int variant, int workgroups, hipStream_t s)
{
    if (workgroups <= 0 || workgroups % 8 != 0 || !tile_persistent_supports(g, variant))
        return hipErrorInvalidValue;
    switch (variant) {
    case TILE_256x192: return launch_persistent_variant<256, 192, 4, 2, 2, 128>(g, workgroups, s);
    case TILE_256x128: return launch_persistent_variant<256, 128, 4, 2, 3, 128>(g, workgroups, s);
    case TILE_128x192: return launch_persistent_variant<128, 192, 4, 2, 3, 128>(g, workgroups, s);
    case TILE_128x128: return launch_persistent_variant<128, 128, 2, 4, 4, 128>(g, workgroups, s);
    case TILE_256x192_W4: return launch_persistent_variant<256, 192, 2, 2, 2, 64>(g, workgroups, s);
    case TILE_256x256: return launch_persistent_variant<256, 256, 4, 2, 2, 128>(g, workgroups, s);
    default: return hipErrorInvalidValue;
    }
}

// every group non-empty, aligned like a single problem, K long enough for the ring
bool tile_grouped_supports(const GroupTable& tab, int n, int k, int variant)
{
    const int stages = persistent_stages(variant);
    if (stages == 0 || variant == TILE_256x192_W4 ||  // the one-wave-per-SIMD loop is written for a single problem
        k / KBLOCK < stages - 1 || tab.groups < 1 || tab.groups > GroupTable::MAX_GROUPS)
        return false;
    for (int g = 0; g < tab.groups; ++g) {
        const GemmArgs ga{tab.a[g], tab.b[g], tab.a_scale[g], tab.b_scale[g], tab.c[g], tab.m[g], n, k, tab.lda[g]};
        if (tab.m[g] <= 0 || !tile_supports(ga))
            return false;
    }
    return true;
}

hipError_t launch_tile_grouped(GroupTable& tab, int n, int k, int variant, int workgroups, hipStream_t s)
{
    if (workgroups <= 0 || workgroups % 8 != 0 || !tile_grouped_supports(tab, n, k, variant))
        return hipErrorInvalidValue;
    switch (variant) {
    case TILE_256x192: return launch_grouped_variant<256, 192, 4, 2, 2, 128>(tab, n, k, workgroups, s);
    case TILE_256x128: return launch_grouped_variant<256, 128, 4, 2, 3, 128>(tab, n, k, workgroups, s);
    case TILE_128x192: return launch_grouped_variant<128, 192, 4, 2, 3, 128>(tab, n, k, workgroups, s);
    case TILE_128x128: return launch_grouped_variant<128, 128, 2, 4, 4, 128>(tab, n, k, workgroups, s);
    case TILE_256x256: return launch_grouped_variant<256, 256, 4, 2, 2, 128>(tab, n, k, workgroups, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace fp8gemm
