// Wide-strip decode kernel for tiny M (M <= 64): HBM-bound, B is read exactly once, in whole
// 128-byte lines.  The reference has no kernel for this regime (its smallest tile needs M >= 64,
// /root/reference/mn_small.hip:16,121-125); the math is the same block-scaled product
// (/root/reference/check.cu:36-48).
//
// Work split.  One workgroup owns a strip of 128 columns of C and a range of K blocks; with 56
// strips (N = 7168) the K range is cut in four so that 224 workgroups pull on the memory system at
// once, each fetching a [K/4 x 128 B] slab of B (whole cache lines) and the matching quarter of A.
// The narrow-strip kernel (k_skinny.hip) fills the chip without a K split but uses 32 bytes of every
// 128-byte line per workgroup and re-reads all of A in every workgroup.
//
// Inside a workgroup the eight waves copy one K block per stage together (global -> LDS, 16 bytes
// per lane, written by the load itself), meet at one barrier per stage, and then each wave multiplies
// its own 16 columns against all rows of A with v_mfma_f32_16x16x128_f8f6f4 (rows = n, columns = m,
// operands through ds_read_b64_tr_b8 as in the tile kernel): a wave ends with the complete partial
// result of its 32 x 16 patch for the workgroup's K range and no reduction across waves is needed.
//
// The K splits of a strip are added inside the kernel, wave by wave, without a second launch and without
// a ticket or a fence:
//   * the workgroups of one strip are given linear ids that agree modulo 8, which the dispatcher
//     places on one XCD (checked once per device by a probe grid, xcd_placement_confirmed): their
//     stores and loads meet in that XCD's L2, and no device-scope fence -- a write-back of the whole
//     L2 on this part -- is needed;
//   * the partial patches travel through a mailbox, a region of the workspace that only this kernel
//     writes and that holds zeros whenever no launch is running.  A wave of every split but the last
//     stores its fp32 partial patch there (register order, 1 KiB per instruction) with every +0.0 replaced
//     by -0.0, so that no word it writes is zero, and is done: it waits for nothing;
//   * the wave of the last split -- the workgroup with the highest id of its strip, dispatched after the
//     others -- loads the patches of its 16 columns past its L1 (sc1) again and again until no word of
//     them is zero, stores zeros back for the next launch, and adds them in split order, its own registers
//     last: the sum does not depend on timing (adding -0.0 changes nothing, and a running sum that starts
//     from +0.0 is never -0.0 itself).  A wave that has polled for a second gives up and writes NaN.
// Against storing, waiting for the acknowledgement, taking a ticket with an atomic and loading as the last
// arrival (three round trips to the L2, 2.8 us on the timeline of M = 32, N = 7168, K = 2048 split in
// four) this is one store and the polling load.
//
// M <= 32 runs with two 16-row tiles of A (32-byte LDS rows), M <= 64 with four (64-byte rows); the same
// body runs grouped problems (common N and K, own M <= 64, own operands: the experts of an MoE layer in a
// decode step), whose strips form one list of work items.
//
// Variants of the same body (template arguments): a row count off the 16-byte grid (RAGGED: A's packed K-block
// slabs are copied whole and spread into padded rows in the LDS); strips of 256 columns (NB = 2: two
// 128-column halves per stage; 256 contiguous bytes of a k-row come 10 % faster from HBM than 128, at half
// the workgroups per split); one copy of the K loop per number of row tiles, so that no branch surrounds its
// LDS operations.  The streaming form (decode_stream_body) is for launches with more strips than the device
// holds workgroups and no K split: 256 workgroups walk through the strips -- of one problem or of all groups --
// and the K blocks of all strips of a workgroup form one copy stream.
//
// LDS stage: 128 k-rows x 128 B of B (chunk c of row r at position c ^ ((r >> 1) & 7)), 128 x 32 B
// of A (chunk c at c ^ ((r >> 3) & 1); 64-byte rows: c ^ ((r >> 2) & 3)), the block's a_scale and b_scale values; six stages form a
// ring, up to five in flight while one is multiplied.  A CU takes in about 50 bytes per clock through
// this path whatever the instruction mix, so the copy instructions of a workgroup's whole K range
// (80 KB for a quarter of K = 2048) are what its run time is made of; small stages let the multiplying
// start when the first 20 KB have landed.
#include "device_common.h"
#include "launchers.h"

#include <mutex>
#include <type_traits>

namespace fp8gemm {

namespace {

constexpr int DS_BN = 128;
constexpr int DS_THREADS = 512;
constexpr int RAGGED4_NS = 4;  // ring stages of the four-row-tile kernel that also holds A's packed slabs
constexpr unsigned AUX_L1_MISS = 16;  // cache policy of the partial-patch loads (sc1): past the L1, served by the L2
constexpr unsigned long long SPIN_LIMIT_TICKS = 100000000ull;  // one second of the constant 100 MHz counter (s_memrealtime)

// MT = 16-row tiles of A a workgroup multiplies (2: M <= 32, 4: M <= 64); DS_NS = stages of the LDS ring (6: one
// workgroup per CU with its whole K range in flight when that is short; 3: two workgroups per CU, so that one
// streams while the other starts up or hands over -- for launches of many workgroups with long K ranges)
// RAGGED = the row count is not a multiple of 16, so that k-rows of A do not start on 16-byte boundaries: a stage
// then also holds the K block's slab of A as it lies in memory, [128][M] bytes packed -- which does start on a
// 16-byte boundary, 128 * M * kb bytes into A -- and the threads spread it into the padded rows the reads expect.
// NB = 128-column halves of a strip (1; 2 in the streaming form of wide problems: 256 contiguous bytes of every
// k-row instead of 128, which the memory system serves 10 % faster, and A's fragments used twice).  Each half is a
// [128][128] byte matrix of its own in the stage, laid out and swizzled alike.
template <int MT, int DS_NS, bool RAGGED = false, int NB = 1>
struct DecodeShape {
    static constexpr int RSA = 16 * MT;                 // LDS bytes per k-row of A
    static constexpr int HALF_B = KBLOCK * 128;
    static constexpr int MAT_B = HALF_B * NB;
    static constexpr int MAT_A = KBLOCK * RSA;
    static constexpr int SA_OFF = MAT_B + MAT_A;        // up to 64 a_scale floats
    static constexpr int SB_OFF = SA_OFF + 256;         // NB floats (every wave that brings them writes the same bytes)
    static constexpr int PACK_OFF = SB_OFF + 256;       // RAGGED: the packed slab of A, up to MAT_A bytes, and 16
    // bytes the last row's reads may run into; stages start on 512-byte boundaries
    static constexpr int STAGE = RAGGED ? (PACK_OFF + MAT_A + 16 + 511) / 512 * 512 : PACK_OFF;
    static constexpr int LDS = DS_NS * STAGE;
    // copy instructions per wave and stage: two of B, then A / scales
    //   MT = 2: waves 0..3 A (32 rows x 32 B each), wave 4 a_scale, waves 5..7 b_scale
    //   MT = 4: every wave A (16 rows x 64 B each), then wave 0 a_scale, waves 1..7 b_scale
    static constexpr int COPIES = 2 * NB + (MT == 2 ? 1 : 2);
    static_assert(MT == 2 || MT == 4, "two or four row tiles");
    static_assert(LDS <= 160 * 1024, "ring exceeds the LDS");
    static_assert(COPIES * (DS_NS - 1) < 64, "vmcnt is a 6-bit field");
};

template <int N>
__device__ __forceinline__ void ds_wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// one problem as the kernel sees it
struct DecodeProblem {
    const uint8_t* a;
    const uint8_t* b;
    const float* a_scale;
    const float* b_scale;
    uint16_t* c;
    int M;    // rows of c
    int lda;  // elements between consecutive k-rows of a and of a_scale (>= M; rows M .. lda-1 hold zeros)
};

// Work units = (problem, strip), numbered problem-major; `units` of them.  Linear workgroup ids that
// agree modulo 8 share an XCD: the ksplit workgroups of unit u sit at ids xcd + 8 * (grp * ksplit + split)
// with u = grp * 8 + xcd.
// TILES = the number of 16-row tiles when the launch knows it (a single problem: the count is then a constant
// in the epilogue as well), 0 = read from the problem (grouped launches).
template <int MT, bool GROUPED, int DS_NS, bool RAGGED, int TILES, int NB>
__device__ __forceinline__ void decode_body(const DecodeProblem& one, const GroupTable* tab, float* mailbox, int N, int K,
                                            int strips, int units, int ksplit, int kb_per_split)
{
    using S = DecodeShape<MT, DS_NS, RAGGED, NB>;
    constexpr int BN = DS_BN * NB;  // columns of a strip
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    auto lds = LDS_PTR(uint8_t, smem);
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    const int pid = blockIdx.x;
    const int xcd = pid & 7, j = pid >> 3;
    const int grp = j / ksplit, split = j - grp * ksplit;
    const int unit = grp * 8 + xcd;
    if (unit >= units)
        return;
    DecodeProblem pr = one;
    int strip = unit;
    if (GROUPED) {
        const int g = unit / strips;
        strip = unit - g * strips;
        pr = DecodeProblem{tab->a[g], tab->b[g], tab->a_scale[g], tab->b_scale[g], tab->c[g], tab->m[g], tab->lda[g]};
    }
    const uint8_t* __restrict__ a = pr.a;
    const uint8_t* __restrict__ b = pr.b;
    const float* __restrict__ a_scale = pr.a_scale;
    const float* __restrict__ b_scale = pr.b_scale;
    uint16_t* __restrict__ c = pr.c;
    const int M = pr.M, lda = pr.lda;
    const int n0 = strip * BN;

    const int nkb = K / KBLOCK;
    const int kb0 = split * kb_per_split;
    const int kb1 = (kb0 + kb_per_split < nkb) ? (kb0 + kb_per_split) : nkb;
    const int sn = (N + KBLOCK - 1) / KBLOCK;
    const int mtiles = TILES > 0 ? TILES : (M + 15) >> 4;  // 1 .. MT

    // ---- copy plan.  B: instruction q (0, 1) of a wave fills stage rows 16*wave + 8*q + (lane >> 3), chunk
    // position lane & 7; the chunk swizzle (r >> 1) & 7 is (4*q + (lane >> 4)) & 7.  A, 32-byte rows: waves
    // 0..3, rows 32*wave + (lane >> 1), position lane & 1, swizzle (r >> 3) & 1 = (lane >> 4) & 1; 64-byte
    // rows: every wave, rows 16*wave + (lane >> 2), position lane & 3, swizzle (r >> 2) & 3 = (lane >> 4) & 3.
    const uint32_t a_bytes = (uint32_t)lda * (uint32_t)K, b_bytes = (uint32_t)N * (uint32_t)K;
    uint32_t voff_b[NB][2];  // per 128-column half of the strip
#pragma unroll
    for (int h = 0; h < NB; ++h)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int cc = (lane & 7) ^ ((4 * q + (lane >> 4)) & 7);
            const bool ok = n0 + DS_BN * h + 16 * cc < N;
            voff_b[h][q] = ok ? (uint32_t)((16 * wave + 8 * q + (lane >> 3)) * N + n0 + DS_BN * h + 16 * cc) : 0x80000000u;
        }
    const uint32_t voff_sa = lane < lda ? (uint32_t)(lane * 4) : 0x80000000u;
    const uint32_t voff_sb = lane < NB ? (uint32_t)((strip * NB + lane) * 4) : 0x80000000u;  // past the last block: zeros
    uint32_t voff_a;
    if (RAGGED) {
        // the K block's slab of A, 128 * M contiguous bytes, in 16-byte pieces: piece 64 * wave + lane
        const int piece = 64 * wave + lane;
        voff_a = 16 * piece < KBLOCK * lda ? (uint32_t)(16 * piece) : 0x80000000u;
    } else if (MT == 2) {
        const int cc = (lane & 1) ^ ((lane >> 4) & 1);
        voff_a = 16 * cc < lda ? (uint32_t)((32 * wave + (lane >> 1)) * lda + 16 * cc) : 0x80000000u;
    } else {
        const int cc = (lane & 3) ^ ((lane >> 4) & 3);
        voff_a = 16 * cc < lda ? (uint32_t)((16 * wave + (lane >> 2)) * lda + 16 * cc) : 0x80000000u;
    }

    // Stage `slot` <- K block kb.  The resources of A and B start at the block's first k-row.
    auto issue_stage = [&](int slot, int kb) __attribute__((always_inline)) {
        const uint32_t stage = lds_base + (uint32_t)(slot * S::STAGE);
        const uint32_t skip_b = (uint32_t)kb * KBLOCK * (uint32_t)N;
        const uint32_t skip_a = (uint32_t)kb * KBLOCK * (uint32_t)lda;
        const v4i rb = make_rsrc_words(b + skip_b, b_bytes - skip_b);
#pragma unroll
        for (int h = 0; h < NB; ++h) {
            lds_dma16(rb, voff_b[h][0], stage + (uint32_t)(h * S::HALF_B + (2 * wave) * 1024));
            lds_dma16(rb, voff_b[h][1], stage + (uint32_t)(h * S::HALF_B + (2 * wave + 1) * 1024));
        }
        const int scale_wave = MT == 2 ? wave - 4 : wave;  // 0: a_scale, 1..: b_scale, below 0: A (two row tiles)
        if (RAGGED) {
            // the slab of the K block after this one, into the next slot: it has landed with this stage, one
            // stage before it is multiplied, which is when the threads spread it
            if (MT == 4 || wave < 4) {
                const uint32_t next = lds_base + (uint32_t)((slot == DS_NS - 1 ? 0 : slot + 1) * S::STAGE);
                const uint32_t skip_next = skip_a + KBLOCK * (uint32_t)lda;
                lds_dma16(make_rsrc_words(a + skip_next, a_bytes - skip_next), kb + 1 < kb1 ? voff_a : 0x80000000u,
                          next + S::PACK_OFF + (uint32_t)(wave * 1024));
            }
        } else if (MT == 4 || wave < 4)
            lds_dma16(make_rsrc_words(a + skip_a, a_bytes - skip_a), voff_a, stage + S::MAT_B + (uint32_t)(wave * 1024));
        if (scale_wave == 0)
            lds_dma4(make_rsrc_words(a_scale + (size_t)kb * lda, (uint32_t)lda * 4u), voff_sa, stage + S::SA_OFF);
        else if (scale_wave > 0)
            lds_dma4(make_rsrc_words(b_scale + (size_t)kb * sn, (uint32_t)sn * 4u), voff_sb, stage + S::SB_OFF);
    };
    // RAGGED: thread 4 * r + j moves bytes 16 * j .. 16 * j + 15 of packed k-row r (they start at any byte:
    // five aligned words, shifted) to chunk j of the padded, swizzled row, zeros where the row has ended; only
    // the chunks of row tiles that exist are read by the MFMAs.  Every thread reads and writes, so that no branch
    // surrounds the LDS operations: a thread whose chunk belongs to no row tile reads what lies at its address
    // (inside the stage) and writes to the 16 spare bytes behind the slab.  Reading and writing are apart so that
    // the stage's other LDS reads sit between them.
    const int sp_r = (int)threadIdx.x >> 2, sp_j = (int)threadIdx.x & 3;
    const uint32_t sp_src = (uint32_t)(S::PACK_OFF + ((sp_r * lda + 16 * sp_j) & ~3));
    const uint32_t sp_shift = (uint32_t)((sp_r * lda) & 3);
    const uint32_t sp_dst =
        sp_j < mtiles
            ? (uint32_t)(S::MAT_B + sp_r * S::RSA + ((sp_j ^ (MT == 2 ? (sp_r >> 3) & 1 : (sp_r >> 2) & 3)) << 4))
            : (uint32_t)(S::PACK_OFF + S::MAT_A);
    uint32_t sp_mask[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int valid = M - 16 * sp_j - 4 * i;  // bytes of word i inside the row
        sp_mask[i] = valid >= 4 ? 0xFFFFFFFFu : valid <= 0 ? 0u : (1u << (8 * valid)) - 1u;
    }
    uint32_t sp_word[5];
    auto slab_read = [&](int sl) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 5; ++i)
            sp_word[i] = *LDS_PTR(uint32_t, lds + sl * S::STAGE + sp_src + 4 * i);
    };
    auto slab_write = [&](int sl) __attribute__((always_inline)) {
        v4i out;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            out[i] = (int)(__builtin_amdgcn_alignbyte(sp_word[i + 1], sp_word[i], sp_shift) & sp_mask[i]);
        *LDS_PTR(v4i, lds + sl * S::STAGE + sp_dst) = out;
    };
    // wait until at most the copies of `outstanding` stages are in flight (loads complete in order)
    auto wait_landed = [&](int outstanding) __attribute__((always_inline)) {
        switch (outstanding) {
        case 0: ds_wait_vmcnt<0>(); break;
        case 1: ds_wait_vmcnt<S::COPIES>(); break;
        case 2: ds_wait_vmcnt<2 * S::COPIES>(); break;
        case 3: ds_wait_vmcnt<3 * S::COPIES>(); break;
        case 4: ds_wait_vmcnt<4 * S::COPIES>(); break;
        default: ds_wait_vmcnt<(DS_NS - 1) * S::COPIES>(); break;
        }
    };

    // ---- transposing reads.  Lane = 16*g + i; read t of a K block covers k-rows 32*t + 8*g + (i >> 1),
    // so (r >> 1) & 7 = (4*g + (i >> 2)) & 7, (r >> 3) & 1 = g & 1 and (r >> 2) & 3 = (2*g + (i >> 3)) & 3
    // for every t.
    const int g4 = lane >> 4, i16 = lane & 15;
    const uint32_t addr_b = (uint32_t)((8 * g4 + (i16 >> 1)) * 128 + ((wave ^ ((4 * g4 + (i16 >> 2)) & 7)) * 16) +
                                       (i16 & 1) * 8);
    const uint32_t addr_a = (uint32_t)(S::MAT_B + (8 * g4 + (i16 >> 1)) * S::RSA + (i16 & 1) * 8);
    const int swz_a = MT == 2 ? (g4 & 1) : ((2 * g4 + (i16 >> 3)) & 3);
    auto read_frag = [&](uint32_t addr, int step) __attribute__((always_inline)) -> v8i {
        v2i r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr));
        v2i r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + step));
        v2i r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 2 * step));
        v2i r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 3 * step));
        return (v8i){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    };

    v4f acc[NB][MT];
#pragma unroll
    for (int h = 0; h < NB; ++h)
#pragma unroll
        for (int i = 0; i < MT; ++i)
            acc[h][i] = (v4f){0.f, 0.f, 0.f, 0.f};

    const int nstages = kb1 - kb0;
    if (RAGGED && (MT == 4 || wave < 4)) {  // the first K block's slab, ahead of every stage
        const uint32_t skip_a = (uint32_t)kb0 * KBLOCK * (uint32_t)lda;
        lds_dma16(make_rsrc_words(a + skip_a, a_bytes - skip_a), voff_a, lds_base + S::PACK_OFF + (uint32_t)(wave * 1024));
    }
#pragma unroll
    for (int p = 0; p < DS_NS - 1; ++p)
        if (p < nstages)
            issue_stage(p, kb0 + p);
    if (RAGGED) {  // the first slab has landed once only the stages' copies are in flight
        wait_landed(nstages < DS_NS - 1 ? nstages : DS_NS - 1);
        __syncthreads();
        slab_read(0);
        slab_write(0);
    }
    // The K loop, one copy per number of 16-row tiles (chosen below, outside the loop): with the count fixed
    // the loop has no branch around its LDS operations, every read of a stage is issued before the first MFMA,
    // and the compiler's wait counts name exactly the reads each MFMA needs (around a branch it waits for
    // everything in flight, which serialises read latency and MFMAs tile after tile).
    auto k_loop = [&](auto tile_count) __attribute__((always_inline)) {
    constexpr int T = decltype(tile_count)::value;
    int slot = 0;
    for (int s = 0; s < nstages; ++s) {
        // loads complete in order: this wave's copies of stage s have landed once at most those of the
        // younger stages in flight are outstanding
        wait_landed(nstages - 1 - s < DS_NS - 2 ? nstages - 1 - s : DS_NS - 2);
        __syncthreads();  // everyone's copies landed and spreads are done; the slot of stage s - 1 is no longer read
        if (s + DS_NS - 1 < nstages)
            issue_stage(slot == 0 ? DS_NS - 1 : slot - 1, kb0 + s + DS_NS - 1);
        const uint32_t so = (uint32_t)(slot * S::STAGE);
        const int next_slot = slot == DS_NS - 1 ? 0 : slot + 1;
        // RAGGED: the next stage's slab, also behind the last stage (nothing reads what that spreads)
        if (RAGGED)
            slab_read(next_slot);
        v8i fb[NB];
        float sb[NB];
#pragma unroll
        for (int h = 0; h < NB; ++h) {
            fb[h] = read_frag(so + h * S::HALF_B + addr_b, 32 * 128);
            sb[h] = *LDS_PTR(float, lds + so + S::SB_OFF + 4 * h);
        }
        auto multiply = [&](int h, int i, const v8i& fa, float sa) __attribute__((always_inline)) {
            const v4f blk = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb[h], fa, (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0,
                                                                             0, 0, 0, 0);
            const float sc = sa * sb[h];
            acc[h][i] = (v4f){fmaf(sc, blk[0], acc[h][i][0]), fmaf(sc, blk[1], acc[h][i][1]),
                              fmaf(sc, blk[2], acc[h][i][2]), fmaf(sc, blk[3], acc[h][i][3])};
        };
        // the spread words are written behind the stage's reads: the LDS works in order, a write among the
        // reads would hold the later ones back
        v8i fa[T];
        float sa[T];
#pragma unroll
        for (int i = 0; i < T; ++i) {
            sa[i] = *LDS_PTR(float, lds + so + S::SA_OFF + (16 * i + i16) * 4);
            fa[i] = read_frag(so + addr_a + (uint32_t)((i ^ swz_a) * 16), 32 * S::RSA);
        }
        if (RAGGED)
            slab_write(next_slot);
#pragma unroll
        for (int h = 0; h < NB; ++h)
#pragma unroll
            for (int i = 0; i < T; ++i)
                multiply(h, i, fa[i], sa[i]);
        slot = next_slot;
    }
    };
    if (TILES > 0)
        k_loop(std::integral_constant<int, (TILES > 0 ? TILES : 1)>{});
    else
    switch (mtiles) {
    case 1: k_loop(std::integral_constant<int, 1>{}); break;
    case 2: k_loop(std::integral_constant<int, 2>{}); break;
    case 3:
        if (MT == 4)
            k_loop(std::integral_constant<int, MT == 4 ? 3 : 1>{});
        break;
    default:
        if (MT == 4)
            k_loop(std::integral_constant<int, MT == 4 ? 4 : 1>{});
        break;
    }

    // ---- a lane holds C[16*i + (lane & 15)][n0 + 128*h + 16*wave + 4*(lane >> 4) + 0..3]
    auto store_c = [&](const v4f (&v)[NB][MT]) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < NB; ++h) {
            const int ncol = n0 + DS_BN * h + 16 * wave + 4 * g4;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const int mrow = 16 * i + i16;
                if (mrow < M && ncol < N) {
                    uint2 pk;
                    pk.x = pack_bf16x2(v[h][i][0], v[h][i][1]);
                    pk.y = pack_bf16x2(v[h][i][2], v[h][i][3]);
                    *reinterpret_cast<uint2*>(c + (size_t)mrow * N + ncol) = pk;
                }
            }
        }
    };
    if (ksplit == 1) {
        store_c(acc);
        return;
    }

    // ---- mailbox: [unit][split 0 .. ksplit-2][wave][half h][i][lane] x 16 bytes, all zero between launches
    constexpr int PER_WAVE = NB * MT;        // patches of one wave
    constexpr int PER_SPLIT = 8 * PER_WAVE;  // patches of one split of one unit
    const int senders = ksplit - 1;
    const size_t patch = ((size_t)unit * senders * 8 + wave) * PER_WAVE;  // split 0
    if (split < senders) {
        v4i* mine = reinterpret_cast<v4i*>(mailbox) + (patch + (size_t)split * PER_SPLIT) * 64 + lane;
#pragma unroll
        for (int h = 0; h < NB; ++h)
#pragma unroll
            for (int i = 0; i < MT; ++i)
                if (i < mtiles) {
                    v4i bits = __builtin_bit_cast(v4i, acc[h][i]);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        bits[e] = bits[e] == 0 ? (int)0x80000000 : bits[e];  // +0.0 -> -0.0: no word is zero
                    mine[64 * (h * MT + i)] = bits;
                }
        return;
    }
    // last split: wait for the other splits' patches of these 16 columns, four splits at a time
    const uint32_t span = (uint32_t)senders * PER_SPLIT * 64u * 16u;  // bytes from this wave's split-0 patch to past its last
    const __amdgpu_buffer_rsrc_t rp = make_rsrc(reinterpret_cast<const v4i*>(mailbox) + patch * 64, span);
    v4f sum[NB][MT];
#pragma unroll
    for (int h = 0; h < NB; ++h)
#pragma unroll
        for (int i = 0; i < MT; ++i)
            sum[h][i] = (v4f){0.f, 0.f, 0.f, 0.f};
    bool gave_up = false;
    const unsigned long long t_first = __builtin_amdgcn_s_memrealtime();
    for (int z0 = 0; z0 < senders; z0 += 4) {
#pragma unroll
        for (int hp = 0; hp < NB * (MT / 2); ++hp) {  // two row tiles of a half at a time
            const int hb = hp / (MT / 2), h = hp % (MT / 2);
            if (2 * h < mtiles) {
                v4i v[4][2];
                for (;;) {
                    asm volatile("" ::: "memory");  // the loads belong to this round of the loop
                    // a split past the last reads outside the resource, which fetches zeros
#pragma unroll
                    for (int z = 0; z < 4; ++z)
#pragma unroll
                        for (int i = 0; i < 2; ++i)
                            v[z][i] = __builtin_amdgcn_raw_buffer_load_b128(
                                rp, (uint32_t)(((z0 + z) * PER_SPLIT + hb * MT + 2 * h + i) * 64 + lane) * 16u, 0, AUX_L1_MISS);
                    bool missing = false;
#pragma unroll
                    for (int z = 0; z < 4; ++z)
#pragma unroll
                        for (int i = 0; i < 2; ++i)
                            if (z0 + z < senders && 2 * h + i < mtiles)
                                missing = missing || v[z][i][0] == 0 || v[z][i][1] == 0 || v[z][i][2] == 0 || v[z][i][3] == 0;
                    if (__builtin_amdgcn_ballot_w64(missing) == 0)
                        break;
                    if (__builtin_amdgcn_s_memrealtime() - t_first > SPIN_LIMIT_TICKS) {
                        gave_up = true;
                        break;
                    }
                }
#pragma unroll
                for (int z = 0; z < 4; ++z)
                    if (z0 + z < senders) {
#pragma unroll
                        for (int i = 0; i < 2; ++i) {
                            if (2 * h + i < mtiles)
                                __builtin_amdgcn_raw_buffer_store_b128(
                                    (v4i){0, 0, 0, 0}, rp,
                                    (uint32_t)(((z0 + z) * PER_SPLIT + hb * MT + 2 * h + i) * 64 + lane) * 16u, 0, 0);
                            const v4f f = __builtin_bit_cast(v4f, v[z][i]);
                            sum[hb][2 * h + i] = z0 + z == 0 ? f : sum[hb][2 * h + i] + f;
                        }
                    }
            }
        }
    }
#pragma unroll
    for (int h = 0; h < NB; ++h)
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            sum[h][i] = sum[h][i] + acc[h][i];
            if (gave_up)
                sum[h][i] = (v4f){__builtin_nanf(""), __builtin_nanf(""), __builtin_nanf(""), __builtin_nanf("")};
        }
    store_c(sum);
}

template <int MT, int DS_NS, bool RAGGED, int TILES, int NB>
__global__ void __launch_bounds__(DS_THREADS)
decode_strip_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b, const float* __restrict__ a_scale,
                    const float* __restrict__ b_scale, uint16_t* __restrict__ c, float* mailbox, int M, int lda, int N,
                    int K, int strips, int ksplit, int kb_per_split)
{
    const DecodeProblem one{a, b, a_scale, b_scale, c, M, lda};
    decode_body<MT, false, DS_NS, RAGGED, TILES, NB>(one, nullptr, mailbox, N, K, strips, strips, ksplit, kb_per_split);
}

template <int MT, int DS_NS, bool RAGGED>
__global__ void __launch_bounds__(DS_THREADS)
decode_strip_grouped_kernel(const GroupTable tab, float* mailbox, int N, int K, int strips, int ksplit, int kb_per_split)
{
    const DecodeProblem none{nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0};
    decode_body<MT, true, DS_NS, RAGGED, 0, 1>(none, &tab, mailbox, N, K, strips, strips * tab.groups, ksplit, kb_per_split);
}

// The streaming form, for a single problem without a K split whose strips outnumber the workgroups the
// device holds at once (N > 32768: the output projection onto a vocabulary): gridDim.x workgroups walk
// through the strips (workgroup w takes strips w, w + gridDim.x, ...) and the K blocks of all strips of a
// workgroup form ONE copy stream, so the first stages of the next strip are on their way while the current one
// is multiplied and stored, instead of every strip starting from an empty ring (M = 32, N = 65536, K = 2048:
// 23.4 against 26.3 us = 5.7 TB/s).  Same stages, same reads, same arithmetic per strip as decode_body:
// bit-identical results.  Grouped launches gain nothing from it (64 groups x 56 strips: 225 against 220 us)
// and keep the plain form.  (A strip's two stores per wave share the vmcnt counter with the copies and may
// complete after younger copies; counting them as outstanding copies only makes a wait longer, never shorter.)
// STAGED: a strip's C goes through the LDS (behind the ring) and leaves in whole rows, 16 bytes per lane, instead
// of 32 bytes of a row per wave straight from the accumulators (3 - 10 % on four row tiles, nothing on two: what
// C costs a long stream -- 15 % of the run time for 3 % of the bytes at 32 rows and K = 2048 -- is the price of
// writes to HBM among the reads, whatever their shape).  Needs c on a 16-byte boundary.
// GROUPED: units run through the strips of all problems of `tab` (TILES = 0: the tile count is the unit's own, and
// the stage's math is chosen by it -- one straight-line copy per count).
template <int MT, int DS_NS, int TILES, bool STAGED, int NB, bool GROUPED>
__device__ __forceinline__ void decode_stream_body(const DecodeProblem& one, const GroupTable* tab, int N, int K, int strips,
                                                   int units)
{
    using S = DecodeShape<MT, DS_NS, false, NB>;
    constexpr int BN = DS_BN * NB;                 // columns of a strip
    constexpr int C_STAGE_ROW = 2 * BN + 16;       // bytes per staged row of C (16 more than the data: rows 4 banks apart)
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    auto lds = LDS_PTR(uint8_t, smem);
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int G = (int)gridDim.x, w = (int)blockIdx.x;
    if (w >= units)
        return;
    const int nkb = K / KBLOCK;
    const int sn = (N + KBLOCK - 1) / KBLOCK;
    const int total = ((units - w + G - 1) / G) * nkb;  // stages of this workgroup's stream

    auto problem_of = [&](int unit, int* strip) __attribute__((always_inline)) -> DecodeProblem {
        if (!GROUPED) {
            *strip = unit;
            return one;
        }
        const int g = unit / strips;
        *strip = unit - g * strips;
        return DecodeProblem{tab->a[g], tab->b[g], tab->a_scale[g], tab->b_scale[g], tab->c[g], tab->m[g], tab->lda[g]};
    };
    // ---- copy side: what the strip being copied needs (see decode_body for the plan)
    DecodeProblem cp = one;
    int cp_strip = 0;
    uint32_t voff_b[NB][2], voff_a = 0, voff_sa = 0, voff_sb = 0;
    auto enter_copy_unit = [&](int unit) __attribute__((always_inline)) {
        cp = problem_of(unit, &cp_strip);
#pragma unroll
        for (int h = 0; h < NB; ++h) {
            const int n0 = cp_strip * BN + DS_BN * h;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int cc = (lane & 7) ^ ((4 * q + (lane >> 4)) & 7);
                const bool ok = n0 + 16 * cc < N;
                voff_b[h][q] = ok ? (uint32_t)((16 * wave + 8 * q + (lane >> 3)) * N + n0 + 16 * cc) : 0x80000000u;
            }
        }
        voff_sa = lane < cp.lda ? (uint32_t)(lane * 4) : 0x80000000u;
        voff_sb = lane < NB ? (uint32_t)((cp_strip * NB + lane) * 4) : 0x80000000u;  // past the last block: zeros
        if (MT == 2) {
            const int cc = (lane & 1) ^ ((lane >> 4) & 1);
            voff_a = 16 * cc < cp.lda ? (uint32_t)((32 * wave + (lane >> 1)) * cp.lda + 16 * cc) : 0x80000000u;
        } else {
            const int cc = (lane & 3) ^ ((lane >> 4) & 3);
            voff_a = 16 * cc < cp.lda ? (uint32_t)((16 * wave + (lane >> 2)) * cp.lda + 16 * cc) : 0x80000000u;
        }
    };
    auto issue_stage = [&](int slot, int kb) __attribute__((always_inline)) {
        const uint32_t a_bytes = (uint32_t)cp.lda * (uint32_t)K, b_bytes = (uint32_t)N * (uint32_t)K;
        const uint32_t stage = lds_base + (uint32_t)(slot * S::STAGE);
        const uint32_t skip_b = (uint32_t)kb * KBLOCK * (uint32_t)N;
        const uint32_t skip_a = (uint32_t)kb * KBLOCK * (uint32_t)cp.lda;
        const v4i rb = make_rsrc_words(cp.b + skip_b, b_bytes - skip_b);
#pragma unroll
        for (int h = 0; h < NB; ++h) {
            lds_dma16(rb, voff_b[h][0], stage + (uint32_t)(h * S::HALF_B + (2 * wave) * 1024));
            lds_dma16(rb, voff_b[h][1], stage + (uint32_t)(h * S::HALF_B + (2 * wave + 1) * 1024));
        }
        const int scale_wave = MT == 2 ? wave - 4 : wave;
        if (MT == 4 || wave < 4)
            lds_dma16(make_rsrc_words(cp.a + skip_a, a_bytes - skip_a), voff_a, stage + S::MAT_B + (uint32_t)(wave * 1024));
        if (scale_wave == 0)
            lds_dma4(make_rsrc_words(cp.a_scale + (size_t)kb * cp.lda, (uint32_t)cp.lda * 4u), voff_sa, stage + S::SA_OFF);
        else if (scale_wave > 0)
            lds_dma4(make_rsrc_words(cp.b_scale + (size_t)kb * sn, (uint32_t)sn * 4u), voff_sb, stage + S::SB_OFF);
    };
    int cp_kb = 0, cp_unit = w, cp_slot = 0, issued = 0;
    auto issue_next = [&]() __attribute__((always_inline)) {
        if (issued >= total)
            return;
        if (cp_kb == 0)
            enter_copy_unit(cp_unit);
        issue_stage(cp_slot, cp_kb);
        ++issued;
        cp_slot = cp_slot == DS_NS - 1 ? 0 : cp_slot + 1;
        if (++cp_kb == nkb) {
            cp_kb = 0;
            cp_unit += G;
        }
    };

    // ---- multiply side
    const int g4 = lane >> 4, i16 = lane & 15;
    const uint32_t addr_b = (uint32_t)((8 * g4 + (i16 >> 1)) * 128 + ((wave ^ ((4 * g4 + (i16 >> 2)) & 7)) * 16) +
                                       (i16 & 1) * 8);
    const uint32_t addr_a = (uint32_t)(S::MAT_B + (8 * g4 + (i16 >> 1)) * S::RSA + (i16 & 1) * 8);
    const int swz_a = MT == 2 ? (g4 & 1) : ((2 * g4 + (i16 >> 3)) & 3);
    auto read_frag = [&](uint32_t addr, int step) __attribute__((always_inline)) -> v8i {
        v2i r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr));
        v2i r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + step));
        v2i r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 2 * step));
        v2i r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 3 * step));
        return (v8i){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    };
    v4f acc[NB][MT];
    DecodeProblem mp = one;
    int mp_strip = 0, mp_tiles = TILES;

#pragma unroll
    for (int p = 0; p < DS_NS - 1; ++p)
        issue_next();
    int slot = 0, kb = 0, unit = w;
    for (int t = 0; t < total; ++t) {
        const int younger = total - 1 - t < DS_NS - 2 ? total - 1 - t : DS_NS - 2;
        switch (younger) {
        case 0: ds_wait_vmcnt<0>(); break;
        case 1: ds_wait_vmcnt<S::COPIES>(); break;
        case 2: ds_wait_vmcnt<2 * S::COPIES>(); break;
        case 3: ds_wait_vmcnt<3 * S::COPIES>(); break;
        default: ds_wait_vmcnt<4 * S::COPIES>(); break;
        }
        __syncthreads();  // everyone's copies of stage t landed; the slot of stage t - 1 is no longer read
        issue_next();     // stage t + DS_NS - 1 goes into the slot of stage t - 1
        if (kb == 0) {
            mp = problem_of(unit, &mp_strip);
            if (TILES == 0)
                mp_tiles = (mp.M + 15) >> 4;
#pragma unroll
            for (int h = 0; h < NB; ++h)
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    acc[h][i] = (v4f){0.f, 0.f, 0.f, 0.f};
        }
        const uint32_t so = (uint32_t)(slot * S::STAGE);
        // T 16-row tiles: every read of the stage is issued before the first MFMA, no branch among them
        auto stage_math = [&](auto tile_count) __attribute__((always_inline)) {
            constexpr int T = decltype(tile_count)::value;
            v8i fb[NB], fa[T];
            float sb[NB], sa[T];
#pragma unroll
            for (int h = 0; h < NB; ++h) {
                fb[h] = read_frag(so + h * S::HALF_B + addr_b, 32 * 128);
                sb[h] = *LDS_PTR(float, lds + so + S::SB_OFF + 4 * h);
            }
#pragma unroll
            for (int i = 0; i < T; ++i) {
                sa[i] = *LDS_PTR(float, lds + so + S::SA_OFF + (16 * i + i16) * 4);
                fa[i] = read_frag(so + addr_a + (uint32_t)((i ^ swz_a) * 16), 32 * S::RSA);
            }
#pragma unroll
            for (int h = 0; h < NB; ++h)
#pragma unroll
                for (int i = 0; i < T; ++i) {
                    const v4f blk = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        fb[h], fa[i], (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                    const float sc = sa[i] * sb[h];
                    acc[h][i] = (v4f){fmaf(sc, blk[0], acc[h][i][0]), fmaf(sc, blk[1], acc[h][i][1]),
                                      fmaf(sc, blk[2], acc[h][i][2]), fmaf(sc, blk[3], acc[h][i][3])};
                }
        };
        if (TILES > 0)
            stage_math(std::integral_constant<int, (TILES > 0 ? TILES : 1)>{});
        else
            switch (mp_tiles) {
            case 1: stage_math(std::integral_constant<int, 1>{}); break;
            case 2: stage_math(std::integral_constant<int, 2>{}); break;
            case 3: stage_math(std::integral_constant<int, (MT == 4 ? 3 : 1)>{}); break;
            default: stage_math(std::integral_constant<int, (MT == 4 ? 4 : 1)>{}); break;
            }
        slot = slot == DS_NS - 1 ? 0 : slot + 1;
        if (++kb == nkb) {
            // a lane holds C[16*i + (lane & 15)][n0 + 128*h + 16*wave + 4*(lane >> 4) + 0..3]
            if (STAGED) {
                const uint32_t cbase = (uint32_t)(DS_NS * S::STAGE);
#pragma unroll
                for (int h = 0; h < NB; ++h)
#pragma unroll
                    for (int i = 0; i < (TILES > 0 ? TILES : MT); ++i)
                        if (TILES > 0 || i < mp_tiles)
                            *LDS_PTR(v2i, lds + cbase + (16 * i + i16) * C_STAGE_ROW + (DS_BN * h + 16 * wave + 4 * g4) * 2) =
                                (v2i){(int)pack_bf16x2(acc[h][i][0], acc[h][i][1]),
                                      (int)pack_bf16x2(acc[h][i][2], acc[h][i][3])};
                __syncthreads();  // (the next write to this area lies behind the next stage's barrier)
                constexpr int CPR = BN / 8;  // 16-byte chunks per row
                const int staged_rows = 16 * (TILES > 0 ? TILES : mp_tiles);
                for (int idx = (int)threadIdx.x; idx < staged_rows * CPR; idx += DS_THREADS) {
                    const int row = idx / CPR, ch = idx % CPR;
                    const int ncol = mp_strip * BN + 8 * ch;
                    if (row < mp.M && ncol < N)
                        *reinterpret_cast<v4i*>(mp.c + (size_t)row * N + ncol) =
                            *LDS_PTR(v4i, lds + cbase + row * C_STAGE_ROW + 16 * ch);
                }
            } else {
#pragma unroll
                for (int h = 0; h < NB; ++h) {
                    const int ncol = mp_strip * BN + DS_BN * h + 16 * wave + 4 * g4;
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        const int mrow = 16 * i + i16;
                        if (mrow < mp.M && ncol < N) {
                            uint2 pk;
                            pk.x = pack_bf16x2(acc[h][i][0], acc[h][i][1]);
                            pk.y = pack_bf16x2(acc[h][i][2], acc[h][i][3]);
                            *reinterpret_cast<uint2*>(mp.c + (size_t)mrow * N + ncol) = pk;
                        }
                    }
                }
            }
            kb = 0;
            unit += G;
        }
    }
}

template <int MT, int DS_NS, bool STAGED, int NB>
__global__ void __launch_bounds__(DS_THREADS)
decode_stream_grouped_kernel(const GroupTable tab, int N, int K, int strips, int units)
{
    const DecodeProblem none{};
    decode_stream_body<MT, DS_NS, 0, STAGED, NB, true>(none, &tab, N, K, strips, units);
}

template <int MT, int DS_NS, int TILES, bool STAGED, int NB>
__global__ void __launch_bounds__(DS_THREADS)
decode_stream_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b, const float* __restrict__ a_scale,
                     const float* __restrict__ b_scale, uint16_t* __restrict__ c, int M, int lda, int N, int K,
                     int strips)
{
    const DecodeProblem one{a, b, a_scale, b_scale, c, M, lda};
    decode_stream_body<MT, DS_NS, TILES, STAGED, NB, false>(one, nullptr, N, K, strips, strips);
}

// records the XCC (XCD) id each workgroup of a probe grid runs on
constexpr int XCC_PROBE = 256;
static __device__ unsigned int xcc_probe_out[XCC_PROBE];

__global__ void xcc_probe_kernel(unsigned int* out)
{
    unsigned int x;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(x));
    if (threadIdx.x == 0)
        out[blockIdx.x] = x & 0xFu;
}

inline int row_tiles(int m) { return m <= 32 ? 2 : 4; }

// the streaming form: ring depth and workgroups (one per CU; six stages, five beside four staged row tiles of C)
constexpr int STREAM_NS = 6;
constexpr int STREAM_NS4 = 5;
constexpr int STREAM_NS_WIDE = 3;  // 256-column strips: 32 KB of B per stage
constexpr long GROUPED_STREAM_MIN_UNITS = 256;  // grouped launches: 256-column strips of all groups for the streaming form
template <int MT_, int NS_, int NB_>
struct StreamShape {
    static constexpr int MT = MT_, NS = NS_, NB = NB_;
};
constexpr int STREAM_WORKGROUPS = 256;
constexpr int SLAB_FORM_MIN_KBLOCKS = 28;  // K blocks per workgroup from which up to 32 rows on the grid take the slab-spreading instances too

// Two workgroups per CU with a three-stage ring instead of one with six: one streams while the other starts up.
// Measured on grouped launches: 64 groups x 56 strips, 16 K blocks each: 221 against 236 us; with 768-1152
// workgroups (1.5-2.25 rounds of 512 resident ones) 1-3 % slower than three to four and a half rounds of 256.
inline bool shallow_ring_pays(long workgroups, int kb_per_split) { return workgroups >= 2048 && kb_per_split >= 6; }

}  // namespace

// any 1 <= m <= 64: a row count off the 16-byte grid runs the kernels that spread A's packed slabs in the LDS;
// a and a_scale may have more elements per k-row than c has rows (lda: a multiple of 16, at most 64 -- padded
// copies whose c is written in place)
bool decode_strip_supports(const GemmArgs& g)
{
    return g.m >= 1 && g.m <= 64 && g.n % 16 == 0 &&
           (g.lda == 0 || g.lda == g.m || (g.lda > g.m && g.lda <= 64 && g.lda % 16 == 0)) &&
           (reinterpret_cast<uintptr_t>(g.a) % 16 == 0) && (reinterpret_cast<uintptr_t>(g.b) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.a_scale) % 4 == 0) && (reinterpret_cast<uintptr_t>(g.b_scale) % 4 == 0) &&
           (reinterpret_cast<uintptr_t>(g.c) % 8 == 0);
}

// the mailbox of a K split: one patch per strip, sending split, wave and row tile
bool decode_strip_can_split(const GemmArgs& g, int ksplit, int halves)
{
    return decode_strip_mailbox_bytes(g, ksplit, halves) <= SPLIT_MAILBOX_BYTES;
}

size_t decode_strip_mailbox_bytes(const GemmArgs& g, int ksplit, int halves)
{
    if (ksplit <= 1)
        return 0;
    const size_t strips = (size_t)(g.n + DS_BN * halves - 1) / (DS_BN * halves);
    return strips * (size_t)(ksplit - 1) * 8 * halves * row_tiles(g.m) * 64 * 16;
}
// Microseconds with B streamed from HBM, fitted to M = 16 and 32, N = 1536 ... 16384, K = 1536 ... 7168 and
// 1 to 16 K splits: a launch, then rounds of 256 workgroups, each workgroup living for a start-up, its
// K blocks (0.5 us per block when few workgroups pull on HBM, 0.76 us when 256 do) and, when K is split,
// the in-kernel reduction, whose last split reads one partial patch per other split.
double decode_strip_cost(const GemmArgs& g, int ksplit, int halves)
{
    const int strips = (g.n + DS_BN * halves - 1) / (DS_BN * halves);
    const int nkb = g.k / KBLOCK;
    const int kbs = (nkb + ksplit - 1) / ksplit;
    // An unsplit launch of more strips than the device holds workgroups: 256 workgroups at a time take the strips
    // in turn (the streaming form, which makes them 256 columns wide once there are 256 such strips; with rows off
    // the 16-byte grid the plain kernel's workgroups as CUs free up), a full turn at what HBM delivers (1.33 us
    // per K block of 256-column strips, 0.756 us of 128-column ones), the last, partial turn like a launch of
    // that many workgroups.  (16 x 65792 / 81920 / 98304 x 2048: 32.8 / 36.1 / 39.4 us estimated, 31.2 / 38.7 /
    // 41.2 us measured; 8 x 131072 x 4096: 88.6, 92.9 us; 8 x 163840 x 2048 in 256-column strips 60.6, 64.9 us, in
    // 128-column strips 64.0, 72.6 us.)
    if (ksplit == 1 && strips > STREAM_WORKGROUPS) {
        const long wide_units = (g.n + 2 * DS_BN - 1) / (2 * DS_BN);
        const bool wide = halves == 2 || (leading_dim(g) % 16 == 0 && wide_units >= STREAM_WORKGROUPS);
        const long units = wide ? wide_units : strips;
        const long turns = units / STREAM_WORKGROUPS, tail = units % STREAM_WORKGROUPS;
        return 3.5 + kbs * (turns * (wide ? 1.33 : 0.756) + (tail ? 0.50 + (wide ? 0.0032 : 0.001) * tail : 0.0));
    }
    const long wgs = (long)strips * ksplit;
    // the splits of a strip share an XCD (32 CUs, one workgroup each), strips are dealt out over the eight XCDs:
    // 36 strips x 7 splits are 252 workgroups, but 35 on each of four XCDs, which is two rounds there (measured:
    // 19.8 us against 14.0 us with 6 splits for 4608 x 7168)
    const long rounds = ((long)((strips + 7) / 8) * ksplit + 31) / 32;
    const double active = wgs < 256 ? (double)wgs : 256.0;
    // (a stage of a 256-column strip is twice the bytes for 1.92 times the time in a launch of one round, which
    // lives on latencies, and for 1.8 times in longer unsplit ones, which stream: 256 contiguous bytes come 10 %
    // faster)
    double per_block = (0.50 + 0.001 * active) * (halves == 2 ? (rounds > 1 && ksplit == 1 ? 1.8 : 1.92) : 1.0);
    // (one round of unsplit 256-column strips streams its whole K range and is bound by what HBM delivers to all
    // of them: 0.81 / 0.99 / 1.06 / 1.22 us per block with 129 / 160 / 192 / 224 workgroups -- 33024 ... 57344
    // columns, K = 2048 and 8192 -- which is 5.1 ... 5.9 TB/s)
    if (halves == 2 && ksplit == 1 && rounds == 1)
        per_block = 0.50 + 0.0032 * active;
    const double life = 1.0 + kbs * per_block + (ksplit > 1 ? 0.39 * ksplit : 0.0);
    return 2.5 + (double)rounds * life;
}

// Workgroups whose linear ids agree modulo 8 run on one XCD when the dispatcher deals workgroups out
// round-robin; the in-kernel reduction of K splits relies on it.  Looked at once per device: a probe
// grid records the XCC id of every workgroup into an array of the library's device image, and the call
// waits for it (may_probe = false, e.g. under stream capture: only a result already known is returned).
int xcd_placement_confirmed(bool may_probe)
{
    constexpr int MAX_DEVICES = 64;
    static std::mutex mutex;
    static signed char known[MAX_DEVICES] = {};  // 0 = not looked at, 1 = confirmed, -1 = not round-robin
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
        return 0;
    std::lock_guard<std::mutex> lock(mutex);
    if (known[dev] != 0)
        return known[dev] > 0;
    if (!may_probe)
        return -1;
    unsigned int* out = nullptr;
    unsigned int h[XCC_PROBE];
    bool ok = hipGetSymbolAddress(reinterpret_cast<void**>(&out), HIP_SYMBOL(xcc_probe_out)) == hipSuccess;
    for (int rep = 0; rep < 2 && ok; ++rep) {
        hipLaunchKernelGGL(xcc_probe_kernel, dim3(XCC_PROBE), dim3(64), 0, nullptr, out);
        ok = hipMemcpy(h, out, sizeof(h), hipMemcpyDeviceToHost) == hipSuccess;
        for (int i = 8; i < XCC_PROBE && ok; ++i)
            ok = h[i] == h[i & 7];
    }
    known[dev] = ok ? 1 : -1;
    return ok;
}

hipError_t launch_decode_strips(const GemmArgs& g, int ksplit, int halves, float* mailbox, hipStream_t s)
{
    if (halves != 1 && halves != 2)
        return hipErrorInvalidValue;
    const int strips = (g.n + DS_BN * halves - 1) / (DS_BN * halves);
    const int nkb = g.k / KBLOCK;
    if (!decode_strip_supports(g) || ksplit < 1 || ksplit > nkb || ksplit > DECODE_MAX_KSPLIT ||
        (ksplit > 1 && (!mailbox || !decode_strip_can_split(g, ksplit, halves))))
        return hipErrorInvalidValue;
    const int kb_per_split = (nkb + ksplit - 1) / ksplit;
    if ((ksplit - 1) * kb_per_split >= nkb)  // every split owns at least one K block
        return hipErrorInvalidValue;
    const dim3 grid(8 * ((strips + 7) / 8) * ksplit);
    auto go = [&](auto kern, int lds) -> hipError_t {
        FP8GEMM_ALLOW_LDS(kern, lds);
        hipLaunchKernelGGL(kern, grid, dim3(DS_THREADS), lds, s, g.a, g.b, g.a_scale, g.b_scale, g.c, mailbox, g.m,
                           leading_dim(g), g.n, g.k, strips, ksplit, kb_per_split);
        return hipGetLastError();
    };
    // more strips than resident workgroups, no K split: one copy stream per workgroup (the streaming form chooses
    // its strip width itself).  Strips of the width asked for: 57344 columns are 448 strips of 128 -- two turns of
    // the streaming workgroups, the second three quarters full, 96.9 us for 16 x 57344 x 8192 -- but 224 strips of
    // 256, one round of plain workgroups, 80.8 us.
    const int strips128 = (g.n + DS_BN - 1) / DS_BN;
    if (ksplit == 1 && strips > STREAM_WORKGROUPS && leading_dim(g) % 16 == 0) {
        const bool staged = reinterpret_cast<uintptr_t>(g.c) % 16 == 0;
        const int wide_units = (g.n + 2 * DS_BN - 1) / (2 * DS_BN);
        const bool wide = wide_units >= STREAM_WORKGROUPS;  // 256-column strips while every CU gets one
        const int units = wide ? wide_units : strips128;
        auto stream = [&](auto shape, auto tiles_c, auto staged_c) -> hipError_t {
            constexpr int MT = decltype(shape)::MT, NS = decltype(shape)::NS, NB = decltype(shape)::NB;
            constexpr int T = decltype(tiles_c)::value;
            constexpr bool ST = decltype(staged_c)::value;
            constexpr int lds = DecodeShape<MT, NS, false, NB>::LDS + (ST ? 16 * T * (2 * DS_BN * NB + 16) : 0);
            static_assert(lds <= 160 * 1024, "ring and staged C exceed the LDS");
            auto kern = decode_stream_kernel<MT, NS, T, ST, NB>;
            FP8GEMM_ALLOW_LDS(kern, lds);
            hipLaunchKernelGGL(kern, dim3(STREAM_WORKGROUPS), dim3(DS_THREADS), lds, s, g.a, g.b, g.a_scale, g.b_scale, g.c,
                               g.m, leading_dim(g), g.n, g.k, units);
            return hipGetLastError();
        };
        auto by_staging = [&](auto shape, auto tiles_c) -> hipError_t {
            return staged ? stream(shape, tiles_c, std::true_type{}) : stream(shape, tiles_c, std::false_type{});
        };
        auto by_tiles = [&](auto shape2, auto shape4) -> hipError_t {
            switch ((g.m + 15) / 16) {
            case 1: return by_staging(shape2, std::integral_constant<int, 1>{});
            case 2: return by_staging(shape2, std::integral_constant<int, 2>{});
            case 3: return by_staging(shape4, std::integral_constant<int, 3>{});
            default: return by_staging(shape4, std::integral_constant<int, 4>{});
            }
        };
        return wide ? by_tiles(StreamShape<2, STREAM_NS_WIDE, 2>{}, StreamShape<4, STREAM_NS_WIDE, 2>{})
                    : by_tiles(StreamShape<2, STREAM_NS, 1>{}, StreamShape<4, STREAM_NS4, 1>{});
    }
    if (halves == 2) {  // 256-column strips: three stages of 32 KB of B
        const int tiles = (g.m + 15) / 16;
        auto wide = [&](auto mt_c, auto ragged_c, auto tiles_c) -> hipError_t {
            constexpr int MT = decltype(mt_c)::value, T = decltype(tiles_c)::value;
            constexpr bool RG = decltype(ragged_c)::value;
            return go(decode_strip_kernel<MT, STREAM_NS_WIDE, RG, T, 2>, DecodeShape<MT, STREAM_NS_WIDE, RG, 2>::LDS);
        };
        auto by_tiles = [&](auto ragged_c) -> hipError_t {
            switch (tiles) {
            case 1: return wide(std::integral_constant<int, 2>{}, ragged_c, std::integral_constant<int, 1>{});
            case 2: return wide(std::integral_constant<int, 2>{}, ragged_c, std::integral_constant<int, 2>{});
            case 3: return wide(std::integral_constant<int, 4>{}, ragged_c, std::integral_constant<int, 3>{});
            default: return wide(std::integral_constant<int, 4>{}, ragged_c, std::integral_constant<int, 4>{});
            }
        };
        return leading_dim(g) % 16 != 0 ? by_tiles(std::true_type{}) : by_tiles(std::false_type{});
    }
    const int tiles = (g.m + 15) / 16;
    // The instances that spread A's packed slabs take rows on the grid as well, and a workgroup with a long K
    // range runs 3 - 8 % faster in them (28672 x 8192 unsplit, 15 / 16 / 31 / 32 rows: 43.2 / 45.8 / 45.1 / 47.1 us;
    // 16384 x 7168 in two splits, 47 / 48 rows: 26.3 / 27.8 us), a short one 3 - 10 % slower (24576 x 2048 unsplit,
    // 31 / 32 rows: 14.4 / 13.9 us; 7168 x 2048 in four splits: 8.0 / 7.3 us).  With three or four row tiles the
    // two measure level (their slab form has a ring of four stages, not six).
    if (leading_dim(g) % 16 != 0 || (kb_per_split >= SLAB_FORM_MIN_KBLOCKS && tiles <= 2)) {
        constexpr int L2 = DecodeShape<2, 6, true>::LDS, L4 = DecodeShape<4, RAGGED4_NS, true>::LDS;
        switch (tiles) {
        case 1: return go(decode_strip_kernel<2, 6, true, 1, 1>, L2);
        case 2: return go(decode_strip_kernel<2, 6, true, 2, 1>, L2);
        case 3: return go(decode_strip_kernel<4, RAGGED4_NS, true, 3, 1>, L4);
        default: return go(decode_strip_kernel<4, RAGGED4_NS, true, 4, 1>, L4);
        }
    }
    const bool deep = !shallow_ring_pays((long)strips * ksplit, kb_per_split);
    constexpr int D2 = DecodeShape<2, 6>::LDS, S2 = DecodeShape<2, 3>::LDS, D4 = DecodeShape<4, 6>::LDS,
                  S4 = DecodeShape<4, 3>::LDS;
    switch (tiles) {
    case 1: return deep ? go(decode_strip_kernel<2, 6, false, 1, 1>, D2) : go(decode_strip_kernel<2, 3, false, 1, 1>, S2);
    case 2: return deep ? go(decode_strip_kernel<2, 6, false, 2, 1>, D2) : go(decode_strip_kernel<2, 3, false, 2, 1>, S2);
    case 3: return deep ? go(decode_strip_kernel<4, 6, false, 3, 1>, D4) : go(decode_strip_kernel<4, 3, false, 3, 1>, S4);
    default: return deep ? go(decode_strip_kernel<4, 6, false, 4, 1>, D4) : go(decode_strip_kernel<4, 3, false, 4, 1>, S4);
    }
}

// every group: 1 <= m <= lda <= 64 (rows m .. lda-1 of a and a_scale readable), operands aligned like a
// single problem's; one lda off the 16-byte grid sends the whole launch to the slab-spreading kernels
bool decode_grouped_supports(const GroupTable& tab, int n, int k)
{
    if (tab.groups < 1 || tab.groups > GroupTable::MAX_GROUPS || k % KBLOCK != 0)
        return false;
    for (int g = 0; g < tab.groups; ++g) {
        const GemmArgs ga{tab.a[g], tab.b[g], tab.a_scale[g], tab.b_scale[g], tab.c[g], tab.lda[g], n, k};
        if (tab.m[g] <= 0 || tab.m[g] > tab.lda[g] || !decode_strip_supports(ga))
            return false;
    }
    return true;
}

size_t decode_grouped_mailbox_bytes(const GroupTable& tab, int n, int ksplit)
{
    if (ksplit <= 1)
        return 0;
    int mmax = 0;
    for (int g = 0; g < tab.groups; ++g)
        mmax = tab.lda[g] > mmax ? tab.lda[g] : mmax;
    const size_t units = (size_t)tab.groups * ((n + DS_BN - 1) / DS_BN);
    return units * (size_t)(ksplit - 1) * 8 * row_tiles(mmax) * 64 * 16;
}

// the K split for a grouped launch: what the cost model picks for one problem with all the groups' strips
// among the splits whose patches fit the mailbox; 1 when the in-kernel reduction cannot be used
int decode_grouped_ksplit(const GroupTable& tab, int n, int k, bool fused_ok)
{
    const int strips = (n + DS_BN - 1) / DS_BN, nkb = k / KBLOCK;
    const long units = (long)strips * tab.groups;
    if (!fused_ok || units * DS_BN > 0x7FFFFFFFl)
        return 1;
    GemmArgs all{tab.a[0], tab.b[0], tab.a_scale[0], tab.b_scale[0], tab.c[0], 32, (int)(units * DS_BN), k};
    int best = 1;
    double best_cost = decode_strip_cost(all, 1);
    for (int ks = 2; ks <= DECODE_MAX_KSPLIT && ks <= nkb; ++ks) {
        if ((ks - 1) * ((nkb + ks - 1) / ks) >= nkb || decode_grouped_mailbox_bytes(tab, n, ks) > SPLIT_MAILBOX_BYTES)
            continue;
        const double cst = decode_strip_cost(all, ks);
        if (cst < best_cost) {
            best_cost = cst;
            best = ks;
        }
    }
    return best;
}

// Whether a grouped launch of this many groups is one for the streaming form with 256-column strips: 256
// workgroups take the units in turn, which pays while the last turn is not too empty (288 units are two turns for
// 56 % of the work of two: 145 us against 121 us for 16 x (4608 x 7168); 448 units: 44 against 49 us).
bool decode_grouped_streams(int groups, int n)
{
    const long wide_units = (long)((n + 2 * DS_BN - 1) / (2 * DS_BN)) * groups;
    const long turns = (wide_units + STREAM_WORKGROUPS - 1) / STREAM_WORKGROUPS;
    return wide_units >= GROUPED_STREAM_MIN_UNITS && 5 * wide_units >= 4 * turns * STREAM_WORKGROUPS;
}

hipError_t launch_decode_grouped(const GroupTable& tab, int n, int k, int ksplit, float* mailbox, hipStream_t s)
{
    const int strips = (n + DS_BN - 1) / DS_BN;
    const int nkb = k / KBLOCK;
    const long units = (long)strips * tab.groups;
    if (!decode_grouped_supports(tab, n, k) || ksplit < 1 || ksplit > nkb || ksplit > DECODE_MAX_KSPLIT ||
        units > 0x0FFFFFFF / DECODE_MAX_KSPLIT ||
        (ksplit > 1 && (!mailbox || decode_grouped_mailbox_bytes(tab, n, ksplit) > SPLIT_MAILBOX_BYTES)))
        return hipErrorInvalidValue;
    const int kb_per_split = (nkb + ksplit - 1) / ksplit;
    if ((ksplit - 1) * kb_per_split >= nkb)
        return hipErrorInvalidValue;
    int mmax = 0;
    bool ragged = false;
    for (int g = 0; g < tab.groups; ++g) {
        mmax = tab.lda[g] > mmax ? tab.lda[g] : mmax;
        ragged |= tab.lda[g] % 16 != 0;
    }
    // many strips, rows on the 16-byte grid, no K split: the streaming form with 256-column strips
    const int wide_strips = (n + 2 * DS_BN - 1) / (2 * DS_BN);
    const long wide_units = (long)wide_strips * tab.groups;
    if (ksplit == 1 && !ragged && decode_grouped_streams(tab.groups, n)) {
        bool staged = true;
        for (int g = 0; g < tab.groups; ++g)
            staged = staged && reinterpret_cast<uintptr_t>(tab.c[g]) % 16 == 0;
        auto stream = [&](auto shape, auto staged_c) -> hipError_t {
            constexpr int MT = decltype(shape)::MT, NS = decltype(shape)::NS, NB = decltype(shape)::NB;
            constexpr bool ST = decltype(staged_c)::value;
            constexpr int lds = DecodeShape<MT, NS, false, NB>::LDS + (ST ? 16 * MT * (2 * DS_BN * NB + 16) : 0);
            static_assert(lds <= 160 * 1024, "ring and staged C exceed the LDS");
            auto kern = decode_stream_grouped_kernel<MT, NS, ST, NB>;
            FP8GEMM_ALLOW_LDS(kern, lds);
            hipLaunchKernelGGL(kern, dim3(STREAM_WORKGROUPS), dim3(DS_THREADS), lds, s, tab, n, k, wide_strips,
                               (int)wide_units);
            return hipGetLastError();
        };
        if (row_tiles(mmax) == 2)
            return staged ? stream(StreamShape<2, STREAM_NS_WIDE, 2>{}, std::true_type{})
                          : stream(StreamShape<2, STREAM_NS_WIDE, 2>{}, std::false_type{});
        return staged ? stream(StreamShape<4, STREAM_NS_WIDE, 2>{}, std::true_type{})
                      : stream(StreamShape<4, STREAM_NS_WIDE, 2>{}, std::false_type{});
    }
    const dim3 grid((unsigned)(8 * ((units + 7) / 8) * ksplit));
    auto go = [&](auto kern, int lds) -> hipError_t {
        FP8GEMM_ALLOW_LDS(kern, lds);
        hipLaunchKernelGGL(kern, grid, dim3(DS_THREADS), lds, s, tab, mailbox, n, k, strips, ksplit, kb_per_split);
        return hipGetLastError();
    };
    if (ragged)
        return row_tiles(mmax) == 2
                   ? go(decode_strip_grouped_kernel<2, 6, true>, DecodeShape<2, 6, true>::LDS)
                   : go(decode_strip_grouped_kernel<4, RAGGED4_NS, true>, DecodeShape<4, RAGGED4_NS, true>::LDS);
    const bool deep = !shallow_ring_pays(units * ksplit, kb_per_split);
    if (row_tiles(mmax) == 2)
        return deep ? go(decode_strip_grouped_kernel<2, 6, false>, DecodeShape<2, 6>::LDS)
                    : go(decode_strip_grouped_kernel<2, 3, false>, DecodeShape<2, 3>::LDS);
    return deep ? go(decode_strip_grouped_kernel<4, 6, false>, DecodeShape<4, 6>::LDS)
                : go(decode_strip_grouped_kernel<4, 3, false>, DecodeShape<4, 3>::LDS);
}

}  // namespace fp8gemm
