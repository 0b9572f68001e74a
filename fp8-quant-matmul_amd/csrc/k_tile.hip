// MFMA tile kernel for gfx950: the successor of in_smem_kernel (/root/reference/mn_large.hip:11-128)
// and, with the K range split over workgroups, of k_large_kernel (/root/reference/mn_small.hip:10-137).
//
// Data path (all of it differs from the reference, which scatters single bytes into LDS):
//   * A ([K][M], m contiguous) and B ([K][N], n contiguous) tiles of 128 K-rows are copied
//     global -> LDS with 16-byte buffer loads that write LDS directly (no VGPR round trip),
//     keeping the global orientation: one LDS row per k, 128 or 256 bytes per row.  The
//     16-byte column chunk c of row r is stored at chunk position c ^ swizzle(r), which makes
//     the transposing reads below bank-conflict free (measured: 0 conflicts).
//   * Operands are fetched with ds_read_b64_tr_b8: 16 lanes read an 8(k) x 16(m|n) byte
//     patch and receive it transposed, i.e. lane i holds 8 consecutive k of column i.  Four
//     such reads give the 32 bytes per lane that v_mfma_f32_32x32x64_f8f6f4 consumes.
//     The k order inside the instruction is permuted identically for both operands, which
//     leaves the dot product unchanged.
//   * Two MFMAs (K = 64 each) cover a 128-wide scale block of one 32x32 patch; the block sum
//     lives in 16 registers for a moment and is folded into the running result with
//     a_scale[kb][m] * b_scale[kb][n/128] by one FMA per element (mn_large.hip:100-106,
//     mn_small.hip:85-88 do the same with a second full-size accumulator).
//   * The MFMA computes the transposed patch (rows = n, columns = m) as mn_small.hip does,
//     so that a lane owns one m (one a_scale value) and runs of 4 consecutive n.
//   * The finished tile goes through the idle LDS ring (row-major, padded rows) and leaves as
//     16 bytes per lane along whole tile rows; straight from the accumulators a store
//     instruction would write 8-byte pieces of 32 different rows.
//   * a_scale values of the tile travel through LDS with the stage (one extra 1 KiB copy), so
//     the K loop holds no compiler-visible global load and every wait on the copies is the
//     explicit one below.
//   * NS LDS stages form a ring: the copies of K blocks kb+1 .. kb+NS-1 are in flight while
//     block kb is multiplied.  Large tiles fit two stages; smaller tiles get three or four,
//     which is what hides the global latency when a K block is only a few MFMAs long.
//   * The copy instructions of a K block ride on the first MFMAs of an earlier block instead
//     of being issued in one burst after the barrier (a burst queues up in the address unit
//     and holds every wave back from its LDS reads).
//
// Work decomposition: grid.x = tiles (XCD-aware order), grid.y = K splits.
#include "tile_common.h"

namespace fp8gemm {

namespace {

template <int BM, int BN, int WM, int WN, int NS, bool SPLIT>
__global__ void __launch_bounds__(NTHREADS)
tile_gemm_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                 const float* __restrict__ a_scale, const float* __restrict__ b_scale,
                 uint16_t* __restrict__ c, float* __restrict__ partial, float* mailbox,
                 int M, int lda, int N, int K, int tiles_m, int tiles_n, int kb_per_split, int group_m)
{
    using S = TileShape<BM, BN, WM, WN, NS>;
    // Eight waves copy; WM x WN of them (all eight, or the first four for the smallest tile)
    // also multiply.
    static_assert(WM * WN == 8 || WM * WN == 4, "eight or four multiplying waves");
    constexpr int NCW = WM * WN;
    static_assert(NS >= 2 && NS <= 4, "two to four LDS stages");
    constexpr int TM = BM / WM, TN = BN / WN;      // wave tile
    constexpr int MI = TM / 32, NJ = TN / 32;      // 32x32 patches per wave
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile is made of 32x32 patches");
    static_assert(TN <= 128, "a wave's n range touches at most two 128-wide scale blocks");
    static_assert(BM <= 256 && BN <= 256, "LDS rows hold at most 256 bytes");
    constexpr int RSA = S::RSA, RSB = S::RSB, NA = S::NA, NB = S::NB, NCOPY = S::NCOPY;

    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    auto lds = LDS_PTR(uint8_t, smem);
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = (wave / WM) % WN;
    const bool compute = NCW == 8 || wave < NCW;

    // ---- which tile: consecutive workgroup ids land on different XCDs (id % 8), so give
    // each XCD a contiguous run of tile numbers, and walk tiles in groups of group_m rows
    // so that the tiles an XCD works on together share A and B panels in its L2 (the host picks
    // group_m so that an XCD's co-resident tiles form a block that is about square in bytes).
    const int T = tiles_m * tiles_n;
    const int pid = blockIdx.x;
    if (pid >= T)  // grid.x is rounded up to a multiple of 8 when the K splits of a tile have to share an XCD
        return;
    const int xcd = pid & 7, q8 = T >> 3, r8 = T & 7;
    const int logical = xcd * q8 + (xcd < r8 ? xcd : r8) + (pid >> 3);
    const int per_group = group_m * tiles_n;
    const int group = logical / per_group;
    const int first_m = group * group_m;
    const int gsz = (tiles_m - first_m < group_m) ? (tiles_m - first_m) : group_m;
    const int in_group = logical - group * per_group;
    const int m0 = (first_m + in_group % gsz) * BM;
    const int n0 = (in_group / gsz) * BN;

    const int nkb = K / KBLOCK;
    const int kb0 = blockIdx.y * kb_per_split;
    const int kb1 = (kb0 + kb_per_split < nkb) ? (kb0 + kb_per_split) : nkb;

    // ---- global -> LDS copy plan.  One 16-byte load per lane fills 1 KiB of LDS (LDS address
    // = base + lane*16): 4 rows of 256 B, 8 rows of 128 B or 16 rows of 64 B.  Wave w owns instructions
    // NA*w .. NA*w+NA-1 of the A tile and likewise of B.  A lane writes chunk position p of
    // row r and therefore fetches column chunk p ^ swizzle(r).  Chunks outside the tile or the
    // matrix get an out-of-range offset: the buffer load then writes zeros and reads nothing.
    uint32_t voff_a[S::NVA], voff_b[S::NVB];
#pragma unroll
    for (int q = 0; q < S::NVA; ++q) {
        const int r = (NA * wave + q) * (1024 / RSA) + S::template copy_row<RSA>(lane);
        const int cc = S::template copy_pos<RSA>(lane) ^ row_swizzle<RSA>(r & 7);
        const bool ok = (16 * cc < BM) && (m0 + 16 * cc < M);
        voff_a[q] = ok ? (uint32_t)(r * lda + m0 + 16 * cc) : 0x80000000u;
    }
#pragma unroll
    for (int q = 0; q < S::NVB; ++q) {
        const int r = (NB * wave + q) * (1024 / RSB) + S::template copy_row<RSB>(lane);
        const int cc = S::template copy_pos<RSB>(lane) ^ row_swizzle<RSB>(r & 7);
        const bool ok = (16 * cc < BN) && (n0 + 16 * cc < N);
        voff_b[q] = ok ? (uint32_t)(r * N + n0 + 16 * cc) : 0x80000000u;
    }
    const uint32_t a_bytes = (uint32_t)lda * (uint32_t)K, b_bytes = (uint32_t)N * (uint32_t)K;
    const uint32_t as_bytes = (uint32_t)nkb * (uint32_t)lda * 4u;
    const uint32_t voff_s =
        (4 * lane < BM && m0 + 4 * lane < M) ? (uint32_t)((m0 + 4 * lane) * 4) : 0x80000000u;

    // copy instruction q (0..NCOPY-1) of K block kb into ring slot `slot`.  The three buffer
    // resources stay fixed; the K block's byte offset rides in the scalar offset operand.
    const v4i rsrc_a = make_rsrc_words(a, a_bytes), rsrc_b = make_rsrc_words(b, b_bytes);
    const v4i rsrc_s = make_rsrc_words(a_scale, as_bytes);
    auto copy_step = [&](int slot, int kb, int q) __attribute__((always_inline)) {
        const uint32_t stage = lds_base + (uint32_t)(slot * S::STAGE);
        if (q < NA) {
            lds_dma16(rsrc_a, voff_a[S::template voff_index<RSA>(q)], stage + (uint32_t)((NA * wave + q) * 1024),
                      (uint32_t)(kb * KBLOCK + S::template extra_rows<RSA>(q)) * (uint32_t)lda);
        } else if (q < NA + NB) {
            lds_dma16(rsrc_b, voff_b[S::template voff_index<RSB>(q - NA)],
                      stage + S::MAT_A + (uint32_t)((NB * wave + (q - NA)) * 1024),
                      (uint32_t)(kb * KBLOCK + S::template extra_rows<RSB>(q - NA)) * (uint32_t)N);
        } else if (wave == 0) {
            lds_dma16(rsrc_s, voff_s, stage + S::SCALE_OFF, (uint32_t)kb * (uint32_t)lda * 4u);
        }
    };

    // ---- transposing LDS reads.  Lane l = 16*g + i feeds MFMA row/column (l & 31) and k half
    // (l >> 5).  For K step ks (64 wide) read t of the lane covers k rows
    // 64*ks + 32*(g>>1) + 8*t + (i>>1), 8-byte half (i & 1) of 16-byte chunk (patch chunk + (g&1)).
    // (row & 7) = (i >> 1) does not depend on t or ks: one address per patch plus immediates.
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

    // 32 bytes per lane of one operand for K step ks; rs = row stride of the matrix read
    auto read_frag = [&](uint32_t addr, int ks, int rs) __attribute__((always_inline)) -> v8i {
        const uint32_t base = addr + (uint32_t)(ks * 64 * rs);
        v2i r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base));
        v2i r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 8 * rs));
        v2i r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 16 * rs));
        v2i r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + base + 24 * rs));
        return (v8i){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    };

    // ---- scales.  One a_scale per lane and 32-row patch (the lane's m).  A wave's n range is at
    // most 128 wide, so it touches at most two 128-wide b_scale blocks (nb_lo, nb_hi); a 32-wide
    // patch never straddles a block boundary.
    const int sn = (N + KBLOCK - 1) / KBLOCK;
    const int n_wave = n0 + wn * TN;
    int nb_lo = n_wave >> 7, nb_hi = (n_wave + TN - 1) >> 7;
    nb_lo = nb_lo < sn ? nb_lo : sn - 1;
    nb_hi = nb_hi < sn ? nb_hi : sn - 1;
    uint32_t hi_mask[NJ];  // all ones when patch j lies in the wave's second b_scale block
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        hi_mask[j] = (uint32_t)-(int)(((n_wave + 32 * j) >> 7) > (n_wave >> 7));

    v16f acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                acc[i][j][r] = 0.f;
    const v16f zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    // ---- prologue: the first NS-1 K blocks go into ring slots 0 .. NS-2
#pragma unroll
    for (int p = 0; p < NS - 1; ++p)
        if (kb0 + p < kb1) {
#pragma unroll
            for (int q = 0; q < NCOPY; ++q)
                copy_step(p, kb0 + p, q);
        }

    int slot = 0;             // ring slot of block kb
    int slot_fill = NS - 1;   // ring slot that block kb + NS - 1 goes into (= slot of kb - 1)

    // One K block.  MORE = block kb+NS-1 exists and is copied here; two instantiations keep the
    // steady-state body free of branches.
    auto k_block = [&](auto more_tag, int kb) {
        constexpr bool more = decltype(more_tag)::value;
        // Block kb has landed once at most the copies of the younger blocks in flight are
        // outstanding (loads complete in order).  NCOPY - 1 per block is exact for waves 1..7
        // and one short for wave 0, which then waits for one more copy than it must.
        if (more) {
            wait_vmcnt<(NS - 2) * (NCOPY - 1)>();
        } else {
            const int younger = (kb1 - 1 - kb < NS - 2) ? (kb1 - 1 - kb) : (NS - 2);
            if (NS >= 4 && younger >= 2)
                wait_vmcnt<2 * (NCOPY - 1)>();
            else if (NS >= 3 && younger >= 1)
                wait_vmcnt<NCOPY - 1>();
            else
                wait_vmcnt<0>();
        }
        __syncthreads();  // everyone's copies of block kb landed; slot_fill is no longer read
        if (!compute) {  // copy-only wave
            if (more) {
#pragma unroll
                for (int q = 0; q < NCOPY; ++q)
                    copy_step(slot_fill, kb + NS - 1, q);
            }
            slot_fill = slot;
            slot = (slot + 1 == NS) ? 0 : slot + 1;
            return;
        }
        const uint32_t so = (uint32_t)(slot * S::STAGE);
        float sa[MI];
#pragma unroll
        for (int i = 0; i < MI; ++i)
            sa[i] = *LDS_PTR(float, lds + so + addr_s + 128 * i);
        // wave-uniform addresses: scalar loads
        const float sb_lo = b_scale[__builtin_amdgcn_readfirstlane(kb * sn + nb_lo)];
        const float sb_hi = b_scale[__builtin_amdgcn_readfirstlane(kb * sn + nb_hi)];

        v8i fa[MI][2];
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            fa[i][0] = read_frag(addr_a[i] + so, 0, RSA);
            fa[i][1] = read_frag(addr_a[i] + so, 1, RSA);
        }

        // the wave's NCOPY copy instructions of block kb+NS-1 ride on the first MFMAs
        constexpr int N_MFMA = MI * NJ * 2;
        constexpr int PER_MFMA = (NCOPY + N_MFMA - 1) / N_MFMA;  // copies behind each MFMA
        int cq = 0;
        auto copy_slot = [&](int n) {
#pragma unroll
            for (int u = 0; u < NCOPY; ++u)
                if (u < n && cq < NCOPY) {
                    if (more)
                        copy_step(slot_fill, kb + NS - 1, cq);
                    ++cq;
                }
        };

#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const v8i fb0 = read_frag(addr_b[j] + so, 0, RSB);
            const v8i fb1 = read_frag(addr_b[j] + so, 1, RSB);
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
                const float sbj = __uint_as_float((__float_as_uint(sb_hi) & hi_mask[j]) |
                                                  (__float_as_uint(sb_lo) & ~hi_mask[j]));
                const float sc = sa[i] * sbj;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[i][j][r] = fmaf(sc, blk[i][r], acc[i][j][r]);
            }
        }
        copy_slot(NCOPY);  // whatever is left (tiles with few MFMAs per K block)

        slot_fill = slot;
        slot = (slot + 1 == NS) ? 0 : slot + 1;
    };
    int kb = kb0;
    for (; kb + NS - 1 < kb1; ++kb)
        k_block(std::true_type{}, kb);
    for (; kb < kb1; ++kb)
        k_block(std::false_type{}, kb);

    // ---- K splits added inside the kernel (mailbox != nullptr).  grid.x is a multiple of 8, so the
    // workgroups of one tile (same blockIdx.x) have linear ids that agree modulo 8 and share an XCD: what
    // they store and load meets in that XCD's L2.  The mailbox holds zeros between launches.  A wave of every
    // split but the last stores its accumulators there in register order (1 KiB per instruction) with
    // every +0.0 replaced by -0.0, so that no word it writes is zero, and is done.  The waves of the last
    // split -- the workgroup with the highest id of its tile, dispatched after the others -- load the other
    // splits' patches past their L1 until no word is zero, store zeros back, add them in split order, their
    // own registers last (the arithmetic of splitk_reduce_kernel: adding -0.0 changes nothing), and the
    // workgroup leaves through the bf16 epilogue.  A wave that has polled for a second gives up and
    // writes NaN.
    bool as_partial = SPLIT;
    if constexpr (SPLIT) {
        if (mailbox != nullptr) {
            as_partial = false;
            constexpr int PATCHES = NCW * MI * NJ;  // 32x32 patches of a tile: 4 KiB of fp32 each
            const int senders = (int)gridDim.y - 1;
            const size_t first = ((size_t)pid * senders * PATCHES + (size_t)wave * (MI * NJ)) * 256;  // in 16-byte units
            if ((int)blockIdx.y < senders) {
                if (compute) {
                    v4i* mine = reinterpret_cast<v4i*>(mailbox) + first + (size_t)blockIdx.y * PATCHES * 256 + lane;
#pragma unroll
                    for (int i = 0; i < MI; ++i)
#pragma unroll
                        for (int j = 0; j < NJ; ++j)
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                v4i bits;
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    const int w = (int)__float_as_uint(acc[i][j][4 * q + e]);
                                    bits[e] = w == 0 ? (int)0x80000000 : w;
                                }
                                mine[((i * NJ + j) * 4 + q) * 64] = bits;
                            }
                }
                return;
            }
            if (compute) {
                constexpr int ZC = MI * NJ <= 2 ? 4 : 2;  // splits polled together (registers)
                const uint32_t span = (uint32_t)senders * PATCHES * 4096u;
                const __amdgpu_buffer_rsrc_t rp = make_rsrc(reinterpret_cast<const v4i*>(mailbox) + first, span);
                const unsigned long long t_first = __builtin_amdgcn_s_memrealtime();
                bool gave_up = false;
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        v4f sum[4];
                        for (int z0 = 0; z0 < senders; z0 += ZC) {
                            v4i v[ZC][4];
                            for (;;) {
                                asm volatile("" ::: "memory");  // the loads belong to this round of the loop
#pragma unroll
                                for (int z = 0; z < ZC; ++z)
#pragma unroll
                                    for (int q = 0; q < 4; ++q)  // a split past the last: outside the resource, zeros
                                        v[z][q] = __builtin_amdgcn_raw_buffer_load_b128(
                                            rp, (uint32_t)((((z0 + z) * PATCHES + i * NJ + j) * 4 + q) * 64 + lane) * 16u, 0, 16);
                                bool missing = false;
#pragma unroll
                                for (int z = 0; z < ZC; ++z)
#pragma unroll
                                    for (int q = 0; q < 4; ++q)
                                        if (z0 + z < senders)
                                            missing = missing || v[z][q][0] == 0 || v[z][q][1] == 0 || v[z][q][2] == 0 ||
                                                      v[z][q][3] == 0;
                                if (__builtin_amdgcn_ballot_w64(missing) == 0)
                                    break;
                                if (__builtin_amdgcn_s_memrealtime() - t_first > 100000000ull) {  // one second at 100 MHz
                                    gave_up = true;
                                    break;
                                }
                            }
#pragma unroll
                            for (int z = 0; z < ZC; ++z)
                                if (z0 + z < senders) {
#pragma unroll
                                    for (int q = 0; q < 4; ++q) {
                                        __builtin_amdgcn_raw_buffer_store_b128(
                                            (v4i){0, 0, 0, 0}, rp,
                                            (uint32_t)((((z0 + z) * PATCHES + i * NJ + j) * 4 + q) * 64 + lane) * 16u, 0, 0);
                                        const v4f f = __builtin_bit_cast(v4f, v[z][q]);
                                        sum[q] = z0 + z == 0 ? f : sum[q] + f;
                                    }
                                }
                        }
#pragma unroll
                        for (int q = 0; q < 4; ++q)
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                acc[i][j][4 * q + e] = gave_up ? __builtin_nanf("") : sum[q][e] + acc[i][j][4 * q + e];
                    }
            }
        }
    }

    // ---- epilogue.  A lane owns row m = .. + (lane & 31) and, per patch, four runs of 4 columns
    // (accumulator register 4*q + e is column 8*q + 4*(lane >> 5) + e of the patch): stored
    // straight from the registers that would be 8- or 16-byte pieces of 32 different rows per
    // instruction.  The tile therefore goes through the (now idle) LDS ring, row-major with a
    // padded row stride that keeps the writes conflict free, and leaves as 16 bytes per lane
    // along whole rows of the tile.  A tile larger than the ring is written in two halves.
    // PARTIAL = fp32 into this split's partial tile (the reduction kernel follows), else bf16 into c.
    auto write_tile = [&](auto partial_tag) __attribute__((always_inline)) {
        constexpr bool PARTIAL = decltype(partial_tag)::value;
        constexpr int ESZ = PARTIAL ? 4 : 2;
        constexpr int CROW = BN * ESZ + (PARTIAL ? 16 : 8);  // LDS bytes per tile row
        constexpr int HALVES = (BM * CROW <= S::LDS_BYTES) ? 1 : 2;
        constexpr int HROWS = BM / HALVES;
        static_assert(HROWS * CROW <= S::LDS_BYTES, "half a tile must fit the ring");
        static_assert(HROWS % 32 == 0, "a 32-row patch lies in one half");
        constexpr int CPR = BN * ESZ / 16;                 // 16-byte chunks per tile row
        constexpr int CHUNKS = HROWS * CPR;
#pragma unroll
        for (int h = 0; h < HALVES; ++h) {
            __syncthreads();  // nobody reads the ring (or the previous half) any more
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int prow = wm * TM + 32 * i;  // first tile row of the patch
                if (compute && prow / HROWS == h) {
                    const uint32_t rbase = (uint32_t)((prow - h * HROWS + (lane & 31)) * CROW);
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const int col = wn * TN + 32 * j + 8 * q + 4 * (lane >> 5);
                            const v4f v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                           acc[i][j][4 * q + 3]};
                            if (PARTIAL) {
                                *LDS_PTR(v4f, lds + rbase + col * 4) = v;
                            } else {
                                v2i pk = {(int)pack_bf16x2(v[0], v[1]), (int)pack_bf16x2(v[2], v[3])};
                                *LDS_PTR(v2i, lds + rbase + col * 2) = pk;
                            }
                        }
                }
            }
            __syncthreads();
#pragma unroll
            for (int it = 0; it < (CHUNKS + NTHREADS - 1) / NTHREADS; ++it) {
                const int idx = it * NTHREADS + (int)threadIdx.x;
                const int row = idx / CPR, ch = idx - row * CPR;
                const int mrow = m0 + h * HROWS + row;
                const int ncol = n0 + ch * (16 / ESZ);
                if (idx < CHUNKS && mrow < M && ncol < N) {
                    const size_t o = (size_t)mrow * N + ncol;
                    if (PARTIAL) {
                        const v4f v = *LDS_PTR(v4f, lds + row * CROW + ch * 16);
                        *reinterpret_cast<v4f*>(partial + (size_t)blockIdx.y * M * N + o) = v;
                    } else {
                        const v2i lo = *LDS_PTR(v2i, lds + row * CROW + ch * 16);
                        const v2i hi = *LDS_PTR(v2i, lds + row * CROW + ch * 16 + 8);
                        *reinterpret_cast<v4i*>(c + o) = (v4i){lo.x, lo.y, hi.x, hi.y};
                    }
                }
            }
        }
    };
    if constexpr (SPLIT) {
        if (as_partial)
            write_tile(std::true_type{});
        else
            write_tile(std::false_type{});
    } else {
        write_tile(std::false_type{});
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
    // four splits' loads in flight at a time (one after the other, each add waits a trip to the L2: 0.4 us per
    // split of a small problem); the sum keeps its order
    v4f s = *reinterpret_cast<const v4f*>(partial + i4);
    int z = 1;
    for (; z + 3 < ksplit; z += 4) {
        v4f p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            p[u] = *reinterpret_cast<const v4f*>(partial + (size_t)(z + u) * mn + i4);
#pragma unroll
        for (int u = 0; u < 4; ++u)
            s += p[u];
    }
    for (; z < ksplit; ++z) {
        v4f p = *reinterpret_cast<const v4f*>(partial + (size_t)z * mn + i4);
        s += p;
    }
    uint2 pk;
    pk.x = pack_bf16x2(s[0], s[1]);
    pk.y = pack_bf16x2(s[2], s[3]);
    *reinterpret_cast<uint2*>(c + i4) = pk;
}

// Tile rows per locality group.  The kernel gives XCD x (workgroup id % 8) a contiguous run of the
// tile order, which walks the tile grid in groups of group_m rows, column by column.  The tiles an
// XCD works on together (its first 32: one per CU) then touch some rows of A and some of B; the
// group size that makes the eight XCDs touch the fewest bytes is found by walking the order, and
// remembered for the last few grids.
int choose_group_m(int tiles_m, int tiles_n, int bm, int bn)
{
    struct Entry { int tm, tn, bm, bn, g; };
    static thread_local Entry cache[8] = {};
    static thread_local int next = 0;
    for (const Entry& e : cache)
        if (e.tm == tiles_m && e.tn == tiles_n && e.bm == bm && e.bn == bn)
            return e.g;
    const int T = tiles_m * tiles_n;
    int best_g = GROUP_M;
    long best_cost = -1;
    for (int gm = 1; gm <= GROUP_M; ++gm) {
        long cost = 0;
        for (int xcd = 0; xcd < 8; ++xcd) {
            const int q8 = T >> 3, r8 = T & 7;
            const int start = xcd * q8 + (xcd < r8 ? xcd : r8);
            int len = q8 + (xcd < r8 ? 1 : 0);
            len = len < 32 ? len : 32;
            unsigned long long rows[4] = {0, 0, 0, 0}, cols[4] = {0, 0, 0, 0};  // up to 256 tile rows / columns tracked
            int nrows = 0, ncols = 0;
            for (int t = start; t < start + len; ++t) {
                const int per_group = gm * tiles_n, group = t / per_group, first_m = group * gm;
                const int gsz = tiles_m - first_m < gm ? tiles_m - first_m : gm;
                const int in_group = t - group * per_group;
                const int r = (first_m + in_group % gsz) & 255, c = (in_group / gsz) & 255;
                if (!(rows[r >> 6] >> (r & 63) & 1)) {
                    rows[r >> 6] |= 1ull << (r & 63);
                    ++nrows;
                }
                if (!(cols[c >> 6] >> (c & 63) & 1)) {
                    cols[c >> 6] |= 1ull << (c & 63);
                    ++ncols;
                }
            }
            cost += (long)nrows * bm + (long)ncols * bn;
        }
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best_g = gm;
        }
    }
    cache[next] = Entry{tiles_m, tiles_n, bm, bn, best_g};
    next = (next + 1) & 7;
    return best_g;
}

template <int BM, int BN, int WM, int WN, int NS>
hipError_t launch_variant(const GemmArgs& g, int ksplit, float* partial, float* mailbox, hipStream_t s)
{
    using S = TileShape<BM, BN, WM, WN, NS>;
    constexpr int LDS_TOTAL = S::LDS_BYTES;
    const int tiles_m = (g.m + BM - 1) / BM, tiles_n = (g.n + BN - 1) / BN;
    const int nkb = g.k / KBLOCK;
    const int kb_per_split = (nkb + ksplit - 1) / ksplit;
    const int tiles = tiles_m * tiles_n;
    const int group_m = choose_group_m(tiles_m, tiles_n, BM, BN);
    if (ksplit > 1) {
        // in-kernel reduction: the other splits' patches of every tile fit the mailbox
        if (mailbox && (size_t)tiles * (ksplit - 1) * BM * BN * 4 > SPLIT_MAILBOX_BYTES)
            return hipErrorInvalidValue;
        dim3 grid(mailbox ? (tiles + 7) & ~7 : tiles, ksplit);
        auto kern = tile_gemm_kernel<BM, BN, WM, WN, NS, true>;
        FP8GEMM_ALLOW_LDS(kern, LDS_TOTAL);
        hipLaunchKernelGGL(kern, grid, dim3(NTHREADS), LDS_TOTAL, s, g.a, g.b, g.a_scale, g.b_scale, g.c, partial,
                           mailbox, g.m, leading_dim(g), g.n, g.k, tiles_m, tiles_n, kb_per_split, group_m);
    } else {
        auto kern = tile_gemm_kernel<BM, BN, WM, WN, NS, false>;
        FP8GEMM_ALLOW_LDS(kern, LDS_TOTAL);
        hipLaunchKernelGGL(kern, dim3(tiles, 1), dim3(NTHREADS), LDS_TOTAL, s, g.a, g.b, g.a_scale, g.b_scale, g.c,
                           partial, static_cast<float*>(nullptr), g.m, leading_dim(g), g.n, g.k, tiles_m,
                           tiles_n, kb_per_split, group_m);
    }
    return hipGetLastError();
}

}  // namespace

bool tile_supports(const GemmArgs& g)
{
    // 16-byte copies need every k-row of a, b and a_scale to start 16-byte aligned; rows of a
    // and a_scale beyond m, up to the leading dimension, are read (and must be finite: zeros)
    return leading_dim(g) % 16 == 0 && leading_dim(g) >= g.m && g.n % 16 == 0 &&
           (reinterpret_cast<uintptr_t>(g.a) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.b) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.a_scale) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.c) % 16 == 0);
}

const char* tile_variant_name(int variant)
{
    switch (variant) {
    case TILE_256x128: return "tile256x128";
    case TILE_128x128: return "tile128x128";
    case TILE_256x192: return "tile256x192";
    case TILE_128x192: return "tile128x192";
    case TILE_64x64: return "tile64x64";
    case TILE_256x192_W4: return "tile256x192w4";
    case TILE_256x256: return "tile256x256";
    default: return "tile?";
    }
}

void tile_variant_dims(int variant, int* bm, int* bn)
{
    switch (variant) {
    case TILE_256x128: *bm = 256; *bn = 128; break;
    case TILE_256x192:
    case TILE_256x192_W4: *bm = 256; *bn = 192; break;
    case TILE_128x192: *bm = 128; *bn = 192; break;
    case TILE_64x64: *bm = 64; *bn = 64; break;
    case TILE_256x256: *bm = 256; *bn = 256; break;
    default: *bm = 128; *bn = 128; break;
    }
}

size_t tile_mailbox_bytes(const GemmArgs& g, int variant, int ksplit)
{
    int bm, bn;
    tile_variant_dims(variant, &bm, &bn);
    const size_t tiles = (size_t)((g.m + bm - 1) / bm) * ((g.n + bn - 1) / bn);
    return ksplit > 1 ? tiles * (size_t)(ksplit - 1) * bm * bn * 4 : 0;
}

hipError_t launch_tile(const GemmArgs& g, int variant, int ksplit, float* partial, float* mailbox,
                       hipStream_t s)
{
    switch (variant) {
    case TILE_256x192: return launch_variant<256, 192, 4, 2, 2>(g, ksplit, partial, mailbox, s);
    case TILE_256x128: return launch_variant<256, 128, 4, 2, 3>(g, ksplit, partial, mailbox, s);
    case TILE_128x192: return launch_variant<128, 192, 4, 2, 3>(g, ksplit, partial, mailbox, s);
    case TILE_128x128: return launch_variant<128, 128, 2, 4, 4>(g, ksplit, partial, mailbox, s);
    case TILE_64x64: return launch_variant<64, 64, 2, 2, 4>(g, ksplit, partial, mailbox, s);
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
