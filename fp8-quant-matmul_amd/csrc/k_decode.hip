// Wide-strip decode kernel for tiny M (M <= 32): HBM-bound, B is read exactly once, in whole
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
// The K splits of a strip are added inside the kernel, wave by wave, without a second launch:
//   * the workgroups of one strip are given linear ids that agree modulo 8, which the dispatcher
//     places on one XCD (checked once per device by a probe grid, xcd_placement_confirmed): their
//     stores and loads meet in that XCD's L2, and no device-scope fence -- a write-back of the whole
//     L2 on this part -- is needed;
//   * a wave stores its fp32 partial patch (register order, 1 KiB per instruction), waits for the
//     stores' acknowledgement from L2 (s_waitcnt vmcnt(0)), and takes a ticket for (strip, wave) with
//     a workgroup-scope atomic, which executes in that same L2;
//   * the wave whose ticket says it arrived last loads all partial patches of its columns past its L1
//     (sc0: a device-scope load, sc1, would also pass the L2 and cost a round trip to memory), adds them in split order -- the result does not depend on who arrived last -- and stores
//     bf16.  The ticket wraps to zero with the last arrival (atomic inc with wrap), so the ticket
//     words stay zero between launches; they must be zero before the first one.
//
// LDS stage: 128 k-rows x 128 B of B (chunk c of row r at position c ^ ((r >> 1) & 7)), 128 x 32 B
// of A (chunk c at c ^ ((r >> 3) & 1)), the block's a_scale and b_scale values; six stages form a
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
constexpr int DS_MAT_B = KBLOCK * 128;
constexpr int DS_MAT_A = KBLOCK * 32;
constexpr int DS_SA_OFF = DS_MAT_B + DS_MAT_A;  // M floats (wave 4's copy)
constexpr int DS_SB_OFF = DS_SA_OFF + 256;      // 1 float (wave 5's copy; waves 6 and 7 bring it again, 256 B apart)
constexpr int DS_STAGE = DS_SB_OFF + 3 * 256;
constexpr int DS_NS = 6;
constexpr int DS_LDS = DS_NS * DS_STAGE;
constexpr int DS_COPIES = 3;                    // copy instructions per wave and stage
constexpr unsigned AUX_L1_MISS = 1;             // cache policy of the buffer loads (sc0): served by the L2
static_assert(DS_LDS <= 160 * 1024, "ring exceeds the LDS");
static_assert(DS_COPIES * (DS_NS - 2) < 64, "vmcnt is a 6-bit field");

template <int N>
__device__ __forceinline__ void ds_wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__global__ void __launch_bounds__(DS_THREADS)
decode_strip_kernel(const uint8_t* __restrict__ a, const uint8_t* __restrict__ b,
                    const float* __restrict__ a_scale, const float* __restrict__ b_scale,
                    uint16_t* __restrict__ c, float* __restrict__ partial, unsigned int* __restrict__ tickets,
                    int M, int N, int K, int strips, int ksplit, int kb_per_split)
{
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    auto lds = LDS_PTR(uint8_t, smem);
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // linear ids that agree modulo 8 share an XCD: the ksplit workgroups of a strip sit at
    // ids xcd + 8 * (group * ksplit + split)
    const int pid = blockIdx.x;
    const int xcd = pid & 7, j = pid >> 3;
    const int grp = j / ksplit, split = j - grp * ksplit;
    const int strip = grp * 8 + xcd;
    if (strip >= strips)
        return;
    const int n0 = strip * DS_BN;

    const int nkb = K / KBLOCK;
    const int kb0 = split * kb_per_split;
    const int kb1 = (kb0 + kb_per_split < nkb) ? (kb0 + kb_per_split) : nkb;
    const int sn = (N + KBLOCK - 1) / KBLOCK;
    const int mtiles = (M + 15) >> 4;  // 1 or 2

    // ---- copy plan, three instructions per wave and stage.  B: instruction q (0, 1) of a wave fills
    // stage rows 16*wave + 8*q + (lane >> 3), chunk position lane & 7; the chunk swizzle (r >> 1) & 7 is
    // (4*q + (lane >> 4)) & 7.  A: waves 0..3, rows 32*wave + (lane >> 1), position lane & 1, swizzle
    // (r >> 3) & 1 = (lane >> 4) & 1.  Wave 4 brings the block's a_scale values, waves 5..7 its b_scale
    // value (each into a slot of its own; wave 5's is read), so that every wave counts the same.
    const uint32_t a_bytes = (uint32_t)M * (uint32_t)K, b_bytes = (uint32_t)N * (uint32_t)K;
    uint32_t voff_b[2];
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const int cc = (lane & 7) ^ ((4 * q + (lane >> 4)) & 7);
        const bool ok = n0 + 16 * cc < N;
        voff_b[q] = ok ? (uint32_t)((16 * wave + 8 * q + (lane >> 3)) * N + n0 + 16 * cc) : 0x80000000u;
    }
    const int cca = (lane & 1) ^ ((lane >> 4) & 1);
    uint32_t voff_3;  // the wave's third instruction
    if (wave < 4)
        voff_3 = 16 * cca < M ? (uint32_t)((32 * wave + (lane >> 1)) * M + 16 * cca) : 0x80000000u;
    else if (wave == 4)
        voff_3 = lane < M ? (uint32_t)(lane * 4) : 0x80000000u;
    else
        voff_3 = lane == 0 ? (uint32_t)(strip * 4) : 0x80000000u;

    // Stage `slot` <- K block kb.  The resources of A and B start at the block's first k-row.
    auto issue_stage = [&](int slot, int kb) __attribute__((always_inline)) {
        const uint32_t stage = lds_base + (uint32_t)(slot * DS_STAGE);
        const uint32_t skip_b = (uint32_t)kb * KBLOCK * (uint32_t)N;
        const v4i rb = make_rsrc_words(b + skip_b, b_bytes - skip_b);
        lds_dma16(rb, voff_b[0], stage + (uint32_t)((2 * wave) * 1024));
        lds_dma16(rb, voff_b[1], stage + (uint32_t)((2 * wave + 1) * 1024));
        if (wave < 4) {
            const uint32_t skip_a = (uint32_t)kb * KBLOCK * (uint32_t)M;
            lds_dma16(make_rsrc_words(a + skip_a, a_bytes - skip_a), voff_3, stage + DS_MAT_B + (uint32_t)(wave * 1024));
        } else if (wave == 4) {
            lds_dma4(make_rsrc_words(a_scale + (size_t)kb * M, (uint32_t)M * 4u), voff_3, stage + DS_SA_OFF);
        } else {
            lds_dma4(make_rsrc_words(b_scale + (size_t)kb * sn, (uint32_t)sn * 4u), voff_3,
                     stage + DS_SB_OFF + (uint32_t)((wave - 5) * 256));
        }
    };

    // ---- transposing reads.  Lane = 16*g + i; read t of a K block covers k-rows 32*t + 8*g + (i >> 1),
    // so (r >> 1) & 7 = (4*g + (i >> 2)) & 7 and (r >> 3) & 1 = g & 1 for every t and both blocks.
    const int g4 = lane >> 4, i16 = lane & 15;
    const uint32_t addr_b = (uint32_t)((8 * g4 + (i16 >> 1)) * 128 + ((wave ^ ((4 * g4 + (i16 >> 2)) & 7)) * 16) +
                                       (i16 & 1) * 8);
    const uint32_t addr_a = (uint32_t)(DS_MAT_B + (8 * g4 + (i16 >> 1)) * 32 + (i16 & 1) * 8);
    const uint32_t chunk_a[2] = {(uint32_t)((0 ^ (g4 & 1)) * 16), (uint32_t)((1 ^ (g4 & 1)) * 16)};
    auto read_frag = [&](uint32_t addr, int step) __attribute__((always_inline)) -> v8i {
        v2i r0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr));
        v2i r1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + step));
        v2i r2 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 2 * step));
        v2i r3 = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, lds + addr + 3 * step));
        return (v8i){r0.x, r0.y, r1.x, r1.y, r2.x, r2.y, r3.x, r3.y};
    };

    v4f acc[2] = {(v4f){0.f, 0.f, 0.f, 0.f}, (v4f){0.f, 0.f, 0.f, 0.f}};

    const int nstages = kb1 - kb0;
#pragma unroll
    for (int p = 0; p < DS_NS - 1; ++p)
        if (p < nstages)
            issue_stage(p, kb0 + p);
    int slot = 0;
    for (int s = 0; s < nstages; ++s) {
        // loads complete in order: this wave's copies of stage s have landed once at most those of the
        // younger stages in flight are outstanding
        const int younger = nstages - 1 - s < DS_NS - 2 ? nstages - 1 - s : DS_NS - 2;
        switch (younger) {
        case 0: ds_wait_vmcnt<0>(); break;
        case 1: ds_wait_vmcnt<DS_COPIES>(); break;
        case 2: ds_wait_vmcnt<2 * DS_COPIES>(); break;
        case 3: ds_wait_vmcnt<3 * DS_COPIES>(); break;
        default: ds_wait_vmcnt<4 * DS_COPIES>(); break;
        }
        __syncthreads();  // everyone's copies of stage s landed; the slot of stage s - 1 is no longer read
        if (s + DS_NS - 1 < nstages)
            issue_stage(slot == 0 ? DS_NS - 1 : slot - 1, kb0 + s + DS_NS - 1);
        const uint32_t so = (uint32_t)(slot * DS_STAGE);
        const v8i fb = read_frag(so + addr_b, 32 * 128);
        const float sb = *LDS_PTR(float, lds + so + DS_SB_OFF);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (i < mtiles) {
                const v8i fa = read_frag(so + addr_a + chunk_a[i], 32 * 32);
                const float sa = *LDS_PTR(float, lds + so + DS_SA_OFF + (16 * i + i16) * 4);
                const v4f blk = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                    fb, fa, (v4f){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                const float sc = sa * sb;
                acc[i] = (v4f){fmaf(sc, blk[0], acc[i][0]), fmaf(sc, blk[1], acc[i][1]),
                               fmaf(sc, blk[2], acc[i][2]), fmaf(sc, blk[3], acc[i][3])};
            }
        }
        slot = slot == DS_NS - 1 ? 0 : slot + 1;
    }

    // ---- a lane holds C[16*i + (lane & 15)][n0 + 16*wave + 4*(lane >> 4) + 0..3]
    const int ncol = n0 + 16 * wave + 4 * g4;
    auto store_c = [&](const v4f (&v)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int mrow = 16 * i + i16;
            if (mrow < M && ncol < N) {
                uint2 pk;
                pk.x = pack_bf16x2(v[i][0], v[i][1]);
                pk.y = pack_bf16x2(v[i][2], v[i][3]);
                *reinterpret_cast<uint2*>(c + (size_t)mrow * N + ncol) = pk;
            }
        }
    };
    if (ksplit == 1) {
        store_c(acc);
        return;
    }

    // ---- this wave's partial patch, in register order: [strip][split][wave][i][lane] x 16 bytes
    const size_t patch = ((size_t)(strip * ksplit) * 8 + wave) * 2;  // split 0; splits lie 16 patches apart
    v4f* mine = reinterpret_cast<v4f*>(partial) + (patch + (size_t)split * 16) * 64 + lane;
    mine[0] = acc[0];
    mine[64] = acc[1];
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // acknowledged by the L2 this XCD's workgroups share
    unsigned int ticket = 0;
    if (lane == 0)
        ticket = __builtin_amdgcn_atomic_inc32(tickets + strip * 8 + wave, (unsigned int)(ksplit - 1),
                                               __ATOMIC_RELAXED, "workgroup");
    ticket = (unsigned int)__builtin_amdgcn_readfirstlane((int)ticket);
    if (ticket != (unsigned int)(ksplit - 1))
        return;
    // last to arrive for these 16 columns: every split's patch is in L2
    const uint32_t span = (uint32_t)ksplit * 16u * 64u * 16u;  // bytes from this wave's split-0 patch to past its last
    const __amdgpu_buffer_rsrc_t rp = make_rsrc(reinterpret_cast<const v4f*>(partial) + patch * 64, span);
    // Every load goes out before the first sum.  A split past the last reads outside the resource, which
    // fetches nothing.  (Taking this wave's own patch from its registers instead of loading it back was
    // measured slower, 4 000 against 3 200 clocks for this phase.)
    v4f sum[2] = {(v4f){0.f, 0.f, 0.f, 0.f}, (v4f){0.f, 0.f, 0.f, 0.f}};
    auto gather = [&](auto nz_tag) __attribute__((always_inline)) {
        constexpr int NZ = decltype(nz_tag)::value;
        v4i v[NZ][2];
#pragma unroll
        for (int z = 0; z < NZ; ++z)
#pragma unroll
            for (int i = 0; i < 2; ++i)
                v[z][i] = __builtin_amdgcn_raw_buffer_load_b128(rp, (uint32_t)((z * 16 + i) * 64 + lane) * 16u, 0,
                                                                AUX_L1_MISS);
#pragma unroll
        for (int z = 0; z < NZ; ++z)
            if (z < ksplit) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const v4f f = __builtin_bit_cast(v4f, v[z][i]);
                    sum[i] = z == 0 ? f : sum[i] + f;
                }
            }
    };
    if (ksplit <= 4)
        gather(std::integral_constant<int, 4>{});
    else if (ksplit <= 8)
        gather(std::integral_constant<int, 8>{});
    else
        gather(std::integral_constant<int, DECODE_MAX_KSPLIT>{});
    store_c(sum);
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

}  // namespace

bool decode_strip_supports(const GemmArgs& g)
{
    return g.m <= 32 && g.m % 16 == 0 && g.n % 16 == 0 && (g.lda == 0 || g.lda == g.m) &&
           (g.n + DS_BN - 1) / DS_BN * 8 <= DECODE_TICKET_WORDS &&
           (reinterpret_cast<uintptr_t>(g.a) % 16 == 0) && (reinterpret_cast<uintptr_t>(g.b) % 16 == 0) &&
           (reinterpret_cast<uintptr_t>(g.a_scale) % 4 == 0) && (reinterpret_cast<uintptr_t>(g.c) % 8 == 0);
}

size_t decode_strip_partial_bytes(const GemmArgs& g, int ksplit)
{
    if (ksplit <= 1)
        return 0;
    const size_t strips = (size_t)(g.n + DS_BN - 1) / DS_BN;
    return strips * (size_t)ksplit * 8 * 2 * 64 * 16;
}

// Microseconds with B streamed from HBM, fitted to M = 16 and 32, N = 1536 ... 16384, K = 1536 ... 7168 and
// 1 to 16 K splits: a launch, then rounds of 256 workgroups, each workgroup living for a start-up, its
// K blocks (0.5 us per block when few workgroups pull on HBM, 0.76 us when 256 do) and, when K is split,
// the in-kernel reduction, whose last arrival reads one partial patch per split.
double decode_strip_cost(const GemmArgs& g, int ksplit)
{
    const int strips = (g.n + DS_BN - 1) / DS_BN;
    const int nkb = g.k / KBLOCK;
    const int kbs = (nkb + ksplit - 1) / ksplit;
    const long wgs = (long)strips * ksplit;
    const long rounds = (wgs + 255) / 256;
    const double active = wgs < 256 ? (double)wgs : 256.0;
    const double per_block = 0.50 + 0.001 * active;
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

hipError_t launch_decode_strips(const GemmArgs& g, int ksplit, float* partial, unsigned int* tickets, hipStream_t s)
{
    const int strips = (g.n + DS_BN - 1) / DS_BN;
    const int nkb = g.k / KBLOCK;
    if (!decode_strip_supports(g) || ksplit < 1 || ksplit > nkb || ksplit > DECODE_MAX_KSPLIT || (ksplit > 1 && (!partial || !tickets)))
        return hipErrorInvalidValue;
    const int kb_per_split = (nkb + ksplit - 1) / ksplit;
    if ((ksplit - 1) * kb_per_split >= nkb)  // every split owns at least one K block
        return hipErrorInvalidValue;
    const int groups = (strips + 7) / 8;
    auto kern = decode_strip_kernel;
    FP8GEMM_ALLOW_LDS(kern, DS_LDS);
    hipLaunchKernelGGL(kern, dim3(8 * groups * ksplit), dim3(DS_THREADS), DS_LDS, s, g.a, g.b, g.a_scale, g.b_scale,
                       g.c, partial, tickets, g.m, g.n, g.k, strips, ksplit, kb_per_split);
    return hipGetLastError();
}

}  // namespace fp8gemm
