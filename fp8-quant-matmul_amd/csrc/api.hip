// C ABI of the library (include/fp8_block_gemm.h): argument validation, kernel dispatch,
// split-K workspace.  The dispatcher is the run-time counterpart of the reference's
// compile-time kernel choice (#include "mn_large.hip" / "mn_small.hip", check.cu:13, and the
// OPTION macro, mn_large.hip:9) and of gemmGPU's grid arithmetic (check.cu:92-114).
#include "../../include/fp8_block_gemm.h"
#include "launchers.h"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <vector>

using namespace fp8gemm;

namespace {

constexpr int NUM_CU = 256;

// Process-wide defaults, set by fp8_block_gemm_select / _force_config / _set_persistent and read by
// the entry points without an options argument.  The _ex / _ws entry points read none of this.
std::atomic<int> g_selected{FP8GEMM_KERNEL_AUTO};
std::atomic<int> g_force_variant{-1};
std::atomic<int> g_force_ksplit{0};
std::atomic<int> g_persistent{-1};  // -1 = when tiles outnumber the CUs, 0 = never, 1 = whenever possible
std::atomic<int> g_fused{-1};       // K splits added inside the GEMM kernel: -1 = by cost, 0 = never, 1 = whenever possible
thread_local const char* t_last_kernel = "none";
thread_local char t_name_buf[96];

// what decides a plan besides the shape
struct Config {
    int selected;       // FP8GEMM_KERNEL_*
    int force_variant;  // tile shape, -1 = cost model
    int force_ksplit;   // 0 = cost model
    int persistent;     // -1 / 0 / 1 as above
    // plans that add K splits inside the kernel may be chosen: the workspace starts with a zeroed header
    // and the device places workgroups on XCDs as those kernels assume (set by run())
    bool fused_ok = true;
    int fused_mode = -1;  // -1 = by cost, 0 = never, 1 = whenever fused_ok and the plan allows
};
Config global_config()
{
    Config c{g_selected.load(), g_force_variant.load(), g_force_ksplit.load(), g_persistent.load()};
    c.fused_mode = g_fused.load();
    c.fused_ok = c.fused_mode != 0;
    return c;
}
constexpr int MAX_KSPLIT = 16;

// device memory a call may use beyond its operands: fp32 partial sums of plans that split K, padded
// copies of operands off the 16-byte grid
// The first WS_HEADER bytes belong to the kernels that add their K splits themselves and are zero before
// the first call and after every call: the mailbox through which the splits of a tile or strip hand over
// their partial results.  Plans keep their data behind it.
struct Workspace {
    float* ptr;
    size_t bytes;
    bool zeroed;  // the header was zero-filled when the buffer was taken on and only this library wrote to it since
};
constexpr size_t WS_HEADER = SPLIT_MAILBOX_BYTES;
static_assert(WS_HEADER == FP8GEMM_WORKSPACE_HEADER_BYTES, "the header size is part of the ABI");
inline float* ws_data(const Workspace& w) { return w.ptr ? reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(w.ptr) + WS_HEADER) : nullptr; }
inline float* ws_mailbox(const Workspace& w) { return w.ptr; }

std::mutex g_ws_mutex;
float* g_ws_own = nullptr;       // library-owned workspace
size_t g_ws_own_bytes = 0;
bool g_ws_own_captured = false;  // handed out to a call whose stream was being captured: a graph holds its address
hipStream_t g_ws_last_stream = nullptr;  // stream of the last call that was given the library-owned workspace
// Outgrown library-owned buffers.  Kernels of earlier calls may still use one: it is freed by a later
// growth once the event recorded behind its last use has completed.  One that a captured graph may hold
// (pinned) lives until fp8_block_gemm_release().
struct Retired {
    void* ptr;
    hipEvent_t done;  // nullptr when pinned
    bool pinned;
};
std::vector<Retired> g_ws_retired;
float* g_ws_user = nullptr;      // caller-supplied workspace
size_t g_ws_user_bytes = 0;
bool g_ws_user_zeroed = false;

// Size the library-owned workspace grows to when a call needs `need` bytes and `have` are there: at
// least double, so that the buffers retired on the way never add up to more than the live one.
size_t growth_target(size_t have, size_t need)
{
    if (need <= have)
        return have;
    const size_t twice = have > (SIZE_MAX >> 1) ? SIZE_MAX : 2 * have;
    return need > twice ? need : twice;
}

struct Plan {
    int family;   // FP8GEMM_KERNEL_*
    int variant;  // TileVariant for the tile families
    int ksplit;
    bool persistent = false;  // tile families, ksplit == 1: workgroups walk through the tiles
    bool padded = false;      // the plan is for the problem with m and n rounded up to 16 (run_padded)
    bool wide = false;        // decode family: 128-column strips, K splits added inside the kernel (k_decode.hip)
    bool fused = false;       // tile family, ksplit > 1: the last workgroup of a tile adds the partial tiles (no reduction launch)
    int halves = 1;           // wide decode strips: 128-column halves per strip (2 = 256-column strips)
};

// Shapes or addresses the MFMA kernels cannot take (m or n not a multiple of 16, a base not
// 16-byte aligned) run on padded copies in the workspace: which operands are copied, and where.
struct PadLayout {
    bool a, as, b, c;
    int m16, n16;
    size_t off_a, off_as, off_b, off_c, off_partial, total;
};

inline size_t round256(size_t x) { return (x + 255) & ~(size_t)255; }
inline bool misaligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; }

// conservative = true: every operand copied (an upper bound that does not depend on addresses).
// keeps_rows = the kernels of the plan take a leading dimension for a and a_scale apart from m
// (the tile kernels and the wide decode strips): c then needs no copy on account of m.
PadLayout pad_layout(const GemmArgs& g, size_t partial_bytes, bool conservative, bool keeps_rows)
{
    PadLayout L{};
    L.m16 = (g.m + 15) & ~15;
    L.n16 = (g.n + 15) & ~15;
    const bool rm = L.m16 != g.m, rn = L.n16 != g.n;
    L.a = conservative || rm || misaligned16(g.a);
    L.as = conservative || rm || misaligned16(g.a_scale);
    L.b = conservative || rn || misaligned16(g.b);
    L.c = conservative || (rm && !keeps_rows) || rn || misaligned16(g.c);
    const size_t nkb = (size_t)g.k / 128;
    size_t off = 0;
    L.off_a = off;
    off += L.a ? round256((size_t)g.k * L.m16) : 0;
    L.off_as = off;
    off += L.as ? round256(nkb * L.m16 * sizeof(float)) : 0;
    L.off_b = off;
    off += L.b ? round256((size_t)g.k * L.n16) : 0;
    L.off_c = off;
    off += L.c ? round256((size_t)L.m16 * L.n16 * 2) : 0;
    L.off_partial = off;
    off += partial_bytes;
    L.total = off;
    return L;
}

int validate(const void* a, const void* b, const float* as, const float* bs, const void* c, int m,
             int n, int k)
{
    if (!a || !b || !as || !bs || !c)
        return FP8GEMM_E_NULLPTR;
    if (m <= 0 || n <= 0 || k <= 0 || (k % 128) != 0)
        return FP8GEMM_E_SHAPE;
    const long long lim = 0x7FFFFFFFll;
    if ((long long)m * k > lim || (long long)n * k > lim || (long long)m * n > lim)
        return FP8GEMM_E_TOOLARGE;
    return FP8GEMM_OK;
}

// Estimated run time of a tile plan in microseconds.  The form is launch + rounds of 256
// workgroups x (pipeline fill + K blocks + store) + the split-K reduction; the constants are a
// least-squares fit to a sweep of every tile variant x ksplit over the 18 shapes of the
// reference's table (/root/reference/README.md:15-25) and the five benchmark shapes (rms
// error 10 %, the chosen plan within 6 % of the best measured one on all of them).
double tile_cost(const GemmArgs& g, int variant, int ksplit, bool fused = false)
{
    int bm, bn;
    tile_variant_dims(variant, &bm, &bn);
    const long tiles = (long)((g.m + bm - 1) / bm) * ((g.n + bn - 1) / bn);
    const int nkb = g.k / 128;
    const int kbs = (nkb + ksplit - 1) / ksplit;
    const double area = (double)bm * bn / 65536.0;
    // (the 256x256 tile measures 3-5 % ahead of 256x192 per flop where both fill their rounds; the fitted
    // line, extrapolated to its area, would put it 6 % ahead)
    // (a single row of tiles reads every byte of B once and from HBM -- decode weights do not fit the caches --,
    // where a K block takes a quarter longer than the fit to cached operands says: without this factor
    // 48 x 7168 x 1536 stays unsplit, 9.4 us from HBM against 8.1 us with two splits; the same for two rows of
    // to four rows of 64x64 tiles over a B of 16 MB or more, which they fetch in 64-byte pieces: 128 x 4096 x 7168
    // as tile64x64_k2f 22.2 us, as tile128x128_k7 17.1 us; 176 x 4608 x 4096 as tile64x64_k1 21.2 us from HBM and
    // 12.8 us with B in the Infinity Cache, as tile128x128_k3f 16.6 and 15.9 us -- while over 1536 x 7168
    // tile64x64_k5f stays ahead, 11.9 against 12.9 us)
    const bool streams_b = g.m <= 64 || (variant == TILE_64x64 && g.m <= 256 && (long long)g.n * g.k >= 16000000ll);
    // (with the splits added inside the kernel the grid holds a multiple of 8 tiles, so that the splits of a tile
    // share an XCD: the workgroups beyond the tiles exit at once but take their turn -- 85 tiles x 3 splits are
    // 264 workgroups, and the last of them start when a CU frees up: 20.2 us against 13.9 us with two splits)
    const long items = (ksplit > 1 && fused ? (tiles + 7) / 8 * 8 : tiles) * ksplit;
    // (a problem of at most 64 tiles of 64x64: a K block takes 0.265 us whether 4 or 64 tiles run -- M, N = 96 ... 512
    // with K = 1536 ... 8192 -- where the fit, made on launches of several rounds, says 0.34, and the hand-over of
    // the splits inside the kernel starts 0.3 us earlier.  Problems of 96 ... 256 such tiles measure as the fit
    // says, or slower.)
    const bool light = variant == TILE_64x64 && !streams_b && tiles <= 64;
    const double per_kb = (1.19 * area + 0.267) * (variant == TILE_256x256 ? 1.03 : 1.0) * (streams_b ? 1.25 : 1.0) *
                          (light ? 0.8 : 1.0);
    // (unsplit 128x192 tiles in more than one round of workgroups: the fit has them 8 % too fast against the 256-row
    // tiles -- 36 random shapes of 512 ... 8192 rows where that margin decides, before / after: the 256x256 or
    // 256x128 plan +5.6 % with B cached, +10.3 % with B from HBM on average, worst -2.3 %)
    const double in_rounds = variant == TILE_128x192 && ksplit == 1 && tiles > NUM_CU ? 1.08 : 1.0;
    const double per_item = 0.95 + 4.38 * area + kbs * per_kb * in_rounds;
    // (two 64x64 workgroups share a CU, but a single row of tiles with B from HBM is fastest with at most one
    // workgroup per CU: M = 48, 64 on 12 shapes, the split that keeps tiles x splits within 256 is the best
    // measured or within 2 % of it)
    const long rounds = (items + NUM_CU - 1) / NUM_CU;
    double cost = 1.79 + rounds * per_item;
    if (ksplit > 1 && fused)  // the last split of a tile waits for the others' accumulators and reads them
        cost += (light ? 1.5 : 1.8) + 0.35 * (ksplit - 1) * (double)(bm * bn) / 4096.0;
    else if (ksplit > 1) {  // second launch + partial write and read-back
        cost += 2.86 + (double)g.m * g.n * ksplit * 8.0 / 7.38e6;
        // (a GEMM kernel shorter than a launch takes cannot hide the reduction's launch behind it: two such kernels
        // take 9 - 9.5 us back to back whatever the split, 112 x 96 x 1536 ... 256 x 256 x 7168)
        const double first = rounds * per_item;
        cost += first < 4.5 ? 4.5 - first : 0.0;
    }
    return cost;
}

// The in-kernel reduction against the reduction kernel, measured on 11 shapes x 13 split plans (all
// bit-identical): the workgroup of a tile's last split reads the other splits' accumulators at the 15-20
// bytes per clock one CU takes in, so it pays while that is little -- 64x64 tiles (16 KB per split): 2-35 %
// faster up to 8 splits; 128x128 tiles (64 KB per split): 0-45 % faster with two or three splits unless
// only a handful of workgroups run (256 x 256 x 7168: 2-6 % slower) -- and loses beyond (128x128 with six
// splits +25 %, 256x192 up to 2 x), where the reduction kernel's 256 CUs read the partials together.
bool tile_fused_pays(const GemmArgs& g, int variant, int ksplit)
{
    if (variant == TILE_64x64)
        return ksplit <= 8;
    if (variant == TILE_128x128) {
        const long tiles = (long)((g.m + 127) / 128) * ((g.n + 127) / 128);
        return ksplit <= 3 && tiles * ksplit >= 64;
    }
    return false;
}

// whether a tile plan that splits K would add its splits inside the kernel
bool tile_plan_fused(const GemmArgs& g, int variant, int ksplit, const Config& cfg)
{
    if (ksplit <= 1 || !cfg.fused_ok || cfg.fused_mode == 0 || tile_mailbox_bytes(g, variant, ksplit) > SPLIT_MAILBOX_BYTES)
        return false;
    return cfg.fused_mode == 1 || tile_fused_pays(g, variant, ksplit);
}

// Shapes whose best measured plan differs from the model's choice: {m, n, k, variant, ksplit}.
struct TunedShape { int m, n, k, variant, ksplit; };
constexpr TunedShape kTuned[] = {
    {1024, 512, 7168, TILE_64x64, 2},
    {1024, 576, 7168, TILE_128x128, 4},
    {6144, 3072, 1536, TILE_256x192, 1},
    {8192, 7168, 2048, TILE_256x192, 1},
};

// tile shapes that exist in the persistent form only (and run only when asked for by number)
inline bool persistent_only(int variant) { return variant == TILE_256x192_W4 || variant == TILE_256x256; }
// ... of which the dispatcher may pick this one by itself
inline bool persistent_only_auto(int variant) { return variant == TILE_256x256; }

// A persistent launch pays off when a CU gets more than one tile.
void decide_persistent(const GemmArgs& g, Plan& p, const Config& cfg)
{
    p.persistent = false;
    const int mode = cfg.persistent;
    if (persistent_only(p.variant)) {
        p.persistent = p.ksplit == 1 && tile_persistent_supports(g, p.variant);
        return;
    }
    if (mode == 0 || p.ksplit != 1 || !tile_persistent_supports(g, p.variant))
        return;
    int bm, bn;
    tile_variant_dims(p.variant, &bm, &bn);
    const long tiles = (long)((g.m + bm - 1) / bm) * ((g.n + bn - 1) / bn);
    p.persistent = mode == 1 || tiles > NUM_CU;
}

// Whether a tile plan that splits K adds the partial tiles inside the GEMM kernel (the last workgroup of
// a tile to finish) or leaves them to the reduction kernel.
void decide_fused(const GemmArgs& g, Plan& p, const Config& cfg)
{
    p.fused = tile_plan_fused(g, p.variant, p.ksplit, cfg);
}

Plan compute_plan(const GemmArgs& g, const Config& cfg);

// The plan of a problem depends on its sizes, on the low address bits of its operands and on the switches: a
// serving loop asks for the same few again and again, and working one out costs a microsecond or two of host
// time (three are worked out per call), which is what a launch-bound decode loop runs on.  Each thread keeps the
// last plans it worked out, 64 slots indexed by a hash of the sizes.
struct PlanKey {
    int m, n, k, lda;
    uint32_t low_bits;  // 6 low address bits of a, b, a_scale, b_scale and c
    int selected, force_variant, force_ksplit, persistent, fused_mode;
    int fused_ok;
    bool operator==(const PlanKey& o) const
    {
        return m == o.m && n == o.n && k == o.k && lda == o.lda && low_bits == o.low_bits && selected == o.selected &&
               force_variant == o.force_variant && force_ksplit == o.force_ksplit && persistent == o.persistent &&
               fused_mode == o.fused_mode && fused_ok == o.fused_ok;
    }
};
struct PlanSlot {
    PlanKey key;
    Plan plan;
    bool used = false;
};
Plan make_plan(const GemmArgs& g, const Config& cfg)
{
    thread_local PlanSlot slots[64];
    auto low6 = [](const void* p) { return (uint32_t)(reinterpret_cast<uintptr_t>(p) & 63); };
    const PlanKey key{g.m, g.n, g.k, g.lda,
                      low6(g.a) | low6(g.b) << 6 | low6(g.a_scale) << 12 | low6(g.b_scale) << 18 | low6(g.c) << 24,
                      cfg.selected, cfg.force_variant, cfg.force_ksplit, cfg.persistent, cfg.fused_mode, cfg.fused_ok ? 1 : 0};
    const uint32_t h = ((uint32_t)g.m * 2654435761u) ^ ((uint32_t)g.n * 40503u) ^ ((uint32_t)g.k * 2246822519u) ^
                       (cfg.fused_ok ? 0x9E3779B9u : 0u);
    PlanSlot& slot = slots[(h >> 16 ^ h) & 63];
    if (slot.used && slot.key == key)
        return slot.plan;
    slot.plan = compute_plan(g, cfg);
    slot.key = key;
    slot.used = true;
    return slot.plan;
}

Plan compute_plan(const GemmArgs& g, const Config& cfg)
{
    const int selected = cfg.selected;
    Plan p{FP8GEMM_KERNEL_SCALAR, 0, 1};
    if (selected == FP8GEMM_KERNEL_SCALAR)
        return p;
    // The decode kernels (M <= 32): narrow strips (k_skinny.hip) or wide strips whose K splits are added
    // inside the kernel (k_decode.hip), whichever the cost model prefers; with the family asked for by name,
    // tile_variant 0 / 1 pins the narrow / wide form.  Under automatic dispatch the family has to hold its own
    // against the best tile plan by cost: with a long K range and many column strips 64x64 tiles with the K
    // range split are faster than the narrow kernel (measured: 12-14 us against 15-20 us for M = 16 / 32,
    // N >= 4608, K = 7168).
    Plan decode{FP8GEMM_KERNEL_SKINNY, 0, 1};
    double decode_us = -1.0;  // >= 0: the decode family is a candidate, at this cost
    const bool narrow_ok = skinny_supports(g), wide_ok = decode_strip_supports(g);
    if (selected == FP8GEMM_KERNEL_SKINNY && !narrow_ok && !wide_ok) {
        p.family = -1;
        return p;
    }
    if ((narrow_ok || wide_ok) && (selected == FP8GEMM_KERNEL_SKINNY || selected == FP8GEMM_KERNEL_AUTO)) {
        const int nkb = g.k / 128;
        const bool by_name = selected == FP8GEMM_KERNEL_SKINNY;
        auto valid_split = [&](int ks) { return ks >= 1 && ks <= nkb && (ks - 1) * ((nkb + ks - 1) / ks) < nkb; };
        int forced_ks = 0;
        if (cfg.force_ksplit > 0) {  // every split has to own at least one K block
            forced_ks = cfg.force_ksplit < nkb ? cfg.force_ksplit : nkb;
            while (!valid_split(forced_ks))
                --forced_ks;
        }
        double narrow_us = 1e300, wide_us = 1e300;
        Plan narrow = decode, wide = decode;
        wide.wide = true;
        if (narrow_ok && !(by_name && cfg.force_variant >= 1)) {
            narrow.ksplit = forced_ks ? forced_ks : skinny_ksplit(g);
            narrow_us = skinny_cost(g, narrow.ksplit);
        }
        if (wide_ok && (by_name ? cfg.force_variant != 0 : cfg.force_variant < 0)) {
            // without the in-kernel reduction (no zeroed mailbox, or workgroup placement not confirmed) only
            // the unsplit form exists.  By name, tile_variant 2 pins the 256-column strips.
            // Left to the cost model, 256-column strips have to be 7 % ahead where K is split: they halve the
            // workgroups of a split and win where that saves a round (144 strips x 3 splits are 54 workgroups on
            // an XCD's 32 CUs, 72 x 3 are 27: 18432 x 7168 from HBM 28.6 against 34.6 us), and lose 15 - 40 % on
            // cfg5-sized problems.  Unsplit launches stream, and there the wider strips are ahead throughout (a
            // projection onto a vocabulary with 8 rows, 131072 x 4096: 93.3 against 101.7 us; 16 x 49152 x 4096 in
            // one round of 192 workgroups 39.0 us, against 48.4 us in 384 strips of 128 columns).
            const int hi = cfg.fused_ok ? (nkb < MAX_KSPLIT ? nkb : MAX_KSPLIT) : 1;
            for (int halves = 1; halves <= 2; ++halves) {
                if (by_name ? halves != (cfg.force_variant == 2 ? 2 : 1) : cfg.force_variant >= 0 && halves == 2)
                    continue;
                for (int ks = 1; ks <= hi; ++ks) {
                    if (!valid_split(ks) || (forced_ks && ks != forced_ks) || !decode_strip_can_split(g, ks, halves))
                        continue;
                    const double cst =
                        decode_strip_cost(g, ks, halves) * (halves == 2 && !by_name && ks > 1 ? 1.07 : 1.0);
                    if (cst < wide_us) {
                        wide_us = cst;
                        wide.ksplit = ks;
                        wide.halves = halves;
                    }
                }
            }
        }
        // Decode weights come from HBM (a model's layers do not fit the caches): there the wide strips are
        // ahead of the narrow ones and of every tile plan on all 40 shapes measured (M = 16, 32; N = 1536 ...
        // 16384; K = 1536 ... 7168: 6.0-27 us against 7.3-60 us), although the narrow kernel is 1-2 us faster
        // on short K when B happens to sit in the Infinity Cache.  They need the in-kernel reduction.
        // With more than 32 rows the 64x64 tile plans that add their K splits in the kernel are ahead of the wide
        // strips on 22 of 24 shapes (M = 48, 64; same N and K; from HBM 6.2-15 us against 7.5-16 us): the
        // four-row-tile form is there for grouped launches and runs single problems only when asked for by name.
        // ... except where N x K is large (N = 7168, K >= 4096: 12.2 - 17.4 us against 13.7 - 20.4 us), and for row
        // counts off the 16-byte grid, which the strips take as they are while the tiles need padded copies
        // (M = 33 ... 63 on the same 12 shapes: 6.8 - 16.9 us against 10.8 - 23.8 us).
        if (!by_name && g.m > 32 && g.m % 16 == 0 && !(g.n >= 6144 && (long long)g.n * g.k >= 28000000ll))
            wide_us = 1e300;

        if (!by_name && cfg.force_variant < 0 && cfg.force_ksplit <= 0 && wide_us < 1e300 && cfg.fused_ok)
            return wide;
        if (!by_name && !cfg.fused_ok)
            wide_us = 1e300;  // unsplit wide strips leave most CUs idle: the narrow kernel and the tile plans compete
        if (narrow_us == 1e300 && wide_us == 1e300) {
            if (by_name) {
                p.family = -1;
                return p;
            }
        } else {
            decode = wide_us < narrow_us ? wide : narrow;
            decode_us = wide_us < narrow_us ? wide_us : narrow_us;
            if (by_name || cfg.force_variant >= 0 || cfg.force_ksplit > 0 || !tile_supports(g))
                return decode;
            // one pass of one round of workgroups: nothing here is faster
            if (decode_us <= skinny_cost(g, 0))
                return decode;
        }
    }
    if (!tile_supports(g)) {
        if (selected != FP8GEMM_KERNEL_AUTO) {
            p.family = -1;
            return p;
        }
        // rows without 16-byte alignment: the padded problem (its one or two extra launches cost
        // about 5 us; the scalar kernel, one dependent load after the other, takes 30 us for
        // K = 128 already), unless padding pushes an operand past the size limit
        const long long m16 = (g.m + 15) & ~15, n16 = (g.n + 15) & ~15, lim = 0x7FFFFFFFll;
        if (m16 * g.k > lim || n16 * g.k > lim || m16 * n16 > lim)
            return p;
        const uint8_t* const al8 = reinterpret_cast<const uint8_t*>(uintptr_t(4096));
        GemmArgs gp{al8, al8, reinterpret_cast<const float*>(uintptr_t(4096)), g.b_scale,
                    reinterpret_cast<uint16_t*>(uintptr_t(4096)), (int)m16, (int)n16, g.k};
        p = make_plan(gp, cfg);
        p.padded = p.family != FP8GEMM_KERNEL_SCALAR && p.family >= 0;
        return p;
    }
    const int fv = cfg.force_variant, fk = cfg.force_ksplit;
    const int nkb = g.k / 128;
    if (selected == FP8GEMM_KERNEL_AUTO && fv < 0 && fk <= 0)
        for (const TunedShape& t : kTuned)
            if (t.m == g.m && t.n == g.n && t.k == g.k) {
                p.family = t.ksplit > 1 ? FP8GEMM_KERNEL_SPLITK : FP8GEMM_KERNEL_LARGE;
                p.variant = t.variant;
                p.ksplit = t.ksplit;
                decide_persistent(g, p, cfg);
                decide_fused(g, p, cfg);
                return p;
            }
    double best = 1e300, best_256x128 = 1e300;
    int ks_256x128 = 1;
    for (int v = 0; v < TILE_VARIANT_COUNT; ++v) {
        if (fv >= 0 && v != fv)
            continue;
        if (tile_variant_name(v)[4] == '?')
            continue;
        if (persistent_only(v) && fv != v) {
            // the one-wave-per-SIMD form: only when asked for; the 256x256 tile: when its persistent form can
            // run (a ring's worth of K blocks) and the persistent kernel is not switched off
            if (!persistent_only_auto(v) || cfg.persistent == 0 || !tile_persistent_supports(g, v) ||
                selected == FP8GEMM_KERNEL_SPLITK)
                continue;
        }
        if (g.m <= 64 && fv < 0 && selected == FP8GEMM_KERNEL_AUTO && v != TILE_64x64)
            continue;  // a single row of tiles: taller tiles only multiply rows that do not exist
        for (int ks = 1; ks <= MAX_KSPLIT && ks <= nkb; ++ks) {
            if (persistent_only(v) && ks != 1)
                continue;
            if (fk > 0 && ks != (fk < nkb ? fk : nkb))
                continue;
            if (selected == FP8GEMM_KERNEL_LARGE && ks != 1)
                continue;
            if (selected == FP8GEMM_KERNEL_SPLITK && ks == 1 && nkb > 1)
                continue;
            // every split must own at least one K block
            const int kbs = (nkb + ks - 1) / ks;
            if ((ks - 1) * kbs >= nkb)
                continue;
            // a single row of tiles: the fitted constants overrate a split into short K ranges (measured for
            // M = 16 ... 64: with the reduction kernel the best split never leaves a workgroup fewer than 8 K
            // blocks; with the splits added inside the kernel, never fewer than 3)
            if (g.m <= 64 && fk <= 0 && selected == FP8GEMM_KERNEL_AUTO && ks > 1 &&
                kbs < (tile_plan_fused(g, v, ks, cfg) ? 3 : 8))
                continue;
            // 128x128 tiles that add their splits inside the kernel hand over 64 KB per split: with fewer than 8 K
            // blocks per workgroup that costs more than the split saves (27 shapes with K = 1536, 96 ... 128 tiles,
            // two splits of 6 blocks against unsplit: 10 - 28 % slower with B cached, -2 ... +15 % from HBM)
            if (v == TILE_128x128 && ks > 1 && kbs < 8 && fk <= 0 && selected == FP8GEMM_KERNEL_AUTO &&
                tile_plan_fused(g, v, ks, cfg))
                continue;
            const double cst = tile_cost(g, v, ks, tile_plan_fused(g, v, ks, cfg));
            if (cst < best) {
                best = cst;
                p.family = ks > 1 ? FP8GEMM_KERNEL_SPLITK : FP8GEMM_KERNEL_LARGE;
                p.variant = v;
                p.ksplit = ks;
            }
            if (v == TILE_256x128 && cst < best_256x128) {
                best_256x128 = cst;
                ks_256x128 = ks;
            }
        }
    }
    if (decode_us >= 0.0 && decode_us <= 0.95 * best)  // measured: at equal estimates the decode kernel is ahead
        return decode;
    if (best == 1e300) {
        p.family = -1;
        return p;
    }
    // 129 ... 1536 rows over a B of 16 MB or more with a long K: 128-row tiles read B twice as often as 256-row
    // tiles.  Where the model takes 128x128 tiles with a 256x128 plan within 12 % of them, that plan -- mostly two
    // to four splits with the reduction kernel -- measures ahead with B cached and with B from HBM: 45 random
    // shapes of up to 256 rows over 32 MB or more all faster, by 12 and 17 % on average; 56 more of up to 512 rows
    // or 18 ... 32 MB with K >= 4096: +8.3 and +6.4 % on average, worst -3.8 % (K = 3072, where an unsplit 128x128
    // plan would give way to three splits, loses 4 - 10 % and is left out); 49 of 528 ... 1536 rows: +7.4 and +6.1 %, worst
    // -3.0 %.  The same where the model takes a 128x192 plan with splits: 56 shapes, +3.6 and +7.4 %, worst -4.6 %.
    if (selected == FP8GEMM_KERNEL_AUTO && fv < 0 && fk <= 0 && (p.variant == TILE_128x128 || p.variant == TILE_128x192) && g.m > 128 && g.m <= 1536 &&
        g.k >= 4096 && (long long)g.n * g.k >= 16000000ll && best_256x128 <= 1.12 * best) {
        p.variant = TILE_256x128;
        p.ksplit = ks_256x128;
        p.family = p.ksplit > 1 ? FP8GEMM_KERNEL_SPLITK : FP8GEMM_KERNEL_LARGE;
    }
    // The same rows where the model takes the 128x192 tile: one row of 256x128 tiles streams B once where the 128x192 tile
    // the fit to cached operands prefers reads it twice.  With B from HBM -- which is what such a B is in a
    // model -- the taller tile is 2 - 13 % ahead on 22 random shapes (208 x 18816 x 3072: +12.8 %), with B in the
    // Infinity Cache -5 ... +4 %; with more rows (two to four tile rows against four to eight) the two are level.
    if (selected == FP8GEMM_KERNEL_AUTO && fv < 0 && fk <= 0 && p.variant == TILE_128x192 && p.ksplit == 1 &&
        g.m <= 256 && (long long)g.n * g.k >= 32000000ll && (g.n + 127) / 128 <= NUM_CU)
        p.variant = TILE_256x128;
    decide_persistent(g, p, cfg);
    decide_fused(g, p, cfg);
    if (persistent_only(p.variant) && !p.persistent)
        p.family = -1;
    return p;
}

// The process-wide workspace for a call on `stream` that needs `bytes`: the caller-supplied one, else
// the library-owned one, grown on demand (growth_target).  Growing allocates, which a stream under
// capture does not allow (and which would leave the graph with a buffer it was not recorded with): such
// a call gets FP8GEMM_E_WORKSPACE and the capture stays valid.  An outgrown buffer is retired, not
// freed on the spot: kernels in flight may still use it.
int acquire_workspace(size_t bytes, hipStream_t stream, Workspace* out)
{
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if (g_ws_user) {
        if (g_ws_user_bytes < bytes)
            return FP8GEMM_E_WORKSPACE;
        *out = Workspace{g_ws_user, g_ws_user_bytes, g_ws_user_zeroed};
        return FP8GEMM_OK;
    }
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    hipError_t e = hipStreamIsCapturing(stream, &status);
    if (e != hipSuccess)
        return (int)e;
    const bool capturing = status != hipStreamCaptureStatusNone;
    if (g_ws_own_bytes < bytes) {
        if (capturing)
            return FP8GEMM_E_WORKSPACE;
        // retired buffers whose last use has completed go back to the allocator now
        for (size_t i = 0; i < g_ws_retired.size();) {
            Retired& r = g_ws_retired[i];
            if (!r.pinned && hipEventQuery(r.done) == hipSuccess) {
                (void)hipEventDestroy(r.done);
                (void)hipFree(r.ptr);
                g_ws_retired.erase(g_ws_retired.begin() + (long)i);
            } else {
                ++i;
            }
        }
        (void)hipGetLastError();  // hipEventQuery reports "not ready" as an error
        size_t want = growth_target(g_ws_own_bytes, bytes);
        void* p = nullptr;
        e = hipMalloc(&p, want);
        if (e != hipSuccess && want > bytes) {
            (void)hipGetLastError();
            want = bytes;
            e = hipMalloc(&p, want);
        }
        if (e != hipSuccess)
            return (int)e;
        e = hipMemset(p, 0, WS_HEADER);  // the mailbox (bytes >= WS_HEADER whenever a plan needs a workspace)
        if (e != hipSuccess) {
            (void)hipFree(p);
            return (int)e;
        }
        if (g_ws_own) {
            Retired r{g_ws_own, nullptr, g_ws_own_captured};
            if (!r.pinned) {
                if (hipEventCreateWithFlags(&r.done, hipEventDisableTiming) != hipSuccess ||
                    hipEventRecord(r.done, g_ws_last_stream) != hipSuccess) {
                    (void)hipGetLastError();
                    if (r.done)
                        (void)hipEventDestroy(r.done);
                    r.done = nullptr;
                    r.pinned = true;  // no way to tell when its last use ends: kept until release
                }
            }
            g_ws_retired.push_back(r);
        }
        g_ws_own = static_cast<float*>(p);
        g_ws_own_bytes = want;
        g_ws_own_captured = false;
    }
    g_ws_own_captured = g_ws_own_captured || capturing;
    g_ws_last_stream = stream;
    *out = Workspace{g_ws_own, g_ws_own_bytes, true};
    return FP8GEMM_OK;
}

// bytes of partial sums a plan keeps behind the workspace header
size_t plan_workspace_bytes(const GemmArgs& g, const Plan& p)
{
    // splits that are added inside the kernel meet in the header
    if (p.ksplit <= 1 || (p.family == FP8GEMM_KERNEL_SKINNY && p.wide) || p.fused)
        return 0;
    return (size_t)p.ksplit * g.m * g.n * sizeof(float);
}
// whether a plan uses the header although it keeps nothing behind it
inline bool plan_uses_header(const Plan& p) { return p.ksplit > 1 && ((p.family == FP8GEMM_KERNEL_SKINNY && p.wide) || p.fused); }
// a workspace that holds `data` bytes of a plan: nothing, or the header and the data
inline size_t with_header(size_t data, bool header_alone = false) { return data || header_alone ? data + WS_HEADER : 0; }

void plan_name(const Plan& p, char* out, size_t cap)
{
    const char* pre = p.padded ? "padded_" : "";
    if (p.family == FP8GEMM_KERNEL_SCALAR)
        snprintf(out, cap, "scalar");
    else if (p.family == FP8GEMM_KERNEL_SKINNY)
        snprintf(out, cap, p.wide ? (p.halves == 2 ? "%sdecode256_k%d" : "%sdecode128_k%d") : "%sskinny_k%d", pre, p.ksplit);
    else
        snprintf(out, cap, "%s%s_k%d%s", pre, tile_variant_name(p.variant), p.ksplit,
                 p.persistent ? "_persistent" : (p.fused ? "f" : ""));
}

// the kernels of a plan on operands they can take; `partial` holds plan_workspace_bytes, `w` is the
// workspace whose zeroed header the plans use that add their K splits inside the kernel
hipError_t launch_plan(const GemmArgs& g, const Plan& p, float* partial, const Workspace& w, hipStream_t stream)
{
    switch (p.family) {
    case FP8GEMM_KERNEL_SCALAR:
        return launch_scalar(g, stream);
    case FP8GEMM_KERNEL_SKINNY:
        if (p.wide)
            return launch_decode_strips(g, p.ksplit, p.halves, ws_mailbox(w), stream);
        return launch_skinny(g, p.ksplit, partial, stream);
    default: {
        if (p.persistent)
            return launch_tile_persistent(g, p.variant, NUM_CU, stream);
        hipError_t e = launch_tile(g, p.variant, p.ksplit, partial, p.fused ? ws_mailbox(w) : nullptr, stream);
        if (e == hipSuccess && p.ksplit > 1 && !p.fused)
            e = launch_splitk_reduce(g, p.ksplit, partial, stream);
        return e;
    }
    }
}

// pad what needs padding into the workspace, run the plan there, copy C's corner out
// bytes run_padded needs for this call (depends on which operands are off the grid)
size_t padded_bytes(const GemmArgs& g, const Plan& p)
{
    GemmArgs gp = g;
    gp.m = (g.m + 15) & ~15;
    gp.n = (g.n + 15) & ~15;
    const bool keeps_rows = p.family == FP8GEMM_KERNEL_LARGE || p.family == FP8GEMM_KERNEL_SPLITK ||
                            (p.family == FP8GEMM_KERNEL_SKINNY && p.wide);
    return with_header(pad_layout(g, plan_workspace_bytes(gp, p), false, keeps_rows).total, plan_uses_header(p));
}

int run_padded(const GemmArgs& g, const Plan& p, const Workspace& w, hipStream_t stream)
{
    GemmArgs gp = g;
    const int m16 = (g.m + 15) & ~15;
    gp.m = m16;
    gp.n = (g.n + 15) & ~15;
    const bool keeps_rows = p.family == FP8GEMM_KERNEL_LARGE || p.family == FP8GEMM_KERNEL_SPLITK ||
                            (p.family == FP8GEMM_KERNEL_SKINNY && p.wide);
    const PadLayout L = pad_layout(g, plan_workspace_bytes(gp, p), false, keeps_rows);
    if (!L.c) {  // c is written in place: its m rows, while a and a_scale have m16 per k-row
        gp.m = g.m;
        gp.lda = m16;
    }
    if (!w.ptr || w.bytes < with_header(L.total))
        return FP8GEMM_E_WORKSPACE;
    uint8_t* base = reinterpret_cast<uint8_t*>(ws_data(w));
    const int nkb = g.k / 128;
    // every operand that needs a padded copy, in one launch
    PadJobs jobs;
    jobs.count = 0;
    if (L.a) {
        jobs.job[jobs.count++] = PadJob{g.a, base + L.off_a, g.k, g.m, m16, 0};
        gp.a = base + L.off_a;
    }
    if (L.as) {
        float* as = reinterpret_cast<float*>(base + L.off_as);
        jobs.job[jobs.count++] = PadJob{g.a_scale, as, nkb, g.m, m16, 1};
        gp.a_scale = as;
    }
    if (L.b) {
        jobs.job[jobs.count++] = PadJob{g.b, base + L.off_b, g.k, g.n, gp.n, 0};
        gp.b = base + L.off_b;
    }
    hipError_t e = launch_pad_jobs(jobs, stream);
    if (L.c)
        gp.c = reinterpret_cast<uint16_t*>(base + L.off_c);
    if (e == hipSuccess)
        e = launch_plan(gp, p, reinterpret_cast<float*>(base + L.off_partial), w, stream);
    if (e == hipSuccess && L.c)
        e = launch_crop_bf16(gp.c, g.c, g.m, g.n, gp.n, stream);
    return (int)e;
}

// Whether plans that add their K splits inside the kernel may run for a call on `stream`: the device
// must place workgroups on XCDs as those kernels assume.  The first call on a device finds out with a
// probe grid that it waits for; while `stream` is being captured nothing is probed and an unknown
// placement counts as "no".
bool placement_ok(hipStream_t stream)
{
    int known = xcd_placement_confirmed(false);
    if (known >= 0)
        return known == 1;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess || status != hipStreamCaptureStatusNone)
        return false;
    return xcd_placement_confirmed(true) == 1;
}

// One GEMM.  explicit_ws = the caller's per-call workspace (its bytes may be 0 / its pointer NULL when the
// plan needs none); nullptr = the process-wide workspace.
int run(const void* a, const void* b, const float* as, const float* bs, void* c, int m, int n, int k,
        hipStream_t stream, Config cfg, const Workspace* explicit_ws)
{
    int v = validate(a, b, as, bs, c, m, n, k);
    if (v != FP8GEMM_OK)
        return v;
    GemmArgs g{static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), as, bs,
               static_cast<uint16_t*>(c), m, n, k};
    // in-kernel K-split reduction: a zeroed header (every process-wide workspace has one; a per-call
    // one when the caller says so) and a confirmed workgroup placement
    cfg.fused_ok = cfg.fused_ok && (!explicit_ws || explicit_ws->zeroed);
    if (cfg.fused_ok) {
        Config probe = cfg;
        probe.fused_ok = false;
        const Plan with = make_plan(g, cfg), without = make_plan(g, probe);
        const bool differs = with.family != without.family || with.ksplit != without.ksplit ||
                             with.wide != without.wide || with.fused != without.fused || with.halves != without.halves;
        if (differs && !placement_ok(stream))
            cfg.fused_ok = false;
    }
    Plan p = make_plan(g, cfg);
    if (p.family < 0)
        return FP8GEMM_E_KERNEL;
    Workspace w{nullptr, 0, false};
    for (int attempt = 0;; ++attempt) {
        const size_t need = p.padded ? padded_bytes(g, p) : with_header(plan_workspace_bytes(g, p), plan_uses_header(p));
        int rc = FP8GEMM_OK;
        if (need) {
            if (explicit_ws) {
                if (!explicit_ws->ptr || explicit_ws->bytes < need ||
                    (reinterpret_cast<uintptr_t>(explicit_ws->ptr) % 256) != 0)
                    rc = FP8GEMM_E_WORKSPACE;
                else
                    w = *explicit_ws;
            } else {
                rc = acquire_workspace(need, stream, &w);
            }
        }
        if (rc == FP8GEMM_OK)
            break;
        // A plan that adds its K splits inside the kernel needs the header; when the workspace at hand cannot
        // hold it (a small caller-owned buffer, or none while the stream is being captured) the plan without
        // it may still run -- cfg1-like shapes then need no workspace at all.  Not when that form was asked for.
        if (rc != FP8GEMM_E_WORKSPACE || attempt > 0 || !cfg.fused_ok || cfg.fused_mode == 1 || !plan_uses_header(p))
            return rc;
        cfg.fused_ok = false;
        p = make_plan(g, cfg);
        if (p.family < 0)
            return FP8GEMM_E_WORKSPACE;
    }
    const int rc = p.padded ? run_padded(g, p, w, stream) : (int)launch_plan(g, p, ws_data(w), w, stream);
    if (rc == FP8GEMM_OK) {
        plan_name(p, t_name_buf, sizeof(t_name_buf));
        t_last_kernel = t_name_buf;
    }
    return rc;
}

// ---- the entry point that allocates nothing: its workspace is this array, part of the library's device
// image (every GPU the library runs on holds its own copy, at its own address, until the process
// ends).  In host code the array's name is only a handle for hipGetSymbolAddress: the device address is
// looked up once per device, with that device current, and everything else uses that pointer.
static __device__ __align__(256) unsigned char scratch[FP8GEMM_NOALLOC_MAX_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[MAX_DEVICES] = {};

int scratch_for_current_device(void** out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES)
        return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess)
            return (int)e;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return FP8GEMM_OK;
}

// the tiles of a grouped launch: every group starts a tile row of its own
long grouped_tiles(const GroupTable& tab, int n, int variant)
{
    int bm, bn;
    tile_variant_dims(variant, &bm, &bn);
    long rows = 0;
    for (int g = 0; g < tab.groups; ++g)
        rows += (tab.m[g] + bm - 1) / bm;
    return rows * ((n + bn - 1) / bn);
}

// Estimated run time of a grouped tile launch in microseconds: tile_cost's form -- launch + rounds of 256
// workgroups x (fill + K blocks + store) -- on the launch's own tile count, with a K block priced for operands
// that come from HBM: every group brings its own B, and a tile row of a group reads all of it, so the launch
// moves more bytes per flop than the single problems tile_cost was fitted on, the more the smaller the tile.
// Factors on the K block from 25 launches (1 ... 64 groups of 65 ... 3000 rows, N = 1536 ... 7168, K = 2048 and
// 7168, every tile shape pinned): 1.12 for 256x256, 1.5 for 256x192 and 256x128, 1.7 for 128x192 and 128x128 --
// e.g. 8 groups of 300 ... 3000 rows, 4608 x 7168: 498 / 610 / 680 / 775 / 893 us estimated for 256x256 / 256x192 /
// 256x128 / 128x192 / 128x128, 515 / 615 / 727 / 875 / 1042 us measured; 4 groups of 65 ... 256 rows, 7168 x 2048:
// 35 / 34 / 26 / 46 / 37 us estimated, 32 / 33 / 25 / 42 / 36 us measured.
double grouped_tile_cost(const GroupTable& tab, int n, int k, int variant)
{
    int bm, bn;
    tile_variant_dims(variant, &bm, &bn);
    const double area = (double)bm * bn / 65536.0;
    const double from_hbm = variant == TILE_256x256 ? 1.12 : bm == 256 ? 1.5 : 1.7;
    const double per_kb = (1.19 * area + 0.267) * (variant == TILE_256x256 ? 1.03 : 1.0) * from_hbm;
    const double per_item = 0.95 + 4.38 * area + (k / 128) * per_kb;
    const long rounds = (grouped_tiles(tab, n, variant) + NUM_CU - 1) / NUM_CU;
    return 1.79 + rounds * per_item;
}

// tile shape for a grouped launch: the cheapest by grouped_tile_cost among the shapes that have a grouped form
// (no K split); -1 when none can take the table
int grouped_variant(const GroupTable& tab, int n, int k, const Config& cfg)
{
    long long m_total = 0;
    for (int g = 0; g < tab.groups; ++g)
        m_total += tab.m[g];
    if (m_total > 0x7FFFFFFFll)
        return -1;
    int best_v = -1;
    double best = 1e300;
    const int fv = cfg.force_variant;
    for (int v = 0; v < TILE_VARIANT_COUNT; ++v) {
        if ((fv >= 0 && v != fv) || !tile_grouped_supports(tab, n, k, v))
            continue;
        if (fv < 0 && persistent_only(v) && !persistent_only_auto(v))
            continue;
        const double cst = grouped_tile_cost(tab, n, k, v);
        if (cst < best) {
            best = cst;
            best_v = v;
        }
    }
    return best_v;
}

// the workspace of a call: the caller's per-call one, else the process-wide one
int workspace_for(size_t need, hipStream_t stream, const Workspace* explicit_ws, Workspace* out)
{
    *out = Workspace{nullptr, 0, false};
    if (!need)
        return FP8GEMM_OK;
    if (explicit_ws) {
        if (!explicit_ws->ptr || explicit_ws->bytes < need || (reinterpret_cast<uintptr_t>(explicit_ws->ptr) % 256) != 0)
            return FP8GEMM_E_WORKSPACE;
        *out = *explicit_ws;
        return FP8GEMM_OK;
    }
    return acquire_workspace(need, stream, out);
}

// One grouped launch for the problems of `tab` (same n and k): the decode kernel when every group has at
// most 64 rows (decode = true), else the persistent tile kernel.  Groups off the 16-byte grid (n, or for the
// tile kernel m, not a multiple of 16; an operand off a 16-byte boundary) run on zero-padded copies in the
// workspace made by one batched copy launch per operand kind.  Returns GROUPED_NOT_APPLICABLE when it cannot run (the caller
// then takes the groups one by one).
constexpr int GROUPED_NOT_APPLICABLE = -1000;
int run_grouped_table(const GroupTable& tab, int n, int k, bool decode, hipStream_t s, const Config& cfg,
                      const Workspace* explicit_ws)
{
    const long long lim = 0x7FFFFFFFll;
    const int n16 = (n + 15) & ~15;
    const size_t nkb = (size_t)k / 128;
    bool pad_a = false, pad_b = n16 != n, pad_c = n16 != n;
    // The decode kernel takes row counts off the 16-byte grid as they are (it spreads A's packed slabs in the
    // LDS) and 4-byte aligned scales: measured on 2 to 64 groups of 1 - 64 rows, N = 1536 ... 7168, K = 2048 and
    // 7168, level with the padded copies (one more launch, then the plain kernel) or up to 20 % ahead.  Launches
    // large enough for the streaming form, which wants rows on the grid, are the exception: 9 % for one copy launch.
    const bool streams = decode && decode_grouped_streams(tab.groups, n16);
    for (int g = 0; g < tab.groups; ++g) {
        pad_a = pad_a || misaligned16(tab.a[g]) || (tab.m[g] % 16 != 0 && (!decode || streams)) ||
                (!decode && misaligned16(tab.a_scale[g]));
        pad_b = pad_b || misaligned16(tab.b[g]);
        pad_c = pad_c || misaligned16(tab.c[g]);
    }
    const bool padded = pad_a || pad_b || pad_c;
    size_t off_a[GroupTable::MAX_GROUPS], off_as[GroupTable::MAX_GROUPS], off_b[GroupTable::MAX_GROUPS],
        off_c[GroupTable::MAX_GROUPS];
    size_t off = 0;
    if (padded)
        for (int g = 0; g < tab.groups; ++g) {
            const long long m16 = (tab.m[g] + 15) & ~15;
            if (m16 * k > lim || (long long)n16 * k > lim || m16 * n16 > lim)
                return GROUPED_NOT_APPLICABLE;
            off_a[g] = off;
            off += round256((size_t)k * m16);
            off_as[g] = off;
            off += round256(nkb * m16 * sizeof(float));
            off_b[g] = off;
            off += pad_b ? round256((size_t)k * n16) : 0;
            off_c[g] = off;
            off += pad_c ? round256((size_t)m16 * n16 * 2) : 0;
        }
    // the problems as the GEMM kernel sees them (addresses in the workspace are filled in below): c in place
    // keeps its m rows, a and a_scale have m16 per k-row
    GroupTable pt = tab;
    if (padded)
        for (int g = 0; g < tab.groups; ++g) {
            const int m16 = (tab.m[g] + 15) & ~15;
            pt.m[g] = pad_c ? m16 : tab.m[g];
            pt.lda[g] = m16;
        }
    // decode kernel: K split by cost (it needs the zeroed mailbox and the XCD placement); tile kernel: none
    int ksplit = 1;
    int variant = -1;
    if (decode) {
        // placeholder addresses that pass the alignment checks while the real ones are not known yet
        GroupTable probe = pt;
        if (padded)
            for (int g = 0; g < tab.groups; ++g) {
                probe.a[g] = reinterpret_cast<const uint8_t*>(uintptr_t(4096));
                probe.a_scale[g] = reinterpret_cast<const float*>(uintptr_t(4096));
                if (pad_b)
                    probe.b[g] = reinterpret_cast<const uint8_t*>(uintptr_t(4096));
                if (pad_c)
                    probe.c[g] = reinterpret_cast<uint16_t*>(uintptr_t(4096));
            }
        if (!decode_grouped_supports(probe, n16, k))
            return GROUPED_NOT_APPLICABLE;
        bool fused_ok = cfg.fused_ok && (!explicit_ws || explicit_ws->zeroed);
        if (fused_ok && decode_grouped_ksplit(pt, n16, k, true) > 1)
            fused_ok = placement_ok(s);
        ksplit = cfg.force_ksplit > 0 && fused_ok ? cfg.force_ksplit : decode_grouped_ksplit(pt, n16, k, fused_ok);
        const int nkb_i = k / 128;
        while (ksplit > 1 && (ksplit > nkb_i || (ksplit - 1) * ((nkb_i + ksplit - 1) / ksplit) >= nkb_i))
            --ksplit;
        if (decode_grouped_mailbox_bytes(pt, n16, ksplit) > SPLIT_MAILBOX_BYTES)
            ksplit = 1;
    }
    Workspace w;
    const int wrc = workspace_for(with_header(off, ksplit > 1), s, explicit_ws, &w);
    if (wrc == FP8GEMM_E_WORKSPACE)
        return GROUPED_NOT_APPLICABLE;  // a workspace sized for single problems: one by one
    if (wrc != FP8GEMM_OK)
        return wrc;
    uint8_t* base = reinterpret_cast<uint8_t*>(ws_data(w));
    RepackTable ta, tas, tb, tc;
    ta.groups = tas.groups = tb.groups = tc.groups = tab.groups;
    if (padded)
        for (int g = 0; g < tab.groups; ++g) {
            const int m = tab.m[g], m16 = (m + 15) & ~15;
            pt.a[g] = base + off_a[g];
            pt.a_scale[g] = reinterpret_cast<const float*>(base + off_as[g]);
            pt.b[g] = pad_b ? base + off_b[g] : tab.b[g];
            pt.c[g] = pad_c ? reinterpret_cast<uint16_t*>(base + off_c[g]) : tab.c[g];
            ta.src[g] = tab.a[g], ta.dst[g] = base + off_a[g], ta.rows[g] = k, ta.ld_src[g] = m, ta.ld_dst[g] = m16;
            tas.src[g] = tab.a_scale[g], tas.dst[g] = base + off_as[g], tas.rows[g] = (int)nkb, tas.ld_src[g] = m,
            tas.ld_dst[g] = m16;
            tb.src[g] = tab.b[g], tb.dst[g] = base + off_b[g], tb.rows[g] = k, tb.ld_src[g] = n, tb.ld_dst[g] = n16;
            tc.src[g] = base + off_c[g], tc.dst[g] = tab.c[g], tc.rows[g] = m, tc.ld_src[g] = n16, tc.ld_dst[g] = n;
        }
    if (!decode) {
        variant = grouped_variant(pt, n16, k, cfg);
        if (variant < 0)
            return GROUPED_NOT_APPLICABLE;
        // A launch that leaves a third of the CUs without a tile while each tile walks a long K range: single
        // problems split K (one group of 200 x 4096 x 7168: 19 us against 52 us, two: 42 against 56 us; four groups
        // of 1536 x 7168: level; with K = 2048 one group 13.4 against 15.6 us, two 26 against 19 us).
        if (cfg.force_variant < 0 && tab.groups <= 8 && k >= 2048 && grouped_tiles(pt, n16, variant) < 160)
            return GROUPED_NOT_APPLICABLE;
    }
    hipError_t e = hipSuccess;
    if (padded) {
        e = launch_pad_pair_batched(ta, tas, s);
        if (e == hipSuccess && pad_b)
            e = launch_pad_bytes_batched(tb, s);
    }
    if (e == hipSuccess)
        e = decode ? launch_decode_grouped(pt, n16, k, ksplit, ws_mailbox(w), s)
                   : launch_tile_grouped(pt, n16, k, variant, NUM_CU, s);
    if (e == hipSuccess && pad_c)
        e = launch_crop_bf16_batched(tc, s);
    if (e == hipSuccess) {
        if (decode)
            snprintf(t_name_buf, sizeof(t_name_buf), "%sdecode128_k%d_grouped%d", padded ? "padded_" : "", ksplit, tab.groups);
        else
            snprintf(t_name_buf, sizeof(t_name_buf), "%s%s_k1_grouped%d", padded ? "padded_" : "", tile_variant_name(variant),
                     tab.groups);
        t_last_kernel = t_name_buf;
    }
    return (int)e;
}

// nullptr = automatic dispatch; rc = FP8GEMM_OK when the options are usable
Config config_from_options(const fp8gemm_options* opt, int* rc)
{
    *rc = FP8GEMM_OK;
    if (!opt)
        return Config{FP8GEMM_KERNEL_AUTO, -1, 0, -1};
    if (opt->kernel < FP8GEMM_KERNEL_AUTO || opt->kernel > FP8GEMM_KERNEL_SKINNY ||
        opt->tile_variant >= TILE_VARIANT_COUNT || opt->ksplit < 0 || opt->ksplit > MAX_KSPLIT ||
        opt->persistent < -1 || opt->persistent > 1 || (opt->flags & ~FP8GEMM_FLAG_WORKSPACE_ZEROED) != 0)
        *rc = FP8GEMM_E_KERNEL;
    return Config{opt->kernel, opt->tile_variant < 0 ? -1 : opt->tile_variant, opt->ksplit, opt->persistent};
}

// aligned = the plan for 16-byte aligned operands; otherwise the larger of that and what the padded
// plan needs when every operand has to be copied
size_t workspace_bytes_for(int m, int n, int k, const Config& cfg_in, bool any_alignment)
{
    if (m <= 0 || n <= 0 || k <= 0 || (k % 128) != 0)
        return 0;
    const uintptr_t al = 4096;
    GemmArgs g{reinterpret_cast<const uint8_t*>(al), reinterpret_cast<const uint8_t*>(al),
               reinterpret_cast<const float*>(al), nullptr, reinterpret_cast<uint16_t*>(al), m, n, k};
    GemmArgs gp = g;
    gp.m = (m + 15) & ~15;
    gp.n = (n + 15) & ~15;
    size_t need = 0;
    // the larger need of the plans a call may settle on: with the K splits added inside the kernel, and
    // -- when the device turns out not to place workgroups as that needs -- with the reduction kernel
    for (int fused = 0; fused < 2; ++fused) {
        Config cfg = cfg_in;
        if (!fused)
            cfg.fused_ok = false;
        const Plan p = make_plan(g, cfg);
        size_t one = 0;
        if (p.family >= 0)
            one = with_header(p.padded ? pad_layout(g, plan_workspace_bytes(gp, p), true, false).total
                                       : plan_workspace_bytes(g, p), plan_uses_header(p));
        if (any_alignment && !(p.family >= 0 && p.padded)) {
            // the same shape with an operand off a 16-byte boundary: the plan of the padded shape on copies
            const long long lim = 0x7FFFFFFFll;
            if ((long long)gp.m * k <= lim && (long long)gp.n * k <= lim && (long long)gp.m * gp.n <= lim &&
                cfg.selected != FP8GEMM_KERNEL_SCALAR) {
                const Plan pp = make_plan(gp, cfg);
                if (pp.family >= 0 && pp.family != FP8GEMM_KERNEL_SCALAR) {
                    const size_t all = with_header(pad_layout(g, plan_workspace_bytes(gp, pp), true, false).total,
                                                   plan_uses_header(pp));
                    one = all > one ? all : one;
                }
            }
        }
        need = one > need ? one : need;
    }
    return need;
}

}  // namespace

extern "C" {

int fp8_block_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale, void* c,
                   int m, int n, int k)
{
    return run(a, b, a_scale, b_scale, c, m, n, k, nullptr, global_config(), nullptr);
}

int fp8_block_gemm_stream(const void* a, const void* b, const float* a_scale, const float* b_scale,
                          void* c, int m, int n, int k, void* stream)
{
    return run(a, b, a_scale, b_scale, c, m, n, k, static_cast<hipStream_t>(stream), global_config(), nullptr);
}

int fp8_block_gemm_ex(const void* a, const void* b, const float* a_scale, const float* b_scale, void* c,
                      int m, int n, int k, const fp8gemm_options* options, void* workspace,
                      size_t workspace_bytes, void* stream)
{
    int rc;
    const Config cfg = config_from_options(options, &rc);
    if (rc != FP8GEMM_OK)
        return rc;
    const bool zeroed = options && (options->flags & FP8GEMM_FLAG_WORKSPACE_ZEROED) != 0;
    const Workspace w{static_cast<float*>(workspace), workspace ? workspace_bytes : 0, zeroed};
    return run(a, b, a_scale, b_scale, c, m, n, k, static_cast<hipStream_t>(stream), cfg, &w);
}

int fp8_block_gemm_ws(const void* a, const void* b, const float* a_scale, const float* b_scale, void* c,
                      int m, int n, int k, void* workspace, size_t workspace_bytes, void* stream)
{
    return fp8_block_gemm_ex(a, b, a_scale, b_scale, c, m, n, k, nullptr, workspace, workspace_bytes, stream);
}

int fp8_block_gemm_noalloc(const void* a, const void* b, const float* a_scale, const float* b_scale, void* c,
                           int m, int n, int k, void* stream)
{
    // arguments first (no device call), then the plan's need against the fixed size: a plan that does
    // not fit is refused here, with the code a too small workspace always gets
    const int v = validate(a, b, a_scale, b_scale, c, m, n, k);
    if (v != FP8GEMM_OK)
        return v;
    const Config cfg = global_config();
    const GemmArgs g{static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), a_scale, b_scale,
                     static_cast<uint16_t*>(c), m, n, k};
    // the largest need among the plans run() may settle on (with and without the in-kernel reduction)
    size_t need = 0;
    for (int fused = 0; fused < 2; ++fused) {
        Config probe = cfg;
        probe.fused_ok = fused != 0;
        const Plan p = make_plan(g, probe);
        if (p.family < 0)
            return FP8GEMM_E_KERNEL;
        const size_t bytes = p.padded ? padded_bytes(g, p) : with_header(plan_workspace_bytes(g, p), plan_uses_header(p));
        need = bytes > need ? bytes : need;
    }
    if (need > (size_t)FP8GEMM_NOALLOC_MAX_BYTES)
        return FP8GEMM_E_WORKSPACE;
    void* ptr = nullptr;
    const int rc = scratch_for_current_device(&ptr);
    if (rc != FP8GEMM_OK)
        return rc;
    // the array starts out zero and every kernel that uses the header leaves it zero
    const Workspace w{static_cast<float*>(ptr), (size_t)FP8GEMM_NOALLOC_MAX_BYTES, true};
    return run(a, b, a_scale, b_scale, c, m, n, k, static_cast<hipStream_t>(stream), cfg, &w);
}

int fp8_block_gemm_scalar(const void* a, const void* b, const float* a_scale, const float* b_scale,
                          void* c, int m, int n, int k, void* stream)
{
    return run(a, b, a_scale, b_scale, c, m, n, k, static_cast<hipStream_t>(stream),
               Config{FP8GEMM_KERNEL_SCALAR, -1, 0, -1}, nullptr);
}

int fp8_block_gemm_select(int kernel_id)
{
    if (kernel_id < FP8GEMM_KERNEL_AUTO || kernel_id > FP8GEMM_KERNEL_SKINNY)
        return FP8GEMM_E_KERNEL;
    g_selected.store(kernel_id);
    return FP8GEMM_OK;
}

int fp8_block_gemm_force_config(int tile_variant, int ksplit)
{
    if (tile_variant >= TILE_VARIANT_COUNT || ksplit < 0 || ksplit > MAX_KSPLIT)
        return FP8GEMM_E_KERNEL;
    g_force_variant.store(tile_variant < 0 ? -1 : tile_variant);
    g_force_ksplit.store(ksplit);
    return FP8GEMM_OK;
}

// Grouped GEMM behind both entry points.  explicit_ws = the caller's per-call workspace, nullptr = the
// process-wide one.
static int run_grouped(int groups, const void* const* a, const void* const* b, const float* const* a_scale,
                       const float* const* b_scale, void* const* c, const int* m, int n, int k, hipStream_t s,
                       const Config& cfg, const Workspace* explicit_ws)
{
    if (groups < 0)
        return FP8GEMM_E_SHAPE;
    if (groups == 0)
        return FP8GEMM_OK;
    if (!a || !b || !a_scale || !b_scale || !c || !m)
        return FP8GEMM_E_NULLPTR;
    // Groups of at most 64 rows (an MoE layer in a decode step) go to the decode kernel, which streams
    // every group's B once in whole lines; taller groups to the persistent tile kernel.  A pinned tile
    // shape sends everything to the tile kernel.
    // A few small groups beside many taller ones ride along in the tile launch: their tiles fill its last round,
    // which costs less than a launch of their own (15 small + 49 tall groups, N = 2048, K = 7168: 258 us against
    // 281 us; 32 + 32: 284 against 257 us) -- unless that would put an on-grid tile launch on padded copies.
    bool small_to_tiles = cfg.force_variant >= 0;
    if (!small_to_tiles) {
        int small_n = 0, tall_n = 0;
        bool small_ragged = false, tall_ragged = false;
        for (int g = 0; g < groups; ++g) {
            if (m[g] <= 0)
                continue;
            (m[g] <= 64 ? small_n : tall_n) += 1;
            (m[g] <= 64 ? small_ragged : tall_ragged) |= m[g] % 16 != 0;
        }
        small_to_tiles = small_n > 0 && 3 * small_n <= tall_n && (!small_ragged || tall_ragged);
    }
    auto is_small = [&](int g) { return m[g] <= 64 && !small_to_tiles; };
    // every problem is validated before anything is launched
    long long m_total = 0;
    int count[2] = {0, 0};  // small, tall
    for (int g = 0; g < groups; ++g) {
        if (m[g] < 0)
            return FP8GEMM_E_SHAPE;
        if (m[g] == 0)
            continue;
        const int v = validate(a[g], b[g], a_scale[g], b_scale[g], c[g], m[g], n, k);
        if (v != FP8GEMM_OK)
            return v;
        m_total += m[g];
        ++count[is_small(g) ? 0 : 1];
    }
    if (count[0] + count[1] == 0)
        return FP8GEMM_OK;
    if (count[0] + count[1] == 1 && cfg.force_variant < 0)  // one problem: the dispatcher for single problems
        for (int g = 0; g < groups; ++g)
            if (m[g] > 0)
                return run(a[g], b[g], a_scale[g], b_scale[g], c[g], m[g], n, k, s, cfg, explicit_ws);
    static_assert(GroupTable::MAX_GROUPS == FP8GEMM_MAX_GROUPS, "table size mirrors the ABI constant");
    if (cfg.selected == FP8GEMM_KERNEL_AUTO && m_total <= 0x7FFFFFFFll) {
        // One launch holds MAX_GROUPS problems (the table travels in the kernel arguments): more of a kind run
        // as the fewest launches that hold them, of equal size, one after the other on the stream.
        int rc = FP8GEMM_OK;
        char first_name[sizeof(t_name_buf)] = "";
        for (int kind = 0; kind < 2 && rc == FP8GEMM_OK; ++kind) {
            if (count[kind] == 0)
                continue;
            const int launches = (count[kind] + GroupTable::MAX_GROUPS - 1) / GroupTable::MAX_GROUPS;
            const int per_launch = (count[kind] + launches - 1) / launches;
            GroupTable tab;
            tab.groups = 0;
            int seen = 0;
            for (int g = 0; g < groups && rc == FP8GEMM_OK; ++g) {
                if (m[g] == 0 || is_small(g) != (kind == 0))
                    continue;
                const int t = tab.groups++;
                tab.a[t] = static_cast<const uint8_t*>(a[g]);
                tab.b[t] = static_cast<const uint8_t*>(b[g]);
                tab.a_scale[t] = a_scale[g];
                tab.b_scale[t] = b_scale[g];
                tab.c[t] = static_cast<uint16_t*>(c[g]);
                tab.m[t] = m[g];
                tab.lda[t] = m[g];
                ++seen;
                if (tab.groups == per_launch || seen == count[kind]) {
                    rc = run_grouped_table(tab, n, k, kind == 0, s, cfg, explicit_ws);
                    if (rc == GROUPED_NOT_APPLICABLE) {  // these groups one by one
                        rc = FP8GEMM_OK;
                        for (int t = 0; t < tab.groups && rc == FP8GEMM_OK; ++t)
                            rc = run(tab.a[t], tab.b[t], tab.a_scale[t], tab.b_scale[t], tab.c[t], tab.m[t], n, k, s, cfg,
                                     explicit_ws);
                    }
                    tab.groups = 0;
                }
            }
            if (rc != FP8GEMM_OK)
                break;
            if (launches > 1) {  // the last launch's name and how many there were
                char many[sizeof(t_name_buf)];
                snprintf(many, sizeof(many), "%.88sx%d", t_name_buf, launches);
                snprintf(t_name_buf, sizeof(t_name_buf), "%s", many);
            }
            if (kind == 0 && count[1] > 0)
                snprintf(first_name, sizeof(first_name), "%s", t_name_buf);
            if (kind == 1 && first_name[0]) {  // both kernels ran: name both
                char both[sizeof(t_name_buf)];
                snprintf(both, sizeof(both), "%.46s+%.46s", first_name, t_name_buf);
                snprintf(t_name_buf, sizeof(t_name_buf), "%s", both);
            }
        }
        return rc;
    }
    for (int g = 0; g < groups; ++g) {
        if (m[g] == 0)
            continue;
        const int rc = run(a[g], b[g], a_scale[g], b_scale[g], c[g], m[g], n, k, s, cfg, explicit_ws);
        if (rc != FP8GEMM_OK)
            return rc;
    }
    return FP8GEMM_OK;
}

int fp8_block_gemm_grouped(int groups, const void* const* a, const void* const* b,
                           const float* const* a_scale, const float* const* b_scale,
                           void* const* c, const int* m, int n, int k, void* stream)
{
    return run_grouped(groups, a, b, a_scale, b_scale, c, m, n, k, static_cast<hipStream_t>(stream), global_config(),
                       nullptr);
}

int fp8_block_gemm_grouped_ex(int groups, const void* const* a, const void* const* b, const float* const* a_scale,
                              const float* const* b_scale, void* const* c, const int* m, int n, int k,
                              const fp8gemm_options* options, void* workspace, size_t workspace_bytes, void* stream)
{
    int rc;
    const Config cfg = config_from_options(options, &rc);
    if (rc != FP8GEMM_OK)
        return rc;
    const bool zeroed = options && (options->flags & FP8GEMM_FLAG_WORKSPACE_ZEROED) != 0;
    const Workspace w{static_cast<float*>(workspace), workspace ? workspace_bytes : 0, zeroed};
    return run_grouped(groups, a, b, a_scale, b_scale, c, m, n, k, static_cast<hipStream_t>(stream), cfg, &w);
}

int fp8_block_gemm_set_fused_reduction(int mode)
{
    if (mode < -1 || mode > 1)
        return FP8GEMM_E_KERNEL;
    g_fused.store(mode);
    return FP8GEMM_OK;
}

int fp8_block_gemm_set_persistent(int mode)
{
    if (mode < -1 || mode > 1)
        return FP8GEMM_E_KERNEL;
    g_persistent.store(mode);
    return FP8GEMM_OK;
}

const char* fp8_block_gemm_last_kernel(void) { return t_last_kernel; }

int fp8_block_gemm_plan(int m, int n, int k, char* name, size_t cap)
{
    if (!name || cap == 0)
        return FP8GEMM_E_NULLPTR;
    if (m <= 0 || n <= 0 || k <= 0 || (k % 128) != 0)
        return FP8GEMM_E_SHAPE;
    // aligned dummy addresses: only their alignment is inspected
    GemmArgs g{reinterpret_cast<const uint8_t*>(uintptr_t(4096)), reinterpret_cast<const uint8_t*>(uintptr_t(4096)),
               reinterpret_cast<const float*>(uintptr_t(4096)), nullptr, reinterpret_cast<uint16_t*>(uintptr_t(4096)),
               m, n, k};
    Plan p = make_plan(g, global_config());
    if (p.family < 0)
        return FP8GEMM_E_KERNEL;
    plan_name(p, name, cap);
    return FP8GEMM_OK;
}

size_t fp8_block_gemm_workspace_bytes(int m, int n, int k)
{
    return workspace_bytes_for(m, n, k, global_config(), false);
}

size_t fp8_block_gemm_workspace_bytes_ex(int m, int n, int k, const fp8gemm_options* options, int any_alignment)
{
    int rc;
    const Config cfg = config_from_options(options, &rc);
    if (rc != FP8GEMM_OK)
        return 0;
    return workspace_bytes_for(m, n, k, cfg, any_alignment != 0);
}

static size_t grouped_bytes(int groups, const int* m, int n, int k, const Config& cfg)
{
    if (groups <= 0 || !m || n <= 0 || k <= 0 || (k % 128) != 0)
        return 0;
    // a grouped launch on padded copies takes every group's copies at once (the decode kernel's splits meet
    // in the header); one by one the largest single need would do
    const int n16 = (n + 15) & ~15;
    const size_t nkb = (size_t)k / 128;
    size_t total = 0, small_groups = 0;
    for (int g = 0; g < groups; ++g) {
        if (m[g] <= 0)
            continue;
        const size_t m16 = ((size_t)m[g] + 15) & ~(size_t)15;
        total += round256((size_t)k * m16) + round256(nkb * m16 * sizeof(float)) + round256((size_t)k * n16) +
                 round256(m16 * n16 * 2);
        small_groups += m[g] <= 64 ? 1 : 0;
    }
    total = with_header(total, small_groups > 0);
    for (int g = 0; g < groups; ++g) {
        if (m[g] <= 0)
            continue;
        const size_t single = workspace_bytes_for(m[g], n, k, cfg, true);
        total = total > single ? total : single;
    }
    return total;
}

size_t fp8_block_gemm_grouped_workspace_bytes(int groups, const int* m, int n, int k)
{
    return grouped_bytes(groups, m, n, k, global_config());
}

size_t fp8_block_gemm_grouped_workspace_bytes_ex(int groups, const int* m, int n, int k, const fp8gemm_options* options)
{
    int rc;
    const Config cfg = config_from_options(options, &rc);
    return rc == FP8GEMM_OK ? grouped_bytes(groups, m, n, k, cfg) : 0;
}

int fp8_block_gemm_set_workspace(void* device_ptr, size_t bytes)
{
    if (device_ptr && (reinterpret_cast<uintptr_t>(device_ptr) % 256) != 0)
        return FP8GEMM_E_WORKSPACE;
    // the header at its start is zero-filled here (the call waits for that fill); a buffer too
    // small to hold it can serve no plan anyway
    bool zeroed = false;
    if (device_ptr && bytes >= WS_HEADER) {
        const hipError_t e = hipMemset(device_ptr, 0, WS_HEADER);
        if (e != hipSuccess)
            return (int)e;
        zeroed = true;
    }
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    g_ws_user = static_cast<float*>(device_ptr);
    g_ws_user_bytes = device_ptr ? bytes : 0;
    g_ws_user_zeroed = zeroed;
    return FP8GEMM_OK;
}

int fp8_block_gemm_release(void)
{
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if (!g_ws_own && g_ws_retired.empty())
        return FP8GEMM_OK;
    hipError_t e = hipDeviceSynchronize();  // kernels of earlier calls may still use the buffers
    if (e != hipSuccess)
        return (int)e;
    hipError_t first = hipSuccess;
    for (Retired& r : g_ws_retired) {
        if (r.done)
            (void)hipEventDestroy(r.done);
        e = hipFree(r.ptr);
        first = first == hipSuccess ? e : first;
    }
    g_ws_retired.clear();
    g_ws_own_captured = false;
    if (g_ws_own) {
        e = hipFree(g_ws_own);
        first = first == hipSuccess ? e : first;
        g_ws_own = nullptr;
        g_ws_own_bytes = 0;
    }
    return (int)first;
}

int fp8_convert_f32_to_e4m3fn(const float* in, void* out, size_t count, void* stream)
{
    if (count == 0)
        return FP8GEMM_OK;
    if (!in || !out)
        return FP8GEMM_E_NULLPTR;
    if (reinterpret_cast<uintptr_t>(in) % 16 != 0 || reinterpret_cast<uintptr_t>(out) % 4 != 0)
        return FP8GEMM_E_ALIGN;  // the kernel reads four floats and writes four codes at a time
    return (int)launch_convert(in, static_cast<uint8_t*>(out), count, static_cast<hipStream_t>(stream));
}

static int quantize_entry(const void* x, int x_dtype, void* q, float* scale, int rows, int k,
                          void* stream, bool block128)
{
    if (!x || !q || !scale)
        return FP8GEMM_E_NULLPTR;
    if (rows <= 0 || k <= 0 || (k % 128) != 0)
        return FP8GEMM_E_SHAPE;
    if ((long long)rows * k > 0x7FFFFFFFll)
        return FP8GEMM_E_TOOLARGE;
    if (x_dtype != FP8GEMM_DTYPE_BF16 && x_dtype != FP8GEMM_DTYPE_F32 && x_dtype != FP8GEMM_DTYPE_BF16_F32MATH)
        return FP8GEMM_E_DTYPE;
    if (reinterpret_cast<uintptr_t>(x) % 16 != 0)
        return FP8GEMM_E_ALIGN;
    static_assert(QUANT_SOURCE_BF16 == FP8GEMM_DTYPE_BF16 && QUANT_SOURCE_F32 == FP8GEMM_DTYPE_F32 &&
                      QUANT_SOURCE_BF16_F32MATH == FP8GEMM_DTYPE_BF16_F32MATH,
                  "launcher enum mirrors the ABI constants");
    return (int)launch_quantize(x, static_cast<QuantSource>(x_dtype), static_cast<uint8_t*>(q), scale, rows,
                                k, block128, static_cast<hipStream_t>(stream));
}

int fp8_quantize_a_1x128(const void* x, int x_dtype, void* a, float* a_scale, int m, int k,
                         void* stream)
{
    return quantize_entry(x, x_dtype, a, a_scale, m, k, stream, false);
}

int fp8_quantize_b_128x128(const void* x, int x_dtype, void* b, float* b_scale, int n, int k,
                           void* stream)
{
    return quantize_entry(x, x_dtype, b, b_scale, n, k, stream, true);
}

const char* fp8_block_gemm_error_string(int code)
{
    switch (code) {
    case FP8GEMM_OK: return "success";
    case FP8GEMM_E_NULLPTR: return "a required pointer is NULL";
    case FP8GEMM_E_SHAPE: return "m, n, k must be positive and k a multiple of 128";
    case FP8GEMM_E_KERNEL: return "unknown kernel id or kernel not applicable to this shape";
    case FP8GEMM_E_WORKSPACE: return "workspace missing, too small or misaligned (or it would have to grow under stream capture)";
    case FP8GEMM_E_TOOLARGE: return "operand exceeds 2^31-1 elements";
    case FP8GEMM_E_DTYPE: return "unknown source element type";
    case FP8GEMM_E_ALIGN: return "pointer alignment: 16 bytes for a source, 4 for the converter's output";
    default: break;
    }
    if (code > 0)
        return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error code";
}

size_t fp8_block_gemm_workspace_growth(size_t have, size_t need) { return growth_target(have, need); }

int fp8_block_gemm_abi_version(void) { return 5; }

}  // extern "C"
