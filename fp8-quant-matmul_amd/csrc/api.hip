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

using namespace fp8gemm;

namespace {

constexpr int NUM_CU = 256;

std::atomic<int> g_selected{FP8GEMM_KERNEL_AUTO};
std::atomic<int> g_force_variant{-1};
std::atomic<int> g_force_ksplit{0};
std::atomic<int> g_persistent{-1};  // -1 = when tiles outnumber the CUs, 0 = never, 1 = whenever possible
thread_local const char* t_last_kernel = "none";
thread_local char t_name_buf[64];

std::mutex g_ws_mutex;
float* g_ws_own = nullptr;       // library-owned workspace
size_t g_ws_own_bytes = 0;
float* g_ws_user = nullptr;      // caller-supplied workspace
size_t g_ws_user_bytes = 0;

struct Plan {
    int family;   // FP8GEMM_KERNEL_*
    int variant;  // TileVariant for the tile families
    int ksplit;
    bool persistent = false;  // tile families, ksplit == 1: workgroups walk through the tiles
    bool padded = false;      // the plan is for the problem with m and n rounded up to 16 (run_padded)
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
// (the tile kernels): c then needs no copy on account of m.
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
double tile_cost(const GemmArgs& g, int variant, int ksplit)
{
    int bm, bn;
    tile_variant_dims(variant, &bm, &bn);
    const int tiles = ((g.m + bm - 1) / bm) * ((g.n + bn - 1) / bn);
    const int nkb = g.k / 128;
    const int kbs = (nkb + ksplit - 1) / ksplit;
    const double area = (double)bm * bn / 65536.0;
    const double per_kb = 1.19 * area + 0.267;
    const double per_item = 0.95 + 4.38 * area + kbs * per_kb;
    const long items = (long)tiles * ksplit;
    const long rounds = (items + NUM_CU - 1) / NUM_CU;
    double cost = 1.79 + rounds * per_item;
    if (ksplit > 1)  // second launch + partial write and read-back
        cost += 2.86 + (double)g.m * g.n * ksplit * 8.0 / 7.38e6;
    return cost;
}

// Shapes whose best measured plan differs from the model's choice: {m, n, k, variant, ksplit}.
struct TunedShape { int m, n, k, variant, ksplit; };
constexpr TunedShape kTuned[] = {
    {1024, 512, 7168, TILE_64x64, 2},
    {1024, 576, 7168, TILE_128x128, 4},
    {6144, 3072, 1536, TILE_256x192, 1},
    {8192, 7168, 2048, TILE_256x192, 1},
};

// A persistent launch pays off when a CU gets more than one tile.
void decide_persistent(const GemmArgs& g, Plan& p)
{
    p.persistent = false;
    const int mode = g_persistent.load();
    if (p.variant == TILE_256x192_W4) {  // exists in the persistent form only
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

Plan make_plan(const GemmArgs& g, int selected)
{
    Plan p{FP8GEMM_KERNEL_SCALAR, 0, 1};
    if (selected == FP8GEMM_KERNEL_SCALAR)
        return p;
    if (selected == FP8GEMM_KERNEL_SKINNY || (selected == FP8GEMM_KERNEL_AUTO && skinny_supports(g) && g.m <= 64)) {
        if (skinny_supports(g)) {
            p.family = FP8GEMM_KERNEL_SKINNY;
            p.ksplit = skinny_ksplit(g);
            return p;
        }
        if (selected == FP8GEMM_KERNEL_SKINNY) {
            p.family = -1;
            return p;
        }
    }
    if (!tile_supports(g)) {
        if (selected != FP8GEMM_KERNEL_AUTO) {
            p.family = -1;
            return p;
        }
        // rows without 16-byte alignment: the padded problem (its four extra launches cost
        // about 12 us; the scalar kernel, one dependent load after the other, takes 30 us for
        // K = 128 already), unless padding pushes an operand past the size limit
        const long long m16 = (g.m + 15) & ~15, n16 = (g.n + 15) & ~15, lim = 0x7FFFFFFFll;
        if (m16 * g.k > lim || n16 * g.k > lim || m16 * n16 > lim)
            return p;
        const uint8_t* const al8 = reinterpret_cast<const uint8_t*>(uintptr_t(4096));
        GemmArgs gp{al8, al8, reinterpret_cast<const float*>(uintptr_t(4096)), g.b_scale,
                    reinterpret_cast<uint16_t*>(uintptr_t(4096)), (int)m16, (int)n16, g.k};
        p = make_plan(gp, selected);
        p.padded = p.family != FP8GEMM_KERNEL_SCALAR && p.family >= 0;
        return p;
    }
    const int fv = g_force_variant.load(), fk = g_force_ksplit.load();
    const int nkb = g.k / 128;
    if (selected == FP8GEMM_KERNEL_AUTO && fv < 0 && fk <= 0)
        for (const TunedShape& t : kTuned)
            if (t.m == g.m && t.n == g.n && t.k == g.k) {
                p.family = t.ksplit > 1 ? FP8GEMM_KERNEL_SPLITK : FP8GEMM_KERNEL_LARGE;
                p.variant = t.variant;
                p.ksplit = t.ksplit;
                decide_persistent(g, p);
                return p;
            }
    double best = 1e300;
    for (int v = 0; v < TILE_VARIANT_COUNT; ++v) {
        if (fv >= 0 && v != fv)
            continue;
        if (tile_variant_name(v)[4] == '?')
            continue;
        if (v == TILE_256x192_W4 && fv != v)  // one-wave-per-SIMD form: only when asked for
            continue;
        for (int ks = 1; ks <= 16 && ks <= nkb; ++ks) {
            if (v == TILE_256x192_W4 && ks != 1)
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
            const double cst = tile_cost(g, v, ks);
            if (cst < best) {
                best = cst;
                p.family = ks > 1 ? FP8GEMM_KERNEL_SPLITK : FP8GEMM_KERNEL_LARGE;
                p.variant = v;
                p.ksplit = ks;
            }
        }
    }
    if (best == 1e300) {
        p.family = -1;
        return p;
    }
    decide_persistent(g, p);
    if (p.variant == TILE_256x192_W4 && !p.persistent)
        p.family = -1;
    return p;
}

// fp32 partial buffer of at least `bytes`, or nullptr with *err set
float* get_workspace(size_t bytes, int* err)
{
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    *err = FP8GEMM_OK;
    if (g_ws_user) {
        if (g_ws_user_bytes < bytes) {
            *err = FP8GEMM_E_WORKSPACE;
            return nullptr;
        }
        return g_ws_user;
    }
    if (g_ws_own_bytes < bytes) {
        if (g_ws_own) {
            // kernels of earlier calls may still read the old buffer
            hipError_t e = hipDeviceSynchronize();
            if (e != hipSuccess) {
                *err = (int)e;
                return nullptr;
            }
            (void)hipFree(g_ws_own);
            g_ws_own = nullptr;
            g_ws_own_bytes = 0;
        }
        void* p = nullptr;
        hipError_t e = hipMalloc(&p, bytes);
        if (e != hipSuccess) {
            *err = (int)e;
            return nullptr;
        }
        g_ws_own = static_cast<float*>(p);
        g_ws_own_bytes = bytes;
    }
    return g_ws_own;
}

size_t plan_workspace_bytes(const GemmArgs& g, const Plan& p)
{
    if (p.ksplit <= 1)
        return 0;
    return (size_t)p.ksplit * g.m * g.n * sizeof(float);
}

void plan_name(const Plan& p, char* out, size_t cap)
{
    const char* pre = p.padded ? "padded_" : "";
    if (p.family == FP8GEMM_KERNEL_SCALAR)
        snprintf(out, cap, "scalar");
    else if (p.family == FP8GEMM_KERNEL_SKINNY)
        snprintf(out, cap, "%sskinny_k%d", pre, p.ksplit);
    else
        snprintf(out, cap, "%s%s_k%d%s", pre, tile_variant_name(p.variant), p.ksplit,
                 p.persistent ? "_persistent" : "");
}

// the kernels of a plan on operands they can take; `partial` holds plan_workspace_bytes
hipError_t launch_plan(const GemmArgs& g, const Plan& p, float* partial, hipStream_t stream)
{
    switch (p.family) {
    case FP8GEMM_KERNEL_SCALAR:
        return launch_scalar(g, stream);
    case FP8GEMM_KERNEL_SKINNY:
        return launch_skinny(g, partial, stream);
    default: {
        if (p.persistent)
            return launch_tile_persistent(g, p.variant, NUM_CU, stream);
        hipError_t e = launch_tile(g, p.variant, p.ksplit, partial, stream);
        if (e == hipSuccess && p.ksplit > 1)
            e = launch_splitk_reduce(g, p.ksplit, partial, stream);
        return e;
    }
    }
}

// pad what needs padding into the workspace, run the plan there, copy C's corner out
int run_padded(const GemmArgs& g, const Plan& p, hipStream_t stream)
{
    GemmArgs gp = g;
    const int m16 = (g.m + 15) & ~15;
    gp.m = m16;
    gp.n = (g.n + 15) & ~15;
    const bool keeps_rows = p.family == FP8GEMM_KERNEL_LARGE || p.family == FP8GEMM_KERNEL_SPLITK;
    const PadLayout L = pad_layout(g, plan_workspace_bytes(gp, p), false, keeps_rows);
    if (!L.c) {  // c is written in place: its m rows, while a and a_scale have m16 per k-row
        gp.m = g.m;
        gp.lda = m16;
    }
    int err;
    float* ws = get_workspace(L.total, &err);
    if (!ws)
        return err;
    uint8_t* base = reinterpret_cast<uint8_t*>(ws);
    const int nkb = g.k / 128;
    hipError_t e = hipSuccess;
    if (L.a) {
        e = launch_pad_bytes(g.a, base + L.off_a, g.k, g.m, m16, stream);
        gp.a = base + L.off_a;
    }
    if (e == hipSuccess && L.as) {
        float* as = reinterpret_cast<float*>(base + L.off_as);
        e = launch_pad_floats(g.a_scale, as, nkb, g.m, m16, stream);
        gp.a_scale = as;
    }
    if (e == hipSuccess && L.b) {
        e = launch_pad_bytes(g.b, base + L.off_b, g.k, g.n, gp.n, stream);
        gp.b = base + L.off_b;
    }
    if (L.c)
        gp.c = reinterpret_cast<uint16_t*>(base + L.off_c);
    if (e == hipSuccess)
        e = launch_plan(gp, p, reinterpret_cast<float*>(base + L.off_partial), stream);
    if (e == hipSuccess && L.c)
        e = launch_crop_bf16(gp.c, g.c, g.m, g.n, gp.n, stream);
    return (int)e;
}

int run(const void* a, const void* b, const float* as, const float* bs, void* c, int m, int n, int k,
        hipStream_t stream, int selected)
{
    int v = validate(a, b, as, bs, c, m, n, k);
    if (v != FP8GEMM_OK)
        return v;
    GemmArgs g{static_cast<const uint8_t*>(a), static_cast<const uint8_t*>(b), as, bs,
               static_cast<uint16_t*>(c), m, n, k};
    const Plan p = make_plan(g, selected);
    if (p.family < 0)
        return FP8GEMM_E_KERNEL;
    int rc;
    if (p.padded) {
        rc = run_padded(g, p, stream);
    } else {
        float* ws = nullptr;
        const size_t need = plan_workspace_bytes(g, p);
        if (need) {
            int err;
            ws = get_workspace(need, &err);
            if (!ws)
                return err;
        }
        rc = (int)launch_plan(g, p, ws, stream);
    }
    plan_name(p, t_name_buf, sizeof(t_name_buf));
    t_last_kernel = t_name_buf;
    return rc;
}

// tile shape for a grouped launch: what the cost model picks for the stacked problem, among the
// shapes that have a persistent form, without a K split; -1 when none can take the table
int grouped_variant(const GroupTable& tab, int n, int k)
{
    long long m_total = 0;
    for (int g = 0; g < tab.groups; ++g)
        m_total += tab.m[g];
    if (m_total > 0x7FFFFFFFll)
        return -1;
    int best_v = -1;
    double best = 1e300;
    const int fv = g_force_variant.load();
    const GemmArgs stacked{tab.a[0], tab.b[0], tab.a_scale[0], tab.b_scale[0], tab.c[0], (int)m_total, n, k};
    for (int v = 0; v < TILE_VARIANT_COUNT; ++v) {
        if ((fv >= 0 && v != fv) || !tile_grouped_supports(tab, n, k, v))
            continue;
        const double cst = tile_cost(stacked, v, 1);
        if (cst < best) {
            best = cst;
            best_v = v;
        }
    }
    return best_v;
}

// Grouped launch for problems off the 16-byte grid: A and a_scale of every group (B and C too
// when n or one of their addresses is off the grid) go through padded copies in the workspace,
// one batched copy launch per kind around one grouped GEMM.  Returns GROUPED_NOT_APPLICABLE when it cannot run
// (the caller then takes the groups one by one).
constexpr int GROUPED_NOT_APPLICABLE = -1000;
int run_grouped_padded(const GroupTable& tab, int n, int k, hipStream_t s)
{
    const long long lim = 0x7FFFFFFFll;
    const int n16 = (n + 15) & ~15;
    const size_t nkb = (size_t)k / 128;
    bool pad_b = n16 != n, pad_c = n16 != n;
    for (int g = 0; g < tab.groups; ++g) {
        pad_b = pad_b || misaligned16(tab.b[g]);
        pad_c = pad_c || misaligned16(tab.c[g]);
    }
    size_t off_a[GroupTable::MAX_GROUPS], off_as[GroupTable::MAX_GROUPS], off_b[GroupTable::MAX_GROUPS],
        off_c[GroupTable::MAX_GROUPS];
    size_t off = 0;
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
    int err;
    float* ws = get_workspace(off, &err);
    if (!ws)
        return err;
    uint8_t* base = reinterpret_cast<uint8_t*>(ws);
    GroupTable pt;
    RepackTable ta, tas, tb, tc;
    pt.groups = ta.groups = tas.groups = tb.groups = tc.groups = tab.groups;
    for (int g = 0; g < tab.groups; ++g) {
        const int m = tab.m[g], m16 = (m + 15) & ~15;
        pt.a[g] = base + off_a[g];
        pt.a_scale[g] = reinterpret_cast<const float*>(base + off_as[g]);
        pt.b[g] = pad_b ? base + off_b[g] : tab.b[g];
        pt.b_scale[g] = tab.b_scale[g];
        // c in place keeps its m rows; a and a_scale have m16 per k-row either way
        pt.c[g] = pad_c ? reinterpret_cast<uint16_t*>(base + off_c[g]) : tab.c[g];
        pt.m[g] = pad_c ? m16 : m;
        pt.lda[g] = m16;
        ta.src[g] = tab.a[g], ta.dst[g] = base + off_a[g], ta.rows[g] = k, ta.ld_src[g] = m, ta.ld_dst[g] = m16;
        tas.src[g] = tab.a_scale[g], tas.dst[g] = base + off_as[g], tas.rows[g] = (int)nkb, tas.ld_src[g] = m,
        tas.ld_dst[g] = m16;
        tb.src[g] = tab.b[g], tb.dst[g] = base + off_b[g], tb.rows[g] = k, tb.ld_src[g] = n, tb.ld_dst[g] = n16;
        tc.src[g] = base + off_c[g], tc.dst[g] = tab.c[g], tc.rows[g] = m, tc.ld_src[g] = n16, tc.ld_dst[g] = n;
    }
    const int v = grouped_variant(pt, n16, k);
    if (v < 0)
        return GROUPED_NOT_APPLICABLE;
    hipError_t e = launch_pad_bytes_batched(ta, s);
    if (e == hipSuccess)
        e = launch_pad_floats_batched(tas, s);
    if (e == hipSuccess && pad_b)
        e = launch_pad_bytes_batched(tb, s);
    if (e == hipSuccess)
        e = launch_tile_grouped(pt, n16, k, v, NUM_CU, s);
    if (e == hipSuccess && pad_c)
        e = launch_crop_bf16_batched(tc, s);
    if (e == hipSuccess) {
        snprintf(t_name_buf, sizeof(t_name_buf), "padded_%s_k1_grouped%d", tile_variant_name(v), tab.groups);
        t_last_kernel = t_name_buf;
    }
    return (int)e;
}

}  // namespace

extern "C" {

int fp8_block_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale, void* c,
                   int m, int n, int k)
{
    return run(a, b, a_scale, b_scale, c, m, n, k, nullptr, g_selected.load());
}

int fp8_block_gemm_stream(const void* a, const void* b, const float* a_scale, const float* b_scale,
                          void* c, int m, int n, int k, void* stream)
{
    return run(a, b, a_scale, b_scale, c, m, n, k, static_cast<hipStream_t>(stream),
               g_selected.load());
}

int fp8_block_gemm_scalar(const void* a, const void* b, const float* a_scale, const float* b_scale,
                          void* c, int m, int n, int k, void* stream)
{
    return run(a, b, a_scale, b_scale, c, m, n, k, static_cast<hipStream_t>(stream),
               FP8GEMM_KERNEL_SCALAR);
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
    if (tile_variant >= TILE_VARIANT_COUNT || ksplit < 0 || ksplit > 64)
        return FP8GEMM_E_KERNEL;
    g_force_variant.store(tile_variant < 0 ? -1 : tile_variant);
    g_force_ksplit.store(ksplit);
    return FP8GEMM_OK;
}

int fp8_block_gemm_grouped(int groups, const void* const* a, const void* const* b,
                           const float* const* a_scale, const float* const* b_scale,
                           void* const* c, const int* m, int n, int k, void* stream)
{
    if (groups < 0)
        return FP8GEMM_E_SHAPE;
    if (groups == 0)
        return FP8GEMM_OK;
    if (!a || !b || !a_scale || !b_scale || !c || !m)
        return FP8GEMM_E_NULLPTR;
    // every problem is validated before anything is launched
    long long m_total = 0;
    int live = 0;
    for (int g = 0; g < groups; ++g) {
        if (m[g] < 0)
            return FP8GEMM_E_SHAPE;
        if (m[g] == 0)
            continue;
        const int v = validate(a[g], b[g], a_scale[g], b_scale[g], c[g], m[g], n, k);
        if (v != FP8GEMM_OK)
            return v;
        m_total += m[g];
        ++live;
    }
    if (live == 0)
        return FP8GEMM_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    static_assert(GroupTable::MAX_GROUPS == FP8GEMM_MAX_GROUPS, "table size mirrors the ABI constant");
    if (live <= GroupTable::MAX_GROUPS && g_selected.load() == FP8GEMM_KERNEL_AUTO && m_total <= 0x7FFFFFFFll) {
        GroupTable tab;
        tab.groups = 0;
        for (int g = 0; g < groups; ++g) {
            if (m[g] == 0)
                continue;
            const int t = tab.groups++;
            tab.a[t] = static_cast<const uint8_t*>(a[g]);
            tab.b[t] = static_cast<const uint8_t*>(b[g]);
            tab.a_scale[t] = a_scale[g];
            tab.b_scale[t] = b_scale[g];
            tab.c[t] = static_cast<uint16_t*>(c[g]);
            tab.m[t] = m[g];
            tab.lda[t] = m[g];
        }
        const int best_v = grouped_variant(tab, n, k);
        if (best_v >= 0) {
            const hipError_t e = launch_tile_grouped(tab, n, k, best_v, NUM_CU, s);
            if (e == hipSuccess) {
                snprintf(t_name_buf, sizeof(t_name_buf), "%s_k1_grouped%d", tile_variant_name(best_v), tab.groups);
                t_last_kernel = t_name_buf;
            }
            return (int)e;
        }
        const int rc = run_grouped_padded(tab, n, k, s);
        if (rc != GROUPED_NOT_APPLICABLE)
            return rc;
    }
    for (int g = 0; g < groups; ++g) {
        if (m[g] == 0)
            continue;
        const int rc = run(a[g], b[g], a_scale[g], b_scale[g], c[g], m[g], n, k, s, g_selected.load());
        if (rc != FP8GEMM_OK)
            return rc;
    }
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
               nullptr, nullptr, reinterpret_cast<uint16_t*>(uintptr_t(4096)), m, n, k};
    Plan p = make_plan(g, g_selected.load());
    if (p.family < 0)
        return FP8GEMM_E_KERNEL;
    plan_name(p, name, cap);
    return FP8GEMM_OK;
}

size_t fp8_block_gemm_workspace_bytes(int m, int n, int k)
{
    if (m <= 0 || n <= 0 || k <= 0 || (k % 128) != 0)
        return 0;
    // what the plan for 16-byte aligned operands needs under the current selection and forced
    // configuration; operands with less alignment run kernels that need the same or nothing
    GemmArgs g{reinterpret_cast<const uint8_t*>(uintptr_t(4096)), reinterpret_cast<const uint8_t*>(uintptr_t(4096)),
               nullptr, nullptr, reinterpret_cast<uint16_t*>(uintptr_t(4096)), m, n, k};
    const Plan p = make_plan(g, g_selected.load());
    if (p.family < 0)
        return 0;
    if (!p.padded)
        return plan_workspace_bytes(g, p);
    GemmArgs gp = g;
    gp.m = (m + 15) & ~15;
    gp.n = (n + 15) & ~15;
    return pad_layout(g, plan_workspace_bytes(gp, p), true, false).total;
}

int fp8_block_gemm_set_workspace(void* device_ptr, size_t bytes)
{
    if (device_ptr && (reinterpret_cast<uintptr_t>(device_ptr) % 256) != 0)
        return FP8GEMM_E_WORKSPACE;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    g_ws_user = static_cast<float*>(device_ptr);
    g_ws_user_bytes = device_ptr ? bytes : 0;
    return FP8GEMM_OK;
}

int fp8_block_gemm_release(void)
{
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    if (g_ws_own) {
        hipError_t e = hipDeviceSynchronize();
        if (e != hipSuccess)
            return (int)e;
        e = hipFree(g_ws_own);
        g_ws_own = nullptr;
        g_ws_own_bytes = 0;
        return (int)e;
    }
    return FP8GEMM_OK;
}

int fp8_convert_f32_to_e4m3fn(const float* in, void* out, size_t count, void* stream)
{
    if (count == 0)
        return FP8GEMM_OK;
    if (!in || !out)
        return FP8GEMM_E_NULLPTR;
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
    case FP8GEMM_E_WORKSPACE: return "workspace too small or misaligned";
    case FP8GEMM_E_TOOLARGE: return "operand exceeds 2^31-1 elements";
    case FP8GEMM_E_DTYPE: return "unknown source element type";
    case FP8GEMM_E_ALIGN: return "source pointer is not 16-byte aligned";
    default: break;
    }
    if (code > 0)
        return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown error code";
}

int fp8_block_gemm_abi_version(void) { return 2; }

}  // extern "C"
