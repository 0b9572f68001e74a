// Internal (C++) launch functions behind the C ABI in include/fp8_block_gemm.h.
// Each returns a hipError_t; none synchronises.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

namespace fp8gemm {

struct GemmArgs {
    const uint8_t* a;
    const uint8_t* b;
    const float* a_scale;
    const float* b_scale;
    uint16_t* c;
    int m, n, k;
    // elements between consecutive k-rows of a and of a_scale; 0 = m (the layout of the ABI).
    // Only the tile kernels take another value (padded copies whose c keeps m rows).
    int lda = 0;
};
inline int leading_dim(const GemmArgs& g) { return g.lda ? g.lda : g.m; }

// Kernels with more than 64 KiB of dynamic LDS need the attribute raised before their first launch
// on a device.  Once per kernel and device (a bit per device in a word the call site owns) instead of
// once per launch: the runtime call costs as much as a short kernel takes.
#define FP8GEMM_ALLOW_LDS(kern, bytes)                                                                       \
    do {                                                                                                     \
        static std::atomic<uint64_t> done_{0};                                                               \
        int dev_ = 0;                                                                                        \
        hipError_t e_ = hipGetDevice(&dev_);                                                                 \
        if (e_ != hipSuccess)                                                                                \
            return e_;                                                                                       \
        const uint64_t bit_ = 1ull << (dev_ & 63);                                                           \
        if (!(done_.load(std::memory_order_acquire) & bit_)) {                                               \
            e_ = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                    \
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (bytes));                   \
            if (e_ != hipSuccess)                                                                            \
                return e_;                                                                                   \
            done_.fetch_or(bit_, std::memory_order_release);                                                 \
        }                                                                                                    \
    } while (0)

// one thread per C element (check.cu:30-49)
hipError_t launch_scalar(const GemmArgs& g, hipStream_t s);

// The mailbox: device memory that only the kernels that add their K splits themselves write, all zero
// before a launch and all zero again after it; the splits of a tile or strip hand their partial results
// over through it.
constexpr size_t SPLIT_MAILBOX_BYTES = (size_t)16 << 20;

// MFMA tile kernel family.  `variant` picks the workgroup tile; ksplit > 1 writes fp32
// partial sums to `partial` ([ksplit][m][n]) instead of c.  With mailbox == nullptr it must be followed
// by launch_splitk_reduce; with a mailbox (SPLIT_MAILBOX_BYTES) the workgroup of a tile's last split
// adds the other splits' accumulators itself and writes c, with the same arithmetic, and `partial` is
// not used.  The latter needs xcd_placement_confirmed() and tile_mailbox_bytes() <= SPLIT_MAILBOX_BYTES.
enum TileVariant { TILE_256x192 = 0, TILE_256x128 = 1, TILE_128x128 = 2, TILE_128x192 = 3,
                   TILE_64x64 = 4, TILE_256x192_W4 = 5, TILE_256x256 = 6, TILE_VARIANT_COUNT };
bool tile_supports(const GemmArgs& g);
const char* tile_variant_name(int variant);
void tile_variant_dims(int variant, int* bm, int* bn);
size_t tile_mailbox_bytes(const GemmArgs& g, int variant, int ksplit);
hipError_t launch_tile(const GemmArgs& g, int variant, int ksplit, float* partial, float* mailbox,
                       hipStream_t s);
// Persistent form (ksplit = 1 only): `workgroups` (a multiple of 8) workgroups walk through
// all tiles, the copies of a tile's first K blocks overlap the previous tile's epilogue.
bool tile_persistent_supports(const GemmArgs& g, int variant);
hipError_t launch_tile_persistent(const GemmArgs& g, int variant, int workgroups, hipStream_t s);
// Grouped form: several problems with the same n and k and their own m in one persistent launch
// (the table travels by value in the kernel arguments; tile_start is filled by the launcher).
struct GroupTable {
    static constexpr int MAX_GROUPS = 64;
    const uint8_t* a[MAX_GROUPS];
    const uint8_t* b[MAX_GROUPS];
    const float* a_scale[MAX_GROUPS];
    const float* b_scale[MAX_GROUPS];
    uint16_t* c[MAX_GROUPS];
    int m[MAX_GROUPS];
    int lda[MAX_GROUPS];  // as GemmArgs::lda, but always filled in
    int tile_start[MAX_GROUPS + 1];
    int groups;
};
bool tile_grouped_supports(const GroupTable& tab, int n, int k, int variant);
hipError_t launch_tile_grouped(GroupTable& tab, int n, int k, int variant, int workgroups, hipStream_t s);
hipError_t launch_splitk_reduce(const GemmArgs& g, int ksplit, const float* partial, hipStream_t s);

// tiny-M streaming kernel (decode shapes)
bool skinny_supports(const GemmArgs& g);
int skinny_ksplit(const GemmArgs& g);
double skinny_cost(const GemmArgs& g, int ksplit);
hipError_t launch_skinny(const GemmArgs& g, int ksplit, float* partial, hipStream_t s);

// wide-strip decode kernel (M <= 64): 128-column strips, the K splits of a strip added inside the
// kernel.  `mailbox` = SPLIT_MAILBOX_BYTES as above.  ksplit > 1 needs xcd_placement_confirmed() and
// decode_strip_can_split.
constexpr int DECODE_MAX_KSPLIT = 16;
bool decode_strip_supports(const GemmArgs& g);
// halves = 128-column halves of a strip: 1, or 2 (256-column strips: 256 contiguous bytes of every k-row of B)
size_t decode_strip_mailbox_bytes(const GemmArgs& g, int ksplit, int halves = 1);
bool decode_strip_can_split(const GemmArgs& g, int ksplit, int halves = 1);
double decode_strip_cost(const GemmArgs& g, int ksplit, int halves = 1);
hipError_t launch_decode_strips(const GemmArgs& g, int ksplit, int halves, float* mailbox, hipStream_t s);
// The same kernel on several problems with common n and k and their own m <= 64 (multiples of 16), whose
// strips form one list of work items; tile_start of the table is not used.
bool decode_grouped_supports(const GroupTable& tab, int n, int k);
int decode_grouped_ksplit(const GroupTable& tab, int n, int k, bool fused_ok);
size_t decode_grouped_mailbox_bytes(const GroupTable& tab, int n, int ksplit);
bool decode_grouped_streams(int groups, int n);  // the launch takes the streaming form (rows on the 16-byte grid, no K split)
hipError_t launch_decode_grouped(const GroupTable& tab, int n, int k, int ksplit, float* mailbox, hipStream_t s);
// 1 = workgroups whose linear ids agree modulo 8 share an XCD on the current device (looked at once
// per device with a probe grid, which the first call waits for: not under stream capture),
// 0 = they do not, or it could not be looked at; -1 = not looked at yet and may_probe is false
int xcd_placement_confirmed(bool may_probe);

// Padding: rows of ld_src elements copied into rows of ld_dst >= ld_src elements, the rest zero (dst
// 16-byte aligned, ld_dst a multiple of 16 bytes).  Cropping: the m x n corner of a bf16 matrix with
// ld_src elements per row copied into a dense one.
hipError_t launch_crop_bf16(const uint16_t* src, uint16_t* dst, int m, int n, int ld_src, hipStream_t s);
// the padding copies of one problem (bytes of a and b, fp32 values of a_scale) in one launch
struct PadJob {
    const void* src;
    void* dst;
    int rows, ld_src, ld_dst;
    int floats;  // 0 = bytes (ld_dst a multiple of 16), 1 = fp32 values (ld_dst a multiple of 4)
};
struct PadJobs {
    static constexpr int MAX = 4;
    PadJob job[MAX];
    int count;
};
hipError_t launch_pad_jobs(const PadJobs& jobs, hipStream_t s);
// one kind of copy for several matrices in one launch (the table travels by value in the kernel
// arguments).  Padding: rows x ld_src -> rows x ld_dst.  Cropping: rows = m, ld_src = elements
// per source row, ld_dst = n.
struct RepackTable {
    static constexpr int MAX_GROUPS = 64;
    const void* src[MAX_GROUPS];
    void* dst[MAX_GROUPS];
    int rows[MAX_GROUPS];
    int ld_src[MAX_GROUPS];
    int ld_dst[MAX_GROUPS];
    int groups;
};
hipError_t launch_pad_bytes_batched(const RepackTable& tab, hipStream_t s);
// byte copies (a of every group) and fp32 copies (a_scale of every group) in one launch; same group count
hipError_t launch_pad_pair_batched(const RepackTable& bytes, const RepackTable& floats, hipStream_t s);
hipError_t launch_crop_bf16_batched(const RepackTable& tab, hipStream_t s);

// fp32 -> e4m3fn (check.cu:17-22)
hipError_t launch_convert(const float* in, uint8_t* out, size_t count, hipStream_t s);

// 1 x 128 (block128 = false) or 128 x 128 quantiser of a row-major [rows][k] matrix into the
// GEMM's column-major fp8 layout and scale layout (quantize.py:16-67)
// source: element type of x and the arithmetic (values of FP8GEMM_DTYPE_*)
enum QuantSource { QUANT_SOURCE_BF16 = 0, QUANT_SOURCE_F32 = 1, QUANT_SOURCE_BF16_F32MATH = 2 };
hipError_t launch_quantize(const void* x, QuantSource source, uint8_t* q, float* scale_out, int rows,
                           int k, bool block128, hipStream_t s);

}  // namespace fp8gemm
