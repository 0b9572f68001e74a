/*
 * C ABI of the MI355X (gfx950) block-scaled FP8 GEMM.
 *
 *   C[M,N] (bf16, row-major) = sum over 128-wide K blocks kb of
 *        a_scale[kb][m] * b_scale[kb][n/128] * ( A[m, kb-block] . B[n, kb-block] )
 *
 * Every pointer is a DEVICE pointer owned by the caller; the library never frees caller
 * memory and fully overwrites c (no beta).  Layouts are the reference's, unchanged
 * (/root/reference/check.cu:42-48):
 *   a        fp8 e4m3fn (OCP) bytes, element (m,k) at  m + k*M          (M x K column-major)
 *   b        fp8 e4m3fn (OCP) bytes, element (n,k) at  n + k*N          (N x K column-major)
 *   a_scale  fp32, (kb,m)  at  m  + kb*M                                ([K/128][M])
 *   b_scale  fp32, (kb,nb) at  nb + kb*ceil(N/128)                      ([K/128][ceil(N/128)])
 *   c        bf16 bits, element (m,n) at m*N + n
 * Preconditions: m, n, k > 0, k % 128 == 0, non-null pointers.  Any m and n are accepted.
 *
 * Return value: 0 on success; a negative FP8GEMM_E_* code for argument errors, detected
 * before any device call; a positive hipError_t value when the HIP runtime reports one.
 * Nothing is thrown across this boundary.  Launches are asynchronous on the given stream; no
 * entry point waits for the device except fp8_block_gemm_release and fp8_gemm_host.
 *
 * Threads and streams.  fp8_block_gemm_ex / fp8_block_gemm_ws take everything they depend on as
 * arguments (options, workspace, stream) and read no process-wide state: any number of host
 * threads may call them at once, on any streams, as long as calls that run concurrently on the
 * device use different workspaces.  The shorter entry points use process-wide defaults
 * (fp8_block_gemm_select, _force_config, _set_persistent: meant for tests, benchmarks and drivers
 * that mirror the reference's compile-time switches) and ONE process-wide workspace.
 */
#ifndef FP8_BLOCK_GEMM_H
#define FP8_BLOCK_GEMM_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FP8GEMM_OK 0
#define FP8GEMM_E_NULLPTR (-1)   /* a required pointer is NULL */
#define FP8GEMM_E_SHAPE (-2)     /* m, n or k <= 0, or k not a multiple of 128 */
#define FP8GEMM_E_KERNEL (-3)    /* unknown kernel id, or the kernel cannot run this shape */
#define FP8GEMM_E_WORKSPACE (-4) /* workspace missing, too small or misaligned; or the library-owned one
                                    would have to be (re)allocated while the stream is being captured */
#define FP8GEMM_E_TOOLARGE (-5)  /* m*k, n*k or m*n does not fit the 32-bit offsets used */
#define FP8GEMM_E_DTYPE (-6)     /* unknown FP8GEMM_DTYPE_* value */
#define FP8GEMM_E_ALIGN (-7)     /* a source pointer is not 16-byte aligned (converter: output not 4-byte aligned) */

/* Element type of a quantiser's source matrix, and with it the arithmetic: quantize.py computes
 * in the tensor's own dtype, i.e. torch rounds every element-wise result to bf16 for a bf16
 * tensor.  BF16 and F32 reproduce the reference's outputs bit for bit for that source type;
 * BF16_F32MATH reads bf16 but keeps fp32 intermediates (more accurate, not what quantize.py
 * computes). */
#define FP8GEMM_DTYPE_BF16 0
#define FP8GEMM_DTYPE_F32 1
#define FP8GEMM_DTYPE_BF16_F32MATH 2

/* Kernel ids for fp8_block_gemm_select (the run-time counterpart of the reference's
 * compile-time OPTION / #include swap, mn_large.hip:9, check.cu:13). */
#define FP8GEMM_KERNEL_AUTO 0   /* shape-based dispatch (default) */
#define FP8GEMM_KERNEL_SCALAR 1 /* one thread per C element: ref_kernel, check.cu:30-49 */
#define FP8GEMM_KERNEL_LARGE 2  /* MFMA tile kernel for large M and N: mn_large.hip:11 */
#define FP8GEMM_KERNEL_SPLITK 3 /* MFMA tile kernel with the K range split over workgroups:
                                   mn_small.hip:10 (small M*N, large K) */
#define FP8GEMM_KERNEL_SKINNY 4 /* tiny-M streaming kernel (decode shapes) */

/* The GEMM on the null stream.  Replaces the reference launch
 * in_smem_kernel<<<grid, block, 0, 0>>>(A, B, As, Bs, C, M, N, K)
 * (/root/reference/check.cu:106-114, kernel mn_large.hip:11 / mn_small.hip:10):
 * same argument order and meaning.  Any m, n > 0 and k % 128 == 0.  The MFMA kernels take
 * m % 16 == 0, n % 16 == 0 and 16-byte aligned a, b, a_scale, c as they are; for anything else
 * the library copies the operands concerned into zero-padded buffers in its workspace, runs
 * there and copies c's m x n corner out (plans named "padded_...": one extra launch for the copies and
 * one for c's corner, about 2 bytes of extra traffic per operand byte).  The decode kernel ("decode128_kN",
 * chosen for m <= 32) takes any m as it is: a decode batch of 1 ... 15 rows needs no copy.  The reference
 * requires M, N % 64 (32) == 0
 * and reads out of bounds otherwise (mn_large.hip:16). */
int fp8_block_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
                   void* c, int m, int n, int k);

/* Same, on a caller-supplied hipStream_t (passed as void* so that this header needs no HIP
 * include).  The reference only ever uses stream 0 (check.cu:113). */
int fp8_block_gemm_stream(const void* a, const void* b, const float* a_scale,
                          const float* b_scale, void* c, int m, int n, int k, void* stream);

/* The scalar definition kernel: one thread per C element, sequential fp32 block sums.
 * Replaces ref_kernel<<<...>>> (/root/reference/check.cu:30-49, launch check.cu:88). */
int fp8_block_gemm_scalar(const void* a, const void* b, const float* a_scale,
                          const float* b_scale, void* c, int m, int n, int k, void* stream);

/* Force one kernel family for later calls from this process (FP8GEMM_KERNEL_*), or return
 * to automatic dispatch.  Replaces the OPTION macro (/root/reference/mn_large.hip:9) and the
 * `option` argument of gemmGPU (/root/reference/check.cu:51-52, 86-116). */
int fp8_block_gemm_select(int kernel_id);

/* Pin the MFMA tile kernels to one workgroup tile (0 = 256x192, 1 = 256x128, 2 = 128x128,
 * 3 = 128x192, 4 = 64x64 rows x columns of C, 5 = 256x192 with one wave per SIMD (persistent
 * form only, never chosen automatically), 6 = 256x256 (persistent form only, no K split);
 * -1 = choose by cost model) and one K-split count
 * (0 = choose, at most 16; more returns FP8GEMM_E_KERNEL).  With FP8GEMM_KERNEL_SKINNY selected the
 * first argument picks the decode kernel instead: 0 = 32-column strips, 1 = 128-column strips whose K
 * splits are added inside the kernel, 2 = the same with 256-column strips, -1 = by cost.  Benchmarking and test aid; no counterpart in the reference beyond editing its WMMA_* / NUM_WARP_* macros
 * (/root/reference/mn_large.hip:1-8). */
int fp8_block_gemm_force_config(int tile_variant, int ksplit);

/* The tile kernels have a persistent form (ksplit = 1): 256 workgroups walk through all
 * tiles and copy a tile's first K blocks while the previous tile is stored.  mode -1 = use it
 * when there are more tiles than compute units (default), 0 = never, 1 = whenever the shape
 * allows.  The reference names such a kernel as future work (/root/reference/README.md:29). */
int fp8_block_gemm_set_persistent(int mode);

/* Plans that split K ("..._kN") write fp32 partial results; they are added either by a second kernel or
 * inside the GEMM kernel ("..._kNf", "decode128_kN"): the K splits of a tile are placed on one XCD and meet
 * in its L2.  Every split but the last stores its accumulators into a zero-initialised mailbox (with +0.0
 * written as -0.0, so that no word is zero); the waves of the last split poll the mailbox until nothing is
 * missing, store zeros back and add the partials in split order, their own last -- the second kernel's
 * arithmetic, so the result equals its bit for bit and does not depend on timing (a wave that polls for a
 * second gives up and writes NaN).  mode -1 = by cost (default), 0 = never,
 * 1 = whenever the plan allows.  The first call that could use it on a device looks once at where that
 * device places workgroups (a probe grid the call waits for; skipped, and the two-kernel form used, while
 * the stream is being captured and the answer is not known yet).  The reference does not split K
 * (/root/reference/mn_small.hip:28); its README names filling the CUs for skinny shapes as the open
 * problem (/root/reference/README.md:161). */
int fp8_block_gemm_set_fused_reduction(int mode);

/* Grouped GEMM: `groups` independent problems with the same n and k and their own m[g]
 * (ragged M, e.g. the experts of one MoE layer), C[g] = A[g] . B[g]^T with the layouts above.
 * a, b, a_scale, b_scale, c and m are HOST arrays of `groups` entries; the pointers they hold
 * are device pointers.  Groups with m[g] == 0 are skipped; a call with one group left is
 * fp8_block_gemm_stream on that group.  Up to FP8GEMM_MAX_GROUPS problems
 * run as ONE launch of the persistent tile kernel (their tiles form one list that 256
 * workgroups walk through): as they are when every m[g] and n are multiples of 16 and the
 * operands 16-byte aligned, else on zero-padded copies in the workspace made by one batched copy
 * launch per operand kind ("padded_..._groupedN").  Groups of at most 64 rows (the experts of an MoE
 * layer in a decode step) do not go through 128-row tiles: they run as ONE launch of the decode kernel
 * ("decode128_kN_groupedG": 128-column strips of every group in one work list, every group's B read
 * once, the K range split and added inside the kernel as for a single problem; row counts off the 16-row
 * grid as they are, without copies, except in launches large enough for the streaming form -- 256 or more
 * strips of 256 columns over all groups --, which runs on padded copies of A and a_scale); a call that mixes
 * both kinds launches each kernel once, unless the small groups are few beside the taller ones (at most a third
 * as many), which then join the tile launch.  The tile shape of a grouped launch comes from a cost model of its
 * own (its own tile count, K blocks priced for operands from HBM: mostly the 256x256 tile, which streams a
 * group's B once per 256 rows in pieces of 256 bytes).  A tile launch of at most 8 groups that
 * would leave more than a third of the CUs without a tile while K >= 2048 is not made: those groups run one by
 * one, where the dispatcher splits K.  A launch holds FP8GEMM_MAX_GROUPS problems; more of a kind run as
 * the fewest launches that hold them, of equal size, one after the other on the stream ("...groupedGxL":
 * L launches, the last of G groups).  Each C[g] is bit-identical to
 * what fp8_block_gemm_stream gives for that problem with the same tile shape (decode kernel: with the
 * same K split).  No counterpart in the
 * reference, which launches one problem at a time (/root/reference/check.cu:106-114). */
#define FP8GEMM_MAX_GROUPS 64
int fp8_block_gemm_grouped(int groups, const void* const* a, const void* const* b,
                           const float* const* a_scale, const float* const* b_scale,
                           void* const* c, const int* m, int n, int k, void* stream);

/* Per-call form.  `options` (NULL = automatic dispatch) replaces the process-wide switches above for
 * this call only; `workspace` (256-byte aligned device memory of `workspace_bytes`; NULL / 0 when the
 * plan needs none) replaces the process-wide workspace: the call allocates nothing, synchronises
 * nothing and returns FP8GEMM_E_WORKSPACE when the plan needs more than it was given
 * (fp8_block_gemm_workspace_bytes_ex tells how much).  Safe to call from several host threads and on
 * several streams at once with distinct workspaces, and under stream capture.  No counterpart in the
 * reference, whose launcher is single-threaded on stream 0 (/root/reference/check.cu:106-119). */
typedef struct fp8gemm_options {
    int kernel;       /* FP8GEMM_KERNEL_* */
    int tile_variant; /* as fp8_block_gemm_force_config; -1 = cost model */
    int ksplit;       /* 0 = cost model, else 1..16 */
    int persistent;   /* as fp8_block_gemm_set_persistent */
    int flags;        /* FP8GEMM_FLAG_* or 0 */
} fp8gemm_options;
/* The first FP8GEMM_WORKSPACE_HEADER_BYTES of the workspace handed to this call were zero-filled by the
 * caller before the first call that used this workspace, and nothing but this library has written to the
 * workspace since.  The plans that add the K splits of a tile or strip inside the GEMM kernel instead of
 * launching a reduction kernel ("decode128_kN", "..._kNf") hand their partial results over through it (a
 * mailbox of 16 MiB) and leave all of it zero again after every call; without the flag a per-call workspace
 * only gets the two-kernel plans.
 * The process-wide workspace and fp8_block_gemm_noalloc's array always have a zeroed header.  Calls that
 * share a workspace and overlap on the device (which the contract forbids) can leave the header non-zero
 * and later results wrong: zero it again before the next use (fp8_block_gemm_release() drops the
 * library-owned buffer, whose successor starts out zeroed). */
#define FP8GEMM_FLAG_WORKSPACE_ZEROED 1
#define FP8GEMM_WORKSPACE_HEADER_BYTES (16u << 20)
int fp8_block_gemm_ex(const void* a, const void* b, const float* a_scale, const float* b_scale, void* c,
                      int m, int n, int k, const fp8gemm_options* options, void* workspace,
                      size_t workspace_bytes, void* stream);
/* fp8_block_gemm_ex with automatic dispatch. */
int fp8_block_gemm_ws(const void* a, const void* b, const float* a_scale, const float* b_scale, void* c,
                      int m, int n, int k, void* workspace, size_t workspace_bytes, void* stream);
/* Workspace bytes fp8_block_gemm_ex needs for (m, n, k) under `options` (NULL = automatic).
 * any_alignment = 0: for a, b, a_scale, c on 16-byte boundaries (what allocators return);
 * any_alignment != 0: an upper bound that also covers operands off such a boundary, which run on
 * padded copies of every operand concerned (for cfg-sized shapes that is the size of all operands).
 * Touches no device.  0 for an invalid shape or options. */
size_t fp8_block_gemm_workspace_bytes_ex(int m, int n, int k, const fp8gemm_options* options,
                                         int any_alignment);
/* Per-call form of fp8_block_gemm_grouped: same arguments and results, with `options` and `workspace`
 * as for fp8_block_gemm_ex (nothing process-wide is read or written, nothing is allocated; safe from
 * several host threads on several streams with distinct workspaces, and under stream capture).
 * fp8_block_gemm_grouped_workspace_bytes_ex bounds the workspace for any alignment of the operands;
 * with less than that (or none) the groups that need a workspace run one by one, or the call returns
 * FP8GEMM_E_WORKSPACE when a single group needs more than it was given.  The decode kernel splits K
 * only with FP8GEMM_FLAG_WORKSPACE_ZEROED.  No counterpart in the reference (one problem at a time on
 * stream 0, /root/reference/check.cu:106-119). */
int fp8_block_gemm_grouped_ex(int groups, const void* const* a, const void* const* b,
                              const float* const* a_scale, const float* const* b_scale, void* const* c,
                              const int* m, int n, int k, const fp8gemm_options* options, void* workspace,
                              size_t workspace_bytes, void* stream);
size_t fp8_block_gemm_grouped_workspace_bytes_ex(int groups, const int* m, int n, int k,
                                                 const fp8gemm_options* options);

/* fp8_block_gemm_stream for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same dispatch under the same process-wide switches, but
 * the workspace of plans that split K or pad is a fixed array inside the library's device image,
 * FP8GEMM_NOALLOC_MAX_BYTES per GPU, held until the process ends.  The call allocates and frees nothing.
 * A plan that needs more than that returns FP8GEMM_E_WORKSPACE (ask fp8_block_gemm_workspace_bytes /
 * _ex beforehand; plans that neither split K nor pad need nothing and always fit).  All calls on one
 * GPU share that GPU's array: calls that use it and overlap on the device (different streams) race, as
 * with the process-wide workspace.  The caller clears nothing: the array starts out zero, the plans that
 * use its first FP8GEMM_WORKSPACE_HEADER_BYTES (the mailbox of the K splits) leave them zero, every other
 * plan writes what it later reads.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress); make that call outside a stream capture.  This entry point has no counterpart in
 * the reference. */
#define FP8GEMM_NOALLOC_MAX_BYTES (32u << 20)
int fp8_block_gemm_noalloc(const void* a, const void* b, const float* a_scale, const float* b_scale,
                           void* c, int m, int n, int k, void* stream);

/* Writes the name of the kernel plan the dispatcher would launch for (m, n, k) with
 * 16-byte aligned operands into name[0..cap), e.g. "tile256x192_k1_persistent", "tile128x128_k3", "skinny_k1", "padded_tile64x64_k1", "scalar".
 * Touches no device.  Returns 0, or a negative code for an invalid shape.  No counterpart
 * in the reference (its choice is made by editing the source, README.md:55). */
int fp8_block_gemm_plan(int m, int n, int k, char* name, size_t cap);

/* Name of the kernel plan the last successful GEMM call on this thread launched
 * (static storage, never NULL).  No counterpart in the reference: diagnostics. */
const char* fp8_block_gemm_last_kernel(void);

/* The process-wide workspace of the entry points without a workspace argument.  Plans that split K
 * ("..._kN", N > 1) keep fp32 partial tiles there, plans for operands off the 16-byte grid
 * ("padded_...") their copies; other plans never touch it.  By default the library owns a buffer that
 * it allocates on first need and replaces by a larger one when a call needs more; the outgrown buffer
 * is kept until fp8_block_gemm_release, so kernels in flight and graphs captured earlier stay valid --
 * but a graph replays into the buffer it was captured with, which later calls no longer share: give
 * captured work a workspace of its own.  A call that would have to allocate while its stream is being
 * captured returns FP8GEMM_E_WORKSPACE and leaves the capture valid.
 * fp8_block_gemm_set_workspace supplies a caller-owned buffer instead (256-byte aligned; NULL returns
 * to the library-owned one); it must hold fp8_block_gemm_workspace_bytes(m, n, k) for every shape
 * passed: what the plan needs under the switches in force when asked, for 16-byte aligned operands
 * (0 when the plan neither splits K nor pads; operands off a 16-byte boundary need what
 * fp8_block_gemm_workspace_bytes_ex(m, n, k, NULL, 1) returns).  fp8_block_gemm_grouped_workspace_bytes
 * bounds what fp8_block_gemm_grouped takes for any alignment; with a smaller caller-owned buffer the
 * groups run one by one.  There is ONE such workspace per process, on the device that was current when
 * it was allocated or supplied: calls that use it must not overlap on different streams.  The reference
 * has no workspace (its kernels do not split K: mn_small.hip:28). */
size_t fp8_block_gemm_workspace_bytes(int m, int n, int k);
size_t fp8_block_gemm_grouped_workspace_bytes(int groups, const int* m, int n, int k);
int fp8_block_gemm_set_workspace(void* device_ptr, size_t bytes);
int fp8_block_gemm_release(void);
/* Growth policy of the library-owned workspace: the size it is (re)allocated with when a call needs
 * `need` bytes and it holds `have` (at least twice `have`, so that outgrown buffers never add up to more
 * than the live one).  An outgrown buffer is freed by a later growth once the work that last used it has
 * completed; one that was handed to a call under stream capture is kept until fp8_block_gemm_release.
 * Touches no device.  No counterpart in the reference. */
size_t fp8_block_gemm_workspace_growth(size_t have, size_t need);

/* fp32 -> fp8 e4m3fn, round to nearest even, saturating to +-448; count elements; `in` 16-byte and
 * `out` 4-byte aligned (FP8GEMM_E_ALIGN otherwise).
 * Replaces convert_float_to_fp8<<<M*K/256, 256>>> (/root/reference/check.cu:17-22, 83-84);
 * unlike that launch it also converts a tail that is not a multiple of 256. */
int fp8_convert_f32_to_e4m3fn(const float* in, void* out, size_t count, void* stream);

/* Quantise activations for the GEMM's `a` operand: x is [m][k] row-major (k contiguous),
 * bf16 or fp32 (x_dtype = FP8GEMM_DTYPE_*), 16-byte aligned.  Per row and 128-wide K group:
 * scale = (1 / max(amax, 1e-12)) * 448 (torch's evaluation order of finfo.max / amax),
 * a = fp8_rne(clamp(x * scale, +-448)) written at m + k*M, a_scale = 1 / scale written at
 * m + kb*M.  Replaces
 * to_float8_rowwise_scale (/root/reference/quantize.py:43-67, with the e4m3fn maximum 448
 * instead of fnuz's 240) together with the host-side transposes that bring its outputs into
 * the kernel's layouts (row_to_col_major, /root/reference/check.cu:164-167). */
int fp8_quantize_a_1x128(const void* x, int x_dtype, void* a, float* a_scale, int m, int k,
                         void* stream);

/* Quantise weights for the GEMM's `b` operand: x is [n][k] row-major, one scale per
 * 128 x 128 block (a last block of fewer than 128 rows takes its amax over the rows that
 * exist), b written at n + k*N, b_scale at nb + kb*ceil(N/128).  Replaces
 * to_float8_block_scale (/root/reference/quantize.py:16-41; that function drops a partial
 * last block, quantize.py:23-26) and the same transposes. */
int fp8_quantize_b_128x128(const void* x, int x_dtype, void* b, float* b_scale, int n, int k,
                           void* stream);

/* Text for a return code of any function above (static storage). */
const char* fp8_block_gemm_error_string(int code);

/* ABI version of this header: bumped on any incompatible change. */
int fp8_block_gemm_abi_version(void);

/* ---- host-buffer convenience layer: the reference's host launcher ----
 * Counterpart of gemmGPU (/root/reference/check.cu:51-130): takes HOST buffers with fp32
 * values for a and b (already in the column-major layouts above), allocates device
 * memory, uploads, converts fp32 -> fp8 on the device, runs the kernel selected by
 * `option`, downloads c (bf16 bits) and frees.  option: 2 = scalar definition kernel,
 * 0 = automatic dispatch, 1 = same as 0 (the reference's "reverse" grid has no meaning
 * here), or 100 + FP8GEMM_KERNEL_* to force a family.  Synchronous. */
int fp8_gemm_host(unsigned short* c, const float* a, const float* b, const float* a_scale,
                  const float* b_scale, size_t m, size_t n, size_t k, int option);

#ifdef __cplusplus
}
#endif
#endif /* FP8_BLOCK_GEMM_H */
