// Host-buffer launcher: the counterpart of gemmGPU (/root/reference/check.cu:51-130,
// /root/reference/sgemm.cu:24-191).  Allocate, upload, convert fp32 -> fp8 on the device,
// launch, download, free -- with every HIP return code checked instead of discarded.
#include "../../include/fp8_block_gemm.h"
#include "launchers.h"

#include <cstdint>

namespace {

struct DeviceBuf {
    void* p = nullptr;
    ~DeviceBuf()
    {
        if (p)
            (void)hipFree(p);
    }
    hipError_t alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 1); }
};

}  // namespace

extern "C" int fp8_gemm_host(unsigned short* c, const float* a, const float* b, const float* a_scale,
                             const float* b_scale, size_t m, size_t n, size_t k, int option)
{
    if (!c || !a || !b || !a_scale || !b_scale)
        return FP8GEMM_E_NULLPTR;
    if (m == 0 || n == 0 || k == 0 || k % 128 != 0)
        return FP8GEMM_E_SHAPE;
    if (m * k > 0x7FFFFFFFull || n * k > 0x7FFFFFFFull || m * n > 0x7FFFFFFFull)
        return FP8GEMM_E_TOOLARGE;
    const size_t nkb = k / 128, sn = (n + 127) / 128;
    DeviceBuf d_a32, d_b32, d_a8, d_b8, d_as, d_bs, d_c;
    hipError_t e;
#define TRY(x)                 \
    do {                       \
        e = (x);               \
        if (e != hipSuccess)   \
            return (int)e;     \
    } while (0)
    TRY(d_a32.alloc(m * k * sizeof(float)));
    TRY(d_b32.alloc(n * k * sizeof(float)));
    TRY(d_a8.alloc(m * k));
    TRY(d_b8.alloc(n * k));
    TRY(d_as.alloc(nkb * m * sizeof(float)));
    TRY(d_bs.alloc(nkb * sn * sizeof(float)));
    TRY(d_c.alloc(m * n * 2));
    TRY(hipMemcpy(d_a32.p, a, m * k * sizeof(float), hipMemcpyHostToDevice));
    TRY(hipMemcpy(d_b32.p, b, n * k * sizeof(float), hipMemcpyHostToDevice));
    TRY(hipMemcpy(d_as.p, a_scale, nkb * m * sizeof(float), hipMemcpyHostToDevice));
    TRY(hipMemcpy(d_bs.p, b_scale, nkb * sn * sizeof(float), hipMemcpyHostToDevice));
    int rc = fp8_convert_f32_to_e4m3fn(static_cast<const float*>(d_a32.p), d_a8.p, m * k, nullptr);
    if (rc != 0)
        return rc;
    rc = fp8_convert_f32_to_e4m3fn(static_cast<const float*>(d_b32.p), d_b8.p, n * k, nullptr);
    if (rc != 0)
        return rc;
    const float* das = static_cast<const float*>(d_as.p);
    const float* dbs = static_cast<const float*>(d_bs.p);
    // per-call options and a workspace of this call's own: no process-wide switch is touched
    fp8gemm_options opt{FP8GEMM_KERNEL_AUTO, -1, 0, -1, 0};
    if (option == 2)
        opt.kernel = FP8GEMM_KERNEL_SCALAR;
    else if (option >= 100 && option <= 100 + FP8GEMM_KERNEL_SKINNY)
        opt.kernel = option - 100;
    else if (option != 0 && option != 1)
        return FP8GEMM_E_KERNEL;
    const size_t ws_bytes = fp8_block_gemm_workspace_bytes_ex((int)m, (int)n, (int)k, &opt, 0);
    DeviceBuf d_ws;
    if (ws_bytes)
        TRY(d_ws.alloc(ws_bytes));
    rc = fp8_block_gemm_ex(d_a8.p, d_b8.p, das, dbs, d_c.p, (int)m, (int)n, (int)k, &opt, d_ws.p, ws_bytes,
                           nullptr);
    if (rc != 0)
        return rc;
    TRY(hipMemcpy(c, d_c.p, m * n * 2, hipMemcpyDeviceToHost));  // blocking: also the sync
#undef TRY
    return FP8GEMM_OK;
}
