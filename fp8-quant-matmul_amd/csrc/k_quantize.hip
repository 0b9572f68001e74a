// Device-side quantisers: the producers of the GEMM's inputs.
//
//   1 x 128 groups along K per row   (to_float8_rowwise_scale, /root/reference/quantize.py:43-67)
//   128 x 128 blocks                 (to_float8_block_scale,   /root/reference/quantize.py:16-41)
//
// Arithmetic of both, with the OCP e4m3fn maximum 448:
//   scale = (1 / max(amax, 1e-12)) * 448;  q = fp8_rne(clamp(x * scale, -448, 448));  stored = 1 / scale
// (reciprocal first, then the product: that is how torch evaluates `finfo.max / amax`,
// quantize.py:28,54).  For an fp32 source every step is fp32.  For a bf16 source torch rounds
// every element-wise result to bf16 (1e-12, the reciprocal, the product with 448, x * scale);
// BF16MATH reproduces that, so that bytes and scales equal the reference's own outputs for
// either source type.  A bf16 source can also be quantised with fp32 arithmetic (more
// accurate, not what quantize.py computes).
//
// The source x is row-major [rows][K] (K contiguous), bf16 or fp32.  The outputs are written
// directly in the GEMM's layouts, which the reference produces with host-side transposes
// (/root/reference/check.cu:164-167):  q at row + k*rows, the 1 x 128 scales at row + kb*rows,
// the 128 x 128 scales at nb + kb*ceil(rows/128).
//
// One workgroup owns a 128-row x 128-k tile (one scale block, or 128 scale groups).  Sixteen
// lanes read one row's 128 elements as 16- or 32-byte pieces (whole cache lines per row); the
// fp8 bytes go through LDS transposed, and leave as 16-byte pieces of 128-byte row segments.
// The kernel moves 2 (or 4) bytes in and 1 byte out per element: it is bound by HBM.
#include "device_common.h"
#include "launchers.h"

namespace fp8gemm {

namespace {

// LDS bytes per k-row of the transposed tile of 128 (64) rows.  33 (17) dwords: the byte stores of a wave (16
// k-rows 8 apart, 4 adjacent rows of the source) fall into 8 banks two deep, the dword reads into distinct banks.
constexpr int q_stride(int rows) { return rows + 4; }

__device__ __forceinline__ void load8(const uint16_t* p, float (&v)[8])
{
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(u[i] << 16);
        v[2 * i + 1] = __uint_as_float(u[i] & 0xFFFF0000u);
    }
}

__device__ __forceinline__ void load8(const float* p, float (&v)[8])
{
    const float4 lo = reinterpret_cast<const float4*>(p)[0];
    const float4 hi = reinterpret_cast<const float4*>(p)[1];
    v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
    v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
}

__device__ __forceinline__ float clamp_pm448(float v)
{
    return fminf(fmaxf(v, -448.0f), 448.0f);
}

template <bool BF16MATH>
__device__ __forceinline__ float q_round(float v)
{
    return BF16MATH ? __uint_as_float(pack_bf16x2(v, 0.0f) << 16) : v;
}

template <bool BF16MATH>
__device__ __forceinline__ float q_value(float x, float scale)
{
    return clamp_pm448(q_round<BF16MATH>(x * scale));
}

// BLOCK = false: one scale per row and tile (1 x 128).  BLOCK = true: one per tile (128 x 128).
// QTILE = rows of a workgroup's tile: 128, or 64 for the 1 x 128 quantiser on matrices of a few hundred to a few
// thousand rows, whose 128-row tiles are too few workgroups to overlap one's loads with another's stores.
template <typename TIn, bool BLOCK, bool BF16MATH, int QTILE = 128>
__global__ void __launch_bounds__(256)
quantize_kernel(const TIn* __restrict__ x, uint8_t* __restrict__ q, float* __restrict__ scale_out,
                int rows, int K, int vec_store)
{
    static_assert(QTILE == 128 || (QTILE == 64 && !BLOCK), "128 rows, or 64 for the row-wise scales");
    constexpr int QSTRIDE = q_stride(QTILE);
    constexpr int PASSES = QTILE / 16;  // rows per thread
    __shared__ __attribute__((aligned(16))) uint8_t tile[128 * QSTRIDE];
    __shared__ float s_inv[QTILE];
    __shared__ float s_red[4];

    const int t = threadIdx.x;
    const int c = t & 15;   // 8-element piece of the row's 128
    const int r0 = t >> 4;  // row of the first pass; pass p handles row r0 + 16 p
    const int row0 = blockIdx.x * QTILE;
    const int kb = blockIdx.y;

    float v[PASSES][8];
    float amax[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int row = row0 + r0 + 16 * p;
        if (row < rows) {
            load8(x + (size_t)row * K + (size_t)kb * 128 + 8 * c, v[p]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                v[p][j] = 0.0f;
        }
        float a = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            a = fmaxf(a, __builtin_fabsf(v[p][j]));
        amax[p] = a;
    }

    if (BLOCK) {
        float a = amax[0];
#pragma unroll
        for (int p = 1; p < PASSES; ++p)
            a = fmaxf(a, amax[p]);
#pragma unroll
        for (int d = 1; d < 64; d <<= 1)
            a = fmaxf(a, __shfl_xor(a, d));
        if ((t & 63) == 0)
            s_red[t >> 6] = a;
        __syncthreads();
        a = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            amax[p] = a;
    } else {
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
#pragma unroll
            for (int d = 1; d < 16; d <<= 1)
                amax[p] = fmaxf(amax[p], __shfl_xor(amax[p], d));
    }

#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int r = r0 + 16 * p;
        const float recip = q_round<BF16MATH>(1.0f / fmaxf(amax[p], q_round<BF16MATH>(1e-12f)));
        const float scale = q_round<BF16MATH>(recip * 448.0f);
        int w0 = 0, w1 = 0;
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q_value<BF16MATH>(v[p][0], scale), q_value<BF16MATH>(v[p][1], scale), w0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q_value<BF16MATH>(v[p][2], scale), q_value<BF16MATH>(v[p][3], scale), w0, true);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q_value<BF16MATH>(v[p][4], scale), q_value<BF16MATH>(v[p][5], scale), w1, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q_value<BF16MATH>(v[p][6], scale), q_value<BF16MATH>(v[p][7], scale), w1, true);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            tile[(8 * c + j) * QSTRIDE + r] = (uint8_t)((uint32_t)w0 >> (8 * j));
            tile[(8 * c + 4 + j) * QSTRIDE + r] = (uint8_t)((uint32_t)w1 >> (8 * j));
        }
        if (!BLOCK && c == 0)
            s_inv[r] = 1.0f / scale;
        if (BLOCK && t == 0 && p == 0)
            scale_out[(size_t)kb * gridDim.x + blockIdx.x] = 1.0f / scale;
    }
    __syncthreads();

    if (!BLOCK && t < QTILE && row0 + t < rows)
        scale_out[(size_t)kb * rows + row0 + t] = s_inv[t];

    // k-row kk of the tile: QTILE bytes, one per source row; lane takes 16 of them
    constexpr int LPR = QTILE / 16;  // lanes per k-row
    const int dq = t % LPR;
#pragma unroll
    for (int pass = 0; pass < 128 * LPR / 256; ++pass) {
        const int kk = t / LPR + (256 / LPR) * pass;
        const uint32_t* src = reinterpret_cast<const uint32_t*>(tile + kk * QSTRIDE + 16 * dq);
        const uint32_t w[4] = {src[0], src[1], src[2], src[3]};
        const int first = row0 + 16 * dq;
        const size_t o = (size_t)(kb * 128 + kk) * rows + first;
        if (vec_store && first + 16 <= rows) {
            *reinterpret_cast<uint4*>(q + o) = make_uint4(w[0], w[1], w[2], w[3]);
        } else if (first + 16 <= rows) {
            // a row count off the 16-byte grid: the piece starts at any byte.  The bytes up to the next dword
            // boundary one by one, three whole dwords shifted into place, the rest one by one
            uint8_t* d = q + o;
            const uint32_t head = (4u - (uint32_t)(reinterpret_cast<uintptr_t>(d) & 3)) & 3;  // 0 ... 3 bytes
            if (head == 0) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    reinterpret_cast<uint32_t*>(d)[i] = w[i];
            } else {
#pragma unroll
                for (int j = 0; j < 3; ++j)
                    if ((uint32_t)j < head)
                        d[j] = (uint8_t)(w[0] >> (8 * j));
#pragma unroll
                for (int i = 0; i < 3; ++i)
                    *reinterpret_cast<uint32_t*>(d + head + 4 * i) = __builtin_amdgcn_alignbyte(w[i + 1], w[i], head);
#pragma unroll
                for (int j = 1; j < 4; ++j)  // bytes head + 12 ... 15 are bytes head ... 3 of the last dword
                    if ((uint32_t)j >= head)
                        d[12 + j] = (uint8_t)(w[3] >> (8 * j));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j)
                if (first + j < rows)
                    q[o + j] = (uint8_t)(w[j >> 2] >> (8 * (j & 3)));
        }
    }
}

// 128-row tiles of the 1 x 128 quantiser between these counts run as 64-row tiles
constexpr long HALF_TILE_LO = 1, HALF_TILE_HI = 2500;

template <typename TIn, bool BF16MATH>
void launch_quantize_typed(const TIn* x, uint8_t* q, float* scale_out, int rows, int k, bool block128,
                           hipStream_t s)
{
    const dim3 grid((rows + 127) / 128, k / 128);
    const int vec_store = (rows % 16 == 0) && (reinterpret_cast<uintptr_t>(q) % 16 == 0);
    if (block128)
        hipLaunchKernelGGL((quantize_kernel<TIn, true, BF16MATH>), grid, dim3(256), 0, s, x, q, scale_out, rows,
                           k, vec_store);
    else if (HALF_TILE_LO <= (long)grid.x * grid.y && (long)grid.x * grid.y <= HALF_TILE_HI)
        hipLaunchKernelGGL((quantize_kernel<TIn, false, BF16MATH, 64>), dim3((rows + 63) / 64, k / 128), dim3(256), 0, s, x,
                           q, scale_out, rows, k, vec_store);
    else
        hipLaunchKernelGGL((quantize_kernel<TIn, false, BF16MATH>), grid, dim3(256), 0, s, x, q, scale_out, rows,
                           k, vec_store);
}

}  // namespace

hipError_t launch_quantize(const void* x, QuantSource source, uint8_t* q, float* scale_out, int rows,
                           int k, bool block128, hipStream_t s)
{
    switch (source) {
    case QUANT_SOURCE_BF16:
        launch_quantize_typed<uint16_t, true>(static_cast<const uint16_t*>(x), q, scale_out, rows, k, block128, s);
        break;
    case QUANT_SOURCE_F32:
        launch_quantize_typed<float, false>(static_cast<const float*>(x), q, scale_out, rows, k, block128, s);
        break;
    case QUANT_SOURCE_BF16_F32MATH:
        launch_quantize_typed<uint16_t, false>(static_cast<const uint16_t*>(x), q, scale_out, rows, k, block128, s);
        break;
    default:
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace fp8gemm
