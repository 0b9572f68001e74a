// Padding copies for shapes the MFMA kernels cannot take as they are.
//
// The tile kernels move 16-byte pieces of A's and B's columns, which start at k*M and k*N:
// they need M and N to be multiples of 16 (and 16-byte aligned bases).  The reference asks
// for multiples of 64 or 32 and reads out of bounds otherwise (/root/reference/mn_large.hip:16).
// For any other shape the operands are copied into buffers whose leading dimension is rounded
// up to 16 (new rows zero), the GEMM runs on the padded problem into a padded C, and C's
// m x n corner is copied out.  All of it is plain data movement: 2 bytes moved per byte of a
// padded operand, 4 per element of C.
#include "device_common.h"
#include "launchers.h"

namespace fp8gemm {

namespace {

// dst[r][0..ld_dst) = src[r][0..ld_src) followed by zeros; ld_dst is a multiple of V elements
// and dst is 16-byte aligned.  One thread writes one 16-byte piece.
template <typename T>
__global__ void __launch_bounds__(256)
pad_rows_kernel(const T* __restrict__ src, T* __restrict__ dst, int rows, int ld_src, int ld_dst)
{
    constexpr int V = 16 / (int)sizeof(T);
    const int chunks = ld_dst / V;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * chunks)
        return;
    const int r = (int)(idx / chunks), ch = (int)(idx - (size_t)r * chunks);
    union {
        T v[V];
        uint4 q;
    } u;
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const int col = ch * V + j;
        u.v[j] = col < ld_src ? src[(size_t)r * ld_src + col] : T(0);
    }
    *reinterpret_cast<uint4*>(dst + (size_t)r * ld_dst + (size_t)ch * V) = u.q;
}

// The same for bytes, at dword speed whatever the alignment of a source row: the (up to five)
// aligned dwords that hold the 16 source bytes are read and shifted into place.  The first and
// the last dword may reach up to 3 bytes beyond the row: they stay inside the aligned dwords
// that hold the matrix's first and last byte, so no access leaves its pages.
__global__ void __launch_bounds__(256)
pad_rows_bytes_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int rows, int ld_src, int ld_dst)
{
    const int chunks = ld_dst / 16;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)rows * chunks)
        return;
    const int r = (int)(idx / chunks), ch = (int)(idx - (size_t)r * chunks);
    int valid = ld_src - 16 * ch;  // source bytes of this piece
    valid = valid < 0 ? 0 : (valid > 16 ? 16 : valid);
    const uintptr_t ad = reinterpret_cast<uintptr_t>(src) + (size_t)r * ld_src + (size_t)ch * 16;
    const uint32_t sh = (uint32_t)(ad & 3);
    const uint32_t* w = reinterpret_cast<const uint32_t*>(ad - sh);
    const int need = valid > 0 ? ((int)sh + valid + 3) >> 2 : 0;
    uint32_t in[5];
#pragma unroll
    for (int i = 0; i < 5; ++i)
        in[i] = i < need ? w[i] : 0u;
    uint32_t out[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t v = __builtin_amdgcn_alignbyte(in[i + 1], in[i], sh);
        const int left = valid - 4 * i;  // bytes of this dword that belong to the row
        out[i] = left >= 4 ? v : (left <= 0 ? 0u : (v & ((1u << (8 * left)) - 1u)));
    }
    *reinterpret_cast<uint4*>(dst + (size_t)r * ld_dst + (size_t)ch * 16) = make_uint4(out[0], out[1], out[2], out[3]);
}

// dst[m][n] (dense) = src[m][0..n) of a matrix with ld_src elements per row (a multiple of 8, base
// 16-byte aligned).  One thread moves 8 elements of a row: one 16-byte load, and one store as
// wide as the destination's alignment allows.
__global__ void __launch_bounds__(256)
crop_rows_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int m, int n, int ld_src)
{
    const int chunks = (n + 7) / 8;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)m * chunks)
        return;
    const int r = (int)(idx / chunks), ch = (int)(idx - (size_t)r * chunks);
    const uint4 v = *reinterpret_cast<const uint4*>(src + (size_t)r * ld_src + (size_t)ch * 8);
    uint16_t* d = dst + (size_t)r * n + (size_t)ch * 8;
    const int count = n - 8 * ch < 8 ? n - 8 * ch : 8;
    const uintptr_t ad = reinterpret_cast<uintptr_t>(d);
    const uint32_t wv[4] = {v.x, v.y, v.z, v.w};
    if (count == 8 && (ad & 15) == 0) {
        *reinterpret_cast<uint4*>(d) = v;
    } else if (count == 8 && (ad & 3) == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            reinterpret_cast<uint32_t*>(d)[i] = wv[i];
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (i < count)
                d[i] = (uint16_t)(wv[i >> 1] >> (16 * (i & 1)));
    }
}

template <typename T>
hipError_t launch_pad_typed(const T* src, T* dst, int rows, int ld_src, int ld_dst, hipStream_t s)
{
    const size_t pieces = (size_t)rows * (ld_dst / (16 / (int)sizeof(T)));
    if (pieces == 0)
        return hipSuccess;
    hipLaunchKernelGGL((pad_rows_kernel<T>), dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, s, src, dst,
                       rows, ld_src, ld_dst);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_pad_bytes(const uint8_t* src, uint8_t* dst, int rows, int ld_src, int ld_dst, hipStream_t s)
{
    const size_t pieces = (size_t)rows * (ld_dst / 16);
    if (pieces == 0)
        return hipSuccess;
    hipLaunchKernelGGL(pad_rows_bytes_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, s, src, dst,
                       rows, ld_src, ld_dst);
    return hipGetLastError();
}

hipError_t launch_pad_floats(const float* src, float* dst, int rows, int ld_src, int ld_dst, hipStream_t s)
{
    return launch_pad_typed<float>(src, dst, rows, ld_src, ld_dst, s);
}

hipError_t launch_crop_bf16(const uint16_t* src, uint16_t* dst, int m, int n, int ld_src, hipStream_t s)
{
    const size_t count = (size_t)m * ((n + 7) / 8);
    hipLaunchKernelGGL(crop_rows_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, src, dst, m, n,
                       ld_src);
    return hipGetLastError();
}

}  // namespace fp8gemm
