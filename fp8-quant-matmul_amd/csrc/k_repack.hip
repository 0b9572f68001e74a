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

// dst[r][0..ld_dst) = src[r][0..ld_src) followed by zeros; ld_dst is a multiple of 4 floats and
// dst is 16-byte aligned.  One thread (number idx) writes one 16-byte piece.
__device__ __forceinline__ void pad_piece_floats(const float* __restrict__ src, float* __restrict__ dst, int rows,
                                                 int ld_src, int ld_dst, size_t idx)
{
    const int chunks = ld_dst / 4;
    if (idx >= (size_t)rows * chunks)
        return;
    const int r = (int)(idx / chunks), ch = (int)(idx - (size_t)r * chunks);
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = ch * 4 + j;
        v[j] = col < ld_src ? src[(size_t)r * ld_src + col] : 0.0f;
    }
    *reinterpret_cast<float4*>(dst + (size_t)r * ld_dst + (size_t)ch * 4) = make_float4(v[0], v[1], v[2], v[3]);
}

// The same for bytes (ld_dst a multiple of 16), at dword speed whatever the alignment of a source
// row: the (up to five) aligned dwords that hold the 16 source bytes are read and shifted into
// place.  The first and the last dword may reach up to 3 bytes beyond the row: they stay inside
// the aligned dwords that hold the matrix's first and last byte, so no access leaves its pages.
__device__ __forceinline__ void pad_piece_bytes(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, int rows,
                                                int ld_src, int ld_dst, size_t idx)
{
    const int chunks = ld_dst / 16;
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
__device__ __forceinline__ void crop_piece(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int m, int n,
                                           int ld_src, size_t idx)
{
    const int chunks = (n + 7) / 8;
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

enum RepackKind { REPACK_PAD_BYTES, REPACK_PAD_FLOATS, REPACK_CROP_BF16 };

template <int KIND>
__device__ __forceinline__ void repack_piece(const void* src, void* dst, int rows, int ld_src, int ld_dst, size_t idx)
{
    if (KIND == REPACK_PAD_BYTES)
        pad_piece_bytes(static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), rows, ld_src, ld_dst, idx);
    else if (KIND == REPACK_PAD_FLOATS)
        pad_piece_floats(static_cast<const float*>(src), static_cast<float*>(dst), rows, ld_src, ld_dst, idx);
    else  // rows = m, ld_dst = n
        crop_piece(static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), rows, ld_dst, ld_src, idx);
}

template <int KIND>
__host__ __device__ inline size_t repack_pieces(int rows, int ld_dst)
{
    return (size_t)rows * (KIND == REPACK_PAD_BYTES ? ld_dst / 16 : KIND == REPACK_PAD_FLOATS ? ld_dst / 4
                                                                                                : (ld_dst + 7) / 8);
}

template <int KIND>
__global__ void __launch_bounds__(256)
repack_kernel(const void* __restrict__ src, void* __restrict__ dst, int rows, int ld_src, int ld_dst)
{
    repack_piece<KIND>(src, dst, rows, ld_src, ld_dst, (size_t)blockIdx.x * blockDim.x + threadIdx.x);
}

// one matrix per blockIdx.y
template <int KIND>
__global__ void __launch_bounds__(256) repack_batched_kernel(const RepackTable tab)
{
    const int g = blockIdx.y;
    repack_piece<KIND>(tab.src[g], tab.dst[g], tab.rows[g], tab.ld_src[g], tab.ld_dst[g],
                       (size_t)blockIdx.x * blockDim.x + threadIdx.x);
}

// up to PadJobs::MAX padding copies of either kind in one launch, one per blockIdx.y
__global__ void __launch_bounds__(256) pad_jobs_kernel(const PadJobs jobs)
{
    const PadJob& j = jobs.job[blockIdx.y];
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j.floats)
        pad_piece_floats(static_cast<const float*>(j.src), static_cast<float*>(j.dst), j.rows, j.ld_src, j.ld_dst, idx);
    else
        pad_piece_bytes(static_cast<const uint8_t*>(j.src), static_cast<uint8_t*>(j.dst), j.rows, j.ld_src, j.ld_dst, idx);
}

// the byte copies (blockIdx.z = 0) and the fp32 copies (blockIdx.z = 1) of several problems in one launch
__global__ void __launch_bounds__(256) pad_pair_batched_kernel(const RepackTable bytes, const RepackTable floats)
{
    const int g = blockIdx.y;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (blockIdx.z == 0)
        repack_piece<REPACK_PAD_BYTES>(bytes.src[g], bytes.dst[g], bytes.rows[g], bytes.ld_src[g], bytes.ld_dst[g], idx);
    else
        repack_piece<REPACK_PAD_FLOATS>(floats.src[g], floats.dst[g], floats.rows[g], floats.ld_src[g], floats.ld_dst[g], idx);
}

template <int KIND>
hipError_t launch_repack(const void* src, void* dst, int rows, int ld_src, int ld_dst, hipStream_t s)
{
    const size_t pieces = repack_pieces<KIND>(rows, ld_dst);
    if (pieces == 0)
        return hipSuccess;
    hipLaunchKernelGGL((repack_kernel<KIND>), dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, s, src, dst,
                       rows, ld_src, ld_dst);
    return hipGetLastError();
}

template <int KIND>
hipError_t launch_repack_batched(const RepackTable& tab, hipStream_t s)
{
    if (tab.groups < 1 || tab.groups > RepackTable::MAX_GROUPS)
        return hipErrorInvalidValue;
    size_t most = 0;
    for (int g = 0; g < tab.groups; ++g) {
        const size_t pieces = repack_pieces<KIND>(tab.rows[g], tab.ld_dst[g]);
        most = pieces > most ? pieces : most;
    }
    if (most == 0)
        return hipSuccess;
    hipLaunchKernelGGL((repack_batched_kernel<KIND>), dim3((unsigned)((most + 255) / 256), (unsigned)tab.groups),
                       dim3(256), 0, s, tab);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_pad_jobs(const PadJobs& jobs, hipStream_t s)
{
    if (jobs.count < 0 || jobs.count > PadJobs::MAX)
        return hipErrorInvalidValue;
    size_t most = 0;
    for (int i = 0; i < jobs.count; ++i) {
        const PadJob& j = jobs.job[i];
        const size_t pieces = j.floats ? repack_pieces<REPACK_PAD_FLOATS>(j.rows, j.ld_dst)
                                       : repack_pieces<REPACK_PAD_BYTES>(j.rows, j.ld_dst);
        most = pieces > most ? pieces : most;
    }
    if (most == 0)
        return hipSuccess;
    hipLaunchKernelGGL(pad_jobs_kernel, dim3((unsigned)((most + 255) / 256), (unsigned)jobs.count), dim3(256), 0, s, jobs);
    return hipGetLastError();
}

hipError_t launch_crop_bf16(const uint16_t* src, uint16_t* dst, int m, int n, int ld_src, hipStream_t s)
{
    return launch_repack<REPACK_CROP_BF16>(src, dst, m, ld_src, n, s);
}

hipError_t launch_pad_pair_batched(const RepackTable& bytes, const RepackTable& floats, hipStream_t s)
{
    if (bytes.groups < 1 || bytes.groups > RepackTable::MAX_GROUPS || floats.groups != bytes.groups)
        return hipErrorInvalidValue;
    size_t most = 0;
    for (int g = 0; g < bytes.groups; ++g) {
        const size_t pb = repack_pieces<REPACK_PAD_BYTES>(bytes.rows[g], bytes.ld_dst[g]);
        const size_t pf = repack_pieces<REPACK_PAD_FLOATS>(floats.rows[g], floats.ld_dst[g]);
        most = pb > most ? pb : most;
        most = pf > most ? pf : most;
    }
    if (most == 0)
        return hipSuccess;
    hipLaunchKernelGGL(pad_pair_batched_kernel, dim3((unsigned)((most + 255) / 256), (unsigned)bytes.groups, 2), dim3(256), 0, s,
                       bytes, floats);
    return hipGetLastError();
}

hipError_t launch_pad_bytes_batched(const RepackTable& tab, hipStream_t s)
{
    return launch_repack_batched<REPACK_PAD_BYTES>(tab, s);
}

hipError_t launch_crop_bf16_batched(const RepackTable& tab, hipStream_t s)
{
    return launch_repack_batched<REPACK_CROP_BF16>(tab, s);
}

}  // namespace fp8gemm
