// Pieces shared by the tile kernels (k_tile.hip, k_tile_persistent.hip): LDS stage geometry,
// the chunk swizzle, the explicit wait on the copy counter.
#pragma once
#include "device_common.h"
#include "launchers.h"

#include <type_traits>

namespace fp8gemm {
namespace {

constexpr int NTHREADS = 512;
constexpr int GROUP_M = 8;  // tile rows per L2 locality group

// NW = waves of the workgroup (all of them copy): eight, or four for the kernels that run one wave
// per SIMD with twice the registers.
template <int BM, int BN, int WM, int WN, int NS, int NW = 8>
struct TileShape {
    static constexpr int RSA = BM > 128 ? 256 : (BM > 64 ? 128 : 64);  // LDS bytes per k-row of the A tile
    static constexpr int RSB = BN > 128 ? 256 : (BN > 64 ? 128 : 64);
    static constexpr int MAT_A = KBLOCK * RSA;
    static constexpr int MAT_B = KBLOCK * RSB;
    static constexpr int SCALE_OFF = MAT_A + MAT_B;       // BM a_scale floats
    static constexpr int SB_OFF = SCALE_OFF + 1024;       // four waves: 64 dwords, the first four = b_scale
    static constexpr int STAGE = MAT_A + MAT_B + 1024 + (NW == 4 ? 256 : 0);
    static constexpr int LDS_BYTES = NS * STAGE;
    static constexpr int NA = RSA / (8 * NW);             // copy instructions per wave, A tile
    static constexpr int NB = RSB / (8 * NW);
    static constexpr int NCOPY = NA + NB + 1;             // + the a_scale slice (wave 0 only; four
                                                          // waves: wave 1 brings b_scale as well)
    static_assert(NW == 4 || NW == 8, "four or eight waves");
    static_assert(NA * 8 * NW == RSA && NB * 8 * NW == RSB, "whole copy instructions per wave");
    // A wave's copy instructions of one matrix lie 4 (256-byte rows), 8 (128-byte rows) or 16
    // (64-byte rows) k-rows apart.  Instructions 8 rows apart share the chunk swizzle and hence
    // the per-lane offset: only NV distinct offsets are kept in registers, the row distance goes
    // into the instruction's scalar offset.
    static constexpr int NVA = RSA == 256 ? 2 : 1;
    static constexpr int NVB = RSB == 256 ? 2 : 1;
    // instruction q of a matrix with row stride RS: which kept offset, and how many k-rows on top
    template <int RS> static constexpr int voff_index(int q) { return RS == 256 ? (q & 1) : 0; }
    template <int RS> static constexpr int extra_rows(int q)
    {
        return RS == 256 ? (q >> 1) * 8 : q * (1024 / RS);
    }
    // lane of a copy instruction -> k-row within the instruction's 1 KiB and chunk position in it
    template <int RS> static __device__ __forceinline__ int copy_row(int lane) { return lane / (RS / 16); }
    template <int RS> static __device__ __forceinline__ int copy_pos(int lane) { return lane % (RS / 16); }
    static_assert(LDS_BYTES <= 160 * 1024, "stages exceed the 160 KiB of LDS");
};

// chunk swizzle of row r (0..7 within an 8-row group) for a row stride of RS bytes
template <int RS>
__device__ __forceinline__ int row_swizzle(int r)
{
    return RS == 256 ? 2 * (r & 7) : (RS == 128 ? 2 * ((r >> 1) & 3) : 2 * ((r >> 2) & 1));
}

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

}  // namespace
}  // namespace fp8gemm
