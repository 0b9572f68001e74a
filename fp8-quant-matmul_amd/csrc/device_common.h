// Device-side helpers shared by the gfx950 kernels: vector types, fp8 e4m3fn (OCP) decode,
// bf16 packing, LDS / buffer-resource pointer casts.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef int v32i __attribute__((ext_vector_type(32)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

constexpr int KBLOCK = 128;  // K extent of one scale block (check.cu:15 BLOCK)

// e4m3fn bit pattern -> fp32.  Exponent bias 7, subnormal step 2^-9, 0x7F/0xFF = NaN.
__device__ __forceinline__ float e4m3fn_to_f32(uint8_t v)
{
    uint32_t sign = (uint32_t)(v & 0x80) << 24;
    uint32_t e = (v >> 3) & 15, m = v & 7;
    uint32_t bits;
    if (e == 15 && m == 7)
        bits = 0x7FC00000u;
    else if (e == 0)
        bits = __float_as_uint((float)m * 0.001953125f);  // m * 2^-9
    else
        bits = ((e + 120) << 23) | (m << 20);
    return __uint_as_float(bits | sign);
}

// two fp32 -> packed bf16 (round to nearest even, hardware v_cvt_pk_bf16_f32); low half = x
__device__ __forceinline__ uint32_t pack_bf16x2(float x, float y)
{
    v2f f = {x, y};
    v2bf h = __builtin_convertvector(f, v2bf);
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float x)
{
    return (uint16_t)(pack_bf16x2(x, 0.0f) & 0xFFFFu);
}

// Raw buffer resource over [base, base+bytes): loads past the end return 0 instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// The same resource as four plain words, for inline assembly operands.
__device__ __forceinline__ v4i make_rsrc_words(const void* base, uint32_t bytes)
{
    const uint64_t ad = reinterpret_cast<uint64_t>(base);
    return (v4i){(int)(uint32_t)ad, (int)((ad >> 32) & 0xFFFFu), (int)bytes, 0x00020000};
}

// One 16-byte-per-lane buffer load whose destination is LDS: lane l's 16 bytes land at
// lds_addr + 16*l (lds_addr wave-uniform, handed over in M0); a lane whose voffset is
// outside the resource writes zeros.  Written as assembly on purpose: the compiler's wait
// insertion treats every LDS read after a compiler-visible LDS-writing load as dependent on
// it and would wait for the copy of the NEXT stage before reading the current one.  The
// caller orders these copies itself (s_waitcnt vmcnt(0) + barrier before the data is read).
// M0 is a reserved register: the compiler writes it immediately before each of its own uses and
// keeps no value in it across other code, and clang rejects it in a clobber list for that reason.
// soffset is a wave-uniform byte offset added to the global address only (not range checked,
// not part of the LDS address).
__device__ __forceinline__ void lds_dma16(v4i rsrc, uint32_t voffset, uint32_t lds_addr,
                                          uint32_t soffset = 0)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %3 offen lds"
                 :
                 : "v"(voffset), "s"(rsrc), "s"(lds_addr), "s"(soffset)
                 : "memory");
}

// The same with 4 bytes per lane: lane l's dword lands at lds_addr + 4*l (256 bytes per wave).
__device__ __forceinline__ void lds_dma4(v4i rsrc, uint32_t voffset, uint32_t lds_addr, uint32_t soffset = 0)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tbuffer_load_dword %0, %1, %3 offen lds"
                 :
                 : "v"(voffset), "s"(rsrc), "s"(lds_addr), "s"(soffset)
                 : "memory");
}
