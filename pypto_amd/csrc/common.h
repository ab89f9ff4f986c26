// Shared device/host helpers for the gfx950 kernels of the sparse-attention path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pto {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// two fp32 -> packed bf16 pair, round-to-nearest-even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    f32x2 v = {lo, hi};
    bf16x2 r = __builtin_convertvector(v, bf16x2);
    return __builtin_bit_cast(uint32_t, r);
}

// two fp32 -> packed fp16 pair, round-to-nearest-even (v_cvt_pk_f16_f32)
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi)
{
    f32x2 v = {lo, hi};
    f16x2 r = __builtin_convertvector(v, f16x2);
    return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// LDS transposing read (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane i receives
// element (i % 4) of the 4-element rows addressed by lanes i/4, 4 + i/4, 8 + i/4 and 12 + i/4.
__device__ __forceinline__ s16x4 lds_read_tr16(const uint16_t *p)
{
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(p));
}

typedef __attribute__((address_space(3))) uint8_t lds_byte_t;

// One LDS-DMA request: lane i's 16 bytes at base + lane_off land at lds_dst + 16*i.  base and lds_dst
// are wave-uniform.  Written as assembly so that the compiler tracks none of these requests: an
// explicit vmcnt wait follows them.
__device__ __forceinline__ void dma16_base(const void *base, const uint32_t lane_off, const uint32_t lds_dst)
{
    const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    const uint64_t ub = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32)) << 32);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(ub), "s"(dst) : "memory", "m0");
}
// the same with a full address per lane
__device__ __forceinline__ void dma16(const void *gaddr, const uint32_t lds_dst)
{
    const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gaddr), "s"(dst) : "memory", "m0");
}

// the same for the lanes of a mask only (the others request and write nothing); the mask is applied
// inside the statement, so no branch splits the caller's instruction stream
__device__ __forceinline__ void dma16_lanes(const void *gaddr, const uint32_t lds_dst, const uint64_t lanes)
{
    const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %3\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, off\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved) : "v"(gaddr), "s"(dst), "s"(lanes) : "memory", "m0");
}

// four bytes per lane: lane i's dword at gaddr lands at lds_dst + 4*i
__device__ __forceinline__ void dma4(const void *gaddr, const uint32_t lds_dst)
{
    const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_dst);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gaddr), "s"(dst) : "memory", "m0");
}
// s_waitcnt immediate for "at most n vector-memory operations outstanding" (the other counters unconstrained)
// compute units of the current device, cached per device ordinal; 0 if the device cannot be asked
// (host side, defined with the C ABI)
int cu_count();

constexpr int vmcnt_imm(const int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

}  // namespace pto
