// Small device helpers shared by the int8 matrix-core kernels: vector types, LDS reads whose wait is written by hand,
// saturating packs, magic-number division.
#pragma once

#include <hip/hip_runtime.h>

namespace n2d2hip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

template <int OFF>
__device__ __forceinline__ void lds_read128_nowait(v4i& v, unsigned addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
}
template <int OFF>
__device__ __forceinline__ void lds_read64_nowait(v2i& v, unsigned addr)
{
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_lgkm()
{
    asm volatile("s_waitcnt lgkmcnt(%0)" : : "n"(N) : "memory");
}
// Makes a register filled by an earlier asynchronous LDS read depend on the wait that precedes this call.
__device__ __forceinline__ void tie(v4i& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void tie(v2i& x) { asm volatile("" : "+v"(x)); }
typedef short v2s __attribute__((ext_vector_type(2)));
__device__ __forceinline__ v2s as_v2s(int x) { return __builtin_bit_cast(v2s, x); }
__device__ __forceinline__ v2s splat_v2s(int x) { return v2s{(short)x, (short)x}; }
__device__ __forceinline__ v2s clamp_v2s(v2s x, v2s lo, v2s hi)
{
    return __builtin_elementwise_min(__builtin_elementwise_max(x, lo), hi);
}
// two 16-bit values saturated to [0, 255], as the two low bytes of the result
__device__ __forceinline__ unsigned sat_pk_u8(v2s x)
{
    unsigned r;
    asm("v_sat_pk_u8_i16 %0, %1" : "=v"(r) : "v"(x));
    return r;
}
// four 32-bit values saturated to [0, 255], one byte each (first value in the lowest byte)
__device__ __forceinline__ unsigned sat_bytes_u8(int r0, int r1, int r2, int r3)
{
    const v2s lo = __builtin_amdgcn_cvt_pk_i16(r0, r1), hi = __builtin_amdgcn_cvt_pk_i16(r2, r3);   // saturating
    return sat_pk_u8(lo) | (sat_pk_u8(hi) << 16);
}
template <int N>
__device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(N) : "memory");
}
__device__ __forceinline__ int med3_i32(int x, int lo, int hi)
{
    int r;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(lo), "v"(hi));
    return r;
}
__device__ __forceinline__ float med3_f32(float x, float lo, float hi)
{
    float r;
    asm("v_med3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(lo), "v"(hi));
    return r;
}
// 4 saturated values -> one dword of bytes
__device__ __forceinline__ unsigned pack_bytes(int r0, int r1, int r2, int r3)
{
    const unsigned t01 = __builtin_amdgcn_perm((unsigned)r1, (unsigned)r0, 0x0c0c0400u);
    const unsigned t23 = __builtin_amdgcn_perm((unsigned)r3, (unsigned)r2, 0x0c0c0400u);
    return __builtin_amdgcn_perm(t23, t01, 0x05040100u);
}
// n / d for 0 <= n < 2^31 with a host-made (multiplier, shift); multiplier 0 stands for d == 1
__device__ __forceinline__ int div_magic(int n, unsigned mul, unsigned sh)
{
    return mul ? (int)(__umulhi((unsigned)n, mul) >> sh) : n;
}

} // namespace n2d2hip
