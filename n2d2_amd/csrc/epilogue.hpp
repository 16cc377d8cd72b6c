// Device-side rescale / saturate / activation shared by every kernel that ends
// an N2D2 cell: the integer restatement of Scaling::propagate
// (ref: src/Scaling_Kernels.cpp:29-199) followed by the Rectifier / Linear pass.
#pragma once

#include "common.h"

namespace n2d2hip {

__device__ __forceinline__ float as_f32(int x) { return __int_as_float(x); }

// std::round: half away from zero.  x - trunc(x) is exact in float.
__device__ __forceinline__ float round_half_away(float x)
{
    float r = truncf(x);
    float d = x - r;
    if (fabsf(d) >= 0.5f)
        r += copysignf(1.0f, x);
    return r;
}

__device__ __forceinline__ int clamp_i32(int v, int lo, int hi) { return min(max(v, lo), hi); }

// v: exact integer accumulator (bias included).  a..e: this channel's table row.
template <int KIND>
__device__ __forceinline__ int epi_apply(int v, int a, int b, int c, int d, int e, int lo, int hi, int relu)
{
    if (KIND == EPI_RAW) {
        return relu ? max(v, 0) : v;
    } else if (KIND == EPI_I24) {
        // Pre-clamped so that t*c + d fits 32 bits and t, c fit 24 bits.
        const int t = clamp_i32(v, a, b);
        const int r = (__mul24(t, c) + d) >> e;
        return clamp_i32(r, lo, hi);
    } else if (KIND == EPI_I64) {
        const int t = clamp_i32(v, a, b);
        const long long half = (e > 0) ? (1ll << (e - 1)) : 0ll;
        long long r = ((long long)t * (long long)c + half) >> e;
        r = r < (long long)lo ? (long long)lo : (r > (long long)hi ? (long long)hi : r);
        return (int)r;
    } else {
        float f = (float)v;
        f = fminf(fmaxf(f, as_f32(a)), as_f32(b));   // Clip (no-op bounds are -inf/+inf)
        f = f * as_f32(c);                            // one IEEE float32 multiply
        f = round_half_away(f);
        f = fminf(fmaxf(f, (float)lo), (float)hi);
        return (int)f;
    }
}

// Run-time dispatch for the bandwidth kernels (the branch is wave-uniform).
__device__ __forceinline__ int epi_apply_dyn(const EpiArgs& p, int v, int ch)
{
    switch (p.kind) {
    case EPI_RAW: return epi_apply<EPI_RAW>(v, 0, 0, 0, 0, 0, p.lo, p.hi, p.relu);
    case EPI_I24: return epi_apply<EPI_I24>(v, p.a[ch], p.b[ch], p.c[ch], p.d[ch], p.e[ch], p.lo, p.hi, 0);
    case EPI_I64: return epi_apply<EPI_I64>(v, p.a[ch], p.b[ch], p.c[ch], 0, p.e[ch], p.lo, p.hi, 0);
    default: return epi_apply<EPI_F32>(v, p.a[ch], p.b[ch], p.c[ch], 0, 0, p.lo, p.hi, 0);
    }
}

// Float-valued input (ElemWise with non-integer coefficients): the integer
// modes round it first, as the reference's `round(realInput)` does.
__device__ __forceinline__ int epi_apply_dyn_f(const EpiArgs& p, float f, int ch)
{
    if (p.kind == EPI_F32) {
        f = fminf(fmaxf(f, as_f32(p.a[ch])), as_f32(p.b[ch]));
        f = f * as_f32(p.c[ch]);
        f = round_half_away(f);
        f = fminf(fmaxf(f, (float)p.lo), (float)p.hi);
        return (int)f;
    }
    const float r = round_half_away(f);
    const int v = (int)fminf(fmaxf(r, -2147483520.0f), 2147483520.0f);
    return epi_apply_dyn(p, v, ch);
}

// Logical value of a stored element.
__device__ __forceinline__ int load_value(const void* p, size_t i, int dtype)
{
    switch (dtype) {
    case N2D2HIP_U8: return (int)((const unsigned char*)p)[i];
    case N2D2HIP_I8: return (int)((const signed char*)p)[i];
    case N2D2HIP_U8B: return (int)((const signed char*)p)[i] + 128;
    case N2D2HIP_I32: return ((const int*)p)[i];
    default: return (int)round_half_away(((const float*)p)[i]);
    }
}

// Stores a logical value, saturating to the destination type.
__device__ __forceinline__ void store_value(void* p, size_t i, int dtype, int v)
{
    switch (dtype) {
    case N2D2HIP_U8: ((unsigned char*)p)[i] = (unsigned char)clamp_i32(v, 0, 255); break;
    case N2D2HIP_I8: ((signed char*)p)[i] = (signed char)clamp_i32(v, -128, 127); break;
    case N2D2HIP_U8B: ((signed char*)p)[i] = (signed char)(clamp_i32(v, 0, 255) - 128); break;
    case N2D2HIP_I32: ((int*)p)[i] = v; break;
    default: ((float*)p)[i] = (float)v; break;
    }
}

} // namespace n2d2hip
