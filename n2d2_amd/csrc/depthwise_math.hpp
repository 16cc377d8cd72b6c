// Device arithmetic shared by the kernels that compute a 3x3 depthwise convolution (depthwise.hip, dw_pw.hip).
#pragma once

#include <hip/hip_runtime.h>

namespace n2d2hip {

// One input row of a column as the dot products want it: per channel a dword (left, middle, right, 0).
struct Row4 { int c[4]; };

// xm, x0, xp: the 4 channel bytes of the pixels left of, at and right of the column
__device__ __forceinline__ Row4 transpose3(unsigned xm, unsigned x0, unsigned xp)
{
    const unsigned lo = __builtin_amdgcn_perm(x0, xm, 0x05010400u);   // m0 c0 m1 c1
    const unsigned hi = __builtin_amdgcn_perm(x0, xm, 0x07030602u);   // m2 c2 m3 c3
    Row4 r;
    r.c[0] = (int)__builtin_amdgcn_perm(xp, lo, 0x0c040100u);
    r.c[1] = (int)__builtin_amdgcn_perm(xp, lo, 0x0c050302u);
    r.c[2] = (int)__builtin_amdgcn_perm(xp, hi, 0x0c060100u);
    r.c[3] = (int)__builtin_amdgcn_perm(xp, hi, 0x0c070302u);
    return r;
}

} // namespace n2d2hip
