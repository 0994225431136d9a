// Pieces shared by every kernel that PRODUCES BlockQ8 activations: the block
// quantizer itself and the deterministic elementwise functions of the fused
// producers.
//
// Everything here has a bit-level definition that the CPU checker restates
// operation by operation: only IEEE add / mul / fma / div / sqrt (the build asks for
// correctly rounded division and square root), no hardware approximations
// (v_rcp / v_rsq / v_exp), no contraction the source does not spell out.  That is
// what lets a fused producer be compared byte for byte instead of "within a quant
// step".
#pragma once

#include "rein_common.h"

// ---- a 32-value sub-block lives in one 16-lane DPP row, two values per lane -------
// Lane l (0..15) of the row holds elements l ("lo") and l + 16 ("hi").  The xor
// butterfly 16, 8, 4, 2, 1 over the 32 elements is then: one local combine (level
// 16), and four cross-lane levels that all stay inside the row and run as DPP
// operand modifiers on the VALU (no LDS crossbar round trip per level):
//   xor 8  row_ror:8          xor 4  row_shl:4 on banks 0,2 + row_shr:4 on banks 1,3
//   xor 2  quad_perm [2,3,0,1]  xor 1  quad_perm [1,0,3,2]
// Every lane of the row ends with the result; the association order is exactly that
// of the 32-lane butterfly, level by level.
__device__ __forceinline__ float rein_row_xor4(float x)
{
    float t = rein_dpp_f32<0x104, 0xF, 0x5>(x, x);     // lanes 0-3, 8-11 <- lane + 4
    return rein_dpp_f32<0x114, 0xF, 0xA>(t, x);        // lanes 4-7, 12-15 <- lane - 4
}

__device__ __forceinline__ float rein_row_sum(float lo, float hi)
{
#pragma clang fp contract(off)
    float s = lo + hi;
    s = s + rein_dpp_f32<0x128>(s, s);
    s = s + rein_row_xor4(s);
    s = s + rein_dpp_f32<0x4E>(s, s);
    s = s + rein_dpp_f32<0xB1>(s, s);
    return s;
}

__device__ __forceinline__ float rein_row_max(float lo, float hi)
{
    float m = fmaxf(lo, hi);
    m = fmaxf(m, rein_dpp_f32<0x128>(m, m));
    m = fmaxf(m, rein_row_xor4(m));
    m = fmaxf(m, rein_dpp_f32<0x4E>(m, m));
    m = fmaxf(m, rein_dpp_f32<0xB1>(m, m));
    return m;
}

// Quantize the sub-block held by a row (lane l: elements l and l + 16) into *o.
// amax and sum reduce with the xor butterfly 16, 8, 4, 2, 1; d = amax/127 and
// inv = 127/amax are IEEE divisions; q = clamp(rint(v*inv), -127, 127), ties to
// even; an all-zero block stores d = 1.  Same output as
// kernels/quantize_q8.cpp:37-53 of the reference up to its use of v_rcp_f32 for inv.
struct ReinQ8Lane { int w0, w1; float d, sum; };   // what lane l of a row holds of the finished block

__device__ __forceinline__ ReinQ8Lane rein_q8_quantize_sub(float lo, float hi)
{
#pragma clang fp contract(off)
    const float amax = rein_row_max(fabsf(lo), fabsf(hi));
    const float sum  = rein_row_sum(lo, hi);
    const float d   = amax > 0.0f ? amax / 127.0f : 1.0f;
    const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
    const int q0 = max(-127, min(127, (int)rintf(lo * inv))) & 0xFF;
    const int q1 = max(-127, min(127, (int)rintf(hi * inv))) & 0xFF;
    // bytes of a lane quad -> one dword per 16-element half: pairs, then pairs of pairs
    int p = q0 | (q1 << 16);                                                          // [q0, -, q1, -]
    p = p | (__builtin_amdgcn_update_dpp(0, p, 0xB1, 0xF, 0xF, false) << 8);          // even lanes: + lane^1
    ReinQ8Lane r;
    r.w0 = (p & 0xFFFF) | (__builtin_amdgcn_update_dpp(0, p, 0x4E, 0xF, 0xF, false) << 16);
    r.w1 = ((unsigned)p >> 16) | (__builtin_amdgcn_update_dpp(0, p, 0x4E, 0xF, 0xF, false) & 0xFFFF0000);
    r.d = d;
    r.sum = sum;
    return r;
}

__device__ __forceinline__ void rein_q8_store_lane(BlockQ8* __restrict__ o, unsigned l, const ReinQ8Lane& r)
{
    if ((l & 3u) == 0u) { o->qs[l >> 2] = r.w0; o->qs[4 + (l >> 2)] = r.w1; }
    if (l == 0u) { o->d = r.d; o->xsum = r.sum; }
}

__device__ __forceinline__ void rein_q8_store_sub(BlockQ8* __restrict__ o, unsigned l, float lo, float hi)
{
    rein_q8_store_lane(o, l, rein_q8_quantize_sub(lo, hi));
}

// exp(x), |relative error| < 3e-7 on [-87, 88]; outside, x is clamped (the result
// saturates at exp(-87) ~ 1.6e-38 resp. exp(88) ~ 1.7e38 instead of 0 / inf).
// n = rint(x*log2(e)); r = x - n*ln2 in two fma steps (ln2 split hi + lo);
// degree-6 Horner polynomial in fma; result scaled by 2^n through the exponent
// field.
__device__ __forceinline__ float rein_exp_det(float x)
{
#pragma clang fp contract(off)
    x = fminf(fmaxf(x, -87.0f), 88.0f);
    const float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693145751953125f, x);           // ln2 hi: 0x3F317200
    r = fmaf(n, -1.42860682030941723e-6f, r);            // ln2 lo
    float p = 1.0f / 720.0f;
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    // 2^n with n in [-126, 127]: n = -126 needs two steps to stay normal
    const int ni = (int)n;
    const int n1 = ni / 2, n2 = ni - n1;
    const float s1 = __builtin_bit_cast(float, (unsigned)(n1 + 127) << 23);
    const float s2 = __builtin_bit_cast(float, (unsigned)(n2 + 127) << 23);
    return p * s1 * s2;
}

// x / (1 + exp(-x))   (src/cpu/ops.rs:14-16 of the reference)
__device__ __forceinline__ float rein_silu_det(float x)
{
#pragma clang fp contract(off)
    return x / (1.0f + rein_exp_det(-x));
}

// 1 / (1 + exp(-x))   (src/cpu/ops.rs:20-22)
__device__ __forceinline__ float rein_sigmoid_det(float x)
{
#pragma clang fp contract(off)
    return 1.0f / (1.0f + rein_exp_det(-x));
}

// GELU, tanh form: 0.5 x (1 + tanh(z)), z = sqrt(2/pi) (x + 0.044715 x^3)
// (src/cpu/ops.rs:33-36; kernels/moe_geglu_q8.cpp:25-29), evaluated as the identical
// x / (1 + exp(-2z)): one exp, one division, and no cancellation in the negative tail
// (where 1 + tanh(z) loses every digit in fp32).
__device__ __forceinline__ float rein_gelu_det(float x)
{
#pragma clang fp contract(off)
    const float c = x + 0.044715f * x * x * x;
    return x / (1.0f + rein_exp_det(-2.0f * (0.7978845608028654f * c)));
}

// Sum of squares of a vector whose 32-value sub-blocks are spread over the 16-lane
// rows of a workgroup, in an order that does not depend on the launch geometry:
//   part[sb] = butterfly 16, 8, 4, 2, 1 over the 32 squares of sub-block sb
//              (rein_row_sum of the two squares a lane holds)
//   lane l of wavefront 0 adds part[l], part[l+64], part[l+128], ... in that order
//   the 64 lane sums reduce with the butterfly 32, 16, 8, 4, 2, 1
// `part` is LDS with room for n_sub floats; the caller has stored part[sb] (from
// lane 0 of the row that owns sb).  Returns the total to every thread.
// Needs blockDim.x >= 64.
__device__ __forceinline__ float rein_sumsq_finish(float* part, unsigned n_sub, float* bcast)
{
#pragma clang fp contract(off)
    __syncthreads();
    if (threadIdx.x < 64u) {
        float t = 0.0f;
        for (unsigned i = threadIdx.x; i < n_sub; i += 64u) t = t + part[i];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) t = t + __shfl_xor(t, off);
        if (threadIdx.x == 0u) *bcast = t;
    }
    __syncthreads();
    return *bcast;
}
