// Repacked-v2 weight formats as the kernels see them.
//
// A repacked slab is a concatenation of planes, each row-major with row stride
// nsp (padded sub-blocks per row); layouts are fixed by the reference's
// repack_for_matvec functions:
//   Q4_K   nib 16 | (sc,m) 2          per sub-block, (f16 d, f16 dmin) per superblock   src/quant/q4_k.rs:126-176
//   Q5_K   nib 16 | qh 4 | (sc,m) 2   per sub-block, (f16 d, f16 dmin) per superblock   src/quant/q5_k.rs:97-151
//   Q6_K   nib 16 | hi2 8 | (i8,i8) 2 per sub-block, f16 d per superblock               src/quant/q6_k.rs:86-148
//   Q8_0   lo 16 | hi 16 | f16 d 2    per sub-block                                     src/quant/q8_0.rs:93-119
//   Q4_0   nib 16 | f16 d 2           per sub-block                                     src/quant/q4_0.rs:86-104
//   IQ4_XS nib 16 | f16 dl 2          per sub-block                                     src/quant/iq4_xs.rs:106-136
//
// Every format exposes the same three steps:
//   load(row, sb)     raw words of one 32-weight sub-block, straight from HBM
//   unpack(raw, W)    eight int8x4 words in dot order (word j pairs with
//                     activation word j: words 0-3 = weights 0-15, 4-7 = 16-31)
//                     plus the fp32 scales
//   term(...)         the sub-block's fp32 contribution from the integer dots
#pragma once

#include "rein_common.h"

enum ReinFmt : int {
    REIN_Q4_0   = 2,
    REIN_Q8_0   = 8,
    REIN_Q4_K   = 12,
    REIN_Q5_K   = 13,
    REIN_Q6_K   = 14,
    REIN_IQ4_XS = 23,
    // relabelled formats: another format's planes and kernels with one decode step swapped
    REIN_Q5_1   = 7,    // Q5_K's nibble and qh planes, raw fp16 (d, m) per sub-block (src/quant/q5_1.rs:12-20)
    REIN_IQ3_S  = 21,   // IQ4_XS's planes, codebook value 2n - 15 (src/quant/iq3_s.rs:13-19)
};

// Unpacked sub-block.
struct SubW {
    int   w[8];     // int8x4, dot order
    float s0;       // K-quants: d*sc (Q6_K: d*sc_lo); others: d
    float s1;       // Q4_K/Q5_K: dmin*m; Q6_K: d*sc_hi
};

// Integer sums of an activation block's quants (needed by Q6_K and Q4_0 only).
struct XSums { int lo, hi; };

__device__ __forceinline__ XSums rein_xsums(const int x[8])
{
    XSums s;
    s.lo = 0; s.hi = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        s.lo = rein_dot4(x[j], 0x01010101, s.lo);
        s.hi = rein_dot4(x[j + 4], 0x01010101, s.hi);
    }
    return s;
}

// bits 0..3 of h -> bit 0 of bytes 0..3 (one 24-bit multiply: bit i lands on 8i)
__device__ __forceinline__ uint32_t rein_spread4(uint32_t h)
{
    return __umul24(h & 0xFu, 0x204081u) & 0x01010101u;
}

// The four 2-bit fields of the byte at bit `shift` of word hw -> bits 4,5 of bytes 0..3.
// Two 24-bit multiplies place fields (0, 2) and (1, 3) -- the masks go on before the
// multiply (so the copies cannot run into each other) and after it (to drop the copies
// that landed elsewhere); no field is ever shifted into place on its own.
__device__ __forceinline__ uint32_t rein_spread2(uint32_t hw, unsigned shift)
{
    const uint32_t h = hw >> shift;
    const uint32_t even = __umul24(h & 0x33u, 0x10010u) & 0x00300030u;          // field 0 -> bit 4, field 2 -> bit 20
    const uint32_t odd  = __umul24(h & 0xCCu, 0x400400u);                        // field 1 -> bit 12, field 3 -> bit 28
    return (odd & 0x30003000u) | even;
}

// IQ4_NL / IQ4_XS codebook (src/quant/iq4_xs.rs:28-31), four entries per word.
#define REIN_KV_0_3   0xbfad9881u
#define REIN_KV_4_7   0xf6eaddcfu
#define REIN_KV_8_11  0x26190d01u
#define REIN_KV_12_15 0x71594535u

// (x - c) per byte for bytes x in [0,127], c < 128: no borrow crosses a byte
__device__ __forceinline__ int rein_sub_bytes(uint32_t x, uint32_t c4)
{
    return (int)(((x | 0x80808080u) - c4) ^ 0x80808080u);
}

// The four int8 weight values of a codebook format from the nibbles at bit `shift` (0 or 4)
// of the four bytes of w.
//   IQ4_XS: two byte permutes look the low three index bits up in either half of the
//   codebook, a third picks per byte between the halves (selector byte i = i or 4 + i by
//   index bit 3); no nibble is ever isolated.
//   IQ3_S:  KVALUES_IQ3S[n] = 2n - 15 (src/quant/iq3_s.rs:161-162), computed per byte.
template <int FMT> __device__ __forceinline__ int rein_codebook4(uint32_t w, unsigned shift)
{
    const uint32_t v = w >> shift;
    if constexpr (FMT == REIN_IQ3_S) {
        return rein_sub_bytes((v << 1) & 0x1E1E1E1Eu, 0x0F0F0F0Fu);
    } else {
        const uint32_t sel  = v & 0x07070707u;
        const uint32_t lo   = __builtin_amdgcn_perm(REIN_KV_4_7, REIN_KV_0_3, sel);
        const uint32_t hi   = __builtin_amdgcn_perm(REIN_KV_12_15, REIN_KV_8_11, sel);
        const uint32_t pick = ((v >> 1) & 0x04040404u) | 0x03020100u;
        return (int)__builtin_amdgcn_perm(hi, lo, pick);
    }
}

// Streaming (nontemporal) loads for the matvec weight planes: every weight byte is
// read exactly once per launch, so it should not displace the activations in L2.
typedef uint32_t rein_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t rein_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 rein_ldw(const uint4* p)
{
    const rein_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const rein_u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 rein_ldw(const uint2* p)
{
    const rein_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const rein_u32x2*>(p));
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t rein_ldw(const uint32_t* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ uint16_t rein_ldw(const uint16_t* p) { return __builtin_nontemporal_load(p); }

template <int FMT> struct Fmt;

// ------------------------------------------------------------------ Q4_K
template <> struct Fmt<REIN_Q4_K> {
    static constexpr bool kNeedsXSums = false;
    struct Raw { uint4 q; uint16_t sm; uint32_t dd; };
    const uint4*    nib;
    const uint16_t* smp;
    const uint32_t* ddp;
    unsigned nsp, n_super;
    __device__ Fmt(const uint8_t* w, unsigned n_sub, unsigned out_dim)
    {
        nsp = rein_nsp(n_sub);
        n_super = n_sub >> 3;
        const size_t n = (size_t)out_dim * nsp;
        nib = reinterpret_cast<const uint4*>(w);
        smp = reinterpret_cast<const uint16_t*>(w + n * 16);
        ddp = reinterpret_cast<const uint32_t*>(w + n * 18);
    }
    __device__ __forceinline__ Raw load(unsigned row, unsigned sb) const
    {
        const size_t i = (size_t)row * nsp + sb;
        Raw r;
        r.q  = rein_ldw(&nib[i]);
        r.sm = rein_ldw(&smp[i]);
        r.dd = rein_ldw(&ddp[(size_t)row * n_super + (sb >> 3)]);
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, SubW& s)
    {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            s.w[j]     = (int)(q[j] & 0x0F0F0F0Fu);
            s.w[j + 4] = (int)((q[j] >> 4) & 0x0F0F0F0Fu);
        }
        s.s0 = rein_h2f((uint16_t)(r.dd & 0xFFFFu)) * (float)(r.sm & 0xFFu);
        s.s1 = rein_h2f((uint16_t)(r.dd >> 16)) * (float)(r.sm >> 8);
    }
    // dsc*dx*idot - deff*xsum   (kernels/matvec_q4k_repacked.cpp:106-121)
    static __device__ __forceinline__ float term(const SubW& s, int i0, int i1, float dx, float xsum, XSums)
    {
        return s.s0 * dx * (float)(i0 + i1) - s.s1 * xsum;
    }
    static constexpr int kDotParts = 1;
    static __device__ __forceinline__ void parts(int i0, int i1, XSums, int out[2]) { out[0] = i0 + i1; out[1] = 0; }
};

// ------------------------------------------------------------------ Q5_K
template <> struct Fmt<REIN_Q5_K> {
    static constexpr bool kNeedsXSums = false;
    struct Raw { uint4 q; uint32_t qh; uint16_t sm; uint32_t dd; };
    const uint4*    nib;
    const uint32_t* qhp;
    const uint16_t* smp;
    const uint32_t* ddp;
    unsigned nsp, n_super;
    __device__ Fmt(const uint8_t* w, unsigned n_sub, unsigned out_dim)
    {
        nsp = rein_nsp(n_sub);
        n_super = n_sub >> 3;
        const size_t n = (size_t)out_dim * nsp;
        nib = reinterpret_cast<const uint4*>(w);
        qhp = reinterpret_cast<const uint32_t*>(w + n * 16);
        smp = reinterpret_cast<const uint16_t*>(w + n * 20);
        ddp = reinterpret_cast<const uint32_t*>(w + n * 22);
    }
    __device__ __forceinline__ Raw load(unsigned row, unsigned sb) const
    {
        const size_t i = (size_t)row * nsp + sb;
        Raw r;
        r.q  = rein_ldw(&nib[i]);
        r.qh = rein_ldw(&qhp[i]);
        r.sm = rein_ldw(&smp[i]);
        r.dd = rein_ldw(&ddp[(size_t)row * n_super + (sb >> 3)]);
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, SubW& s)
    {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // bit 4g+b of qh is the 5th bit of weight b of dot group g; the low
            // nibbles of word j are group 2j, the high nibbles group 2j+1
            // (kernels/matvec_q5k_repacked.cpp:90-91)
            s.w[j]     = (int)((q[j] & 0x0F0F0F0Fu) | (rein_spread4(r.qh >> (8 * j)) << 4));
            s.w[j + 4] = (int)(((q[j] >> 4) & 0x0F0F0F0Fu) | (rein_spread4(r.qh >> (8 * j + 4)) << 4));
        }
        s.s0 = rein_h2f((uint16_t)(r.dd & 0xFFFFu)) * (float)(r.sm & 0xFFu);
        s.s1 = rein_h2f((uint16_t)(r.dd >> 16)) * (float)(r.sm >> 8);
    }
    static __device__ __forceinline__ float term(const SubW& s, int i0, int i1, float dx, float xsum, XSums)
    {
        return s.s0 * dx * (float)(i0 + i1) - s.s1 * xsum;
    }
    static constexpr int kDotParts = 1;
    static __device__ __forceinline__ void parts(int i0, int i1, XSums, int out[2]) { out[0] = i0 + i1; out[1] = 0; }
};

// ------------------------------------------------------------------ Q6_K
template <> struct Fmt<REIN_Q6_K> {
    static constexpr bool kNeedsXSums = true;
    struct Raw { uint4 q; uint2 h2; uint16_t sm; uint16_t d; };
    const uint4*    nib;
    const uint2*    h2p;
    const uint16_t* smp;
    const uint16_t* dp;
    unsigned nsp, n_super;
    __device__ Fmt(const uint8_t* w, unsigned n_sub, unsigned out_dim)
    {
        nsp = rein_nsp(n_sub);
        n_super = n_sub >> 3;
        const size_t n = (size_t)out_dim * nsp;
        nib = reinterpret_cast<const uint4*>(w);
        h2p = reinterpret_cast<const uint2*>(w + n * 16);
        smp = reinterpret_cast<const uint16_t*>(w + n * 24);
        dp  = reinterpret_cast<const uint16_t*>(w + n * 26);
    }
    __device__ __forceinline__ Raw load(unsigned row, unsigned sb) const
    {
        const size_t i = (size_t)row * nsp + sb;
        Raw r;
        r.q  = rein_ldw(&nib[i]);
        r.h2 = rein_ldw(&h2p[i]);
        r.sm = rein_ldw(&smp[i]);
        r.d  = rein_ldw(&dp[(size_t)row * n_super + (sb >> 3)]);
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, SubW& s)
    {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // byte g of the hi2 plane holds dot group g's four 2-bit fields;
            // group 2j -> low nibbles of word j, group 2j+1 -> high nibbles
            // (kernels/matvec_q6k_repacked.cpp:97-103)
            const uint32_t hw = j < 2 ? r.h2.x : r.h2.y;
            s.w[j]     = (int)((q[j] & 0x0F0F0F0Fu) | rein_spread2(hw, 16 * (j & 1)));
            s.w[j + 4] = (int)(((q[j] >> 4) & 0x0F0F0F0Fu) | rein_spread2(hw, 16 * (j & 1) + 8));
        }
        const float d = rein_h2f(r.d);
        s.s0 = d * (float)(int)(int8_t)(r.sm & 0xFFu);
        s.s1 = d * (float)(int)(int8_t)(r.sm >> 8);
    }
    // dsc_lo*dx*(idot0-32*xis0) + dsc_hi*dx*(idot1-32*xis1)  (kernels/matvec_q6k_repacked.cpp:91-108)
    static __device__ __forceinline__ float term(const SubW& s, int i0, int i1, float dx, float, XSums xs)
    {
        return s.s0 * dx * (float)(i0 - 32 * xs.lo) + s.s1 * dx * (float)(i1 - 32 * xs.hi);
    }
    static constexpr int kDotParts = 2;
    static __device__ __forceinline__ void parts(int i0, int i1, XSums xs, int out[2])
    {
        out[0] = i0 - 32 * xs.lo;
        out[1] = i1 - 32 * xs.hi;
    }
};

// ------------------------------------------------------------------ Q8_0
template <> struct Fmt<REIN_Q8_0> {
    static constexpr bool kNeedsXSums = false;
    struct Raw { uint4 lo, hi; uint16_t d; };
    const uint4*    lop;
    const uint4*    hip_;
    const uint16_t* dp;
    unsigned nsp;
    __device__ Fmt(const uint8_t* w, unsigned n_sub, unsigned out_dim)
    {
        nsp = rein_nsp(n_sub);
        const size_t n = (size_t)out_dim * nsp;
        lop  = reinterpret_cast<const uint4*>(w);
        hip_ = reinterpret_cast<const uint4*>(w + n * 16);
        dp   = reinterpret_cast<const uint16_t*>(w + n * 32);
    }
    __device__ __forceinline__ Raw load(unsigned row, unsigned sb) const
    {
        const size_t i = (size_t)row * nsp + sb;
        Raw r;
        r.lo = rein_ldw(&lop[i]);
        r.hi = rein_ldw(&hip_[i]);
        r.d  = rein_ldw(&dp[i]);
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, SubW& s)
    {
        s.w[0] = (int)r.lo.x; s.w[1] = (int)r.lo.y; s.w[2] = (int)r.lo.z; s.w[3] = (int)r.lo.w;
        s.w[4] = (int)r.hi.x; s.w[5] = (int)r.hi.y; s.w[6] = (int)r.hi.z; s.w[7] = (int)r.hi.w;
        s.s0 = rein_h2f(r.d);
        s.s1 = 0.0f;
    }
    // dw*dx*idot   (kernels/matvec_q8_0_repacked.cpp:78-85)
    static __device__ __forceinline__ float term(const SubW& s, int i0, int i1, float dx, float, XSums)
    {
        return s.s0 * dx * (float)(i0 + i1);
    }
    static constexpr int kDotParts = 1;
    static __device__ __forceinline__ void parts(int i0, int i1, XSums, int out[2]) { out[0] = i0 + i1; out[1] = 0; }
};

// ------------------------------------------------------------------ Q4_0
template <> struct Fmt<REIN_Q4_0> {
    static constexpr bool kNeedsXSums = true;
    struct Raw { uint4 q; uint16_t d; };
    const uint4*    nib;
    const uint16_t* dp;
    unsigned nsp;
    __device__ Fmt(const uint8_t* w, unsigned n_sub, unsigned out_dim)
    {
        nsp = rein_nsp(n_sub);
        const size_t n = (size_t)out_dim * nsp;
        nib = reinterpret_cast<const uint4*>(w);
        dp  = reinterpret_cast<const uint16_t*>(w + n * 16);
    }
    __device__ __forceinline__ Raw load(unsigned row, unsigned sb) const
    {
        const size_t i = (size_t)row * nsp + sb;
        Raw r;
        r.q = rein_ldw(&nib[i]);
        r.d = rein_ldw(&dp[i]);
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, SubW& s)
    {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            s.w[j]     = (int)(q[j] & 0x0F0F0F0Fu);
            s.w[j + 4] = (int)((q[j] >> 4) & 0x0F0F0F0Fu);
        }
        s.s0 = rein_h2f(r.d);
        s.s1 = 0.0f;
    }
    // dw*dx*(idot - 8*xqsum), the offset against the *quantized* activation sum
    // (kernels/matvec_q4_0_repacked.cpp:13-23,99-110)
    static __device__ __forceinline__ float term(const SubW& s, int i0, int i1, float dx, float, XSums xs)
    {
        return s.s0 * dx * (float)(i0 + i1 - 8 * (xs.lo + xs.hi));
    }
    static constexpr int kDotParts = 1;
    static __device__ __forceinline__ void parts(int i0, int i1, XSums xs, int out[2])
    {
        out[0] = i0 + i1 - 8 * (xs.lo + xs.hi);
        out[1] = 0;
    }
};

// ---------------------------------------------------------------- IQ4_XS
// IQ4_XS and IQ3_S share planes and arithmetic; FMT selects the codebook.
template <int FMT> struct FmtCodebook16 {
    static constexpr bool kNeedsXSums = false;
    struct Raw { uint4 q; uint16_t d; };
    const uint4*    nib;
    const uint16_t* dp;
    unsigned nsp;
    __device__ FmtCodebook16(const uint8_t* w, unsigned n_sub, unsigned out_dim)
    {
        nsp = rein_nsp(n_sub);
        const size_t n = (size_t)out_dim * nsp;
        nib = reinterpret_cast<const uint4*>(w);
        dp  = reinterpret_cast<const uint16_t*>(w + n * 16);
    }
    __device__ __forceinline__ Raw load(unsigned row, unsigned sb) const
    {
        const size_t i = (size_t)row * nsp + sb;
        Raw r;
        r.q = rein_ldw(&nib[i]);
        r.d = rein_ldw(&dp[i]);
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, SubW& s)
    {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            s.w[j]     = rein_codebook4<FMT>(q[j], 0);
            s.w[j + 4] = rein_codebook4<FMT>(q[j], 4);
        }
        s.s0 = rein_h2f(r.d);
        s.s1 = 0.0f;
    }
    // dl*dx*idot   (kernels/matvec_iq4xs_repacked.cpp:105-115)
    static __device__ __forceinline__ float term(const SubW& s, int i0, int i1, float dx, float, XSums)
    {
        return s.s0 * dx * (float)(i0 + i1);
    }
    static constexpr int kDotParts = 1;
    static __device__ __forceinline__ void parts(int i0, int i1, XSums, int out[2]) { out[0] = i0 + i1; out[1] = 0; }
};
template <> struct Fmt<REIN_IQ4_XS> : FmtCodebook16<REIN_IQ4_XS> { using FmtCodebook16<REIN_IQ4_XS>::FmtCodebook16; };
template <> struct Fmt<REIN_IQ3_S> : FmtCodebook16<REIN_IQ3_S> { using FmtCodebook16<REIN_IQ3_S>::FmtCodebook16; };

// ------------------------------------------------------------------ Q5_1
// The Q5_K unpack with the scale decode of the reference's Q5_1_SCALES build
// (kernels/moe_matvec_q5k_repacked.cpp:57-60,86-91): dsc = d, deff = -m, both raw fp16
// per sub-block.  in_dim is a multiple of 32 only.
template <> struct Fmt<REIN_Q5_1> {
    static constexpr bool kNeedsXSums = false;
    struct Raw { uint4 q; uint32_t qh; uint32_t dm; };
    const uint4*    nib;
    const uint32_t* qhp;
    const uint32_t* dmp;
    unsigned nsp;
    __device__ Fmt(const uint8_t* w, unsigned n_sub, unsigned out_dim)
    {
        nsp = rein_nsp(n_sub);
        const size_t n = (size_t)out_dim * nsp;
        nib = reinterpret_cast<const uint4*>(w);
        qhp = reinterpret_cast<const uint32_t*>(w + n * 16);
        dmp = reinterpret_cast<const uint32_t*>(w + n * 20);
    }
    __device__ __forceinline__ Raw load(unsigned row, unsigned sb) const
    {
        const size_t i = (size_t)row * nsp + sb;
        Raw r;
        r.q  = rein_ldw(&nib[i]);
        r.qh = rein_ldw(&qhp[i]);
        r.dm = rein_ldw(&dmp[i]);
        return r;
    }
    static __device__ __forceinline__ void unpack(const Raw& r, SubW& s)
    {
        const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            s.w[j]     = (int)((q[j] & 0x0F0F0F0Fu) | (rein_spread4(r.qh >> (8 * j)) << 4));
            s.w[j + 4] = (int)(((q[j] >> 4) & 0x0F0F0F0Fu) | (rein_spread4(r.qh >> (8 * j + 4)) << 4));
        }
        s.s0 = rein_h2f((uint16_t)(r.dm & 0xFFFFu));
        s.s1 = -rein_h2f((uint16_t)(r.dm >> 16));
    }
    static __device__ __forceinline__ float term(const SubW& s, int i0, int i1, float dx, float xsum, XSums)
    {
        return s.s0 * dx * (float)(i0 + i1) - s.s1 * xsum;
    }
    static constexpr int kDotParts = 1;
    static __device__ __forceinline__ void parts(int i0, int i1, XSums, int out[2]) { out[0] = i0 + i1; out[1] = 0; }
};
