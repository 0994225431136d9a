// Skinny MMQ: Y[P][N] for a handful of activation rows (P <= 8 or <= 16), the
// batched-decode shapes, on the int8 matrix cores but built like a matvec:
// HBM-bound, every wavefront an independent weight stream, no workgroup barrier in
// the main loop.
//
//   * A workgroup is KS wavefronts (blockDim.x / 64, chosen by the host) that all own
//     the same 32 weight rows and split the contraction: wavefront k walks superblock
//     chunks [k*C/KS, (k+1)*C/KS).
//     The KS partial tiles are summed through LDS at the end in wavefront order, so
//     the result does not depend on timing.  grid.x = ceil(N/32) row tiles,
//     grid.y = token groups of TOK rows.
//   * Everything a wavefront consumes travels HBM/L2 -> LDS by asynchronous transfer
//     (global_load_lds): the 16-byte weight plane through the same two-slot ring as
//     the tuned MMQ (a slot is refilled as soon as it is read), the small weight
//     words and the TOK x 8 activation blocks of a chunk one chunk ahead into
//     double-buffered images.  No register loads in the loop: the waits are placed by
//     hand and count transfers.
//   * Per sub-block one v_mfma_i32_32x32x32_i8 with the tokens as tile rows: tile row
//     m = 8*(v/4) + 4*(lane/32) + v%4, so tokens 0..7 are registers 0..3 of every lane
//     (0..7 for 16 tokens) and only those NV registers are converted and scaled; the
//     padding rows of the tile repeat the real tokens and are never read.  With
//     NV = 4 the fp32 work per sub-block is a dozen instructions, which is what makes
//     this faster than eight dot4 chains per row.
//   * Scales on the VALU: the lane's row scale times the four dx values of its
//     tokens (one ds_read_b128); Q4_K/Q5_K subtract dmin*m*xsum the same way.
//
// Same sub-block formulas as the matvec (src: kernels/matvec_*_repacked.cpp of the
// reference); the integer dots are the MMQ's.  No counterpart in the reference,
// which runs these batches on dot4 kernels (kernels/matvec_*_repacked_batched.cpp).
#pragma once

#include "mmq_gemm.h"

// 4-byte-per-lane HBM -> LDS transfer, lane l's dword lands at lds_base + 4 l.
__device__ __forceinline__ void rein_lds_dma4(const void* gptr, unsigned lds_base)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
                 :
                 : "v"(gptr), "s"(lds_base)
                 : "memory", "m0");
}

__device__ __forceinline__ unsigned rein_lds_addr(const void* p)
{
    typedef const __attribute__((address_space(3))) void* lptr_t;
    return __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)p);
}

// Per-format small words of one chunk (aux bits, scales, fp16 pair).  They travel
// HBM -> LDS like everything else in this kernel (lanes 0..31 request their row's
// words, lane l reads entry l % 32 back), so that the main loop has no register
// loads for the compiler to wait on.  begin()/pair()/rotate() turn the words into
// the per-sub-block scales of the lane's row (both lane halves need every
// sub-block's scale here); operand() is MmqChunk's.
template <int FMT> struct SkinnyFmt;

template <int FMT> struct SkinnyKQuant {
    using C = MmqChunk<FMT>;
    using Small = typename C::Small;
    static constexpr bool kHasMin = C::kHasMin, kTwoScales = C::kTwoScales;
    static __device__ __forceinline__ rein_v4i operand(const uint4& q, const Small& r, int s, unsigned h)
    {
        return C::operand(q, r, s, h);
    }
};

template <> struct SkinnyFmt<REIN_Q4_K> : SkinnyKQuant<REIN_Q4_K> {
    struct Lds { uint4 sm[32]; uint32_t dd[32]; };
    static constexpr int kDma = 2;
    static __device__ __forceinline__ void request(Lds& l, const Fmt<REIN_Q4_K>& f, unsigned row, unsigned sb0, unsigned)
    {
        rein_lds_dma16(f.smp + (size_t)row * f.nsp + sb0, rein_lds_addr(l.sm));
        rein_lds_dma4(f.ddp + (size_t)row * f.n_super + (sb0 >> 3), rein_lds_addr(l.dd));
    }
    static __device__ __forceinline__ Small read(const Lds& l, unsigned j, unsigned, unsigned)
    {
        Small r;
        r.sm = __builtin_bit_cast(ReinU16x8, l.sm[j]);
        r.dd = l.dd[j];
        return r;
    }
    float d, dmin;
    __device__ __forceinline__ void begin(const Small& r, unsigned, unsigned)
    {
        d = rein_h2f((uint16_t)(r.dd & 0xFFFFu));
        dmin = rein_h2f((uint16_t)(r.dd >> 16));
    }
    // scales of sub-blocks 0 and 1 of the (rotated) chunk words
    __device__ __forceinline__ void pair(const Small& r, float sc[2], float sc_hi[2], float mn[2])
    {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            sc[s] = d * (float)(r.sm.v[s] & 0xFFu);
            mn[s] = dmin * (float)(r.sm.v[s] >> 8);
            sc_hi[s] = 0.0f;
        }
    }
    static __device__ __forceinline__ void rotate(Small& r)
    {
#pragma unroll
        for (int i = 0; i < 6; i++) r.sm.v[i] = r.sm.v[i + 2];
    }
};

template <> struct SkinnyFmt<REIN_Q5_K> : SkinnyKQuant<REIN_Q5_K> {
    struct Lds { uint4 sm[32]; uint4 qh[2][32]; uint32_t dd[32]; };
    static constexpr int kDma = 4;
    static __device__ __forceinline__ void request(Lds& l, const Fmt<REIN_Q5_K>& f, unsigned row, unsigned sb0, unsigned)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
        rein_lds_dma16(f.smp + i, rein_lds_addr(l.sm));
        rein_lds_dma16(f.qhp + i, rein_lds_addr(l.qh[0]));
        rein_lds_dma16(f.qhp + i + 4, rein_lds_addr(l.qh[1]));
        rein_lds_dma4(f.ddp + (size_t)row * f.n_super + (sb0 >> 3), rein_lds_addr(l.dd));
    }
    static __device__ __forceinline__ Small read(const Lds& l, unsigned j, unsigned, unsigned)
    {
        Small r;
        r.sm = __builtin_bit_cast(ReinU16x8, l.sm[j]);
        const uint4 a = l.qh[0][j], b = l.qh[1][j];
        r.qh.v[0] = a.x; r.qh.v[1] = a.y; r.qh.v[2] = a.z; r.qh.v[3] = a.w;
        r.qh.v[4] = b.x; r.qh.v[5] = b.y; r.qh.v[6] = b.z; r.qh.v[7] = b.w;
        r.dd = l.dd[j];
        return r;
    }
    float d, dmin;
    __device__ __forceinline__ void begin(const Small& r, unsigned, unsigned)
    {
        d = rein_h2f((uint16_t)(r.dd & 0xFFFFu));
        dmin = rein_h2f((uint16_t)(r.dd >> 16));
    }
    __device__ __forceinline__ void pair(const Small& r, float sc[2], float sc_hi[2], float mn[2])
    {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            sc[s] = d * (float)(r.sm.v[s] & 0xFFu);
            mn[s] = dmin * (float)(r.sm.v[s] >> 8);
            sc_hi[s] = 0.0f;
        }
    }
    static __device__ __forceinline__ void rotate(Small& r)
    {
#pragma unroll
        for (int i = 0; i < 6; i++) { r.sm.v[i] = r.sm.v[i + 2]; r.qh.v[i] = r.qh.v[i + 2]; }
    }
};

template <> struct SkinnyFmt<REIN_Q6_K> : SkinnyKQuant<REIN_Q6_K> {
    struct Lds { uint4 sm[32]; uint4 h2[4][32]; uint32_t d[32]; };
    static constexpr int kDma = 6;
    static __device__ __forceinline__ void request(Lds& l, const Fmt<REIN_Q6_K>& f, unsigned row, unsigned sb0, unsigned)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
        rein_lds_dma16(f.smp + i, rein_lds_addr(l.sm));
#pragma unroll
        for (int k = 0; k < 4; k++) rein_lds_dma16(f.h2p + i + 2 * k, rein_lds_addr(l.h2[k]));
        // the fp16 d sits at a 2-byte address: fetch the aligned dword that holds it
        const uint16_t* dp = f.dp + (size_t)row * f.n_super + (sb0 >> 3);
        rein_lds_dma4(reinterpret_cast<const void*>(reinterpret_cast<size_t>(dp) & ~(size_t)3), rein_lds_addr(l.d));
    }
    static __device__ __forceinline__ Small read(const Lds& l, unsigned j, unsigned d_odd, unsigned)
    {
        Small r;
        r.sm = __builtin_bit_cast(ReinU16x8, l.sm[j]);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint4 a = l.h2[k][j];
            r.h2.v[2 * k] = make_uint2(a.x, a.y);
            r.h2.v[2 * k + 1] = make_uint2(a.z, a.w);
        }
        r.d = (uint16_t)(l.d[j] >> (16u * d_odd));
        return r;
    }
    float d;
    __device__ __forceinline__ void begin(const Small& r, unsigned, unsigned) { d = rein_h2f(r.d); }
    __device__ __forceinline__ void pair(const Small& r, float sc[2], float sc_hi[2], float mn[2])
    {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            sc[s]    = d * (float)(int)(int8_t)(r.sm.v[s] & 0xFFu);
            sc_hi[s] = d * (float)(int)(int8_t)(r.sm.v[s] >> 8);
            mn[s] = 0.0f;
        }
    }
    static __device__ __forceinline__ void rotate(Small& r)
    {
#pragma unroll
        for (int i = 0; i < 6; i++) { r.sm.v[i] = r.sm.v[i + 2]; r.h2.v[i] = r.h2.v[i + 2]; }
    }
};

// Q8_0 / Q4_0 / IQ4_XS: eight fp16 scales.  A ragged last chunk (in_dim only a
// multiple of 32) requests the last eight scales of the row instead, so the 16
// bytes never run past the end of the scale plane, and read() rotates them into
// place; sub-blocks past the end are zero-scaled.  Needs n_sub >= 8.
template <int FMT> struct SkinnyD16 {
    using C = MmqChunk<FMT>;
    struct Small { uint16_t d[8]; };
    struct Lds { uint4 d[32]; };
    static constexpr int kDma = 1;
    static constexpr bool kHasMin = false, kTwoScales = false;
    unsigned left;                                   // valid sub-blocks from the front of the rotated words
    static __device__ __forceinline__ void request(Lds& l, const Fmt<FMT>& f, unsigned row, unsigned sb0, unsigned n_sub)
    {
        const unsigned first = sb0 + 8u <= n_sub ? sb0 : n_sub - 8u;
        rein_lds_dma16(f.dp + (size_t)row * f.nsp + first, rein_lds_addr(l.d));
    }
    static __device__ __forceinline__ Small read(const Lds& l, unsigned j, unsigned, unsigned shift)
    {
        Small r = __builtin_bit_cast(Small, l.d[j]);
        for (unsigned k = 0; k < shift; k++) {       // wave-uniform trip count
#pragma unroll
            for (int i = 0; i < 7; i++) r.d[i] = r.d[i + 1];
        }
        return r;
    }
    static __device__ __forceinline__ rein_v4i operand(const uint4& q, const Small&, int s, unsigned h)
    {
        return C::operand(q, typename C::Small{}, s, h);
    }
    __device__ __forceinline__ void begin(const Small&, unsigned sb0, unsigned n_sub) { left = n_sub - sb0; }
    __device__ __forceinline__ void pair(const Small& r, float sc[2], float sc_hi[2], float mn[2])
    {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            sc[s] = (unsigned)s < left ? rein_h2f(r.d[s]) : 0.0f;
            sc_hi[s] = 0.0f;
            mn[s] = 0.0f;
        }
        left = left > 2u ? left - 2u : 0u;
    }
    static __device__ __forceinline__ void rotate(Small& r)
    {
#pragma unroll
        for (int i = 0; i < 6; i++) r.d[i] = r.d[i + 2];
    }
};
template <> struct SkinnyFmt<REIN_Q8_0> : SkinnyD16<REIN_Q8_0> {};
template <> struct SkinnyFmt<REIN_Q4_0> : SkinnyD16<REIN_Q4_0> {};
template <> struct SkinnyFmt<REIN_IQ4_XS> : SkinnyD16<REIN_IQ4_XS> {};

// One wavefront's LDS image of one activation chunk: TOK rows x 8 sub-blocks, in
// the order the transfers deliver it (lane l of a transfer = sub-block l/8 ... of
// row l%TOK).
template <int TOK>
struct SkinnyAct {
    uint4 qs[2][8][TOK];                                 // [half][sub-block][row]
    float dx[8][TOK];
    float xs[8][TOK];
};

// HBM/L2 -> LDS: lane l of transfer k covers block e = 64k + l, sub-block e / TOK,
// row e % TOK (rows past tok_end and sub-blocks past n_sub repeat the last valid
// one: their results are never stored, resp. are zero-scaled on the weight side).
// 4 (3 without xsum) transfers per 64 blocks.
template <int TOK, bool XS>
__device__ __forceinline__ void rein_skinny_xrequest(SkinnyAct<TOK>& a, const BlockQ8* __restrict__ xq, unsigned n_sub,
                                                     unsigned tok_base, unsigned tok_end, unsigned sb0, unsigned lane)
{
#pragma unroll
    for (int k = 0; k < TOK * 8 / 64; k++) {
        const unsigned e = 64u * k + lane;
        const unsigned tok = min(tok_base + e % TOK, tok_end - 1u), sb = rein_clamp_sb(sb0 + e / TOK, n_sub);
        const uint8_t* blk = reinterpret_cast<const uint8_t*>(xq + (size_t)tok * n_sub + sb);
        rein_lds_dma16(blk + 8, rein_lds_addr(&a.qs[0][0][0] + 64 * k));
        rein_lds_dma16(blk + 24, rein_lds_addr(&a.qs[1][0][0] + 64 * k));
        rein_lds_dma4(blk, rein_lds_addr(&a.dx[0][0] + 64 * k));
        if (XS) rein_lds_dma4(blk + 4, rein_lds_addr(&a.xs[0][0] + 64 * k));
    }
}

// Per-wavefront LDS of the skinny kernel: the weight plane in a ring of two
// half-chunk slots, the activation blocks and small words of a chunk double-buffered.
// Kept small on purpose -- the kernel hides latency with resident wavefronts (four
// per SIMD), and LDS is what limits them.  The launch passes KS of these as dynamic
// shared memory.
template <int FMT, int TOK>
struct SkinnyWaveLds {
    MmqWLds<FMT> ring;
    SkinnyAct<TOK> act[2];
    typename SkinnyFmt<FMT>::Lds small[2];
};
static_assert(sizeof(SkinnyWaveLds<REIN_Q4_K, 8>) == 4096 + 2 * (320 * 8 + 640), "host launcher mirrors this");
static_assert(sizeof(SkinnyWaveLds<REIN_Q5_K, 8>) == 4096 + 2 * (320 * 8 + 1664), "host launcher mirrors this");
static_assert(sizeof(SkinnyWaveLds<REIN_Q6_K, 16>) == 4096 + 2 * (320 * 16 + 2688), "host launcher mirrors this");
static_assert(sizeof(SkinnyWaveLds<REIN_Q8_0, 8>) == 2 * 4096 + 2 * (320 * 8 + 512), "host launcher mirrors this");
static_assert(sizeof(SkinnyWaveLds<REIN_Q4_0, 16>) == 4096 + 2 * (320 * 16 + 512), "host launcher mirrors this");

template <int FMT, int NV>
__device__ __forceinline__ void rein_mmq_skinny(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                unsigned p_rows)
{
    using F = Fmt<FMT>;
    using SK = SkinnyFmt<FMT>;
    constexpr int TOK = 2 * NV;
    constexpr bool XS = SK::kHasMin;
    constexpr int kRing = 2 * MmqWLds<FMT>::kPlanes;                       // transfers per ring half
    constexpr int kStage = SK::kDma + (TOK * 8 / 64) * (XS ? 4 : 3);       // small words + activations of a chunk
    static_assert(kStage + kRing <= 63, "vmcnt is six bits");
    typedef SkinnyWaveLds<FMT, TOK> WaveLds;
    extern __shared__ uint4 rein_skinny_lds[];
    static_assert(sizeof(WaveLds) >= 32 * TOK * 4, "partial tiles are reduced through the per-wavefront LDS");
    const unsigned KS = blockDim.x >> 6;

    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned j = lane & 31u, h = lane >> 5;
    const unsigned n_sub = in_dim >> 5;
    const unsigned n_chunks = (n_sub + 7u) >> 3;
    const F fmt(w, n_sub, out_dim);
    const unsigned row_base = blockIdx.x * 32u;
    const unsigned row = row_base + j;
    const unsigned rowc = row < out_dim ? row : out_dim - 1;
    const unsigned tok_base = blockIdx.y * TOK;
    const unsigned tok_end = min(p_rows, tok_base + TOK);
    const unsigned wsel = FMT == REIN_Q8_0 ? h : 0u;
    const unsigned ja = j & (TOK - 1);                 // tile rows >= TOK repeat real tokens (never read back)
    WaveLds& my = reinterpret_cast<WaveLds*>(rein_skinny_lds)[wave];
    MmqWLds<FMT>& wl = my.ring;

    const unsigned c_begin = wave * n_chunks / KS, c_end = (wave + 1u) * n_chunks / KS;

    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) acc[v] = 0.0f;
    rein_v16i cinit;
#pragma unroll
    for (int v = 0; v < 16; v++) cinit[v] = REIN_MMQ_MAGIC_I;

    // Everything the loop consumes arrives by LDS transfer, so every wait below is
    // placed by hand and counts transfers only (they complete in order; vmcnt = those
    // in flight).  Per chunk c:
    //   top            stage(c+1): small words + activation blocks of c+1   [kStage]
    //   after pair 1   ring slot 0 <- c+1                                   [kRing]
    //   before pair 2  slot 1 of c must be in: younger are stage(c+1), slot 0 refill
    //   after pair 3   ring slot 1 <- c+1                                   [kRing]
    //   end            stage(c+1) and slot 0 of c+1 must be in: younger is the slot 1 refill
    if (c_begin < c_end) {
        const unsigned sb_first = c_begin * 8u;
        if (lane < 32u) SK::request(my.small[0], fmt, rowc, sb_first, n_sub);      // one request per row
        rein_skinny_xrequest<TOK, XS>(my.act[0], xq, n_sub, tok_base, tok_end, sb_first, lane);
        rein_mmq_wload<FMT>(wl, 0, fmt, row_base, out_dim, sb_first, n_sub, lane);
        rein_mmq_wload<FMT>(wl, 1, fmt, row_base, out_dim, sb_first + 4u, n_sub, lane);
        REIN_WAIT_VMCNT(kRing);                      // all but slot 1 of the first chunk has landed

        unsigned buf = 0;
        for (unsigned c = c_begin; c < c_end; c++, buf ^= 1u) {
            const unsigned sb0 = c * 8u;
            const bool more = c + 1u < c_end;
            // Q6_K's fp16 d may be the odd half of the dword that was fetched; a ragged
            // D16 chunk was requested from n_sub-8 and is shifted into place
            unsigned d_odd = 0;
            if constexpr (FMT == REIN_Q6_K)
                d_odd = (unsigned)(((reinterpret_cast<size_t>(fmt.dp) >> 1) + (size_t)rowc * fmt.n_super + (sb0 >> 3)) & 1u);
            const unsigned shift = sb0 + 8u <= n_sub ? 0u : sb0 + 8u - n_sub;
            typename SK::Small cur = SK::read(my.small[buf], j, d_odd, shift);
            SK sk;
            sk.begin(cur, sb0, n_sub);
            if (more) {
                if (lane < 32u) SK::request(my.small[buf ^ 1u], fmt, rowc, sb0 + 8u, n_sub);
                rein_skinny_xrequest<TOK, XS>(my.act[buf ^ 1u], xq, n_sub, tok_base, tok_end, sb0 + 8u, lane);
            }
            const SkinnyAct<TOK>& a = my.act[buf];
            const unsigned rot = j >> 1;

#pragma unroll 1
            for (unsigned p = 0; p < 4; p++) {
                if (p == 2) {
                    if (more) REIN_WAIT_VMCNT(kStage + kRing); else REIN_WAIT_VMCNT(0);
                }
                const uint4* slot = wl.q[wsel][p >> 1];
                const unsigned s4 = 2u * (p & 1u);
                rein_v4i b[2];
                b[0] = SK::operand(slot[4u * j + ((s4 + rot) & 3u)], cur, 0, h);
                b[1] = SK::operand(slot[4u * j + ((s4 + 1u + rot) & 3u)], cur, 1, h);
                if (more && (p & 1u)) {
                    __builtin_amdgcn_s_waitcnt(0xC07F);            // lgkmcnt(0): the slot has been read
                    rein_mmq_wload<FMT>(wl, p >> 1, fmt, row_base, out_dim, sb0 + 8u + 4u * (p >> 1), n_sub, lane);
                }
                float sc[2], sc_hi[2], mn[2];
                sk.pair(cur, sc, sc_hi, mn);
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    const unsigned sb = 2u * p + s;
                    const uint4 a4 = a.qs[h][sb][ja];
                    rein_v4i av;
                    av[0] = (int)a4.x; av[1] = (int)a4.y; av[2] = (int)a4.z; av[3] = (int)a4.w;
                    float dxv[NV], xsv[NV];
#pragma unroll
                    for (int q = 0; q < NV / 4; q++) {
                        const float4 d4 = *reinterpret_cast<const float4*>(&a.dx[sb][8 * q + 4 * h]);
                        dxv[4 * q] = d4.x; dxv[4 * q + 1] = d4.y; dxv[4 * q + 2] = d4.z; dxv[4 * q + 3] = d4.w;
                        if constexpr (XS) {
                            const float4 x4 = *reinterpret_cast<const float4*>(&a.xs[sb][8 * q + 4 * h]);
                            xsv[4 * q] = x4.x; xsv[4 * q + 1] = x4.y; xsv[4 * q + 2] = x4.z; xsv[4 * q + 3] = x4.w;
                        }
                    }
                    if constexpr (SK::kTwoScales) {
                        rein_v4i blo, bhi;
#pragma unroll
                        for (int k = 0; k < 4; k++) { blo[k] = h ? 0 : b[s][k]; bhi[k] = h ? b[s][k] : 0; }
                        const rein_v16f flo = rein_mmq_unbias(__builtin_amdgcn_mfma_i32_32x32x32_i8(av, blo, cinit, 0, 0, 0));
                        const rein_v16f fhi = rein_mmq_unbias(__builtin_amdgcn_mfma_i32_32x32x32_i8(av, bhi, cinit, 0, 0, 0));
#pragma unroll
                        for (int v = 0; v < NV; v++)
                            acc[v] = fmaf(fmaf(fhi[v], sc_hi[s], flo[v] * sc[s]), dxv[v], acc[v]);
                    } else {
                        const rein_v16f f = rein_mmq_unbias(__builtin_amdgcn_mfma_i32_32x32x32_i8(av, b[s], cinit, 0, 0, 0));
#pragma unroll
                        for (int v = 0; v < NV; v++) {
                            acc[v] = fmaf(f[v], sc[s] * dxv[v], acc[v]);
                            if constexpr (XS) acc[v] = fmaf(-mn[s], xsv[v], acc[v]);
                        }
                    }
                }
                SK::rotate(cur);
            }
            if (more) {
                REIN_WAIT_VMCNT(kRing);              // stage(c+1) and slot 0 of c+1 have landed
                __builtin_amdgcn_s_waitcnt(0xC07F);  // this chunk's LDS reads have returned before stage(c+2) overwrites
            }
        }
    }

    // sum the KS partial tiles in wavefront order
    __syncthreads();                                 // every wavefront is done with its LDS
    constexpr unsigned kStride = sizeof(WaveLds) / 4;                           // floats between wavefronts' partials
    float* red = reinterpret_cast<float*>(rein_skinny_lds);                     // wavefront k: [NV][64] at k*kStride
#pragma unroll
    for (int v = 0; v < NV; v++) red[wave * kStride + v * 64 + lane] = acc[v];
    __syncthreads();
    for (unsigned e = threadIdx.x; e < NV * 64u; e += blockDim.x) {
        float s = red[e];
#pragma unroll 1
        for (unsigned k = 1; k < KS; k++) s += red[k * kStride + e];
        const unsigned v = e >> 6, l = e & 63u;
        const unsigned tok = tok_base + 8u * (v >> 2) + 4u * (l >> 5) + (v & 3u);
        const unsigned r = row_base + (l & 31u);
        if (tok < tok_end && r < out_dim) y[(size_t)tok * out_dim + r] = s;
    }
}

// name(w, xq, y, in_dim, out_dim, p_rows): block = 64*KS threads (KS = 1..16 wavefronts
// splitting the contraction), grid = (ceil(out_dim/32), ceil(p_rows/(2*NV))), dynamic
// shared memory = KS * sizeof(SkinnyWaveLds<FMT, 2*NV>).  Q8_0 / Q4_0 / IQ4_XS need
// in_dim >= 256.
#define REIN_DEFINE_MMQ_SKINNY(name, FMT, NV)                                                    \
    extern "C" __global__ __launch_bounds__(1024) void name(REIN_MMQ_ARGS)                       \
    {                                                                                            \
        rein_mmq_skinny<FMT, NV>(w, xq, y, in_dim, out_dim, p_rows);                             \
    }
