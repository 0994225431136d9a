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
//   * What bounds a weight stream is the number of bytes in flight, and registers are
//     the largest place to keep them: a wavefront holds the 16-byte weight plane of
//     several chunks ahead in registers (eight lanes walk a row's 128 contiguous bytes
//     per load, four loads per chunk), plus the chunk's small words (scales, aux bits) and
//     the TOK x 8 activation blocks of the next chunk.  Plain loads, so the compiler
//     counts them and waits for exactly the chunk that is consumed.
//   * A chunk's plane goes registers -> LDS -> registers once, because the MFMA wants
//     lane = weight row while a coalesced load wants lane = consecutive bytes; the
//     image is private to the wavefront (LDS operations of a wavefront execute in
//     order, so no barrier) and swizzled so that neither side has bank conflicts.
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

// Per-format small words of one chunk (aux bits, scales, fp16 pair) of the lane's
// row, fetched straight into registers (both lane halves need every sub-block's
// scale here).  begin()/pair()/rotate() turn the words into the per-sub-block scales;
// operand() is MmqChunk's.
template <int FMT> struct SkinnyFmt;

template <int FMT> struct SkinnyKQuant {
    using C = MmqChunk<FMT>;
    using Small = typename C::Small;
    static constexpr bool kHasMin = C::kHasMin, kTwoScales = C::kTwoScales;
    static __device__ __forceinline__ void fetch(Small& r, const Fmt<FMT>& f, unsigned row, unsigned sb0, unsigned n_sub)
    {
        C::fetch_small(r, f, row, sb0, n_sub, 0);
    }
    static __device__ __forceinline__ void place(Small&, unsigned) {}
    static __device__ __forceinline__ rein_v4i operand(const uint4& q, const Small& r, int s, unsigned h)
    {
        return C::operand(q, r, s, h);
    }
};

template <> struct SkinnyFmt<REIN_Q4_K> : SkinnyKQuant<REIN_Q4_K> {
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
// multiple of 32) fetches the last eight scales of the row instead, so the 16
// bytes never run past the end of the scale plane, and place() shifts them into
// position; sub-blocks past the end are zero-scaled.  Needs n_sub >= 8.
template <int FMT> struct SkinnyD16 {
    using C = MmqChunk<FMT>;
    struct Small { uint16_t d[8]; };
    static constexpr bool kHasMin = false, kTwoScales = false;
    unsigned left;                                   // valid sub-blocks from the front of the rotated words
    static __device__ __forceinline__ void fetch(Small& r, const Fmt<FMT>& f, unsigned row, unsigned sb0, unsigned n_sub)
    {
        const unsigned first = sb0 + 8u <= n_sub ? sb0 : n_sub - 8u;
        r = __builtin_bit_cast(Small, *reinterpret_cast<const ReinU16x8*>(f.dp + (size_t)row * f.nsp + first));
    }
    static __device__ __forceinline__ void place(Small& r, unsigned shift)
    {
        for (unsigned k = 0; k < shift; k++) {       // wave-uniform trip count
#pragma unroll
            for (int i = 0; i < 7; i++) r.d[i] = r.d[i + 1];
        }
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
template <> struct SkinnyFmt<REIN_IQ3_S> : SkinnyD16<REIN_IQ3_S> {};

// ---- the 16-byte weight plane(s) of one chunk: 32 rows x 8 sub-blocks -------------
// In registers as loaded: lane l of load i holds row 8i + l/8, sub-block l%8.
template <int FMT> struct SkinnyWRegs { uint4 q[MmqWLds<FMT>::kPlanes][4]; };
// In LDS: entry (row n, sub-block s) at 8n + ((s + n/2) & 7).  A ds_read_b128 of one
// sub-block by rows 0..15 (one quarter-wave pass) then covers all 64 banks once, and
// so does the store of two rows x 8 sub-blocks by lanes 0..15.
template <int FMT> struct SkinnyWImage { uint4 q[MmqWLds<FMT>::kPlanes][256]; };

template <int FMT>
__device__ __forceinline__ void rein_skinny_wfetch(SkinnyWRegs<FMT>& r, const Fmt<FMT>& fmt, unsigned row_base,
                                                   unsigned out_dim, unsigned sb0, unsigned n_sub, unsigned lane, bool live)
{
    const unsigned sb = rein_clamp_sb(sb0 + (lane & 7u), n_sub);
#pragma unroll
    for (int pl = 0; pl < MmqWLds<FMT>::kPlanes; pl++) {
        const uint4* plane = MmqChunk<FMT>::plane(fmt, (unsigned)pl);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const unsigned row = min(row_base + 8u * i + (lane >> 3), out_dim - 1u);
            r.q[pl][i] = rein_ldw(live ? plane + (size_t)row * fmt.nsp + sb : plane);
        }
    }
}

template <int FMT>
__device__ __forceinline__ void rein_skinny_wstash(SkinnyWImage<FMT>& l, const SkinnyWRegs<FMT>& r, unsigned lane)
{
#pragma unroll
    for (int pl = 0; pl < MmqWLds<FMT>::kPlanes; pl++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const unsigned n = 8u * i + (lane >> 3);
            l.q[pl][8u * n + (((lane & 7u) + (n >> 1)) & 7u)] = r.q[pl][i];
        }
    }
}

// ---- the activation blocks of one chunk: TOK rows x 8 sub-blocks -------------------
// In registers: lane l of load k holds block e = 64k + l, sub-block e / TOK of row
// e % TOK (rows past tok_end and sub-blocks past n_sub repeat the last valid one:
// their results are never stored, resp. are zero-scaled on the weight side).
//
// The fetches past a wavefront's last chunk are not branched around: a load under a
// branch makes its destination a merge of two values, which costs copies and a wait
// right behind the load.  `live == false` points every lane at the first bytes of the
// plane instead (one cache line, always valid) and the result is never used.
template <int TOK> struct SkinnyARegs { BlockQ8 b[(TOK * 8 + 63) / 64]; };      // TOK < 8: lanes past TOK*8 idle
template <int TOK>
struct SkinnyAct {
    uint4 qs[2][8][TOK];                                 // [half][sub-block][row]
    float dx[8][TOK];
    float xs[8][TOK];
};

template <int TOK>
__device__ __forceinline__ void rein_skinny_afetch(SkinnyARegs<TOK>& r, const BlockQ8* __restrict__ xq, unsigned n_sub,
                                                   unsigned tok_base, unsigned tok_end, unsigned sb0, unsigned lane,
                                                   bool live)
{
#pragma unroll
    for (int k = 0; k < (TOK * 8 + 63) / 64; k++) {
        const unsigned e = min(64u * k + lane, TOK * 8u - 1u);
        const unsigned tok = min(tok_base + e % TOK, tok_end - 1u), sb = rein_clamp_sb(sb0 + e / TOK, n_sub);
        r.b[k] = *(live ? xq + (size_t)tok * n_sub + sb : xq);
    }
}

template <int TOK, bool XS>
__device__ __forceinline__ void rein_skinny_astash(SkinnyAct<TOK>& a, const SkinnyARegs<TOK>& r, unsigned lane)
{
#pragma unroll
    for (int k = 0; k < (TOK * 8 + 63) / 64; k++) {
        const unsigned e = 64u * k + lane;
        if (TOK * 8 < 64 && e >= TOK * 8u) continue;
        const BlockQ8& b = r.b[k];
        a.qs[0][e / TOK][e % TOK] = make_uint4((unsigned)b.qs[0], (unsigned)b.qs[1], (unsigned)b.qs[2], (unsigned)b.qs[3]);
        a.qs[1][e / TOK][e % TOK] = make_uint4((unsigned)b.qs[4], (unsigned)b.qs[5], (unsigned)b.qs[6], (unsigned)b.qs[7]);
        a.dx[e / TOK][e % TOK] = b.d;
        if (XS) a.xs[e / TOK][e % TOK] = b.xsum;
    }
}

// Per-wavefront LDS of the skinny kernel: one chunk of the weight plane and of the
// activation blocks.  The launch passes KS of these as dynamic shared memory.
template <int FMT, int TOK>
struct SkinnyWaveLds {
    SkinnyWImage<FMT> w;
    SkinnyAct<TOK> act;
};
static_assert(sizeof(SkinnyWaveLds<REIN_Q4_K, 8>) == 4096 + 320 * 8, "host launcher mirrors this");
static_assert(sizeof(SkinnyWaveLds<REIN_Q6_K, 16>) == 4096 + 320 * 16, "host launcher mirrors this");
static_assert(sizeof(SkinnyWaveLds<REIN_Q8_0, 8>) == 2 * 4096 + 320 * 8, "host launcher mirrors this");

// Chunks of weight plane a wavefront keeps in flight.  What the loaded memory system
// needs to stream at full rate is on the order of 100 KB in flight per CU; at two
// wavefronts per SIMD (256 registers each) that is 12-16 KB per wavefront.
template <int FMT, int NV> struct SkinnyDepth { static constexpr int value = FMT == REIN_Q8_0 ? 2 : 3; };

template <int FMT, int NV>
__device__ __forceinline__ void rein_mmq_skinny(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                unsigned p_rows)
{
    using F = Fmt<FMT>;
    using SK = SkinnyFmt<FMT>;
    typedef typename SK::Small Small;
    constexpr int TOK = 2 * NV;
    constexpr bool XS = SK::kHasMin;
    typedef SkinnyWaveLds<FMT, TOK> WaveLds;
    extern __shared__ uint4 rein_skinny_lds[];
    static_assert(sizeof(WaveLds) >= 64 * NV * 4, "partial tiles are reduced through the per-wavefront LDS");
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
    // tile row of lane half h, register v is 8(v/4) + 4h + v%4: with NV <= 4 the tokens a lane
    // converts are NV*h + v, i.e. token t sits in tile row (t % NV) + 4(t / NV); the other
    // rows repeat real tokens and are never read back
    const unsigned ja = NV >= 4 ? (j & (TOK - 1)) : ((j & (NV - 1)) | (((j >> 2) & 1u) * NV));
    const unsigned rot = j >> 1;
    WaveLds& my = reinterpret_cast<WaveLds*>(rein_skinny_lds)[wave];

    const unsigned c_begin = wave * n_chunks / KS, c_end = (wave + 1u) * n_chunks / KS;

    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) acc[v] = 0.0f;
    rein_v16i czero;
#pragma unroll
    for (int v = 0; v < 16; v++) czero[v] = 0;

    // Queue: weight plane and small words of chunks c .. c+D-1, activation blocks of
    // chunk c.  Chunk c: move its registers to LDS, refill them (activations of c+1
    // first, then the plane of c+D, so that the next chunk's wait for its activations
    // leaves the younger plane requests in flight), then the math, then the small
    // words of c+D.  The loop body is D chunks, so every queue slot is a fixed set of
    // registers.
    constexpr int D = SkinnyDepth<FMT, NV>::value;
    SkinnyWRegs<FMT> wq[D];
    Small sq[D];
    SkinnyARegs<TOK> aq;

    auto step = [&](unsigned c, SkinnyWRegs<FMT>& wr, Small& sr) {
        const unsigned sb0 = c * 8u;
        rein_skinny_wstash<FMT>(my.w, wr, lane);
        rein_skinny_astash<TOK, XS>(my.act, aq, lane);
        Small cur = sr;
        rein_skinny_afetch<TOK>(aq, xq, n_sub, tok_base, tok_end, sb0 + 8u, lane, c + 1u < c_end);
        const bool live2 = c + D < c_end;
        rein_skinny_wfetch<FMT>(wr, fmt, row_base, out_dim, live2 ? sb0 + 8u * D : 0u, n_sub, lane, live2);
        SK::place(cur, sb0 + 8u <= n_sub ? 0u : sb0 + 8u - n_sub);     // a ragged chunk was fetched from n_sub - 8
        SK sk;
        sk.begin(cur, sb0, n_sub);
        const SkinnyAct<TOK>& a = my.act;

#pragma unroll 1
        for (unsigned p = 0; p < 4; p++) {
            rein_v4i b[2];
            b[0] = SK::operand(my.w.q[wsel][8u * j + ((2u * p + rot) & 7u)], cur, 0, h);
            b[1] = SK::operand(my.w.q[wsel][8u * j + ((2u * p + 1u + rot) & 7u)], cur, 1, h);
            float sc[2], sc_hi[2], mn[2];
            sk.pair(cur, sc, sc_hi, mn);
#pragma unroll
            for (int s = 0; s < 2; s++) {
                const unsigned sb = 2u * p + s;
                const uint4 a4 = a.qs[h][sb][ja];
                rein_v4i av;
                av[0] = (int)a4.x; av[1] = (int)a4.y; av[2] = (int)a4.z; av[3] = (int)a4.w;
                float dxv[NV], xsv[NV];
                if constexpr (NV >= 4) {
#pragma unroll
                    for (int q = 0; q < NV / 4; q++) {
                        const float4 d4 = *reinterpret_cast<const float4*>(&a.dx[sb][8 * q + 4 * h]);
                        dxv[4 * q] = d4.x; dxv[4 * q + 1] = d4.y; dxv[4 * q + 2] = d4.z; dxv[4 * q + 3] = d4.w;
                        if constexpr (XS) {
                            const float4 x4 = *reinterpret_cast<const float4*>(&a.xs[sb][8 * q + 4 * h]);
                            xsv[4 * q] = x4.x; xsv[4 * q + 1] = x4.y; xsv[4 * q + 2] = x4.z; xsv[4 * q + 3] = x4.w;
                        }
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < NV; v++) {
                        dxv[v] = a.dx[sb][NV * h + v];
                        if constexpr (XS) xsv[v] = a.xs[sb][NV * h + v];
                    }
                }
                if constexpr (SK::kTwoScales) {
                    rein_v4i blo, bhi;
#pragma unroll
                    for (int k = 0; k < 4; k++) { blo[k] = h ? 0 : b[s][k]; bhi[k] = h ? b[s][k] : 0; }
                    const rein_v16i ilo = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, blo, czero, 0, 0, 0);
                    const rein_v16i ihi = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bhi, czero, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < NV; v++)
                        acc[v] = fmaf(fmaf((float)ihi[v], sc_hi[s], (float)ilo[v] * sc[s]), dxv[v], acc[v]);
                } else {
                    const rein_v16i id = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, b[s], czero, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < NV; v++) {
                        acc[v] = fmaf((float)id[v], sc[s] * dxv[v], acc[v]);
                        if constexpr (XS) acc[v] = fmaf(-mn[s], xsv[v], acc[v]);
                    }
                }
            }
            SK::rotate(cur);
        }
        // the small words of c+2 go into the registers `cur` has just left (requested
        // earlier they would need a third set, and copies at the loop end that wait)
        SK::fetch(sr, fmt, live2 ? rowc : 0u, live2 ? sb0 + 8u * D : 0u, n_sub);
    };

    if (c_begin < c_end) {
        rein_skinny_afetch<TOK>(aq, xq, n_sub, tok_base, tok_end, c_begin * 8u, lane, true);
#pragma unroll
        for (int u = 0; u < D; u++) {
            const bool live = c_begin + u < c_end;
            rein_skinny_wfetch<FMT>(wq[u], fmt, row_base, out_dim, live ? (c_begin + u) * 8u : 0u, n_sub, lane, live);
            SK::fetch(sq[u], fmt, live ? rowc : 0u, live ? (c_begin + u) * 8u : 0u, n_sub);
        }
        unsigned c = c_begin;
        for (; c + D <= c_end; c += D) {
#pragma unroll
            for (int u = 0; u < D; u++) step(c + u, wq[u], sq[u]);
        }
#pragma unroll
        for (int u = 0; u < D - 1; u++)
            if (c + u < c_end) step(c + u, wq[u], sq[u]);
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
        const unsigned tok = tok_base + (NV >= 4 ? 8u * (v >> 2) + 4u * (l >> 5) + (v & 3u) : NV * (l >> 5) + v);
        const unsigned r = row_base + (l & 31u);
        if (tok < tok_end && r < out_dim) y[(size_t)tok * out_dim + r] = s;
    }
}

// name(w, xq, y, in_dim, out_dim, p_rows): block = 64*KS threads (KS = 1..8 wavefronts
// splitting the contraction; OCC = wavefronts per SIMD the register budget is set for), grid = (ceil(out_dim/32), ceil(p_rows/(2*NV))), dynamic
// shared memory = KS * sizeof(SkinnyWaveLds<FMT, 2*NV>).  Q8_0 / Q4_0 / IQ4_XS need
// in_dim >= 256.
#define REIN_DEFINE_MMQ_SKINNY(name, FMT, NV, OCC)                                                \
    extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(OCC, OCC)))   \
    void name(REIN_MMQ_ARGS)                                                                      \
    {                                                                                             \
        rein_mmq_skinny<FMT, NV>(w, xq, y, in_dim, out_dim, p_rows);                              \
    }
