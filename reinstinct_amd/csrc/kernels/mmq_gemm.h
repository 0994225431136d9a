// Prefill MMQ GEMM on the int8 matrix cores:  Y[P][N] = Xq[P][K] . W^T  with W in a
// repacked-v2 format and Xq in 40-byte BlockQ8 rows.
//
// Tiling (gfx950, wave64).  A workgroup of W wavefronts (4 in the tuned launch)
// owns TM tokens x 32W weight rows; wavefront w owns 32 of those rows and all TM
// tokens, as TM/32 MFMA tiles of 32x32.  The contraction is walked one
// 256-weight superblock (8 sub-blocks of 32) at a time:
//
//   * activations: the TM x 8 BlockQ8 of the chunk are staged in LDS, split into
//     the two 16-quant halves (so an MFMA operand is one conflict-free
//     ds_read_b128) plus planes of dx and xsum;
//   * weights: lane (j = lane%32, h = lane/32) streams row j's eight sub-blocks
//     straight from HBM/L2 (8 x 16 B contiguous = one cache line, scales as one
//     16 B load), expands half h of each to int8 in registers, and keeps them
//     for all TM/32 token tiles.  Weights have no reuse across wavefronts in
//     this mapping, so they never touch LDS;
//   * per sub-block and tile one v_mfma_i32_32x32x32_i8 (tokens = rows of the
//     tile, weights = columns) yields the exact int32 block dots; MFMA K = 32
//     is exactly one sub-block, lane half h carries quants 16h..16h+15 on both
//     operands;
//   * scales: v_mfma_f32_32x32x1_2b forms the outer products dx[token] *
//     dsc[row] for two sub-blocks at once in the accumulator layout, so the
//     combine is one convert and one fma per element; the -deff*xsum term of
//     Q4_K/Q5_K is a v_mfma_f32_32x32x2 (K = the two sub-blocks) straight into
//     the fp32 accumulators;
//   * Q6_K has one scale per 16 weights: two int8 MFMAs per sub-block with the
//     other half of the weight operand zeroed, and the 2-block outer product
//     holds dx*dsc_lo and dx*dsc_hi.  The -32 (Q6_K) and -8 (Q4_0) offsets are
//     folded into the int8 weights, which is integer-identical to the matvec's
//     idot - 32*sum(q8) form.
//
// Accumulator layout of a 32x32 tile: lane -> column (weight row) lane%32,
// register v -> tile row (token) 8*(v/4) + 4*(lane/32) + v%4.
//
// Replaces kernels/mmq_gemm_*_repacked.cpp (wide and narrow) and
// kernels/mmq_gemm_*_grouped.cpp of the reference; same arguments.  Any
// grid and any block size that is a multiple of 64 is correct: blockIdx.x walks
// row blocks, blockIdx.y token tiles, both as grid-stride loops.
#pragma once

#include "rein_formats.h"

typedef int   rein_v4i  __attribute__((ext_vector_type(4)));
typedef int   rein_v16i __attribute__((ext_vector_type(16)));
typedef float rein_v16f __attribute__((ext_vector_type(16)));
typedef float rein_v32f __attribute__((ext_vector_type(32)));

struct __attribute__((packed, aligned(2))) ReinU16x8 { uint16_t v[8]; };
struct __attribute__((packed, aligned(4))) ReinU32x8 { uint32_t v[8]; };
struct __attribute__((packed, aligned(8))) ReinU64x8 { uint2 v[8]; };

// (x - c) per byte for bytes x in [0,127], c < 128: no borrow crosses a byte
__device__ __forceinline__ int rein_sub_bytes(uint32_t x, uint32_t c4)
{
    return (int)(((x | 0x80808080u) - c4) ^ 0x80808080u);
}

// Weight side of one superblock chunk (8 sub-blocks) for lane (row, half h).
//   fetch()   raw plane words HBM/L2 -> registers (so the next chunk can be in
//             flight while this one is multiplied)
//   expand()  raw -> b[s]: int8 operand (quants 16h..16h+15 of sub-block s, offsets
//             folded), sc[u]: fp32 scale feeding the outer-product MFMA, mn[u]:
//             negated min term
// One-scale formats: u = pair index p, value for sub-block 2p+h.
// Q6_K: u = s, value = d*sc_h for this lane's 16-weight half.
template <int FMT> struct MmqChunk;

__device__ __forceinline__ unsigned rein_clamp_sb(unsigned sb, unsigned n_sub) { return sb < n_sub ? sb : n_sub - 1; }

template <> struct MmqChunk<REIN_Q4_K> {
    static constexpr bool kTwoScales = false, kHasMin = true;
    struct Raw { uint4 q[8]; ReinU16x8 sm; uint32_t dd; };
    rein_v4i b[8];
    float sc[4], mn[4];
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<REIN_Q4_K>& f, unsigned row, unsigned sb0, unsigned, unsigned)
    {
        const size_t i = (size_t)row * f.nsp + sb0;      // K-quants: n_sub % 8 == 0, the whole chunk is valid
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = f.nib[i + s];
        r.sm = *reinterpret_cast<const ReinU16x8*>(f.smp + i);
        r.dd = f.ddp[(size_t)row * f.n_super + (sb0 >> 3)];
    }
    __device__ __forceinline__ void expand(const Raw& r, unsigned, unsigned, unsigned h)
    {
        const float d = rein_h2f((uint16_t)(r.dd & 0xFFFFu)), dmin = rein_h2f((uint16_t)(r.dd >> 16));
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const uint32_t w[4] = {r.q[s].x, r.q[s].y, r.q[s].z, r.q[s].w};
#pragma unroll
            for (int j = 0; j < 4; j++) b[s][j] = (int)((w[j] >> (4 * h)) & 0x0F0F0F0Fu);
        }
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint16_t v = h ? r.sm.v[2 * p + 1] : r.sm.v[2 * p];
            sc[p] = d * (float)(v & 0xFFu);
            mn[p] = -(dmin * (float)(v >> 8));
        }
    }
};

template <> struct MmqChunk<REIN_Q5_K> {
    static constexpr bool kTwoScales = false, kHasMin = true;
    struct Raw { uint4 q[8]; ReinU32x8 qh; ReinU16x8 sm; uint32_t dd; };
    rein_v4i b[8];
    float sc[4], mn[4];
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<REIN_Q5_K>& f, unsigned row, unsigned sb0, unsigned, unsigned)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = f.nib[i + s];
        r.qh = *reinterpret_cast<const ReinU32x8*>(f.qhp + i);
        r.sm = *reinterpret_cast<const ReinU16x8*>(f.smp + i);
        r.dd = f.ddp[(size_t)row * f.n_super + (sb0 >> 3)];
    }
    __device__ __forceinline__ void expand(const Raw& r, unsigned, unsigned, unsigned h)
    {
        const float d = rein_h2f((uint16_t)(r.dd & 0xFFFFu)), dmin = rein_h2f((uint16_t)(r.dd >> 16));
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const uint32_t w[4] = {r.q[s].x, r.q[s].y, r.q[s].z, r.q[s].w};
#pragma unroll
            for (int j = 0; j < 4; j++)
                b[s][j] = (int)(((w[j] >> (4 * h)) & 0x0F0F0F0Fu) | (rein_spread4(r.qh.v[s] >> (8 * j + 4 * h)) << 4));
        }
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint16_t v = h ? r.sm.v[2 * p + 1] : r.sm.v[2 * p];
            sc[p] = d * (float)(v & 0xFFu);
            mn[p] = -(dmin * (float)(v >> 8));
        }
    }
};

template <> struct MmqChunk<REIN_Q6_K> {
    static constexpr bool kTwoScales = true, kHasMin = false;
    struct Raw { uint4 q[8]; ReinU64x8 h2; ReinU16x8 sm; uint16_t d; };
    rein_v4i b[8];
    float sc[8];
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<REIN_Q6_K>& f, unsigned row, unsigned sb0, unsigned, unsigned)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = f.nib[i + s];
        r.h2 = *reinterpret_cast<const ReinU64x8*>(f.h2p + i);
        r.sm = *reinterpret_cast<const ReinU16x8*>(f.smp + i);
        r.d  = f.dp[(size_t)row * f.n_super + (sb0 >> 3)];
    }
    __device__ __forceinline__ void expand(const Raw& r, unsigned, unsigned, unsigned h)
    {
        const float d = rein_h2f(r.d);
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const uint32_t w[4] = {r.q[s].x, r.q[s].y, r.q[s].z, r.q[s].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // hi2 byte 2j+h holds the 2-bit fields of this half's word j
                const uint32_t hw = j < 2 ? r.h2.v[s].x : r.h2.v[s].y;
                const uint32_t hb = (hw >> (16 * (j & 1) + 8 * h)) & 0xFFu;
                const uint32_t q6 = ((w[j] >> (4 * h)) & 0x0F0F0F0Fu) | rein_spread2(hb);
                b[s][j] = rein_sub_bytes(q6, 0x20202020u);
            }
            const uint16_t v = r.sm.v[s];
            sc[s] = d * (float)(int)(int8_t)(h ? (v >> 8) : (v & 0xFFu));
        }
    }
};

// Q8_0 / Q4_0 / IQ4_XS: one fp16 scale per sub-block, the chunk may be ragged
// (in_dim is only a multiple of 32): sub-blocks past the end are clamped and
// their scale is forced to zero.
template <int FMT> struct MmqChunkD16 {
    static constexpr bool kTwoScales = false, kHasMin = false;
    struct Raw { uint4 q[8]; uint16_t d[4]; };
    rein_v4i b[8];
    float sc[4], mn[4];
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<FMT>& f, unsigned row, unsigned sb0, unsigned n_sub, unsigned h)
    {
        const uint4* plane;
        if constexpr (FMT == REIN_Q8_0) plane = h ? f.hip_ : f.lop;     // this lane's 16 quants are one plane entry
        else plane = f.nib;
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = plane[(size_t)row * f.nsp + rein_clamp_sb(sb0 + s, n_sub)];
#pragma unroll
        for (int p = 0; p < 4; p++) r.d[p] = f.dp[(size_t)row * f.nsp + rein_clamp_sb(sb0 + 2 * p + h, n_sub)];
    }
    __device__ __forceinline__ void expand(const Raw& r, unsigned sb0, unsigned n_sub, unsigned h)
    {
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const uint32_t w[4] = {r.q[s].x, r.q[s].y, r.q[s].z, r.q[s].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if constexpr (FMT == REIN_Q8_0) b[s][j] = (int)w[j];
                else if constexpr (FMT == REIN_Q4_0) b[s][j] = rein_sub_bytes((w[j] >> (4 * h)) & 0x0F0F0F0Fu, 0x08080808u);
                else b[s][j] = rein_iq4_lut4((w[j] >> (4 * h)) & 0x0F0F0F0Fu);
            }
        }
#pragma unroll
        for (int p = 0; p < 4; p++) {
            sc[p] = sb0 + 2 * p + h < n_sub ? rein_h2f(r.d[p]) : 0.0f;
            mn[p] = 0.0f;
        }
    }
};
template <> struct MmqChunk<REIN_Q8_0> : MmqChunkD16<REIN_Q8_0> {};
template <> struct MmqChunk<REIN_Q4_0> : MmqChunkD16<REIN_Q4_0> {};
template <> struct MmqChunk<REIN_IQ4_XS> : MmqChunkD16<REIN_IQ4_XS> {};

// LDS image of one activation chunk: TM tokens x 8 sub-blocks.
template <int TM>
struct MmqLds {
    static constexpr int kPlane = TM + 1;                 // +1 entry: sub-block planes land on different banks
    uint4 qs[2][8][kPlane];                               // [half][sub-block][token]
    float dx[8][kPlane];
    float xsum[8][kPlane];
};

// Stage xq rows tok_base .. tok_base+TM (rows >= tok_end are zero-scaled) for
// sub-blocks sb0..sb0+8 into LDS, all threads of the workgroup.
template <int TM>
__device__ __forceinline__ void rein_mmq_stage(MmqLds<TM>& l, const BlockQ8* __restrict__ xq, unsigned n_sub,
                                               unsigned tok_base, unsigned tok_end, unsigned sb0)
{
    for (unsigned e = threadIdx.x; e < TM * 8; e += blockDim.x) {
        const unsigned tl = e >> 3, s = e & 7;
        const unsigned tok = tok_base + tl;
        const unsigned sb = sb0 + s;
        const bool ok = tok < tok_end && sb < n_sub;
        const BlockQ8* p = xq + (size_t)(tok < tok_end ? tok : tok_end - 1) * n_sub + (sb < n_sub ? sb : n_sub - 1);
        const float d = p->d, xs = p->xsum;
        uint4 lo, hi;
        lo.x = p->qs[0]; lo.y = p->qs[1]; lo.z = p->qs[2]; lo.w = p->qs[3];
        hi.x = p->qs[4]; hi.y = p->qs[5]; hi.z = p->qs[6]; hi.w = p->qs[7];
        l.qs[0][s][tl] = lo;
        l.qs[1][s][tl] = hi;
        l.dx[s][tl]   = ok ? d : 0.0f;
        l.xsum[s][tl] = ok ? xs : 0.0f;
    }
}

// One workgroup tile.  w: weight slab; xq/y rows tok_base..tok_end (exclusive) are
// this tile's tokens (at most TM); DOTS != 0 stores the int32 block dots to
// `dots` instead of computing y.
template <int FMT, int TM, int DOTS>
__device__ __forceinline__ void rein_mmq_tile(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                              float* __restrict__ y, int* __restrict__ dots,
                                              unsigned in_dim, unsigned out_dim, unsigned row_block,
                                              unsigned tok_base, unsigned tok_end)
{
    using F = Fmt<FMT>;
    using C = MmqChunk<FMT>;
    constexpr int NT = TM / 32;
    __shared__ MmqLds<TM> lds;

    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned j = lane & 31u, h = lane >> 5;
    const unsigned n_sub = in_dim >> 5;
    const F fmt(w, n_sub, out_dim);
    const unsigned row = (row_block * (blockDim.x >> 6) + wave) * 32u + j;
    const unsigned rowc = row < out_dim ? row : out_dim - 1;

    rein_v16f acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.0f;

    for (unsigned sb0 = 0; sb0 < n_sub; sb0 += 8) {
        C ck;
        {
            typename C::Raw raw;
            C::fetch(raw, fmt, rowc, sb0, n_sub, h);   // HBM/L2 -> registers, overlaps the staging below
            ck.expand(raw, sb0, n_sub, h);
        }
        __syncthreads();                           // previous chunk's LDS reads are done
        rein_mmq_stage<TM>(lds, xq, n_sub, tok_base, tok_end, sb0);
        __syncthreads();

        if constexpr (C::kTwoScales) {
#pragma unroll
            for (int s = 0; s < 8; s++) {
                rein_v4i blo, bhi;
#pragma unroll
                for (int k = 0; k < 4; k++) { blo[k] = h ? 0 : ck.b[s][k]; bhi[k] = h ? ck.b[s][k] : 0; }
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const uint4 a4 = lds.qs[h][s][t * 32 + j];
                    rein_v4i a;
                    a[0] = (int)a4.x; a[1] = (int)a4.y; a[2] = (int)a4.z; a[3] = (int)a4.w;
                    rein_v16i z;
#pragma unroll
                    for (int v = 0; v < 16; v++) z[v] = 0;
                    const rein_v16i clo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, blo, z, 0, 0, 0);
                    const rein_v16i chi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bhi, z, 0, 0, 0);
                    if (DOTS) {
#pragma unroll
                        for (int v = 0; v < 16; v++) {
                            const unsigned tok = tok_base + t * 32 + 8 * (v / 4) + 4 * h + (v % 4);
                            if (tok < tok_end && row < out_dim && sb0 + s < n_sub) {
                                int* o = dots + (((size_t)tok * out_dim + row) * n_sub + sb0 + s) * 2;
                                o[0] = clo[v];
                                o[1] = chi[v];
                            }
                        }
                    } else {
                        rein_v32f z32;
#pragma unroll
                        for (int v = 0; v < 32; v++) z32[v] = 0.0f;
                        // block 0 (lanes 0-31 of both operands): dx * dsc_lo, block 1: dx * dsc_hi
                        const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(lds.dx[s][t * 32 + j], ck.sc[s], z32, 0, 0, 0);
#pragma unroll
                        for (int v = 0; v < 16; v++) {
                            acc[t][v] = fmaf((float)clo[v], sx[v], acc[t][v]);
                            acc[t][v] = fmaf((float)chi[v], sx[16 + v], acc[t][v]);
                        }
                    }
                }
            }
        } else {
#pragma unroll
            for (int p = 0; p < 4; p++) {
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const uint4 a40 = lds.qs[h][2 * p][t * 32 + j];
                    const uint4 a41 = lds.qs[h][2 * p + 1][t * 32 + j];
                    rein_v4i a0, a1;
                    a0[0] = (int)a40.x; a0[1] = (int)a40.y; a0[2] = (int)a40.z; a0[3] = (int)a40.w;
                    a1[0] = (int)a41.x; a1[1] = (int)a41.y; a1[2] = (int)a41.z; a1[3] = (int)a41.w;
                    rein_v16i z;
#pragma unroll
                    for (int v = 0; v < 16; v++) z[v] = 0;
                    const rein_v16i c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, ck.b[2 * p], z, 0, 0, 0);
                    const rein_v16i c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, ck.b[2 * p + 1], z, 0, 0, 0);
                    if (DOTS) {
#pragma unroll
                        for (int v = 0; v < 16; v++) {
                            const unsigned tok = tok_base + t * 32 + 8 * (v / 4) + 4 * h + (v % 4);
                            if (tok < tok_end && row < out_dim) {
                                int* o = dots + ((size_t)tok * out_dim + row) * n_sub + sb0 + 2 * p;
                                if (sb0 + 2 * p < n_sub) o[0] = c0[v];
                                if (sb0 + 2 * p + 1 < n_sub) o[1] = c1[v];
                            }
                        }
                    } else {
                        rein_v32f z32;
#pragma unroll
                        for (int v = 0; v < 32; v++) z32[v] = 0.0f;
                        // lane half h feeds sub-block 2p+h: block 0 = sub-block 2p, block 1 = 2p+1
                        const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(lds.dx[2 * p + h][t * 32 + j], ck.sc[p], z32, 0, 0, 0);
                        if constexpr (C::kHasMin)
                            acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(lds.xsum[2 * p + h][t * 32 + j], ck.mn[p], acc[t], 0, 0, 0);
#pragma unroll
                        for (int v = 0; v < 16; v++) {
                            acc[t][v] = fmaf((float)c0[v], sx[v], acc[t][v]);
                            acc[t][v] = fmaf((float)c1[v], sx[16 + v], acc[t][v]);
                        }
                    }
                }
            }
        }
    }

    if (!DOTS) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const unsigned tok = tok_base + t * 32 + 8 * (v / 4) + 4 * h + (v % 4);
                if (tok < tok_end && row < out_dim) y[(size_t)tok * out_dim + row] = acc[t][v];
            }
    }
}

// ---------------------------------------------------------------------------
// Pipelined dense MMQ (the tuned launch).  Same math and layouts as
// rein_mmq_tile, plus:
//   * the next chunk's weight words and activation blocks are fetched into
//     registers before the current chunk is multiplied, the LDS image is
//     double-buffered, and there is one barrier per chunk;
//   * a fixed workgroup of 4 wavefronts (128 rows x TM tokens);
//   * a 1-D grid whose workgroup -> tile map keeps all token tiles of one
//     128-row weight block on the same XCD (workgroups are dealt round-robin
//     over the 8 XCDs, each with its own L2), so a weight block is pulled from
//     HBM once and re-read from that L2.
// Grid: 8 * ceil(n_row_blocks / 8) * n_token_tiles workgroups of 256 threads.
template <int TM>
struct MmqXRegs {
    static constexpr int kPer = TM * 8 / 256;            // activation blocks per thread per chunk
    uint2 hdr[kPer];
    uint4 lo[kPer], hi[kPer];
};

template <int TM>
__device__ __forceinline__ void rein_mmq_xfetch(MmqXRegs<TM>& r, const BlockQ8* __restrict__ xq, unsigned n_sub,
                                                unsigned tok_base, unsigned tok_end, unsigned sb0)
{
    // loads only: nothing here may consume a loaded value, or the wait for it
    // lands in front of the chunk's math and the prefetch is lost
#pragma unroll
    for (int k = 0; k < MmqXRegs<TM>::kPer; k++) {
        const unsigned e = threadIdx.x + k * 256;
        const unsigned tl = e >> 3, s = e & 7;
        const unsigned tok = tok_base + tl, sb = sb0 + s;
        const uint2* p = reinterpret_cast<const uint2*>(
            xq + (size_t)(tok < tok_end ? tok : tok_end - 1) * n_sub + (sb < n_sub ? sb : n_sub - 1));
        const uint2 w0 = p[0], w1 = p[1], w2 = p[2], w3 = p[3], w4 = p[4];   // 8-byte aligned words
        r.hdr[k] = w0;
        r.lo[k].x = w1.x; r.lo[k].y = w1.y; r.lo[k].z = w2.x; r.lo[k].w = w2.y;
        r.hi[k].x = w3.x; r.hi[k].y = w3.y; r.hi[k].z = w4.x; r.hi[k].w = w4.y;
    }
}

// rows past tok_end / sub-blocks past n_sub get zero scales here
template <int TM>
__device__ __forceinline__ void rein_mmq_xstore(MmqLds<TM>& l, const MmqXRegs<TM>& r, unsigned n_sub,
                                                unsigned tok_base, unsigned tok_end, unsigned sb0)
{
#pragma unroll
    for (int k = 0; k < MmqXRegs<TM>::kPer; k++) {
        const unsigned e = threadIdx.x + k * 256;
        const unsigned tl = e >> 3, s = e & 7;
        const bool ok = tok_base + tl < tok_end && sb0 + s < n_sub;
        l.qs[0][s][tl] = r.lo[k];
        l.qs[1][s][tl] = r.hi[k];
        l.dx[s][tl]    = ok ? __builtin_bit_cast(float, r.hdr[k].x) : 0.0f;
        l.xsum[s][tl]  = ok ? __builtin_bit_cast(float, r.hdr[k].y) : 0.0f;
    }
}

// multiply one staged chunk into the accumulators
template <int FMT, int TM>
__device__ __forceinline__ void rein_mmq_chunk_math(const MmqLds<TM>& lds, const MmqChunk<FMT>& ck,
                                                    rein_v16f (&acc)[TM / 32], unsigned j, unsigned h)
{
    using C = MmqChunk<FMT>;
    constexpr int NT = TM / 32;
    rein_v16i z;
#pragma unroll
    for (int v = 0; v < 16; v++) z[v] = 0;
    rein_v32f z32;
#pragma unroll
    for (int v = 0; v < 32; v++) z32[v] = 0.0f;

    if constexpr (C::kTwoScales) {
#pragma unroll
        for (int s = 0; s < 8; s++) {
            rein_v4i blo, bhi;
#pragma unroll
            for (int k = 0; k < 4; k++) { blo[k] = h ? 0 : ck.b[s][k]; bhi[k] = h ? ck.b[s][k] : 0; }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 a4 = lds.qs[h][s][t * 32 + j];
                rein_v4i a;
                a[0] = (int)a4.x; a[1] = (int)a4.y; a[2] = (int)a4.z; a[3] = (int)a4.w;
                const rein_v16i clo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, blo, z, 0, 0, 0);
                const rein_v16i chi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bhi, z, 0, 0, 0);
                const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(lds.dx[s][t * 32 + j], ck.sc[s], z32, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    acc[t][v] = fmaf((float)clo[v], sx[v], acc[t][v]);
                    acc[t][v] = fmaf((float)chi[v], sx[16 + v], acc[t][v]);
                }
            }
        }
    } else {
#pragma unroll
        for (int p = 0; p < 4; p++) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 a40 = lds.qs[h][2 * p][t * 32 + j];
                const uint4 a41 = lds.qs[h][2 * p + 1][t * 32 + j];
                rein_v4i a0, a1;
                a0[0] = (int)a40.x; a0[1] = (int)a40.y; a0[2] = (int)a40.z; a0[3] = (int)a40.w;
                a1[0] = (int)a41.x; a1[1] = (int)a41.y; a1[2] = (int)a41.z; a1[3] = (int)a41.w;
                const rein_v16i c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, ck.b[2 * p], z, 0, 0, 0);
                const rein_v16i c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, ck.b[2 * p + 1], z, 0, 0, 0);
                const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(lds.dx[2 * p + h][t * 32 + j], ck.sc[p], z32, 0, 0, 0);
                if constexpr (C::kHasMin)
                    acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(lds.xsum[2 * p + h][t * 32 + j], ck.mn[p], acc[t], 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    acc[t][v] = fmaf((float)c0[v], sx[v], acc[t][v]);
                    acc[t][v] = fmaf((float)c1[v], sx[16 + v], acc[t][v]);
                }
            }
        }
    }
}

template <int FMT, int TM>
__device__ __forceinline__ void rein_mmq_pipelined(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                   float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                   unsigned p_rows)
{
    using F = Fmt<FMT>;
    using C = MmqChunk<FMT>;
    constexpr int NT = TM / 32;
    __shared__ MmqLds<TM> lds[2];

    // workgroup -> (row block, token tile), XCD-aware
    const unsigned n_rb = (out_dim + 127u) / 128u;
    const unsigned n_tt = (p_rows + TM - 1) / TM;
    const unsigned xcd = blockIdx.x & 7u, k = blockIdx.x >> 3;
    const unsigned rb = (k / n_tt) * 8u + xcd, tt = k % n_tt;
    if (rb >= n_rb) return;

    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned j = lane & 31u, h = lane >> 5;
    const unsigned n_sub = in_dim >> 5;
    const F fmt(w, n_sub, out_dim);
    const unsigned row = rb * 128u + wave * 32u + j;
    const unsigned rowc = row < out_dim ? row : out_dim - 1;
    const unsigned tok_base = tt * TM;
    const unsigned tok_end = min(p_rows, tok_base + TM);

    rein_v16f acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.0f;

    typename C::Raw raw;
    MmqXRegs<TM> xr;
    C::fetch(raw, fmt, rowc, 0, n_sub, h);
    rein_mmq_xfetch<TM>(xr, xq, n_sub, tok_base, tok_end, 0);
    rein_mmq_xstore<TM>(lds[0], xr, n_sub, tok_base, tok_end, 0);
    __syncthreads();

    unsigned buf = 0;
    for (unsigned sb0 = 0; sb0 < n_sub; sb0 += 8, buf ^= 1u) {
        C ck;
        ck.expand(raw, sb0, n_sub, h);
        const bool more = sb0 + 8 < n_sub;
        if (more) {                                  // next chunk goes out before the math
            C::fetch(raw, fmt, rowc, sb0 + 8, n_sub, h);
            rein_mmq_xfetch<TM>(xr, xq, n_sub, tok_base, tok_end, sb0 + 8);
        }
        rein_mmq_chunk_math<FMT, TM>(lds[buf], ck, acc, j, h);
        if (more) rein_mmq_xstore<TM>(lds[buf ^ 1u], xr, n_sub, tok_base, tok_end, sb0 + 8);
        __syncthreads();
    }

#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const unsigned tok = tok_base + t * 32 + 8 * (v / 4) + 4 * h + (v % 4);
            if (tok < tok_end && row < out_dim) y[(size_t)tok * out_dim + row] = acc[t][v];
        }
}

// Dense GEMM: grid-stride over (row block, token tile).
template <int FMT, int TM, int DOTS>
__device__ __forceinline__ void rein_mmq_dense(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                               float* __restrict__ y, int* __restrict__ dots,
                                               unsigned in_dim, unsigned out_dim, unsigned p_rows)
{
    const unsigned rpb = 32u * (blockDim.x >> 6);
    const unsigned n_rb = (out_dim + rpb - 1u) / rpb;
    const unsigned n_tt = (p_rows + TM - 1) / TM;
    for (unsigned tt = blockIdx.y; tt < n_tt; tt += gridDim.y)
        for (unsigned rb = blockIdx.x; rb < n_rb; rb += gridDim.x) {
            const unsigned tok_base = tt * TM;
            const unsigned tok_end = min(p_rows, tok_base + TM);
            rein_mmq_tile<FMT, TM, DOTS>(w, xq, y, dots, in_dim, out_dim, rb, tok_base, tok_end);
        }
}

// Grouped-expert GEMM (kernels/mmq_gemm_q4k_grouped.cpp:38-165): tile index
// blockIdx.y -> expert by binary search over tile_off; the tile's tokens are
// rows expert_off[e] + 32*local .. of the expert-sorted xq / y.
template <int FMT>
__device__ __forceinline__ void rein_mmq_grouped(const uint8_t* __restrict__ slab, unsigned bytes_per_expert,
                                                 const int* __restrict__ expert_off, const int* __restrict__ tile_off,
                                                 unsigned n_expert, const BlockQ8* __restrict__ xq,
                                                 float* __restrict__ y, unsigned in_dim, unsigned out_dim)
{
    const unsigned rpb = 32u * (blockDim.x >> 6);
    const unsigned n_rb = (out_dim + rpb - 1u) / rpb;
    const unsigned n_tiles = (unsigned)tile_off[n_expert];
    for (unsigned tile = blockIdx.y; tile < n_tiles; tile += gridDim.y) {
        unsigned lo = 0, hi = n_expert;            // largest e with tile_off[e] <= tile
        while (hi - lo > 1) {
            const unsigned mid = (lo + hi) >> 1;
            if ((unsigned)tile_off[mid] <= tile) lo = mid; else hi = mid;
        }
        const unsigned e = lo;
        const unsigned tok_base = (unsigned)expert_off[e] + (tile - (unsigned)tile_off[e]) * 32u;
        const unsigned tok_end = (unsigned)expert_off[e + 1];
        if (tok_base >= tok_end) continue;         // host counted tiles with a smaller bn
        for (unsigned rb = blockIdx.x; rb < n_rb; rb += gridDim.x)
            rein_mmq_tile<FMT, 32, 0>(slab + (size_t)e * bytes_per_expert, xq, y, nullptr, in_dim, out_dim, rb,
                                      tok_base, min(tok_end, tok_base + 32u));
    }
}

#define REIN_MMQ_ARGS                                                                            \
    const unsigned char* __restrict__ w, const BlockQ8* __restrict__ xq, float* __restrict__ y, \
        unsigned int in_dim, unsigned int out_dim, unsigned int p_rows

#define REIN_DEFINE_MMQ(name, FMT, TM)                                                           \
    extern "C" __global__ __launch_bounds__(256) void name(REIN_MMQ_ARGS)                        \
    {                                                                                            \
        rein_mmq_dense<FMT, TM, 0>(w, xq, y, nullptr, in_dim, out_dim, p_rows);                  \
    }

// tuned entry: fixed 256-thread workgroups, 1-D XCD-aware grid
#define REIN_DEFINE_MMQ_PIPE(name, FMT, TM)                                                      \
    extern "C" __global__ __launch_bounds__(256) void name(REIN_MMQ_ARGS)                        \
    {                                                                                            \
        rein_mmq_pipelined<FMT, TM>(w, xq, y, in_dim, out_dim, p_rows);                          \
    }

#define REIN_DEFINE_MMQ_DOTS(name, FMT)                                                          \
    extern "C" __global__ __launch_bounds__(256) void name(                                      \
        const unsigned char* __restrict__ w, const BlockQ8* __restrict__ xq, int* __restrict__ out, \
        unsigned int in_dim, unsigned int out_dim, unsigned int p_rows)                          \
    {                                                                                            \
        rein_mmq_dense<FMT, 32, 1>(w, xq, nullptr, out, in_dim, out_dim, p_rows);                \
    }

#define REIN_DEFINE_MMQ_GROUPED(name, FMT)                                                       \
    extern "C" __global__ __launch_bounds__(256) void name(                                      \
        const unsigned char* __restrict__ slab, unsigned int bytes_per_expert,                   \
        const int* __restrict__ expert_off, const int* __restrict__ tile_off, unsigned int n_expert, \
        const BlockQ8* __restrict__ xq, float* __restrict__ y, unsigned int in_dim,              \
        unsigned int out_dim)                                                                    \
    {                                                                                            \
        rein_mmq_grouped<FMT>(slab, bytes_per_expert, expert_off, tile_off, n_expert, xq, y,     \
                              in_dim, out_dim);                                                  \
    }
