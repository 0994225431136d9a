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
//     ds_read_b128) plus planes of dx and of the bf16 splits of xsum;
//   * weights: lane (j = lane%32, h = lane/32) owns row j's eight sub-blocks, expands
//     half h of each to int8 in registers and keeps them for all TM/32 token tiles.
//     Weights have no reuse across wavefronts in this mapping.  The plain kernels
//     (rein_mmq_tile) load them straight into registers (8 x 16 B contiguous = one
//     cache line, scales as one 16 B load); the tuned kernel (rein_mmq_pipelined_tile)
//     moves the 16-byte plane HBM -> LDS asynchronously into a per-wavefront ring and
//     reads it back as it is consumed;
//   * per sub-block and tile one v_mfma_i32_32x32x32_i8 (tokens = rows of the
//     tile, weights = columns) yields the exact int32 block dots; MFMA K = 32
//     is exactly one sub-block, lane half h carries quants 16h..16h+15 on both
//     operands;
//   * scales: v_mfma_f32_32x32x1_2b forms the outer products dx[token] *
//     dsc[row] for two sub-blocks at once in the accumulator layout, so the
//     combine is one subtract (the int32 dots come out biased so that their bits
//     read as fp32) and one fma per element; the -dmin*m*xsum term of Q4_K/Q5_K
//     is one superblock-wide pair of bf16 MFMAs on the three-way bf16 split of
//     xsum against the integer mins (exact products), scaled by -dmin;
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
#include "q8_block.h"

typedef int   rein_v4i  __attribute__((ext_vector_type(4)));
typedef int   rein_v16i __attribute__((ext_vector_type(16)));
typedef float rein_v16f __attribute__((ext_vector_type(16)));
typedef float rein_v32f __attribute__((ext_vector_type(32)));
typedef __bf16 rein_v8bf __attribute__((ext_vector_type(8)));

// The int8 MFMA accumulates on top of this bias, so its int32 result read as
// fp32 is exactly 12582912 + dot (|dot| < 2^22), and one v_sub_f32 replaces the
// slower v_cvt_f32_i32.
#define REIN_MMQ_MAGIC_I 0x4B400000
#define REIN_MMQ_MAGIC_F 12582912.0f

// Whole-vector form on purpose: written per element (bit_cast of c[v], then the
// subtract) hipcc 7.2 reuses element 0 for all sixteen lanes of the tile.
__device__ __forceinline__ rein_v16f rein_mmq_unbias(rein_v16i c)
{
    return __builtin_bit_cast(rein_v16f, c) - REIN_MMQ_MAGIC_F;
}

// The tuned kernels bias the int8 MFMA through its accumulator operand with the inline
// constant 1/(2 pi) = 0x3E22F983 instead: no registers hold the bias.  Integer addition of
// `dot` to that bit pattern stays inside the binade [1/8, 1/4) for -2292099 <= dot <=
// 6096508 (every format's 32-element dot is below 2^20), whose ulp is 2^-26, so the result
// read as fp32 is exactly 1/(2 pi) + dot * 2^-26 and the subtraction below returns
// dot * 2^-26 exactly.  The activation scales are staged multiplied by 2^26
// (rein_mmq_xstore), a power of two, so every product and sum rounds as without the trick.
// The instruction is written as asm because the compiler does not fold a splat of that
// constant into the operand.  The compiler cannot see that this is an MFMA, so the wait
// states it would have placed are written out: two between a VALU write of an operand and
// the MFMA that reads it, twelve between an 8-pass MFMA and a read of its result.
#define REIN_MMQ_INV2PI 0.15915494f
#define REIN_MMQ_XSCALE 67108864.0f
// SBIAS: subtract the constant out of a scalar register (four-byte encodings) instead of a
// literal; measured per tile shape, the 64-token tile gains 4 % from it, the 32-token tile
// loses 1 %.
template <bool SBIAS>
__device__ __forceinline__ rein_v16f rein_mmq_dot_tile(rein_v4i a, rein_v4i b)
{
    rein_v16f r;
    asm("s_nop 1\n\tv_mfma_i32_32x32x32_i8 %0, %1, %2, 0.15915494\n\ts_nop 11" : "=&v"(r) : "v"(a), "v"(b));
    float c0 = REIN_MMQ_INV2PI;
    if constexpr (SBIAS) asm("" : "+s"(c0));
    rein_v16f f = r - c0;
    // all sixteen subtractions (in place) before the first fma: independent fp32
    // instructions issue faster than sixteen dependent subtract / fma pairs
    asm("" : "+v"(f));
    return f;
}

// bf16 bit pattern of a small non-negative integer (exact below 256)
__device__ __forceinline__ uint32_t rein_bf16_of_u8(uint32_t v) { return __builtin_bit_cast(uint32_t, (float)v) >> 16; }

struct __attribute__((packed, aligned(2))) ReinU16x8 { uint16_t v[8]; };
struct __attribute__((packed, aligned(4))) ReinU32x8 { uint32_t v[8]; };
struct __attribute__((packed, aligned(8))) ReinU64x8 { uint2 v[8]; };

// Weight side of one superblock chunk (8 sub-blocks) for lane (row, half h).
// The 16-byte-per-sub-block plane (nibbles; Q8_0: the lane half's quant plane) is
// kept apart from the small words (aux bits, scales, fp16 pair), because the tuned
// kernel moves the former through LDS and only the latter through registers:
//   Small / fetch_small()  aux + scale words HBM/L2 -> registers
//   prepare()   Small -> sc[u]: fp32 scale feeding the outer-product MFMA; Q4_K/Q5_K
//               also mb: the eight 6-bit mins as bf16 and ndmin = -dmin
//   operand()   16 plane bytes of sub-block s -> int8 MFMA operand (quants
//               16h..16h+15, offsets folded)
//   plane()     which 16-byte plane this lane half reads
// One-scale formats: u = pair index p, value for sub-block 2p+h.
// Q6_K: u = s, value = d*sc_h for this lane's 16-weight half.
// The plain kernels use Raw / fetch() / expand(): everything through registers.
template <int FMT> struct MmqChunk;

__device__ __forceinline__ unsigned rein_clamp_sb(unsigned sb, unsigned n_sub) { return sb < n_sub ? sb : n_sub - 1; }

template <int FMT, class Self> struct MmqChunkBase {
    // kSplitK: the lane halves of the tuned kernel split a sub-block's contraction as
    // {0..7, 16..23} / {8..15, 24..31} instead of {0..15} / {16..31} (rein_mmq_xstore stages
    // the activations to match); operand_at() then reads only its 8 plane bytes
    static constexpr bool kSplitK = false;
    rein_v4i b[8];
    template <class Small>
    static __device__ __forceinline__ rein_v4i operand_at(const uint4* e, const Small& sm, int s, unsigned h)
    {
        return Self::operand(*e, sm, s, h);
    }
    // what the tuned kernel needs of prepare(); the same unless a format says otherwise
    template <class Small>
    __device__ __forceinline__ void prepare_tuned(const Small& r, unsigned sb0, unsigned n_sub, unsigned h)
    {
        static_cast<Self*>(this)->prepare(r, sb0, n_sub, h);
    }
    template <class Raw>
    __device__ __forceinline__ void expand(const Raw& r, unsigned sb0, unsigned n_sub, unsigned h)
    {
        Self& self = *static_cast<Self*>(this);
        self.prepare(r.sm, sb0, n_sub, h);
#pragma unroll
        for (int s = 0; s < 8; s++) b[s] = Self::operand(r.q[s], r.sm, s, h);
    }
};

template <> struct MmqChunk<REIN_Q4_K> : MmqChunkBase<REIN_Q4_K, MmqChunk<REIN_Q4_K>> {
    static constexpr bool kTwoScales = false, kHasMin = true, kMinSplit = false;
    struct Small { ReinU16x8 sm; uint32_t dd; };
    struct Raw { uint4 q[8]; Small sm; };
    float sc[4], ndmin;
    rein_v8bf mb;
    static __device__ __forceinline__ const uint4* plane(const Fmt<REIN_Q4_K>& f, unsigned) { return f.nib; }
    static __device__ __forceinline__ void fetch_small(Small& r, const Fmt<REIN_Q4_K>& f, unsigned row, unsigned sb0, unsigned, unsigned)
    {
        const size_t i = (size_t)row * f.nsp + sb0;      // K-quants: n_sub % 8 == 0, the whole chunk is valid
        r.sm = *reinterpret_cast<const ReinU16x8*>(f.smp + i);
        r.dd = f.ddp[(size_t)row * f.n_super + (sb0 >> 3)];
    }
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<REIN_Q4_K>& f, unsigned row, unsigned sb0, unsigned n_sub, unsigned h)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = f.nib[i + s];
        fetch_small(r.sm, f, row, sb0, n_sub, h);
    }
    __device__ __forceinline__ void prepare(const Small& r, unsigned, unsigned, unsigned h)
    {
        const float d = rein_h2f((uint16_t)(r.dd & 0xFFFFu)), dmin = rein_h2f((uint16_t)(r.dd >> 16));
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint16_t v = h ? r.sm.v[2 * p + 1] : r.sm.v[2 * p];
            sc[p] = d * (float)(v & 0xFFu);
        }
        uint4 m4;                                   // the eight 6-bit mins as bf16, sub-block order
        m4.x = rein_bf16_of_u8(r.sm.v[0] >> 8) | (rein_bf16_of_u8(r.sm.v[1] >> 8) << 16);
        m4.y = rein_bf16_of_u8(r.sm.v[2] >> 8) | (rein_bf16_of_u8(r.sm.v[3] >> 8) << 16);
        m4.z = rein_bf16_of_u8(r.sm.v[4] >> 8) | (rein_bf16_of_u8(r.sm.v[5] >> 8) << 16);
        m4.w = rein_bf16_of_u8(r.sm.v[6] >> 8) | (rein_bf16_of_u8(r.sm.v[7] >> 8) << 16);
        mb = __builtin_bit_cast(rein_v8bf, m4);
        ndmin = -dmin;
    }
    static __device__ __forceinline__ rein_v4i operand(const uint4& q, const Small&, int, unsigned h)
    {
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        rein_v4i o;
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = (int)((w[j] >> (4 * h)) & 0x0F0F0F0Fu);
        return o;
    }
    // Plane byte i holds weights i (low nibble) and 16 + i (high nibble): the 8 bytes
    // 8h..8h+7 give weights {8h..8h+7, 16+8h..16+8h+7} with two masks and two shifts + masks.
    static constexpr bool kSplitK = true;
    static __device__ __forceinline__ rein_v4i operand_at(const uint4* e, const Small&, int, unsigned h)
    {
        const uint2 q = reinterpret_cast<const uint2*>(e)[h];
        rein_v4i o;
        o[0] = (int)(q.x & 0x0F0F0F0Fu);
        o[1] = (int)(q.y & 0x0F0F0F0Fu);
        o[2] = (int)((q.x >> 4) & 0x0F0F0F0Fu);
        o[3] = (int)((q.y >> 4) & 0x0F0F0F0Fu);
        return o;
    }
    // next sub-block pair to the front (the rolled loop of the tuned kernel only
    // ever indexes entries 0 and 1)
    __device__ __forceinline__ void rotate(Small&) { sc[0] = sc[1]; sc[1] = sc[2]; sc[2] = sc[3]; }
};

template <> struct MmqChunk<REIN_Q5_K> : MmqChunkBase<REIN_Q5_K, MmqChunk<REIN_Q5_K>> {
    static constexpr bool kTwoScales = false, kHasMin = true, kMinSplit = false;
    struct Small { ReinU32x8 qh; ReinU16x8 sm; uint32_t dd; };
    struct Raw { uint4 q[8]; Small sm; };
    float sc[4], ndmin;
    rein_v8bf mb;
    static __device__ __forceinline__ const uint4* plane(const Fmt<REIN_Q5_K>& f, unsigned) { return f.nib; }
    static __device__ __forceinline__ void fetch_small(Small& r, const Fmt<REIN_Q5_K>& f, unsigned row, unsigned sb0, unsigned, unsigned)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
        r.qh = *reinterpret_cast<const ReinU32x8*>(f.qhp + i);
        r.sm = *reinterpret_cast<const ReinU16x8*>(f.smp + i);
        r.dd = f.ddp[(size_t)row * f.n_super + (sb0 >> 3)];
    }
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<REIN_Q5_K>& f, unsigned row, unsigned sb0, unsigned n_sub, unsigned h)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = f.nib[i + s];
        fetch_small(r.sm, f, row, sb0, n_sub, h);
    }
    __device__ __forceinline__ void prepare(const Small& r, unsigned, unsigned, unsigned h)
    {
        const float d = rein_h2f((uint16_t)(r.dd & 0xFFFFu)), dmin = rein_h2f((uint16_t)(r.dd >> 16));
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint16_t v = h ? r.sm.v[2 * p + 1] : r.sm.v[2 * p];
            sc[p] = d * (float)(v & 0xFFu);
        }
        uint4 m4;
        m4.x = rein_bf16_of_u8(r.sm.v[0] >> 8) | (rein_bf16_of_u8(r.sm.v[1] >> 8) << 16);
        m4.y = rein_bf16_of_u8(r.sm.v[2] >> 8) | (rein_bf16_of_u8(r.sm.v[3] >> 8) << 16);
        m4.z = rein_bf16_of_u8(r.sm.v[4] >> 8) | (rein_bf16_of_u8(r.sm.v[5] >> 8) << 16);
        m4.w = rein_bf16_of_u8(r.sm.v[6] >> 8) | (rein_bf16_of_u8(r.sm.v[7] >> 8) << 16);
        mb = __builtin_bit_cast(rein_v8bf, m4);
        ndmin = -dmin;
    }
    static __device__ __forceinline__ rein_v4i operand(const uint4& q, const Small& r, int s, unsigned h)
    {
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        rein_v4i o;
#pragma unroll
        for (int j = 0; j < 4; j++)
            o[j] = (int)(((w[j] >> (4 * h)) & 0x0F0F0F0Fu) | (rein_spread4(r.qh.v[s] >> (8 * j + 4 * h)) << 4));
        return o;
    }
    __device__ __forceinline__ void rotate(Small& r)
    {
        sc[0] = sc[1]; sc[1] = sc[2]; sc[2] = sc[3];
#pragma unroll
        for (int i = 0; i < 6; i++) r.qh.v[i] = r.qh.v[i + 2];
    }
};

// Q5_1: the Q5_K operand with a raw fp16 (d, m) per sub-block.  The minimum term
// sum_s m_s * xsum_s goes through the bf16 MFMA like Q5_K's, but m_s is an fp16 value, not
// a 6-bit integer under a shared dmin: it is split into a bf16 head (8 significant bits)
// and the exact remainder (the other 3), so the products stay exact.  in_dim is only a
// multiple of 32: sub-blocks past the end are clamped and zero-scaled.
template <> struct MmqChunk<REIN_Q5_1> : MmqChunkBase<REIN_Q5_1, MmqChunk<REIN_Q5_1>> {
    static constexpr bool kTwoScales = false, kHasMin = true, kMinSplit = true;
    struct Small { ReinU32x8 qh; ReinU32x8 dm; };
    struct Raw { uint4 q[8]; Small sm; };
    float sc[4], ndmin;
    rein_v8bf mb, mb_lo;
    static __device__ __forceinline__ const uint4* plane(const Fmt<REIN_Q5_1>& f, unsigned) { return f.nib; }
    static __device__ __forceinline__ void fetch_small(Small& r, const Fmt<REIN_Q5_1>& f, unsigned row, unsigned sb0, unsigned n_sub, unsigned)
    {
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const size_t i = (size_t)row * f.nsp + rein_clamp_sb(sb0 + s, n_sub);
            r.qh.v[s] = f.qhp[i];
            r.dm.v[s] = f.dmp[i];
        }
    }
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<REIN_Q5_1>& f, unsigned row, unsigned sb0, unsigned n_sub, unsigned h)
    {
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = f.nib[(size_t)row * f.nsp + rein_clamp_sb(sb0 + s, n_sub)];
        fetch_small(r.sm, f, row, sb0, n_sub, h);
    }
    __device__ __forceinline__ void prepare(const Small& r, unsigned sb0, unsigned n_sub, unsigned h)
    {
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint32_t v = h ? r.dm.v[2 * p + 1] : r.dm.v[2 * p];
            sc[p] = sb0 + 2 * p + h < n_sub ? rein_h2f((uint16_t)(v & 0xFFFFu)) : 0.0f;
        }
        uint32_t hi[8], lo[8];
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const float m = sb0 + s < n_sub ? rein_h2f((uint16_t)(r.dm.v[s] >> 16)) : 0.0f;
            const uint32_t head = __builtin_bit_cast(uint32_t, m) & 0xFFFF0000u;
            const float rest = m - __builtin_bit_cast(float, head);          // at most 3 significant bits: exact in bf16
            hi[s] = head >> 16;
            lo[s] = __builtin_bit_cast(uint32_t, rest) >> 16;
        }
        uint4 m4;
        m4.x = hi[0] | (hi[1] << 16); m4.y = hi[2] | (hi[3] << 16); m4.z = hi[4] | (hi[5] << 16); m4.w = hi[6] | (hi[7] << 16);
        mb = __builtin_bit_cast(rein_v8bf, m4);
        m4.x = lo[0] | (lo[1] << 16); m4.y = lo[2] | (lo[3] << 16); m4.z = lo[4] | (lo[5] << 16); m4.w = lo[6] | (lo[7] << 16);
        mb_lo = __builtin_bit_cast(rein_v8bf, m4);
        ndmin = 1.0f;                                                        // the term is + m * xsum (deff = -m)
    }
    static __device__ __forceinline__ rein_v4i operand(const uint4& q, const Small& r, int s, unsigned h)
    {
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        rein_v4i o;
#pragma unroll
        for (int j = 0; j < 4; j++)
            o[j] = (int)(((w[j] >> (4 * h)) & 0x0F0F0F0Fu) | (rein_spread4(r.qh.v[s] >> (8 * j + 4 * h)) << 4));
        return o;
    }
    __device__ __forceinline__ void rotate(Small& r)
    {
        sc[0] = sc[1]; sc[1] = sc[2]; sc[2] = sc[3];
#pragma unroll
        for (int i = 0; i < 6; i++) r.qh.v[i] = r.qh.v[i + 2];
    }
};

template <> struct MmqChunk<REIN_Q6_K> : MmqChunkBase<REIN_Q6_K, MmqChunk<REIN_Q6_K>> {
    static constexpr bool kTwoScales = true, kHasMin = false;
    struct Small { ReinU64x8 h2; ReinU16x8 sm; uint16_t d; };
    struct Raw { uint4 q[8]; Small sm; };
    float sc[8];
    static __device__ __forceinline__ const uint4* plane(const Fmt<REIN_Q6_K>& f, unsigned) { return f.nib; }
    static __device__ __forceinline__ void fetch_small(Small& r, const Fmt<REIN_Q6_K>& f, unsigned row, unsigned sb0, unsigned, unsigned)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
        r.h2 = *reinterpret_cast<const ReinU64x8*>(f.h2p + i);
        r.sm = *reinterpret_cast<const ReinU16x8*>(f.smp + i);
        r.d  = f.dp[(size_t)row * f.n_super + (sb0 >> 3)];
    }
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<REIN_Q6_K>& f, unsigned row, unsigned sb0, unsigned n_sub, unsigned h)
    {
        const size_t i = (size_t)row * f.nsp + sb0;
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = f.nib[i + s];
        fetch_small(r.sm, f, row, sb0, n_sub, h);
    }
    __device__ __forceinline__ void prepare(const Small& r, unsigned, unsigned, unsigned h)
    {
        const float d = rein_h2f(r.d);
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const uint16_t v = r.sm.v[s];
            sc[s] = d * (float)(int)(int8_t)(h ? (v >> 8) : (v & 0xFFu));
        }
    }
    static __device__ __forceinline__ rein_v4i operand(const uint4& q, const Small& r, int s, unsigned h)
    {
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        rein_v4i o;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // hi2 byte 2j+h holds the 2-bit fields of this half's word j
            const uint32_t hw = j < 2 ? r.h2.v[s].x : r.h2.v[s].y;
            const uint32_t q6 = ((w[j] >> (4 * h)) & 0x0F0F0F0Fu) | rein_spread2(hw, 16 * (j & 1) + 8 * h);
            o[j] = rein_sub_bytes(q6, 0x20202020u);
        }
        return o;
    }
    // Tuned kernel.  The lane halves split a sub-block as {0..7, 16..23} / {8..15, 24..31}:
    // operand registers 0,1 then belong to the first 16-weight scale group and 2,3 to the
    // second in BOTH halves, so the two groups' dots come from two MFMAs whose other
    // registers are constant zeros (no per-lane masking).  The int8 group scales combine the
    // two int32 dots exactly (|dot| <= 16*32*127, |sum| < 2^24), which leaves one fp32 scale
    // per sub-block, d * dx, as in the one-scale formats.  dq = d * 2^-26 undoes the factor
    // the activation scales are staged with.  hi2 dword h holds this half's 2-bit fields:
    // byte 0 -> weights 8h.., byte 2 -> 8h+4.., byte 1 -> 16+8h.., byte 3 -> 20+8h...
    static constexpr bool kSplitK = true;
    float dq;
    __device__ __forceinline__ void prepare_tuned(const Small& r, unsigned, unsigned, unsigned)
    {
        dq = rein_h2f(r.d) * (1.0f / REIN_MMQ_XSCALE);
    }
    static __device__ __forceinline__ rein_v4i operand_at(const uint4* e, const Small& r, int s, unsigned h)
    {
        const uint2 q = reinterpret_cast<const uint2*>(e)[h];
        const uint32_t hw = h ? r.h2.v[s].y : r.h2.v[s].x;
        rein_v4i o;
        o[0] = rein_sub_bytes((q.x & 0x0F0F0F0Fu) | rein_spread2(hw, 0), 0x20202020u);
        o[1] = rein_sub_bytes((q.y & 0x0F0F0F0Fu) | rein_spread2(hw, 16), 0x20202020u);
        o[2] = rein_sub_bytes(((q.x >> 4) & 0x0F0F0F0Fu) | rein_spread2(hw, 8), 0x20202020u);
        o[3] = rein_sub_bytes(((q.y >> 4) & 0x0F0F0F0Fu) | rein_spread2(hw, 24), 0x20202020u);
        return o;
    }
    // the int8 scales of sub-block s (0 or 1 after rotation) for the two groups
    static __device__ __forceinline__ int group_scale(const Small& r, int s, int g)
    {
        return (int)(int8_t)(g ? (r.sm.v[s] >> 8) : (r.sm.v[s] & 0xFFu));
    }
    __device__ __forceinline__ void rotate(Small& r)
    {
#pragma unroll
        for (int i = 0; i < 6; i++) { sc[i] = sc[i + 2]; r.h2.v[i] = r.h2.v[i + 2]; r.sm.v[i] = r.sm.v[i + 2]; }
    }
};

// Q8_0 / Q4_0 / IQ4_XS / IQ3_S: one fp16 scale per sub-block, the chunk may be ragged
// (in_dim is only a multiple of 32): sub-blocks past the end are clamped and
// their scale is forced to zero.
template <int FMT> struct MmqChunkD16 : MmqChunkBase<FMT, MmqChunk<FMT>> {
    static constexpr bool kTwoScales = false, kHasMin = false;
    struct Small { uint16_t d[4]; };
    struct Raw { uint4 q[8]; Small sm; };
    float sc[4];
    static __device__ __forceinline__ const uint4* plane(const Fmt<FMT>& f, unsigned h)
    {
        if constexpr (FMT == REIN_Q8_0) return h ? f.hip_ : f.lop;      // this lane's 16 quants are one plane entry
        else return f.nib;
    }
    static __device__ __forceinline__ void fetch_small(Small& r, const Fmt<FMT>& f, unsigned row, unsigned sb0, unsigned n_sub, unsigned h)
    {
#pragma unroll
        for (int p = 0; p < 4; p++) r.d[p] = f.dp[(size_t)row * f.nsp + rein_clamp_sb(sb0 + 2 * p + h, n_sub)];
    }
    static __device__ __forceinline__ void fetch(Raw& r, const Fmt<FMT>& f, unsigned row, unsigned sb0, unsigned n_sub, unsigned h)
    {
        const uint4* pl = plane(f, h);
#pragma unroll
        for (int s = 0; s < 8; s++) r.q[s] = pl[(size_t)row * f.nsp + rein_clamp_sb(sb0 + s, n_sub)];
        fetch_small(r.sm, f, row, sb0, n_sub, h);
    }
    __device__ __forceinline__ void prepare(const Small& r, unsigned sb0, unsigned n_sub, unsigned h)
    {
#pragma unroll
        for (int p = 0; p < 4; p++) sc[p] = sb0 + 2 * p + h < n_sub ? rein_h2f(r.d[p]) : 0.0f;
    }
    static __device__ __forceinline__ rein_v4i operand(const uint4& q, const Small&, int, unsigned h)
    {
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        rein_v4i o;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if constexpr (FMT == REIN_Q8_0) o[j] = (int)w[j];
            else if constexpr (FMT == REIN_Q4_0) o[j] = rein_sub_bytes((w[j] >> (4 * h)) & 0x0F0F0F0Fu, 0x08080808u);
            else o[j] = rein_codebook4<FMT>(w[j], 4 * h);
        }
        return o;
    }
    __device__ __forceinline__ void rotate(Small&) { sc[0] = sc[1]; sc[1] = sc[2]; sc[2] = sc[3]; }
};
template <> struct MmqChunk<REIN_Q8_0> : MmqChunkD16<REIN_Q8_0> {};
template <> struct MmqChunk<REIN_Q4_0> : MmqChunkD16<REIN_Q4_0> {};
template <> struct MmqChunk<REIN_IQ4_XS> : MmqChunkD16<REIN_IQ4_XS> {};
template <> struct MmqChunk<REIN_IQ3_S> : MmqChunkD16<REIN_IQ3_S> {};

// LDS image of one activation chunk: TM tokens x 8 sub-blocks.  xsb holds each
// block's xsum split into three bf16 (truncated head, then the exact remainders),
// which together carry all 24 significand bits: the -dmin*m*xsum term of
// Q4_K/Q5_K is then one superblock-wide bf16 MFMA against the integer mins with
// exact products and fp32 accumulation.
template <int TM>
struct MmqLds {
    static constexpr int kPlane = TM + 1;                 // +1 entry: sub-block planes land on different banks
    uint4 qs[2][8][kPlane];                               // [half][sub-block][token]
    float dx[8][kPlane];
    uint16_t xsb[3][TM][8];                               // [split][token][sub-block]
};

__device__ __forceinline__ void rein_mmq_split_xsum(float xs, uint16_t out[3])
{
    const uint32_t b0 = __builtin_bit_cast(uint32_t, xs) & 0xFFFF0000u;
    const float r1 = xs - __builtin_bit_cast(float, b0);
    const uint32_t b1 = __builtin_bit_cast(uint32_t, r1) & 0xFFFF0000u;
    const float r2 = r1 - __builtin_bit_cast(float, b1);
    out[0] = (uint16_t)(b0 >> 16);
    out[1] = (uint16_t)(b1 >> 16);
    out[2] = (uint16_t)(__builtin_bit_cast(uint32_t, r2) >> 16);
}

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
        uint16_t sp[3];
        rein_mmq_split_xsum(ok ? xs : 0.0f, sp);
        l.xsb[0][tl][s] = sp[0];
        l.xsb[1][tl][s] = sp[1];
        l.xsb[2][tl][s] = sp[2];
    }
}

// Multiply one staged chunk (8 sub-blocks) into the accumulators of this
// wavefront's TM/32 tiles.  DOTS != 0: store the raw int32 block dots instead.
template <int FMT, int TM, int DOTS, class BSrc>
__device__ __forceinline__ void rein_mmq_chunk_math(const MmqLds<TM>& lds, const MmqChunk<FMT>& ck, const BSrc& bsrc,
                                                    rein_v16f (&acc)[TM / 32], unsigned j, unsigned h,
                                                    int* __restrict__ dots, unsigned row, unsigned out_dim,
                                                    unsigned tok_base, unsigned tok_end, unsigned sb0, unsigned n_sub)
{
    using C = MmqChunk<FMT>;
    constexpr int NT = TM / 32;
    rein_v16i cinit;
#pragma unroll
    for (int v = 0; v < 16; v++) cinit[v] = DOTS ? 0 : REIN_MMQ_MAGIC_I;
    rein_v32f z32;
#pragma unroll
    for (int v = 0; v < 32; v++) z32[v] = 0.0f;

    if constexpr (C::kTwoScales) {
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const rein_v4i bs = bsrc(s);
            rein_v4i blo, bhi;
#pragma unroll
            for (int k = 0; k < 4; k++) { blo[k] = h ? 0 : bs[k]; bhi[k] = h ? bs[k] : 0; }
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 a4 = lds.qs[h][s][t * 32 + j];
                rein_v4i a;
                a[0] = (int)a4.x; a[1] = (int)a4.y; a[2] = (int)a4.z; a[3] = (int)a4.w;
                const rein_v16i clo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, blo, cinit, 0, 0, 0);
                const rein_v16i chi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bhi, cinit, 0, 0, 0);
                if constexpr (DOTS != 0) {
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
                    // block 0 (lanes 0-31 of both operands): dx * dsc_lo, block 1: dx * dsc_hi
                    const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(lds.dx[s][t * 32 + j], ck.sc[s], z32, 0, 0, 0);
                    const rein_v16f flo = rein_mmq_unbias(clo), fhi = rein_mmq_unbias(chi);
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        acc[t][v] = fmaf(flo[v], sx[v], acc[t][v]);
                        acc[t][v] = fmaf(fhi[v], sx[16 + v], acc[t][v]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const rein_v4i b0 = bsrc(2 * p), b1 = bsrc(2 * p + 1);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 a40 = lds.qs[h][2 * p][t * 32 + j];
                const uint4 a41 = lds.qs[h][2 * p + 1][t * 32 + j];
                rein_v4i a0, a1;
                a0[0] = (int)a40.x; a0[1] = (int)a40.y; a0[2] = (int)a40.z; a0[3] = (int)a40.w;
                a1[0] = (int)a41.x; a1[1] = (int)a41.y; a1[2] = (int)a41.z; a1[3] = (int)a41.w;
                const rein_v16i c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b0, cinit, 0, 0, 0);
                const rein_v16i c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b1, cinit, 0, 0, 0);
                if constexpr (DOTS != 0) {
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
                    // lane half h feeds sub-block 2p+h: block 0 = sub-block 2p, block 1 = 2p+1
                    const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(lds.dx[2 * p + h][t * 32 + j], ck.sc[p], z32, 0, 0, 0);
                    const rein_v16f f0 = rein_mmq_unbias(c0), f1 = rein_mmq_unbias(c1);
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        acc[t][v] = fmaf(f0[v], sx[v], acc[t][v]);
                        acc[t][v] = fmaf(f1[v], sx[16 + v], acc[t][v]);
                    }
                }
            }
            // keep the pairs apart: interleaving them buys nothing (MFMA and VALU of
            // a SIMD do not overlap) and costs a second set of 96 live registers
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (C::kHasMin && DOTS == 0) {
            static_assert(!C::kMinSplit, "split minimums are handled by the pipelined tile only");
            // sum over the 8 sub-blocks of m * xsum: lane half 0 carries the heads of
            // the xsum splits, half 1 the first remainders, a second MFMA the last
            // remainders (its half 1 multiplies zeros)
            const uint4 z4 = make_uint4(0u, 0u, 0u, 0u);
            const rein_v8bf mb2 = h ? __builtin_bit_cast(rein_v8bf, z4) : ck.mb;
            rein_v16f z16;
#pragma unroll
            for (int v = 0; v < 16; v++) z16[v] = 0.0f;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 x01 = *reinterpret_cast<const uint4*>(lds.xsb[h][t * 32 + j]);
                const uint4 x2  = *reinterpret_cast<const uint4*>(lds.xsb[2][t * 32 + j]);
                rein_v16f m = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rein_v8bf, x01), ck.mb, z16, 0, 0, 0);
                m = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rein_v8bf, x2), mb2, m, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][v] = fmaf(m[v], ck.ndmin, acc[t][v]);
            }
        }
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
        rein_mmq_chunk_math<FMT, TM, DOTS>(lds, ck, [&](int s) { return ck.b[s]; }, acc, j, h, dots, row, out_dim,
                                           tok_base, tok_end, sb0, n_sub);
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
//   * the 16-byte weight plane travels HBM -> LDS directly
//     (global_load_lds_dwordx4, no registers), each wavefront into its own ring
//     of two half-chunk slots, so it needs no barrier; a slot is refilled with
//     the next chunk's half as soon as it has been read;
//   * the next chunk's small weight words and activation blocks are fetched into
//     registers before the current chunk is multiplied, the activation LDS image
//     is double-buffered, and there is one barrier per chunk;
//   * a fixed workgroup of 4 wavefronts (128 rows x TM tokens);
//   * a 1-D grid whose workgroup -> tile map keeps all token tiles of one
//     128-row weight block on the same XCD (workgroups are dealt round-robin
//     over the 8 XCDs, each with its own L2), so a weight block is pulled from
//     HBM once and re-read from that L2.
// Grid: 8 * ceil(n_row_blocks / 8) * n_token_tiles workgroups of 256 threads.
struct __attribute__((packed, aligned(8))) ReinQ8Words { uint32_t v[4]; };   // 16 bytes at 8-byte alignment

template <int TM>
struct MmqXRegs {
    static constexpr int kPer = TM * 8 / 256;            // activation blocks per thread per chunk
    uint2 hdr[kPer];                                     // d, xsum
    rein_v4i lo[kPer], hi[kPer];                         // quants 0..15, 16..31: the two 16-byte loads
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
        const char* p = reinterpret_cast<const char*>(
            xq + (size_t)(tok < tok_end ? tok : tok_end - 1) * n_sub + (sb < n_sub ? sb : n_sub - 1));
        const ReinQ8Words lo = *reinterpret_cast<const ReinQ8Words*>(p + 8), hi = *reinterpret_cast<const ReinQ8Words*>(p + 24);
#pragma unroll
        for (int i = 0; i < 4; i++) { r.lo[k][i] = (int)lo.v[i]; r.hi[k][i] = (int)hi.v[i]; }
        // keeps the header out of the two 16-byte loads above (merged with it they would be
        // cut at offsets 0 / 16 / 32 and the quads would have to be reassembled)
        asm volatile("" ::: "memory");
        r.hdr[k] = *reinterpret_cast<const uint2*>(p);
    }
}

// rows past tok_end / sub-blocks past n_sub get zero scales here; dx is staged times 2^26
// (see rein_mmq_dot_tile).  Lane half 0 / 1 of the math reads quants 0..15 / 16..31, or
// {0..7, 16..23} / {8..15, 24..31} when the format splits the contraction that way
// (MmqChunkBase::kSplitK).
template <int TM, bool SPLITK>
__device__ __forceinline__ void rein_mmq_xstore(MmqLds<TM>& l, MmqXRegs<TM>& r, unsigned n_sub,
                                                unsigned tok_base, unsigned tok_end, unsigned sb0)
{
#pragma unroll
    for (int k = 0; k < MmqXRegs<TM>::kPer; k++) {
        const unsigned e = threadIdx.x + k * 256;
        const unsigned tl = e >> 3, s = e & 7;
        const bool ok = tok_base + tl < tok_end && sb0 + s < n_sub;
        if constexpr (SPLITK) {
            // Pin the two quads as loaded: the regrouping then happens here, on values that
            // arrived a chunk ago, and the next fetch lands in these registers directly.
            // Left to itself the compiler keeps the store grouping across the loop and
            // regroups right behind the loads, which waits for them in mid-chunk.
            asm volatile("" : "+v"(r.lo[k]), "+v"(r.hi[k]));
            l.qs[0][s][tl] = make_uint4((unsigned)r.lo[k][0], (unsigned)r.lo[k][1], (unsigned)r.hi[k][0], (unsigned)r.hi[k][1]);
            l.qs[1][s][tl] = make_uint4((unsigned)r.lo[k][2], (unsigned)r.lo[k][3], (unsigned)r.hi[k][2], (unsigned)r.hi[k][3]);
        } else {
            l.qs[0][s][tl] = __builtin_bit_cast(uint4, r.lo[k]);
            l.qs[1][s][tl] = __builtin_bit_cast(uint4, r.hi[k]);
        }
        l.dx[s][tl]    = ok ? __builtin_bit_cast(float, r.hdr[k].x) * REIN_MMQ_XSCALE : 0.0f;
        uint16_t sp[3];
        rein_mmq_split_xsum(ok ? __builtin_bit_cast(float, r.hdr[k].y) : 0.0f, sp);
        l.xsb[0][tl][s] = sp[0];
        l.xsb[1][tl][s] = sp[1];
        l.xsb[2][tl][s] = sp[2];
    }
}

// One wavefront's LDS ring for the 16-byte weight plane(s): two slots of half a
// chunk (32 rows x 4 sub-blocks, 2 KiB) each.  Slot entry of (row n, sub-block
// s4 of the half) is 4n + ((s4 + n/2) & 3), which spreads the 32 rows of a
// ds_read_b128 over all banks.  Q8_0 has one plane per lane half.
template <int FMT>
struct MmqWLds {
    static constexpr int kPlanes = FMT == REIN_Q8_0 ? 2 : 1;
    uint4 q[kPlanes][2][128];
};

// One 16-byte-per-lane HBM -> LDS transfer: lane l's bytes land at lds_base + 16 l
// (lds_base wave-uniform, passed in M0).  Written as inline assembly on purpose:
// through the builtin the compiler treats every later LDS read as a possible reader
// of the transfer and waits for it on the spot (s_waitcnt vmcnt(0)), which turns the
// prefetch into a blocking load.  Here the waits are placed by hand with
// REIN_WAIT_VMCNT.  The compiler's own vmcnt waits stay correct: requests complete in
// order and it can only under-count the younger ones, i.e. wait for more.
__device__ __forceinline__ void rein_lds_dma16(const void* gptr, unsigned lds_base)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_base)
                 : "memory", "m0");
}

// The same with the address as scalar base + 32-bit lane offset: the per-transfer address
// arithmetic of the tuned kernel then runs on the scalar unit.
__device__ __forceinline__ void rein_lds_dma16_s(unsigned voff, const void* sbase, unsigned lds_base)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(sbase), "s"(lds_base)
                 : "memory", "m0");
}

// Where a wavefront's ring transfers come from and go to.  row_off[k]: byte offset of lane
// l's row in transfer k (row 16k + l/4 of the wavefront's 32, clamped to the matrix)
// relative to the wavefront's first row; s4: which of the half chunk's four sub-blocks the
// lane fetches (four lanes walk a row's 64 contiguous bytes; the rotation by row / 2 is the
// ring's bank swizzle); lds: LDS address of the wavefront's ring.  K-quant rows hold whole
// chunks, so the lane offset is constant and only the scalar base moves; the 32-weight
// formats clamp the sub-block to the row (ragged last chunk).
template <int FMT>
struct MmqWSrc {
    static constexpr bool kRagged = !(FMT == REIN_Q4_K || FMT == REIN_Q5_K || FMT == REIN_Q6_K);
    unsigned row_off[2], s4[2], lds;
    size_t wave_off;                               // byte offset of the wavefront's first row in a plane
    __device__ __forceinline__ void init(const MmqWLds<FMT>& ring, const Fmt<FMT>& fmt, unsigned row_base, unsigned out_dim,
                                         unsigned lane)
    {
        typedef __attribute__((address_space(3))) const void* lptr_t;
        lds = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)&ring);
        // a wavefront whose rows all lie past the matrix reads the last row (and stores nothing)
        const unsigned first = min(row_base, out_dim - 1u);
        wave_off = (size_t)first * fmt.nsp * 16u;
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const unsigned n = 16u * k + (lane >> 2);
            s4[k] = ((lane & 3u) - (n >> 1)) & 3u;
            const unsigned nrow = min(row_base + n, out_dim - 1u) - first;
            row_off[k] = nrow * fmt.nsp * 16u + (kRagged ? 0u : s4[k] * 16u);
        }
    }
};

// HBM -> LDS, asynchronous (counted by vmcnt), sub-blocks sb_first .. sb_first+3 of
// the wavefront's 32 rows into slot `half`.  2 * kPlanes transfers.
template <int FMT>
__device__ __forceinline__ void rein_mmq_wload(const MmqWSrc<FMT>& src, unsigned half, const Fmt<FMT>& fmt,
                                               unsigned sb_first, unsigned n_sub)
{
#pragma unroll
    for (int pl = 0; pl < MmqWLds<FMT>::kPlanes; pl++) {
        const char* plane = reinterpret_cast<const char*>(MmqChunk<FMT>::plane(fmt, (unsigned)pl));
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const unsigned lds_base = src.lds + (((unsigned)pl * 2u + half) * 128u + 64u * k) * 16u;
            if constexpr (MmqWSrc<FMT>::kRagged) {
                const unsigned sb = rein_clamp_sb(sb_first + src.s4[k], n_sub);
                rein_lds_dma16_s(src.row_off[k] + sb * 16u, plane + src.wave_off, lds_base);
            } else {
                rein_lds_dma16_s(src.row_off[k], plane + src.wave_off + (size_t)sb_first * 16u, lds_base);
            }
        }
    }
}

// s_waitcnt vmcnt(N) with the other counters left alone (gfx9 encoding)
#define REIN_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(0x0F70 | ((N) & 15) | (((N) >> 4) << 14))

// int8 MFMA operand of token `tok`, sub-block `blk` for lane half h (the 16 quants staged
// for that half by rein_mmq_xstore)
template <int TM>
__device__ __forceinline__ rein_v4i rein_mmq_act_operand(const MmqLds<TM>& lds, unsigned h, unsigned blk, unsigned tok)
{
    const uint4 a4 = lds.qs[h][blk][tok];
    rein_v4i a;
    a[0] = (int)a4.x; a[1] = (int)a4.y; a[2] = (int)a4.z; a[3] = (int)a4.w;
    return a;
}

// The chunk math of the tuned kernel: one rolled iteration per sub-block pair so
// that only one pair's tiles (two int32 dot tiles, one 2-block scale tile) are
// live at a time.  Pairs 0,1 read ring slot 0 and pairs 2,3 slot 1; as soon as a
// slot has been read, the same half of the NEXT chunk is requested into it
// (`more`), so a weight request is in flight for about three quarters of a chunk.
// `refill(half)` is the caller's: it issues the loads (see rein_mmq_pipelined for the
// order that keeps every wait off the freshest requests).
// `ck` and `sm` are private copies; they are rotated so the loop indexes entries
// 0 and 1.
template <int FMT, int TM, class Refill, class Prefetch>
__device__ __forceinline__ void rein_mmq_chunk_math_rolled(const MmqLds<TM>& lds, MmqWLds<FMT>& wl, unsigned wsel,
                                                           MmqChunk<FMT> ck, typename MmqChunk<FMT>::Small sm,
                                                           rein_v16f (&acc)[TM / 32], unsigned j, unsigned h,
                                                           bool more, const Refill& refill, const Prefetch& prefetch)
{
    using C = MmqChunk<FMT>;
    constexpr int NT = TM / 32;
    constexpr int kDma = 2 * MmqWLds<FMT>::kPlanes;
    rein_v32f z32;
#pragma unroll
    for (int v = 0; v < 32; v++) z32[v] = 0.0f;
    const unsigned rot = j >> 1;
    rein_v4i zlo[2], zhi[2];
    if constexpr (C::kTwoScales) {
        // opaque zeros: otherwise the compiler rebuilds the half-zero operands from
        // constants for every MFMA
#pragma unroll
        for (int s = 0; s < 2; s++) {
            zlo[s] = rein_v4i{0, 0, 0, 0};
            zhi[s] = rein_v4i{0, 0, 0, 0};
            asm volatile("" : "+v"(zlo[s]), "+v"(zhi[s]));
        }
    }

    // two pairs per trip at 32 tokens (the ring addresses of a slot become four adds and
    // the branches on the pair's parity go); at 64 tokens that would spill
    constexpr int kPairUnroll = (NT == 1 && !C::kTwoScales) ? 2 : 1;
#pragma unroll kPairUnroll
    for (unsigned p = 0; p < 4; p++) {
        if (p == 2) {
            // slot 1 of this chunk: only the refill of slot 0 (if any) is younger
            if (more) REIN_WAIT_VMCNT(kDma); else REIN_WAIT_VMCNT(0);
            // the next activation blocks are requested here, behind the wait, so that it
            // does not wait for them: they have until the end of the chunk
            __builtin_amdgcn_sched_barrier(0);
            if (more) prefetch();
        }
        const uint4* slot = wl.q[wsel][p >> 1];
        const unsigned s4 = 2u * (p & 1u);
        const rein_v4i b0 = C::operand_at(&slot[4u * j + ((s4 + rot) & 3u)], sm, 0, h);
        const rein_v4i b1 = C::operand_at(&slot[4u * j + ((s4 + 1u + rot) & 3u)], sm, 1, h);
        if (more && (p & 1u)) {
            // both pairs of the slot are in registers: refill it.  The LDS reads above
            // must have returned before the DMA may overwrite the slot.
            __builtin_amdgcn_s_waitcnt(0xC07F);                    // lgkmcnt(0)
            refill(p >> 1);
        }
        if constexpr (C::kTwoScales) {
            rein_v16i zi;
#pragma unroll
            for (int v = 0; v < 16; v++) zi[v] = 0;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(lds.dx[2 * p + h][t * 32 + j], ck.dq, z32, 0, 0, 0);
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    const rein_v4i bs = s ? b1 : b0;
                    // the zero halves of the two operands live in the same registers all along
                    zlo[s][0] = bs[0]; zlo[s][1] = bs[1];
                    zhi[s][2] = bs[2]; zhi[s][3] = bs[3];
                    const rein_v4i a = rein_mmq_act_operand(lds, h, 2 * p + s, t * 32 + j);
                    const rein_v16i ilo = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, zlo[s], zi, 0, 0, 0);
                    const rein_v16i ihi = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, zhi[s], zi, 0, 0, 0);
                    const int sl = C::group_scale(sm, s, 0), sh = C::group_scale(sm, s, 1);
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int both = __mul24(ilo[v], sl) + __mul24(ihi[v], sh);
                        acc[t][v] = fmaf((float)both, sx[16 * s + v], acc[t][v]);
                    }
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const rein_v4i a0 = rein_mmq_act_operand(lds, h, 2 * p, t * 32 + j);
                const rein_v4i a1 = rein_mmq_act_operand(lds, h, 2 * p + 1, t * 32 + j);
                const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(lds.dx[2 * p + h][t * 32 + j], ck.sc[0], z32, 0, 0, 0);
                const rein_v16f f0 = rein_mmq_dot_tile<NT == 2>(a0, b0);
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][v] = fmaf(f0[v], sx[v], acc[t][v]);
                const rein_v16f f1 = rein_mmq_dot_tile<NT == 2>(a1, b1);
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][v] = fmaf(f1[v], sx[16 + v], acc[t][v]);
            }
        }
        ck.rotate(sm);
    }
    if constexpr (C::kHasMin) {
        rein_v16f z16;
#pragma unroll
        for (int v = 0; v < 16; v++) z16[v] = 0.0f;
        if constexpr (C::kMinSplit) {
            // fp16 minimums as head + remainder: six (xsum split, minimum part) products
            // of eight sub-blocks each, two per MFMA (one per lane half)
            const rein_v8bf b_mid = h ? ck.mb_lo : ck.mb;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 x0 = *reinterpret_cast<const uint4*>(lds.xsb[0][t * 32 + j]);
                const uint4 x1 = *reinterpret_cast<const uint4*>(lds.xsb[1][t * 32 + j]);
                const uint4 x2 = *reinterpret_cast<const uint4*>(lds.xsb[2][t * 32 + j]);
                const uint4 a1 = h ? x1 : x0, a2 = h ? x0 : x2, a3 = h ? x2 : x1;
                rein_v16f m = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rein_v8bf, a1), ck.mb, z16, 0, 0, 0);
                m = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rein_v8bf, a2), b_mid, m, 0, 0, 0);
                m = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rein_v8bf, a3), ck.mb_lo, m, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][v] = fmaf(m[v], ck.ndmin, acc[t][v]);
            }
        } else {
            const uint4 z4 = make_uint4(0u, 0u, 0u, 0u);
            const rein_v8bf mb2 = h ? __builtin_bit_cast(rein_v8bf, z4) : ck.mb;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const uint4 x01 = *reinterpret_cast<const uint4*>(lds.xsb[h][t * 32 + j]);
                const uint4 x2  = *reinterpret_cast<const uint4*>(lds.xsb[2][t * 32 + j]);
                rein_v16f m = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rein_v8bf, x01), ck.mb, z16, 0, 0, 0);
                m = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rein_v8bf, x2), mb2, m, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][v] = fmaf(m[v], ck.ndmin, acc[t][v]);
            }
        }
    }
}

// One workgroup tile of the tuned kernel: 256 threads, rows 128*rb .., tokens
// tok_base .. tok_end (at most TM) of xq / y.  Ends on a barrier, so a workgroup may
// run several tiles in a row.
// LDS of one tile: two activation images and the four wavefronts' weight rings.  The
// buffer is one variable per size, so a kernel that runs tiles of both token counts
// (LDSB = the larger size for both) holds one buffer, not two.
template <int FMT, int TM>
constexpr int rein_mmq_tile_lds_bytes() { return 2 * (int)sizeof(MmqLds<TM>) + 4 * (int)sizeof(MmqWLds<FMT>); }

template <int BYTES>
__device__ __forceinline__ unsigned char* rein_mmq_tile_lds()
{
    __shared__ __attribute__((aligned(16))) unsigned char raw[BYTES];
    return raw;
}

// The contraction of one workgroup tile: wavefront `wave` accumulates tokens tok_base ..
// tok_end (at most TM) against the 32 weight rows from `row_base` of the matrix at `w`
// (both may differ from wavefront to wavefront, but are uniform within one).  Ends on a
// barrier: the tile's LDS is free again when it returns.  sb_begin / sb_stop (multiples of 8;
// sb_stop = 0: the end) restrict the sum to the sub-blocks [sb_begin, sb_stop) of the contraction.
template <int FMT, int TM, int LDSB = rein_mmq_tile_lds_bytes<FMT, TM>()>
__device__ __forceinline__ void rein_mmq_pipelined_acc(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                       unsigned in_dim, unsigned out_dim, unsigned row_base,
                                                       unsigned tok_base, unsigned tok_end, rein_v16f (&acc)[TM / 32],
                                                       unsigned sb_begin = 0u, unsigned sb_stop = 0u)
{
    using F = Fmt<FMT>;
    using C = MmqChunk<FMT>;
    constexpr int NT = TM / 32;
    constexpr int kDma = 2 * MmqWLds<FMT>::kPlanes;
    static_assert(LDSB >= rein_mmq_tile_lds_bytes<FMT, TM>(), "tile LDS buffer too small");
    static_assert(sizeof(MmqLds<TM>) % 16 == 0, "weight rings must stay 16-byte aligned");
    unsigned char* const raw = rein_mmq_tile_lds<LDSB>();
    MmqLds<TM>* const lds = reinterpret_cast<MmqLds<TM>*>(raw);
    MmqWLds<FMT>* const wlds = reinterpret_cast<MmqWLds<FMT>*>(raw + 2 * sizeof(MmqLds<TM>));

    const unsigned lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned j = lane & 31u, h = lane >> 5;
    const unsigned n_sub = in_dim >> 5;
    const F fmt(w, n_sub, out_dim);
    const unsigned row = row_base + j;
    const unsigned rowc = row < out_dim ? row : out_dim - 1;
    const unsigned wsel = FMT == REIN_Q8_0 ? h : 0u;
    MmqWLds<FMT>& wl = wlds[wave];
    MmqWSrc<FMT> wsrc;
    wsrc.init(wl, fmt, row_base, out_dim, lane);

#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.0f;

    // Request order per chunk c.  Requests complete in order and vmcnt counts those in
    // flight.  The ring DMA is invisible to the compiler's own bookkeeping, so its waits
    // for the register loads can only be stronger than it thinks; the hand-placed waits
    // only ever count ring requests, never the compiler's (whose number of instructions
    // is its own business):
    //   top of c        small words of c+1                                  (registers)
    //   after pair 1    activation image of c+1 -> LDS (blocks fetched during c-1), then ring
    //                   slot 0 <- c+1
    //   before pair 2   wait until only the slot 0 refill is in flight (slot 1 of c is in);
    //                   behind the wait, activation blocks of c+2 (registers): they have until
    //                   the end of the chunk and the wait does not include them
    //   after pair 3    ring slot 1 <- c+1
    //   end of c        wait until only the slot 1 refill is in flight (slot 0 of c+1 is
    //                   in), barrier
    // Fill: the ring requests go first, so that one memory latency covers them and the first
    // activation blocks together: the store of those blocks waits for them, and by then the
    // older ring requests have landed too (requests complete in order); the explicit wait
    // behind the store costs nothing in that case and holds if the compiler moved a load.
    typename C::Small small;
    MmqXRegs<TM> xr;
    const unsigned sb_end = sb_stop ? min(sb_stop, n_sub) : n_sub;
    rein_mmq_wload<FMT>(wsrc, 0, fmt, sb_begin, n_sub);
    rein_mmq_wload<FMT>(wsrc, 1, fmt, sb_begin + 4u, n_sub);
    C::fetch_small(small, fmt, rowc, sb_begin, n_sub, h);
    rein_mmq_xfetch<TM>(xr, xq, n_sub, tok_base, tok_end, sb_begin);
    rein_mmq_xstore<TM, C::kSplitK>(lds[0], xr, n_sub, tok_base, tok_end, sb_begin);
    REIN_WAIT_VMCNT(0);                              // both slots of the first chunk have landed
    __builtin_amdgcn_sched_barrier(0);               // the next fetch reuses the registers just stored
    rein_mmq_xfetch<TM>(xr, xq, n_sub, tok_base, tok_end, sb_begin + 8u < sb_end ? sb_begin + 8u : sb_begin);
    __syncthreads();

    unsigned buf = 0;
    for (unsigned sb0 = sb_begin; sb0 < sb_end; sb0 += 8, buf ^= 1u) {
        C ck;
        ck.prepare_tuned(small, sb0, n_sub, h);
        const typename C::Small cur = small;
        const bool more = sb0 + 8 < sb_end, more2 = sb0 + 16 < sb_end;
        if (more) C::fetch_small(small, fmt, rowc, sb0 + 8, n_sub, h);
        MmqLds<TM>& nxt = lds[buf ^ 1u];
        rein_mmq_chunk_math_rolled<FMT, TM>(lds[buf], wl, wsel, ck, cur, acc, j, h, more, [&](unsigned half) {
            if (half == 0) {
                rein_mmq_xstore<TM, C::kSplitK>(nxt, xr, n_sub, tok_base, tok_end, sb0 + 8);
                // the next fetch (behind the wait of pair 2) lands in the registers these stores
                // have read; the fence keeps the compiler from issuing it up here into others
                __builtin_amdgcn_sched_barrier(0);
            }
            rein_mmq_wload<FMT>(wsrc, half, fmt, sb0 + 8 + 4 * half, n_sub);
        }, [&]() {
            // past the last chunk the fetch repeats on clamped addresses and is never stored
            rein_mmq_xfetch<TM>(xr, xq, n_sub, tok_base, tok_end, more2 ? sb0 + 16 : sb0 + 8);
        });
        if (more) REIN_WAIT_VMCNT(kDma);             // slot 0 of the next chunk has landed
        __syncthreads();
    }
}

template <int FMT, int TM, int LDSB = rein_mmq_tile_lds_bytes<FMT, TM>()>
__device__ __forceinline__ void rein_mmq_pipelined_tile(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                        float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                        unsigned rb, unsigned tok_base, unsigned tok_end)
{
    constexpr int NT = TM / 32;
    const unsigned lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned j = lane & 31u, h = lane >> 5;
    const unsigned row = rb * 128u + wave * 32u + j;
    rein_v16f acc[NT];
    rein_mmq_pipelined_acc<FMT, TM, LDSB>(w, xq, in_dim, out_dim, rb * 128u + wave * 32u, tok_base, tok_end, acc);
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const unsigned tok = tok_base + t * 32 + 8 * (v / 4) + 4 * h + (v % 4);
            if (tok < tok_end && row < out_dim) y[(size_t)tok * out_dim + row] = acc[t][v];
        }
}

template <int FMT, int TM>
__device__ __forceinline__ void rein_mmq_pipelined(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                   float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                   unsigned p_rows)
{
    // workgroup -> (row block, token tile), XCD-aware
    const unsigned n_rb = (out_dim + 127u) / 128u;
    const unsigned n_tt = (p_rows + TM - 1) / TM;
    const unsigned xcd = blockIdx.x & 7u, k = blockIdx.x >> 3;
    const unsigned rb = (k / n_tt) * 8u + xcd, tt = k % n_tt;
    if (rb >= n_rb) return;
    rein_mmq_pipelined_tile<FMT, TM>(w, xq, y, in_dim, out_dim, rb, tt * TM, min(p_rows, tt * TM + TM));
}

// The same with token tiles of two sizes in one launch: per row block the first n64
// tiles take 64 tokens, the rest of the tokens goes in 32-token tiles.  The 64-token tile
// costs less per token (one weight unpack feeds two MFMA tiles) but its coarser grain
// leaves the last round of workgroups badly filled at a few hundred tokens; launched
// first, with the small tiles behind them as fillers, the machine drains evenly.  The
// host picks n64.  Workgroup -> tile keeps one weight block on one XCD, as above.
template <int FMT>
__device__ __forceinline__ void rein_mmq_pipelined_mixed(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                         float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                         unsigned p_rows, unsigned n64)
{
    constexpr int kLds = rein_mmq_tile_lds_bytes<FMT, 64>();
    const unsigned n_rb = (out_dim + 127u) / 128u, n_rbg = (n_rb + 7u) / 8u;
    const unsigned tok64 = min(p_rows, n64 * 64u);
    const unsigned n32 = (p_rows - tok64 + 31u) / 32u;
    const unsigned xcd = blockIdx.x & 7u;
    unsigned k = blockIdx.x >> 3;
    if (k < n_rbg * n64) {
        const unsigned rb = (k / n64) * 8u + xcd, tt = k % n64;
        if (rb >= n_rb || tt * 64u >= tok64) return;
        rein_mmq_pipelined_tile<FMT, 64, kLds>(w, xq, y, in_dim, out_dim, rb, tt * 64u, min(tok64, tt * 64u + 64u));
        return;
    }
    k -= n_rbg * n64;
    if (n32 == 0u) return;
    const unsigned rb = (k / n32) * 8u + xcd, tt = k % n32;
    if (rb >= n_rb) return;
    const unsigned t0 = tok64 + tt * 32u;
    rein_mmq_pipelined_tile<FMT, 32, kLds>(w, xq, y, in_dim, out_dim, rb, t0, min(p_rows, t0 + 32u));
}

// Split-tail launch of the tuned tile: the grid IS the resident slots (gridDim.x = G
// workgroups, a multiple of 8, two per CU).  Units -- unit u = (row block u / n_tg, TM-token
// group u % n_tg) -- are dealt in rounds: in round r workgroup `pos` computes unit r G + pos
// whole.  The U mod G units left after the whole rounds are split along the contraction, `split`
// workgroups per unit, each a contiguous range of 256-weight chunks, all at the same time; range
// k of tail unit t stores its partial tile to slot t * split + k of `part`
// ([tile][register][thread], TM / 32 x 16 x 256 floats), and rein_mmq_tail_sum_body, launched behind
// this kernel, adds the partial tiles of every tail unit in range order (a fixed order:
// reproducible).  pos = (blockIdx.x % 8) * G / 8 + blockIdx.x / 8: the workgroups of one XCD
// hold neighbouring units, so the token groups of a row block -- and the ranges of a tail unit
// -- meet in one L2 at the same time.
template <int FMT, int TM>
__device__ __forceinline__ void rein_mmq_split_tail(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                    float* __restrict__ y, float* __restrict__ part,
                                                    unsigned in_dim, unsigned out_dim, unsigned p_rows, unsigned split)
{
    constexpr int NT = TM / 32;
    constexpr unsigned kPart = (unsigned)NT * 16u * 256u;                // floats per partial tile
    const unsigned n_rb = (out_dim + 127u) / 128u, n_tg = (p_rows + TM - 1u) / TM;
    const unsigned n_chunk = ((in_dim >> 5) + 7u) >> 3, g = gridDim.x, n_unit = n_rb * n_tg;
    const unsigned pos = (blockIdx.x & 7u) * (g >> 3) + (blockIdx.x >> 3);
    const unsigned rounds = n_unit / g, n_tail = n_unit - rounds * g;
    if (blockDim.x != 256u) return;

    // the tail's ranges are dealt evenly over the XCDs, each XCD a contiguous run of them
    const unsigned n_seg = n_tail * split, per_xcd = (n_seg + 7u) >> 3;
    const unsigned seg = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    const unsigned lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned j = lane & 31u, h = lane >> 5;

    for (unsigned r = 0; r <= rounds; r++) {                             // whole units, then this workgroup's tail range
        unsigned u = r * g + pos, c0 = 0u, c1 = n_chunk;
        float* dst = nullptr;
        if (r == rounds) {
            if ((blockIdx.x >> 3) >= per_xcd || seg >= n_seg) return;
            const unsigned tu = seg / split, k = seg - tu * split;       // tail unit, range within it
            u = rounds * g + tu;
            c0 = n_chunk * k / split; c1 = n_chunk * (k + 1u) / split;
            if (c0 == c1) return;                                        // more ranges than chunks: nothing to add
            if (split > 1u) dst = part + (size_t)seg * kPart;
        }
        const unsigned rb = u / n_tg, tg = u % n_tg;
        const unsigned tok_base = tg * TM, tok_end = min(p_rows, tok_base + TM);
        const unsigned row = rb * 128u + wave * 32u + j;
        rein_v16f acc[NT];
        rein_mmq_pipelined_acc<FMT, TM>(w, xq, in_dim, out_dim, rb * 128u + wave * 32u, tok_base, tok_end, acc, c0 * 8u, c1 * 8u);
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const unsigned tok = tok_base + t * 32 + 8 * (v / 4) + 4 * h + (v % 4);
                if (dst) dst[(t * 16 + v) * 256 + threadIdx.x] = acc[t][v];
                else if (tok < tok_end && row < out_dim) y[(size_t)tok * out_dim + row] = acc[t][v];
            }
    }
}

// y of the tail units = their partial tiles added in range order.  Grid (tail units, NT, 4):
// blockIdx.y = 32-token tile of the unit's NT, blockIdx.z = register quad, 256 threads as in the
// GEMM (thread -> weight row, register -> token).  `first_unit` = the whole rounds' unit count, n_chunk = chunks of
// the contraction (an empty range stored nothing).
template <int NT>
__device__ __forceinline__ void rein_mmq_tail_sum_body(const float* __restrict__ part, float* __restrict__ y,
                                                       unsigned n_chunk, unsigned out_dim, unsigned p_rows,
                                                       unsigned first_unit, unsigned split)
{
    constexpr unsigned kPart = (unsigned)NT * 16u * 256u;
    const unsigned n_tg = (p_rows + 32u * NT - 1u) / (32u * NT);
    const unsigned tu = blockIdx.x, t = blockIdx.y, u = first_unit + tu, rb = u / n_tg, tg = u % n_tg;
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, j = lane & 31u, h = lane >> 5;
    const unsigned row = rb * 128u + wave * 32u + j;
    // blockIdx.z = which four of the sixteen registers: four times the workgroups, a quarter of the serial loads each
    const unsigned v0 = 4u * blockIdx.z;
    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 4
    for (unsigned q = 0; q < split; q++) {
        if (n_chunk * q / split == n_chunk * (q + 1u) / split) continue;
        const float* src = part + (size_t)(tu * split + q) * kPart + (t * 16u + v0) * 256u + threadIdx.x;
#pragma unroll
        for (int v = 0; v < 4; v++) sum[v] += src[v * 256];
    }
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const unsigned tok = tg * 32u * NT + t * 32u + 8u * blockIdx.z + 4u * h + v;
        if (tok < p_rows && row < out_dim) y[(size_t)tok * out_dim + row] = sum[v];
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
// rows expert_off[e] + 32*local .. of the expert-sorted xq / y.  Each tile runs
// the tuned 32-token workgroup tile; any grid is correct, the block must be 256
// threads (src/runtime/qwen35.rs:3062).
// Expert of a token tile: the largest e with tile_off[e] <= tile.  Every wavefront counts the
// entries that are <= tile with one load per lane and 64 experts (a binary search would be
// seven dependent loads deep at 128 experts, in front of every workgroup's first fetch).
__device__ __forceinline__ unsigned rein_mmq_tile_expert(const int* __restrict__ tile_off, unsigned n_expert, unsigned tile)
{
    const unsigned lane = threadIdx.x & 63u;
    unsigned n_le = 0;
    for (unsigned e0 = 0; e0 < n_expert; e0 += 64u) {
        const unsigned e = e0 + lane;
        const bool le = e < n_expert && (unsigned)tile_off[e < n_expert ? e : 0u] <= tile;
        n_le += (unsigned)__popcll(__ballot(le));
    }
    return n_le - 1u;                              // tile_off[0] = 0 <= tile: at least one
}

// The same with the expert's rows in the same round trip: every lane also loads its experts' expert_off[e],
// expert_off[e + 1] and keeps tile_off[e], and the three words of the expert found are read out of the lane
// that holds them -- one memory latency in front of a workgroup's first fetch instead of two.  Up to 256
// experts; beyond, the words are loaded once the expert is known.
struct ReinTileRows { unsigned expert, tok_base, tok_end; };
__device__ __forceinline__ ReinTileRows rein_mmq_tile_rows(const int* __restrict__ tile_off, const int* __restrict__ expert_off,
                                                           unsigned n_expert, unsigned tile)
{
    const unsigned lane = threadIdx.x & 63u;
    if (n_expert > 256u) {
        const unsigned lo = rein_mmq_tile_expert(tile_off, n_expert, tile);
        return ReinTileRows{lo, (unsigned)expert_off[lo] + (tile - (unsigned)tile_off[lo]) * 32u, (unsigned)expert_off[lo + 1]};
    }
    int to[4], e0[4], e1[4];
    unsigned n_le = 0;
#pragma unroll
    for (unsigned k = 0; k < 4u; k++) {
        const unsigned e = min(k * 64u + lane, n_expert - 1u);
        to[k] = tile_off[e]; e0[k] = expert_off[e]; e1[k] = expert_off[e + 1u];
    }
#pragma unroll
    for (unsigned k = 0; k < 4u; k++) {
        const bool le = k * 64u + lane < n_expert && (unsigned)to[k] <= tile;
        n_le += (unsigned)__popcll(__ballot(le));
    }
    const unsigned lo = n_le - 1u, src = lo & 63u;                       // tile_off[0] = 0 <= tile: at least one
    int t = 0, a = 0, b = 0;
#pragma unroll
    for (unsigned k = 0; k < 4u; k++) {
        const int tk = __builtin_amdgcn_readlane(to[k], src), ak = __builtin_amdgcn_readlane(e0[k], src), bk = __builtin_amdgcn_readlane(e1[k], src);
        if ((lo >> 6) == k) { t = tk; a = ak; b = bk; }
    }
    return ReinTileRows{lo, (unsigned)a + (tile - (unsigned)t) * 32u, (unsigned)b};
}

template <int FMT>
__device__ __forceinline__ void rein_mmq_grouped(const uint8_t* __restrict__ slab, unsigned bytes_per_expert,
                                                 const int* __restrict__ expert_off, const int* __restrict__ tile_off,
                                                 unsigned n_expert, const BlockQ8* __restrict__ xq,
                                                 float* __restrict__ y, unsigned in_dim, unsigned out_dim)
{
    if (blockDim.x != 256u) return;                // the tuned tile is built for 4 wavefronts (the reference's launch)
    const unsigned n_rb = (out_dim + 127u) / 128u;
    const unsigned n_tiles = (unsigned)tile_off[n_expert];
    for (unsigned tile = blockIdx.y; tile < n_tiles; tile += gridDim.y) {
        const unsigned e = rein_mmq_tile_expert(tile_off, n_expert, tile);
        const unsigned tok_base = (unsigned)expert_off[e] + (tile - (unsigned)tile_off[e]) * 32u;
        const unsigned tok_end = (unsigned)expert_off[e + 1];
        if (tok_base >= tok_end) continue;         // host counted tiles with a smaller bn
        for (unsigned rb = blockIdx.x; rb < n_rb; rb += gridDim.x)
            rein_mmq_pipelined_tile<FMT, 32>(slab + (size_t)e * bytes_per_expert, xq, y, in_dim, out_dim, rb,
                                             tok_base, min(tok_end, tok_base + 32u));
    }
}

// The library's own launch of the grouped GEMM: exactly one (token tile, 128-row block, slab)
// per workgroup of a 1-D grid of 8 * ceil(tile_ub / 8) * n_slab * ceil(out_dim / 128)
// workgroups (tile_ub = the host's upper bound of the tile count; surplus workgroups leave
// at once).  Workgroup i runs on XCD i % 8, and all row blocks and slabs of a token tile are
// dealt to the same XCD, so the tile's activation blocks are pulled into one L2 and re-read
// there by the others; XCD x takes the x-th eighth of the tiles, so the tiles of an expert
// meet in one L2 too.  Two slabs with their outputs let the gate and the up projection of
// an expert FFN run in one launch (twice the workgroups fill the machine better than two
// launches of half the size, and the second launch's fill / drain disappears).  Without the grid-stride loops
// of rein_mmq_grouped around it the tile keeps to the register budget of three
// wavefronts per SIMD, which is what hides the pipeline fill of the short contractions
// of expert FFNs (24 to 64 sub-blocks).
template <int FMT>
__device__ __forceinline__ void rein_mmq_grouped_one(const uint8_t* __restrict__ slab0, const uint8_t* __restrict__ slab1,
                                                     unsigned bytes_per_expert, const int* __restrict__ expert_off,
                                                     const int* __restrict__ tile_off, unsigned n_expert,
                                                     const BlockQ8* __restrict__ xq, float* __restrict__ y0,
                                                     float* __restrict__ y1, unsigned in_dim, unsigned out_dim,
                                                     unsigned n_slab)
{
    // XCD x takes the x-th eighth of the tiles that exist: neighbouring tiles -- the tiles of one
    // expert -- run on one XCD at the same time and share the expert's weights in its L2
    const unsigned n_rb = (out_dim + 127u) / 128u, per = n_slab * n_rb;
    const unsigned xcd = blockIdx.x & 7u, k = blockIdx.x >> 3;
    const unsigned n_tile = (unsigned)tile_off[n_expert], per_xcd = (n_tile + 7u) >> 3;
    const unsigned tile = xcd * per_xcd + k / per, rb = (k % per) % n_rb, z = (k % per) / n_rb;
    if (blockDim.x != 256u || k / per >= per_xcd || tile >= n_tile) return;
    const ReinTileRows tr = rein_mmq_tile_rows(tile_off, expert_off, n_expert, tile);
    const unsigned lo = tr.expert, tok_base = tr.tok_base, tok_end = tr.tok_end;
    if (tok_base >= tok_end) return;
    const uint8_t* slab = z ? slab1 : slab0;
    rein_mmq_pipelined_tile<FMT, 32>(slab + (size_t)lo * bytes_per_expert, xq, z ? y1 : y0, in_dim, out_dim, rb,
                                     tok_base, min(tok_end, tok_base + 32u));
}

// Gate and up projection of an expert FFN with SwiGLU and the BlockQ8 quantizer in the
// epilogue: a workgroup owns one 32-token tile and 64 columns of the expert's ff dimension;
// wavefronts 0, 1 run the gate rows of those columns, wavefronts 2, 3 the up rows (the same
// contraction as rein_mmq_grouped_one, term for term, so gate and up carry the same bits as
// the two-output launch).  The four 32 x 32 tiles then meet in LDS as [wavefront][token][column]
// and the workgroup's sixteen 16-lane rows turn them into the 2 x 32 BlockQ8 blocks of
// silu(gate) * up with the quantizer and the silu of swiglu_q8_f32 -- the same bytes as
// rein_mmq_grouped_one + swiglu_q8_f32, without the two fp32 matrices between them.
// Launch: 1-D, 8 * ceil(tile_ub / 8) * ceil(out_dim / 64) workgroups of 256 threads, tiles
// dealt to XCDs as in rein_mmq_grouped_one.  out_dim a multiple of 32.
template <int FMT>
__device__ __forceinline__ void rein_mmq_grouped_swiglu(const uint8_t* __restrict__ gate_slab,
                                                        const uint8_t* __restrict__ up_slab, unsigned bytes_per_expert,
                                                        const int* __restrict__ expert_off, const int* __restrict__ tile_off,
                                                        unsigned n_expert, const BlockQ8* __restrict__ xq,
                                                        BlockQ8* __restrict__ out, unsigned in_dim, unsigned out_dim)
{
#pragma clang fp contract(off)
    constexpr unsigned kPitch = 40;                   // floats per token row of a wavefront's tile: the two lane
                                                      // halves (tokens 4 apart) land on different banks
    static_assert(rein_mmq_tile_lds_bytes<FMT, 32>() >= 4 * 32 * (int)kPitch * 4, "epilogue image does not fit the tile LDS");
    const unsigned n_cb = (out_dim + 63u) / 64u;
    const unsigned xcd = blockIdx.x & 7u, k = blockIdx.x >> 3;
    const unsigned n_tile = (unsigned)tile_off[n_expert], per_xcd = (n_tile + 7u) >> 3;
    const unsigned tile = xcd * per_xcd + k / n_cb, cb = k % n_cb;
    if (blockDim.x != 256u || k / n_cb >= per_xcd || tile >= n_tile) return;
    const ReinTileRows tr = rein_mmq_tile_rows(tile_off, expert_off, n_expert, tile);
    const unsigned lo = tr.expert, tok_base = tr.tok_base, tok_end = min(tr.tok_end, tok_base + 32u);
    if (tok_base >= tok_end) return;

    const unsigned lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint8_t* slab = (wave >> 1) ? up_slab : gate_slab;
    rein_v16f acc[1];
    rein_mmq_pipelined_acc<FMT, 32>(slab + (size_t)lo * bytes_per_expert, xq, in_dim, out_dim,
                                    cb * 64u + (wave & 1u) * 32u, tok_base, tok_end, acc);

    float* const img = reinterpret_cast<float*>(rein_mmq_tile_lds<rein_mmq_tile_lds_bytes<FMT, 32>()>());
    const unsigned j = lane & 31u, h = lane >> 5;
#pragma unroll
    for (int v = 0; v < 16; v++) img[(wave * 32u + 8u * (v / 4) + 4u * h + (v % 4)) * kPitch + j] = acc[0][v];
    __syncthreads();
    const unsigned n_sub_out = out_dim >> 5;
    const unsigned l = threadIdx.x & 15u, g = threadIdx.x >> 4;
#pragma unroll
    for (unsigned it = 0; it < 4u; it++) {
        const unsigned idx = it * 16u + g, half = idx >> 5, tok = idx & 31u;
        const unsigned blk = cb * 2u + half;
        if (tok_base + tok < tok_end && blk < n_sub_out) {
            const float* gt = img + (half * 32u + tok) * kPitch;
            const float* ut = img + ((2u + half) * 32u + tok) * kPitch;
            const float v0 = rein_silu_det(gt[l]) * ut[l], v1 = rein_silu_det(gt[l + 16]) * ut[l + 16];
            rein_q8_store_sub(out + (size_t)(tok_base + tok) * n_sub_out + blk, l, v0, v1);
        }
    }
}

// Two wavefronts per SIMD: a 256-register budget, which makes the compiler keep
// MFMA results in ordinary VGPRs (no AGPR round trips) without spilling.
#define REIN_MMQ_OCC __attribute__((amdgpu_waves_per_eu(2)))

#define REIN_MMQ_ARGS                                                                            \
    const unsigned char* __restrict__ w, const BlockQ8* __restrict__ xq, float* __restrict__ y, \
        unsigned int in_dim, unsigned int out_dim, unsigned int p_rows

#define REIN_DEFINE_MMQ(name, FMT, TM)                                                           \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(REIN_MMQ_ARGS)                        \
    {                                                                                            \
        rein_mmq_dense<FMT, TM, 0>(w, xq, y, nullptr, in_dim, out_dim, p_rows);                  \
    }

// tuned entry: fixed 256-thread workgroups, 1-D XCD-aware grid
#define REIN_DEFINE_MMQ_PIPE(name, FMT, TM)                                                      \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(REIN_MMQ_ARGS)                        \
    {                                                                                            \
        rein_mmq_pipelined<FMT, TM>(w, xq, y, in_dim, out_dim, p_rows);                          \
    }

#define REIN_DEFINE_MMQ_MIXED(name, FMT)                                                         \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(REIN_MMQ_ARGS, unsigned int n64) \
    {                                                                                            \
        rein_mmq_pipelined_mixed<FMT>(w, xq, y, in_dim, out_dim, p_rows, n64);                   \
    }

#define REIN_DEFINE_MMQ_DOTS(name, FMT)                                                          \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                         \
        const unsigned char* __restrict__ w, const BlockQ8* __restrict__ xq, int* __restrict__ out, \
        unsigned int in_dim, unsigned int out_dim, unsigned int p_rows)                          \
    {                                                                                            \
        rein_mmq_dense<FMT, 32, 1>(w, xq, nullptr, out, in_dim, out_dim, p_rows);                \
    }

#define REIN_DEFINE_MMQ_GROUPED(name, FMT)                                                       \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                         \
        const unsigned char* __restrict__ slab, unsigned int bytes_per_expert,                   \
        const int* __restrict__ expert_off, const int* __restrict__ tile_off, unsigned int n_expert, \
        const BlockQ8* __restrict__ xq, float* __restrict__ y, unsigned int in_dim,              \
        unsigned int out_dim)                                                                    \
    {                                                                                            \
        rein_mmq_grouped<FMT>(slab, bytes_per_expert, expert_off, tile_off, n_expert, xq, y,     \
                              in_dim, out_dim);                                                  \
    }

#define REIN_DEFINE_MMQ_GROUPED_ONE(name, FMT)                                                   \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                         \
        const unsigned char* __restrict__ slab0, const unsigned char* __restrict__ slab1,        \
        unsigned int bytes_per_expert, const int* __restrict__ expert_off,                       \
        const int* __restrict__ tile_off, unsigned int n_expert, const BlockQ8* __restrict__ xq, \
        float* __restrict__ y0, float* __restrict__ y1, unsigned int in_dim, unsigned int out_dim, \
        unsigned int n_slab)                                                                     \
    {                                                                                            \
        rein_mmq_grouped_one<FMT>(slab0, slab1, bytes_per_expert, expert_off, tile_off,          \
                                  n_expert, xq, y0, y1, in_dim, out_dim, n_slab);                \
    }

#define REIN_DEFINE_MMQ_GROUPED_SWIGLU(name, FMT)                                                \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                         \
        const unsigned char* __restrict__ gate_slab, const unsigned char* __restrict__ up_slab,  \
        unsigned int bytes_per_expert, const int* __restrict__ expert_off,                       \
        const int* __restrict__ tile_off, unsigned int n_expert, const BlockQ8* __restrict__ xq, \
        BlockQ8* __restrict__ out, unsigned int in_dim, unsigned int out_dim)                    \
    {                                                                                            \
        rein_mmq_grouped_swiglu<FMT>(gate_slab, up_slab, bytes_per_expert, expert_off, tile_off, \
                                     n_expert, xq, out, in_dim, out_dim);                        \
    }

#define REIN_DEFINE_MMQ_SPLIT_TAIL(name, FMT, TM)                                                \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                         \
        const unsigned char* __restrict__ w, const BlockQ8* __restrict__ xq, float* __restrict__ y, \
        float* __restrict__ part, unsigned int in_dim, unsigned int out_dim, unsigned int p_rows, \
        unsigned int split)                                                                      \
    {                                                                                            \
        rein_mmq_split_tail<FMT, TM>(w, xq, y, part, in_dim, out_dim, p_rows, split);            \
    }

#define REIN_DEFINE_MMQ_TAIL_SUM(name, NT)                                                       \
    extern "C" __global__ __launch_bounds__(256) void name(                                      \
        const float* __restrict__ part, float* __restrict__ y, unsigned int n_chunk,             \
        unsigned int out_dim, unsigned int p_rows, unsigned int first_unit, unsigned int split)  \
    {                                                                                            \
        rein_mmq_tail_sum_body<NT>(part, y, n_chunk, out_dim, p_rows, first_unit, split);        \
    }
