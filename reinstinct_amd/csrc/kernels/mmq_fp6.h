// Prefill MMQ GEMM for the 4-bit formats on the block-scaled fp6 matrix instruction.
//
// v_mfma_scale_f32_32x32x64_f8f6f4 with both operands in fp6 (E2M3) runs at the rate of the
// int8 32x32x32 instruction, contracts 64 slots per issue and returns fp32.  E2M3 code n
// (0..15) is the value n / 8, bit 5 is the sign, so a 4-bit magnitude IS its own fp6 code:
//   * a Q4_K weight nibble q goes into a 6-bit slot unchanged (value q / 8);
//   * an int8 activation x = sign * (16 a + b), a <= 7, b <= 15, becomes two codes
//     sign | a and sign | b: lanes 0..31 of the A operand carry the a parts of a token's 32
//     quants with block scale 2^7, lanes 32..63 the b parts with block scale 2^3, and the
//     weight operand carries the same 32 nibbles in both lane halves with block scale 2^3.
// One instruction therefore yields sum_k x_k q_k for a whole 32-weight sub-block of a
// 32-token x 32-row tile, exactly (every partial sum is an integer below 2^24), already in
// fp32: the int8 formulation's convert step disappears, and what is left per tile and
// sub-block is one fp32 multiply-add per element with the scale tile dx (x) d*sc, which a
// 2-block fp32 outer-product MFMA forms for two sub-blocks at a time.  The -dmin*m*xsum term
// is accumulated by a bf16 MFMA straight into the accumulators: xsum as three bf16 pieces,
// -dmin*m (17 significant bits, exact in fp32) as three bf16 pieces, the six products that
// matter per sub-block in six of the instruction's sixteen slots.
//
// Activations are brought into operand form once per GEMM by rein_mmq6_prep (every workgroup
// of the GEMM would otherwise redo it): the "X6 image", one 4352-byte record per (pair of
// sub-blocks, 32-token tile), laid out as the GEMM's LDS image so that it travels HBM/L2 ->
// LDS by global_load_lds_dwordx4 without touching registers.
//
// Replaces, for Q4_K, kernels/mmq_gemm_q4k_repacked.cpp:63-178 of the reference (same
// product, same per-sub-block terms (d*sc)*dx*idot - (dmin*m)*xsum).
#pragma once

#include "mmq_gemm.h"

typedef int rein_v8i __attribute__((ext_vector_type(8)));

// ---- slot order -----------------------------------------------------------------------
// The 16-byte nibble plane entry of a sub-block is four words W0..W3; nibble n of word j is
// weight 4j + n/2 (+16 when n is odd).  Words (W0, W1) fill slots 0..15, (W2, W3) slots
// 16..31, each pair by rein_fp6_pack16 below.  Source nibble (word of the pair, nibble) per
// slot, as that function places them:
//   a0 a1 a3 a4 a6 a7 b1 b2 b4 b5 b7 b0 a2 b3 a5 b6
__host__ __device__ constexpr int rein_fp6_slot_weight(int slot)
{
    constexpr int word[16]   = {0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1, 0, 1, 0, 1};
    constexpr int nibble[16] = {0, 1, 3, 4, 6, 7, 1, 2, 4, 5, 7, 0, 2, 3, 5, 6};
    const int pair = slot >> 4, i = slot & 15;
    const int j = 2 * pair + word[i], n = nibble[i];
    return 4 * j + (n >> 1) + 16 * (n & 1);
}

// Sixteen nibbles of (wa, wb) -> sixteen 6-bit slots in three words: every nibble moves by a
// shift of 0 or 2 (the one nibble that straddles words 0 and 1 by 2 and by -30), so three
// masks of the unshifted and three of the shifted words place fifteen of them.
__device__ __forceinline__ void rein_fp6_pack16(uint32_t wa, uint32_t wb, int& o0, int& o1, int& o2)
{
    const uint32_t sa = wa << 2, sb = wb << 2;
    o0 = (int)((wa & 0x0F00F00Fu) | (sa & 0xC03C03C0u));
    o1 = (int)((wb & 0xF00F00F0u) | (sb & 0x03C03C00u) | (wa >> 30));
    o2 = (int)((sb & 0x3C03C03Cu) | (wa & 0x00F00F00u));
}

__device__ __forceinline__ rein_v8i rein_fp6_weights(const uint4& q)
{
    int o[6];
    rein_fp6_pack16(q.x, q.y, o[0], o[1], o[2]);
    rein_fp6_pack16(q.z, q.w, o[3], o[4], o[5]);
    return rein_v8i{o[0], o[1], o[2], o[3], o[4], o[5], 0, 0};
}

// ---- X6 image -------------------------------------------------------------------------
// Record of (sub-block pair, token tile): 4352 bytes
//   [   0, 3072)  A operands: sub-block s of the pair at 1536 s:
//                   [0, 1024)    lane l = 32 h + j: words 0..3 of token j's part h (h = 0: the
//                                16's digits, h = 1: the units)
//                   [1024, 1536) lane l: words 4, 5
//   [3072, 3328)  dx: [s][j] fp32 (0 for tokens past the end)
//   [3328, 4352)  xs: [s][j] 16 bytes, the bf16 operand of the minimum term: the pieces x0, x1,
//                 x2 of xsum in slot order x0 x0 x1 x0 x1 x2 0 0
// Records are ordered [pair][token tile].
#define REIN_X6_REC 4352u

__host__ __device__ constexpr size_t rein_x6_bytes(unsigned n_sub, unsigned p_rows)
{
    return (size_t)((n_sub + 1u) / 2u) * ((p_rows + 31u) / 32u) * REIN_X6_REC + 1024u;   // + slack, see issue_acts
}

// One lane's share of the image: BlockQ8 block `sb` of row `tok` of xq (ok: the row and the
// block exist) goes into token slot j of record `rec`; n_rec = records per sub-block pair.
__device__ __forceinline__ void rein_mmq6_prep_lane(const BlockQ8* __restrict__ xq, uint8_t* __restrict__ img,
                                                    unsigned n_sub, unsigned n_rec, unsigned rec, unsigned j,
                                                    unsigned sb, unsigned tok, bool ok)
{
    float d = 0.0f, xs = 0.0f;
    int q[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (ok) {
        const BlockQ8* p = xq + (size_t)tok * n_sub + sb;
        d = p->d; xs = p->xsum;
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = p->qs[i];
    }
    uint32_t hi[6] = {0, 0, 0, 0, 0, 0}, lo[6] = {0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int slot = 0; slot < 32; slot++) {
        const int k = rein_fp6_slot_weight(slot);
        const int v = (int)(int8_t)((uint32_t)q[k >> 2] >> (8 * (k & 3)));
        const uint32_t mag = (uint32_t)(v < 0 ? -v : v), sgn = v < 0 ? 32u : 0u;
        const uint32_t ch = sgn | (mag >> 4), cl = sgn | (mag & 15u);
        const int bit = 6 * slot, wd = bit >> 5, sh = bit & 31;
        hi[wd] |= ch << sh; lo[wd] |= cl << sh;
        if (sh > 26) { hi[wd + 1] |= ch >> (32 - sh); lo[wd + 1] |= cl >> (32 - sh); }
    }
    uint8_t* r = img + ((size_t)(sb >> 1) * n_rec + rec) * REIN_X6_REC;
    uint8_t* a = r + (sb & 1u) * 1536u;
    *reinterpret_cast<uint4*>(a + j * 16u)          = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    *reinterpret_cast<uint4*>(a + 512u + j * 16u)   = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    *reinterpret_cast<uint2*>(a + 1024u + j * 8u)   = make_uint2(hi[4], hi[5]);
    *reinterpret_cast<uint2*>(a + 1280u + j * 8u)   = make_uint2(lo[4], lo[5]);
    *reinterpret_cast<float*>(r + 3072u + (sb & 1u) * 128u + j * 4u) = ok ? d : 0.0f;
    uint16_t sp[3];
    rein_mmq_split_xsum(ok ? xs : 0.0f, sp);
    const uint32_t x0 = sp[0], x1 = sp[1], x2 = sp[2];
    *reinterpret_cast<uint4*>(r + 3328u + (sb & 1u) * 512u + j * 16u) = make_uint4(x0 | (x0 << 16), x1 | (x0 << 16), x1 | (x2 << 16), 0u);
}

// xq [p_rows][n_sub] BlockQ8 -> X6 image.  One lane per (token, sub-block): the eight lanes
// of a token read eight consecutive blocks (320 contiguous bytes); blockIdx.x = token tile,
// blockIdx.y = group of 8 sub-blocks (4 pairs), 256 threads.
__device__ __forceinline__ void rein_mmq6_prep_body(const BlockQ8* __restrict__ xq, uint8_t* __restrict__ img,
                                                    unsigned n_sub, unsigned p_rows)
{
    const unsigned n_tt = (p_rows + 31u) / 32u;
    const unsigned tt = blockIdx.x;
    const unsigned j = threadIdx.x >> 3, s8 = threadIdx.x & 7u;
    const unsigned sb = blockIdx.y * 8u + s8, tok = tt * 32u + j;
    if (tt >= n_tt || sb >= ((n_sub + 1u) & ~1u)) return;
    rein_mmq6_prep_lane(xq, img, n_sub, n_tt, tt, j, sb, tok, tok < p_rows && sb < n_sub);
}

// ---- DMA helpers ----------------------------------------------------------------------
// Narrow HBM -> LDS transfers for the small weight words: each lane loads one 16-bit / 32-bit
// value, which lands as a dword at lds_base + 4 * lane.
__device__ __forceinline__ void rein_lds_dma_u16(const void* gptr, unsigned lds_base)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_ushort %0, off" : : "v"(gptr), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void rein_lds_dma_u32(const void* gptr, unsigned lds_base)
{
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(gptr), "s"(lds_base) : "memory", "m0");
}

// ---- the tile -------------------------------------------------------------------------
// LDS of one workgroup (4 wavefronts, 128 weight rows x 32 NT tokens):
//   acts   D x NT x 4352       activation records of D consecutive sub-block pairs
//   ring   4 x R x 2048        per wavefront: R slots of 4 sub-blocks x 32 rows x 16 B
//   small  4 x S x 1280        per wavefront: S buffers of (sc, m) of a superblock [row][8] as
//                              dwords, then (d, dmin) [row]
// The depths set how far ahead of their use the transfers are requested: D - 1 pair-steps for
// the records, R - 1 ring stages (2 pair-steps each) for the weights, 4 S - 2 pair-steps for
// the small words.  A pair-step of a 4-tile group computes for about a microsecond, which covers
// the memory latency at the shallowest depths; the narrow groups, whose pair-steps are a
// quarter as long, are given the weights several stages ahead.
template <int NT> struct Mmq6Cfg;
template <> struct Mmq6Cfg<4> { static constexpr int R = 2, D = 3, S = 1; };
template <> struct Mmq6Cfg<2> { static constexpr int R = 4, D = 4, S = 2; };
template <> struct Mmq6Cfg<1> { static constexpr int R = 3, D = 4, S = 1; };

template <int NT>
constexpr unsigned rein_mmq6_act_stride() { return (NT * REIN_X6_REC + 1023u) & ~1023u; }   // whole 1 KiB transfers
template <int NT>
constexpr int rein_mmq6_lds_bytes()
{
    return Mmq6Cfg<NT>::D * (int)rein_mmq6_act_stride<NT>() + 4 * Mmq6Cfg<NT>::R * 2048 + 4 * Mmq6Cfg<NT>::S * 1280;
}

// All global -> LDS traffic of the loop is DMA that the compiler cannot see; the waits are
// placed by hand and count exactly the transfers below.  Per pair-step i (one pair of
// sub-blocks), every wavefront issues, in this order:
//   acts(i + D - 1)                     K transfers   into record buffer (i + D - 1) % D
//   i % 2 == 0: ring(i / 2 + R - 1)     2 transfers   into slot (i / 2 + R - 1) % R
//   i % 4 == 2: small(i / 4 + S)        5 transfers   into small buffer (i / 4) % S (last read in this step)
// Transfers complete in order, so "X has landed" is "at most as many transfers are in flight as
// were issued after X".  At the top of step i the step needs acts(i), at even i the ring stage
// i / 2, at i % 4 == 0 the small words of chunk i / 4; Mmq6Waits counts what was issued after the
// oldest of those, per i % 4.  The prologue issues everything the first steps need and drains
// it, so the counts of the steady state hold from the first step.  Past the end of the pair
// range the same transfers are issued (into buffers nobody reads again; past the end of the
// contraction on clamped addresses), which keeps the counts uniform; the tile drains them
// before it ends.
template <int K, int R, int D, int S>
struct Mmq6Waits {
    static constexpr int ring(int s) { return s % 2 == 0 ? 2 : 0; }
    static constexpr int small(int s) { return s % 4 == 2 ? 5 : 0; }
    static constexpr int cnt(int s) { return K + ring(s) + small(s); }
    static constexpr int sum(int a, int b) { int t = 0; for (int s = a; s <= b; s++) t += cnt(s); return t; }
    static constexpr int at(int r)                 // r = i % 4; the step is taken as r + 64 (period 4)
    {
        const int i = r + 64;
        int n = ring(i - D + 1) + small(i - D + 1) + sum(i - D + 2, i - 1);                    // after acts(i)
        if (r % 2 == 0) {
            const int m = small(i - 2 * R + 2) + sum(i - 2 * R + 3, i - 1);                    // after ring(i / 2)
            n = m < n ? m : n;
        }
        if (r == 0) {
            const int m = sum(i - 4 * S + 3, i - 1);                                           // after small(i / 4)
            n = m < n ? m : n;
        }
        return n;
    }
};

// The records and the rows of xq / y that one workgroup covers.
struct Mmq6Span {
    unsigned n_rec;      // records per sub-block pair in the image
    unsigned rec0;       // first record of this workgroup
    unsigned rec_cnt;    // records that exist from rec0 on (>= 1); min(NT, rec_cnt) are computed
    unsigned tok_base;   // row of y of token 0 of record rec0; record rec0 + t starts 32 t rows on
    unsigned tok_end;    // one past the last row of this span
    unsigned pair_begin; // the sub-block pairs [pair_begin, pair_end) of the contraction are summed,
    unsigned pair_end;   // both multiples of 4 (whole superblocks); pair_end = 0 stands for the whole contraction
    float* part;         // nullptr: the sums are the result, stored to y; else: a partial tile, stored
                         // here as [tile][register][thread] (NT * 16 * 256 floats) for rein_mmq6_tail_sum
};

template <int NT, int DOTS>
__device__ __forceinline__ void rein_mmq6_tile(const uint8_t* __restrict__ w, const uint8_t* __restrict__ img,
                                               float* __restrict__ y, int* __restrict__ dots, unsigned in_dim,
                                               unsigned out_dim, unsigned rb, const Mmq6Span span)
{
    constexpr int FMT = REIN_Q4_K;
    using F = Fmt<FMT>;
    constexpr unsigned kActBytes = rein_mmq6_act_stride<NT>();           // LDS buffer of one pair (records + pad)
    constexpr unsigned kActDma = (kActBytes + 4095u) / 4096u;          // transfers per wavefront and pair-step
    constexpr unsigned R = Mmq6Cfg<NT>::R, D = Mmq6Cfg<NT>::D, S = Mmq6Cfg<NT>::S;
    using Waits = Mmq6Waits<(int)kActDma, (int)R, (int)D, (int)S>;
    static_assert(Waits::at(0) < 64 && Waits::at(1) < 64 && Waits::at(2) < 64 && Waits::at(3) < 64, "vmcnt holds 6 bits");
    extern __shared__ __attribute__((aligned(16))) unsigned char rein_mmq6_lds[];
    unsigned char* const raw = rein_mmq6_lds;
    typedef __attribute__((address_space(3))) const void* lptr_t;

    const unsigned lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned j = lane & 31u, h = lane >> 5;
    const unsigned n_sub = in_dim >> 5, n_pair = n_sub >> 1, n_tt = span.n_rec, tt0 = span.rec0;
    const F fmt(w, n_sub, out_dim);
    const unsigned row_base = rb * 128u + wave * 32u;
    const unsigned row = row_base + j;
    const unsigned rowc = min(row, out_dim - 1u);

    const uint4* const ring = reinterpret_cast<const uint4*>(raw + D * kActBytes + wave * (R * 2048u));
    const uint32_t* const small0 = reinterpret_cast<const uint32_t*>(raw + D * kActBytes + 4u * R * 2048u + wave * (S * 1280u));
    const unsigned lds_acts = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)raw);
    const unsigned lds_small = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)small0);
    MmqWSrc<FMT> wsrc;                               // slot s of the ring is 2048 s bytes on, as rein_mmq_wload addresses it
    wsrc.init(*reinterpret_cast<const MmqWLds<FMT>*>(ring), fmt, row_base, out_dim, lane);

    // activation source: this workgroup's NT records of a pair are contiguous
    const unsigned tt_cnt = min((unsigned)NT, span.rec_cnt);              // records that exist (>= 1)
    const size_t pair_stride = (size_t)n_tt * REIN_X6_REC;
    auto issue_acts = [&](unsigned pair) {
        const unsigned p = min(pair, n_pair - 1u);
        const uint8_t* src = img + (size_t)p * pair_stride + (size_t)tt0 * REIN_X6_REC;
        const unsigned buf = lds_acts + (pair % D) * kActBytes;
#pragma unroll
        for (unsigned k = 0; k < kActDma; k++) {
            // transfer k of this wavefront covers bytes [off, off + 1024) of the records; one
            // that starts past the records that exist repeats the first kilobyte onto itself,
            // one that straddles their end drags in what follows them in the image (the image
            // is allocated with a kilobyte of slack) and drops it on the buffer's pad
            unsigned off = (k * 4u + wave) * 1024u;
            if (off >= tt_cnt * REIN_X6_REC) off = 0u;
            rein_lds_dma16(src + off + lane * 16u, buf + off);
        }
    };
    auto issue_ring = [&](unsigned stage) {
        const unsigned sb_first = min(stage * 4u, n_sub - 4u);
        rein_mmq_wload<FMT>(wsrc, stage % R, fmt, sb_first, n_sub);
    };
    auto issue_small = [&](unsigned chunk) {
        const unsigned sup = min(chunk, (n_sub >> 3) - 1u);
        const unsigned dst = lds_small + (chunk % S) * 1280u;
#pragma unroll
        for (unsigned k = 0; k < 4; k++) {
            const unsigned r = min(row_base + 8u * k + (lane >> 3), out_dim - 1u);
            rein_lds_dma_u16(fmt.smp + (size_t)r * fmt.nsp + sup * 8u + (lane & 7u), dst + k * 256u);
        }
        rein_lds_dma_u32(fmt.ddp + (size_t)rowc * fmt.n_super + sup, dst + 1024u);
    };

    rein_v16f acc[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[t][v] = 0.0f;
    rein_v16f z16;
#pragma unroll
    for (int v = 0; v < 16; v++) z16[v] = 0.0f;
    rein_v32f z32;
#pragma unroll
    for (int v = 0; v < 32; v++) z32[v] = 0.0f;
    const int scale_a = h ? 130 : 134, scale_b = 130;                   // 2^3, 2^7 | 2^3 (E8M0)

    // prologue: everything the steps before the first in-loop requests land need.  A workgroup
    // may run several tiles in a row: the barrier keeps the first transfers off buffers that a
    // slower wavefront still reads for the previous tile.
    const unsigned pb = span.pair_begin, pe = span.pair_end ? span.pair_end : n_pair;     // 0: the whole contraction
    __syncthreads();
#pragma unroll
    for (unsigned k = 0; k + 1u < D; k++) issue_acts(pb + k);
#pragma unroll
    for (unsigned k = 0; k + 1u < R; k++) issue_ring((pb >> 1) + k);
#pragma unroll
    for (unsigned k = 0; k < S; k++) issue_small((pb >> 2) + k);
    REIN_WAIT_VMCNT(0);

    // Words 4, 5 of the second operand of a pair are addressed through an offset the compiler
    // cannot see through: with a common base it pairs that read with the first operand's in
    // one ds_read2, whose result then has to be moved into the two operands' register tuples.
    unsigned lane8b = lane * 8u;
    asm volatile("" : "+v"(lane8b));

    float scq[2];                    // d * sc of sub-block 2q + h of the current stage
    rein_v8bf pmin[2];               // bf16 pieces of -dmin * m of that sub-block, in slot order
    const unsigned rot = j >> 1;

    for (unsigned i = pb; i < pe; i++) {
        if ((i & 3u) == 0u) REIN_WAIT_VMCNT(Waits::at(0));
        else if ((i & 3u) == 1u) REIN_WAIT_VMCNT(Waits::at(1));
        else if ((i & 3u) == 2u) REIN_WAIT_VMCNT(Waits::at(2));
        else REIN_WAIT_VMCNT(Waits::at(3));
        __syncthreads();
        issue_acts(i + D - 1u);
        if ((i & 1u) == 0u) {
            issue_ring((i >> 1) + R - 1u);
            // scales of this stage's four sub-blocks from the small buffer
            const unsigned half = (i >> 1) & 1u;                         // which half of the superblock
            const uint32_t* const small = small0 + ((i >> 2) % S) * 320u;
            const uint32_t dd = small[256 + lane];
            const float d = rein_h2f((uint16_t)(dd & 0xFFFFu)), ndmin = -rein_h2f((uint16_t)(dd >> 16));
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const uint32_t sm = small[j * 8u + half * 4u + 2u * q + h];
                scq[q] = d * (float)(sm & 0xFFu);
                const float pm = ndmin * (float)(sm >> 8);               // exact: 11 x 6 significant bits
                const uint32_t b0 = __builtin_bit_cast(uint32_t, pm) & 0xFFFF0000u;
                const float r1 = pm - __builtin_bit_cast(float, b0);
                const uint32_t b1 = __builtin_bit_cast(uint32_t, r1) & 0xFFFF0000u;
                const float r2 = r1 - __builtin_bit_cast(float, b1);
                const uint32_t p0 = b0 >> 16, p1 = b1 >> 16, p2 = __builtin_bit_cast(uint32_t, r2) >> 16;
                // slots: (x0,p0) (x0,p1) (x1,p0) (x0,p2) (x1,p1) (x2,p0)
                const uint4 pk = make_uint4(p0 | (p1 << 16), p0 | (p2 << 16), p1 | (p0 << 16), 0u);
                pmin[q] = __builtin_bit_cast(rein_v8bf, pk);
            }
            if ((i & 3u) == 2u) {
                __builtin_amdgcn_s_waitcnt(0xC07F);                      // the small buffer has been read
                issue_small((i >> 2) + S);
            }
        }
        const unsigned char* const act = raw + (i % D) * kActBytes;
        const unsigned q = i & 1u;
        const uint4* slot = ring + ((i >> 1) % R) * 128u;
        const rein_v8i b0 = rein_fp6_weights(slot[4u * j + ((2u * q + rot) & 3u)]);
        const rein_v8i b1 = rein_fp6_weights(slot[4u * j + ((2u * q + 1u + rot) & 3u)]);
        const float sc = q ? scq[1] : scq[0];
        const rein_v8bf pm = q ? pmin[1] : pmin[0];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const unsigned char* rec = act + t * REIN_X6_REC;
            rein_v8i a0, a1;
            {
                const uint4 lo4 = *reinterpret_cast<const uint4*>(rec + lane * 16u);
                const uint2 hi2 = *reinterpret_cast<const uint2*>(rec + 1024u + lane * 8u);
                a0[0] = (int)lo4.x; a0[1] = (int)lo4.y; a0[2] = (int)lo4.z; a0[3] = (int)lo4.w; a0[4] = (int)hi2.x; a0[5] = (int)hi2.y; a0[6] = 0; a0[7] = 0;
                const uint4 lo4b = *reinterpret_cast<const uint4*>(rec + 1536u + lane * 16u);
                const uint2 hi2b = *reinterpret_cast<const uint2*>(rec + 1536u + 1024u + lane8b);
                a1[0] = (int)lo4b.x; a1[1] = (int)lo4b.y; a1[2] = (int)lo4b.z; a1[3] = (int)lo4b.w; a1[4] = (int)hi2b.x; a1[5] = (int)hi2b.y; a1[6] = 0; a1[7] = 0;
            }
            const rein_v16f d0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a0, b0, z16, 2, 2, 0, scale_a, 0, scale_b);
            const rein_v16f d1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a1, b1, z16, 2, 2, 0, scale_a, 0, scale_b);
            if constexpr (DOTS != 0) {
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const unsigned tok = span.tok_base + t * 32u + 8 * (v / 4) + 4 * h + (v % 4);
                    if (tok < span.tok_end && row < out_dim) {
                        int* o = dots + ((size_t)tok * out_dim + row) * n_sub + 2u * i;
                        o[0] = (int)d0[v];
                        o[1] = (int)d1[v];
                    }
                }
            } else {
                const float dxv = *reinterpret_cast<const float*>(rec + 3072u + lane * 4u);
                const rein_v32f sx = __builtin_amdgcn_mfma_f32_32x32x1f32(dxv, sc, z32, 0, 0, 0);
                const uint4 xa = *reinterpret_cast<const uint4*>(rec + 3328u + lane * 16u);
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][v] = fmaf(d0[v], sx[v], acc[t][v]);
#pragma unroll
                for (int v = 0; v < 16; v++) acc[t][v] = fmaf(d1[v], sx[16 + v], acc[t][v]);
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rein_v8bf, xa), pm, acc[t], 0, 0, 0);
            }
        }
    }
    REIN_WAIT_VMCNT(0);

    if constexpr (DOTS == 0) {
        if (span.part) {
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int v = 0; v < 16; v++) span.part[(t * 16 + v) * 256 + threadIdx.x] = acc[t][v];
            return;
        }
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const unsigned tok = span.tok_base + t * 32u + 8 * (v / 4) + 4 * h + (v % 4);
                if (tok < span.tok_end && row < out_dim) y[(size_t)tok * out_dim + row] = acc[t][v];
            }
    }
}

// Workgroup -> (row block, token tiles), XCD-aware as rein_mmq_pipelined: workgroup i runs on
// XCD i % 8, and all token groups of one 128-row weight block are dealt to the same XCD, so the
// block is pulled from HBM once and re-read from that L2.  The tokens of a row block are cut
// into n4 groups of four 32-token tiles, then n2 groups of two, then single tiles: the wide
// groups spend least per token (one weight unpack feeds four MFMA tiles) but at a few hundred
// tokens their coarse grain leaves the last round of workgroups badly filled; launched first,
// with the narrow ones behind them as fillers, the machine drains evenly.  The host picks
// n4 and n2 (n4 * 4 + n2 * 2 <= token tiles).
// Grid: 8 * ceil(n_row_blocks / 8) * (n4 + n2 + n1) workgroups of 256 threads, n1 = the rest.
__device__ __forceinline__ Mmq6Span rein_mmq6_dense_span(unsigned p_rows, unsigned tt0)
{
    const unsigned n_tt = (p_rows + 31u) / 32u;
    return Mmq6Span{n_tt, tt0, n_tt - tt0, tt0 * 32u, p_rows, 0u, 0u, nullptr};
}

__device__ __forceinline__ void rein_mmq6_mixed(const uint8_t* __restrict__ w, const uint8_t* __restrict__ img,
                                                float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                unsigned p_rows, unsigned n4, unsigned n2)
{
    const unsigned n_rb = (out_dim + 127u) / 128u, n_rbg = (n_rb + 7u) / 8u;
    const unsigned n_tt = (p_rows + 31u) / 32u;
    const unsigned n1 = n_tt - 4u * n4 - 2u * n2;
    const unsigned xcd = blockIdx.x & 7u;
    unsigned k = blockIdx.x >> 3;
    if (k < n_rbg * n4) {
        const unsigned rb = (k / n4) * 8u + xcd;
        if (rb < n_rb) rein_mmq6_tile<4, 0>(w, img, y, nullptr, in_dim, out_dim, rb, rein_mmq6_dense_span(p_rows, (k % n4) * 4u));
        return;
    }
    k -= n_rbg * n4;
    if (k < n_rbg * n2) {
        const unsigned rb = (k / n2) * 8u + xcd;
        if (rb < n_rb) rein_mmq6_tile<2, 0>(w, img, y, nullptr, in_dim, out_dim, rb, rein_mmq6_dense_span(p_rows, 4u * n4 + (k % n2) * 2u));
        return;
    }
    k -= n_rbg * n2;
    if (n1 == 0u) return;
    const unsigned rb = (k / n1) * 8u + xcd;
    if (rb < n_rb) rein_mmq6_tile<1, 0>(w, img, y, nullptr, in_dim, out_dim, rb, rein_mmq6_dense_span(p_rows, 4u * n4 + 2u * n2 + k % n1));
}

template <int NT, int DOTS>
__device__ __forceinline__ void rein_mmq6_dense(const uint8_t* __restrict__ w, const uint8_t* __restrict__ img,
                                                float* __restrict__ y, int* __restrict__ dots, unsigned in_dim,
                                                unsigned out_dim, unsigned p_rows)
{
    const unsigned n_rb = (out_dim + 127u) / 128u;
    const unsigned n_tt = (p_rows + 31u) / 32u, n_tg = (n_tt + NT - 1) / NT;
    const unsigned xcd = blockIdx.x & 7u, k = blockIdx.x >> 3;
    const unsigned rb = (k / n_tg) * 8u + xcd, tg = k % n_tg;
    if (rb >= n_rb) return;
    rein_mmq6_tile<NT, DOTS>(w, img, y, dots, in_dim, out_dim, rb, rein_mmq6_dense_span(p_rows, tg * NT));
}

// ---- split-tail launch ----------------------------------------------------------------
// 17408 rows are 136 row blocks, 512 tokens four 4-tile groups: 544 workgroup tiles on 512
// resident slots is 1.06 rounds, and no tiling by powers of two changes that 17/16.  Here the
// launch is exactly the resident slots (gridDim.x = G workgroups, a multiple of 8), and the
// units -- unit u = (row block u / n_tg, 4-tile token group u % n_tg) -- are dealt in rounds:
// in round r workgroup `pos` computes unit r G + pos whole.  What is left after the whole
// rounds (U mod G units, the tail) is split along the contraction: `split` workgroups per
// unit, each a contiguous range of superblock chunks, all at the same time; the workgroup of
// range k of tail unit t stores its partial tile to slot t * split + k of `part`, and
// rein_mmq6_tail_sum, launched behind this kernel, adds the partial tiles of every tail unit
// in range order.
// pos = (blockIdx.x % 8) * G / 8 + blockIdx.x / 8: the workgroups of one XCD hold neighbouring
// units, so the token groups of a row block -- and the ranges of a tail unit -- meet in one
// L2 at the same time.
__device__ __forceinline__ void rein_mmq6_split_tail(const uint8_t* __restrict__ w, const uint8_t* __restrict__ img,
                                                     float* __restrict__ y, float* __restrict__ part,
                                                     unsigned in_dim, unsigned out_dim, unsigned p_rows, unsigned split)
{
    constexpr unsigned kPart = 4u * 16u * 256u;                          // floats per partial tile
    const unsigned n_rb = (out_dim + 127u) / 128u, n_tt = (p_rows + 31u) / 32u, n_tg = (n_tt + 3u) / 4u;
    const unsigned n_chunk = in_dim >> 8, g = gridDim.x, n_unit = n_rb * n_tg;
    const unsigned pos = (blockIdx.x & 7u) * (g >> 3) + (blockIdx.x >> 3);
    const unsigned rounds = n_unit / g, n_tail = n_unit - rounds * g;

    for (unsigned r = 0; r < rounds; r++) {
        const unsigned u = r * g + pos, rb = u / n_tg, tg = u % n_tg;
        const Mmq6Span span{n_tt, tg * 4u, n_tt - tg * 4u, tg * 128u, p_rows, 0u, 0u, nullptr};
        rein_mmq6_tile<4, 0>(w, img, y, nullptr, in_dim, out_dim, rb, span);
    }
    // the tail's ranges are dealt evenly over the XCDs, each XCD a contiguous run of them
    const unsigned n_seg = n_tail * split, per_xcd = (n_seg + 7u) >> 3;
    const unsigned seg = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
    if ((blockIdx.x >> 3) >= per_xcd || seg >= n_seg) return;

    const unsigned tu = seg / split, k = seg - tu * split;               // tail unit, range within it
    const unsigned u = rounds * g + tu, rb = u / n_tg, tg = u % n_tg;
    const unsigned c0 = n_chunk * k / split, c1 = n_chunk * (k + 1u) / split;
    if (c0 == c1) return;                                                // more ranges than chunks: nothing to add
    const Mmq6Span span{n_tt, tg * 4u, n_tt - tg * 4u, tg * 128u, p_rows, 4u * c0, 4u * c1,
                        split > 1u ? part + (size_t)seg * kPart : nullptr};
    rein_mmq6_tile<4, 0>(w, img, y, nullptr, in_dim, out_dim, rb, span);
}

// y of the tail units = their partial tiles added in range order.  Grid (tail units, 4, 4): blockIdx.x = tail unit,
// blockIdx.y = 32-token tile of the unit's four, blockIdx.z = register quad, 256 threads as in the GEMM (thread -> weight
// row, register -> token).  `first_unit` = the whole rounds' unit count.
__device__ __forceinline__ void rein_mmq6_tail_sum_body(const float* __restrict__ part, float* __restrict__ y,
                                                        unsigned in_dim, unsigned out_dim, unsigned p_rows,
                                                        unsigned first_unit, unsigned split)
{
    constexpr unsigned kPart = 4u * 16u * 256u;
    const unsigned n_tt = (p_rows + 31u) / 32u, n_tg = (n_tt + 3u) / 4u, n_chunk = in_dim >> 8;
    const unsigned tu = blockIdx.x, t = blockIdx.y, u = first_unit + tu, rb = u / n_tg, tg = u % n_tg;
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, j = lane & 31u, h = lane >> 5;
    const unsigned row = rb * 128u + wave * 32u + j;
    // blockIdx.z = which four of the sixteen registers: four times the workgroups, a quarter of the serial loads each
    const unsigned v0 = 4u * blockIdx.z;
    float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 4
    for (unsigned q = 0; q < split; q++) {
        if (n_chunk * q / split == n_chunk * (q + 1u) / split) continue;           // an empty range stored nothing
        const float* src = part + (size_t)(tu * split + q) * kPart + (t * 16u + v0) * 256u + threadIdx.x;
#pragma unroll
        for (int v = 0; v < 4; v++) sum[v] += src[v * 256];
    }
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const unsigned tok = tg * 128u + t * 32u + 8u * blockIdx.z + 4u * h + v;
        if (tok < p_rows && row < out_dim) y[(size_t)tok * out_dim + row] = sum[v];
    }
}

#define REIN_DEFINE_MMQ6_PREP(name)                                                                 \
    extern "C" __global__ __launch_bounds__(256) void name(const BlockQ8* __restrict__ xq,          \
                                                           unsigned char* __restrict__ img,         \
                                                           unsigned int n_sub, unsigned int p_rows) \
    {                                                                                               \
        rein_mmq6_prep_body(xq, img, n_sub, p_rows);                                                \
    }

#define REIN_DEFINE_MMQ6_MIXED(name)                                                                \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                            \
        const unsigned char* __restrict__ w, const unsigned char* __restrict__ img,                 \
        float* __restrict__ y, unsigned int in_dim, unsigned int out_dim, unsigned int p_rows,      \
        unsigned int n4, unsigned int n2)                                                           \
    {                                                                                               \
        rein_mmq6_mixed(w, img, y, in_dim, out_dim, p_rows, n4, n2);                                \
    }

#define REIN_DEFINE_MMQ6_SPLIT_TAIL(name)                                                           \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                            \
        const unsigned char* __restrict__ w, const unsigned char* __restrict__ img,                 \
        float* __restrict__ y, float* __restrict__ part, unsigned int in_dim,                       \
        unsigned int out_dim, unsigned int p_rows, unsigned int split)                              \
    {                                                                                               \
        rein_mmq6_split_tail(w, img, y, part, in_dim, out_dim, p_rows, split);                      \
    }

#define REIN_DEFINE_MMQ6_TAIL_SUM(name)                                                             \
    extern "C" __global__ __launch_bounds__(256) void name(                                         \
        const float* __restrict__ part, float* __restrict__ y, unsigned int in_dim,                 \
        unsigned int out_dim, unsigned int p_rows, unsigned int first_unit, unsigned int split)     \
    {                                                                                               \
        rein_mmq6_tail_sum_body(part, y, in_dim, out_dim, p_rows, first_unit, split);               \
    }

#define REIN_DEFINE_MMQ6_DOTS(name)                                                                 \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                            \
        const unsigned char* __restrict__ w, const unsigned char* __restrict__ img,                 \
        int* __restrict__ out, unsigned int in_dim, unsigned int out_dim, unsigned int p_rows)      \
    {                                                                                               \
        rein_mmq6_dense<1, 1>(w, img, nullptr, out, in_dim, out_dim, p_rows);                       \
    }
