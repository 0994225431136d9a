// Prefill MMQ GEMM for Q4_K on the fp16 matrix instruction, with the contraction of a whole
// 256-weight superblock accumulated inside the matrix unit.
//
// The int8 and fp6 formulations leave one fp32 multiply-add per output element and 32-weight
// sub-block on the vector ALU (the scale (d*sc) * dx differs per sub-block on both sides), and
// that is what bounds them.  Here both per-sub-block factors go into the operands instead:
//   * weight operand  q * sc           (nibble times 6-bit scale, at most 945: exact in fp16);
//   * token operand   x * dx * 2^-e    as a pair of fp16 numbers hi + lo (22 significant bits;
//                     e per token row, so that the largest |x * dx| of the row lands in
//                     [2^14, 2^15) -- the fp32 range of dx never reaches the fp16 one).
// v_mfma_f32_32x32x16_f16 multiplies exactly and accumulates in fp32, so
//   S1 = sum over the superblock of (q sc) (x dx)        -- four instructions per sub-block
//   S2 = sum over its 8 sub-blocks of m * (xsum 2^-e-6)  -- one instruction per superblock
// and per superblock and output element the vector ALU does  y += d S1 - (64 dmin) S2, once per
// 256 weights instead of once per 32.  The result is multiplied by 2^e when it is stored.
// Differences to the per-sub-block fp32 chain of the other kernels are of the order of fp32
// rounding (the token operand carries 22 of its 24 bits).
//
// A wavefront owns 64 weight rows x 64 tokens (2 x 2 instruction tiles: every operand register
// feeds two instructions), a workgroup of four wavefronts 256 rows x 64 tokens.  The token
// operands are made once per GEMM by rein_mmq16_prep (the "X16 image") and travel L2 -> LDS by
// DMA; the weight nibbles go through the per-wavefront LDS ring of the other tile kernels.
//
// Replaces, for Q4_K, kernels/mmq_gemm_q4k_repacked.cpp:63-178 of the reference (same product,
// same per-sub-block terms (d*sc)*dx*idot - (dmin*m)*xsum, summed per superblock first).
#pragma once

#include "mmq_fp6.h"

typedef _Float16 rein_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 rein_v8h __attribute__((ext_vector_type(8)));

// ---- operand slot order ---------------------------------------------------------------
// An instruction contracts 16 slots; lane half h holds slots 8h .. 8h+7 of both operands.  The
// two instructions kh = 0, 1 of a sub-block take word 2h + kh of the sub-block's 16-byte nibble
// entry (nibble n of word j is weight 4j + n/2, + 16 when n is odd), and the eight nibbles of
// a word land in the slots in the order the masks below produce them: n0 n4 n1 n5 n2 n6 n3 n7.
__host__ __device__ constexpr int rein_f16_slot_weight(int kh, int h, int e)
{
    constexpr int t[8] = {0, 2, 16, 18, 1, 3, 17, 19};
    return 4 * (2 * h + kh) + t[e];
}

// ---- X16 image ------------------------------------------------------------------------
//   records   [sub-block pair][64-token group] of 16384 bytes:
//               [q: sub-block of the pair][t: 32-token tile][op = 2 kh + part][lane][8 x fp16]
//               part 0 = hi, 1 = lo; lane = 32 h + token
//   xs        [superblock][64-token group] of 2048 bytes: [t][lane][8 x fp16], lane half 0 the
//             hi parts of xsum * 2^(-e-6) of the superblock's 8 sub-blocks, half 1 the lo parts
//   tokscale  [64-token group][64] fp32: 2^e per token
#define REIN_X16_REC 16384u
#define REIN_X16_XS  2048u

__host__ __device__ constexpr size_t rein_x16_xs_offset(unsigned n_sub, unsigned p_rows)
{
    return (size_t)(n_sub / 2u) * ((p_rows + 63u) / 64u) * REIN_X16_REC;
}
__host__ __device__ constexpr size_t rein_x16_scale_offset(unsigned n_sub, unsigned p_rows)
{
    return rein_x16_xs_offset(n_sub, p_rows) + (size_t)(n_sub / 8u) * ((p_rows + 63u) / 64u) * REIN_X16_XS;
}
__host__ __device__ constexpr size_t rein_x16_bytes(unsigned n_sub, unsigned p_rows)
{
    return rein_x16_scale_offset(n_sub, p_rows) + (size_t)((p_rows + 63u) / 64u) * 256u + 1024u;
}

// xq [p_rows][n_sub] BlockQ8 -> X16 image.  blockIdx.x = 32-token tile, blockIdx.y = superblock,
// 256 threads: thread 8 j + s handles token j of the tile, sub-block s of the superblock.
__device__ __forceinline__ void rein_mmq16_prep_body(const BlockQ8* __restrict__ xq, uint8_t* __restrict__ img,
                                                     unsigned n_sub, unsigned p_rows)
{
    const unsigned n_grp = (p_rows + 63u) / 64u;
    const unsigned tt = blockIdx.x, c = blockIdx.y;
    const unsigned j = threadIdx.x >> 3, s8 = threadIdx.x & 7u, lane = threadIdx.x & 63u;
    const unsigned tok = tt * 32u + j, sb = c * 8u + s8;
    const bool ok = tok < p_rows;
    const BlockQ8* row = xq + (size_t)(ok ? tok : 0u) * n_sub;

    // e of the token row from its largest dx (every workgroup of the row finds the same one)
    float dmax = 0.0f;
    for (unsigned s = s8; s < n_sub; s += 8u) dmax = fmaxf(dmax, ok ? fabsf(row[s].d) : 0.0f);
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) dmax = fmaxf(dmax, __shfl_xor(dmax, m));
    int e = 0;
    if (dmax > 0.0f && dmax < INFINITY) {
        int ex;
        (void)frexpf(dmax, &ex);                     // dmax = f 2^ex, f in [0.5, 1)
        e = ex - 8;                                  // dmax 2^-e in [2^7, 2^8): |x dx| 2^-e < 2^15
    }

    float d = 0.0f, xs = 0.0f;
    int q[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (ok) {
        const BlockQ8* p = row + sb;
        d = p->d; xs = p->xsum;
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = p->qs[i];
    }
    const float ds = ldexpf(d, -e);
    uint8_t* rec = img + ((size_t)(sb >> 1) * n_grp + (tt >> 1)) * REIN_X16_REC + (sb & 1u) * 8192u + (tt & 1u) * 4096u;
#pragma unroll
    for (int kh = 0; kh < 2; kh++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            uint32_t hi[4], lo[4];
#pragma unroll
            for (int e2 = 0; e2 < 8; e2++) {
                const int k = rein_f16_slot_weight(kh, h, e2);
                const float v = (float)(int)(int8_t)((uint32_t)q[k >> 2] >> (8 * (k & 3))) * ds;
                const _Float16 vh = (_Float16)v;
                const _Float16 vl = (_Float16)(v - (float)vh);
                const uint32_t bh = __builtin_bit_cast(uint16_t, vh), bl = __builtin_bit_cast(uint16_t, vl);
                if (e2 & 1) { hi[e2 >> 1] |= bh << 16; lo[e2 >> 1] |= bl << 16; }
                else        { hi[e2 >> 1] = bh;        lo[e2 >> 1] = bl; }
            }
            uint8_t* o = rec + (2u * kh) * 1024u + (32u * h + j) * 16u;
            *reinterpret_cast<uint4*>(o)         = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            *reinterpret_cast<uint4*>(o + 1024u) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        }

    // xsum operand of the superblock: the token's 8 lanes each hold one sub-block's pair
    const float xv = ldexpf(xs, -e - 6);
    const _Float16 xh = (_Float16)xv;
    const _Float16 xl = (_Float16)(xv - (float)xh);
    const uint32_t mine = (uint32_t)__builtin_bit_cast(uint16_t, xh) | ((uint32_t)__builtin_bit_cast(uint16_t, xl) << 16);
    uint32_t all[8];
#pragma unroll
    for (int k = 0; k < 8; k++) all[k] = (uint32_t)__shfl((int)mine, (int)((lane & ~7u) + k));
    if (s8 == 0u) {
        uint8_t* x = img + rein_x16_xs_offset(n_sub, p_rows) + ((size_t)c * n_grp + (tt >> 1)) * REIN_X16_XS + (tt & 1u) * 1024u;
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            hi[k] = (all[2 * k] & 0xFFFFu) | (all[2 * k + 1] << 16);
            lo[k] = (all[2 * k] >> 16) | (all[2 * k + 1] & 0xFFFF0000u);
        }
        *reinterpret_cast<uint4*>(x + j * 16u)          = make_uint4(hi[0], hi[1], hi[2], hi[3]);
        *reinterpret_cast<uint4*>(x + (32u + j) * 16u)  = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        if (c == 0u)
            reinterpret_cast<float*>(img + rein_x16_scale_offset(n_sub, p_rows))[tt * 32u + j] = ldexpf(1.0f, e);
    }
}

// ---- the tile -------------------------------------------------------------------------
// LDS of one workgroup (4 wavefronts, 256 weight rows x 64 tokens):
//   acts   D x 16384           records of D consecutive sub-block pairs
//   xs     2 x 2048            xsum operands of two consecutive superblocks
//   ring   4 x 2 x R x 2048    per wavefront and 32-row tile: R slots of 4 sub-blocks x 32 rows x 16 B
//   small  4 x 2 x 1280        per wavefront and 32-row tile: (sc, m) of a superblock [row][8] as
//                              dwords, then (d, dmin) [row]
struct Mmq16Cfg { static constexpr int R = 2, D = 2; };
constexpr int rein_mmq16_lds_bytes()
{
    return Mmq16Cfg::D * (int)REIN_X16_REC + 2 * (int)REIN_X16_XS + 4 * 2 * Mmq16Cfg::R * 2048 + 4 * 2 * 1280;
}

// Transfers per wavefront and pair-step i, in issue order (all DMA, counted by hand as in
// mmq_fp6.h):
//   acts(i + D - 1)                   4
//   i % 2 == 0: ring(i / 2 + R - 1)   4   (two 32-row tiles)
//   i % 4 == 1: small(i / 4 + 1)     12   (two tiles x 5, and this wavefront's quarter of the xsum operands)
template <int R, int D>
struct Mmq16Waits {
    static constexpr int ring(int s) { return s % 2 == 0 ? 4 : 0; }
    static constexpr int small(int s) { return s % 4 == 1 ? 12 : 0; }
    static constexpr int cnt(int s) { return 4 + ring(s) + small(s); }
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
            const int m = sum(i - 2, i - 1);                                                   // after small(i / 4), issued last in step i - 3
            n = m < n ? m : n;
        }
        return n;
    }
};

template <unsigned N> struct ReinConst { static constexpr unsigned value = N; };

struct Mmq16Span {
    unsigned n_grp;      // 64-token groups in the image
    unsigned grp;        // this workgroup's group
    unsigned tok_end;    // rows of y
    unsigned pair_begin; // the sub-block pairs [pair_begin, pair_end) are summed, both multiples of 4;
    unsigned pair_end;   // pair_end = 0 stands for the whole contraction
    float* part;         // nullptr: the sums are the result; else a partial tile [tile][register][thread]
};

__device__ __forceinline__ rein_v8h rein_f16_weights(uint32_t w, rein_h2 sc, rein_h2 c1024, rein_h2 c64)
{
    const uint32_t w8 = w >> 8;
    const rein_h2 r0 = __builtin_bit_cast(rein_h2, (w & 0x000F000Fu) | 0x64006400u);      // 1024 + n0, 1024 + n4
    const rein_h2 r1 = __builtin_bit_cast(rein_h2, (w & 0x00F000F0u) | 0x54005400u);      //   64 + n1,   64 + n5
    const rein_h2 r2 = __builtin_bit_cast(rein_h2, (w8 & 0x000F000Fu) | 0x64006400u);
    const rein_h2 r3 = __builtin_bit_cast(rein_h2, (w8 & 0x00F000F0u) | 0x54005400u);
    const rein_h2 o0 = __builtin_elementwise_fma(r0, sc, c1024), o1 = __builtin_elementwise_fma(r1, sc, c64);
    const rein_h2 o2 = __builtin_elementwise_fma(r2, sc, c1024), o3 = __builtin_elementwise_fma(r3, sc, c64);
    return rein_v8h{o0[0], o0[1], o1[0], o1[1], o2[0], o2[1], o3[0], o3[1]};
}

__device__ __forceinline__ void rein_mmq16_tile(const uint8_t* __restrict__ w, const uint8_t* __restrict__ img,
                                                float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                unsigned rb, const Mmq16Span span)
{
    constexpr int FMT = REIN_Q4_K;
    using F = Fmt<FMT>;
    constexpr unsigned R = Mmq16Cfg::R, D = Mmq16Cfg::D;
    using Waits = Mmq16Waits<(int)R, (int)D>;
    static_assert(Waits::at(0) < 64 && Waits::at(1) < 64 && Waits::at(2) < 64 && Waits::at(3) < 64, "vmcnt holds 6 bits");
    extern __shared__ __attribute__((aligned(16))) unsigned char rein_mmq16_lds[];
    unsigned char* const raw = rein_mmq16_lds;
    typedef __attribute__((address_space(3))) const void* lptr_t;

    const unsigned lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned j = lane & 31u, h = lane >> 5;
    const unsigned n_sub = in_dim >> 5, n_pair = n_sub >> 1, n_chunk = n_sub >> 3, n_grp = span.n_grp;
    const F fmt(w, n_sub, out_dim);
    const unsigned row_base = rb * 256u + wave * 64u;

    constexpr unsigned kXs = D * REIN_X16_REC, kRing = kXs + 2u * REIN_X16_XS, kSmall = kRing + 4u * 2u * R * 2048u;
    const unsigned char* const xsbuf = raw + kXs;
    const uint4* const ring0 = reinterpret_cast<const uint4*>(raw + kRing + wave * (2u * R * 2048u));
    const uint32_t* const small0 = reinterpret_cast<const uint32_t*>(raw + kSmall + wave * (2u * 1280u));
    const unsigned lds_acts = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)raw);
    const unsigned lds_xs = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)xsbuf);
    const unsigned lds_small = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(lptr_t)small0);
    MmqWSrc<FMT> wsrc[2];                            // 32-row tile rt: its R slots are R * 2048 bytes on
    unsigned rowc[2];
#pragma unroll
    for (int rt = 0; rt < 2; rt++) {
        wsrc[rt].init(*reinterpret_cast<const MmqWLds<FMT>*>(ring0 + rt * (R * 128u)), fmt, row_base + 32u * rt, out_dim, lane);
        rowc[rt] = min(row_base + 32u * rt + j, out_dim - 1u);
    }

    const uint8_t* const xsimg = img + rein_x16_xs_offset(n_sub, span.tok_end);
    auto issue_acts = [&](unsigned pair) {
        const unsigned p = min(pair, n_pair - 1u);
        const uint8_t* src = img + ((size_t)p * n_grp + span.grp) * REIN_X16_REC;
        const unsigned buf = lds_acts + (pair % D) * REIN_X16_REC;
#pragma unroll
        for (unsigned k = 0; k < 4; k++) {
            const unsigned off = (k * 4u + wave) * 1024u;
            rein_lds_dma16(src + off + lane * 16u, buf + off);
        }
    };
    auto issue_ring = [&](unsigned stage) {
        const unsigned sb_first = min(stage * 4u, n_sub - 4u);
#pragma unroll
        for (int rt = 0; rt < 2; rt++) rein_mmq_wload<FMT>(wsrc[rt], stage % R, fmt, sb_first, n_sub);
    };
    auto issue_small = [&](unsigned chunk) {
        const unsigned sup = min(chunk, n_chunk - 1u);
#pragma unroll
        for (int rt = 0; rt < 2; rt++) {
            const unsigned dst = lds_small + rt * 1280u;
#pragma unroll
            for (unsigned k = 0; k < 4; k++) {
                const unsigned r = min(row_base + 32u * rt + 8u * k + (lane >> 3), out_dim - 1u);
                rein_lds_dma_u16(fmt.smp + (size_t)r * fmt.nsp + sup * 8u + (lane & 7u), dst + k * 256u);
            }
            rein_lds_dma_u32(fmt.ddp + (size_t)rowc[rt] * fmt.n_super + sup, dst + 1024u);
        }
        // this wavefront's quarter (512 bytes) of the superblock's xsum operands
        const uint8_t* xsrc = xsimg + ((size_t)sup * n_grp + span.grp) * REIN_X16_XS + wave * 512u;
        const unsigned xdst = lds_xs + (chunk & 1u) * REIN_X16_XS + wave * 512u;
        rein_lds_dma_u32(xsrc + lane * 4u, xdst);
        rein_lds_dma_u32(xsrc + 256u + lane * 4u, xdst + 256u);
    };

    rein_v16f acc[2][2], s1[2][2];
    rein_v16f z16;
#pragma unroll
    for (int v = 0; v < 16; v++) z16[v] = 0.0f;
#pragma unroll
    for (int rt = 0; rt < 2; rt++)
#pragma unroll
        for (int t = 0; t < 2; t++) { acc[rt][t] = z16; s1[rt][t] = z16; }

    const unsigned pb = span.pair_begin, pe = span.pair_end ? span.pair_end : n_pair;
    __syncthreads();
#pragma unroll
    for (unsigned k = 0; k + 1u < D; k++) issue_acts(pb + k);
#pragma unroll
    for (unsigned k = 0; k + 1u < R; k++) issue_ring((pb >> 1) + k);
    issue_small(pb >> 2);
    REIN_WAIT_VMCNT(0);

    const unsigned rot = j >> 1;
    float d[2] = {0.0f, 0.0f}, nd[2] = {0.0f, 0.0f};
    rein_h2 sch[2][4];                               // sc of the superblock's 8 sub-blocks as fp16, per tile
    uint32_t mpk[2][4];                              // m likewise: the weight-side operand of S2

    // Weight operands of the coming step's first sub-block, [32-row tile][kh]: steps 1..3 of a superblock find
    // them made by the step before (under its instructions), step 0 makes them itself.
    rein_v8h bq0[2][2];

    // pair-step u of superblock c
    auto step = [&](auto u_tag, const unsigned c) {
        constexpr unsigned u = decltype(u_tag)::value;
        const unsigned i = 4u * c + u;
        REIN_WAIT_VMCNT(Waits::at((int)u));
        __syncthreads();
        if (u == 0u) {
            // all small words of the superblock into registers: the buffer is free for the next one
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                const uint32_t* const small = small0 + rt * 320u;
                const uint4 lo4 = *reinterpret_cast<const uint4*>(small + j * 8u);
                const uint4 hi4 = *reinterpret_cast<const uint4*>(small + j * 8u + 4u);
                const uint32_t sm[8] = {lo4.x, lo4.y, lo4.z, lo4.w, hi4.x, hi4.y, hi4.z, hi4.w};
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    sch[rt][k] = rein_h2{(_Float16)(float)(sm[2 * k] & 0xFFu), (_Float16)(float)(sm[2 * k + 1] & 0xFFu)};
                    const rein_h2 mh = {(_Float16)(float)(sm[2 * k] >> 8), (_Float16)(float)(sm[2 * k + 1] >> 8)};
                    mpk[rt][k] = __builtin_bit_cast(uint32_t, mh);
                }
                const uint32_t dd = small[256 + lane];
                d[rt] = rein_h2f((uint16_t)(dd & 0xFFFFu));
                nd[rt] = -64.0f * rein_h2f((uint16_t)(dd >> 16));
            }
        }
        const unsigned char* const act = raw + (i % D) * REIN_X16_REC + lane * 16u;
        // nibble words of sub-block q of pair-step v of this superblock (ring slot v / 2)
        auto nib = [&](unsigned v, unsigned q, int rt) {
            const uint4* const slot = ring0 + ((v >> 1) % R) * 128u;
            return reinterpret_cast<const uint2*>(slot + rt * (R * 128u) + 4u * j + ((2u * (v & 1u) + q + rot) & 3u))[h];
        };
        // one weight operand; `word` goes through an empty asm so that the unpack stays in the stage it is
        // written in (it has no other tie to it and would be moved in front of the step's first instruction)
        auto unpack = [&](rein_v8h& out, uint32_t word, _Float16 scf) {
            asm volatile("" : "+v"(word));
            const rein_h2 sc = {scf, scf};
            out = rein_f16_weights(word, sc, sc * rein_h2{(_Float16)-1024.0f, (_Float16)-1024.0f},
                                   sc * rein_h2{(_Float16)-64.0f, (_Float16)-64.0f});
        };
        auto a_read = [&](unsigned k) {
            const unsigned q = k >> 3, op = (k >> 1) & 3u, t = k & 1u;
            return *reinterpret_cast<const rein_v8h*>(act + q * 8192u + t * 4096u + op * 1024u);
        };
        uint2 w1[2] = {nib(u, 1u, 0), nib(u, 1u, 1)}, wn[2];
        rein_v8h b1[2][2];
        rein_v8h aw[4];
        aw[0] = a_read(0); aw[1] = a_read(1); aw[2] = a_read(2);
        if (u == 0u) {
            const uint2 w0[2] = {nib(0u, 0u, 0), nib(0u, 0u, 1)};
#pragma unroll
            for (int rt = 0; rt < 2; rt++) {
                unpack(bq0[rt][0], w0[rt].x, sch[rt][0][0]);
                unpack(bq0[rt][1], w0[rt].y, sch[rt][0][0]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // Stage k: the two instructions of token operand k (k = 8 q + 2 op + t), the read of operand k + 3, and a
        // piece of the unpack of what comes next: stages 0..3 the second sub-block's operands, stages 9..12 the
        // next step's first.  The fences keep the stages as written.
#pragma unroll
        for (unsigned k = 0; k < 16; k++) {
            const unsigned q = k >> 3, op = (k >> 1) & 3u, t = k & 1u;
            if (k + 3u < 16u) aw[(k + 3u) & 3u] = a_read(k + 3u);
#pragma unroll
            for (int rt = 0; rt < 2; rt++)
                s1[rt][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aw[k & 3u], q ? b1[rt][op >> 1] : bq0[rt][op >> 1], s1[rt][t], 0, 0, 0);
            // this step's transfers go out under the instructions (in the order the wait counts assume: records,
            // ring, small words); the barrier at the top of the step has freed their buffers
            if (k == 1u) issue_acts(i + D - 1u);
            if (k == 3u && (u & 1u) == 0u) issue_ring((i >> 1) + R - 1u);
            if (k == 3u && u == 1u) issue_small(c + 1u);
            if (k < 4u) unpack(b1[k >> 1][k & 1u], (k & 1u) ? w1[k >> 1].y : w1[k >> 1].x, sch[k >> 1][u][1]);
            if (u < 3u) {
                if (k == 7u && (u & 1u)) {
                    // the next step's ring stage: behind it only this step's acts and, in step 1, the small words
                    if (u == 1u) REIN_WAIT_VMCNT(16); else REIN_WAIT_VMCNT(4);
                }
                if (k == 8u) { wn[0] = nib(u + 1u, 0u, 0); wn[1] = nib(u + 1u, 0u, 1); }
                if (k >= 9u && k < 13u) {
                    const unsigned e = k - 9u;
                    unpack(bq0[e >> 1][e & 1u], (e & 1u) ? wn[e >> 1].y : wn[e >> 1].x, sch[e >> 1][(u + 1u) & 3u][0]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (u == 3u) {
            const unsigned char* const xb = xsbuf + (c & 1u) * REIN_X16_XS;
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const rein_v8h a2 = *reinterpret_cast<const rein_v8h*>(xb + t * 1024u + lane * 16u);
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const uint4 mk = make_uint4(mpk[rt][0], mpk[rt][1], mpk[rt][2], mpk[rt][3]);
                    const rein_v16f s2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, __builtin_bit_cast(rein_v8h, mk), z16, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[rt][t][v] = fmaf(nd[rt], s2[v], fmaf(d[rt], s1[rt][t][v], acc[rt][t][v]));
                    s1[rt][t] = z16;
                }
            }
        }
    };
    for (unsigned c = pb >> 2; c < (pe >> 2); c++) {
        step(ReinConst<0>{}, c);
        step(ReinConst<1>{}, c);
        step(ReinConst<2>{}, c);
        step(ReinConst<3>{}, c);
    }
    REIN_WAIT_VMCNT(0);

    const float* const tokscale = reinterpret_cast<const float*>(img + rein_x16_scale_offset(n_sub, span.tok_end)) + span.grp * 64u;
    if (span.part) {
#pragma unroll
        for (int rt = 0; rt < 2; rt++)
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int v = 0; v < 16; v++) span.part[((rt * 2 + t) * 16 + v) * 256 + threadIdx.x] = acc[rt][t][v];
        return;
    }
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const unsigned tl = t * 32u + 8 * (v / 4) + 4 * h + (v % 4), tok = span.grp * 64u + tl;
            if (tok < span.tok_end) {
                const float ts = tokscale[tl];
#pragma unroll
                for (int rt = 0; rt < 2; rt++) {
                    const unsigned row = row_base + 32u * rt + j;
                    if (row < out_dim) y[(size_t)tok * out_dim + row] = acc[rt][t][v] * ts;
                }
            }
        }
}

// Workgroup -> (256-row block, 64-token group): workgroup i runs on XCD i % 8 and all token
// groups of a row block are dealt to the same XCD, so the block's weights are pulled from HBM
// once and re-read from that L2.  Grid: 8 * ceil(n_row_blocks / 8) * n_groups workgroups of 256.
__device__ __forceinline__ void rein_mmq16_dense(const uint8_t* __restrict__ w, const uint8_t* __restrict__ img,
                                                 float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                 unsigned p_rows)
{
    const unsigned n_rb = (out_dim + 255u) / 256u, n_grp = (p_rows + 63u) / 64u;
    const unsigned xcd = blockIdx.x & 7u, k = blockIdx.x >> 3;
    const unsigned rb = (k / n_grp) * 8u + xcd, grp = k % n_grp;
    if (rb >= n_rb) return;
    rein_mmq16_tile(w, img, y, in_dim, out_dim, rb, Mmq16Span{n_grp, grp, p_rows, 0u, 0u, nullptr});
}

#define REIN_DEFINE_MMQ16_PREP(name)                                                                \
    extern "C" __global__ __launch_bounds__(256) void name(const BlockQ8* __restrict__ xq,          \
                                                           unsigned char* __restrict__ img,         \
                                                           unsigned int n_sub, unsigned int p_rows) \
    {                                                                                               \
        rein_mmq16_prep_body(xq, img, n_sub, p_rows);                                               \
    }

#define REIN_DEFINE_MMQ16_DENSE(name)                                                               \
    extern "C" __global__ __launch_bounds__(256) REIN_MMQ_OCC void name(                            \
        const unsigned char* __restrict__ w, const unsigned char* __restrict__ img,                 \
        float* __restrict__ y, unsigned int in_dim, unsigned int out_dim, unsigned int p_rows)      \
    {                                                                                               \
        rein_mmq16_dense(w, img, y, in_dim, out_dim, p_rows);                                       \
    }
