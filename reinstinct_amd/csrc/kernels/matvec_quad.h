// Batched decode matvec on the small int8 matrix instruction: 3 to 8 activation rows (the
// first kernel below; the library picks it for the formats whose weight unpack is expensive,
// Q6_K, Q5_K, IQ4_XS) and 3 to 32 rows with the activation rows staged in LDS (the second
// kernel, every format).
//
// On the dot4 matvec every activation row costs eight v_dot4_i32_i8 per weight sub-block
// and lane, and the weight unpack is repeated per output row.  v_mfma_i32_4x4x4_16b_i8
// multiplies, in each of the 16 four-lane blocks of a wavefront, a 4x4 int8 matrix A
// (lane j of the block supplies row j: four consecutive k) with a 4x4 matrix B (lane j
// supplies column j) in 8 cycles (measured), so the dots of four weight rows with four
// activation rows cost what one row pair costs on dot4, and every (row, sub-block) is
// unpacked exactly once.  What remains per output is the fp32 scaling, as in every
// formulation of this path.  Mapping:
//
//   block  b = lane / 4   -> sub-block b (+16 per trip) of the contraction
//   lane   j = lane % 4   -> weight row 4g + j  (A side)  and  activation row 4t + j  (B side)
//
// so lane (b, j) works on exactly one (row, sub-block) of the weights -- 16 bytes of the
// nibble plane plus its scale words, through the same Fmt<FMT>::load / unpack as the dot4
// kernels -- and one BlockQ8 of one activation row.  Eight chained instructions walk the
// 32 k of the sub-block; D register r of lane j then holds the int32 dot of weight row r
// with activation row j.  The scales of the four rows are spread over the block with DPP
// quad broadcasts, the fp32 term is the format's own (Fmt<FMT>::term), partial sums over
// sub-blocks stay in registers and are reduced across the 16 blocks at the end.
//
// The integer offsets of Q6_K (-32) and Q4_0 (-8) are folded into the weight bytes, which
// gives the same integers as the dot4 kernels' "dot - offset * sum of activation quants".
//
// A wavefront owns four output rows and NT groups of four activation rows; weights are read
// once per wavefront whatever NT.  Correct for any grid (grid-stride over row groups); the
// block must be 256 threads.  No counterpart in the reference, whose
// batched kernels are dot4 loops (kernels/matvec_*_repacked_batched.cpp); same arguments.
#pragma once

#include "rein_formats.h"

typedef int rein_quad_v4i __attribute__((ext_vector_type(4)));

template <int FMT> __device__ __forceinline__ int rein_fold_offset(int w)
{
    if constexpr (FMT == REIN_Q6_K) return rein_sub_bytes((uint32_t)w, 0x20202020u);
    else if constexpr (FMT == REIN_Q4_0) return rein_sub_bytes((uint32_t)w, 0x08080808u);
    else return w;
}

// value of lane R of every four-lane block, in all four lanes of the block
template <int R> __device__ __forceinline__ float rein_quad_bcast(float v)
{
    return rein_dpp_f32<R * 0x55>(0.0f, v);
}

// One trip of a wavefront through LDS.  Memory wants lane l to read row l / 16, sub-block
// l % 16 (16 lanes x 16 B contiguous per row and load); the matrix instruction wants lane
// 4b + j to hold row j, sub-block b.  Each wavefront turns its 4 x 16 tile of 16-byte
// entries through a private LDS image: entry e is stored at e + 4 (e / 16), which makes
// both the row-major store and the column-major load conflict-free (a quarter-wave pass
// of 16 lanes covers all 64 banks once).  LDS operations of one wavefront execute in
// order, so no barrier is involved.
template <int FMT, int NT>
struct QuadStage {
    static constexpr int kRawParts = (sizeof(typename Fmt<FMT>::Raw) + 15) / 16;
    uint4 raw[kRawParts][76];
    uint4 qs[NT][2][76];
    uint2 hdr[NT][76];
};

template <int FMT> struct QuadRawBits {
    static constexpr int kParts = (sizeof(typename Fmt<FMT>::Raw) + 15) / 16;
    uint4 p[kParts];
};

template <int FMT>
__device__ __forceinline__ QuadRawBits<FMT> rein_quad_raw_bits(const typename Fmt<FMT>::Raw& r)
{
    QuadRawBits<FMT> b;
#pragma unroll
    for (int i = 0; i < QuadRawBits<FMT>::kParts; i++) b.p[i] = make_uint4(0u, 0u, 0u, 0u);
    __builtin_memcpy(&b, &r, sizeof(r));
    return b;
}

struct QuadAct {
    uint2 hdr;           // fp32 d, fp32 xsum
    uint4 lo, hi;        // quants 0-15, 16-31
};

template <int FMT, int NT>
__device__ __forceinline__ void rein_matvec_quad_body(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                      float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                      unsigned n_rows)
{
    using F = Fmt<FMT>;
    using Raw = typename F::Raw;
    constexpr bool kTwo = F::kDotParts == 2;          // Q6_K: one scale per 16 weights
    constexpr int kParts = QuadRawBits<FMT>::kParts;
    __shared__ QuadStage<FMT, NT> stages[4];
    if (blockDim.x != 256u) return;                   // four wavefronts, four LDS images
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned j = lane & 3u, blk = lane >> 2;    // compute side: row / activation row j, sub-block slot blk
    const unsigned lr = lane >> 4, ls = lane & 15u;   // memory side: row lr, sub-block slot ls
    const unsigned put = lane + 4u * lr;              // entry 16 lr + ls
    const unsigned get = 16u * j + blk + 4u * j;      // entry 16 j + blk
    QuadStage<FMT, NT>& st = stages[wave];
    const unsigned n_sub = in_dim >> 5;
    const F fmt(w, n_sub, out_dim);
    const unsigned n_groups = (out_dim + 3u) / 4u;
    const XSums no_xs = {0, 0};

    for (unsigned g = blockIdx.x * 4u + wave; g < n_groups; g += gridDim.x * 4u) {
        const unsigned row = min(g * 4u + lr, out_dim - 1u);
        float acc[NT][4];
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[t][r] = 0.0f;

        Raw rq;
        QuadAct aq[NT];
        auto fetch = [&](Raw& raw, QuadAct (&act)[NT], unsigned sb0) {
            const unsigned sb = min(sb0 + ls, n_sub - 1u);             // loads stay unconditional
            raw = fmt.load(row, sb);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const BlockQ8* p = xq + (size_t)min(4u * t + lr, n_rows - 1u) * n_sub + sb;
                act[t].hdr = *reinterpret_cast<const uint2*>(p);
                act[t].lo = make_uint4((uint32_t)p->qs[0], (uint32_t)p->qs[1], (uint32_t)p->qs[2], (uint32_t)p->qs[3]);
                act[t].hi = make_uint4((uint32_t)p->qs[4], (uint32_t)p->qs[5], (uint32_t)p->qs[6], (uint32_t)p->qs[7]);
            }
        };
        auto step = [&](Raw& raw, QuadAct (&act)[NT], unsigned sb0) {
            // through LDS: what lane (lr, ls) fetched goes to lane (blk, j)
            const QuadRawBits<FMT> bits = rein_quad_raw_bits<FMT>(raw);
#pragma unroll
            for (int i = 0; i < kParts; i++) st.raw[i][put] = bits.p[i];
#pragma unroll
            for (int t = 0; t < NT; t++) {
                st.hdr[t][put] = act[t].hdr;
                st.qs[t][0][put] = act[t].lo;
                st.qs[t][1][put] = act[t].hi;
            }
            // The load registers are free again: request the next trip now, so that it is in
            // flight while this one is read back and multiplied (past the end the fetch repeats
            // the last sub-blocks and is never used: no load sits under a branch).  The
            // scheduling barriers pin that order; left alone the compiler sinks the loads to
            // where their results are needed and the kernel loses a third of its speed (measured,
            // as were the placements behind the read-back and behind the arithmetic: both slower).
            __builtin_amdgcn_sched_barrier(0);
            fetch(raw, act, sb0 + 16u);
            __builtin_amdgcn_sched_barrier(0);
            QuadRawBits<FMT> mine;
#pragma unroll
            for (int i = 0; i < kParts; i++) mine.p[i] = st.raw[i][get];
            QuadAct ma[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) {
                ma[t].hdr = st.hdr[t][get];
                ma[t].lo = st.qs[t][0][get];
                ma[t].hi = st.qs[t][1][get];
            }

            Raw my;
            __builtin_memcpy(&my, &mine, sizeof(my));
            SubW sw;
            F::unpack(my, sw);
            const bool live = sb0 + blk < n_sub;
            int a[8];
#pragma unroll
            for (int k = 0; k < 8; k++) a[k] = rein_fold_offset<FMT>(sw.w[k]);
            // the scales of the block's four rows, in every lane of the block
            float s0[4], s1[4];
            s0[0] = rein_quad_bcast<0>(sw.s0); s0[1] = rein_quad_bcast<1>(sw.s0);
            s0[2] = rein_quad_bcast<2>(sw.s0); s0[3] = rein_quad_bcast<3>(sw.s0);
            s1[0] = rein_quad_bcast<0>(sw.s1); s1[1] = rein_quad_bcast<1>(sw.s1);
            s1[2] = rein_quad_bcast<2>(sw.s1); s1[3] = rein_quad_bcast<3>(sw.s1);
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const bool on = live && 4u * t + j < n_rows;
                const float dx = on ? __builtin_bit_cast(float, ma[t].hdr.x) : 0.0f;
                const float xsum = on ? __builtin_bit_cast(float, ma[t].hdr.y) : 0.0f;
                const int q[8] = {(int)ma[t].lo.x, (int)ma[t].lo.y, (int)ma[t].lo.z, (int)ma[t].lo.w,
                                  (int)ma[t].hi.x, (int)ma[t].hi.y, (int)ma[t].hi.z, (int)ma[t].hi.w};
                rein_quad_v4i d0 = {0, 0, 0, 0}, d1 = {0, 0, 0, 0};
#pragma unroll
                for (int k = 0; k < 4; k++) d0 = __builtin_amdgcn_mfma_i32_4x4x4i8(a[k], q[k], d0, 0, 0, 0);
                if (kTwo) {
#pragma unroll
                    for (int k = 4; k < 8; k++) d1 = __builtin_amdgcn_mfma_i32_4x4x4i8(a[k], q[k], d1, 0, 0, 0);
                } else {
#pragma unroll
                    for (int k = 4; k < 8; k++) d0 = __builtin_amdgcn_mfma_i32_4x4x4i8(a[k], q[k], d0, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    SubW sc;
                    sc.s0 = s0[r];
                    sc.s1 = s1[r];
                    acc[t][r] += F::term(sc, d0[r], d1[r], dx, xsum, no_xs);
                }
            }
        };

        // One trip (16 sub-blocks x 4 rows, 1 KiB of the nibble plane) per iteration and one
        // trip of loads in flight per wavefront; the other wavefronts of the SIMD cover the rest
        // of the latency.  Deeper register queues were measured and lose to the registers they
        // cost.
        fetch(rq, aq, 0u);
        for (unsigned sb0 = 0; sb0 < n_sub; sb0 += 16u) step(rq, aq, sb0);

        // sum over the 16 blocks (lane bits 2..5); lanes 0..3 (block 0) store
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float v = acc[t][r];
                v += __shfl_xor(v, 4);
                v += __shfl_xor(v, 8);
                v += __shfl_xor(v, 16);
                v += __shfl_xor(v, 32);
                const unsigned tok = 4u * t + j, orow = g * 4u + r;
                if (blk == 0u && tok < n_rows && orow < out_dim) y[(size_t)tok * out_dim + orow] = v;
            }
    }
}

// name(w, xq[n_rows][n_sub], y[n_rows][out_dim], in_dim, out_dim, n_rows), n_rows <= 4 * NT
#define REIN_DEFINE_MATVEC_QUAD(name, FMT, NT)                                                    \
    extern "C" __global__ __launch_bounds__(256) void name(                                       \
        const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq, float* __restrict__ y,    \
        unsigned int in_dim, unsigned int out_dim, unsigned int n_rows)                           \
    {                                                                                             \
        rein_matvec_quad_body<FMT, NT>(w, xq, y, in_dim, out_dim, n_rows);                        \
    }

// ---- the same kernel with the activation rows staged in LDS once per workgroup ----------------------
// In the kernel above a lane fetches one BlockQ8 per group of four activation rows and trip from memory
// (40-byte records at a 40-byte stride) and hands it to the lane that needs it through LDS, like the
// weights: at eight rows that is five times the weight bytes through the vector cache, plus six LDS
// stores per trip.  Here the workgroup (up to 16 wavefronts) copies the 4*NT activation rows into LDS
// once, as planes (quants 0..15, quants 16..31, {d, xsum}) whose row stride is 4 mod 16 entries, so that
// the compute-side lane (block b, row j) reads its operand at (4t + j) * stride + sub-block directly and a
// quarter-wave pass covers 64 different banks.  Only the weights still take the trip through the
// wavefront's private LDS image.  A trip requests the next trip's weights (or the first trip of the
// wavefront's next row group) before it computes.  Same arithmetic in the same order as the kernel above (the
// compiler's choice of fused multiply-adds may differ between the two, so the last bits may).
//
// A contraction whose rows do not fit the LDS is staged in phases of `phase_sub` sub-blocks (a multiple
// of 16): every wavefront then owns at most ONE row group (the launch has at least as many wavefronts as
// row groups), keeps its partial sums in registers across the phases, and the workgroup re-stages between
// two barriers that every wavefront reaches, with or without a row group.  phase_sub >= in_dim / 32 is the
// single-phase form, in which -- with slices == 1 -- wavefronts may stride over several row groups.
//
// A matrix with few rows has few row groups (5120 rows: 1280, five per CU), each with one trip of weights
// in flight: a latency-bound launch.  With `slices` = S > 1 wavefront w of the workgroup takes row group
// w / S and every S-th trip of its contraction, from trip w % S on; the S partial sums meet in LDS (in the
// wavefronts' weight images) and the first slice's wavefront adds them in slice order, so the result does
// not depend on timing (it differs in the last bits from the S = 1 order).  Again one row group per
// wavefront at most; with phases, phase_sub is a multiple of 16 * S, so that a wavefront's next trip is
// the same sub-blocks whether or not a phase boundary lies in between.
// Launch: block = 64 x W threads (W <= 16, a multiple of S), dynamic shared memory =
//   4*NT * stride * 40 + W * kParts * 76 * 16 bytes, stride = n + ((20 - n % 16) % 16) for
//   n = min(in_dim / 32, phase_sub); grid >= ceil(row groups / (W / S)) unless single-phase with S = 1.
template <int FMT, int NT>
__device__ __forceinline__ void rein_matvec_quad_lds_body(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                          float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                          unsigned n_rows, unsigned phase_sub, unsigned slices, unsigned depth)
{
    using F = Fmt<FMT>;
    using Raw = typename F::Raw;
    constexpr bool kTwo = F::kDotParts == 2;
    constexpr int kParts = QuadRawBits<FMT>::kParts;
    constexpr unsigned T = 4u * NT;
    // the second register set of weights (depth 2) exists for 3-8 rows only: at 16 and 32 rows the code of its loops costs
    // the one-set loops registers (32 rows 17408 -> 5120: 57 -> 64 us for Q4_K, 131 -> 159 for Q6_K with it compiled in)
    constexpr bool kTwoSets = NT <= 2;
    static_assert(kParts * 76 * 16 >= NT * 16 * 4, "a wavefront's partial sums go through its weight image");
    extern __shared__ uint4 rein_mvql_lds[];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, wpb = blockDim.x >> 6;
    const unsigned j = lane & 3u, blk = lane >> 2;
    const unsigned lr = lane >> 4, ls = lane & 15u;
    const unsigned put = lane + 4u * lr;
    const unsigned get = 16u * j + blk + 4u * j;
    const unsigned n_sub = in_dim >> 5;
    const unsigned n_stage = min(n_sub, phase_sub);                   // sub-blocks staged at a time
    const unsigned stride = n_stage + ((20u - (n_stage & 15u)) & 15u);
    uint4* xlo = rein_mvql_lds;
    uint4* xhi = xlo + T * stride;
    uint2* xhd = reinterpret_cast<uint2*>(xhi + T * stride);
    uint4* stage = reinterpret_cast<uint4*>(xhd + T * stride) + wave * (kParts * 76u);
    const F fmt(w, n_sub, out_dim);
    const unsigned n_groups = (out_dim + 3u) / 4u;
    const unsigned step = gridDim.x * wpb;
    const XSums no_xs = {0, 0};

    // sub-blocks [first, first + count) of every activation row -> planes
    auto stage_x = [&](unsigned first, unsigned count) {
        for (unsigned e = threadIdx.x; e < T * count; e += blockDim.x) {
            const unsigned t = e / count, sb = e - t * count;
            const BlockQ8 v = xq[(size_t)min(t, n_rows - 1u) * n_sub + first + sb];
            xlo[t * stride + sb] = make_uint4((unsigned)v.qs[0], (unsigned)v.qs[1], (unsigned)v.qs[2], (unsigned)v.qs[3]);
            xhi[t * stride + sb] = make_uint4((unsigned)v.qs[4], (unsigned)v.qs[5], (unsigned)v.qs[6], (unsigned)v.qs[7]);
            xhd[t * stride + sb] = make_uint2(__builtin_bit_cast(unsigned, v.d), __builtin_bit_cast(unsigned, v.xsum));
        }
    };

    Raw rq;
    // one trip of row group g: 16 sub-blocks from sb0, whose activations sit at plane index x0 + block; the
    // wavefront's next trip starts `ahead` sub-blocks further on
    // (the weights of the trip arrive in rqx; the same registers then take the request for sub-blocks psb.. of row group png)
    auto trip_on = [&](Raw& rqx, unsigned sb0, unsigned x0, unsigned png, unsigned psb, float (&acc)[NT][4]) {
        const QuadRawBits<FMT> bits = rein_quad_raw_bits<FMT>(rqx);
#pragma unroll
        for (int i = 0; i < kParts; i++) stage[i * 76 + put] = bits.p[i];
        // the load registers are free again: a later trip (of this row group, or of the wavefront's next one) is
        // requested now, pinned between scheduling barriers as in the kernel above
        __builtin_amdgcn_sched_barrier(0);
        {
            const unsigned nrow = min(min(png, n_groups - 1u) * 4u + lr, out_dim - 1u);
            rqx = fmt.load(nrow, min(psb + ls, n_sub - 1u));
        }
        __builtin_amdgcn_sched_barrier(0);
        QuadRawBits<FMT> mine;
#pragma unroll
        for (int i = 0; i < kParts; i++) mine.p[i] = stage[i * 76 + get];
        Raw my;
        __builtin_memcpy(&my, &mine, sizeof(my));
        SubW sw;
        F::unpack(my, sw);
        const bool live = sb0 + blk < n_sub;
        const unsigned sbx = x0 + min(blk, n_sub - 1u - sb0);
        int a[8];
#pragma unroll
        for (int k = 0; k < 8; k++) a[k] = rein_fold_offset<FMT>(sw.w[k]);
        float s0[4], s1[4];
        s0[0] = rein_quad_bcast<0>(sw.s0); s0[1] = rein_quad_bcast<1>(sw.s0);
        s0[2] = rein_quad_bcast<2>(sw.s0); s0[3] = rein_quad_bcast<3>(sw.s0);
        s1[0] = rein_quad_bcast<0>(sw.s1); s1[1] = rein_quad_bcast<1>(sw.s1);
        s1[2] = rein_quad_bcast<2>(sw.s1); s1[3] = rein_quad_bcast<3>(sw.s1);
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const unsigned at = (4u * t + j) * stride + sbx;
            const uint4 lo = xlo[at], hi = xhi[at];
            const uint2 hd = xhd[at];
            const bool on = live && 4u * t + j < n_rows;
            const float dx = on ? __builtin_bit_cast(float, hd.x) : 0.0f;
            const float xsum = on ? __builtin_bit_cast(float, hd.y) : 0.0f;
            const int q[8] = {(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            rein_quad_v4i d0 = {0, 0, 0, 0}, d1 = {0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < 4; k++) d0 = __builtin_amdgcn_mfma_i32_4x4x4i8(a[k], q[k], d0, 0, 0, 0);
            if (kTwo) {
#pragma unroll
                for (int k = 4; k < 8; k++) d1 = __builtin_amdgcn_mfma_i32_4x4x4i8(a[k], q[k], d1, 0, 0, 0);
            } else {
#pragma unroll
                for (int k = 4; k < 8; k++) d0 = __builtin_amdgcn_mfma_i32_4x4x4i8(a[k], q[k], d0, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                SubW sc;
                sc.s0 = s0[r];
                sc.s1 = s1[r];
                acc[t][r] += F::term(sc, d0[r], d1[r], dx, xsum, no_xs);
            }
        }
    };
    auto trip = [&](unsigned g, unsigned sb0, unsigned x0, unsigned ahead, float (&acc)[NT][4]) {
        const bool last = sb0 + ahead >= n_sub;
        trip_on(rq, sb0, x0, last ? g + step : g, last ? 0u : sb0 + ahead, acc);
    };
    // sum over the 16 blocks (lane bits 2..5); lanes 0..3 (block 0) store
    auto finish = [&](unsigned g, float (&acc)[NT][4]) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float v = acc[t][r];
                v += __shfl_xor(v, 4);
                v += __shfl_xor(v, 8);
                v += __shfl_xor(v, 16);
                v += __shfl_xor(v, 32);
                const unsigned tok = 4u * t + j, orow = g * 4u + r;
                if (blk == 0u && tok < n_rows && orow < out_dim) y[(size_t)tok * out_dim + orow] = v;
            }
    };

    float acc[NT][4];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[t][r] = 0.0f;
    if (phase_sub >= n_sub && slices <= 1u) {
        unsigned g = blockIdx.x * wpb + wave;
        {   // the first trip's weights are on their way while the activations are staged
            const unsigned row = min(min(g, n_groups - 1u) * 4u + lr, out_dim - 1u);
            rq = fmt.load(row, min(ls, n_sub - 1u));
        }
        if (kTwoSets && depth >= 2u) {
            // two trips of weights in flight per wavefront: two register sets take turns, each refilled with the trip
            // after next as soon as its own has gone to LDS
            struct Pos { unsigned g, sb0; };
            auto nxt = [&](Pos p) { Pos q; const bool last = p.sb0 + 16u >= n_sub; q.g = last ? p.g + step : p.g; q.sb0 = last ? 0u : p.sb0 + 16u; return q; };
            Pos p; p.g = g; p.sb0 = 0u;
            Pos q = nxt(p), r2 = nxt(q);
            Raw rq2;
            {
                const unsigned row = min(min(q.g, n_groups - 1u) * 4u + lr, out_dim - 1u);
                rq2 = fmt.load(row, min(q.sb0 + ls, n_sub - 1u));
            }
            stage_x(0u, n_sub);
            __syncthreads();
            auto one = [&](Raw& rqx) {
                trip_on(rqx, p.sb0, p.sb0, r2.g, r2.sb0, acc);
                if (p.sb0 + 16u >= n_sub) {
                    finish(p.g, acc);
#pragma unroll
                    for (int t = 0; t < NT; t++)
#pragma unroll
                        for (int r = 0; r < 4; r++) acc[t][r] = 0.0f;
                }
                p = q; q = r2; r2 = nxt(r2);
            };
            while (p.g < n_groups) {
                one(rq);
                if (!(p.g < n_groups)) break;
                one(rq2);
            }
            return;
        }
        stage_x(0u, n_sub);
        __syncthreads();
        for (; g < n_groups; g += step) {
            for (unsigned sb0 = 0; sb0 < n_sub; sb0 += 16u) trip(g, sb0, sb0, 16u, acc);
            finish(g, acc);
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[t][r] = 0.0f;
        }
    } else {
        // one (row group, slice) per wavefront: wavefront w of the workgroup takes row group w / slices and every
        // slices-th trip of it, from trip w % slices on
        const unsigned gpb = wpb / slices;                       // row groups per workgroup
        const unsigned slice = wave % slices;
        const unsigned g = blockIdx.x * gpb + wave / slices;
        const bool has = wave < gpb * slices && g < n_groups;    // wave-uniform
        const unsigned ahead = 16u * slices;
        const bool two = kTwoSets && depth >= 2u;                // two register sets of weights taking turns
        Raw rq2;
        {
            const unsigned row = min(min(g, n_groups - 1u) * 4u + lr, out_dim - 1u);
            rq = fmt.load(row, min(16u * slice + ls, n_sub - 1u));
            if (two) rq2 = fmt.load(row, min(16u * slice + ahead + ls, n_sub - 1u));
        }
        bool odd = false;
        for (unsigned ph0 = 0; ph0 < n_sub; ph0 += phase_sub) {
            const unsigned count = min(phase_sub, n_sub - ph0);
            if (ph0 != 0u) __syncthreads();            // every wavefront is done with the previous phase's planes
            stage_x(ph0, count);
            __syncthreads();
            if (has && !two) {
                for (unsigned sb0 = ph0 + 16u * slice; sb0 < ph0 + count; sb0 += ahead) trip(g, sb0, sb0 - ph0, ahead, acc);
            } else if (has) {
                for (unsigned sb0 = ph0 + 16u * slice; sb0 < ph0 + count; sb0 += ahead) {
                    if (!odd) trip_on(rq, sb0, sb0 - ph0, g, sb0 + 2u * ahead, acc);
                    else trip_on(rq2, sb0, sb0 - ph0, g, sb0 + 2u * ahead, acc);
                    odd = !odd;
                }
            }
        }
        if (slices <= 1u) {
            if (has) finish(g, acc);
        } else {
            // The slices' partial sums meet in LDS (each wavefront's weight image has room for its 16 x NT
            // values) and are added in slice order by the first slice's wavefront: the result does not depend on timing.
            float* part = reinterpret_cast<float*>(stage);
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float v = acc[t][r];
                    v += __shfl_xor(v, 4);
                    v += __shfl_xor(v, 8);
                    v += __shfl_xor(v, 16);
                    v += __shfl_xor(v, 32);
                    if (blk == 0u) part[(t * 4 + r) * 4 + j] = v;
                }
            __syncthreads();
            if (has && slice == 0u) {
                for (unsigned e = lane; e < 16u * NT; e += 64u) {
                    float v = part[e];
                    for (unsigned k = 1; k < slices; k++) v += part[k * (kParts * 76u * 4u) + e];
                    const unsigned t = e >> 4, r = (e >> 2) & 3u, jj = e & 3u;
                    const unsigned tok = 4u * t + jj, orow = g * 4u + r;
                    if (tok < n_rows && orow < out_dim) y[(size_t)tok * out_dim + orow] = v;
                }
            }
        }
    }
}

// name(w, xq[n_rows][n_sub], y[n_rows][out_dim], in_dim, out_dim, n_rows, phase_sub, slices, depth), n_rows <= 4 * NT
// (32 rows: by default for eight wavefronts per workgroup at most, so that the 32 partial sums and the eight activation
// tiles of a trip stay in registers; REIN_DEFINE_MATVEC_QUAD_LDS_BOUND builds it for sixteen wavefronts' 128 registers as
// well, where the heavier formats spill)
#define REIN_DEFINE_MATVEC_QUAD_LDS(name, FMT, NT) REIN_DEFINE_MATVEC_QUAD_LDS_BOUND(name, FMT, NT, (NT >= 8 ? 512 : 1024))
#define REIN_DEFINE_MATVEC_QUAD_LDS_BOUND(name, FMT, NT, BOUND)                                   \
    extern "C" __global__ __launch_bounds__(BOUND) void name(                                     \
        const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq, float* __restrict__ y,    \
        unsigned int in_dim, unsigned int out_dim, unsigned int n_rows, unsigned int phase_sub,   \
        unsigned int slices, unsigned int depth)                                                  \
    {                                                                                             \
        rein_matvec_quad_lds_body<FMT, NT>(w, xq, y, in_dim, out_dim, n_rows, phase_sub, slices,  \
                                           depth);                                                \
    }
