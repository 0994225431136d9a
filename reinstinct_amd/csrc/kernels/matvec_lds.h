// Decode matvec for 2..4 activation rows with the activation rows staged in LDS.
//
// The dot4 matvec (matvec_repacked.h) reads a lane's BlockQ8 of every activation
// row straight from memory: 40-byte records at a 40-byte lane stride, three load
// instructions that each touch twenty 128-byte lines for 2.5 KB of payload.  At one
// row that hides behind the weight stream; from two rows on the vector cache spends
// more time on the activations than on the weights (per trip of R x 1 KiB of weights,
// B x 2.5 KB of activations), which is what makes two and four rows cost 1.3-2 x one.
// Here a workgroup copies the B rows into LDS once, split into planes that a lane
// reads with conflict-free 16-byte and 4-byte accesses
//   qlo[b][sb], qhi[b][sb] (16 B each: quants 0..15, 16..31), dx[b][sb], xsum[b][sb]
// and its wavefronts then walk their output rows as in the dot4 kernel.  The first
// trip's weights are requested before the copy, and every trip requests the next
// one's (or the next row group's first) before it computes, so the weight stream
// never waits for the staging.
//
// The arithmetic is the dot4 kernel's, operation for operation and in the same
// order (lane l owns sub-blocks l, l + 64, ..., fp32 partials per lane, the same
// wave reduction), so the outputs are bit-identical to rein_mv_<fmt>_r<R>_b<B>.
// No counterpart in the reference (kernels/matvec_*_repacked_batched.cpp read the
// activations from memory).
//
// Launch: block = 64 x W threads, W <= 16; dynamic shared memory = B * (in_dim/32) * 40
// bytes (at most 160 KB: B = 4 up to in_dim 32768); any grid -- wavefronts stride
// over the row groups.
#pragma once

#include "matvec_repacked.h"

template <int FMT, int R, int B>
__device__ __forceinline__ void rein_matvec_lds_body(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                     float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                     unsigned n_rows)
{
    using F = Fmt<FMT>;
    extern __shared__ uint4 rein_mvl_lds[];
    const unsigned lane = threadIdx.x & 63u;
    const unsigned wpb = blockDim.x >> 6;
    const unsigned n_sub = in_dim >> 5;
    const F fmt(w, n_sub, out_dim);
    const unsigned n_groups = (out_dim + R - 1) / R;
    const unsigned rmax = out_dim - 1, bmax = n_rows - 1;
    const unsigned stride = gridDim.x * wpb;
    uint4* qlo = rein_mvl_lds;
    uint4* qhi = rein_mvl_lds + (size_t)B * n_sub;
    float* dxs = reinterpret_cast<float*>(rein_mvl_lds + 2u * B * n_sub);
    float* xss = dxs + (size_t)B * n_sub;

    unsigned g = blockIdx.x * wpb + (threadIdx.x >> 6);
    // A wavefront's trips in order: position (row group, first sub-block); the one after the last trip of a row
    // group is the first of the wavefront's next row group.  Lanes past the end of a row re-read its last
    // sub-block (loads stay unconditional) and are zeroed through dx / xsum; a position past the last row group
    // reads the last one and is never used.
    struct Pos { unsigned g, sb0; };
    auto nxt = [&](Pos p) {
        Pos q;
        const bool last = p.sb0 + 64u >= n_sub;
        q.g = last ? p.g + stride : p.g;
        q.sb0 = last ? 0u : p.sb0 + 64u;
        return q;
    };
    auto request = [&](typename F::Raw (&r)[R], Pos p) {
        const unsigned row0 = min(p.g, n_groups - 1) * R;
        const unsigned sb = p.sb0 + lane < n_sub ? p.sb0 + lane : n_sub - 1;
#pragma unroll
        for (int rr = 0; rr < R; rr++) r[rr] = fmt.load(min(row0 + rr, rmax), sb);
    };
    Pos p, q;
    p.g = g; p.sb0 = 0u;
    q = nxt(p);
    typename F::Raw raw[R];
    request(raw, p);

    for (unsigned e = threadIdx.x; e < B * n_sub; e += blockDim.x) {
        const unsigned b = e / n_sub, sb = e - b * n_sub;
        const BlockQ8 v = xq[(size_t)min(b, bmax) * n_sub + sb];
        qlo[e] = make_uint4((unsigned)v.qs[0], (unsigned)v.qs[1], (unsigned)v.qs[2], (unsigned)v.qs[3]);
        qhi[e] = make_uint4((unsigned)v.qs[4], (unsigned)v.qs[5], (unsigned)v.qs[6], (unsigned)v.qs[7]);
        dxs[e] = v.d;
        xss[e] = v.xsum;
    }
    __syncthreads();

    float acc[R][B];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int b = 0; b < B; b++) acc[r][b] = 0.0f;

    // one trip: the weights that arrived in `raw`, whose registers then take the request for the next position.
    // (Two register sets taking turns, each refilled with the trip after next, were measured on this kernel: 0.85-1.0
    // of this form's speed at every shape and format.)
    while (p.g < n_groups) {
        const bool live = p.sb0 + lane < n_sub;
        const unsigned sb = live ? p.sb0 + lane : n_sub - 1;
        typename F::Raw cur[R];
#pragma unroll
        for (int r = 0; r < R; r++) cur[r] = raw[r];
        request(raw, q);
        SubW sw[R];
#pragma unroll
        for (int r = 0; r < R; r++) F::unpack(cur[r], sw[r]);
#pragma unroll
        for (int b = 0; b < B; b++) {
            const uint4 lo = qlo[b * n_sub + sb], hi = qhi[b * n_sub + sb];
            const float d0 = dxs[b * n_sub + sb], s0 = xss[b * n_sub + sb];
            const float d = live ? d0 : 0.0f, xsum = live ? s0 : 0.0f;
            const int qv[8] = {(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            XSums xs;
            if (F::kNeedsXSums) xs = rein_xsums(qv);
            else { xs.lo = 0; xs.hi = 0; }
#pragma unroll
            for (int r = 0; r < R; r++) {
                int i0 = 0, i1 = 0;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    i0 = rein_dot4(sw[r].w[j], qv[j], i0);
                    i1 = rein_dot4(sw[r].w[j + 4], qv[j + 4], i1);
                }
                acc[r][b] += F::term(sw[r], i0, i1, d, xsum, xs);
            }
        }
        if (p.sb0 + 64u >= n_sub) {                       // the row group is complete
            const unsigned row0 = p.g * R;
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int b = 0; b < B; b++) {
                    const float s = rein_wave_sum(acc[r][b]);
                    if (lane == 0 && row0 + r < out_dim && (unsigned)b < n_rows) y[(size_t)b * out_dim + row0 + r] = s;
                    acc[r][b] = 0.0f;
                }
        }
        p = q;
        q = nxt(q);
    }
}

// name(w, xq[n_rows][n_sub], y[n_rows][out_dim], in_dim, out_dim, n_rows), n_rows <= B
#define REIN_DEFINE_MATVEC_LDS(name, FMT, R, B)                                                   \
    extern "C" __global__ __launch_bounds__(1024) void name(REIN_MATVEC_ARGS, unsigned int n_rows) \
    {                                                                                             \
        rein_matvec_lds_body<FMT, R, B>(w, xq, y, in_dim, out_dim, n_rows);                       \
    }
