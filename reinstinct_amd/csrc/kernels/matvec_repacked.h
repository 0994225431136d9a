// Decode matvec over repacked-v2 weights, 1..B activation rows, wave64, HBM-bound.
//
//   y[b][row] = sum over 32-weight sub-blocks of Fmt::term(int8 dot, scales)
//
// One wavefront owns R consecutive output rows at a time and walks the
// contraction with lane l on sub-blocks l, l+64, ...: every load instruction of
// the nibble / quant plane is 64 lanes x 16 contiguous bytes (one 1 KiB burst),
// the scale plane 64 x 2 B.  Each weight sub-block is read once and dotted with
// all B activation rows (v_dot4_i32_i8), partials are kept per lane in fp32 and
// summed across the wave with DPP at the end.  No LDS, no MFMA.
//
// Wave -> row-group mapping is a grid-stride loop, so the kernel is correct for
// any (grid, block) with blockDim.x a multiple of 64.  In particular the
// reference launches -- grid ceil(out/8) x 256 threads with R = 2
// (src/runtime/qwen35.rs:2232-2280), grid ceil(out/R) x 64 threads for Q8_0 --
// give each wave exactly one group.  The tuned host launcher picks R and the
// grid for 256 CUs itself.
//
// Replaces the bodies of kernels/matvec_{q4_0,q4k,q5k,q6k,q8_0,iq4xs}_repacked.cpp
// and kernels/matvec_*_repacked_batched.cpp of the reference.
#pragma once

#include "rein_formats.h"

template <int B>
struct XBlocks {
    float dx[B];
    float xsum[B];
    int   q[B][8];
};

// The row groups first, first + step, ... of one matrix, walked by the calling wavefront.
template <int FMT, int R, int B, int U = 1>
__device__ __forceinline__ void rein_matvec_span(const uint8_t* __restrict__ w,
                                                 const BlockQ8* __restrict__ xq,
                                                 float* __restrict__ y,
                                                 unsigned in_dim, unsigned out_dim, unsigned n_rows,
                                                 unsigned first, unsigned step)
{
    using F = Fmt<FMT>;
    const unsigned lane  = threadIdx.x & 63u;
    const unsigned n_sub = in_dim >> 5;
    const F fmt(w, n_sub, out_dim);

    const unsigned n_groups = (out_dim + R - 1) / R;
    const unsigned rmax = out_dim - 1;
    const unsigned bmax = n_rows - 1;

    for (unsigned g = first; g < n_groups; g += step) {
        const unsigned row0 = g * R;
        float acc[R][B];
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int b = 0; b < B; b++) acc[r][b] = 0.0f;

        // U trips of 64 sub-blocks per iteration: every load of the iteration is
        // issued before the first dot, so U*R weight bursts per wave are in flight.
        for (unsigned sb0 = 0; sb0 < n_sub; sb0 += 64 * U) {
            bool     live[U];
            unsigned sb[U];
            typename F::Raw raw[U][R];
            XBlocks<B> xb[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                // Lanes past the end of the row re-read the last sub-block (loads
                // stay unconditional) and are zeroed through dx/xsum below.
                live[u] = sb0 + 64 * u + lane < n_sub;
                sb[u]   = live[u] ? sb0 + 64 * u + lane : n_sub - 1;
#pragma unroll
                for (int r = 0; r < R; r++) raw[u][r] = fmt.load(min(row0 + r, rmax), sb[u]);
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int b = 0; b < B; b++) {
                    const BlockQ8* p = xq + (size_t)min((unsigned)b, bmax) * n_sub + sb[u];
                    const float d = p->d, xs = p->xsum;
                    xb[u].dx[b]   = live[u] ? d : 0.0f;
                    xb[u].xsum[b] = live[u] ? xs : 0.0f;
#pragma unroll
                    for (int j = 0; j < 8; j++) xb[u].q[b][j] = p->qs[j];
                }

#pragma unroll
            for (int u = 0; u < U; u++) {
                XSums xs[B];
#pragma unroll
                for (int b = 0; b < B; b++) {
                    if (F::kNeedsXSums) xs[b] = rein_xsums(xb[u].q[b]);
                    else { xs[b].lo = 0; xs[b].hi = 0; }
                }
#pragma unroll
                for (int r = 0; r < R; r++) {
                    SubW sw;
                    F::unpack(raw[u][r], sw);
#pragma unroll
                    for (int b = 0; b < B; b++) {
                        int i0 = 0, i1 = 0;
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            i0 = rein_dot4(sw.w[j], xb[u].q[b][j], i0);
                            i1 = rein_dot4(sw.w[j + 4], xb[u].q[b][j + 4], i1);
                        }
                        acc[r][b] += F::term(sw, i0, i1, xb[u].dx[b], xb[u].xsum[b], xs[b]);
                    }
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int b = 0; b < B; b++) {
                const float s = rein_wave_sum(acc[r][b]);
                if (lane == 0 && row0 + r < out_dim && (unsigned)b < n_rows)
                    y[(size_t)b * out_dim + row0 + r] = s;
            }
    }
}

// Every wavefront of the launch takes the row groups of its own index, striding by the launch's wavefront count.
template <int FMT, int R, int B, int U = 1>
__device__ __forceinline__ void rein_matvec_body(const uint8_t* __restrict__ w,
                                                 const BlockQ8* __restrict__ xq,
                                                 float* __restrict__ y,
                                                 unsigned in_dim, unsigned out_dim, unsigned n_rows)
{
    const unsigned wpb = blockDim.x >> 6;
    rein_matvec_span<FMT, R, B, U>(w, xq, y, in_dim, out_dim, n_rows, blockIdx.x * wpb + (threadIdx.x >> 6), gridDim.x * wpb);
}

// Per-block integer dots exactly as the matvec forms them, for the bit-exact
// parity check: out[((t*out_dim + row)*n_sub + sb)*parts + p].  One lane per
// (row, sub-block); grid-stride over rows; blockIdx.y = activation row t.
template <int FMT>
__device__ __forceinline__ void rein_block_dots_body(const uint8_t* __restrict__ w,
                                                     const BlockQ8* __restrict__ xq,
                                                     int* __restrict__ out,
                                                     unsigned in_dim, unsigned out_dim)
{
    using F = Fmt<FMT>;
    const unsigned n_sub = in_dim >> 5;
    const F fmt(w, n_sub, out_dim);
    const unsigned t = blockIdx.y;
    for (unsigned row = blockIdx.x; row < out_dim; row += gridDim.x)
        for (unsigned sb = threadIdx.x; sb < n_sub; sb += blockDim.x) {
            SubW sw;
            F::unpack(fmt.load(row, sb), sw);
            const BlockQ8* p = xq + (size_t)t * n_sub + sb;
            int x[8];
#pragma unroll
            for (int j = 0; j < 8; j++) x[j] = p->qs[j];
            int i0 = 0, i1 = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                i0 = rein_dot4(sw.w[j], x[j], i0);
                i1 = rein_dot4(sw.w[j + 4], x[j + 4], i1);
            }
            int parts[2];
            F::parts(i0, i1, rein_xsums(x), parts);
            int* o = out + (((size_t)t * out_dim + row) * n_sub + sb) * F::kDotParts;
#pragma unroll
            for (int k = 0; k < F::kDotParts; k++) o[k] = parts[k];
        }
}

#define REIN_MATVEC_ARGS                                                                          \
    const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq, float* __restrict__ y,        \
        unsigned int in_dim, unsigned int out_dim

// name(w, xq, y, in_dim, out_dim): single activation row
#define REIN_DEFINE_MATVEC(name, FMT, R)                                                          \
    extern "C" __global__ __launch_bounds__(256) void name(REIN_MATVEC_ARGS)                      \
    {                                                                                             \
        rein_matvec_body<FMT, R, 1>(w, xq, y, in_dim, out_dim, 1u);                               \
    }

// name(w, xq[n_rows][n_sub], y[n_rows][out_dim], in_dim, out_dim, n_rows), n_rows <= B
#define REIN_DEFINE_MATVEC_BATCHED(name, FMT, R, B)                                               \
    extern "C" __global__ __launch_bounds__(256) void name(REIN_MATVEC_ARGS, unsigned int n_rows) \
    {                                                                                             \
        rein_matvec_body<FMT, R, B>(w, xq, y, in_dim, out_dim, n_rows);                           \
    }

// tuned variant with U trips of loads in flight per iteration
#define REIN_DEFINE_MATVEC_TUNED(name, FMT, R, B, U)                                              \
    extern "C" __global__ __launch_bounds__(256) void name(REIN_MATVEC_ARGS, unsigned int n_rows) \
    {                                                                                             \
        rein_matvec_body<FMT, R, B, U>(w, xq, y, in_dim, out_dim, n_rows);                        \
    }

#define REIN_DEFINE_BLOCK_DOTS(name, FMT)                                                         \
    extern "C" __global__ __launch_bounds__(256) void name(                                       \
        const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq, int* __restrict__ out,    \
        unsigned int in_dim, unsigned int out_dim)                                                \
    {                                                                                             \
        rein_block_dots_body<FMT>(w, xq, out, in_dim, out_dim);                                   \
    }
