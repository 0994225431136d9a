// Several decode matvecs that share their activation rows (one, or the two to four of a speculative-decode
// verify step), in one launch: rein_mv_multi_r<R>_b<B>.
//
// The reference's decode step launches the Q, K and V projections one after the other on the same
// quantized activations, and likewise the gate and up projections of a dense FFN
// (src/runtime/qwen35.rs:2670-2672, 2702-2703, 3612-3614, 3662-3663); on this machine every launch of
// that size costs one to two microseconds of gap and ramp that no kernel can win back.  Here the
// wavefronts of one launch are dealt over up to four matrices: wavefront i belongs to the first
// matrix whose cumulative row-group count exceeds i and runs that matrix's row group exactly as the
// single-matrix kernel rein_mv_<fmt>_r<R>_b<B> does (the same function, the same sums in the same
// order: the outputs are the bits of those kernels).  The matrices may differ in format and in their
// number of rows; they share in_dim and the activation rows.
#include "matvec_repacked.h"

#define REIN_MULTI_MAX 4

struct ReinMultiMat {
    const uint8_t* w;
    float*         y;
    unsigned       out_dim;
    int            fmt;          // REIN_* format id of rein_formats.h
    unsigned       group_end;    // row groups of this matrix and of those before it
    unsigned       pad;
};
struct ReinMultiArgs {
    ReinMultiMat m[REIN_MULTI_MAX];
};

template <int R, int B>
__device__ __forceinline__ void rein_matvec_multi_body(const ReinMultiArgs& a, const BlockQ8* __restrict__ xq,
                                                       unsigned in_dim, unsigned n_mat, unsigned n_rows)
{
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned wid = blockIdx.x * (blockDim.x >> 6) + wave;
    unsigned base = 0, end = a.m[0].group_end, out_dim = a.m[0].out_dim;
    const uint8_t* w = a.m[0].w;
    float* y = a.m[0].y;
    int fmt = a.m[0].fmt;
#pragma unroll
    for (int i = 1; i < REIN_MULTI_MAX; i++)
        if ((unsigned)i < n_mat && wid >= a.m[i - 1].group_end) {
            base = a.m[i - 1].group_end; end = a.m[i].group_end; out_dim = a.m[i].out_dim;
            w = a.m[i].w; y = a.m[i].y; fmt = a.m[i].fmt;
        }
    if (wid >= end) return;
    const unsigned g = wid - base;
    // one row group per wavefront: first = g, and a step that ends the walk after it
    const unsigned step = 0x40000000u;
    switch (fmt) {
    case REIN_Q4_K:   rein_matvec_span<REIN_Q4_K, R, B>(w, xq, y, in_dim, out_dim, n_rows, g, step); break;
    case REIN_Q6_K:   rein_matvec_span<REIN_Q6_K, R, B>(w, xq, y, in_dim, out_dim, n_rows, g, step); break;
    case REIN_Q5_K:   rein_matvec_span<REIN_Q5_K, R, B>(w, xq, y, in_dim, out_dim, n_rows, g, step); break;
    case REIN_Q8_0:   rein_matvec_span<REIN_Q8_0, R, B>(w, xq, y, in_dim, out_dim, n_rows, g, step); break;
    case REIN_Q4_0:   rein_matvec_span<REIN_Q4_0, R, B>(w, xq, y, in_dim, out_dim, n_rows, g, step); break;
    case REIN_IQ4_XS: rein_matvec_span<REIN_IQ4_XS, R, B>(w, xq, y, in_dim, out_dim, n_rows, g, step); break;
    case REIN_IQ3_S:  rein_matvec_span<REIN_IQ3_S, R, B>(w, xq, y, in_dim, out_dim, n_rows, g, step); break;
    default: break;
    }
}

// name(table, xq[n_rows][in_dim / 32], in_dim, n_mat, n_rows): n_rows <= B; y of matrix i is [n_rows][out_dim i]
#define REIN_DEFINE_MATVEC_MULTI(name, R, B)                                                                 \
    extern "C" __global__ __launch_bounds__(256) void name(ReinMultiArgs a, const BlockQ8* __restrict__ xq,   \
                                                           unsigned int in_dim, unsigned int n_mat,           \
                                                           unsigned int n_rows)                               \
    {                                                                                                        \
        rein_matvec_multi_body<R, B>(a, xq, in_dim, n_mat, n_rows);                                          \
    }

REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r1_b1, 1, 1)
REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r2_b1, 2, 1)
REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r4_b1, 4, 1)
REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r1_b2, 1, 2)
REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r2_b2, 2, 2)
REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r4_b2, 4, 2)
REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r1_b4, 1, 4)
REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r2_b4, 2, 4)
REIN_DEFINE_MATVEC_MULTI(rein_mv_multi_r4_b4, 4, 4)
