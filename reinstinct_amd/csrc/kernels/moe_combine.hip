// Weighted combine of the routed-expert outputs: same entry point and arguments
// as kernels/moe_combine.cpp:15-38 of the reference.
//   out[tok][i] = sum_j weights[tok][j] * down_exps_s[ids[tok][j]] * experts[tok][j][i]
// summed in slot order j = 0..n_used-1 (fp32, one fma-free multiply-add chain).
#include "rein_common.h"

extern "C" __global__ void moe_combine_f32(const float* __restrict__ experts, const int* __restrict__ ids,
                                           const float* __restrict__ weights,
                                           const float* __restrict__ down_exps_s, float* __restrict__ out,
                                           unsigned int hidden, unsigned int n_used)
{
#pragma clang fp contract(off)
    const size_t tok = blockIdx.y;
    experts += tok * n_used * hidden;
    ids     += tok * n_used;
    weights += tok * n_used;
    out     += tok * hidden;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < hidden; i += gridDim.x * blockDim.x) {
        float acc = 0.0f;
        for (unsigned j = 0; j < n_used; j++) {
            const float s = weights[j] * down_exps_s[ids[j]];
            acc += s * experts[(size_t)j * hidden + i];
        }
        out[i] = acc;
    }
}

// The same sum over expert outputs that are still in expert-sorted order:
// row of (tok, j) = sorted[inv[tok * n_used + j]] (moe_scatter_rows + moe_combine_f32 in
// one pass; same slot order, same arithmetic).  Entries with inv < 0 (expert id out of
// range) contribute nothing.
extern "C" __global__ void rein_moe_combine_sorted_f32(const float* __restrict__ sorted, const int* __restrict__ inv,
                                                       const int* __restrict__ ids, const float* __restrict__ weights,
                                                       const float* __restrict__ down_exps_s, float* __restrict__ out,
                                                       unsigned int hidden, unsigned int n_used)
{
#pragma clang fp contract(off)
    const size_t tok = blockIdx.y;
    inv     += tok * n_used;
    ids     += tok * n_used;
    weights += tok * n_used;
    out     += tok * hidden;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < hidden; i += gridDim.x * blockDim.x) {
        float acc = 0.0f;
        for (unsigned j = 0; j < n_used; j++) {
            const int pos = inv[j];
            if (pos < 0) continue;
            const float s = weights[j] * down_exps_s[ids[j]];
            acc += s * sorted[(size_t)pos * hidden + i];
        }
        out[i] = acc;
    }
}
