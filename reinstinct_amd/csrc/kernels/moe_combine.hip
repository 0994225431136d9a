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

// The same, four columns per thread (hidden a multiple of 4, 16-byte aligned rows): 128-bit loads of the
// eight expert rows, the slot order and the per-column arithmetic unchanged (the same bits).
extern "C" __global__ __launch_bounds__(256)
void rein_moe_combine_sorted4_f32(const float* __restrict__ sorted, const int* __restrict__ inv,
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
    const unsigned h4 = hidden >> 2;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < h4; i += gridDim.x * blockDim.x) {
        float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll 8
        for (unsigned j = 0; j < n_used; j++) {
            const int pos = inv[j];
            if (pos < 0) continue;
            const float s = weights[j] * down_exps_s[ids[j]];
            const float4 v = *reinterpret_cast<const float4*>(sorted + (size_t)pos * hidden + 4u * i);
            acc.x += s * v.x; acc.y += s * v.y; acc.z += s * v.z; acc.w += s * v.w;
        }
        *reinterpret_cast<float4*>(out + 4u * i) = acc;
    }
}

