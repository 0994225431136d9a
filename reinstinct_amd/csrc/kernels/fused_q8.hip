// Fused BlockQ8 producers: the step in front of a quantized matvec (norm, gate
// or activation function) writes the BlockQ8 blocks the matvec reads, so the fp32
// vector does not make a round trip through HBM and one launch disappears per
// linear layer.
//
// Same symbols and argument lists as the reference's kernels/rmsnorm_q8.cpp:38-103,
// kernels/qwen35_fused.cpp:66-151,195-217 and kernels/moe_geglu_q8.cpp:31-66; correct
// under the reference's launch geometry and under any block that is a multiple of 64
// (16-lane rows stride over sub-blocks, two values per lane; n a multiple of 32).
//
// Bit-level definition, shared with the CPU checker: the quantizer is
// rein_q8_store_sub; exp / silu / sigmoid / gelu are the deterministic forms of
// q8_block.h; rrms = 1 / sqrt(sumsq / n + eps) with IEEE division and square root
// and the geometry-independent summation order of rein_sumsq_finish;
// normalized value = (x * rrms) * w, two roundings.
#include "q8_block.h"

#define REIN_FUSED_MAX_SUB 1024        // n <= 32768 per vector
#define REIN_FUSED_KEEP    4           // sub-blocks per 16-lane row held in registers

// (hidden += add) -> rmsnorm * w -> fp32 y and/or BlockQ8.  One workgroup per
// vector (blockIdx.y).  add, y may be null; hidden is written only when add is given.
__device__ __forceinline__ void rein_add_rmsnorm_q8(float* __restrict__ hidden, const float* __restrict__ add,
                                                    const float* __restrict__ w, float* __restrict__ y,
                                                    BlockQ8* __restrict__ out, unsigned n, float eps)
{
#pragma clang fp contract(off)
    __shared__ float part[REIN_FUSED_MAX_SUB];
    __shared__ float total;
    const unsigned n_sub = n >> 5;
    const unsigned l = threadIdx.x & 15u, g = threadIdx.x >> 4, n_g = blockDim.x >> 4;

    // every load first: this is one workgroup working on one vector, and what it
    // waits for is memory latency, once
    float v0[REIN_FUSED_KEEP], v1[REIN_FUSED_KEEP], w0[REIN_FUSED_KEEP], w1[REIN_FUSED_KEEP];
#pragma unroll
    for (int k = 0; k < REIN_FUSED_KEEP; k++) {
        const unsigned sb = min(g + k * n_g, n_sub - 1u);
        const unsigned i = sb * 32u + l;
        v0[k] = hidden[i];
        v1[k] = hidden[i + 16];
        if (add) { v0[k] = v0[k] + add[i]; v1[k] = v1[k] + add[i + 16]; }
        w0[k] = w[i];
        w1[k] = w[i + 16];
    }
#pragma unroll
    for (int k = 0; k < REIN_FUSED_KEEP; k++) {
        const unsigned sb = g + k * n_g;
        if (sb < n_sub) {
            if (add) { hidden[sb * 32u + l] = v0[k]; hidden[sb * 32u + l + 16] = v1[k]; }
            const float s = rein_row_sum(v0[k] * v0[k], v1[k] * v1[k]);
            if (l == 0u) part[sb] = s;
        }
    }
    for (unsigned sb = g + REIN_FUSED_KEEP * n_g; sb < n_sub; sb += n_g) {      // vectors too long for the registers
        const unsigned i = sb * 32u + l;
        float a0 = hidden[i], a1 = hidden[i + 16];
        if (add) { a0 = a0 + add[i]; a1 = a1 + add[i + 16]; hidden[i] = a0; hidden[i + 16] = a1; }
        const float s = rein_row_sum(a0 * a0, a1 * a1);
        if (l == 0u) part[sb] = s;
    }
    const float sumsq = rein_sumsq_finish(part, n_sub, &total);
    const float rrms = 1.0f / sqrtf(sumsq / (float)n + eps);

#pragma unroll
    for (int k = 0; k < REIN_FUSED_KEEP; k++) {
        const unsigned sb = g + k * n_g;
        if (sb < n_sub) {
            const float o0 = (v0[k] * rrms) * w0[k], o1 = (v1[k] * rrms) * w1[k];
            if (y) { y[sb * 32u + l] = o0; y[sb * 32u + l + 16] = o1; }
            rein_q8_store_sub(out + sb, l, o0, o1);
        }
    }
    for (unsigned sb = g + REIN_FUSED_KEEP * n_g; sb < n_sub; sb += n_g) {
        const unsigned i = sb * 32u + l;
        const float o0 = (hidden[i] * rrms) * w[i], o1 = (hidden[i + 16] * rrms) * w[i + 16];   // hidden holds x + add
        if (y) { y[i] = o0; y[i + 16] = o1; }
        rein_q8_store_sub(out + sb, l, o0, o1);
    }
}

// kernels/rmsnorm_q8.cpp:38-42: grid = (1, n_vec), block = 512 in the reference
extern "C" __global__ __launch_bounds__(1024)
void rmsnorm_q8_f32(const float* __restrict__ x, const float* __restrict__ w, BlockQ8* __restrict__ out,
                    unsigned int n, float eps)
{
    const size_t vec = blockIdx.y;
    rein_add_rmsnorm_q8(const_cast<float*>(x) + vec * n, nullptr, w, nullptr, out + vec * (n >> 5), n, eps);
}

// kernels/qwen35_fused.cpp:66-74: grid = 1, block = 1024 in the reference; here
// blockIdx.y selects the vector of hidden / add / y / out (w is shared)
extern "C" __global__ __launch_bounds__(1024)
void add_rmsnorm_q8_f32(float* __restrict__ hidden, const float* __restrict__ add, const float* __restrict__ w,
                        float* __restrict__ y, BlockQ8* __restrict__ out, unsigned int n, float eps)
{
    const size_t vec = blockIdx.y;
    rein_add_rmsnorm_q8(hidden + vec * n, add ? add + vec * n : nullptr, w, y ? y + vec * n : nullptr,
                        out + vec * (n >> 5), n, eps);
}

// out = silu(gate) * up, fp32 and BlockQ8.  kernels/qwen35_fused.cpp:132-146
// (grid = ceil(n/256), block = 256 there).  `out` may be null.
extern "C" __global__ __launch_bounds__(1024)
void swiglu_q8_f32(const float* __restrict__ gate, const float* __restrict__ up, float* __restrict__ out,
                   BlockQ8* __restrict__ q8, unsigned int n)
{
#pragma clang fp contract(off)
    const unsigned n_sub = n >> 5, l = threadIdx.x & 15u, n_g = blockDim.x >> 4;
    for (unsigned sb = blockIdx.x * n_g + (threadIdx.x >> 4); sb < n_sub; sb += gridDim.x * n_g) {
        const unsigned i = sb * 32u + l;
        const float v0 = rein_silu_det(gate[i]) * up[i], v1 = rein_silu_det(gate[i + 16]) * up[i + 16];
        if (out) { out[i] = v0; out[i + 16] = v1; }
        rein_q8_store_sub(q8 + sb, l, v0, v1);
    }
}

// x *= sigmoid(gate) in place, plus BlockQ8.  kernels/qwen35_fused.cpp:149-162
extern "C" __global__ __launch_bounds__(1024)
void sigmoid_mul_q8_f32(float* __restrict__ x, const float* __restrict__ gate, BlockQ8* __restrict__ q8,
                        unsigned int n)
{
#pragma clang fp contract(off)
    const unsigned n_sub = n >> 5, l = threadIdx.x & 15u, n_g = blockDim.x >> 4;
    for (unsigned sb = blockIdx.x * n_g + (threadIdx.x >> 4); sb < n_sub; sb += gridDim.x * n_g) {
        const unsigned i = sb * 32u + l;
        const float v0 = x[i] * rein_sigmoid_det(gate[i]), v1 = x[i + 16] * rein_sigmoid_det(gate[i + 16]);
        x[i] = v0;
        x[i + 16] = v1;
        rein_q8_store_sub(q8 + sb, l, v0, v1);
    }
}

// Per-head gated RMSNorm: y = rmsnorm(x) * w * silu(z), fp32 and BlockQ8.
// kernels/qwen35_fused.cpp:195-217 (grid = n_heads blocks of head_dim threads
// there; any block of >= 64 threads here).  head_dim a multiple of 32, <= 32768.
extern "C" __global__ __launch_bounds__(1024)
void rmsnorm_gated_q8_f32(const float* __restrict__ x, const float* __restrict__ z, const float* __restrict__ w,
                          float* __restrict__ y, BlockQ8* __restrict__ q8, unsigned int n_heads,
                          unsigned int head_dim, float eps)
{
#pragma clang fp contract(off)
    __shared__ float part[REIN_FUSED_MAX_SUB];
    __shared__ float total;
    const unsigned n_sub = head_dim >> 5, l = threadIdx.x & 15u, g = threadIdx.x >> 4, n_g = blockDim.x >> 4;
    for (unsigned h = blockIdx.x; h < n_heads; h += gridDim.x) {
        const size_t base = (size_t)h * head_dim;
        for (unsigned sb = g; sb < n_sub; sb += n_g) {
            const float a0 = x[base + sb * 32u + l], a1 = x[base + sb * 32u + l + 16];
            const float s = rein_row_sum(a0 * a0, a1 * a1);
            if (l == 0u) part[sb] = s;
        }
        const float sumsq = rein_sumsq_finish(part, n_sub, &total);
        const float rrms = 1.0f / sqrtf(sumsq / (float)head_dim + eps);
        for (unsigned sb = g; sb < n_sub; sb += n_g) {
            const unsigned c = sb * 32u + l;
            const float v0 = ((x[base + c] * rrms) * w[c]) * rein_silu_det(z[base + c]);
            const float v1 = ((x[base + c + 16] * rrms) * w[c + 16]) * rein_silu_det(z[base + c + 16]);
            if (y) { y[base + c] = v0; y[base + c + 16] = v1; }
            rein_q8_store_sub(q8 + (base >> 5) + sb, l, v0, v1);
        }
        __syncthreads();                                  // part / total are reused by the next head
    }
}

// act = gelu(gate) * up per expert slot, straight to BlockQ8.
// kernels/moe_geglu_q8.cpp:31-66: gu is [n_slot, 2*ff_exp] (gate half, up half),
// grid = (ceil(ff_exp/256), n_slot), block = 256 there.
extern "C" __global__ __launch_bounds__(1024)
void moe_geglu_q8_f32(const float* __restrict__ gu, BlockQ8* __restrict__ out, unsigned int ff_exp)
{
#pragma clang fp contract(off)
    const unsigned slot = blockIdx.y;
    const unsigned n_sub = ff_exp >> 5, l = threadIdx.x & 15u, n_g = blockDim.x >> 4;
    const float* g = gu + (size_t)slot * 2u * ff_exp;
    BlockQ8* o = out + (size_t)slot * n_sub;
    for (unsigned sb = blockIdx.x * n_g + (threadIdx.x >> 4); sb < n_sub; sb += gridDim.x * n_g) {
        const unsigned i = sb * 32u + l;
        const float v0 = rein_gelu_det(g[i]) * g[ff_exp + i], v1 = rein_gelu_det(g[i + 16]) * g[ff_exp + i + 16];
        rein_q8_store_sub(o + sb, l, v0, v1);
    }
}
