// MoE router: softmax over the expert logits, top-k, selected weights
// renormalised.  Same entry point, arguments and launch contract as
// kernels/moe_topk.cpp:17-108 of the reference: one workgroup of 128 threads per
// token, dynamic shared memory = n_expert floats.
//
// The result depends on the reduction order (fp32 softmax sum; which index
// survives an argmax tie), so the order is fixed to the 128-slot halving tree
// (slot t owns experts t, t+128, ...; 64 then 32 ... then 1, the lower slot
// surviving a tie).  Here the tree runs in registers: the 64-step crosses the two
// wavefronts through one LDS exchange, the remaining six steps are wave64
// shuffles.  Launches with more than 128 threads idle the extra waves.
#include "rein_common.h"
#include "q8_block.h"
#include "moe_topk_wave.h"

namespace {

struct Best { float v; int i; };

__device__ __forceinline__ float topk_tree_max(float v, float* xchg, int t)
{
    if (t >= 64 && t < 128) xchg[t - 64] = v;
    __syncthreads();
    if (t < 64) {
        v = fmaxf(v, xchg[t]);
#pragma unroll
        for (int s = 32; s > 0; s >>= 1) v = fmaxf(v, __shfl_down(v, s));
    }
    __syncthreads();
    if (t == 0) xchg[0] = v;
    __syncthreads();
    const float r = xchg[0];
    __syncthreads();
    return r;
}

__device__ __forceinline__ float topk_tree_sum(float v, float* xchg, int t)
{
    if (t >= 64 && t < 128) xchg[t - 64] = v;
    __syncthreads();
    if (t < 64) {
        v = v + xchg[t];
#pragma unroll
        for (int s = 32; s > 0; s >>= 1) v = v + __shfl_down(v, s);
    }
    __syncthreads();
    if (t == 0) xchg[0] = v;
    __syncthreads();
    const float r = xchg[0];
    __syncthreads();
    return r;
}

// strict '>' : the lower slot keeps its candidate on a tie
__device__ __forceinline__ Best topk_tree_argmax(Best b, float* xv, int* xi, int t)
{
    if (t >= 64 && t < 128) { xv[t - 64] = b.v; xi[t - 64] = b.i; }
    __syncthreads();
    if (t < 64) {
        if (xv[t] > b.v) { b.v = xv[t]; b.i = xi[t]; }
#pragma unroll
        for (int s = 32; s > 0; s >>= 1) {
            const float ov = __shfl_down(b.v, s);
            const int   oi = __shfl_down(b.i, s);
            if (ov > b.v) { b.v = ov; b.i = oi; }
        }
    }
    __syncthreads();
    return b;     // valid in thread 0
}

}  // namespace

extern "C" __global__ void moe_topk_f32(const float* __restrict__ logits, int n_expert, int n_used,
                                        int* __restrict__ out_ids, float* __restrict__ out_weights)
{
    extern __shared__ float probs[];          // n_expert floats
    __shared__ float xchg_v[64];
    __shared__ int   xchg_i[64];
    __shared__ float picked[64];              // n_used <= 64
    const int  t      = threadIdx.x;
    const bool worker = t < 128;

    logits      += (size_t)blockIdx.x * n_expert;
    out_ids     += (size_t)blockIdx.x * n_used;
    out_weights += (size_t)blockIdx.x * n_used;

    // load (NaN counts as -inf, so it can never be the maximum) and maximum
    float part = -INFINITY;
    if (worker)
        for (int i = t; i < n_expert; i += 128) {
            float v = logits[i];
            if (isnan(v)) v = -INFINITY;
            probs[i] = v;
            part = fmaxf(part, v);
        }
    const float m = topk_tree_max(part, xchg_v, t);

    part = 0.0f;
    if (worker)
        for (int i = t; i < n_expert; i += 128) {
            const float e = expf(probs[i] - m);
            probs[i] = e;
            part += e;
        }
    const float inv_sum = 1.0f / topk_tree_sum(part, xchg_v, t);
    if (worker)
        for (int i = t; i < n_expert; i += 128) probs[i] *= inv_sum;
    __syncthreads();

    // n_used rounds of argmax; a chosen expert is marked -1 and drops out
    for (int k = 0; k < n_used; k++) {
        Best b;
        b.v = -1.0f;
        b.i = 0;
        if (worker)
            for (int i = t; i < n_expert; i += 128) {
                const float v = probs[i];
                if (v > b.v) { b.v = v; b.i = i; }
            }
        b = topk_tree_argmax(b, xchg_v, xchg_i, t);
        if (t == 0) {
            out_ids[k]  = b.i;
            picked[k]   = b.v;
            probs[b.i]  = -1.0f;
        }
        __syncthreads();
    }

    if (t == 0) {
        float wsum = 0.0f;
        for (int k = 0; k < n_used; k++) wsum += picked[k];
        wsum = fmaxf(wsum, 6.103515625e-5f);      // 2^-14 floor
        for (int k = 0; k < n_used; k++) out_weights[k] = picked[k] / wsum;
    }
}

// Four tokens per 256-thread workgroup.
extern "C" __global__ __launch_bounds__(256) void rein_moe_topk_wave(const float* __restrict__ logits, int n_expert,
                                                                     int n_used, int* __restrict__ out_ids,
                                                                     float* __restrict__ out_weights, int n_tok)
{
    const int tok = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (tok >= n_tok) return;                       // whole wavefronts leave: no barrier anywhere
    rein_topk::topk_one_wave(logits + (size_t)tok * n_expert, n_expert, n_used, out_ids + (size_t)tok * n_used,
                  out_weights + (size_t)tok * n_used, threadIdx.x & 63);
}

// The router and quantize_q8_f32 of the token rows in one launch (the few-token form of the expert FFN runs both on
// the same inputs' stream with nothing between them): workgroups [0, ceil(n_tok / 4)) route four tokens each, the
// following n_tok * q_per_tok quantize 16 sub-blocks of 32 values each (q_per_tok = ceil(in_dim / 512)).  The bytes
// of both outputs are those of the two launches.
extern "C" __global__ __launch_bounds__(256) void rein_moe_route_quantize(const float* __restrict__ logits, int n_expert,
                                                                          int n_used, int* __restrict__ out_ids,
                                                                          float* __restrict__ out_weights, int n_tok,
                                                                          const float* __restrict__ x,
                                                                          BlockQ8* __restrict__ xq, unsigned in_dim,
                                                                          unsigned q_per_tok)
{
    const unsigned n_route = ((unsigned)n_tok + 3u) >> 2;
    if (blockIdx.x < n_route) {
        const int tok = blockIdx.x * 4 + (threadIdx.x >> 6);
        if (tok >= n_tok) return;
        rein_topk::topk_one_wave(logits + (size_t)tok * n_expert, n_expert, n_used, out_ids + (size_t)tok * n_used,
                      out_weights + (size_t)tok * n_used, threadIdx.x & 63);
        return;
    }
    const unsigned w = blockIdx.x - n_route;
    const unsigned vec = w / q_per_tok, chunk = w - vec * q_per_tok;
    const unsigned n_sub = in_dim >> 5;
    const unsigned blk = chunk * 16u + (threadIdx.x >> 4), l = threadIdx.x & 15u;
    if (blk >= n_sub) return;
    const float* v = x + (size_t)vec * in_dim + (size_t)blk * 32 + l;
    rein_q8_store_sub(xq + (size_t)vec * n_sub + blk, l, v[0], v[16]);
}
