// MoE router on one wavefront per token (up to 256 experts): softmax, top-k and renormalised weights with the ids
// and the weight bits of moe_topk_f32 (kernels/moe_topk.cpp:17-108 of the reference: its 128-slot halving tree).
// Shared by rein_moe_topk_wave (moe_topk.hip) and by the few-token expert FFN, whose gate / up launch routes its
// token itself (moe_matvec.hip).
#pragma once

#include "rein_common.h"

// ---- one wavefront per token (up to 256 experts) -----------------------------------------------------------
//
// Slot s of the 128-slot tree owns experts s and s + 128; lane l holds slots l and l + 64, so the tree's 64-step is
// an operation between two registers of a lane and no LDS or barrier is needed.
//  * maximum: order-free, reduced with DPP row shifts and row broadcasts.
//  * softmax sum: the tree's additions in the tree's order (64-step in the lane, 32 and 16 by shuffle, 8..1 by DPP
//    row shift -- lane 0 only ever reads lanes of its own 16-lane row there).
//  * arg-max rounds: the tree keeps the lower slot on a tie at every step, and two slots meet at the step of their
//    lowest differing bit, so among equal probabilities the winner is the expert with the smallest bit-reversed
//    8-bit index (bit 7 = second expert of a slot, lowest priority).  That is a total order, so each round is two
//    order-free reductions: the maximum probability, then the minimum bit-reversed index among its holders.
// Same ids and same weight bits as moe_topk_f32 (tested); 128 experts, top-8: 4.6 instead of 6.5 us for one token,
// 7.9 instead of 11.4 us for 4096.
namespace rein_topk {

template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f(float keep, float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, keep), __builtin_bit_cast(int, v),
                                                                 CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ unsigned dpp_u(unsigned keep, unsigned v)
{
    return (unsigned)__builtin_amdgcn_update_dpp((int)keep, (int)v, CTRL, ROW_MASK, 0xf, false);
}
constexpr int kRowShr = 0x110, kRowShl = 0x100, kRowBcast15 = 0x142, kRowBcast31 = 0x143;

// maximum over the wavefront, returned in every lane (lanes without a source keep their own value)
__device__ __forceinline__ float wave_max(float v)
{
    v = fmaxf(v, dpp_f<kRowShr + 1>(v, v));
    v = fmaxf(v, dpp_f<kRowShr + 2>(v, v));
    v = fmaxf(v, dpp_f<kRowShr + 4>(v, v));
    v = fmaxf(v, dpp_f<kRowShr + 8>(v, v));
    v = fmaxf(v, dpp_f<kRowBcast15, 0xa>(v, v));
    v = fmaxf(v, dpp_f<kRowBcast31, 0xc>(v, v));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ unsigned wave_min(unsigned v)
{
    v = min(v, dpp_u<kRowShr + 1>(v, v));
    v = min(v, dpp_u<kRowShr + 2>(v, v));
    v = min(v, dpp_u<kRowShr + 4>(v, v));
    v = min(v, dpp_u<kRowShr + 8>(v, v));
    v = min(v, dpp_u<kRowBcast15, 0xa>(v, v));
    v = min(v, dpp_u<kRowBcast31, 0xc>(v, v));
    return (unsigned)__builtin_amdgcn_readlane((int)v, 63);
}
// lane 0's value of the halving tree v[i] += v[i + s], s = 32 .. 1, in every lane
__device__ __forceinline__ float wave_tree_sum(float v)
{
    v = v + __shfl_down(v, 32);
    v = v + __shfl_down(v, 16);
    v = v + dpp_f<kRowShl + 8>(0.0f, v);
    v = v + dpp_f<kRowShl + 4>(0.0f, v);
    v = v + dpp_f<kRowShl + 2>(0.0f, v);
    v = v + dpp_f<kRowShl + 1>(0.0f, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
}

__device__ __forceinline__ void topk_one_wave(const float* __restrict__ logits, int n_expert, int n_used,
                                              int* __restrict__ out_ids, float* __restrict__ out_weights, int lane)
{
    // q[a][b]: expert lane + 64 a + 128 b, i.e. slot lane + 64 a, the slot's b-th expert
    float q[2][2];
    bool  have[2][2];
    float part[2];
#pragma unroll
    for (int a = 0; a < 2; a++) {
        part[a] = -INFINITY;
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int i = lane + 64 * a + 128 * b;
            have[a][b] = i < n_expert;
            float v = have[a][b] ? logits[i] : -INFINITY;
            if (isnan(v)) v = -INFINITY;
            q[a][b] = v;
            part[a] = fmaxf(part[a], v);
        }
    }
    const float m = wave_max(fmaxf(part[0], part[1]));

#pragma unroll
    for (int a = 0; a < 2; a++) {
        part[a] = 0.0f;
#pragma unroll
        for (int b = 0; b < 2; b++)
            if (have[a][b]) {
                q[a][b] = expf(q[a][b] - m);
                part[a] += q[a][b];
            }
    }
    const float inv_sum = 1.0f / wave_tree_sum(part[0] + part[1]);
    // an expert that can be chosen holds its probability, every other one (absent, NaN, already chosen) -1: the
    // workgroup kernel starts each slot's candidate at {-1, expert 0} and replaces it on a strict '>'
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const float pr = q[a][b] * inv_sum;
            q[a][b] = (have[a][b] && pr > -1.0f) ? pr : -1.0f;
        }

    float picked = 0.0f;                            // lane k keeps the k-th selected probability
    for (int k = 0; k < n_used; k++) {
        const float bv = wave_max(fmaxf(fmaxf(q[0][0], q[0][1]), fmaxf(q[1][0], q[1][1])));
        int bi = 0;                                 // nothing left to choose: {-1, expert 0}, as the tree gives
        if (bv > -1.0f) {
            unsigned key = 0xFFFFFFFFu;
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++)
                    if (q[a][b] == bv) key = min(key, __builtin_bitreverse32((unsigned)(lane + 64 * a + 128 * b)) >> 24);
            bi = (int)(__builtin_bitreverse32(wave_min(key)) >> 24);
        }
        if (lane == 0) out_ids[k] = bi;
        if (lane == k) picked = bv;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < 2; b++)
                if (lane + 64 * a + 128 * b == bi) q[a][b] = -1.0f;
    }

    float wsum = 0.0f;
    for (int k = 0; k < n_used; k++)
        wsum += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, picked), k));
    wsum = fmaxf(wsum, 6.103515625e-5f);            // 2^-14 floor
    if (lane < n_used) out_weights[lane] = picked / wsum;
}

}  // namespace rein_topk
