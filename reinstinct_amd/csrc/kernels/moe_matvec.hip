// MoE decode: expert matvecs with the expert id read on the device.
//
//   y[tok][slot][row] = W[ids[tok][slot]] . xq[tok(, slot)]
//
// Same symbols and argument lists as the reference's kernels/moe_matvec_{q4k,q5k,q6k,
// q8_0}_repacked.cpp, moe_matvec_{q5k,q6k}_down.cpp and
// moe_gate_up_swiglu_q4k_repacked.cpp: grid = (row blocks, n_used, n_tok) x 256
// threads there; here grid.x is a stride, so any grid.x and any block that is a
// multiple of 64 is correct, and grid.y / grid.z still carry the slot and the token.
//
// LANES = 64: a wavefront owns R rows, lane l walks sub-blocks l, l+64, ... (the
// decode matvec's mapping: 1 KiB bursts of the nibble plane per row).
// LANES = 32: each half of a wavefront owns its own R rows and walks sub-blocks
// l, l+32, ...; this is what the "down" symbols use: the down projection contracts
// over the expert's intermediate size (768 -> 24 sub-blocks), which would leave 40
// of 64 lanes idle.  The reference packs rows into a workgroup and sums through LDS
// for the same reason (moe_matvec_q6k_down.cpp:1-6).
//
// Per-sub-block formulas are the decode matvec's (rein_formats.h); the gate+up form
// writes silu(gate) * up with the deterministic silu of q8_block.h.
#include "rein_formats.h"
#include "q8_block.h"

template <int FMT, int R, int LANES, bool GATE_UP>
__device__ __forceinline__ void rein_moe_matvec(const uint8_t* __restrict__ slab0, const uint8_t* __restrict__ slab1,
                                                const int* __restrict__ ids, const BlockQ8* __restrict__ xq,
                                                float* __restrict__ y, unsigned in_dim, unsigned out_dim,
                                                unsigned bytes_per_expert, unsigned xq_tok_stride,
                                                unsigned xq_slot_stride, unsigned n_used)
{
    using F = Fmt<FMT>;
    static_assert(LANES == 64 || LANES == 32, "a row group is a wavefront or half of one");
    const unsigned tok = blockIdx.z, slot = blockIdx.y;
    const unsigned eid = (unsigned)ids[(size_t)tok * n_used + slot];
    const BlockQ8* xqs = xq + (size_t)tok * xq_tok_stride + (size_t)slot * xq_slot_stride;
    float* yo = y + ((size_t)tok * n_used + slot) * out_dim;
    const unsigned n_sub = in_dim >> 5;
    const F w0(slab0 + (size_t)eid * bytes_per_expert, n_sub, out_dim);
    const F w1((GATE_UP ? slab1 : slab0) + (size_t)eid * bytes_per_expert, n_sub, out_dim);

    const unsigned lane = threadIdx.x & (LANES - 1u);
    const unsigned teams_per_block = blockDim.x / LANES;
    const unsigned n_groups = (out_dim + R - 1) / R;
    const unsigned rmax = out_dim - 1;

    // trip count made uniform across the wavefront (both halves run the same number of
    // passes; a half past the end works on clamped rows and stores nothing)
    const unsigned team0 = blockIdx.x * teams_per_block + threadIdx.x / LANES;
    const unsigned wave_team0 = blockIdx.x * teams_per_block + (threadIdx.x >> 6) * (64 / LANES);
    for (unsigned g = team0, gw = wave_team0; gw < n_groups; g += gridDim.x * teams_per_block, gw += gridDim.x * teams_per_block) {
        const unsigned row0 = g * R;
        float a0[R], a1[R];
#pragma unroll
        for (int r = 0; r < R; r++) { a0[r] = 0.0f; a1[r] = 0.0f; }

        for (unsigned sb0 = 0; sb0 < n_sub; sb0 += LANES) {
            const bool live = sb0 + lane < n_sub;
            const unsigned sb = live ? sb0 + lane : n_sub - 1;
            typename F::Raw raw0[R], raw1[R];
#pragma unroll
            for (int r = 0; r < R; r++) {
                raw0[r] = w0.load(min(row0 + r, rmax), sb);
                if (GATE_UP) raw1[r] = w1.load(min(row0 + r, rmax), sb);
            }
            const BlockQ8* p = xqs + sb;
            const float dx = live ? p->d : 0.0f, xsum = live ? p->xsum : 0.0f;
            int q[8];
#pragma unroll
            for (int j = 0; j < 8; j++) q[j] = p->qs[j];
            XSums xs;
            if (F::kNeedsXSums) xs = rein_xsums(q);
            else { xs.lo = 0; xs.hi = 0; }
#pragma unroll
            for (int r = 0; r < R; r++) {
                SubW sw;
                F::unpack(raw0[r], sw);
                int i0 = 0, i1 = 0;
#pragma unroll
                for (int j = 0; j < 4; j++) { i0 = rein_dot4(sw.w[j], q[j], i0); i1 = rein_dot4(sw.w[j + 4], q[j + 4], i1); }
                a0[r] += F::term(sw, i0, i1, dx, xsum, xs);
                if (GATE_UP) {
                    F::unpack(raw1[r], sw);
                    i0 = 0; i1 = 0;
#pragma unroll
                    for (int j = 0; j < 4; j++) { i0 = rein_dot4(sw.w[j], q[j], i0); i1 = rein_dot4(sw.w[j + 4], q[j + 4], i1); }
                    a1[r] += F::term(sw, i0, i1, dx, xsum, xs);
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; r++) {
            float s0, s1 = 0.0f;
            if (LANES == 64) {
                s0 = rein_wave_sum(a0[r]);
                if (GATE_UP) s1 = rein_wave_sum(a1[r]);
            } else {
                // row sums of the four 16-lane rows; a half owns rows {0,1} or {2,3}
                const float t = rein_row16_sum(a0[r]);
                const int b = __builtin_bit_cast(int, t);
                const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) +
                                 __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
                const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) +
                                 __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
                s0 = (threadIdx.x & 32u) ? hi : lo;
            }
            if (lane == 0 && row0 + r < out_dim) yo[row0 + r] = GATE_UP ? rein_silu_det(s0) * s1 : s0;
        }
    }
}

#define REIN_MOE_MV_ARGS                                                                                  \
    const unsigned char *__restrict__ slab, const int *__restrict__ ids, const BlockQ8 *__restrict__ xq,  \
        float *__restrict__ y, unsigned int in_dim, unsigned int out_dim, unsigned int bytes_per_expert,  \
        unsigned int xq_tok_stride, unsigned int xq_slot_stride, unsigned int n_used

#define REIN_DEFINE_MOE_MV(name, FMT, R, LANES)                                                           \
    extern "C" __global__ __launch_bounds__(256) void name(REIN_MOE_MV_ARGS)                              \
    {                                                                                                     \
        rein_moe_matvec<FMT, R, LANES, false>(slab, slab, ids, xq, y, in_dim, out_dim, bytes_per_expert,  \
                                              xq_tok_stride, xq_slot_stride, n_used);                     \
    }

// kernels/moe_matvec_q4k_repacked.cpp:23-100 and its Q5_K / Q6_K / Q8_0 siblings
REIN_DEFINE_MOE_MV(moe_matvec_q4k_repacked_f32, REIN_Q4_K, 2, 64)
REIN_DEFINE_MOE_MV(moe_matvec_q5k_repacked_f32, REIN_Q5_K, 2, 64)
REIN_DEFINE_MOE_MV(moe_matvec_q6k_repacked_f32, REIN_Q6_K, 2, 64)
REIN_DEFINE_MOE_MV(moe_matvec_q8_0_repacked_f32, REIN_Q8_0, 2, 64)
// kernels/moe_matvec_q5k_down.cpp, moe_matvec_q6k_down.cpp:24-112 and the Q8_0 down entry
// of moe_matvec_q8_0_repacked.cpp: short contractions
REIN_DEFINE_MOE_MV(moe_matvec_q5k_down_f32, REIN_Q5_K, 2, 32)
REIN_DEFINE_MOE_MV(moe_matvec_q6k_down_f32, REIN_Q6_K, 2, 32)
REIN_DEFINE_MOE_MV(moe_matvec_q8_0_repacked_down_f32, REIN_Q8_0, 2, 32)
// Q5_1 experts: the Q5_K kernels with the raw (d, m) scale decode (the reference's second
// compilation with Q5_1_SCALES, qwen35.rs:3082,3116)
REIN_DEFINE_MOE_MV(moe_matvec_q5_1_repacked_f32, REIN_Q5_1, 2, 64)
REIN_DEFINE_MOE_MV(moe_matvec_q5_1_down_f32, REIN_Q5_1, 2, 32)
// the same for the format the reference has no down kernel for (it falls back to the
// generic one, qwen35.rs:3118-3120)
REIN_DEFINE_MOE_MV(rein_moe_matvec_q4k_down_f32, REIN_Q4_K, 2, 32)

// kernels/moe_gate_up_swiglu_q4k_repacked.cpp:28-129: y = silu(gate . x) * (up . x)
extern "C" __global__ __launch_bounds__(256)
void moe_gate_up_swiglu_q4k_repacked_f32(const unsigned char* __restrict__ gate_slab,
                                         const unsigned char* __restrict__ up_slab, const int* __restrict__ ids,
                                         const BlockQ8* __restrict__ xq, float* __restrict__ y, unsigned int in_dim,
                                         unsigned int out_dim, unsigned int bytes_per_expert,
                                         unsigned int xq_tok_stride, unsigned int xq_slot_stride, unsigned int n_used)
{
    rein_moe_matvec<REIN_Q4_K, 2, 64, true>(gate_slab, up_slab, ids, xq, y, in_dim, out_dim, bytes_per_expert,
                                            xq_tok_stride, xq_slot_stride, n_used);
}
