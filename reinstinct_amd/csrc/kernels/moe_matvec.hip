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
#include "moe_topk_wave.h"

// Dot products of rows row0 .. row0+R-1 of one expert (w0; GATE_UP: also w1) with the
// BlockQ8 row xqs, for a team of LANES lanes (lane = index in the team).  s0 / s1 are valid
// in every lane of the team.  Rows past rmax are clamped (the caller stores nothing for them).
template <int FMT, int R, int LANES, bool GATE_UP>
__device__ __forceinline__ void rein_moe_row_sums(const Fmt<FMT>& w0, const Fmt<FMT>& w1, const BlockQ8* __restrict__ xqs,
                                                  unsigned n_sub, unsigned row0, unsigned rmax, unsigned lane,
                                                  float (&s0)[R], float (&s1)[R])
{
    using F = Fmt<FMT>;
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
        s1[r] = 0.0f;
        if (LANES == 64) {
            s0[r] = rein_wave_sum(a0[r]);
            if (GATE_UP) s1[r] = rein_wave_sum(a1[r]);
        } else {
            // row sums of the four 16-lane rows; a half owns rows {0,1} or {2,3}
            const float t = rein_row16_sum(a0[r]);
            const int b = __builtin_bit_cast(int, t);
            const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) +
                             __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
            const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) +
                             __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
            s0[r] = (threadIdx.x & 32u) ? hi : lo;
        }
    }
}

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
        float s0[R], s1[R];
        rein_moe_row_sums<FMT, R, LANES, GATE_UP>(w0, w1, xqs, n_sub, row0, rmax, lane, s0, s1);
#pragma unroll
        for (int r = 0; r < R; r++)
            if (lane == 0 && row0 + r < out_dim) yo[row0 + r] = GATE_UP ? rein_silu_det(s0[r]) * s1[r] : s0[r];
    }
}

// gate + up + SwiGLU + quantize_q8 in one launch: xq_out[tok][slot][blk] is the BlockQ8 block
// of outputs 32 blk .. 32 blk + 31 of silu(gate . x) * (up . x) -- byte for byte what
// moe_gate_up_swiglu_*_f32 followed by quantize_q8_f32 writes (same per-row sums, same silu,
// same block quantizer).  One workgroup of 1024 threads per block of 32 outputs: wavefront w
// computes rows 2w, 2w + 1 (the mapping of the two-launch form), the 32 values meet in LDS and
// one 16-lane row quantizes them.  grid = (out_dim / 32, n_used, n_tok); out_dim % 32 == 0.
template <int FMT, int R>
__device__ __forceinline__ void rein_moe_gate_up_swiglu_q8_core(const uint8_t* __restrict__ gate_slab, const uint8_t* __restrict__ up_slab,
                                                                unsigned eid, const BlockQ8* __restrict__ xqs,
                                                                BlockQ8* __restrict__ xq_out, unsigned in_dim, unsigned out_dim,
                                                                unsigned bytes_per_expert, unsigned n_used, float* vals)
{
    using F = Fmt<FMT>;
    const unsigned tok = blockIdx.z, slot = blockIdx.y, blk = blockIdx.x;
    const unsigned n_blk = out_dim >> 5;
    const unsigned n_sub = in_dim >> 5;
    const F w0(gate_slab + (size_t)eid * bytes_per_expert, n_sub, out_dim);
    const F w1(up_slab + (size_t)eid * bytes_per_expert, n_sub, out_dim);
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned row0 = blk * 32u + wave * R;
    float s0[R], s1[R];
    rein_moe_row_sums<FMT, R, 64, true>(w0, w1, xqs, n_sub, row0, out_dim - 1u, lane, s0, s1);
#pragma unroll
    for (int r = 0; r < R; r++)
        if (lane == (unsigned)r) vals[wave * R + r] = rein_silu_det(s0[r]) * s1[r];
    __syncthreads();
    if (threadIdx.x < 16u)
        rein_q8_store_sub(xq_out + ((size_t)tok * n_used + slot) * n_blk + blk, threadIdx.x, vals[threadIdx.x], vals[threadIdx.x + 16u]);
}

template <int FMT, int R>
__device__ __forceinline__ void rein_moe_gate_up_swiglu_q8(const uint8_t* __restrict__ gate_slab, const uint8_t* __restrict__ up_slab,
                                                           const int* __restrict__ ids, const BlockQ8* __restrict__ xq,
                                                           BlockQ8* __restrict__ xq_out, unsigned in_dim, unsigned out_dim,
                                                           unsigned bytes_per_expert, unsigned xq_tok_stride,
                                                           unsigned xq_slot_stride, unsigned n_used)
{
    __shared__ float vals[32];
    if (blockDim.x != 64u * (32u / R)) return;
    const unsigned tok = blockIdx.z, slot = blockIdx.y;
    if (blockIdx.x >= (out_dim >> 5)) return;
    const unsigned eid = (unsigned)ids[(size_t)tok * n_used + slot];
    rein_moe_gate_up_swiglu_q8_core<FMT, R>(gate_slab, up_slab, eid, xq + (size_t)tok * xq_tok_stride + (size_t)slot * xq_slot_stride,
                                         xq_out, in_dim, out_dim, bytes_per_expert, n_used, vals);
}

// The same with the router and quantize_q8_f32 in front, for the few-token expert FFN: every workgroup routes its
// token on its first wavefront (rein_topk::topk_one_wave: the ids and weight bits of moe_topk_f32) while all
// sixteen quantize the token's row into LDS (the bytes of quantize_q8_f32), then runs the launch above on its
// expert.  The workgroup (0, 0, tok) stores the token's ids and weights for the down projection.  One launch
// instead of three in front of the down projection: the router is a few microseconds of one wavefront's time,
// the launch it replaces costs as much on the whole GPU.  Up to 256 experts and 64 used; dynamic shared memory =
// in_dim / 32 * 40 bytes; grid = (out_dim / 32, n_used, n_tok) x 1024 threads.
template <int FMT, int R>
__device__ __forceinline__ void rein_moe_route_gate_up_swiglu_q8(const uint8_t* __restrict__ gate_slab, const uint8_t* __restrict__ up_slab,
                                                                 const float* __restrict__ logits, const float* __restrict__ x,
                                                                 int* __restrict__ ids_out, float* __restrict__ weights_out,
                                                                 BlockQ8* __restrict__ xq_out, unsigned in_dim, unsigned out_dim,
                                                                 unsigned bytes_per_expert, unsigned n_expert, unsigned n_used)
{
    extern __shared__ BlockQ8 rein_moe_xq_row[];             // in_dim / 32 blocks
    __shared__ float vals[32];
    __shared__ int ids_s[64];
    __shared__ float weights_s[64];
    if (blockDim.x != 64u * (32u / R)) return;
    const unsigned tok = blockIdx.z, slot = blockIdx.y;
    if (blockIdx.x >= (out_dim >> 5)) return;
    const unsigned n_sub = in_dim >> 5;
    if (threadIdx.x < 64u)
        rein_topk::topk_one_wave(logits + (size_t)tok * n_expert, (int)n_expert, (int)n_used, ids_s, weights_s, (int)threadIdx.x);
    const float* xr = x + (size_t)tok * in_dim;
    const unsigned l = threadIdx.x & 15u;
    for (unsigned sb = threadIdx.x >> 4; sb < n_sub; sb += blockDim.x >> 4) {
        const float* v = xr + (size_t)sb * 32 + l;
        rein_q8_store_sub(rein_moe_xq_row + sb, l, v[0], v[16]);
    }
    __syncthreads();
    if (blockIdx.x == 0u && slot == 0u && threadIdx.x < n_used) {
        ids_out[(size_t)tok * n_used + threadIdx.x] = ids_s[threadIdx.x];
        weights_out[(size_t)tok * n_used + threadIdx.x] = weights_s[threadIdx.x];
    }
    rein_moe_gate_up_swiglu_q8_core<FMT, R>(gate_slab, up_slab, (unsigned)ids_s[slot], rein_moe_xq_row, xq_out, in_dim, out_dim,
                                         bytes_per_expert, n_used, vals);
}

// down projection + weighted combine in one launch:
//   out[tok][i] = sum_j (weights[tok][j] * down_exps_s[ids[tok][j]]) * (W[ids[tok][j]] . xq[tok][j])[i]
// in slot order j = 0 .. n_used-1, a multiply and an add per slot (no fma): bit for bit what
// moe_matvec_*_f32 followed by moe_combine_f32 writes.  A workgroup owns R rows; its teams of
// LANES lanes take one slot each (all slots of a row group are in flight at once, as in the
// two-launch form), the per-slot results meet in LDS and thread r sums row r in slot order.
// grid = (row groups, 1, n_tok); any grid.x is correct; block a multiple of 64, at most 512.
template <int FMT, int R, int LANES>
__device__ __forceinline__ void rein_moe_down_combine(const uint8_t* __restrict__ slab, const int* __restrict__ ids,
                                                      const float* __restrict__ weights, const float* __restrict__ down_exps_s,
                                                      const BlockQ8* __restrict__ xq, float* __restrict__ out, unsigned in_dim,
                                                      unsigned out_dim, unsigned bytes_per_expert, unsigned xq_tok_stride,
                                                      unsigned xq_slot_stride, unsigned n_used)
{
#pragma clang fp contract(off)
    using F = Fmt<FMT>;
    constexpr unsigned kMaxTeams = 512 / LANES;
    __shared__ float vals[kMaxTeams][R];
    const unsigned n_teams = blockDim.x / LANES;
    if (n_teams == 0u || n_teams > kMaxTeams || (blockDim.x & 63u)) return;
    const unsigned tok = blockIdx.z;
    ids     += (size_t)tok * n_used;
    weights += (size_t)tok * n_used;
    out     += (size_t)tok * out_dim;
    const unsigned n_sub = in_dim >> 5;
    const unsigned lane = threadIdx.x & (LANES - 1u), team = threadIdx.x / LANES;
    const unsigned n_groups = (out_dim + R - 1) / R;
    const unsigned rmax = out_dim - 1;
    for (unsigned g = blockIdx.x; g < n_groups; g += gridDim.x) {
        const unsigned row0 = g * R;
        float acc = 0.0f;                                        // thread r < R: row row0 + r
        for (unsigned j0 = 0; j0 < n_used; j0 += n_teams) {
            // a team past the last slot repeats the last slot and stores nothing
            const unsigned j = min(j0 + team, n_used - 1u);
            const unsigned eid = (unsigned)ids[j];
            // the slots' scales are requested in front of the weights, so that the sum behind the barrier finds
            // them in registers instead of starting two dependent loads (ids -> down_exps_s) there
            const unsigned n_here = min(n_teams, n_used - j0);
            float scl[kMaxTeams];
            if (threadIdx.x < (unsigned)R) {
#pragma unroll
                for (unsigned t = 0; t < kMaxTeams; t++)
                    scl[t] = t < n_here ? weights[j0 + t] * down_exps_s[ids[j0 + t]] : 0.0f;
            }
            const F w(slab + (size_t)eid * bytes_per_expert, n_sub, out_dim);
            const BlockQ8* xqs = xq + (size_t)tok * xq_tok_stride + (size_t)j * xq_slot_stride;
            float s0[R], s1[R];
            rein_moe_row_sums<FMT, R, LANES, false>(w, w, xqs, n_sub, row0, rmax, lane, s0, s1);
            if (lane == 0u && j0 + team < n_used) {
#pragma unroll
                for (int r = 0; r < R; r++) vals[team][r] = s0[r];
            }
            __syncthreads();
            if (threadIdx.x < (unsigned)R) {
#pragma unroll
                for (unsigned t = 0; t < kMaxTeams; t++)
                    if (t < n_here) acc += scl[t] * vals[t][threadIdx.x];
            }
            __syncthreads();
        }
        if (threadIdx.x < (unsigned)R && row0 + threadIdx.x < out_dim) out[row0 + threadIdx.x] = acc;
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

// The two fused launches of the one-token expert FFN (no counterpart in the reference, which
// runs the four-launch chain of src/runtime/qwen35.rs:3071-3167).
#define REIN_DEFINE_MOE_GUQ8(name, FMT, R)                                                                \
    extern "C" __global__ __launch_bounds__(64 * (32 / R)) void name(                                     \
        const unsigned char* __restrict__ gate_slab, const unsigned char* __restrict__ up_slab,           \
        const int* __restrict__ ids, const BlockQ8* __restrict__ xq, BlockQ8* __restrict__ xq_out,        \
        unsigned int in_dim, unsigned int out_dim, unsigned int bytes_per_expert,                         \
        unsigned int xq_tok_stride, unsigned int xq_slot_stride, unsigned int n_used)                     \
    {                                                                                                     \
        rein_moe_gate_up_swiglu_q8<FMT, R>(gate_slab, up_slab, ids, xq, xq_out, in_dim, out_dim,          \
                                           bytes_per_expert, xq_tok_stride, xq_slot_stride, n_used);      \
    }
// two rows per wavefront and 1024 threads, or four and 512 (more bytes in flight per lane, half the wavefronts)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q4k, REIN_Q4_K, 2)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q4k_r4, REIN_Q4_K, 4)
// the other expert formats (the reference fuses gate + up + SwiGLU for Q4_K only and runs two matvecs otherwise)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q5k, REIN_Q5_K, 2)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q5k_r4, REIN_Q5_K, 4)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q6k, REIN_Q6_K, 2)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q6k_r4, REIN_Q6_K, 4)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q8_0, REIN_Q8_0, 2)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q8_0_r4, REIN_Q8_0, 4)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q5_1, REIN_Q5_1, 2)
REIN_DEFINE_MOE_GUQ8(rein_moe_gate_up_swiglu_q8_q5_1_r4, REIN_Q5_1, 4)

#define REIN_DEFINE_MOE_RGUQ8(name, FMT, R)                                                               \
    extern "C" __global__ __launch_bounds__(64 * (32 / R)) void name(                                     \
        const unsigned char* __restrict__ gate_slab, const unsigned char* __restrict__ up_slab,           \
        const float* __restrict__ logits, const float* __restrict__ x, int* __restrict__ ids_out,         \
        float* __restrict__ weights_out, BlockQ8* __restrict__ xq_out, unsigned int in_dim,               \
        unsigned int out_dim, unsigned int bytes_per_expert, unsigned int n_expert, unsigned int n_used)  \
    {                                                                                                     \
        rein_moe_route_gate_up_swiglu_q8<FMT, R>(gate_slab, up_slab, logits, x, ids_out, weights_out,     \
                                                 xq_out, in_dim, out_dim, bytes_per_expert, n_expert,     \
                                                 n_used);                                                 \
    }
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q4k, REIN_Q4_K, 2)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q4k_r4, REIN_Q4_K, 4)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q5k, REIN_Q5_K, 2)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q5k_r4, REIN_Q5_K, 4)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q6k, REIN_Q6_K, 2)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q6k_r4, REIN_Q6_K, 4)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q8_0, REIN_Q8_0, 2)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q8_0_r4, REIN_Q8_0, 4)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q5_1, REIN_Q5_1, 2)
REIN_DEFINE_MOE_RGUQ8(rein_moe_route_gate_up_swiglu_q8_q5_1_r4, REIN_Q5_1, 4)

#define REIN_DEFINE_MOE_DC(name, FMT, R, LANES)                                                           \
    extern "C" __global__ __launch_bounds__(512) void name(                                               \
        const unsigned char* __restrict__ slab, const int* __restrict__ ids, const float* __restrict__ weights, \
        const float* __restrict__ down_exps_s, const BlockQ8* __restrict__ xq, float* __restrict__ out,   \
        unsigned int in_dim, unsigned int out_dim, unsigned int bytes_per_expert,                         \
        unsigned int xq_tok_stride, unsigned int xq_slot_stride, unsigned int n_used)                     \
    {                                                                                                     \
        rein_moe_down_combine<FMT, R, LANES>(slab, ids, weights, down_exps_s, xq, out, in_dim, out_dim,   \
                                             bytes_per_expert, xq_tok_stride, xq_slot_stride, n_used);    \
    }
// Two, four or eight rows per workgroup (the host takes the most rows that still leave the machine four workgroups
// per CU: more rows are more bytes in flight per lane and fewer workgroups to start -- 16 tokens x 128 experts
// top-8, Q6_K 768 -> 2048: 110 / 99 / 96 us per FFN at 2 / 4 / 8 rows, one token 15.6 / 15.5 / 16.0).  Short
// contractions (at most 32 sub-blocks): half-wavefront teams (_h), as the *_down symbols.
#define REIN_DEFINE_MOE_DC_ROWS(stem, FMT)                      \
    REIN_DEFINE_MOE_DC(stem##_h, FMT, 2, 32)                    \
    REIN_DEFINE_MOE_DC(stem##_h_r4, FMT, 4, 32)                 \
    REIN_DEFINE_MOE_DC(stem##_h_r8, FMT, 8, 32)                 \
    REIN_DEFINE_MOE_DC(stem, FMT, 2, 64)                        \
    REIN_DEFINE_MOE_DC(stem##_r4, FMT, 4, 64)                   \
    REIN_DEFINE_MOE_DC(stem##_r8, FMT, 8, 64)
REIN_DEFINE_MOE_DC_ROWS(rein_moe_down_combine_q4k, REIN_Q4_K)
REIN_DEFINE_MOE_DC_ROWS(rein_moe_down_combine_q5k, REIN_Q5_K)
REIN_DEFINE_MOE_DC_ROWS(rein_moe_down_combine_q6k, REIN_Q6_K)
REIN_DEFINE_MOE_DC_ROWS(rein_moe_down_combine_q8_0, REIN_Q8_0)
REIN_DEFINE_MOE_DC_ROWS(rein_moe_down_combine_q5_1, REIN_Q5_1)
