// The matvec call sites that are left once every layer weight is repacked:
//
//   * matvec_{q4_k,q5_k,q6_k,q8_0}_dp4a_f32: weights in the ON-DISK (GGUF) block
//     layout.  Only a tied token_embd that doubles as the output projection still
//     reaches them (src/runtime/qwen35.rs:2209-2229): the embedding lookup wants the
//     on-disk blocks, so the matrix is not repacked.  Same symbols and arguments as
//     kernels/matvec_q4_k_dp4a.cpp:52-116 and its Q5_K / Q6_K / Q8_0 siblings.
//   * matvec_q8_0_repacked_splitk_f32: split-K over grid.y for projections with a
//     tiny out_dim (kernels/matvec_q8_0_repacked.cpp:117-176): partial sums go to
//     y[blockIdx.y][out_dim], the consumer adds them.
//
// Lane l of a wavefront walks sub-blocks l, l+64, ... of R rows exactly as the
// repacked matvec does; only the address arithmetic differs (a sub-block's bytes sit
// inside its 256-weight block), and the per-sub-block math is Fmt<FMT>::term.  Any
// grid.x and any block that is a multiple of 64 is correct.
#include "rein_formats.h"

// One sub-block of one row, read from on-disk blocks into dot order.
template <int FMT> struct DiskFmt;

// ggml get_scale_min_k4 (src/quant/q4_k.rs:40-48) on the 12 scale bytes held as three dwords
__device__ __forceinline__ void rein_scale_min_k4(unsigned j, const uint32_t s[3], uint32_t& sc, uint32_t& m)
{
    auto byte = [&](unsigned i) { return (s[i >> 2] >> (8u * (i & 3u))) & 0xFFu; };
    if (j < 4u) {
        sc = byte(j) & 63u;
        m  = byte(j + 4u) & 63u;
    } else {
        sc = (byte(j + 4u) & 0x0Fu) | ((byte(j - 4u) >> 6) << 4);
        m  = (byte(j + 4u) >> 4) | ((byte(j) >> 6) << 4);
    }
}

// Q4_K block, 144 B: {f16 d, f16 dmin, u8 scales[12], u8 qs[128]}; sub-block j holds
// the low (j even) or high (j odd) nibbles of qs[32*(j/2) .. +32)  (src/quant/q4_k.rs:50-84)
template <> struct DiskFmt<REIN_Q4_K> {
    static constexpr unsigned kBlock = 144;
    static __device__ __forceinline__ void load(const uint8_t* w, size_t row, unsigned n_sub, unsigned sb, SubW& s)
    {
        const uint8_t* blk = w + (row * (n_sub >> 3) + (sb >> 3)) * kBlock;
        const unsigned j = sb & 7u, shift = 4u * (j & 1u);
        const uint4* qs = reinterpret_cast<const uint4*>(blk + 16 + 32 * (j >> 1));
        const uint4 a = qs[0], b = qs[1];
        const uint32_t q[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int k = 0; k < 8; k++) s.w[k] = (int)((q[k] >> shift) & 0x0F0F0F0Fu);
        const uint32_t* h = reinterpret_cast<const uint32_t*>(blk);
        const uint32_t sc3[3] = {h[1], h[2], h[3]};
        uint32_t sc, m;
        rein_scale_min_k4(j, sc3, sc, m);
        s.s0 = rein_h2f((uint16_t)(h[0] & 0xFFFFu)) * (float)sc;
        s.s1 = rein_h2f((uint16_t)(h[0] >> 16)) * (float)m;
    }
};

// Q5_K block, 176 B: {d, dmin, scales[12], u8 qh[32], u8 qs[128]}; weight i of
// sub-block j = nibble as in Q4_K | bit j of qh[i] << 4  (src/quant/q5_k.rs:47-86)
template <> struct DiskFmt<REIN_Q5_K> {
    static constexpr unsigned kBlock = 176;
    static __device__ __forceinline__ void load(const uint8_t* w, size_t row, unsigned n_sub, unsigned sb, SubW& s)
    {
        const uint8_t* blk = w + (row * (n_sub >> 3) + (sb >> 3)) * kBlock;
        const unsigned j = sb & 7u, shift = 4u * (j & 1u);
        const uint4* qh = reinterpret_cast<const uint4*>(blk + 16);
        const uint4* qs = reinterpret_cast<const uint4*>(blk + 48 + 32 * (j >> 1));
        const uint4 a = qs[0], b = qs[1], ha = qh[0], hb = qh[1];
        const uint32_t q[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        const uint32_t h8[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
#pragma unroll
        for (int k = 0; k < 8; k++)
            s.w[k] = (int)(((q[k] >> shift) & 0x0F0F0F0Fu) | (((h8[k] >> j) & 0x01010101u) << 4));
        const uint32_t* h = reinterpret_cast<const uint32_t*>(blk);
        const uint32_t sc3[3] = {h[1], h[2], h[3]};
        uint32_t sc, m;
        rein_scale_min_k4(j, sc3, sc, m);
        s.s0 = rein_h2f((uint16_t)(h[0] & 0xFFFFu)) * (float)sc;
        s.s1 = rein_h2f((uint16_t)(h[0] >> 16)) * (float)m;
    }
};

// Q6_K block, 210 B (2-byte aligned): {u8 ql[128], u8 qh[64], i8 scales[16], f16 d}.
// Sub-block j = 4n + g: weight l = nibble (g >> 1) of ql[64n + 32(g & 1) + l] |
// bits 2g..2g+1 of qh[32n + l] << 4, scale scales[8n + 2g + l/16]; the -32 offset is
// folded by Fmt<REIN_Q6_K>::term  (src/quant/q6_k.rs:31-69)
struct __attribute__((packed, aligned(2))) ReinU32A2 { uint32_t v; };
template <> struct DiskFmt<REIN_Q6_K> {
    static constexpr unsigned kBlock = 210;
    static __device__ __forceinline__ void load(const uint8_t* w, size_t row, unsigned n_sub, unsigned sb, SubW& s)
    {
        const uint8_t* blk = w + (row * (n_sub >> 3) + (sb >> 3)) * kBlock;
        const unsigned j = sb & 7u, n = j >> 2, g = j & 3u;
        const ReinU32A2* ql = reinterpret_cast<const ReinU32A2*>(blk + 64 * n + 32 * (g & 1u));
        const ReinU32A2* qh = reinterpret_cast<const ReinU32A2*>(blk + 128 + 32 * n);
        const unsigned lo_shift = 4u * (g >> 1), hi_shift = 2u * g;
#pragma unroll
        for (int k = 0; k < 8; k++)
            s.w[k] = (int)(((ql[k].v >> lo_shift) & 0x0F0F0F0Fu) | (((qh[k].v >> hi_shift) & 0x03030303u) << 4));
        const uint16_t sm = *reinterpret_cast<const uint16_t*>(blk + 192 + 8 * n + 2 * g);
        const float d = rein_h2f(*reinterpret_cast<const uint16_t*>(blk + 208));
        s.s0 = d * (float)(int)(int8_t)(sm & 0xFFu);
        s.s1 = d * (float)(int)(int8_t)(sm >> 8);
    }
};

// Q8_0 block, 34 B (2-byte aligned): {f16 d, i8 qs[32]}  (src/quant/q8_0.rs:13-38)
template <> struct DiskFmt<REIN_Q8_0> {
    static constexpr unsigned kBlock = 34;
    static __device__ __forceinline__ void load(const uint8_t* w, size_t row, unsigned n_sub, unsigned sb, SubW& s)
    {
        const uint8_t* blk = w + (row * n_sub + sb) * kBlock;
        const ReinU32A2* q = reinterpret_cast<const ReinU32A2*>(blk + 2);
#pragma unroll
        for (int k = 0; k < 8; k++) s.w[k] = (int)q[k].v;
        s.s0 = rein_h2f(*reinterpret_cast<const uint16_t*>(blk));
        s.s1 = 0.0f;
    }
};

template <int FMT, int R>
__device__ __forceinline__ void rein_matvec_ondisk(const uint8_t* __restrict__ w, const BlockQ8* __restrict__ xq,
                                                   float* __restrict__ y, unsigned in_dim, unsigned out_dim)
{
    using F = Fmt<FMT>;
    const unsigned lane = threadIdx.x & 63u, wpb = blockDim.x >> 6;
    const unsigned n_sub = in_dim >> 5;
    const unsigned n_groups = (out_dim + R - 1) / R, rmax = out_dim - 1;
    for (unsigned g = blockIdx.x * wpb + (threadIdx.x >> 6); g < n_groups; g += gridDim.x * wpb) {
        const unsigned row0 = g * R;
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = 0.0f;
        for (unsigned sb0 = 0; sb0 < n_sub; sb0 += 64) {
            const bool live = sb0 + lane < n_sub;
            const unsigned sb = live ? sb0 + lane : n_sub - 1;
            SubW sw[R];
#pragma unroll
            for (int r = 0; r < R; r++) DiskFmt<FMT>::load(w, min(row0 + r, rmax), n_sub, sb, sw[r]);
            const BlockQ8* p = xq + sb;
            const float dx = live ? p->d : 0.0f, xsum = live ? p->xsum : 0.0f;
            int q[8];
#pragma unroll
            for (int j = 0; j < 8; j++) q[j] = p->qs[j];
            XSums xs;
            if (F::kNeedsXSums) xs = rein_xsums(q);
            else { xs.lo = 0; xs.hi = 0; }
#pragma unroll
            for (int r = 0; r < R; r++) {
                int i0 = 0, i1 = 0;
#pragma unroll
                for (int j = 0; j < 4; j++) { i0 = rein_dot4(sw[r].w[j], q[j], i0); i1 = rein_dot4(sw[r].w[j + 4], q[j + 4], i1); }
                acc[r] += F::term(sw[r], i0, i1, dx, xsum, xs);
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float s = rein_wave_sum(acc[r]);
            if (lane == 0 && row0 + r < out_dim) y[row0 + r] = s;
        }
    }
}

#define REIN_DEFINE_MATVEC_ONDISK(name, FMT)                                                                  \
    extern "C" __global__ __launch_bounds__(256) void name(const unsigned char* __restrict__ w_blocks,        \
                                                           const BlockQ8* __restrict__ xq, float* __restrict__ y, \
                                                           unsigned int in_dim, unsigned int out_dim)        \
    {                                                                                                         \
        rein_matvec_ondisk<FMT, 2>(w_blocks, xq, y, in_dim, out_dim);                                         \
    }

REIN_DEFINE_MATVEC_ONDISK(matvec_q4_k_dp4a_f32, REIN_Q4_K)
REIN_DEFINE_MATVEC_ONDISK(matvec_q5_k_dp4a_f32, REIN_Q5_K)
REIN_DEFINE_MATVEC_ONDISK(matvec_q6_k_dp4a_f32, REIN_Q6_K)
REIN_DEFINE_MATVEC_ONDISK(matvec_q8_0_dp4a_f32, REIN_Q8_0)

// Split-K over repacked Q8_0: blockIdx.y owns sub-blocks [y*chunk, (y+1)*chunk),
// chunk = ceil(n_sub / n_split), and writes its partial sums to y[blockIdx.y][out_dim].
extern "C" __global__ __launch_bounds__(256)
void matvec_q8_0_repacked_splitk_f32(const unsigned char* __restrict__ slab, const BlockQ8* __restrict__ xq,
                                     float* __restrict__ y, unsigned int in_dim, unsigned int out_dim,
                                     unsigned int n_split)
{
    using F = Fmt<REIN_Q8_0>;
    constexpr int R = 2;
    const unsigned lane = threadIdx.x & 63u, wpb = blockDim.x >> 6;
    const unsigned n_sub = in_dim >> 5;
    const F fmt(slab, n_sub, out_dim);
    const unsigned chunk = (n_sub + n_split - 1) / n_split;
    const unsigned n_groups = (out_dim + R - 1) / R, rmax = out_dim - 1;
    for (unsigned part = blockIdx.y; part < n_split; part += gridDim.y) {
        const unsigned sb_lo = part * chunk, sb_hi = min(sb_lo + chunk, n_sub);
        for (unsigned g = blockIdx.x * wpb + (threadIdx.x >> 6); g < n_groups; g += gridDim.x * wpb) {
            const unsigned row0 = g * R;
            float acc[R] = {0.0f, 0.0f};
            for (unsigned sb0 = sb_lo; sb0 < sb_hi; sb0 += 64) {
                const bool live = sb0 + lane < sb_hi;
                const unsigned sb = live ? sb0 + lane : n_sub - 1;
                F::Raw raw[R];
#pragma unroll
                for (int r = 0; r < R; r++) raw[r] = fmt.load(min(row0 + r, rmax), sb);
                const BlockQ8* p = xq + sb;
                const float dx = live ? p->d : 0.0f;
                int q[8];
#pragma unroll
                for (int j = 0; j < 8; j++) q[j] = p->qs[j];
                XSums xs;
                xs.lo = 0; xs.hi = 0;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    SubW sw;
                    F::unpack(raw[r], sw);
                    int i0 = 0, i1 = 0;
#pragma unroll
                    for (int j = 0; j < 4; j++) { i0 = rein_dot4(sw.w[j], q[j], i0); i1 = rein_dot4(sw.w[j + 4], q[j + 4], i1); }
                    acc[r] += F::term(sw, i0, i1, dx, 0.0f, xs);
                }
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float s = rein_wave_sum(acc[r]);
                if (lane == 0 && row0 + r < out_dim) y[(size_t)part * out_dim + row0 + r] = s;
            }
        }
    }
}
