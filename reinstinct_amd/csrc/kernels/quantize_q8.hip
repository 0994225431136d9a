// fp32 activations -> BlockQ8 {f32 d; f32 xsum; i8 qs[32]} (40 B per 32 values).
//
// Replaces kernels/quantize_q8.cpp:23-54 of the reference: same symbol, same
// arguments, same output format.  Correct under the reference launch
// (grid = (ceil(in_dim/256), n_vec), block = 256) and under any other grid.x /
// blockDim.x that is a multiple of 16: 16-lane rows stride over sub-blocks.
//
// Bit-level definition (shared with the CPU oracle) in rein_q8_store_sub: amax and
// sum are reduced with the xor butterfly 16, 8, 4, 2, 1; d = amax/127 and
// inv = 127/amax are IEEE divisions; q = clamp(rint(v*inv), -127, 127), ties to even.
#include "q8_block.h"

extern "C" __global__ __launch_bounds__(1024)
void quantize_q8_f32(const float* __restrict__ x, BlockQ8* __restrict__ out, unsigned int in_dim)
{
    const unsigned vec = blockIdx.y;
    const unsigned n_sub = in_dim >> 5;
    x   += (size_t)vec * in_dim;
    out += (size_t)vec * n_sub;

    // one 16-lane row per sub-block, two values per lane
    const unsigned rows_per_block = blockDim.x >> 4;
    const unsigned l = threadIdx.x & 15u;
    for (unsigned blk = blockIdx.x * rows_per_block + (threadIdx.x >> 4); blk < n_sub;
         blk += gridDim.x * rows_per_block) {
        const float* v = x + (size_t)blk * 32 + l;
        rein_q8_store_sub(out + blk, l, v[0], v[16]);
    }
}

// quantize_q8_f32 + moe_gather_xq in one launch: every token row is quantized once and each
// finished block is written to the n_used places its routing entries have in the
// expert-sorted order (inv[tok * n_used + j], as the sort records them; negative = dropped
// entry) -- the same bytes as the two launches, without the quantized table between them.
// grid = (blocks of rows, n_tok); any grid.x and any block that is a multiple of 16.
extern "C" __global__ __launch_bounds__(1024)
void rein_moe_quantize_scatter(const float* __restrict__ x, const int* __restrict__ inv, BlockQ8* __restrict__ out,
                               unsigned int in_dim, unsigned int n_used, unsigned int n_entries)
{
    const unsigned tok = blockIdx.y;
    const unsigned n_sub = in_dim >> 5;
    x   += (size_t)tok * in_dim;
    inv += (size_t)tok * n_used;
    const unsigned rows_per_block = blockDim.x >> 4;
    const unsigned l = threadIdx.x & 15u;
    for (unsigned blk = blockIdx.x * rows_per_block + (threadIdx.x >> 4); blk < n_sub; blk += gridDim.x * rows_per_block) {
        const float* v = x + (size_t)blk * 32 + l;
        const ReinQ8Lane q = rein_q8_quantize_sub(v[0], v[16]);
        for (unsigned j = 0; j < n_used; j++) {
            const int pos = inv[j];
            if (pos >= 0 && (unsigned)pos < n_entries) rein_q8_store_lane(out + (size_t)pos * n_sub + blk, l, q);
        }
    }
}
