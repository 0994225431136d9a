// fp32 activations -> BlockQ8 {f32 d; f32 xsum; i8 qs[32]} (40 B per 32 values).
//
// Replaces kernels/quantize_q8.cpp:23-54 of the reference: same symbol, same
// arguments, same output format.  Correct under the reference launch
// (grid = (ceil(in_dim/256), n_vec), block = 256) and under any other grid.x /
// blockDim.x that is a multiple of 32: 32-lane groups stride over sub-blocks.
//
// Bit-level definition (shared with the CPU oracle): amax and sum are reduced
// with the xor butterfly 16, 8, 4, 2, 1; d = amax/127 and inv = 127/amax are
// IEEE divisions; q = clamp(rint(v*inv), -127, 127) with ties to even.
#include "rein_common.h"

extern "C" __global__ __launch_bounds__(1024)
void quantize_q8_f32(const float* __restrict__ x, BlockQ8* __restrict__ out, unsigned int in_dim)
{
#pragma clang fp contract(off)
    const unsigned vec = blockIdx.y;
    const unsigned n_sub = in_dim >> 5;
    x   += (size_t)vec * in_dim;
    out += (size_t)vec * n_sub;

    const unsigned groups_per_block = blockDim.x >> 5;
    const unsigned l = threadIdx.x & 31u;
    for (unsigned blk = blockIdx.x * groups_per_block + (threadIdx.x >> 5); blk < n_sub;
         blk += gridDim.x * groups_per_block) {
        const float v = x[(size_t)blk * 32 + l];
        float amax = fabsf(v);
        float sum  = v;
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) {
            amax = fmaxf(amax, __shfl_xor(amax, o));
            sum  = sum + __shfl_xor(sum, o);
        }
        const float d   = amax > 0.0f ? amax / 127.0f : 1.0f;
        const float inv = amax > 0.0f ? 127.0f / amax : 0.0f;
        int q = (int)rintf(v * inv);
        q = max(-127, min(127, q));

        // pack four quants per lane-quad into one dword store
        const int b  = q & 0xFF;
        const int w0 = b | (__shfl_down(b, 1) << 8) | (__shfl_down(b, 2) << 16) | (__shfl_down(b, 3) << 24);
        BlockQ8* o = out + blk;
        if ((l & 3u) == 0u) o->qs[l >> 2] = w0;
        if (l == 0u) { o->d = d; o->xsum = sum; }
    }
}
