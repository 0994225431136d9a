// Shared device helpers for the gfx950 (CDNA4, wave64) quantized-matmul kernels.
//
// Activation block layout follows the reference's BlockQ8
// (kernels/quantize_q8.cpp:16-21): packed {f32 d; f32 xsum; i8 qs[32]} = 40 B.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define REIN_WAVE 64

// 40-byte activation block. Rows of blocks are 8-byte aligned only, so the
// struct is declared with 4-byte alignment and read with dword loads.
struct __attribute__((packed, aligned(4))) BlockQ8 {
    float   d;
    float   xsum;
    int32_t qs[8];   // 32 int8, word j = quants 4j..4j+3
};
static_assert(sizeof(BlockQ8) == 40, "BlockQ8 must be 40 bytes");

// Sub-blocks per repacked row: one pad sub-block when the count is a power of
// two (must match quant::*::repacked_n_sub_padded, src/quant/q4_k.rs:92-95).
__device__ __forceinline__ unsigned rein_nsp(unsigned n_sub)
{
    return ((n_sub & (n_sub - 1u)) == 0u) ? (n_sub + 1u) : n_sub;
}

__device__ __forceinline__ float rein_h2f(uint16_t bits)
{
    return (float)__builtin_bit_cast(_Float16, bits);
}

__device__ __forceinline__ int rein_dot4(int a, int b, int c)
{
    return __builtin_amdgcn_sdot4(a, b, c, false);
}

// ---- wave64 reductions over DPP (gfx9 row ops + row broadcasts) -------------
// dpp_ctrl encodings: quad_perm = low 8 bits; row_half_mirror 0x141;
// row_mirror 0x140; row_bcast15 0x142; row_bcast31 0x143.
// row_shl:n 0x100+n (lane <- lane+n), row_shr:n 0x110+n (lane <- lane-n),
// row_ror:n 0x120+n.  Lanes masked out by ROW_MASK / BANK_MASK (bank = 4 lanes of a
// row) keep `old`.
template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF>
__device__ __forceinline__ float rein_dpp_f32(float old, float v)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v),
                                           CTRL, ROW_MASK, BANK_MASK, false));
}

// Sum over the 16 lanes of each DPP row; every lane of the row ends with it.
__device__ __forceinline__ float rein_row16_sum(float v)
{
    v += rein_dpp_f32<0xB1>(0.0f, v);    // quad_perm [1,0,3,2]  : lane ^ 1
    v += rein_dpp_f32<0x4E>(0.0f, v);    // quad_perm [2,3,0,1]  : lane ^ 2
    v += rein_dpp_f32<0x141>(0.0f, v);   // row_half_mirror      : quad <-> quad within 8
    v += rein_dpp_f32<0x140>(0.0f, v);   // row_mirror           : low 8 <-> high 8
    return v;
}

// Full wave64 sum, result valid in every lane (uniform).
__device__ __forceinline__ float rein_wave_sum(float v)
{
    v = rein_row16_sum(v);
    const int b = __builtin_bit_cast(int, v);
    float s = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
    s += __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
    s += __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
    s += __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
    return s;
}

__device__ __forceinline__ float rein_wave_max(float v)
{
    v = fmaxf(v, rein_dpp_f32<0xB1>(v, v));
    v = fmaxf(v, rein_dpp_f32<0x4E>(v, v));
    v = fmaxf(v, rein_dpp_f32<0x141>(v, v));
    v = fmaxf(v, rein_dpp_f32<0x140>(v, v));
    const int b = __builtin_bit_cast(int, v);
    float s = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
    s = fmaxf(s, __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)));
    s = fmaxf(s, __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)));
    s = fmaxf(s, __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48)));
    return s;
}
