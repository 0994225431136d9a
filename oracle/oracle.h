/*
 * CPU oracle for the quantized-weight matmul path of sixvolts/reinstinct.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * algorithm (formats, repack-v2 layouts, quantize_q8, per-block integer dots,
 * fp32 combine, the dequantize -> f32 matvec CPU path and the MoE glue).  It is
 * linked or loaded only by the tests, by the smoke check and by the
 * cpu_baseline leg of the benchmark, always as the checker and never as the
 * thing measured or shipped.  The product library does not link it.
 *
 * Every function cites the reference file:line it restates (paths relative to
 * the reference checkout).
 *
 * What pins each function (checked in tests/test_oracle_*.py):
 *   orc_f16_to_f32 / orc_f32_to_f16  known values half.rs:93-106,132-135 and an
 *                                    exhaustive cross-check against numpy.float16
 *   orc_get_scale_min_k4, dequant    closed forms from the unit tests of
 *                                    q4_k.rs, q5_k.rs, q6_k.rs, q4_0.rs,
 *                                    q8_0.rs, iq4_xs.rs
 *   repack / decode_repacked         decode(repack(w)) == dequant(w) (the
 *                                    reference's own invariant), byte-level
 *                                    expectations of q4_0.rs:132-160, pad rule
 *   orc_q8_0_quantize_from_f32       closed forms (q8_0.rs:45-61)
 *   orc_quantize_q8                  special cases + invariants; the reciprocal
 *                                    is IEEE 127/amax (the reference uses the
 *                                    gfx906 v_rcp_f32 approximation, which has
 *                                    no portable bit-exact definition):
 *                                    PARITY UNPINNED at bit level vs the
 *                                    reference kernel for that one rounding.
 *   orc_block_dots, orc_matvec_q8    integer-activation identity against
 *                                    dequant -> f32 matvec; brute force
 *   orc_moe_*                        textbook softmax/top-k, sort invariants,
 *                                    closed forms
 *   orc_exp_det and the functions    libm expf / tanhf to a few ulp over the whole
 *   built on it; orc_*_q8            range, the known values of ops.rs:176-188, the
 *                                    reference CPU forms (orc_rmsnorm_ref etc.,
 *                                    ops.rs:14-76) to rounding, and the identity
 *                                    fused == quantize_q8(unfused)
 */
#ifndef REIN_ORACLE_H
#define REIN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Format ids = the reference's GgmlType discriminants (src/gguf/types.rs:16-35). */
enum {
    ORC_Q4_0   = 2,
    ORC_Q8_0   = 8,
    ORC_Q4_K   = 12,
    ORC_Q5_K   = 13,
    ORC_Q6_K   = 14,
    ORC_IQ4_XS = 23,
    ORC_Q5_1   = 7,    /* runs on the Q5_K kernels with raw (d, m) scales, src/quant/q5_1.rs:12-20 */
    ORC_IQ3_S  = 21    /* runs on the IQ4_XS kernels with the codebook 2n-15, src/quant/iq3_s.rs:13-19 */
};

/* src/quant/half.rs:9-40, 51-84 */
float    orc_f16_to_f32(uint16_t bits);
uint16_t orc_f32_to_f16(float value);

/* weights per on-disk block / bytes per on-disk block; 0 for unknown fmt */
int orc_block_size(int fmt);
int orc_bytes_per_block(int fmt);

/* src/quant/q4_k.rs:40-48 */
void orc_get_scale_min_k4(int j, const uint8_t *q12, uint8_t *sc, uint8_t *m);

/* <fmt>::dequantize_to_f32 — n_elems must be a multiple of the block size.
 * returns 0, or -1 on a bad format/size. */
int orc_dequantize_to_f32(int fmt, const uint8_t *bytes, float *out, size_t n_elems);

/* repacked_n_sub_padded (q4_k.rs:92-95 and its per-format twins) */
size_t orc_repacked_n_sub_padded(size_t in_dim);
/* <fmt>::repacked_len */
size_t orc_repacked_len(int fmt, size_t in_dim, size_t out_dim);
/* <fmt>::repack_for_matvec; `out` must hold orc_repacked_len bytes (zeroed here). */
int orc_repack_for_matvec(int fmt, const uint8_t *bytes, size_t in_dim, size_t out_dim,
                          uint8_t *out);
/* Read the repacked planes back to f32 with the kernels' index arithmetic
 * (q4_k.rs:276-299 style).  Output is [out_dim][in_dim] in original weight
 * order, i.e. directly comparable with orc_dequantize_to_f32. */
int orc_decode_repacked_to_f32(int fmt, const uint8_t *packed, size_t in_dim, size_t out_dim,
                               float *out);

/* q8_0::quantize_from_f32 (q8_0.rs:45-61); out = n/32 blocks of 34 bytes */
void orc_q8_0_quantize_from_f32(const float *vals, size_t n, uint8_t *out);

/* kernels/quantize_q8.cpp:23-54 — out is n_vec * (in_dim/32) packed 40-byte
 * blocks {f32 d; f32 xsum; i8 qs[32]} */
void orc_quantize_q8(const float *x, size_t in_dim, size_t n_vec, uint8_t *out);

/* Number of int32 values per (token,row,sub-block) that orc_block_dots emits:
 * 2 for Q6_K (one per 16-weight half, each already minus 32*sum(q8)), 1 otherwise
 * (Q4_0: idot - 8*sum(q8); others: the raw dot). */
int orc_block_dot_parts(int fmt);
/* Per-block integer dots exactly as the matvec kernels form them
 * (matvec_*_repacked.cpp inner loops).  out[((t*out_dim + r)*n_sub + sb)*parts + p] */
int orc_block_dots(int fmt, const uint8_t *packed, size_t in_dim, size_t out_dim,
                   const uint8_t *xq, size_t n_rows, int32_t *out);
/* int8 path: y[t][r] = sum over sub-blocks of the per-format fp32 combine,
 * accumulated in the reference's order (lane-strided partials, then the
 * xor-1,2,4,8,16,32 tree of kernels/gfx906_dpp.h:69-77). */
int orc_matvec_q8(int fmt, const uint8_t *packed, size_t in_dim, size_t out_dim,
                  const uint8_t *xq, size_t n_rows, float *y, int n_threads);

/* src/cpu/ops.rs:108-140 — the reference's CPU path after dequantize_to_f32:
 * y[j] = sum_i x[i]*w[j*in_dim+i], sequential in i, rows split over threads
 * when in_dim*out_dim >= 65536 (n_threads<=1 keeps it sequential). */
void orc_matvec_f32(const float *x, const float *w, size_t in_dim, size_t out_dim, float *y,
                    int n_threads);

/* kernels/moe_topk.cpp:17-108 */
void orc_moe_topk(const float *logits, int n_tok, int n_expert, int n_used, int32_t *out_ids,
                  float *out_weights);
/* kernels/moe_expert_sort.cpp:27-75 — stable (entry-order) variant; the GPU
 * order inside one expert is free. expert_off/tile_off have n_expert+1 entries. */
void orc_moe_sort(const int32_t *ids, int n_entries, int n_expert, int bn, int32_t *perm,
                  int32_t *expert_off, int32_t *tile_off);
/* kernels/moe_expert_sort.cpp:81-110 */
void orc_moe_gather_xq(const uint8_t *xq_src, const int32_t *perm, uint8_t *xq_dst, int nsub,
                       int n_used, int n_entries);
void orc_moe_scatter_rows(const float *src, const int32_t *perm, float *dst, int dim,
                          int n_entries);
/* kernels/moe_combine.cpp:15-38 */
void orc_moe_combine(const float *experts, const int32_t *ids, const float *weights,
                     const float *down_exps_s, float *out, int n_tok, int hidden, int n_used);
/* ---- fused BlockQ8 producers -------------------------------------------------
 * Deterministic elementwise functions: IEEE add/mul/fma/div/sqrt only, in the
 * order the device code spells out, so that device and checker agree bit for bit.
 * exp: n = rint(x*log2 e), two-step fma reduction by ln 2, degree-6 Horner, scaled
 * by 2^n in two exact steps; x clamped to [-87, 88]. */
float orc_exp_det(float x);
float orc_silu_det(float x);      /* x / (1 + exp(-x))           src/cpu/ops.rs:14-16 */
float orc_sigmoid_det(float x);   /* 1 / (1 + exp(-x))           src/cpu/ops.rs:20-22 */
float orc_gelu_det(float x);      /* tanh form as x / (1 + exp(-2z))   src/cpu/ops.rs:33-36 */
void orc_map_det(int which, const float *x, float *out, size_t n);   /* 0 exp 1 silu 2 sigmoid 4 gelu */
/* sum of squares in the order of the fused norm kernels: per 32-value sub-block
 * the xor butterfly 16..1, then 64 strided running sums, then the butterfly 32..1 */
float orc_sumsq_det(const float *x, size_t n);
/* kernels/qwen35_fused.cpp:66-121 (add may be NULL; hidden is updated when it is
 * not): y[v] = ((hidden[v] * rrms) * w), rrms = 1 / sqrt(sumsq/n + eps) */
void orc_add_rmsnorm(float *hidden, const float *add, const float *w, float *y, size_t n, size_t n_vec, float eps);
/* kernels/qwen35_fused.cpp:195-217: y = ((x * rrms) * w) * silu(z) per head */
void orc_rmsnorm_gated(const float *x, const float *z, const float *w, float *y, size_t n_heads, size_t head_dim, float eps);
/* kernels/qwen35_fused.cpp:132-146 / 149-162 / kernels/moe_geglu_q8.cpp:31-66 (fp32 results;
 * the BlockQ8 form is orc_quantize_q8 of them) */
void orc_swiglu_det(const float *gate, const float *up, float *out, size_t n);
void orc_sigmoid_mul_det(const float *x, const float *gate, float *out, size_t n);
void orc_geglu_det(const float *gu, float *out, size_t ff_exp, size_t n_slot);
/* The reference's CPU forms, libm and sequential sums: src/cpu/ops.rs:47-57, 63-76,
 * 14-16, 20-22, 33-36.  which: 1 silu 2 sigmoid 4 gelu */
void orc_rmsnorm_ref(const float *x, const float *w, float eps, float *out, size_t n);
void orc_rmsnorm_gated_ref(const float *x, const float *gate, const float *w, float eps, float *out, size_t n);
void orc_map_ref(int which, const float *x, float *out, size_t n);

/* ---- relabelled GGUF types: CPU dequantizers of the source formats -----------------
 * src/quant/q3_k.rs:124-165 (110-byte blocks), src/quant/iq4_nl.rs:34-50 (18-byte blocks),
 * src/quant/half.rs:42-46 (bf16 = high half of an f32) */
void orc_q3_k_dequantize(const uint8_t *src, float *out, size_t n);
void orc_iq4_nl_dequantize(const uint8_t *src, float *out, size_t n);
/* entry idx (0..511) of the IQ3_S grid as the reference states it: four magnitude bytes,
 * weight 0 in the low byte (IQ3S_GRID, src/quant/iq3_s.rs:41-107) */
uint32_t orc_iq3s_grid_entry(int idx);
void orc_bf16_to_f32(const uint16_t *src, float *out, size_t n);

/* kernels/swiglu.cpp:10-21 (expf in place of __expf) */
void orc_swiglu_mul(const float *gate, const float *up, float *out, size_t n);
/* kernels/mmq_gemm_q4k_grouped.cpp:38-165 — per expert e, rows
 * expert_off[e]..expert_off[e+1] of the sorted xq/y against slab + e*bytes_per_expert */
int orc_grouped_gemm(int fmt, const uint8_t *slab, size_t bytes_per_expert,
                     const int32_t *expert_off, int n_expert, const uint8_t *xq, float *y,
                     size_t in_dim, size_t out_dim, int n_threads);

#ifdef __cplusplus
}
#endif
#endif
