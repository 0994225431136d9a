// Grouped-expert MMQ GEMM, repacked Q5K expert slabs (kernels/mmq_gemm_q5k_grouped.cpp
// of the reference; launch grid (ceil(out/64), tile upper bound) x 256).  Token
// tiles are 32 rows of the expert-sorted activations; a host that counted tiles
// with a smaller bn only over-launches.
#include "mmq_gemm.h"

REIN_DEFINE_MMQ_GROUPED(mmq_gemm_q5k_grouped_f32, REIN_Q5_K)
// the library's launch: one tile per workgroup; two slabs run gate and up of an expert FFN at once
REIN_DEFINE_MMQ_GROUPED_ONE(rein_mmq_q5k_grouped_t32, REIN_Q5_K)

// Q5_1 experts: the reference compiles this file a second time with Q5_1_SCALES
// (src/quant/q5_1.rs:58-60, qwen35.rs:3045) and looks up the same symbol in that module.
REIN_DEFINE_MMQ_GROUPED(mmq_gemm_q5_1_grouped_f32, REIN_Q5_1)
REIN_DEFINE_MMQ_GROUPED_ONE(rein_mmq_q5_1_grouped_t32, REIN_Q5_1)
// gate + up + SwiGLU + BlockQ8 of an expert FFN in one launch
REIN_DEFINE_MMQ_GROUPED_SWIGLU(rein_mmq_q5k_grouped_swiglu_q8, REIN_Q5_K)
