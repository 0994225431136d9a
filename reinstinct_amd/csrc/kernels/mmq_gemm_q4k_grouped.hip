// Grouped-expert MMQ GEMM, repacked Q4K expert slabs (kernels/mmq_gemm_q4k_grouped.cpp
// of the reference; launch grid (ceil(out/64), tile upper bound) x 256).  Token
// tiles are 32 rows of the expert-sorted activations; a host that counted tiles
// with a smaller bn only over-launches.
#include "mmq_gemm.h"

REIN_DEFINE_MMQ_GROUPED(mmq_gemm_q4k_grouped_f32, REIN_Q4_K)
// the library's launch: one tile per workgroup; two slabs run gate and up of an expert FFN at once
REIN_DEFINE_MMQ_GROUPED_ONE(rein_mmq_q4k_grouped_t32, REIN_Q4_K)
// gate + up + SwiGLU + BlockQ8 of an expert FFN in one launch
REIN_DEFINE_MMQ_GROUPED_SWIGLU(rein_mmq_q4k_grouped_swiglu_q8, REIN_Q4_K)
