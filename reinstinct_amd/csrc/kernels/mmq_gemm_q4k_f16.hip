// Prefill MMQ GEMM for repacked Q4_K weights on the fp16 matrix instruction with whole
// superblocks accumulated in the matrix unit (mmq_f16.h).  No counterpart file in the reference;
// the product computed is that of kernels/mmq_gemm_q4k_repacked.cpp.
//   rein_mmq16_prep    BlockQ8 rows -> fp16 operand image (once per GEMM)
//   rein_mmq16_q4k     the GEMM, one 256-row x 64-token tile per workgroup
#include "mmq_f16.h"

REIN_DEFINE_MMQ16_PREP(rein_mmq16_prep)
REIN_DEFINE_MMQ16_DENSE(rein_mmq16_q4k)
