// Prefill MMQ GEMM for repacked Q4_K weights on the block-scaled fp6 matrix instruction
// (mmq_fp6.h): the library's tuned launch for more than 16 activation rows when the caller
// provides a workspace.  No counterpart file in the reference; the product computed is that
// of kernels/mmq_gemm_q4k_repacked.cpp.
//   rein_mmq6_prep       BlockQ8 rows -> operand image (once per GEMM)
//   rein_mmq6_q4k_mix    the GEMM, token groups of 4 / 2 / 1 tiles in one launch
//   rein_mmq6_q4k_sk     the GEMM as a split-tail launch: one workgroup per resident slot, whole tiles in
//                        rounds, the tiles left over split along the contraction into partial tiles
//   rein_mmq6_tail_sum   adds the partial tiles of the tail in range order (second launch)
//   rein_mmq6_q4k_dots   the raw block dots out of the fp6 instruction (parity tests)
#include "mmq_fp6.h"

REIN_DEFINE_MMQ6_PREP(rein_mmq6_prep)
REIN_DEFINE_MMQ6_MIXED(rein_mmq6_q4k_mix)
REIN_DEFINE_MMQ6_SPLIT_TAIL(rein_mmq6_q4k_sk)
REIN_DEFINE_MMQ6_TAIL_SUM(rein_mmq6_tail_sum)
REIN_DEFINE_MMQ6_DOTS(rein_mmq6_q4k_dots)
