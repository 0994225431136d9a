// Prefill MMQ GEMM, repacked Q4K weights, on the int8 matrix cores.  Entry
// points the reference host looks up by name (kernels/mmq_gemm_q4k_repacked.cpp):
//   _f32         wide tile   (reference launch: grid (ceil(out/64), ceil(P/64)) x 256)
//   _narrow_f32  <= 16 rows  (reference launch: grid (ceil(out/16), ceil(P/16)) x 64)
// plus the tuned token-tile variants the C-ABI launcher picks from and the MFMA
// block-dot dump used by the parity tests.
#include "mmq_gemm.h"

REIN_DEFINE_MMQ(mmq_gemm_q4k_repacked_f32, REIN_Q4_K, 64)
REIN_DEFINE_MMQ(mmq_gemm_q4k_repacked_narrow_f32, REIN_Q4_K, 32)
REIN_DEFINE_MMQ_PIPE(rein_mmq_q4k_t32, REIN_Q4_K, 32)
REIN_DEFINE_MMQ_PIPE(rein_mmq_q4k_t64, REIN_Q4_K, 64)
REIN_DEFINE_MMQ_MIXED(rein_mmq_q4k_mix, REIN_Q4_K)
REIN_DEFINE_MMQ_SPLIT_TAIL(rein_mmq_q4k_sk, REIN_Q4_K, 64)
REIN_DEFINE_MMQ_SPLIT_TAIL(rein_mmq_q4k_sk32, REIN_Q4_K, 32)
// adds the partial tiles of a split-tail launch (any format): second launch behind rein_mmq_<fmt>_sk
REIN_DEFINE_MMQ_TAIL_SUM(rein_mmq_tail_sum_t64, 2)
REIN_DEFINE_MMQ_TAIL_SUM(rein_mmq_tail_sum_t32, 1)
REIN_DEFINE_MMQ_DOTS(rein_mmq_dots_q4k, REIN_Q4_K)
