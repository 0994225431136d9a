// Prefill MMQ GEMM, repacked Q4_0 weights, on the int8 matrix cores.  Entry
// points the reference host looks up by name (kernels/mmq_gemm_q4_0_repacked.cpp):
//   _f32         wide tile   (reference launch: grid (ceil(out/64), ceil(P/64)) x 256)
//   _narrow_f32  <= 16 rows  (reference launch: grid (ceil(out/16), ceil(P/16)) x 64)
// plus the tuned token-tile variants the C-ABI launcher picks from and the MFMA
// block-dot dump used by the parity tests.
#include "mmq_gemm.h"

REIN_DEFINE_MMQ(mmq_gemm_q4_0_repacked_f32, REIN_Q4_0, 64)
REIN_DEFINE_MMQ(mmq_gemm_q4_0_repacked_narrow_f32, REIN_Q4_0, 32)
REIN_DEFINE_MMQ_PIPE(rein_mmq_q4_0_t32, REIN_Q4_0, 32)
REIN_DEFINE_MMQ_PIPE(rein_mmq_q4_0_t64, REIN_Q4_0, 64)
REIN_DEFINE_MMQ_MIXED(rein_mmq_q4_0_mix, REIN_Q4_0)
REIN_DEFINE_MMQ_SPLIT_TAIL(rein_mmq_q4_0_sk, REIN_Q4_0, 64)
REIN_DEFINE_MMQ_SPLIT_TAIL(rein_mmq_q4_0_sk32, REIN_Q4_0, 32)
REIN_DEFINE_MMQ_DOTS(rein_mmq_dots_q4_0, REIN_Q4_0)
