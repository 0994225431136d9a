// Prefill MMQ GEMM, repacked IQ4XS weights, on the int8 matrix cores.  Entry
// points the reference host looks up by name (kernels/mmq_gemm_iq4xs_repacked.cpp):
//   _f32         wide tile   (reference launch: grid (ceil(out/64), ceil(P/64)) x 256)
//   _narrow_f32  <= 16 rows  (reference launch: grid (ceil(out/16), ceil(P/16)) x 64)
// plus the tuned token-tile variants the C-ABI launcher picks from and the MFMA
// block-dot dump used by the parity tests.
#include "mmq_gemm.h"

REIN_DEFINE_MMQ(mmq_gemm_iq4xs_repacked_f32, REIN_IQ4_XS, 64)
REIN_DEFINE_MMQ(mmq_gemm_iq4xs_repacked_narrow_f32, REIN_IQ4_XS, 32)
REIN_DEFINE_MMQ_PIPE(rein_mmq_iq4xs_t32, REIN_IQ4_XS, 32)
REIN_DEFINE_MMQ_PIPE(rein_mmq_iq4xs_t64, REIN_IQ4_XS, 64)
REIN_DEFINE_MMQ_MIXED(rein_mmq_iq4xs_mix, REIN_IQ4_XS)
REIN_DEFINE_MMQ_SPLIT_TAIL(rein_mmq_iq4xs_sk, REIN_IQ4_XS, 64)
REIN_DEFINE_MMQ_SPLIT_TAIL(rein_mmq_iq4xs_sk32, REIN_IQ4_XS, 32)
REIN_DEFINE_MMQ_DOTS(rein_mmq_dots_iq4xs, REIN_IQ4_XS)

// the same kernels with the IQ3_S codebook (src/runtime/prefill.rs:528-529)
REIN_DEFINE_MMQ(mmq_gemm_iq3s_repacked_f32, REIN_IQ3_S, 64)
REIN_DEFINE_MMQ(mmq_gemm_iq3s_repacked_narrow_f32, REIN_IQ3_S, 32)
REIN_DEFINE_MMQ_PIPE(rein_mmq_iq3s_t32, REIN_IQ3_S, 32)
REIN_DEFINE_MMQ_PIPE(rein_mmq_iq3s_t64, REIN_IQ3_S, 64)
REIN_DEFINE_MMQ_MIXED(rein_mmq_iq3s_mix, REIN_IQ3_S)
REIN_DEFINE_MMQ_SPLIT_TAIL(rein_mmq_iq3s_sk, REIN_IQ3_S, 64)
REIN_DEFINE_MMQ_SPLIT_TAIL(rein_mmq_iq3s_sk32, REIN_IQ3_S, 32)
REIN_DEFINE_MMQ_DOTS(rein_mmq_dots_iq3s, REIN_IQ3_S)
