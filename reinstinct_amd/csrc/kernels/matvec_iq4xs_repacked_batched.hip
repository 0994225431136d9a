// Small-batch decode matvec, repacked IQ4XS weights: every weight sub-block is
// read once and dotted with all activation rows (kernels/matvec_iq4xs_repacked_batched.cpp).
//   _batched_f32    up to 4 rows  (reference launch: grid ceil(out/8) x 256)
//   _batched16_f32  up to 16 rows (reference launch: grid ceil(out/4) x 256)
#include "matvec_repacked.h"

REIN_DEFINE_MATVEC_BATCHED(matvec_iq4xs_repacked_batched_f32, REIN_IQ4_XS, 2, 4)
REIN_DEFINE_MATVEC_BATCHED(matvec_iq4xs_repacked_batched16_f32, REIN_IQ4_XS, 1, 16)

// the same kernels with the IQ3_S codebook (src/runtime/prefill.rs:473-474)
REIN_DEFINE_MATVEC_BATCHED(matvec_iq3s_repacked_batched_f32, REIN_IQ3_S, 2, 4)
REIN_DEFINE_MATVEC_BATCHED(matvec_iq3s_repacked_batched16_f32, REIN_IQ3_S, 1, 16)
