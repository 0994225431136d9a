// Small-batch decode matvec, repacked Q4_0 weights: every weight sub-block is
// read once and dotted with all activation rows (kernels/matvec_q4_0_repacked_batched.cpp).
//   _batched_f32    up to 4 rows  (reference launch: grid ceil(out/8) x 256)
//   _batched16_f32  up to 16 rows (reference launch: grid ceil(out/4) x 256)
#include "matvec_repacked.h"

REIN_DEFINE_MATVEC_BATCHED(matvec_q4_0_repacked_batched_f32, REIN_Q4_0, 2, 4)
REIN_DEFINE_MATVEC_BATCHED(matvec_q4_0_repacked_batched16_f32, REIN_Q4_0, 1, 16)
