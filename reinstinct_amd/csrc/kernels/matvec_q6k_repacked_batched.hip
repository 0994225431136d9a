// Small-batch decode matvec, repacked Q6K weights: every weight sub-block is
// read once and dotted with all activation rows (kernels/matvec_q6k_repacked_batched.cpp).
//   _batched_f32    up to 4 rows  (reference launch: grid ceil(out/8) x 256)
//   _batched16_f32  up to 16 rows (reference launch: grid ceil(out/4) x 256)
#include "matvec_repacked.h"

REIN_DEFINE_MATVEC_BATCHED(matvec_q6k_repacked_batched_f32, REIN_Q6_K, 2, 4)
REIN_DEFINE_MATVEC_BATCHED(matvec_q6k_repacked_batched16_f32, REIN_Q6_K, 1, 16)
