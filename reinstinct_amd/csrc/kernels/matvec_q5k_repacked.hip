// Decode matvec, repacked Q5K weights: the entry points the reference host
// looks up by name (kernels/matvec_q5k_repacked.cpp:36-105), rebuilt on the shared wave64 body in
// matvec_repacked.h.  Same arguments; correct under the reference launch geometry.
#include "matvec_repacked.h"

REIN_DEFINE_MATVEC(matvec_q5k_repacked_f32, REIN_Q5_K, 2)

// Per-block int32 dots (debug / parity entry point; no counterpart in the reference).
REIN_DEFINE_BLOCK_DOTS(rein_block_dots_q5k, REIN_Q5_K)
// Q5_1 has expert kernels only (as in the reference); its sub-block decode is checked
// through the same per-block dot dump.
REIN_DEFINE_BLOCK_DOTS(rein_block_dots_q5_1, REIN_Q5_1)
