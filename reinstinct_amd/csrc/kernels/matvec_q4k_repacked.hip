// Decode matvec, repacked Q4K weights: the entry points the reference host
// looks up by name (kernels/matvec_q4k_repacked.cpp:132-160), rebuilt on the shared wave64 body in
// matvec_repacked.h.  Same arguments; correct under the reference launch geometry.
#include "matvec_repacked.h"

REIN_DEFINE_MATVEC(matvec_q4k_repacked_f32, REIN_Q4_K, 2)
REIN_DEFINE_MATVEC(matvec_q4k_repacked_r1_f32, REIN_Q4_K, 1)
REIN_DEFINE_MATVEC(matvec_q4k_repacked_r4_f32, REIN_Q4_K, 4)

// Per-block int32 dots (debug / parity entry point; no counterpart in the reference).
REIN_DEFINE_BLOCK_DOTS(rein_block_dots_q4k, REIN_Q4_K)
