// Decode matvec, repacked Q4_0 weights: the entry points the reference host
// looks up by name (kernels/matvec_q4_0_repacked.cpp:121-149), rebuilt on the shared wave64 body in
// matvec_repacked.h.  Same arguments; correct under the reference launch geometry.
#include "matvec_repacked.h"

REIN_DEFINE_MATVEC(matvec_q4_0_repacked_f32, REIN_Q4_0, 2)
REIN_DEFINE_MATVEC(matvec_q4_0_repacked_r1_f32, REIN_Q4_0, 1)
REIN_DEFINE_MATVEC(matvec_q4_0_repacked_r4_f32, REIN_Q4_0, 4)

// Per-block int32 dots (debug / parity entry point; no counterpart in the reference).
REIN_DEFINE_BLOCK_DOTS(rein_block_dots_q4_0, REIN_Q4_0)
