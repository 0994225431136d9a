// Decode matvec, repacked IQ4XS weights: the entry points the reference host
// looks up by name (kernels/matvec_iq4xs_repacked.cpp:126-154), rebuilt on the shared wave64 body in
// matvec_repacked.h.  Same arguments; correct under the reference launch geometry.
#include "matvec_repacked.h"

REIN_DEFINE_MATVEC(matvec_iq4xs_repacked_f32, REIN_IQ4_XS, 2)
REIN_DEFINE_MATVEC(matvec_iq4xs_repacked_r1_f32, REIN_IQ4_XS, 1)
REIN_DEFINE_MATVEC(matvec_iq4xs_repacked_r4_f32, REIN_IQ4_XS, 4)

// Per-block int32 dots (debug / parity entry point; no counterpart in the reference).
REIN_DEFINE_BLOCK_DOTS(rein_block_dots_iq4xs, REIN_IQ4_XS)

// IQ3_S: the reference compiles this file a second time with the IQ3_S codebook
// (src/quant/iq3_s.rs:164-177, qwen35.rs:2264) and looks up the same symbol in that module;
// one code object cannot hold two symbols of one name, hence the _iq3s_ names.
REIN_DEFINE_MATVEC(matvec_iq3s_repacked_f32, REIN_IQ3_S, 2)
REIN_DEFINE_MATVEC(matvec_iq3s_repacked_r1_f32, REIN_IQ3_S, 1)
REIN_DEFINE_MATVEC(matvec_iq3s_repacked_r4_f32, REIN_IQ3_S, 4)
REIN_DEFINE_BLOCK_DOTS(rein_block_dots_iq3s, REIN_IQ3_S)
