// Skinny MMQ instantiations: rein_mmqs_<fmt>_v<NV> -- up to 2*NV activation rows per
// workgroup; the number of wavefronts that split the contraction is the launch's
// block size / 64 (1..8); last argument: wavefronts per SIMD the kernel is built for.
#include "mmq_skinny.h"

REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q4_0_v4, REIN_Q4_0, 4, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q4_0_v8, REIN_Q4_0, 8, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q4k_v4, REIN_Q4_K, 4, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q4k_v8, REIN_Q4_K, 8, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q5k_v4, REIN_Q5_K, 4, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q5k_v8, REIN_Q5_K, 8, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q6k_v4, REIN_Q6_K, 4, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q6k_v8, REIN_Q6_K, 8, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q8_0_v4, REIN_Q8_0, 4, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q8_0_v8, REIN_Q8_0, 8, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_iq4xs_v4, REIN_IQ4_XS, 4, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_iq4xs_v8, REIN_IQ4_XS, 8, 2)
// two and four activation rows: fewer accumulator registers are converted and scaled per sub-block
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q4_0_v1, REIN_Q4_0, 1, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q4_0_v2, REIN_Q4_0, 2, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q4k_v1, REIN_Q4_K, 1, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q4k_v2, REIN_Q4_K, 2, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q5k_v1, REIN_Q5_K, 1, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q5k_v2, REIN_Q5_K, 2, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q6k_v1, REIN_Q6_K, 1, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q6k_v2, REIN_Q6_K, 2, 2)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q8_0_v1, REIN_Q8_0, 1, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_q8_0_v2, REIN_Q8_0, 2, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_iq4xs_v1, REIN_IQ4_XS, 1, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_iq4xs_v2, REIN_IQ4_XS, 2, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_iq3s_v1, REIN_IQ3_S, 1, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_iq3s_v2, REIN_IQ3_S, 2, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_iq3s_v4, REIN_IQ3_S, 4, 3)
REIN_DEFINE_MMQ_SKINNY(rein_mmqs_iq3s_v8, REIN_IQ3_S, 8, 2)
