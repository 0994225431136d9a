// Instantiations of the LDS-staged decode matvec for 2..4 activation rows:
// rein_mvl_<fmt>_r<R>_b<B> (R output rows per wavefront pass, up to B activation rows).
// The host launcher picks R, the workgroup size and the grid from the shape.  No
// counterpart in the reference.
#include "matvec_lds.h"

REIN_DEFINE_MATVEC_LDS(rein_mvl_q4_0_r1_b2, REIN_Q4_0, 1, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4_0_r1_b4, REIN_Q4_0, 1, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4_0_r2_b2, REIN_Q4_0, 2, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4_0_r2_b4, REIN_Q4_0, 2, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4_0_r4_b2, REIN_Q4_0, 4, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4_0_r4_b4, REIN_Q4_0, 4, 4)

REIN_DEFINE_MATVEC_LDS(rein_mvl_q4k_r1_b2, REIN_Q4_K, 1, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4k_r1_b4, REIN_Q4_K, 1, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4k_r2_b2, REIN_Q4_K, 2, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4k_r2_b4, REIN_Q4_K, 2, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4k_r4_b2, REIN_Q4_K, 4, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q4k_r4_b4, REIN_Q4_K, 4, 4)

REIN_DEFINE_MATVEC_LDS(rein_mvl_q5k_r1_b2, REIN_Q5_K, 1, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q5k_r1_b4, REIN_Q5_K, 1, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q5k_r2_b2, REIN_Q5_K, 2, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q5k_r2_b4, REIN_Q5_K, 2, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q5k_r4_b2, REIN_Q5_K, 4, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q5k_r4_b4, REIN_Q5_K, 4, 4)

REIN_DEFINE_MATVEC_LDS(rein_mvl_q6k_r1_b2, REIN_Q6_K, 1, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q6k_r1_b4, REIN_Q6_K, 1, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q6k_r2_b2, REIN_Q6_K, 2, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q6k_r2_b4, REIN_Q6_K, 2, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q6k_r4_b2, REIN_Q6_K, 4, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q6k_r4_b4, REIN_Q6_K, 4, 4)

REIN_DEFINE_MATVEC_LDS(rein_mvl_q8_0_r1_b2, REIN_Q8_0, 1, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q8_0_r1_b4, REIN_Q8_0, 1, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q8_0_r2_b2, REIN_Q8_0, 2, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q8_0_r2_b4, REIN_Q8_0, 2, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q8_0_r4_b2, REIN_Q8_0, 4, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_q8_0_r4_b4, REIN_Q8_0, 4, 4)

REIN_DEFINE_MATVEC_LDS(rein_mvl_iq4xs_r1_b2, REIN_IQ4_XS, 1, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq4xs_r1_b4, REIN_IQ4_XS, 1, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq4xs_r2_b2, REIN_IQ4_XS, 2, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq4xs_r2_b4, REIN_IQ4_XS, 2, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq4xs_r4_b2, REIN_IQ4_XS, 4, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq4xs_r4_b4, REIN_IQ4_XS, 4, 4)

REIN_DEFINE_MATVEC_LDS(rein_mvl_iq3s_r1_b2, REIN_IQ3_S, 1, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq3s_r1_b4, REIN_IQ3_S, 1, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq3s_r2_b2, REIN_IQ3_S, 2, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq3s_r2_b4, REIN_IQ3_S, 2, 4)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq3s_r4_b2, REIN_IQ3_S, 4, 2)
REIN_DEFINE_MATVEC_LDS(rein_mvl_iq3s_r4_b4, REIN_IQ3_S, 4, 4)
