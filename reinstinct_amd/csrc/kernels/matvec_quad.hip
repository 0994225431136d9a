// Batched decode matvec on v_mfma_i32_4x4x4_16b_i8: rein_mvq_<fmt>_t4 takes up to 4
// activation rows, _t8 up to 8 (two groups of four over the same weight registers).
#include "matvec_quad.h"

REIN_DEFINE_MATVEC_QUAD(rein_mvq_q4_0_t4, REIN_Q4_0, 1)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q4_0_t8, REIN_Q4_0, 2)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q4k_t4, REIN_Q4_K, 1)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q4k_t8, REIN_Q4_K, 2)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q5k_t4, REIN_Q5_K, 1)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q5k_t8, REIN_Q5_K, 2)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q6k_t4, REIN_Q6_K, 1)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q6k_t8, REIN_Q6_K, 2)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q8_0_t4, REIN_Q8_0, 1)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_q8_0_t8, REIN_Q8_0, 2)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_iq4xs_t4, REIN_IQ4_XS, 1)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_iq4xs_t8, REIN_IQ4_XS, 2)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_iq3s_t4, REIN_IQ3_S, 1)
REIN_DEFINE_MATVEC_QUAD(rein_mvq_iq3s_t8, REIN_IQ3_S, 2)

// rein_mvql_<fmt>_t4 / _t8: the same with the activation rows staged in LDS once per workgroup
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q4_0_t4, REIN_Q4_0, 1)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q4_0_t8, REIN_Q4_0, 2)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q4k_t4, REIN_Q4_K, 1)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q4k_t8, REIN_Q4_K, 2)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q5k_t4, REIN_Q5_K, 1)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q5k_t8, REIN_Q5_K, 2)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q6k_t4, REIN_Q6_K, 1)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q6k_t8, REIN_Q6_K, 2)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q8_0_t4, REIN_Q8_0, 1)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_q8_0_t8, REIN_Q8_0, 2)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_iq4xs_t4, REIN_IQ4_XS, 1)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_iq4xs_t8, REIN_IQ4_XS, 2)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_iq3s_t4, REIN_IQ3_S, 1)
REIN_DEFINE_MATVEC_QUAD_LDS(rein_mvql_iq3s_t8, REIN_IQ3_S, 2)
