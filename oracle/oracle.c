/*
 * CPU oracle — TEST INFRASTRUCTURE ONLY (see oracle.h for what pins each
 * function).  Plain C, built with -O2 -ffp-contract=off and no fast-math so
 * every fp32 operation below is a single IEEE operation in source order.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ half */

/* src/quant/half.rs:9-40 */
float orc_f16_to_f32(uint16_t bits)
{
    uint32_t sign = (uint32_t)(bits & 0x8000u) << 16;
    uint32_t ex   = (bits >> 10) & 0x1Fu;
    uint32_t man  = bits & 0x03FFu;
    uint32_t u;
    if (ex == 0) {
        if (man == 0) {
            u = sign;
        } else {
            /* subnormal half: normalise, unbiased exponent -14 minus the shifts */
            int shifts = 0;
            while ((man & 0x0400u) == 0) { man <<= 1; shifts++; }
            man &= 0x03FFu;
            u = sign | ((uint32_t)(127 - 14 - shifts) << 23) | (man << 13);
        }
    } else if (ex == 0x1F) {
        u = sign | 0x7F800000u | (man << 13);
    } else {
        u = sign | ((ex + (127 - 15)) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* src/quant/half.rs:51-84 — RNE for normal results; the subnormal-result
 * branch truncates (half.rs:69-73), restated as such. */
uint16_t orc_f32_to_f16(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, 4);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    int      ex   = (int)((bits >> 23) & 0xFFu);
    uint32_t man  = bits & 0x007FFFFFu;

    if (ex == 0xFF) return (uint16_t)(sign | 0x7C00u | (man ? 0x0200u : 0u));
    int unbiased = ex - 127;
    if (unbiased >= 16) return (uint16_t)(sign | 0x7C00u);
    if (unbiased < -24) return sign;
    if (unbiased < -14) {
        uint32_t m = (man | 0x00800000u) >> (unsigned)((-14 - unbiased) + 13);
        return (uint16_t)(sign | (uint16_t)m);
    }
    uint16_t out = (uint16_t)(sign | (uint16_t)((unbiased + 15) << 10) | (uint16_t)(man >> 13));
    uint32_t round_bit = (man >> 12) & 1u;
    uint32_t sticky    = man & 0x0FFFu;
    if (round_bit && (sticky || (out & 1u))) out = (uint16_t)(out + 1u);
    return out;
}

static inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline void     wr16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); }
static inline uint32_t rd32(const uint8_t *p)
{
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* ------------------------------------------------------- format constants */

/* src/quant/iq4_xs.rs:28-31 */
static const int8_t KVALUES_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10,
                                         1,    13,   25,  38,  53,  69,  89,  113};

/* The IQ3_S grid (IQ3S_GRID of src/quant/iq3_s.rs:41-107, ggml's iq3s_grid): 512 groups
 * of four magnitudes.  Every magnitude is odd, 2*l + 1 with l in 0..7, so a group is four
 * octal digits; they are written here weight 0 first. */
static const char IQ3S_GRID_OCTAL[2048 + 1] =
    "000010002000500070000100110021004100610002001200520033000400240054007400150035000600260017004700"
    "770000101010201040100110111051100210321072101310531044101610561027100020102050207020012031206120"
    "122052200320432024205420742015203520072037203030113051300230223013303330633044300530253076301730"
    "573000403140714012404240234004403440154007402050405002502250625033501450545074506650375060601160"
    "316013602560176000702070407002702270627033700570457000011001200140010101110131015101710102012201"
    "130143016301450165011601270100111011301160110111411112110311331114110511251107116711002121215121"
    "712102214221232104213421552106212721103140317031013131311231723103314331143126310731304150412141"
    "414113413341244164410541454110510151315112510351235115510261426172614461646110713071017121711271"
    "537114712671077100021002300250027002010221024102610212023202720203022302140234025402050225027602"
    "070237025702001220120112311271122212521213124312241215121022402270221222322203227322142235227522"
    "172247220032203250321132223242321332333224320532663210427042024232422342534214422742574240521152"
    "225273520452355207520062206270621262556216625072117262720372347205722003110331035103710322031303"
    "330353032403440374031503360317031013301350134113121332130413061327136713002321230223232343230523"
    "103301334133123332337233033314333433743355333733304311436143224313432543064346431053015321535253"
    "235344536553375361631463107330730273227353730004400421040204420472042304140405040704201470141114"
    "311422140314531434141514551410243024012451241224332404247524262407244034113431340234223413345334"
    "004420444244734404441744505470541254265431644364066401745174037434741574200501054105220504054405"
    "740525056605470510153015501521151215231527150025112532250325632535252035703501357235443515355635"
    "373510454045024523456445215562551555355524652075407522751106310651061306330606060016021672164616"
    "212643262426552626260726003641361236043652463446264600563056435606565066046611763176000740077007"
    "020722076307040745072607201711174217341754171027402701276127122703271527203723375337353710475047"
    "31470247054722572457206713670077";

/* magnitude of weight j (0..3) of grid entry idx (0..511) */
static inline int iq3s_grid_mag(int idx, int j) { return 2 * (IQ3S_GRID_OCTAL[4 * idx + j] - '0') + 1; }

uint32_t orc_iq3s_grid_entry(int idx)
{
    uint32_t v = 0;
    for (int j = 0; j < 4; j++) v |= (uint32_t)iq3s_grid_mag(idx, j) << (8 * j);
    return v;
}

int orc_block_size(int fmt)
{
    switch (fmt) {
    case ORC_Q4_0: case ORC_Q8_0: case ORC_Q5_1: return 32;       /* q4_0.rs:22, q8_0.rs:8, q5_1.rs:25 */
    case ORC_IQ3_S:                                               /* iq3_s.rs:24 */
    case ORC_Q4_K: case ORC_Q5_K: case ORC_Q6_K: case ORC_IQ4_XS: return 256;
    default: return 0;
    }
}

int orc_bytes_per_block(int fmt)
{
    switch (fmt) {
    case ORC_Q4_0:   return 18;    /* q4_0.rs:23  */
    case ORC_Q8_0:   return 34;    /* q8_0.rs:9   */
    case ORC_Q4_K:   return 144;   /* q4_k.rs:18  */
    case ORC_Q5_K:   return 176;   /* q5_k.rs:22  */
    case ORC_Q6_K:   return 210;   /* q6_k.rs:19  */
    case ORC_IQ4_XS: return 136;   /* iq4_xs.rs:24 */
    case ORC_Q5_1:   return 24;    /* q5_1.rs:26  */
    case ORC_IQ3_S:  return 110;   /* iq3_s.rs:25 */
    default: return 0;
    }
}

/* src/quant/q4_k.rs:40-48 */
void orc_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m)
{
    if (j < 4) {
        *sc = q[j] & 63;
        *m  = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m  = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* IQ4_XS 6-bit sub-scale (iq4_xs.rs:55-57, 121-123) */
static inline int iq4xs_ls(const uint8_t *blk, int ib)
{
    uint16_t scales_h = rd16(blk + 2);
    const uint8_t *scales_l = blk + 4;
    int lo = (scales_l[ib / 2] >> (4 * (ib & 1))) & 0x0F;
    int hi = (scales_h >> (2 * ib)) & 3;
    return lo | (hi << 4);
}

/* ---------------------------------------------------------------- dequant */

/* src/quant/q4_k.rs:50-84 */
static void dequant_q4_k(const uint8_t *b, float *y)
{
    float d = orc_f16_to_f32(rd16(b)), dmin = orc_f16_to_f32(rd16(b + 2));
    const uint8_t *scales = b + 4, *qs = b + 16;
    for (int chunk = 0; chunk < 4; chunk++) {
        uint8_t sa, ma, sb, mb;
        orc_get_scale_min_k4(2 * chunk, scales, &sa, &ma);
        orc_get_scale_min_k4(2 * chunk + 1, scales, &sb, &mb);
        float d1 = d * (float)sa, m1 = dmin * (float)ma;
        float d2 = d * (float)sb, m2 = dmin * (float)mb;
        for (int l = 0; l < 32; l++) {
            uint8_t q = qs[chunk * 32 + l];
            y[chunk * 64 + l]      = d1 * (float)(q & 0x0F) - m1;
            y[chunk * 64 + l + 32] = d2 * (float)(q >> 4) - m2;
        }
    }
}

/* src/quant/q5_k.rs:47-86 */
static void dequant_q5_k(const uint8_t *b, float *y)
{
    float d = orc_f16_to_f32(rd16(b)), dmin = orc_f16_to_f32(rd16(b + 2));
    const uint8_t *scales = b + 4, *qh = b + 16, *qs = b + 48;
    uint8_t u1 = 1, u2 = 2;
    for (int chunk = 0; chunk < 4; chunk++) {
        uint8_t sa, ma, sb, mb;
        orc_get_scale_min_k4(2 * chunk, scales, &sa, &ma);
        orc_get_scale_min_k4(2 * chunk + 1, scales, &sb, &mb);
        float d1 = d * (float)sa, m1 = dmin * (float)ma;
        float d2 = d * (float)sb, m2 = dmin * (float)mb;
        for (int l = 0; l < 32; l++) {
            uint8_t q = qs[chunk * 32 + l];
            int qlo = (q & 0x0F) + ((qh[l] & u1) ? 16 : 0);
            int qhi = (q >> 4) + ((qh[l] & u2) ? 16 : 0);
            y[chunk * 64 + l]      = d1 * (float)qlo - m1;
            y[chunk * 64 + l + 32] = d2 * (float)qhi - m2;
        }
        u1 = (uint8_t)(u1 << 2);
        u2 = (uint8_t)(u2 << 2);
    }
}

/* src/quant/q6_k.rs:31-69 — note the product order d * scale * q */
static void dequant_q6_k(const uint8_t *b, float *y)
{
    const uint8_t *ql = b, *qh = b + 128;
    const int8_t  *sc = (const int8_t *)(b + 192);
    float d = orc_f16_to_f32(rd16(b + 208));
    for (int chunk = 0; chunk < 2; chunk++) {
        const uint8_t *l4 = ql + chunk * 64, *h2 = qh + chunk * 32;
        const int8_t  *s  = sc + chunk * 8;
        float *o = y + chunk * 128;
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            uint8_t h = h2[l];
            int q1 = (int)((l4[l] & 0x0F) | (((h >> 0) & 3) << 4)) - 32;
            int q2 = (int)((l4[l + 32] & 0x0F) | (((h >> 2) & 3) << 4)) - 32;
            int q3 = (int)((l4[l] >> 4) | (((h >> 4) & 3) << 4)) - 32;
            int q4 = (int)((l4[l + 32] >> 4) | (((h >> 6) & 3) << 4)) - 32;
            o[l]      = d * (float)s[is] * (float)q1;
            o[l + 32] = d * (float)s[is + 2] * (float)q2;
            o[l + 64] = d * (float)s[is + 4] * (float)q3;
            o[l + 96] = d * (float)s[is + 6] * (float)q4;
        }
    }
}

/* src/quant/q8_0.rs:24-38 */
static void dequant_q8_0(const uint8_t *b, float *y)
{
    float d = orc_f16_to_f32(rd16(b));
    const int8_t *qs = (const int8_t *)(b + 2);
    for (int i = 0; i < 32; i++) y[i] = d * (float)qs[i];
}

/* src/quant/q4_0.rs:36-53 */
static void dequant_q4_0(const uint8_t *b, float *y)
{
    float d = orc_f16_to_f32(rd16(b));
    for (int k = 0; k < 16; k++) {
        int lo = (int)(b[2 + k] & 0x0F) - 8, hi = (int)(b[2 + k] >> 4) - 8;
        y[k]      = d * (float)lo;
        y[k + 16] = d * (float)hi;
    }
}

/* src/quant/iq4_xs.rs:44-71 */
static void dequant_iq4_xs(const uint8_t *b, float *y)
{
    float d = orc_f16_to_f32(rd16(b));
    const uint8_t *qs = b + 8;
    for (int ib = 0; ib < 8; ib++) {
        float dl = d * (float)(iq4xs_ls(b, ib) - 32);
        for (int l = 0; l < 16; l++) {
            uint8_t q = qs[ib * 16 + l];
            y[ib * 32 + l]      = dl * (float)KVALUES_IQ4NL[q & 0x0F];
            y[ib * 32 + l + 16] = dl * (float)KVALUES_IQ4NL[q >> 4];
        }
    }
}

/* src/quant/q5_1.rs:38-56: w = d*q5 + m, the 5th bit of weight i is bit i of qh */
static void dequant_q5_1(const uint8_t *b, float *y)
{
    float d = orc_f16_to_f32(rd16(b)), m = orc_f16_to_f32(rd16(b + 2));
    uint32_t qh = rd32(b + 4);
    const uint8_t *qs = b + 8;
    for (int k = 0; k < 16; k++) {
        int lo = (qs[k] & 0x0F) | (int)(((qh >> k) & 1u) << 4);
        int hi = (qs[k] >> 4) | (int)(((qh >> (k + 16)) & 1u) << 4);
        y[k] = d * (float)lo + m;
        y[k + 16] = d * (float)hi + m;
    }
}

/* The eight sub-blocks of an IQ3_S block as (db, 32 signed odd values), src/quant/iq3_s.rs:
 * 113-147: sub-block s reads 8 index bytes qs[8s..], one qh byte (bit i = 9th bit of index
 * i), 4 sign bytes (bit j of byte l flips weight 8l + j) and the nibble s of scales;
 * db = d * (1 + 2*nibble). */
static void iq3s_sub_block(const uint8_t *b, int s, float *db, int vals[32])
{
    const uint8_t *qs = b + 2 + 8 * s, *signs = b + 2 + 64 + 8 + 4 * s;
    int qh = b[2 + 64 + s];
    int sc = (b[2 + 64 + 8 + 32 + s / 2] >> (4 * (s & 1))) & 0x0F;
    *db = orc_f16_to_f32(rd16(b)) * (1.0f + 2.0f * (float)sc);
    for (int i = 0; i < 8; i++) {                /* index i covers weights 4i .. 4i+3 */
        int idx = qs[i] | (((qh >> i) & 1) << 8);
        for (int j = 0; j < 4; j++) {
            int w = 4 * i + j;
            int mag = iq3s_grid_mag(idx, j);
            vals[w] = (signs[w >> 3] >> (w & 7)) & 1 ? -mag : mag;
        }
    }
}

static void dequant_iq3_s(const uint8_t *b, float *y)
{
    for (int s = 0; s < 8; s++) {
        float db;
        int v[32];
        iq3s_sub_block(b, s, &db, v);
        for (int i = 0; i < 32; i++) y[32 * s + i] = db * (float)v[i];
    }
}

int orc_dequantize_to_f32(int fmt, const uint8_t *bytes, float *out, size_t n)
{
    int bs = orc_block_size(fmt), bb = orc_bytes_per_block(fmt);
    if (!bs || n % (size_t)bs) return -1;
    size_t nb = n / (size_t)bs;
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *b = bytes + i * (size_t)bb;
        float *y = out + i * (size_t)bs;
        switch (fmt) {
        case ORC_Q4_K:   dequant_q4_k(b, y); break;
        case ORC_Q5_K:   dequant_q5_k(b, y); break;
        case ORC_Q6_K:   dequant_q6_k(b, y); break;
        case ORC_Q8_0:   dequant_q8_0(b, y); break;
        case ORC_Q4_0:   dequant_q4_0(b, y); break;
        case ORC_IQ4_XS: dequant_iq4_xs(b, y); break;
        case ORC_Q5_1:   dequant_q5_1(b, y); break;
        case ORC_IQ3_S:  dequant_iq3_s(b, y); break;
        }
    }
    return 0;
}

/* ----------------------------------------------------------------- repack */

/* src/quant/q4_k.rs:92-95 (same rule in q8_0.rs:68-71, q4_0.rs:60-63, iq4_xs.rs:79-82) */
size_t orc_repacked_n_sub_padded(size_t in_dim)
{
    size_t n = in_dim / 32;
    return (n != 0 && (n & (n - 1)) == 0) ? n + 1 : n;
}

/* bytes per sub-block in the per-sub-block planes, bytes per superblock in the
 * per-superblock plane (0 = no such plane) */
static void plane_bytes(int fmt, size_t *per_sub, size_t *per_super)
{
    switch (fmt) {
    case ORC_Q4_K:   *per_sub = 16 + 2;     *per_super = 4; break;  /* q4_k.rs:98-102  */
    case ORC_Q5_K:   *per_sub = 16 + 4 + 2; *per_super = 4; break;  /* q5_k.rs:100-104 */
    case ORC_Q6_K:   *per_sub = 16 + 8 + 2; *per_super = 2; break;  /* q6_k.rs:89-93   */
    case ORC_Q8_0:   *per_sub = 32 + 2;     *per_super = 0; break;  /* q8_0.rs:74-77   */
    case ORC_Q4_0:   *per_sub = 16 + 2;     *per_super = 0; break;  /* q4_0.rs:66-69   */
    case ORC_IQ4_XS: *per_sub = 16 + 2;     *per_super = 0; break;  /* iq4_xs.rs:85-88 */
    case ORC_IQ3_S:  *per_sub = 16 + 2;     *per_super = 0; break;  /* iq3_s.rs:178-184 */
    case ORC_Q5_1:   *per_sub = 16 + 4 + 4; *per_super = 0; break;  /* q5_1.rs:76-81   */
    default:         *per_sub = 0;          *per_super = 0; break;
    }
}

size_t orc_repacked_len(int fmt, size_t in_dim, size_t out_dim)
{
    size_t ps, pp;
    plane_bytes(fmt, &ps, &pp);
    if (!ps) return 0;
    return out_dim * orc_repacked_n_sub_padded(in_dim) * ps + out_dim * (in_dim / 256) * pp;
}

/* nibble byte 4j+b = w[4j+b] | w[16+4j+b] << 4   (q4_k.rs:158-165) */
static void pack_nibbles(const uint8_t w[32], uint8_t *dst)
{
    for (int j = 0; j < 4; j++)
        for (int b = 0; b < 4; b++)
            dst[4 * j + b] = (uint8_t)(w[4 * j + b] | (w[16 + 4 * j + b] << 4));
}

/* src/quant/q4_k.rs:126-176 */
static void repack_q4_k(const uint8_t *bytes, size_t in_dim, size_t out_dim, uint8_t *out)
{
    size_t nb = in_dim / 256, nsp = orc_repacked_n_sub_padded(in_dim);
    size_t nib_len = out_dim * nsp * 16, sm_len = out_dim * nsp * 2;
    for (size_t row = 0; row < out_dim; row++)
        for (size_t blk = 0; blk < nb; blk++) {
            const uint8_t *b = bytes + (row * nb + blk) * 144;
            uint8_t *dd = out + nib_len + sm_len + (row * nb + blk) * 4;
            memcpy(dd, b, 4); /* d, dmin raw fp16 */
            for (int s = 0; s < 8; s++) {
                size_t gsb = blk * 8 + (size_t)s;
                const uint8_t *qs = b + 16 + (s >> 1) * 32;
                uint8_t w[32];
                for (int k = 0; k < 32; k++) w[k] = (s & 1) ? (uint8_t)(qs[k] >> 4) : (uint8_t)(qs[k] & 0x0F);
                pack_nibbles(w, out + (row * nsp + gsb) * 16);
                uint8_t sc, m;
                orc_get_scale_min_k4(s, b + 4, &sc, &m);
                out[nib_len + (row * nsp + gsb) * 2]     = sc;
                out[nib_len + (row * nsp + gsb) * 2 + 1] = m;
            }
        }
}

/* src/quant/q5_k.rs:97-151 */
static void repack_q5_k(const uint8_t *bytes, size_t in_dim, size_t out_dim, uint8_t *out)
{
    size_t nb = in_dim / 256, nsp = orc_repacked_n_sub_padded(in_dim);
    size_t nib_len = out_dim * nsp * 16, qh_len = out_dim * nsp * 4, sm_len = out_dim * nsp * 2;
    for (size_t row = 0; row < out_dim; row++)
        for (size_t blk = 0; blk < nb; blk++) {
            const uint8_t *b = bytes + (row * nb + blk) * 176;
            const uint8_t *qhs = b + 16;
            memcpy(out + nib_len + qh_len + sm_len + (row * nb + blk) * 4, b, 4);
            for (int s = 0; s < 8; s++) {
                size_t gsb = blk * 8 + (size_t)s;
                const uint8_t *qs = b + 48 + (s >> 1) * 32;
                uint8_t w[32], hb[32];
                for (int l = 0; l < 32; l++) {
                    w[l]  = (s & 1) ? (uint8_t)(qs[l] >> 4) : (uint8_t)(qs[l] & 0x0F);
                    hb[l] = (uint8_t)((qhs[l] >> s) & 1);
                }
                pack_nibbles(w, out + (row * nsp + gsb) * 16);
                uint32_t packed = 0;
                for (int j = 0; j < 4; j++)
                    for (int bb = 0; bb < 4; bb++) {
                        packed |= (uint32_t)hb[4 * j + bb] << (4 * (2 * j) + bb);
                        packed |= (uint32_t)hb[16 + 4 * j + bb] << (4 * (2 * j + 1) + bb);
                    }
                uint8_t *q = out + nib_len + (row * nsp + gsb) * 4;
                q[0] = (uint8_t)packed; q[1] = (uint8_t)(packed >> 8);
                q[2] = (uint8_t)(packed >> 16); q[3] = (uint8_t)(packed >> 24);
                uint8_t sc, m;
                orc_get_scale_min_k4(s, b + 4, &sc, &m);
                out[nib_len + qh_len + (row * nsp + gsb) * 2]     = sc;
                out[nib_len + qh_len + (row * nsp + gsb) * 2 + 1] = m;
            }
        }
}

/* src/quant/q6_k.rs:86-148 */
static void repack_q6_k(const uint8_t *bytes, size_t in_dim, size_t out_dim, uint8_t *out)
{
    size_t nb = in_dim / 256, nsp = orc_repacked_n_sub_padded(in_dim);
    size_t nib_len = out_dim * nsp * 16, h2_len = out_dim * nsp * 8, sm_len = out_dim * nsp * 2;
    for (size_t row = 0; row < out_dim; row++)
        for (size_t blk = 0; blk < nb; blk++) {
            const uint8_t *b = bytes + (row * nb + blk) * 210;
            const uint8_t *ql = b, *qh = b + 128, *scales = b + 192;
            memcpy(out + nib_len + h2_len + sm_len + (row * nb + blk) * 2, b + 208, 2);
            for (int s = 0; s < 8; s++) {
                size_t gsb = blk * 8 + (size_t)s;
                int chunk = s / 4, quad = s % 4;
                uint8_t lo[32], hi[32];
                for (int l = 0; l < 32; l++) {
                    uint8_t h = qh[chunk * 32 + l];
                    uint8_t a = ql[chunk * 64 + l], c = ql[chunk * 64 + l + 32];
                    switch (quad) {
                    case 0:  lo[l] = a & 0x0F; hi[l] = h & 3; break;
                    case 1:  lo[l] = c & 0x0F; hi[l] = (h >> 2) & 3; break;
                    case 2:  lo[l] = a >> 4;   hi[l] = (h >> 4) & 3; break;
                    default: lo[l] = c >> 4;   hi[l] = (h >> 6) & 3; break;
                    }
                }
                pack_nibbles(lo, out + (row * nsp + gsb) * 16);
                uint8_t h2p[8] = {0};
                for (int j = 0; j < 4; j++)
                    for (int bb = 0; bb < 4; bb++) {
                        h2p[2 * j]     |= (uint8_t)(hi[4 * j + bb] << (2 * bb));
                        h2p[2 * j + 1] |= (uint8_t)(hi[16 + 4 * j + bb] << (2 * bb));
                    }
                memcpy(out + nib_len + (row * nsp + gsb) * 8, h2p, 8);
                out[nib_len + h2_len + (row * nsp + gsb) * 2]     = scales[chunk * 8 + quad * 2];
                out[nib_len + h2_len + (row * nsp + gsb) * 2 + 1] = scales[chunk * 8 + quad * 2 + 1];
            }
        }
}

/* src/quant/q8_0.rs:93-119 */
static void repack_q8_0(const uint8_t *bytes, size_t in_dim, size_t out_dim, uint8_t *out)
{
    size_t nb = in_dim / 32, nsp = orc_repacked_n_sub_padded(in_dim);
    size_t half_len = out_dim * nsp * 16;
    for (size_t row = 0; row < out_dim; row++)
        for (size_t blk = 0; blk < nb; blk++) {
            const uint8_t *src = bytes + (row * nb + blk) * 34;
            size_t i = row * nsp + blk;
            memcpy(out + i * 16, src + 2, 16);
            memcpy(out + half_len + i * 16, src + 18, 16);
            memcpy(out + 2 * half_len + i * 2, src, 2);
        }
}

/* src/quant/q4_0.rs:86-104 */
static void repack_q4_0(const uint8_t *bytes, size_t in_dim, size_t out_dim, uint8_t *out)
{
    size_t nb = in_dim / 32, nsp = orc_repacked_n_sub_padded(in_dim);
    size_t nib_len = out_dim * nsp * 16;
    for (size_t row = 0; row < out_dim; row++)
        for (size_t blk = 0; blk < nb; blk++) {
            const uint8_t *src = bytes + (row * nb + blk) * 18;
            memcpy(out + nib_len + (row * nsp + blk) * 2, src, 2);
            memcpy(out + (row * nsp + blk) * 16, src + 2, 16);
        }
}

/* src/quant/iq4_xs.rs:106-136 */
static void repack_iq4_xs(const uint8_t *bytes, size_t in_dim, size_t out_dim, uint8_t *out)
{
    size_t nb = in_dim / 256, nsp = orc_repacked_n_sub_padded(in_dim);
    size_t nib_len = out_dim * nsp * 16;
    for (size_t row = 0; row < out_dim; row++)
        for (size_t blk = 0; blk < nb; blk++) {
            const uint8_t *b = bytes + (row * nb + blk) * 136;
            float d = orc_f16_to_f32(rd16(b));
            for (int ib = 0; ib < 8; ib++) {
                size_t sb = blk * 8 + (size_t)ib;
                float dl = d * (float)(iq4xs_ls(b, ib) - 32);
                memcpy(out + (row * nsp + sb) * 16, b + 8 + ib * 16, 16);
                wr16(out + nib_len + (row * nsp + sb) * 2, orc_f32_to_f16(dl));
            }
        }
}

/* src/quant/q5_1.rs:61-104: nibbles verbatim; qh re-ordered so that bit 8j+b is the 5th
 * bit of weight 4j+b and bit 8j+4+b that of weight 16+4j+b; raw fp16 d | m << 16 */
static void repack_q5_1(const uint8_t *bytes, size_t in_dim, size_t out_dim, uint8_t *out)
{
    size_t n_sub = in_dim / 32, nsp = orc_repacked_n_sub_padded(in_dim);
    size_t nib_len = out_dim * nsp * 16, qh_len = out_dim * nsp * 4;
    for (size_t row = 0; row < out_dim; row++)
        for (size_t sb = 0; sb < n_sub; sb++) {
            const uint8_t *b = bytes + (row * n_sub + sb) * 24;
            size_t i = row * nsp + sb;
            memcpy(out + i * 16, b + 8, 16);
            uint32_t qh = rd32(b + 4), packed = 0;
            for (int w = 0; w < 32; w++) {
                int j = (w & 15) >> 2, bb = w & 3, upper = w >> 4;
                packed |= ((qh >> w) & 1u) << (8 * j + 4 * upper + bb);
            }
            uint8_t *q = out + nib_len + i * 4;
            q[0] = (uint8_t)packed; q[1] = (uint8_t)(packed >> 8); q[2] = (uint8_t)(packed >> 16); q[3] = (uint8_t)(packed >> 24);
            memcpy(out + nib_len + qh_len + i * 4, b, 4);
        }
}

/* src/quant/iq3_s.rs:186-207: nibble (v + 15) / 2 of weight k low / k+16 high, fp16(db) */
static void repack_iq3_s(const uint8_t *bytes, size_t in_dim, size_t out_dim, uint8_t *out)
{
    size_t nb = in_dim / 256, nsp = orc_repacked_n_sub_padded(in_dim);
    size_t nib_len = out_dim * nsp * 16;
    for (size_t row = 0; row < out_dim; row++)
        for (size_t blk = 0; blk < nb; blk++)
            for (int s = 0; s < 8; s++) {
                float db;
                int v[32];
                iq3s_sub_block(bytes + (row * nb + blk) * 110, s, &db, v);
                size_t i = row * nsp + blk * 8 + (size_t)s;
                for (int k = 0; k < 16; k++)
                    out[i * 16 + (size_t)k] = (uint8_t)(((v[k] + 15) / 2) | (((v[k + 16] + 15) / 2) << 4));
                wr16(out + nib_len + i * 2, orc_f32_to_f16(db));
            }
}

int orc_repack_for_matvec(int fmt, const uint8_t *bytes, size_t in_dim, size_t out_dim,
                          uint8_t *out)
{
    int bs = orc_block_size(fmt);
    if (!bs || in_dim % (size_t)bs) return -1;
    memset(out, 0, orc_repacked_len(fmt, in_dim, out_dim));
    switch (fmt) {
    case ORC_Q4_K:   repack_q4_k(bytes, in_dim, out_dim, out); break;
    case ORC_Q5_K:   repack_q5_k(bytes, in_dim, out_dim, out); break;
    case ORC_Q6_K:   repack_q6_k(bytes, in_dim, out_dim, out); break;
    case ORC_Q8_0:   repack_q8_0(bytes, in_dim, out_dim, out); break;
    case ORC_Q4_0:   repack_q4_0(bytes, in_dim, out_dim, out); break;
    case ORC_IQ4_XS: repack_iq4_xs(bytes, in_dim, out_dim, out); break;
    case ORC_Q5_1:   repack_q5_1(bytes, in_dim, out_dim, out); break;
    case ORC_IQ3_S:  repack_iq3_s(bytes, in_dim, out_dim, out); break;
    }
    return 0;
}

/* ------------------------------------------- repacked planes, kernel view */

typedef struct {
    const uint8_t *nib;   /* 16 B / sub-block (Q8_0: lo plane)            */
    const uint8_t *aux;   /* Q5_K qh (4 B), Q6_K hi2 (8 B), Q8_0 hi plane */
    const uint8_t *sm;    /* 2 B / sub-block                               */
    const uint8_t *sup;   /* per-superblock plane                          */
    size_t nsp, n_sub, n_super;
} planes_t;

/* plane offsets exactly as the kernels compute them
 * (matvec_q4k_repacked.cpp:66-71, matvec_q5k_repacked.cpp:50-57,
 *  matvec_q6k_repacked.cpp:54-61, matvec_q8_0_repacked.cpp:48-53,
 *  matvec_q4_0_repacked.cpp:73-75) */
static planes_t planes_of(int fmt, const uint8_t *w, size_t in_dim, size_t out_dim)
{
    planes_t p;
    p.n_sub = in_dim >> 5;
    p.nsp = orc_repacked_n_sub_padded(in_dim);
    p.n_super = p.n_sub >> 3;
    size_t n = out_dim * p.nsp;
    p.nib = w;
    p.aux = p.sm = p.sup = NULL;
    switch (fmt) {
    case ORC_Q4_K:   p.sm = w + n * 16; p.sup = p.sm + n * 2; break;
    case ORC_Q5_K:   p.aux = w + n * 16; p.sm = p.aux + n * 4; p.sup = p.sm + n * 2; break;
    case ORC_Q6_K:   p.aux = w + n * 16; p.sm = p.aux + n * 8; p.sup = p.sm + n * 2; break;
    case ORC_Q8_0:   p.aux = w + n * 16; p.sm = w + n * 32; break;
    case ORC_Q5_1:   p.aux = w + n * 16; p.sm = p.aux + n * 4; break;      /* sm: 4 B / sub-block here */
    case ORC_Q4_0:
    case ORC_IQ3_S:
    case ORC_IQ4_XS: p.sm = w + n * 16; break;
    }
    return p;
}

/* The 32 integer weight values of sub-block (row, sb) in dot order:
 * wq[0..15] pair with activation qs[0..15], wq[16..31] with qs[16..31]
 * (nibble word j low = weights 4j..4j+3, high = 16+4j..; matvec_q4k_repacked.cpp:112-120).
 * Q4_K/Q4_0: 0..15; Q5_K: 0..31; Q6_K: 0..63; Q8_0: int8; IQ4_XS: codebook value. */
static void sub_block_ints(int fmt, const planes_t *p, size_t row, size_t sb, int wq[32])
{
    size_t idx = row * p->nsp + sb;
    const uint8_t *nb = p->nib + idx * 16;
    if (fmt == ORC_Q8_0) {
        const int8_t *lo = (const int8_t *)nb, *hi = (const int8_t *)(p->aux + idx * 16);
        for (int k = 0; k < 16; k++) { wq[k] = lo[k]; wq[16 + k] = hi[k]; }
        return;
    }
    for (int k = 0; k < 16; k++) { wq[k] = nb[k] & 0x0F; wq[16 + k] = nb[k] >> 4; }
    if (fmt == ORC_Q5_K || fmt == ORC_Q5_1) {
        /* bit 4g+b of qh = 5th bit of weight b of dot group g; group 2j = weights
         * 4j.., group 2j+1 = weights 16+4j.. (matvec_q5k_repacked.cpp:90-91) */
        uint32_t qh = rd32(p->aux + idx * 4);
        for (int j = 0; j < 4; j++)
            for (int b = 0; b < 4; b++) {
                wq[4 * j + b]      |= (int)((qh >> (8 * j + b)) & 1u) << 4;
                wq[16 + 4 * j + b] |= (int)((qh >> (8 * j + 4 + b)) & 1u) << 4;
            }
    } else if (fmt == ORC_Q6_K) {
        /* byte g of the hi2 plane = the four 2-bit fields of dot group g
         * (matvec_q6k_repacked.cpp:97-103) */
        const uint8_t *h2 = p->aux + idx * 8;
        for (int j = 0; j < 4; j++)
            for (int b = 0; b < 4; b++) {
                wq[4 * j + b]      |= ((h2[2 * j] >> (2 * b)) & 3) << 4;
                wq[16 + 4 * j + b] |= ((h2[2 * j + 1] >> (2 * b)) & 3) << 4;
            }
    } else if (fmt == ORC_IQ4_XS) {
        for (int k = 0; k < 32; k++) wq[k] = KVALUES_IQ4NL[wq[k]];
    } else if (fmt == ORC_IQ3_S) {
        for (int k = 0; k < 32; k++) wq[k] = 2 * wq[k] - 15;      /* KVALUES_IQ3S, iq3_s.rs:161-162 */
    }
}

/* original position inside the row of weight k (dot order) of sub-block sb
 * (q4_k.rs:294-295 for the K-quants; q6_k.rs:106-143; contiguous otherwise) */
static size_t orig_pos(int fmt, size_t sb, int k)
{
    size_t blk = sb / 8, s = sb % 8;
    switch (fmt) {
    case ORC_Q4_K:
    case ORC_Q5_K: return blk * 256 + (s / 2) * 64 + (s & 1) * 32 + (size_t)k;
    case ORC_Q6_K: return blk * 256 + (s / 4) * 128 + (s % 4) * 32 + (size_t)k;
    default:       return sb * 32 + (size_t)k;
    }
}

int orc_decode_repacked_to_f32(int fmt, const uint8_t *packed, size_t in_dim, size_t out_dim,
                               float *out)
{
    if (!orc_block_size(fmt)) return -1;
    planes_t p = planes_of(fmt, packed, in_dim, out_dim);
    for (size_t row = 0; row < out_dim; row++)
        for (size_t sb = 0; sb < p.n_sub; sb++) {
            int wq[32];
            sub_block_ints(fmt, &p, row, sb, wq);
            size_t idx = row * p.nsp + sb;
            float *o = out + row * in_dim;
            if (fmt == ORC_Q4_K || fmt == ORC_Q5_K) {
                const uint8_t *dd = p.sup + (row * p.n_super + sb / 8) * 4;
                float dsc  = orc_f16_to_f32(rd16(dd)) * (float)p.sm[idx * 2];
                float deff = orc_f16_to_f32(rd16(dd + 2)) * (float)p.sm[idx * 2 + 1];
                for (int k = 0; k < 32; k++) o[orig_pos(fmt, sb, k)] = dsc * (float)wq[k] - deff;
            } else if (fmt == ORC_Q5_1) {
                float dsc = orc_f16_to_f32(rd16(p.sm + idx * 4)), deff = -orc_f16_to_f32(rd16(p.sm + idx * 4 + 2));
                for (int k = 0; k < 32; k++) o[orig_pos(fmt, sb, k)] = dsc * (float)wq[k] - deff;
            } else if (fmt == ORC_Q6_K) {
                float d = orc_f16_to_f32(rd16(p.sup + (row * p.n_super + sb / 8) * 2));
                float s0 = (float)(int8_t)p.sm[idx * 2], s1 = (float)(int8_t)p.sm[idx * 2 + 1];
                for (int k = 0; k < 32; k++)
                    o[orig_pos(fmt, sb, k)] = d * (k < 16 ? s0 : s1) * (float)(wq[k] - 32);
            } else {
                float d = orc_f16_to_f32(rd16(p.sm + idx * 2));
                int off = (fmt == ORC_Q4_0) ? 8 : 0;
                for (int k = 0; k < 32; k++) o[orig_pos(fmt, sb, k)] = d * (float)(wq[k] - off);
            }
        }
    return 0;
}

/* ------------------------------------------------------------- quantizers */

/* src/quant/q8_0.rs:45-61 — Rust f32::round is half-away-from-zero = roundf */
void orc_q8_0_quantize_from_f32(const float *vals, size_t n, uint8_t *out)
{
    for (size_t b = 0; b < n / 32; b++) {
        const float *v = vals + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) { float a = fabsf(v[i]); if (a > amax) amax = a; }
        float d = amax / 127.0f;
        float inv = d > 0.0f ? 1.0f / d : 0.0f;
        uint8_t *o = out + b * 34;
        wr16(o, orc_f32_to_f16(d));
        for (int i = 0; i < 32; i++) {
            float r = roundf(v[i] * inv);
            if (r < -127.0f) r = -127.0f;
            if (r > 127.0f) r = 127.0f;
            o[2 + i] = (uint8_t)(int8_t)r;
        }
    }
}

/* kernels/quantize_q8.cpp:37-53.  The butterfly (offsets 16,8,4,2,1, every lane
 * updated from the previous level) is restated literally; lane 0 is stored.
 * inv is IEEE 127/amax (the reference's v_rcp_f32 form is not portable). */
void orc_quantize_q8(const float *x, size_t in_dim, size_t n_vec, uint8_t *out)
{
    size_t n_sub = in_dim >> 5;
    for (size_t vec = 0; vec < n_vec; vec++)
        for (size_t blk = 0; blk < n_sub; blk++) {
            const float *v = x + vec * in_dim + blk * 32;
            float amax[32], sum[32], ta[32], ts[32];
            for (int l = 0; l < 32; l++) { amax[l] = fabsf(v[l]); sum[l] = v[l]; }
            for (int o = 16; o > 0; o >>= 1) {
                for (int l = 0; l < 32; l++) {
                    ta[l] = fmaxf(amax[l], amax[l ^ o]);
                    ts[l] = sum[l] + sum[l ^ o];
                }
                memcpy(amax, ta, sizeof ta);
                memcpy(sum, ts, sizeof ts);
            }
            float am = amax[0];
            float d = am > 0.0f ? am / 127.0f : 1.0f;
            float inv = am > 0.0f ? 127.0f / am : 0.0f;
            uint8_t *o = out + (vec * n_sub + blk) * 40;
            memcpy(o, &d, 4);
            memcpy(o + 4, &sum[0], 4);
            for (int l = 0; l < 32; l++) {
                int q = (int)rintf(v[l] * inv);
                if (q < -127) q = -127;
                if (q > 127) q = 127;
                o[8 + l] = (uint8_t)(int8_t)q;
            }
        }
}

/* ------------------------------------------------------------- int8 path */

int orc_block_dot_parts(int fmt) { return fmt == ORC_Q6_K ? 2 : 1; }

/* integer part of one (row, sub-block, activation block): what the kernels hold
 * in idot (and xis/xqsum) just before the fp32 combine */
static void block_dot(int fmt, const planes_t *p, size_t row, size_t sb, const int8_t *q8,
                      int32_t parts[2])
{
    int wq[32];
    sub_block_ints(fmt, p, row, sb, wq);
    int32_t lo = 0, hi = 0, xlo = 0, xhi = 0;
    for (int k = 0; k < 16; k++) {
        lo += wq[k] * q8[k];        xlo += q8[k];
        hi += wq[16 + k] * q8[16 + k]; xhi += q8[16 + k];
    }
    switch (fmt) {
    case ORC_Q6_K:                                   /* matvec_q6k_repacked.cpp:83-108 */
        parts[0] = lo - 32 * xlo;
        parts[1] = hi - 32 * xhi;
        break;
    case ORC_Q4_0:                                   /* matvec_q4_0_repacked.cpp:85-110 */
        parts[0] = lo + hi - 8 * (xlo + xhi);
        parts[1] = 0;
        break;
    default:
        parts[0] = lo + hi;
        parts[1] = 0;
        break;
    }
}

int orc_block_dots(int fmt, const uint8_t *packed, size_t in_dim, size_t out_dim,
                   const uint8_t *xq, size_t n_rows, int32_t *out)
{
    if (!orc_block_size(fmt)) return -1;
    planes_t p = planes_of(fmt, packed, in_dim, out_dim);
    int np = orc_block_dot_parts(fmt);
    for (size_t t = 0; t < n_rows; t++)
        for (size_t r = 0; r < out_dim; r++)
            for (size_t sb = 0; sb < p.n_sub; sb++) {
                int32_t parts[2];
                block_dot(fmt, &p, r, sb, (const int8_t *)(xq + (t * p.n_sub + sb) * 40 + 8), parts);
                for (int k = 0; k < np; k++) out[((t * out_dim + r) * p.n_sub + sb) * (size_t)np + (size_t)k] = parts[k];
            }
    return 0;
}

/* fp32 contribution of one sub-block, expression order as in the kernels:
 *   Q4_K/Q5_K  dsc*dx*(float)idot - deff*xsum      matvec_q4k_repacked.cpp:106-121
 *   Q6_K       dsc_lo*dx*(float)i0 + dsc_hi*dx*(float)i1   matvec_q6k_repacked.cpp:91-108
 *   Q4_0       dw*dx*(float)(idot - 8*xqsum)       matvec_q4_0_repacked.cpp:99-110
 *   Q8_0       dw*dx*(float)idot                   matvec_q8_0_repacked.cpp:78-85
 *   IQ4_XS     dw*dx*(float)idot                   matvec_iq4xs_repacked.cpp:105-115 */
static float block_term(int fmt, const planes_t *p, size_t row, size_t sb, const uint8_t *xb)
{
    float dx, xsum;
    memcpy(&dx, xb, 4);
    memcpy(&xsum, xb + 4, 4);
    int32_t parts[2];
    block_dot(fmt, p, row, sb, (const int8_t *)(xb + 8), parts);
    size_t idx = row * p->nsp + sb;
    if (fmt == ORC_Q4_K || fmt == ORC_Q5_K) {
        const uint8_t *dd = p->sup + (row * p->n_super + sb / 8) * 4;
        float dsc  = orc_f16_to_f32(rd16(dd)) * (float)p->sm[idx * 2];
        float deff = orc_f16_to_f32(rd16(dd + 2)) * (float)p->sm[idx * 2 + 1];
        return dsc * dx * (float)parts[0] - deff * xsum;
    }
    if (fmt == ORC_Q5_1) {                           /* moe_matvec_q5k_repacked.cpp:86-91: dsc = d, deff = -m */
        float dsc = orc_f16_to_f32(rd16(p->sm + idx * 4)), deff = -orc_f16_to_f32(rd16(p->sm + idx * 4 + 2));
        return dsc * dx * (float)parts[0] - deff * xsum;
    }
    if (fmt == ORC_Q6_K) {
        float d = orc_f16_to_f32(rd16(p->sup + (row * p->n_super + sb / 8) * 2));
        float dlo = d * (float)(int)(int8_t)p->sm[idx * 2];
        float dhi = d * (float)(int)(int8_t)p->sm[idx * 2 + 1];
        return dlo * dx * (float)parts[0] + dhi * dx * (float)parts[1];
    }
    float dw = orc_f16_to_f32(rd16(p->sm + idx * 2));
    return dw * dx * (float)parts[0];
}

static float row_dot_q8(int fmt, const planes_t *p, size_t row, const uint8_t *xrow)
{
    /* lane l accumulates sub-blocks l, l+64, ... in order, then the wave64
     * xor tree 1,2,4,8,16,32 (kernels/gfx906_dpp.h:69-77); lane 0 is stored */
    float acc[64], t[64];
    for (int l = 0; l < 64; l++) {
        float a = 0.0f;
        for (size_t sb = (size_t)l; sb < p->n_sub; sb += 64)
            a += block_term(fmt, p, row, sb, xrow + sb * 40);
        acc[l] = a;
    }
    for (int o = 1; o < 64; o <<= 1) {
        for (int l = 0; l < 64; l++) t[l] = acc[l] + acc[l ^ o];
        memcpy(acc, t, sizeof t);
    }
    return acc[0];
}

int orc_matvec_q8(int fmt, const uint8_t *packed, size_t in_dim, size_t out_dim,
                  const uint8_t *xq, size_t n_rows, float *y, int n_threads)
{
    if (!orc_block_size(fmt)) return -1;
    planes_t p = planes_of(fmt, packed, in_dim, out_dim);
    long total = (long)(n_rows * out_dim);
    (void)n_threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(n_threads > 0 ? n_threads : 1)
#endif
    for (long i = 0; i < total; i++) {
        size_t t = (size_t)i / out_dim, r = (size_t)i % out_dim;
        y[i] = row_dot_q8(fmt, &p, r, xq + t * p.n_sub * 40);
    }
    return 0;
}

/* ---------------------------------------------------------------- f32 path */

/* src/cpu/ops.rs:108-140 */
void orc_matvec_f32(const float *x, const float *w, size_t in_dim, size_t out_dim, float *y,
                    int n_threads)
{
    int par = (in_dim * out_dim >= ((size_t)1 << 16)) && n_threads > 1;
    (void)par;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) if (par) num_threads(n_threads > 0 ? n_threads : 1)
#endif
    for (long j = 0; j < (long)out_dim; j++) {
        const float *row = w + (size_t)j * in_dim;
        float acc = 0.0f;
        for (size_t i = 0; i < in_dim; i++) acc += x[i] * row[i];
        y[j] = acc;
    }
}

/* --------------------------------------------------------------------- MoE */

/* kernels/moe_topk.cpp:17-108.  The block reductions there are max/sum trees
 * over 128 threads; the max is order-free, and the softmax sum below follows
 * the same thread-strided partials + halving tree so the probabilities match
 * a 128-thread launch bit for bit. */
void orc_moe_topk(const float *logits, int n_tok, int n_expert, int n_used, int32_t *out_ids,
                  float *out_weights)
{
    const int nt = 128;
    float *probs = (float *)malloc(sizeof(float) * (size_t)n_expert);
    for (int tok = 0; tok < n_tok; tok++) {
        const float *lg = logits + (size_t)tok * (size_t)n_expert;
        float m = -INFINITY;
        for (int i = 0; i < n_expert; i++) {
            float v = lg[i];
            if (isnan(v)) v = -INFINITY;
            probs[i] = v;
            m = fmaxf(m, v);
        }
        float red[128];
        for (int t = 0; t < nt; t++) {
            float s = 0.0f;
            for (int i = t; i < n_expert; i += nt) {
                float e = expf(probs[i] - m);
                probs[i] = e;
                s += e;
            }
            red[t] = s;
        }
        for (int s = nt >> 1; s > 0; s >>= 1)
            for (int t = 0; t < s; t++) red[t] += red[t + s];
        float inv_sum = 1.0f / red[0];
        for (int i = 0; i < n_expert; i++) probs[i] *= inv_sum;

        float chosen[64];
        for (int k = 0; k < n_used; k++) {
            /* per-thread strided argmax, then the halving tree, strict '>' at
             * both levels (moe_topk.cpp:78-93): a tie keeps the lower thread,
             * which is the lowest index whenever n_expert <= 128 */
            int ridx[128];
            for (int t = 0; t < nt; t++) {
                float bv = -1.0f;
                int bi = 0;
                for (int i = t; i < n_expert; i += nt)
                    if (probs[i] > bv) { bv = probs[i]; bi = i; }
                red[t] = bv;
                ridx[t] = bi;
            }
            for (int s = nt >> 1; s > 0; s >>= 1)
                for (int t = 0; t < s; t++)
                    if (red[t + s] > red[t]) { red[t] = red[t + s]; ridx[t] = ridx[t + s]; }
            out_ids[(size_t)tok * (size_t)n_used + (size_t)k] = ridx[0];
            chosen[k] = red[0];
            probs[ridx[0]] = -1.0f;
        }
        float wsum = 0.0f;
        for (int k = 0; k < n_used; k++) wsum += chosen[k];
        if (wsum < 6.103515625e-5f) wsum = 6.103515625e-5f;
        for (int k = 0; k < n_used; k++) out_weights[(size_t)tok * (size_t)n_used + (size_t)k] = chosen[k] / wsum;
    }
    free(probs);
}

/* kernels/moe_expert_sort.cpp:33-75; ranks taken in entry order */
void orc_moe_sort(const int32_t *ids, int n_entries, int n_expert, int bn, int32_t *perm,
                  int32_t *expert_off, int32_t *tile_off)
{
    int32_t *count = (int32_t *)calloc((size_t)n_expert, sizeof(int32_t));
    for (int i = 0; i < n_entries; i++)
        if (ids[i] >= 0 && ids[i] < n_expert) count[ids[i]]++;
    int eacc = 0, tacc = 0;
    for (int e = 0; e < n_expert; e++) {
        expert_off[e] = eacc;
        tile_off[e] = tacc;
        eacc += count[e];
        tacc += (count[e] + bn - 1) / bn;
    }
    expert_off[n_expert] = eacc;
    tile_off[n_expert] = tacc;
    memset(count, 0, sizeof(int32_t) * (size_t)n_expert);
    for (int i = 0; i < n_entries; i++) {
        int e = ids[i];
        if (e < 0 || e >= n_expert) continue;
        perm[expert_off[e] + count[e]++] = i;
    }
    free(count);
}

/* kernels/moe_expert_sort.cpp:81-97 */
void orc_moe_gather_xq(const uint8_t *xq_src, const int32_t *perm, uint8_t *xq_dst, int nsub,
                       int n_used, int n_entries)
{
    for (int p = 0; p < n_entries; p++) {
        size_t tok = (size_t)((unsigned)perm[p] / (unsigned)n_used);
        memcpy(xq_dst + (size_t)p * (size_t)nsub * 40, xq_src + tok * (size_t)nsub * 40, (size_t)nsub * 40);
    }
}

/* kernels/moe_expert_sort.cpp:101-110 */
void orc_moe_scatter_rows(const float *src, const int32_t *perm, float *dst, int dim,
                          int n_entries)
{
    for (int p = 0; p < n_entries; p++)
        memcpy(dst + (size_t)perm[p] * (size_t)dim, src + (size_t)p * (size_t)dim, sizeof(float) * (size_t)dim);
}

/* kernels/moe_combine.cpp:15-38 */
void orc_moe_combine(const float *experts, const int32_t *ids, const float *weights,
                     const float *down_exps_s, float *out, int n_tok, int hidden, int n_used)
{
    for (int tok = 0; tok < n_tok; tok++) {
        const float *ex = experts + (size_t)tok * (size_t)n_used * (size_t)hidden;
        const int32_t *id = ids + (size_t)tok * (size_t)n_used;
        const float *w = weights + (size_t)tok * (size_t)n_used;
        for (int i = 0; i < hidden; i++) {
            float acc = 0.0f;
            for (int j = 0; j < n_used; j++) {
                float s = w[j] * down_exps_s[id[j]];
                acc += s * ex[(size_t)j * (size_t)hidden + (size_t)i];
            }
            out[(size_t)tok * (size_t)hidden + (size_t)i] = acc;
        }
    }
}

/* ---- relabelled GGUF types -------------------------------------------------- */

/* src/quant/q3_k.rs:124-165, the walk of ggml's dequantize_row_q3_K: two halves of 128
 * weights, four 2-bit shift levels each, two 16-weight sub-blocks per level; the third
 * quant bit comes from hmask with one mask bit per (half, level); bit CLEAR subtracts 4 */
static void q3k_scales(const uint8_t *sc, int out[16])
{
    /* src/quant/q3_k.rs:41-61: low nibbles of scales 0..7 in bytes 0..7, of 8..15 in their
     * high nibbles, the two top bits four per byte in bytes 8..11 */
    uint32_t a0, a1, tmp;
    memcpy(&a0, sc, 4);
    memcpy(&a1, sc + 4, 4);
    memcpy(&tmp, sc + 8, 4);
    const uint32_t k1 = 0x03030303u, k2 = 0x0f0f0f0fu;
    uint32_t aux[4];
    aux[0] = (a0 & k2) | (((tmp >> 0) & k1) << 4);
    aux[1] = (a1 & k2) | (((tmp >> 2) & k1) << 4);
    aux[2] = ((a0 >> 4) & k2) | (((tmp >> 4) & k1) << 4);
    aux[3] = ((a1 >> 4) & k2) | (((tmp >> 6) & k1) << 4);
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++) out[4 * i + j] = (int)(int8_t)((aux[i] >> (8 * j)) & 0xFF);
}

void orc_q3_k_dequantize(const uint8_t *src, float *out, size_t n)
{
    for (size_t b = 0; b < n / 256; b++) {
        const uint8_t *blk = src + b * 110;
        const uint8_t *hmask = blk, *qs = blk + 32;
        uint16_t dbits;
        memcpy(&dbits, blk + 108, 2);
        const float d_all = orc_f16_to_f32(dbits);
        int scales[16];
        q3k_scales(blk + 96, scales);
        float *ob = out + b * 256;
        size_t y = 0;
        int is = 0;
        unsigned m = 1;
        for (int half = 0; half < 2; half++) {
            const uint8_t *q = qs + 32 * half;
            for (int shift = 0; shift < 8; shift += 2) {
                for (int part = 0; part < 2; part++) {
                    const float dl = d_all * (float)(scales[is++] - 32);
                    for (int l = 0; l < 16; l++) {
                        const int lo = (q[l + 16 * part] >> shift) & 3;
                        const int hi = (hmask[l + 16 * part] & m) ? 0 : 4;
                        ob[y++] = dl * (float)(lo - hi);
                    }
                }
                m <<= 1;
            }
        }
    }
}

/* src/quant/iq4_nl.rs:34-50: w[k] = d * kvalues[qs[k] & 15], w[k+16] = d * kvalues[qs[k] >> 4] */
void orc_iq4_nl_dequantize(const uint8_t *src, float *out, size_t n)
{
    for (size_t b = 0; b < n / 32; b++) {
        const uint8_t *blk = src + b * 18;
        uint16_t dbits;
        memcpy(&dbits, blk, 2);
        const float d = orc_f16_to_f32(dbits);
        for (int k = 0; k < 16; k++) {
            out[b * 32 + k] = d * (float)KVALUES_IQ4NL[blk[2 + k] & 15];
            out[b * 32 + k + 16] = d * (float)KVALUES_IQ4NL[blk[2 + k] >> 4];
        }
    }
}

void orc_bf16_to_f32(const uint16_t *src, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        const uint32_t bits = (uint32_t)src[i] << 16;
        memcpy(&out[i], &bits, 4);
    }
}

/* ---- fused BlockQ8 producers ---------------------------------------------- */

float orc_exp_det(float x)
{
    x = fminf(fmaxf(x, -87.0f), 88.0f);
    const float n = rintf(x * 1.44269504088896341f);
    float r = fmaf(n, -0.693145751953125f, x);
    r = fmaf(n, -1.42860682030941723e-6f, r);
    float p = 1.0f / 720.0f;
    p = fmaf(p, r, 1.0f / 120.0f);
    p = fmaf(p, r, 1.0f / 24.0f);
    p = fmaf(p, r, 1.0f / 6.0f);
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    const int ni = (int)n;
    const int n1 = ni / 2, n2 = ni - n1;
    const uint32_t b1 = (uint32_t)(n1 + 127) << 23, b2 = (uint32_t)(n2 + 127) << 23;
    float s1, s2;
    memcpy(&s1, &b1, 4);
    memcpy(&s2, &b2, 4);
    return p * s1 * s2;
}

float orc_silu_det(float x) { return x / (1.0f + orc_exp_det(-x)); }
float orc_sigmoid_det(float x) { return 1.0f / (1.0f + orc_exp_det(-x)); }
float orc_gelu_det(float x)
{
    const float c = x + 0.044715f * x * x * x;
    return x / (1.0f + orc_exp_det(-2.0f * (0.7978845608028654f * c)));
}

void orc_map_det(int which, const float *x, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++)
        out[i] = which == 0 ? orc_exp_det(x[i]) : which == 1 ? orc_silu_det(x[i]) : which == 2 ? orc_sigmoid_det(x[i])
               : orc_gelu_det(x[i]);
}

/* src/cpu/ops.rs:14-16, 20-22, 33-36 with libm */
void orc_map_ref(int which, const float *x, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        const float v = x[i];
        if (which == 1) out[i] = v / (1.0f + expf(-v));
        else if (which == 2) out[i] = 1.0f / (1.0f + expf(-v));
        else out[i] = 0.5f * v * (1.0f + tanhf(0.79788456f * (v + 0.044715f * v * v * v)));
    }
}

float orc_sumsq_det(const float *x, size_t n)
{
    const size_t n_sub = n >> 5;
    float lane[64];
    for (int l = 0; l < 64; l++) lane[l] = 0.0f;
    for (size_t sb = 0; sb < n_sub; sb++) {           /* ascending sb visits each lane's addends in its order */
        float s[32], t[32];
        for (int l = 0; l < 32; l++) s[l] = x[sb * 32 + l] * x[sb * 32 + l];
        for (int o = 16; o > 0; o >>= 1) {
            for (int l = 0; l < 32; l++) t[l] = s[l] + s[l ^ o];
            memcpy(s, t, sizeof s);
        }
        lane[sb & 63] = lane[sb & 63] + s[0];
    }
    float t[64];
    for (int o = 32; o > 0; o >>= 1) {
        for (int l = 0; l < 64; l++) t[l] = lane[l] + lane[l ^ o];
        memcpy(lane, t, sizeof lane);
    }
    return lane[0];
}

void orc_add_rmsnorm(float *hidden, const float *add, const float *w, float *y, size_t n, size_t n_vec, float eps)
{
    for (size_t v = 0; v < n_vec; v++) {
        float *h = hidden + v * n;
        if (add)
            for (size_t i = 0; i < n; i++) h[i] = h[i] + add[v * n + i];
        const float rrms = 1.0f / sqrtf(orc_sumsq_det(h, n) / (float)n + eps);
        for (size_t i = 0; i < n; i++) y[v * n + i] = (h[i] * rrms) * w[i];
    }
}

void orc_rmsnorm_gated(const float *x, const float *z, const float *w, float *y, size_t n_heads, size_t head_dim, float eps)
{
    for (size_t h = 0; h < n_heads; h++) {
        const float *xh = x + h * head_dim, *zh = z + h * head_dim;
        const float rrms = 1.0f / sqrtf(orc_sumsq_det(xh, head_dim) / (float)head_dim + eps);
        for (size_t i = 0; i < head_dim; i++) y[h * head_dim + i] = ((xh[i] * rrms) * w[i]) * orc_silu_det(zh[i]);
    }
}

void orc_swiglu_det(const float *gate, const float *up, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++) out[i] = orc_silu_det(gate[i]) * up[i];
}

void orc_sigmoid_mul_det(const float *x, const float *gate, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++) out[i] = x[i] * orc_sigmoid_det(gate[i]);
}

void orc_geglu_det(const float *gu, float *out, size_t ff_exp, size_t n_slot)
{
    for (size_t s = 0; s < n_slot; s++)
        for (size_t i = 0; i < ff_exp; i++)
            out[s * ff_exp + i] = orc_gelu_det(gu[s * 2 * ff_exp + i]) * gu[s * 2 * ff_exp + ff_exp + i];
}

/* src/cpu/ops.rs:47-57 */
void orc_rmsnorm_ref(const float *x, const float *w, float eps, float *out, size_t n)
{
    float sum_sq = 0.0f;
    for (size_t i = 0; i < n; i++) sum_sq += x[i] * x[i];
    const float rrms = 1.0f / sqrtf(sum_sq / (float)n + eps);
    for (size_t i = 0; i < n; i++) out[i] = x[i] * rrms * w[i];
}

/* src/cpu/ops.rs:63-76 */
void orc_rmsnorm_gated_ref(const float *x, const float *gate, const float *w, float eps, float *out, size_t n)
{
    float sum_sq = 0.0f;
    for (size_t i = 0; i < n; i++) sum_sq += x[i] * x[i];
    const float rrms = 1.0f / sqrtf(sum_sq / (float)n + eps);
    for (size_t i = 0; i < n; i++) out[i] = x[i] * rrms * w[i] * (gate[i] / (1.0f + expf(-gate[i])));
}

/* kernels/swiglu.cpp:10-21 */
void orc_swiglu_mul(const float *gate, const float *up, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        float g = gate[i];
        float s = g / (1.0f + expf(-g));
        out[i] = s * up[i];
    }
}

/* kernels/mmq_gemm_q4k_grouped.cpp:38-165 — per (token,row) the same
 * per-sub-block terms as the matvec, summed in sub-block order */
int orc_grouped_gemm(int fmt, const uint8_t *slab, size_t bytes_per_expert,
                     const int32_t *expert_off, int n_expert, const uint8_t *xq, float *y,
                     size_t in_dim, size_t out_dim, int n_threads)
{
    if (!orc_block_size(fmt)) return -1;
    size_t n_sub = in_dim >> 5;
    for (int e = 0; e < n_expert; e++) {
        int t0 = expert_off[e], t1 = expert_off[e + 1];
        if (t1 <= t0) continue;
        int rc = orc_matvec_q8(fmt, slab + (size_t)e * bytes_per_expert, in_dim, out_dim,
                               xq + (size_t)t0 * n_sub * 40, (size_t)(t1 - t0),
                               y + (size_t)t0 * out_dim, n_threads);
        if (rc) return rc;
    }
    return 0;
}
