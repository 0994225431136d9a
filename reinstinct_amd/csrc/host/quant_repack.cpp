// Host-side mirror of the reference's src/quant layout contract: repacked_len,
// repacked_n_sub_padded and repack_for_matvec for the six formats.  Load-time
// code (runs once per weight, host to host), written destination-first: for
// every 32-weight sub-block of the output it pulls that sub-block's fields out
// of the on-disk block and emits the planes.  Rows are split over threads.
#include <algorithm>
#include <cstring>
#include <thread>
#include <vector>

#include "../../../include/rein.h"
#include "hip_api.h"
#include "iq3s_grid.h"

namespace {

struct Geometry {
    int    block;        // weights per on-disk block
    int    bytes;        // bytes per on-disk block
    size_t per_sub;      // bytes per sub-block over all per-sub-block planes
    size_t per_super;    // bytes per 256-weight superblock plane entry
};

bool geometry(int fmt, Geometry* g)
{
    switch (fmt) {
    case REIN_TYPE_Q4_0:   *g = {32, 18, 16 + 2, 0}; return true;       // src/quant/q4_0.rs:22-23,66-69
    case REIN_TYPE_Q8_0:   *g = {32, 34, 32 + 2, 0}; return true;       // src/quant/q8_0.rs:8-9,74-77
    case REIN_TYPE_Q4_K:   *g = {256, 144, 16 + 2, 4}; return true;     // src/quant/q4_k.rs:17-18,98-102
    case REIN_TYPE_Q5_K:   *g = {256, 176, 16 + 4 + 2, 4}; return true; // src/quant/q5_k.rs:21-22,100-104
    case REIN_TYPE_Q6_K:   *g = {256, 210, 16 + 8 + 2, 2}; return true; // src/quant/q6_k.rs:18-19,89-93
    case REIN_TYPE_IQ4_XS: *g = {256, 136, 16 + 2, 0}; return true;     // src/quant/iq4_xs.rs:23-24,85-88
    case REIN_TYPE_Q5_1:   *g = {32, 24, 16 + 4 + 4, 0}; return true;   // src/quant/q5_1.rs:25-26,76-81
    case REIN_TYPE_IQ3_S:  *g = {256, 110, 16 + 2, 0}; return true;     // src/quant/iq3_s.rs:24-25,178-184
    default: return false;
    }
}

inline uint16_t load16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }
inline void store16(uint8_t* p, uint16_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); }

// IEEE half <-> float with the reference's rounding behaviour
// (src/quant/half.rs:9-40, 51-84: RNE for normal results, truncation for
// subnormal results).
float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    int      e = (h >> 10) & 31;
    uint32_t m = h & 1023u;
    uint32_t bits;
    if (e == 31) {
        bits = sign | 0x7F800000u | (m << 13);
    } else if (e != 0) {
        bits = sign | ((uint32_t)(e + 112) << 23) | (m << 13);
    } else if (m == 0) {
        bits = sign;
    } else {
        e = 113;
        while (!(m & 1024u)) { m <<= 1; e--; }
        bits = sign | ((uint32_t)e << 23) | ((m & 1023u) << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

uint16_t float_to_half(float f)
{
    uint32_t b;
    std::memcpy(&b, &f, 4);
    const uint16_t sign = (uint16_t)((b >> 16) & 0x8000u);
    const int      e = (int)((b >> 23) & 255u) - 127;
    const uint32_t m = b & 0x7FFFFFu;
    if (e == 128) return (uint16_t)(sign | 0x7C00u | (m ? 0x200u : 0u));
    if (e > 15) return (uint16_t)(sign | 0x7C00u);
    if (e < -24) return sign;
    if (e < -14) return (uint16_t)(sign | (uint16_t)((m | 0x800000u) >> (unsigned)(-1 - e)));
    uint16_t h = (uint16_t)(sign | (uint16_t)((e + 15) << 10) | (uint16_t)(m >> 13));
    const uint32_t rest = m & 0x1FFFu;
    if (rest > 0x1000u || (rest == 0x1000u && (h & 1u))) h = (uint16_t)(h + 1u);
    return h;
}

// 6-bit (scale, min) of sub-block j from the 12 packed bytes (q4_k.rs:40-48).
inline void scale_min_k4(const uint8_t* q, int j, uint8_t* sc, uint8_t* mn)
{
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[4 + j] & 63;
    } else {
        *sc = (uint8_t)((q[4 + j] & 15) | ((q[j - 4] >> 6) << 4));
        *mn = (uint8_t)((q[4 + j] >> 4) | ((q[j] >> 6) << 4));
    }
}

// One 32-weight sub-block in dot order: element k pairs with activation quant k.
struct SubBlock {
    uint8_t lo4[32];     // low four bits of every weight
    uint8_t ext[32];     // Q5_K: bit 4; Q6_K: bits 4-5
    uint8_t sm[2];       // per-sub-block scale bytes
};

// nibble plane: byte 4j+b = lo4[4j+b] | lo4[16+4j+b] << 4 (q4_k.rs:158-165); the
// two halves of the sub-block end up in the low / high nibbles of 16 bytes.
inline void emit_nibbles(const SubBlock& s, uint8_t* dst)
{
    for (int k = 0; k < 16; k++) dst[k] = (uint8_t)(s.lo4[k] | (s.lo4[16 + k] << 4));
}

// qh word of the Q5_K kernels: bit 4g+b = 5th bit of weight b of dot group g; group 2j is
// weights 4j.., group 2j+1 weights 16+4j.. (q5_k.rs:122-141, q5_1.rs:70-73)
inline uint32_t fifth_bits(const SubBlock& w)
{
    uint32_t qh = 0;
    for (int k = 0; k < 16; k++) {
        qh |= (uint32_t)(w.ext[k] & 1) << (8 * (k / 4) + (k % 4));
        qh |= (uint32_t)(w.ext[16 + k] & 1) << (8 * (k / 4) + 4 + (k % 4));
    }
    return qh;
}

void repack_rows(int fmt, const Geometry& g, const uint8_t* src, size_t in_dim, size_t out_dim,
                 uint8_t* dst, size_t row_begin, size_t row_end)
{
    const size_t n_sub   = in_dim / 32;
    const size_t nsp     = rein_repacked_n_sub_padded(in_dim);
    const size_t n_super = in_dim / 256;
    const size_t n       = out_dim * nsp;
    uint8_t* const nib = dst;

    for (size_t row = row_begin; row < row_end; row++) {
        for (size_t sb = 0; sb < n_sub; sb++) {
            const size_t i = row * nsp + sb;
            switch (fmt) {
            case REIN_TYPE_Q4_0: {     // q4_0.rs:86-104: nibble bytes verbatim, fp16 d split out
                const uint8_t* b = src + (row * n_sub + sb) * 18;
                std::memcpy(nib + i * 16, b + 2, 16);
                std::memcpy(dst + n * 16 + i * 2, b, 2);
                break;
            }
            case REIN_TYPE_Q8_0: {     // q8_0.rs:93-119: quants 0-15 | quants 16-31 | fp16 d
                const uint8_t* b = src + (row * n_sub + sb) * 34;
                std::memcpy(nib + i * 16, b + 2, 16);
                std::memcpy(dst + n * 16 + i * 16, b + 18, 16);
                std::memcpy(dst + n * 32 + i * 2, b, 2);
                break;
            }
            case REIN_TYPE_IQ4_XS: {   // iq4_xs.rs:106-136: nibbles verbatim, fp16(d*(ls-32))
                const uint8_t* b = src + (row * n_super + sb / 8) * 136;
                const int ib = (int)(sb % 8);
                const int ls = ((b[4 + ib / 2] >> (4 * (ib & 1))) & 15) | (((load16(b + 2) >> (2 * ib)) & 3) << 4);
                std::memcpy(nib + i * 16, b + 8 + ib * 16, 16);
                store16(dst + n * 16 + i * 2, float_to_half(half_to_float(load16(b)) * (float)(ls - 32)));
                break;
            }
            case REIN_TYPE_Q5_1: {     // q5_1.rs:82-104: nibbles verbatim, qh in dot-group order, raw fp16 d | m
                const uint8_t* b = src + (row * n_sub + sb) * 24;
                std::memcpy(nib + i * 16, b + 8, 16);
                const uint32_t bits = (uint32_t)b[4] | ((uint32_t)b[5] << 8) | ((uint32_t)b[6] << 16) | ((uint32_t)b[7] << 24);
                SubBlock w;
                for (int k = 0; k < 32; k++) w.ext[k] = (uint8_t)((bits >> k) & 1);   // on disk bit k is weight k
                const uint32_t qh = fifth_bits(w);
                std::memcpy(dst + n * 16 + i * 4, &qh, 4);
                std::memcpy(dst + n * 20 + i * 4, b, 4);
                break;
            }
            case REIN_TYPE_IQ3_S: {    // iq3_s.rs:186-207: signed odd values -> nibble (v + 15) / 2, fp16(d * (1 + 2*scale))
                const uint8_t* b = src + (row * n_super + sb / 8) * 110;
                const int s = (int)(sb % 8);
                const uint8_t* index = b + 2 + 8 * s;                // eight grid indices, low 8 bits
                const unsigned high = b[66 + s];                     // their 9th bits
                const uint8_t* sign = b + 74 + 4 * s;                // one bit per weight
                const int scale = (b[106 + s / 2] >> (4 * (s & 1))) & 15;
                SubBlock w;
                for (int k = 0; k < 32; k++) {
                    const unsigned entry = index[k / 4] | (((high >> (k / 4)) & 1u) << 8);
                    const int mag = rein::iq3s_magnitude(entry, (unsigned)k % 4);
                    const int v = ((sign[k / 8] >> (k % 8)) & 1) ? -mag : mag;
                    w.lo4[k] = (uint8_t)((v + 15) / 2);
                }
                emit_nibbles(w, nib + i * 16);
                store16(dst + n * 16 + i * 2, float_to_half(half_to_float(load16(b)) * (1.0f + 2.0f * (float)scale)));
                break;
            }
            case REIN_TYPE_Q4_K:       // q4_k.rs:126-176
            case REIN_TYPE_Q5_K: {     // q5_k.rs:97-151
                const bool q5 = fmt == REIN_TYPE_Q5_K;
                const uint8_t* b = src + (row * n_super + sb / 8) * (size_t)g.bytes;
                const int s = (int)(sb % 8);
                const uint8_t* qs = b + (q5 ? 48 : 16) + (s / 2) * 32;
                SubBlock w;
                for (int k = 0; k < 32; k++) {
                    w.lo4[k] = (s & 1) ? (uint8_t)(qs[k] >> 4) : (uint8_t)(qs[k] & 15);
                    w.ext[k] = q5 ? (uint8_t)((b[16 + k] >> s) & 1) : (uint8_t)0;
                }
                scale_min_k4(b + 4, s, &w.sm[0], &w.sm[1]);
                emit_nibbles(w, nib + i * 16);
                size_t off = n * 16;
                if (q5) {
                    const uint32_t qh = fifth_bits(w);
                    std::memcpy(dst + off + i * 4, &qh, 4);
                    off += n * 4;
                }
                dst[off + i * 2]     = w.sm[0];
                dst[off + i * 2 + 1] = w.sm[1];
                if (s == 0) std::memcpy(dst + off + n * 2 + (row * n_super + sb / 8) * 4, b, 4);
                break;
            }
            case REIN_TYPE_Q6_K: {     // q6_k.rs:86-148
                const uint8_t* b = src + (row * n_super + sb / 8) * 210;
                const int s = (int)(sb % 8), chunk = s / 4, quad = s % 4;
                const uint8_t* ql = b + chunk * 64 + (quad & 1) * 32;
                const uint8_t* qh = b + 128 + chunk * 32;
                SubBlock w;
                for (int k = 0; k < 32; k++) {
                    w.lo4[k] = (quad & 2) ? (uint8_t)(ql[k] >> 4) : (uint8_t)(ql[k] & 15);
                    w.ext[k] = (uint8_t)((qh[k] >> (2 * quad)) & 3);
                }
                emit_nibbles(w, nib + i * 16);
                // byte g = the four 2-bit fields of dot group g (q6_k.rs:128-138)
                uint8_t h2[8] = {0, 0, 0, 0, 0, 0, 0, 0};
                for (int k = 0; k < 16; k++) {
                    h2[2 * (k / 4)]     |= (uint8_t)(w.ext[k] << (2 * (k % 4)));
                    h2[2 * (k / 4) + 1] |= (uint8_t)(w.ext[16 + k] << (2 * (k % 4)));
                }
                std::memcpy(dst + n * 16 + i * 8, h2, 8);
                dst[n * 24 + i * 2]     = b[192 + chunk * 8 + quad * 2];
                dst[n * 24 + i * 2 + 1] = b[192 + chunk * 8 + quad * 2 + 1];
                if (s == 0) std::memcpy(dst + n * 26 + (row * n_super + sb / 8) * 2, b + 208, 2);
                break;
            }
            }
        }
    }
}

}  // namespace

extern "C" {

size_t rein_repacked_n_sub_padded(size_t in_dim)
{
    const size_t n = in_dim / 32;
    return (n != 0 && (n & (n - 1)) == 0) ? n + 1 : n;
}

size_t rein_repacked_len(int fmt, size_t in_dim, size_t out_dim)
{
    Geometry g;
    if (!geometry(fmt, &g)) return 0;
    return out_dim * rein_repacked_n_sub_padded(in_dim) * g.per_sub + out_dim * (in_dim / 256) * g.per_super;
}

int rein_block_size(int fmt)
{
    Geometry g;
    return geometry(fmt, &g) ? g.block : 0;
}

int rein_bytes_per_block(int fmt)
{
    Geometry g;
    return geometry(fmt, &g) ? g.bytes : 0;
}

int rein_repack_for_matvec(int fmt, const uint8_t* src, size_t in_dim, size_t out_dim, uint8_t* dst)
{
    Geometry g;
    if (!geometry(fmt, &g)) return rein::fail(REIN_E_BAD_FORMAT, "rein_repack_for_matvec: unknown format " + std::to_string(fmt));
    if (in_dim == 0 || in_dim % (size_t)g.block != 0)
        return rein::fail(REIN_E_BAD_SHAPE, "rein_repack_for_matvec: in_dim must be a non-zero multiple of " + std::to_string(g.block));
    if (!src || !dst) return rein::fail(REIN_E_BAD_POINTER, "rein_repack_for_matvec: null pointer");
    std::memset(dst, 0, rein_repacked_len(fmt, in_dim, out_dim));

    size_t n_threads = std::min<size_t>(std::max(1u, std::thread::hardware_concurrency()), 16);
    if (in_dim * out_dim < ((size_t)1 << 22)) n_threads = 1;
    n_threads = std::min(n_threads, std::max<size_t>(out_dim, 1));
    if (n_threads <= 1) {
        repack_rows(fmt, g, src, in_dim, out_dim, dst, 0, out_dim);
        return 0;
    }
    std::vector<std::thread> pool;
    const size_t step = (out_dim + n_threads - 1) / n_threads;
    for (size_t t = 0; t < n_threads; t++) {
        const size_t a = t * step, b = std::min(out_dim, a + step);
        if (a >= b) break;
        pool.emplace_back(repack_rows, fmt, std::cref(g), src, in_dim, out_dim, dst, a, b);
    }
    for (auto& th : pool) th.join();
    return 0;
}

}  // extern "C"
