// fp32 -> on-disk quantized blocks, for building synthetic weights of the
// benchmark / test shapes ("fp32 ~N(0,0.02) quantized to <fmt>").  Only Q8_0 has
// a counterpart in the reference (q8_0::quantize_from_f32, src/quant/q8_0.rs:45-61);
// the other five follow the structure of ggml's reference quantizers
// (per-sub-block affine or symmetric fit, then 6-/8-bit quantization of the
// sub-block scales against a per-superblock fp16) without their iterative
// refinement.  Any output is a valid block of its format, which is all the
// matmul path requires: GPU kernels and the CPU checker consume the same bytes.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "../../../include/rein.h"
#include "hip_api.h"

namespace {

inline void store16(uint8_t* p, uint16_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); }

uint16_t to_half(float f)
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

float from_half(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h >> 15) << 31;
    int      e = (h >> 10) & 31;
    uint32_t m = h & 1023u;
    uint32_t bits;
    if (e == 31) bits = sign | 0x7F800000u | (m << 13);
    else if (e != 0) bits = sign | ((uint32_t)(e + 112) << 23) | (m << 13);
    else if (m == 0) bits = sign;
    else {
        e = 113;
        while (!(m & 1024u)) { m <<= 1; e--; }
        bits = sign | ((uint32_t)e << 23) | ((m & 1023u) << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }
inline int nearest(float v) { return (int)std::lrintf(v); }

// src/quant/q8_0.rs:45-61 (round half away from zero)
void quant_q8_0(const float* x, uint8_t* o)
{
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) amax = std::max(amax, std::fabs(x[i]));
    const float d = amax / 127.0f;
    const float inv = d > 0.0f ? 1.0f / d : 0.0f;
    store16(o, to_half(d));
    for (int i = 0; i < 32; i++) {
        float r = std::round(x[i] * inv);
        r = std::min(127.0f, std::max(-127.0f, r));
        o[2 + i] = (uint8_t)(int8_t)r;
    }
}

// w = d*(q-8): d = (value of largest magnitude)/-8, q = min(15, trunc(x/d + 8.5))
void quant_q4_0(const float* x, uint8_t* o)
{
    float amax = 0.0f, vmax = 0.0f;
    for (int i = 0; i < 32; i++)
        if (std::fabs(x[i]) > amax) { amax = std::fabs(x[i]); vmax = x[i]; }
    const float d = vmax / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    store16(o, to_half(d));
    for (int k = 0; k < 16; k++) {
        const int a = std::min(15, (int)(x[k] * id + 8.5f));
        const int b = std::min(15, (int)(x[16 + k] * id + 8.5f));
        o[2 + k] = (uint8_t)(std::max(a, 0) | (std::max(b, 0) << 4));
    }
}

// 12-byte packing of eight 6-bit (scale, min) pairs: inverse of get_scale_min_k4
// (src/quant/q4_k.rs:32-48)
void pack_scales_k4(const uint8_t sc[8], const uint8_t mn[8], uint8_t* q)
{
    std::memset(q, 0, 12);
    for (int j = 0; j < 8; j++) {
        if (j < 4) {
            q[j]     |= sc[j] & 63;
            q[4 + j] |= mn[j] & 63;
        } else {
            q[4 + j] = (uint8_t)((sc[j] & 15) | ((mn[j] & 15) << 4));
            q[j - 4] |= (uint8_t)((sc[j] >> 4) << 6);
            q[j]     |= (uint8_t)((mn[j] >> 4) << 6);
        }
    }
}

// Q4_K (nmax = 15) / Q5_K (nmax = 31): w = d*sc*q - dmin*m, q in [0, nmax]
void quant_q45_k(const float* x, uint8_t* o, int nmax)
{
    float scale[8], mins[8];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int s = 0; s < 8; s++) {
        float lo = x[s * 32], hi = x[s * 32];
        for (int k = 1; k < 32; k++) { lo = std::min(lo, x[s * 32 + k]); hi = std::max(hi, x[s * 32 + k]); }
        lo = std::min(lo, 0.0f);                         // the min term is subtracted, so m >= 0
        scale[s] = (hi - lo) / (float)nmax;
        mins[s]  = -lo;
        max_scale = std::max(max_scale, scale[s]);
        max_min   = std::max(max_min, mins[s]);
    }
    const float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    const float inv_min   = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    uint8_t sc[8], mn[8];
    for (int s = 0; s < 8; s++) {
        sc[s] = (uint8_t)clampi(nearest(inv_scale * scale[s]), 0, 63);
        mn[s] = (uint8_t)clampi(nearest(inv_min * mins[s]), 0, 63);
    }
    const uint16_t dh = to_half(max_scale / 63.0f), dmh = to_half(max_min / 63.0f);
    store16(o, dh);
    store16(o + 2, dmh);
    pack_scales_k4(sc, mn, o + 4);
    const float d = from_half(dh), dmin = from_half(dmh);
    uint8_t q[256];
    for (int s = 0; s < 8; s++) {
        const float ds = d * (float)sc[s], dm = dmin * (float)mn[s];
        for (int k = 0; k < 32; k++)
            q[s * 32 + k] = ds != 0.0f ? (uint8_t)clampi(nearest((x[s * 32 + k] + dm) / ds), 0, nmax) : (uint8_t)0;
    }
    uint8_t* qs = o + (nmax == 31 ? 48 : 16);
    if (nmax == 31) std::memset(o + 16, 0, 32);
    for (int chunk = 0; chunk < 4; chunk++)
        for (int l = 0; l < 32; l++) {
            const uint8_t a = q[chunk * 64 + l], b = q[chunk * 64 + 32 + l];
            qs[chunk * 32 + l] = (uint8_t)((a & 15) | ((b & 15) << 4));
            if (nmax == 31) o[16 + l] |= (uint8_t)(((a >> 4) << (2 * chunk)) | ((b >> 4) << (2 * chunk + 1)));
        }
}

// Q6_K: w = d*sc*(q-32), sixteen 16-weight groups with int8 scales
void quant_q6_k(const float* x, uint8_t* o)
{
    float scales[16];
    float max_abs = 0.0f, max_scale = 0.0f;
    for (int g = 0; g < 16; g++) {
        float amax = 0.0f, vmax = 0.0f;
        for (int k = 0; k < 16; k++)
            if (std::fabs(x[g * 16 + k]) > amax) { amax = std::fabs(x[g * 16 + k]); vmax = x[g * 16 + k]; }
        scales[g] = vmax / -32.0f;                        // largest value maps to -32
        if (std::fabs(scales[g]) > max_abs) { max_abs = std::fabs(scales[g]); max_scale = scales[g]; }
    }
    std::memset(o, 0, 210);
    if (max_abs == 0.0f) return;
    const float iscale = -128.0f / max_scale;
    const uint16_t dh = to_half(1.0f / iscale);
    store16(o + 208, dh);
    const float d = from_half(dh);
    int8_t sc[16];
    uint8_t q[256];
    for (int g = 0; g < 16; g++) {
        sc[g] = (int8_t)std::min(127, nearest(iscale * scales[g]));
        o[192 + g] = (uint8_t)sc[g];
        const float ds = d * (float)sc[g];
        for (int k = 0; k < 16; k++)
            q[g * 16 + k] = ds != 0.0f ? (uint8_t)(clampi(nearest(x[g * 16 + k] / ds), -32, 31) + 32) : (uint8_t)32;
    }
    for (int chunk = 0; chunk < 2; chunk++)
        for (int l = 0; l < 32; l++) {
            const uint8_t q1 = q[chunk * 128 + l], q2 = q[chunk * 128 + 32 + l];
            const uint8_t q3 = q[chunk * 128 + 64 + l], q4 = q[chunk * 128 + 96 + l];
            o[chunk * 64 + l]      = (uint8_t)((q1 & 15) | ((q3 & 15) << 4));
            o[chunk * 64 + 32 + l] = (uint8_t)((q2 & 15) | ((q4 & 15) << 4));
            o[128 + chunk * 32 + l] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
}

const int8_t kIq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

inline int best_iq4nl(float v)
{
    int best = 0;
    float err = std::fabs(v - (float)kIq4nl[0]);
    for (int i = 1; i < 16; i++) {
        const float e = std::fabs(v - (float)kIq4nl[i]);
        if (e < err) { err = e; best = i; }
    }
    return best;
}

// IQ4_XS: w = d*(ls-32)*codebook[q]
void quant_iq4_xs(const float* x, uint8_t* o)
{
    float dl[8];
    float max_abs = 0.0f;
    for (int s = 0; s < 8; s++) {
        float amax = 0.0f, vmax = 0.0f;
        for (int k = 0; k < 32; k++)
            if (std::fabs(x[s * 32 + k]) > amax) { amax = std::fabs(x[s * 32 + k]); vmax = x[s * 32 + k]; }
        dl[s] = vmax / -127.0f;                          // largest value maps to codebook[0]
        max_abs = std::max(max_abs, std::fabs(dl[s]));
    }
    std::memset(o, 0, 136);
    const uint16_t dh = to_half(max_abs / 32.0f);
    store16(o, dh);
    const float d = from_half(dh);
    uint16_t scales_h = 0;
    for (int s = 0; s < 8; s++) {
        const int l = d > 0.0f ? clampi(nearest(dl[s] / d), -32, 31) : 0;
        const int ls = l + 32;
        o[4 + s / 2] |= (uint8_t)((ls & 15) << (4 * (s & 1)));
        scales_h |= (uint16_t)(((ls >> 4) & 3) << (2 * s));
        const float step = d * (float)l;
        const float id = step != 0.0f ? 1.0f / step : 0.0f;
        for (int k = 0; k < 16; k++) {
            const int a = best_iq4nl(x[s * 32 + k] * id), b = best_iq4nl(x[s * 32 + 16 + k] * id);
            o[8 + s * 16 + k] = (uint8_t)(a | (b << 4));
        }
    }
    store16(o + 2, scales_h);
}

void quant_range(int fmt, const float* src, uint8_t* dst, size_t blk_begin, size_t blk_end)
{
    const int bs = rein_block_size(fmt), bb = rein_bytes_per_block(fmt);
    for (size_t i = blk_begin; i < blk_end; i++) {
        const float* x = src + i * (size_t)bs;
        uint8_t* o = dst + i * (size_t)bb;
        switch (fmt) {
        case REIN_TYPE_Q8_0:   quant_q8_0(x, o); break;
        case REIN_TYPE_Q4_0:   quant_q4_0(x, o); break;
        case REIN_TYPE_Q4_K:   quant_q45_k(x, o, 15); break;
        case REIN_TYPE_Q5_K:   quant_q45_k(x, o, 31); break;
        case REIN_TYPE_Q6_K:   quant_q6_k(x, o); break;
        case REIN_TYPE_IQ4_XS: quant_iq4_xs(x, o); break;
        }
    }
}

}  // namespace

extern "C" int rein_quantize_weights(int fmt, const float* src, size_t n, uint8_t* dst)
{
    const int bs = rein_block_size(fmt);
    if (!bs) return rein::fail(REIN_E_BAD_FORMAT, "rein_quantize_weights: unknown format " + std::to_string(fmt));
    if (n % (size_t)bs) return rein::fail(REIN_E_BAD_SHAPE, "rein_quantize_weights: n must be a multiple of " + std::to_string(bs));
    if (!src || !dst) return rein::fail(REIN_E_BAD_POINTER, "rein_quantize_weights: null pointer");
    const size_t n_blk = n / (size_t)bs;
    size_t n_threads = std::min<size_t>(std::max(1u, std::thread::hardware_concurrency()), 16);
    if (n < ((size_t)1 << 20)) n_threads = 1;
    if (n_threads <= 1) {
        quant_range(fmt, src, dst, 0, n_blk);
        return 0;
    }
    std::vector<std::thread> pool;
    const size_t step = (n_blk + n_threads - 1) / n_threads;
    for (size_t t = 0; t < n_threads; t++) {
        const size_t a = t * step, b = std::min(n_blk, a + step);
        if (a >= b) break;
        pool.emplace_back(quant_range, fmt, src, dst, a, b);
    }
    for (auto& th : pool) th.join();
    return 0;
}
