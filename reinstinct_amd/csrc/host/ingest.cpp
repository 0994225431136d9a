// Load-time ingestion of GGUF tensor bytes into the repacked layouts the kernels read:
// the dispatch of GpuMatvecTensor::from_bytes_matvec (src/runtime/qwen35.rs:251-331).
// Six formats repack as they are; three more are RELABELLED onto a layout that has
// kernels, without rounding (IQ4_NL, Q3_K) or with one Q8_0 quantization step (BF16):
//
//   IQ4_NL (18-byte blocks {f16 d, 16 nibble bytes})   -> IQ4_XS planes: the nibble bytes
//            verbatim, the fp16 scale verbatim (src/quant/iq4_nl.rs:52-75).  The block is
//            byte-compatible with Q4_0's, so the Q4_0 repack does the move.
//   Q3_K   (110-byte blocks)  -> Q6_K blocks with q6 = q3 + 28 and sc6 = sc3 - 32, the
//            same d: w = d * sc6 * (q6 - 32) = d * (sc3 - 32) * (q3 - 4) factor for
//            factor (src/quant/q3_k.rs:85-122), then the Q6_K repack.
//   BF16   -> f32 (high half of the word) -> Q8_0 blocks (src/quant/q8_0.rs:45-61) -> Q8_0 repack.
//
// IQ3_S repacks onto the IQ4_XS planes under its own format id (the kernels differ in the
// codebook).  Q5_1 is an expert-tensor format only (rein_ingest_expert_format), as in the
// reference, where a dense Q5_1 tensor stays in its on-disk layout.
#include <cstring>
#include <string>
#include <vector>

#include "../../../include/rein.h"
#include "hip_api.h"

namespace {

constexpr size_t kQ3kBytes = 110, kQ6kBytes = 210;

// the sixteen 6-bit scales of a Q3_K block: scale k = 4i + j has its low nibble in
// byte 4(i & 1) + j (upper nibble for i >= 2) and its two high bits in byte 8 + j at 2i
inline int q3k_scale(const uint8_t* scales, int k)
{
    const int i = k >> 2, j = k & 3;
    const int lo = i < 2 ? (scales[4 * i + j] & 0x0F) : (scales[4 * (i - 2) + j] >> 4);
    const int hi = (scales[8 + j] >> (2 * i)) & 3;
    return lo | (hi << 4);
}

// stored 3-bit quant of weight y (0..255): low two bits from qs, third bit from hmask.
// The weight is d * (sc - 32) * (q3 - 4): hmask bit set means "no -4".
inline int q3k_quant(const uint8_t* hmask, const uint8_t* qs, int y)
{
    const int n = y >> 7, s = (y >> 5) & 3, l = y & 31;
    const int lo = (qs[32 * n + l] >> (2 * s)) & 3;
    const int hi = (hmask[l] >> (4 * n + s)) & 1;
    return lo | (hi << 2);
}

void q3k_block_to_q6k(const uint8_t* src, uint8_t* dst)
{
    const uint8_t* hmask = src;
    const uint8_t* qs = src + 32;
    const uint8_t* scales = src + 96;
    uint8_t* ql = dst;
    uint8_t* qh = dst + 128;
    int8_t* sc6 = reinterpret_cast<int8_t*>(dst + 192);
    std::memset(dst, 0, 192);
    for (int k = 0; k < 16; k++) sc6[k] = (int8_t)(q3k_scale(scales, k) - 32);
    for (int y = 0; y < 256; y++) {
        const int q6 = q3k_quant(hmask, qs, y) + 28;
        // Q6_K placement of weight y (src/quant/q6_k.rs:31-69): half n, group g of 32, lane l
        const int n = y >> 7, g = (y >> 5) & 3, l = y & 31;
        ql[64 * n + 32 * (g & 1) + l] |= (uint8_t)((q6 & 0x0F) << (4 * (g >> 1)));
        qh[32 * n + l] |= (uint8_t)((q6 >> 4) << (2 * g));
    }
    dst[208] = src[108];
    dst[209] = src[109];
}

int label_of(int ggml_type)
{
    switch (ggml_type) {
    case REIN_TYPE_Q4_0: case REIN_TYPE_Q8_0: case REIN_TYPE_Q4_K: case REIN_TYPE_Q5_K: case REIN_TYPE_Q6_K:
    case REIN_TYPE_IQ4_XS: case REIN_TYPE_IQ3_S: return ggml_type;
    case REIN_GGML_IQ4_NL: return REIN_TYPE_IQ4_XS;
    case REIN_GGML_Q3_K:   return REIN_TYPE_Q6_K;
    case REIN_GGML_BF16:   return REIN_TYPE_Q8_0;
    default: return 0;
    }
}

}  // namespace

extern "C" int rein_ingest_format(int ggml_type) { return label_of(ggml_type); }

// the types GpuExpertTensor::from_gguf repacks (src/runtime/qwen35.rs:415-425)
extern "C" int rein_ingest_expert_format(int ggml_type)
{
    switch (ggml_type) {
    case REIN_TYPE_Q4_K: case REIN_TYPE_Q5_K: case REIN_TYPE_Q6_K: case REIN_TYPE_Q8_0: case REIN_TYPE_Q5_1: return ggml_type;
    default: return 0;
    }
}

extern "C" size_t rein_ingest_src_len(int ggml_type, size_t in_dim, size_t out_dim)
{
    const size_t n = in_dim * out_dim;
    switch (ggml_type) {
    case REIN_GGML_IQ4_NL: return n / 32 * 18;
    case REIN_GGML_Q3_K:   return n / 256 * kQ3kBytes;
    case REIN_GGML_BF16:   return n * 2;
    default: {
        const int bs = rein_block_size(ggml_type);
        return bs ? n / (size_t)bs * (size_t)rein_bytes_per_block(ggml_type) : 0;
    }
    }
}

extern "C" int rein_transcode_q3_k_to_q6_k(const uint8_t* src, size_t n_weights, uint8_t* dst)
{
    if (!src || !dst) return rein::fail(REIN_E_BAD_POINTER, "rein_transcode_q3_k_to_q6_k: null pointer");
    if (n_weights == 0 || n_weights % 256) return rein::fail(REIN_E_BAD_SHAPE, "rein_transcode_q3_k_to_q6_k: n_weights must be a non-zero multiple of 256");
    for (size_t b = 0; b < n_weights / 256; b++) q3k_block_to_q6k(src + b * kQ3kBytes, dst + b * kQ6kBytes);
    return 0;
}

extern "C" int rein_ingest_for_matvec(int ggml_type, const uint8_t* src, size_t in_dim, size_t out_dim, uint8_t* dst,
                                      int* out_fmt)
{
    const char* who = "rein_ingest_for_matvec";
    const int label = label_of(ggml_type);
    if (!label)
        return rein::fail(REIN_E_BAD_FORMAT, std::string(who) + ": no repacked layout for ggml type " + std::to_string(ggml_type) +
                                             " (handled: Q4_0, Q8_0, Q3_K, Q4_K, Q5_K, Q6_K, IQ3_S, IQ4_NL, IQ4_XS, BF16)");
    if (!src || !dst) return rein::fail(REIN_E_BAD_POINTER, std::string(who) + ": null pointer");
    if (out_fmt) *out_fmt = label;
    if (label == ggml_type) return rein_repack_for_matvec(ggml_type, src, in_dim, out_dim, dst);
    if (in_dim == 0 || out_dim == 0) return rein::fail(REIN_E_BAD_SHAPE, std::string(who) + ": zero dimension");
    switch (ggml_type) {
    case REIN_GGML_IQ4_NL:
        // {f16 d, 16 nibble bytes}: Q4_0's block, Q4_0's planes; only the kernels' codebook differs
        return rein_repack_for_matvec(REIN_TYPE_Q4_0, src, in_dim, out_dim, dst);
    case REIN_GGML_Q3_K: {
        if (in_dim % 256) return rein::fail(REIN_E_BAD_SHAPE, std::string(who) + ": Q3_K in_dim must be a multiple of 256");
        std::vector<uint8_t> q6(in_dim * out_dim / 256 * kQ6kBytes);
        if (int rc = rein_transcode_q3_k_to_q6_k(src, in_dim * out_dim, q6.data())) return rc;
        return rein_repack_for_matvec(REIN_TYPE_Q6_K, q6.data(), in_dim, out_dim, dst);
    }
    case REIN_GGML_BF16: {
        if (in_dim % 32) return rein::fail(REIN_E_BAD_SHAPE, std::string(who) + ": BF16 in_dim must be a multiple of 32");
        const size_t n = in_dim * out_dim;
        std::vector<float> f(n);
        for (size_t i = 0; i < n; i++) {
            const uint32_t bits = (uint32_t)(src[2 * i] | (src[2 * i + 1] << 8)) << 16;
            std::memcpy(&f[i], &bits, 4);
        }
        std::vector<uint8_t> q8(n / 32 * 34);
        if (int rc = rein_quantize_weights(REIN_TYPE_Q8_0, f.data(), n, q8.data())) return rc;
        return rein_repack_for_matvec(REIN_TYPE_Q8_0, q8.data(), in_dim, out_dim, dst);
    }
    default: return rein::fail(REIN_E_BAD_FORMAT, std::string(who) + ": unreachable");
    }
}
