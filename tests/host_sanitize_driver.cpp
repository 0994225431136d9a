// Driver for tests/test_host_sanitized.py: the host library's load-time code (repacks of
// every format at ragged shapes, the synthetic quantizers, the ingestion of relabelled
// types, a small GGUF container) on exactly-sized heap buffers, built with AddressSanitizer
// and UndefinedBehaviorSanitizer.  Host code only; nothing here touches a GPU.
#include "../include/rein.h"
#include <cstdio>
#include <cstdlib>
#include <vector>
#include <random>
#include <cstring>
int main() {
    std::mt19937 rng(1);
    int fmts[] = {2, 8, 12, 13, 14, 23, 7, 21};
    int n_ok = 0;
    for (int fmt : fmts) {
        int bs = rein_block_size(fmt), bb = rein_bytes_per_block(fmt);
        for (size_t in_dim : {(size_t)bs, (size_t)bs * 2, (size_t)bs * 3, (size_t)256 * 4, (size_t)256 * 5 + (bs == 32 ? 96 : 0), (size_t)4096}) {
            for (size_t out_dim : {(size_t)1, (size_t)3, (size_t)17, (size_t)1100}) {
                if (in_dim * out_dim > (1u << 23)) continue;
                size_t src_len = in_dim * out_dim / bs * bb;
                uint8_t* src = (uint8_t*)malloc(src_len);           // exact size: ASan sees overreads
                for (size_t i = 0; i < src_len; i++) src[i] = (uint8_t)rng();
                size_t dl = rein_repacked_len(fmt, in_dim, out_dim);
                uint8_t* dst = (uint8_t*)malloc(dl);
                int rc = rein_repack_for_matvec(fmt, src, in_dim, out_dim, dst);
                if (rc) { printf("repack fmt %d %zu %zu rc %d %s\n", fmt, in_dim, out_dim, rc, rein_last_error()); return 1; }
                n_ok++;
                free(src); free(dst);
            }
        }
        // weight quantizer
        if (fmt != 7 && fmt != 21) {
            size_t n = 256 * 37;
            std::vector<float> w(n);
            for (auto& v : w) v = (float)((int)(rng() % 2001) - 1000) * 1e-4f;
            w[5] = 0.0f; w[300] = 1e30f; w[700] = -1e-30f;
            uint8_t* dst = (uint8_t*)malloc(n / bs * bb);
            int rc = rein_quantize_weights(fmt, w.data(), n, dst);
            if (rc) { printf("quantize fmt %d rc %d\n", fmt, rc); return 1; }
            free(dst);
        }
    }
    // ingestion of relabelled types
    for (int ty : {11, 20, 30, 21}) {
        size_t in_dim = 512, out_dim = 9;
        size_t sl = rein_ingest_src_len(ty, in_dim, out_dim);
        uint8_t* src = (uint8_t*)malloc(sl);
        for (size_t i = 0; i < sl; i++) src[i] = (uint8_t)rng();
        int label = rein_ingest_format(ty);
        size_t dl = rein_repacked_len(label, in_dim, out_dim);
        uint8_t* dst = (uint8_t*)malloc(dl);
        int fmt = 0;
        int rc = rein_ingest_for_matvec(ty, src, in_dim, out_dim, dst, &fmt);
        if (rc || fmt != label) { printf("ingest ty %d rc %d\n", ty, rc); return 1; }
        free(src); free(dst);
        n_ok++;
    }
    // a small container: header, one string entry, one Q8_0 tensor; then every truncation of it
    {
        std::vector<uint8_t> f;
        auto put = [&](const void* p, size_t n) { f.insert(f.end(), (const uint8_t*)p, (const uint8_t*)p + n); };
        auto u32 = [&](uint32_t v) { put(&v, 4); };
        auto u64 = [&](uint64_t v) { put(&v, 8); };
        auto str = [&](const char* s) { u64(strlen(s)); put(s, strlen(s)); };
        put("GGUF", 4); u32(3); u64(1); u64(1);
        str("general.architecture"); u32(8); str("qwen35");
        str("w"); u32(2); u64(64); u64(2); u32(8); u64(0);
        while (f.size() % 32) f.push_back(0);
        for (int i = 0; i < 4 * 34; i++) f.push_back((uint8_t)rng());
        for (size_t cut = 0; cut <= f.size(); cut++) {
            uint8_t* p = (uint8_t*)malloc(cut ? cut : 1);
            memcpy(p, f.data(), cut);
            rein_gguf* g = nullptr;
            const int rc = rein_gguf_from_bytes(p, cut, &g);
            if ((rc == 0) != (cut == f.size())) { printf("gguf cut %zu rc %d\n", cut, rc); return 1; }
            if (g) {
                rein_gguf_dims d; int fmt = 0;
                std::vector<uint8_t> dst(rein_repacked_len(8, 64, 2));
                if (rein_gguf_load_for_matvec(g, "w", dst.data(), dst.size(), &fmt, &d) || fmt != 8) { printf("gguf load\n"); return 1; }
                rein_gguf_close(g);
                n_ok++;
            }
            free(p);
        }
    }
    // argument errors never touch memory
    rein_repack_for_matvec(12, nullptr, 256, 1, nullptr);
    rein_repack_for_matvec(12, (const uint8_t*)"", 100, 1, (uint8_t*)"");
    rein_ingest_for_matvec(99, nullptr, 0, 0, nullptr, nullptr);
    printf("ok %d\n", n_ok);
}
