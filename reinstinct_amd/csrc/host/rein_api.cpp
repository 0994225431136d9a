// librein C ABI: runtime (dlopen'd HIP, code-object loading, kernel lookup by
// name) and the host-side dispatch of the quantized matmul path.  Mirrors the
// reference's src/hip (module / launch surface) and the launch sites in
// src/runtime/{qwen35,prefill}.rs; geometry is chosen here for MI355X
// (256 CUs, wave64) instead of being fixed per kernel.
#include <dlfcn.h>

#include <cmath>
#include <cstdlib>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <algorithm>
#include <atomic>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../../include/rein.h"
#include "hip_api.h"

using namespace rein;

namespace {

struct Runtime {
    const HipApi* api = nullptr;
    hipModule_t   module = nullptr;
    std::mutex    mu;
    std::unordered_map<std::string, hipFunction_t> fns;
    bool loaded = false;
};

Runtime g_rt;
std::mutex g_init_mu;

std::string default_hsaco_path()
{
    Dl_info info;
    if (dladdr(reinterpret_cast<const void*>(&default_hsaco_path), &info) && info.dli_fname) {
        std::string p(info.dli_fname);
        const size_t slash = p.find_last_of('/');
        const std::string dir = slash == std::string::npos ? std::string(".") : p.substr(0, slash);
        return dir + "/rein_gfx950.hsaco";
    }
    return "rein_gfx950.hsaco";
}

int need_api(const HipApi** out)
{
    std::string err;
    const HipApi* api = hip_api(&err);
    if (!api) return fail(REIN_E_NOT_LOADED, err);
    *out = api;
    return 0;
}

int need_runtime()
{
    if (!g_rt.loaded) return fail(REIN_E_NOT_LOADED, "librein: rein_init has not succeeded; no CPU fallback exists");
    return 0;
}

int get_fn(const std::string& name, hipFunction_t* f)
{
    if (int rc = need_runtime()) return rc;
    std::lock_guard<std::mutex> lock(g_rt.mu);
    auto it = g_rt.fns.find(name);
    if (it != g_rt.fns.end()) {
        *f = it->second;
        return 0;
    }
    hipFunction_t fn = nullptr;
    const hipError_t e = g_rt.api->ModuleGetFunction(&fn, g_rt.module, name.c_str());
    if (e != 0) {
        check_hip(g_rt.api, e, ("hipModuleGetFunction(" + name + ")").c_str());
        return REIN_E_NO_KERNEL;
    }
    g_rt.fns.emplace(name, fn);
    *f = fn;
    return 0;
}

int launch(const std::string& name, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned shmem,
           rein_stream_t s, void** args)
{
    hipFunction_t f;
    if (int rc = get_fn(name, &f)) return rc;
    return check_hip(g_rt.api, g_rt.api->ModuleLaunchKernel(f, gx, gy, gz, bx, 1, 1, shmem, s, args, nullptr),
                     ("hipModuleLaunchKernel(" + name + ")").c_str());
}

const char* fmt_tag(int fmt)
{
    switch (fmt) {
    case REIN_TYPE_Q4_0:   return "q4_0";
    case REIN_TYPE_Q8_0:   return "q8_0";
    case REIN_TYPE_Q4_K:   return "q4k";
    case REIN_TYPE_Q5_K:   return "q5k";
    case REIN_TYPE_Q6_K:   return "q6k";
    case REIN_TYPE_IQ4_XS: return "iq4xs";
    case REIN_TYPE_Q5_1:   return "q5_1";
    case REIN_TYPE_IQ3_S:  return "iq3s";
    default: return nullptr;
    }
}

int check_shape(const char* who, int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows)
{
    const int bs = rein_block_size(fmt);
    if (!bs) return fail(REIN_E_BAD_FORMAT, std::string(who) + ": unknown format " + std::to_string(fmt));
    if (in_dim == 0 || in_dim % (unsigned)bs != 0)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": in_dim " + std::to_string(in_dim) + " is not a non-zero multiple of " + std::to_string(bs));
    if (out_dim == 0 || n_rows == 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": out_dim and the row count must be non-zero");
    return 0;
}

// Q5_1 has expert kernels only and IQ3_S dense kernels only (src/runtime/qwen35.rs:2264,3045,
// 3082,3116 are every site the reference dispatches them at).
int check_dense_fmt(const char* who, int fmt)
{
    if (fmt == REIN_TYPE_Q5_1)
        return fail(REIN_E_BAD_FORMAT, std::string(who) + ": Q5_1 has MoE expert kernels only (a dense Q5_1 tensor keeps its on-disk layout)");
    return 0;
}

int check_ptr(const char* who, const void* p, size_t align, const char* what)
{
    if (!p) return fail(REIN_E_BAD_POINTER, std::string(who) + ": " + what + " is NULL");
    if (reinterpret_cast<uintptr_t>(p) % align != 0)
        return fail(REIN_E_BAD_POINTER, std::string(who) + ": " + what + " must be " + std::to_string(align) + "-byte aligned");
    return 0;
}

// ---- options ---------------------------------------------------------------------------------
// Every switch that forces a launch choice (the tests use them to reach each kernel family; a host
// may pin a choice it has measured) lives in this one table.  An option is either unset -- the
// library decides -- or set to a number.  The environment variables of the same names are read
// once per process, on the first look at the table (rein_init does one); afterwards only
// rein_set_option changes an entry, so the launch an entry point chooses depends on its arguments
// and on this table alone.  Entries are single atomic words: setting one while another thread
// launches is safe, the launch sees the old or the new value.
enum Opt : int { O_MV_ROWS, O_MV_WPB, O_MV_LDS, O_QUAD_LDS, O_QUAD_SLICES, O_QUAD_DEPTH, O_QUAD_WIDE32, O_SKINNY_KS, O_SKINNY_FROM, O_QUAD_FROM, O_GROUPED_STRIDED, O_MMQ_TM, O_MMQ_N64, O_MMQ6, O_MMQ6_N4, O_MMQ6_N2, O_MMQ6_SK_GRID, O_MMQ6_SK_SPLIT, O_MMQ6_SK, O_MMQ6_FROM, O_MMQ_SK, O_MMQ_SK_GRID, O_MMQ_SK_SPLIT, O_MMQ_SK_TM, O_MMQ16, O_TOPK_WAVE, O_MOE_SORT_SPLIT, O_MOE_GU_ROWS, O_MOE_DC_ROWS, O_MOE_CHAIN, O_MOE_FUSED, O_COUNT };
const char* const kOptNames[O_COUNT] = {"REIN_MV_ROWS", "REIN_MV_WPB", "REIN_MV_LDS", "REIN_QUAD_LDS", "REIN_QUAD_SLICES", "REIN_QUAD_DEPTH", "REIN_QUAD_WIDE32", "REIN_SKINNY_KS", "REIN_SKINNY_FROM", "REIN_QUAD_FROM", "REIN_GROUPED_STRIDED", "REIN_MMQ_TM", "REIN_MMQ_N64", "REIN_MMQ6", "REIN_MMQ6_N4", "REIN_MMQ6_N2", "REIN_MMQ6_SK_GRID", "REIN_MMQ6_SK_SPLIT", "REIN_MMQ6_SK", "REIN_MMQ6_FROM", "REIN_MMQ_SK", "REIN_MMQ_SK_GRID", "REIN_MMQ_SK_SPLIT", "REIN_MMQ_SK_TM", "REIN_MMQ16", "REIN_TOPK_WAVE", "REIN_MOE_SORT_SPLIT", "REIN_MOE_GU_ROWS", "REIN_MOE_DC_ROWS", "REIN_MOE_CHAIN", "REIN_MOE_FUSED"};
constexpr uint64_t kOptSet = 1ull << 63;
std::atomic<uint64_t> g_opts[O_COUNT];          // zero = unset
std::once_flag g_opts_env_once;

void opts_from_env()
{
    for (int i = 0; i < O_COUNT; i++) {
        const char* v = std::getenv(kOptNames[i]);
        if (v && *v) g_opts[i].store(kOptSet | (uint32_t)std::strtoul(v, nullptr, 10), std::memory_order_relaxed);
    }
}

uint64_t opt_raw(Opt id)
{
    std::call_once(g_opts_env_once, opts_from_env);
    return g_opts[id].load(std::memory_order_relaxed);
}
// the option's value, or dflt while it is unset
unsigned opt_u(Opt id, unsigned dflt)
{
    const uint64_t r = opt_raw(id);
    return (r & kOptSet) ? (unsigned)(r & 0xFFFFFFFFull) : dflt;
}
// whether the option has been set (a set option pins a choice; several cost models step aside then)
bool opt_is_set(Opt id) { return (opt_raw(id) & kOptSet) != 0; }

constexpr unsigned kCUs = 256;    // MI355X

// Rows per wavefront pass for the decode matvec.  More rows per wave amortise
// the activation read and the cross-lane reduction; fewer rows put more waves in
// flight.  Measured on MI355X (Q4_K, batch 1): 4 rows win once that still leaves
// ~32 waves per CU (N = 34816), 2 rows down to ~8 waves per CU (N = 5120), 1 row
// below that.
unsigned pick_rows_per_wave(int fmt, unsigned out_dim, unsigned batch)
{
    const unsigned forced = opt_u(O_MV_ROWS, 0);
    unsigned r = 1;
    if ((out_dim + 3) / 4 >= kCUs * 32) r = 4;
    else if ((out_dim + 1) / 2 >= kCUs * 8) r = 2;
    // Per-format corrections, measured at 5120 -> 34816, 5120 -> 5120 and 17408 -> 5120: the
    // formats with the most work per sub-block run out of issue slots before bandwidth, and
    // there fewer rows per wave (more waves) or more rows (fewer activation reads) can win.
    if ((fmt == REIN_TYPE_Q4_K || fmt == REIN_TYPE_Q4_0) && batch == 1 && out_dim >= 7168) r = 4;   // 7168 rows: 7.6 -> 7.1 us, 16384: 12.4 -> 11.8
    if (fmt == REIN_TYPE_Q8_0 && r == 4 && batch <= 2) r = 2;        // 34.9 -> 32.3 us (b1), 43.1 -> 37.0 (b2)
    if (fmt == REIN_TYPE_Q6_K && r == 4 && batch == 2) r = 2;        // 48.1 -> 38.6 us
    if (fmt == REIN_TYPE_Q6_K && r == 2 && batch == 4) r = 1;        // 15.8 -> 14.0, 42.7 -> 39.4 us
    if (fmt == REIN_TYPE_Q5_K && r == 2 && batch == 4) r = 4;        // 13.9 -> 12.9, 39.2 -> 32.1 us
    if (forced == 1 || forced == 2 || forced == 4) r = forced;
    while (r > 1 && r * batch > 16) r >>= 1;
    return r;
}

unsigned batch_slot(unsigned n_rows) { return n_rows <= 1 ? 1 : n_rows <= 2 ? 2 : n_rows <= 4 ? 4 : 8; }

// Wavefronts per workgroup of the dot4 matvec (they share nothing): four, or two where the finer grain deals the
// wavefronts more evenly over the CUs -- every format at two activation rows (Q4_K 17408 -> 5120: 18.5 -> 15.4 us,
// 5120 -> 5120: 7.5 -> 6.7; IQ3_S 16.4 -> 14.5), Q8_0 also at one (19.8 -> 17.1, 7.1 -> 6.5), and one to three percent for
// Q4_K / Q5_K at one row; Q4_0, IQ4_XS and IQ3_S at one row lose 3-10 % on 5120 -> 5120 and stay at four.
// The workgroups of a launch this short are all resident at once, so a CU that holds three workgroups of four
// wavefronts beside CUs that hold two ends 20 % late (5120 rows at two rows per wavefront: 640 workgroups of four, 1280
// of two).  At one row the pairs are taken only where they even the deal out by more than 3 %; otherwise four wavefronts
// halve the workgroups to start (us, two -> four: Q4_K 2048 -> 5632 4.17 -> 3.58, 4096 -> 6144 5.44 -> 4.94, 16384 -> 6144
// 13.9 -> 12.9; Q5_K 4.44 -> 3.85, 6.24 -> 5.68; Q8_0 4.62 -> 4.18; 48 cells of three formats x 16 shapes then sit within
// 3 % of the better of the two).
unsigned pick_wpb(int fmt, unsigned groups, unsigned b)
{
    const unsigned forced = opt_u(O_MV_WPB, 0);
    if (forced == 1 || forced == 2 || forced == 4) return forced;
    const auto uneven = [&](unsigned w) { const unsigned n = (groups + w - 1) / w; return (double)((n + kCUs - 1) / kCUs * kCUs) / n; };
    unsigned wpb = 4;
    if (b == 2 || (fmt == REIN_TYPE_Q8_0 && b <= 2) || (b == 1 && (fmt == REIN_TYPE_Q4_K || fmt == REIN_TYPE_Q5_K))) wpb = 2;
    if (wpb == 2 && b == 1 && !(uneven(2) < uneven(4) - 0.03)) wpb = 4;
    return wpb;
}

// Skinny MMQ launch: grid.x = 32-row tiles, grid.y = token groups, block = KS
// wavefronts that split the contraction of one tile.  The kernels keep several
// chunks of weights in flight in registers, which leaves room for two or three
// wavefronts per SIMD (the table below mirrors the kernels' register budgets).
// Measured on MI355X (Q4_K): a wavefront alone on its SIMD takes 1.5 us per chunk;
// m >= 2 wavefronts sharing a SIMD take 1.14 us x m each (the SIMD is then busy).
// KS is chosen by that model: when every wavefront is resident at once the fullest
// SIMD sets the time; otherwise the work streams through the slots and the last
// workgroups run underoccupied.
int launch_skinny(int fmt, const void* w, const void* xq, float* y, unsigned in_dim, unsigned out_dim,
                  unsigned n_rows, rein_stream_t s)
{
    const unsigned nv = n_rows <= 2 ? 1 : n_rows <= 4 ? 2 : n_rows <= 8 ? 4 : 8, tok = 2 * nv;
    const unsigned tiles = ((out_dim + 31) / 32) * ((n_rows + tok - 1) / tok);
    const unsigned n_chunks = (in_dim / 32 + 7) / 8;
    const unsigned planes = fmt == REIN_TYPE_Q8_0 ? 2 : 1;
    const unsigned lds_per_wave = planes * 4096 + 320 * tok;                       // sizeof(SkinnyWaveLds<FMT, TOK>)
    const bool three = nv <= 4 && (fmt == REIN_TYPE_Q4_0 || fmt == REIN_TYPE_Q4_K || fmt == REIN_TYPE_Q8_0 ||
                                   fmt == REIN_TYPE_IQ4_XS || fmt == REIN_TYPE_IQ3_S);
    const unsigned occ = three ? 3 : 2;                                            // wavefronts per SIMD (registers)
    const unsigned waves_per_cu = std::min(4 * occ, 160u * 1024u / lds_per_wave);
    const unsigned ks_max = std::min(std::min(8u, waves_per_cu), n_chunks);        // the kernels' launch bound is 512 threads
    unsigned ks = 1;
    double best = 1e30;
    for (unsigned k = 1; k <= ks_max; k++) {
        const unsigned wg_per_cu = waves_per_cu / k;
        const double waves = (double)tiles * k, slots = (double)kCUs * wg_per_cu * k;
        const double per_wave = (n_chunks + k - 1) / k + 2.0;                      // chunks, plus pipeline fill and the reduction
        double cost;
        if (waves <= slots) {
            const double m = std::ceil(waves / (kCUs * 4.0));
            cost = per_wave * std::max(1.5, 1.14 * m);
        } else {
            cost = waves * per_wave / (kCUs * 4.0) * 1.14 + 0.5 * per_wave * 1.5;
        }
        if (cost < best) { best = cost; ks = k; }
    }
    // Measured correction for the two-wavefronts-per-SIMD kernels (Q5_K, Q6_K) at 5-8 rows against many row
    // tiles: four wavefronts per tile, i.e. two tiles per CU at a time, beat the model's two (Q5_K 5120 -> 34816
    // at 8 rows: 46.6 -> 41.0 us, Q6_K 58.8 -> 52.8; 2 / 4 / 8 wavefronts: 46.6 / 41.0 / 56.5)
    if (occ == 2 && nv == 4 && tiles >= 1024 && ks < 4 && ks_max >= 4) ks = 4;
    const unsigned forced = opt_u(O_SKINNY_KS, 0);
    if (forced >= 1 && forced <= ks_max) ks = forced;
    const std::string name = std::string("rein_mmqs_") + fmt_tag(fmt) + "_v" + std::to_string(nv);
    void* args[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&n_rows};
    return launch(name, (out_dim + 31) / 32, (n_rows + tok - 1) / tok, 1, ks * 64, ks * lds_per_wave, s, args);
}

// Activation rows from which the batched decode leaves the dot4 kernels for the
// skinny MMQ.  Every extra row is eight more v_dot4 and one more fp32 term per sub-block
// and lane, which costs the dot4 kernels ~7 us at 5120 -> 34816 (Q4_K: 21 / 28 / 39 us at 1 / 2 / 3-4
// rows) while the skinny MMQ takes 27 / 30 / 33 us for up to 2 / 4 / 8 rows.  Two rows
// stay on dot4 (level at large N, faster at small N).  Q6_K would switch at 5 (two MFMAs and
// the most aux words per sub-block), but use_quad sends its 3+ rows elsewhere first.
unsigned skinny_from_rows(int fmt)
{
    unsigned dflt = 3;
    if (fmt == REIN_TYPE_Q6_K) dflt = 5;
    return opt_u(O_SKINNY_FROM, dflt);
}

// Whether a batched decode of n_rows (<= 8) activation rows runs on the 4x4x4 int8 matrix
// instruction (rein_mvq_*: four weight rows x four activation rows per instruction chain,
// every weight sub-block unpacked once).  From one run of all three kernel families at
// 5120 -> 34816, 5120 -> 5120 and 17408 -> 5120 (us, best of dot4 / skinny MMQ -> this):
//   Q6_K    3..8 rows everywhere           3-4 rows: 58.3 -> 40.5, 13.8 -> 13.2, 38.7 -> 37.5
//                                          5-8 rows: 63.6 -> 58.2, 18.2 -> 15.5, 44.5 -> 43.0
//   Q5_K    3..4 rows everywhere           43.6 -> 37.4, 12.6 -> 10.1, 29.8 -> 27.8
//           5..8 rows below 16384 rows     13.2 -> 12.0, 31.8 -> 31.7 (34816 rows: 46.7 vs 50.8, stays)
//   IQ4_XS  3..4 rows everywhere           34.1 -> 31.1, 13.1 -> 10.1, 31.9 -> 25.7
//           5..8 rows below 16384 rows     13.3 -> 12.4, 32.4 -> 32.3 (34816 rows: 35.3 vs 45.6, stays)
// The formats with a cheap unpack (Q4_K, Q4_0, Q8_0, IQ3_S) stay on dot4 / skinny MMQ
// (Q4_K 4 rows at 34816 output rows: skinny 29.6, this 34.3).
// ... except at 3-4 rows against 8192-20480 output rows, where the skinny MMQ's 32-row tiles do not fill the
// machine as evenly as four-row groups do (us, skinny -> this: Q4_K 4096 -> 14336 17.7 -> 14.0, 5120 -> 17408 21.8 ->
// 19.4, 8192 -> 8192 19.7 -> 17.0; Q4_0 17.0 -> 13.1, 21.1 -> 17.4, 18.4 -> 17.2; Q8_0 23.0 -> 21.0, 25.9 -> 25.6, 25.5 ->
// 21.3; level at 7168 rows, behind at 5120 and 34816).
bool use_quad(int fmt, unsigned out_dim, unsigned n_rows)
{
    const unsigned forced = opt_u(O_QUAD_FROM, 0);
    if (forced) return n_rows >= forced;
    if (n_rows < 3) return false;
    switch (fmt) {
    case REIN_TYPE_Q6_K:   return true;
    case REIN_TYPE_Q5_K:
    case REIN_TYPE_IQ4_XS: return n_rows <= 4 || out_dim < 16384;
    case REIN_TYPE_Q4_K:
    case REIN_TYPE_Q4_0:
    case REIN_TYPE_Q8_0:   return n_rows <= 4 && out_dim >= 8192 && out_dim <= 20480;
    default:               return false;
    }
}

// Small matrices stay on dot4 at every row count: the matrix-core kernels hand out 32-row tiles or 16-row
// workgroups, too few of them for 256 CUs, and carry a pipeline fill that a 5 us launch does not earn back.
// One run of all kernel families over 12 shapes x 6 formats (us, matrix-core choice -> dot4): 5120 -> 1024 at 3-4
// rows Q4_K 8.6 -> 4.8, Q8_0 9.1 -> 5.2, Q5_K 8.4 -> 5.6, IQ4_XS 8.5 -> 4.9, Q6_K 10.8 -> 7.9; 5120 -> 2048 8.8 -> 6.3
// ... 11.2 -> 9.7; 2048 -> 1536 6.0 -> 3.5.  Beyond 2048 output rows only the formats of the skinny MMQ gain, up to
// 2^24 weights (4096 -> 4096 Q4_K 9.0 -> 7.1, Q8_0 11.0 -> 8.6; 2048 -> 5120 6.5 -> 5.5; 5120 -> 5120: 9.8 against
// 11.6, stays), the 4x4x4 kernel of the others is level there (Q5_K 2048 -> 5120 5.8 = 5.8).  At 5-8 rows dot4 is
// ahead up to about six million weights (5120 -> 1024 Q4_K 9.5 -> 7.7, Q5_K 9.8 -> 6.8; 2048 -> 1536 6.2 -> 5.1;
// 5120 -> 2048 9.7 against 10.7, stays).
bool small_for_matrix_cores(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows)
{
    if (n_rows < 3 || opt_is_set(O_QUAD_FROM) || opt_is_set(O_SKINNY_FROM)) return false;
    const unsigned long long weights = (unsigned long long)in_dim * out_dim;
    if (n_rows > 4) return weights <= (6ull << 20);
    const bool quad_family = fmt == REIN_TYPE_Q6_K || fmt == REIN_TYPE_Q5_K || fmt == REIN_TYPE_IQ4_XS;
    // (... except short contractions against 8192 rows and more, which the 4x4x4 kernel takes: 1536 -> 8960 at 4 rows Q4_K
    // 7.3 -> 5.6 us, Q8_0 7.7 -> 6.4)
    return out_dim <= 2048 || (!quad_family && weights <= (1ull << 24) && out_dim < 8192);
}

// LDS-staged dot4 matvec (rein_mvl_*, kernels/matvec_lds.h), 2..4 activation rows: the rows of a
// workgroup's activations live in LDS, B x (in_dim / 32) x 40 bytes of it.
constexpr size_t kLdsPerCu = 160u * 1024u;
size_t mvl_lds_bytes(unsigned in_dim, unsigned n_rows) { return (size_t)(n_rows <= 2 ? 2 : 4) * (in_dim / 32) * 40; }

// Launch geometry, from a sweep over R 1/2/4, 4-16 wavefronts per workgroup and 1-4 resident workgroups
// per CU on 15 shapes (Q4_K and Q6_K, 2 and 4 rows).  Up to 16 wavefronts per workgroup share one
// copy of the activations.
//   * A matrix whose row groups all fit the machine at once (at most two workgroups of 16 wavefronts per
//     CU) is dealt out evenly, each wavefront one row group: 5120 rows are 512 workgroups of ten
//     wavefronts at one row per wavefront, 256 of ten at two.  R is the smallest rows-per-wavefront for
//     which that works and the copies fit the CU's LDS (Q6_K starts at two from in_dim 8192: 14336 -> 4096
//     at 4 rows 17.8 us against 19.2, 18944 -> 3584 23.0 against 25.2).
//   * Wider matrices run persistent: up to four workgroups per CU of four (2 rows) or eight (3-4 rows)
//     wavefronts at two rows per wavefront, striding over the row groups, each trip requesting the
//     next row group's first one.
// us, Q4_K, this geometry against the best other one: 5120 -> 5120 at 4 rows 7.89 (8.12); 17408 -> 5120
// 13.72 (14.28) and 18.84 (22.6); 14336 -> 4096 9.49 (10.04) and 12.40 (12.75); 5120 -> 34816 at 2 rows
// 22.26 (22.61); 5120 -> 17408 13.22 (13.29); 8192 -> 28672 at 4 rows 33.03 (33.99).
void mvl_geometry(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows, unsigned* r_out, unsigned* wpb_out, unsigned* grid_out)
{
    const unsigned copies = (unsigned)std::min<size_t>(4, kLdsPerCu / mvl_lds_bytes(in_dim, n_rows));
    unsigned r = 0, wpb = 0, grid = 0;
    for (unsigned rr = fmt == REIN_TYPE_Q6_K && in_dim >= 8192 ? 2 : 1; rr <= 2 && r == 0; rr *= 2) {
        const unsigned groups = (out_dim + rr - 1) / rr;
        const unsigned c = (groups + kCUs * 16 - 1) / (kCUs * 16);
        if (c > 2) break;                    // too wide for one row group per wavefront: persistent
        if (c > copies) continue;            // the CU's LDS holds fewer copies: more rows per wavefront
        r = rr;
        wpb = (groups + kCUs * c - 1) / (kCUs * c);
        grid = (groups + wpb - 1) / wpb;
    }
    if (r == 0) {
        r = 2;
        wpb = n_rows <= 2 ? 4 : 8;
        while (copies * wpb < 16) wpb *= 2;
        const unsigned groups = (out_dim + 1) / 2;
        grid = std::min(kCUs * copies, (groups + wpb - 1) / wpb);
    }
    const unsigned r_forced = opt_u(O_MV_ROWS, 0), wpb_forced = opt_u(O_MV_WPB, 0);
    if (r_forced == 1 || r_forced == 2 || r_forced == 4 || (wpb_forced >= 1 && wpb_forced <= 16)) {
        if (r_forced == 1 || r_forced == 2 || r_forced == 4) r = r_forced;
        if (wpb_forced >= 1 && wpb_forced <= 16) wpb = wpb_forced;
        grid = ((out_dim + r - 1) / r + wpb - 1) / wpb;
    }
    *r_out = r; *wpb_out = wpb; *grid_out = grid;
}

// Whether a batched decode of 2..4 rows runs on the LDS-staged kernel.  From one run of the library's choice
// among the other three families against this kernel, six formats x 16 shapes x 2 / 3 / 4 rows (ratio of the two
// times; the kernel's outputs are those of the dot4 family bit for bit):
//   3-4 rows  ahead for every format when the matrix has at most 6144 rows or a contraction of 8192 and more,
//             from 2^24 weights: 5120 -> 5120 1.07-1.24, 17408 -> 5120 1.18-1.29, 4096 -> 4096 1.28-1.47,
//             14336 -> 4096 1.22-1.57, 18944 -> 3584 1.15-1.58, 8192 -> 8192 1.00-1.11, 28672 -> 8192 1.07-1.25,
//             8192 -> 28672 1.17-1.59.  Behind on short contractions against many rows (5120 -> 34816 0.76-1.05,
//             5120 -> 17408 0.77-1.08, 3584 -> 18944 0.77-1.01, 5120 -> 7168 0.84-1.02), where the skinny MMQ and
//             the 4x4x4 kernel stream best, and on small matrices (2048 -> 2048 0.86-1.04).
//   2 rows    ahead for every format at contractions of 8192 and more from 2^25 weights (17408 -> 5120 0.98-1.11,
//             14336 -> 4096 0.97-1.24, 8192 -> 8192 1.03-1.16, 28672 -> 8192 1.12-1.28, 18944 -> 3584 1.10-1.63,
//             8192 -> 28672 1.10-1.34); on shorter contractions only Q4_K, Q4_0 and Q5_K against 14336 rows and
//             more (5120 -> 34816 1.13 / 1.08 / 1.06, 5120 -> 17408 1.17 / 1.14 / 1.09, 3584 -> 18944 1.16 / 1.13 /
//             1.05, 4096 -> 14336 1.04 / 1.08 / 1.03) and IQ3_S (1.05-1.14); Q6_K 0.91-1.10 and IQ4_XS 0.97-1.06
//             there; Q8_0 from 13824 rows at contractions of 4096 and more (timed from steady clocks: 1.06-1.09).
// Three and four rows on the 4x4x4 kernel with the rows in LDS (the shape part of use_mvql's rule, shared with use_mvl):
//   * up to 8192 rows and from 20 * 2^20 weights, every format but Q8_0 (contraction sliced over wavefronts);
//   * Q6_K with a long contraction against very few rows (us at 4 rows, dot4 / LDS dot4 / this: 8192 -> 1024 10.5 / 9.4 /
//     7.0, 8960 -> 1536 14.9 / 10.6 / 9.3);
//   * between 8192 and 14336 rows: Q4_K, Q5_K, Q6_K and their kin (5120 -> 13824 at 4 rows, 4x4x4 without LDS -> this: Q4_K
//     14.0 -> 12.4, Q5_K 17.7 -> 14.7; 8192 -> 10240, LDS dot4 -> this: 16.8 -> 15.6, 20.0 -> 19.1, Q6_K 24.5 -> 21.9), Q8_0
//     from 12288 rows (19.8 -> 17.1; 8192 -> 10240 21.4 on LDS dot4 against 22.9);
//   * from 14336 rows: every format but IQ4_XS (measured again from steady clocks, 4x4x4 without LDS -> this at 4 rows: Q6_K
//     5120 -> 34816 40.7 -> 36.7, 6144 -> 16384 23.6 -> 21.7, 3584 -> 18944 18.2 -> 17.9).
bool mvql_few_rows(int fmt, unsigned in_dim, unsigned out_dim)
{
    const unsigned long long weights = (unsigned long long)in_dim * out_dim;
    if (fmt != REIN_TYPE_Q8_0 && out_dim <= 8192 && weights >= (20ull << 20)) return true;
    if (fmt == REIN_TYPE_Q6_K && weights >= (6ull << 20) && in_dim >= 8192 && out_dim <= 1536) return true;
    // (short contractions against 8192 rows and more, below 2^24 weights: 1536 -> 8960 at 4 rows, us, dot4 / 4x4x4 / this:
    // Q4_K 7.3 / 5.6 / 5.6, Q8_0 7.7 / 6.4 / 6.4, Q6_K 10.2 / 6.9 / 6.6, IQ3_S 6.6 / 5.7 / 5.4, Q4_0 7.0 / 5.6 / 5.4)
    if (weights >= (6ull << 20) && weights < (1ull << 24)) return out_dim >= 8192;
    if (weights < (1ull << 24)) return false;
    const bool light_or_q5k = fmt == REIN_TYPE_Q5_K || fmt == REIN_TYPE_IQ3_S || fmt == REIN_TYPE_Q4_K || fmt == REIN_TYPE_Q4_0;
    if (out_dim >= 14336) return light_or_q5k || fmt == REIN_TYPE_Q8_0 || fmt == REIN_TYPE_Q6_K;
    if (out_dim > 8192) return light_or_q5k || fmt == REIN_TYPE_Q6_K || (fmt == REIN_TYPE_Q8_0 && out_dim >= 12288);
    return false;
}

bool use_mvl(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows)
{
    if (n_rows < 2 || n_rows > 4 || mvl_lds_bytes(in_dim, n_rows) > kLdsPerCu) return false;
    if (opt_is_set(O_MV_LDS)) return opt_u(O_MV_LDS, 0) != 0;
    if (opt_is_set(O_SKINNY_FROM) || opt_is_set(O_QUAD_FROM) || opt_is_set(O_MV_ROWS) || opt_is_set(O_MV_WPB)) return false;
    const unsigned long long weights = (unsigned long long)in_dim * out_dim;
    if (n_rows >= 3) {
        // (where the 4x4x4 kernel with the rows in LDS is ahead of this one, it goes first -- mvql_few_rows)
        if (opt_u(O_QUAD_LDS, 1) != 0 && mvql_few_rows(fmt, in_dim, out_dim)) return false;
        if (weights >= (1ull << 24)) return out_dim <= 6144 || in_dim >= 8192;
        // Smaller matrices with a contraction of 3584 and more: ahead of the plain dot4 kernel from six million weights
        // (us at 4 rows, dot4 -> this: 8960 -> 1536 Q4_K 9.3 -> 6.7, Q8_0 9.2 -> 7.1, Q5_K 10.0 -> 7.0; 5632 -> 2048 6.6 -> 5.2,
        // 6.4 -> 5.7, 7.1 -> 5.5, Q6_K 9.9 -> 6.4; 3584 -> 4608 8.3 -> 6.1, 9.7 -> 6.4; 8192 -> 1024 6.2 -> 5.8, 7.4 -> 5.9;
        // level at four million weights and with short contractions -- 2048 -> 5632 5.7 = 5.7, 1536 -> 8960 7.3 -> 6.9, where
        // the 4x4x4 kernels take 5.6)
        // (Q6_K, whose unpack weighs most on the plain kernel, from four million weights and at any contraction: 4096 -> 1024
        // 6.4 -> 4.7, 2048 -> 2048 4.7 -> 4.1, 2048 -> 5632 7.2 on the 4x4x4 kernel -> 6.8)
        if (fmt == REIN_TYPE_Q6_K) return weights >= (4ull << 20) && out_dim <= 6144;
        return weights >= (6ull << 20) && in_dim >= 3584 && out_dim <= 6144;
    }
    if (weights < (1ull << 25)) return false;
    if (in_dim >= 8192) return true;
    // (5120 -> 7168 Q4_K 8.5 -> 7.7 us, Q5_K 9.5 -> 9.2; 5120 -> 13824 13.0 -> 11.6, 14.8 -> 13.2; Q8_0 from 13824 rows:
    // 5120 -> 34816 35.4 -> 32.4, 5120 -> 13824 16.1 -> 15.2, 6144 -> 16384 20.7 -> 19.6, level at 7168 rows and at 3584 -> 18944)
    if (fmt == REIN_TYPE_Q8_0) return out_dim >= 13824 && in_dim >= 4096;
    return out_dim >= 7168 && (fmt == REIN_TYPE_Q4_K || fmt == REIN_TYPE_Q4_0 || fmt == REIN_TYPE_Q5_K || fmt == REIN_TYPE_IQ3_S);
}

int launch_matvec_lds(int fmt, const void* w, const void* xq, float* y, unsigned in_dim, unsigned out_dim,
                      unsigned n_rows, rein_stream_t s)
{
    unsigned r, wpb, grid;
    mvl_geometry(fmt, in_dim, out_dim, n_rows, &r, &wpb, &grid);
    const unsigned b = n_rows <= 2 ? 2 : 4;
    const std::string name = std::string("rein_mvl_") + fmt_tag(fmt) + "_r" + std::to_string(r) + "_b" + std::to_string(b);
    void* args[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&n_rows};
    return launch(name, grid, 1, 1, wpb * 64, (unsigned)mvl_lds_bytes(in_dim, n_rows), s, args);
}

// The 4x4x4 kernel with the activation rows staged in LDS (rein_mvql_*, kernels/matvec_quad.h), 3..8 rows.
// Geometry from a sweep over 4-16 wavefronts per workgroup, 1-4 resident workgroups per CU and one row group
// per wavefront or persistent wavefronts (Q4_K, Q6_K, Q5_K, Q8_0 on six shapes): up to 16384 rows 256
// workgroups with one group of four rows per wavefront (5120 rows: five wavefronts, 14336: fourteen); beyond,
// 512 workgroups of eight wavefronts that stride over the row groups.
struct QuadLdsGeometry { unsigned wpb, grid, phase_sub, slices; size_t lds; };       // lds == 0: no launch fits
// Which build of the 32-row kernel: the one for sixteen wavefronts per workgroup (128 registers, a few spilled) lets
// three wavefronts slice a row group's contraction and wins for every format but Q6_K, whose loop spills 204 bytes
// there (us at 32 rows, 512-thread build / 1024-thread build: Q4_K 17408 -> 5120 69.9 / 53.3, 5120 -> 5120 25.3 / 22.2,
// 8192 -> 8192 39.4 / 38.3; Q8_0 66.5 / 53.0, 24.3 / 24.1; Q5_K 73.0 / 55.8, 26.4 / 23.5; Q6_K 87.2 / 121.6, 30.5 / 47.9,
// 48.7 / 90.5).
bool mvql_wide32(int fmt)
{
    return opt_u(O_QUAD_WIDE32, fmt == REIN_TYPE_Q6_K ? 0u : 1u) != 0;
}
QuadLdsGeometry mvql_geometry(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows)
{
    const unsigned n_sub = in_dim / 32, t = n_rows <= 4 ? 4 : n_rows <= 8 ? 8 : n_rows <= 16 ? 16 : 32;
    const unsigned parts = fmt == REIN_TYPE_Q8_0 ? 3 : 2;               // 16-byte parts of Fmt<FMT>::Raw
    const unsigned groups = (out_dim + 3) / 4;
    QuadLdsGeometry g;
    g.slices = 1;
    // the 32-row kernels are built for 512 threads (no spills) and, as rein_mvql_<fmt>_t32w, for 1024
    const bool wide32 = t == 32 && mvql_wide32(fmt);
    const unsigned max_wpb = t == 32 && !wide32 ? 8 : 16;
    unsigned gpb = std::min(max_wpb, (groups + kCUs - 1) / kCUs);      // row groups per workgroup
    // 32 rows: every workgroup stages all 32 activation rows (700 KB at in_dim 17408, in phases), more than its share of
    // the weights, so fewer and fuller workgroups win as long as 160 CUs have one: 5120 rows as 160 workgroups of
    // eight wavefronts instead of 256 of five (us: Q4_K 17408 -> 5120 67.1 -> 64.2, 5120 -> 5120 24.7 -> 24.0; Q6_K
    // 85.6 -> 82.8, 30.6 -> 29.6)
    if (t == 32 && !wide32 && groups >= 8 * 160) gpb = 8;
    const bool persistent = groups > kCUs * 16;
    const unsigned wpb_forced = opt_u(O_MV_WPB, 0);
    if (wpb_forced >= 1 && wpb_forced <= max_wpb) gpb = wpb_forced;
    if (persistent && !(wpb_forced >= 1 && wpb_forced <= max_wpb)) { g.wpb = 8; g.grid = 2 * kCUs; }
    else {
        // few row groups per CU: several wavefronts share a row group, each taking every slices-th trip
        // (us, Q4_K at 8 rows, slices 1 / 2 / 3-4: 17408 -> 5120 28.7 / 21.1 / 19.9, 14336 -> 4096 22.5 / 16.1 / 14.6,
        // 5120 -> 5120 10.5 / 8.8 / 9.0, 8192 -> 8192 16.8 / 15.1, 5120 -> 1024 12.0 / 8.4 / 6.9: one trip in flight per
        // wavefront and five wavefronts per CU is a latency-bound launch): as many slices as give a workgroup 16
        // wavefronts, each with two trips at least
        const unsigned want = opt_u(O_QUAD_SLICES, 0);
        const unsigned trips = (n_sub + 15) / 16;
        g.slices = want >= 1 && want <= 8 ? want : std::min(8u, std::max(1u, trips / 2));
        g.slices = std::max(1u, std::min(g.slices, max_wpb / gpb));
        g.slices = std::min(g.slices, std::max(1u, trips));
        g.wpb = gpb * g.slices;
        g.grid = (groups + gpb - 1) / gpb;
    }
    const auto bytes = [&](unsigned n_stage) {
        const unsigned stride = n_stage + ((20u - (n_stage & 15u)) & 15u);
        return (size_t)t * stride * 40 + (size_t)g.wpb * parts * 76 * 16;
    };
    g.phase_sub = n_sub;
    g.lds = bytes(n_sub);
    if (g.lds > kLdsPerCu) {
        // The rows do not fit: stage the contraction in phases.  That form keeps a wavefront's partial sums in
        // registers across the phases, so it needs one row group per wavefront at most; a phase is a whole number
        // of rounds of the slices' trips.
        g.lds = 0;
        const unsigned round = 16u * g.slices;
        if (!persistent || (unsigned long long)g.grid * g.wpb >= groups)
            for (unsigned phases = 2; phases <= 32 && g.lds == 0; phases++) {
                const unsigned per = (((n_sub + phases - 1) / phases) + round - 1) / round * round;
                if (bytes(per) <= kLdsPerCu) { g.phase_sub = per; g.lds = bytes(per); }
            }
    }
    return g;
}

// Whether a batched decode of 3..32 rows runs on it.  Runs of the library's other choice against this kernel, seven
// formats x 16 shapes x 3 / 4 / 5 / 6 / 8 rows (ratio of the two times):
//   5-8 rows  Q6_K, Q5_K, IQ4_XS (the formats of the 4x4x4 kernel): level or ahead everywhere from 5 * 2^20 weights --
//             5120 -> 5120 1.05-1.18 (1.15-1.37 with slices), 5120 -> 34816 1.02-1.25, 4096 -> 14336 1.31-1.47, 8192 -> 8192
//             1.04-1.16, 2048 -> 16384 1.30-1.45, 17408 -> 5120 1.39-1.40, 18944 -> 3584 1.47-1.57, 5120 -> 1024 1.0-1.47.
//             Q4_K, Q8_0, Q4_0, IQ3_S (skinny MMQ otherwise): ahead up to 20480 rows -- 17408 -> 5120 1.21-1.37, 14336 ->
//             4096 1.25-1.46, 18944 -> 3584 1.27-1.50, 5120 -> 5120 1.12-1.16, 4096 -> 4096 1.12-1.35, 5120 -> 1024
//             1.20-1.51, 8192 -> 8192 1.00-1.23, 4096 -> 14336 1.21-1.36, 2048 -> 16384 1.20-1.35 -- except where the rows
//             need phases against more than 6144 rows (28672 -> 8192 0.88-1.06); behind or level beyond 20480 rows
//             (5120 -> 34816 0.95-1.08, 8192 -> 28672 0.92-1.20).
//   3-4 rows  up to 8192 rows and from 20 * 2^20 weights ahead of the LDS-staged dot4 kernel for every format but Q8_0
//             (0.95-1.02): Q4_K 5120 -> 5120 1.05-1.08, 17408 -> 5120 1.24-1.26, 14336 -> 4096 1.09, 28672 -> 8192
//             1.15-1.18, 18944 -> 3584 1.17, 5120 -> 7168 1.18-1.20, 8192 -> 8192 0.96; Q4_0 1.08-1.33; Q6_K 1.07-1.22;
//             Q5_K 1.05-1.27; IQ4_XS 1.01-1.17; IQ3_S 0.99-1.21; 4096 -> 4096 (2^24 weights) 0.86-0.97 and stays.
//             Against 14336 rows and more, where neither of those applies: Q5_K 1.03-1.18, Q8_0 0.99-1.17, IQ3_S
//             1.08-1.51, Q4_K 0.98-1.18, Q4_0 (with two trips in flight) 1.03-1.18; mixed for IQ4_XS 0.93-1.08 and Q6_K
//             0.89-1.09, which stay.
bool use_mvql(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows)
{
    if (n_rows < 3 || n_rows > 32) return false;
    const QuadLdsGeometry g = mvql_geometry(fmt, in_dim, out_dim, n_rows);
    if (g.lds == 0) return false;
    if (opt_is_set(O_QUAD_LDS)) return opt_u(O_QUAD_LDS, 0) != 0;
    if (opt_is_set(O_SKINNY_FROM) || opt_is_set(O_QUAD_FROM) || opt_is_set(O_MV_ROWS) || opt_is_set(O_MV_WPB)) return false;
    const unsigned long long weights = (unsigned long long)in_dim * out_dim;
    if (n_rows > 16)
        // 17-32 rows, against the 32-token tile launch of rein_mmq_xq8, which hands out one workgroup per 128 rows (40
        // workgroups for 5120 rows): ahead up to 8192 rows for every format -- 24 / 32 rows, us: Q4_K 5120 -> 5120 39 ->
        // 23, 17408 -> 5120 127 -> 56, 14336 -> 4096 104 -> 40, 8192 -> 8192 70 -> 38, 28672 -> 8192 207 -> 111, 5120 -> 1024
        // 38 -> 14; Q6_K 69 -> 50, 230 -> 127, 188 -> 91, 114 -> 92; beyond (4096 -> 14336 0.72-1.30, 2048 -> 16384
        // 0.65-1.13) the tile launch has workgroups enough
        // A sweep over 20 further shapes moved the limit: the tile launch stays short of workgroups up to 16384 rows
        // (tile launch / this at 24-32 rows: 8192 -> 10240 1.45-1.9, 4096 -> 14336 1.06-1.36, 5120 -> 13824 1.02-1.21,
        // 6144 -> 16384 1.05-1.21) unless the contraction is short (1536 -> 8960 0.88-1.06).
        return weights >= (1ull << 22) && (out_dim <= 8192 || (out_dim <= 16384 && in_dim >= 4096));
    if (n_rows > 8) {
        // 9-16 rows (rein_mmq_xq8 sends them here), against the skinny MMQ at 12 and 16 rows: Q6_K and Q5_K ahead on
        // narrow and on short-and-mid matrices (5120 -> 5120 1.27 / 1.13, 17408 -> 5120 1.29 / 1.17, 14336 -> 4096 1.30 /
        // 1.19, 18944 -> 3584 1.32 / 1.20, 4096 -> 14336 1.15, 2048 -> 16384 1.32 / 1.12, 8192 -> 8192 1.04-1.10, 5120 ->
        // 1024 1.9 / 1.6), the other formats by 1.00-1.22 against at most 4096 rows with a long contraction and 1.28-1.42
        // at 5120 -> 1024; everything behind against many rows (5120 -> 34816 0.72-0.93, 5120 -> 17408 0.69-0.85,
        // 28672 -> 8192 0.69-0.92, 5120 -> 7168 0.83-1.01)
        // The same 20 further shapes at 12 and 16 rows (skinny MMQ / this): every format 1.27-1.48 at 8192 -> 10240, where 320
        // tiles of 32 rows deal badly over 256 CUs; the formats of the skinny MMQ also 1.25-1.37 at 4096 -> 1024 (four million
        // weights), 1.18-1.28 at 5632 -> 2048, 1.08-1.28 at 16384 -> 6144 (0.99-1.08 at 13824 -> 5120, 0.84-0.91 at 3584 -> 4608,
        // 0.86-1.03 at 2048 -> 2048: they stay).
        if (weights < (1ull << 22)) return false;
        if (in_dim >= 8192 && out_dim > 8192 && out_dim <= 10240) return true;
        if (fmt == REIN_TYPE_Q6_K || fmt == REIN_TYPE_Q5_K)
            return out_dim <= 6144 || (in_dim <= 4096 && out_dim <= 16384) || (in_dim <= 8192 && out_dim <= 8192);
        // Measured again with every timing from steady clocks (the sweeps above ran the families of a cell one after the
        // other from cold clocks, the skinny MMQ last): contractions that are a multiple of 4096 -- the slices of a row
        // group's contraction come out even -- are ahead up to 14336 rows (skinny MMQ / this at 12 / 16 rows, Q4_K and Q8_0:
        // 4096 -> 4096 1.06 / 1.09 and 1.14 / 1.18, 4096 -> 6144 1.07 / 1.09 and 1.08 / 1.12, 4096 -> 14336 1.09 / 1.08 and
        // 1.20 / 1.22), and 13824 -> 5120 (1.07 / 1.10, 1.07 / 1.12) joins the long contractions against at most 6144 rows;
        // 5120 -> 5120 (0.95-1.04), 3584 -> 4608 (0.88-0.94), 5120 -> 7168 (0.81-0.88), 5120 -> 13824 (0.93-1.04) stay.
        return out_dim <= 1536 || (out_dim <= 2048 && in_dim >= 4096) || (out_dim <= 6144 && in_dim >= 13824) ||
               (in_dim % 4096 == 0 && out_dim <= 14336);
    }
    if (n_rows >= 5) {
        // (from four million weights with a contraction of 4096, every format but Q5_K: 4096 -> 1024 at 8 rows Q6_K 8.6 -> 6.7 us,
        // Q8_0 7.4 -> 6.4, IQ4_XS 8.0 -> 6.3, Q4_0 7.7 -> 6.3, IQ3_S 7.5 -> 6.2, Q4_K 6.5 -> 6.3; Q5_K 5.8 -> 6.5 and 2048 -> 2048
        // Q4_K 5.6 -> 6.0, Q5_K 5.3 -> 6.1 stay on dot4)
        const bool from_4m = fmt != REIN_TYPE_Q5_K && weights >= (4ull << 20) && in_dim >= 4096;
        if (weights < (5ull << 20) && !from_4m) return false;
        if (fmt == REIN_TYPE_Q6_K || fmt == REIN_TYPE_Q5_K || fmt == REIN_TYPE_IQ4_XS) return true;
        const bool phased = g.phase_sub < in_dim / 32;
        return out_dim <= 20480 && !(phased && out_dim > 6144);
    }
    return mvql_few_rows(fmt, in_dim, out_dim);
}

int launch_quad_lds(int fmt, const void* w, const void* xq, float* y, unsigned in_dim, unsigned out_dim,
                    unsigned n_rows, rein_stream_t s)
{
    const QuadLdsGeometry g = mvql_geometry(fmt, in_dim, out_dim, n_rows);
    const std::string name = std::string("rein_mvql_") + fmt_tag(fmt) + (n_rows <= 4 ? "_t4" : n_rows <= 8 ? "_t8" : n_rows <= 16 ? "_t16" :
                                                                         mvql_wide32(fmt) ? "_t32w" : "_t32");
    // Trips of weights in flight per wavefront where wavefronts stride over row groups or own a whole one (no slices,
    // no phases): two for the formats with little arithmetic per sub-block at 3-4 rows -- two register sets taking
    // turns -- (us, 5120 -> 34816 / 5120 -> 17408 / 3584 -> 18944 at 4 rows, one -> two: Q4_K 28.3 -> 26.0, 18.8 -> 17.3,
    // 14.2 -> 13.0; Q4_0 27.4 -> 23.7, 18.9 -> 16.1, 14.4 -> 12.2; IQ3_S 27.8 -> 24.2, 18.7 -> 16.2; Q8_0 40.1 -> 37.5,
    // 25.8 -> 23.0; Q5_K 33.0 -> 32.3, 21.2 -> 20.3) and for Q8_0 / Q4_0 / IQ3_S at 5-8 rows against 16384 rows and more
    // (1.05-1.07 x); Q6_K and IQ4_XS lose 3-10 % to the registers it costs, Q4_K and Q5_K at 8 rows 1-4 %.
    const bool light = fmt == REIN_TYPE_Q4_K || fmt == REIN_TYPE_Q4_0 || fmt == REIN_TYPE_Q8_0 || fmt == REIN_TYPE_IQ3_S || fmt == REIN_TYPE_Q5_K;
    // With slices or phases (narrow matrices) the second register set gains only where a wavefront has the CU nearly to
    // itself: 5120 -> 1024 1.05-1.20 x for every format at 4 and 8 rows, 0.86-1.05 from 4096 rows on.
    const bool strided = g.slices == 1 && g.phase_sub >= in_dim / 32;
    unsigned depth = 1;
    if (!strided) depth = out_dim <= 1536 ? 2 : 1;
    else if (n_rows <= 4 && light) depth = 2;
    else if (n_rows <= 8 && out_dim >= 16384 && (fmt == REIN_TYPE_Q8_0 || fmt == REIN_TYPE_Q4_0 || fmt == REIN_TYPE_IQ3_S)) depth = 2;
    depth = opt_u(O_QUAD_DEPTH, depth);
    void* args[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&n_rows, (void*)&g.phase_sub, (void*)&g.slices,
                    (void*)&depth};
    return launch(name, g.grid, 1, 1, g.wpb * 64, (unsigned)g.lds, s, args);
}

// Which kernel family a decode of 1..8 activation rows runs on.
enum class MvFamily { Dot4, Dot4Lds, Skinny, Quad, QuadLds };
MvFamily matvec_family(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows)
{
    // (an option that forces one LDS-staged family on goes first)
    const bool mvql_forced = opt_u(O_QUAD_LDS, 0) != 0 && opt_u(O_MV_LDS, 0) == 0;
    if (mvql_forced && use_mvql(fmt, in_dim, out_dim, n_rows)) return MvFamily::QuadLds;
    if (use_mvl(fmt, in_dim, out_dim, n_rows)) return MvFamily::Dot4Lds;
    if (use_mvql(fmt, in_dim, out_dim, n_rows)) return MvFamily::QuadLds;
    const bool small = small_for_matrix_cores(fmt, in_dim, out_dim, n_rows);
    if (!small && use_quad(fmt, out_dim, n_rows)) return MvFamily::Quad;
    // (the skinny kernel fetches a row's eight fp16 scales at once: in_dim >= 256)
    if (!small && n_rows >= skinny_from_rows(fmt) && in_dim >= 256) return MvFamily::Skinny;
    return MvFamily::Dot4;
}

// The kernel a few-row product launches: 1..8 rows as rein_matvec_batched_xq8 dispatches them, 9..32 rows the few-row
// kernels behind rein_mmq_xq8 ("" where that entry point launches token tiles).
std::string matvec_kernel_name(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows)
{
    const std::string tag = fmt_tag(fmt);
    const std::string t = n_rows <= 4 ? "_t4" : n_rows <= 8 ? "_t8" : n_rows <= 16 ? "_t16" : mvql_wide32(fmt) ? "_t32w" : "_t32";
    if (n_rows > 8) {
        if (n_rows <= 32 && use_mvql(fmt, in_dim, out_dim, n_rows)) return "rein_mvql_" + tag + t;
        if (n_rows <= 16 && in_dim >= 256 && skinny_from_rows(fmt) <= 16) return "rein_mmqs_" + tag + "_v8";
        return "";
    }
    switch (matvec_family(fmt, in_dim, out_dim, n_rows)) {
    case MvFamily::QuadLds: return "rein_mvql_" + tag + t;
    case MvFamily::Quad:    return "rein_mvq_" + tag + t;
    case MvFamily::Skinny:  return "rein_mmqs_" + tag + "_v" + std::to_string(n_rows <= 2 ? 1 : n_rows <= 4 ? 2 : 4);
    case MvFamily::Dot4Lds: {
        unsigned r, wpb, grid;
        mvl_geometry(fmt, in_dim, out_dim, n_rows, &r, &wpb, &grid);
        return "rein_mvl_" + tag + "_r" + std::to_string(r) + "_b" + std::to_string(n_rows <= 2 ? 2 : 4);
    }
    default: {
        const unsigned b = batch_slot(n_rows);
        return "rein_mv_" + tag + "_r" + std::to_string(pick_rows_per_wave(fmt, out_dim, b)) + "_b" + std::to_string(b);
    }
    }
}

int launch_matvec(const char* who, int fmt, const void* w, const void* xq, float* y, unsigned in_dim,
                  unsigned out_dim, unsigned n_rows, rein_stream_t s)
{
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_rows)) return rc;
    if (int rc = check_dense_fmt(who, fmt)) return rc;
    if (n_rows > 8) return fail(REIN_E_TOO_LARGE, std::string(who) + ": at most 8 activation rows");
    if (int rc = check_ptr(who, w, 16, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, y, 4, "y")) return rc;
    const MvFamily family = matvec_family(fmt, in_dim, out_dim, n_rows);
    if (family == MvFamily::QuadLds) return launch_quad_lds(fmt, w, xq, y, in_dim, out_dim, n_rows, s);
    if (family == MvFamily::Dot4Lds) return launch_matvec_lds(fmt, w, xq, y, in_dim, out_dim, n_rows, s);
    if (family == MvFamily::Quad) {
        // four output rows per wavefront, four wavefronts per workgroup
        const std::string name = std::string("rein_mvq_") + fmt_tag(fmt) + (n_rows <= 4 ? "_t4" : "_t8");
        void* args[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&n_rows};
        return launch(name, ((out_dim + 3) / 4 + 3) / 4, 1, 1, 256, 0, s, args);
    }
    if (family == MvFamily::Skinny) return launch_skinny(fmt, w, xq, y, in_dim, out_dim, n_rows, s);
    const unsigned b = batch_slot(n_rows);
    const unsigned r = pick_rows_per_wave(fmt, out_dim, b);
    const unsigned groups = (out_dim + r - 1) / r;
    const unsigned wpb = pick_wpb(fmt, groups, b);
    const unsigned grid = (groups + wpb - 1) / wpb;
    const std::string name = std::string("rein_mv_") + fmt_tag(fmt) + "_r" + std::to_string(r) + "_b" + std::to_string(b);
    void* args[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&n_rows};
    return launch(name, grid, 1, 1, wpb * 64, 0, s, args);
}

// Grouped GEMM launch.  The tile count lives on the device; the grid covers its upper bound
// (qwen35.rs:3051).  One tile per workgroup (rein_mmq_<fmt>_grouped_t32, both slabs in one
// launch when a second slab / output pair is given) as long as that bound fits a 1-D grid;
// beyond it the reference-named kernel, which strides over tiles, once per slab.
int launch_grouped(int fmt, const void* slab0, const void* slab1, unsigned bytes_per_expert, const int32_t* expert_off,
                   const int32_t* tile_off, unsigned n_expert, const void* xq, float* y0, float* y1, unsigned in_dim,
                   unsigned out_dim, unsigned n_entries, rein_stream_t s)
{
    const unsigned bn = rein_moe_gemm_bn();
    const unsigned tile_ub = (n_entries + bn - 1) / bn + n_expert;
    const unsigned gx = (out_dim + 127) / 128;
    const unsigned n_slab = slab1 ? 2 : 1;
    const unsigned long long grid = 8ull * ((tile_ub + 7) / 8) * n_slab * gx;
    if (grid <= 0x7FFFFFFFull && opt_u(O_GROUPED_STRIDED, 0) == 0) {
        const void* s1 = slab1 ? slab1 : slab0;
        float* o1 = y1 ? y1 : y0;
        void* a[] = {(void*)&slab0, (void*)&s1, (void*)&bytes_per_expert, (void*)&expert_off, (void*)&tile_off,
                     (void*)&n_expert, (void*)&xq, (void*)&y0, (void*)&o1, (void*)&in_dim, (void*)&out_dim, (void*)&n_slab};
        return launch(std::string("rein_mmq_") + fmt_tag(fmt) + "_grouped_t32", (unsigned)grid, 1, 1, 256, 0, s, a);
    }
    const std::string name = std::string("mmq_gemm_") + fmt_tag(fmt) + "_grouped_f32";
    for (int z = 0; z < (slab1 ? 2 : 1); z++) {
        const void* slab = z ? slab1 : slab0;
        float* y = z ? y1 : y0;
        void* a[] = {(void*)&slab, (void*)&bytes_per_expert, (void*)&expert_off, (void*)&tile_off, (void*)&n_expert,
                     (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim};
        if (int rc = launch(name, gx, std::min(tile_ub, 65535u), 1, 256, 0, s, a)) return rc;
    }
    return 0;
}

}  // namespace

extern "C" {

const char* rein_last_error(void) { return last_error(); }

// ---- options (the table at the top of this file)
namespace {
int opt_find(const char* name)
{
    if (!name) return -1;
    for (int i = 0; i < O_COUNT; i++)
        if (std::strcmp(name, kOptNames[i]) == 0) return i;
    return -1;
}
}  // namespace

int rein_set_option(const char* name, const char* value)
{
    const int i = opt_find(name);
    if (i < 0) return fail(REIN_E_NOT_FOUND, std::string("rein_set_option: no option named ") + (name ? name : "(null)"));
    (void)opt_raw((Opt)i);               // the environment is read before the first explicit change, never after it
    if (!value || !*value) {
        g_opts[i].store(0, std::memory_order_relaxed);
        return 0;
    }
    char* end = nullptr;
    const unsigned long v = std::strtoul(value, &end, 10);
    if (end == value || *end != 0 || v > 0xFFFFFFFFul)
        return fail(REIN_E_BAD_SHAPE, std::string("rein_set_option: ") + name + " takes an unsigned 32-bit decimal number, got \"" + value + "\"");
    g_opts[i].store(kOptSet | (uint64_t)v, std::memory_order_relaxed);
    return 0;
}

int rein_get_option(const char* name, unsigned* value, int* is_set)
{
    const int i = opt_find(name);
    if (i < 0) return fail(REIN_E_NOT_FOUND, std::string("rein_get_option: no option named ") + (name ? name : "(null)"));
    const uint64_t r = opt_raw((Opt)i);
    if (value) *value = (unsigned)(r & 0xFFFFFFFFull);
    if (is_set) *is_set = (r & kOptSet) ? 1 : 0;
    return 0;
}

int rein_option_count(void) { return O_COUNT; }
const char* rein_option_name(int index) { return index >= 0 && index < O_COUNT ? kOptNames[index] : nullptr; }

int rein_reset_options(void)
{
    (void)opt_raw(O_MV_ROWS);
    for (int i = 0; i < O_COUNT; i++) g_opts[i].store(0, std::memory_order_relaxed);
    return 0;
}

int rein_init(const char* hsaco_path)
{
    std::lock_guard<std::mutex> lock(g_init_mu);
    if (g_rt.loaded) return 0;
    const HipApi* api;
    if (int rc = need_api(&api)) return rc;
    const std::string path = hsaco_path && *hsaco_path ? hsaco_path : default_hsaco_path();
    hipModule_t m = nullptr;
    if (int rc = check_hip(api, api->ModuleLoad(&m, path.c_str()), ("hipModuleLoad(" + path + ")").c_str())) return rc;
    g_rt.api = api;
    g_rt.module = m;
    g_rt.loaded = true;
    (void)opt_raw(O_MV_ROWS);            // the one read of the environment, if nothing looked at the table before
    return 0;
}

int rein_is_loaded(void) { return g_rt.loaded ? 1 : 0; }

#define API_OR_RETURN() const HipApi* api; if (int rc_ = need_api(&api)) return rc_

int rein_device_count(int* n) { API_OR_RETURN(); return check_hip(api, api->GetDeviceCount(n), "hipGetDeviceCount"); }
int rein_set_device(int d) { API_OR_RETURN(); return check_hip(api, api->SetDevice(d), "hipSetDevice"); }
int rein_get_device(int* d) { API_OR_RETURN(); return check_hip(api, api->GetDevice(d), "hipGetDevice"); }
int rein_device_name(int d, char* buf, int len) { API_OR_RETURN(); return check_hip(api, api->DeviceGetName(buf, len, d), "hipDeviceGetName"); }
int rein_device_total_mem(int d, size_t* b) { API_OR_RETURN(); return check_hip(api, api->DeviceTotalMem(b, d), "hipDeviceTotalMem"); }
int rein_mem_info(size_t* f, size_t* t) { API_OR_RETURN(); return check_hip(api, api->MemGetInfo(f, t), "hipMemGetInfo"); }
int rein_device_synchronize(void) { API_OR_RETURN(); return check_hip(api, api->DeviceSynchronize(), "hipDeviceSynchronize"); }

int rein_malloc(void** p, size_t bytes) { API_OR_RETURN(); return check_hip(api, api->Malloc(p, bytes), "hipMalloc"); }
int rein_free(void* p) { API_OR_RETURN(); return check_hip(api, api->Free(p), "hipFree"); }
int rein_memcpy_h2d(void* d, const void* s, size_t n) { API_OR_RETURN(); return check_hip(api, api->Memcpy(d, s, n, hipMemcpyHostToDevice), "hipMemcpy H2D"); }
int rein_memcpy_d2h(void* d, const void* s, size_t n) { API_OR_RETURN(); return check_hip(api, api->Memcpy(d, s, n, hipMemcpyDeviceToHost), "hipMemcpy D2H"); }
int rein_memcpy_d2d(void* d, const void* s, size_t n) { API_OR_RETURN(); return check_hip(api, api->Memcpy(d, s, n, hipMemcpyDeviceToDevice), "hipMemcpy D2D"); }
int rein_memcpy_h2d_async(void* d, const void* s, size_t n, rein_stream_t st) { API_OR_RETURN(); return check_hip(api, api->MemcpyAsync(d, s, n, hipMemcpyHostToDevice, st), "hipMemcpyAsync H2D"); }
int rein_memcpy_d2h_async(void* d, const void* s, size_t n, rein_stream_t st) { API_OR_RETURN(); return check_hip(api, api->MemcpyAsync(d, s, n, hipMemcpyDeviceToHost, st), "hipMemcpyAsync D2H"); }
int rein_memcpy_d2d_async(void* d, const void* s, size_t n, rein_stream_t st) { API_OR_RETURN(); return check_hip(api, api->MemcpyAsync(d, s, n, hipMemcpyDeviceToDevice, st), "hipMemcpyAsync D2D"); }

int rein_stream_create(rein_stream_t* s) { API_OR_RETURN(); return check_hip(api, api->StreamCreate(s), "hipStreamCreate"); }
int rein_stream_destroy(rein_stream_t s) { API_OR_RETURN(); return check_hip(api, api->StreamDestroy(s), "hipStreamDestroy"); }
int rein_stream_synchronize(rein_stream_t s) { API_OR_RETURN(); return check_hip(api, api->StreamSynchronize(s), "hipStreamSynchronize"); }
int rein_stream_wait_event(rein_stream_t s, rein_event_t e) { API_OR_RETURN(); return check_hip(api, api->StreamWaitEvent(s, e, 0), "hipStreamWaitEvent"); }
int rein_event_create(rein_event_t* e) { API_OR_RETURN(); return check_hip(api, api->EventCreate(e), "hipEventCreate"); }
int rein_event_record(rein_event_t e, rein_stream_t s) { API_OR_RETURN(); return check_hip(api, api->EventRecord(e, s), "hipEventRecord"); }
int rein_event_synchronize(rein_event_t e) { API_OR_RETURN(); return check_hip(api, api->EventSynchronize(e), "hipEventSynchronize"); }
int rein_event_elapsed_ms(float* ms, rein_event_t a, rein_event_t b) { API_OR_RETURN(); return check_hip(api, api->EventElapsedTime(ms, a, b), "hipEventElapsedTime"); }
int rein_event_destroy(rein_event_t e) { API_OR_RETURN(); return check_hip(api, api->EventDestroy(e), "hipEventDestroy"); }
int rein_stream_begin_capture(rein_stream_t s) { API_OR_RETURN(); return check_hip(api, api->StreamBeginCapture(s, hipStreamCaptureModeGlobal), "hipStreamBeginCapture"); }
int rein_stream_end_capture(rein_stream_t s, rein_graph_t* g) { API_OR_RETURN(); return check_hip(api, api->StreamEndCapture(s, g), "hipStreamEndCapture"); }
int rein_graph_instantiate(rein_graph_exec_t* ge, rein_graph_t g) { API_OR_RETURN(); return check_hip(api, api->GraphInstantiate(ge, g, nullptr, nullptr, 0), "hipGraphInstantiate"); }
int rein_graph_launch(rein_graph_exec_t ge, rein_stream_t s) { API_OR_RETURN(); return check_hip(api, api->GraphLaunch(ge, s), "hipGraphLaunch"); }
int rein_graph_destroy(rein_graph_t g) { API_OR_RETURN(); return check_hip(api, api->GraphDestroy(g), "hipGraphDestroy"); }
int rein_graph_exec_destroy(rein_graph_exec_t ge) { API_OR_RETURN(); return check_hip(api, api->GraphExecDestroy(ge), "hipGraphExecDestroy"); }

int rein_module_load(rein_module_t* m, const char* path)
{
    API_OR_RETURN();
    if (!path) return fail(REIN_E_BAD_POINTER, "rein_module_load: path is NULL");
    return check_hip(api, api->ModuleLoad(m, path), "hipModuleLoad");
}
int rein_module_unload(rein_module_t m) { API_OR_RETURN(); return check_hip(api, api->ModuleUnload(m), "hipModuleUnload"); }
int rein_module_get_function(rein_function_t* f, rein_module_t m, const char* name)
{
    API_OR_RETURN();
    if (!name) return fail(REIN_E_BAD_POINTER, "rein_module_get_function: name is NULL");
    return check_hip(api, api->ModuleGetFunction(f, m, name), "hipModuleGetFunction");
}
int rein_builtin_module(rein_module_t* m)
{
    if (int rc = need_runtime()) return rc;
    *m = g_rt.module;
    return 0;
}
int rein_launch_kernel(rein_function_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
                       unsigned bz, unsigned shared_bytes, rein_stream_t s, void** args)
{
    API_OR_RETURN();
    return check_hip(api, api->ModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, shared_bytes, s, args, nullptr),
                     "hipModuleLaunchKernel");
}

// ------------------------------------------------------------------ hot path

int rein_quantize_q8(const float* x, void* xq, unsigned in_dim, unsigned n_vec, rein_stream_t s)
{
    if (in_dim == 0 || in_dim % 32 != 0 || n_vec == 0)
        return fail(REIN_E_BAD_SHAPE, "rein_quantize_q8: in_dim must be a non-zero multiple of 32 and n_vec non-zero");
    if (n_vec > 65535) return fail(REIN_E_TOO_LARGE, "rein_quantize_q8: at most 65535 vectors per call");
    if (int rc = check_ptr("rein_quantize_q8", x, 4, "x")) return rc;
    if (int rc = check_ptr("rein_quantize_q8", xq, 8, "xq")) return rc;
    // 16 sub-blocks per 256-thread workgroup (a 16-lane row each); the reference launches
    // 8 per workgroup (qwen35.rs:3202-3211), which the kernel accepts as well
    const unsigned gx = (in_dim + 511) / 512;
    void* args[] = {(void*)&x, (void*)&xq, (void*)&in_dim};
    return launch("quantize_q8_f32", gx, n_vec, 1, 256, 0, s, args);
}

// ---- fused BlockQ8 producers (kernels/fused_q8.hip)

namespace {
int check_fused_n(const char* who, unsigned n, unsigned n_vec, unsigned n_max)
{
    if (n == 0 || n % 32 != 0 || n_vec == 0)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": the vector length must be a non-zero multiple of 32 and the count non-zero");
    if (n_max && n > n_max) return fail(REIN_E_TOO_LARGE, std::string(who) + ": at most " + std::to_string(n_max) + " values per vector");
    if (n_vec > 65535) return fail(REIN_E_TOO_LARGE, std::string(who) + ": at most 65535 vectors per call");
    return 0;
}
// one workgroup per vector, a 16-lane row per sub-block: as many rows as the vector has
// sub-blocks (the serial part of the kernel is per row), whole wavefronts, at most 1024
// threads (the kernel keeps up to four sub-blocks per row in registers and re-reads
// beyond that)
unsigned fused_norm_block(unsigned n)
{
    const unsigned rows = n / 32;
    return std::min(1024u, (rows * 16 + 63) / 64 * 64);
}
unsigned elementwise_grid(unsigned n)
{
    unsigned g = (n + 511) / 512;              // 16 rows of a 256-thread block, 32 values each
    return std::min(g, kCUs * 32);
}
}  // namespace

int rein_rmsnorm_q8(const float* x, const float* w, void* xq, unsigned n, unsigned n_vec, float eps, rein_stream_t s)
{
    const char* who = "rein_rmsnorm_q8";
    if (int rc = check_fused_n(who, n, n_vec, 32768)) return rc;
    if (int rc = check_ptr(who, x, 4, "x")) return rc;
    if (int rc = check_ptr(who, w, 4, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    void* a[] = {(void*)&x, (void*)&w, (void*)&xq, (void*)&n, (void*)&eps};
    return launch("rmsnorm_q8_f32", 1, n_vec, 1, fused_norm_block(n), 0, s, a);
}

int rein_add_rmsnorm_q8(float* hidden, const float* add, const float* w, float* y, void* xq, unsigned n,
                        unsigned n_vec, float eps, rein_stream_t s)
{
    const char* who = "rein_add_rmsnorm_q8";
    if (int rc = check_fused_n(who, n, n_vec, 32768)) return rc;
    if (int rc = check_ptr(who, hidden, 4, "hidden")) return rc;
    if (int rc = check_ptr(who, w, 4, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (add) if (int rc = check_ptr(who, add, 4, "add")) return rc;
    if (y) if (int rc = check_ptr(who, y, 4, "y")) return rc;
    void* a[] = {(void*)&hidden, (void*)&add, (void*)&w, (void*)&y, (void*)&xq, (void*)&n, (void*)&eps};
    return launch("add_rmsnorm_q8_f32", 1, n_vec, 1, fused_norm_block(n), 0, s, a);
}

int rein_swiglu_q8(const float* gate, const float* up, float* out, void* xq, unsigned n, rein_stream_t s)
{
    const char* who = "rein_swiglu_q8";
    if (int rc = check_fused_n(who, n, 1, 0)) return rc;
    if (int rc = check_ptr(who, gate, 4, "gate")) return rc;
    if (int rc = check_ptr(who, up, 4, "up")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (out) if (int rc = check_ptr(who, out, 4, "out")) return rc;
    void* a[] = {(void*)&gate, (void*)&up, (void*)&out, (void*)&xq, (void*)&n};
    return launch("swiglu_q8_f32", elementwise_grid(n), 1, 1, 256, 0, s, a);
}

int rein_sigmoid_mul_q8(float* x, const float* gate, void* xq, unsigned n, rein_stream_t s)
{
    const char* who = "rein_sigmoid_mul_q8";
    if (int rc = check_fused_n(who, n, 1, 0)) return rc;
    if (int rc = check_ptr(who, x, 4, "x")) return rc;
    if (int rc = check_ptr(who, gate, 4, "gate")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    void* a[] = {(void*)&x, (void*)&gate, (void*)&xq, (void*)&n};
    return launch("sigmoid_mul_q8_f32", elementwise_grid(n), 1, 1, 256, 0, s, a);
}

int rein_rmsnorm_gated_q8(const float* x, const float* z, const float* w, float* y, void* xq, unsigned n_heads,
                          unsigned head_dim, float eps, rein_stream_t s)
{
    const char* who = "rein_rmsnorm_gated_q8";
    if (int rc = check_fused_n(who, head_dim, 1, 32768)) return rc;
    if (n_heads == 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": n_heads is zero");
    if (int rc = check_ptr(who, x, 4, "x")) return rc;
    if (int rc = check_ptr(who, z, 4, "z")) return rc;
    if (int rc = check_ptr(who, w, 4, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (y) if (int rc = check_ptr(who, y, 4, "y")) return rc;
    const unsigned block = std::max(64u, std::min(1024u, head_dim));
    void* a[] = {(void*)&x, (void*)&z, (void*)&w, (void*)&y, (void*)&xq, (void*)&n_heads, (void*)&head_dim, (void*)&eps};
    return launch("rmsnorm_gated_q8_f32", std::min(n_heads, kCUs * 16), 1, 1, block, 0, s, a);
}

int rein_moe_geglu_q8(const float* gu, void* xq, unsigned ff_exp, unsigned n_slot, rein_stream_t s)
{
    const char* who = "rein_moe_geglu_q8";
    if (int rc = check_fused_n(who, ff_exp, n_slot, 0)) return rc;
    if (int rc = check_ptr(who, gu, 4, "gu")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    void* a[] = {(void*)&gu, (void*)&xq, (void*)&ff_exp};
    return launch("moe_geglu_q8_f32", (ff_exp + 511) / 512, n_slot, 1, 256, 0, s, a);
}

int rein_matvec_xq8(int fmt, const void* w, const void* xq, float* y, unsigned in_dim, unsigned out_dim,
                    rein_stream_t s)
{
    return launch_matvec("rein_matvec_xq8", fmt, w, xq, y, in_dim, out_dim, 1, s);
}

int rein_matvec_batched_xq8(int fmt, const void* w, const void* xq, float* y, unsigned in_dim,
                            unsigned out_dim, unsigned n_rows, rein_stream_t s)
{
    return launch_matvec("rein_matvec_batched_xq8", fmt, w, xq, y, in_dim, out_dim, n_rows, s);
}

// Up to four matvecs on the same activation rows in one launch (kernels/matvec_multi.hip): the wavefronts of the
// launch are dealt over the matrices' row groups, each runs its group as rein_mv_<fmt>_r<R>_b<B> would.
int rein_matvec_multi_xq8(unsigned n_mat, const int* fmts, const void* const* ws, float* const* ys,
                          const unsigned* out_dims, const void* xq, unsigned in_dim, unsigned n_rows,
                          rein_stream_t s)
{
    const char* who = "rein_matvec_multi_xq8";
    constexpr unsigned kMax = 4;
    if (n_mat == 0 || n_mat > kMax)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": " + std::to_string(n_mat) + " matrices, 1 to " + std::to_string(kMax) + " go into one launch");
    if (n_rows > 4) return fail(REIN_E_TOO_LARGE, std::string(who) + ": at most 4 activation rows");
    if (!fmts || !ws || !ys || !out_dims) return fail(REIN_E_BAD_POINTER, std::string(who) + ": a NULL table");
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    unsigned long long total = 0;
    unsigned widest = 0;
    for (unsigned i = 0; i < n_mat; i++) {
        if (int rc = check_shape(who, fmts[i], in_dim, out_dims[i], n_rows)) return rc;
        if (int rc = check_dense_fmt(who, fmts[i])) return rc;
        if (int rc = check_ptr(who, ws[i], 16, "w")) return rc;
        if (int rc = check_ptr(who, ys[i], 4, "y")) return rc;
        total += out_dims[i];
        if (out_dims[i] > out_dims[widest]) widest = i;
    }
    if (total > 0x3FFFFFFFull) return fail(REIN_E_TOO_LARGE, std::string(who) + ": too many rows for one launch");
    // One matrix, or three to four rows against matrices of the size of an FFN's: the launches of the matrices one by
    // one, whose few-row kernels (activations staged in LDS, matrix instructions) are further ahead of dot4 there than
    // a launch costs (gate + up 5120 -> 17408 at 4 rows: 34.0 us as two launches, 38.6 as one; Q + K + V 5120 -> 5120 /
    // 1024 / 1024: 20.7 against 14.1, stays one launch; at 2 rows 26.9 against 25.7 and 15.4 against 10.1).
    const bool one_by_one = n_mat == 1 || (n_rows >= 3 && total * in_dim >= (64ull << 20) && !opt_is_set(O_MV_ROWS));
    if (one_by_one) {
        for (unsigned i = 0; i < n_mat; i++)
            if (int rc = launch_matvec(who, fmts[i], ws[i], xq, ys[i], in_dim, out_dims[i], n_rows, s)) return rc;
        return 0;
    }
    // rows per wavefront and wavefronts per workgroup as the dot4 launch of all the rows in the widest matrix's
    // format would take them
    // the fewest rows any of the formats would take at this total height, and four only from 16384 rows on: the
    // wavefronts of the heaviest format finish last (Q + K + V 5120 -> 5120 / 1024 / 1024 with a Q6_K value
    // projection: 9.6 us at four rows per wavefront, 7.7 at two, 8.7 at one; all Q4_K: 7.7 / 6.9 / 8.1)
    const int lead = fmts[widest];
    const unsigned b = batch_slot(n_rows);
    unsigned r = pick_rows_per_wave(lead, (unsigned)total, b);       // two to four rows: the widest matrix's choice (14.1 us against 17.6)
    for (unsigned i = 0; i < n_mat && b == 1; i++) {
        unsigned ri = pick_rows_per_wave(fmts[i], (unsigned)total, b);
        if (ri == 4 && total < 16384 && !opt_is_set(O_MV_ROWS)) ri = 2;
        r = std::min(r, ri);
    }
    struct Mat { const void* w; float* y; unsigned out_dim; int fmt; unsigned group_end; unsigned pad; };
    struct Args { Mat m[kMax]; } a{};
    unsigned groups = 0;
    for (unsigned i = 0; i < n_mat; i++) {
        groups += (out_dims[i] + r - 1) / r;
        a.m[i] = Mat{ws[i], ys[i], out_dims[i], fmts[i], groups, 0u};
    }
    for (unsigned i = n_mat; i < kMax; i++) a.m[i] = a.m[n_mat - 1];
    const unsigned wpb = pick_wpb(lead, groups, b);
    void* args[] = {(void*)&a, (void*)&xq, (void*)&in_dim, (void*)&n_mat, (void*)&n_rows};
    return launch("rein_mv_multi_r" + std::to_string(r) + "_b" + std::to_string(b), (groups + wpb - 1) / wpb, 1, 1, wpb * 64, 0, s, args);
}

int rein_matvec_kernel_name(int fmt, unsigned in_dim, unsigned out_dim, unsigned n_rows, char* name, size_t name_len)
{
    const char* who = "rein_matvec_kernel_name";
    if (!name || name_len == 0) return fail(REIN_E_BAD_POINTER, std::string(who) + ": no room for the name");
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_rows)) return rc;
    if (int rc = check_dense_fmt(who, fmt)) return rc;
    const std::string k = matvec_kernel_name(fmt, in_dim, out_dim, n_rows);
    if (k.size() + 1 > name_len) return fail(REIN_E_TOO_LARGE, std::string(who) + ": the name needs " + std::to_string(k.size() + 1) + " bytes");
    std::memcpy(name, k.c_str(), k.size() + 1);
    return 0;
}

int rein_matvec_ondisk_xq8(int fmt, const void* w_blocks, const void* xq, float* y, unsigned in_dim,
                           unsigned out_dim, rein_stream_t s)
{
    const char* who = "rein_matvec_ondisk_xq8";
    if (int rc = check_shape(who, fmt, in_dim, out_dim, 1)) return rc;
    const char* name = fmt == REIN_TYPE_Q4_K ? "matvec_q4_k_dp4a_f32" : fmt == REIN_TYPE_Q5_K ? "matvec_q5_k_dp4a_f32"
                     : fmt == REIN_TYPE_Q6_K ? "matvec_q6_k_dp4a_f32" : fmt == REIN_TYPE_Q8_0 ? "matvec_q8_0_dp4a_f32" : nullptr;
    if (!name) return fail(REIN_E_BAD_FORMAT, std::string(who) + ": formats are Q4_K, Q5_K, Q6_K, Q8_0");
    if (int rc = check_ptr(who, w_blocks, 16, "w_blocks")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, y, 4, "y")) return rc;
    // 4 wavefronts x 2 rows per workgroup; the kernel strides, so cap the grid at a few waves per SIMD
    const unsigned gx = std::min((out_dim + 7) / 8, kCUs * 16);
    void* a[] = {(void*)&w_blocks, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim};
    return launch(name, gx, 1, 1, 256, 0, s, a);
}

int rein_matvec_q8_0_splitk(const void* w, const void* xq, float* y_partials, unsigned in_dim, unsigned out_dim,
                            unsigned n_split, rein_stream_t s)
{
    const char* who = "rein_matvec_q8_0_splitk";
    if (int rc = check_shape(who, REIN_TYPE_Q8_0, in_dim, out_dim, 1)) return rc;
    if (n_split == 0 || n_split > 65535) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": n_split must be in 1..65535");
    if (int rc = check_ptr(who, w, 16, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, y_partials, 4, "y_partials")) return rc;
    void* a[] = {(void*)&w, (void*)&xq, (void*)&y_partials, (void*)&in_dim, (void*)&out_dim, (void*)&n_split};
    // one wavefront per row pair, as the reference (block 64, grid (ceil(out/2), n_split))
    return launch("matvec_q8_0_repacked_splitk_f32", (out_dim + 1) / 2, n_split, 1, 64, 0, s, a);
}

// How many 64-token tiles per row block the MMQ launch uses (0 = the 32-token kernel).
// A 64-token tile costs c64 times a 32-token tile of the 32-token kernel (one weight unpack
// feeds two MFMA tiles); a 32-token tile inside the mixed kernel costs 1.17 (two workgroups
// per CU there, three in its own kernel).  c64 is per format, from the 32- and 64-token kernels
// at 1024 and 2048 tokens against 17408 and 34816 rows: Q8_0 1.56, Q6_K and Q5_K 1.74, and Q4_K,
// whose 32-token kernel is the leanest, 2.1 -- unless the rows of the slab are padded (a
// power-of-two sub-block count), where every fetch of a weight tile straddles cache lines and
// sharing it between two token tiles is worth more: 0.3 less for every format (Q4_K 1.77 at
// 8192 x 8192 and 4096 x 14336).
// Workgroups are handed to CUs in launch order, 64-token tiles first; a CU's finish time is
// the sum of what it was handed.  The candidate with the earliest last finish wins.  Up to
// three 32-token workgroups per CU (everything resident at once) nothing beats the fine
// grain.  The estimate walks at most a few thousand workgroups, so it is kept per shape.
static double mmq_c64(int fmt, unsigned in_dim)
{
    const unsigned n_sub = in_dim / 32;
    const double padded = n_sub != 0 && (n_sub & (n_sub - 1)) == 0 ? 0.3 : 0.0;
    switch (fmt) {
    case REIN_TYPE_Q8_0: return 1.56 - padded;
    case REIN_TYPE_Q6_K:
    case REIN_TYPE_Q5_K: return 1.74 - padded;
    case REIN_TYPE_Q4_K: return 2.1 - padded;
    default:             return 1.68 - padded;
    }
}
static unsigned mmq_pick_n64(int fmt, unsigned in_dim, unsigned out_dim, unsigned p_rows)
{
    const unsigned n_rb = (out_dim + 127) / 128, t32 = (p_rows + 31) / 32;
    const unsigned long long wg32 = (unsigned long long)n_rb * t32;
    if (p_rows < 64 || wg32 <= 2ull * kCUs) return 0;
    const double c64 = mmq_c64(fmt, in_dim), c32mix = 1.17;
    if (wg32 <= 3ull * kCUs) {
        // everything resident at once either way: three 32-token workgroups on the fullest CUs (1.75 each)
        // against one or two 64-token ones (0.71 or 1.0 x c64) -- Q8_0 8192 x 8192 at 384 tokens 155 -> 133 us,
        // 17408 -> 5120 at 512 tokens 274 -> 251; Q4_K stays (119 against 140)
        const unsigned long long u64 = (unsigned long long)n_rb * ((p_rows + 63) / 64);
        return c64 * (u64 <= kCUs ? 0.71 : 1.0) < 0.97 * 1.75 ? p_rows / 64 : 0;
    }
    static std::mutex mu;
    static std::unordered_map<unsigned long long, unsigned> memo;
    const unsigned long long key = ((unsigned long long)out_dim << 32) | ((unsigned long long)p_rows << 8) | (unsigned)(c64 * 100.0 - 100.0);
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = memo.find(key);
        if (it != memo.end()) return it->second;
    }
    const unsigned a_max = p_rows / 64;
    unsigned best_n64 = c64 > 2.0 ? 0 : a_max;                 // very large grids: granularity no longer matters
    if (wg32 <= 64ull * kCUs) {
        double best = std::ceil((double)wg32 / kCUs);          // the 32-token kernel
        best_n64 = 0;
        std::vector<double> load(kCUs);
        for (unsigned a = a_max > 6 ? a_max - 6 : 1; a <= a_max; a++) {
            const unsigned long long big = (unsigned long long)n_rb * a;
            const unsigned long long small = (unsigned long long)n_rb * ((p_rows - a * 64 + 31) / 32);
            for (unsigned c = 0; c < kCUs; c++) load[c] = -c64 * (double)(big / kCUs + (c < big % kCUs ? 1 : 0));
            std::make_heap(load.begin(), load.end());          // max-heap of negated loads: top = least loaded CU
            for (unsigned long long i = 0; i < small; i++) {
                std::pop_heap(load.begin(), load.end());
                load.back() -= c32mix;
                std::push_heap(load.begin(), load.end());
            }
            const double finish = -*std::min_element(load.begin(), load.end());
            if (finish < best - 1e-9) { best = finish; best_n64 = a; }
        }
    }
    std::lock_guard<std::mutex> lock(mu);
    if (memo.size() > 4096) memo.clear();
    memo[key] = best_n64;
    return best_n64;
}

int rein_mmq_xq8(int fmt, const void* w, const void* xq, float* y, unsigned in_dim, unsigned out_dim,
                 unsigned p_rows, rein_stream_t s)
{
    const char* who = "rein_mmq_xq8";
    if (int rc = check_shape(who, fmt, in_dim, out_dim, p_rows)) return rc;
    if (int rc = check_dense_fmt(who, fmt)) return rc;
    if (int rc = check_ptr(who, w, 16, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, y, 4, "y")) return rc;
    // few rows: the batched-decode kernels (up to eight rows the choice of rein_matvec_batched_xq8, the same outputs)
    if (p_rows <= 8) return launch_matvec(who, fmt, w, xq, y, in_dim, out_dim, p_rows, s);
    if (p_rows <= 32 && use_mvql(fmt, in_dim, out_dim, p_rows)) return launch_quad_lds(fmt, w, xq, y, in_dim, out_dim, p_rows, s);
    if (p_rows <= 16 && in_dim >= 256 && skinny_from_rows(fmt) <= 16) return launch_skinny(fmt, w, xq, y, in_dim, out_dim, p_rows, s);
    // Token tiles: 32 tokens (rein_mmq_<fmt>_t32, three workgroups per CU) or the mixed launch
    // (rein_mmq_<fmt>_mix: n64 tiles of 64 tokens per row block, the rest in 32-token tiles).
    const unsigned n_rb = (out_dim + 127) / 128;
    unsigned n64 = mmq_pick_n64(fmt, in_dim, out_dim, p_rows);
    const unsigned forced_tm = opt_u(O_MMQ_TM, 0), forced_n64 = opt_u(O_MMQ_N64, 0xFFFFFFFFu);
    if (forced_n64 != 0xFFFFFFFFu) n64 = std::min(forced_n64, p_rows / 64);
    if (forced_tm == 32) n64 = 0;
    // every token in a 64-token tile: the 64-token kernel itself, 5-7 % ahead of the mixed kernel launched without
    // fillers (Q8_0 5120 x 34816 at 1024 tokens 681 -> 639 us, 8192 x 8192 at 2048 527 -> 501)
    const bool all64 = forced_n64 == 0xFFFFFFFFu && forced_tm == 0 && n64 > 0 && n64 * 64 >= p_rows;
    if (forced_tm == 64 || all64) {
        const unsigned long long g = 8ull * ((n_rb + 7) / 8) * ((p_rows + 63) / 64);
        if (g > 0x7FFFFFFFull) return fail(REIN_E_TOO_LARGE, "rein_mmq_xq8: too many tiles for one launch");
        void* a[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&p_rows};
        return launch(std::string("rein_mmq_") + fmt_tag(fmt) + "_t64", (unsigned)g, 1, 1, 256, 0, s, a);
    }
    // 1-D grids; workgroup i runs on XCD i % 8 and the kernels map it to (row block, token
    // tile) so that one weight block stays on one XCD
    if (n64 > 0 || forced_n64 != 0xFFFFFFFFu) {
        const unsigned n32 = (p_rows - n64 * 64 + 31) / 32;
        const unsigned long long g = 8ull * ((n_rb + 7) / 8) * (n64 + n32);
        if (g > 0x7FFFFFFFull) return fail(REIN_E_TOO_LARGE, "rein_mmq_xq8: too many tiles for one launch");
        void* a[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&p_rows, (void*)&n64};
        return launch(std::string("rein_mmq_") + fmt_tag(fmt) + "_mix", (unsigned)g, 1, 1, 256, 0, s, a);
    }
    const unsigned long long grid = 8ull * ((n_rb + 7) / 8) * ((p_rows + 31) / 32);
    if (grid > 0x7FFFFFFFull) return fail(REIN_E_TOO_LARGE, "rein_mmq_xq8: too many tiles for one launch");
    void* args[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&p_rows};
    return launch(std::string("rein_mmq_") + fmt_tag(fmt) + "_t32", (unsigned)grid, 1, 1, 256, 0, s, args);
}

// ---- Q4_K on the block-scaled fp6 matrix instruction (kernels/mmq_fp6.h)
namespace {
constexpr unsigned kX6Rec = 4352;          // REIN_X6_REC: bytes per (sub-block pair, 32-token tile) record
size_t x6_image_bytes(unsigned n_sub, unsigned p_rows)
{
    return (size_t)((n_sub + 1) / 2) * ((p_rows + 31) / 32) * kX6Rec + 1024;      // rein_x6_bytes
}
bool mmq6_format(int fmt) { return fmt == REIN_TYPE_Q4_K && opt_u(O_MMQ6, 1) != 0; }
unsigned mmq6_lds_bytes(unsigned nt)       // rein_mmq6_lds_bytes<NT>(), depths of Mmq6Cfg<NT>
{
    const unsigned r = nt == 4 ? 2 : nt == 2 ? 4 : 3, d = nt == 4 ? 3 : 4, sm = nt == 2 ? 2 : 1;
    return d * ((nt * kX6Rec + 1023u) & ~1023u) + 4 * r * 2048 + 4 * sm * 1280;
}
// a launch whose workgroups run tiles of several widths holds the largest layout
unsigned mmq6_lds_max() { return std::max(mmq6_lds_bytes(4), std::max(mmq6_lds_bytes(2), mmq6_lds_bytes(1))); }
// Token groups per 128-row block: n4 groups of four 32-token tiles, n2 of two, the rest single.
// Relative cost of a workgroup per 32-token tile, fitted to a sweep of the splits of 512 x 5120
// x 17408: 1.00 in a group of four, 1.15 in a group of two, 1.8 alone (the weight unpack is
// shared by fewer tiles, and a narrow workgroup still holds a wide one's LDS).  Workgroups are
// handed to CUs in launch order, widest first; a CU's finish time is the sum of what it was
// handed, and the split with the earliest last finish wins (ties: the least total work).
void mmq6_pick(unsigned out_dim, unsigned p_rows, unsigned* n4_out, unsigned* n2_out)
{
    const unsigned n_rb = (out_dim + 127) / 128, n_tt = (p_rows + 31) / 32;
    const unsigned f4 = opt_u(O_MMQ6_N4, 0xFFFFFFFFu), f2 = opt_u(O_MMQ6_N2, 0xFFFFFFFFu);
    if (f4 != 0xFFFFFFFFu || f2 != 0xFFFFFFFFu) {
        unsigned n4 = f4 == 0xFFFFFFFFu ? 0 : std::min(f4, n_tt / 4);
        unsigned n2 = f2 == 0xFFFFFFFFu ? 0 : std::min(f2, (n_tt - 4 * n4) / 2);
        *n4_out = n4; *n2_out = n2;
        return;
    }
    const unsigned a4 = n_tt / 4, rest = n_tt - 4 * a4;
    *n4_out = a4; *n2_out = rest / 2;
    // from about three rounds of wide workgroups the grain no longer matters (2048 x 17408: all
    // wide 591 us, the split the walk below prefers 611 us)
    if ((unsigned long long)n_rb * a4 > 6ull * kCUs) return;
    static std::mutex mu;
    static std::unordered_map<unsigned long long, unsigned> memo;
    const unsigned long long key = ((unsigned long long)out_dim << 32) | p_rows;
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = memo.find(key);
        if (it != memo.end()) { *n4_out = it->second >> 16; *n2_out = it->second & 0xFFFFu; return; }
    }
    const double c4 = 4.0, c2 = 2.3, c1 = 1.8;
    double best = 1e30;
    unsigned b4 = 0, b2 = 0;
    std::vector<double> load(kCUs);
    for (unsigned n4 = a4 > 3 ? a4 - 3 : 0; n4 <= a4; n4++) {
        const unsigned left = n_tt - 4 * n4;
        for (unsigned n2 = 0; 2 * n2 <= left && n2 <= 8; n2++) {
            const unsigned n1 = left - 2 * n2;
            std::fill(load.begin(), load.end(), 0.0);
            std::make_heap(load.begin(), load.end());          // max-heap of negated loads: top = least loaded CU
            const unsigned long long cnt[3] = {(unsigned long long)n_rb * n4, (unsigned long long)n_rb * n2, (unsigned long long)n_rb * n1};
            const double cost[3] = {c4, c2, c1};
            for (int kind = 0; kind < 3; kind++)
                for (unsigned long long i = 0; i < cnt[kind]; i++) {
                    std::pop_heap(load.begin(), load.end());
                    load.back() -= cost[kind];
                    std::push_heap(load.begin(), load.end());
                }
            const double total = (cnt[0] * c4 + cnt[1] * c2 + cnt[2] * c1) / kCUs;
            const double finish = -*std::min_element(load.begin(), load.end()) + 1e-3 * total;
            if (finish < best - 1e-9) { best = finish; b4 = n4; b2 = n2; }
        }
    }
    *n4_out = b4; *n2_out = b2;
    std::lock_guard<std::mutex> lock(mu);
    if (memo.size() > 4096) memo.clear();
    memo[key] = (b4 << 16) | b2;
}
int mmq6_prep(const void* xq, void* img, unsigned n_sub, unsigned p_rows, rein_stream_t s)
{
    void* a[] = {(void*)&xq, (void*)&img, (void*)&n_sub, (void*)&p_rows};
    return launch("rein_mmq6_prep", (p_rows + 31) / 32, (n_sub + 7) / 8, 1, 256, 0, s, a);
}

// Split-tail launch (rein_mmq6_split_tail): one workgroup per resident slot, two per CU; whole
// 4-tile units in rounds, the units left over split along the contraction.  Behind the activation
// image the workspace then holds one partial tile per workgroup.
constexpr unsigned kSkGrid = 2 * kCUs;
constexpr size_t kSkPartBytes = (size_t)4 * 16 * 256 * 4;                 // one partial tile: 4 x 32 tokens x 128 rows fp32
size_t sk_image_bytes(unsigned in_dim, unsigned p_rows) { return (x6_image_bytes(in_dim / 32, p_rows) + 255) & ~(size_t)255; }
size_t sk_workspace_bytes(unsigned in_dim, unsigned p_rows)
{
    return sk_image_bytes(in_dim, p_rows) + (size_t)kSkGrid * kSkPartBytes;
}
unsigned sk_grid()                 // REIN_MMQ6_SK_GRID: fewer workgroups (a multiple of 8), for tests of several rounds
{
    const unsigned g = opt_u(O_MMQ6_SK_GRID, kSkGrid) & ~7u;
    return g >= 8 && g <= kSkGrid ? g : kSkGrid;
}
// Workgroups per tail unit: at most 8 (every range pays a pipeline fill and a partial tile), at most one per
// chunk; behind whole rounds as many as fill one workgroup per CU, without them both slots.  Measured at
// 5120 x 17408 (us at split 1 / 2 / 4 / 8): 128 tokens 97 / 77 / 63 / 63 (3 in effect), 512 tokens 216 / 181 /
// 169 / 167, 2048 tokens 570 / 575 / 586 / 595.
unsigned sk_split(unsigned in_dim, unsigned out_dim, unsigned p_rows)
{
    const unsigned g = sk_grid(), n_unit = ((out_dim + 127) / 128) * (((p_rows + 31) / 32 + 3) / 4), n_tail = n_unit % g;
    if (n_tail == 0) return 1;
    const unsigned forced = opt_u(O_MMQ6_SK_SPLIT, 0);
    const unsigned room = (n_unit >= g ? g / 2 : g) / n_tail;
    const unsigned most = std::min(g / n_tail, in_dim / 256);
    return std::max(1u, std::min(forced ? forced : std::min(8u, room), most));
}
// The launch wants whole 4-tile token groups (a ragged last group computes its missing tiles all the same).
// Against the mixed launch, over 23 model shapes x 14 token counts (us, split-tail / mixed): a tail that splits
// two ways or more wins behind one to three rounds (4096 -> 11008 at 768 tokens 0.88, 5120 -> 17408 at 512
// 154 / 175, at 1024 289 / 308) and most without one (17408 -> 5120 at 512: 183 / 290); an unsplit tail
// behind one to three rounds is level or just ahead (0.92-1.06, median 0.98).  Behind four rounds and more the
// mixed launch, whose workgroups drift apart and overlap their fills and stores, is as good without the second
// launch (0.97-1.01) and steadier (2048 tokens x 17408: 575-690 us over runs against 586-617).  Without a whole round and with more units than CUs: up
// to 1.3 units per CU the second slots of a quarter of the CUs set the time and the mixed launch's narrower
// groups win (320-336 units: 1.12-1.23), from there on the launch is level (400-480 units 0.97-1.03) or
// ahead (4096 -> 6144 at 1024 tokens, 384 units, 104 / 134).  REIN_MMQ6_SK = 2 forces the launch wherever it
// is valid.
bool mmq6_split_tail(unsigned in_dim, unsigned out_dim, unsigned p_rows)
{
    const unsigned mode = opt_u(O_MMQ6_SK, 1);
    if (mode == 0) return false;
    if (opt_is_set(O_MMQ6_N4) || opt_is_set(O_MMQ6_N2)) return false;      // a forced token-group split
    const unsigned n_tt = (p_rows + 31) / 32, n_tg = (n_tt + 3) / 4;
    if (8 * (4 * n_tg - n_tt) > n_tt) return false;                       // more than an eighth of the tiles empty
    if (mode == 2 || opt_is_set(O_MMQ6_SK_GRID)) return true;
    const unsigned long long units = (unsigned long long)((out_dim + 127) / 128) * n_tg;
    const unsigned long long rounds = units / sk_grid();
    if (units % sk_grid() == 0 || rounds > 3) return false;
    if (sk_split(in_dim, out_dim, p_rows) >= 2) return true;
    return rounds != 0 || units >= kSkGrid * 2 / 3;
}

// Split-tail launch of the int8 tile (rein_mmq_split_tail in mmq_gemm.h): the same scheme for every dense
// format, with 64-token units, or 32-token units where a 64-token unit would be half empty (at most 32
// tokens, or an odd number of 32-token tiles below nine).  The workspace holds one partial tile per
// workgroup (32 KiB at 64 tokens).  Small GEMMs are what it is for: 17408 -> 5120 at 64 tokens is 40 units
// on 256 CUs as whole tiles (126 us for Q8_0, 228 for Q6_K) and 480 ranges split twelve ways (46 and 83 us).
constexpr size_t kSk8PartBytes = (size_t)2 * 16 * 256 * 4;
struct Sk8Plan { unsigned tm, g, n_unit, n_tail, split; bool take; double cost; };
// One unit width: units, ranges per tail unit, whether the launch pays, and a cost to compare widths by (a
// 64-token unit costs 1.68 32-token units; workgroups that have a CU to themselves run 1.4 times faster).
Sk8Plan sk8_width(int fmt, unsigned tm, unsigned g, unsigned in_dim, unsigned out_dim, unsigned p_rows)
{
    Sk8Plan p{tm, g, 0, 0, 1, false, 0.0};
    const unsigned n_chunk = (in_dim + 255) / 256;
    p.n_unit = ((out_dim + 127) / 128) * ((p_rows + tm - 1) / tm);
    p.n_tail = p.n_unit % g;
    const unsigned rounds = p.n_unit / g;
    if (p.n_tail) {
        // behind whole rounds: ranges that fill one workgroup per CU, at most 8; without them both slots, ranges
        // of two chunks and more, at most 12 (us at 4 / 8 / 10 / 12 ranges, Q8_0 17408 -> 5120 at 64 tokens:
        // 62 / 54 / 48 / 46; 5120 -> 1024: 20 / 18 / 16 / 16 at 5 / 8 / 10 / 20)
        const unsigned room = (rounds ? g / 2 : g) / p.n_tail, cap = rounds ? 8u : std::min(12u, std::max(1u, n_chunk / 2));
        const unsigned forced = opt_u(O_MMQ_SK_SPLIT, 0);
        p.split = std::max(1u, std::min(std::min(forced ? forced : std::min(cap, room), g / p.n_tail), n_chunk));
    }
    // it pays where the tail decides: no whole round and a tail that splits, or one whole round and a tail that
    // splits four ways (5120 x 17408 at 256 tokens: 117 -> 106 us Q8_0, 210 -> 184 Q6_K).  With 64-token units
    // also behind one or two whole rounds when the tail's workgroups have a CU each, split or not: over 23 model
    // shapes x 14 token counts Q6_K gains in all 43 such cells (1.01-1.29 x, median 1.08; 17408 -> 5120 at 1024
    // tokens 699 -> 566 us) and Q8_0 in all 42 (1.00-1.26 x; 346 -> 274 at 13824 -> 5120), while a tail on more
    // than half the slots loses (0.85-1.07, median 0.96) and so does Q6_K behind three rounds and more (0.89-1.00
    // without a tail, whose workgroups the plain launch lets drift apart).  Q4_K on the int8 tile gains only with a
    // tail that splits (0.96-1.24 against 0.88-1.04 unsplit).  Q5_K, Q4_0 and IQ4_XS, timed from steady clocks on the same
    // shapes: 1.13-1.16 x in the median with a tail that splits (0.95-1.28), 1.01-1.03 x unsplit (0.99-1.20); IQ3_S follows IQ4_XS.
    // Q8_0, the cheapest chunk against the same fills, stays ahead up to six rounds (1.01-1.15 x in all 19 cells).
    const bool any_split = fmt != REIN_TYPE_Q4_K;
    // Behind a third round the other formats but Q4_K are level or ahead as well (0.98-1.16, median 1.02 over 32 cells).
    const unsigned most_rounds = fmt == REIN_TYPE_Q8_0 ? 6 : fmt == REIN_TYPE_Q4_K ? 2 : 3;
    p.take = (rounds == 0 && p.split >= 2) || (rounds == 1 && p.split >= 4) ||
             (tm == 64 && rounds >= 1 && rounds <= most_rounds && p.n_tail != 0 && p.n_tail <= g / 2 && (any_split || p.split >= 2));
    const unsigned n_seg = p.n_tail * p.split;
    const double alone = rounds || n_seg >= g ? 1.0 : n_seg <= g / 2 ? 0.71 : 0.71 + 0.29 * (n_seg - g / 2) / (g / 2);
    p.cost = (tm == 64 ? 1.68 : 1.0) * (rounds + (p.n_tail ? alone / p.split : 0.0));
    return p;
}
Sk8Plan sk8_plan(int fmt, unsigned in_dim, unsigned out_dim, unsigned p_rows)
{
    const Sk8Plan none{64, kSkGrid, 0, 0, 1, false, 0.0};
    const unsigned mode = opt_u(O_MMQ_SK, 1);
    if (mode == 0 || p_rows <= 16 || in_dim == 0 || out_dim == 0 || !fmt_tag(fmt) || fmt == REIN_TYPE_Q5_1) return none;
    if (opt_is_set(O_MMQ_TM) || opt_is_set(O_MMQ_N64)) return none;        // a forced tiling
    const unsigned gg = opt_u(O_MMQ_SK_GRID, kSkGrid) & ~7u;        // fewer workgroups: tests of several rounds
    const unsigned g = gg >= 8 && gg <= kSkGrid ? gg : kSkGrid;
    const bool force = mode == 2 || opt_is_set(O_MMQ_SK_GRID);
    const unsigned n_tt = (p_rows + 31) / 32;
    const bool half_empty = 8 * (2 * ((n_tt + 1) / 2) - n_tt) > n_tt;   // more than an eighth of the 64-token units' tiles
    Sk8Plan w64 = sk8_width(fmt, 64, g, in_dim, out_dim, p_rows), w32 = sk8_width(fmt, 32, g, in_dim, out_dim, p_rows);
    if (const unsigned forced_tm = opt_u(O_MMQ_SK_TM, 0)) {
        Sk8Plan p = forced_tm == 32 ? w32 : w64;
        p.take = p.take || force;
        return p;
    }
    if (half_empty) w64.take = false;
    // Without a whole round the launch competes with the plain one, whose workgroups are then all resident at
    // once.  Both are priced in chunk times of a 32-token workgroup that shares its CU with one other (alone
    // 0.71, three on a CU 1.75 each, in between by the fill; a 64-token unit 1.68 of a 32-token one), plus three
    // chunk times for the second launch and the partial tiles.  Over 282 measured shapes x formats that removes
    // the losses of 5-46 % (1536 -> 6144 at 320 tokens: 26.5 us against 18.2 plain; 2048 -> 1536 at 512 tokens:
    // 21-23 against 17-19) and gives up two gains of 3-5 %.  Q6_K and Q5_K, whose chunk costs more against the
    // same second launch, gained in every measured shape and are left alone.
    if (!force && fmt != REIN_TYPE_Q6_K && fmt != REIN_TYPE_Q5_K) {
        const unsigned n_chunk = (in_dim + 255) / 256, n_rb = (out_dim + 127) / 128;
        const unsigned long long wg32 = (unsigned long long)n_rb * n_tt, u64 = (unsigned long long)n_rb * ((p_rows + 63) / 64);
        double plain;
        if (wg32 <= kCUs) plain = 0.71;
        else if (wg32 <= 2ull * kCUs) plain = 0.71 + 0.29 * (double)(wg32 - kCUs) / kCUs;
        else if (wg32 <= 3ull * kCUs) plain = 1.0 + 0.75 * (double)(wg32 - 2ull * kCUs) / kCUs;
        else { const unsigned long long r = u64 % kSkGrid; plain = 1.68 * ((double)(u64 / kSkGrid) + (r == 0 ? 0.0 : r <= kCUs ? 0.71 : 1.0)); }
        for (Sk8Plan* w : {&w64, &w32}) {
            if (w->take && w->n_unit < g && !(w->cost * n_chunk + 3.0 < plain * n_chunk)) w->take = false;
            // behind one whole round the same, against a plain launch that is resident at once (its fullest CUs
            // set its time: 1536 -> 6144 at 384 tokens 25.9 us against 22.8 plain)
            if (w->take && w->n_unit >= g && wg32 <= 3ull * kCUs &&
                !(w->cost * n_chunk + 3.0 < (wg32 <= kCUs ? 0.71 : wg32 <= 2ull * kCUs ? 1.0 : 1.75) * n_chunk)) w->take = false;
        }
    }
    // 128 tokens x 17408 rows: 544 units of 32 tokens are one round and a tail split eight ways (Q8_0 93 -> 73 us,
    // Q6_K 143 -> 117), 272 units of 64 tokens fill half the slots and do not split
    Sk8Plan p = w64.take && (!w32.take || w64.cost <= w32.cost) ? w64 : w32.take ? w32 : half_empty ? w32 : w64;
    p.take = p.take || force;
    return p;
}

}  // namespace

size_t rein_mmq_workspace_min_bytes(int fmt, unsigned in_dim, unsigned p_rows);

namespace {
// Which launch a workspace of `bytes` gets: 0 plain int8, 1 fp6 one token group per workgroup, 2 fp6 split-tail,
// 3 int8 split-tail.  REIN_MMQ6_FROM asks for the fp6 path by name wherever its workspace is there.
int mmq_form(int fmt, unsigned in_dim, unsigned out_dim, unsigned p_rows, size_t bytes)
{
    const size_t need = rein_mmq_workspace_min_bytes(fmt, in_dim, p_rows);
    const bool asked = opt_is_set(O_MMQ6_FROM) || opt_is_set(O_MMQ6_N4) || opt_is_set(O_MMQ6_N2);
    // The fp6 launches carry the image kernel in front and, split-tail, the sum behind: below about 50 us of
    // GEMM (2 M N K < 2.8e10) that costs more than the tile saves (768 -> 2048 at 512 tokens: 21 us against 9,
    // 2048 -> 1536: 26 against 19, 1536 -> 6144: 38 against 24; 5120 -> 2560 at 1536 tokens, 4.0e10: 90 against 139).
    const bool large = 2.0 * p_rows * (double)out_dim * in_dim >= 2.8e10;
    if (need != 0 && bytes >= need && (large || asked)) {
        if (bytes >= sk_workspace_bytes(in_dim, p_rows) && mmq6_split_tail(in_dim, out_dim, p_rows)) return 2;
        const unsigned n_tt = (p_rows + 31) / 32, n_tg = (n_tt + 3) / 4;
        const unsigned long long units = (unsigned long long)((out_dim + 127) / 128) * n_tg;
        if (8 * (4 * n_tg - n_tt) <= n_tt) {
            // Whole 4-tile token groups: from 1.25 groups per CU the fp6 tile is ahead of the int8 launches in
            // every measured shape but two (int8 / fp6 0.93-1.25, median 1.15, over 110 cells of 23 model shapes);
            // below that an unsplit launch leaves too many CUs with one workgroup against the int8 launch's
            // finer grain (258-296 groups: 0.78-0.99) and the GEMM stays there.
            if (units >= kSkGrid * 5 / 8 || asked) return 1;
        } else {
            // A ragged last group: the mixed launch cuts it into narrower workgroups, and comes out even over the
            // CUs' two slots with up to two 128-token workgroups per CU (from three 32-token tiles per slot),
            // whole multiples, or five and more (units per CU -> us fp6 against int8: 1.9 153 / 172, 2.0 129 / 151,
            // 3.0 193 / 233, 5.0 385 / 399, 8.5 622 / 665; in between level or behind, 3584 -> 18944 at 320 tokens
            // 108 / 94, 5120 -> 13824 at 448 tokens 1.15 x).  Below 320 tokens a ragged count stays on the int8 tile.
            const unsigned long long u128 = (unsigned long long)((out_dim + 127) / 128) * ((p_rows + 127) / 128);
            const unsigned long long tiles = (unsigned long long)((out_dim + 127) / 128) * n_tt;
            const bool even = p_rows >= 320 && tiles >= 3ull * kSkGrid && (u128 <= kSkGrid || u128 % kCUs == 0 || u128 >= 5ull * kCUs);
            if (even || asked) return 1;
        }
    }
    return bytes >= (size_t)kSkGrid * kSk8PartBytes && sk8_plan(fmt, in_dim, out_dim, p_rows).take ? 3 : 0;
}
}  // namespace

namespace {
// ---- Q4_K on the fp16 matrix instruction, superblocks accumulated in the matrix unit (kernels/mmq_f16.h)
size_t x16_image_bytes(unsigned n_sub, unsigned p_rows)                        // rein_x16_bytes
{
    const size_t n_grp = (p_rows + 63) / 64;
    return (size_t)(n_sub / 2) * n_grp * 16384 + (size_t)(n_sub / 8) * n_grp * 2048 + n_grp * 256 + 1024;
}
constexpr unsigned kMmq16Lds = 2 * 16384 + 2 * 2048 + 4 * 2 * 2 * 2048 + 4 * 2 * 1280;    // rein_mmq16_lds_bytes()
// The fp16 formulation is a study kernel: slower than the default launches and compiled into the code object
// only when the build asks for it (make MMQ16=1).  The option is ignored where the kernel is absent.
bool mmq16_built()
{
    static std::atomic<int> state{0};                   // 0 unknown, 1 present, 2 absent
    int st = state.load(std::memory_order_relaxed);
    if (st == 0) {
        if (!g_rt.loaded) return false;
        hipFunction_t f = nullptr;
        std::lock_guard<std::mutex> lock(g_rt.mu);
        st = g_rt.api->ModuleGetFunction(&f, g_rt.module, "rein_mmq16_q4k") == 0 && f ? 1 : 2;
        state.store(st, std::memory_order_relaxed);
    }
    return st == 1;
}
bool mmq16_asked(int fmt, unsigned in_dim)
{
    return fmt == REIN_TYPE_Q4_K && in_dim != 0 && in_dim % 256 == 0 && opt_u(O_MMQ16, 0) != 0 && mmq16_built();
}
}  // namespace

size_t rein_mmq_workspace_min_bytes(int fmt, unsigned in_dim, unsigned p_rows)
{
    if (!mmq6_format(fmt) || in_dim == 0 || in_dim % 256 != 0 || p_rows < opt_u(O_MMQ6_FROM, 128)) return 0;
    return x6_image_bytes(in_dim / 32, p_rows);
}

size_t rein_mmq_workspace_bytes(int fmt, unsigned in_dim, unsigned p_rows)
{
    // below 128 rows the fp6 launches never paid (their 4-tile token group is then mostly empty)
    if (rein_mmq_workspace_min_bytes(fmt, in_dim, p_rows) == 0) {
        // the int8 launch needs none; with room for its partial tiles it may run as a split-tail launch
        const bool dense = fmt_tag(fmt) && fmt != REIN_TYPE_Q5_1 && in_dim != 0 && p_rows > 16;
        return dense && opt_u(O_MMQ_SK, 1) != 0 ? (size_t)kSkGrid * kSk8PartBytes : 0;
    }
    const size_t fp6 = opt_u(O_MMQ6_SK, 1) != 0 ? sk_workspace_bytes(in_dim, p_rows) : x6_image_bytes(in_dim / 32, p_rows);
    return mmq16_asked(fmt, in_dim) ? std::max(fp6, x16_image_bytes(in_dim / 32, p_rows)) : fp6;
}

int rein_mmq_xq8_ws(int fmt, const void* w, const void* xq, float* y, unsigned in_dim, unsigned out_dim,
                    unsigned p_rows, void* workspace, size_t workspace_bytes, rein_stream_t s)
{
    const char* who = "rein_mmq_xq8_ws";
    const size_t need = rein_mmq_workspace_min_bytes(fmt, in_dim, p_rows);
    if (workspace && need != 0 && workspace_bytes < need)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": workspace of " + std::to_string(workspace_bytes) + " bytes, rein_mmq_workspace_min_bytes asks for " + std::to_string(need));
    if (workspace && mmq16_asked(fmt, in_dim) && p_rows > 16 && workspace_bytes >= x16_image_bytes(in_dim / 32, p_rows)) {
        if (int rc = check_shape(who, fmt, in_dim, out_dim, p_rows)) return rc;
        if (int rc = check_ptr(who, w, 16, "w")) return rc;
        if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
        if (int rc = check_ptr(who, y, 4, "y")) return rc;
        if (int rc = check_ptr(who, workspace, 16, "workspace")) return rc;
        const unsigned n_sub = in_dim / 32, n_grp = (p_rows + 63) / 64, n_rb = (out_dim + 255) / 256;
        void* pa[] = {(void*)&xq, (void*)&workspace, (void*)&n_sub, (void*)&p_rows};
        if (int rc = launch("rein_mmq16_prep", 2 * n_grp, n_sub / 8, 1, 256, 0, s, pa)) return rc;
        const unsigned long long grid = 8ull * ((n_rb + 7) / 8) * n_grp;
        if (grid > 0x7FFFFFFFull) return fail(REIN_E_TOO_LARGE, std::string(who) + ": too many tiles for one launch");
        void* a[] = {(void*)&w, (void*)&workspace, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&p_rows};
        return launch("rein_mmq16_q4k", (unsigned)grid, 1, 1, 256, kMmq16Lds, s, a);
    }
    const int form = workspace ? mmq_form(fmt, in_dim, out_dim, p_rows, workspace_bytes) : 0;
    if (form == 3) {
        const Sk8Plan sk8 = sk8_plan(fmt, in_dim, out_dim, p_rows);
        if (int rc = check_shape(who, fmt, in_dim, out_dim, p_rows)) return rc;
        if (int rc = check_dense_fmt(who, fmt)) return rc;
        if (int rc = check_ptr(who, w, 16, "w")) return rc;
        if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
        if (int rc = check_ptr(who, y, 4, "y")) return rc;
        if (int rc = check_ptr(who, workspace, 16, "workspace")) return rc;
        const unsigned first = sk8.n_unit - sk8.n_tail, n_chunk = (in_dim / 32 + 7) / 8, split = sk8.split;
        void* a[] = {(void*)&w, (void*)&xq, (void*)&y, (void*)&workspace, (void*)&in_dim, (void*)&out_dim, (void*)&p_rows, (void*)&split};
        if (int rc = launch(std::string("rein_mmq_") + fmt_tag(fmt) + (sk8.tm == 32 ? "_sk32" : "_sk"), sk8.g, 1, 1, 256, 0, s, a)) return rc;
        if (sk8.n_tail == 0 || split == 1) return 0;
        void* b[] = {(void*)&workspace, (void*)&y, (void*)&n_chunk, (void*)&out_dim, (void*)&p_rows, (void*)&first, (void*)&split};
        return launch(sk8.tm == 32 ? "rein_mmq_tail_sum_t32" : "rein_mmq_tail_sum_t64", sk8.n_tail, sk8.tm / 32, 4, 256, 0, s, b);
    }
    if (form == 0) return rein_mmq_xq8(fmt, w, xq, y, in_dim, out_dim, p_rows, s);
    if (int rc = check_shape(who, fmt, in_dim, out_dim, p_rows)) return rc;
    if (int rc = check_ptr(who, w, 16, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, y, 4, "y")) return rc;
    if (int rc = check_ptr(who, workspace, 16, "workspace")) return rc;
    if (form == 2) {
        char* base = static_cast<char*>(workspace);
        float* part = reinterpret_cast<float*>(base + sk_image_bytes(in_dim, p_rows));
        const unsigned split = sk_split(in_dim, out_dim, p_rows), g = sk_grid();
        const unsigned n_unit = ((out_dim + 127) / 128) * (((p_rows + 31) / 32 + 3) / 4), n_tail = n_unit % g, first = n_unit - n_tail;
        if (int rc = mmq6_prep(xq, workspace, in_dim / 32, p_rows, s)) return rc;
        void* a[] = {(void*)&w, (void*)&workspace, (void*)&y, (void*)&part, (void*)&in_dim, (void*)&out_dim, (void*)&p_rows, (void*)&split};
        if (int rc = launch("rein_mmq6_q4k_sk", g, 1, 1, 256, mmq6_lds_bytes(4), s, a)) return rc;
        if (n_tail == 0 || split == 1) return 0;
        void* b[] = {(void*)&part, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&p_rows, (void*)&first, (void*)&split};
        return launch("rein_mmq6_tail_sum", n_tail, 4, 4, 256, 0, s, b);
    }
    unsigned n4, n2;
    mmq6_pick(out_dim, p_rows, &n4, &n2);
    const unsigned n_rb = (out_dim + 127) / 128, n_tt = (p_rows + 31) / 32, n1 = n_tt - 4 * n4 - 2 * n2;
    const unsigned long long grid = 8ull * ((n_rb + 7) / 8) * (n4 + n2 + n1);
    if (grid > 0x7FFFFFFFull) return fail(REIN_E_TOO_LARGE, std::string(who) + ": too many tiles for one launch");
    if (int rc = mmq6_prep(xq, workspace, in_dim / 32, p_rows, s)) return rc;
    void* a[] = {(void*)&w, (void*)&workspace, (void*)&y, (void*)&in_dim, (void*)&out_dim, (void*)&p_rows, (void*)&n4, (void*)&n2};
    return launch("rein_mmq6_q4k_mix", (unsigned)grid, 1, 1, 256, mmq6_lds_max(), s, a);
}

// ---- the entry point that allocates nothing
namespace {
typedef int (*static_scratch_fn)(void**, size_t*);
std::mutex g_scratch_mu;
static_scratch_fn g_scratch_fn = nullptr;

// librein_scratch.so (host/static_scratch.hip) next to this library: loaded on first use
int static_scratch(void** ptr, size_t* bytes)
{
    {
        std::lock_guard<std::mutex> lock(g_scratch_mu);
        if (!g_scratch_fn) {
            std::string path = default_hsaco_path();
            const size_t slash = path.find_last_of('/');
            path = (slash == std::string::npos ? std::string(".") : path.substr(0, slash)) + "/librein_scratch.so";
            void* h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
            if (!h) {
                const char* err = dlerror();
                return fail(REIN_E_NOT_LOADED, "rein_mmq_xq8_noalloc: cannot load " + path + ": " + (err ? err : "unknown error"));
            }
            g_scratch_fn = reinterpret_cast<static_scratch_fn>(dlsym(h, "rein_static_scratch"));
            if (!g_scratch_fn) return fail(REIN_E_NOT_LOADED, "rein_mmq_xq8_noalloc: " + path + " does not export rein_static_scratch");
        }
    }
    const int e = g_scratch_fn(ptr, bytes);
    if (e != 0) return check_hip(g_rt.api, (hipError_t)e, "hipGetSymbolAddress(scratch)");
    return 0;
}
}  // namespace

int rein_noalloc_prepare(void)
{
    if (int rc = need_runtime()) return rc;
    void* ptr = nullptr;
    size_t bytes = 0;
    if (int rc = static_scratch(&ptr, &bytes)) return rc;
    // the kernels the entry point can launch: their handles are looked up now, not under a capture
    static const char* const names[] = {"rein_mmq6_prep", "rein_mmq6_q4k_mix", "rein_mmq6_q4k_sk", "rein_mmq6_tail_sum",
                                        "rein_mmq_tail_sum_t32", "rein_mmq_tail_sum_t64"};
    for (const char* n : names) {
        hipFunction_t f;
        if (int rc = get_fn(n, &f)) return rc;
    }
    static const int fmts[] = {REIN_TYPE_Q4_0, REIN_TYPE_Q4_K, REIN_TYPE_Q5_K, REIN_TYPE_Q6_K, REIN_TYPE_Q8_0, REIN_TYPE_IQ4_XS, REIN_TYPE_IQ3_S};
    static const char* const forms[] = {"_t32", "_t64", "_mix", "_sk", "_sk32"};
    // (up to 32 rows the entry point launches the few-row kernels: skinny MMQ, both 4x4x4 kernels, and from eight rows
    // down the decode matvecs in every rows-per-wavefront x batch-slot instantiation there is)
    static const char* const few[] = {"rein_mmqs_%s_v1", "rein_mmqs_%s_v2", "rein_mmqs_%s_v4", "rein_mmqs_%s_v8", "rein_mvql_%s_t4", "rein_mvql_%s_t8",
                                      "rein_mvql_%s_t16", "rein_mvql_%s_t32", "rein_mvql_%s_t32w", "rein_mvq_%s_t4", "rein_mvq_%s_t8"};
    for (int fmt : fmts) {
        for (const char* form : forms) {
            hipFunction_t f;
            if (int rc = get_fn(std::string("rein_mmq_") + fmt_tag(fmt) + form, &f)) return rc;
        }
        for (const char* pattern : few) {
            char name[64];
            std::snprintf(name, sizeof(name), pattern, fmt_tag(fmt));
            hipFunction_t f;
            if (int rc = get_fn(name, &f)) return rc;
        }
        for (unsigned r = 1; r <= 4; r *= 2)
            for (unsigned b = 1; b <= 8; b *= 2) {
                hipFunction_t f;
                if (r * b <= 16)
                    if (int rc = get_fn(std::string("rein_mv_") + fmt_tag(fmt) + "_r" + std::to_string(r) + "_b" + std::to_string(b), &f)) return rc;
                if (b == 2 || b == 4)
                    if (int rc = get_fn(std::string("rein_mvl_") + fmt_tag(fmt) + "_r" + std::to_string(r) + "_b" + std::to_string(b), &f)) return rc;
            }
    }
    return 0;
}

int rein_mmq_xq8_noalloc(int fmt, const void* w, const void* xq, float* y, unsigned in_dim, unsigned out_dim,
                         unsigned p_rows, rein_stream_t s)
{
    if (int rc = need_runtime()) return rc;
    // rein_mmq_xq8_ws on the fixed array: whichever launch that entry point picks for a workspace of the array's
    // size (split-tail forms included where their partial tiles fit behind the activation image)
    const size_t need = rein_mmq_workspace_min_bytes(fmt, in_dim, p_rows);
    void* ptr = nullptr;
    size_t bytes = 0;
    if (int rc = static_scratch(&ptr, &bytes)) return rc;
    if (need > bytes)
        return fail(REIN_E_TOO_LARGE, "rein_mmq_xq8_noalloc: this shape needs " + std::to_string(need) + " bytes of scratch, the fixed array holds " +
                                          std::to_string(bytes) + "; use rein_mmq_xq8_ws with a workspace of your own");
    return rein_mmq_xq8_ws(fmt, w, xq, y, in_dim, out_dim, p_rows, ptr, bytes, s);
}

int rein_mmq_form_ws(int fmt, unsigned in_dim, unsigned out_dim, unsigned p_rows, size_t workspace_bytes)
{
    const size_t need = rein_mmq_workspace_min_bytes(fmt, in_dim, p_rows);
    if (need != 0 && workspace_bytes < need) return 0;                   // rein_mmq_xq8_ws refuses such a workspace
    if (mmq16_asked(fmt, in_dim) && p_rows > 16 && workspace_bytes >= x16_image_bytes(in_dim / 32, p_rows)) return 4;
    return mmq_form(fmt, in_dim, out_dim, p_rows, workspace_bytes);
}

int rein_mmq_tile_plan_ws(int fmt, unsigned out_dim, unsigned p_rows, unsigned* n4, unsigned* n2)
{
    if (!n4 || !n2) return fail(REIN_E_BAD_POINTER, "rein_mmq_tile_plan_ws: NULL output");
    if (!mmq6_format(fmt)) return fail(REIN_E_BAD_FORMAT, "rein_mmq_tile_plan_ws: the format has no workspace launch");
    if (out_dim == 0 || p_rows == 0) return fail(REIN_E_BAD_SHAPE, "rein_mmq_tile_plan_ws: empty shape");
    mmq6_pick(out_dim, p_rows, n4, n2);
    return 0;
}

int rein_mmq_block_dots_ws(int fmt, const void* w, const void* xq, int32_t* out, unsigned in_dim, unsigned out_dim,
                           unsigned n_rows, void* workspace, size_t workspace_bytes, rein_stream_t s)
{
    const char* who = "rein_mmq_block_dots_ws";
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_rows)) return rc;
    if (!mmq6_format(fmt)) return fail(REIN_E_BAD_FORMAT, std::string(who) + ": the format has no workspace launch");
    if (int rc = check_ptr(who, w, 16, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, out, 4, "out")) return rc;
    if (int rc = check_ptr(who, workspace, 16, "workspace")) return rc;
    if (workspace_bytes < x6_image_bytes(in_dim / 32, n_rows))
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": workspace too small");
    const unsigned n_rb = (out_dim + 127) / 128, n_tt = (n_rows + 31) / 32;
    const unsigned long long grid = 8ull * ((n_rb + 7) / 8) * n_tt;
    if (grid > 0x7FFFFFFFull) return fail(REIN_E_TOO_LARGE, std::string(who) + ": too many tiles for one launch");
    if (int rc = mmq6_prep(xq, workspace, in_dim / 32, n_rows, s)) return rc;
    void* a[] = {(void*)&w, (void*)&workspace, (void*)&out, (void*)&in_dim, (void*)&out_dim, (void*)&n_rows};
    return launch("rein_mmq6_q4k_dots", (unsigned)grid, 1, 1, 256, mmq6_lds_bytes(1), s, a);
}

int rein_mmq_tile_plan(int fmt, unsigned in_dim, unsigned out_dim, unsigned p_rows)
{
    if (!rein_block_size(fmt)) return fail(REIN_E_BAD_FORMAT, "rein_mmq_tile_plan: unknown format " + std::to_string(fmt));
    if (in_dim == 0 || out_dim == 0 || p_rows == 0) return fail(REIN_E_BAD_SHAPE, "rein_mmq_tile_plan: empty shape");
    return (int)mmq_pick_n64(fmt, in_dim, out_dim, p_rows);
}

int rein_matmul_path(int fmt, unsigned n_rows)
{
    if (!rein_block_size(fmt)) return fail(REIN_E_BAD_FORMAT, "rein_matmul_path: unknown format " + std::to_string(fmt));
    if (n_rows == 0) return fail(REIN_E_BAD_SHAPE, "rein_matmul_path: n_rows is zero");
    if (n_rows == 1) return 0;
    return n_rows <= 8 ? 1 : 2;
}

int rein_matmul(int fmt, const void* w, const float* x, float* y, unsigned in_dim, unsigned out_dim,
                unsigned n_rows, void* xq_scratch, rein_stream_t s)
{
    if (int rc = check_shape("rein_matmul", fmt, in_dim, out_dim, n_rows)) return rc;
    if (int rc = check_dense_fmt("rein_matmul", fmt)) return rc;
    if (int rc = rein_quantize_q8(x, xq_scratch, in_dim, n_rows, s)) return rc;
    switch (rein_matmul_path(fmt, n_rows)) {
    case 0:  return rein_matvec_xq8(fmt, w, xq_scratch, y, in_dim, out_dim, s);
    case 1:  return rein_matvec_batched_xq8(fmt, w, xq_scratch, y, in_dim, out_dim, n_rows, s);
    default: return rein_mmq_xq8(fmt, w, xq_scratch, y, in_dim, out_dim, n_rows, s);
    }
}

size_t rein_matmul_scratch_bytes(int fmt, unsigned in_dim, unsigned n_rows)
{
    if (!rein_block_size(fmt) || in_dim == 0 || in_dim % 32 != 0 || n_rows == 0) return 0;
    const size_t xq = ((size_t)n_rows * (in_dim / 32) * 40 + 255) & ~(size_t)255;
    return xq + (rein_matmul_path(fmt, n_rows) == 2 ? rein_mmq_workspace_bytes(fmt, in_dim, n_rows) : 0);
}

int rein_matmul_ws(int fmt, const void* w, const float* x, float* y, unsigned in_dim, unsigned out_dim,
                   unsigned n_rows, void* scratch, size_t scratch_bytes, rein_stream_t s)
{
    if (int rc = check_shape("rein_matmul_ws", fmt, in_dim, out_dim, n_rows)) return rc;
    if (int rc = check_dense_fmt("rein_matmul_ws", fmt)) return rc;
    if (int rc = check_ptr("rein_matmul_ws", scratch, 16, "scratch")) return rc;
    const size_t xq = ((size_t)n_rows * (in_dim / 32) * 40 + 255) & ~(size_t)255;
    if (scratch_bytes < (size_t)n_rows * (in_dim / 32) * 40)
        return fail(REIN_E_BAD_SHAPE, "rein_matmul_ws: scratch smaller than the quantized activations");
    // nothing behind the activations that a workspace launch could use: the plain dispatch
    const size_t least = rein_mmq_workspace_min_bytes(fmt, in_dim, n_rows);
    if (rein_matmul_path(fmt, n_rows) != 2 || rein_mmq_workspace_bytes(fmt, in_dim, n_rows) == 0 ||
        scratch_bytes < xq + std::max<size_t>(least, 16))
        return rein_matmul(fmt, w, x, y, in_dim, out_dim, n_rows, scratch, s);
    if (int rc = rein_quantize_q8(x, scratch, in_dim, n_rows, s)) return rc;
    return rein_mmq_xq8_ws(fmt, w, scratch, y, in_dim, out_dim, n_rows, static_cast<char*>(scratch) + xq, scratch_bytes - xq, s);
}

int rein_block_dot_parts(int fmt) { return fmt == REIN_TYPE_Q6_K ? 2 : (rein_block_size(fmt) ? 1 : 0); }

int rein_block_dots(int fmt, const void* w, const void* xq, int32_t* out, unsigned in_dim, unsigned out_dim,
                    unsigned n_rows, int via_mfma, rein_stream_t s)
{
    const char* who = "rein_block_dots";
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_rows)) return rc;
    if (int rc = check_ptr(who, w, 16, "w")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, out, 4, "out")) return rc;
    if (n_rows > 65535) return fail(REIN_E_TOO_LARGE, "rein_block_dots: at most 65535 rows");
    if (via_mfma) {
        if (int rc = check_dense_fmt(who, fmt)) return rc;
        const std::string name = std::string("rein_mmq_dots_") + fmt_tag(fmt);
        void* args[] = {(void*)&w, (void*)&xq, (void*)&out, (void*)&in_dim, (void*)&out_dim, (void*)&n_rows};
        return launch(name, (out_dim + 127) / 128, (n_rows + 31) / 32, 1, 256, 0, s, args);
    }
    const std::string name = std::string("rein_block_dots_") + fmt_tag(fmt);
    void* args[] = {(void*)&w, (void*)&xq, (void*)&out, (void*)&in_dim, (void*)&out_dim};
    return launch(name, out_dim < 4096 ? out_dim : 4096, n_rows, 1, 64, 0, s, args);
}

// ------------------------------------------------------------------------ MoE

unsigned rein_moe_gemm_bn(void) { return 32; }

int rein_moe_topk(const float* logits, unsigned n_tok, unsigned n_expert, unsigned n_used, int32_t* out_ids,
                  float* out_weights, rein_stream_t s)
{
    if (n_tok == 0 || n_expert == 0 || n_used == 0 || n_used > 64 || n_used > n_expert)
        return fail(REIN_E_BAD_SHAPE, "rein_moe_topk: need n_tok > 0 and 1 <= n_used <= min(64, n_expert)");
    if (n_expert > 12288) return fail(REIN_E_TOO_LARGE, "rein_moe_topk: at most 12288 experts (LDS)");
    if (int rc = check_ptr("rein_moe_topk", logits, 4, "logits")) return rc;
    if (int rc = check_ptr("rein_moe_topk", out_ids, 4, "out_ids")) return rc;
    if (int rc = check_ptr("rein_moe_topk", out_weights, 4, "out_weights")) return rc;
    int ne = (int)n_expert, nu = (int)n_used;
    if (n_expert <= 256 && opt_u(O_TOPK_WAVE, 1) != 0) {
        // one wavefront per token, the tree's decisions as register reductions (no LDS, no barrier): the same ids
        // and weight bits as moe_topk_f32
        int nt = (int)n_tok;
        void* a[] = {(void*)&logits, (void*)&ne, (void*)&nu, (void*)&out_ids, (void*)&out_weights, (void*)&nt};
        return launch("rein_moe_topk_wave", (n_tok + 3) / 4, 1, 1, 256, 0, s, a);
    }
    void* args[] = {(void*)&logits, (void*)&ne, (void*)&nu, (void*)&out_ids, (void*)&out_weights};
    return launch("moe_topk_f32", n_tok, 1, 1, 128, n_expert * 4, s, args);
}

namespace {
// Small routing tables are sorted by one workgroup (one launch instead of four or five): the
// 4096 entries of 512 tokens x top-8 take it ~5 us, about one launch of the split form.
bool moe_sort_in_one_block(unsigned n_entries, unsigned n_expert)
{
    return n_entries <= 32768 && n_expert <= 2048 && opt_u(O_MOE_SORT_SPLIT, 0) == 0;
}
}  // namespace

int rein_moe_sort(const int32_t* ids, unsigned n_entries, unsigned n_expert, unsigned bn, int32_t* count,
                  int32_t* cursor, int32_t* perm, int32_t* expert_off, int32_t* tile_off, rein_stream_t s)
{
    if (n_entries == 0 || n_expert == 0 || bn == 0)
        return fail(REIN_E_BAD_SHAPE, "rein_moe_sort: n_entries, n_expert and bn must be non-zero");
    const void* ptrs[] = {ids, count, cursor, perm, expert_off, tile_off};
    for (const void* p : ptrs)
        if (int rc = check_ptr("rein_moe_sort", p, 4, "buffer")) return rc;
    if (moe_sort_in_one_block(n_entries, n_expert)) {
        // cursor is left as it is: the rank counters of the one-workgroup sort live in LDS
        int32_t* inv = nullptr;
        void* a[] = {(void*)&ids, (void*)&count, (void*)&expert_off, (void*)&tile_off, (void*)&perm, (void*)&inv,
                     (void*)&n_entries, (void*)&n_expert, (void*)&bn};
        return launch("rein_moe_sort_one_block", 1, 1, 1, 1024, 0, s, a);
    }
    const unsigned ge = (n_expert + 255) / 256, gn = (n_entries + 255) / 256;
    {
        void* a[] = {(void*)&count, (void*)&n_expert};
        if (int rc = launch("moe_sort_zero", ge, 1, 1, 256, 0, s, a)) return rc;
    }
    {
        void* a[] = {(void*)&ids, (void*)&count, (void*)&n_entries, (void*)&n_expert};
        if (int rc = launch("moe_sort_histogram", gn, 1, 1, 256, 0, s, a)) return rc;
    }
    {
        void* a[] = {(void*)&count, (void*)&expert_off, (void*)&tile_off, (void*)&n_expert, (void*)&bn};
        if (int rc = launch("moe_sort_scan", 1, 1, 1, 64, 0, s, a)) return rc;
    }
    {
        void* a[] = {(void*)&cursor, (void*)&n_expert};
        if (int rc = launch("moe_sort_zero", ge, 1, 1, 256, 0, s, a)) return rc;
    }
    void* a[] = {(void*)&ids, (void*)&expert_off, (void*)&cursor, (void*)&perm, (void*)&n_entries, (void*)&n_expert};
    return launch("moe_sort_scatter", gn, 1, 1, 256, 0, s, a);
}

int rein_moe_gather_xq(const void* xq_src, const int32_t* perm, void* xq_dst, unsigned nsub, unsigned n_used,
                       unsigned n_entries, rein_stream_t s)
{
    if (nsub == 0 || n_used == 0 || n_entries == 0) return fail(REIN_E_BAD_SHAPE, "rein_moe_gather_xq: zero dimension");
    if (int rc = check_ptr("rein_moe_gather_xq", xq_src, 8, "xq_src")) return rc;
    if (int rc = check_ptr("rein_moe_gather_xq", xq_dst, 8, "xq_dst")) return rc;
    if (int rc = check_ptr("rein_moe_gather_xq", perm, 4, "perm")) return rc;
    const unsigned gx = (nsub * 5 + 255) / 256, gy = n_entries < 65535 ? n_entries : 65535;
    void* a[] = {(void*)&xq_src, (void*)&perm, (void*)&xq_dst, (void*)&nsub, (void*)&n_used, (void*)&n_entries};
    return launch("moe_gather_xq", gx, gy, 1, 256, 0, s, a);
}

int rein_moe_quantize_scatter(const float* x, const int32_t* inv, void* xq_dst, unsigned in_dim, unsigned n_used,
                              unsigned n_tok, rein_stream_t s)
{
    const char* who = "rein_moe_quantize_scatter";
    if (in_dim == 0 || in_dim % 32 != 0 || n_used == 0 || n_tok == 0)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": in_dim must be a non-zero multiple of 32, the counts non-zero");
    if (n_tok > 65535) return fail(REIN_E_TOO_LARGE, std::string(who) + ": at most 65535 tokens per call");
    if (int rc = check_ptr(who, x, 4, "x")) return rc;
    if (int rc = check_ptr(who, inv, 4, "inv")) return rc;
    if (int rc = check_ptr(who, xq_dst, 8, "xq_dst")) return rc;
    const unsigned gx = (in_dim + 511) / 512;
    const unsigned n_entries = n_tok * n_used;
    void* a[] = {(void*)&x, (void*)&inv, (void*)&xq_dst, (void*)&in_dim, (void*)&n_used, (void*)&n_entries};
    return launch("rein_moe_quantize_scatter", gx, n_tok, 1, 256, 0, s, a);
}

int rein_moe_scatter_rows(const float* src, const int32_t* perm, float* dst, unsigned dim, unsigned n_entries,
                          rein_stream_t s)
{
    if (dim == 0 || n_entries == 0) return fail(REIN_E_BAD_SHAPE, "rein_moe_scatter_rows: zero dimension");
    if (int rc = check_ptr("rein_moe_scatter_rows", src, 4, "src")) return rc;
    if (int rc = check_ptr("rein_moe_scatter_rows", dst, 4, "dst")) return rc;
    if (int rc = check_ptr("rein_moe_scatter_rows", perm, 4, "perm")) return rc;
    const unsigned gx = (dim + 255) / 256, gy = n_entries < 65535 ? n_entries : 65535;
    void* a[] = {(void*)&src, (void*)&perm, (void*)&dst, (void*)&dim, (void*)&n_entries};
    return launch("moe_scatter_rows", gx, gy, 1, 256, 0, s, a);
}

int rein_moe_grouped_gemm(int fmt, const void* slab, unsigned bytes_per_expert, const int32_t* expert_off,
                          const int32_t* tile_off, unsigned n_expert, const void* xq, float* y, unsigned in_dim,
                          unsigned out_dim, unsigned n_entries, rein_stream_t s)
{
    const char* who = "rein_moe_grouped_gemm";
    if (!rein_ingest_expert_format(fmt))
        return fail(REIN_E_BAD_FORMAT, std::string(who) + ": formats are Q4_K, Q5_K, Q6_K, Q8_0, Q5_1");
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_entries)) return rc;
    if (n_expert == 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": n_expert is zero");
    if (bytes_per_expert % 16 != 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": bytes_per_expert must be a multiple of 16");
    if (int rc = check_ptr(who, slab, 16, "slab")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, y, 4, "y")) return rc;
    if (int rc = check_ptr(who, expert_off, 4, "expert_off")) return rc;
    if (int rc = check_ptr(who, tile_off, 4, "tile_off")) return rc;
    return launch_grouped(fmt, slab, nullptr, bytes_per_expert, expert_off, tile_off, n_expert, xq, y, nullptr, in_dim,
                          out_dim, n_entries, s);
}

// Gate + up + SwiGLU + BlockQ8 in one launch (rein_mmq_<fmt>_grouped_swiglu_q8): the grid is
// 8 * ceil(tile_ub / 8) * ceil(out_dim / 64) workgroups, tile_ub as in launch_grouped.
int rein_moe_grouped_swiglu_q8(int fmt, const void* gate_slab, const void* up_slab, unsigned bytes_per_expert,
                               const int32_t* expert_off, const int32_t* tile_off, unsigned n_expert, const void* xq,
                               void* xq_out, unsigned in_dim, unsigned out_dim, unsigned n_entries, rein_stream_t s)
{
    const char* who = "rein_moe_grouped_swiglu_q8";
    if (fmt != REIN_TYPE_Q4_K && fmt != REIN_TYPE_Q5_K && fmt != REIN_TYPE_Q6_K && fmt != REIN_TYPE_Q8_0)
        return fail(REIN_E_BAD_FORMAT, std::string(who) + ": formats are Q4_K, Q5_K, Q6_K, Q8_0");
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_entries)) return rc;
    if (n_expert == 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": n_expert is zero");
    if (out_dim % 32 != 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": out_dim must be a multiple of 32 (whole BlockQ8 blocks)");
    if (bytes_per_expert % 16 != 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": bytes_per_expert must be a multiple of 16");
    if (int rc = check_ptr(who, gate_slab, 16, "gate_slab")) return rc;
    if (int rc = check_ptr(who, up_slab, 16, "up_slab")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, xq_out, 8, "xq_out")) return rc;
    if (int rc = check_ptr(who, expert_off, 4, "expert_off")) return rc;
    if (int rc = check_ptr(who, tile_off, 4, "tile_off")) return rc;
    const unsigned bn = rein_moe_gemm_bn();
    const unsigned tile_ub = (n_entries + bn - 1) / bn + n_expert;
    const unsigned long long grid = 8ull * ((tile_ub + 7) / 8) * ((out_dim + 63) / 64);
    if (grid > 0x7FFFFFFFull) return fail(REIN_E_TOO_LARGE, std::string(who) + ": more than 2^31 workgroup tiles");
    void* a[] = {(void*)&gate_slab, (void*)&up_slab, (void*)&bytes_per_expert, (void*)&expert_off, (void*)&tile_off,
                 (void*)&n_expert, (void*)&xq, (void*)&xq_out, (void*)&in_dim, (void*)&out_dim};
    return launch(std::string("rein_mmq_") + fmt_tag(fmt) + "_grouped_swiglu_q8", (unsigned)grid, 1, 1, 256, 0, s, a);
}

namespace {
int moe_mv_launch(const char* who, const std::string& kernel, unsigned rows_per_block, int fmt, const void* slab0,
                  const void* slab1, const int32_t* ids, const void* xq, float* y, unsigned in_dim, unsigned out_dim,
                  unsigned bytes_per_expert, unsigned xq_tok_stride, unsigned xq_slot_stride, unsigned n_used,
                  unsigned n_tok, rein_stream_t s)
{
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_tok)) return rc;
    if (n_used == 0 || n_used > 65535 || n_tok > 65535)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": n_used and n_tok must be in 1..65535");
    if (bytes_per_expert < rein_repacked_len(fmt, in_dim, out_dim))
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": bytes_per_expert is smaller than one repacked expert");
    if (int rc = check_ptr(who, slab0, 16, "slab")) return rc;
    if (slab1) if (int rc = check_ptr(who, slab1, 16, "up_slab")) return rc;
    if (bytes_per_expert % 16 != 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": bytes_per_expert must be a multiple of 16");
    if (int rc = check_ptr(who, ids, 4, "ids")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, y, 4, "y")) return rc;
    const unsigned gx = (out_dim + rows_per_block - 1) / rows_per_block;
    if (slab1) {
        void* a[] = {(void*)&slab0, (void*)&slab1, (void*)&ids, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim,
                     (void*)&bytes_per_expert, (void*)&xq_tok_stride, (void*)&xq_slot_stride, (void*)&n_used};
        return launch(kernel, gx, n_used, n_tok, 256, 0, s, a);
    }
    void* a[] = {(void*)&slab0, (void*)&ids, (void*)&xq, (void*)&y, (void*)&in_dim, (void*)&out_dim,
                 (void*)&bytes_per_expert, (void*)&xq_tok_stride, (void*)&xq_slot_stride, (void*)&n_used};
    return launch(kernel, gx, n_used, n_tok, 256, 0, s, a);
}
bool moe_mv_fmt(int fmt) { return rein_ingest_expert_format(fmt) != 0; }       // Q4_K, Q5_K, Q6_K, Q8_0, Q5_1
}  // namespace

int rein_moe_expert_matvec(int fmt, const void* slab, const int32_t* ids, const void* xq, float* y, unsigned in_dim,
                           unsigned out_dim, unsigned bytes_per_expert, unsigned xq_tok_stride,
                           unsigned xq_slot_stride, unsigned n_used, unsigned n_tok, rein_stream_t s)
{
    const char* who = "rein_moe_expert_matvec";
    if (!moe_mv_fmt(fmt)) return fail(REIN_E_BAD_FORMAT, std::string(who) + ": formats are Q4_K, Q5_K, Q6_K, Q8_0, Q5_1");
    // 4 wavefronts x 2 rows per 256-thread workgroup (the reference's grid, qwen35.rs:3086)
    return moe_mv_launch(who, std::string("moe_matvec_") + fmt_tag(fmt) + "_repacked_f32", 8, fmt, slab, nullptr, ids, xq,
                         y, in_dim, out_dim, bytes_per_expert, xq_tok_stride, xq_slot_stride, n_used, n_tok, s);
}

int rein_moe_down(int fmt, const void* slab, const int32_t* ids, const void* xq, float* y, unsigned in_dim,
                  unsigned out_dim, unsigned bytes_per_expert, unsigned xq_tok_stride, unsigned xq_slot_stride,
                  unsigned n_used, unsigned n_tok, rein_stream_t s)
{
    const char* who = "rein_moe_down";
    if (!moe_mv_fmt(fmt)) return fail(REIN_E_BAD_FORMAT, std::string(who) + ": formats are Q4_K, Q5_K, Q6_K, Q8_0, Q5_1");
    if (in_dim / 32 > 32)       // long contraction: the full-wavefront mapping wastes nothing
        return rein_moe_expert_matvec(fmt, slab, ids, xq, y, in_dim, out_dim, bytes_per_expert, xq_tok_stride,
                                      xq_slot_stride, n_used, n_tok, s);
    const std::string kernel = fmt == REIN_TYPE_Q4_K   ? "rein_moe_matvec_q4k_down_f32"
                               : fmt == REIN_TYPE_Q8_0 ? "moe_matvec_q8_0_repacked_down_f32"
                                                       : std::string("moe_matvec_") + fmt_tag(fmt) + "_down_f32";
    // 8 half-wavefronts x 2 rows per workgroup
    return moe_mv_launch(who, kernel, 16, fmt, slab, nullptr, ids, xq, y, in_dim, out_dim, bytes_per_expert,
                         xq_tok_stride, xq_slot_stride, n_used, n_tok, s);
}

int rein_moe_gate_up_swiglu(int fmt, const void* gate_slab, const void* up_slab, const int32_t* ids, const void* xq,
                            float* y, unsigned in_dim, unsigned out_dim, unsigned bytes_per_expert,
                            unsigned xq_tok_stride, unsigned xq_slot_stride, unsigned n_used, unsigned n_tok,
                            rein_stream_t s)
{
    const char* who = "rein_moe_gate_up_swiglu";
    if (fmt != REIN_TYPE_Q4_K) return fail(REIN_E_BAD_FORMAT, std::string(who) + ": the fused form exists for Q4_K experts");
    if (!up_slab) return fail(REIN_E_BAD_POINTER, std::string(who) + ": up_slab is NULL");
    return moe_mv_launch(who, "moe_gate_up_swiglu_q4k_repacked_f32", 8, fmt, gate_slab, up_slab, ids, xq, y, in_dim,
                         out_dim, bytes_per_expert, xq_tok_stride, xq_slot_stride, n_used, n_tok, s);
}

int rein_moe_gate_up_swiglu_q8(int fmt, const void* gate_slab, const void* up_slab, const int32_t* ids, const void* xq,
                               void* xq_out, unsigned in_dim, unsigned out_dim, unsigned bytes_per_expert,
                               unsigned xq_tok_stride, unsigned xq_slot_stride, unsigned n_used, unsigned n_tok,
                               rein_stream_t s)
{
    const char* who = "rein_moe_gate_up_swiglu_q8";
    if (!moe_mv_fmt(fmt)) return fail(REIN_E_BAD_FORMAT, std::string(who) + ": formats are Q4_K, Q5_K, Q6_K, Q8_0, Q5_1");
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_tok)) return rc;
    if (out_dim % 32 != 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": out_dim must be a multiple of 32 (whole BlockQ8 blocks)");
    if (n_used == 0 || n_used > 65535 || n_tok > 65535)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": n_used and n_tok must be in 1..65535");
    if (bytes_per_expert < rein_repacked_len(fmt, in_dim, out_dim))
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": bytes_per_expert is smaller than one repacked expert");
    if (bytes_per_expert % 16 != 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": bytes_per_expert must be a multiple of 16");
    if (int rc = check_ptr(who, gate_slab, 16, "gate_slab")) return rc;
    if (int rc = check_ptr(who, up_slab, 16, "up_slab")) return rc;
    if (int rc = check_ptr(who, ids, 4, "ids")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, xq_out, 8, "xq_out")) return rc;
    void* a[] = {(void*)&gate_slab, (void*)&up_slab, (void*)&ids, (void*)&xq, (void*)&xq_out, (void*)&in_dim, (void*)&out_dim,
                 (void*)&bytes_per_expert, (void*)&xq_tok_stride, (void*)&xq_slot_stride, (void*)&n_used};
    // two rows per wavefront (1024 threads per 32 outputs) or four (512): four once the launch is two workgroups
    // per CU -- more bytes in flight per lane, half the wavefronts to start; 128 experts top-8, 2048 -> 768 at
    // 4 / 8 / 16 tokens 32.9 / 51.9 / 88.4 us per FFN against 34.1 / 55.9 / 99.3, one token 16.9 against 15.9
    const unsigned gu_rows = opt_u(O_MOE_GU_ROWS, 0);
    const bool r4 = gu_rows == 4 || (gu_rows != 2 && (unsigned long long)(out_dim / 32) * n_used * n_tok >= 2ull * kCUs);
    return launch(std::string("rein_moe_gate_up_swiglu_q8_") + fmt_tag(fmt) + (r4 ? "_r4" : ""), out_dim / 32, n_used, n_tok, r4 ? 512 : 1024, 0, s, a);
}

int rein_moe_down_combine(int fmt, const void* slab, const int32_t* ids, const float* weights, const float* down_exps_s,
                          const void* xq, float* out, unsigned in_dim, unsigned out_dim, unsigned bytes_per_expert,
                          unsigned xq_tok_stride, unsigned xq_slot_stride, unsigned n_used, unsigned n_tok, rein_stream_t s)
{
    const char* who = "rein_moe_down_combine";
    if (!moe_mv_fmt(fmt)) return fail(REIN_E_BAD_FORMAT, std::string(who) + ": formats are Q4_K, Q5_K, Q6_K, Q8_0, Q5_1");
    if (int rc = check_shape(who, fmt, in_dim, out_dim, n_tok)) return rc;
    if (n_used == 0 || n_used > 65535 || n_tok > 65535)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": n_used and n_tok must be in 1..65535");
    if (bytes_per_expert < rein_repacked_len(fmt, in_dim, out_dim))
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": bytes_per_expert is smaller than one repacked expert");
    if (bytes_per_expert % 16 != 0) return fail(REIN_E_BAD_SHAPE, std::string(who) + ": bytes_per_expert must be a multiple of 16");
    if (int rc = check_ptr(who, slab, 16, "slab")) return rc;
    if (int rc = check_ptr(who, ids, 4, "ids")) return rc;
    if (int rc = check_ptr(who, weights, 4, "weights")) return rc;
    if (int rc = check_ptr(who, down_exps_s, 4, "down_exps_s")) return rc;
    if (int rc = check_ptr(who, xq, 8, "xq")) return rc;
    if (int rc = check_ptr(who, out, 4, "out")) return rc;
    // A workgroup owns `rows` rows, one team per slot: half-wavefront teams for contractions of at most 32
    // sub-blocks, whole wavefronts otherwise; as many teams as slots, up to 512 threads.  rows = the most of 8, 4, 2
    // that leaves four workgroups per CU (REIN_MOE_DC_ROWS forces it); every choice gives the same bits.
    const bool half = in_dim / 32 <= 32;
    const unsigned lanes = half ? 32 : 64;
    unsigned threads = ((n_used * lanes + 63) / 64) * 64;
    if (threads > 512) threads = 512;
    unsigned rows = opt_u(O_MOE_DC_ROWS, 0);
    if (rows != 2 && rows != 4 && rows != 8) {
        rows = 8;
        while (rows > 2 && (unsigned long long)((out_dim + rows - 1) / rows) * n_tok < 4ull * kCUs) rows /= 2;
    }
    void* a[] = {(void*)&slab, (void*)&ids, (void*)&weights, (void*)&down_exps_s, (void*)&xq, (void*)&out, (void*)&in_dim,
                 (void*)&out_dim, (void*)&bytes_per_expert, (void*)&xq_tok_stride, (void*)&xq_slot_stride, (void*)&n_used};
    return launch(std::string("rein_moe_down_combine_") + fmt_tag(fmt) + (half ? "_h" : "") + (rows == 2 ? "" : rows == 4 ? "_r4" : "_r8"),
                  (out_dim + rows - 1) / rows, 1, n_tok, threads, 0, s, a);
}

int rein_swiglu_mul(const float* gate, const float* up, float* out, unsigned n, rein_stream_t s)
{
    if (n == 0) return fail(REIN_E_BAD_SHAPE, "rein_swiglu_mul: n is zero");
    if (int rc = check_ptr("rein_swiglu_mul", gate, 4, "gate")) return rc;
    if (int rc = check_ptr("rein_swiglu_mul", up, 4, "up")) return rc;
    if (int rc = check_ptr("rein_swiglu_mul", out, 4, "out")) return rc;
    unsigned g = (n + 255) / 256;
    if (g > kCUs * 32) g = kCUs * 32;
    void* a[] = {(void*)&gate, (void*)&up, (void*)&out, (void*)&n};
    return launch("swiglu_mul_f32", g, 1, 1, 256, 0, s, a);
}

int rein_moe_combine(const float* experts, const int32_t* ids, const float* weights, const float* down_exps_s,
                     float* out, unsigned n_tok, unsigned hidden, unsigned n_used, rein_stream_t s)
{
    if (n_tok == 0 || hidden == 0 || n_used == 0) return fail(REIN_E_BAD_SHAPE, "rein_moe_combine: zero dimension");
    if (n_tok > 65535) return fail(REIN_E_TOO_LARGE, "rein_moe_combine: at most 65535 tokens per call");
    const void* ptrs[] = {experts, ids, weights, down_exps_s, out};
    for (const void* p : ptrs)
        if (int rc = check_ptr("rein_moe_combine", p, 4, "buffer")) return rc;
    void* a[] = {(void*)&experts, (void*)&ids, (void*)&weights, (void*)&down_exps_s, (void*)&out, (void*)&hidden, (void*)&n_used};
    return launch("moe_combine_f32", (hidden + 255) / 256, n_tok, 1, 256, 0, s, a);
}

// Workspace carve-up for rein_moe_ffn (all offsets 256-byte aligned).
namespace {
struct MoeWs {
    size_t ids, weights, count, cursor, perm, inv, eoff, toff, xq_in, g_in, e_gate, e_up, xq_exp, g_out, total;
};
size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }
MoeWs moe_ws(const rein_moe_shape& sh)
{
    const size_t ne = (size_t)sh.n_tok * sh.n_used;
    MoeWs w;
    size_t o = 0;
    auto take = [&](size_t bytes) { const size_t at = o; o += up256(bytes); return at; };
    w.ids     = take(ne * 4);
    w.weights = take(ne * 4);
    w.count   = take((size_t)sh.n_expert * 4);
    w.cursor  = take((size_t)sh.n_expert * 4);
    w.perm    = take(ne * 4);
    w.inv     = take(ne * 4);
    w.eoff    = take(((size_t)sh.n_expert + 1) * 4);
    w.toff    = take(((size_t)sh.n_expert + 1) * 4);
    w.xq_in   = take((size_t)sh.n_tok * (sh.hidden / 32) * 40);
    w.g_in    = take(ne * (sh.hidden / 32) * 40);
    w.e_gate  = take(ne * sh.expert_ff * 4);
    w.e_up    = take(ne * sh.expert_ff * 4);
    w.xq_exp  = take(ne * (sh.expert_ff / 32) * 40);
    w.g_out   = take(ne * sh.hidden * 4);
    w.total   = o;
    return w;
}
}  // namespace

size_t rein_moe_workspace_bytes(const rein_moe_shape* sh)
{
    if (!sh) return 0;
    return moe_ws(*sh).total;
}

int rein_moe_ffn(const rein_moe_shape* shp, const float* x, const float* logits, const void* gate_exps,
                 const void* up_exps, const void* down_exps, const float* down_exps_s, void* workspace,
                 float* out, rein_stream_t s)
{
    const char* who = "rein_moe_ffn";
    if (!shp) return fail(REIN_E_BAD_POINTER, std::string(who) + ": shape is NULL");
    const rein_moe_shape sh = *shp;
    if (sh.n_tok == 0 || sh.hidden == 0 || sh.n_expert == 0 || sh.n_used == 0 || sh.expert_ff == 0)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": zero dimension");
    if (int rc = check_shape(who, sh.gate_up_fmt, sh.hidden, sh.expert_ff, sh.n_tok)) return rc;
    if (int rc = check_shape(who, sh.down_fmt, sh.expert_ff, sh.hidden, sh.n_tok)) return rc;
    if (int rc = check_ptr(who, workspace, 256, "workspace")) return rc;
    if (!moe_mv_fmt(sh.gate_up_fmt) || !moe_mv_fmt(sh.down_fmt))
        return fail(REIN_E_BAD_FORMAT, std::string(who) + ": expert formats are Q4_K, Q5_K, Q6_K, Q8_0");
    if (sh.n_tok > 65535) return fail(REIN_E_TOO_LARGE, std::string(who) + ": at most 65535 tokens per call");
    if (int rc = check_ptr(who, x, 4, "x")) return rc;
    if (int rc = check_ptr(who, logits, 4, "logits")) return rc;
    if (int rc = check_ptr(who, gate_exps, 16, "gate_exps")) return rc;
    if (int rc = check_ptr(who, up_exps, 16, "up_exps")) return rc;
    if (int rc = check_ptr(who, down_exps, 16, "down_exps")) return rc;
    if (int rc = check_ptr(who, down_exps_s, 4, "down_exps_s")) return rc;
    if (int rc = check_ptr(who, out, 4, "out")) return rc;
    const size_t bpe_gu = rein_repacked_len(sh.gate_up_fmt, sh.hidden, sh.expert_ff);
    const size_t bpe_dn = rein_repacked_len(sh.down_fmt, sh.expert_ff, sh.hidden);
    if (bpe_gu > 0xFFFFFFFFull || bpe_dn > 0xFFFFFFFFull)
        return fail(REIN_E_TOO_LARGE, std::string(who) + ": an expert slab must stay below 4 GiB");   // u32, qwen35.rs:3052
    if (bpe_gu % 16 != 0 || bpe_dn % 16 != 0)
        return fail(REIN_E_BAD_SHAPE, std::string(who) + ": expert slabs must be multiples of 16 bytes (hidden and expert_ff multiples of 8 rows)");

    const MoeWs w = moe_ws(sh);
    char* base = static_cast<char*>(workspace);
    int32_t* ids = (int32_t*)(base + w.ids);
    float* weights = (float*)(base + w.weights);
    int32_t* perm = (int32_t*)(base + w.perm);
    int32_t* eoff = (int32_t*)(base + w.eoff);
    int32_t* toff = (int32_t*)(base + w.toff);
    const unsigned ne = sh.n_tok * sh.n_used;

    // Few tokens: with about one routing entry per expert nearly every entry meets an expert of its own, a
    // 32-token tile of the grouped GEMM holds one or two tokens, and the sort is pure overhead.  The decode kernels
    // (qwen35.rs:3071-3167, here in their two fused launches) read an expert per entry -- streaming, where a
    // mostly empty tile pays its full matrix work -- and are ahead up to 1.6 entries per expert: 128 experts top-8
    // at 1 / 4 / 16 / 24 tokens 16 / 33 / 89 / 125 us against 48 / 61 / 126 / 141 for the pipeline below, at 28
    // tokens 141 against 143, at 32 tokens 160 against 145.  Same integer dots, fp32 sums in the decode kernels' order.
    const bool chain = 5ull * ne <= 8ull * sh.n_expert && sh.expert_ff % 32 == 0 && opt_u(O_MOE_CHAIN, 1) != 0;
    if (chain) {
        const unsigned ns_h = sh.hidden / 32, ns_f = sh.expert_ff / 32;
        // Where the one-wavefront router applies it shares a launch: for one or two tokens the gate / up launch
        // routes and quantizes its token itself (every workgroup again: 15.9 / 23.8 us against 17.3 / 25.4), beyond
        // that router and quantizer run as one small launch in front (16 tokens: 105 us against 111)
        const bool wave = sh.n_expert <= 256 && sh.n_used <= 64 && sh.n_used <= sh.n_expert && opt_u(O_TOPK_WAVE, 1) != 0;
        const bool routed = wave && sh.n_tok <= 2 && ns_h * 40u <= 48u * 1024u;
        if (routed) {
            void* xq_exp = base + w.xq_exp;
            const unsigned bpe = (unsigned)bpe_gu;
            void* a[] = {(void*)&gate_exps, (void*)&up_exps, (void*)&logits, (void*)&x, (void*)&ids, (void*)&weights, (void*)&xq_exp,
                         (void*)&sh.hidden, (void*)&sh.expert_ff, (void*)&bpe, (void*)&sh.n_expert, (void*)&sh.n_used};
            const unsigned gu_rows = opt_u(O_MOE_GU_ROWS, 0);
            const bool r4 = gu_rows == 4 || (gu_rows != 2 && (unsigned long long)(sh.expert_ff / 32) * sh.n_used * sh.n_tok >= 2ull * kCUs);
            if (int rc = launch(std::string("rein_moe_route_gate_up_swiglu_q8_") + fmt_tag(sh.gate_up_fmt) + (r4 ? "_r4" : ""), sh.expert_ff / 32,
                                sh.n_used, sh.n_tok, r4 ? 512 : 1024, ns_h * 40u, s, a)) return rc;
        } else {
            if (wave) {
                int n_e = (int)sh.n_expert, n_u = (int)sh.n_used, n_t = (int)sh.n_tok;
                void* xq = base + w.xq_in;
                unsigned q_per_tok = (sh.hidden + 511) / 512;
                void* a[] = {(void*)&logits, (void*)&n_e, (void*)&n_u, (void*)&ids, (void*)&weights, (void*)&n_t,
                             (void*)&x, (void*)&xq, (void*)&sh.hidden, (void*)&q_per_tok};
                if (int rc = launch("rein_moe_route_quantize", (sh.n_tok + 3) / 4 + sh.n_tok * q_per_tok, 1, 1, 256, 0, s, a)) return rc;
            } else {
                if (int rc = rein_moe_topk(logits, sh.n_tok, sh.n_expert, sh.n_used, ids, weights, s)) return rc;
                if (int rc = rein_quantize_q8(x, base + w.xq_in, sh.hidden, sh.n_tok, s)) return rc;
            }
            if (int rc = rein_moe_gate_up_swiglu_q8(sh.gate_up_fmt, gate_exps, up_exps, ids, base + w.xq_in, base + w.xq_exp, sh.hidden,
                                                    sh.expert_ff, (unsigned)bpe_gu, ns_h, 0, sh.n_used, sh.n_tok, s)) return rc;
        }
        return rein_moe_down_combine(sh.down_fmt, down_exps, ids, weights, down_exps_s, base + w.xq_exp, out, sh.expert_ff, sh.hidden,
                                     (unsigned)bpe_dn, sh.n_used * ns_f, ns_f, sh.n_used, sh.n_tok, s);
    }
    if (int rc = rein_moe_topk(logits, sh.n_tok, sh.n_expert, sh.n_used, ids, weights, s)) return rc;
    // counting sort by expert (moe_expert_sort.hip), with the inverse permutation kept so
    // that the combine can read the sorted expert outputs in place
    int32_t* count = (int32_t*)(base + w.count);
    int32_t* inv = (int32_t*)(base + w.inv);
    const unsigned bn = rein_moe_gemm_bn();
    if (moe_sort_in_one_block(ne, sh.n_expert)) {
        void* a[] = {(void*)&ids, (void*)&count, (void*)&eoff, (void*)&toff, (void*)&perm, (void*)&inv, (void*)&ne,
                     (void*)&sh.n_expert, (void*)&bn};
        if (int rc = launch("rein_moe_sort_one_block", 1, 1, 1, 1024, 0, s, a)) return rc;
    } else {
        int32_t* cursor = (int32_t*)(base + w.cursor);
        const unsigned zn = (unsigned)((w.cursor - w.count) / 4) + sh.n_expert;     // count .. cursor are adjacent
        const unsigned gn = (ne + 255) / 256;
        void* a0[] = {(void*)&count, (void*)&zn};
        if (int rc = launch("moe_sort_zero", (zn + 255) / 256, 1, 1, 256, 0, s, a0)) return rc;
        void* a1[] = {(void*)&ids, (void*)&count, (void*)&ne, (void*)&sh.n_expert};
        if (int rc = launch("moe_sort_histogram", gn, 1, 1, 256, 0, s, a1)) return rc;
        void* a2[] = {(void*)&count, (void*)&eoff, (void*)&toff, (void*)&sh.n_expert, (void*)&bn};
        if (int rc = launch("moe_sort_scan", 1, 1, 1, 64, 0, s, a2)) return rc;
        void* a3[] = {(void*)&ids, (void*)&eoff, (void*)&cursor, (void*)&perm, (void*)&inv, (void*)&ne, (void*)&sh.n_expert};
        if (int rc = launch("rein_moe_sort_scatter_inv", gn, 1, 1, 256, 0, s, a3)) return rc;
    }
    // the expert-sorted BlockQ8 rows straight from x (quantize_q8 + moe_gather_xq in one launch)
    if (int rc = rein_moe_quantize_scatter(x, inv, base + w.g_in, sh.hidden, sh.n_used, sh.n_tok, s)) return rc;
    // gate and up projections, SwiGLU and the down projection's BlockQ8 rows in one launch;
    // REIN_MOE_FUSED=0 takes the two-output GEMM and swiglu_q8_f32 instead (the same bytes)
    const unsigned long long fused_grid = 8ull * (((ne + bn - 1) / bn + sh.n_expert + 7) / 8) * ((sh.expert_ff + 63) / 64);
    if (sh.expert_ff % 32 == 0 && fused_grid <= 0x7FFFFFFFull && opt_u(O_MOE_FUSED, 1) != 0) {
        if (int rc = rein_moe_grouped_swiglu_q8(sh.gate_up_fmt, gate_exps, up_exps, (unsigned)bpe_gu, eoff, toff, sh.n_expert,
                                                base + w.g_in, base + w.xq_exp, sh.hidden, sh.expert_ff, ne, s)) return rc;
    } else {
    // gate and up projections in one launch (two slabs)
    if (int rc = launch_grouped(sh.gate_up_fmt, gate_exps, up_exps, (unsigned)bpe_gu, eoff, toff, sh.n_expert, base + w.g_in,
                                (float*)(base + w.e_gate), (float*)(base + w.e_up), sh.hidden, sh.expert_ff, ne, s)) return rc;
    // SwiGLU straight into the down projection's BlockQ8 rows (rows are expert_ff long,
    // a multiple of 32, so the flat array quantizes as one vector)
    for (size_t e0 = 0; e0 < (size_t)ne * sh.expert_ff; e0 += (size_t)1 << 30) {
        const size_t left = (size_t)ne * sh.expert_ff - e0;
        const unsigned cnt = (unsigned)std::min(left, (size_t)1 << 30);
        if (int rc = rein_swiglu_q8((float*)(base + w.e_gate) + e0, (float*)(base + w.e_up) + e0, nullptr,
                                    base + w.xq_exp + e0 / 32 * 40, cnt, s)) return rc;
    }
    }
    if (int rc = rein_moe_grouped_gemm(sh.down_fmt, down_exps, (unsigned)bpe_dn, eoff, toff, sh.n_expert,
                                       base + w.xq_exp, (float*)(base + w.g_out), sh.expert_ff, sh.hidden, ne, s)) return rc;
    // scatter + weighted combine in one pass over the sorted rows
    {
        const float* sorted = (const float*)(base + w.g_out);
        const int32_t* inv = (const int32_t*)(base + w.inv);
        void* a[] = {(void*)&sorted, (void*)&inv, (void*)&ids, (void*)&weights, (void*)&down_exps_s, (void*)&out,
                     (void*)&sh.hidden, (void*)&sh.n_used};
        // four columns per thread where the rows allow 128-bit accesses (the same bits)
        if (sh.hidden % 4 == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)sorted & 15) == 0)
            return launch("rein_moe_combine_sorted4_f32", (sh.hidden / 4 + 127) / 128, sh.n_tok, 1, 128, 0, s, a);
        return launch("rein_moe_combine_sorted_f32", (sh.hidden + 255) / 256, sh.n_tok, 1, 256, 0, s, a);
    }
}

}  // extern "C"
