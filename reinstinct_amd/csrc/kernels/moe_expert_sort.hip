// MoE expert-routing counting sort, gather and scatter: same entry points and
// arguments as kernels/moe_expert_sort.cpp:27-110 of the reference.
//
//   moe_sort_zero       buf[0..n) = 0
//   moe_sort_histogram  count[e] = number of routing entries with ids[i] == e
//   moe_sort_scan       expert_off[e], tile_off[e] = exclusive prefix sums of
//                       count and ceil(count/bn); entry n_expert holds the totals
//   moe_sort_scatter    perm[expert_off[e] + rank] = i   (rank by atomic counter:
//                       the order inside one expert is not deterministic)
//   moe_gather_xq       xq_dst[p] = xq_src[perm[p] / n_used]   (rows of 40-byte blocks)
//   moe_scatter_rows    dst[perm[p]] = src[p]                  (rows of `dim` floats)
//
// Every kernel is a grid-stride loop, so any launch geometry is correct; the
// scan is one wavefront doing a DPP-free shuffle scan instead of a serial loop.
#include "rein_common.h"

extern "C" __global__ void moe_sort_zero(int* __restrict__ buf, unsigned int n)
{
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) buf[i] = 0;
}

extern "C" __global__ void moe_sort_histogram(const int* __restrict__ ids, int* __restrict__ count,
                                              unsigned int n_entries, unsigned int n_expert)
{
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n_entries; i += gridDim.x * blockDim.x) {
        const int e = ids[i];
        if (e >= 0 && (unsigned)e < n_expert) atomicAdd(&count[e], 1);
    }
}

// Inclusive scan over one wavefront.
__device__ __forceinline__ int rein_wave_scan_incl(int v, unsigned lane)
{
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(v, o);
        if (lane >= (unsigned)o) v += t;
    }
    return v;
}

// Only wavefront 0 of block 0 works (the reference launches one block of 64).
extern "C" __global__ void moe_sort_scan(const int* __restrict__ count, int* __restrict__ expert_off,
                                         int* __restrict__ tile_off, unsigned int n_expert,
                                         unsigned int bn)
{
    if (blockIdx.x != 0 || threadIdx.x >= 64) return;
    const unsigned lane = threadIdx.x;
    int ebase = 0, tbase = 0;
    for (unsigned e0 = 0; e0 < n_expert; e0 += 64) {
        const unsigned e = e0 + lane;
        const int c = e < n_expert ? count[e] : 0;
        const int t = (int)(((unsigned)c + bn - 1u) / bn);
        const int ce = rein_wave_scan_incl(c, lane);
        const int te = rein_wave_scan_incl(t, lane);
        if (e < n_expert) {
            expert_off[e] = ebase + ce - c;
            tile_off[e]   = tbase + te - t;
        }
        ebase += __shfl(ce, 63);
        tbase += __shfl(te, 63);
    }
    if (lane == 0) {
        expert_off[n_expert] = ebase;
        tile_off[n_expert]   = tbase;
    }
}

extern "C" __global__ void moe_sort_scatter(const int* __restrict__ ids, const int* __restrict__ expert_off,
                                            int* __restrict__ cursor, int* __restrict__ perm,
                                            unsigned int n_entries, unsigned int n_expert)
{
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n_entries; i += gridDim.x * blockDim.x) {
        const int e = ids[i];
        if (e < 0 || (unsigned)e >= n_expert) continue;
        const int rank = atomicAdd(&cursor[e], 1);
        perm[expert_off[e] + rank] = (int)i;
    }
}

// One 40-byte block = five 8-byte words per thread; blockIdx.y strides over entries.
extern "C" __global__ void moe_gather_xq(const unsigned char* __restrict__ xq_src, const int* __restrict__ perm,
                                         unsigned char* __restrict__ xq_dst, unsigned int nsub,
                                         unsigned int n_used, unsigned int n_entries)
{
    for (unsigned p = blockIdx.y; p < n_entries; p += gridDim.y) {
        const unsigned tok = (unsigned)perm[p] / n_used;
        const uint2* s = reinterpret_cast<const uint2*>(xq_src + (size_t)tok * nsub * 40);
        uint2*       d = reinterpret_cast<uint2*>(xq_dst + (size_t)p * nsub * 40);
        for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < nsub * 5; i += gridDim.x * blockDim.x) d[i] = s[i];
    }
}

extern "C" __global__ void moe_scatter_rows(const float* __restrict__ src, const int* __restrict__ perm,
                                            float* __restrict__ dst, unsigned int dim, unsigned int n_entries)
{
    for (unsigned p = blockIdx.y; p < n_entries; p += gridDim.y) {
        const float* s = src + (size_t)p * dim;
        float*       d = dst + (size_t)perm[p] * dim;
        for (unsigned c = blockIdx.x * blockDim.x + threadIdx.x; c < dim; c += gridDim.x * blockDim.x) d[c] = s[c];
    }
}

// moe_sort_scatter that also records where each routing entry went: inv[i] = position
// of entry i in the sorted order (perm[inv[i]] == i).  Lets the combine read the
// sorted expert outputs directly instead of through a scatter pass.
extern "C" __global__ void rein_moe_sort_scatter_inv(const int* __restrict__ ids, const int* __restrict__ expert_off,
                                                     int* __restrict__ cursor, int* __restrict__ perm,
                                                     int* __restrict__ inv, unsigned int n_entries,
                                                     unsigned int n_expert)
{
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n_entries; i += gridDim.x * blockDim.x) {
        const int e = ids[i];
        if (e < 0 || (unsigned)e >= n_expert) { inv[i] = -1; continue; }
        const int pos = expert_off[e] + atomicAdd(&cursor[e], 1);
        perm[pos] = (int)i;
        inv[i] = pos;
    }
}

// The whole counting sort in one workgroup of 1024 threads, for routing tables small enough
// that launches, not work, are what the four-kernel form costs (512 tokens x top-8 = 4096
// entries): histogram and rank counters live in LDS, wavefront 0 scans, the same threads
// scatter.  Writes count, expert_off, tile_off, perm and (if inv != nullptr) inv exactly as
// moe_sort_zero + moe_sort_histogram + moe_sort_scan + rein_moe_sort_scatter_inv would
// (the order inside one expert is as undetermined here as there).  n_expert <= 2048.
#define REIN_SORT1_MAX_EXPERT 2048
extern "C" __global__ __launch_bounds__(1024)
void rein_moe_sort_one_block(const int* __restrict__ ids, int* __restrict__ count, int* __restrict__ expert_off,
                             int* __restrict__ tile_off, int* __restrict__ perm, int* __restrict__ inv,
                             unsigned int n_entries, unsigned int n_expert, unsigned int bn)
{
    __shared__ int cnt[REIN_SORT1_MAX_EXPERT], off[REIN_SORT1_MAX_EXPERT], cur[REIN_SORT1_MAX_EXPERT];
    if (blockIdx.x != 0 || n_expert > REIN_SORT1_MAX_EXPERT) return;
    for (unsigned e = threadIdx.x; e < n_expert; e += blockDim.x) { cnt[e] = 0; cur[e] = 0; }
    __syncthreads();
    for (unsigned i = threadIdx.x; i < n_entries; i += blockDim.x) {
        const int e = ids[i];
        if (e >= 0 && (unsigned)e < n_expert) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        const unsigned lane = threadIdx.x;
        int ebase = 0, tbase = 0;
        for (unsigned e0 = 0; e0 < n_expert; e0 += 64) {
            const unsigned e = e0 + lane;
            const int c = e < n_expert ? cnt[e] : 0;
            const int t = (int)(((unsigned)c + bn - 1u) / bn);
            const int ce = rein_wave_scan_incl(c, lane);
            const int te = rein_wave_scan_incl(t, lane);
            if (e < n_expert) {
                off[e] = ebase + ce - c;
                count[e] = c;
                expert_off[e] = ebase + ce - c;
                tile_off[e]   = tbase + te - t;
            }
            ebase += __shfl(ce, 63);
            tbase += __shfl(te, 63);
        }
        if (lane == 0) {
            expert_off[n_expert] = ebase;
            tile_off[n_expert]   = tbase;
        }
    }
    __syncthreads();
    for (unsigned i = threadIdx.x; i < n_entries; i += blockDim.x) {
        const int e = ids[i];
        if (e < 0 || (unsigned)e >= n_expert) { if (inv) inv[i] = -1; continue; }
        const int pos = off[e] + atomicAdd(&cur[e], 1);
        perm[pos] = (int)i;
        if (inv) inv[i] = pos;
    }
}
