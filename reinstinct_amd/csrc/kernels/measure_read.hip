// Measurement kernel, not part of the path: a plain streaming read of n16 16-byte words, one
// 128-bit load per lane and trip, four trips in flight.  The benchmark runs it over the same
// weight rotations as the decode matvecs, so that "what a read of these bytes takes on this
// machine" is measured next to every matvec figure.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef unsigned int rein_read_v4u __attribute__((ext_vector_type(4)));

extern "C" __global__ __launch_bounds__(256) void rein_measure_read16(const rein_read_v4u* __restrict__ p, size_t n16,
                                                                      unsigned int* __restrict__ sink)
{
    const size_t tid = (size_t)blockIdx.x * 256u + threadIdx.x;
    const size_t nth = (size_t)gridDim.x * 256u;
    unsigned acc = 0u;
    for (size_t i = tid; i < n16; i += nth * 4u) {
        rein_read_v4u v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const size_t j = i + (size_t)u * nth;
            v[u] = __builtin_nontemporal_load(p + (j < n16 ? j : n16 - 1u));
        }
#pragma unroll
        for (int u = 0; u < 4; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x12345678u) sink[0] = 1u;            // keeps the loads alive; practically never taken
}

// Measurement kernel, not part of the path: what a barrier across all workgroups of a launch costs on this
// machine when it goes through device memory (the L2s of the XCDs are not coherent with each other, so flags
// that every CU must see are agent-scope accesses that go to memory).  Launched with one workgroup per CU
// (all resident at once), it does nothing but the barrier; every wait is bounded by spin_limit polls, after
// which a workgroup sets out[1] and leaves, so every wavefront ends whatever happens.  The words are never
// reset: a launch reads the generation g, stores g + 1 to its flags, and workgroup 0 publishes g + 1 as the
// next generation once it has seen every flag, so launches replay.
//   mode 0  no barrier (an empty launch of the same shape)
//   mode 1  every workgroup polls every flag
//   mode 2  workgroup 0 gathers the flags into one word that the others poll
//   mode 3  mode 2 without the release's L2 write-back in front of the flag store
struct ReinMeasureSync {
    unsigned gen, open, pad[62];
    unsigned flag[1024];
};
__device__ ReinMeasureSync rein_measure_sync;

extern "C" __global__ __launch_bounds__(1024) void rein_measure_barrier(unsigned int mode, unsigned int spin_limit,
                                                                        unsigned int* __restrict__ out)
{
    __shared__ unsigned open_s;
    if (mode == 0u || gridDim.x > 1024u) return;
    ReinMeasureSync& S = rein_measure_sync;
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned gen = __hip_atomic_load(&S.gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (wave == 0u) {
        if (mode != 3u) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        if (lane == 0u) __hip_atomic_store(&S.flag[blockIdx.x], gen + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned open = 0u;
        if (mode == 1u || blockIdx.x == 0u) {
            for (unsigned s = 0; s < spin_limit; s++) {
                bool all = true;
                for (unsigned i = lane; i < gridDim.x; i += 64u)
                    all = all && __hip_atomic_load(&S.flag[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gen + 1u;
                if (__all(all)) { open = 1u; break; }
                __builtin_amdgcn_s_sleep(2);
            }
            if (mode != 1u && open && lane == 0u) __hip_atomic_store(&S.open, gen + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            for (unsigned s = 0; s < spin_limit; s++) {
                if (__hip_atomic_load(&S.open, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == gen + 1u) { open = 1u; break; }
                __builtin_amdgcn_s_sleep(2);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        if (lane == 0u) open_s = open;
    }
    __syncthreads();
    if (open_s == 0u) {
        if (threadIdx.x == 0u) out[1] = 1u;
        return;
    }
    if (blockIdx.x == 0u && threadIdx.x == 0u) {
        __hip_atomic_store(&S.gen, gen + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        out[0] = gen + 1u;
    }
}
