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
