// SwiGLU: out[i] = gate[i] / (1 + exp(-gate[i])) * up[i]; same entry point and
// arguments as kernels/swiglu.cpp:10-21 of the reference.
#include "rein_common.h"

extern "C" __global__ void swiglu_mul_f32(const float* __restrict__ gate, const float* __restrict__ up,
                                          float* __restrict__ out, unsigned int n)
{
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) {
        const float g = gate[i];
        out[i] = g / (1.0f + __expf(-g)) * up[i];
    }
}
