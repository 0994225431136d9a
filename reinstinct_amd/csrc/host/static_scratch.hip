// The one piece of librein that is compiled by hipcc as host + device code: a fixed scratch
// array in device memory for rein_mmq_xq8_noalloc, the entry point for callers that cannot
// allocate (code under graph capture, serving loops, harnesses that forbid hipMalloc).  It is
// built into its own small shared object (librein_scratch.so) so that librein.so itself keeps
// binding the HIP runtime at run time only; librein.so loads it on the first call of that
// entry point.
//
// Every GPU the process uses holds its own copy of the array, at its own address, until the
// process ends.  In host code the array's name is only a handle for the runtime: the address
// kernels can use comes from hipGetSymbolAddress, asked once per device with that device
// current, and is what the library passes on as the workspace pointer.
#include <hip/hip_runtime.h>

#include <mutex>

#define REIN_STATIC_SCRATCH_BYTES (48u << 20)      // 48 MiB per GPU: the activation image and the partial tiles of a
                                                   // split-tail launch at 512 tokens x 5120, with room to 1500 tokens
#define REIN_MAX_DEVICES 64

static __device__ __align__(256) unsigned char scratch[REIN_STATIC_SCRATCH_BYTES];

namespace {
std::mutex g_mu;
void* g_ptr[REIN_MAX_DEVICES];
bool  g_known[REIN_MAX_DEVICES];
}  // namespace

// *ptr = device address of the current device's scratch array, *bytes = its size.
// Returns 0 or the hipError_t of the failing runtime call.  Allocates nothing.
extern "C" int rein_static_scratch(void** ptr, size_t* bytes)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= REIN_MAX_DEVICES) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_known[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return (int)hipErrorInvalidSymbol;
        g_ptr[dev] = p;
        g_known[dev] = true;
    }
    *ptr = g_ptr[dev];
    *bytes = REIN_STATIC_SCRATCH_BYTES;
    return 0;
}
