// Run-time binding of libamdhip64.so: the same entry points the reference
// resolves (src/hip/sys.rs:57-101), as a table of C function pointers.  No
// link-time ROCm dependency and no HIP headers needed on the host side.
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>

namespace rein {

using hipError_t   = int;
using hipStream_t  = void*;
using hipEvent_t   = void*;
using hipGraph_t   = void*;
using hipGraphExec_t = void*;
using hipModule_t  = void*;
using hipFunction_t = void*;

enum : int { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum : int { hipStreamCaptureModeGlobal = 0 };

struct HipApi {
    void* lib = nullptr;
    hipError_t (*GetDeviceCount)(int*);
    hipError_t (*SetDevice)(int);
    hipError_t (*GetDevice)(int*);
    hipError_t (*DeviceCanAccessPeer)(int*, int, int);
    hipError_t (*DeviceEnablePeerAccess)(int, unsigned);
    hipError_t (*DeviceGetName)(char*, int, int);
    hipError_t (*DeviceTotalMem)(size_t*, int);
    hipError_t (*MemGetInfo)(size_t*, size_t*);
    const char* (*GetErrorString)(hipError_t);
    hipError_t (*Malloc)(void**, size_t);
    hipError_t (*Free)(void*);
    hipError_t (*Memcpy)(void*, const void*, size_t, int);
    hipError_t (*MemcpyAsync)(void*, const void*, size_t, int, hipStream_t);
    hipError_t (*MemcpyPeerAsync)(void*, int, const void*, int, size_t, hipStream_t);
    hipError_t (*StreamCreate)(hipStream_t*);
    hipError_t (*StreamDestroy)(hipStream_t);
    hipError_t (*StreamSynchronize)(hipStream_t);
    hipError_t (*StreamWaitEvent)(hipStream_t, hipEvent_t, unsigned);
    hipError_t (*DeviceSynchronize)();
    hipError_t (*ModuleLoad)(hipModule_t*, const char*);
    hipError_t (*ModuleUnload)(hipModule_t);
    hipError_t (*ModuleGetFunction)(hipFunction_t*, hipModule_t, const char*);
    hipError_t (*ModuleLaunchKernel)(hipFunction_t, unsigned, unsigned, unsigned, unsigned, unsigned,
                                     unsigned, unsigned, hipStream_t, void**, void**);
    hipError_t (*StreamBeginCapture)(hipStream_t, int);
    hipError_t (*StreamEndCapture)(hipStream_t, hipGraph_t*);
    hipError_t (*GraphInstantiate)(hipGraphExec_t*, hipGraph_t, void*, char*, size_t);
    hipError_t (*GraphLaunch)(hipGraphExec_t, hipStream_t);
    hipError_t (*GraphDestroy)(hipGraph_t);
    hipError_t (*GraphExecDestroy)(hipGraphExec_t);
    hipError_t (*EventCreate)(hipEvent_t*);
    hipError_t (*EventRecord)(hipEvent_t, hipStream_t);
    hipError_t (*EventSynchronize)(hipEvent_t);
    hipError_t (*EventElapsedTime)(float*, hipEvent_t, hipEvent_t);
    hipError_t (*EventDestroy)(hipEvent_t);
};

// Loads the library on first use; returns nullptr and fills `err` on failure.
const HipApi* hip_api(std::string* err);

// thread-local last-error string
void set_error(const std::string& msg);
const char* last_error();
// returns e; when e != 0 also records "<ctx>: <hipGetErrorString> (code N)"
int check_hip(const HipApi* api, hipError_t e, const char* ctx);
int fail(int code, const std::string& msg);

}  // namespace rein
