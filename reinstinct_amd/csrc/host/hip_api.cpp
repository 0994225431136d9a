#include "hip_api.h"

#include <dlfcn.h>

#include <mutex>

namespace rein {

static thread_local std::string g_last_error;

void set_error(const std::string& msg) { g_last_error = msg; }
const char* last_error() { return g_last_error.c_str(); }

int fail(int code, const std::string& msg)
{
    set_error(msg + " (code " + std::to_string(code) + ")");
    return code;
}

int check_hip(const HipApi* api, hipError_t e, const char* ctx)
{
    if (e == 0) return 0;
    const char* s = api && api->GetErrorString ? api->GetErrorString(e) : nullptr;
    set_error(std::string(ctx) + ": " + (s ? s : "unknown HIP error") + " (code " + std::to_string(e) + ")");
    return e;
}

static HipApi     g_api;
static bool       g_ok = false;
static std::string g_load_error;
static std::once_flag g_once;

static void load_once()
{
    // Prefer a runtime some other library in this process already mapped, so
    // that device pointers and streams are shared with it.
    static const char* const names[] = {
        "libamdhip64.so", "libamdhip64.so.7", "libamdhip64.so.6", "libamdhip64.so.5",
        "/opt/rocm/lib/libamdhip64.so", "/usr/lib/x86_64-linux-gnu/libamdhip64.so"};
    void* lib = nullptr;
    std::string last = "no candidate paths";
    for (const char* n : names) {
        lib = dlopen(n, RTLD_NOW | RTLD_NOLOAD | RTLD_GLOBAL);
        if (lib) break;
    }
    for (size_t i = 0; !lib && i < sizeof(names) / sizeof(names[0]); i++) {
        lib = dlopen(names[i], RTLD_NOW | RTLD_GLOBAL);
        if (!lib) {
            const char* e = dlerror();
            last = std::string(names[i]) + ": " + (e ? e : "?");
        }
    }
    if (!lib) {
        g_load_error = "could not load libamdhip64.so (" + last + ")";
        return;
    }
    g_api.lib = lib;
    bool ok = true;
    auto sym = [&](const char* name) -> void* {
        void* p = dlsym(lib, name);
        if (!p && ok) {
            ok = false;
            g_load_error = std::string("missing ") + name;
        }
        return p;
    };
#define BIND(field, name) g_api.field = reinterpret_cast<decltype(g_api.field)>(sym(name))
    BIND(GetDeviceCount, "hipGetDeviceCount");
    BIND(SetDevice, "hipSetDevice");
    BIND(GetDevice, "hipGetDevice");
    BIND(DeviceCanAccessPeer, "hipDeviceCanAccessPeer");
    BIND(DeviceEnablePeerAccess, "hipDeviceEnablePeerAccess");
    BIND(DeviceGetName, "hipDeviceGetName");
    BIND(DeviceTotalMem, "hipDeviceTotalMem");
    BIND(MemGetInfo, "hipMemGetInfo");
    BIND(GetErrorString, "hipGetErrorString");
    BIND(Malloc, "hipMalloc");
    BIND(Free, "hipFree");
    BIND(Memcpy, "hipMemcpy");
    BIND(MemcpyAsync, "hipMemcpyAsync");
    BIND(MemcpyPeerAsync, "hipMemcpyPeerAsync");
    BIND(StreamCreate, "hipStreamCreate");
    BIND(StreamDestroy, "hipStreamDestroy");
    BIND(StreamSynchronize, "hipStreamSynchronize");
    BIND(StreamWaitEvent, "hipStreamWaitEvent");
    BIND(DeviceSynchronize, "hipDeviceSynchronize");
    BIND(ModuleLoad, "hipModuleLoad");
    BIND(ModuleUnload, "hipModuleUnload");
    BIND(ModuleGetFunction, "hipModuleGetFunction");
    BIND(ModuleLaunchKernel, "hipModuleLaunchKernel");
    BIND(StreamBeginCapture, "hipStreamBeginCapture");
    BIND(StreamEndCapture, "hipStreamEndCapture");
    BIND(GraphInstantiate, "hipGraphInstantiate");
    BIND(GraphLaunch, "hipGraphLaunch");
    BIND(GraphDestroy, "hipGraphDestroy");
    BIND(GraphExecDestroy, "hipGraphExecDestroy");
    BIND(EventCreate, "hipEventCreate");
    BIND(EventRecord, "hipEventRecord");
    BIND(EventSynchronize, "hipEventSynchronize");
    BIND(EventElapsedTime, "hipEventElapsedTime");
    BIND(EventDestroy, "hipEventDestroy");
#undef BIND
    g_ok = ok;
}

const HipApi* hip_api(std::string* err)
{
    std::call_once(g_once, load_once);
    if (!g_ok) {
        if (err) *err = g_load_error;
        return nullptr;
    }
    return &g_api;
}

}  // namespace rein
