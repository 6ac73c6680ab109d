// A workspace that needs no allocation: 64 MiB of device memory that is part of this library's
// code object on every GPU it is loaded on, for callers that may not allocate when they
// execute an einsummable (code under HIP graph capture, serving loops, harnesses that forbid
// it).  The array's name means something only to device code and to hipGetSymbolAddress; host
// code uses the address looked up once per device.
#include "static_workspace.h"

#include "kernel_manager.h"

#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

static __device__ __align__(256) unsigned char scratch[es::STATIC_WORKSPACE_BYTES];

namespace es
{

namespace
{

constexpr int MAX_DEVICES = 64;
std::mutex    g_mu;
void*         g_ptr[MAX_DEVICES];  // device address of `scratch` on each device, once looked up

}  // namespace

void* static_workspace_init(int device)
{
    if (device < 0 || device >= MAX_DEVICES) {
        throw km_error(km_status::device, "static workspace: device index out of range");
    }
    std::lock_guard<std::mutex> lock(g_mu);
    if (g_ptr[device]) return g_ptr[device];
    int current = -1;
    hipError_t err = hipGetDevice(&current);
    if (err != hipSuccess || current != device) {
        throw km_error(km_status::device,
                       "static workspace: device " + std::to_string(device) + " is not current");
    }
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr) {
        throw km_error(km_status::device,
                       std::string("hipGetSymbolAddress(static workspace): ") +
                           hipGetErrorString(err));
    }
    g_ptr[device] = ptr;
    return ptr;
}

void* static_workspace(int device)
{
    if (device < 0 || device >= MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(g_mu);
    return g_ptr[device];
}

}  // namespace es
