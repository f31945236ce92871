// The only device code that is compiled into the library ahead of time (everything else is
// generated and compiled at run time through hipRTC): the static device buffer that the entry
// point which allocates nothing (qmlp_network_inference_noalloc) uses in place of device
// memory from hipMalloc.
#include "qmlp/device_code.h"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>
#include <string>

namespace {

// Workspace of qmlp_network_inference_noalloc: every GPU the library runs on holds one copy of
// it from the moment this code object is loaded until the process ends. In host code the name
// of the array is only a handle for hipGetSymbolAddress, never an address.
static __device__ __align__(256) unsigned char scratch[QMLP_STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
void* g_scratchAddress[MAX_DEVICES] = {};   // per device: where that device holds its copy
std::mutex g_scratchMutex;

std::string describe(hipError_t e, const char* what)
{
    return std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")";
}

} // namespace

namespace qmlp { namespace device_code {

int staticScratch(void** ptr, size_t* bytes, std::string& error)
{
    *ptr = nullptr;
    *bytes = QMLP_STATIC_SCRATCH_BYTES;
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        error = describe(e, "hipGetDevice");
        return 1;
    }
    if (device < 0 || device >= MAX_DEVICES) {
        error = "device index " + std::to_string(device) + " beyond the " + std::to_string(MAX_DEVICES) + " this library tracks";
        return 1;
    }
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    if (g_scratchAddress[device] == nullptr) {
        // once per device, with that device current: each GPU has its own copy at its own address
        void* address = nullptr;
        e = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (e != hipSuccess || address == nullptr) {
            error = describe(e, "hipGetSymbolAddress(scratch)");
            return 1;
        }
        g_scratchAddress[device] = address;
    }
    *ptr = g_scratchAddress[device];
    return 0;
}

}} // namespace qmlp::device_code
