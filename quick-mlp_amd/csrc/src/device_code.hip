// The only device code that is compiled into the library ahead of time (everything else is
// generated and compiled at run time through hipRTC):
//   * a fill kernel that stands in for hipMemsetAsync, so that a caller may capture any call
//     of this library into a HIP graph without recording a memset node;
//   * the static device buffer that the entry point which allocates nothing
//     (qmlp_network_inference_noalloc) uses in place of device memory from hipMalloc.
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
hipStream_t g_scratchStream[MAX_DEVICES] = {};   // per device: the stream of the last call that used it
bool g_scratchUsed[MAX_DEVICES] = {};
std::mutex g_scratchMutex;

__global__ void __launch_bounds__(256) FillBytesKernel(unsigned char* __restrict__ p, unsigned char value, size_t bytes)
{
    const size_t tid = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t numThreads = static_cast<size_t>(gridDim.x) * 256;
    // bytes up to the first 16-byte boundary, 16-byte stores in the middle, the rest bytewise
    size_t head = (16 - reinterpret_cast<uintptr_t>(p) % 16) % 16;
    if (head > bytes) head = bytes;
    const size_t body = (bytes - head) / 16;
    const size_t tail = bytes - head - body * 16;
    if (tid < head) p[tid] = value;
    if (tid < tail) p[head + body * 16 + tid] = value;
    const unsigned int w = value * 0x01010101u;
    const uint4 word = make_uint4(w, w, w, w);
    uint4* __restrict__ q = reinterpret_cast<uint4*>(p + head);
    for (size_t i = tid; i < body; i += numThreads) q[i] = word;
}

std::string describe(hipError_t e, const char* what)
{
    return std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")";
}

} // namespace

namespace qmlp { namespace device_code {

int fillAsync(void* ptr, int value, size_t bytes, void* stream, std::string& error)
{
    if (bytes == 0) return 0;
    const size_t blocks = (bytes / 16 + 255) / 256 + 1;
    const unsigned grid = static_cast<unsigned>(blocks < 4096 ? blocks : 4096);
    // launched through the call that returns this launch's own status: hipGetLastError() would also report (and
    // clear) an error that another library left on this thread, e.g. hipErrorNotReady of an event query
    unsigned char* p = static_cast<unsigned char*>(ptr);
    unsigned char v = static_cast<unsigned char>(value);
    void* args[] = {&p, &v, &bytes};
    const hipError_t e = hipLaunchKernel(reinterpret_cast<const void*>(FillBytesKernel), dim3(grid), dim3(256), args, 0,
                                         static_cast<hipStream_t>(stream));
    if (e != hipSuccess) {
        error = describe(e, "launch of the fill kernel");
        return 1;
    }
    return 0;
}

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

int claimStaticScratch(void* stream, std::string& error)
{
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess || device < 0 || device >= MAX_DEVICES) {
        error = describe(e, "hipGetDevice");
        return 1;
    }
    const hipStream_t s = static_cast<hipStream_t>(stream);
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    if (g_scratchUsed[device] && g_scratchStream[device] != s) {
        // Work of another stream may still read or write the buffer. While this stream is being captured nothing
        // may be asked of other streams; otherwise the other stream says whether it is done (a stream that its
        // owner has destroyed meanwhile reports an error, which means that its work is over).
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &capture) != hipSuccess) (void)hipGetLastError();
        const bool busy = capture != hipStreamCaptureStatusNone || hipStreamQuery(g_scratchStream[device]) == hipErrorNotReady;
        (void)hipGetLastError();   // a not-ready or invalid-handle answer is no error of this call
        if (busy) {
            error = "the static workspace of the call that allocates nothing was last used on another stream whose work has "
                    "not finished (or this stream is being captured): calls that share it on one device must follow each "
                    "other on one stream, or be synchronised by the caller";
            return 1;
        }
    }
    g_scratchUsed[device] = true;
    g_scratchStream[device] = s;
    return 0;
}

}} // namespace qmlp::device_code
