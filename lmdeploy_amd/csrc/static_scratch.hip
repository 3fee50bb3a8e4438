// Scratch memory for callers that cannot allocate (code under HIP graph capture, serving loops and
// harnesses that forbid hipMalloc): a file-scope device array that the split-K kernels use for their
// partial tiles and arrival counters instead of a handle's workspace.
//
// Every GPU the library runs on holds its own copy of the array, at its own address, from the
// moment the code object is loaded there until the process ends.  In host code the array's name is
// only a stand-in for those copies: its device address comes from hipGetSymbolAddress, once per
// device with that device current, and only that address is ever handed to a kernel.
#include "w4a16_internal.h"

#include <algorithm>
#include <mutex>

namespace w4a16 {

namespace {

constexpr size_t kCounterBytes = kStaticCounters * sizeof(int);
constexpr size_t kStaticBytes  = kCounterBytes + kStaticWorkspaceBytes;
constexpr int    kMaxDevices   = 64;

// [arrival counters: kStaticCounters ints][fp32 partial tiles: kStaticWorkspaceBytes]
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

std::mutex     g_mutex;
unsigned char* g_ptr[kMaxDevices];  // device address of `scratch` on each device, null until looked up

__global__ void __launch_bounds__(256) fill_zero_kernel(int* p, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

}  // namespace

hipError_t static_scratch(Scratch* out)
{
    int        dev = 0;
    hipError_t e   = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    unsigned char* ptr;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        if (!g_ptr[dev]) {
            void* p = nullptr;
            e       = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess) return e;
            if (!p) return hipErrorInvalidSymbol;
            g_ptr[dev] = static_cast<unsigned char*>(p);
        }
        ptr = g_ptr[dev];
    }
    out->cnt      = reinterpret_cast<int*>(ptr);
    out->cnt_len  = (int)kStaticCounters;
    out->ws       = reinterpret_cast<float*>(ptr + kCounterBytes);
    out->ws_bytes = kStaticWorkspaceBytes;
    return hipSuccess;
}

hipError_t clear_counters(const Scratch& sc, int n, hipStream_t st)
{
    n = std::min(n, sc.cnt_len);
    if (!sc.cnt || n <= 0) return hipSuccess;
    // a kernel, not hipMemsetAsync: the call may be recorded into a graph
    return launch_kernel(fill_zero_kernel, dim3((n + 255) / 256), dim3(256), 0, st, sc.cnt, n);
}

}  // namespace w4a16
