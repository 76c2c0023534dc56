// Fixed scratch memory for the entry point that allocates nothing (ovfcc_fc_run_device_static): the split-K
// workspaces and arrival counters that the other entry points keep in buffers of the request live here in one
// file-scope device array, 64 KiB of counters followed by 32 MiB of f32 partial tiles.  Every GPU the library runs
// on holds its own copy of the array at its own address until the process ends; the address is looked up once per
// device, with that device current, and host code uses that pointer -- never the array's name, which on the host
// is only a stand-in for the symbol.
#include <hip/hip_runtime.h>

#include "ovfcc_internal.h"

namespace ovfcc {

static __device__ __align__(256) unsigned char scratch[kStaticCounterBytes + kStaticWorkspaceBytes];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

// Called by ovfcc_init with `device` current.  Returns a HIP error code (0 = success).
int static_scratch_setup(int device) {
    if (device < 0 || device >= kMaxDevices)
        return (int)hipErrorInvalidDevice;
    if (g_scratch_ptr[device])
        return 0;
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess)
        return (int)e;
    if (!ptr)
        return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[device] = ptr;
    return 0;
}

// Device address of the array on `device` (null before static_scratch_setup succeeded there).
void* static_scratch_ptr(int device) {
    return device >= 0 && device < kMaxDevices ? g_scratch_ptr[device] : nullptr;
}

__global__ __launch_bounds__(256) void fcc_zero_u32_kernel(unsigned* __restrict__ p, unsigned n) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        p[i] = 0u;
}

// p[0 .. n) = 0 with a small fill kernel (a caller may be capturing the stream into a graph)
int launch_zero_u32(unsigned* p, size_t n, void* stream) {
    if (n == 0)
        return 0;
    if (n > 0xFFFFFFFFull)
        return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fcc_zero_u32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), p, (unsigned)n);
    return (int)hipGetLastError();
}

}  // namespace ovfcc
