// Test support: fills the LDS of every compute unit with all-ones bits (a NaN as fp32, bf16 and fp16).
// Kernels that read LDS they (or their workgroup) have not written, or read it before the write is visible, then
// produce results that differ from an undisturbed run instead of silently reusing plausible leftovers.
#include <hip/hip_runtime.h>

namespace {
constexpr int kLdsBytes = 160 * 1024;  // the whole LDS of a gfx950 compute unit

__global__ __launch_bounds__(256) void lds_fill_kernel(unsigned* sink) {
    extern __shared__ unsigned lds[];
    constexpr int n = kLdsBytes / 4;
    for (int i = threadIdx.x; i < n; i += 256) lds[i] = 0xFFFFFFFFu;
    __syncthreads();
    unsigned acc = 0;  // read everything back so that the stores cannot be dropped
    for (int i = threadIdx.x; i < n; i += 256) acc &= lds[i];
    if (acc == 0x12345678u) sink[0] = acc;  // never true
}
}  // namespace

// One workgroup occupies a whole compute unit; 1024 of them visit each of the 256 units several times.
extern "C" int lds_fill(void* sink, void* stream) {
    hipError_t e = hipFuncSetAttribute((const void*)lds_fill_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(lds_fill_kernel, dim3(1024), dim3(256), kLdsBytes, (hipStream_t)stream, (unsigned*)sink);
    return (int)hipGetLastError();
}
