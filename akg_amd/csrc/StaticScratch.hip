/**
 * The library's fixed device scratch array and what touches it from the host.
 *
 * akg_hip_launch_static_scratch (HipRuntime.cpp) serves callers that may not allocate device memory at launch
 * time or ever for this purpose (code under HIP graph capture, serving loops with a frozen memory plan). Kernels
 * whose family needs device memory beyond inputs and outputs (arrival counters and partial results of streaming
 * reductions and of GEMMs with K split over workgroups, grouped segment sums, the tensors between the kernels of a
 * staged description) normally get it from a per-handle hipMalloc; here they get a piece of `scratch` instead.
 *
 * `scratch` is a device symbol: in host code its name is only a stand-in for the device array, so its address on the
 * current device is asked for once per device with hipGetSymbolAddress and every host-side use (kernel arguments,
 * clearing) goes through that pointer. Every device the library's code object is loaded on holds its own copy until
 * the process ends.
 */
#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>

#include "StaticScratch.h"

static __device__ __align__(256) unsigned char scratch[AKG_HIP_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_mu;
void *g_scratchOnDevice[kMaxDevices] = {};

// 16 bytes per thread and step; `n16` counts 16-byte pieces.
__global__ void __launch_bounds__(256) akgScratchFillZero(uint4 *p, uint64_t n16) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride) {
    p[i] = make_uint4(0u, 0u, 0u, 0u);
  }
}

}  // namespace

namespace akg {

hipError_t staticScratchOnCurrentDevice(void **ptr) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_mu);
  if (g_scratchOnDevice[device] == nullptr) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (p == nullptr) return hipErrorInvalidSymbol;
    g_scratchOnDevice[device] = p;
  }
  *ptr = g_scratchOnDevice[device];
  return hipSuccess;
}

hipError_t staticScratchClear(void *ptr, uint64_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  const uint64_t n16 = (bytes + 15) / 16;   // the array is a multiple of 256 bytes, so rounding up stays inside it
  uint64_t blocks = (n16 + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  akgScratchFillZero<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream>>>(static_cast<uint4 *>(ptr), n16);
  return hipGetLastError();
}

}  // namespace akg
