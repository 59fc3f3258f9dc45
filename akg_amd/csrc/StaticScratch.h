/**
 * Host-side access to the library's fixed device scratch array (StaticScratch.hip).
 */
#ifndef AKG_HIP_STATICSCRATCH_H_
#define AKG_HIP_STATICSCRATCH_H_

#include <hip/hip_runtime_api.h>

#include <cstdint>

// Size of the array every device holds once the library's own code object is loaded there.
#define AKG_HIP_STATIC_SCRATCH_BYTES (16u << 20)

namespace akg {

// Address of the scratch array on the current device (looked up once per device, then remembered).
hipError_t staticScratchOnCurrentDevice(void **ptr);

// Enqueue a fill kernel that zeroes the first `bytes` bytes at `ptr` (a pointer into the array) on `stream`.
hipError_t staticScratchClear(void *ptr, uint64_t bytes, hipStream_t stream);

}  // namespace akg

#endif  // AKG_HIP_STATICSCRATCH_H_
