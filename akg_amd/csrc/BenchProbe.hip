/**
 * Measurement probes for bench.py (built into libakg_bench_probe.so, NOT part of libakg_hip.so).
 *
 * What a matrix unit of this part sustains when nothing else is in the way: every wavefront keeps its MFMA operands in
 * registers and issues nothing but MFMAs, in the shape the GEMM kernel issues them (2 x 4 accumulator tiles of
 * 32 x 32 per wavefront, two wavefronts per SIMD, eight per workgroup). The operands come from a caller's buffer,
 * so the same loop can run on zeros and on random data: the part is power limited, and how far the clock drops under
 * the toggling of real operands is what decides the ceiling a GEMM kernel can approach. Four operand sets are
 * rotated so that consecutive MFMAs do not see the same registers.
 *
 * Entry points (plain C, asynchronous on the given stream; the caller times them with events):
 *   akg_probe_mfma_i8 / akg_probe_mfma_bf16 (stream, operands, iterations, workgroups, sink)
 *     operands: device buffer of at least 24 KiB (24 fragments of 64 lanes x 16 bytes), sink: workgroups * 512 ints
 *     work done = workgroups * 8 wavefronts * iterations * 32 MFMAs * 65536 ops (int8, 32 x 32 x 32) or 32768 (bf16, 32 x 32 x 16)
 */
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ inline int bitsOf(int x) { return x; }
__device__ inline int bitsOf(float x) { return __float_as_int(x); }

template <bool INT8>
__global__ void __launch_bounds__(512) mfmaLoop(const v4i *__restrict__ operands, int iterations, int *__restrict__ sink) {
  const int lane = static_cast<int>(threadIdx.x) & 63;
  v4i a[4][2], b[4][4];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
#pragma unroll
    for (int i = 0; i < 2; ++i) a[s][i] = operands[(s * 6 + i) * 64 + lane];
#pragma unroll
    for (int j = 0; j < 4; ++j) b[s][j] = operands[(s * 6 + 2 + j) * 64 + lane];
  }
  typedef typename std::conditional<INT8, v16i, v16f>::type acc_v;
  acc_v acc[2][4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    }
  }
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (INT8) {
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
          } else {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[s][i]),
                                                                __builtin_bit_cast(bf16x8, b[s][j]), acc[i][j], 0, 0, 0);
          }
        }
      }
    }
  }
  int fold = 0;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) fold ^= bitsOf(acc[i][j][v]);
    }
  }
  sink[static_cast<size_t>(blockIdx.x) * 512 + threadIdx.x] = fold;
}

}  // namespace

extern "C" {

int akg_probe_mfma_i8(void *stream, const void *operands, int iterations, int workgroups, void *sink) {
  if (operands == nullptr || sink == nullptr || iterations <= 0 || workgroups <= 0) return -1;
  mfmaLoop<true><<<dim3(static_cast<unsigned>(workgroups)), dim3(512), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const v4i *>(operands), iterations, static_cast<int *>(sink));
  return hipGetLastError() == hipSuccess ? 0 : -7;
}

int akg_probe_mfma_bf16(void *stream, const void *operands, int iterations, int workgroups, void *sink) {
  if (operands == nullptr || sink == nullptr || iterations <= 0 || workgroups <= 0) return -1;
  mfmaLoop<false><<<dim3(static_cast<unsigned>(workgroups)), dim3(512), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const v4i *>(operands), iterations, static_cast<int *>(sink));
  return hipGetLastError() == hipSuccess ? 0 : -7;
}

}  // extern "C"
