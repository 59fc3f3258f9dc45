/**
 * Measurement probes for bench.py (built into libakg_bench_probe.so, NOT part of libakg_hip.so).
 *
 * What a matrix unit of this part sustains when nothing else is in the way: every wavefront keeps its MFMA operands in
 * registers and issues nothing but MFMAs (two wavefronts per SIMD, eight per workgroup), either in the shape the GEMM
 * kernel issues them (4 x 4 accumulator tiles of 16 x 16 per wavefront, 64 bytes of K per MFMA) or in the 32 x 32 shape
 * (2 x 4 tiles, 32 bytes of K). The operands come from a caller's buffer, so the same loop can run on zeros and on
 * random data: the part is power limited, and how far the clock drops under the toggling of real operands is what
 * decides the ceiling a GEMM kernel can approach - and it drops less in the 16 x 16 shapes. Four operand sets are
 * rotated so that consecutive MFMAs do not see the same registers.
 *
 * Entry points (plain C, asynchronous on the given stream; the caller times them with events):
 *   akg_probe_mfma_i8 / akg_probe_mfma_bf16 / akg_probe_mfma_i8_32x32 / akg_probe_mfma_bf16_32x32
 *       (stream, operands, iterations, workgroups, sink)
 *     operands: device buffer of at least 32 KiB (32 fragments of 64 lanes x 16 bytes), sink: workgroups * 512 ints
 *     work done = workgroups * 8 wavefronts * iterations * 2097152 ops (int8) or 1048576 flops (bf16): 64 MFMAs of
 *     16 x 16 x 64 (int8) / 16 x 16 x 32 (bf16), or 32 MFMAs of 32 x 32 x 32 / 32 x 32 x 16
 */
#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ inline int bitsOf(int x) { return x; }
__device__ inline int bitsOf(float x) { return __float_as_int(x); }

// SHAPE 16: 4 x 4 tiles of 16 x 16, SHAPE 32: 2 x 4 tiles of 32 x 32
template <bool INT8, int SHAPE>
struct Tile;
template <>
struct Tile<true, 32> {
  typedef v16i acc_v;
  static __device__ inline acc_v mma(v4i a, v4i b, acc_v c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0); }
};
template <>
struct Tile<false, 32> {
  typedef v16f acc_v;
  static __device__ inline acc_v mma(v4i a, v4i b, acc_v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <>
struct Tile<true, 16> {
  typedef v4i acc_v;
  static __device__ inline acc_v mma(v4i a, v4i b, acc_v c) { return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0); }
};
template <>
struct Tile<false, 16> {
  typedef v4f acc_v;
  static __device__ inline acc_v mma(v4i a, v4i b, acc_v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};

template <bool INT8, int SHAPE>
__global__ void __launch_bounds__(512) mfmaLoop(const v4i *__restrict__ operands, int iterations, int *__restrict__ sink) {
  constexpr int I = SHAPE == 16 ? 4 : 2, J = 4;
  typedef typename Tile<INT8, SHAPE>::acc_v acc_v;
  constexpr int kAccRegs = sizeof(acc_v) / 4;
  const int lane = static_cast<int>(threadIdx.x) & 63;
  v4i a[4][I], b[4][J];
#pragma unroll
  for (int s = 0; s < 4; ++s) {
#pragma unroll
    for (int i = 0; i < I; ++i) a[s][i] = operands[(s * (I + J) + i) * 64 + lane];
#pragma unroll
    for (int j = 0; j < J; ++j) b[s][j] = operands[(s * (I + J) + I + j) * 64 + lane];
  }
  acc_v acc[I][J];
#pragma unroll
  for (int i = 0; i < I; ++i) {
#pragma unroll
    for (int j = 0; j < J; ++j) {
#pragma unroll
      for (int v = 0; v < kAccRegs; ++v) acc[i][j][v] = 0;
    }
  }
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int i = 0; i < I; ++i) {
#pragma unroll
        for (int j = 0; j < J; ++j) acc[i][j] = Tile<INT8, SHAPE>::mma(a[s][i], b[s][j], acc[i][j]);
      }
    }
  }
  int fold = 0;
#pragma unroll
  for (int i = 0; i < I; ++i) {
#pragma unroll
    for (int j = 0; j < J; ++j) {
#pragma unroll
      for (int v = 0; v < kAccRegs; ++v) fold ^= bitsOf(acc[i][j][v]);
    }
  }
  sink[static_cast<size_t>(blockIdx.x) * 512 + threadIdx.x] = fold;
}

template <bool INT8, int SHAPE>
int launchLoop(void *stream, const void *operands, int iterations, int workgroups, void *sink) {
  if (operands == nullptr || sink == nullptr || iterations <= 0 || workgroups <= 0) return -1;
  mfmaLoop<INT8, SHAPE><<<dim3(static_cast<unsigned>(workgroups)), dim3(512), 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const v4i *>(operands), iterations, static_cast<int *>(sink));
  return hipGetLastError() == hipSuccess ? 0 : -7;
}

}  // namespace

extern "C" {

int akg_probe_mfma_i8(void *stream, const void *operands, int iterations, int workgroups, void *sink) {
  return launchLoop<true, 16>(stream, operands, iterations, workgroups, sink);
}
int akg_probe_mfma_bf16(void *stream, const void *operands, int iterations, int workgroups, void *sink) {
  return launchLoop<false, 16>(stream, operands, iterations, workgroups, sink);
}
int akg_probe_mfma_i8_32x32(void *stream, const void *operands, int iterations, int workgroups, void *sink) {
  return launchLoop<true, 32>(stream, operands, iterations, workgroups, sink);
}
int akg_probe_mfma_bf16_32x32(void *stream, const void *operands, int iterations, int workgroups, void *sink) {
  return launchLoop<false, 32>(stream, operands, iterations, workgroups, sink);
}

}  // extern "C"
