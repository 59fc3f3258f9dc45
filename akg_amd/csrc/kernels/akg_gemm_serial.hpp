/**
 * MatMul in the reference's own arithmetic, for the descriptions the MFMA kernels do not take.
 *
 * The reference lowers MatMul to linalg.matmul on a zero-filled accumulator of the declared result type
 * (akg-mlir/lib/Conversion/MindSporeToLinalg/MindSporeToLinalg.cpp:1453-1546) and then to plain loops in (i, j, k)
 * order: both operands are converted to the accumulator's element type, multiplied in it and added in it, one k after
 * the other. For a float16 / bfloat16 result that means a product rounded to 16 bits and a sum rounded to 16 bits at
 * every step - a result no matrix unit reproduces (they sum in float32). This kernel keeps that order and that
 * rounding exactly: every output element is one serial chain over k on the vector ALUs, so a description with a 16-bit
 * MatMul result gets the reference's value bit for bit (slowly: descriptions that want the matrix units declare a
 * float32 result and cast it, which is what the measured GEMM fusions do). It also serves shapes and element types the
 * MFMA kernels refuse (N not a multiple of 4, rows of K that are not whole 16-byte pieces, float32 / float64 / wider
 * integer operands), where it is the reference's float32 sum in the reference's order.
 *
 * Work split: a workgroup of 256 threads (16 x 16) owns 64 rows x 16*W columns of the result, a thread 4 rows x W
 * adjacent columns (W = 4, or 1 when N is not a multiple of 4); K is walked in slabs of 32 through LDS, both tiles
 * stored as compute-type values. Out-of-range rows / columns compute on zeros and are not stored; the k loop runs
 * exactly K steps (an extra step with a zero product could turn an accumulated -0 into +0).
 */
#pragma once

#include "akg_rt.hpp"

namespace akg {

template <typename ACC>
struct SerialMac {
  // float / double accumulators: one rounded product, one rounded sum (the build never contracts them into an fma)
  template <typename CT>
  static AKG_DEV ACC step(ACC acc, ACC a, ACC b) {
    return CT::rnd(acc + CT::rnd(a * b));
  }
};
template <>
struct SerialMac<int> {
  template <typename CT>
  static AKG_DEV int step(int acc, int a, int b) {
    return CT::rnd(op_add(acc, CT::rnd(op_mul(a, b))));
  }
};
template <>
struct SerialMac<long long> {
  template <typename CT>
  static AKG_DEV long long step(long long acc, long long a, long long b) {
    return op_add(acc, op_mul(a, b));
  }
};

// AT: element type tag of both operands, CT: tag of the accumulator (the MatMul's declared result type).
template <typename AT, typename CT, long M, long N, long K, bool TRANSB, int W, typename Epilogue>
AKG_DEV void gemm_serial(const typename AT::storage *__restrict__ A, const typename AT::storage *__restrict__ B,
                         Epilogue &epi) {
  typedef typename CT::compute ACC;
  constexpr int kRowsPerThread = 4, kSlab = 32;
  constexpr int kTileRows = 16 * kRowsPerThread, kTileCols = 16 * W;
  constexpr long kColTiles = (N + kTileCols - 1) / kTileCols;
  __shared__ ACC As[kTileRows][kSlab + 1];
  __shared__ ACC Bs[kSlab][kTileCols + 1];

  const int tid = static_cast<int>(threadIdx.x);
  const int tx = tid % 16, ty = tid / 16;
  const long tile = static_cast<long>(blockIdx.x);
  const long row0 = (tile / kColTiles) * kTileRows;
  const long col0 = (tile % kColTiles) * kTileCols;

  ACC acc[kRowsPerThread][W];
#pragma unroll
  for (int i = 0; i < kRowsPerThread; ++i) {
#pragma unroll
    for (int j = 0; j < W; ++j) acc[i][j] = static_cast<ACC>(0);
  }

  for (long k0 = 0; k0 < K; k0 += kSlab) {
    const int kmax = static_cast<int>((K - k0) < kSlab ? (K - k0) : kSlab);
    // A slab: kTileRows x kSlab values, consecutive threads along k
    for (int e = tid; e < kTileRows * kSlab; e += 256) {
      const int r = e / kSlab, kk = e % kSlab;
      const long row = row0 + r, k = k0 + kk;
      ACC v = static_cast<ACC>(0);
      if (row < M && k < K) v = static_cast<ACC>(AT::load(A[row * K + k]));
      As[r][kk] = v;
    }
    // B slab: kSlab x kTileCols values; consecutive threads along the operand's contiguous axis
    for (int e = tid; e < kSlab * kTileCols; e += 256) {
      int kk, c;
      if (TRANSB) {
        c = e / kSlab;
        kk = e % kSlab;
      } else {
        kk = e / kTileCols;
        c = e % kTileCols;
      }
      const long col = col0 + c, k = k0 + kk;
      ACC v = static_cast<ACC>(0);
      if (col < N && k < K) v = static_cast<ACC>(AT::load(TRANSB ? B[col * K + k] : B[k * N + col]));
      Bs[kk][c] = v;
    }
    __syncthreads();
    for (int kk = 0; kk < kmax; ++kk) {
      ACC a[kRowsPerThread], b[W];
#pragma unroll
      for (int i = 0; i < kRowsPerThread; ++i) a[i] = As[ty * kRowsPerThread + i][kk];
#pragma unroll
      for (int j = 0; j < W; ++j) b[j] = Bs[kk][tx * W + j];
#pragma unroll
      for (int i = 0; i < kRowsPerThread; ++i) {
#pragma unroll
        for (int j = 0; j < W; ++j) acc[i][j] = SerialMac<ACC>::template step<CT>(acc[i][j], a[i], b[j]);
      }
    }
    __syncthreads();
  }

  const long col = col0 + tx * W;
  if (col < N) {   // W divides N, so a thread's W columns are inside the row or all outside
    epi.prepare(col);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
      const long row = row0 + ty * kRowsPerThread + i;
      if (row < M) epi.apply(acc[i], row, col);
    }
  }
}

}  // namespace akg
