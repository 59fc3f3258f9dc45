/**
 * int8 x int8 -> int32 GEMM tile kernel for gfx950 (CDNA4) with a caller-supplied epilogue applied to the
 * int32 accumulators while they are still in registers (dequantise / bias / activation / cast fusions).
 *
 * Shape of the computation (all sizes are compile-time constants of the emitted kernel):
 *   C[M,N] = A[M,K] * B[K,N]            A row-major int8, B row-major int8 ([N,K] when TRANSB)
 *   workgroup = 256 threads = 4 wavefronts (2 x 2), workgroup tile 256 x 256, K step 64
 *   wavefront tile 128 x 128 = 4 x 4 MFMA tiles of v_mfma_i32_32x32x32_i8 (16 accumulator registers each)
 *
 * Data movement:
 *   global -> registers -> LDS, double buffered in LDS (one barrier per K step); the global loads of step
 *   i+1 are issued before the MFMAs of step i.
 *   A: each thread moves 4 x 16 bytes (16 consecutive k of one row) straight into LDS.
 *   B (not transposed) is row-major along N but the MFMA wants, per lane, 16 consecutive k of one column.
 *   Each thread therefore loads a 16(k) x 4(n) byte block as 16 dwords, transposes it in registers with
 *   v_perm_b32 (8 permutes per 4 x 4 sub-block) and writes four 16-byte k-vectors to LDS.
 *   LDS rows are 64 data bytes + 16 pad bytes: with a row pitch of 80 bytes eight consecutive rows start in
 *   eight different 16-byte bank groups, so the ds_read_b128 fragment loads are conflict free.
 *   LDS row r of the B tile holds global column 4 * (r % 64) + r / 64 of the tile. A wavefront's four column
 *   tiles are r / 64 = 0..3 with the same r % 64 range, so each lane ends up owning 4 ADJACENT output columns:
 *   the epilogue works on 4-element chunks and a wavefront stores 256 contiguous bytes per output row.
 *
 * Workgroup -> tile mapping: consecutive workgroup ids go round-robin to the 8 XCDs (each with its own L2), so
 * ids are first regrouped per XCD and then walked in column-major groups of 8 tile-rows, which keeps the A and B
 * panels that an XCD's resident workgroups share inside that XCD's L2.
 */
#pragma once

namespace akg {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kGemmBM = 256;
constexpr int kGemmBN = 256;
constexpr int kGemmBK = 64;
constexpr int kGemmPitch = 80;  // bytes per LDS row: 64 data + 16 pad
constexpr int kGemmThreads = 256;
constexpr int kGemmXcds = 8;
constexpr int kGemmGroupRows = 8;  // tile-rows per group in the swizzled walk

// 4 x 4 byte transpose: in r[i] byte j  ->  out t[j] byte i.
AKG_DEV void transpose4x4_bytes(const u32 (&r)[4], u32 (&t)[4]) {
  const u32 lo01 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);
  const u32 hi01 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
  const u32 lo23 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
  const u32 hi23 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
  t[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
  t[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
  t[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
  t[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

// Number of workgroups to launch for an M x N problem (multiple of the XCD count).
constexpr long gemm_i8_grid(long m, long n) {
  const long tiles = ((m + kGemmBM - 1) / kGemmBM) * ((n + kGemmBN - 1) / kGemmBN);
  return ((tiles + kGemmXcds - 1) / kGemmXcds) * kGemmXcds;
}

template <long M, long N, long K, bool TRANSB, typename Epilogue>
AKG_DEV void gemm_i8_256x256(const s8 *__restrict__ A, const s8 *__restrict__ B, Epilogue &epi) {
  static_assert(K % 16 == 0, "K must be a multiple of 16");
  static_assert(TRANSB || (N % 4 == 0), "N must be a multiple of 4");
  constexpr long kTilesM = (M + kGemmBM - 1) / kGemmBM;
  constexpr long kTilesN = (N + kGemmBN - 1) / kGemmBN;
  constexpr long kTiles = kTilesM * kTilesN;
  constexpr long kPerXcd = (kTiles + kGemmXcds - 1) / kGemmXcds;
  constexpr long kSteps = (K + kGemmBK - 1) / kGemmBK;
  constexpr bool kFull = (M % kGemmBM == 0) && (N % kGemmBN == 0) && (K % kGemmBK == 0);
  constexpr int kTileBytes = kGemmBM * kGemmPitch;  // one operand tile in LDS

  __shared__ __attribute__((aligned(16))) u8 lds[2][2][kTileBytes];  // [buffer][A|B]

  // ---- workgroup -> tile
  const long wg = static_cast<long>(blockIdx.x);
  const long linear = (wg % kGemmXcds) * kPerXcd + wg / kGemmXcds;
  if (linear >= kTiles) return;
  constexpr long kGroupSize = kGemmGroupRows * kTilesN;
  const long group = linear / kGroupSize;
  const long firstRow = group * kGemmGroupRows;
  const long rowsInGroup = (kTilesM - firstRow) < kGemmGroupRows ? (kTilesM - firstRow) : kGemmGroupRows;
  const long inGroup = linear % kGroupSize;
  const long tileM = firstRow + inGroup % rowsInGroup;
  const long tileN = inGroup / rowsInGroup;
  const long m0 = tileM * kGemmBM;
  const long n0 = tileN * kGemmBN;

  const int tid = static_cast<int>(threadIdx.x);
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1;
  const int wn = wave & 1;

  v16i acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    }
  }

  // ---- staging registers
  v4i ga[4];
  u32 gb[16];   // !TRANSB: 16 k-rows x 4 columns
  v4i gbt[4];   // TRANSB: like A

  const int aRow = tid >> 2;       // + 64 * i
  const int aChunk = tid & 3;
  const int bN4 = tid & 63;
  const int bKq = tid >> 6;

  auto loadGlobal = [&](long step) {
    const long k0 = step * kGemmBK;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const long row = m0 + aRow + 64 * i;
      const long k = k0 + aChunk * 16;
      if (kFull || (row < M && k < K)) {
        ga[i] = *reinterpret_cast<const v4i *>(A + row * K + k);
      } else {
        ga[i] = v4i{0, 0, 0, 0};
      }
    }
    if constexpr (TRANSB) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const long col = n0 + aRow + 64 * i;
        const long k = k0 + aChunk * 16;
        if (kFull || (col < N && k < K)) {
          gbt[i] = *reinterpret_cast<const v4i *>(B + col * K + k);
        } else {
          gbt[i] = v4i{0, 0, 0, 0};
        }
      }
    } else {
      const long col = n0 + 4 * bN4;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const long k = k0 + bKq * 16 + i;
        if (kFull || (col < N && k < K)) {
          gb[i] = *reinterpret_cast<const u32 *>(B + k * N + col);
        } else {
          gb[i] = 0u;
        }
      }
    }
  };

  auto storeLds = [&](int buf) {
    u8 *la = lds[buf][0];
    u8 *lb = lds[buf][1];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<v4i *>(la + (aRow + 64 * i) * kGemmPitch + aChunk * 16) = ga[i];
    }
    if constexpr (TRANSB) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int col = aRow + 64 * i;                 // column of the tile
        const int r = (col & 3) * 64 + (col >> 2);     // its LDS row
        *reinterpret_cast<v4i *>(lb + r * kGemmPitch + aChunk * 16) = gbt[i];
      }
    } else {
      u32 t[4][4];
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const u32 rows[4] = {gb[4 * g], gb[4 * g + 1], gb[4 * g + 2], gb[4 * g + 3]};
        transpose4x4_bytes(rows, t[g]);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v4i w;
        w[0] = static_cast<int>(t[0][j]);
        w[1] = static_cast<int>(t[1][j]);
        w[2] = static_cast<int>(t[2][j]);
        w[3] = static_cast<int>(t[3][j]);
        *reinterpret_cast<v4i *>(lb + (j * 64 + bN4) * kGemmPitch + bKq * 16) = w;
      }
    }
  };

  const int fragRow = lane & 31;
  const int fragHalf = (lane >> 5) * 16;

  auto compute = [&](int buf) {
    const u8 *la = lds[buf][0] + (wm * 128 + fragRow) * kGemmPitch + fragHalf;
    const u8 *lb = lds[buf][1] + (wn * 32 + fragRow) * kGemmPitch + fragHalf;
#pragma unroll
    for (int ks = 0; ks < kGemmBK / 32; ++ks) {
      v4i af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const v4i *>(la + i * 32 * kGemmPitch + ks * 32);
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[j] = *reinterpret_cast<const v4i *>(lb + j * 64 * kGemmPitch + ks * 32);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
      }
    }
  };

  // ---- main loop
  loadGlobal(0);
  storeLds(0);
  __syncthreads();
  for (long step = 0; step < kSteps; ++step) {
    const int buf = static_cast<int>(step & 1);
    if (step + 1 < kSteps) loadGlobal(step + 1);
    compute(buf);
    if (step + 1 < kSteps) storeLds(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: lane owns columns col4 .. col4+3 of 64 rows
  const long col4 = n0 + 4 * (wn * 32 + fragRow);
  if (kFull || col4 < N) {
    epi.prepare(col4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const long row = m0 + wm * 128 + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        if (kFull || row < M) {
          const int a4[4] = {acc[i][0][v], acc[i][1][v], acc[i][2][v], acc[i][3][v]};
          epi.apply(a4, row, col4);
        }
      }
    }
  }
}

}  // namespace akg
