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

// WAVES_M x 2 wavefronts per workgroup: 2 x 2 (one wavefront per SIMD, 128 x 128 per wavefront, 256 accumulator
// registers) or 4 x 2 (two wavefronts per SIMD, 64 x 128 per wavefront, 128 accumulator registers: the second
// wavefront's MFMAs cover the first one's loads, transposes and barriers).
template <long M, long N, long K, bool TRANSB, int WAVES_M, typename Epilogue>
AKG_DEV void gemm_i8_256x256(const s8 *__restrict__ A, const s8 *__restrict__ B, Epilogue &epi) {
  static_assert(K % 16 == 0, "K must be a multiple of 16");
  static_assert(TRANSB || (N % 4 == 0), "N must be a multiple of 4");
  static_assert(WAVES_M == 2 || WAVES_M == 4, "2 x 2 or 4 x 2 wavefronts");
  constexpr int kWaves = WAVES_M * 2;
  constexpr int kThreads = kWaves * 64;
  constexpr int kTM = kGemmBM / (32 * WAVES_M);       // MFMA row tiles per wavefront
  constexpr int kWaveRows = kGemmBM / WAVES_M;
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

  v16i acc[kTM][4];
#pragma unroll
  for (int i = 0; i < kTM; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    }
  }

  // ---- staging registers (one K step ahead of LDS, two ahead of the MFMAs)
  // 2 x 2 wavefronts: every thread stages 4 chunks of A and a 16 x 4 block of B.
  // 4 x 2 wavefronts: wavefronts 0..3 stage all of B (16 x 4 blocks, 128-bit LDS writes stay conflict free),
  //                   wavefronts 4..7 stage all of A.
  constexpr bool kSplitDuty = (WAVES_M == 4);
  v4i ga[4];
  u32 gb[16];   // !TRANSB: 16 k-rows x 4 columns
  v4i gbt[4];   // TRANSB: like A

  const int ltid = tid & 255;
  const bool stageA = !kSplitDuty || tid >= 256;
  const bool stageB = !kSplitDuty || tid < 256;
  const int aRow = ltid >> 2;   // + 64 * i
  const int aChunk = ltid & 3;
  const int bN4 = ltid & 63;
  const int bKq = ltid >> 6;

  const s8 *aSrc = A + (m0 + aRow) * K + aChunk * 16;
  const s8 *bSrc = TRANSB ? (B + (n0 + aRow) * K + aChunk * 16) : (B + (bKq * 16) * N + n0 + 4 * bN4);

  auto loadGlobal = [&](long step) {
    const long k0 = step * kGemmBK;
    if (stageA) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (kFull || (m0 + aRow + 64 * i < M && k0 + aChunk * 16 < K)) {
          ga[i] = *reinterpret_cast<const v4i *>(aSrc + (64 * i) * K + k0);
        } else {
          ga[i] = v4i{0, 0, 0, 0};
        }
      }
    }
    if (stageB) {
      if constexpr (TRANSB) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (kFull || (n0 + aRow + 64 * i < N && k0 + aChunk * 16 < K)) {
            gbt[i] = *reinterpret_cast<const v4i *>(bSrc + (64 * i) * K + k0);
          } else {
            gbt[i] = v4i{0, 0, 0, 0};
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if (kFull || (n0 + 4 * bN4 < N && k0 + bKq * 16 + i < K)) {
            gb[i] = *reinterpret_cast<const u32 *>(bSrc + (k0 + i) * N);
          } else {
            gb[i] = 0u;
          }
        }
      }
    }
  };

  auto storeLds = [&](int buf) {
    u8 *la = lds[buf][0];
    u8 *lb = lds[buf][1];
    if (stageA) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *reinterpret_cast<v4i *>(la + (aRow + 64 * i) * kGemmPitch + aChunk * 16) = ga[i];
      }
    }
    if (stageB) {
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
    }
  };

  const int fragRow = lane & 31;
  const int fragHalf = (lane >> 5) * 16;
  const int aFragOff = (wm * kWaveRows + fragRow) * kGemmPitch + fragHalf;
  const int bFragOff = (wn * 32 + fragRow) * kGemmPitch + fragHalf;

  auto readFrags = [&](int buf, int ks, v4i (&af)[kTM], v4i (&bf)[4]) {
    const u8 *la = lds[buf][0] + aFragOff + ks * 32;
    const u8 *lb = lds[buf][1] + bFragOff + ks * 32;
#pragma unroll
    for (int i = 0; i < kTM; ++i) af[i] = *reinterpret_cast<const v4i *>(la + i * 32 * kGemmPitch);
#pragma unroll
    for (int j = 0; j < 4; ++j) bf[j] = *reinterpret_cast<const v4i *>(lb + j * 64 * kGemmPitch);
  };
  auto mfmaAll = [&](const v4i (&af)[kTM], const v4i (&bf)[4]) {
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
    }
  };

  // ---- main loop. Invariant at the top of step s: LDS buffer s&1 holds tile s (complete), the staging registers
  // hold tile s+1, and f0 holds the fragments of the first half (k 0..31) of tile s.
  //   a. staged tile s+1 -> LDS buffer (s+1)&1        (its last readers finished before the previous barrier)
  //   b. issue the global loads of tile s+2 into the staging registers
  //   c. read the second-half fragments f1 of tile s
  //   d. MFMAs on f0
  //   e. barrier: everybody has read tile s completely and has written tile s+1
  //   f. read the first-half fragments of tile s+1     (its latency hides behind the MFMAs of g)
  //   g. MFMAs on f1
  v4i f0a[kTM], f0b[4], f1a[kTM], f1b[4];
  loadGlobal(0);
  storeLds(0);
  if (kSteps > 1) loadGlobal(1);
  __syncthreads();
  readFrags(0, 0, f0a, f0b);
  for (long step = 0; step < kSteps; ++step) {
    const int buf = static_cast<int>(step & 1);
#ifndef AKG_DIAG_NO_LDS_STORE
    if (step + 1 < kSteps) storeLds(buf ^ 1);
#endif
#ifndef AKG_DIAG_NO_GLOBAL_LOAD
    if (step + 2 < kSteps) loadGlobal(step + 2);
#endif
    // Keep the global loads here: left to itself the scheduler sinks them to the end of the step (shorter live
    // ranges), which exposes the full memory latency at the top of the next step.
    __builtin_amdgcn_sched_barrier(0);
#ifndef AKG_DIAG_NO_FRAG_READ
    readFrags(buf, 1, f1a, f1b);
#endif
#ifndef AKG_DIAG_NO_MFMA
    mfmaAll(f0a, f0b);
#endif
#ifndef AKG_DIAG_NO_BARRIER
    __syncthreads();
#endif
#ifndef AKG_DIAG_NO_FRAG_READ
    if (step + 1 < kSteps) readFrags(buf ^ 1, 0, f0a, f0b);
#endif
#ifndef AKG_DIAG_NO_MFMA
    mfmaAll(f1a, f1b);
#endif
  }

  // ---- epilogue: lane owns columns col4 .. col4+3 of 16 * kTM rows
  const long col4 = n0 + 4 * (wn * 32 + fragRow);
  if (kFull || col4 < N) {
    epi.prepare(col4);
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const long row = m0 + wm * kWaveRows + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        if (kFull || row < M) {
          const int a4[4] = {acc[i][0][v], acc[i][1][v], acc[i][2][v], acc[i][3][v]};
          epi.apply(a4, row, col4);
        }
      }
    }
  }
}

}  // namespace akg
