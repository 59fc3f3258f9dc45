/**
 * MFMA GEMM tile kernel for gfx950 (CDNA4) with a caller-supplied epilogue applied to the accumulators while they
 * are still in registers (dequantise / bias / activation / cast fusions). The element type is a template
 * parameter (`Mma`): int8 x int8 -> int32 (v_mfma_i32_32x32x32_i8), bfloat16 or float16 -> float32
 * (v_mfma_f32_32x32x16_bf16 / _f16). Both instruction shapes consume 32 BYTES of K per row and MFMA (a lane holds 16
 * consecutive bytes), so the kernel is written in bytes along K and the LDS layout, the fragment reads and the A
 * staging are the same for every element type; only the in-register transpose of a row-major B differs.
 *
 * Shape of the computation (all sizes are compile-time constants of the emitted kernel):
 *   C[M,N] = A[M,K] * B[K,N]            A row-major, B row-major ([N,K] when TRANSB)
 *   workgroup tile 256 x 256, K step 128 bytes, 4 x 2 wavefronts
 *   wavefront tile 64 x 128 = 2 x 4 MFMA tiles of 32 x 32 (16 accumulator registers each)
 *
 * Data movement:
 *   global -> registers -> LDS, double buffered in LDS (one barrier per K step); the global loads of step
 *   i+1 are issued before the MFMAs of step i.
 *   A: each thread moves 4 x 16 bytes (16 consecutive k of one row) straight into LDS.
 *   B (not transposed) is row-major along N but the MFMA wants, per lane, 16 consecutive k of one column. By default
 *   (TRB) its tile goes to LDS as it lies in memory, 16-byte chunks of a k-row, and the fragments are read with the
 *   transposing LDS reads of gfx950 (ds_read_b64_tr_b8 / _b16: sixteen lanes hand in 8 bytes of a k-row each and get
 *   back, per column, 8 or 4 consecutive k); the staging of both operands is then a plain copy, spread over the
 *   substeps, and the order of MFMAs, LDS accesses and loads inside a substep is fixed with scheduling groups
 *   (int8 4096 x 8192 x 8192: 0.428 -> 0.463 of the MFMA peak, bfloat16: 0.465 -> 0.516; MFMA units busy 58 -> 68 %).
 *   Without TRB each thread loads a 16(k) x 4(n) byte block as 16 dwords, transposes it in registers with
 *   v_perm_b32 (8 permutes per 4 x 4 sub-block) and writes four 16-byte k-vectors to LDS.
 *   LDS rows are 128 data bytes + 16 pad bytes: with a row pitch of 144 bytes consecutive rows start in
 *   different 16-byte bank groups, and the ds_read_b128 fragment loads are conflict free (SQ_LDS_BANK_CONFLICT reads 0).
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
typedef float v16f __attribute__((ext_vector_type(16)));

// Element-type traits of the contraction: bytes per element, accumulator type, and the MFMA on one 16-byte
// fragment per operand (32 x 32 outputs, 32 bytes of K).
struct MmaI8 {
  static constexpr int kElemBytes = 1;
  typedef int acc_t;
  typedef v16i acc_v;
  static AKG_DEV acc_v mma(v4i a, v4i b, acc_v c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0); }
};
struct MmaBF16 {
  static constexpr int kElemBytes = 2;
  typedef float acc_t;
  typedef v16f acc_v;
  typedef __bf16 frag __attribute__((ext_vector_type(8)));
  static AKG_DEV acc_v mma(v4i a, v4i b, acc_v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(frag, a), __builtin_bit_cast(frag, b), c, 0, 0, 0);
  }
};
struct MmaF16 {
  static constexpr int kElemBytes = 2;
  typedef float acc_t;
  typedef v16f acc_v;
  typedef _Float16 frag __attribute__((ext_vector_type(8)));
  static AKG_DEV acc_v mma(v4i a, v4i b, acc_v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(frag, a), __builtin_bit_cast(frag, b), c, 0, 0, 0);
  }
};

constexpr int kGemmBM = 256;
constexpr int kGemmBN = 256;
constexpr int kGemmXcds = 8;
constexpr int kGemmGroupRows = 8;  // tile-rows per group in the swizzled walk

template <bool B>
struct BoolTag {
  static constexpr bool value = B;
};

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

// 2 x 16-bit pairs: out word = (lo or hi half of x, same half of y).
AKG_DEV u32 pack_lo16(u32 x, u32 y) { return __builtin_amdgcn_perm(y, x, 0x05040100u); }
AKG_DEV u32 pack_hi16(u32 x, u32 y) { return __builtin_amdgcn_perm(y, x, 0x07060302u); }

// KE is the K extent in elements; everything below counts K in bytes (K = KE * element size).
// KSPLIT > 1 (few tiles, long K: a skinny A in front of a big weight matrix) gives every tile to KSPLIT workgroups,
// each with a contiguous range of K steps; they leave their accumulators in the workspace `ws` (one arrival counter per
// tile, then kPartRows x 256 accumulators per tile and split), and the last one to arrive adds the partials in split
// order and runs the epilogue: deterministic, and the weight matrix is still read exactly once. The launch has
// KSPLIT times the workgroups; the counters are left at zero.
// Instruction order of a substep of 8 MFMAs with R LDS reads, W LDS writes and L memory loads beside them: after every
// MFMA its share of the others, reads first. (Scheduling-group barriers: the compiler orders the instructions of the
// region to match the sequence of groups, as far as their dependences allow.)
template <int R, int W, int L, int M = 0>
struct SubstepOrder {
  static constexpr int kAll = R + W + L;
  static constexpr int kFrom = M * kAll / 8, kUpto = (M + 1) * kAll / 8;
  static constexpr int within(int lo, int hi) {
    const int a = kFrom > lo ? kFrom : lo, b = kUpto < hi ? kUpto : hi;
    return b > a ? b - a : 0;
  }
  static AKG_DEV void emit() {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (within(0, R) > 0) __builtin_amdgcn_sched_group_barrier(0x100, within(0, R), 0);
    if constexpr (within(R, R + W) > 0) __builtin_amdgcn_sched_group_barrier(0x200, within(R, R + W), 0);
    if constexpr (within(R + W, kAll) > 0) __builtin_amdgcn_sched_group_barrier(0x020, within(R + W, kAll), 0);
    if constexpr (M < 7) SubstepOrder<R, W, L, M + 1>::emit();
  }
};

template <typename Mma, long M, long N, long KE, bool TRANSB, typename Epilogue, int KSPLIT = 1, bool TRB = false>
AKG_DEV void gemm_256x256(const void *__restrict__ A, const void *__restrict__ B, Epilogue &epi,
                          unsigned *__restrict__ ws = nullptr) {
  constexpr int EB = Mma::kElemBytes;
  constexpr long K = KE * EB;    // bytes of K per row of A (and per column of B)
  constexpr long NB = N * EB;    // bytes per k-row of a row-major B
  static_assert(K % 16 == 0, "K must be a multiple of 16 bytes");
  static_assert(TRANSB || (N % 4 == 0), "N must be a multiple of 4");
  // 4 x 2 wavefronts (two per SIMD: one's MFMAs cover the other's loads, transposes and waits), 128 bytes of K per step
  // (every row of A contributes one whole cache line, half as many barriers as with 64; LDS holds 2 x 72 KiB).
  // Staging (global -> registers -> LDS) is done by every thread for both operands: uniform control flow, so the whole
  // K step is one basic block and loads, transposes and LDS writes interleave with the MFMAs. (Measured and dropped:
  // 2 x 2 wavefronts of 128 x 128 each (a third less LDS traffic, one wavefront per SIMD: 2 to 4 % slower, also with the
  // fixed instruction order below), 64-byte steps, staging split between two groups of wavefronts, 256 x 128 tiles
  // with two workgroups per CU; tiles fetched memory -> LDS directly (buffer_load_dwordx4 ... lds into rows without
  // padding, chunks permuted against bank conflicts): correct, 2 % slower than the staging through registers; the K
  // steps of different tiles in rotated order: 8 to 25 % slower, the workgroups of an XCD share their panels in L2
  // only while they walk K together. With the staging switched off altogether the loop runs 17 % faster, whichever
  // way the tiles travel: what is left is the price of moving 64 KB per step and CU on a power-limited part.)
  constexpr int WAVES_M = 4;
  constexpr int BK = 128;
  constexpr int kThreads = WAVES_M * 128;
  constexpr int kStageThreads = kThreads;             // threads that share one operand tile
  constexpr int kPitch = BK + 16;                     // LDS row: BK data bytes + 16 pad (odd multiple of 16)
  constexpr int kSub = BK / 32;                       // MFMA k-substeps per step (2 or 4)
  constexpr int kChunksPerRow = BK / 16;              // 16-byte chunks per row of a K-contiguous operand tile
  constexpr int kRowChunks = 256 * kChunksPerRow / kStageThreads;  // 16-byte chunks per staging thread and operand
  constexpr int kRowStep = kStageThreads / kChunksPerRow;          // rows between two chunks of one thread
  constexpr int kBlockRows = 4 * kRowChunks / EB;     // k-rows of B per staging thread, 4 columns each (16 k-bytes per chunk)
  constexpr int kTM = kGemmBM / (32 * WAVES_M);       // MFMA row tiles per wavefront
  constexpr int kWaveRows = kGemmBM / WAVES_M;
  constexpr long kTilesM = (M + kGemmBM - 1) / kGemmBM;
  constexpr long kTilesN = (N + kGemmBN - 1) / kGemmBN;
  constexpr long kTiles = kTilesM * kTilesN;
  constexpr long kPerXcd = (kTiles + kGemmXcds - 1) / kGemmXcds;
  constexpr long kSteps = (K + BK - 1) / BK;
  constexpr bool kFull = (M % kGemmBM == 0) && (N % kGemmBN == 0) && (K % BK == 0);
  constexpr int kTileBytes = kGemmBM * kPitch;        // one operand tile in LDS
  // TRB: a row-major B goes to LDS as it lies in memory, k-rows of 256 columns, and the fragments are read with the
  // transposing LDS reads (ds_read_b64_tr_b8 / _b16): no transposes in registers.
  static_assert(!(TRB && TRANSB), "the transposing reads are for a row-major B");
  constexpr int kRowBytesB = kGemmBN * EB;            // bytes of one k-row of the B tile
  // Row pitch: the 16 lanes of a transposing read hand in 8 rows x 16 bytes (8-bit) or 4 rows x 32 bytes (16-bit), and the
  // neighbouring 16 lanes the 16 or 32 bytes beside them; with rows 32 (64) bytes apart modulo the 256 bytes of the
  // banks, the two groups of a half wavefront interleave without sharing a bank.
  constexpr int kPitchB = kRowBytesB + (EB == 1 ? 32 : 64);
  constexpr int kRowsB = BK / EB;                     // k-rows per step
  constexpr int kChunksPerRowB = kRowBytesB / 16;
  constexpr int kRowStepB = kStageThreads / kChunksPerRowB;
  static_assert(!TRB || kRowsB * kPitchB <= kTileBytes, "the row-major B tile must fit the operand's LDS space");

  __shared__ __attribute__((aligned(16))) u8 lds[2][2][kTileBytes];  // [buffer][A|B]

  // ---- workgroup -> tile
  constexpr long kGridTiles = kPerXcd * kGemmXcds;   // workgroups per K split (a multiple of the XCD count)
  const long wgAll = static_cast<long>(blockIdx.x);
  const long ksplit = KSPLIT > 1 ? wgAll / kGridTiles : 0;
  const long wg = KSPLIT > 1 ? wgAll % kGridTiles : wgAll;
  const long linear = (wg % kGemmXcds) * kPerXcd + wg / kGemmXcds;
  if (linear >= kTiles) return;
  constexpr long kStepsPer = (kSteps + KSPLIT - 1) / KSPLIT;
  static_assert((KSPLIT - 1) * kStepsPer < kSteps, "every K split needs at least one step");
  const long stepBase = ksplit * kStepsPer;
  const long mySteps = KSPLIT == 1 ? kSteps : ((kSteps - stepBase) < kStepsPer ? (kSteps - stepBase) : kStepsPer);
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

  typename Mma::acc_v acc[kTM][4];
#pragma unroll
  for (int i = 0; i < kTM; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    }
  }

  // ---- staging registers: the tile of step s+1 travels memory -> registers during step s-1.. s and is written to
  // LDS at the top of step s.
  // Every thread stages its share of A (x) and of B (y).
  struct Stage {
    v4i x[kRowChunks];
    v4i y[kRowChunks];
  };
  Stage stage;

  const int ltid = tid;
  const int aRow = ltid / kChunksPerRow;   // + kRowStep * i
  const int aChunk = ltid % kChunksPerRow;
  const int bN4 = ltid & 63;
  const int bKq = ltid >> 6;

  // Global loads are buffer loads: the per-lane offset is computed once, everything that changes from load to load
  // (row block, k-row, K step) is a scalar offset, so the loop spends no vector instructions on addresses (vector
  // instructions and MFMAs compete for issue cycles). Out-of-range lanes read zero through the descriptor's size.
  static_assert(M * K < (1L << 31) && N * K < (1L << 31), "operand too large for 32-bit buffer offsets");
  const __amdgpu_buffer_rsrc_t aRsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void *>(A), 0, static_cast<int>(M * K), 0x00020000);
  const __amdgpu_buffer_rsrc_t bRsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<void *>(B), 0, static_cast<int>(N * K), 0x00020000);
  const int aVoff = static_cast<int>((m0 + aRow) * K + aChunk * 16);
  const int bVoff = TRANSB ? static_cast<int>((n0 + aRow) * K + aChunk * 16)
                           : static_cast<int>((bKq * kBlockRows) * NB + (n0 + 4 * bN4) * EB);
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const int bRowT = ltid / kChunksPerRowB;     // + kRowStepB * i
  const int bChunkT = ltid % kChunksPerRowB;
  const int bVoffT = static_cast<int>(bRowT * NB + n0 * EB + bChunkT * 16);

  auto loadRows = [&](__amdgpu_buffer_rsrc_t rsrc, int voff, long rowBase, long rowLimit, long k0,
                      v4i (&dst)[kRowChunks]) {
    // kRowChunks chunks of 16 consecutive k, rows rowBase + kRowStep * i of a K-contiguous operand
#pragma unroll
    for (int i = 0; i < kRowChunks; ++i) {
      if (kFull || (rowBase + kRowStep * i < rowLimit && k0 + aChunk * 16 < K)) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, static_cast<int>((kRowStep * i) * K + k0), 0);
        dst[i] = v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
      } else {
        dst[i] = v4i{0, 0, 0, 0};
      }
    }
  };
  auto loadBlock = [&](long k0, v4i (&dst)[kRowChunks]) {
    // kBlockRows k-rows x 4 columns of row-major B: one dword (8-bit elements) or two (16-bit) per k-row.
    // k0 is in bytes of K: the first k-row of the step is k0 / EB.
#pragma unroll
    for (int i = 0; i < kBlockRows; ++i) {
      const bool ok = kFull || (n0 + 4 * bN4 < N && k0 / EB + bKq * kBlockRows + i < KE);
      if constexpr (EB == 1) {
        u32 v = 0u;
        if (ok) v = __builtin_amdgcn_raw_buffer_load_b32(bRsrc, bVoff, static_cast<int>((k0 + i) * NB), 0);
        dst[i >> 2][i & 3] = static_cast<int>(v);
      } else {
        typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
        u32x2 v = {0u, 0u};
        if (ok) v = __builtin_amdgcn_raw_buffer_load_b64(bRsrc, bVoff, static_cast<int>((k0 / EB + i) * NB), 0);
        dst[i >> 1][(i & 1) * 2] = static_cast<int>(v[0]);
        dst[i >> 1][(i & 1) * 2 + 1] = static_cast<int>(v[1]);
      }
    }
  };
  auto loadGlobal = [&](long step, Stage &st) {
    const long k0 = (stepBase + step) * BK;
    loadRows(aRsrc, aVoff, m0 + aRow, M, k0, st.x);
    if constexpr (TRANSB) {
      loadRows(bRsrc, bVoff, n0 + aRow, N, k0, st.y);
    } else if constexpr (TRB) {
      // kRowChunks chunks of 16 bytes along n: k-rows bRowT + kRowStepB * i of the step
#pragma unroll
      for (int i = 0; i < kRowChunks; ++i) {
        const long krow = k0 / EB + bRowT + kRowStepB * i;
        if (kFull || (krow < KE && n0 * EB + bChunkT * 16 < NB)) {
          const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(bRsrc, bVoffT, static_cast<int>((k0 / EB + kRowStepB * i) * NB), 0);
          st.y[i] = v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
        } else {
          st.y[i] = v4i{0, 0, 0, 0};
        }
      }
    } else {
      loadBlock(k0, st.y);
    }
  };

  auto storeRowsA = [&](u8 *la, const v4i (&src)[kRowChunks]) {
#pragma unroll
    for (int i = 0; i < kRowChunks; ++i) {
      *reinterpret_cast<v4i *>(la + (aRow + kRowStep * i) * kPitch + aChunk * 16) = src[i];
    }
  };
  auto storeRowsBt = [&](u8 *lb, const v4i (&src)[kRowChunks]) {
#pragma unroll
    for (int i = 0; i < kRowChunks; ++i) {
      const int col = aRow + kRowStep * i;           // column of the tile
      const int r = (col & 3) * 64 + (col >> 2);     // its LDS row
      *reinterpret_cast<v4i *>(lb + r * kPitch + aChunk * 16) = src[i];
    }
  };
  auto storeBlockB16 = [&](u8 *lb, const v4i (&src)[kRowChunks]) {
    // 16-bit elements: src[g] = k-rows 2g, 2g+1, each as (columns 0 1 | columns 2 3). A column's 8 consecutive k
    // (16 bytes) are gathered two at a time with v_perm_b32; a thread holds 8 k-rows.
    static_assert(kRowChunks == 4, "the staging is written for four 16-byte chunks per thread and operand");
    if constexpr (EB == 2) {
#pragma unroll
      for (int h = 0; h < kRowChunks / 4; ++h) {
        v4i w[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32 c01a = static_cast<u32>(src[4 * h + g][0]), c23a = static_cast<u32>(src[4 * h + g][1]);  // k-row 2g
          const u32 c01b = static_cast<u32>(src[4 * h + g][2]), c23b = static_cast<u32>(src[4 * h + g][3]);  // k-row 2g + 1
          w[0][g] = static_cast<int>(pack_lo16(c01a, c01b));
          w[1][g] = static_cast<int>(pack_hi16(c01a, c01b));
          w[2][g] = static_cast<int>(pack_lo16(c23a, c23b));
          w[3][g] = static_cast<int>(pack_hi16(c23a, c23b));
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          *reinterpret_cast<v4i *>(lb + (j * 64 + bN4) * kPitch + bKq * (kRowChunks * 4) + h * 16) = w[j];
        }
      }
    }
  };
  auto storeBlockB8 = [&](u8 *lb, const v4i (&src)[kRowChunks]) {
    // src[g] = 4 k-rows x 4 columns; after the byte transpose t[g][j] = 4 consecutive k of column j
    u32 t[kRowChunks][4];
#pragma unroll
    for (int g = 0; g < kRowChunks; ++g) {
      const u32 rows[4] = {static_cast<u32>(src[g][0]), static_cast<u32>(src[g][1]), static_cast<u32>(src[g][2]),
                           static_cast<u32>(src[g][3])};
      transpose4x4_bytes(rows, t[g]);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int h = 0; h < kRowChunks / 4; ++h) {
        v4i w;
        w[0] = static_cast<int>(t[4 * h + 0][j]);
        w[1] = static_cast<int>(t[4 * h + 1][j]);
        w[2] = static_cast<int>(t[4 * h + 2][j]);
        w[3] = static_cast<int>(t[4 * h + 3][j]);
        *reinterpret_cast<v4i *>(lb + (j * 64 + bN4) * kPitch + bKq * kBlockRows + h * 16) = w;
      }
    }
  };
  auto storeBlockB = [&](u8 *lb, const v4i (&src)[kRowChunks]) {
    if constexpr (EB == 1) {
      storeBlockB8(lb, src);
    } else {
      storeBlockB16(lb, src);
    }
  };
  auto storeLds = [&](int buf, const Stage &st) {
    u8 *la = lds[buf][0];
    u8 *lb = lds[buf][1];
    storeRowsA(la, st.x);
    if constexpr (TRANSB) {
      storeRowsBt(lb, st.y);
    } else if constexpr (TRB) {
#pragma unroll
      for (int i = 0; i < kRowChunks; ++i) {
        *reinterpret_cast<v4i *>(lb + (bRowT + kRowStepB * i) * kPitchB + bChunkT * 16) = st.y[i];
      }
    } else {
      storeBlockB(lb, st.y);
    }
  };

  const int fragRow = lane & 31;
  const int fragHalf = (lane >> 5) * 16;
  const int aFragOff = (wm * kWaveRows + fragRow) * kPitch + fragHalf;
  const int bFragOff = (wn * 32 + fragRow) * kPitch + fragHalf;
  // TRB: lane = 16 g + s. Group g reads the columns 16 (g & 1) .. of the fragment's 32 for the k-half g >> 1; inside
  // the group, 8-bit: lane s hands in k-row s >> 1, column octet s & 1; 16-bit: k-row s >> 2, column quad s & 3.
  const int trS = lane & 15, trG = lane >> 4;
  const int bFragOffT = EB == 1
      ? ((trG >> 1) * 16 + (trS >> 1)) * kPitchB + (wn * 128 + (trG & 1) * 16 + (trS & 1) * 8)
      : ((trG >> 1) * 8 + (trS >> 2)) * kPitchB + (wn * 128 + (trG & 1) * 16 + (trS & 3) * 4) * 2;

  // Wavefronts whose rows all lie below the last row of A (a skinny A: M = 16 leaves three of the four wavefront rows
  // without a single real row) take part in the staging and the barriers but skip fragment reads and MFMAs.
  constexpr bool kAllRowsReal = (M % kGemmBM == 0);
  const bool waveHasRows = kAllRowsReal || (m0 + wm * kWaveRows < M);
  auto readFrags = [&](int buf, int ks, v4i (&af)[kTM], v4i (&bf)[4]) {
    if (!kAllRowsReal && !waveHasRows) return;
    const u8 *la = lds[buf][0] + aFragOff + ks * 32;
    const u8 *lb = lds[buf][1] + bFragOff + ks * 32;
#pragma unroll
    for (int i = 0; i < kTM; ++i) af[i] = *reinterpret_cast<const v4i *>(la + i * 32 * kPitch);
    if constexpr (TRB) {
      // Sixteen lanes share a transposing read: each hands in 8 bytes of one k-row and gets back, for one column,
      // the elements of 8 (8-bit) or 4 (16-bit) consecutive k-rows. Two reads make the 16 bytes of K of a fragment.
      typedef int v2i __attribute__((ext_vector_type(2)));
      typedef short v4s __attribute__((ext_vector_type(4)));
      const u8 *lt = lds[buf][1] + bFragOffT + ks * (32 / EB) * kPitchB;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u8 *p0 = lt + j * 32 * EB;
        const u8 *p1 = p0 + (8 / EB) * kPitchB;
        if constexpr (EB == 1) {
          const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)(p0));
          const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)(p1));
          bf[j] = v4i{lo[0], lo[1], hi[0], hi[1]};
        } else {
          const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)(p0));
          const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4s *)(p1));
          const v2i l2 = __builtin_bit_cast(v2i, lo), h2 = __builtin_bit_cast(v2i, hi);
          bf[j] = v4i{l2[0], l2[1], h2[0], h2[1]};
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) bf[j] = *reinterpret_cast<const v4i *>(lb + j * 64 * kPitch);
    }
  };
  auto mfmaAll = [&](const v4i (&af)[kTM], const v4i (&bf)[4]) {
    if (!kAllRowsReal && !waveHasRows) return;
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[i][j] = Mma::mma(af[i], bf[j], acc[i][j]);
      }
    }
  };

  // ---- main loop. Invariant at the top of step s: LDS buffer s&1 holds tile s (complete), the staging registers hold
  // tile s+1 (possibly still in flight), and f0 holds the fragments of the first 32 k of tile s.
  //   a. staged tile s+1 -> LDS buffer (s+1)&1      (its last readers finished before the previous barrier)
  //   b. issue the global loads of tile s+2 into the staging registers (they have a whole step to arrive)
  //   c. for every k-substep but the last: read the next substep's fragments, MFMAs on the current ones
  //      (a and b interleave with the MFMAs of the early substeps)
  //   d. barrier: everybody has read tile s completely and has written tile s+1
  //   e. read the first fragments of tile s+1         (their latency hides behind the MFMAs of f)
  //   f. MFMAs on the last substep's fragments
  v4i f0a[kTM], f0b[4], f1a[kTM], f1b[4];
  // One K step. kStore / kLoad are compile-time so that the steady-state loop body is a single basic block (the
  // last two steps, which have nothing left to store or load, are peeled off below).
  auto stepBody = [&](long step, auto storeTag, auto loadTag) {
    constexpr bool kStore = decltype(storeTag)::value;
    constexpr bool kLoad = decltype(loadTag)::value;
    const int buf = static_cast<int>(step & 1);
    // The staged tile goes to the other LDS buffer at the very top of the step (its last readers finished before
    // the previous step's barrier), and the freed staging registers are refilled at once: the LDS writes complete
    // and the global loads travel while the step's MFMAs run, instead of piling up in front of the barrier.
    if constexpr (kStore) storeLds(buf ^ 1, stage);
    if constexpr (kLoad) loadGlobal(step + 2, stage);
#pragma unroll
    for (int ks = 0; ks + 2 < kSub; ks += 2) {
      readFrags(buf, ks + 1, f1a, f1b);
      mfmaAll(f0a, f0b);
      readFrags(buf, ks + 2, f0a, f0b);
      mfmaAll(f1a, f1b);
    }
    if constexpr (kSub > 2) __builtin_amdgcn_sched_barrier(0);  // keep the staging work in the early substeps
    readFrags(buf, kSub - 1, f1a, f1b);
    mfmaAll(f0a, f0b);
    __syncthreads();
    // ---- after the barrier: MFMAs on the last fragments of this tile; meanwhile fetch the first fragments of the next
    if constexpr (kStore) readFrags(buf ^ 1, 0, f0a, f0b);
    mfmaAll(f1a, f1b);
  };
  // ---- the same step with the staging spread over the substeps (operands whose staging is a plain copy of 16-byte
  // chunks: B transposed in memory, or read with the transposing LDS reads): substep ks writes chunk ks of both operands
  // to LDS and refills its registers from the tile after next, so that every group of 8 MFMAs has about the same
  // number of LDS and memory instructions to cover; the order inside a substep is then fixed instruction by
  // instruction (one MFMA, then a few of the others) instead of left to the scheduler, which clusters them.
  constexpr bool kSpread = (TRB || TRANSB) && kSub == 4 && kRowChunks == 4;
  auto storeChunk = [&](int buf, int i) {
    u8 *la = lds[buf][0];
    u8 *lb = lds[buf][1];
    *reinterpret_cast<v4i *>(la + (aRow + kRowStep * i) * kPitch + aChunk * 16) = stage.x[i];
    if constexpr (TRANSB) {
      const int col = aRow + kRowStep * i;
      const int r = (col & 3) * 64 + (col >> 2);
      *reinterpret_cast<v4i *>(lb + r * kPitch + aChunk * 16) = stage.y[i];
    } else {
      *reinterpret_cast<v4i *>(lb + (bRowT + kRowStepB * i) * kPitchB + bChunkT * 16) = stage.y[i];
    }
  };
  auto loadChunk = [&](long step, int i) {
    const long k0 = (stepBase + step) * BK;
    if (kFull || (m0 + aRow + kRowStep * i < M && k0 + aChunk * 16 < K)) {
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(aRsrc, aVoff, static_cast<int>((kRowStep * i) * K + k0), 0);
      stage.x[i] = v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
    } else {
      stage.x[i] = v4i{0, 0, 0, 0};
    }
    if constexpr (TRANSB) {
      if (kFull || (n0 + aRow + kRowStep * i < N && k0 + aChunk * 16 < K)) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(bRsrc, bVoff, static_cast<int>((kRowStep * i) * K + k0), 0);
        stage.y[i] = v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
      } else {
        stage.y[i] = v4i{0, 0, 0, 0};
      }
    } else {
      const long krow = k0 / EB + bRowT + kRowStepB * i;
      if (kFull || (krow < KE && n0 * EB + bChunkT * 16 < NB)) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(bRsrc, bVoffT, static_cast<int>((k0 / EB + kRowStepB * i) * NB), 0);
        stage.y[i] = v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
      } else {
        stage.y[i] = v4i{0, 0, 0, 0};
      }
    }
  };
  auto stepSpread = [&](long step, auto storeTag, auto loadTag) {
    constexpr bool kStore = decltype(storeTag)::value;
    constexpr bool kLoad = decltype(loadTag)::value;
    constexpr int kFragReads = kTM + (TRB ? 8 : 4);
    const int buf = static_cast<int>(step & 1);
    // substep 0: fragments of substep 1; chunks 0 and 1 of tile s+1 to LDS
    readFrags(buf, 1, f1a, f1b);
    if constexpr (kStore) {
      storeChunk(buf ^ 1, 0);
      storeChunk(buf ^ 1, 1);
    }
    mfmaAll(f0a, f0b);
    SubstepOrder<kFragReads, kStore ? 4 : 0, 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    // substep 1: fragments of substep 2; chunk 2 to LDS; chunks 0 and 1 of tile s+2 on their way
    readFrags(buf, 2, f0a, f0b);
    if constexpr (kStore) storeChunk(buf ^ 1, 2);
    if constexpr (kLoad) {
      loadChunk(step + 2, 0);
      loadChunk(step + 2, 1);
    }
    mfmaAll(f1a, f1b);
    SubstepOrder<kFragReads, kStore ? 2 : 0, kLoad ? 4 : 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    // substep 2: fragments of substep 3; chunk 3 to LDS; chunk 2 on its way
    readFrags(buf, 3, f1a, f1b);
    if constexpr (kStore) storeChunk(buf ^ 1, 3);
    if constexpr (kLoad) loadChunk(step + 2, 2);
    mfmaAll(f0a, f0b);
    SubstepOrder<kFragReads, kStore ? 2 : 0, kLoad ? 2 : 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();   // everybody has read tile s completely and has written tile s+1
    // substep 3: first fragments of tile s+1; chunk 3 on its way
    if constexpr (kStore) readFrags(buf ^ 1, 0, f0a, f0b);
    if constexpr (kLoad) loadChunk(step + 2, 3);
    mfmaAll(f1a, f1b);
    SubstepOrder<kStore ? kFragReads : 0, 0, kLoad ? 2 : 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
  };
  loadGlobal(0, stage);
  storeLds(0, stage);
  if (mySteps > 1) loadGlobal(1, stage);
  __syncthreads();
  readFrags(0, 0, f0a, f0b);
  long step = 0;
  if constexpr (kSpread) {
    for (; step + 2 < mySteps; ++step) stepSpread(step, BoolTag<true>(), BoolTag<true>());
    if (step + 1 < mySteps) {
      stepSpread(step, BoolTag<true>(), BoolTag<false>());
      ++step;
    }
    stepSpread(step, BoolTag<false>(), BoolTag<false>());
  } else {
    for (; step + 2 < mySteps; ++step) stepBody(step, BoolTag<true>(), BoolTag<true>());
    if (step + 1 < mySteps) {
      stepBody(step, BoolTag<true>(), BoolTag<false>());
      ++step;
    }
    stepBody(step, BoolTag<false>(), BoolTag<false>());
  }

  // ---- epilogue: lane owns columns col4 .. col4+3 of 16 * kTM rows
  // With the transposing reads column tile j holds the columns 32 j .. 32 j + 31 of the wavefront's 128, lane by lane,
  // so the four lanes of a quad hold four neighbouring columns of each of the four tiles: a 4 x 4 transpose between
  // the lanes of the quad and the tiles (two exchanges with quad permutations) gives lane c the four columns of tile c.
  if constexpr (TRB) {
    const bool odd = (lane & 1) != 0, upper = (lane & 2) != 0;
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        typename Mma::acc_t a0 = acc[i][0][v], a1 = acc[i][1][v], a2 = acc[i][2][v], a3 = acc[i][3][v];
        const typename Mma::acc_t r01 = lane_partner<1>(odd ? a0 : a1), r23 = lane_partner<1>(odd ? a2 : a3);
        if (odd) { a0 = r01; a2 = r23; } else { a1 = r01; a3 = r23; }
        const typename Mma::acc_t r02 = lane_partner<2>(upper ? a0 : a2), r13 = lane_partner<2>(upper ? a1 : a3);
        if (upper) { a0 = r02; a1 = r13; } else { a2 = r02; a3 = r13; }
        acc[i][0][v] = a0;
        acc[i][1][v] = a1;
        acc[i][2][v] = a2;
        acc[i][3][v] = a3;
      }
    }
  }
  const long col4 = TRB ? n0 + wn * 128 + 32 * (lane & 3) + (fragRow & ~3) : n0 + 4 * (wn * 32 + fragRow);
  if constexpr (KSPLIT > 1) {
    constexpr long kPartRows = M < kGemmBM ? M : kGemmBM;            // rows of a tile that can hold results
    constexpr long kCounterBytes = (kGridTiles * 4 + 255) / 256 * 256;
    constexpr long kPartBytes = kPartRows * kGemmBN * static_cast<long>(sizeof(typename Mma::acc_t));
    constexpr long kWsBytes = kCounterBytes + kTiles * KSPLIT * kPartBytes;
    static_assert(kWsBytes < (1L << 31), "split-K workspace too large");
    const Buffer wsBuf = make_buffer(ws, kWsBytes);
    const u32 tileBase = static_cast<u32>(kCounterBytes + linear * KSPLIT * kPartBytes);
    const bool colOk = kFull || col4 < N;
    auto partOffset = [&](int i, int v) {
      const long rowInTile = wm * kWaveRows + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
      return static_cast<long>((rowInTile * kGemmBN + (col4 - n0)) * static_cast<long>(sizeof(typename Mma::acc_t)));
    };
    auto rowOk = [&](int i, int v) {
      const long rowInTile = wm * kWaveRows + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
      return rowInTile < kPartRows && m0 + rowInTile < M;
    };
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        if (colOk && rowOk(i, v)) {
          const typename Mma::acc_t a4[4] = {acc[i][0][v], acc[i][1][v], acc[i][2][v], acc[i][3][v]};
          ws_store_chunk<4>(wsBuf, tileBase + static_cast<u32>(ksplit * kPartBytes + partOffset(i, v)), a4);
        }
      }
    }
    __shared__ unsigned akg_gemm_flag;
    if (!last_workgroup(ws, linear, KSPLIT, tid, &akg_gemm_flag)) return;
    if (!colOk) return;
    epi.prepare(col4);
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        if (!rowOk(i, v)) continue;
        typename Mma::acc_t sum[4] = {0, 0, 0, 0};
        for (int p = 0; p < KSPLIT; ++p) {
          typename Mma::acc_t part[4];
          ws_load_chunk<4>(wsBuf, tileBase + static_cast<u32>(p * kPartBytes + partOffset(i, v)), part);
#pragma unroll
          for (int c = 0; c < 4; ++c) sum[c] += part[c];
        }
        const long row = m0 + wm * kWaveRows + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        epi.apply(sum, row, col4);
      }
    }
    return;
  }
  if (kFull || col4 < N) {
    epi.prepare(col4);
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const long row = m0 + wm * kWaveRows + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
        if (kFull || row < M) {
          const typename Mma::acc_t a4[4] = {acc[i][0][v], acc[i][1][v], acc[i][2][v], acc[i][3][v]};
          epi.apply(a4, row, col4);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// Skinny A (M <= 64 rows: a decoding step, a GEMV): the time is that of streaming B once, so B goes from global memory
// straight into MFMA operands, without LDS and without barriers in the main loop.
//   workgroup = 4 wavefronts, one strip of 128 columns, one range of K (KSPLIT ranges per strip)
//   wavefront w takes the MFMA steps (32 bytes of K each) w, w + 4, ... of that range, two steps' loads in flight
//   lane (n = lane % 32, g = lane / 32) owns the 4 ADJACENT columns 4n .. 4n+3 of the strip and the 16 bytes
//   [32 t + 16 g, +16) of K: for a row-major B it loads a (16 bytes of K) x (4 columns) block (8 rows x 8 bytes or
//   16 rows x 4 bytes) and transposes it in registers into four operands, for [N,K] it loads the four operands as they
//   are; one MFMA per column of the four, all against the same one or two A operands (32 rows each; rows beyond M repeat row M-1 and are dropped)
// The four wavefronts add their accumulators through LDS (only the M real rows), the KSPLIT workgroups of a strip
// through the workspace in split order (counter per strip, then M x 128 partials per strip and split), and the thread
// that owns (row, 4 columns) runs the epilogue on the sums. Deterministic; B is read exactly once.
template <typename Mma, long M, long N, long KE, bool TRANSB, typename Epilogue, int KSPLIT, int WAVES = 4, int UNROLL = 2, bool NT = false>
AKG_DEV void gemm_skinny(const void *__restrict__ Av, const void *__restrict__ Bv, Epilogue &epi,
                         unsigned *__restrict__ ws, long group0) {
  constexpr int EB = Mma::kElemBytes;
  constexpr long K = KE * EB;   // bytes of K per row of A
  constexpr long NB = N * EB;   // bytes per k-row of a row-major B
  static_assert(M >= 1 && M <= 128, "at most 128 rows");
  constexpr int kRowTiles = static_cast<int>((M + 31) / 32);   // MFMA tiles of 32 rows
  static_assert(K % 32 == 0, "K must be a multiple of 32 bytes");
  static_assert(TRANSB || N % 4 == 0, "N must be a multiple of 4");
  constexpr long kSteps = K / 32;
  constexpr long kStrips = (N + 127) / 128;
  constexpr int kWaves = WAVES, U = UNROLL;
  static_assert(WAVES == 4 || WAVES == 8, "4 or 8 wavefronts");
  constexpr int kRawWords = 16;   // dwords a lane loads per step: 64 bytes whatever the layout
  typedef typename Mma::acc_t acc_t;
  typedef typename Mma::acc_v acc_v;
  const int tid = static_cast<int>(threadIdx.x), lane = tid & 63, wave = tid >> 6;
  const long strip = static_cast<long>(blockIdx.x) % kStrips;   // neighbours in launch order read neighbouring columns
  const int ksplit = static_cast<int>(static_cast<long>(blockIdx.x) / kStrips);
  const long t0 = kSteps * ksplit / KSPLIT, t1 = kSteps * (ksplit + 1) / KSPLIT;
  const int n32 = lane & 31, kg = lane >> 5;
  const long myCol = strip * 128 + 4 * n32;
  const long ldCol = myCol + 3 < N ? myCol : 0;   // columns beyond N: load something valid, the results are dropped
  const char *__restrict__ A[kRowTiles];
#pragma unroll
  for (int rt = 0; rt < kRowTiles; ++rt) {
    const long rowA = 32 * rt + n32 < M ? 32 * rt + n32 : M - 1;
    A[rt] = static_cast<const char *>(Av) + rowA * K + kg * 16;
  }
  const char *__restrict__ B = static_cast<const char *>(Bv);
  acc_v acc[kRowTiles][4];
#pragma unroll
  for (int rt = 0; rt < kRowTiles; ++rt) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[rt][c][v] = 0;
    }
  }
  struct Raw {
    v4i a[kRowTiles];
    u32 w[kRawWords];
  };
  auto load = [&](long t, Raw &r) {
    const long kb = t * 32 + kg * 16;   // this lane's first byte of K
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt) r.a[rt] = *reinterpret_cast<const v4i *>(A[rt] + t * 32);
    if constexpr (TRANSB) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const v4i *bp = reinterpret_cast<const v4i *>(B + (ldCol + c) * K + kb);
        const v4i q = NT ? __builtin_nontemporal_load(bp) : *bp;
        r.w[4 * c + 0] = static_cast<u32>(q[0]);
        r.w[4 * c + 1] = static_cast<u32>(q[1]);
        r.w[4 * c + 2] = static_cast<u32>(q[2]);
        r.w[4 * c + 3] = static_cast<u32>(q[3]);
      }
    } else if constexpr (EB == 2) {
      const long k0 = kb / 2;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        typedef u32 v2u __attribute__((ext_vector_type(2)));
        const v2u *bp = reinterpret_cast<const v2u *>(B + (k0 + j) * NB + ldCol * 2);
        const v2u q = NT ? __builtin_nontemporal_load(bp) : *bp;
        r.w[2 * j] = q[0];
        r.w[2 * j + 1] = q[1];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const u32 *bp = reinterpret_cast<const u32 *>(B + (kb + j) * NB + ldCol);
        r.w[j] = NT ? __builtin_nontemporal_load(bp) : *bp;
      }
    }
  };
  auto mfma = [&](const Raw &r) {
    v4i b[4];
    if constexpr (TRANSB) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
#pragma unroll
        for (int i = 0; i < 4; ++i) b[c][i] = static_cast<int>(r.w[4 * c + i]);
      }
    } else if constexpr (EB == 2) {
      // rows 2i, 2i+1 of the block -> word i of every column's operand
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        b[0][i] = static_cast<int>(pack_lo16(r.w[4 * i], r.w[4 * i + 2]));
        b[1][i] = static_cast<int>(pack_hi16(r.w[4 * i], r.w[4 * i + 2]));
        b[2][i] = static_cast<int>(pack_lo16(r.w[4 * i + 1], r.w[4 * i + 3]));
        b[3][i] = static_cast<int>(pack_hi16(r.w[4 * i + 1], r.w[4 * i + 3]));
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const u32 rows[4] = {r.w[4 * i], r.w[4 * i + 1], r.w[4 * i + 2], r.w[4 * i + 3]};
        u32 cols[4];
        transpose4x4_bytes(rows, cols);
#pragma unroll
        for (int c = 0; c < 4; ++c) b[c][i] = static_cast<int>(cols[c]);
      }
    }
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt) {
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[rt][c] = Mma::mma(r.a[rt], b[c], acc[rt][c]);
    }
  };
  for (long t = t0 + wave; t < t1; t += kWaves * U) {   // (uniform per wavefront)
    Raw r[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (t + u * kWaves < t1) load(t + u * kWaves, r[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (t + u * kWaves < t1) mfma(r[u]);
    }
  }

  // ---- the four wavefronts' sums, rows below M only, 16 rows at a time: accumulator v of a lane is row
  // 8 (v / 4) + 4 g + v % 4; thread (c4, r0) then owns 4 columns of the strip and the rows r0, r0 + 8, ...
  constexpr int kHalfRows = M < 16 ? static_cast<int>(M) : 16;
  __shared__ acc_t akg_skinny_sum[kWaves][kHalfRows][128];
  const int c4 = tid & 31, r0 = (tid >> 5) & 7;
  const long col = strip * 128 + 4 * c4;
  const bool colOk = col < N && tid < 256;   // (of 8 wavefronts the first four finish the sums)
  constexpr int kRowsPerThread = (M + 7) / 8;
  acc_t sum[kRowsPerThread][4];
#pragma unroll
  for (int h = 0; h < (M + 15) / 16; ++h) {
    if (h > 0) __syncthreads();
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      if ((v >> 3) != (h & 1)) continue;            // rows 16 h .. 16 h + 15: tile h / 2, accumulators 8 (h % 2) .. + 7
      const int row = 32 * (h >> 1) + 8 * (v >> 2) + 4 * kg + (v & 3);
      if (row < M) {
#pragma unroll
        for (int c = 0; c < 4; ++c) akg_skinny_sum[wave][row - 16 * h][4 * n32 + c] = acc[h >> 1][c][v];
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 2 * h; i < 2 * h + 2 && i < kRowsPerThread; ++i) {
      const int row = r0 + 8 * i;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        sum[i][c] = 0;
        if (row < M) {
#pragma unroll
          for (int w = 0; w < kWaves; ++w) sum[i][c] += akg_skinny_sum[w][row - 16 * h][4 * c4 + c];
        }
      }
    }
  }
  if constexpr (KSPLIT > 1) {
    constexpr long kPartBytes = M * 128 * static_cast<long>(sizeof(acc_t));
    const long group = group0 + strip;
    // layout: [groups x 4 bytes of counters, rounded up to 256][group][split][M][128]
    const long groups = static_cast<long>(gridDim.y) * kStrips;
    const long counterBytes = (groups * 4 + 255) / 256 * 256;
    const Buffer wsBuf = make_buffer(ws, counterBytes + groups * KSPLIT * kPartBytes);
    const u32 base = static_cast<u32>(counterBytes + group * KSPLIT * kPartBytes);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
      const int row = r0 + 8 * i;
      if (row < M && colOk) {
        ws_store_chunk<4>(wsBuf, base + static_cast<u32>(ksplit * kPartBytes + (row * 128 + 4 * c4) * static_cast<long>(sizeof(acc_t))), sum[i]);
      }
    }
    __shared__ unsigned akg_skinny_flag;
    if (!last_workgroup(ws, group, KSPLIT, tid, &akg_skinny_flag)) return;
    if (!colOk) return;
    epi.prepare(col);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
      const int row = r0 + 8 * i;
      if (row >= M) continue;
      acc_t total[4] = {0, 0, 0, 0};
      for (int p = 0; p < KSPLIT; ++p) {
        acc_t part[4];
        ws_load_chunk<4>(wsBuf, base + static_cast<u32>(p * kPartBytes + (row * 128 + 4 * c4) * static_cast<long>(sizeof(acc_t))), part);
#pragma unroll
        for (int c = 0; c < 4; ++c) total[c] += part[c];
      }
      epi.apply(total, row, col);
    }
    return;
  }
  if (!colOk) return;
  epi.prepare(col);
#pragma unroll
  for (int i = 0; i < kRowsPerThread; ++i) {
    const int row = r0 + 8 * i;
    if (row < M) epi.apply(sum[i], row, col);
  }
}

}  // namespace akg
