/**
 * MFMA GEMM tile kernel for gfx950 (CDNA4) with a caller-supplied epilogue applied to the accumulators while they
 * are still in registers (dequantise / bias / activation / cast fusions). The element type is a template
 * parameter (`Mma`): int8 x int8 -> int32 (v_mfma_i32_16x16x64_i8), bfloat16 or float16 -> float32
 * (v_mfma_f32_16x16x32_bf16 / _f16). Both instruction shapes consume 64 BYTES of K per row and MFMA (a lane holds 16
 * consecutive bytes), so the kernel is written in bytes along K and the LDS layout, the fragment reads and the
 * staging are the same for every element type.
 * Why 16 x 16 tiles and not 32 x 32 (half the MFMAs for the same work): the part is power limited, and a loop of
 * nothing but MFMAs on random operands sustains 0.85 of the nominal peak in the 16 x 16 shapes against 0.72 (int8) and
 * 0.75 (bfloat16) in the 32 x 32 ones; the same kernel on 32 x 32 MFMAs was 5 % (int8) and 3 % (bfloat16) slower.
 *
 * Shape of the computation (all sizes are compile-time constants of the emitted kernel):
 *   C[M,N] = A[M,K] * B[K,N]            A row-major, B row-major ([N,K] when TRANSB)
 *   workgroup tile 256 x 256, K step 128 bytes, 4 x 2 wavefronts (WM = 4) or 2 x 4 (WM = 2)
 *   wavefront tile 64 x 128 = 4 x 8 MFMA tiles of 16 x 16 (4 accumulator registers each), or 128 x 64 = 8 x 4
 *
 * Data movement:
 *   global -> registers -> LDS, double buffered in LDS (one barrier per K step); the global loads of step
 *   i+2 are issued during step i. Both operands travel as 16-byte chunks, a plain copy.
 *   A (and a B given as [N,K]): rows of 128 data bytes + 16 pad bytes; with a row pitch of 144 bytes consecutive rows
 *   start in different 16-byte bank groups. Fragments are read with ds_read_b128.
 *   B row-major: its tile goes to LDS as it lies in memory, k-rows of 256 columns, and the fragments are read with the
 *   transposing LDS reads of gfx950 (ds_read_b64_tr_b8 / _b16: sixteen lanes hand in 8 bytes of a k-row each and get
 *   back, per column, 8 or 4 consecutive k): no transposes in registers.
 *   SQ_LDS_BANK_CONFLICT reads 0 for both layouts (how the chunks are placed for that is said where they are written).
 *   Every lane ends up owning 4 ADJACENT output columns (by the order of the LDS rows of an [N,K] B; by a 4 x 4
 *   exchange inside each lane quad for a row-major B): the epilogue works on 4-element chunks and sixteen lanes store
 *   one aligned piece of 64 columns per output row.
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
typedef float v4f __attribute__((ext_vector_type(4)));

// Element-type traits of the contraction: bytes per element, accumulator type, and the MFMA on one 16-byte
// fragment per operand: `mma16` 16 x 16 outputs and 64 bytes of K (the tile kernel), `mma` 32 x 32 outputs and 32 bytes
// of K (the skinny kernel, whose time is that of streaming B).
struct MmaI8 {
  static constexpr int kElemBytes = 1;
  typedef int acc_t;
  typedef v16i acc_v;
  typedef v4i acc4_v;
  static AKG_DEV acc_v mma(v4i a, v4i b, acc_v c) { return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0); }
  static AKG_DEV acc4_v mma16(v4i a, v4i b, acc4_v c) { return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0); }
};
struct MmaBF16 {
  static constexpr int kElemBytes = 2;
  typedef float acc_t;
  typedef v16f acc_v;
  typedef __bf16 frag __attribute__((ext_vector_type(8)));
  static AKG_DEV acc_v mma(v4i a, v4i b, acc_v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(frag, a), __builtin_bit_cast(frag, b), c, 0, 0, 0);
  }
  typedef v4f acc4_v;
  static AKG_DEV acc4_v mma16(v4i a, v4i b, acc4_v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(frag, a), __builtin_bit_cast(frag, b), c, 0, 0, 0);
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
  typedef v4f acc4_v;
  static AKG_DEV acc4_v mma16(v4i a, v4i b, acc4_v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(frag, a), __builtin_bit_cast(frag, b), c, 0, 0, 0);
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

// The same for the substeps of the 16 x 16 kernel, whose MFMAs are half as long: the others go in front, two after each
// of the first MFMAs, reads first (their results are wanted by the very next substep), then writes, then loads.
template <int R, int W, int L, int M = 0>
struct SubstepFront {
  static constexpr int kAll = R + W + L;
  static constexpr int kFrom = 2 * M < kAll ? 2 * M : kAll, kUpto = 2 * M + 2 < kAll ? 2 * M + 2 : kAll;
  static constexpr int within(int lo, int hi) {
    const int a = kFrom > lo ? kFrom : lo, b = kUpto < hi ? kUpto : hi;
    return b > a ? b - a : 0;
  }
  static AKG_DEV void emit() {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (within(0, R) > 0) __builtin_amdgcn_sched_group_barrier(0x100, within(0, R), 0);
    if constexpr (within(R, R + W) > 0) __builtin_amdgcn_sched_group_barrier(0x200, within(R, R + W), 0);
    if constexpr (within(R + W, kAll) > 0) __builtin_amdgcn_sched_group_barrier(0x020, within(R + W, kAll), 0);
    if constexpr (M < 7) SubstepFront<R, W, L, M + 1>::emit();
  }
};

// DYN: the row count of A and the number of K splits are kernel arguments (`mDyn`, `ksDyn`; the template's M and KSPLIT
// are then ignored): one code object serves every M of a description whose leading extents are open, and the host
// chooses the split for each call. Rows are bounds-checked at run time; `ws` is always a valid pointer.
template <typename Mma, long MS, long N, long KE, bool TRANSB, typename Epilogue, int KSPLIT = 1, int WM = 4, bool DYN = false>
AKG_DEV void gemm_256x256(const void *__restrict__ A, const void *__restrict__ B, Epilogue &epi,
                          unsigned *__restrict__ ws = nullptr, long mDyn = 0, int ksDyn = 1) {
  const long M = DYN ? mDyn : MS;                 // (a constant after inlining unless DYN)
  const int kSplits = DYN ? ksDyn : KSPLIT;
  constexpr bool kSplitPossible = DYN || KSPLIT > 1;
  constexpr int EB = Mma::kElemBytes;
  constexpr long K = KE * EB;    // bytes of K per row of A (and per column of B)
  constexpr long NB = N * EB;    // bytes per k-row of a row-major B
  static_assert(K % 16 == 0, "K must be a multiple of 16 bytes");
  static_assert(TRANSB || (N % 4 == 0), "N must be a multiple of 4");
  // 4 x 2 wavefronts (two per SIMD: one's MFMAs cover the other's LDS accesses and waits), 128 bytes of K per step
  // (every row of A contributes one whole cache line; LDS holds 2 x 72 KiB). Every thread stages its share of both
  // operands: uniform control flow, so a K step is one basic block.
  // (Measured and dropped: 2 x 2 wavefronts of 128 x 128 each (a third less LDS traffic, one wavefront per SIMD: 2 to 4 %
  // slower), 64-byte steps, staging split between two groups of wavefronts, 256 x 128 tiles with two workgroups per
  // CU; tiles fetched memory -> LDS directly (buffer_load_dwordx4 ... lds into rows without padding, chunks permuted
  // against bank conflicts; tried with both MFMA shapes): correct, the LDS pipe a third less busy, and 2 % slower (int8) or
  // equal (bfloat16): the cycles saved on LDS writes are spent waiting for the tile to land before the barrier; the K steps of different tiles in
  // rotated order: 8 to 25 % slower, the workgroups of an XCD share their panels in L2 only while they walk K
  // together. With the staging switched off altogether the loop runs 17 % faster, whichever way the tiles travel: what
  // is left is the price of moving 64 KB per step and CU on a power-limited part.)
  constexpr int WAVES_M = WM;            // 4 x 2 wavefronts of 64 x 128, or 2 x 4 of 128 x 64
  constexpr int WAVES_N = 8 / WM;
  constexpr int BK = 128;
  constexpr int kThreads = 512;
  constexpr int kPitch = BK + 16;                     // LDS row of a K-contiguous tile: BK data bytes + 16 pad
  constexpr int kChunksPerRow = BK / 16;              // 16-byte chunks per row of a K-contiguous operand tile
  constexpr int kRowChunks = 256 * kChunksPerRow / kThreads;  // 16-byte chunks per thread and operand (4)
  constexpr int kRowStep = kThreads / kChunksPerRow;  // rows between two chunks of one thread
  constexpr int kWaveRows = kGemmBM / WAVES_M;        // 64 (128)
  constexpr int kWaveCols = kGemmBN / WAVES_N;        // 128 (64)
  constexpr int kTM = kWaveRows / 16;                 // MFMA row tiles (16 rows) per wavefront
  constexpr int kTN = kWaveCols / 16;                 // MFMA column tiles (16 columns) per wavefront
  constexpr int kHM = kTM / 2, kHN = kTN / 2;         // tiles per half: a quarter of the wavefront tile is kHM x kHN = 8 MFMAs
  static_assert(kHM * kHN == 8, "a substep is 8 MFMAs");
  const long kTilesM = (M + kGemmBM - 1) / kGemmBM;
  constexpr long kTilesN = (N + kGemmBN - 1) / kGemmBN;
  const long kTiles = kTilesM * kTilesN;
  const long kPerXcd = (kTiles + kGemmXcds - 1) / kGemmXcds;
  constexpr long kSteps = (K + BK - 1) / BK;
  constexpr bool kFull = !DYN && (MS % kGemmBM == 0) && (N % kGemmBN == 0) && (K % BK == 0);
  // Whole tiles along N and K, and an M that is an argument or leaves a ragged last tile behind full ones: the loads need
  // no checks either. Every thread clamps the rows of A it stages to the last row once, in front of the loop (the scalar
  // offset of a buffer load takes no part in the descriptor's range check, so the descriptor alone would not keep the
  // rows of a ragged last tile inside A); rows beyond M then hold copies of row M - 1 and their accumulators are
  // dropped by the epilogue's row check. The main loop is the one of a whole shape: no compares, one basic block per K
  // step. (A single ragged tile, M < 256, keeps the checks: there the wavefronts without rows skip their MFMAs.)
  constexpr bool kClampRows = !kFull && (DYN || MS > kGemmBM) && (N % kGemmBN == 0) && (K % BK == 0);
  constexpr bool kLoadsInRange = kFull || kClampRows;
  constexpr int kTileBytes = kGemmBM * kPitch;        // one operand tile in LDS
  static_assert(kRowChunks == 4, "the staging schedule is written for four 16-byte chunks per thread and operand");
  // A row-major B goes to LDS as it lies in memory, k-rows of 256 columns. Sixteen lanes share a transposing read:
  // each hands in 8 bytes of one k-row (8-bit: 8 k-rows x 16 bytes, 16-bit: 4 k-rows x 32 bytes) and gets back, for one
  // column, 8 or 4 consecutive k. The four 16-lane groups of a wavefront read the same 16 columns, each its own
  // sixteen (8-bit) or eight (16-bit) k-rows; the rows of neighbouring groups are a multiple of 256 bytes apart whatever
  // the pitch, so odd groups find their columns in the neighbouring 16-column unit of the row (units swapped in pairs
  // when the row is written), and with rows 32 (64) bytes apart modulo the 256 bytes of the banks the two groups of a
  // half wavefront interleave without sharing a bank.
  constexpr int kRowBytesB = kGemmBN * EB;            // bytes of one k-row of the B tile
  constexpr int kPitchB = kRowBytesB + (EB == 1 ? 32 : 64);
  constexpr int kRowsB = BK / EB;                     // k-rows per step
  constexpr int kChunksPerRowB = kRowBytesB / 16;
  constexpr int kRowStepB = kThreads / kChunksPerRowB;
  constexpr int kGroupRowsB = 16 / EB;                // k-rows one 16-lane group owns per MFMA
  static_assert(TRANSB || kRowsB * kPitchB <= kTileBytes, "the row-major B tile must fit the operand's LDS space");

  __shared__ __attribute__((aligned(16))) u8 lds[2][2][kTileBytes];  // [buffer][A|B]

  // ---- workgroup -> tile
  const long kGridTiles = kPerXcd * kGemmXcds;   // workgroups per K split (a multiple of the XCD count)
  const long wgAll = static_cast<long>(blockIdx.x);
  const long ksplit = kSplitPossible ? wgAll / kGridTiles : 0;
  const long wg = kSplitPossible ? wgAll % kGridTiles : wgAll;
  const long linear = (wg % kGemmXcds) * kPerXcd + wg / kGemmXcds;
  if (linear >= kTiles) return;
  const long kStepsPer = (kSteps + kSplits - 1) / kSplits;
  static_assert(DYN || (KSPLIT - 1) * ((kSteps + KSPLIT - 1) / KSPLIT) < kSteps, "every K split needs at least one step");
  const long stepBase = ksplit * kStepsPer;
  const long mySteps = !kSplitPossible ? kSteps : ((kSteps - stepBase) < kStepsPer ? (kSteps - stepBase) : kStepsPer);
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
  const int wm = wave / WAVES_N;
  const int wn = wave % WAVES_N;

  typename Mma::acc4_v acc[kTM][kTN];
#pragma unroll
  for (int i = 0; i < kTM; ++i) {
#pragma unroll
    for (int j = 0; j < kTN; ++j) {
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0;
    }
  }

  // ---- staging registers: chunk i of tile s+1 waits here from its load (during step s-1) to its LDS write (step s).
  struct Stage {
    v4i x[kRowChunks];   // A
    v4i y[kRowChunks];   // B
  };
  Stage stage;

  const int aRow = tid / kChunksPerRow;   // + kRowStep * i
  const int aChunk = tid % kChunksPerRow;
  // Global loads are buffer loads: the per-lane offset is computed once, everything that changes from load to load
  // (row block, k-row, K step) is a scalar offset, so the loop spends no vector instructions on addresses (vector
  // instructions and MFMAs compete for issue cycles). Out-of-range lanes read zero through the descriptor's size.
  // The descriptor of A (and of a [N,K] B) starts at the tile's first row, so the 32-bit offsets only have to span a
  // tile and A may be of any size (131072 tokens x 8192 bf16 are 2 GiB); a row-major B is addressed from its start.
  static_assert(kGemmBM * K < (1L << 31) && (TRANSB ? kGemmBN * K : N * K) < (1L << 31), "operand too large for 32-bit buffer offsets");
  auto bytesLeft = [](long bytes) { return static_cast<int>(bytes < 0 ? 0 : (bytes < 0x7fffffffL ? bytes : 0x7fffffffL)); };
  const __amdgpu_buffer_rsrc_t aRsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char *>(static_cast<const char *>(A)) + m0 * K, 0, bytesLeft((M - m0) * K), 0x00020000);
  const __amdgpu_buffer_rsrc_t bRsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char *>(static_cast<const char *>(B)) + (TRANSB ? n0 * K : 0L), 0, bytesLeft(TRANSB ? (N - n0) * K : N * K), 0x00020000);
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const int aVoff = static_cast<int>(aRow * K + aChunk * 16);
  int aVoffClamped[kRowChunks];   // kClampRows: one vector offset per staged chunk, its row clamped to M - 1
#pragma unroll
  for (int i = 0; i < kRowChunks; ++i) {
    const long row = m0 + aRow + kRowStep * i;
    aVoffClamped[i] = static_cast<int>(((row < M ? row : M - 1) - m0) * K + aChunk * 16);
  }
  const int bRowT = tid / kChunksPerRowB;     // + kRowStepB * i
  const int bChunkT = tid % kChunksPerRowB;
  const int bVoff = TRANSB ? static_cast<int>(aRow * K + aChunk * 16)
                           : static_cast<int>(bRowT * NB + n0 * EB + bChunkT * 16);
  // LDS write offsets. [N,K] B: the LDS row of a column is chosen so that the 16 lanes of a fragment read find, in the
  // four column tiles 4 q .. 4 q + 3, four ADJACENT columns (row 64 q + 16 t + c holds column 64 q + 4 c + t).
  // Row-major B: the 16-column units of a k-row are swapped in pairs for the k-rows of odd 16-lane groups.
  // K-contiguous tiles: a 128-bit LDS read is served sixteen lanes at a time, and not sixteen neighbours: the lane
  // quads 0, 3, 5, 6 of a half wavefront go together, then 1, 2, 4, 7 (measured). The 16 rows x 2 quarters of K such a
  // group reads fall into 16 different bank groups when rows 4 .. 11 of every 16 keep their 16-byte chunks swapped in pairs.
  auto pairSwap = [](int row) { return ((row >> 2) ^ (row >> 3)) & 1; };
  const int aStoreOff = aRow * kPitch + (aChunk ^ pairSwap(aRow)) * 16;
  int bStoreOff[kRowChunks];
#pragma unroll
  for (int i = 0; i < kRowChunks; ++i) {
    if constexpr (TRANSB) {
      const int col = aRow + kRowStep * i;
      const int r = (col & ~63) + (col & 3) * 16 + ((col >> 2) & 15);
      bStoreOff[i] = r * kPitch + (aChunk ^ pairSwap(r)) * 16;
    } else {
      const int krow = bRowT + kRowStepB * i;
      const int odd = (krow / kGroupRowsB) & 1;
      bStoreOff[i] = krow * kPitchB + (bChunkT ^ (odd * EB)) * 16;
    }
  }

  auto loadChunk = [&](long step, int i) {
    const long k0 = (stepBase + step) * BK;
    if (kLoadsInRange || (m0 + aRow + kRowStep * i < M && k0 + aChunk * 16 < K)) {
      const u32x4 v = kClampRows ? __builtin_amdgcn_raw_buffer_load_b128(aRsrc, aVoffClamped[i], static_cast<int>(k0), 0)
                                 : __builtin_amdgcn_raw_buffer_load_b128(aRsrc, aVoff, static_cast<int>((kRowStep * i) * K + k0), 0);
      stage.x[i] = v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
    } else {
      stage.x[i] = v4i{0, 0, 0, 0};
    }
    if constexpr (TRANSB) {
      if (kLoadsInRange || (n0 + aRow + kRowStep * i < N && k0 + aChunk * 16 < K)) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(bRsrc, bVoff, static_cast<int>((kRowStep * i) * K + k0), 0);
        stage.y[i] = v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
      } else {
        stage.y[i] = v4i{0, 0, 0, 0};
      }
    } else {
      const long krow = k0 / EB + bRowT + kRowStepB * i;
      if (kLoadsInRange || (krow < KE && n0 * EB + bChunkT * 16 < NB)) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(bRsrc, bVoff, static_cast<int>((k0 / EB + kRowStepB * i) * NB), 0);
        stage.y[i] = v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
      } else {
        stage.y[i] = v4i{0, 0, 0, 0};
      }
    }
  };
  auto storeChunk = [&](int buf, int i) {
    *reinterpret_cast<v4i *>(lds[buf][0] + aStoreOff + (kRowStep * i) * kPitch) = stage.x[i];
    *reinterpret_cast<v4i *>(lds[buf][1] + bStoreOff[i]) = stage.y[i];
  };

  // ---- fragments. Every MFMA takes 64 bytes of K per row: lane (c = lane % 16, g = lane / 16) holds the 16 bytes
  // [16 g, +16) of row c of its A tile and of column c of its B tile (the same bytes of K in both, which is all the
  // instruction needs), and receives rows 4 g .. 4 g + 3 of column c of the 16 x 16 result.
  const int fragC = lane & 15, fragG = lane >> 4;
  const int aFragOff = (wm * kWaveRows + fragC) * kPitch + (fragG ^ pairSwap(fragC)) * 16;
  const int bFragOff = (wn * kWaveCols + fragC) * kPitch + (fragG ^ pairSwap(fragC)) * 16;
  // Row-major B: group g reads k-rows kGroupRowsB * g .. of the 64 bytes of K; inside the group, 8-bit: lane s hands in
  // k-row s >> 1, column octet s & 1; 16-bit: k-row s >> 2, column quad s & 3. Even and odd column tiles have their own
  // base because of the swap of units in the rows of odd groups.
  const int trRow = fragG * kGroupRowsB + (EB == 1 ? (fragC >> 1) : (fragC >> 2));
  const int trCol = EB == 1 ? (fragC & 1) * 8 : (fragC & 3) * 8;
  const int trSwap = (fragG & 1) * 16 * EB;
  const int bFragOffEven = trRow * kPitchB + wn * kWaveCols * EB + trSwap + trCol;
  const int bFragOffOdd = trRow * kPitchB + wn * kWaveCols * EB - trSwap + trCol;

  // Wavefronts whose rows all lie below the last row of A (a skinny A: M = 16 leaves three of the four wavefront rows
  // without a single real row) take part in the staging and the barriers but skip fragment reads and MFMAs.
  constexpr bool kAllRowsReal = kClampRows || (!DYN && MS % kGemmBM == 0);   // (clamped rows: every wavefront computes)
  const bool waveHasRows = kAllRowsReal || (m0 + wm * kWaveRows < M);
  // A fragments of row half rh (2 tiles of 16 rows), K half kh (64 bytes)
  auto readA = [&](int buf, int kh, int rh, v4i (&af)[kHM]) {
    if (!kAllRowsReal && !waveHasRows) return;
    const u8 *la = lds[buf][0] + aFragOff + kh * 64 + rh * (kHM * 16) * kPitch;
#pragma unroll
    for (int i = 0; i < kHM; ++i) af[i] = *reinterpret_cast<const v4i *>(la + i * 16 * kPitch);
  };
  // B fragments of column half ch (4 tiles of 16 columns), K half kh
  auto readB = [&](int buf, int kh, int ch, v4i (&bf)[kHN]) {
    if (!kAllRowsReal && !waveHasRows) return;
    if constexpr (TRANSB) {
      const u8 *lb = lds[buf][1] + bFragOff + kh * 64 + ch * (kHN * 16) * kPitch;
#pragma unroll
      for (int j = 0; j < kHN; ++j) bf[j] = *reinterpret_cast<const v4i *>(lb + j * 16 * kPitch);
    } else {
      typedef int v2i __attribute__((ext_vector_type(2)));
      typedef short v4s __attribute__((ext_vector_type(4)));
      const u8 *lt = lds[buf][1] + kh * (64 / EB) * kPitchB + ch * (kHN * 16) * EB;
#pragma unroll
      for (int j = 0; j < kHN; ++j) {
        const u8 *p0 = lt + ((j & 1) ? bFragOffOdd : bFragOffEven) + j * 16 * EB;
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
    }
  };
  // bFresh: the B fragments are the ones that have just been read: walk them one after the other (both row tiles on
  // each) so that the last to arrive is wanted last; else the A fragments one after the other.
  auto mfma8 = [&](int rh, int ch, const v4i (&af)[kHM], const v4i (&bf)[kHN], auto bFresh) {
    if (!kAllRowsReal && !waveHasRows) return;
    if constexpr (decltype(bFresh)::value) {
#pragma unroll
      for (int j = 0; j < kHN; ++j) {
#pragma unroll
        for (int i = 0; i < kHM; ++i) {
          acc[rh * kHM + i][ch * kHN + j] = Mma::mma16(af[i], bf[j], acc[rh * kHM + i][ch * kHN + j]);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < kHM; ++i) {
#pragma unroll
        for (int j = 0; j < kHN; ++j) {
          acc[rh * kHM + i][ch * kHN + j] = Mma::mma16(af[i], bf[j], acc[rh * kHM + i][ch * kHN + j]);
        }
      }
    }
  };

  // ---- main loop. A step is 8 substeps of 8 MFMAs: the wavefront's 64 x 128 tile in quarters (row half rh, column half
  // ch), for each of the two 64-byte halves of K, walked so that consecutive substeps share one operand half and only the
  // other is read anew: (0,0) (0,1) (1,1) (1,0) | (0,1) (0,0) (1,0) (1,1). Two register sets per operand: while one
  // half feeds the MFMAs, the half needed next arrives in the other. Invariant at the top of step s: LDS buffer s & 1
  // holds tile s, the staging registers hold tile s + 1 (possibly still in flight), fa[0] and fb[0] hold the fragments
  // (rh 0, ch 0) of the first K half of tile s. The eight chunks of tile s + 1 go to the other LDS buffer in the
  // substeps that read only A fragments (1, 2 and 5: an LDS write of 1 KiB occupies the LDS twice as long as a read, and
  // eight wavefronts in step writing at once cost more cycles than the same writes one per MFMA), and their registers
  // are refilled from tile s + 2 in substeps 3, 4 and 6; all fragment reads of tile s are issued by substep 5, the
  // barrier follows it, and substeps 6 and 7 fetch the first fragments of tile s + 1. The order of MFMAs, LDS accesses
  // and loads inside a substep is fixed instruction by instruction with scheduling groups instead of left to the
  // scheduler, which clusters them: fragment reads two after each of the first MFMAs (their results are wanted by the
  // next substep), writes one per MFMA.
  v4i fa[2][kHM], fb[2][kHN];
  auto stepSpread = [&](long step, auto storeTag, auto loadTag) {
    constexpr bool kStore = decltype(storeTag)::value;
    constexpr bool kLoad = decltype(loadTag)::value;
    constexpr int kReadsA = kHM, kReadsB = TRANSB ? kHN : 2 * kHN;
    const int buf = static_cast<int>(step & 1);
    auto storeX = [&](int i) { *reinterpret_cast<v4i *>(lds[buf ^ 1][0] + aStoreOff + (kRowStep * i) * kPitch) = stage.x[i]; };
    auto storeY = [&](int i) { *reinterpret_cast<v4i *>(lds[buf ^ 1][1] + bStoreOff[i]) = stage.y[i]; };
    // substep 0: (0,0) of K half 0; B (ch 1) arrives
    readB(buf, 0, 1, fb[1]);
    mfma8(0, 0, fa[0], fb[0], BoolTag<true>());
    SubstepFront<kReadsB, 0, 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    // substep 1: (0,1); A (rh 1) arrives; three chunks of tile s+1 to LDS
    readA(buf, 0, 1, fa[1]);
    if constexpr (kStore) {
      storeX(0);
      storeY(0);
      storeX(1);
    }
    mfma8(0, 1, fa[0], fb[1], BoolTag<true>());
    SubstepOrder<kReadsA, kStore ? 3 : 0, 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    // substep 2: (1,1); A (rh 0) of K half 1 arrives; three more chunks to LDS
    readA(buf, 1, 0, fa[0]);
    if constexpr (kStore) {
      storeY(1);
      storeX(2);
      storeY(2);
    }
    mfma8(1, 1, fa[1], fb[1], BoolTag<false>());
    SubstepOrder<kReadsA, kStore ? 3 : 0, 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    // substep 3: (1,0); B (ch 1) of K half 1 arrives; chunks 0 and 1 of tile s+2 on their way
    readB(buf, 1, 1, fb[1]);
    if constexpr (kLoad) {
      loadChunk(step + 2, 0);
      loadChunk(step + 2, 1);
    }
    mfma8(1, 0, fa[1], fb[0], BoolTag<false>());
    SubstepFront<kReadsB, 0, kLoad ? 4 : 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    // substep 4: K half 1, (0,1); B (ch 0) arrives; chunk 2 on its way
    readB(buf, 1, 0, fb[0]);
    if constexpr (kLoad) loadChunk(step + 2, 2);
    mfma8(0, 1, fa[0], fb[1], BoolTag<true>());
    SubstepFront<kReadsB, 0, kLoad ? 2 : 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    // substep 5: (0,0); A (rh 1) arrives: the last read of tile s; the last two chunks to LDS
    readA(buf, 1, 1, fa[1]);
    if constexpr (kStore) {
      storeX(3);
      storeY(3);
    }
    mfma8(0, 0, fa[0], fb[0], BoolTag<true>());
    SubstepOrder<kReadsA, kStore ? 2 : 0, 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();   // everybody has read tile s completely and has written tile s+1
    // substep 6: (1,0); first A fragments of tile s+1; chunk 3 of tile s+2 on its way
    if constexpr (kStore) readA(buf ^ 1, 0, 0, fa[0]);
    if constexpr (kLoad) loadChunk(step + 2, 3);
    mfma8(1, 0, fa[1], fb[0], BoolTag<false>());
    SubstepFront<kStore ? kReadsA : 0, 0, kLoad ? 2 : 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
    // substep 7: (1,1); first B fragments of tile s+1
    if constexpr (kStore) readB(buf ^ 1, 0, 0, fb[0]);
    mfma8(1, 1, fa[1], fb[1], BoolTag<false>());
    SubstepFront<kStore ? kReadsB : 0, 0, 0>::emit();
    __builtin_amdgcn_sched_barrier(0);
  };
#pragma unroll
  for (int i = 0; i < kRowChunks; ++i) loadChunk(0, i);
#pragma unroll
  for (int i = 0; i < kRowChunks; ++i) storeChunk(0, i);
  if (mySteps > 1) {
#pragma unroll
    for (int i = 0; i < kRowChunks; ++i) loadChunk(1, i);
  }
  __syncthreads();
  readA(0, 0, 0, fa[0]);
  readB(0, 0, 0, fb[0]);
  long step = 0;
  for (; step + 2 < mySteps; ++step) stepSpread(step, BoolTag<true>(), BoolTag<true>());
  if (step + 1 < mySteps) {
    stepSpread(step, BoolTag<true>(), BoolTag<false>());
    ++step;
  }
  stepSpread(step, BoolTag<false>(), BoolTag<false>());

  // ---- epilogue: a lane owns, per group of four column tiles (q = 0, 1), four ADJACENT columns of 16 rows.
  // [N,K] B: the LDS row order gave tile 4 q + t of lane c column 64 q + 4 c + t. Row-major B: tile j holds the columns
  // 16 j .. 16 j + 15 lane by lane, so the four lanes of a quad hold four neighbouring columns of each of four tiles:
  // a 4 x 4 transpose between the lanes of the quad and the tiles (two exchanges with quad permutations) gives lane s
  // of the quad the four columns of tile 4 q + s.
  if constexpr (!TRANSB) {
    const bool odd = (lane & 1) != 0, upper = (lane & 2) != 0;
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int q = 0; q < kTN / 4; ++q) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          typename Mma::acc_t a0 = acc[i][4 * q][v], a1 = acc[i][4 * q + 1][v], a2 = acc[i][4 * q + 2][v], a3 = acc[i][4 * q + 3][v];
          const typename Mma::acc_t r01 = lane_partner<1>(odd ? a0 : a1), r23 = lane_partner<1>(odd ? a2 : a3);
          if (odd) { a0 = r01; a2 = r23; } else { a1 = r01; a3 = r23; }
          const typename Mma::acc_t r02 = lane_partner<2>(upper ? a0 : a2), r13 = lane_partner<2>(upper ? a1 : a3);
          if (upper) { a0 = r02; a1 = r13; } else { a2 = r02; a3 = r13; }
          acc[i][4 * q][v] = a0;
          acc[i][4 * q + 1][v] = a1;
          acc[i][4 * q + 2][v] = a2;
          acc[i][4 * q + 3][v] = a3;
        }
      }
    }
  }
  // first of the lane's four columns in column group q, and the row of accumulator v of row tile i inside the tile
  const long colBase = n0 + wn * kWaveCols + (TRANSB ? 4 * fragC : 16 * (fragC & 3) + (fragC & ~3));
  auto rowInTileOf = [&](int i, int v) { return static_cast<long>(wm * kWaveRows + i * 16 + fragG * 4 + v); };
  if (kSplitPossible && kSplits > 1) {
    const long kPartRows = M < kGemmBM ? M : kGemmBM;            // rows of a tile that can hold results
    const long kCounterBytes = (kGridTiles * 4 + 255) / 256 * 256;
    const long kPartBytes = kPartRows * kGemmBN * static_cast<long>(sizeof(typename Mma::acc_t));
    const long kWsBytes = kCounterBytes + kTiles * kSplits * kPartBytes;   // (below 2 GiB: checked by the host)
    const Buffer wsBuf = make_buffer(ws, kWsBytes);
    const u32 tileBase = static_cast<u32>(kCounterBytes + linear * kSplits * kPartBytes);
    auto partOffset = [&](int i, int q, int v) {
      return static_cast<long>((rowInTileOf(i, v) * kGemmBN + (colBase + 64 * q - n0)) * static_cast<long>(sizeof(typename Mma::acc_t)));
    };
    auto rowOk = [&](int i, int v) { return rowInTileOf(i, v) < kPartRows && m0 + rowInTileOf(i, v) < M; };
#pragma unroll
    for (int q = 0; q < kTN / 4; ++q) {
      if (!(kFull || colBase + 64 * q < N)) continue;
#pragma unroll
      for (int i = 0; i < kTM; ++i) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          // (a row beyond M stores to beyond the workspace, which drops it)
          const typename Mma::acc_t a4[4] = {acc[i][4 * q][v], acc[i][4 * q + 1][v], acc[i][4 * q + 2][v], acc[i][4 * q + 3][v]};
          ws_store_chunk<4>(wsBuf, rowOk(i, v) ? tileBase + static_cast<u32>(ksplit * kPartBytes + partOffset(i, q, v)) : kBeyondEveryBuffer, a4);
        }
      }
    }
    __shared__ unsigned akg_gemm_flag;
    if (!last_workgroup(ws, linear, kSplits, tid, &akg_gemm_flag)) return;
    if constexpr (!DYN) {
      // The number of splits is a constant: sum and epilogue per group of four accumulators, the loads of all splits of
      // the group in flight together (the compiler unrolls the splits and overlaps the groups).
#pragma unroll
      for (int q = 0; q < kTN / 4; ++q) {
        const long col4 = colBase + 64 * q;
        if (!(kFull || col4 < N)) continue;
        epi.prepare(col4);
#pragma unroll
        for (int i = 0; i < kTM; ++i) {
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            if (!rowOk(i, v)) continue;
            typename Mma::acc_t sum[4] = {0, 0, 0, 0};
            for (int p = 0; p < kSplits; ++p) {
              typename Mma::acc_t part[4];
              ws_load_chunk<4>(wsBuf, tileBase + static_cast<u32>(p * kPartBytes + partOffset(i, q, v)), part);
#pragma unroll
              for (int c = 0; c < 4; ++c) sum[c] += part[c];
            }
            epi.apply(sum, m0 + rowInTileOf(i, v), col4);
          }
        }
      }
      return;
    } else {
      // The last workgroup of the tile: the sums of the partials, in split order, into the accumulators (this workgroup's
      // own partial is among them). One round per split with every load of the round issued before the first addition
      // (the number of splits may be an argument: a loop over the splits inside the loops over the accumulators would
      // wait for every load by itself); a row beyond M loads from beyond the workspace, which reads zero.
#pragma unroll
      for (int i = 0; i < kTM; ++i) {
#pragma unroll
        for (int j = 0; j < kTN; ++j) {
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[i][j][v] = 0;
        }
      }
      for (int p = 0; p < kSplits; ++p) {
        const u32 splitBase = tileBase + static_cast<u32>(p * kPartBytes);
#pragma unroll
        for (int q = 0; q < kTN / 4; ++q) {
          if (!(kFull || colBase + 64 * q < N)) continue;
#pragma unroll
          for (int i = 0; i < kTM; ++i) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              typename Mma::acc_t part[4];
              ws_load_chunk<4>(wsBuf, rowOk(i, v) ? splitBase + static_cast<u32>(partOffset(i, q, v)) : kBeyondEveryBuffer, part);
#pragma unroll
              for (int c = 0; c < 4; ++c) acc[i][4 * q + c][v] += part[c];
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int q = 0; q < kTN / 4; ++q) {
    const long col4 = colBase + 64 * q;
    if (!(kFull || col4 < N)) continue;
    epi.prepare(col4);
#pragma unroll
    for (int i = 0; i < kTM; ++i) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const long row = m0 + rowInTileOf(i, v);
        if (kFull || row < M) {
          const typename Mma::acc_t a4[4] = {acc[i][4 * q][v], acc[i][4 * q + 1][v], acc[i][4 * q + 2][v], acc[i][4 * q + 3][v]};
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
// DYN: MS is the most rows the code object takes (16, 32 or 64), the actual row count and the number of K splits are
// kernel arguments (`mDyn` <= MS, `ksDyn`); `ws` is always a valid pointer.
template <typename Mma, long MS, long N, long KE, bool TRANSB, typename Epilogue, int KSPLIT, int WAVES = 4, int UNROLL = 2, bool NT = false, bool DYN = false>
AKG_DEV void gemm_skinny(const void *__restrict__ Av, const void *__restrict__ Bv, Epilogue &epi,
                         unsigned *__restrict__ ws, long group0, long mDyn = 0, int ksDyn = 1) {
  const long M = DYN ? mDyn : MS;
  const int kSplits = DYN ? ksDyn : KSPLIT;
  constexpr bool kSplitPossible = DYN || KSPLIT > 1;
  constexpr int EB = Mma::kElemBytes;
  constexpr long K = KE * EB;   // bytes of K per row of A
  constexpr long NB = N * EB;   // bytes per k-row of a row-major B
  static_assert(MS >= 1 && MS <= 128, "at most 128 rows");
  constexpr int kRowTiles = static_cast<int>((MS + 31) / 32);   // MFMA tiles of 32 rows
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
  const long t0 = kSteps * ksplit / kSplits, t1 = kSteps * (ksplit + 1) / kSplits;
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
  // (For a [N,K] weight, whose columns are contiguous along K, giving a wavefront a run of adjacent steps instead of
  // every fourth changes nothing: 36.9 us either way on bf16 16 x 8192 x 8192; the L1 merges the pieces of a line.)
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
  constexpr int kHalfRows = MS < 16 ? static_cast<int>(MS) : 16;
  __shared__ acc_t akg_skinny_sum[kWaves][kHalfRows][128];
  const int c4 = tid & 31, r0 = (tid >> 5) & 7;
  const long col = strip * 128 + 4 * c4;
  const bool colOk = col < N && tid < 256;   // (of 8 wavefronts the first four finish the sums)
  constexpr int kRowsPerThread = (MS + 7) / 8;
  acc_t sum[kRowsPerThread][4];
#pragma unroll
  for (int h = 0; h < (MS + 15) / 16; ++h) {
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
  if (kSplitPossible && kSplits > 1) {
    const long kPartBytes = M * 128 * static_cast<long>(sizeof(acc_t));
    const long group = group0 + strip;
    // layout: [groups x 4 bytes of counters, rounded up to 256][group][split][M][128]
    const long groups = static_cast<long>(gridDim.y) * kStrips;
    const long counterBytes = (groups * 4 + 255) / 256 * 256;
    const Buffer wsBuf = make_buffer(ws, counterBytes + groups * kSplits * kPartBytes);
    const u32 base = static_cast<u32>(counterBytes + group * kSplits * kPartBytes);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
      const int row = r0 + 8 * i;
      if (row < M && colOk) {
        ws_store_chunk<4>(wsBuf, base + static_cast<u32>(ksplit * kPartBytes + (row * 128 + 4 * c4) * static_cast<long>(sizeof(acc_t))), sum[i]);
      }
    }
    __shared__ unsigned akg_skinny_flag;
    if (!last_workgroup(ws, group, kSplits, tid, &akg_skinny_flag)) return;
    if (!colOk) return;
    epi.prepare(col);
    // Rounds of two or four splits, the loads of all rows of a round issued together (a row beyond M or a split beyond
    // the last loads from beyond the workspace, which reads zero); sums in split order, whether the number of splits
    // is an argument or a constant.
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
#pragma unroll
      for (int c = 0; c < 4; ++c) sum[i][c] = 0;
    }
    constexpr int kRound = kRowsPerThread <= 4 ? 4 : 2;   // splits per round: at most 16 loads of 16 bytes in flight
    for (int p0 = 0; p0 < kSplits; p0 += kRound) {
      acc_t part[kRound][kRowsPerThread][4];
#pragma unroll
      for (int u = 0; u < kRound; ++u) {
#pragma unroll
        for (int i = 0; i < kRowsPerThread; ++i) {
          const int row = r0 + 8 * i;
          const bool there = row < M && p0 + u < kSplits;
          ws_load_chunk<4>(wsBuf, there ? base + static_cast<u32>((p0 + u) * kPartBytes + (row * 128 + 4 * c4) * static_cast<long>(sizeof(acc_t))) : kBeyondEveryBuffer, part[u][i]);
        }
      }
#pragma unroll
      for (int u = 0; u < kRound; ++u) {
#pragma unroll
        for (int i = 0; i < kRowsPerThread; ++i) {
#pragma unroll
          for (int c = 0; c < 4; ++c) sum[i][c] += part[u][i][c];
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
      const int row = r0 + 8 * i;
      if (row < M) epi.apply(sum[i], row, col);
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
