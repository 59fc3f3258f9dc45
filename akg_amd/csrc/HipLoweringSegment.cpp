/**
 * UnsortedSegmentSum: out[ids[i], ...] += data[i, ...] for the index positions i in increasing order.
 *
 * The reference lowers it to a serial loop over the (collapsed) index positions that adds one data slice to the
 * accumulator slice its id names (MindSporeToLinalg.cpp:596-745). A GPU scatter with float atomics would add in arrival
 * order; this kernel keeps the reference's order, bit for bit, without atomics and without a zero-filled output.
 *
 * A workgroup owns a range of segments (and a tile of the slice) whose accumulators live in LDS. Every wavefront of it
 * scans ALL index positions, 64 lanes x 16 bytes of ids per load and several loads in flight, and ballots the lanes
 * whose ids fall into the range; the few matches are handled in ascending position order. For slices of up to four
 * elements the matching lane adds the whole slice itself (its data loads are issued before the serial part); for wider
 * slices thread t adds columns t, t + block, ... and only ever touches its own columns, so the wavefronts of a workgroup
 * repeat the (cheap) scan instead of sharing it and no barrier is needed. Either way the order per output element is
 * the serial one.
 * Ids outside [0, segments) match nobody and are dropped. The id array is read once per workgroup (from L2 after the
 * first), the data once overall.
 *
 * That scan costs (workgroups x positions) id reads. Inputs with many positions are grouped by segment first instead
 * (lowerSegmentSorted below): same result, bit for bit.
 */
#include <algorithm>
#include <sstream>

#include "HipLowering.h"

namespace akg {

namespace {

// The shapes both schedules need.
struct SegmentShapes {
  const OpNode *op = nullptr;
  const TensorValue *data = nullptr, *ids = nullptr, *out = nullptr;
  int64_t positions = 0, segments = 0, slice = 0;
};

SegmentShapes checkSegmentSum(const OpGraph &g) {
  if (g.ops.size() != 1 || g.ops[0].kind != OpKind::SegmentSum || g.outputs.size() != 1 ||
      g.outputs[0] != g.ops[0].outputs[0]) {
    throw LoweringError("UnsortedSegmentSum can only be lowered as a kernel of its own (no fused neighbours yet)");
  }
  SegmentShapes sh;
  sh.op = &g.ops[0];
  const OpNode &op = *sh.op;
  sh.data = &g.tensor(op.inputs[0]);
  sh.ids = &g.tensor(op.inputs[1]);
  sh.out = &g.tensor(op.outputs[0]);
  if (sh.data->inputIndex < 0 || sh.ids->inputIndex < 0) throw LoweringError("op " + op.name + ": operands must be kernel inputs");
  if (sh.data->dtype != sh.out->dtype) throw LoweringError("op " + op.name + ": data and result element types differ");
  if (sh.out->dtype == DType::Bool) throw LoweringError("op " + op.name + ": bool data is not supported");
  sh.positions = sh.ids->numel();
  sh.segments = op.padValue;
  sh.slice = sh.positions > 0 ? sh.data->numel() / sh.positions : 0;
  if (sh.positions <= 0 || sh.slice <= 0 || sh.out->numel() != sh.segments * sh.slice) {
    throw LoweringError("op " + op.name + ": inconsistent shapes");
  }
  if (sh.positions >= (1LL << 31) || sh.out->numel() >= (1LL << 31) || sh.data->numel() >= (1LL << 40)) {
    throw LoweringError("op " + op.name + ": too large");
  }
  return sh;
}

// The three counting launches both grouped schedules share. The generated source must define POSITIONS, KEYS (counters
// per run), RUNS, RUN, W_HIST, W_TOTAL, W_START, as_segment() and key_of(segment):
//   <op>_count    workgroup b counts the keys of its run of positions (LDS counters) -> hist[b][key]
//   <op>_offsets  per key, the exclusive prefix of hist over b (in place) and the key's total
//   <op>_starts   exclusive prefix of the totals: where each key's list starts (and, at [KEYS], where the last one ends)
// Workgroups of the <op>_offsets launch for `keys` counters per run (see emitCountingLaunches).
int64_t offsetsGrid(int64_t keys) {
  const int64_t perWg = keys >= 4096 ? 16 : 4, groups = (keys + perWg - 1) / perWg;
  return (groups + 7) / 8 * 8;
}

void emitCountingLaunches(std::ostringstream &s, const std::string &name, const std::string &paramList, const std::string &idTag,
                          const std::string &idsName, int64_t runs, int64_t keys) {
  const int perStart = static_cast<int>((keys + 1023) / 1024);
  // ---- count ----
  s << "extern \"C\" __global__ __launch_bounds__(256) void " << name << "_count(" << paramList << ") {\n";
  s << "  __shared__ unsigned akg_cnt[KEYS];\n";
  s << "  const int tid = static_cast<int>(threadIdx.x), run = static_cast<int>(blockIdx.x);\n";
  s << "  for (int k = tid; k < KEYS; k += 256) akg_cnt[k] = 0u;\n";
  s << "  __syncthreads();\n";
  s << "  const int p0 = run * RUN, p1 = p0 + RUN < POSITIONS ? p0 + RUN : POSITIONS;\n";
  s << "#pragma unroll 4\n";
  s << "  for (int p = p0 + tid; p < p1; p += 256) {\n";
  s << "    const int id = as_segment(" << idTag << "::load(" << idsName << "[p]));\n";
  s << "    if (id >= 0) atomicAdd(&akg_cnt[key_of(id)], 1u);\n";
  s << "  }\n";
  s << "  __syncthreads();\n";
  s << "  for (int k = tid; k < KEYS; k += 256) akg_ws[W_HIST + static_cast<long>(run) * KEYS + k] = akg_cnt[k];\n";
  s << "}\n\n";

  // ---- offsets ----
  // A workgroup takes a few keys and splits the runs among its threads: KPW keys x (256 / KPW) slabs of runs. Few keys
  // (the bucketed schedule) take 4 a workgroup, so that the launch still fills the chip.
  const int keysPerWg = keys >= 4096 ? 16 : 4, slabs = 256 / keysPerWg;
  const int64_t runsPer = (runs + slabs - 1) / slabs;
  s << "extern \"C\" __global__ __launch_bounds__(256) void " << name << "_offsets(" << paramList << ") {\n";
  s << "  constexpr int PER = " << runsPer << ", KPW = " << keysPerWg << ", SLABS = " << slabs << ";   // runs per thread, keys per workgroup, threads a key\n";
  s << "  __shared__ unsigned akg_part[SLABS][KPW + 1];\n";
  s << "  const int tid = static_cast<int>(threadIdx.x), sl = tid % KPW, bl = tid / KPW;\n";
  s << "  // (workgroups of one XCD - launch order: workgroup b runs on XCD b mod 8 - take neighbouring keys, which share lines)\n";
  s << "  constexpr int GROUPS = (KEYS + KPW - 1) / KPW, PER_XCD = (GROUPS + 7) / 8;\n";
  s << "  const int group = static_cast<int>(blockIdx.x & 7u) * PER_XCD + static_cast<int>(blockIdx.x >> 3);\n";
  s << "  if (group >= GROUPS) return;   // (uniform)\n";
  s << "  const int seg = group * KPW + sl;\n";
  s << "  const int b0 = bl * PER < RUNS ? bl * PER : RUNS, b1 = b0 + PER < RUNS ? b0 + PER : RUNS;\n";
  s << "  unsigned *__restrict__ col = akg_ws + W_HIST + seg;\n";
  s << "  unsigned sum = 0u;\n";
  s << "  if (seg < KEYS) {\n";
  s << "#pragma unroll 8\n";
  s << "    for (int b = b0; b < b1; ++b) sum += col[static_cast<long>(b) * KEYS];\n";
  s << "  }\n";
  s << "  akg_part[bl][sl] = sum;\n";
  s << "  __syncthreads();\n";
  s << "  unsigned before = 0u;\n";
  s << "  for (int j = 0; j < bl; ++j) before += akg_part[j][sl];\n";
  s << "  if (seg >= KEYS) return;\n";
  s << "  if (bl == SLABS - 1) akg_ws[W_TOTAL + seg] = before + sum;\n";
  s << "  for (int b = b0; b < b1; b += 8) {\n";
  s << "    unsigned v[8];\n";
  s << "#pragma unroll\n";
  s << "    for (int j = 0; j < 8; ++j) v[j] = b + j < b1 ? col[static_cast<long>(b + j) * KEYS] : 0u;\n";
  s << "#pragma unroll\n";
  s << "    for (int j = 0; j < 8; ++j) {\n";
  s << "      if (b + j < b1) col[static_cast<long>(b + j) * KEYS] = before;\n";
  s << "      before += v[j];\n";
  s << "    }\n  }\n";
  s << "}\n\n";

  // ---- starts ----
  s << "extern \"C\" __global__ __launch_bounds__(1024) void " << name << "_starts(" << paramList << ") {\n";
  s << "  constexpr int PER = " << perStart << ";\n";
  s << "  __shared__ unsigned akg_scan[1024];\n";
  s << "  const int tid = static_cast<int>(threadIdx.x);\n";
  s << "  unsigned v[PER], sum = 0u;\n";
  s << "#pragma unroll\n";
  s << "  for (int j = 0; j < PER; ++j) {\n";
  s << "    const int seg = tid * PER + j;\n";
  s << "    v[j] = seg < KEYS ? akg_ws[W_TOTAL + seg] : 0u;\n";
  s << "    sum += v[j];\n";
  s << "  }\n";
  s << "  akg_scan[tid] = sum;\n";
  s << "  __syncthreads();\n";
  s << "  for (int d = 1; d < 1024; d <<= 1) {\n";
  s << "    const unsigned add = tid >= d ? akg_scan[tid - d] : 0u;\n";
  s << "    __syncthreads();\n";
  s << "    akg_scan[tid] += add;\n";
  s << "    __syncthreads();\n";
  s << "  }\n";
  s << "  unsigned run = akg_scan[tid] - sum;\n";
  s << "#pragma unroll\n";
  s << "  for (int j = 0; j < PER; ++j) {\n";
  s << "    const int seg = tid * PER + j;\n";
  s << "    if (seg < KEYS) akg_ws[W_START + seg] = run;\n";
  s << "    run += v[j];\n";
  s << "  }\n";
  s << "  if (tid == 1023) akg_ws[W_START + KEYS] = akg_scan[1023];\n";
  s << "}\n\n";

}

/**
 * Many positions: the scan above costs (workgroups x positions) id reads, which dominates from a few hundred thousand
 * positions on. Here the positions are first grouped by segment, in position order within a segment (a counting sort
 * whose passes only use integer counters, so nothing depends on arrival order), and then every output element is one
 * serial chain of additions over its segment's list, one lane per element, all elements in parallel:
 *
 *   <op>_count    workgroup b counts the ids of its run of positions per segment (LDS counters) -> hist[b][segment]
 *   <op>_offsets  per segment, the exclusive prefix of hist over b (in place) and the segment's total
 *   <op>_starts   exclusive prefix of the totals: where each segment's list starts
 *   <op>_place    one wavefront per run: lanes with equal ids rank themselves with ballots over the id's bits, so the
 *                 positions of a segment land in increasing order; position -> sorted[start + prefix + rank]
 *   <op>_kernel   lane c adds data[sorted[k], column] for k over its segment's list, in order, and stores the sum
 *
 * The five launches take the same arguments and share one workspace (histogram, totals, starts, sorted positions).
 */
LoweredKernel lowerSegmentSorted(const OpGraph &g, const LoweringOptions &options, const SegmentShapes &sh) {
  using lowering::computeTypeName;
  using lowering::dtypeTag;
  const TensorValue &data = *sh.data, &ids = *sh.ids, &out = *sh.out;
  const int64_t positions = sh.positions, segments = sh.segments, slice = sh.slice;
  const std::string ct = computeTypeName(out.dtype), tag = dtypeTag(out.dtype), idTag = dtypeTag(ids.dtype);
  const bool narrow = out.dtype == DType::F16 || out.dtype == DType::BF16 || out.dtype == DType::I8 || out.dtype == DType::I16;
  const std::string rndOpen = narrow ? tag + "::rnd(" : std::string("(");
  // Runs of positions: a multiple of 64 positions, at least 1024, at most 2048 runs. One wavefront places a run, and
  // the placement is bound by latency with few wavefronts and by the scattered partial-line writes with many (24.5
  // million positions of 12-byte rows: 512 runs 1.56 ms, 1024 1.06 ms, 2048 0.82 ms, 4096 1.03 ms for all launches).
  int64_t runs = options.split > 0 ? options.split : std::min<int64_t>(2048, std::max<int64_t>(1, positions / 1024));
  int64_t runLength = (positions + runs - 1) / runs;
  runLength = (runLength + 63) / 64 * 64;
  runs = (positions + runLength - 1) / runLength;
  int idBits = 1;
  while ((1LL << idBits) < segments) ++idBits;
  const int64_t chains = segments * slice;
  const int unroll = options.chunks > 0 ? options.chunks : 8;
  // Short slices (one 16-byte load per data row) are moved into segment order themselves; of wider ones only the
  // positions are.
  const int elemBytes = static_cast<int>(dtypeSize(out.dtype));
  const bool staged = slice * elemBytes <= 16;
  // workspace, in 4-byte words
  const int64_t wHist = 0, wTotal = wHist + runs * segments, wStart = wTotal + segments,
                wSorted = (wStart + segments + 1 + 3) / 4 * 4;   // 16-byte aligned
  const int64_t words = wSorted + (staged ? (positions * slice * elemBytes + 3) / 4 : positions);
  std::ostringstream s;
  s << "// Generated by the akg HIP lowering for gfx950. Op description: " << g.name << "\n";
  s << "// family: segment_sum (positions grouped by segment first), fusion class: " << operatorTemplateName(g.operatorTemplate) << "\n";
  s << "#include \"akg_rt.hpp\"\n\n";
  s << "namespace {\n";
  s << "constexpr int POSITIONS = " << positions << ", SEGMENTS = " << segments << ", KEYS = SEGMENTS, RUNS = " << runs << ", RUN = " << runLength
    << ", ID_BITS = " << idBits << ";\n";
  s << "constexpr long SLICE = " << slice << ", CHAINS = " << chains << ";\n";
  s << "constexpr long W_HIST = " << wHist << ", W_TOTAL = " << wTotal << ", W_START = " << wStart << ", W_SORTED = " << wSorted << ";\n";
  s << "using id_t = " << idTag << "::storage;\n";
  // ids as int: anything outside [0, SEGMENTS) becomes -1 (belongs to no segment and is dropped)
  if (ids.dtype == DType::I64) {
    s << "__device__ inline int as_segment(long v) { return v < 0 || v >= SEGMENTS ? -1 : static_cast<int>(v); }\n";
  } else {
    s << "__device__ inline int as_segment(int v) { return v < 0 || v >= SEGMENTS ? -1 : v; }\n";
  }
  s << "__device__ inline int key_of(int segment) { return segment; }\n";
  s << "}  // namespace\n\n";
  std::ostringstream params;
  for (size_t i = 0; i < g.inputs.size(); ++i) {
    params << (i ? ", " : "") << "const " << dtypeTag(g.tensor(g.inputs[i]).dtype) << "::storage *__restrict__ in" << i;
  }
  params << ", " << tag << "::storage *__restrict__ out0, unsigned *__restrict__ akg_ws";
  const std::string idsName = "in" + std::to_string(ids.inputIndex), dataName = "in" + std::to_string(data.inputIndex);

  emitCountingLaunches(s, g.name, params.str(), idTag, idsName, runs, segments);

  // ---- place ----
  s << "extern \"C\" __global__ __launch_bounds__(64) void " << g.name << "_place(" << params.str() << ") {\n";
  s << "  constexpr int U = 8;   // tiles of 64 positions whose ids are in flight together\n";
  s << "  __shared__ unsigned akg_next[SEGMENTS];\n";
  s << "  const int lane = static_cast<int>(threadIdx.x), run = static_cast<int>(blockIdx.x);\n";
  s << "  for (int k = lane; k < SEGMENTS; k += 64) {\n";
  s << "    akg_next[k] = akg_ws[W_START + k] + akg_ws[W_HIST + static_cast<long>(run) * SEGMENTS + k];\n";
  s << "  }\n";
  s << "  __syncthreads();\n";
  s << "  // one wavefront: its LDS accesses complete in program order, so the loop needs no barrier\n";
  s << "  const int p0 = run * RUN, p1 = p0 + RUN < POSITIONS ? p0 + RUN : POSITIONS;\n";
  s << "  const unsigned long long below = (1ull << lane) - 1ull;\n";
  if (staged) {
    // rows are copied in the widest unit that divides them (their values are not looked at)
    const int64_t rowBytes = slice * elemBytes;
    const int unitBytes = rowBytes % 4 == 0 ? 4 : rowBytes % 2 == 0 ? 2 : 1;
    s << "  using unit_t = " << (unitBytes == 4 ? "unsigned" : unitBytes == 2 ? "unsigned short" : "unsigned char") << ";\n";
    s << "  constexpr int UNITS = " << rowBytes / unitBytes << ";\n";
    s << "  const unit_t *__restrict__ rows = reinterpret_cast<const unit_t *>(" << dataName << ");\n";
    s << "  unit_t *__restrict__ placed = reinterpret_cast<unit_t *>(akg_ws + W_SORTED);\n";
  }
  s << "  for (int base = p0; base < p1; base += 64 * U) {\n";
  s << "    int id[U];\n";
  if (staged) s << "    unit_t row[U][UNITS];\n";
  s << "#pragma unroll\n";
  s << "    for (int u = 0; u < U; ++u) {\n";
  s << "      const int p = base + u * 64 + lane;\n";
  s << "      id[u] = p < p1 ? as_segment(" << idTag << "::load(" << idsName << "[p])) : -1;\n";
  if (staged) {
    s << "#pragma unroll\n";
    s << "      for (int c = 0; c < UNITS; ++c) row[u][c] = p < p1 ? rows[static_cast<long>(p) * UNITS + c] : unit_t(0);\n";
  }
  s << "    }\n";
  s << "#pragma unroll\n";
  s << "    for (int u = 0; u < U; ++u) {\n";
  s << "      if (base + u * 64 < p1) {   // (uniform; a guard and not a break, so that the tiles stay in registers)\n";
  s << "      // lanes of this tile with the same id as mine\n";
  s << "      unsigned long long same = __ballot(id[u] >= 0);\n";
  s << "#pragma unroll\n";
  s << "      for (int bit = 0; bit < ID_BITS; ++bit) {\n";
  s << "        const bool set = ((id[u] >> bit) & 1) != 0;\n";
  s << "        const unsigned long long with = __ballot(set);\n";
  s << "        same &= set ? with : ~with;\n";
  s << "      }\n";
  s << "      if (id[u] >= 0) {\n";
  s << "        const unsigned at = akg_next[id[u]];\n";
  s << "        const unsigned rank = static_cast<unsigned>(__popcll(same & below));\n";
  if (staged) {
    s << "#pragma unroll\n";
    s << "        for (int c = 0; c < UNITS; ++c) placed[static_cast<long>(at + rank) * UNITS + c] = row[u][c];\n";
  } else {
    s << "        akg_ws[W_SORTED + at + rank] = static_cast<unsigned>(base + u * 64 + lane);\n";
  }
  s << "        if ((same >> lane) >> 1 == 0ull) akg_next[id[u]] = at + rank + 1u;   // the group's highest lane\n";
  s << "      }\n";
  s << "      }\n";
  s << "    }\n";
  s << "  }\n";
  s << "}\n\n";

  // ---- chains ----
  // Short slices (one 16-byte load per data row): the wavefront of a few segments fetches 256 list entries per segment
  // and round with all its lanes (positions, then rows, many loads in flight), stages the rows in LDS, and one lane
  // per output element adds them in list order. Wide slices have enough output elements to hide the latency of a
  // plain loop per element, whose lanes read neighbouring columns of the same rows.
  int64_t segsPerWave = 1;
  if (staged) {
    segsPerWave = std::max<int64_t>(1, std::min<int64_t>(segments / 2048, 64 / slice));
    segsPerWave = std::min<int64_t>(segsPerWave, 8);
    s << "extern \"C\" __global__ __launch_bounds__(64) void " << g.name << "_kernel(" << params.str() << ") {\n";
    s << "  constexpr int S = " << segsPerWave << ", E = 256, ROW = " << slice << ";   // segments per wavefront, entries per round\n";
    s << "  __shared__ " << ct << " akg_tile[S * E * ROW];\n";
    s << "  const int lane = static_cast<int>(threadIdx.x), seg0 = static_cast<int>(blockIdx.x) * S;\n";
    s << "  const " << tag << "::storage *__restrict__ placed = reinterpret_cast<const " << tag << "::storage *>(akg_ws + W_SORTED);\n";
    s << "  unsigned from[S], upto[S], longest = 0u;\n";
    s << "#pragma unroll\n";
    s << "  for (int i = 0; i < S; ++i) {\n";
    s << "    const bool real = seg0 + i < SEGMENTS;\n";
    s << "    from[i] = real ? akg_ws[W_START + seg0 + i] : 0u;\n";
    s << "    upto[i] = real ? akg_ws[W_START + seg0 + i + 1] : 0u;\n";
    s << "    longest = upto[i] - from[i] > longest ? upto[i] - from[i] : longest;\n";
    s << "  }\n";
    s << "  // the output element of this lane, if it has one\n";
    s << "  const int cs = lane / ROW, cc = lane - cs * ROW;\n";
    s << "  const bool adds = lane < S * ROW && seg0 + cs < SEGMENTS;\n";
    s << "  unsigned mine = 0u;\n";
    s << "#pragma unroll\n";
    s << "  for (int i = 0; i < S; ++i) mine = cs == i ? upto[i] - from[i] : mine;\n";
    s << "  " << ct << " acc = " << lowering::literalFor(out.dtype, 0.0) << ";\n";
    s << "  for (unsigned r = 0; r < longest; r += E) {\n";
    s << "    " << ct << " v[S][4 * ROW];\n";
    s << "#pragma unroll\n";
    s << "    for (int i = 0; i < S; ++i) {\n";
    s << "      const unsigned k = from[i] + r + lane * 4;\n";
    s << "      if (k + 4 <= upto[i]) {\n";
    s << "        akg::load_chunk_unaligned<" << tag << ", 4 * ROW>(placed + static_cast<long>(k) * ROW, v[i]);\n";
    s << "      } else {\n";
    s << "#pragma unroll\n";
    s << "        for (int e = 0; e < 4 * ROW; ++e) {\n";
    s << "          if (k + e / ROW < upto[i]) v[i][e] = " << tag << "::load(placed[static_cast<long>(k) * ROW + e]);\n";
    s << "        }\n";
    s << "      }\n";
    s << "    }\n";
    s << "#pragma unroll\n";
    s << "    for (int i = 0; i < S; ++i) {\n";
    s << "      const unsigned k = from[i] + r + lane * 4;\n";
    s << "#pragma unroll\n";
    s << "      for (int e = 0; e < 4; ++e) {\n";
    s << "        if (k + e < upto[i]) {\n";
    s << "#pragma unroll\n";
    s << "          for (int c = 0; c < ROW; ++c) akg_tile[((i * E) + lane * 4 + e) * ROW + c] = v[i][e * ROW + c];\n";
    s << "        }\n";
    s << "      }\n";
    s << "    }\n";
    s << "    __syncthreads();\n";
    s << "    if (adds && r < mine) {\n";
    s << "      const int n = mine - r < static_cast<unsigned>(E) ? static_cast<int>(mine - r) : E;\n";
    s << "      const " << ct << " *__restrict__ row = akg_tile + cs * E * ROW + cc;\n";
    s << "      int j = 0;\n";
    s << "      for (; j + 8 <= n; j += 8) {\n";
    s << "        " << ct << " t[8];\n";
    s << "#pragma unroll\n";
    s << "        for (int u = 0; u < 8; ++u) t[u] = row[(j + u) * ROW];\n";
    s << "#pragma unroll\n";
    s << "        for (int u = 0; u < 8; ++u) acc = " << rndOpen << "akg::op_add(t[u], acc));\n";
    s << "      }\n";
    s << "      for (; j < n; ++j) acc = " << rndOpen << "akg::op_add(row[j * ROW], acc));\n";
    s << "    }\n";
    s << "    __syncthreads();\n";
    s << "  }\n";
    s << "  if (adds) out0[static_cast<long>(seg0 + cs) * ROW + cc] = " << tag << "::store(acc);\n";
    s << "}\n";
  } else {
    s << "extern \"C\" __global__ __launch_bounds__(256) void " << g.name << "_kernel(" << params.str() << ") {\n";
    s << "  constexpr int U = " << unroll << ";\n";
    s << "  const long c = static_cast<long>(blockIdx.x) * 256 + static_cast<long>(threadIdx.x);\n";
    s << "  if (c >= CHAINS) return;\n";
    s << "  const int seg = static_cast<int>(c / SLICE);\n";
    s << "  const long col = c - static_cast<long>(seg) * SLICE;\n";
    s << "  const unsigned *__restrict__ sorted = akg_ws + W_SORTED;\n";
    s << "  const " << tag << "::storage *__restrict__ data = " << dataName << " + col;\n";
    s << "  unsigned k = akg_ws[W_START + seg];\n";
    s << "  const unsigned end = akg_ws[W_START + seg + 1];\n";
    s << "  " << ct << " acc = " << lowering::literalFor(out.dtype, 0.0) << ";\n";
    s << "  for (; k + U <= end; k += U) {\n";
    s << "    unsigned p[U];\n";
    s << "    " << ct << " v[U];\n";
    s << "#pragma unroll\n";
    s << "    for (int u = 0; u < U; ++u) p[u] = sorted[k + u];\n";
    s << "#pragma unroll\n";
    s << "    for (int u = 0; u < U; ++u) v[u] = " << tag << "::load(data[static_cast<long>(p[u]) * SLICE]);\n";
    s << "#pragma unroll\n";
    s << "    for (int u = 0; u < U; ++u) acc = " << rndOpen << "akg::op_add(v[u], acc));\n";
    s << "  }\n";
    s << "  for (; k < end; ++k) acc = " << rndOpen << "akg::op_add(" << tag << "::load(data[static_cast<long>(sorted[k]) * SLICE]), acc));\n";
    s << "  out0[c] = " << tag << "::store(acc);\n";
    s << "}\n";
  }

  LoweredKernel k;
  k.kernelName = g.name + "_kernel";
  k.source = s.str();
  k.family = KernelFamily::SegmentSum;
  k.grid[0] = static_cast<unsigned>(staged ? (segments + segsPerWave - 1) / segsPerWave : (chains + 255) / 256);
  k.block[0] = staged ? 64 : 256;
  const auto phase = [&](const char *suffix, int64_t grid, unsigned block) {
    KernelPhase ph;
    ph.kernelName = g.name + suffix;
    ph.grid[0] = static_cast<unsigned>(grid);
    ph.block[0] = block;
    k.earlierPhases.push_back(ph);
  };
  phase("_count", runs, 256);
  phase("_offsets", offsetsGrid(segments), 256);
  phase("_starts", 1, 1024);
  phase("_place", runs, 64);
  k.workspaceBytes = static_cast<uint64_t>(words) * 4;
  k.algorithmicBytes = lowering::countAlgorithmicBytes(g);
  k.shapeArgs = lowering::buildShapeArgs(g);
  std::ostringstream note;
  note << "segment_sum positions=" << positions << " segments=" << segments << " slice=" << slice << " grouped by segment: runs="
       << runs << " of " << runLength << " positions, 5 launches";
  k.scheduleNote = note.str();
  return k;
}

// Device code both launches of the bucketed schedule share: a stable counting sort of a chunk by key inside a workgroup.
const char *const kChunkSort = R"AKG(
// Stable counting sort of a chunk of NW x TILES x 64 items by key, inside a workgroup of NW wavefronts. Item (w, u, lane)
// - wavefront, tile, lane, in this order of significance - has key[u] (negative: the item takes no part); the function
// returns its place among the sorted items in slot[u]. First every wavefront ranks its own items: lanes of a tile with
// the same key find each other with one ballot per key bit and stand behind the wavefront's running counter of that
// key (its LDS accesses complete in program order, so the counters need no barrier between the tiles). Then the
// counters are summed over the wavefronts and the keys (each key's run starts at a multiple of ALIGN), and every item
// adds where the run of its key and wavefront starts. On return start[k] is where key k's run starts, len[k] its
// length; a barrier has been passed since they were written. cnt: NW * KEYS counters, scan: NW words.
template <int NW, int KEYS, int KEY_BITS, int TILES, int ALIGN>
__device__ inline void chunk_sort(const int (&key)[TILES], unsigned (&slot)[TILES], unsigned short *cnt, unsigned *start,
                                  unsigned *len, unsigned *scan) {
  constexpr int THREADS = NW * 64, PER = (KEYS + THREADS - 1) / THREADS;
  const int tid = static_cast<int>(threadIdx.x), lane = tid & 63, w = tid >> 6;
  for (int k = tid; k < NW * KEYS; k += THREADS) cnt[k] = 0;
  __syncthreads();
  const unsigned long long below = (1ull << lane) - 1ull;
  unsigned short *mine = cnt + w * KEYS;
#pragma unroll
  for (int u = 0; u < TILES; ++u) {
    const int k = key[u] >= 0 ? key[u] : 0;
    unsigned long long same = __ballot(key[u] >= 0);
#pragma unroll
    for (int bit = 0; bit < KEY_BITS; ++bit) {
      const int mine_bit = __builtin_amdgcn_sbfe(k, bit, 1);   // 0 or all ones
      const unsigned long long with = __ballot(mine_bit != 0);
      const unsigned lo = ~(static_cast<unsigned>(with) ^ static_cast<unsigned>(mine_bit));
      const unsigned hi = ~(static_cast<unsigned>(with >> 32) ^ static_cast<unsigned>(mine_bit));
      same &= (static_cast<unsigned long long>(hi) << 32) | lo;   // lanes whose bit equals mine
    }
    slot[u] = 0u;
    if (key[u] >= 0) {
      const unsigned at = mine[k] + static_cast<unsigned>(__popcll(same & below));
      slot[u] = at;
      if ((same >> lane) >> 1 == 0ull) mine[k] = static_cast<unsigned short>(at + 1u);   // the group's highest lane
    }
  }
  __syncthreads();
  unsigned total[PER], sum = 0u;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int k = tid * PER + j;
    unsigned before = 0u;
    if (k < KEYS) {
#pragma unroll
      for (int h = 0; h < NW; ++h) {
        const unsigned c = cnt[h * KEYS + k];
        cnt[h * KEYS + k] = static_cast<unsigned short>(before);
        before += c;
      }
      len[k] = before;
    }
    total[j] = (before + ALIGN - 1) / ALIGN * ALIGN;
    sum += total[j];
  }
  unsigned incl = sum;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const unsigned o = __shfl_up(incl, d);
    if (lane >= d) incl += o;
  }
  if (lane == 63) scan[w] = incl;
  __syncthreads();
  unsigned at = incl - sum;
#pragma unroll
  for (int j = 0; j < NW; ++j) at += j < w ? scan[j] : 0u;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int k = tid * PER + j;
    if (k < KEYS) {
      start[k] = at;
#pragma unroll
      for (int h = 0; h < NW; ++h) cnt[h * KEYS + k] += static_cast<unsigned short>(at);
    }
    at += total[j];
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < TILES; ++u) {
    if (key[u] >= 0) slot[u] += mine[key[u]];
  }
}
)AKG";

/**
 * Very many positions of short rows (at most 12 bytes): grouping by segment in one step writes every row to a place of
 * its own, a partial cache line each time (24.5 million 12-byte rows: 1.07 GB written for 0.29 GB of rows). Here the
 * positions are first grouped by BUCKET, a few neighbouring segments, and the last step to the segment happens in LDS:
 *
 *   <op>_count / _offsets / _starts   as above, with the bucket as the key and chunks of 4096 positions as the runs
 *   <op>_place    a workgroup sorts its chunk by bucket in LDS (chunk_sort above) and copies the sorted chunk out, one
 *                 16-byte entry per position {row, segment}: a bucket's entries of one chunk are contiguous, so the
 *                 stores fill whole sectors
 *   <op>_kernel   a workgroup per bucket walks the bucket's entries, 4096 per round: the same sort, by segment now,
 *                 puts the rows' columns into LDS lists per segment, and one lane per output element adds its list
 *
 * Both sorts are stable, so the order per output element is the position order and the result is the serial loop's,
 * bit for bit.
 */
LoweredKernel lowerSegmentBucketed(const OpGraph &g, const LoweringOptions &, const SegmentShapes &sh, int bucketBits) {
  using lowering::computeTypeName;
  using lowering::dtypeTag;
  const TensorValue &data = *sh.data, &ids = *sh.ids, &out = *sh.out;
  const int64_t positions = sh.positions, segments = sh.segments, slice = sh.slice;
  const std::string ct = computeTypeName(out.dtype), tag = dtypeTag(out.dtype), idTag = dtypeTag(ids.dtype);
  const bool narrow = out.dtype == DType::F16 || out.dtype == DType::BF16 || out.dtype == DType::I8 || out.dtype == DType::I16;
  const std::string rndOpen = narrow ? tag + "::rnd(" : std::string("(");
  const int elemBytes = static_cast<int>(dtypeSize(out.dtype));
  const int64_t rowWords = slice * elemBytes / 4;
  const int64_t perBucket = 1LL << bucketBits, buckets = (segments + perBucket - 1) / perBucket;
  const int64_t chunk = 4096, chunks = (positions + chunk - 1) / chunk;
  int keyBits = 1;
  while ((1LL << keyBits) < buckets) ++keyBits;
  // workspace, in 4-byte words
  const int64_t wHist = 0, wTotal = wHist + chunks * buckets, wStart = wTotal + buckets,
                wSorted = (wStart + buckets + 1 + 3) / 4 * 4;   // 16-byte aligned
  const int64_t words = wSorted + positions * 4;

  std::ostringstream s;
  s << "// Generated by the akg HIP lowering for gfx950. Op description: " << g.name << "\n";
  s << "// family: segment_sum (positions grouped by bucket of segments first), fusion class: " << operatorTemplateName(g.operatorTemplate) << "\n";
  s << "#include \"akg_rt.hpp\"\n\n";
  s << "namespace {\n";
  s << "constexpr int POSITIONS = " << positions << ", SEGMENTS = " << segments << ", BUCKET_BITS = " << bucketBits << ", KEYS = " << buckets
    << ", KEY_BITS = " << keyBits << ", RUNS = " << chunks << ", RUN = " << chunk << ";\n";
  s << "constexpr int ROW = " << slice << ", ROW_WORDS = " << rowWords << ", NW = 8, TILES = RUN / (64 * NW);\n";
  s << "constexpr long W_HIST = " << wHist << ", W_TOTAL = " << wTotal << ", W_START = " << wStart << ", W_SORTED = " << wSorted << ";\n";
  s << "using id_t = " << idTag << "::storage;\n";
  if (ids.dtype == DType::I64) {
    s << "__device__ inline int as_segment(long v) { return v < 0 || v >= SEGMENTS ? -1 : static_cast<int>(v); }\n";
  } else {
    s << "__device__ inline int as_segment(int v) { return v < 0 || v >= SEGMENTS ? -1 : v; }\n";
  }
  s << "__device__ inline int key_of(int segment) { return segment >> BUCKET_BITS; }\n";
  s << "typedef unsigned entry_t __attribute__((ext_vector_type(4)));   // x, y, z: the row's words, zero filled; w: segment\n";
  s << kChunkSort;
  s << "}  // namespace\n\n";
  std::ostringstream params;
  for (size_t i = 0; i < g.inputs.size(); ++i) {
    params << (i ? ", " : "") << "const " << dtypeTag(g.tensor(g.inputs[i]).dtype) << "::storage *__restrict__ in" << i;
  }
  params << ", " << tag << "::storage *__restrict__ out0, unsigned *__restrict__ akg_ws";
  const std::string idsName = "in" + std::to_string(ids.inputIndex), dataName = "in" + std::to_string(data.inputIndex);

  emitCountingLaunches(s, g.name, params.str(), idTag, idsName, chunks, buckets);

  // ---- place ----
  // Workgroups that run at the same time on one XCD (launch order: workgroup b runs on XCD b mod 8) take neighbouring
  // chunks, whose entries are neighbours in every bucket: the line two chunks share is completed in that XCD's L2.
  const int64_t perXcd = (chunks + 7) / 8;
  s << "extern \"C\" __global__ __launch_bounds__(512) void " << g.name << "_place(" << params.str() << ") {\n";
  s << "  __shared__ entry_t akg_stage[RUN];\n";
  s << "  __shared__ unsigned short akg_cnt[NW * KEYS];\n";
  s << "  __shared__ unsigned akg_start[KEYS], akg_len[KEYS], akg_scan[NW];\n";
  s << "  const int tid = static_cast<int>(threadIdx.x), lane = tid & 63, w = tid >> 6;\n";
  s << "  const int run = static_cast<int>(blockIdx.x & 7u) * " << perXcd << " + static_cast<int>(blockIdx.x >> 3);\n";
  s << "  if (run >= RUNS) return;   // (uniform)\n";
  s << "  const int p0 = run * RUN + w * (64 * TILES);\n";
  s << "  const unsigned *__restrict__ rows = reinterpret_cast<const unsigned *>(" << dataName << ");\n";
  s << "  int id[TILES], key[TILES];\n  unsigned row[TILES][ROW_WORDS], slot[TILES];\n";
  s << "#pragma unroll\n";
  s << "  for (int u = 0; u < TILES; ++u) {\n";
  s << "    const int p = p0 + u * 64 + lane;\n";
  s << "    id[u] = p < POSITIONS ? as_segment(" << idTag << "::load(" << idsName << "[p])) : -1;\n";
  s << "    key[u] = id[u] >= 0 ? key_of(id[u]) : -1;\n";
  s << "#pragma unroll\n";
  s << "    for (int c = 0; c < ROW_WORDS; ++c) row[u][c] = p < POSITIONS ? rows[static_cast<long>(p) * ROW_WORDS + c] : 0u;\n";
  s << "  }\n";
  s << "  chunk_sort<NW, KEYS, KEY_BITS, TILES, 1>(key, slot, akg_cnt, akg_start, akg_len, akg_scan);\n";
  s << "#pragma unroll\n";
  s << "  for (int u = 0; u < TILES; ++u) {\n";
  s << "    if (id[u] >= 0) {\n";
  s << "      entry_t e = {0u, 0u, 0u, static_cast<unsigned>(id[u])};\n";
  s << "      e.x = row[u][0];\n";
  if (rowWords > 1) s << "      e.y = row[u][1];\n";
  if (rowWords > 2) s << "      e.z = row[u][2];\n";
  s << "      akg_stage[slot[u]] = e;\n";
  s << "    }\n";
  s << "  }\n";
  s << "  // where the bucket's entries of this chunk go, less where they are in the sorted chunk\n";
  s << "  unsigned valid = 0u;\n";
  s << "  for (int k = tid; k < KEYS; k += 64 * NW) {\n";
  s << "    if (k == KEYS - 1) akg_scan[0] = akg_start[k] + akg_len[k];\n";
  s << "    akg_start[k] = akg_ws[W_START + k] + akg_ws[W_HIST + static_cast<long>(run) * KEYS + k] - akg_start[k];\n";
  s << "  }\n";
  s << "  __syncthreads();\n";
  s << "  valid = akg_scan[0];\n";
  s << "  entry_t *__restrict__ placed = reinterpret_cast<entry_t *>(akg_ws + W_SORTED);\n";
  s << "  for (unsigned i = tid; i < valid; i += 64 * NW) {\n";
  s << "    const entry_t e = akg_stage[i];\n";
  s << "    placed[akg_start[key_of(static_cast<int>(e.w))] + i] = e;\n";
  s << "  }\n";
  s << "}\n\n";

  // ---- chains ----
  const int64_t chains = perBucket * slice, chainsPerWave = (chains + 7) / 8;
  s << "extern \"C\" __global__ __launch_bounds__(512) void " << g.name << "_kernel(" << params.str() << ") {\n";
  s << "  constexpr int S = 1 << BUCKET_BITS, PLANE = RUN + 4 * S + 8, CHAINS = " << chains << ", PER_WAVE = " << chainsPerWave << ";\n";
  s << "  __shared__ __attribute__((aligned(16))) " << ct << " akg_plane[ROW][PLANE];   // column c of the rows, lists per segment\n";
  s << "  __shared__ unsigned short akg_cnt[NW * S];\n";
  s << "  __shared__ unsigned akg_start[S], akg_len[S], akg_scan[NW];\n";
  s << "  const int tid = static_cast<int>(threadIdx.x), lane = tid & 63, w = tid >> 6, bucket = static_cast<int>(blockIdx.x);\n";
  s << "  const entry_t *__restrict__ placed = reinterpret_cast<const entry_t *>(akg_ws + W_SORTED);\n";
  s << "  const unsigned from = akg_ws[W_START + bucket], upto = akg_ws[W_START + bucket + 1];\n";
  s << "  constexpr unsigned LAST = POSITIONS - 1;\n";
  s << "  // the output element of this lane, if it has one: wavefront w adds chains w * PER_WAVE ...\n";
  s << "  const int chain = w * PER_WAVE + lane;\n";
  s << "  const bool has = lane < PER_WAVE && chain < CHAINS;\n";
  s << "  const int cs = has ? chain / ROW : 0, cc = has ? chain - cs * ROW : 0;\n";
  s << "  union cell_t { entry_t q; " << tag << "::storage v[16 / sizeof(" << tag << "::storage)]; };\n";
  s << "  typedef " << ct << " quad_t __attribute__((ext_vector_type(4)));\n";
  s << "  " << ct << " acc = " << lowering::literalFor(out.dtype, 0.0) << ";\n";
  s << "  for (unsigned r = from; r < upto; r += RUN) {\n";
  s << "    cell_t cur[TILES];\n";
  s << "    int key[TILES];\n";
  s << "    unsigned slot[TILES];\n";
  s << "    // (every load is issued, the address clamped to the workspace's last entry: no branch between the loads)\n";
  s << "#pragma unroll\n";
  s << "    for (int u = 0; u < TILES; ++u) {\n";
  s << "      const unsigned k = r + (w * TILES + u) * 64 + lane;\n";
  s << "      cur[u].q = __builtin_nontemporal_load(placed + (k < LAST ? k : LAST));\n";
  s << "    }\n";
  s << "#pragma unroll\n";
  s << "    for (int u = 0; u < TILES; ++u) {\n";
  s << "      const unsigned k = r + (w * TILES + u) * 64 + lane;\n";
  s << "      key[u] = k < upto ? static_cast<int>(cur[u].q.w) & (S - 1) : -1;\n";
  s << "    }\n";
  s << "    chunk_sort<NW, S, BUCKET_BITS, TILES, 4>(key, slot, akg_cnt, akg_start, akg_len, akg_scan);\n";
  s << "#pragma unroll\n";
  s << "    for (int u = 0; u < TILES; ++u) {\n";
  s << "      if (key[u] >= 0) {\n";
  s << "#pragma unroll\n";
  s << "        for (int c = 0; c < ROW; ++c) akg_plane[c][slot[u]] = " << tag << "::load(cur[u].v[c]);\n";
  s << "      }\n";
  s << "    }\n";
  s << "    __syncthreads();\n";
  s << "    if (has) {\n";
  s << "      const int n = static_cast<int>(akg_len[cs]);\n";
  s << "      const quad_t *__restrict__ list = reinterpret_cast<const quad_t *>(&akg_plane[cc][akg_start[cs]]);   // (a multiple of 4)\n";
  s << "      int j = 0;\n";
  s << "      for (; j + 8 <= n; j += 8) {\n";
  s << "        const quad_t a = list[j / 4], b = list[j / 4 + 1];\n";
  s << "#pragma unroll\n";
  s << "        for (int u = 0; u < 4; ++u) acc = " << rndOpen << "akg::op_add(a[u], acc));\n";
  s << "#pragma unroll\n";
  s << "        for (int u = 0; u < 4; ++u) acc = " << rndOpen << "akg::op_add(b[u], acc));\n";
  s << "      }\n";
  s << "      if (j < n) {   // (what lies behind the list's end is read, inside the plane, and not added)\n";
  s << "        const quad_t a = list[j / 4], b = list[j / 4 + 1];\n";
  s << "#pragma unroll\n";
  s << "        for (int u = 0; u < 8; ++u) {\n";
  s << "          const " << ct << " sum = " << rndOpen << "akg::op_add(u < 4 ? a[u & 3] : b[u & 3], acc));\n";
  s << "          acc = j + u < n ? sum : acc;\n";
  s << "        }\n";
  s << "      }\n";
  s << "    }\n";
  s << "    __syncthreads();\n";
  s << "  }\n";
  s << "  if (has && bucket * S + cs < SEGMENTS) out0[static_cast<long>(bucket * S + cs) * ROW + cc] = " << tag << "::store(acc);\n";
  s << "}\n";

  LoweredKernel k;
  k.kernelName = g.name + "_kernel";
  k.source = s.str();
  k.family = KernelFamily::SegmentSum;
  k.grid[0] = static_cast<unsigned>(buckets);
  k.block[0] = 512;
  const auto phase = [&](const char *suffix, int64_t grid, unsigned block) {
    KernelPhase ph;
    ph.kernelName = g.name + suffix;
    ph.grid[0] = static_cast<unsigned>(grid);
    ph.block[0] = block;
    k.earlierPhases.push_back(ph);
  };
  phase("_count", chunks, 256);
  phase("_offsets", offsetsGrid(buckets), 256);
  phase("_starts", 1, 1024);
  phase("_place", perXcd * 8, 512);
  k.workspaceBytes = static_cast<uint64_t>(words) * 4;
  k.algorithmicBytes = lowering::countAlgorithmicBytes(g);
  k.shapeArgs = lowering::buildShapeArgs(g);
  std::ostringstream note;
  note << "segment_sum positions=" << positions << " segments=" << segments << " slice=" << slice << " grouped by bucket of " << perBucket
       << " segments: " << buckets << " buckets, chunks=" << chunks << " of " << chunk << " positions, 5 launches";
  k.scheduleNote = note.str();
  return k;
}

LoweredKernel lowerSegmentScan(const OpGraph &g, const LoweringOptions &options, const SegmentShapes &sh) {
  using lowering::computeTypeName;
  using lowering::dtypeTag;
  const OpNode &op = *sh.op;
  const TensorValue &data = *sh.data, &ids = *sh.ids, &out = *sh.out;
  const int64_t positions = sh.positions, segments = sh.segments, slice = sh.slice;
  const std::string ct = computeTypeName(out.dtype), tag = dtypeTag(out.dtype), idTag = dtypeTag(ids.dtype);
  const bool narrow = out.dtype == DType::F16 || out.dtype == DType::BF16 || out.dtype == DType::I8 || out.dtype == DType::I16;
  const int accBytes = out.dtype == DType::I64 || out.dtype == DType::F64 ? 8 : 4;
  // Short slices: the lane that found the id adds the whole slice itself (its data loads are issued before the
  // serial part). Otherwise the threads of the workgroup share the columns of the slice.
  const bool laneOwned = slice <= 4;
  const int block = options.block > 0 ? options.block : (slice <= 64 ? 64 : 256);
  if (block % 64 != 0 || block > 1024 || (laneOwned && block != 64)) throw LoweringError("op " + op.name + ": unsupported block size");
  const int64_t sliceTile = std::min<int64_t>(slice, 8192 / (accBytes / 4));
  const int64_t sliceTiles = (slice + sliceTile - 1) / sliceTile;
  // segments per workgroup: about 1024 workgroups (every one of them scans all ids; measured on 24.5 million positions
  // into 4954 segments: 256 -> 36 ms, 512 -> 26 ms, 1024 -> 21.6 ms, 2048 -> 20.4 ms), bounded by 32 KB of accumulators
  const int64_t wantGroups = options.split > 0 ? options.split : 1024;
  int64_t segsPerWg = std::max<int64_t>(1, (segments * sliceTiles + wantGroups - 1) / wantGroups);
  segsPerWg = std::min<int64_t>(segsPerWg, std::max<int64_t>(1, 32768 / (sliceTile * accBytes)));
  const int64_t groups = (segments + segsPerWg - 1) / segsPerWg;
  if (groups >= (1LL << 31) || sliceTiles >= 65536) throw LoweringError("op " + op.name + ": too large");
  // ids per lane and load (one 16-byte load where the id type allows), loads in flight per lane
  const int idv = ids.dtype == DType::I32 ? 4 : ids.dtype == DType::I64 ? 2 : 1;
  const int unroll = options.chunks > 0 ? options.chunks : 4;
  const std::string rndOpen = narrow ? tag + "::rnd(" : std::string("(");
  std::ostringstream s;
  s << "// Generated by the akg HIP lowering for gfx950. Op description: " << g.name << "\n";
  s << "// family: segment_sum, fusion class: " << operatorTemplateName(g.operatorTemplate) << "\n";
  s << "#include \"akg_rt.hpp\"\n\n";
  s << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << g.name << "_kernel(";
  for (size_t i = 0; i < g.inputs.size(); ++i) {
    s << (i ? ", " : "") << "const " << dtypeTag(g.tensor(g.inputs[i]).dtype) << "::storage *__restrict__ in" << i;
  }
  s << ", " << tag << "::storage *__restrict__ out0) {\n";
  s << "  constexpr int POSITIONS = " << positions << ", SEGMENTS = " << segments << ", SEGS = " << segsPerWg << ";\n";
  s << "  constexpr long SLICE = " << slice << ";\n  constexpr int TILE = " << sliceTile << ", BLOCK = " << block
    << ", IDV = " << idv << ", U = " << unroll << ";\n";
  s << "  using id_t = " << idTag << "::storage;\n";
  s << "  struct __attribute__((aligned(sizeof(id_t) * IDV))) id_chunk { id_t v[IDV]; };\n";
  s << "  __shared__ " << ct << " akg_acc[SEGS * TILE];\n";
  s << "  const int tid = static_cast<int>(threadIdx.x), lane = tid & 63;\n";
  s << "  const int seg0 = static_cast<int>(blockIdx.x) * SEGS;\n";
  s << "  const int seg1 = seg0 + SEGS < SEGMENTS ? seg0 + SEGS : SEGMENTS;\n";
  s << "  const long col0 = static_cast<long>(blockIdx.y) * TILE;\n";
  s << "  const int cols = SLICE - col0 < TILE ? static_cast<int>(SLICE - col0) : TILE;\n";
  s << "  const id_t *__restrict__ ids = in" << ids.inputIndex << ";\n";
  s << "  const " << tag << "::storage *__restrict__ data = in" << data.inputIndex << ";\n";
  s << "  for (int k = tid; k < SEGS * TILE; k += BLOCK) akg_acc[k] = " << lowering::literalFor(out.dtype, 0.0) << ";\n";
  s << "  __syncthreads();\n";
  if (laneOwned) {
    s << "  // one wavefront: LDS accesses of a wavefront complete in program order, so the loop needs no barrier\n";
  } else {
    s << "  // from here on a thread reads and writes only its own accumulator columns: no further barrier\n";
  }
  // ids as int: anything outside [0, SEGMENTS) becomes -1 (matches nobody)
  const std::string toInt = ids.dtype == DType::I64
      ? "[](long v) { return v < 0 || v >= SEGMENTS ? -1 : static_cast<int>(v); }"
      : "[](int v) { return v; }";
  s << "  const auto as_int = " << toInt << ";\n";
  // The part every lane can load without a bounds check runs double-buffered: the ids of the next step are in flight
  // while the hits of the current one are handled. The last, partial step loads element by element.
  const auto emitHits = [&](const std::string &ind) {
    const std::string isHit = "(id[u][e] >= seg0 && id[u][e] < seg1)";
    if (laneOwned) {
      // first every data load of the step (all lanes, all chunks at once), then the additions in position order
      s << ind << "unsigned long long hits[U];\n";
      s << ind << ct << " v[U][IDV][" << slice << "];\n";
      s << ind << "#pragma unroll\n";
      s << ind << "for (int u = 0; u < U; ++u) {\n";
      s << ind << "  bool mine = false;\n";
      s << ind << "#pragma unroll\n";
      s << ind << "  for (int e = 0; e < IDV; ++e) mine = mine || " << isHit << ";\n";
      s << ind << "  hits[u] = __ballot(mine);\n";
      s << ind << "  if (hits[u] == 0) continue;\n";
      s << ind << "  const long mypos = static_cast<long>(base) + static_cast<long>(u * 64 + lane) * IDV;\n";
      s << ind << "#pragma unroll\n";
      s << ind << "  for (int e = 0; e < IDV; ++e) {\n";
      s << ind << "    if " << isHit << " {\n";
      s << ind << "#pragma unroll\n";
      s << ind << "      for (int c = 0; c < " << slice << "; ++c) v[u][e][c] = " << tag << "::load(data[(mypos + e) * SLICE + c]);\n";
      s << ind << "    }\n" << ind << "  }\n" << ind << "}\n";
      s << ind << "#pragma unroll\n";
      s << ind << "for (int u = 0; u < U; ++u) {\n";
      s << ind << "  unsigned long long todo = hits[u];\n";
      s << ind << "  while (todo) {   // ascending lanes = ascending positions\n";
      s << ind << "    const int b = __builtin_ctzll(todo);\n";
      s << ind << "    todo &= todo - 1;\n";
      s << ind << "    if (lane == b) {\n";
      s << ind << "#pragma unroll\n";
      s << ind << "      for (int e = 0; e < IDV; ++e) {\n";
      s << ind << "        if " << isHit << " {\n";
      s << ind << "          const int row = id[u][e] - seg0;\n";
      s << ind << "#pragma unroll\n";
      s << ind << "          for (int c = 0; c < " << slice << "; ++c) {\n";
      s << ind << "            akg_acc[row * TILE + c] = " << rndOpen << "akg::op_add(v[u][e][c], akg_acc[row * TILE + c]));\n";
      s << ind << "          }\n" << ind << "        }\n" << ind << "      }\n" << ind << "    }\n" << ind << "  }\n";
      s << ind << "}\n";
      return;
    }
    s << ind << "#pragma unroll\n";
    s << ind << "for (int u = 0; u < U; ++u) {\n";
    s << ind << "  bool mine = false;\n";
    s << ind << "#pragma unroll\n";
    s << ind << "  for (int e = 0; e < IDV; ++e) mine = mine || " << isHit << ";\n";
    s << ind << "  unsigned long long hits = __ballot(mine);\n";
    s << ind << "  if (hits == 0) continue;\n";
    s << ind << "  const long first = static_cast<long>(base) + static_cast<long>(u * 64) * IDV;   // lane 0, element 0\n";
    s << ind << "  while (hits) {   // ascending lanes, then ascending elements = ascending positions\n";
    s << ind << "    const int b = __builtin_ctzll(hits);\n";
    s << ind << "    hits &= hits - 1;\n";
    s << ind << "#pragma unroll\n";
    s << ind << "    for (int e = 0; e < IDV; ++e) {\n";
    s << ind << "      const int sid = __builtin_amdgcn_readlane(id[u][e], b);\n";
    s << ind << "      if (sid < seg0 || sid >= seg1) continue;\n";
    s << ind << "      const int row = sid - seg0;\n";
    s << ind << "      const long from = (first + b * IDV + e) * SLICE + col0;\n";
    s << ind << "      for (int c = tid; c < cols; c += BLOCK) {\n";
    s << ind << "        akg_acc[row * TILE + c] = " << rndOpen << "akg::op_add(" << tag
      << "::load(data[from + c]), akg_acc[row * TILE + c]));\n";
    s << ind << "      }\n" << ind << "    }\n" << ind << "  }\n";
    s << ind << "}\n";
  };
  s << "  constexpr int STEP = 64 * IDV * U, FULL = POSITIONS / STEP * STEP;\n";
  s << "  if (FULL > 0) {\n";
  s << "    id_chunk next[U];\n";
  s << "#pragma unroll\n";
  s << "    for (int u = 0; u < U; ++u) next[u] = *reinterpret_cast<const id_chunk *>(ids + (u * 64 + lane) * IDV);\n";
  s << "    for (int base = 0; base < FULL; base += STEP) {\n";
  s << "      int id[U][IDV];\n";
  s << "#pragma unroll\n";
  s << "      for (int u = 0; u < U; ++u) {\n";
  s << "#pragma unroll\n";
  s << "        for (int e = 0; e < IDV; ++e) id[u][e] = as_int(" << idTag << "::load(next[u].v[e]));\n";
  s << "      }\n";
  s << "      if (base + STEP < FULL) {\n";
  s << "#pragma unroll\n";
  s << "        for (int u = 0; u < U; ++u) next[u] = *reinterpret_cast<const id_chunk *>(ids + base + STEP + (u * 64 + lane) * IDV);\n";
  s << "      }\n";
  emitHits("      ");
  s << "    }\n  }\n";
  s << "  if (FULL < POSITIONS) {\n";
  s << "    constexpr int base = FULL;\n";
  s << "    int id[U][IDV];\n";
  s << "#pragma unroll\n";
  s << "    for (int u = 0; u < U; ++u) {\n";
  s << "#pragma unroll\n";
  s << "      for (int e = 0; e < IDV; ++e) {\n";
  s << "        const int p = base + (u * 64 + lane) * IDV + e;\n";
  s << "        id[u][e] = p < POSITIONS ? as_int(" << idTag << "::load(ids[p])) : -1;\n";
  s << "      }\n    }\n";
  emitHits("    ");
  s << "  }\n";
  s << "  for (int r = 0; r < seg1 - seg0; ++r) {\n";
  s << "    for (int c = tid; c < cols; c += BLOCK) {\n";
  s << "      out0[static_cast<long>(seg0 + r) * SLICE + col0 + c] = " << tag << "::store(akg_acc[r * TILE + c]);\n";
  s << "    }\n  }\n}\n";

  LoweredKernel k;
  k.kernelName = g.name + "_kernel";
  k.source = s.str();
  k.family = KernelFamily::SegmentSum;
  k.grid[0] = static_cast<unsigned>(groups);
  k.grid[1] = static_cast<unsigned>(sliceTiles);
  k.block[0] = block;
  k.algorithmicBytes = lowering::countAlgorithmicBytes(g);
  k.shapeArgs = lowering::buildShapeArgs(g);
  std::ostringstream note;
  note << "segment_sum positions=" << positions << " segments=" << segments << " slice=" << slice << " segments/workgroup=" << segsPerWg << " slice tile=" << sliceTile;
  k.scheduleNote = note.str();
  return k;
}

}  // namespace

LoweredKernel lowerSegmentSumToHip(const OpGraph &g, const LoweringOptions &options) {
  const SegmentShapes sh = checkSegmentSum(g);
  // Grouping pays once the repeated id scan costs more than a few launches: from 2^16 positions on
  // (69 thousand positions into 4954 segments: 0.050 ms grouped, 0.069 ms scanned). Its LDS counters
  // hold one word per segment.
  const bool canGroup = sh.segments <= 16384 && sh.segments * sh.slice + 256 < (1LL << 31);
  const bool group = options.variant >= 2 ? canGroup : options.variant == 1 ? false : canGroup && sh.positions >= (1 << 16);
  // Short rows (4, 8 or 12 bytes, 4-byte arithmetic) into many segments: by bucket first. The bucket is the largest power
  // of two of segments whose output elements number at most 32; there are at most 640 buckets (the counters of a chunk
  // must leave room for two workgroups per CU) and, unless asked for, at least 96 (the last launch has one workgroup
  // per bucket: 1 to 4 million positions into 300 segments run 1.3 to 1.9 times slower than grouped by segment; 0.3 to
  // 4 million into 5000 segments 1.7 to 2.2 times faster, 24.5 million 1.9 times).
  const int64_t rowBytes = sh.slice * static_cast<int64_t>(dtypeSize(sh.out->dtype));
  const bool wide = sh.out->dtype == DType::I64 || sh.out->dtype == DType::F64;
  int bucketBits = 4;
  while (bucketBits > 0 && (sh.slice << bucketBits) > 32) --bucketBits;
  const int64_t buckets = (sh.segments + (1LL << bucketBits) - 1) >> bucketBits;
  const bool canBucket = group && !wide && rowBytes <= 12 && rowBytes % 4 == 0 && bucketBits >= 2 && buckets <= 640 && buckets >= 2;
  if (canBucket && (options.variant == 3 || (options.variant == 0 && buckets >= 96))) {
    return lowerSegmentBucketed(g, options, sh, bucketBits);
  }
  return group ? lowerSegmentSorted(g, options, sh) : lowerSegmentScan(g, options, sh);
}

}  // namespace akg
