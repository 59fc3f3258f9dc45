/**
 * Elementwise and row-reduction kernels: the op chain of a fused description on register arrays, one thread per
 * group of 16-byte chunks (family `elementwise`), or one row per group of threads with the row resident in registers
 * across the reductions of the fusion (family `row_reduce`).
 */
#include "HipLowering.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <sstream>

namespace akg {

namespace {

using lowering::computeTypeName;
using lowering::dtypeTag;

int64_t product(const std::vector<int64_t> &v, size_t from = 0, size_t to = static_cast<size_t>(-1)) {
  int64_t p = 1;
  if (to > v.size()) to = v.size();
  for (size_t i = from; i < to; ++i) p *= v[i];
  return p;
}

int64_t ceilDiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

int pow2AtLeast(int64_t x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

// Right-aligns `shape` to `rank` dims (numpy broadcasting), dropping surplus leading 1s.
std::vector<int64_t> padShape(const std::vector<int64_t> &shape, size_t rank, const std::string &what) {
  std::vector<int64_t> s = shape;
  while (s.size() > rank && s.front() == 1) s.erase(s.begin());
  if (s.size() > rank) throw LoweringError(what + ": rank exceeds the kernel's iteration space");
  std::vector<int64_t> out(rank - s.size(), 1);
  out.insert(out.end(), s.begin(), s.end());
  return out;
}

enum class ValRank { Const, Uniform, Tile };

struct ValInfo {
  bool defined = false;
  ValRank rank = ValRank::Const;
  std::string ident;         // variable name (Tile: array, Uniform: scalar); Const: literal text
  bool rowvecNoKeep = false; // Uniform value whose tensor shape lacks the trailing 1 (reduce without keep_dims)
};

// How a kernel input is addressed relative to the iteration space [rows, cols].
struct InputAccess {
  bool lastDimFull = false;          // true: V consecutive elements per chunk; false: one element per row
  std::vector<int64_t> foldedShape;  // shape aligned to the (possibly folded) iteration space
};

class TileEmitter {
 public:
  TileEmitter(const OpGraph &g, const LoweringOptions &o) : g_(g), opt_(o) { nonTemporal_ = (o.nonTemporal != 0); }

  LoweredKernel run() {
    analyse();
    pickSchedule();
    emit();
    LoweredKernel k;
    k.kernelName = g_.name + "_kernel";
    k.source = src_.str();
    k.family = rowMode_ ? KernelFamily::RowReduce : KernelFamily::Elementwise;
    k.grid[0] = static_cast<unsigned>(grid_);
    k.block[0] = static_cast<unsigned>(block_);
    k.algorithmicBytes = lowering::countAlgorithmicBytes(g_);
    k.shapeArgs = lowering::buildShapeArgs(g_);
    if (extentArg_) k.scalarArgs.push_back(extentIsCols_ ? cols_ : rows_);
    if (colsArg_) k.scalarArgs.push_back(cols_);
    if (dimsArg_) {
      for (size_t d = 0; d + 1 < full_.size(); ++d) k.scalarArgs.push_back(full_[d]);
    }
    std::ostringstream note;
    note << kernelFamilyName(k.family) << " rows=" << rows_ << " cols=" << cols_ << " vec=" << vec_
         << " threads_per_row=" << tpr_ << " chunks=" << chunks_ << " rows_per_block=" << rowsPerBlock_
         << " block=" << block_ << " grid=" << grid_;
    if (overlap_ > 0) note << " tail_overlap=" << overlap_;
    if (colsArg_) note << " (row length is a kernel argument: one code object for rows of " << bucketLow_ << " .. " << bucketHigh_ << " elements" << (colsWhole_ ? " that are whole 64-byte pieces" : "") << ")";
    if (multiPass_) note << " walks_of_groups=" << groups_ << (packedRow_ ? " (row packed in registers)" : "");
    k.scheduleNote = note.str();
    return k;
  }

 private:
  const OpGraph &g_;
  LoweringOptions opt_;
  std::ostringstream src_;

  bool rowMode_ = false;
  std::vector<int64_t> full_;     // iteration space (folded in elementwise mode)
  int64_t rows_ = 1, cols_ = 1, numel_ = 1;
  bool extentArg_ = false;     // the row count (or COLS when everything folded into one dim) is a kernel argument
  bool extentIsCols_ = false;
  // Dynamic descriptions: the row length COLS is a second kernel argument. The schedule (threads per row, chunks per
  // thread) is then chosen for the power-of-two bucket of chunk counts the row falls into, chunks are only
  // element-aligned and the last one of a row starts at COLS - V (the overlap is a run-time value), so that every row
  // length of the bucket shares the source and with it the code object.
  bool colsArg_ = false;
  bool allowColsArg_ = true;
  // ... and every row of every tensor that spans the row is a whole number of 64-byte pieces (hidden sizes usually are):
  // such row lengths have a source of their own, in which chunks never overlap, nothing is skipped in the reductions
  // and whole lines are streamed with the non-temporal hint, like in the kernel of a static description.
  bool colsWhole_ = false;
  // Dynamic descriptions with an operand that spans only some of the leading dimensions (an attention mask shared by
  // the heads): the leading extents of the folded iteration space are kernel arguments too, and the operand's row
  // offset is computed from them, so the source does not carry them as numbers.
  bool dimsArg_ = false;
  int64_t bucketLow_ = 0, bucketHigh_ = 0;
  std::vector<InputAccess> access_;  // per graph input
  std::vector<ValInfo> vals_;        // per tensor

  int vec_ = 1, tpr_ = 1, chunks_ = 1, rowsPerBlock_ = 1, block_ = 256;
  int64_t grid_ = 1;
  bool raggedCols_ = false, raggedRows_ = false, raggedFlat_ = false;
  int reduceCount_ = 0;
  // Some reduction is a float16 / bfloat16 sum or product: its steps run in index order, one thread per row folding
  // the row's LDS image (akg::chain_fold), so rows get few threads each and a workgroup many rows.
  bool ordered_ = false;
  // Rows too long to stay in registers: the row is walked in `groups_` groups of NCHUNK chunks per thread, once per
  // reduction of the fusion and once more for the outputs; every walk recomputes the element values it needs from
  // the kernel inputs (re-read from L2 / the last-level cache after the first walk).
  // Rows whose length is not a multiple of the chunk: chunks keep their full width (the accesses are then only
  // element-aligned, which the hardware serves), and the last chunk of a row starts at COLS - V, overlapping its
  // neighbour by overlap_ elements that reductions skip and that are stored twice with the same value.
  int overlap_ = 0;
  bool multiPass_ = false;
  // Walks over a row of 16-bit inputs that fits the registers in its memory image (half its float image): the row
  // is loaded once, kept packed, and every walk unpacks the group it works on.
  bool packedRow_ = false;
  std::vector<bool> packedInput_;          // per graph input: held packed in registers across the walks
  int64_t groups_ = 1;
  int pass_ = 0;                           // walk being emitted
  std::vector<int> lastPassOfInput_;       // per graph input: the last walk that reads it
  bool nonTemporal_ = true;
  bool useBuffers_ = true;
  std::vector<bool> relaxed_;
  // clamp + integer-cast peephole: ops skipped because a later Cast absorbs them, and what each such Cast computes
  struct ClampCast {
    int source = -1;
    double lo = 0.0, hi = 0.0;
  };
  std::vector<bool> absorbed_;            // per op
  std::vector<ClampCast> clampCast_;      // per op (source < 0: none)

  // ------------------------------------------------------------------ analysis
  void analyse() {
    for (const OpNode &op : g_.ops) {
      if (op.kind == OpKind::Unknown) {
        throw LoweringError("op " + op.name + " is not in the op table (mindspore.unknown cannot be legalized)");
      }
      if (op.kind == OpKind::Unsupported) {
        throw LoweringError("op " + op.name + " has no gfx950 kernel family yet");
      }
      if (op.kind == OpKind::MatMul) throw LoweringError("internal: MatMul reached the tile emitter");
      if (lowering::isReduceKind(op.kind)) {
        rowMode_ = true;
        ordered_ = ordered_ || lowering::reduceSpec(op, g_.tensor(op.outputs[0]).dtype).ordered;
      }
    }
    if (rowMode_) {
      analyseRowSpace();
    } else {
      analyseElementwiseSpace();
    }
  }

  void analyseRowSpace() {
    const OpNode *first = nullptr;
    for (const OpNode &op : g_.ops) {
      if (lowering::isReduceKind(op.kind)) {
        first = &op;
        break;
      }
    }
    std::vector<int64_t> space = g_.tensor(first->inputs[0]).shape;
    while (space.size() > 1 && space.front() == 1) space.erase(space.begin());
    if (space.empty() || space.back() <= 1) {
      throw LoweringError("reduction over an innermost axis of extent 1 is not supported");
    }
    const size_t r = space.size();
    for (const OpNode &op : g_.ops) {
      if (!lowering::isReduceKind(op.kind)) continue;
      const TensorValue &in = g_.tensor(op.inputs[0]);
      std::vector<int64_t> s = padShape(in.shape, r, "reduce operand " + in.name);
      if (s != space) {
        throw LoweringError("all reductions of one kernel must run over the same tensor shape");
      }
      // Real (extent > 1) reduced axes must be exactly the innermost axis: direction X.
      std::vector<int64_t> real;
      int64_t lead = static_cast<int64_t>(in.shape.size()) - static_cast<int64_t>(r);
      for (int64_t a : op.axes) {
        if (in.shape[static_cast<size_t>(a)] > 1) real.push_back(a - lead);
      }
      if (real.size() != 1 || real[0] != static_cast<int64_t>(r) - 1) {
        throw LoweringError("op " + op.name +
                            ": only reductions over the innermost axis (direction X) have a kernel family yet");
      }
    }
    full_ = space;
    cols_ = space.back();
    rows_ = product(space, 0, r - 1);
    numel_ = rows_ * cols_;
    access_.resize(g_.inputs.size());
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      const TensorValue &t = g_.tensor(g_.inputs[i]);
      // an input nothing reads takes no part in the iteration space
      std::vector<int64_t> s = padShape(t.used ? t.shape : std::vector<int64_t>{1}, r, "input " + t.name);
      for (size_t d = 0; d < r; ++d) {
        if (s[d] != 1 && s[d] != space[d]) {
          throw LoweringError("input " + t.name + " is not broadcast-compatible with the reduced tensor");
        }
      }
      access_[i].foldedShape = s;
      access_[i].lastDimFull = (s[r - 1] == cols_);
    }
  }

  void analyseElementwiseSpace() {
    std::vector<int64_t> space = g_.tensor(g_.outputs[0]).shape;
    for (int id : g_.outputs) {
      if (g_.tensor(id).shape != space) {
        throw LoweringError("all outputs of an elementwise kernel must have the same shape");
      }
    }
    const size_t r = space.size();
    std::vector<std::vector<int64_t>> padded;
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      const TensorValue &t = g_.tensor(g_.inputs[i]);
      std::vector<int64_t> s = padShape(t.used ? t.shape : std::vector<int64_t>{1}, r, "input " + t.name);
      for (size_t d = 0; d < r; ++d) {
        if (s[d] != 1 && s[d] != space[d]) {
          throw LoweringError("input " + t.name + " is not broadcast-compatible with the output shape");
        }
      }
      padded.push_back(s);
    }
    // Dimension folding (the role FoldDimension plays in the reference): drop unit dims, then merge adjacent
    // dims that every input either spans fully or broadcasts together.
    std::vector<size_t> keep;
    for (size_t d = 0; d < r; ++d) {
      if (space[d] != 1) keep.push_back(d);
    }
    std::vector<int64_t> folded;
    std::vector<std::vector<int64_t>> foldedIn(padded.size());
    auto status = [&](size_t input, size_t d) { return padded[input][d] == space[d]; };
    for (size_t k = 0; k < keep.size(); ++k) {
      size_t d = keep[k];
      bool merge = !folded.empty();
      if (merge) {
        size_t prev = keep[k - 1];
        for (size_t i = 0; i < padded.size(); ++i) {
          if (status(i, d) != status(i, prev)) {
            merge = false;
            break;
          }
        }
      }
      if (merge) {
        folded.back() *= space[d];
        for (size_t i = 0; i < padded.size(); ++i) foldedIn[i].back() *= padded[i][d];
      } else {
        folded.push_back(space[d]);
        for (size_t i = 0; i < padded.size(); ++i) foldedIn[i].push_back(padded[i][d]);
      }
    }
    if (folded.empty()) {
      folded.push_back(1);
      for (auto &f : foldedIn) f.push_back(1);
    }
    full_ = folded;
    cols_ = folded.back();
    rows_ = product(folded, 0, folded.size() - 1);
    numel_ = rows_ * cols_;
    access_.resize(g_.inputs.size());
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      access_[i].foldedShape = foldedIn[i];
      access_[i].lastDimFull = (foldedIn[i].back() == cols_);
    }
  }

  // ------------------------------------------------------------------ schedule
  void pickSchedule() {
    extentArg_ = opt_.extentAsArgument;
    extentIsCols_ = extentArg_ && !rowMode_ && rows_ == 1;
    dimsArg_ = false;
    if (extentArg_ && !extentIsCols_ && full_.size() >= 3 && rows_ < (1LL << 31)) {
      for (const InputAccess &a : access_) {
        if (a.foldedShape.size() != full_.size()) continue;
        bool allFull = true, allOne = true;
        for (size_t d = 0; d + 1 < full_.size(); ++d) {
          allFull = allFull && a.foldedShape[d] == full_[d];
          allOne = allOne && a.foldedShape[d] == 1;
        }
        dimsArg_ = dimsArg_ || (!allFull && !allOne);
      }
    }
    useBuffers_ = true;
    for (int id : g_.inputs) {
      if (g_.tensor(id).numel() * static_cast<int64_t>(dtypeSize(g_.tensor(id).dtype)) >= (1LL << 31)) useBuffers_ = false;
    }
    for (int id : g_.outputs) {
      if (g_.tensor(id).numel() * static_cast<int64_t>(dtypeSize(g_.tensor(id).dtype)) >= (1LL << 31)) useBuffers_ = false;
    }
    // Chunk width: 16 bytes of the widest element type that is moved chunk-wise, so no tensor needs more than one
    // 128-bit access per chunk (narrower tensors use 64- or 32-bit accesses, which still coalesce fully). Measured
    // on MI355X: many small contiguous accesses per wave beat fewer, wider ones.
    size_t minSize = 1, narrowest = 16;
    bool any = false;
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      if (!access_[i].lastDimFull) continue;
      minSize = std::max(minSize, dtypeSize(g_.tensor(g_.inputs[i]).dtype));
      narrowest = std::min(narrowest, dtypeSize(g_.tensor(g_.inputs[i]).dtype));
      any = true;
    }
    for (int id : g_.outputs) {
      if (rowMode_ && g_.tensor(id).numel() != numel_) continue;
      minSize = std::max(minSize, dtypeSize(g_.tensor(id).dtype));
      narrowest = std::min(narrowest, dtypeSize(g_.tensor(id).dtype));
      any = true;
    }
    if (!any) minSize = 4;
    int v = opt_.vec > 0 ? opt_.vec : static_cast<int>(16 / minSize);
    v = std::max(1, std::min(v, 16));
    if ((v & (v - 1)) != 0) v = 1;
    bool inPlace = false;
    for (const OpNode &op : g_.ops) inPlace = inPlace || op.kind == OpKind::Assign;
    // the row length as an argument: row kernels whose rows hold at least two chunks (tried first, given up below if the
    // bucket's longest row would not stay in registers), elementwise kernels with a row structure
    colsArg_ = allowColsArg_ && extentArg_ && !extentIsCols_ && useBuffers_ && opt_.vec == 0 && opt_.threadsPerRow == 0 && opt_.chunks == 0 &&
               (rowMode_ ? (!inPlace && cols_ >= 2 * v) : rows_ > 1);
    int64_t schedCols = cols_;   // the row length the schedule is made for
    if (colsArg_ && rowMode_) {
      const int64_t bucketChunks = pow2AtLeast(static_cast<int>(std::min<int64_t>(ceilDiv(cols_, v), 1 << 20)));
      bucketHigh_ = bucketChunks * v;
      bucketLow_ = std::max<int64_t>(2 * v, bucketChunks / 2 * v + 1);
      schedCols = bucketHigh_;
    }
    colsWhole_ = colsArg_ && rowMode_ && any && (cols_ * static_cast<int64_t>(narrowest)) % 64 == 0;
    if (colsArg_ && rowMode_) {
      // element-aligned chunks; the overlap of the last one is computed in the kernel (none when rows are whole lines)
    } else if (rowMode_ && useBuffers_ && !inPlace && opt_.vec == 0 && (cols_ % v) != 0 && cols_ >= 2 * v) {
      overlap_ = static_cast<int>(v - cols_ % v);
    } else {
      while (v > 1 && (cols_ % v) != 0) v >>= 1;
    }
    vec_ = v;

    if (rowMode_) {
      // One row per group of tpr threads: one 16-byte chunk (8 elements of a 16-bit type) per thread, at most 1024
      // threads per row (wider rows get more chunks per thread instead). Measured on MI355X: 8192-wide bf16 rows
      // 79.5 % of the HBM peak with 1024 threads per row against 75.8 % with 512; 4096-wide f16 rows 75.0 % with 512
      // against 73.9 % with 256; 4096-wide bf16 rows with two streamed inputs the same either way. The row stays in
      // registers across all reductions of the fusion.
      // Threads per row must be a power of two (butterfly reductions). Among the (threads, chunks per thread) pairs
      // with at least 8 elements and at most 8 chunks per thread, the one that leaves the fewest idle chunk slots
      // wins; between pairs within 3 % of each other the one with fewer chunks per thread. Measured on MI355X
      // (% of the HBM peak): 4096-wide f16 rows 512 x 1 75.0, 256 x 2 73.9; 8192-wide bf16 rows 1024 x 1 79.5,
      // 512 x 2 75.8; 4096-wide f32 rows 512 x 2 78.4, 1024 x 1 69.0; 768-wide bf16 LayerNorm 32 x 3 80.5, 128 x 1
      // (25 % idle) 60.3; 5120-wide 128 x 5 78.7, 1024 x 1 (37 % idle) 50.3; 11008-wide f32 softmax 1024 x 3 72.6,
      // 256 x 11 68.2.
      const int64_t rowChunks = ceilDiv(schedCols, vec_);
      int tpr = 0;
      if (opt_.threadsPerRow > 0) {
        tpr = pow2AtLeast(std::max(1, std::min(opt_.threadsPerRow, 1024)));
      } else {
        const int64_t minChunks = std::max(1, 8 / vec_);
        double best = 0;
        for (int t = 1024; t >= 1; t >>= 1) {
          const int64_t c = ceilDiv(rowChunks, t);
          if (c < minChunks && t > 1) continue;
          if (c > 8 && tpr != 0) break;
          const double slots = static_cast<double>(t) * static_cast<double>(c) / static_cast<double>(rowChunks);
          // candidates come with growing chunks per thread: a later one must be clearly better to win
          if (tpr == 0 || slots < best / 1.03) {
            tpr = t;
            best = slots;
          }
        }
      }
      if (opt_.threadsPerRow == 0 && tpr == 1024 && rowChunks > 512 && rowChunks <= 1024) {
        // One chunk per thread on 1024 threads against two on 512: with two row-sized inputs the 1024 win or draw (the
        // quantisation 79.5 against 75.8 % of the HBM peak, RMSNorm + residual and a masked softmax the same either
        // way), with one input the 512 win: 8192-wide f16 softmax 171.0 -> 165.7 us, bf16 RMSNorm 180.1 -> 172.9 us
        // (32768 rows).
        int64_t rowSized = 0;
        for (size_t i = 0; i < g_.inputs.size(); ++i) {
          if (access_[i].lastDimFull && g_.tensor(g_.inputs[i]).numel() == numel_) ++rowSized;
        }
        if (rowSized <= 1) tpr = 512;
      }
      if (opt_.threadsPerRow == 0 && !ordered_ && normalisationLike() && rowChunks >= 128 && rowChunks <= 2048) {
        // A reduction that waits for another one (mean, then variance) with per-column operands behind them (gamma,
        // beta): LayerNorm. Four to eight chunks per thread on at most 256 threads beat one chunk on many threads
        // there - two workgroup-wide reductions per row are cheap on four wavefronts, and every thread keeps four
        // times the bytes in flight. Measured, bf16 with a residual, 64 M elements, default -> this rule: 2048-wide
        // 64.2 -> 61.5 us, 4096 (C3) 65.2 -> 63.1, 8192 70.5 -> 65.1, 16384 80.2 -> 69.0; without the residual 8192-wide
        // 57.3 -> 48.5. (Softmax, RMSNorm, the quantisation and a LayerNorm of three summed inputs without gamma and
        // beta keep the rule above: they lose 1 ... 6 % this way.)
        // (of 64, 128 and 256 threads with at most 8 chunks each: the fewest idle chunk slots, then nearest to four chunks)
        double bestSlots = 0;
        int64_t bestChunks = 0;
        for (int t = 64; t <= 256; t <<= 1) {
          const int64_t c = ceilDiv(rowChunks, t);
          if (c > 8) continue;
          const double slots = static_cast<double>(t) * static_cast<double>(c) / static_cast<double>(rowChunks);
          const bool fewerIdle = bestChunks == 0 || slots < bestSlots / 1.03;
          const bool sameIdle = bestChunks != 0 && slots <= bestSlots * 1.03 && slots >= bestSlots / 1.03;
          if (fewerIdle || (sameIdle && std::llabs(c - 4) < std::llabs(bestChunks - 4))) {
            tpr = t;
            bestSlots = slots;
            bestChunks = c;
          }
        }
      }
      if (opt_.threadsPerRow == 0 && !ordered_ && rowChunks > 2048 && rowChunks <= 4096 && normalisationLike()) {
        tpr = 512;   // (32768-wide bf16 LayerNorm + residual: 74.9 -> 71.0 us; 65536-wide stays on 1024 threads)
      }
      if (ordered_ && opt_.threadsPerRow == 0) {
        // one thread folds a row while the row's other threads wait: as few threads per row as keep it in registers
        for (int t = 1; t <= 1024; t <<= 1) {
          tpr = t;
          if (ceilDiv(rowChunks, t) <= 8) break;
        }
      }
      tpr_ = tpr;
      int64_t perThread = ceilDiv(schedCols, static_cast<int64_t>(tpr_) * vec_);
      // More than 64 values per thread of one row-sized input, or 96 over all of them, do not stay in registers: walk the row in groups of
      // `chunks` chunks per thread instead. The walks after the first re-read the row from HBM (rows in flight exceed
      // L2), so the register-resident row is kept as long as it fits. Measured, % of the HBM peak, resident / walks:
      // 65536-wide f16 softmax (1 input, 64 values) 62.6 / 46.2; 65536-wide bf16 LayerNorm (2 inputs) 21.9 / 61.3;
      // 32768-wide LayerNorm 70.2 / 63.2; 131072-wide LayerNorm 10.6 / 50.0, softmax 30.1 / 42.3.
      const int rowPasses = opt_.variant;  // 1: force the register-resident row, 2: force the walks, 4: walks, packed if possible
      int64_t rowInputs = 0;
      for (size_t i = 0; i < g_.inputs.size(); ++i) {
        if (access_[i].lastDimFull && g_.tensor(g_.inputs[i]).numel() == numel_) ++rowInputs;
      }
      multiPass_ = rowPasses == 2 || rowPasses == 4 || (rowPasses != 1 && (perThread * vec_ > 64 || perThread * vec_ * rowInputs > 96));
      packedInput_.assign(g_.inputs.size(), false);
      // Measured, % of the HBM peak, float values resident / packed walks: 32768-wide bf16 quantisation 61.6 / 73.0,
      // 32768-wide f16 softmax 67.8 / 70.0, 65536-wide 62.1 / 66.4, 32768-wide LayerNorm 69.6 / 67.4; at 16384 and
      // below the same within a point or two. So rows of 16-bit inputs on 1024 threads go packed from 64 values per
      // thread on.
      // (a single row-sized input goes packed from 32 values per thread on: 32768-wide f16 softmax 49.1 -> 47.9 us,
      // bf16 RMSNorm 49.1 -> 46.4 us; at 16 values the float row is ahead or level)
      const bool preferPacked = rowPasses == 0 && tpr_ == 1024 &&
                                (perThread * vec_ * rowInputs >= 64 || (rowInputs == 1 && perThread * vec_ >= 32));
      if ((multiPass_ || preferPacked) && useBuffers_ && rowPasses != 2) {
        // registers (32-bit) per thread for the packed row; 64 leave room for one group's float values
        int64_t packedRegs = 0;
        bool narrowOnly = true;
        for (size_t i = 0; i < g_.inputs.size(); ++i) {
          const TensorValue &t = g_.tensor(g_.inputs[i]);
          if (!(access_[i].lastDimFull && t.numel() == numel_)) continue;
          if (dtypeSize(t.dtype) > 2) narrowOnly = false;
          packedRegs += perThread * ((vec_ * static_cast<int64_t>(dtypeSize(t.dtype)) + 3) / 4);
        }
        if (narrowOnly && packedRegs > 0 && packedRegs <= 64) {
          packedRow_ = true;
          multiPass_ = true;
          for (size_t i = 0; i < g_.inputs.size(); ++i) {
            packedInput_[i] = access_[i].lastDimFull && g_.tensor(g_.inputs[i]).numel() == numel_;
          }
        }
      }
      if (colsArg_ && (multiPass_ || packedRow_)) {
        // rows of this bucket do not stay in registers: the walked kernels are made per row length
        colsArg_ = allowColsArg_ = false;
        multiPass_ = packedRow_ = false;
        packedInput_.clear();
        pickSchedule();
        return;
      }
      if (multiPass_) {
        const int64_t perGroup = opt_.chunks > 0 ? opt_.chunks : std::max<int64_t>(1, (packedRow_ ? 16 : 32) / vec_);
        chunks_ = static_cast<int>(std::min<int64_t>(perGroup, perThread));
        groups_ = ceilDiv(perThread, chunks_);
      } else {
        if (perThread * vec_ > 256) {
          throw LoweringError("row of " + std::to_string(cols_) + " elements does not fit the register-resident row kernel");
        }
        chunks_ = static_cast<int>(perThread);
        groups_ = 1;
      }
      block_ = opt_.block > 0 ? opt_.block : 256;
      block_ = std::max(block_, tpr_);
      block_ = std::min(block_, 1024);
      if (block_ % tpr_ != 0 || block_ % 64 != 0) block_ = std::max(tpr_, 64);
      rowsPerBlock_ = block_ / tpr_;
      grid_ = ceilDiv(rows_, rowsPerBlock_);
      raggedCols_ = colsArg_ || (groups_ * chunks_ * tpr_ != rowChunks);
      raggedRows_ = (rows_ % rowsPerBlock_) != 0 || extentArg_;
    } else {
      block_ = opt_.block > 0 ? opt_.block : 256;
      if (block_ % 64 != 0 || block_ > 1024) block_ = 256;
      int chunks = opt_.chunks > 0 ? opt_.chunks : std::max(1, 16 / vec_);
      // An operand that is broadcast over the iteration space (a bias per column, a scale per row) is loaded again
      // for every chunk of a thread, and those chunks lie a whole workgroup's width apart: one chunk per thread then
      // (bias + activation on 64 M bf16 elements 43.6 -> 41.9 us, on 16 M float32 elements 23.6 -> 22.2 us).
      if (opt_.chunks == 0) {
        for (size_t i = 0; i < g_.inputs.size(); ++i) {
          const TensorValue &t = g_.tensor(g_.inputs[i]);
          if (t.used && t.numel() > 1 && t.numel() != numel_) chunks = 1;
        }
      }
      // Small problems: fewer chunks per thread so the grid still covers the chip.
      if (extentArg_ && opt_.chunks == 0) {
        // a dynamic description: two sizes only (the source must not follow every element count)
        if (ceilDiv(numel_, static_cast<int64_t>(block_) * vec_ * chunks) < 1024) chunks = 1;
      } else {
        while (chunks > 1 && ceilDiv(numel_, static_cast<int64_t>(block_) * vec_ * chunks) < 1024) chunks >>= 1;
      }
      chunks_ = std::max(1, chunks);
      tpr_ = block_;
      rowsPerBlock_ = 1;
      int64_t perBlock = static_cast<int64_t>(block_) * vec_ * chunks_;
      grid_ = std::max<int64_t>(1, ceilDiv(numel_, perBlock));
      raggedFlat_ = (numel_ % perBlock) != 0 || extentArg_;
    }
    if (grid_ > 2147483647LL) throw LoweringError("grid too large");
  }

  // ------------------------------------------------------------------ peepholes
  // Cast_to_int8/int16(Minimum(Maximum(x, c0), c1)) (either order) with constant bounds and single-use intermediates
  // becomes one clamp_cast: 5 vector instructions instead of 11 on the per-token quantisation path.
  void planPeepholes() {
    absorbed_.assign(g_.ops.size(), false);
    clampCast_.assign(g_.ops.size(), ClampCast());
    std::vector<int> uses(g_.tensors.size(), 0);
    for (const OpNode &op : g_.ops) {
      for (int in : op.inputs) ++uses[static_cast<size_t>(in)];
    }
    auto constOperand = [&](const OpNode &op, int *other, double *value) {
      if (op.inputs.size() != 2) return false;
      for (int side = 0; side < 2; ++side) {
        const TensorValue &c = g_.tensor(op.inputs[static_cast<size_t>(side)]);
        if (c.isConst && c.dtype == DType::F32) {
          *other = op.inputs[static_cast<size_t>(1 - side)];
          *value = static_cast<double>(static_cast<float>(c.constValue));
          return true;
        }
      }
      return false;
    };
    auto fusable = [&](int tensorId) {
      const TensorValue &t = g_.tensor(tensorId);
      return t.producer >= 0 && t.outputIndex < 0 && uses[static_cast<size_t>(tensorId)] == 1 && t.dtype == DType::F32;
    };
    for (size_t k = 0; k < g_.ops.size(); ++k) {
      const OpNode &cast = g_.ops[k];
      if (cast.kind != OpKind::Cast || cast.inputs.size() != 1) continue;
      const DType od = g_.tensor(cast.outputs[0]).dtype;
      if (od != DType::I8 && od != DType::I16) continue;
      const int t1 = cast.inputs[0];
      if (!fusable(t1)) continue;
      const OpNode &p1 = g_.ops[static_cast<size_t>(g_.tensor(t1).producer)];
      if (p1.kind != OpKind::Minimum && p1.kind != OpKind::Maximum) continue;
      int t0 = -1, x = -1;
      double c1 = 0.0, c0 = 0.0;
      if (!constOperand(p1, &t0, &c1) || !fusable(t0)) continue;
      const OpNode &p0 = g_.ops[static_cast<size_t>(g_.tensor(t0).producer)];
      if ((p0.kind != OpKind::Minimum && p0.kind != OpKind::Maximum) || p0.kind == p1.kind) continue;
      if (!constOperand(p0, &x, &c0)) continue;
      if (g_.tensor(x).dtype != DType::F32 || c0 != c0 || c1 != c1) continue;
      double lo = (p0.kind == OpKind::Maximum) ? c0 : c1;
      double hi = (p0.kind == OpKind::Minimum) ? c0 : c1;
      if (lo > hi) continue;  // min(max(x, lo), hi) and max(min(x, hi), lo) differ then: leave it alone
      const double tlo = (od == DType::I8) ? -128.0 : -32768.0;
      const double thi = (od == DType::I8) ? 127.0 : 32767.0;
      lo = std::max(std::nearbyint(lo), tlo);
      hi = std::min(std::nearbyint(hi), thi);
      if (lo > hi) continue;
      absorbed_[static_cast<size_t>(g_.tensor(t1).producer)] = true;
      absorbed_[static_cast<size_t>(g_.tensor(t0).producer)] = true;
      clampCast_[k].source = x;
      clampCast_[k].lo = lo;
      clampCast_[k].hi = hi;
    }
  }

  // ------------------------------------------------------------------ emission helpers
  std::string ctOf(int tensorId) const { return computeTypeName(g_.tensor(tensorId).dtype); }
  std::string tagOf(int tensorId) const { return dtypeTag(g_.tensor(tensorId).dtype); }

  std::string operandExpr(int tensorId) const {
    const ValInfo &v = vals_[static_cast<size_t>(tensorId)];
    if (!v.defined) throw LoweringError("internal: operand " + g_.tensor(tensorId).name + " used before definition");
    if (v.rank == ValRank::Tile) return v.ident + "[j][e]";
    return v.ident;
  }

  void line(const std::string &s) { src_ << s << "\n"; }

  // Memory operand of argument `arg` ("in0", "out1", ...) at element offset `offset`: a buffer descriptor plus
  // offset when every tensor of the kernel is below 2 GiB, a plain pointer otherwise.
  std::string memRef(const std::string &arg, const std::string &offset) const {
    if (useBuffers_) return "b_" + arg + ", " + offset;
    return arg + " + " + offset;
  }
  // The chunks' conditions are run-time values (ragged rows or tails, extents that are arguments) and the tensors are
  // addressed through descriptors: accesses take their condition as an operand instead of standing behind a branch.
  bool conditionalAccesses() const { return useBuffers_ && (rowMode_ ? raggedCols_ : raggedFlat_); }

  // Offset of the first element of `row` for an input, as an expression in `rowVar`.
  std::string rowOffsetExpr(const InputAccess &a, const std::string &rowVar) const {
    const std::vector<int64_t> &s = a.foldedShape;
    const size_t r = full_.size();
    bool allFull = true, allOne = true;
    for (size_t d = 0; d + 1 < r; ++d) {
      if (s[d] != full_[d]) allFull = false;
      if (s[d] != 1) allOne = false;
    }
    if (r == 1 || allOne) return "0L";
    // the innermost extent of the operand: a number, or the kernel argument when the row length is one
    const bool symbolic = colsArg_ && s[r - 1] == cols_ && cols_ != 1;
    const std::string inner = symbolic ? std::string("COLS") : std::to_string(s[r - 1]) + "L";
    if (allFull) return "(" + rowVar + " * " + inner + ")";
    if (dimsArg_) {
      // the same decomposition with the leading extents as kernel arguments (32-bit arithmetic: ROWS is below 2^31)
      std::ostringstream e;
      std::string div;          // product of the extents inside dim d, as an expression ("" = 1)
      std::string own;          // product of the operand's own extents inside dim d
      bool firstTerm = true;
      for (int d = static_cast<int>(r) - 2; d >= 0; --d) {
        const std::string dim = "akg_dim" + std::to_string(d);
        if (s[static_cast<size_t>(d)] != 1) {
          if (!firstTerm) e << " + ";
          std::string idx = div.empty() ? "static_cast<unsigned>(" + rowVar + ")" : "(static_cast<unsigned>(" + rowVar + ") / (" + div + "))";
          if (d > 0) idx = "(" + idx + " % " + dim + ")";
          e << "static_cast<long>(" << idx << ")" << (own.empty() ? "" : " * static_cast<long>(" + own + ")");
          firstTerm = false;
          own = own.empty() ? dim : own + " * " + dim;
        }
        div = div.empty() ? dim : div + " * " + dim;
      }
      if (firstTerm) return "0L";
      return "((" + e.str() + ") * " + inner + ")";
    }
    // general leading-dim broadcast: decompose the row index over the leading dims
    std::vector<int64_t> stride(r, 0);
    int64_t acc = symbolic ? 1 : s[r - 1];
    for (int d = static_cast<int>(r) - 2; d >= 0; --d) {
      stride[static_cast<size_t>(d)] = (s[static_cast<size_t>(d)] == 1) ? 0 : acc;
      acc *= s[static_cast<size_t>(d)];
    }
    // emitted as a sum of ((row / inner_extent) % extent) * stride terms
    std::ostringstream e;
    int64_t div = 1;
    bool firstTerm = true;
    for (int d = static_cast<int>(r) - 2; d >= 0; --d) {
      int64_t extent = full_[static_cast<size_t>(d)];
      if (stride[static_cast<size_t>(d)] != 0) {
        if (!firstTerm) e << " + ";
        e << "((" << rowVar << " / " << div << "L) % " << extent << "L) * " << stride[static_cast<size_t>(d)] << "L";
        firstTerm = false;
      }
      div *= extent;
    }
    if (firstTerm) return "0L";
    if (symbolic) return "((" + e.str() + ") * COLS)";
    return "(" + e.str() + ")";
  }

  // ------------------------------------------------------------------ emission
  void emit() {
    vals_.assign(g_.tensors.size(), ValInfo());
    relaxed_ = lowering::relaxedPrecisionTensors(g_);
    planPeepholes();
    const std::string kname = g_.name + "_kernel";

    line("// Generated by the akg HIP lowering for gfx950. Op description: " + g_.name);
    line("// family: " + std::string(rowMode_ ? "row_reduce" : "elementwise") + ", fusion class: " +
         operatorTemplateName(g_.operatorTemplate));
    line("#include \"akg_rt.hpp\"");
    line("");
    src_ << "extern \"C\" __global__ __launch_bounds__(" << block_ << ") void " << kname << "(";
    size_t argc = 0;
    std::vector<bool> assigned(g_.inputs.size(), false);
    for (const OpNode &op : g_.ops) {
      if (op.kind == OpKind::Assign) assigned[static_cast<size_t>(g_.tensor(op.inputs[0]).inputIndex)] = true;
    }
    for (size_t i = 0; i < g_.inputs.size(); ++i, ++argc) {
      src_ << (argc ? ", " : "") << (assigned[i] ? "" : "const ") << tagOf(g_.inputs[i]) << "::storage *__restrict__ in" << i;
    }
    for (size_t i = 0; i < g_.outputs.size(); ++i, ++argc) {
      src_ << (argc ? ", " : "") << tagOf(g_.outputs[i]) << "::storage *__restrict__ out" << i;
    }
    if (extentArg_) src_ << ", const long akg_extent";
    if (colsArg_) src_ << ", const long akg_cols_arg";
    if (dimsArg_) {
      for (size_t d = 0; d + 1 < full_.size(); ++d) src_ << ", const long akg_dim_arg" << d;
    }
    line(") {");
    if (dimsArg_) {
      for (size_t d = 0; d + 1 < full_.size(); ++d) {
        src_ << "  const unsigned akg_dim" << d << " = static_cast<unsigned>(akg_dim_arg" << d << ");   // leading extent " << d << " of the iteration space\n";
      }
    }
    if (extentArg_ && extentIsCols_) {
      line("  constexpr long ROWS = 1L;");
      line("  const long COLS = akg_extent;   // everything folds into one dimension: the element count");
    } else if (extentArg_ && colsArg_) {
      line("  const long COLS = akg_cols_arg;   // the row length (innermost extent)");
      line("  const long ROWS = akg_extent;   // product of the leading dimensions");
    } else if (extentArg_) {
      src_ << "  constexpr long COLS = " << cols_ << "L;\n";
      line("  const long ROWS = akg_extent;   // product of the leading dimensions");
    } else {
      src_ << "  constexpr long COLS = " << cols_ << "L;\n";
      src_ << "  constexpr long ROWS = " << rows_ << "L;\n";
    }
    if (useBuffers_) {
      for (size_t i = 0; i < g_.inputs.size(); ++i) {
        const TensorValue &t = g_.tensor(g_.inputs[i]);
        src_ << "  const akg::Buffer b_in" << i << " = akg::make_buffer(in" << i << ", "
             << bytesExpr(access_[i].foldedShape, t) << ");\n";
      }
      for (size_t i = 0; i < g_.outputs.size(); ++i) {
        const TensorValue &t = g_.tensor(g_.outputs[i]);
        std::vector<int64_t> folded = full_;
        if (t.numel() != numel_) folded.back() = 1;   // one value per row
        src_ << "  const akg::Buffer b_out" << i << " = akg::make_buffer(out" << i << ", " << bytesExpr(folded, t) << ");\n";
      }
    }
    src_ << "  constexpr int V = " << vec_ << ";\n";
    src_ << "  constexpr int NCHUNK = " << chunks_ << ";\n";
    src_ << "  constexpr int BLOCK = " << block_ << ";\n";
    line("  const int tid = static_cast<int>(threadIdx.x);");
    if (rowMode_) {
      src_ << "  constexpr int TPR = " << tpr_ << ";\n";
      src_ << "  constexpr int RPB = " << rowsPerBlock_ << ";\n";
      line("  const int tcol = tid % TPR;");
      // Launch order is kept even where rows share cache lines with their neighbours: giving every XCD a contiguous
      // range of rows was measured slower (1000-wide f16 softmax 73.1 -> 67.8 % of the HBM peak, 4095-wide 63.0 -> 59.9).
      line("  const int akg_wg = static_cast<int>(blockIdx.x);");
      line("  const long akg_row_raw = static_cast<long>(akg_wg) * RPB + (tid / TPR);");
      if (raggedRows_) {
        line("  const bool akg_row_ok = akg_row_raw < ROWS;");
        line("  const long akg_row = akg_row_ok ? akg_row_raw : (ROWS - 1);");
      } else {
        line("  const long akg_row = akg_row_raw;");
      }
      if (tpr_ > 64) {
        line("  __shared__ double akg_scratch[2][BLOCK / 64];");
      }
      if (ordered_) {
        // the part of every row of the workgroup that is being folded, in its 16-bit type (rows 16 bytes apart in the banks)
        line("  constexpr int CHAIN_PITCH = NCHUNK * TPR * V + 8;");
        line("  __shared__ __attribute__((aligned(16))) unsigned short akg_chain[RPB][CHAIN_PITCH];");
        line("  __shared__ float akg_chain_res[RPB];");
      }
      line("  long akg_rows[NCHUNK];");
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) akg_rows[j] = akg_row;");
      if (multiPass_) {
        src_ << "  constexpr int GROUPS = " << groups_ << ";\n";
      } else {
        if (colsArg_ && !colsWhole_) line("  const int akg_overlap = static_cast<int>((V - COLS % V) % V);   // elements the last chunk of a row shares with its neighbour");
        emitColumnsOfGroup("0");
      }
    } else {
      line("  const long NUMEL = ROWS * COLS;");
      line("  const long akg_base = static_cast<long>(blockIdx.x) * (static_cast<long>(BLOCK) * V * NCHUNK);");
      line("  long akg_rows[NCHUNK];");
      line("  long akg_cols[NCHUNK];");
      line("  long akg_flat[NCHUNK];");
      line("  bool akg_ok[NCHUNK];");
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) {");
      line("    const long i = akg_base + (static_cast<long>(j) * BLOCK + tid) * V;");
      line(std::string("    akg_ok[j] = ") + (raggedFlat_ ? "i < NUMEL;" : "true;"));
      line("    const long ic = akg_ok[j] ? i : 0L;");
      line("    akg_flat[j] = ic;");
      if (rows_ == 1) {
        line("    akg_rows[j] = 0L;");
        line("    akg_cols[j] = ic;");
      } else {
        line("    akg_rows[j] = ic / COLS;");
        line("    akg_cols[j] = ic % COLS;");
      }
      line("  }");
    }
    line("");

    // constants
    for (size_t t = 0; t < g_.tensors.size(); ++t) {
      const TensorValue &tv = g_.tensors[t];
      if (!tv.isConst) continue;
      ValInfo &v = vals_[t];
      v.defined = true;
      v.rank = ValRank::Const;
      v.ident = lowering::literalFor(tv.dtype, tv.constValue);
    }
    if (multiPass_) {
      emitWalks();
      line("}");
      return;
    }
    // loads of kernel inputs
    for (size_t i = 0; i < g_.inputs.size(); ++i) emitInputLoad(i);
    // ops in description order
    for (size_t k = 0; k < g_.ops.size(); ++k) {
      const OpNode &op = g_.ops[k];
      if (absorbed_[k]) continue;
      if (lowering::isReduceKind(op.kind)) {
        emitReduceAccumulator(op);
        emitReduceAccumulate(op);
        emitReduceFinish(op);
      } else {
        emitElementwise(op, clampCast_[k]);
      }
    }
    // stores: the outputs, then the destinations of Assign ops (every thread has read its part of a destination
    // into registers above, and writes exactly the positions it read)
    for (size_t i = 0; i < g_.outputs.size(); ++i) emitOutputStore(i);
    for (const OpNode &op : g_.ops) {
      if (op.kind == OpKind::Assign) emitAssignStore(op);
    }
    line("}");
  }

  // Size in bytes of a tensor with the given shape in the (folded) iteration space, as a C expression: a number, or,
  // when the extent is a kernel argument, a multiple of it for tensors that span all leading dimensions (or the one
  // folded dimension). A tensor that spans only some of the leading dimensions keeps its number: such a source is
  // specific to the shape set, which is correct, just not shared.
  std::string bytesExpr(const std::vector<int64_t> &folded, const TensorValue &t) const {
    const int64_t bytes = t.numel() * static_cast<int64_t>(dtypeSize(t.dtype));
    const std::string number = std::to_string(bytes) + "L";
    if (!extentArg_ || folded.size() != full_.size()) return number;
    if (extentIsCols_) {
      return folded.back() == cols_ ? "akg_extent * " + std::to_string(dtypeSize(t.dtype)) + "L" : number;
    }
    bool leadFull = true, leadOne = true;
    for (size_t d = 0; d + 1 < folded.size(); ++d) {
      if (folded[d] != full_[d]) leadFull = false;
      if (folded[d] != 1) leadOne = false;
    }
    const bool symbolicCols = colsArg_ && folded.back() == cols_ && cols_ != 1;
    if (leadOne && rows_ != 1) return symbolicCols ? "COLS * " + std::to_string(dtypeSize(t.dtype)) + "L" : number;
    if (!leadFull && dimsArg_) {
      std::string e = symbolicCols ? std::string("COLS") : std::to_string(folded.back()) + "L";
      for (size_t d = 0; d + 1 < folded.size(); ++d) {
        if (folded[d] != 1) e += " * static_cast<long>(akg_dim" + std::to_string(d) + ")";
      }
      return e + " * " + std::to_string(dtypeSize(t.dtype)) + "L";
    }
    if (!leadFull) return number;
    if (symbolicCols) return "akg_extent * COLS * " + std::to_string(dtypeSize(t.dtype)) + "L";
    return "akg_extent * " + std::to_string(folded.back() * static_cast<int64_t>(dtypeSize(t.dtype))) + "L";
  }

  // Non-temporal accesses pay off when a workgroup moves whole cache lines. Rows of a row kernel that are not a
  // multiple of 64 bytes share their first and last line with the neighbouring rows, which other workgroups move:
  // with the hint such a line is dropped before the neighbour comes for it (measured on 1000-wide bf16 rows:
  // LayerNorm 62.8 % of the HBM peak with the hint, 68.4 % without; int8 quantisation 58.9 % and 66.9 %).
  bool streamsWholeLines(int tensorId) const {
    if (!nonTemporal_) return false;
    if (!rowMode_) return true;
    if (colsArg_ && !colsWhole_) return false;   // rows of any length: their first and last cache lines may be shared with neighbours
    const int64_t rowBytes = cols_ * static_cast<int64_t>(dtypeSize(g_.tensor(tensorId).dtype));
    return rowBytes % 64 == 0 || rowBytes >= 16384;  // two shared lines in 256 or more do not matter
  }

  // Column of every chunk of the thread in group `group` of the row (an expression; "0" for the only group).
  void emitColumnsOfGroup(const std::string &group) {
    line("  long akg_cols[NCHUNK];");
    line("  bool akg_ok[NCHUNK];");
    const bool tails = overlap_ > 0 || (colsArg_ && rowMode_ && !colsWhole_);
    if (tails) line("  bool akg_tail[NCHUNK];");
    line("#pragma unroll");
    line("  for (int j = 0; j < NCHUNK; ++j) {");
    line("    akg_cols[j] = ((static_cast<long>(" + group + ") * NCHUNK + j) * TPR + tcol) * V;");
    line(std::string("    akg_ok[j] = ") + (raggedCols_ ? "akg_cols[j] < COLS;" : "true;"));
    if (tails) {
      line("    akg_tail[j] = akg_cols[j] > COLS - V;");
      line("    if (akg_tail[j]) akg_cols[j] = COLS - V;");
    }
    line("  }");
  }

  // Two reductions of which one waits for the other, and some per-column operand (an input that spans the row but not
  // the rows): the shape of a LayerNorm.
  bool normalisationLike() const {
    std::vector<int> level(g_.tensors.size(), 0);
    int deepest = 0;
    for (const OpNode &op : g_.ops) {
      int lv = 0;
      for (int in : op.inputs) lv = std::max(lv, level[static_cast<size_t>(in)]);
      if (lowering::isReduceKind(op.kind)) ++lv;
      for (int out : op.outputs) level[static_cast<size_t>(out)] = lv;
      deepest = std::max(deepest, lv);
    }
    bool perColumn = false;
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      const TensorValue &t = g_.tensor(g_.inputs[i]);
      perColumn = perColumn || (t.used && access_[i].lastDimFull && t.numel() == cols_ && rows_ > 1);
    }
    return deepest >= 2 && perColumn;
  }

  // Would the value be a per-element (Tile) value? Inputs that span the row are, and whatever is computed from one.
  std::vector<bool> tileRanks() const {
    std::vector<bool> tile(g_.tensors.size(), false);
    for (size_t i = 0; i < g_.inputs.size(); ++i) tile[static_cast<size_t>(g_.inputs[i])] = access_[i].lastDimFull;
    for (size_t k = 0; k < g_.ops.size(); ++k) {
      const OpNode &op = g_.ops[k];
      if (lowering::isReduceKind(op.kind)) continue;
      bool any = op.kind == OpKind::Iota;
      for (int in : operandsOf(k)) any = any || tile[static_cast<size_t>(in)];
      for (int out : op.outputs) tile[static_cast<size_t>(out)] = any;
    }
    return tile;
  }

  // Operands an op really reads (a Cast that absorbed its clamp reads the clamp's source).
  std::vector<int> operandsOf(size_t k) const {
    std::vector<int> in = g_.ops[k].inputs;
    if (clampCast_[k].source >= 0) in[0] = clampCast_[k].source;
    return in;
  }

  struct Walk {
    std::vector<bool> ops;     // per op: recomputed in this walk
    std::vector<bool> inputs;  // per graph input: loaded in this walk
  };

  // What a walk must load and recompute to have `targets` as per-element values.
  Walk planWalk(const std::vector<int> &targets, const std::vector<bool> &tile) const {
    Walk w;
    w.ops.assign(g_.ops.size(), false);
    w.inputs.assign(g_.inputs.size(), false);
    std::vector<int> producer(g_.tensors.size(), -1);
    for (size_t k = 0; k < g_.ops.size(); ++k) {
      for (int out : g_.ops[k].outputs) producer[static_cast<size_t>(out)] = static_cast<int>(k);
    }
    std::vector<int> todo = targets;
    while (!todo.empty()) {
      const int id = todo.back();
      todo.pop_back();
      if (!tile[static_cast<size_t>(id)]) continue;
      const TensorValue &t = g_.tensor(id);
      if (t.inputIndex >= 0 && producer[static_cast<size_t>(id)] < 0) {
        w.inputs[static_cast<size_t>(t.inputIndex)] = true;
        continue;
      }
      const int k = producer[static_cast<size_t>(id)];
      if (k < 0 || w.ops[static_cast<size_t>(k)]) continue;
      w.ops[static_cast<size_t>(k)] = true;
      for (int in : operandsOf(static_cast<size_t>(k))) todo.push_back(in);
    }
    return w;
  }

  void emitWalkBody(const Walk &w) {
    emitColumnsOfGroup("akg_g");
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      if (w.inputs[i]) emitInputLoad(i);
    }
    for (size_t k = 0; k < g_.ops.size(); ++k) {
      if (w.ops[k] && !absorbed_[k]) emitElementwise(g_.ops[k], clampCast_[k]);
    }
  }

  // The row in several walks: per-row values (inputs with one element per row, reduce results and what is computed
  // from them alone) are emitted once, in description order; every reduction gets a walk over the row that recomputes
  // the elements it sums, and a last walk computes and stores the outputs.
  void emitWalks() {
    const std::vector<bool> tile = tileRanks();
    std::vector<Walk> walks;
    std::vector<size_t> walkOfOp(g_.ops.size(), 0);
    for (size_t k = 0; k < g_.ops.size(); ++k) {
      if (absorbed_[k] || !lowering::isReduceKind(g_.ops[k].kind)) continue;
      walkOfOp[k] = walks.size();
      walks.push_back(planWalk({g_.ops[k].inputs[0]}, tile));
    }
    std::vector<int> finals;
    for (int id : g_.outputs) {
      if (g_.tensor(id).numel() == numel_) finals.push_back(id);
    }
    for (const OpNode &op : g_.ops) {
      if (op.kind == OpKind::Assign) finals.push_back(op.outputs[0]);
    }
    walks.push_back(planWalk(finals, tile));
    lastPassOfInput_.assign(g_.inputs.size(), -1);
    for (size_t p = 0; p < walks.size(); ++p) {
      for (size_t i = 0; i < g_.inputs.size(); ++i) {
        if (walks[p].inputs[i]) lastPassOfInput_[i] = static_cast<int>(p);
      }
    }
    // inputs with one element per row
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      if (!access_[i].lastDimFull) emitInputLoad(i);
    }
    if (packedRow_) {
      // the row, once, as it lies in memory
      for (size_t i = 0; i < g_.inputs.size(); ++i) {
        if (packedInput_[i]) src_ << "  akg::RawChunk<" << tagOf(g_.inputs[i]) << ", V> r_in" << i << "[GROUPS * NCHUNK];\n";
      }
      line("#pragma unroll");
      line("  for (int akg_g = 0; akg_g < GROUPS; ++akg_g) {");
      emitColumnsOfGroup("akg_g");
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) {");
      for (size_t i = 0; i < g_.inputs.size(); ++i) {
        if (!packedInput_[i]) continue;
        const std::string tag = tagOf(g_.inputs[i]);
        if (conditionalAccesses()) {
          src_ << "    akg::load_raw_chunk_if<" << tag << ", V, " << (streamsWholeLines(g_.inputs[i]) ? "true" : "false") << ">(b_in"
               << i << ", akg_ok[j], " << rowOffsetExpr(access_[i], "akg_rows[j]") << " + akg_cols[j], r_in" << i
               << "[akg_g * NCHUNK + j]);\n";
          continue;
        }
        src_ << "    if (akg_ok[j]) {\n";
        src_ << "      akg::load_raw_chunk<" << tag << ", V, " << (streamsWholeLines(g_.inputs[i]) ? "true" : "false") << ">(b_in"
             << i << ", " << rowOffsetExpr(access_[i], "akg_rows[j]") << " + akg_cols[j], r_in" << i
             << "[akg_g * NCHUNK + j]);\n";
        src_ << "    } else {\n";
        src_ << "      akg::zero_raw_chunk<" << tag << ", V>(r_in" << i << "[akg_g * NCHUNK + j]);\n";
        src_ << "    }\n";
      }
      line("  }");
      line("  }");
    }
    for (size_t k = 0; k < g_.ops.size(); ++k) {
      const OpNode &op = g_.ops[k];
      if (absorbed_[k]) continue;
      if (lowering::isReduceKind(op.kind)) {
        if (!tile[static_cast<size_t>(op.inputs[0])]) {
          throw LoweringError("op " + op.name + ": the reduced operand must span the innermost axis");
        }
        pass_ = static_cast<int>(walkOfOp[k]);
        emitReduceAccumulator(op);
        if (packedRow_) line("#pragma unroll");
        line("  for (int akg_g = 0; akg_g < GROUPS; ++akg_g) {");
        emitWalkBody(walks[walkOfOp[k]]);
        emitReduceAccumulate(op);
        line("  }");
        emitReduceFinish(op);
        if (packedRow_) {
          for (size_t i = 0; i < g_.inputs.size(); ++i) {
            if (!packedInput_[i]) continue;
            line("#pragma unroll");
            src_ << "  for (int c = 0; c < GROUPS * NCHUNK; ++c) akg::forget_unpacked<" << tagOf(g_.inputs[i]) << ", V>(r_in" << i
                 << "[c]);\n";
          }
        }
      } else if (!tile[static_cast<size_t>(op.outputs[0])]) {
        emitElementwise(op, clampCast_[k]);
      }
    }
    pass_ = static_cast<int>(walks.size()) - 1;
    if (!finals.empty()) {
      if (packedRow_) line("#pragma unroll");
      line("  for (int akg_g = 0; akg_g < GROUPS; ++akg_g) {");
      emitWalkBody(walks.back());
      for (size_t i = 0; i < g_.outputs.size(); ++i) {
        if (g_.tensor(g_.outputs[i]).numel() == numel_) emitOutputStore(i);
      }
      for (const OpNode &op : g_.ops) {
        if (op.kind == OpKind::Assign) emitAssignStore(op);
      }
      line("  }");
    }
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      if (g_.tensor(g_.outputs[i]).numel() != numel_) emitOutputStore(i);
    }
  }

  void emitInputLoad(size_t i) {
    const int id = g_.inputs[i];
    const TensorValue &t = g_.tensor(id);
    const InputAccess &a = access_[i];
    ValInfo &v = vals_[static_cast<size_t>(id)];
    v.defined = true;
    const std::string tag = tagOf(id);
    const std::string ct = ctOf(id);
    std::ostringstream nm;
    if (a.lastDimFull && packedRow_ && packedInput_[i]) {
      v.rank = ValRank::Tile;
      nm << "t_in" << i;
      v.ident = nm.str();
      src_ << "  " << ct << " " << v.ident << "[NCHUNK][V];\n";
      line("#pragma unroll");
      src_ << "  for (int j = 0; j < NCHUNK; ++j) akg::unpack_chunk<" << tag << ", V>(r_in" << i << "[akg_g * NCHUNK + j], "
           << v.ident << "[j]);\n";
      return;
    }
    if (a.lastDimFull) {
      v.rank = ValRank::Tile;
      nm << "t_in" << i;
      v.ident = nm.str();
      src_ << "  " << ct << " " << v.ident << "[NCHUNK][V];\n";
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) {");
      // a tensor as large as the iteration space is read exactly once: stream it
      const bool streamed = streamsWholeLines(id) && (t.numel() == numel_) &&
                            (!multiPass_ || lastPassOfInput_[i] == pass_);
      if (conditionalAccesses()) {
        src_ << "    akg::load_chunk_if<" << tag << ", V, " << (streamed ? "true" : "false") << ">(b_in" << i << ", akg_ok[j], "
             << rowOffsetExpr(a, "akg_rows[j]") << " + akg_cols[j], " << v.ident << "[j]);\n";
      } else {
        src_ << "    if (akg_ok[j]) {\n";
        src_ << "      akg::load_chunk<" << tag << ", V, " << (streamed ? "true" : "false") << ">("
             << memRef("in" + std::to_string(i), rowOffsetExpr(a, "akg_rows[j]") + " + akg_cols[j]") << ", " << v.ident
             << "[j]);\n";
        src_ << "    } else {\n";
        src_ << "      akg::fill_chunk<" << tag << ", V>(" << v.ident << "[j], " << tag << "::load(" << tag
             << "::storage()));\n";
        src_ << "    }\n";
      }
      line("  }");
    } else if (rowMode_) {
      // one element per row (or a single element for the whole kernel)
      v.rank = ValRank::Uniform;
      nm << "u_in" << i;
      v.ident = nm.str();
      if (useBuffers_) {
        src_ << "  const " << ct << " " << v.ident << " = akg::load_one<" << tag << ">(b_in" << i << ", "
             << rowOffsetExpr(a, "akg_row") << ");\n";
      } else {
        src_ << "  const " << ct << " " << v.ident << " = " << tag << "::load(in" << i << "["
             << rowOffsetExpr(a, "akg_row") << "]);\n";
      }
      (void)t;
    } else {
      // elementwise mode: replicate the per-row element over the chunk
      v.rank = ValRank::Tile;
      nm << "t_in" << i;
      v.ident = nm.str();
      src_ << "  " << ct << " " << v.ident << "[NCHUNK][V];\n";
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) {");
      if (useBuffers_) {
        src_ << "    akg::fill_chunk<" << tag << ", V>(" << v.ident << "[j], akg::load_one<" << tag << ">(b_in" << i << ", "
             << rowOffsetExpr(a, "akg_rows[j]") << "));\n";
      } else {
        src_ << "    akg::fill_chunk<" << tag << ", V>(" << v.ident << "[j], " << tag << "::load(in" << i << "["
             << rowOffsetExpr(a, "akg_rows[j]") << "]));\n";
      }
      line("  }");
    }
  }

  void emitElementwise(const OpNode &opIn, const ClampCast &fused) {
    if (opIn.outputs.size() != 1) throw LoweringError("op " + opIn.name + ": multiple results are not supported");
    // a Cast that absorbed its clamp reads the clamp's source directly
    OpNode op = opIn;
    if (fused.source >= 0) op.inputs[0] = fused.source;
    const int outId = op.outputs[0];
    const TensorValue &outT = g_.tensor(outId);
    ValRank rank = ValRank::Const;
    bool anyNoKeep = false, anyTile = false;
    for (int in : op.inputs) {
      const ValInfo &vi = vals_[static_cast<size_t>(in)];
      if (!vi.defined) throw LoweringError("op " + op.name + ": operand " + g_.tensor(in).name + " is undefined");
      if (vi.rank == ValRank::Tile) {
        rank = ValRank::Tile;
        anyTile = true;
      } else if (vi.rank == ValRank::Uniform && rank != ValRank::Tile) {
        rank = ValRank::Uniform;
      }
      if (vi.rowvecNoKeep) anyNoKeep = true;
    }
    if (rank == ValRank::Const) rank = ValRank::Uniform;
    if (op.kind == OpKind::Iota) {
      if (!rowMode_) throw LoweringError("op Iota: only produced for ArgMax over the innermost axis");
      rank = ValRank::Tile;
    }
    if (anyTile && anyNoKeep) {
      throw LoweringError("op " + op.name + ": a reduce result without keep_dims cannot be broadcast against the "
                          "reduced tensor; reshape it to [...,1] first");
    }
    // shape sanity: a Tile result must span the innermost dim, a Uniform result must not
    if (rowMode_) {
      int64_t last = outT.shape.empty() ? 1 : outT.shape.back();
      if (rank == ValRank::Tile && last != cols_) {
        throw LoweringError("op " + op.name + ": result shape does not match its operands");
      }
    }

    std::vector<std::string> operands;
    for (int in : op.inputs) operands.push_back(operandExpr(in));
    const bool relaxed = relaxed_[static_cast<size_t>(outId)];
    std::string expr;
    // float32 division of a tile by a per-row (or constant) divisor: hoist the reciprocal out of the element loop
    const bool uniformDivisor = op.kind == OpKind::Div && rank == ValRank::Tile && op.inputs.size() == 2 &&
                                vals_[static_cast<size_t>(op.inputs[1])].rank != ValRank::Tile &&
                                std::string(computeTypeName(outT.dtype)) == "float" &&
                                std::string(computeTypeName(g_.tensor(op.inputs[0]).dtype)) == "float" &&
                                std::string(computeTypeName(g_.tensor(op.inputs[1]).dtype)) == "float";
    if (op.kind == OpKind::Iota) {
      expr = "static_cast<int>(akg_cols[j] + e)";   // the column of the element: the innermost axis of the row space
    } else if (fused.source >= 0) {
      expr = "akg::clamp_cast(" + operands[0] + ", " + lowering::literalFor(DType::F32, fused.lo) + ", " +
             lowering::literalFor(DType::F32, fused.hi) + ")";
    } else if (uniformDivisor) {
      const std::string hoisted = "d" + std::to_string(outId);
      std::string q;
      if (relaxed) {
        src_ << "  const float " << hoisted << " = akg::fast_rcp(" << operands[1] << ");\n";
        q = "(" + operands[0] + " * " + hoisted + ")";
      } else {
        src_ << "  const akg::UniformDivisor " << hoisted << " = akg::make_divisor(" << operands[1] << ");\n";
        q = "akg::div_uniform(" + operands[0] + ", " + hoisted + ")";
      }
      const DType od = outT.dtype;
      expr = (od == DType::F16 || od == DType::BF16) ? std::string(dtypeTag(od)) + "::rnd(" + q + ")" : q;
    } else {
      expr = lowering::elementwiseExpr(g_, op, operands, relaxed);
    }

    ValInfo &v = vals_[static_cast<size_t>(outId)];
    v.defined = true;
    v.rank = rank;
    std::ostringstream nm;
    if (rank == ValRank::Tile) {
      nm << "t" << outId;
      v.ident = nm.str();
      src_ << "  " << ctOf(outId) << " " << v.ident << "[NCHUNK][V];  // " << op.name << " -> " << outT.name << "\n";
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) {");
      line("#pragma unroll");
      line("    for (int e = 0; e < V; ++e) {");
      src_ << "      " << v.ident << "[j][e] = " << expr << ";\n";
      line("    }");
      line("  }");
    } else {
      nm << "u" << outId;
      v.ident = nm.str();
      src_ << "  const " << ctOf(outId) << " " << v.ident << " = " << expr << ";  // " << op.name << " -> " << outT.name
           << "\n";
      // A per-row value whose shape lacks the trailing 1 (reduce without keep_dims, or a reshape of one).
      v.rowvecNoKeep = rowMode_ && outT.numel() != 1 && !outT.shape.empty() && outT.shape.back() != 1;
    }
  }

  void emitReduceAccumulator(const OpNode &op) {
    const int inId = op.inputs[0];
    const int outId = op.outputs[0];
    const DType od = g_.tensor(outId).dtype;
    const std::string ct = computeTypeName(od);
    const lowering::ReduceSpec spec = lowering::reduceSpec(op, od);
    if (std::string(computeTypeName(g_.tensor(inId).dtype)) != ct) {
      throw LoweringError("op " + op.name + ": operand and result element types differ");
    }
    src_ << "  " << ct << " acc" << outId << " = " << spec.init << ";  // " << op.name << " -> " << g_.tensor(outId).name
         << "\n";
  }

  void emitReduceAccumulate(const OpNode &op) {
    const int inId = op.inputs[0];
    const int outId = op.outputs[0];
    const ValInfo &in = vals_[static_cast<size_t>(inId)];
    if (!in.defined || in.rank != ValRank::Tile) {
      throw LoweringError("op " + op.name + ": the reduced operand must span the innermost axis");
    }
    const DType od = g_.tensor(outId).dtype;
    const std::string tag = dtypeTag(od);
    const lowering::ReduceSpec spec = lowering::reduceSpec(op, od);
    const std::string acc = "acc" + std::to_string(outId);
    if (spec.ordered) {
      // this group of the row into LDS, then the row's first thread folds it onto its accumulator in index order
      const std::string base = multiPass_ ? "static_cast<long>(akg_g) * (NCHUNK * TPR * V)" : "0L";
      src_ << "  {\n";
      src_ << "    " << tag << "::storage *akg_run = reinterpret_cast<" << tag << "::storage *>(akg_chain[tid / TPR]);\n";
      src_ << "    const long akg_base = " << base << ";\n";
      line("#pragma unroll");
      line("    for (int j = 0; j < NCHUNK; ++j) {");
      std::string from = "0";
      if (colsArg_ && !colsWhole_) {
        from = "akg_tail[j] ? akg_overlap : 0";
      } else if (overlap_ > 0) {
        from = "akg_tail[j] ? " + std::to_string(overlap_) + " : 0";
      }
      src_ << "      " << (raggedCols_ || colsArg_ || overlap_ > 0 ? "if (akg_ok[j]) " : "") << "akg::chain_put<" << tag
           << ", V>(akg_run, static_cast<int>(akg_cols[j] - akg_base), " << in.ident << "[j], " << from << ");\n";
      line("    }");
      line("    __syncthreads();");
      line("    const long akg_left = COLS - akg_base;");
      src_ << "    if (tcol == 0) " << acc << " = akg::chain_fold<" << spec.combiner << ", " << tag << ">(" << acc
           << ", akg_run, static_cast<int>(akg_left < NCHUNK * TPR * V ? akg_left : NCHUNK * TPR * V));\n";
      line("    __syncthreads();");
      src_ << "  }\n";
      return;
    }
    const bool anyOrder = spec.combiner == "akg::RedMax" || spec.combiner == "akg::RedMin";
    if (anyOrder && (raggedCols_ || overlap_ > 0)) {
      // A maximum or minimum does not depend on the order of its steps nor on an element taken twice (the elements a
      // tail chunk shares with its neighbour): the chunk is folded by itself and joins the accumulator under the one
      // condition of the chunk, instead of every element under its own.
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) {");
      src_ << "    " << computeTypeName(od) << " akg_part = " << in.ident << "[j][0];\n";
      line("#pragma unroll");
      src_ << "    for (int e = 1; e < V; ++e) akg_part = " << spec.combiner << "::apply(akg_part, " << in.ident << "[j][e]);\n";
      src_ << "    if (akg_ok[j]) " << acc << " = " << spec.combiner << "::apply(" << acc << ", akg_part);\n";
      line("  }");
      return;
    }
    line("#pragma unroll");
    line("  for (int j = 0; j < NCHUNK; ++j) {");
    line("#pragma unroll");
    line("    for (int e = 0; e < V; ++e) {");
    std::string step = spec.combiner + "::apply(" + acc + ", " + in.ident + "[j][e])";
    if (spec.roundEachStep) step = tag + "::rnd(" + step + ")";
    if (colsArg_ && !colsWhole_) {
      src_ << "      if (akg_ok[j] && (!akg_tail[j] || e >= akg_overlap)) " << acc << " = " << step << ";\n";
    } else if (overlap_ > 0) {
      src_ << "      if (akg_ok[j] && (!akg_tail[j] || e >= " << overlap_ << ")) " << acc << " = " << step << ";\n";
    } else if (raggedCols_) {
      src_ << "      if (akg_ok[j]) " << acc << " = " << step << ";\n";
    } else {
      src_ << "      " << acc << " = " << step << ";\n";
    }
    line("    }");
    line("  }");
  }

  void emitReduceFinish(const OpNode &op) {
    const int outId = op.outputs[0];
    const DType od = g_.tensor(outId).dtype;
    const std::string ct = computeTypeName(od);
    const std::string tag = dtypeTag(od);
    const lowering::ReduceSpec spec = lowering::reduceSpec(op, od);
    const std::string red = spec.combiner;
    const bool roundEachStep = spec.roundEachStep;
    const std::string acc = "acc" + std::to_string(outId);
    ValInfo &v = vals_[static_cast<size_t>(outId)];
    std::ostringstream nm;
    nm << "u" << outId;
    if (spec.ordered) {
      src_ << "  if (tcol == 0) akg_chain_res[tid / TPR] = " << acc << ";\n";
      line("  __syncthreads();");
      src_ << "  const " << ct << " " << nm.str() << " = akg_chain_res[tid / TPR];\n";
      v.defined = true;
      v.rank = ValRank::Uniform;
      v.ident = nm.str();
      const TensorValue &outT = g_.tensor(outId);
      v.rowvecNoKeep = outT.numel() != 1 && !outT.shape.empty() && outT.shape.back() != 1;
      return;
    }
    std::string scratch = tpr_ > 64 ? "reinterpret_cast<" + ct + " *>(akg_scratch[" + std::to_string(reduceCount_ & 1) + "])"
                                    : "static_cast<" + ct + " *>(nullptr)";
    src_ << "  const " << ct << " " << nm.str() << " = " << (roundEachStep ? tag + "::rnd(" : "")
         << "akg::group_reduce<" << red << ", TPR>(" << acc << ", " << scratch << ", tid)" << (roundEachStep ? ")" : "")
         << ";\n";
    ++reduceCount_;
    v.defined = true;
    v.rank = ValRank::Uniform;
    v.ident = nm.str();
    const TensorValue &outT = g_.tensor(outId);
    v.rowvecNoKeep = outT.numel() != 1 && !outT.shape.empty() && outT.shape.back() != 1;
  }

  void emitAssignStore(const OpNode &op) {
    const TensorValue &dst = g_.tensor(op.inputs[0]);
    const int valueId = op.outputs[0];
    const ValInfo &v = vals_[static_cast<size_t>(valueId)];
    if (!v.defined) throw LoweringError("op " + op.name + ": value is never computed");
    if (dst.numel() != numel_ || v.rank != ValRank::Tile) {
      throw LoweringError("op " + op.name + ": only destinations as large as the kernel's iteration space are supported");
    }
    const std::string tag = tagOf(valueId);
    line("#pragma unroll");
    line("  for (int j = 0; j < NCHUNK; ++j) {");
    std::string guard = "akg_ok[j]";
    if (rowMode_ && raggedRows_) guard += " && akg_row_ok";
    const std::string offset = rowMode_ ? "akg_rows[j] * COLS + akg_cols[j]" : "akg_flat[j]";
    if (conditionalAccesses() || (useBuffers_ && guard != "akg_ok[j]")) {
      src_ << "    akg::store_chunk_if<" << tag << ", V, " << (streamsWholeLines(op.inputs[0]) ? "true" : "false") << ">(b_in"
           << dst.inputIndex << ", " << guard << ", " << offset << ", " << v.ident << "[j]);  // " << op.name << " -> "
           << dst.name << "\n";
    } else {
      src_ << "    if (" << guard << ") akg::store_chunk<" << tag << ", V, " << (streamsWholeLines(op.inputs[0]) ? "true" : "false") << ">("
           << memRef("in" + std::to_string(dst.inputIndex), offset) << ", " << v.ident << "[j]);  // " << op.name << " -> "
           << dst.name << "\n";
    }
    line("  }");
  }

  void emitOutputStore(size_t i) {
    const int id = g_.outputs[i];
    const TensorValue &t = g_.tensor(id);
    const ValInfo &v = vals_[static_cast<size_t>(id)];
    if (!v.defined) throw LoweringError("output " + t.name + " is never computed");
    const std::string tag = tagOf(id);
    const std::string ct = ctOf(id);
    const bool fullSized = (t.numel() == numel_);
    if (!rowMode_ || fullSized) {
      if (!fullSized) throw LoweringError("output " + t.name + ": shape does not match the kernel's iteration space");
      std::string src = v.ident;
      if (v.rank != ValRank::Tile) {
        // broadcast a uniform value over the chunk
        src = "t_bcast" + std::to_string(i);
        src_ << "  " << ct << " " << src << "[NCHUNK][V];\n";
        line("#pragma unroll");
        src_ << "  for (int j = 0; j < NCHUNK; ++j) akg::fill_chunk<" << tag << ", V>(" << src << "[j], " << v.ident
             << ");\n";
      }
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) {");
      std::string guard = "akg_ok[j]";
      if (rowMode_ && raggedRows_) guard += " && akg_row_ok";
      std::string offset = rowMode_ ? "akg_rows[j] * COLS + akg_cols[j]" : "akg_flat[j]";
      if (conditionalAccesses() || (useBuffers_ && guard != "akg_ok[j]")) {
        src_ << "    akg::store_chunk_if<" << tag << ", V, " << (streamsWholeLines(id) ? "true" : "false") << ">(b_out" << i << ", "
             << guard << ", " << offset << ", " << src << "[j]);\n";
      } else {
        src_ << "    if (" << guard << ") akg::store_chunk<" << tag << ", V, " << (streamsWholeLines(id) ? "true" : "false") << ">("
             << memRef("out" + std::to_string(i), offset) << ", " << src
             << "[j]);\n";
      }
      line("  }");
    } else {
      if (t.numel() != rows_) {
        throw LoweringError("output " + t.name + ": shape is neither the reduced tensor's nor one value per row");
      }
      if (v.rank == ValRank::Tile) throw LoweringError("output " + t.name + ": internal rank mismatch");
      std::string guard = "tcol == 0";
      if (raggedRows_) guard += " && akg_row_ok";
      if (useBuffers_) {
        src_ << "  if (" << guard << ") akg::store_one<" << tag << ">(b_out" << i << ", akg_row, " << v.ident << ");\n";
      } else {
        src_ << "  if (" << guard << ") out" << i << "[akg_row] = " << tag << "::store(" << v.ident << ");\n";
      }
    }
  }
};

}  // namespace

LoweredKernel lowerTileToHip(const OpGraph &graph, const LoweringOptions &options) {
  TileEmitter emitter(graph, options);
  return emitter.run();
}

}  // namespace akg
