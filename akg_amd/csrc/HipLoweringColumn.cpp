/**
 * Reductions over one axis that is not the innermost one, whose results meet the unreduced tensor again: a softmax over
 * the channels of [N, C, H, W], a LayerNorm over the middle axis of [B, R, I] (family `column_reduce`).
 *
 * The streaming reductions keep nothing of what they read, so such a description would take one pass over the tensor per
 * level of its reductions (max, then sum of exp, then the quotient: three reads). Here the tensor is seen as [O, R, I] -
 * the axes in front of the reduced one, the reduced one, the ones behind it - and a workgroup owns a strip of columns
 * (o, i0 .. i0 + LX * V) for the whole run R: thread (ly, lx) keeps the chunks of V columns at rows ly, ly + RY, ... of
 * every full-sized kernel input in registers, as they came from memory (a 16-bit chunk takes half the registers of its
 * float image). The V lanes of a chunk belong to V different runs, so a reduction is V accumulators per thread, folded
 * over the thread's rows and then over the threads that hold the same columns (akg::column_reduce: partners inside the
 * wavefront, LDS across wavefronts). Every level of reductions is one walk over the resident chunks that recomputes
 * the elementwise ops in front of it; the last walk computes the outputs. The tensor is read once and written once.
 *
 * Reductions follow createInitValueForReduce / createCombinerForReduce of the reference (MindSporeToLinalg.cpp:791-901):
 * same initial values and combiners, narrow result types rounded after every step. A float16 / bfloat16 sum or product
 * keeps the reference's order, one serial chain per column over the rows of the run (akg::column_chain_step); every
 * other combiner gives the same result in any order (integers wrap, a maximum is one of its operands) or is a float32 /
 * float64 sum, whose order is the kernel's own (rows of one thread in increasing order, then the threads).
 */
#include <algorithm>
#include <sstream>

#include "HipLowering.h"

namespace akg {

namespace {

using lowering::computeTypeName;
using lowering::dtypeTag;

enum class Rank { Scalar, RowS, Col, Full };   // one value; one per row; one per column; one per element

struct Flags {
  bool o = false, r = false, i = false;
  Rank rank() const { return r && i ? Rank::Full : r ? Rank::RowS : i ? Rank::Col : Rank::Scalar; }
  bool operator==(const Flags &b) const { return o == b.o && r == b.r && i == b.i; }
};

struct Val {
  bool defined = false;
  Rank rank = Rank::Scalar;
  std::string ident;   // t<id>[e] / c<id>[e] / r<id>[j] / s<id>, or a literal
  int level = 0;
};

class ColumnEmitter {
 public:
  ColumnEmitter(const OpGraph &g, const LoweringOptions &o) : g_(g), opt_(o) {}

  LoweredKernel run() {
    analyse();
    pickSchedule();
    emit();
    LoweredKernel k;
    k.kernelName = g_.name + "_kernel";
    k.source = src_.str();
    k.family = KernelFamily::ColumnReduce;
    k.grid[0] = static_cast<unsigned>(launched_);
    k.block[0] = static_cast<unsigned>(block_);
    k.algorithmicBytes = lowering::countAlgorithmicBytes(g_);
    k.shapeArgs = lowering::buildShapeArgs(g_);
    if (dynOuter_) k.scalarArgs.push_back(outer_);
    std::ostringstream note;
    note << "column_reduce outer=" << outer_ << " run=" << run_ << " inner=" << inner_ << " vec=" << vec_ << " threads=" << ly_ << "x" << lx_
         << " rows/thread=" << chunks_ << " walks=" << (maxLevel_ + 1) << (pipelined_ ? " strips pipelined" : "");
    if (dynOuter_) note << " (the outer extent is a kernel argument)";
    k.scheduleNote = note.str();
    return k;
  }

 private:
  const OpGraph &g_;
  const LoweringOptions &opt_;
  std::ostringstream src_;
  std::vector<int64_t> full_;      // shape of the reduced tensor
  size_t axis_ = 0;
  int64_t outer_ = 1, run_ = 1, inner_ = 1;
  std::vector<Flags> flags_;       // per tensor
  std::vector<Val> vals_;
  std::vector<int> level_;
  std::vector<bool> relaxed_;
  int maxLevel_ = 0;
  int vec_ = 4, lx_ = 8, ly_ = 32, chunks_ = 1, block_ = 256;
  int64_t strips_ = 1;
  bool pipelined_ = false;         // workgroups stay and walk several strips, the next strip's loads issued before the work on this one
  int64_t launched_ = 0;           // workgroups launched
  // A description with open extents: the extent in front of the reduced axis (the batch) is a kernel argument. Nothing
  // else in the source depends on it but the choice between one strip per workgroup and persistent workgroups.
  bool dynOuter_ = false;
  bool aligned_ = true;            // every chunk starts at a multiple of its size and lies inside its row
  int reduceCount_ = 0;
  bool ordered_ = false;           // some reduction is a float16 / bfloat16 sum or product: steps in index order

  static std::string id(const char *prefix, int t) { return std::string(prefix) + std::to_string(t); }

  Flags classify(const TensorValue &t, const std::string &what) const {
    Flags f;
    if (t.numel() == 1) return f;
    const size_t n = full_.size();
    std::vector<int64_t> s = t.shape;
    if (s.size() + 1 == n) {
      std::vector<int64_t> dropped = full_;
      dropped.erase(dropped.begin() + static_cast<long>(axis_));
      if (s == dropped) s.insert(s.begin() + static_cast<long>(axis_), 1);   // a reduction result without keep_dims
    }
    while (s.size() < n) s.insert(s.begin(), 1);
    if (s.size() != n) throw LoweringError(what + ": rank does not fit the reduced tensor's");
    int seenO = -1, seenI = -1;
    for (size_t d = 0; d < n; ++d) {
      if (s[d] != full_[d] && s[d] != 1) throw LoweringError(what + ": shape does not broadcast against the reduced tensor's");
      if (full_[d] == 1) continue;
      const int spans = s[d] != 1 ? 1 : 0;
      if (d == axis_) {
        f.r = spans != 0;
      } else {
        int &seen = d < axis_ ? seenO : seenI;
        if (seen >= 0 && seen != spans) throw LoweringError(what + ": broadcasts along part of the axes on one side of the reduced one");
        seen = spans;
      }
    }
    f.o = seenO == 1;
    f.i = seenI == 1;
    return f;
  }

  void analyse() {
    const OpNode *first = nullptr;
    for (const OpNode &op : g_.ops) {
      if (lowering::isReduceKind(op.kind)) {
        first = &op;
        break;
      }
    }
    if (first == nullptr) throw LoweringError("column kernel: no reduction");
    full_ = g_.tensor(first->inputs[0]).shape;
    const auto realAxes = [&](const OpNode &op) {
      const TensorValue &in = g_.tensor(op.inputs[0]);
      std::vector<size_t> out;
      for (int64_t a : op.axes) {
        if (a >= 0 && static_cast<size_t>(a) < in.shape.size() && in.shape[static_cast<size_t>(a)] > 1) out.push_back(static_cast<size_t>(a));
      }
      return out;
    };
    const std::vector<size_t> axes = realAxes(*first);
    if (axes.size() != 1) throw LoweringError("column kernel: exactly one reduced axis");
    axis_ = axes[0];
    for (size_t d = 0; d < full_.size(); ++d) {
      (d < axis_ ? outer_ : d == axis_ ? run_ : inner_) *= full_[d];
    }
    if (inner_ < 2) throw LoweringError("column kernel: the reduced axis is the innermost one");
    if (outer_ * run_ * inner_ >= (1LL << 40)) throw LoweringError("column kernel: too large");
    const size_t nt = g_.tensors.size();
    flags_.assign(nt, Flags());
    level_.assign(nt, 0);
    for (size_t t = 0; t < nt; ++t) {
      const TensorValue &tv = g_.tensors[t];
      if (tv.isConst) continue;
      flags_[t] = classify(tv, "tensor " + tv.name);
    }
    for (const OpNode &op : g_.ops) {
      if (op.outputs.size() != 1) throw LoweringError("op " + op.name + ": multiple results are not supported");
      const int out = op.outputs[0];
      int lv = 0;
      for (int in : op.inputs) lv = std::max(lv, level_[static_cast<size_t>(in)]);
      if (lowering::isReduceKind(op.kind)) {
        const TensorValue &in = g_.tensor(op.inputs[0]);
        if (in.shape != full_ || realAxes(op) != axes) throw LoweringError("column kernel: all reductions must run over the same axis of the same shape");
        if (flags_[static_cast<size_t>(op.inputs[0])].rank() != Rank::Full) throw LoweringError("op " + op.name + ": operand does not span the reduced axis");
        if (std::string(computeTypeName(in.dtype)) != computeTypeName(g_.tensor(out).dtype)) {
          throw LoweringError("op " + op.name + ": operand and result element types differ");
        }
        if (flags_[static_cast<size_t>(out)].r || !flags_[static_cast<size_t>(out)].i) {
          throw LoweringError("op " + op.name + ": result shape does not match");
        }
        ordered_ = ordered_ || lowering::reduceSpec(op, g_.tensor(out).dtype).ordered;
        lv += 1;
      } else if (!lowering::isElementwiseKind(op.kind) || op.kind == OpKind::Assign || op.kind == OpKind::Iota) {
        throw LoweringError("op " + op.name + ": not an elementwise op or a reduction");
      } else if (op.kind == OpKind::Reshape) {
        if (!(flags_[static_cast<size_t>(out)] == flags_[static_cast<size_t>(op.inputs[0])])) {
          throw LoweringError("op Reshape: more than adding or dropping unit dimensions");
        }
      } else if (axis_ > 0) {
        // A reduction result without keep_dims has lost the reduced axis: against a tensor of the full rank, broadcasting
        // would align it on the right, not where it came from. Only a Reshape may put the axis back.
        bool droppedAxis = false, fullRank = false;
        for (int in : op.inputs) {
          const TensorValue &t = g_.tensor(in);
          if (t.isConst || t.numel() == 1) continue;
          droppedAxis = droppedAxis || (t.shape.size() + 1 == full_.size() && flags_[static_cast<size_t>(in)].rank() == Rank::Col);
          fullRank = fullRank || t.shape.size() == full_.size();
        }
        if (droppedAxis && fullRank) {
          throw LoweringError("op " + op.name + ": a reduce result without keep_dims cannot be broadcast against the reduced tensor; reshape it first");
        }
      }
      level_[static_cast<size_t>(out)] = lv;
      maxLevel_ = std::max(maxLevel_, lv);
    }
    if (maxLevel_ < 1) throw LoweringError("column kernel: no reduction result is used");
    for (int o : g_.outputs) {
      const TensorValue &t = g_.tensor(o);
      if (t.producer < 0) throw LoweringError("output " + t.name + " is a kernel input");
      const Rank r = flags_[static_cast<size_t>(o)].rank();
      if (r == Rank::RowS || (r == Rank::Scalar && t.numel() != 1)) throw LoweringError("output " + t.name + ": one value per row");
      if (r == Rank::Scalar) throw LoweringError("output " + t.name + ": a single value");
      if ((r == Rank::Full || r == Rank::Col) && outer_ > 1 && !flags_[static_cast<size_t>(o)].o) {
        throw LoweringError("output " + t.name + ": does not span the outer axes");
      }
    }
    relaxed_ = lowering::relaxedPrecisionTensors(g_);
  }

  void pickSchedule() {
    int widest = 1, fullInputs = 0, fullBytes = 0;
    for (size_t t = 0; t < g_.tensors.size(); ++t) {
      const TensorValue &tv = g_.tensors[t];
      if (tv.isConst || !flags_[t].i) continue;
      if (tv.inputIndex < 0 && tv.outputIndex < 0) continue;
      widest = std::max(widest, static_cast<int>(dtypeSize(tv.dtype)));
      if (tv.inputIndex >= 0 && tv.used && flags_[t].rank() == Rank::Full) {
        ++fullInputs;
        fullBytes += static_cast<int>(dtypeSize(tv.dtype));
      }
    }
    if (fullInputs == 0) throw LoweringError("column kernel: no full-sized input");
    vec_ = opt_.vec > 0 ? opt_.vec : 16 / widest;
    if (vec_ != 1 && vec_ != 2 && vec_ != 4 && vec_ != 8 && vec_ != 16) throw LoweringError("column kernel: unsupported vector width");
    aligned_ = inner_ % vec_ == 0;
    const auto pow2floor = [](int64_t x) { int64_t p = 1; while (p * 2 <= x) p *= 2; return p; };
    const auto pow2ceil = [](int64_t x) { int64_t p = 1; while (p < x) p *= 2; return p; };
    const int64_t lxMax = std::min<int64_t>(64, pow2ceil((inner_ + vec_ - 1) / vec_));
    // About four rows per thread keep enough loads in flight; the registers of the resident chunks bound the rest:
    // a chunk of every full-sized input per row of the thread, at most 64 registers in all, else a larger workgroup
    // (bf16 [64,768,1024] over the middle axis: 24 rows a thread in 256 threads 50.7 us, 12 in 512 48.6, 6 in 1024 49.4).
    const auto shapeFor = [&](int block) {
      int64_t ly = std::min<int64_t>(std::max<int64_t>(1, pow2floor(run_ / 4)), block / 8);
      int64_t lx = std::min<int64_t>(block / ly, lxMax);
      ly = block / lx;
      block_ = block;
      lx_ = static_cast<int>(lx);
      ly_ = static_cast<int>(ly);
      chunks_ = static_cast<int>((run_ + ly - 1) / ly);
      return static_cast<int64_t>(chunks_) * ((fullBytes * vec_ + 3) / 4);   // registers of a thread's resident chunks
    };
    for (int block = opt_.block > 0 ? opt_.block : 256; ; block *= 2) {
      const int64_t regs = shapeFor(block);
      if (regs <= 64 || (regs <= 96 && block_ >= 1024)) break;
      if (block_ >= 1024 || opt_.block > 0) throw LoweringError("column kernel: the run does not fit the registers of a workgroup");
    }
    // rows beyond the run would idle whole wavefronts: shrink the workgroup to the run
    while (block_ > 64 && static_cast<int64_t>(ly_ / 2) * chunks_ >= run_ && ly_ > 1 && chunks_ == 1) {
      ly_ /= 2;
      block_ /= 2;
    }
    strips_ = (inner_ + static_cast<int64_t>(lx_) * vec_ - 1) / (static_cast<int64_t>(lx_) * vec_);
    if (outer_ * strips_ >= (1LL << 31)) throw LoweringError("column kernel: too many workgroups");
    // A workgroup that keeps tens of KB resident loads, reduces, then stores, and its neighbours on the CU do the same in
    // step: memory idles while they compute. With several strips per workgroup the loads of the next strip are issued
    // before the work on this one (a second set of resident registers, one workgroup per CU). Worth it for large
    // footprints only: many small workgroups per CU drift apart by themselves.
    // (Measured on bf16 [64,768,1024] over the middle axis, LayerNorm: 48.0 us as 1024 workgroups of one strip, 45.0 us as
    // 256 workgroups of four strips each. A 1024-thread workgroup with half the rows per thread, which would fit four
    // wavefronts per SIMD beside the second set, spills under the 128-register limit and takes 87 us; softmax over 21
    // classes of f16 [32,21,512,512], 24 resident registers in 256 threads: 114 us as it is, 150 us pipelined.)
    const int64_t regs = static_cast<int64_t>(chunks_) * ((fullBytes * vec_ + 3) / 4);
    const int64_t kCUs = opt_.computeUnits;
    pipelined_ = !ordered_ && opt_.variant != 5 && regs >= 40 && regs <= 64 && block_ == 512 && outer_ * strips_ >= 2 * kCUs;
    // (two such workgroups per CU where every one still gets two strips and more: 45.0 -> 43.5 us on the shape above)
    launched_ = pipelined_ ? (outer_ * strips_ >= 4 * kCUs ? 2 * kCUs : kCUs) : outer_ * strips_;
    dynOuter_ = opt_.extentAsArgument && outer_ > 1;
  }

  void line(const std::string &s) { src_ << s << "\n"; }

  std::string operandExpr(int t) const {
    const TensorValue &tv = g_.tensor(t);
    if (tv.isConst) return lowering::literalFor(tv.dtype, tv.constValue);
    const Val &v = vals_[static_cast<size_t>(t)];
    if (!v.defined) throw LoweringError("tensor " + tv.name + " is used before it is computed");
    switch (v.rank) {
      case Rank::Full:
      case Rank::Col:
        return v.ident + "[e]";
      case Rank::RowS:
        return v.ident + "[j]";
      default:
        return v.ident;
    }
  }

  // index of element (o, row, col) of a tensor with these flags
  std::string offsetExpr(const Flags &f, const std::string &row, const std::string &col) const {
    const int64_t er = f.r ? run_ : 1, ei = f.i ? inner_ : 1;
    std::ostringstream s;
    s << "(";
    s << (f.o ? "akg_o * " + std::to_string(er * ei) + "L" : std::string("0L"));
    if (f.r) s << " + static_cast<long>(" << row << ") * " << ei << "L";
    if (f.i) s << " + " << col;
    s << ")";
    return s.str();
  }

  Rank resultRank(const OpNode &op) const {
    bool anyFull = false, anyCol = false, anyRow = false;
    for (int in : op.inputs) {
      if (g_.tensor(in).isConst) continue;
      const Rank r = vals_[static_cast<size_t>(in)].rank;
      anyFull = anyFull || r == Rank::Full;
      anyCol = anyCol || r == Rank::Col;
      anyRow = anyRow || r == Rank::RowS;
    }
    if (anyFull || (anyCol && anyRow)) return Rank::Full;
    return anyCol ? Rank::Col : anyRow ? Rank::RowS : Rank::Scalar;
  }

  // Elementwise ops of rank `rank` whose level is `from` .. `upto`, in description order.
  void emitOps(Rank rank, int from, int upto, const std::string &ind) {
    for (const OpNode &op : g_.ops) {
      if (lowering::isReduceKind(op.kind)) continue;
      const int out = op.outputs[0];
      const int lv = level_[static_cast<size_t>(out)];
      if (lv < from || lv > upto) continue;
      bool ready = true;
      for (int in : op.inputs) ready = ready && (g_.tensor(in).isConst || vals_[static_cast<size_t>(in)].defined);
      if (!ready) continue;   // (an operand of another rank that this walk does not compute: a later walk does)
      const Rank r = resultRank(op);
      if (r != rank) continue;
      Val &v = vals_[static_cast<size_t>(out)];
      if (rank != Rank::Full && v.defined) continue;   // computed once, in front of the first walk that can
      const std::string ct = computeTypeName(g_.tensor(out).dtype);
      if (op.kind == OpKind::Reshape || op.kind == OpKind::BroadcastTo) {
        const Val &in = vals_[static_cast<size_t>(op.inputs[0])];
        if (g_.tensor(op.inputs[0]).isConst) throw LoweringError("op " + op.name + ": constant operand");
        v = in;
        v.level = lv;
        continue;
      }
      std::vector<std::string> operands;
      for (int in : op.inputs) operands.push_back(operandExpr(in));
      const std::string expr = lowering::elementwiseExpr(g_, op, operands, relaxed_[static_cast<size_t>(out)]);
      v.defined = true;
      v.rank = rank;
      v.level = lv;
      switch (rank) {
        case Rank::Full:
          v.ident = id("t", out);
          src_ << ind << ct << " " << v.ident << "[V];  // " << op.name << " -> " << g_.tensor(out).name << "\n";
          src_ << ind << "#pragma unroll\n";
          src_ << ind << "for (int e = 0; e < V; ++e) " << v.ident << "[e] = " << expr << ";\n";
          break;
        case Rank::Col:
          v.ident = id("c", out);
          src_ << ind << ct << " " << v.ident << "[V];  // " << op.name << " -> " << g_.tensor(out).name << "\n";
          src_ << ind << "#pragma unroll\n";
          src_ << ind << "for (int e = 0; e < V; ++e) " << v.ident << "[e] = " << expr << ";\n";
          break;
        case Rank::RowS:
          v.ident = id("r", out);
          src_ << ind << ct << " " << v.ident << "[CH];  // " << op.name << " -> " << g_.tensor(out).name << "\n";
          src_ << ind << "#pragma unroll\n";
          src_ << ind << "for (int j = 0; j < CH; ++j) " << v.ident << "[j] = " << expr << ";\n";
          break;
        default:
          v.ident = id("s", out);
          src_ << ind << "const " << ct << " " << v.ident << " = " << expr << ";  // " << op.name << " -> " << g_.tensor(out).name << "\n";
      }
    }
  }

  // Full-rank values live inside one walk only.
  void forgetFull() {
    for (size_t t = 0; t < vals_.size(); ++t) {
      if (vals_[t].defined && vals_[t].rank == Rank::Full && g_.tensors[t].inputIndex < 0) vals_[t].defined = false;
    }
  }

  void emit() {
    vals_.assign(g_.tensors.size(), Val());
    src_ << "// Generated by the akg HIP lowering for gfx950. Op description: " << g_.name << "\n";
    src_ << "// family: column_reduce, fusion class: " << operatorTemplateName(g_.operatorTemplate) << "\n";
    src_ << "#include \"akg_rt.hpp\"\n\n";
    src_ << "extern \"C\" __global__ __launch_bounds__(" << block_ << ") void " << g_.name << "_kernel(";
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      src_ << (i ? ", " : "") << "const " << dtypeTag(g_.tensor(g_.inputs[i]).dtype) << "::storage *__restrict__ in" << i;
    }
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      src_ << ", " << dtypeTag(g_.tensor(g_.outputs[i]).dtype) << "::storage *__restrict__ out" << i;
    }
    if (dynOuter_) src_ << ", const long akg_outer_arg";
    src_ << ") {\n";
    src_ << "  constexpr int V = " << vec_ << ", LX = " << lx_ << ", LY = " << ly_ << ", CH = " << chunks_ << ", BLOCK = " << block_ << ";\n";
    src_ << "  constexpr long RUN = " << run_ << ", INNER = " << inner_ << ", STRIPS = " << strips_ << ";\n";
    if (dynOuter_) {
      line("  const long TOTAL = akg_outer_arg * STRIPS;   // strips in all");
      line("  (void)TOTAL;");
    } else {
      src_ << "  constexpr long TOTAL = " << outer_ * strips_ << ";   // strips in all\n";
    }
    if (block_ > 64) line("  __shared__ __attribute__((aligned(16))) unsigned char akg_scratch[2][(BLOCK / 64) * LX * V * 8];");
    if (ordered_) {
      // the rows of one step of an ordered reduction, in their 16-bit type, and the folded results per column
      line("  constexpr int NOWN = (LX * V + BLOCK - 1) / BLOCK;   // columns a thread folds");
      line("  __shared__ __attribute__((aligned(16))) unsigned short akg_chain[LY * LX * V];");
      line("  __shared__ float akg_chain_res[LX * V];");
    }
    line("  const int tid = static_cast<int>(threadIdx.x), lx = tid % LX, ly = tid / LX;");
    // the resident chunks of one strip: every full-sized input as it came from memory
    std::string packedParams, packedArgsA, packedArgsB;
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      const TensorValue &tv = g_.tensor(g_.inputs[i]);
      if (!tv.used || flags_[static_cast<size_t>(g_.inputs[i])].rank() != Rank::Full) continue;
      const std::string tag = dtypeTag(tv.dtype);
      packedParams += ", akg::PackedChunk<" + tag + ", V> (&p_in" + std::to_string(i) + ")[CH]";
      packedArgsA += ", akg_a" + std::to_string(i);
      packedArgsB += ", akg_b_set" + std::to_string(i);
      src_ << "  akg::PackedChunk<" << tag << ", V> akg_a" << i << "[CH];  // " << tv.name << "\n";
      if (pipelined_) src_ << "  akg::PackedChunk<" << tag << ", V> akg_b_set" << i << "[CH];\n";
    }
    const char *kStripIndex =
        "    const long akg_o = akg_strip / STRIPS;\n"
        "    const long akg_col = (akg_strip % STRIPS) * (LX * V) + lx * V;   // first column of this thread's chunks\n"
        "    const int akg_cols = akg_col >= INNER ? 0 : (INNER - akg_col < V ? static_cast<int>(INNER - akg_col) : V);   // columns inside the tensor\n"
        "    bool akg_row_ok[CH];\n"
        "#pragma unroll\n"
        "    for (int j = 0; j < CH; ++j) akg_row_ok[j] = ly + j * LY < RUN;\n";
    // ---- loads of a strip's resident chunks ----
    src_ << "  auto akg_load = [&](long akg_strip" << packedParams << ") {\n" << kStripIndex;
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      const int t = g_.inputs[i];
      const TensorValue &tv = g_.tensor(t);
      const Flags f = flags_[static_cast<size_t>(t)];
      if (!tv.used || f.rank() != Rank::Full) continue;
      const std::string tag = dtypeTag(tv.dtype), in = "in" + std::to_string(i);
      line("#pragma unroll");
      line("    for (int j = 0; j < CH; ++j) {");
      src_ << "      const " << tag << "::storage *akg_p = " << in << " + " << offsetExpr(f, "ly + j * LY", "akg_col") << ";\n";
      if (aligned_) {
        src_ << "      if (akg_row_ok[j] && akg_cols == V) akg::load_packed<" << tag << ", V, true>(akg_p, p_in" << i << "[j]);\n";
        src_ << "      else akg::zero_packed(p_in" << i << "[j]);\n";
      } else {
        src_ << "      akg::load_packed_partial<" << tag << ", V>(akg_p, akg_row_ok[j] ? akg_cols : 0, p_in" << i << "[j]);\n";
      }
      line("    }");
    }
    line("  };");
    // ---- the work on one strip ----
    // (akg_between runs behind the loads of the strip's small inputs: the place to issue the next strip's resident loads,
    // which then return after them)
    src_ << "  auto akg_work = [&](long akg_strip" << packedParams << ", auto akg_between) {\n" << kStripIndex;

    // ---- inputs ----
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      const int t = g_.inputs[i];
      const TensorValue &tv = g_.tensor(t);
      if (!tv.used) continue;
      const Flags f = flags_[static_cast<size_t>(t)];
      const std::string tag = dtypeTag(tv.dtype), ct = computeTypeName(tv.dtype), in = "in" + std::to_string(i);
      Val &v = vals_[static_cast<size_t>(t)];
      v.rank = f.rank();
      v.level = 0;
      switch (v.rank) {
        case Rank::Full: {
          // kept as it came from memory (akg_load); unpacked at the top of every walk
          v.defined = false;   // defined inside the walks
          v.ident = id("x", static_cast<int>(i));
          break;
        }
        case Rank::Col: {
          v.ident = id("c_in", static_cast<int>(i));
          src_ << "  " << ct << " " << v.ident << "[V];  // " << tv.name << "\n";
          line("  {");
          src_ << "    akg::PackedChunk<" << tag << ", V> akg_c;\n";
          src_ << "    akg::load_packed_partial<" << tag << ", V>(" << in << " + " << offsetExpr(f, "0", "akg_col") << ", akg_cols, akg_c);\n";
          src_ << "    akg::unpack_packed(akg_c, " << v.ident << ");\n";
          line("  }");
          v.defined = true;
          break;
        }
        case Rank::RowS: {
          v.ident = id("r_in", static_cast<int>(i));
          src_ << "  " << ct << " " << v.ident << "[CH];  // " << tv.name << "\n";
          line("#pragma unroll");
          src_ << "  for (int j = 0; j < CH; ++j) " << v.ident << "[j] = " << tag << "::load(akg_row_ok[j] ? " << in << "["
               << offsetExpr(f, "ly + j * LY", "0") << "] : " << tag << "::storage());\n";
          v.defined = true;
          break;
        }
        default: {
          v.ident = id("s_in", static_cast<int>(i));
          src_ << "  const " << ct << " " << v.ident << " = " << tag << "::load(" << in << "[" << offsetExpr(f, "0", "0") << "]);  // " << tv.name << "\n";
          v.defined = true;
        }
      }
    }

    line("    akg_between();");

    // ---- one walk per level ----
    for (int walk = 0; walk <= maxLevel_; ++walk) {
      std::vector<const OpNode *> reduces;
      for (const OpNode &op : g_.ops) {
        if (lowering::isReduceKind(op.kind) && level_[static_cast<size_t>(op.inputs[0])] == walk) reduces.push_back(&op);
      }
      src_ << "  // ---- walk " << walk << " ----\n";
      // values that do not vary along the run, or only along it: once, in front of the walk
      emitOps(Rank::Scalar, 0, walk, "  ");
      emitOps(Rank::Col, 0, walk, "  ");
      emitOps(Rank::RowS, 0, walk, "  ");
      const bool last = walk == maxLevel_;
      bool fullOutputs = false;
      for (int o : g_.outputs) fullOutputs = fullOutputs || flags_[static_cast<size_t>(o)].rank() == Rank::Full;
      if (reduces.empty() && !(last && fullOutputs)) continue;
      for (const OpNode *op : reduces) {
        const int out = op->outputs[0];
        const DType od = g_.tensor(out).dtype;
        const lowering::ReduceSpec spec = lowering::reduceSpec(*op, od);
        src_ << "  " << computeTypeName(od) << " acc" << out << "[V];  // " << op->name << " -> " << g_.tensor(out).name << "\n";
        line("#pragma unroll");
        src_ << "  for (int e = 0; e < V; ++e) acc" << out << "[e] = " << spec.init << ";\n";
        if (spec.ordered) {
          src_ << "  " << computeTypeName(od) << " own" << out << "[NOWN];\n";
          line("#pragma unroll");
          src_ << "  for (int k = 0; k < NOWN; ++k) own" << out << "[k] = " << spec.init << ";\n";
        }
      }
      line("#pragma unroll");
      line("  for (int j = 0; j < CH; ++j) {");
      for (size_t i = 0; i < g_.inputs.size(); ++i) {
        const int t = g_.inputs[i];
        const TensorValue &tv = g_.tensor(t);
        Val &v = vals_[static_cast<size_t>(t)];
        if (!tv.used || v.rank != Rank::Full) continue;
        // (two sets of resident chunks leave no registers for what a walk could hand to the next one)
        if (pipelined_ && walk > 0) src_ << "    akg::forget_derived(p_in" << i << "[j]);\n";
        src_ << "    " << computeTypeName(tv.dtype) << " " << v.ident << "[V];\n";
        src_ << "    akg::unpack_packed(p_in" << i << "[j], " << v.ident << ");\n";
        v.defined = true;
      }
      emitOps(Rank::Full, 0, walk, "    ");
      for (const OpNode *op : reduces) {
        const int out = op->outputs[0];
        const DType od = g_.tensor(out).dtype;
        const lowering::ReduceSpec spec = lowering::reduceSpec(*op, od);
        const Val &in = vals_[static_cast<size_t>(op->inputs[0])];
        if (!in.defined || in.rank != Rank::Full) throw LoweringError("op " + op->name + ": operand is not computed in its walk");
        if (spec.ordered) {
          // rows j * LY .. j * LY + LY - 1 of the run are this step's: through LDS, folded in order by the columns' owners
          src_ << "    akg::column_chain_step<" << spec.combiner << ", " << dtypeTag(od) << ", LX, BLOCK, V, NOWN>(own" << out << ", " << in.ident
               << ", reinterpret_cast<" << dtypeTag(od) << "::storage *>(akg_chain), tid, static_cast<int>(RUN - j * LY < LY ? RUN - j * LY : LY));\n";
          continue;
        }
        std::string step = spec.combiner + "::apply(acc" + std::to_string(out) + "[e], " + in.ident + "[e])";
        if (spec.roundEachStep) step = std::string(dtypeTag(od)) + "::rnd(" + step + ")";
        line("#pragma unroll");
        src_ << "    for (int e = 0; e < V; ++e) {\n";
        src_ << "      if (akg_row_ok[j]) acc" << out << "[e] = " << step << ";\n";
        src_ << "    }\n";
      }
      if (last) {
        for (size_t i = 0; i < g_.outputs.size(); ++i) {
          const int t = g_.outputs[i];
          const Flags f = flags_[static_cast<size_t>(t)];
          if (f.rank() != Rank::Full) continue;
          const Val &v = vals_[static_cast<size_t>(t)];
          if (!v.defined) throw LoweringError("output " + g_.tensor(t).name + " is never computed");
          const std::string tag = dtypeTag(g_.tensor(t).dtype), ct = computeTypeName(g_.tensor(t).dtype);
          std::string src = v.ident;
          if (v.rank != Rank::Full) {
            // a value of lower rank broadcast over the elements
            src = "akg_b" + std::to_string(i);
            src_ << "    " << ct << " " << src << "[V];\n";
            line("#pragma unroll");
            src_ << "    for (int e = 0; e < V; ++e) " << src << "[e] = " << operandExpr(t) << ";\n";
          }
          src_ << "    " << tag << "::storage *akg_q" << i << " = out" << i << " + " << offsetExpr(f, "ly + j * LY", "akg_col") << ";\n";
          if (aligned_) {
            src_ << "    if (akg_row_ok[j] && akg_cols == V) akg::store_chunk<" << tag << ", V, true>(akg_q" << i << ", " << src << ");\n";
          } else {
            src_ << "    akg::store_chunk_partial<" << tag << ", V>(akg_q" << i << ", akg_row_ok[j] ? akg_cols : 0, " << src << ");\n";
          }
        }
      }
      line("  }");
      forgetFull();
      for (const OpNode *op : reduces) {
        const int out = op->outputs[0];
        const DType od = g_.tensor(out).dtype;
        const lowering::ReduceSpec spec = lowering::reduceSpec(*op, od);
        const std::string ct = computeTypeName(od);
        if (spec.ordered) {
          src_ << "  akg::column_chain_finish<" << dtypeTag(od) << ", LX, BLOCK, V, NOWN>(own" << out << ", acc" << out << ", akg_chain_res, tid);\n";
          Val &v = vals_[static_cast<size_t>(out)];
          v.defined = true;
          v.rank = Rank::Col;
          v.ident = "acc" + std::to_string(out);
          v.level = walk + 1;
          continue;
        }
        const std::string scratch = block_ > 64 ? "reinterpret_cast<" + ct + " *>(akg_scratch[" + std::to_string(reduceCount_ & 1) + "])"
                                                : "static_cast<" + ct + " *>(nullptr)";
        src_ << "  akg::column_reduce<" << spec.combiner << ", " << dtypeTag(od) << ", " << (spec.roundEachStep ? "true" : "false")
             << ", LX, BLOCK, V>(acc" << out << ", " << scratch << ", tid);\n";
        ++reduceCount_;
        Val &v = vals_[static_cast<size_t>(out)];
        v.defined = true;
        v.rank = Rank::Col;
        v.ident = "acc" + std::to_string(out);
        v.level = walk + 1;
      }
    }
    // ---- outputs with one value per column ----
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      const int t = g_.outputs[i];
      const Flags f = flags_[static_cast<size_t>(t)];
      if (f.rank() != Rank::Col) continue;
      const Val &v = vals_[static_cast<size_t>(t)];
      if (!v.defined) throw LoweringError("output " + g_.tensor(t).name + " is never computed");
      const std::string tag = dtypeTag(g_.tensor(t).dtype), ct = computeTypeName(g_.tensor(t).dtype);
      std::string src = v.ident;
      if (v.rank != Rank::Col) {
        src = "akg_b" + std::to_string(i);
        src_ << "  " << ct << " " << src << "[V];\n";
        line("#pragma unroll");
        src_ << "  for (int e = 0; e < V; ++e) " << src << "[e] = " << v.ident << ";\n";
      }
      src_ << "  if (ly == 0) akg::store_chunk_partial<" << tag << ", V>(out" << i << " + " << offsetExpr(f, "0", "akg_col") << ", akg_cols, " << src << ");\n";
    }
    if (pipelined_ && block_ > 64) line("  __syncthreads();   // the scratch of the reductions is free for the next strip");
    line("  };");
    if (!pipelined_) {
      src_ << "  akg_load(static_cast<long>(blockIdx.x)" << packedArgsA << ");\n";
      src_ << "  akg_work(static_cast<long>(blockIdx.x)" << packedArgsA << ", [] {});\n";
    } else {
      line("  long akg_at = static_cast<long>(blockIdx.x);");
      line("  if (akg_at >= TOTAL) return;");
      src_ << "  akg_load(akg_at" << packedArgsA << ");\n";
      line("  for (;;) {");
      line("    long akg_next = akg_at + static_cast<long>(gridDim.x);");
      src_ << "    akg_work(akg_at" << packedArgsA << ", [&] { if (akg_next < TOTAL) akg_load(akg_next" << packedArgsB << "); });\n";
      line("    if (akg_next >= TOTAL) break;");
      line("    akg_at = akg_next;");
      line("    akg_next = akg_at + static_cast<long>(gridDim.x);");
      src_ << "    akg_work(akg_at" << packedArgsB << ", [&] { if (akg_next < TOTAL) akg_load(akg_next" << packedArgsA << "); });\n";
      line("    if (akg_next >= TOTAL) break;");
      line("    akg_at = akg_next;");
      line("  }");
    }
    line("}");
  }
};

}  // namespace

LoweredKernel lowerColumnToHip(const OpGraph &graph, const LoweringOptions &options) {
  ColumnEmitter emitter(graph, options);
  return emitter.run();
}

}  // namespace akg
