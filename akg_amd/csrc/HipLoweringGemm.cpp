/**
 * Lowering of the Matmul fusion class: one MatMul (int8 x int8 -> int32, or bfloat16 / float16 operands with a
 * float32 accumulator) followed by an elementwise epilogue over [M,N].
 *
 * The reference lowers MatMul to linalg.matmul and then through the same generic loop mapping as everything else
 * (akg-mlir/lib/Conversion/MindSporeToLinalg/MindSporeToLinalg.cpp:1453-1546; no tensor-core path is wired into
 * its GPU pipeline). Here the contraction runs on the MFMA units (kernels/akg_gemm_mfma.hpp) and the ops that follow
 * it in the description are emitted as an epilogue functor applied to the accumulators in registers, so the
 * [M,N] int32 / float32 intermediates never exist in memory.
 *
 * Float MatMul: the reference accumulates in the MatMul's declared result type, element by element in k order
 * (zero-filled accumulator of the output type, MindSporeToLinalg.cpp:1520-1540). The MFMA kernels serve a declared
 * float32 result (their float32 sum differs from the reference's only in the order of the additions). A declared
 * float16 / bfloat16 result means a product and a sum rounded to 16 bits at every k, which no matrix unit computes:
 * such descriptions, and the shapes and element types the MFMA kernels do not take, go to the serial kernel of
 * kernels/akg_gemm_serial.hpp, which keeps the reference's order and rounding exactly.
 *
 * Epilogue operands are classified by how they vary over the output tile:
 *   Full   [M,N]      4-element chunk per (row, 4 columns), loaded / computed per output chunk
 *   Col    [N]/[1,N]  4 values per lane, loaded / computed once per lane (a lane owns 4 fixed columns)
 *   Row    [M,1]      one value per output row
 *   Scalar [1]        one value
 */
#include <algorithm>
#include <sstream>

#include "HipLowering.h"

namespace akg {
namespace {

using lowering::computeTypeName;
using lowering::dtypeTag;

enum class EpiRank { Const = 0, Scalar = 1, Row = 2, Col = 3, Full = 4 };

struct EpiVal {
  bool defined = false;
  EpiRank rank = EpiRank::Const;
  std::string ident;
};

class GemmEmitter {
 public:
  GemmEmitter(const OpGraph &g, const LoweringOptions &o) : g_(g), opt_(o) {}

  LoweredKernel run() {
    analyse();
    pickSplit();
    emit();
    LoweredKernel k;
    k.kernelName = g_.name + "_kernel";
    k.source = src_.str();
    k.family = KernelFamily::GemmEpilogue;
    const int64_t tiles = ((m_ + 255) / 256) * ((n_ + 255) / 256);
    const int64_t gridTiles = ((tiles + 7) / 8) * 8;
    if (serial_) {
      k.grid[0] = static_cast<unsigned>(((m_ + 63) / 64) * ((n_ + 16 * epiWidth() - 1) / (16 * epiWidth())));
      k.block[0] = 256;
    } else if (skinny_) {
      const int64_t strips = (n_ + 127) / 128;
      k.grid[0] = static_cast<unsigned>(strips * kSplit_);
      if (kSplit_ > 1) {
        const int64_t groups = strips * batch_;
        k.workspaceBytes = static_cast<uint64_t>((groups * 4 + 255) / 256 * 256 + groups * kSplit_ * m_ * 128 * 4);
      }
      k.block[0] = static_cast<unsigned>(skinnyWaves() * 64);
    } else {
      k.grid[0] = static_cast<unsigned>(gridTiles * kSplit_);
      if (kSplit_ > 1) {
        const int64_t partRows = std::min<int64_t>(m_, 256);
        k.workspaceBytes = static_cast<uint64_t>((gridTiles * 4 + 255) / 256 * 256 + tiles * kSplit_ * partRows * 256 * 4);
      }
      k.block[0] = 512;
    }
    if (dyn_) {
      // the row count and the number of K splits travel as kernel arguments, and the workspace pointer is part of the
      // signature whether this shape set splits K or not
      k.scalarArgs.push_back(m_);
      k.scalarArgs.push_back(kSplit_);
      k.workspaceBytes = std::max<uint64_t>(k.workspaceBytes, 256);
    }
    k.grid[1] = static_cast<unsigned>(batch_);
    k.algorithmicBytes = lowering::countAlgorithmicBytes(g_);
    k.algorithmicOps = 2ull * static_cast<uint64_t>(batch_) * static_cast<uint64_t>(m_) * static_cast<uint64_t>(n_) *
                       static_cast<uint64_t>(k_);
    k.shapeArgs = lowering::buildShapeArgs(g_);
    std::ostringstream note;
    note << "gemm_epilogue batch=" << batch_ << " M=" << m_ << " N=" << n_ << " K=" << k_ << " transpose_b=" << (transB_ ? 1 : 0);
    if (serial_) {
      note << " serial: the reference's k-ordered sum in the declared type on the vector ALUs, tile=64x" << 16 * epiWidth()
           << " grid=" << k.grid[0];
    } else if (skinny_) {
      note << " skinny: strips of 128 columns, B straight into MFMA operands, mfma=" << mfmaName(false) << " waves=4 grid=" << k.grid[0];
    } else {
      note << " tile=256x256x" << stepK() / elemBytes() << " mfma=" << mfmaName(true) << " waves=" << (tallWavefrontTiles() ? "2x4" : "4x2") << " grid=" << k.grid[0];
    }
    if (kSplit_ > 1) note << " k_splits=" << kSplit_;
    if (roundedOnce_) note << " (AKG_HIP_MATMUL_F32_ACC: float32 accumulation rounded once to the declared 16-bit type, not the reference's per-step rounding)";
    if (dyn_) note << " (rows of A and K splits are kernel arguments: one code object for " << (skinny_ ? "up to " + std::to_string(skinnyBucket()) + " rows" : "more than 64 rows") << ")";
    k.scheduleNote = note.str();
    return k;
  }

 private:
  const OpGraph &g_;
  LoweringOptions opt_;
  std::ostringstream src_;
  int64_t m_ = 0, n_ = 0, k_ = 0, batch_ = 1;
  int kSplit_ = 1;  // workgroups per tile, each with a range of K steps (see pickSplit)
  int skinnyRows() const { return 64; }   // (96 rows: no faster than the tile kernel; 128: slower)
  int skinnyWaves() const { return opt_.block == 512 ? 8 : 4; }
  int skinnyUnroll() const { return opt_.chunks > 0 ? opt_.chunks : 2; }
  // A [N,K] weight is read in 32-byte pieces, four per cache line, by instructions that follow each other: with the
  // non-temporal hint the line is not kept for the next piece (bf16 16 x 8192 x 8192: 71 us with the hint, 37 without).
  bool skinnyNonTemporal() const { return opt_.nonTemporal != 0 && !transB_; }
  bool serial_ = false;  // no MFMA kernel takes the description: gemm_serial (akg_gemm_serial.hpp)
  int epiWidth() const { return (serial_ && n_ % 4 != 0) ? 1 : 4; }   // adjacent result columns per epilogue call
  bool skinny_ = false;  // M <= 64: the kernel that streams B straight into MFMA operands (gemm_skinny)
  // A dynamic description (extents bound per call): M and the K split are kernel arguments, so the source - and with it
  // the code object - is the same for every token count; the skinny kernel comes in three sizes (16, 32, 64 rows).
  bool dyn_ = false;
  int skinnyBucket() const { return m_ <= 16 ? 16 : (m_ <= 32 ? 32 : 64); }
  bool transB_ = false;
  bool roundedOnce_ = false;   // a 16-bit declared MatMul result on the matrix units by the caller's switch
  int matmulOp_ = -1;
  int aId_ = -1, bId_ = -1, accId_ = -1;
  std::vector<EpiVal> vals_;
  std::vector<bool> relaxed_;
  std::ostringstream members_, prepare_, apply_;
  std::vector<int> assignOnly_;   // inputs that are only written (Assign destinations the description never reads)

  DType elem_ = DType::I8;  // operand element type: I8, BF16 or F16
  int elemBytes() const { return elem_ == DType::I8 ? 1 : 2; }
  const char *mmaTraits() const {
    return elem_ == DType::I8 ? "akg::MmaI8" : (elem_ == DType::BF16 ? "akg::MmaBF16" : "akg::MmaF16");
  }
  // the skinny kernel issues 32 x 32 MFMAs (32 bytes of K), the tile kernel 16 x 16 ones (64 bytes of K)
  const char *mfmaName(bool tileKernel) const {
    if (tileKernel) return elem_ == DType::I8 ? "i32_16x16x64_i8" : (elem_ == DType::BF16 ? "f32_16x16x32_bf16" : "f32_16x16x32_f16");
    return elem_ == DType::I8 ? "i32_32x32x32_i8" : (elem_ == DType::BF16 ? "f32_32x32x16_bf16" : "f32_32x32x16_f16");
  }
  std::string accType() const { return serial_ ? computeTypeName(g_.tensor(accId_).dtype) : (elem_ == DType::I8 ? "int" : "float"); }
  int stepK() const { return 128; }   // bytes of K in one step of the tile kernel
  // 2 x 4 wavefronts of 128 x 64 instead of 4 x 2 of 64 x 128: half as many transposing reads of a row-major B (which move
  // 8 bytes a lane) for twice the 16-byte reads of A. int8 4096 x 8192 x 8192: +1.0 %, bfloat16: -0.4 %.
  // (AKG_HIP_VARIANT bit 5 takes the other one.)
  bool tallWavefrontTiles() const { return (elem_ == DType::I8 && !transB_) != ((opt_.variant & 32) != 0); }

  // Few tiles and a long K (a skinny activation in front of a big weight matrix: M = 16 .. 1024 against 8192 x 8192
  // leaves 32 .. 128 of 256 CUs busy, and the time is that of streaming the weights through those few): split K over
  // enough workgroups to fill the chip, at least four K steps each.
  void pickSplit() {
    kSplit_ = 1;
    if (serial_) return;
    dyn_ = opt_.extentAsArgument && batch_ == 1;
    // At most 64 rows of A (and K a multiple of 32 bytes): the time is that of streaming B, which gemm_skinny reads
    // straight into MFMA operands; 256 workgroups of four wavefronts (one per CU: 16 x 8192 x 8192 bf16 reaches 66 % of
    // the HBM peak with 4 splits of 64 strips, 59 % with 8, 48 % with 2; 8 wavefronts or more steps in flight change
    // nothing), each wavefront with at least 4 MFMA steps.
    // AKG_HIP_VARIANT bit 3 keeps the 256 x 256 tile kernel.
    skinny_ = m_ <= skinnyRows() && (k_ * elemBytes()) % 32 == 0 && (transB_ || n_ % 4 == 0) && !(opt_.variant & 8);
    if (skinny_) {
      const int64_t strips = (n_ + 127) / 128, steps = k_ * elemBytes() / 32;
      int64_t want = opt_.split > 0 ? opt_.split : std::max<int64_t>(1, 256 / (strips * batch_));
      want = std::min<int64_t>(want, std::max<int64_t>(1, opt_.split > 0 ? steps : steps / 16));
      // (the last workgroup of a strip adds the partials of all its splits: 16 x 8192 x 1024 takes 10.1 us with 16
      // splits, 12.9 with the 32 that would fill the chip)
      want = std::min<int64_t>(want, 16);
      while (want > 1 && strips * batch_ * want * m_ * 128 * 4 >= (1LL << 30)) --want;
      kSplit_ = static_cast<int>(want);
      return;
    }
    if (batch_ != 1) return;
    const int64_t tiles = ((m_ + 255) / 256) * ((n_ + 255) / 256);
    const int64_t steps = (k_ * elemBytes() + stepK() - 1) / stepK();
    int64_t want = opt_.split > 0 ? opt_.split : (tiles >= 192 ? 1 : std::min<int64_t>(16, (256 + tiles - 1) / tiles));
    want = std::max<int64_t>(1, std::min<int64_t>(want, opt_.split > 0 ? steps : steps / 4));
    const int64_t partRows = std::min<int64_t>(m_, 256);
    while (want > 1 && tiles * want * partRows * 256 * 4 >= (1LL << 30)) --want;
    if (opt_.split <= 0) {
      // the partials are written and read once: not more of them than four times the operands (2048^3 int8 with four
      // splits moved 134 MB of partials for 8 MB of operands and lost 12 %; bf16 with twice the operands gained 26 %)
      const int64_t operandBytes = (m_ * k_ + k_ * n_) * elemBytes();
      while (want > 1 && 2 * tiles * want * partRows * 256 * 4 > 4 * operandBytes) --want;
    }
    if (opt_.split <= 0) {
      // ... and the one workgroup that finishes a tile reads the partials of all its splits by itself: at most 1 MiB
      // of them (256 x 8192 x 8192: four splits 68.0 us bf16 / 47.3 us int8, eight 75.5 / 60.7; 128 rows: eight are best)
      want = std::min<int64_t>(want, std::max<int64_t>(1, (1LL << 20) / (partRows * 256 * 4)));
    }
    while (want > 1 && (want - 1) * ((steps + want - 1) / want) >= steps) --want;   // no empty split
    kSplit_ = static_cast<int>(std::max<int64_t>(1, want));
  }

  void analyse() {
    for (size_t i = 0; i < g_.ops.size(); ++i) {
      const OpNode &op = g_.ops[i];
      if (op.kind == OpKind::MatMul) {
        if (matmulOp_ >= 0) throw LoweringError("only one MatMul per kernel is supported");
        matmulOp_ = static_cast<int>(i);
      } else if (op.kind == OpKind::Unknown) {
        throw LoweringError("op " + op.name + " is not in the op table (mindspore.unknown cannot be legalized)");
      } else if (op.kind == OpKind::Unsupported || lowering::isReduceKind(op.kind)) {
        throw LoweringError("op " + op.name + " cannot be fused into a MatMul epilogue yet");
      }
    }
    const OpNode &mm = g_.ops[static_cast<size_t>(matmulOp_)];
    if (mm.transposeA) throw LoweringError("MatMul: transpose_a is not supported (as in the reference)");
    transB_ = mm.transposeB;
    aId_ = mm.inputs[0];
    bId_ = mm.inputs[1];
    accId_ = mm.outputs[0];
    const TensorValue &a = g_.tensor(aId_);
    const TensorValue &b = g_.tensor(bId_);
    const TensorValue &c = g_.tensor(accId_);
    if (a.inputIndex < 0 || b.inputIndex < 0) {
      throw LoweringError("MatMul operands must be kernel inputs (prologue fusion is not supported yet)");
    }
    if (a.dtype != b.dtype) throw LoweringError("MatMul: the operands must have one element type");
    if (a.dtype == DType::I8 && c.dtype == DType::I32) {
      elem_ = DType::I8;
    } else if ((a.dtype == DType::BF16 || a.dtype == DType::F16) && c.dtype == DType::F32) {
      elem_ = a.dtype;
    } else if ((a.dtype == DType::BF16 || a.dtype == DType::F16) && c.dtype == a.dtype && opt_.matmulF32Acc) {
      elem_ = a.dtype;   // the caller asked for the matrix units: float32 sum, rounded once (see LoweringOptions)
      roundedOnce_ = true;
    } else {
      // linalg.matmul converts both operands to the accumulator's element type: the same type, a wider integer, or a
      // wider float
      auto isIntType = [](DType t) { return t == DType::I8 || t == DType::I16 || t == DType::I32 || t == DType::I64; };
      const bool sameType = c.dtype == a.dtype && a.dtype != DType::Bool;
      const bool widerInt = isIntType(a.dtype) && isIntType(c.dtype) && dtypeSize(c.dtype) > dtypeSize(a.dtype);
      const bool widerFloat = isFloatType(a.dtype) && isFloatType(c.dtype) && dtypeSize(c.dtype) > dtypeSize(a.dtype);
      if (!sameType && !widerInt && !widerFloat) {
        throw LoweringError("MatMul: the result type must be the operands' type or a wider one of the same kind");
      }
      elem_ = a.dtype;
      serial_ = true;
    }
    // [M,K] x [K,N], or one leading batch dimension on all three ([B,M,K] x [B,K,N] -> [B,M,N]: linalg.batch_matmul,
    // MindSporeToLinalg.cpp:1511-1530); every batch is one grid.y slice of the same tile kernel.
    const size_t rank = a.shape.size();
    if ((rank != 2 && rank != 3) || b.shape.size() != rank || c.shape.size() != rank) {
      throw LoweringError("MatMul: operands and result must all be rank 2, or all rank 3 with one batch dimension");
    }
    const size_t o = rank - 2;
    batch_ = rank == 3 ? a.shape[0] : 1;
    if (rank == 3 && (b.shape[0] != batch_ || c.shape[0] != batch_)) throw LoweringError("MatMul: batch extents differ");
    if (batch_ < 1 || batch_ > 65535) throw LoweringError("MatMul: batch extent out of range");
    m_ = a.shape[o];
    k_ = a.shape[o + 1];
    n_ = transB_ ? b.shape[o] : b.shape[o + 1];
    const int64_t kb = transB_ ? b.shape[o + 1] : b.shape[o];
    if (kb != k_ || c.shape[o] != m_ || c.shape[o + 1] != n_) throw LoweringError("MatMul: inconsistent shapes");
    // rows of K that are not whole 16-byte pieces, N not a multiple of 4: shapes the MFMA kernels' loads do not take
    if ((k_ * elemBytes()) % 16 != 0 || n_ % 4 != 0) serial_ = true;
    if (serial_ && (m_ * k_ >= (1LL << 31) || k_ * n_ >= (1LL << 31) || m_ * n_ >= (1LL << 31))) {
      throw LoweringError("MatMul: operands of 2^31 elements and more need the MFMA kernels' shapes");
    }
    for (const OpNode &op : g_.ops) {
      if (op.kind == OpKind::MatMul) continue;
      for (int in : op.inputs) {
        if (in == aId_ || in == bId_) throw LoweringError("MatMul operands cannot also feed the epilogue");
      }
    }
    if (g_.tensor(accId_).outputIndex >= 0) {
      // the raw int32 product as an output is fine: it is just another Full value
    }
  }

  std::string ctOf(int id) const { return computeTypeName(g_.tensor(id).dtype); }
  std::string tagOf(int id) const { return dtypeTag(g_.tensor(id).dtype); }

  EpiRank classifyInput(const TensorValue &t) const {
    if (t.numel() == 1) return EpiRank::Scalar;
    // the result is addressed as [batch * M, N]: fold a leading batch dimension into the rows
    std::vector<int64_t> s = t.shape;
    while (s.size() > 3 && s.front() == 1) s.erase(s.begin());
    if (s.size() == 3) {
      if (s[0] == batch_ && s[1] == m_) {
        s = {batch_ * m_, s[2]};
      } else if (s[0] == 1 && (batch_ == 1 || s[1] == 1)) {
        s = {s[1], s[2]};
      } else {
        throw LoweringError("epilogue input " + t.name + " does not broadcast to the MatMul result");
      }
    }
    if (s.size() == 1) s.insert(s.begin(), 1);
    if (s.size() != 2) throw LoweringError("epilogue input " + t.name + ": rank exceeds the output's");
    const int64_t rows = batch_ * m_;
    if (s[0] == rows && s[1] == n_) return EpiRank::Full;
    if (s[0] == 1 && s[1] == n_) return EpiRank::Col;
    if (s[0] == rows && s[1] == 1) return EpiRank::Row;
    throw LoweringError("epilogue input " + t.name + " does not broadcast to the MatMul result");
  }

  std::string operand(int id) const {
    const EpiVal &v = vals_[static_cast<size_t>(id)];
    if (!v.defined) throw LoweringError("internal: epilogue operand " + g_.tensor(id).name + " undefined");
    if (v.rank == EpiRank::Full || v.rank == EpiRank::Col) return v.ident + "[e]";
    return v.ident;
  }

  void emit() {
    vals_.assign(g_.tensors.size(), EpiVal());
    relaxed_ = lowering::relaxedPrecisionTensors(g_);
    const bool nt = opt_.nonTemporal != 0;
    const std::string W = std::to_string(epiWidth());   // result columns per epilogue call

    // accumulators
    EpiVal &acc = vals_[static_cast<size_t>(accId_)];
    acc.defined = true;
    acc.rank = EpiRank::Full;
    acc.ident = "acc";
    const DType accDt = g_.tensor(accId_).dtype;
    if (!serial_ && (accDt == DType::F16 || accDt == DType::BF16)) {
      // a 16-bit MatMul result: the float32 sum is rounded to the declared type once
      acc.ident = "accr";
      apply_ << "    float accr[4];\n#pragma unroll\n    for (int e = 0; e < 4; ++e) accr[e] = " << dtypeTag(accDt)
             << "::rnd(acc[e]);\n";
    }

    // constants
    for (size_t t = 0; t < g_.tensors.size(); ++t) {
      if (!g_.tensors[t].isConst) continue;
      vals_[t].defined = true;
      vals_[t].rank = EpiRank::Const;
      vals_[t].ident = lowering::literalFor(g_.tensors[t].dtype, g_.tensors[t].constValue);
    }
    // inputs
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      const int id = g_.inputs[i];
      if (id == aId_ || id == bId_) continue;
      const TensorValue &t = g_.tensor(id);
      if (!t.used) continue;
      const EpiRank r = classifyInput(t);
      EpiVal &v = vals_[static_cast<size_t>(id)];
      v.defined = true;
      v.rank = r;
      const std::string tag = tagOf(id), ct = ctOf(id);
      members_ << "  const " << tag << "::storage *__restrict__ in" << i << ";\n";
      switch (r) {
        case EpiRank::Scalar:
          v.ident = "s_in" + std::to_string(i);
          members_ << "  " << ct << " " << v.ident << ";\n";
          prepare_ << "    " << v.ident << " = " << tag << "::load(in" << i << "[0]);\n";
          break;
        case EpiRank::Col:
          v.ident = "c_in" + std::to_string(i);
          members_ << "  " << ct << " " << v.ident << "[" << W << "];\n";
          prepare_ << "    akg::load_chunk<" << tag << ", " << W << ", false>(in" << i << " + col, " << v.ident << ");\n";
          break;
        case EpiRank::Row:
          v.ident = "r_in" + std::to_string(i);
          apply_ << "    const " << ct << " " << v.ident << " = " << tag << "::load(in" << i << "[grow]);\n";
          break;
        case EpiRank::Full:
          v.ident = "t_in" + std::to_string(i);
          apply_ << "    " << ct << " " << v.ident << "[" << W << "];\n";
          apply_ << "    akg::load_chunk<" << tag << ", " << W << ", " << (nt ? "true" : "false") << ">(in" << i << " + grow * " << n_
                 << "L + col, " << v.ident << ");\n";
          break;
        default:
          break;
      }
    }
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      members_ << "  " << tagOf(g_.outputs[i]) << "::storage *__restrict__ out" << i << ";\n";
    }
    // ops
    for (const OpNode &op : g_.ops) {
      if (op.kind == OpKind::MatMul) continue;
      if (op.outputs.size() != 1) throw LoweringError("op " + op.name + ": multiple results are not supported");
      const int outId = op.outputs[0];
      if (op.kind == OpKind::Assign) {
        // the value is stored over the destination (a kernel input as large as the MatMul result) besides being the
        // op's result: linalg.copy ins=value outs=destination (MindSporeToLinalg.cpp:495-524). Every thread writes
        // exactly the chunk of the destination that it has read (if the description reads it at all) before.
        const TensorValue &dst = g_.tensor(op.inputs[0]);
        if (dst.inputIndex < 0 || op.inputs[0] == aId_ || op.inputs[0] == bId_ || dst.dtype != g_.tensor(outId).dtype ||
            dst.numel() != batch_ * m_ * n_ || classifyInput(dst) != EpiRank::Full) {
          throw LoweringError("op " + op.name + ": in a MatMul fusion the destination must be a kernel input of the result's shape and type (not a MatMul operand)");
        }
        const EpiVal &value = vals_[static_cast<size_t>(op.inputs[1])];
        if (!value.defined) throw LoweringError("op " + op.name + ": value is undefined");
        const std::string ct = ctOf(outId), tag = tagOf(outId);
        EpiVal &v = vals_[static_cast<size_t>(outId)];
        v.defined = true;
        v.rank = EpiRank::Full;
        v.ident = "t" + std::to_string(outId);
        std::vector<std::string> operands = {"", operand(op.inputs[1])};
        apply_ << "    " << ct << " " << v.ident << "[" << W << "];  // " << op.name << " -> " << dst.name << "\n";
        apply_ << "#pragma unroll\n    for (int e = 0; e < " << W << "; ++e) " << v.ident << "[e] = "
               << lowering::elementwiseExpr(g_, op, operands, false) << ";\n";
        if (!g_.tensor(op.inputs[0]).used || !vals_[static_cast<size_t>(op.inputs[0])].defined) {
          members_ << "  const " << tag << "::storage *__restrict__ in" << dst.inputIndex << ";\n";
          assignOnly_.push_back(dst.inputIndex);
        }
        apply_ << "    akg::store_chunk<" << tag << ", " << W << ", false>(const_cast<" << tag << "::storage *>(in" << dst.inputIndex
               << ") + grow * " << n_ << "L + col, " << v.ident << ");\n";
        continue;
      }
      bool hasRow = false, hasCol = false, hasFull = false, hasScalar = false;
      for (int in : op.inputs) {
        const EpiVal &vi = vals_[static_cast<size_t>(in)];
        if (!vi.defined) throw LoweringError("op " + op.name + ": operand " + g_.tensor(in).name + " is undefined");
        hasRow |= vi.rank == EpiRank::Row;
        hasCol |= vi.rank == EpiRank::Col;
        hasFull |= vi.rank == EpiRank::Full;
        hasScalar |= vi.rank == EpiRank::Scalar;
      }
      EpiRank rank = EpiRank::Scalar;
      if (hasFull || (hasRow && hasCol)) {
        rank = EpiRank::Full;
      } else if (hasCol) {
        rank = EpiRank::Col;
      } else if (hasRow) {
        rank = EpiRank::Row;
      }
      (void)hasScalar;
      std::vector<std::string> operands;
      for (int in : op.inputs) operands.push_back(operand(in));
      const std::string expr = lowering::elementwiseExpr(g_, op, operands, relaxed_[static_cast<size_t>(outId)]);
      EpiVal &v = vals_[static_cast<size_t>(outId)];
      v.defined = true;
      v.rank = rank;
      const std::string ct = ctOf(outId);
      const std::string comment = "  // " + op.name + " -> " + g_.tensor(outId).name + "\n";
      switch (rank) {
        case EpiRank::Full:
          v.ident = "t" + std::to_string(outId);
          apply_ << "    " << ct << " " << v.ident << "[" << W << "];" << comment;
          apply_ << "#pragma unroll\n    for (int e = 0; e < " << W << "; ++e) " << v.ident << "[e] = " << expr << ";\n";
          break;
        case EpiRank::Col:
          v.ident = "c" + std::to_string(outId);
          members_ << "  " << ct << " " << v.ident << "[" << W << "];\n";
          prepare_ << "#pragma unroll\n    for (int e = 0; e < " << W << "; ++e) " << v.ident << "[e] = " << expr << ";" << comment;
          break;
        case EpiRank::Row:
          v.ident = "r" + std::to_string(outId);
          apply_ << "    const " << ct << " " << v.ident << " = " << expr << ";" << comment;
          break;
        default:
          v.ident = "s" + std::to_string(outId);
          members_ << "  " << ct << " " << v.ident << ";\n";
          prepare_ << "    " << v.ident << " = " << expr << ";" << comment;
          break;
      }
    }
    // stores
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      const int id = g_.outputs[i];
      const TensorValue &t = g_.tensor(id);
      const EpiVal &v = vals_[static_cast<size_t>(id)];
      if (!v.defined) throw LoweringError("output " + t.name + " is never computed");
      if (t.numel() != batch_ * m_ * n_ || v.rank != EpiRank::Full) {
        throw LoweringError("output " + t.name + ": only [M,N] outputs of a MatMul fusion are supported");
      }
      apply_ << "    akg::store_chunk<" << tagOf(id) << ", " << W << ", " << (nt ? "true" : "false") << ">(out" << i << " + grow * "
             << n_ << "L + col, " << v.ident << ");\n";
    }

    const std::string kname = g_.name + "_kernel";
    src_ << "// Generated by the akg HIP lowering for gfx950. Op description: " << g_.name << "\n";
    src_ << "// family: gemm_epilogue, fusion class: " << operatorTemplateName(g_.operatorTemplate) << "\n";
    src_ << "#include \"akg_rt.hpp\"\n#include \"" << (serial_ ? "akg_gemm_serial.hpp" : "akg_gemm_mfma.hpp") << "\"\n\n";
    src_ << "namespace {\nstruct Epilogue {\n" << members_.str();
    src_ << "  AKG_DEV void prepare(long col) {\n    (void)col;\n" << prepare_.str() << "  }\n";
    src_ << "  long row0;  // first row of this batch in the [batch * M, N] view of the result\n";
    src_ << "  AKG_DEV void apply(const " << accType() << " (&acc)[" << W << "], long row, long col) {\n"
         << "    const long grow = row0 + row;\n    (void)grow;\n" << apply_.str() << "  }\n";
    src_ << "};\n}  // namespace\n\n";
    src_ << "extern \"C\" __global__ __launch_bounds__(" << (serial_ ? 256 : (skinny_ ? skinnyWaves() * 64 : 512)) << ") void " << kname << "(";
    size_t argc = 0;
    for (size_t i = 0; i < g_.inputs.size(); ++i, ++argc) {
      src_ << (argc ? ", " : "") << "const " << tagOf(g_.inputs[i]) << "::storage *__restrict__ in" << i;
    }
    for (size_t i = 0; i < g_.outputs.size(); ++i, ++argc) {
      src_ << (argc ? ", " : "") << tagOf(g_.outputs[i]) << "::storage *__restrict__ out" << i;
    }
    if (dyn_) src_ << ", const long akg_m, const long akg_ksplit";
    if (kSplit_ > 1 || dyn_) src_ << ", unsigned *__restrict__ akg_ws";
    src_ << ") {\n  Epilogue epi;\n  const long akg_batch = static_cast<long>(blockIdx.y);\n";
    if (dyn_) {
      src_ << "  epi.row0 = 0L;   // (one batch)\n";
    } else {
      src_ << "  epi.row0 = akg_batch * " << m_ << "L;\n";
    }
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      const int id = g_.inputs[i];
      const bool written = std::find(assignOnly_.begin(), assignOnly_.end(), static_cast<int>(i)) != assignOnly_.end();
      if (id == aId_ || id == bId_ || (!g_.tensor(id).used && !written)) continue;
      src_ << "  epi.in" << i << " = in" << i << ";\n";
    }
    for (size_t i = 0; i < g_.outputs.size(); ++i) src_ << "  epi.out" << i << " = out" << i << ";\n";
    if (serial_) {
      src_ << "  akg::gemm_serial<" << tagOf(aId_) << ", " << tagOf(accId_) << ", " << m_ << "L, " << n_ << "L, " << k_ << "L, "
           << (transB_ ? "true" : "false") << ", " << W << ", Epilogue>(in" << g_.tensor(aId_).inputIndex << " + akg_batch * "
           << m_ * k_ << "L, in" << g_.tensor(bId_).inputIndex << " + akg_batch * " << k_ * n_ << "L, epi);\n}\n";
      return;
    }
    if (skinny_) {
      if (dyn_) {
        src_ << "  akg::gemm_skinny<" << mmaTraits() << ", " << skinnyBucket() << "L, " << n_ << "L, " << k_ << "L, " << (transB_ ? "true" : "false")
             << ", Epilogue, 1, " << skinnyWaves() << ", " << skinnyUnroll() << ", " << (skinnyNonTemporal() ? "true" : "false") << ", true>(in"
             << g_.tensor(aId_).inputIndex << ", in" << g_.tensor(bId_).inputIndex << ", epi, akg_ws, 0L, akg_m, static_cast<int>(akg_ksplit));\n}\n";
        return;
      }
      src_ << "  akg::gemm_skinny<" << mmaTraits() << ", " << m_ << "L, " << n_ << "L, " << k_ << "L, " << (transB_ ? "true" : "false")
           << ", Epilogue, " << kSplit_ << ", " << skinnyWaves() << ", " << skinnyUnroll() << ", " << (skinnyNonTemporal() ? "true" : "false") << ">(in" << g_.tensor(aId_).inputIndex << " + akg_batch * " << m_ * k_ << "L, in"
           << g_.tensor(bId_).inputIndex << " + akg_batch * " << k_ * n_ << "L, epi, " << (kSplit_ > 1 ? "akg_ws" : "nullptr")
           << ", akg_batch * " << (n_ + 127) / 128 << "L);\n}\n";
      return;
    }
    if (dyn_) {
      src_ << "  akg::gemm_256x256<" << mmaTraits() << ", 0L, " << n_ << "L, " << k_ << "L, " << (transB_ ? "true" : "false")
           << ", Epilogue, 1, " << (tallWavefrontTiles() ? 2 : 4) << ", true>(in" << g_.tensor(aId_).inputIndex << ", in" << g_.tensor(bId_).inputIndex
           << ", epi, akg_ws, akg_m, static_cast<int>(akg_ksplit));\n}\n";
      return;
    }
    src_ << "  akg::gemm_256x256<" << mmaTraits() << ", " << m_ << "L, " << n_ << "L, " << k_ << "L, " << (transB_ ? "true" : "false")
         << ", Epilogue, " << kSplit_ << (tallWavefrontTiles() ? ", 2" : "") << ">(in" << g_.tensor(aId_).inputIndex << " + akg_batch * " << m_ * k_ << "L, in" << g_.tensor(bId_).inputIndex
         << " + akg_batch * " << k_ * n_ << "L, epi" << (kSplit_ > 1 ? ", akg_ws" : "") << ");\n}\n";
  }
};

}  // namespace

LoweredKernel lowerGemmToHip(const OpGraph &graph, const LoweringOptions &options) {
  GemmEmitter emitter(graph, options);
  return emitter.run();
}

}  // namespace akg
