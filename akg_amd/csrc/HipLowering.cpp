#include "HipLowering.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <sstream>

namespace akg {

const char *kernelFamilyName(KernelFamily f) {
  switch (f) {
    case KernelFamily::Elementwise: return "elementwise";
    case KernelFamily::RowReduce: return "row_reduce";
    case KernelFamily::GemmEpilogue: return "gemm_epilogue";
    case KernelFamily::StreamReduce: return "stream_reduce";
    case KernelFamily::Indexed: return "indexed";
    case KernelFamily::SegmentSum: return "segment_sum";
  }
  return "?";
}

LoweringOptions LoweringOptions::fromEnvironment() {
  LoweringOptions o;
  auto readInt = [](const char *name) {
    const char *v = std::getenv(name);
    return (v && *v) ? std::atoi(v) : 0;
  };
  o.vec = readInt("AKG_HIP_VEC");
  o.threadsPerRow = readInt("AKG_HIP_TPR");
  o.chunks = readInt("AKG_HIP_CHUNKS");
  o.block = readInt("AKG_HIP_BLOCK");
  o.split = readInt("AKG_HIP_SPLIT");
  o.gemmVariant = readInt("AKG_HIP_GEMM_VARIANT");
  if (const char *nt = std::getenv("AKG_HIP_NT")) o.nonTemporal = (nt[0] != '0') ? 1 : 0;
  return o;
}

namespace lowering {

const char *dtypeTag(DType t) {
  switch (t) {
    case DType::Bool: return "akg::b1";
    case DType::I8: return "akg::i8";
    case DType::I16: return "akg::i16";
    case DType::I32: return "akg::i32";
    case DType::I64: return "akg::i64";
    case DType::F16: return "akg::f16";
    case DType::BF16: return "akg::bf16";
    case DType::F32: return "akg::f32";
    case DType::F64: return "akg::f64";
  }
  return "?";
}

const char *computeTypeName(DType t) {
  switch (t) {
    case DType::Bool: return "bool";
    case DType::I8:
    case DType::I16:
    case DType::I32: return "int";
    case DType::I64: return "long long";
    case DType::F16:
    case DType::BF16:
    case DType::F32: return "float";
    case DType::F64: return "double";
  }
  return "?";
}

static float roundToBf16(float f) {
  uint32_t u;
  std::memcpy(&u, &f, sizeof(u));
  if ((u & 0x7fffffffu) > 0x7f800000u) return f;
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  std::memcpy(&f, &u, sizeof(u));
  return f;
}

static float roundToF16(float f) {
  if (std::isnan(f) || std::isinf(f) || f == 0.0f) return f;
  double a = std::fabs(static_cast<double>(f));
  if (a >= 65520.0) return std::copysign(INFINITY, f);
  int e = 0;
  (void)std::frexp(a, &e);  // a = m * 2^e with m in [0.5, 1): leading bit has weight 2^(e-1)
  int lead = e - 1;
  double quantum = (lead < -14) ? std::ldexp(1.0, -24) : std::ldexp(1.0, lead - 10);
  double r = std::nearbyint(a / quantum) * quantum;  // default rounding mode: to nearest even
  return static_cast<float>(std::copysign(r, static_cast<double>(f)));
}

std::string literalFor(DType t, double value) {
  char buf[96];
  switch (t) {
    case DType::Bool: return value != 0.0 ? "true" : "false";
    case DType::I8:
    case DType::I16:
    case DType::I32: {
      long long v = static_cast<long long>(value);
      if (t == DType::I8) v = static_cast<signed char>(v);
      if (t == DType::I16) v = static_cast<short>(v);
      if (t == DType::I32) v = static_cast<int>(v);
      if (v == -2147483648LL) return "(-2147483647 - 1)";
      std::snprintf(buf, sizeof(buf), "(%lld)", v);
      return buf;
    }
    case DType::I64: {
      long long v = static_cast<long long>(value);
      if (v == (-9223372036854775807LL - 1)) return "(-9223372036854775807LL - 1)";
      std::snprintf(buf, sizeof(buf), "(%lldLL)", v);
      return buf;
    }
    case DType::F64: {
      if (std::isnan(value)) return "__builtin_nan(\"\")";
      if (std::isinf(value)) return value > 0 ? "__builtin_inf()" : "(-__builtin_inf())";
      std::snprintf(buf, sizeof(buf), "(%a)", value);
      return buf;
    }
    case DType::F16:
    case DType::BF16:
    case DType::F32: {
      float f = static_cast<float>(value);
      if (t == DType::F16) f = roundToF16(f);
      if (t == DType::BF16) f = roundToBf16(f);
      if (std::isnan(f)) return "__builtin_nanf(\"\")";
      if (std::isinf(f)) return f > 0 ? "__builtin_inff()" : "(-__builtin_inff())";
      std::snprintf(buf, sizeof(buf), "(%af)", static_cast<double>(f));
      return buf;
    }
  }
  return "0";
}

uint64_t countAlgorithmicBytes(const OpGraph &g) {
  // Every kernel input and output once. An input that is only read through Slice / StridedSlice / Gather (of which it
  // is the data operand) counts with the bytes those ops take out of it, if that is less: the rest of it is never
  // needed, and counting it would overstate the bandwidth of a kernel that rightly leaves it alone.
  uint64_t bytes = 0;
  for (int id : g.inputs) {
    const TensorValue &t = g.tensor(id);
    const uint64_t whole = static_cast<uint64_t>(t.numel()) * dtypeSize(t.dtype);
    uint64_t taken = 0;
    bool onlyTaken = true, used = false;
    for (const OpNode &op : g.ops) {
      for (size_t i = 0; i < op.inputs.size(); ++i) {
        if (op.inputs[i] != id) continue;
        used = true;
        const bool takes = (op.kind == OpKind::Slice || op.kind == OpKind::StridedSlice || op.kind == OpKind::Gather) && i == 0;
        if (!takes) {
          onlyTaken = false;
        } else {
          taken += static_cast<uint64_t>(g.tensor(op.outputs[0]).numel()) * dtypeSize(t.dtype);
        }
      }
    }
    bytes += (used && onlyTaken) ? std::min(whole, taken) : whole;
  }
  for (int id : g.outputs) bytes += static_cast<uint64_t>(g.tensor(id).numel()) * dtypeSize(g.tensor(id).dtype);
  return bytes;
}

std::vector<std::vector<int64_t>> buildShapeArgs(const OpGraph &g) {
  // One record per kernel argument: [offset, sizes..., strides...] (RecordStaticShapeArgs,
  // KernelOutliningExt.cpp:384-423). All tensors are dense row-major with offset 0.
  std::vector<std::vector<int64_t>> out;
  auto add = [&](const TensorValue &t) {
    std::vector<int64_t> rec;
    rec.push_back(0);
    for (int64_t d : t.shape) rec.push_back(d);
    std::vector<int64_t> strides(t.shape.size(), 1);
    for (int i = static_cast<int>(t.shape.size()) - 2; i >= 0; --i) {
      strides[static_cast<size_t>(i)] = strides[static_cast<size_t>(i) + 1] * t.shape[static_cast<size_t>(i) + 1];
    }
    for (int64_t s : strides) rec.push_back(s);
    out.push_back(rec);
  };
  for (int id : g.inputs) add(g.tensor(id));
  for (int id : g.outputs) add(g.tensor(id));
  return out;
}

bool isReduceKind(OpKind k) {
  return k == OpKind::ReduceSum || k == OpKind::ReduceMax || k == OpKind::ReduceMin || k == OpKind::ReduceProd ||
         k == OpKind::ReduceAll || k == OpKind::ReduceAny;
}

ReduceSpec reduceSpec(const OpNode &op, DType od) {
  ReduceSpec r;
  r.roundEachStep = (od == DType::F16 || od == DType::BF16 || od == DType::I8 || od == DType::I16);
  auto largest = [&](bool negative) -> std::string {
    // largest finite value of the result type (createFloatInitValue, MindSporeToLinalg.cpp:811-827)
    double v = 0.0;
    switch (od) {
      case DType::F16: v = 65504.0; break;
      case DType::BF16: v = 3.3895313892515355e38; break;
      case DType::F32: v = 3.4028234663852886e38; break;
      case DType::F64: v = 1.7976931348623157e308; break;
      default: break;
    }
    return literalFor(od, negative ? -v : v);
  };
  auto intLimit = [&](bool minimum) -> std::string {
    switch (od) {
      case DType::I8: return minimum ? "(-128)" : "(127)";
      case DType::I16: return minimum ? "(-32768)" : "(32767)";
      case DType::I32: return minimum ? "(-2147483647 - 1)" : "(2147483647)";
      case DType::I64: return minimum ? "(-9223372036854775807LL - 1)" : "(9223372036854775807LL)";
      default: break;
    }
    throw LoweringError("op " + op.name + ": unsupported result type");
  };
  switch (op.kind) {
    case OpKind::ReduceSum:
      if (od == DType::Bool) throw LoweringError("ReduceSum on bool is not supported");
      r.combiner = "akg::RedSum";
      r.init = literalFor(od, 0.0);
      break;
    case OpKind::ReduceProd:
      if (od == DType::Bool) throw LoweringError("ReducePrd on bool is not supported");
      r.combiner = "akg::RedProd";
      r.init = literalFor(od, 1.0);
      break;
    case OpKind::ReduceMax:
      if (od == DType::Bool) throw LoweringError("ReduceMax on bool is not supported");
      r.combiner = "akg::RedMax";
      r.init = isFloatType(od) ? largest(true) : intLimit(true);
      r.roundEachStep = false;
      break;
    case OpKind::ReduceMin:
      if (od == DType::Bool) throw LoweringError("ReduceMin on bool is not supported");
      r.combiner = "akg::RedMin";
      r.init = isFloatType(od) ? largest(false) : intLimit(false);
      r.roundEachStep = false;
      break;
    case OpKind::ReduceAll:
      if (od != DType::Bool) throw LoweringError("ReduceAll needs a bool tensor");
      r.combiner = "akg::RedAll";
      r.init = "true";
      r.roundEachStep = false;
      break;
    case OpKind::ReduceAny:
      if (od != DType::Bool) throw LoweringError("ReduceAny needs a bool tensor");
      r.combiner = "akg::RedAny";
      r.init = "false";
      r.roundEachStep = false;
      break;
    default:
      throw LoweringError("internal: not a reduction");
  }
  return r;
}

bool isElementwiseKind(OpKind k) {
  switch (k) {
    case OpKind::MatMul:
    case OpKind::Unknown:
    case OpKind::Unsupported:
    case OpKind::Transpose:
    case OpKind::Tile:
    case OpKind::Slice:
    case OpKind::StridedSlice:
    case OpKind::Pad:
    case OpKind::Concat:
    case OpKind::Gather:
    case OpKind::SegmentSum:
    case OpKind::ArgMax:
      return false;
    default:
      return !isReduceKind(k);
  }
}

std::vector<bool> relaxedPrecisionTensors(const OpGraph &g) {
  const size_t n = g.tensors.size();
  std::vector<bool> relaxed(n, false);
  if (const char *p = std::getenv("AKG_HIP_PRECISE")) {
    if (p[0] == '1') return relaxed;
  }
  // demand[t]: 0 = no consumer seen yet, 1 = relaxed is enough, 2 = needs full precision
  std::vector<int> demand(n, 0);
  auto raise = [&](int t, int d) {
    if (d > demand[static_cast<size_t>(t)]) demand[static_cast<size_t>(t)] = d;
  };
  for (int id : g.outputs) {
    const DType dt = g.tensor(id).dtype;
    raise(id, (dt == DType::F16 || dt == DType::BF16) ? 1 : 2);
  }
  for (size_t k = g.ops.size(); k-- > 0;) {
    const OpNode &op = g.ops[k];
    const int out = op.outputs[0];
    const DType od = g.tensor(out).dtype;
    int outDemand = demand[static_cast<size_t>(out)];
    if (outDemand == 0) outDemand = 2;  // dead value: be conservative
    int inDemand = outDemand;
    switch (op.kind) {
      case OpKind::Cast:
        if (!isFloatType(od)) {
          inDemand = 2;  // rounding to an integer / bool is discontinuous
        } else if ((od == DType::F16 || od == DType::BF16) && outDemand == 1) {
          inDemand = 1;
        }
        break;
      case OpKind::Assign:
        // the value also lands in the destination buffer: a float32 / integer destination needs it exact
        if (!(od == DType::F16 || od == DType::BF16)) inDemand = 2;
        break;
      case OpKind::Equal: case OpKind::NotEqual: case OpKind::Greater: case OpKind::GreaterEqual:
      case OpKind::Less: case OpKind::LessEqual: case OpKind::Floor: case OpKind::IsNan: case OpKind::IsInf:
      case OpKind::IsFinite: case OpKind::LogicalNot: case OpKind::LogicalAnd: case OpKind::LogicalOr:
      case OpKind::MatMul:
        inDemand = 2;
        break;
      default:
        if (!isFloatType(od)) inDemand = 2;
        break;
    }
    for (size_t i = 0; i < op.inputs.size(); ++i) {
      int d = inDemand;
      if (op.kind == OpKind::Select && i == 0) d = 2;
      raise(op.inputs[i], d);
    }
  }
  for (size_t t = 0; t < n; ++t) {
    const DType dt = g.tensors[t].dtype;
    relaxed[t] = demand[t] == 1 && (dt == DType::F32 || dt == DType::F16 || dt == DType::BF16);
  }
  return relaxed;
}

std::string elementwiseExpr(const OpGraph &g, const OpNode &op, const std::vector<std::string> &in, bool relaxed) {
  const DType od = g.tensor(op.outputs[0]).dtype;
  if (od == DType::F64) relaxed = false;
  const std::string tag = dtypeTag(od);
  const std::string ct = computeTypeName(od);
  auto inType = [&](size_t i) { return g.tensor(op.inputs[i]).dtype; };
  auto need = [&](size_t n) {
    if (in.size() != n) {
      throw LoweringError("op " + op.name + ": expected " + std::to_string(n) + " operands, found " +
                          std::to_string(in.size()));
    }
  };
  auto conv = [&](size_t i) {
    if (ct == computeTypeName(inType(i))) return in[i];
    return "static_cast<" + ct + ">(" + in[i] + ")";
  };
  auto asBool = [&](size_t i) {
    if (inType(i) == DType::Bool) return in[i];
    return "(" + in[i] + " != 0)";
  };
  auto rnd = [&](const std::string &e) {
    if (od == DType::F16 || od == DType::BF16 || od == DType::I8 || od == DType::I16) return tag + "::rnd(" + e + ")";
    return e;
  };
  auto arith = [&]() {
    if (od == DType::Bool) throw LoweringError("op " + op.name + ": arithmetic on bool tensors is not supported");
  };
  auto floatOnly = [&]() {
    if (!isFloatType(od)) throw LoweringError("op " + op.name + ": only floating-point tensors are supported");
  };
  auto unaryMath = [&](const char *fn, const char *fastFn = nullptr) {
    need(1);
    floatOnly();
    return rnd(std::string("akg::") + ((relaxed && fastFn) ? fastFn : fn) + "(" + conv(0) + ")");
  };
  auto binary = [&](const char *fn) {
    need(2);
    arith();
    return rnd(std::string("akg::") + fn + "(" + conv(0) + ", " + conv(1) + ")");
  };
  auto compare = [&](const char *sym) {
    need(2);
    std::string a = in[0], b = in[1];
    if (std::string(computeTypeName(inType(0))) != computeTypeName(inType(1))) {
      a = "static_cast<double>(" + a + ")";
      b = "static_cast<double>(" + b + ")";
    }
    std::string e = "(" + a + " " + sym + " " + b + ")";
    if (od == DType::Bool) return e;
    return "static_cast<" + ct + ">(" + e + ")";
  };
  auto predicate = [&](const char *fn) {
    need(1);
    if (!isFloatType(inType(0))) throw LoweringError("op " + op.name + ": operand must be floating point");
    std::string e = std::string("akg::") + fn + "(" + in[0] + ")";
    if (od == DType::Bool) return e;
    return "static_cast<" + ct + ">(" + e + ")";
  };

  switch (op.kind) {
    case OpKind::Add: return binary("op_add");
    case OpKind::Sub: return binary("op_sub");
    case OpKind::Mul: return binary("op_mul");
    case OpKind::Div: return (relaxed && isFloatType(od)) ? binary("fast_div") : binary("op_div");
    case OpKind::Maximum: return binary("op_maximum");
    case OpKind::Minimum: return binary("op_minimum");
    case OpKind::Pow: floatOnly(); return binary("op_pow");
    case OpKind::Atan2: floatOnly(); return binary("op_atan2");
    case OpKind::Neg: need(1); arith(); return rnd("akg::op_neg(" + conv(0) + ")");
    case OpKind::Abs: need(1); arith(); return rnd("akg::op_abs(" + conv(0) + ")");
    case OpKind::Square: need(1); arith(); return rnd("akg::op_mul(" + conv(0) + ", " + conv(0) + ")");
    case OpKind::Exp: return unaryMath("op_exp", "fast_exp");
    case OpKind::Log: return unaryMath("op_log", "fast_log");
    case OpKind::Tanh: return unaryMath("op_tanh", "fast_tanh");
    case OpKind::Rsqrt: return unaryMath("op_rsqrt", "fast_rsqrt");
    case OpKind::Sqrt: return unaryMath("op_sqrt", "fast_sqrt");
    case OpKind::Reciprocal: return unaryMath("op_inv", "fast_rcp");
    case OpKind::Floor: return unaryMath("op_floor");
    case OpKind::Sin: return unaryMath("op_sin");
    case OpKind::Cos: return unaryMath("op_cos");
    case OpKind::Asin: return unaryMath("op_asin");
    case OpKind::Acos: return unaryMath("op_acos");
    case OpKind::Atan: return unaryMath("op_atan");
    case OpKind::Asinh: return unaryMath("op_asinh");
    case OpKind::Acosh: return unaryMath("op_acosh");
    case OpKind::IsNan: return predicate("op_isnan");
    case OpKind::IsInf: return predicate("op_isinf");
    case OpKind::IsFinite: return predicate("op_isfinite");
    case OpKind::Equal: return compare("==");
    case OpKind::NotEqual: return compare("!=");
    case OpKind::Greater: return compare(">");
    case OpKind::GreaterEqual: return compare(">=");
    case OpKind::Less: return compare("<");
    case OpKind::LessEqual: return compare("<=");
    case OpKind::LogicalNot: {
      need(1);
      std::string e = "(!" + asBool(0) + ")";
      return od == DType::Bool ? e : "static_cast<" + ct + ">(" + e + ")";
    }
    case OpKind::LogicalAnd: {
      need(2);
      std::string e = "(" + asBool(0) + " && " + asBool(1) + ")";
      return od == DType::Bool ? e : "static_cast<" + ct + ">(" + e + ")";
    }
    case OpKind::LogicalOr: {
      need(2);
      std::string e = "(" + asBool(0) + " || " + asBool(1) + ")";
      return od == DType::Bool ? e : "static_cast<" + ct + ">(" + e + ")";
    }
    case OpKind::Select: {
      need(3);
      return "(" + asBool(0) + " ? " + conv(1) + " : " + conv(2) + ")";
    }
    case OpKind::Cast: {
      need(1);
      return std::string("akg::cast<") + tag + ", " + dtypeTag(inType(0)) + ">(" + in[0] + ")";
    }
    case OpKind::AddN: {
      if (in.empty()) throw LoweringError("op AddN: no operands");
      arith();
      std::string e = conv(0);
      for (size_t i = 1; i < in.size(); ++i) e = rnd("akg::op_add(" + e + ", " + conv(i) + ")");
      return e;
    }
    case OpKind::Reshape:
    case OpKind::BroadcastTo:
      need(1);
      return conv(0);
    case OpKind::Assign:
      need(2);
      return conv(1);  // the value; the store over the destination is the emitter's job
    default:
      break;
  }
  throw LoweringError("op " + op.name + " has no elementwise lowering");
}

}  // namespace lowering

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
    std::ostringstream note;
    note << kernelFamilyName(k.family) << " rows=" << rows_ << " cols=" << cols_ << " vec=" << vec_
         << " threads_per_row=" << tpr_ << " chunks=" << chunks_ << " rows_per_block=" << rowsPerBlock_
         << " block=" << block_ << " grid=" << grid_;
    if (overlap_ > 0) note << " tail_overlap=" << overlap_;
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
  std::vector<InputAccess> access_;  // per graph input
  std::vector<ValInfo> vals_;        // per tensor

  int vec_ = 1, tpr_ = 1, chunks_ = 1, rowsPerBlock_ = 1, block_ = 256;
  int64_t grid_ = 1;
  bool raggedCols_ = false, raggedRows_ = false, raggedFlat_ = false;
  int reduceCount_ = 0;
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
      if (lowering::isReduceKind(op.kind)) rowMode_ = true;
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
    size_t minSize = 1;
    bool any = false;
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      if (!access_[i].lastDimFull) continue;
      minSize = std::max(minSize, dtypeSize(g_.tensor(g_.inputs[i]).dtype));
      any = true;
    }
    for (int id : g_.outputs) {
      if (rowMode_ && g_.tensor(id).numel() != numel_) continue;
      minSize = std::max(minSize, dtypeSize(g_.tensor(id).dtype));
      any = true;
    }
    if (!any) minSize = 4;
    int v = opt_.vec > 0 ? opt_.vec : static_cast<int>(16 / minSize);
    v = std::max(1, std::min(v, 16));
    if ((v & (v - 1)) != 0) v = 1;
    bool inPlace = false;
    for (const OpNode &op : g_.ops) inPlace = inPlace || op.kind == OpKind::Assign;
    if (rowMode_ && useBuffers_ && !inPlace && opt_.vec == 0 && (cols_ % v) != 0 && cols_ >= 2 * v) {
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
      const int64_t rowChunks = ceilDiv(cols_, vec_);
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
      tpr_ = tpr;
      int64_t perThread = ceilDiv(cols_, static_cast<int64_t>(tpr_) * vec_);
      // More than 64 values per thread of one row-sized input, or 96 over all of them, do not stay in registers: walk the row in groups of
      // `chunks` chunks per thread instead. The walks after the first re-read the row from HBM (rows in flight exceed
      // L2), so the register-resident row is kept as long as it fits. Measured, % of the HBM peak, resident / walks:
      // 65536-wide f16 softmax (1 input, 64 values) 62.6 / 46.2; 65536-wide bf16 LayerNorm (2 inputs) 21.9 / 61.3;
      // 32768-wide LayerNorm 70.2 / 63.2; 131072-wide LayerNorm 10.6 / 50.0, softmax 30.1 / 42.3.
      const int rowPasses = opt_.gemmVariant;  // 1: force the register-resident row, 2: force the walks, 4: walks, packed if possible
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
      const bool preferPacked = rowPasses == 0 && tpr_ == 1024 && perThread * vec_ * rowInputs >= 64;
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
      raggedCols_ = (groups_ * chunks_ * tpr_ != rowChunks);
      raggedRows_ = (rows_ % rowsPerBlock_) != 0;
    } else {
      block_ = opt_.block > 0 ? opt_.block : 256;
      if (block_ % 64 != 0 || block_ > 1024) block_ = 256;
      int chunks = opt_.chunks > 0 ? opt_.chunks : std::max(1, 16 / vec_);
      // Small problems: fewer chunks per thread so the grid still covers the chip.
      while (chunks > 1 && ceilDiv(numel_, static_cast<int64_t>(block_) * vec_ * chunks) < 1024) chunks >>= 1;
      chunks_ = std::max(1, chunks);
      tpr_ = block_;
      rowsPerBlock_ = 1;
      int64_t perBlock = static_cast<int64_t>(block_) * vec_ * chunks_;
      grid_ = std::max<int64_t>(1, ceilDiv(numel_, perBlock));
      raggedFlat_ = (numel_ % perBlock) != 0;
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
    if (allFull) return "(" + rowVar + " * " + std::to_string(s[r - 1]) + "L)";
    // general leading-dim broadcast: decompose the row index over the leading dims
    std::vector<int64_t> stride(r, 0);
    int64_t acc = s[r - 1];
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
    line(") {");
    if (useBuffers_) {
      for (size_t i = 0; i < g_.inputs.size(); ++i) {
        const TensorValue &t = g_.tensor(g_.inputs[i]);
        src_ << "  const akg::Buffer b_in" << i << " = akg::make_buffer(in" << i << ", "
             << t.numel() * static_cast<int64_t>(dtypeSize(t.dtype)) << "L);\n";
      }
      for (size_t i = 0; i < g_.outputs.size(); ++i) {
        const TensorValue &t = g_.tensor(g_.outputs[i]);
        src_ << "  const akg::Buffer b_out" << i << " = akg::make_buffer(out" << i << ", "
             << t.numel() * static_cast<int64_t>(dtypeSize(t.dtype)) << "L);\n";
      }
    }
    src_ << "  constexpr int V = " << vec_ << ";\n";
    src_ << "  constexpr int NCHUNK = " << chunks_ << ";\n";
    src_ << "  constexpr int BLOCK = " << block_ << ";\n";
    src_ << "  constexpr long COLS = " << cols_ << "L;\n";
    src_ << "  constexpr long ROWS = " << rows_ << "L;\n";
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
      line("  long akg_rows[NCHUNK];");
      line("#pragma unroll");
      line("  for (int j = 0; j < NCHUNK; ++j) akg_rows[j] = akg_row;");
      if (multiPass_) {
        src_ << "  constexpr int GROUPS = " << groups_ << ";\n";
      } else {
        emitColumnsOfGroup("0");
      }
    } else {
      line("  constexpr long NUMEL = ROWS * COLS;");
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

  // Non-temporal accesses pay off when a workgroup moves whole cache lines. Rows of a row kernel that are not a
  // multiple of 64 bytes share their first and last line with the neighbouring rows, which other workgroups move:
  // with the hint such a line is dropped before the neighbour comes for it (measured on 1000-wide bf16 rows:
  // LayerNorm 62.8 % of the HBM peak with the hint, 68.4 % without; int8 quantisation 58.9 % and 66.9 %).
  bool streamsWholeLines(int tensorId) const {
    if (!nonTemporal_) return false;
    if (!rowMode_) return true;
    const int64_t rowBytes = cols_ * static_cast<int64_t>(dtypeSize(g_.tensor(tensorId).dtype));
    return rowBytes % 64 == 0 || rowBytes >= 16384;  // two shared lines in 256 or more do not matter
  }

  // Column of every chunk of the thread in group `group` of the row (an expression; "0" for the only group).
  void emitColumnsOfGroup(const std::string &group) {
    line("  long akg_cols[NCHUNK];");
    line("  bool akg_ok[NCHUNK];");
    if (overlap_ > 0) line("  bool akg_tail[NCHUNK];");
    line("#pragma unroll");
    line("  for (int j = 0; j < NCHUNK; ++j) {");
    line("    akg_cols[j] = ((static_cast<long>(" + group + ") * NCHUNK + j) * TPR + tcol) * V;");
    line(std::string("    akg_ok[j] = ") + (raggedCols_ ? "akg_cols[j] < COLS;" : "true;"));
    if (overlap_ > 0) {
      line("    akg_tail[j] = akg_cols[j] > COLS - V;");
      line("    if (akg_tail[j]) akg_cols[j] = COLS - V;");
    }
    line("  }");
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
      src_ << "    if (akg_ok[j]) {\n";
      // a tensor as large as the iteration space is read exactly once: stream it
      const bool streamed = streamsWholeLines(id) && (t.numel() == numel_) &&
                            (!multiPass_ || lastPassOfInput_[i] == pass_);
      src_ << "      akg::load_chunk<" << tag << ", V, " << (streamed ? "true" : "false") << ">("
           << memRef("in" + std::to_string(i), rowOffsetExpr(a, "akg_rows[j]") + " + akg_cols[j]") << ", " << v.ident
           << "[j]);\n";
      src_ << "    } else {\n";
      src_ << "      akg::fill_chunk<" << tag << ", V>(" << v.ident << "[j], " << tag << "::load(" << tag
           << "::storage()));\n";
      src_ << "    }\n";
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
    line("#pragma unroll");
    line("  for (int j = 0; j < NCHUNK; ++j) {");
    line("#pragma unroll");
    line("    for (int e = 0; e < V; ++e) {");
    std::string step = spec.combiner + "::apply(" + acc + ", " + in.ident + "[j][e])";
    if (spec.roundEachStep) step = tag + "::rnd(" + step + ")";
    if (overlap_ > 0) {
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
    src_ << "    if (" << guard << ") akg::store_chunk<" << tag << ", V, " << (streamsWholeLines(op.inputs[0]) ? "true" : "false") << ">("
         << memRef("in" + std::to_string(dst.inputIndex), offset) << ", " << v.ident << "[j]);  // " << op.name << " -> "
         << dst.name << "\n";
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
      src_ << "    if (" << guard << ") akg::store_chunk<" << tag << ", V, " << (streamsWholeLines(id) ? "true" : "false") << ">("
           << memRef("out" + std::to_string(i), offset) << ", " << src
           << "[j]);\n";
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

LoweredKernel lowerToHip(const OpGraph &described, const LoweringOptions &options) {
  if (described.ops.empty()) throw LoweringError("op description has no ops");
  bool hasArgMax = false;
  for (const OpNode &op : described.ops) hasArgMax = hasArgMax || op.kind == OpKind::ArgMax;
  OpGraph expanded;
  if (hasArgMax) {
    expanded = described;
    try {
      expandArgMax(&expanded);
    } catch (const TranslateError &e) {
      throw LoweringError(e.what());
    }
    for (const OpNode &op : expanded.ops) {
      if (op.kind != OpKind::Iota) continue;
      const std::vector<int64_t> &shape = expanded.tensor(op.outputs[0]).shape;
      size_t last = shape.size();
      for (size_t d = shape.size(); d-- > 0;) {
        if (shape[d] > 1) {
          last = d;
          break;
        }
      }
      if (static_cast<size_t>(op.concatAxis) != last || last + 1 != shape.size()) {
        throw LoweringError("op ArgMax: only the innermost axis has a kernel yet");
      }
    }
  }
  const OpGraph &graph = hasArgMax ? expanded : described;
  bool hasMatMul = false;
  for (const OpNode &op : graph.ops) {
    if (op.kind == OpKind::MatMul) hasMatMul = true;
  }
  for (const OpNode &op : graph.ops) {
    if (op.kind == OpKind::SegmentSum) return lowerSegmentSumToHip(graph, options);
  }
  if (wantsIndexedKernel(graph)) return lowerIndexedToHip(graph, options);
  if (hasMatMul) return lowerGemmToHip(graph, options);
  if (wantsStreamReduce(graph)) return lowerStreamReduceToHip(graph, options);
  TileEmitter emitter(graph, options);
  return emitter.run();
}

}  // namespace akg
