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
    case KernelFamily::ColumnReduce: return "column_reduce";
    case KernelFamily::Indexed: return "indexed";
    case KernelFamily::SegmentSum: return "segment_sum";
    case KernelFamily::Staged: return "staged";
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
  o.variant = readInt("AKG_HIP_VARIANT");
  if (const int cus = readInt("AKG_HIP_CUS"); cus >= 1 && cus <= 4096) o.computeUnits = cus;
  o.matmulF32Acc = readInt("AKG_HIP_MATMUL_F32_ACC") == 1;
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
      r.ordered = od == DType::F16 || od == DType::BF16;
      break;
    case OpKind::ReduceProd:
      if (od == DType::Bool) throw LoweringError("ReducePrd on bool is not supported");
      r.combiner = "akg::RedProd";
      r.init = literalFor(od, 1.0);
      r.ordered = od == DType::F16 || od == DType::BF16;
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
      case OpKind::Mul:
      case OpKind::Div: {
        // A constant factor of 1024 and more (a divisor of 1/1024 and less) would carry the absolute error of an
        // approximation (1.2e-7 for the hardware tanh form) into the 16-bit tolerance: exact operands from here on.
        if (!isFloatType(od)) inDemand = 2;
        for (size_t i = 0; i < op.inputs.size(); ++i) {
          const TensorValue &t = g.tensor(op.inputs[i]);
          if (!t.isConst) continue;
          const double c = std::fabs(t.constValue);
          const bool divisor = op.kind == OpKind::Div && i == 1;
          if (divisor ? (c <= 1.0 / 1024.0) : (c >= 1024.0)) inDemand = 2;
        }
        break;
      }
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
  // The hardware tanh form 1 - 2 / (e^2x + 1) is the one approximation whose error is ABSOLUTE (1.2e-7 near zero, where
  // the relative error is unbounded). Sums carry that error on; a product with a computed factor turns it into whatever
  // the factor's magnitude makes of it. Harmless where the factor is tied to the tanh's own argument (GELU:
  // x * (1 + tanh(f(x))) - a large x saturates the tanh, whose form is then exact); anywhere else the Tanh keeps the
  // series-near-zero implementation, whose error is relative. Forward pass over the ops:
  std::vector<std::vector<bool>> ancestors(n);       // per tensor: the tensors it is computed from (itself included)
  std::vector<int> taint(n, -1);                     // per tensor: the relaxed Tanh op whose absolute error it carries
  auto base = [&](int t) {
    // the tensor behind constant factors, casts, sign flips and reshapes
    for (;;) {
      const TensorValue &tv = g.tensor(t);
      if (tv.producer < 0) return t;
      const OpNode &p = g.ops[static_cast<size_t>(tv.producer)];
      int next = -1;
      if (p.kind == OpKind::Cast || p.kind == OpKind::Neg || p.kind == OpKind::Reshape || p.kind == OpKind::BroadcastTo) {
        next = p.inputs[0];
      } else if ((p.kind == OpKind::Mul || p.kind == OpKind::Div) && p.inputs.size() == 2) {
        if (g.tensor(p.inputs[1]).isConst) next = p.inputs[0];
        else if (p.kind == OpKind::Mul && g.tensor(p.inputs[0]).isConst) next = p.inputs[1];
      }
      if (next < 0) return t;
      t = next;
    }
  };
  for (size_t t = 0; t < n; ++t) {
    ancestors[t].assign(n, false);
    ancestors[t][t] = true;
  }
  for (size_t k = 0; k < g.ops.size(); ++k) {
    const OpNode &op = g.ops[k];
    const size_t out = static_cast<size_t>(op.outputs[0]);
    for (int in : op.inputs) {
      for (size_t a = 0; a < n; ++a) ancestors[out][a] = ancestors[out][a] || ancestors[static_cast<size_t>(in)][a];
    }
    auto precise = [&](int tanhOp) { relaxed[static_cast<size_t>(g.ops[static_cast<size_t>(tanhOp)].outputs[0])] = false; };
    switch (op.kind) {
      case OpKind::Tanh:
        if (relaxed[out]) taint[out] = static_cast<int>(k);
        break;
      case OpKind::Add: case OpKind::Sub: case OpKind::AddN: case OpKind::Neg: case OpKind::Reshape:
      case OpKind::BroadcastTo: case OpKind::Cast: case OpKind::Select: case OpKind::Maximum: case OpKind::Minimum:
      case OpKind::Abs:
        for (int in : op.inputs) {
          if (taint[static_cast<size_t>(in)] >= 0) taint[out] = taint[static_cast<size_t>(in)];
        }
        break;
      case OpKind::Mul:
      case OpKind::Div:
        for (size_t i = 0; i < op.inputs.size() && op.inputs.size() == 2; ++i) {
          const int tk = taint[static_cast<size_t>(op.inputs[i])];
          if (tk < 0) continue;
          const int other = op.inputs[1 - i];
          const int arg = g.ops[static_cast<size_t>(tk)].inputs[0];
          if (g.tensor(other).isConst && !(op.kind == OpKind::Div && i == 1)) {
            taint[out] = tk;   // (constants of 1024 and more were answered above)
          } else if (op.kind == OpKind::Mul && ancestors[static_cast<size_t>(arg)][static_cast<size_t>(base(other))]) {
            // the factor is what the tanh's argument is made of: the product's error is relative from here on
          } else {
            precise(tk);
          }
        }
        break;
      default:
        // anything else (Exp, Pow, Sqrt, a reduction ...) may amplify an absolute error near zero: keep the tanh relative
        for (int in : op.inputs) {
          if (taint[static_cast<size_t>(in)] >= 0) precise(taint[static_cast<size_t>(in)]);
        }
        break;
    }
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
    case OpKind::Asinh:
    case OpKind::Acosh: {
      // not the library functions: the reference spells them log(x + sqrt(1 + x*x)) and log(x + sqrt(x*x - 1)), one
      // arith / math op of the result type per step (createAsinhOp / createAcoshOp, MindSporeToLinalg.cpp:156-180), so a
      // large negative x cancels to log(0) and a float16 square overflows - results a caller of the reference sees
      need(1);
      floatOnly();
      const std::string x = conv(0), one = literalFor(od, 1.0);
      const std::string sq = rnd("akg::op_mul(" + x + ", " + x + ")");
      const std::string inner = op.kind == OpKind::Asinh ? rnd("akg::op_add(" + one + ", " + sq + ")")
                                                          : rnd("akg::op_sub(" + sq + ", " + one + ")");
      const std::string root = rnd("akg::op_sqrt(" + inner + ")");
      return rnd("akg::op_log(" + rnd("akg::op_add(" + x + ", " + root + ")") + ")");
    }
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
  if (wantsStreamReduce(graph)) {
    // A reduction result that meets the unreduced tensor again is not for the streaming kernels, which keep nothing of
    // what they read: the column kernel keeps the run in registers, if it fits. Failing both, the first reason stands.
    try {
      return lowerStreamReduceToHip(graph, options);
    } catch (const LoweringError &streaming) {
      if (options.variant == 7) throw;
      try {
        return lowerColumnToHip(graph, options);
      } catch (const LoweringError &) {
        throw streaming;
      }
    }
  }
  return lowerTileToHip(graph, options);
}

}  // namespace akg
