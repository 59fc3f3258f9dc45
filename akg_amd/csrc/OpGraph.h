/**
 * Typed op graph built from a MindSpore graph-kernel JSON description.
 *
 * This is the counterpart of the `mindspore`-dialect func that the reference builds in
 * akg-mlir/lib/Target/MindsporeDialect/TranslateToMindsporeDialect.cpp (MindConverter::parseJson :295,
 * MindBuilder::convertToMLIR :573, convertOpNode :826). There is no MLIR here: the JSON is the IR, and this
 * graph is what the classifier, the scheduler and the HIP emitter work on. The tensor signature is fixed
 * here exactly as the reference fixes it: inputs in `input_desc` order, then outputs in `output_desc` order.
 */
#ifndef AKG_HIP_OPGRAPH_H_
#define AKG_HIP_OPGRAPH_H_

#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace akg {

class TranslateError : public std::runtime_error {
 public:
  explicit TranslateError(const std::string &msg) : std::runtime_error(msg) {}
};

// Element types of the reference's type table (TranslateToMindsporeDialect.cpp:488-502,1409-1456).
enum class DType { Bool, I8, I16, I32, I64, F16, BF16, F32, F64 };

const char *dtypeName(DType t);       // JSON spelling ("float16", "bfloat16", ...)
size_t dtypeSize(DType t);            // bytes per element in memory (bool is one byte)
bool isFloatType(DType t);
// Parses a JSON data_type; "uint8" is treated as int8, as the reference does (:331-333,386-388,735-737).
DType parseDType(const std::string &name);

enum class OpKind {
  // unary
  Abs, Neg, Exp, Log, Tanh, Rsqrt, Sqrt, Reciprocal, Floor, Square, Sin, Cos, Asin, Acos, Atan, Asinh, Acosh,
  IsInf, IsFinite, IsNan, LogicalNot, Cast,
  // binary
  Add, Sub, Mul, Div, Maximum, Minimum, Pow, Atan2, Equal, NotEqual, Greater, GreaterEqual, Less, LessEqual,
  LogicalAnd, LogicalOr,
  // ternary
  Select,
  // reductions
  ReduceSum, ReduceMax, ReduceMin, ReduceProd, ReduceAll, ReduceAny,
  // shape
  Reshape, BroadcastTo,
  // data movement: the result is the operand read through an index map
  Transpose, Tile, Slice, StridedSlice, Pad, Concat, Gather,
  // UnsortedSegmentSum: out[ids[i], ...] += data[i, ...] over the index positions i in increasing order
  SegmentSum,
  // ArgMax over one axis: position of the first greatest element (integer result). Lowered by expandArgMax.
  ArgMax,
  // the index of every element along one axis of its (result) shape, int32; only produced by expandArgMax
  Iota,
  // contraction
  MatMul,
  // n-ary
  AddN,
  // Assign / InplaceAssign: the result is the second operand; as a side effect it is also written over the first
  // operand, which must be a kernel input (linalg.copy ins=input1 outs=input0, MindSporeToLinalg.cpp:495-524)
  Assign,
  // anything in the reference's factory that this backend has no kernel family for, and names outside the
  // factory (the reference turns those into mindspore.unknown, :874-876,939-946)
  Unsupported,
  Unknown,
};

const char *opKindName(OpKind k);

// OperatorTemplate lattice of akg-mlir/include/akg/Utils/AnalysisCommon.hpp:127; the fusion class of a kernel
// is the maximum over its ops (akg-mlir/lib/Transforms/OperatorIdentify.cpp:51-93).
enum class OperatorTemplate { Default = 0, Elementwise, Broadcast, Reshape, Transpose, Reduction, Matmul, Conv };
const char *operatorTemplateName(OperatorTemplate t);

// Reduce direction as in AnalysisCommon.hpp:138 (X = innermost axis, Y = any other single direction).
enum class ReduceDirection { Unknown = 0, X, Y, All };

struct TensorValue {
  std::string name;
  DType dtype = DType::F32;
  std::vector<int64_t> shape;
  bool isConst = false;       // scalar constant carried in the JSON ("value" on a shape-[1] op input)
  double constValue = 0.0;
  int producer = -1;          // index into OpGraph::ops, -1 for graph inputs and constants
  int inputIndex = -1;        // position in the kernel signature if this is a graph input
  int outputIndex = -1;       // position among the outputs if this is a graph output
  bool used = true;           // false for a kernel input that no op on the way to an output reads
  int64_t numel() const;
};

struct OpNode {
  std::string name;           // JSON op name, e.g. "RealDiv"
  OpKind kind = OpKind::Unknown;
  std::vector<int> inputs;    // tensor ids
  std::vector<int> outputs;   // tensor ids
  std::vector<int64_t> axes;  // reductions: normalised, sorted
  bool keepDims = false;
  bool transposeA = false;
  bool transposeB = false;
  // data-movement ops, one entry per dimension of the operand (all normalised by the translator):
  std::vector<int64_t> perm;       // Transpose: result dim d is operand dim perm[d]
  std::vector<int64_t> begin;      // Slice / StridedSlice: first index taken; Pad: elements added in front
  std::vector<int64_t> strides;    // StridedSlice: step (positive); Slice: all ones
  int64_t padValue = 0;            // Pad: the constant written outside the operand; SegmentSum: number of segments
  int64_t concatAxis = 0;          // Concat: axis along which the operands follow one another; Gather: gathered axis
  std::string ptrAddress;
};

struct OpGraph {
  std::string name;                 // JSON "op": also the host-visible function name
  std::string process;              // "cpu" | "cuda" | "aicore" | "hip"
  std::string arch;
  std::string computeCapability;
  std::vector<TensorValue> tensors;
  std::vector<OpNode> ops;
  std::vector<int> inputs;          // tensor ids in signature order
  std::vector<int> outputs;         // tensor ids in signature order

  OperatorTemplate operatorTemplate = OperatorTemplate::Default;
  ReduceDirection reduceDirection = ReduceDirection::Unknown;

  const TensorValue &tensor(int id) const { return tensors[static_cast<size_t>(id)]; }
};

// Concrete shapes for the kernel inputs of a dynamic-shape description (dimensions spelled -1), one per input in
// `input_desc` order. With a binding the translator replaces the -1s of the inputs and derives the shape of every op
// result from its operands (the job of the reference's shape-inference passes and of the runtime shape arguments of its
// dynamic kernels, LLVMParameterPacking.cpp:91-194); the result is an ordinary static graph.
struct ShapeBinding {
  std::vector<std::vector<int64_t>> inputShapes;
};

// JSON text -> op graph. Throws json::ParseError / TranslateError. Without a binding a -1 dimension is an error.
OpGraph translateJsonToOpGraph(const std::string &jsonText, const ShapeBinding *binding = nullptr);

// True if the description has a -1 dimension on any kernel input, op result or kernel output.
bool descriptionIsDynamic(const std::string &jsonText);

// ArgMax(x, axis) as ops the kernel families have: m = ReduceMax(x) (keep_dims), i = ReduceMin(Select(x == m, Iota, BIG)),
// result = Cast(Select(i == BIG, 0, i)). This restates upstream tosa.argmax's linalg lowering (LLVM 19.1.7
// TosaToLinalg ArgMaxConverter: start at index 0 with the lowest finite value, take a later element only if it is
// strictly greater under an ordered comparison): the first of equal maxima wins, NaNs are never taken, and a row that
// holds nothing above the lowest finite value gives 0. The graph's other ops are untouched.
void expandArgMax(OpGraph *graph);

// A reduction whose reduced axes all have extent 1 folds nothing: it becomes a Reshape of its operand
// (RemoveRedundantReduce.cpp:46-75 replaces the keep_dims form by the operand; the other form differs from its operand
// only in shape). Differs from evaluating the one-step reduction only for NaN under max / min and for -0.0 under sum.
void removeRedundantReduces(OpGraph *graph);

// Removes ops whose results no kernel output depends on and marks kernel inputs that nothing reads any more (they stay
// in the signature). The reference gets the same effect from MLIR's dead-code elimination in its canonicalisation runs.
void pruneDeadOps(OpGraph *graph);

// Fusion-class identification (OperatorIdentify.cpp:51-93) and reduce-direction marking
// (akg-mlir/lib/Dialect/Linalg/Transforms/MatchAndMarkReductionOps.cpp:51-88). Fills the two fields above.
void identifyOperator(OpGraph *graph);

// Human-readable dump of the graph in a `mindspore`-dialect-like spelling (for `akg-hip translate`).
std::string printOpGraph(const OpGraph &graph);

}  // namespace akg

#endif  // AKG_HIP_OPGRAPH_H_
