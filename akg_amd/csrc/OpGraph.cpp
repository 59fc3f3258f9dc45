#include "OpGraph.h"

#include <algorithm>
#include <sstream>

#include "Json.h"

namespace akg {
namespace {

// Field names of the description format (TranslateToMindsporeDialect.cpp:55-75).
constexpr auto kProcess = "process";
constexpr auto kArch = "arch";
constexpr auto kComputeCapability = "compute_capability";
constexpr auto kTargetInfo = "target_info";
constexpr auto kInputDesc = "input_desc";
constexpr auto kOutputDesc = "output_desc";
constexpr auto kTensorName = "tensor_name";
constexpr auto kShape = "shape";
constexpr auto kDataType = "data_type";
constexpr auto kOpDesc = "op_desc";
constexpr auto kName = "name";
constexpr auto kAttr = "attr";
constexpr auto kValue = "value";
constexpr auto kPtrAddress = "ptr_address";
constexpr auto kAxis = "axis";
constexpr auto kTransposeA = "transpose_a";
constexpr auto kTransposeB = "transpose_b";

struct OpTableEntry {
  const char *name;
  OpKind kind;
};

// Op-name table: every name of MindBuilder::initMindOpFactory (:417-486). Names that this backend has no
// kernel family for are kept in the table as Unsupported so that the error says so precisely.
const OpTableEntry kOpTable[] = {
  {"Abs", OpKind::Abs},
  {"Neg", OpKind::Neg},
  {"Exp", OpKind::Exp},
  {"Log", OpKind::Log},
  {"Tanh", OpKind::Tanh},
  {"ACos", OpKind::Acos},
  {"ASin", OpKind::Asin},
  {"Sin", OpKind::Sin},
  {"Cos", OpKind::Cos},
  {"Asinh", OpKind::Asinh},
  {"Acosh", OpKind::Acosh},
  {"Atan", OpKind::Atan},
  {"Rsqrt", OpKind::Rsqrt},
  {"Floor", OpKind::Floor},
  {"Square", OpKind::Square},
  {"Sqrt", OpKind::Sqrt},
  {"IsInf", OpKind::IsInf},
  {"IsFinite", OpKind::IsFinite},
  {"IsNan", OpKind::IsNan},
  {"Reciprocal", OpKind::Reciprocal},
  {"LogicalNot", OpKind::LogicalNot},
  {"LogicalAnd", OpKind::LogicalAnd},
  {"LogicalOr", OpKind::LogicalOr},
  {"Pow", OpKind::Pow},
  {"Add", OpKind::Add},
  {"Sub", OpKind::Sub},
  {"Maximum", OpKind::Maximum},
  {"Minimum", OpKind::Minimum},
  {"Mul", OpKind::Mul},
  {"Div", OpKind::Div},
  {"RealDiv", OpKind::Div},
  {"Equal", OpKind::Equal},
  {"GreaterEqual", OpKind::GreaterEqual},
  {"Greater", OpKind::Greater},
  {"LessEqual", OpKind::LessEqual},
  {"Less", OpKind::Less},
  {"NotEqual", OpKind::NotEqual},
  {"Atan2", OpKind::Atan2},
  {"Select", OpKind::Select},
  {"ReduceMax", OpKind::ReduceMax},
  {"ReduceMin", OpKind::ReduceMin},
  {"ReduceSum", OpKind::ReduceSum},
  {"ReducePrd", OpKind::ReduceProd},
  {"ReduceAll", OpKind::ReduceAll},
  {"ReduceAny", OpKind::ReduceAny},
  {"ElemAny", OpKind::ReduceAny},
  {"ArgMax", OpKind::ArgMax},
  {"BroadcastTo", OpKind::BroadcastTo},
  {"Slice", OpKind::Slice},
  {"Tile", OpKind::Tile},
  {"Concat", OpKind::Concat},
  {"Reshape", OpKind::Reshape},
  {"Transpose", OpKind::Transpose},
  {"Split", OpKind::Slice},   // becomes one Slice per result (see the translator)
  {"Pad", OpKind::Pad},
  {"Gather", OpKind::Gather},
  {"InplaceAssign", OpKind::Assign},
  {"Assign", OpKind::Assign},
  {"UnsortedSegmentSum", OpKind::SegmentSum},
  {"StridedSlice", OpKind::StridedSlice},
  {"AddN", OpKind::AddN},
  {"MatMul", OpKind::MatMul},
  {"BatchMatMul", OpKind::MatMul},
  {"Cast", OpKind::Cast},
};

OpKind lookupOpKind(const std::string &name) {
  for (const auto &e : kOpTable) {
    if (name == e.name) return e.kind;
  }
  return OpKind::Unknown;
}

bool isReduceKind(OpKind k) {
  return k == OpKind::ReduceSum || k == OpKind::ReduceMax || k == OpKind::ReduceMin || k == OpKind::ReduceProd ||
         k == OpKind::ReduceAll || k == OpKind::ReduceAny;
}

// Ops whose second JSON input is an attribute in disguise (attrInputOpList, :123-125).
bool isIndex1DAttrAsInput(const std::string &opName, size_t inputIdx) {
  static const char *const kList[] = {"Reshape",   "BroadcastTo", "ReduceMax", "ReduceMin", "ReduceSum", "ReducePrd",
                                      "ReduceAll", "ReduceAny",   "ArgMax",    "Transpose", "Tile"};
  if (inputIdx != 1) return false;
  for (const char *n : kList) {
    if (opName == n) return true;
  }
  return false;
}

std::vector<int64_t> readShape(const json::Value &desc) {
  // A missing shape means [1] (:322-325,393-395).
  if (!desc.contains(kShape)) return {1};
  std::vector<int64_t> shape = desc.at(kShape).asIntVector();
  if (shape.empty()) return {1};
  return shape;
}

const json::Value *findAttr(const json::Value &attrs, const std::string &name) {
  for (size_t i = 0; i < attrs.size(); ++i) {
    const json::Value &a = attrs[i];
    if (a.contains(kName) && a.at(kName).isString() && a.at(kName).asString() == name) {
      return &a.at(kValue);
    }
  }
  return nullptr;
}

void checkAttrTypes(const json::Value &attrs, const std::string &opName) {
  // Attribute records are {name, data_type in {bool,str,listInt,int,float}, value}; anything else is fatal in
  // the reference (createMindsporeAttribute :504-531).
  for (size_t i = 0; i < attrs.size(); ++i) {
    const json::Value &a = attrs[i];
    if (!a.contains(kDataType)) continue;
    const std::string &t = a.at(kDataType).asString();
    if (t != "bool" && t != "str" && t != "listInt" && t != "int" && t != "float") {
      throw TranslateError("op " + opName + ": attribute type " + t + " is not supported");
    }
  }
}

class GraphBuilder {
 public:
  GraphBuilder(const json::Value &root, const ShapeBinding *binding) : root_(root), binding_(binding) {}

  OpGraph build() {
    if (!root_.isObject()) throw TranslateError("op description must be a JSON object");
    graph_.name = root_.at("op").asString();
    if (graph_.name.empty()) graph_.name = "main";
    graph_.process = root_.at(kProcess).asString();
    if (root_.contains(kTargetInfo) && root_.at(kTargetInfo).isObject()) {
      const json::Value &ti = root_.at(kTargetInfo);
      if (ti.contains(kComputeCapability) && ti.at(kComputeCapability).isString()) {
        graph_.computeCapability = ti.at(kComputeCapability).asString();
      }
      if (ti.contains(kArch) && ti.at(kArch).isString()) graph_.arch = ti.at(kArch).asString();
    }
    parseInputs();
    parseOps();
    parseOutputs();
    return std::move(graph_);
  }

 private:
  const json::Value &root_;
  const ShapeBinding *binding_;
  OpGraph graph_;
  std::map<std::string, int> operandList_;  // tensor_name -> tensor id (operandList, :110)

  int addTensor(const std::string &name, DType dtype, const std::vector<int64_t> &shape) {
    for (int64_t d : shape) {
      if (d < 0) {
        throw TranslateError("tensor " + name + ": dynamic dimensions (-1) need the shapes of a call: a dynamic description "
                             "goes through akg_hip_dynamic_create / akg_hip_dynamic_specialize (akg-hip --shapes)");
      }
      // No schedule is made for nothing: the graphs the reference cuts its fused operators from hold no empty tensor.
      if (d == 0) throw TranslateError("tensor " + name + ": an extent of 0 (empty tensors have no kernel)");
    }
    // Beyond what any device holds the schedules' 64-bit products would wrap: 2^40 elements is the limit.
    int64_t count = 1;
    for (int64_t d : shape) {
      if (d > (1LL << 40) / count) throw TranslateError("tensor " + name + ": more than 2^40 elements");
      count *= d;
    }
    TensorValue t;
    t.name = name;
    t.dtype = dtype;
    t.shape = shape;
    graph_.tensors.push_back(t);
    return static_cast<int>(graph_.tensors.size()) - 1;
  }

  void parseInputs() {
    const json::Value &inputs = root_.at(kInputDesc);
    for (size_t i = 0; i < inputs.size(); ++i) {
      // input_desc is a list of single-element lists (:320).
      const json::Value &desc = inputs[i][0];
      std::string tensorName = desc.at(kTensorName).asString();
      DType dtype = parseDType(desc.at(kDataType).asString());
      std::vector<int64_t> shape = readShape(desc);
      if (binding_ != nullptr) {
        if (binding_->inputShapes.size() != inputs.size()) {
          throw TranslateError("shape binding: " + std::to_string(binding_->inputShapes.size()) + " shapes given for " +
                               std::to_string(inputs.size()) + " kernel inputs");
        }
        const std::vector<int64_t> &bound = binding_->inputShapes[i];
        if (bound.size() != shape.size()) throw TranslateError("shape binding: rank of input " + tensorName + " differs");
        for (size_t d = 0; d < shape.size(); ++d) {
          if (bound[d] < 0 || (shape[d] >= 0 && shape[d] != bound[d])) {
            throw TranslateError("shape binding: dimension " + std::to_string(d) + " of input " + tensorName +
                                 " contradicts the description");
          }
        }
        shape = bound;
      }
      int id = addTensor(tensorName, dtype, shape);
      graph_.tensors[static_cast<size_t>(id)].inputIndex = static_cast<int>(i);
      graph_.inputs.push_back(id);
      operandList_[tensorName] = id;
    }
  }

  int operandFor(const json::Value &desc, const std::string &opName) {
    std::string tensorName = desc.at(kTensorName).asString();
    auto it = operandList_.find(tensorName);
    if (it != operandList_.end()) return it->second;
    // Not yet defined: must be a constant carried in the JSON (handleDefaultOperand :793-808).
    if (!desc.contains(kValue)) {
      throw TranslateError("op " + opName + ": operand " + tensorName + " is undefined and carries no value");
    }
    const json::Value &val = desc.at(kValue);
    std::vector<int64_t> shape = readShape(desc);
    DType dtype = parseDType(desc.at(kDataType).asString());
    double v = 0.0;
    if (val.isNumber() || val.isBool()) {
      v = val.asDouble();
    } else if (val.isArray() && val.size() == 1 && (val[0].isNumber() || val[0].isBool())) {
      v = val[0].asDouble();
    } else if (val.isArray()) {
      throw TranslateError("op " + opName + ": array-valued constant operand " + tensorName +
                           " is not supported by the HIP backend");
    } else {
      throw TranslateError("Unexpected value from const input of op: " + opName);
    }
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    if (n != 1) {
      throw TranslateError("op " + opName + ": constant operand " + tensorName + " must have one element");
    }
    int id = addTensor(tensorName, dtype, shape);
    TensorValue &t = graph_.tensors[static_cast<size_t>(id)];
    t.isConst = true;
    // Integer constants are truncated toward zero as in buildDenseElementsAttr (:1390-1393).
    t.constValue = isFloatType(dtype) ? v : static_cast<double>(static_cast<int64_t>(v));
    operandList_[tensorName] = id;
    return id;
  }

  void parseOps() {
    const json::Value &ops = root_.at(kOpDesc);
    for (size_t i = 0; i < ops.size(); ++i) {
      const json::Value &opDesc = ops[i];
      OpNode node;
      node.name = opDesc.at(kName).asString();
      node.kind = lookupOpKind(node.name);
      static const json::Value kNoAttrs;
      const json::Value &attrs = (opDesc.contains(kAttr) && opDesc.at(kAttr).isArray()) ? opDesc.at(kAttr) : kNoAttrs;
      checkAttrTypes(attrs, node.name);
      bool fakeOutput = false;
      if (const json::Value *fake = findAttr(attrs, "fake_output")) {
        fakeOutput = fake->isBool() && fake->asBool();
        if (fakeOutput && node.kind != OpKind::Assign) {
          throw TranslateError("op " + node.name + ": fake_output is only meaningful on Assign / InplaceAssign");
        }
      }
      if (opDesc.contains(kPtrAddress) && opDesc.at(kPtrAddress).isString()) {
        node.ptrAddress = opDesc.at(kPtrAddress).asString();
      }
      const json::Value &inputDesc = opDesc.at(kInputDesc);
      const json::Value &outputDesc = opDesc.at(kOutputDesc);
      if (outputDesc.size() == 0) {
        throw TranslateError("Error occurs when converting json: op name: " + node.name + " has empty outputDesc");
      }

      if (node.kind == OpKind::Unknown || node.kind == OpKind::Unsupported) {
        // Keep the node (the translator itself accepts it); the scheduler rejects the kernel.
        for (size_t j = 0; j < inputDesc.size(); ++j) {
          const json::Value &d = inputDesc[j][0];
          auto it = operandList_.find(d.at(kTensorName).asString());
          if (it != operandList_.end()) node.inputs.push_back(it->second);
        }
      } else {
        for (size_t j = 0; j < inputDesc.size(); ++j) {
          if (node.kind == OpKind::Concat) {
            // the operands of a Concat are the tensors of its input entries, normally ONE entry holding the whole
            // list (handleConcatOperands :772-791)
            for (size_t t = 0; t < inputDesc[j].size(); ++t) node.inputs.push_back(operandFor(inputDesc[j][t], node.name));
            continue;
          }
          if (isIndex1DAttrAsInput(node.name, j)) continue;
          if (node.kind == OpKind::Cast && j > 0) continue;  // convertCastOp keeps the first operand only (:1351-1360)
          if (node.kind == OpKind::StridedSlice && j > 0) continue;  // begin / end / strides carried as constants
          if (node.kind == OpKind::Gather && j > 1) continue;        // the axis carried as a constant
          if (node.kind == OpKind::SegmentSum && j > 1) continue;    // the segment count carried as a constant
          if (node.kind == OpKind::Assign && j > 1) continue;        // convertInplaceAssignOp keeps two operands (:1104-1115)
          node.inputs.push_back(operandFor(inputDesc[j][0], node.name));
        }
      }

      if (node.kind != OpKind::Unknown && node.kind != OpKind::Unsupported) {
        // how many operands the op's kind reads; everything behind the translator indexes them without looking
        const int k = static_cast<int>(node.kind);
        size_t least = 1, most = 1;
        if (k >= static_cast<int>(OpKind::Add) && k <= static_cast<int>(OpKind::LogicalOr)) least = most = 2;
        if (node.kind == OpKind::Select) least = most = 3;
        if (node.kind == OpKind::MatMul || node.kind == OpKind::Gather || node.kind == OpKind::SegmentSum ||
            node.kind == OpKind::Assign) {
          least = most = 2;
        }
        if (node.kind == OpKind::Concat || node.kind == OpKind::AddN) most = static_cast<size_t>(-1);
        if (node.inputs.size() < least || node.inputs.size() > most) {
          throw TranslateError("op " + node.name + ": " + std::to_string(node.inputs.size()) + " operands where " +
                               (most == least ? std::to_string(least) : "at least " + std::to_string(least)) + " are read");
        }
      }

      if (isReduceKind(node.kind) || node.kind == OpKind::ArgMax) {
        // Axis from the second input's value or from attr "axis" (:1280-1300); keep_dims defaults to false.
        std::vector<int64_t> axes;
        if (inputDesc.size() == 2) {
          axes = inputDesc[1][0].at(kValue).asIntVector();
        } else if (const json::Value *a = findAttr(attrs, kAxis)) {
          axes = a->asIntVector();
        } else {
          throw TranslateError("op " + node.name + ": cannot find attribute axis");
        }
        int64_t rank = static_cast<int64_t>(readShape(inputDesc[0][0]).size());
        if (axes.empty()) {
          // An empty listInt becomes [1] in createMindsporeAttribute (:516-518).
          axes.push_back(1);
        }
        for (auto &a : axes) {
          if (a < 0) a += rank;
          if (a < 0 || a >= rank) throw TranslateError("op " + node.name + ": reduce axis out of range");
        }
        std::sort(axes.begin(), axes.end());
        axes.erase(std::unique(axes.begin(), axes.end()), axes.end());
        node.axes = axes;
        if (const json::Value *k = findAttr(attrs, "keep_dims")) node.keepDims = k->asBool();
      }
      if (node.kind == OpKind::MatMul) {
        if (const json::Value *a = findAttr(attrs, kTransposeA)) node.transposeA = a->asBool();
        if (const json::Value *b = findAttr(attrs, kTransposeB)) node.transposeB = b->asBool();
      }

      if (node.kind == OpKind::SegmentSum) {
        // segment count: third input's value, else attr "numSegments" (convertUnsortedSegmentSumOp :981-1017); the
        // reference's own test descriptions spell it "num_segments", which is accepted too
        if (node.inputs.size() != 2) throw TranslateError("op " + node.name + ": needs a data and a segment-id operand");
        int64_t segments = 0;
        if (inputDesc.size() > 2 && inputDesc[2][0].contains(kValue)) {
          const json::Value &v = inputDesc[2][0].at(kValue);
          segments = v.isArray() ? v.asIntVector().at(0) : static_cast<int64_t>(v.asDouble());
        } else if (const json::Value *a = findAttr(attrs, "numSegments")) {
          segments = a->isArray() ? a->asIntVector().at(0) : static_cast<int64_t>(a->asDouble());
        } else if (const json::Value *b = findAttr(attrs, "num_segments")) {
          segments = b->isArray() ? b->asIntVector().at(0) : static_cast<int64_t>(b->asDouble());
        }
        if (segments <= 0) throw TranslateError("UnsortedSegmentSumOp must have attr: numSegments");
        const TensorValue &data = graph_.tensor(node.inputs[0]);
        const TensorValue &ids = graph_.tensor(node.inputs[1]);
        if (isFloatType(ids.dtype) || ids.dtype == DType::Bool) throw TranslateError("op " + node.name + ": segment ids must be integers");
        if (ids.shape.size() > data.shape.size() ||
            !std::equal(ids.shape.begin(), ids.shape.end(), data.shape.begin())) {
          throw TranslateError("op " + node.name + ": the segment ids must have the leading dimensions of the data");
        }
        std::vector<int64_t> expect{segments};
        expect.insert(expect.end(), data.shape.begin() + static_cast<long>(ids.shape.size()), data.shape.end());
        const std::vector<int64_t> declared = readShape(outputDesc[0]);
        int64_t n = 1, m = 1;
        for (int64_t d : expect) n *= d;
        for (int64_t d : declared) m *= d;
        if (n != m) throw TranslateError("op " + node.name + ": the declared result shape does not follow from the operands");
        node.padValue = segments;
      }
      if (node.kind == OpKind::Assign) {
        if (node.inputs.size() != 2) throw TranslateError("op " + node.name + ": needs a destination and a value operand");
        const TensorValue &dst = graph_.tensor(node.inputs[0]);
        const TensorValue &src = graph_.tensor(node.inputs[1]);
        if (dst.inputIndex < 0) throw TranslateError("op " + node.name + ": the destination must be a kernel input");
        if (dst.dtype != src.dtype || dst.numel() != src.numel()) {
          throw TranslateError("op " + node.name + ": destination and value differ in type or size");
        }
      }
      (void)fakeOutput;
      std::vector<int64_t> inferred;  // result shape derived from the operands (empty: take the declared one)
      if (node.name == "Split") {
        // handled below, once the result tensors exist
      } else if (node.kind == OpKind::Transpose || node.kind == OpKind::Tile || node.kind == OpKind::Slice ||
          node.kind == OpKind::StridedSlice || node.kind == OpKind::Pad || node.kind == OpKind::Concat ||
          node.kind == OpKind::Gather) {
        inferred = parseDataMovement(&node, attrs, inputDesc, readShape(outputDesc[0]));
      } else if (binding_ != nullptr) {
        inferred = inferResultShape(node, attrs, inputDesc, readShape(outputDesc[0]));
      }

      int opIndex = static_cast<int>(graph_.ops.size());
      for (size_t j = 0; j < outputDesc.size(); ++j) {
        const json::Value &d = outputDesc[j];
        std::string tensorName = d.at(kTensorName).asString();
        DType dtype = parseDType(d.at(kDataType).asString());
        std::vector<int64_t> shape = readShape(d);
        bool dynamic = false;
        for (int64_t e : shape) dynamic = dynamic || e < 0;
        if (dynamic && binding_ != nullptr && j == 0 && !inferred.empty()) shape = inferred;
        if (node.kind == OpKind::Assign) shape = graph_.tensor(node.inputs[0]).shape;  // (:359-364, :398-404)
        int id = addTensor(tensorName, dtype, shape);
        graph_.tensors[static_cast<size_t>(id)].producer = opIndex;
        node.outputs.push_back(id);
        operandList_[tensorName] = id;
      }
      if (node.name == "Split") {
        splitIntoSlices(node, attrs);
        continue;
      }
      graph_.ops.push_back(node);
    }
  }

  // Split (convertSplitOp :1206-1232 reads attr "axis"; the reference has no lowering for mindspore.split): result k
  // is the piece of the operand along `axis` that follows the pieces before it, each as long as its declared shape
  // says. One Slice node per result, all named Split.
  void splitIntoSlices(const OpNode &node, const json::Value &attrs) {
    if (node.inputs.size() != 1) throw TranslateError("op Split: needs exactly one operand");
    const TensorValue x = graph_.tensor(node.inputs[0]);
    const size_t rank = x.shape.size();
    int64_t axis = 0;
    if (const json::Value *a = findAttr(attrs, "axis")) axis = a->isArray() ? a->asIntVector().at(0) : static_cast<int64_t>(a->asDouble());
    if (axis < 0) axis += static_cast<int64_t>(rank);
    if (axis < 0 || axis >= static_cast<int64_t>(rank)) throw TranslateError("op Split: axis out of range");
    int64_t offset = 0;
    for (int out : node.outputs) {
      const TensorValue &y = graph_.tensor(out);
      if (y.dtype != x.dtype) throw TranslateError("op Split: operand and result element types differ");
      if (y.shape.size() != rank) throw TranslateError("op Split: a result must have the rank of the operand");
      for (size_t d = 0; d < rank; ++d) {
        if (static_cast<int64_t>(d) != axis && y.shape[d] != x.shape[d]) {
          throw TranslateError("op Split: a result differs from the operand outside the split axis");
        }
      }
      OpNode piece = node;
      piece.kind = OpKind::Slice;
      piece.outputs.assign(1, out);
      piece.begin.assign(rank, 0);
      piece.begin[static_cast<size_t>(axis)] = offset;
      piece.strides.assign(rank, 1);
      offset += y.shape[static_cast<size_t>(axis)];
      if (offset > x.shape[static_cast<size_t>(axis)]) throw TranslateError("op Split: the results exceed the operand");
      graph_.tensors[static_cast<size_t>(out)].producer = static_cast<int>(graph_.ops.size());
      graph_.ops.push_back(piece);
    }
    if (offset != x.shape[static_cast<size_t>(axis)]) throw TranslateError("op Split: the results do not cover the operand");
  }

  // Attributes of the data-movement ops, checked against the declared result shape.
  //   Transpose    perm from the second input's value or attr "perm" (convertTransposeOp :965-979)
  //   Tile         multiples from the second input's value or attr "multiples"; rank stays (convertTileOp
  //                :1126-1135, MindSporeToLinalg.cpp:970-1040)
  //   Slice        attrs "begin", "size" (-1: to the end) (convertSliceOp :1089-1101)
  //   StridedSlice attrs or constant inputs begin / end / strides, negative end counted from the back; the
  //                lowering uses these three only (MindSporeFinalizingLower.cpp:102-140): the mask attributes are ignored, as there
  //   Pad          attr "padding" = (before, after) pairs listed from the LAST dimension backwards, "value",
  //                mode "constant" (MindSporeToTosa.cpp:305-376)
  //   Concat       two operands, attr "axis" (default 0) (convertConcatOp :1117-1124)
  // Result shape of a non-data-movement op from its (already concrete) operands; used under a shape binding for
  // results declared with -1 dimensions. Elementwise ops broadcast numpy-style; reductions drop or keep their axes;
  // Reshape solves at most one unknown extent from the element count; MatMul is [M,K] x [K,N] (or [N,K]).
  std::vector<int64_t> inferResultShape(const OpNode &node, const json::Value &attrs, const json::Value &inputDesc,
                                        const std::vector<int64_t> &declared) {
    (void)inputDesc;
    bool dynamic = false;
    for (int64_t e : declared) dynamic = dynamic || e < 0;
    if (!dynamic) return {};
    auto shapeOf = [&](size_t i) { return graph_.tensor(node.inputs[i]).shape; };
    if (node.kind == OpKind::Unknown || node.kind == OpKind::Unsupported) {
      throw TranslateError("op " + node.name + ": cannot derive a dynamic result shape for an op with no lowering");
    }
    if (isReduceKind(node.kind)) {
      const std::vector<int64_t> in = shapeOf(0);
      std::vector<int64_t> out;
      for (size_t d = 0; d < in.size(); ++d) {
        const bool reduced = std::find(node.axes.begin(), node.axes.end(), static_cast<int64_t>(d)) != node.axes.end();
        if (!reduced) {
          out.push_back(in[d]);
        } else if (node.keepDims) {
          out.push_back(1);
        }
      }
      if (out.empty()) out.push_back(1);
      return out;
    }
    if (node.kind == OpKind::MatMul) {
      const std::vector<int64_t> a = shapeOf(0), b = shapeOf(1);
      if (a.size() == 3 && b.size() == 3) return {a[0], a[1], node.transposeB ? b[1] : b[2]};
      if (a.size() != 2 || b.size() != 2) throw TranslateError("op " + node.name + ": MatMul operands must be rank 2 or 3");
      return {a[0], node.transposeB ? b[0] : b[1]};
    }
    if (node.kind == OpKind::Reshape || node.kind == OpKind::BroadcastTo) {
      std::vector<int64_t> out = declared;
      if (node.kind == OpKind::BroadcastTo) {
        // unknown extents come from the operand, right-aligned
        const std::vector<int64_t> in = shapeOf(0);
        for (size_t d = 0; d < out.size(); ++d) {
          if (out[d] >= 0) continue;
          const size_t fromEnd = out.size() - 1 - d;
          if (fromEnd >= in.size()) throw TranslateError("op " + node.name + ": cannot derive the broadcast shape");
          out[d] = in[in.size() - 1 - fromEnd];
        }
        return out;
      }
      int64_t known = 1, total = graph_.tensor(node.inputs[0]).numel();
      int unknown = 0;
      for (int64_t e : out) {
        if (e < 0) {
          ++unknown;
        } else {
          known *= e;
        }
      }
      if (unknown != 1 || known == 0 || total % known != 0) {
        throw TranslateError("op " + node.name + ": a dynamic Reshape may leave exactly one extent open");
      }
      for (int64_t &e : out) {
        if (e < 0) e = total / known;
      }
      return out;
    }
    (void)attrs;
    // elementwise (incl. Cast, Select, AddN): numpy broadcasting over every operand
    std::vector<int64_t> out;
    for (size_t i = 0; i < node.inputs.size(); ++i) {
      const std::vector<int64_t> in = shapeOf(i);
      if (in.size() > out.size()) out.insert(out.begin(), in.size() - out.size(), 1);
      for (size_t d = 0; d < in.size(); ++d) {
        int64_t &o = out[out.size() - in.size() + d];
        if (o == 1) {
          o = in[d];
        } else if (in[d] != 1 && in[d] != o) {
          throw TranslateError("op " + node.name + ": operands do not broadcast under the shape binding");
        }
      }
    }
    if (out.size() != declared.size()) {
      if (out.size() < declared.size()) out.insert(out.begin(), declared.size() - out.size(), 1);
    }
    return out;
  }

  std::vector<int64_t> parseDataMovement(OpNode *node, const json::Value &attrs, const json::Value &inputDesc,
                                         const std::vector<int64_t> &outShape) {
    const std::string &nm = node->name;
    if (node->inputs.empty()) throw TranslateError("op " + nm + ": missing operand");
    const std::vector<int64_t> inShape = graph_.tensor(node->inputs[0]).shape;
    const size_t rank = inShape.size();
    auto listFrom = [&](size_t inputIdx, const char *attrName) -> std::vector<int64_t> {
      if (inputDesc.size() > inputIdx && inputDesc[inputIdx][0].contains(kValue)) {
        const json::Value &v = inputDesc[inputIdx][0].at(kValue);
        if (v.isArray()) return v.asIntVector();
        return {static_cast<int64_t>(v.asDouble())};
      }
      if (const json::Value *a = findAttr(attrs, attrName)) {
        if (a->isArray()) return a->asIntVector();
        return {static_cast<int64_t>(a->asDouble())};
      }
      throw TranslateError("op " + nm + ": cannot find attribute " + attrName);
    };
    auto needRank = [&](const std::vector<int64_t> &v, const char *what) {
      if (v.size() != rank) throw TranslateError("op " + nm + ": " + what + " must have one entry per dimension");
    };
    std::vector<int64_t> expect(rank, 0);
    switch (node->kind) {
      case OpKind::Transpose: {
        node->perm = listFrom(1, "perm");
        needRank(node->perm, "perm");
        std::vector<bool> seen(rank, false);
        for (size_t d = 0; d < rank; ++d) {
          int64_t p = node->perm[d];
          if (p < 0) p += static_cast<int64_t>(rank);
          if (p < 0 || p >= static_cast<int64_t>(rank) || seen[static_cast<size_t>(p)]) {
            throw TranslateError("op " + nm + ": perm is not a permutation");
          }
          seen[static_cast<size_t>(p)] = true;
          node->perm[d] = p;
          expect[d] = inShape[static_cast<size_t>(p)];
        }
        break;
      }
      case OpKind::Tile: {
        const std::vector<int64_t> mult = listFrom(1, "multiples");
        needRank(mult, "multiples");
        for (size_t d = 0; d < rank; ++d) {
          if (mult[d] < 1) throw TranslateError("op " + nm + ": multiples must be positive");
          expect[d] = inShape[d] * mult[d];
        }
        break;
      }
      case OpKind::Slice: {
        node->begin = listFrom(99, "begin");
        std::vector<int64_t> size = listFrom(99, "size");
        needRank(node->begin, "begin");
        needRank(size, "size");
        node->strides.assign(rank, 1);
        for (size_t d = 0; d < rank; ++d) {
          if (size[d] == -1) size[d] = inShape[d] - node->begin[d];
          if (node->begin[d] < 0 || size[d] < 0 || node->begin[d] + size[d] > inShape[d]) {
            throw TranslateError("op " + nm + ": slice exceeds the operand");
          }
          expect[d] = size[d];
        }
        break;
      }
      case OpKind::StridedSlice: {
        const bool withAttr = findAttr(attrs, "begin") != nullptr;
        node->begin = withAttr ? listFrom(99, "begin") : listFrom(1, "begin");
        std::vector<int64_t> end = withAttr ? listFrom(99, "end") : listFrom(2, "end");
        node->strides = withAttr ? listFrom(99, "strides") : listFrom(3, "strides");
        needRank(node->begin, "begin");
        needRank(end, "end");
        needRank(node->strides, "strides");
        // beginMask / endMask / ellipsisMask / newAxisMask / shrinkAxisMask are copied onto the op by the reference's
        // translator (TranslateToMindsporeDialect.cpp:1034-1087) and never read again: its lowering builds the
        // tensor.extract_slice from begin, end and strides alone (MindSporeFinalizingLower.cpp:117-124). They are
        // ignored here the same way. (A declared result that drops unit dimensions, as a shrink mask implies, is
        // refused below with every other shape that does not follow from begin / end / strides.)
        for (size_t d = 0; d < rank; ++d) {
          if (end[d] < 0) end[d] += inShape[d];
          if (node->strides[d] < 1) throw TranslateError("op " + nm + ": strides must be positive");
          if (node->begin[d] < 0 || end[d] > inShape[d] || end[d] < node->begin[d]) {
            throw TranslateError("op " + nm + ": slice exceeds the operand");
          }
          expect[d] = (end[d] - node->begin[d] + node->strides[d] - 1) / node->strides[d];
        }
        break;
      }
      case OpKind::Pad: {
        const std::vector<int64_t> padding = listFrom(99, "padding");
        if (padding.size() % 2 != 0 || padding.size() / 2 > rank) {
          throw TranslateError("op " + nm + ": padding must hold (before, after) pairs for at most every dimension");
        }
        if (const json::Value *m = findAttr(attrs, "mode")) {
          if (m->isString() && m->asString() != "constant") {
            throw TranslateError("op " + nm + ": only constant padding is supported");
          }
        }
        if (const json::Value *v = findAttr(attrs, kValue)) node->padValue = static_cast<int64_t>(v->asDouble());
        node->begin.assign(rank, 0);
        std::vector<int64_t> high(rank, 0);
        for (size_t i = 0; i < padding.size() / 2; ++i) {
          if (padding[2 * i] < 0 || padding[2 * i + 1] < 0) throw TranslateError("op " + nm + ": negative padding");
          node->begin[rank - 1 - i] = padding[2 * i];
          high[rank - 1 - i] = padding[2 * i + 1];
        }
        for (size_t d = 0; d < rank; ++d) expect[d] = inShape[d] + node->begin[d] + high[d];
        break;
      }
      case OpKind::Gather: {
        // out = data.shape[:axis] + indices.shape + data.shape[axis+1:]; axis from the third input's value or attr
        // "axis"; batch_dims must be 0 (convertGatherOp :1208-1233, MindSporeToLinalg.cpp:526-594)
        if (node->inputs.size() != 2) throw TranslateError("op " + nm + ": needs a data and an indices operand");
        int64_t axis = 0;
        if (inputDesc.size() > 2 && inputDesc[2][0].contains(kValue)) {
          const json::Value &v = inputDesc[2][0].at(kValue);
          axis = v.isArray() ? v.asIntVector().at(0) : static_cast<int64_t>(v.asDouble());
        } else if (const json::Value *a = findAttr(attrs, kAxis)) {
          axis = a->isArray() ? a->asIntVector().at(0) : static_cast<int64_t>(a->asDouble());
        }
        if (const json::Value *bd = findAttr(attrs, "batch_dims")) {
          if (bd->asDouble() != 0.0) throw TranslateError("op " + nm + ": batch_dims other than 0 is not supported");
        }
        if (axis < 0) axis += static_cast<int64_t>(rank);
        if (axis < 0 || axis >= static_cast<int64_t>(rank)) throw TranslateError("op " + nm + ": axis out of range");
        node->concatAxis = axis;
        const TensorValue &idx = graph_.tensor(node->inputs[1]);
        if (isFloatType(idx.dtype) || idx.dtype == DType::Bool) throw TranslateError("op " + nm + ": indices must be integers");
        expect.assign(inShape.begin(), inShape.begin() + axis);
        expect.insert(expect.end(), idx.shape.begin(), idx.shape.end());
        expect.insert(expect.end(), inShape.begin() + axis + 1, inShape.end());
        break;
      }
      case OpKind::Concat: {
        if (node->inputs.size() != 2) throw TranslateError("op " + nm + ": exactly two operands are supported");
        int64_t axis = 0;
        if (const json::Value *a = findAttr(attrs, kAxis)) {
          axis = a->isArray() ? a->asIntVector().at(0) : static_cast<int64_t>(a->asDouble());
        }
        if (axis < 0) axis += static_cast<int64_t>(rank);
        if (axis < 0 || axis >= static_cast<int64_t>(rank)) throw TranslateError("op " + nm + ": axis out of range");
        node->concatAxis = axis;
        const std::vector<int64_t> &other = graph_.tensor(node->inputs[1]).shape;
        if (other.size() != rank) throw TranslateError("op " + nm + ": operands differ in rank");
        for (size_t d = 0; d < rank; ++d) {
          if (static_cast<int64_t>(d) != axis && other[d] != inShape[d]) {
            throw TranslateError("op " + nm + ": operands differ outside the concatenation axis");
          }
          expect[d] = inShape[d] + (static_cast<int64_t>(d) == axis ? other[d] : 0);
        }
        break;
      }
      default:
        break;
    }
    bool dynamic = false;
    for (int64_t e : outShape) dynamic = dynamic || e < 0;
    if (!dynamic && expect != outShape) {
      throw TranslateError("op " + nm + ": the declared result shape does not follow from the operand and attributes");
    }
    return expect;
  }

  void parseOutputs() {
    const json::Value &outputs = root_.at(kOutputDesc);
    for (size_t i = 0; i < outputs.size(); ++i) {
      const json::Value &desc = outputs[i];
      std::string tensorName = desc.at(kTensorName).asString();
      auto it = operandList_.find(tensorName);
      if (it == operandList_.end()) {
        throw TranslateError("output " + tensorName + " is not produced by any op");
      }
      TensorValue &t = graph_.tensors[static_cast<size_t>(it->second)];
      DType dtype = parseDType(desc.at(kDataType).asString());
      if (dtype != t.dtype) {
        throw TranslateError("output " + tensorName + ": data_type differs between output_desc and its producer");
      }
      std::vector<int64_t> shape = readShape(desc);
      int64_t n = 1;
      bool dynamic = false;
      for (int64_t d : shape) {
        n *= d;
        dynamic = dynamic || d < 0;
      }
      const bool assigned = t.producer >= 0 && graph_.ops[static_cast<size_t>(t.producer)].kind == OpKind::Assign;
      if (assigned) {
        // a fake output: its declared shape is not binding, the destination's is (:398-404)
      } else if (dynamic && binding_ != nullptr) {
        if (shape.size() != t.shape.size()) throw TranslateError("output " + tensorName + ": rank differs from its producer");
      } else if (n != t.numel()) {
        throw TranslateError("output " + tensorName + ": shape differs between output_desc and its producer");
      }
      // A value may be returned more than once (the reference looks every output up by name and returns what it
      // finds; its own Split test description lists one result twice): every listing gets an output buffer.
      if (t.inputIndex >= 0) throw TranslateError("output " + tensorName + " aliases a kernel input");
      if (t.outputIndex < 0) t.outputIndex = static_cast<int>(i);
      graph_.outputs.push_back(it->second);
    }
    if (graph_.outputs.empty()) throw TranslateError("op description has no outputs");
  }
};

bool sameShape(const std::vector<int64_t> &a, const std::vector<int64_t> &b) { return a == b; }

OperatorTemplate templateOfOp(const OpGraph &g, const OpNode &op) {
  switch (op.kind) {
    case OpKind::ReduceSum:
    case OpKind::ReduceMax:
    case OpKind::ReduceMin:
    case OpKind::ReduceProd:
    case OpKind::ReduceAll:
    case OpKind::ReduceAny:
      return OperatorTemplate::Reduction;
    case OpKind::MatMul:
      return OperatorTemplate::Matmul;
    case OpKind::Reshape:
      return OperatorTemplate::Reshape;
    case OpKind::BroadcastTo:
    case OpKind::Tile:
      return OperatorTemplate::Broadcast;
    case OpKind::Transpose:
      return OperatorTemplate::Transpose;
    case OpKind::Slice:
    case OpKind::StridedSlice:
    case OpKind::Pad:
    case OpKind::Concat:
    case OpKind::Gather:
    case OpKind::SegmentSum:
      return OperatorTemplate::Default;  // not classified by getOperatorTemplate (OperatorIdentify.cpp:51-75)
    case OpKind::Unknown:
    case OpKind::Unsupported:
      return OperatorTemplate::Default;
    case OpKind::ArgMax:
      return OperatorTemplate::Reduction;
    case OpKind::Iota:
      return OperatorTemplate::Elementwise;
    default: {
      // Elementwise when every operand has the result's shape, Broadcast otherwise (elementwiseMatch,
      // OperatorIdentify.cpp:34-48).
      const auto &resShape = g.tensor(op.outputs[0]).shape;
      for (int in : op.inputs) {
        if (!sameShape(g.tensor(in).shape, resShape)) return OperatorTemplate::Broadcast;
      }
      return OperatorTemplate::Elementwise;
    }
  }
}

}  // namespace

int64_t TensorValue::numel() const {
  int64_t n = 1;
  for (int64_t d : shape) n *= d;
  return n;
}

const char *dtypeName(DType t) {
  switch (t) {
    case DType::Bool: return "bool";
    case DType::I8: return "int8";
    case DType::I16: return "int16";
    case DType::I32: return "int32";
    case DType::I64: return "int64";
    case DType::F16: return "float16";
    case DType::BF16: return "bfloat16";
    case DType::F32: return "float32";
    case DType::F64: return "float64";
  }
  return "?";
}

size_t dtypeSize(DType t) {
  switch (t) {
    case DType::Bool:
    case DType::I8: return 1;
    case DType::I16:
    case DType::F16:
    case DType::BF16: return 2;
    case DType::I32:
    case DType::F32: return 4;
    case DType::I64:
    case DType::F64: return 8;
  }
  return 0;
}

bool isFloatType(DType t) { return t == DType::F16 || t == DType::BF16 || t == DType::F32 || t == DType::F64; }

DType parseDType(const std::string &name) {
  if (name == "bool" || name == "int1") return DType::Bool;
  if (name == "int8" || name == "uint8" || name == "sint8") return DType::I8;
  if (name == "int16") return DType::I16;
  if (name == "int32") return DType::I32;
  if (name == "int64") return DType::I64;
  if (name == "float16") return DType::F16;
  if (name == "bfloat16") return DType::BF16;
  if (name == "float32") return DType::F32;
  if (name == "float64") return DType::F64;
  throw TranslateError("Error occurs when converting json: data type " + name + " is not supported");
}

const char *opKindName(OpKind k) {
  switch (k) {
    case OpKind::Abs: return "abs";
    case OpKind::Neg: return "neg";
    case OpKind::Exp: return "exp";
    case OpKind::Log: return "log";
    case OpKind::Tanh: return "tanh";
    case OpKind::Rsqrt: return "rsqrt";
    case OpKind::Sqrt: return "sqrt";
    case OpKind::Reciprocal: return "inv";
    case OpKind::Floor: return "floor";
    case OpKind::Square: return "square";
    case OpKind::Sin: return "sin";
    case OpKind::Cos: return "cos";
    case OpKind::Asin: return "asin";
    case OpKind::Acos: return "acos";
    case OpKind::Atan: return "atan";
    case OpKind::Asinh: return "asinh";
    case OpKind::Acosh: return "acosh";
    case OpKind::IsInf: return "isinf";
    case OpKind::IsFinite: return "isfinite";
    case OpKind::IsNan: return "isnan";
    case OpKind::LogicalNot: return "logical_not";
    case OpKind::Cast: return "cast";
    case OpKind::Add: return "add";
    case OpKind::Sub: return "sub";
    case OpKind::Mul: return "mul";
    case OpKind::Div: return "div";
    case OpKind::Maximum: return "maximum";
    case OpKind::Minimum: return "minimum";
    case OpKind::Pow: return "pow";
    case OpKind::Atan2: return "atan2";
    case OpKind::Equal: return "equal";
    case OpKind::NotEqual: return "not_equal";
    case OpKind::Greater: return "greater";
    case OpKind::GreaterEqual: return "greater_equal";
    case OpKind::Less: return "less";
    case OpKind::LessEqual: return "less_equal";
    case OpKind::LogicalAnd: return "logical_and";
    case OpKind::LogicalOr: return "logical_or";
    case OpKind::Select: return "select";
    case OpKind::ReduceSum: return "reduce_sum";
    case OpKind::ReduceMax: return "reduce_max";
    case OpKind::ReduceMin: return "reduce_min";
    case OpKind::ReduceProd: return "reduce_prod";
    case OpKind::ReduceAll: return "reduce_all";
    case OpKind::ReduceAny: return "reduce_any";
    case OpKind::Reshape: return "reshape";
    case OpKind::BroadcastTo: return "broadcast_to";
    case OpKind::Transpose: return "transpose";
    case OpKind::Tile: return "tile";
    case OpKind::Slice: return "slice";
    case OpKind::StridedSlice: return "strided_slice";
    case OpKind::Pad: return "pad";
    case OpKind::Concat: return "concat";
    case OpKind::Gather: return "gather";
    case OpKind::ArgMax: return "argmax";
    case OpKind::Iota: return "iota";
    case OpKind::SegmentSum: return "unsorted_segment_sum";
    case OpKind::MatMul: return "matmul";
    case OpKind::AddN: return "addn";
    case OpKind::Assign: return "inplace_assign";
    case OpKind::Unsupported: return "unsupported";
    case OpKind::Unknown: return "unknown";
  }
  return "?";
}

const char *operatorTemplateName(OperatorTemplate t) {
  switch (t) {
    case OperatorTemplate::Default: return "Default";
    case OperatorTemplate::Elementwise: return "Elementwise";
    case OperatorTemplate::Broadcast: return "Broadcast";
    case OperatorTemplate::Reshape: return "Reshape";
    case OperatorTemplate::Transpose: return "Transpose";
    case OperatorTemplate::Reduction: return "Reduction";
    case OperatorTemplate::Matmul: return "Matmul";
    case OperatorTemplate::Conv: return "Conv";
  }
  return "?";
}

bool descriptionIsDynamic(const std::string &jsonText) {
  const json::Value root = json::Value::parse(jsonText);
  auto dyn = [](const json::Value &desc) {
    if (!desc.contains(kShape)) return false;
    for (int64_t d : desc.at(kShape).asIntVector()) {
      if (d < 0) return true;
    }
    return false;
  };
  if (!root.isObject()) return false;
  const json::Value &inputs = root.at(kInputDesc);
  for (size_t i = 0; i < inputs.size(); ++i) {
    if (dyn(inputs[i][0])) return true;
  }
  const json::Value &ops = root.at(kOpDesc);
  for (size_t i = 0; i < ops.size(); ++i) {
    const json::Value &outs = ops[i].at(kOutputDesc);
    for (size_t j = 0; j < outs.size(); ++j) {
      if (dyn(outs[j])) return true;
    }
  }
  const json::Value &outputs = root.at(kOutputDesc);
  for (size_t i = 0; i < outputs.size(); ++i) {
    if (dyn(outputs[i])) return true;
  }
  return false;
}

OpGraph translateJsonToOpGraph(const std::string &jsonText, const ShapeBinding *binding) {
  json::Value root = json::Value::parse(jsonText);
  GraphBuilder builder(root, binding);
  OpGraph g = builder.build();
  removeRedundantReduces(&g);
  pruneDeadOps(&g);
  identifyOperator(&g);
  return g;
}

void expandArgMax(OpGraph *graph) {
  bool any = false;
  for (const OpNode &op : graph->ops) any = any || op.kind == OpKind::ArgMax;
  if (!any) return;
  const double kBig = 2147483647.0;
  std::vector<OpNode> ops;
  std::vector<int> newIndex;  // not needed by callers: producers are re-derived below
  auto addTensor = [&](const std::string &name, DType dtype, const std::vector<int64_t> &shape) {
    TensorValue t;
    t.name = name;
    t.dtype = dtype;
    t.shape = shape;
    graph->tensors.push_back(t);
    return static_cast<int>(graph->tensors.size()) - 1;
  };
  auto addConst = [&](const std::string &name, double value) {
    const int id = addTensor(name, DType::I32, {1});
    graph->tensors[static_cast<size_t>(id)].isConst = true;
    graph->tensors[static_cast<size_t>(id)].constValue = value;
    return id;
  };
  auto emit = [&](OpKind kind, const char *name, std::vector<int> inputs, int output) {
    OpNode n;
    n.kind = kind;
    n.name = name;
    n.inputs = std::move(inputs);
    n.outputs.assign(1, output);
    ops.push_back(n);
    return &ops.back();
  };
  int serial = 0;
  for (const OpNode &op : graph->ops) {
    if (op.kind != OpKind::ArgMax) {
      ops.push_back(op);
      continue;
    }
    const int x = op.inputs.at(0);
    const int out = op.outputs.at(0);
    const std::vector<int64_t> inShape = graph->tensor(x).shape;
    const DType xType = graph->tensor(x).dtype, outType = graph->tensor(out).dtype;
    if (op.axes.size() != 1) throw TranslateError("op ArgMax: exactly one axis is supported");
    if (isFloatType(outType) || outType == DType::Bool) throw TranslateError("op ArgMax: the result must be an integer tensor");
    if (xType == DType::Bool) throw TranslateError("op ArgMax: a bool operand is not supported");
    const size_t axis = static_cast<size_t>(op.axes[0]);
    if (inShape[axis] >= (1LL << 31) - 1) throw TranslateError("op ArgMax: axis too long");
    std::vector<int64_t> kept = inShape;
    kept[axis] = 1;
    const std::string base = "argmax" + std::to_string(serial++) + "_";
    const int m = addTensor(base + "max", xType, kept);
    OpNode *r = emit(OpKind::ReduceMax, "ReduceMax", {x}, m);
    r->axes = op.axes;
    r->keepDims = true;
    const int eq = addTensor(base + "hit", DType::Bool, inShape);
    emit(OpKind::Equal, "Equal", {x, m}, eq);
    const int iota = addTensor(base + "iota", DType::I32, inShape);
    emit(OpKind::Iota, "Iota", {}, iota)->concatAxis = static_cast<int64_t>(axis);
    const int big = addConst(base + "big", kBig);
    const int sel = addTensor(base + "pos", DType::I32, inShape);
    emit(OpKind::Select, "Select", {eq, iota, big}, sel);
    const std::vector<int64_t> outShape = graph->tensor(out).shape;
    const int first = addTensor(base + "first", DType::I32, outShape);
    r = emit(OpKind::ReduceMin, "ReduceMin", {sel}, first);
    r->axes = op.axes;
    r->keepDims = op.keepDims;
    const int none = addTensor(base + "none", DType::Bool, outShape);
    emit(OpKind::Equal, "Equal", {first, big}, none);
    const int zero = addConst(base + "zero", 0.0);
    if (outType == DType::I32) {
      emit(OpKind::Select, "Select", {none, zero, first}, out);
    } else {
      const int fixed = addTensor(base + "fixed", DType::I32, outShape);
      emit(OpKind::Select, "Select", {none, zero, first}, fixed);
      emit(OpKind::Cast, "Cast", {fixed}, out);
    }
  }
  graph->ops.swap(ops);
  for (TensorValue &t : graph->tensors) t.producer = -1;
  for (size_t k = 0; k < graph->ops.size(); ++k) {
    for (int id : graph->ops[k].outputs) graph->tensors[static_cast<size_t>(id)].producer = static_cast<int>(k);
  }
  (void)newIndex;
}

void removeRedundantReduces(OpGraph *graph) {
  for (OpNode &op : graph->ops) {
    if (!isReduceKind(op.kind) || op.inputs.empty()) continue;
    const std::vector<int64_t> &in = graph->tensor(op.inputs[0]).shape;
    bool redundant = true;
    for (int64_t a : op.axes) {
      if (a >= 0 && static_cast<size_t>(a) < in.size() && in[static_cast<size_t>(a)] != 1) redundant = false;
    }
    if (!redundant || graph->tensor(op.inputs[0]).dtype != graph->tensor(op.outputs[0]).dtype) continue;
    op.kind = OpKind::Reshape;
    op.axes.clear();
    op.inputs.resize(1);
  }
}

void pruneDeadOps(OpGraph *graph) {
  std::vector<bool> live(graph->tensors.size(), false);
  for (int id : graph->outputs) live[static_cast<size_t>(id)] = true;
  std::vector<bool> keep(graph->ops.size(), false);
  for (size_t k = graph->ops.size(); k-- > 0;) {
    const OpNode &op = graph->ops[k];
    // keep what must be reported, and what has a side effect
    bool needed = op.kind == OpKind::Unknown || op.kind == OpKind::Unsupported || op.kind == OpKind::Assign;
    for (int out : op.outputs) needed = needed || live[static_cast<size_t>(out)];
    if (!needed) continue;
    keep[k] = true;
    for (int in : op.inputs) live[static_cast<size_t>(in)] = true;
  }
  std::vector<int> newIndex(graph->ops.size(), -1);
  std::vector<OpNode> kept;
  for (size_t k = 0; k < graph->ops.size(); ++k) {
    if (!keep[k]) continue;
    newIndex[k] = static_cast<int>(kept.size());
    kept.push_back(graph->ops[k]);
  }
  graph->ops.swap(kept);
  for (size_t t = 0; t < graph->tensors.size(); ++t) {
    TensorValue &tv = graph->tensors[t];
    if (tv.producer >= 0) tv.producer = newIndex[static_cast<size_t>(tv.producer)];
    if (tv.inputIndex >= 0) tv.used = live[t];
  }
}

void identifyOperator(OpGraph *graph) {
  OperatorTemplate cur = OperatorTemplate::Default;
  ReduceDirection dir = ReduceDirection::Unknown;
  for (const OpNode &op : graph->ops) {
    OperatorTemplate t = templateOfOp(*graph, op);
    if (t > cur) cur = t;
    if (t == OperatorTemplate::Reduction && !op.inputs.empty()) {
      const auto &inShape = graph->tensor(op.inputs[0]).shape;
      int64_t rank = static_cast<int64_t>(inShape.size());
      // Count only axes that really reduce something (extent > 1), as size-1 axes are redundant reductions
      // (akg-mlir/lib/Dialect/MindSpore/Transforms/RemoveRedundantReduce.cpp).
      std::vector<int64_t> real;
      int64_t nonUnit = 0;
      for (int64_t d = 0; d < rank; ++d) {
        if (inShape[static_cast<size_t>(d)] > 1) ++nonUnit;
      }
      for (int64_t a : op.axes) {
        if (inShape[static_cast<size_t>(a)] > 1) real.push_back(a);
      }
      ReduceDirection d = ReduceDirection::Unknown;
      if (static_cast<int64_t>(real.size()) == nonUnit) {
        d = ReduceDirection::All;
      } else if (!real.empty()) {
        // X when the reduced axes are exactly the innermost non-unit ones.
        bool innermost = true;
        int64_t expect = rank - 1;
        for (auto it = real.rbegin(); it != real.rend(); ++it) {
          while (expect >= 0 && inShape[static_cast<size_t>(expect)] == 1) --expect;
          if (*it != expect) {
            innermost = false;
            break;
          }
          --expect;
        }
        d = innermost ? ReduceDirection::X : ReduceDirection::Y;
      }
      if (dir == ReduceDirection::Unknown) {
        dir = d;
      } else if (dir != d && d != ReduceDirection::Unknown) {
        dir = ReduceDirection::Y;  // mixed directions: treated as the general (non-X) case
      }
    }
  }
  graph->operatorTemplate = cur;
  graph->reduceDirection = dir;
}

std::string printOpGraph(const OpGraph &g) {
  std::ostringstream os;
  auto typeStr = [&](const TensorValue &t) {
    std::ostringstream s;
    s << "tensor<";
    for (int64_t d : t.shape) s << d << "x";
    s << dtypeName(t.dtype) << ">";
    return s.str();
  };
  os << "func.func @" << g.name << "(";
  for (size_t i = 0; i < g.inputs.size(); ++i) {
    const TensorValue &t = g.tensor(g.inputs[i]);
    os << (i ? ", " : "") << "%" << t.name << ": " << typeStr(t);
  }
  os << ") -> (";
  for (size_t i = 0; i < g.outputs.size(); ++i) os << (i ? ", " : "") << typeStr(g.tensor(g.outputs[i]));
  os << ") attributes {mindspore_kernel, process = \"" << g.process << "\", compute_capability = \""
     << g.computeCapability << "\", arch = \"" << g.arch << "\", OperatorType = \""
     << operatorTemplateName(g.operatorTemplate) << "\"} {\n";
  for (const TensorValue &t : g.tensors) {
    if (t.isConst) {
      os << "  %" << t.name << " = \"mindspore.const\"() {value = " << t.constValue << "} : " << typeStr(t) << "\n";
    }
  }
  for (const OpNode &op : g.ops) {
    os << "  ";
    for (size_t i = 0; i < op.outputs.size(); ++i) os << (i ? ", " : "") << "%" << g.tensor(op.outputs[i]).name;
    os << " = \"mindspore." << opKindName(op.kind) << "\"(";
    for (size_t i = 0; i < op.inputs.size(); ++i) os << (i ? ", " : "") << "%" << g.tensor(op.inputs[i]).name;
    os << ")";
    if (!op.axes.empty()) {
      os << " {axis = [";
      for (size_t i = 0; i < op.axes.size(); ++i) os << (i ? ", " : "") << op.axes[i];
      os << "], keepdims = " << (op.keepDims ? "true" : "false") << "}";
    }
    if (op.kind == OpKind::MatMul) {
      os << " {transpose_a = " << (op.transposeA ? "true" : "false")
         << ", transpose_b = " << (op.transposeB ? "true" : "false") << "}";
    }
    auto list = [&](const char *key, const std::vector<int64_t> &v) {
      os << key << " = [";
      for (size_t i = 0; i < v.size(); ++i) os << (i ? ", " : "") << v[i];
      os << "]";
    };
    if (op.kind == OpKind::Transpose) {
      os << " {";
      list("perm", op.perm);
      os << "}";
    } else if (op.kind == OpKind::Slice || op.kind == OpKind::StridedSlice) {
      os << " {";
      list("start", op.begin);
      os << ", ";
      list("strides", op.strides);
      os << "}";
    } else if (op.kind == OpKind::Pad) {
      os << " {";
      list("low", op.begin);
      os << ", value = " << op.padValue << "}";
    } else if (op.kind == OpKind::Concat || op.kind == OpKind::Gather) {
      os << " {axis = " << op.concatAxis << "}";
    }
    if (op.kind == OpKind::Unknown) os << " {ori_op = \"" << op.name << "\"}";
    os << " : " << typeStr(g.tensor(op.outputs[0])) << "\n";
  }
  os << "  return";
  for (size_t i = 0; i < g.outputs.size(); ++i) os << (i ? ", " : " ") << "%" << g.tensor(g.outputs[i]).name;
  os << "\n}\n";
  return os.str();
}

}  // namespace akg
