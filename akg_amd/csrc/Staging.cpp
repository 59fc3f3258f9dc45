#include "Staging.h"

#include <algorithm>
#include <cstdio>
#include <map>
#include <set>
#include <sstream>

#include "HipLowering.h"
#include "Json.h"

namespace akg {
namespace {

std::string quote(const std::string &s) {
  std::string o = "\"";
  for (char c : s) {
    switch (c) {
      case '"': o += "\\\""; break;
      case '\\': o += "\\\\"; break;
      case '\n': o += "\\n"; break;
      case '\r': o += "\\r"; break;
      case '\t': o += "\\t"; break;
      default:
        if (static_cast<unsigned char>(c) < 0x20) {
          char buf[8];
          std::snprintf(buf, sizeof(buf), "\\u%04x", c);
          o += buf;
        } else {
          o += c;
        }
    }
  }
  return o + "\"";
}

// The document model back to text (numbers written as integers stay integers, others keep 17 digits).
std::string dump(const json::Value &v) {
  switch (v.kind()) {
    case json::Value::Kind::Null: return "null";
    case json::Value::Kind::Bool: return v.asBool() ? "true" : "false";
    case json::Value::Kind::Number: {
      if (v.isInteger()) return std::to_string(v.asInt());
      char buf[40];
      std::snprintf(buf, sizeof(buf), "%.17g", v.asDouble());
      return buf;
    }
    case json::Value::Kind::String: return quote(v.asString());
    case json::Value::Kind::Array: {
      std::string o = "[";
      for (size_t i = 0; i < v.size(); ++i) o += (i ? ", " : "") + dump(v[i]);
      return o + "]";
    }
    case json::Value::Kind::Object: {
      std::string o = "{";
      bool first = true;
      for (const auto &m : v.members()) {
        o += (first ? "" : ", ") + quote(m.first) + ": " + dump(m.second);
        first = false;
      }
      return o + "}";
    }
  }
  return "null";
}

// Ops whose result is read through an index map: kept out of the kernels that reduce.
bool isViewOp(OpKind k) {
  switch (k) {
    case OpKind::Transpose:
    case OpKind::Tile:
    case OpKind::Slice:
    case OpKind::StridedSlice:
    case OpKind::Pad:
    case OpKind::Concat:
    case OpKind::Gather:
    case OpKind::Reshape:
      return true;
    default:
      return false;
  }
}

std::string tensorEntry(const TensorValue &t) {
  std::ostringstream o;
  o << "{\"data_type\": " << quote(dtypeName(t.dtype)) << ", \"format\": \"DefaultFormat\", \"shape\": [";
  for (size_t i = 0; i < t.shape.size(); ++i) o << (i ? ", " : "") << t.shape[i];
  o << "], \"tensor_name\": " << quote(t.name) << "}";
  return o.str();
}

}  // namespace

bool planStages(const std::string &jsonText, const OpGraph &g, bool reductionsToo, StagingPlan *plan, std::string *why) {

  plan->stages.clear();
  plan->tempBytes.clear();
  const json::Value doc = json::Value::parse(jsonText);
  if (!doc.contains("op_desc")) {
    *why = "it has no op entries";
    return false;
  }
  // the op entry behind every translated op, by the name of its result (the translator may have dropped unused entries)
  const json::Value &opDesc = doc.at("op_desc");
  std::map<std::string, size_t> entryOf;
  for (size_t i = 0; i < opDesc.size(); ++i) {
    if (!opDesc[i].contains("output_desc")) continue;
    for (size_t o = 0; o < opDesc[i].at("output_desc").size(); ++o) {   // (a Split entry has one result per piece)
      const json::Value &out = opDesc[i].at("output_desc")[o];
      if (out.contains("tensor_name")) entryOf[out.at("tensor_name").asString()] = i;
    }
  }
  std::vector<size_t> entry(g.ops.size(), 0);
  for (size_t i = 0; i < g.ops.size(); ++i) {
    const OpNode &op = g.ops[i];
    if (op.kind == OpKind::Unknown || op.kind == OpKind::Unsupported) {
      *why = "op " + op.name + " is not cut into stages";
      return false;
    }
    if (op.outputs.size() != 1) {
      *why = "op " + op.name + " has several results";
      return false;
    }
    const auto it = entryOf.find(g.tensor(op.outputs[0]).name);
    // (the translator turns a Split entry into one Slice per piece that is used)
    const bool named = it != entryOf.end() && opDesc[it->second].contains("name");
    const std::string entryName = named ? opDesc[it->second].at("name").asString() : std::string();
    if (!named || (entryName != op.name && !(entryName == "Split" && op.kind == OpKind::Slice))) {
      *why = "its op entries do not map one to one onto the translated ops";
      return false;
    }
    entry[i] = it->second;
  }
  {
    std::set<int> distinct(g.outputs.begin(), g.outputs.end());
    if (distinct.size() != g.outputs.size()) {
      *why = "an output is listed twice";
      return false;
    }
  }
  const size_t nt = g.tensors.size();
  // `reduced`: the tensor is the result of a cut op (a reduction, or a data-movement op) and lives in memory
  // Which results are cut (live in memory): those of data-movement ops and of UnsortedSegmentSum (a kernel of its
  // own); of reductions when asked for; of a
  // contraction when a reduction depends on it (otherwise the ops behind it are its epilogue, in the same kernel); and
  // the operands of a contraction that are computed (the GEMM kernel reads its operands from memory).
  std::vector<bool> cutResult(nt, false);
  {
    std::vector<bool> feedsReduction(nt, false);
    for (size_t i = g.ops.size(); i-- > 0;) {
      const OpNode &op = g.ops[i];
      bool feeds = lowering::isReduceKind(op.kind);
      for (int out : op.outputs) feeds = feeds || feedsReduction[static_cast<size_t>(out)];
      if (feeds) {
        for (int in : op.inputs) feedsReduction[static_cast<size_t>(in)] = true;
      }
    }
    for (const OpNode &op : g.ops) {
      const int out = op.outputs[0];
      if (isViewOp(op.kind) || (reductionsToo && lowering::isReduceKind(op.kind)) ||
          (op.kind == OpKind::MatMul && feedsReduction[static_cast<size_t>(out)]) || op.kind == OpKind::SegmentSum) {
        cutResult[static_cast<size_t>(out)] = true;
      }
      if (op.kind == OpKind::MatMul || op.kind == OpKind::SegmentSum) {   // (their kernels read operands from memory)
        for (int in : op.inputs) {
          if (g.tensor(in).producer >= 0) cutResult[static_cast<size_t>(in)] = true;
        }
      }
    }
  }
  std::vector<int> level(nt, 0);
  std::vector<bool> reduced(nt, false);
  for (const OpNode &op : g.ops) {
    int lv = 0;
    for (int in : op.inputs) lv = std::max(lv, level[static_cast<size_t>(in)]);
    const bool cut = cutResult[static_cast<size_t>(op.outputs[0])];
    for (int out : op.outputs) {
      level[static_cast<size_t>(out)] = lv + (cut ? 1 : 0);
      reduced[static_cast<size_t>(out)] = cut;
    }
  }
  // tensors some output of the description depends on
  std::vector<bool> needed(nt, false);
  {
    std::vector<int> work(g.outputs.begin(), g.outputs.end());
    while (!work.empty()) {
      const int t = work.back();
      work.pop_back();
      if (needed[static_cast<size_t>(t)]) continue;
      needed[static_cast<size_t>(t)] = true;
      const int p = g.tensor(t).producer;
      if (p >= 0) {
        for (int in : g.ops[static_cast<size_t>(p)].inputs) work.push_back(in);
      }
    }
  }
  int maxLevel = 0;
  for (int t : g.outputs) maxLevel = std::max(maxLevel, level[static_cast<size_t>(t)]);
  std::set<std::vector<int64_t>> outputShapes;
  for (int t : g.outputs) outputShapes.insert(g.tensor(t).shape);
  // nothing to cut at: only outputs of different shapes are then a reason for several kernels (one per shape; the
  // single-kernel families write outputs of one iteration space)
  if (maxLevel == 0 && (!reductionsToo || outputShapes.size() < 2)) {
    *why = reductionsToo ? "it has no reduction, contraction or data-movement result to cut at"
                         : "it has no contraction or data-movement result to cut at";
    return false;
  }

  // where the reduction results live
  std::map<int, int> tempOf;
  for (size_t t = 0; t < nt; ++t) {
    if (!reduced[t] || !needed[t] || g.tensors[t].outputIndex >= 0) continue;
    tempOf[static_cast<int>(t)] = static_cast<int>(plan->tempBytes.size());
    plan->tempBytes.push_back(static_cast<uint64_t>(g.tensors[t].numel()) * dtypeSize(g.tensors[t].dtype));
  }

  // per kernel: the description inputs it reads and the Assign ops it holds (for the ordering check at the end)
  std::vector<std::set<int>> kernelReads;
  std::vector<std::vector<size_t>> kernelAssigns;
  // one kernel per target group
  auto addKernel = [&](const std::vector<int> &targets, int stage) {
    // ops on the way to the targets, cut at the description's inputs and at reduction results of earlier stages
    std::set<int> targetSet(targets.begin(), targets.end());
    std::vector<bool> opUsed(g.ops.size(), false);
    std::set<int> cutInputs;       // reduction results read from memory
    std::set<int> graphInputs;     // description inputs read
    std::vector<int> work(targets.begin(), targets.end());
    std::set<int> seen;
    while (!work.empty()) {
      const int t = work.back();
      work.pop_back();
      if (!seen.insert(t).second) continue;
      const TensorValue &tv = g.tensor(t);
      if (tv.isConst) continue;
      if (tv.inputIndex >= 0) {
        graphInputs.insert(tv.inputIndex);
        continue;
      }
      const bool earlier = reduced[static_cast<size_t>(t)] && level[static_cast<size_t>(t)] <= stage && !targetSet.count(t);
      if (earlier) {
        cutInputs.insert(t);
        continue;
      }
      if (tv.producer < 0) continue;
      opUsed[static_cast<size_t>(tv.producer)] = true;
      for (int in : g.ops[static_cast<size_t>(tv.producer)].inputs) work.push_back(in);
    }
    StagePlan sp;
    std::ostringstream o;
    const std::string name = g.name + "_stage" + std::to_string(plan->stages.size());
    o << "{\"op\": " << quote(name);
    for (const char *key : {"process", "platform", "composite", "version", "target_info"}) {
      if (doc.contains(key)) o << ", " << quote(key) << ": " << dump(doc.at(key));
    }
    o << ", \"input_desc\": [";
    bool first = true;
    for (int idx : graphInputs) {
      o << (first ? "" : ", ") << "[" << tensorEntry(g.tensor(g.inputs[static_cast<size_t>(idx)])) << "]";
      first = false;
      StageArg a;
      a.kind = StageArg::Kind::Input;
      a.index = idx;
      sp.args.push_back(a);
      sp.shapes.push_back(g.tensor(g.inputs[static_cast<size_t>(idx)]).shape);
    }
    for (int t : cutInputs) {
      o << (first ? "" : ", ") << "[" << tensorEntry(g.tensor(t)) << "]";
      first = false;
      StageArg a;
      if (g.tensor(t).outputIndex >= 0) {
        a.kind = StageArg::Kind::Output;
        a.index = g.tensor(t).outputIndex;
      } else {
        a.kind = StageArg::Kind::Temp;
        a.index = tempOf.at(t);
      }
      sp.args.push_back(a);
      sp.shapes.push_back(g.tensor(t).shape);
    }
    o << "], \"op_desc\": [";
    first = true;
    std::set<size_t> written;
    for (size_t i = 0; i < g.ops.size(); ++i) {
      if (!opUsed[i] || !written.insert(entry[i]).second) continue;
      o << (first ? "" : ", ") << dump(opDesc[entry[i]]);
      first = false;
    }
    o << "], \"output_desc\": [";
    first = true;
    for (int t : targets) {
      o << (first ? "" : ", ") << tensorEntry(g.tensor(t));
      first = false;
      StageArg a;
      if (g.tensor(t).outputIndex >= 0) {
        a.kind = StageArg::Kind::Output;
        a.index = g.tensor(t).outputIndex;
      } else {
        a.kind = StageArg::Kind::Temp;
        a.index = tempOf.at(t);
      }
      sp.args.push_back(a);
      sp.shapes.push_back(g.tensor(t).shape);
      ++sp.numOutputs;
    }
    o << "]}";
    sp.jsonText = o.str();
    plan->stages.push_back(sp);
    kernelReads.push_back(graphInputs);
    std::vector<size_t> assigns;
    for (size_t i = 0; i < g.ops.size(); ++i) {
      if (opUsed[i] && g.ops[i].kind == OpKind::Assign) assigns.push_back(i);
    }
    kernelAssigns.push_back(assigns);
  };

  for (int s = 0; s <= maxLevel; ++s) {
    // the reductions over operands of level s, grouped by operand shape and axes (one reduction space per kernel)
    std::map<std::string, std::vector<int>> reduceGroups;
    for (const OpNode &op : g.ops) {
      const bool isReduce = lowering::isReduceKind(op.kind);
      if (!cutResult[static_cast<size_t>(op.outputs[0])]) continue;
      const int out = op.outputs[0];
      if (!needed[static_cast<size_t>(out)] || level[static_cast<size_t>(out)] != s + 1) continue;
      std::ostringstream key;
      if (isReduce && reductionsToo) {
        for (int64_t d : g.tensor(op.inputs[0]).shape) key << d << "x";
        key << "/";
        for (int64_t a : op.axes) key << a << ",";
        key << (op.keepDims ? "k" : "");
      } else {
        key << "own" << out;   // a kernel of its own per data-movement result and per contraction
      }
      reduceGroups[key.str()].push_back(out);
    }
    for (const auto &kv : reduceGroups) addKernel(kv.second, s);
    // the description's other outputs of this level, one kernel per shape
    std::map<std::string, std::vector<int>> outputGroups;
    for (int t : g.outputs) {
      if (level[static_cast<size_t>(t)] != s || reduced[static_cast<size_t>(t)]) continue;
      if (g.tensor(t).inputIndex >= 0 || g.tensor(t).isConst) {
        *why = "an output is an input of the description";
        return false;
      }
      std::ostringstream key;
      for (int64_t d : g.tensor(t).shape) key << d << "x";
      std::vector<int> &grp = outputGroups[key.str()];
      if (std::find(grp.begin(), grp.end(), t) == grp.end()) grp.push_back(t);
    }
    for (const auto &kv : outputGroups) addKernel(kv.second, s);
  }
  // Assign writes over an input of the description. The kernels recompute from the inputs, so the write must come after
  // every other kernel's reads of that input, must happen once, and must not be lost.
  for (size_t i = 0; i < g.ops.size(); ++i) {
    if (g.ops[i].kind != OpKind::Assign) continue;
    const int dst = g.tensor(g.ops[i].inputs[0]).inputIndex;
    int holder = -1, holders = 0;
    for (size_t kx = 0; kx < kernelAssigns.size(); ++kx) {
      if (std::find(kernelAssigns[kx].begin(), kernelAssigns[kx].end(), i) != kernelAssigns[kx].end()) {
        holder = static_cast<int>(kx);
        ++holders;
      }
    }
    if (holders != 1 || dst < 0) {
      *why = holders == 0 ? "the result of an Assign is not among the outputs" : "an Assign would run in several kernels";
      return false;
    }
    for (size_t kx = 0; kx < kernelReads.size(); ++kx) {
      if (static_cast<int>(kx) > holder && kernelReads[kx].count(dst)) {
        *why = "a kernel behind an Assign would read the input it overwrites";
        return false;
      }
    }
  }
  if (plan->stages.size() < 2) {
    *why = "it has no reduction or data-movement result to cut at";
    return false;
  }
  return true;
}

bool moveArgMaxToInnermostAxis(const std::string &jsonText, std::string *rewritten) {
  const json::Value doc = json::Value::parse(jsonText);
  if (!doc.isObject() || !doc.contains("op_desc")) return false;
  auto shapeText = [](const std::vector<int64_t> &shape) {
    std::string o = "[";
    for (size_t i = 0; i < shape.size(); ++i) o += (i ? ", " : "") + std::to_string(shape[i]);
    return o + "]";
  };
  auto tensorText = [&](const std::string &name, const std::vector<int64_t> &shape, const std::string &dtype) {
    return "{\"data_type\": " + quote(dtype) + ", \"format\": \"DefaultFormat\", \"shape\": " + shapeText(shape) +
           ", \"tensor_name\": " + quote(name) + "}";
  };
  bool changed = false;
  std::string ops = "[";
  const json::Value &opDesc = doc.at("op_desc");
  for (size_t k = 0; k < opDesc.size(); ++k) {
    const json::Value &entry = opDesc[k];
    std::string text = dump(entry);
    do {
      if (!entry.contains("name") || entry.at("name").asString() != "ArgMax") break;
      const json::Value &in = entry.at("input_desc")[0][0];
      const json::Value &out = entry.at("output_desc")[0];
      if (!in.contains("shape") || !out.contains("shape")) break;
      const std::vector<int64_t> shape = in.at("shape").asIntVector();
      const std::vector<int64_t> outShape = out.at("shape").asIntVector();
      bool open = false;
      for (int64_t d : shape) open = open || d < 0;
      if (open || shape.size() < 2) break;
      // the axis: value of the second input, else the attribute
      std::vector<int64_t> axes;
      bool keep = false;
      if (entry.at("input_desc").size() > 1 && entry.at("input_desc")[1][0].contains("value")) {
        const json::Value &v = entry.at("input_desc")[1][0].at("value");
        axes = v.isArray() ? v.asIntVector() : std::vector<int64_t>{v.asInt()};
      }
      const json::Value &attrs = entry.contains("attr") ? entry.at("attr") : json::Value();
      for (size_t a = 0; a < attrs.size(); ++a) {
        const std::string an = attrs[a].at("name").asString();
        if (an == "axis" && axes.empty()) {
          const json::Value &v = attrs[a].at("value");
          axes = v.isArray() ? v.asIntVector() : std::vector<int64_t>{v.asInt()};
        } else if (an == "keep_dims") {
          keep = attrs[a].at("value").asBool();
        }
      }
      if (axes.size() != 1) break;
      const int64_t rank = static_cast<int64_t>(shape.size());
      const int64_t axis = axes[0] < 0 ? axes[0] + rank : axes[0];
      if (axis < 0 || axis >= rank) break;
      // innermost already (extent-1 dimensions behind it do not count)
      bool innermost = true;
      for (int64_t d = axis + 1; d < rank; ++d) innermost = innermost && shape[static_cast<size_t>(d)] == 1;
      if (innermost) break;
      std::vector<int64_t> perm, moved, without;
      for (int64_t d = 0; d < rank; ++d) {
        if (d == axis) continue;
        perm.push_back(d);
        moved.push_back(shape[static_cast<size_t>(d)]);
        without.push_back(shape[static_cast<size_t>(d)]);
      }
      perm.push_back(axis);
      moved.push_back(shape[static_cast<size_t>(axis)]);
      const std::string inName = in.at("tensor_name").asString(), outName = out.at("tensor_name").asString();
      const std::string inType = in.at("data_type").asString(), outType = out.at("data_type").asString();
      const std::string tName = outName + "_akg_moved", iName = outName + "_akg_index";
      const bool reshape = keep || without != outShape;
      std::string t = "{\"attr\": [{\"data_type\": \"listInt\", \"name\": \"perm\", \"value\": " + shapeText(perm) +
                      "}], \"impl_path\": \"\", \"input_desc\": [[" + dump(in) + "]], \"name\": \"Transpose\", \"output_desc\": [" +
                      tensorText(tName, moved, inType) + "]}";
      std::string a = "{\"attr\": [{\"data_type\": \"listInt\", \"name\": \"axis\", \"value\": [" + std::to_string(rank - 1) +
                      "]}, {\"data_type\": \"bool\", \"name\": \"keep_dims\", \"value\": false}], \"impl_path\": \"\", \"input_desc\": [[" +
                      tensorText(tName, moved, inType) + "]], \"name\": \"ArgMax\", \"output_desc\": [" +
                      (reshape ? tensorText(iName, without, outType) : dump(out)) + "]}";
      text = t + ", " + a;
      if (reshape) {
        text += ", {\"attr\": [{\"data_type\": \"listInt\", \"name\": \"shape\", \"value\": " + shapeText(outShape) +
                "}], \"impl_path\": \"\", \"input_desc\": [[" + tensorText(iName, without, outType) +
                "]], \"name\": \"Reshape\", \"output_desc\": [" + dump(out) + "]}";
      }
      changed = true;
    } while (false);
    ops += (k ? ", " : "") + text;
  }
  ops += "]";
  if (!changed) return false;
  std::string o = "{";
  bool first = true;
  for (const auto &m : doc.members()) {
    o += (first ? "" : ", ") + quote(m.first) + ": " + (m.first == "op_desc" ? ops : dump(m.second));
    first = false;
  }
  *rewritten = o + "}";
  return true;
}

}  // namespace akg
