/**
 * Indexed elementwise kernels: fusions that contain data-movement ops (Transpose, Tile, Slice, StridedSlice, Pad,
 * Concat, and Reshape / BroadcastTo between them), where an output element no longer sits at the linear position of
 * the input elements it is computed from.
 *
 * The reference lowers these ops to tosa.transpose / tosa.pad / tosa.concat / tensor.extract_slice / a
 * linalg.generic with a read map (MindSporeToTosa.cpp:46-58,305-376,479; MindSporeToLinalg.cpp:970-1040;
 * MindSporeFinalizingLower.cpp:102-140) and materialises every one of them in memory. Here the whole fusion is
 * one kernel that works backwards from the outputs: a thread owns V consecutive elements of the output's
 * innermost dimension; for each of them the value of every tensor it depends on is produced on demand at the
 * index the ops in between map it to, down to scalar loads of the kernel inputs. Nothing intermediate touches
 * memory and a value needed twice at the same index is computed once. Outputs are stored as V-element chunks.
 *
 * Vector loads. Every index component carries how it varies over the V elements of a thread's chunk: not at all,
 * as `u + e` with a chunk-uniform `u` (and whether `u` is a multiple of V), or arbitrarily. Slices, pads, concats and
 * tiles whose offsets and extents are multiples of V keep the second form, conditions on such components hold for
 * the whole chunk or for none of it, and a kernel input whose innermost index has that form (all other components
 * uniform, every enclosing condition chunk-uniform) is read once per chunk with one 16-byte load placed in front of
 * the element loop. Index loads of a Gather whose position is chunk-uniform are placed there too, so an embedding
 * lookup reads its table rows with vector loads. Anything else falls back to scalar loads inside the element loop.
 *
 * Transposed kernel inputs. Pulled element by element, the reads of a transposed operand are strided across a
 * wavefront (measured 11 % of the HBM peak on a [32,2048,1024] bfloat16 transpose). When a kernel input X goes
 * through a Transpose that moves its innermost axis, and the result has the shape of the outputs, the kernel is
 * tiled instead: a workgroup owns a 64 x 64 patch of the plane spanned by the outputs' innermost axis and the axis
 * X's innermost one lands on, copies X's side of the patch to LDS with 16-byte loads along X's innermost axis, and
 * the on-demand read of the transposed value becomes an LDS read (row pitch 64 + 2 elements, so a wavefront's
 * column reads spread over the banks). Everything else is pulled as before.
 */
#include <map>
#include <sstream>

#include "HipLowering.h"

namespace akg {
namespace {

using lowering::computeTypeName;
using lowering::dtypeTag;

bool isViewKind(OpKind k) {
  return k == OpKind::Transpose || k == OpKind::Tile || k == OpKind::Slice || k == OpKind::StridedSlice ||
         k == OpKind::Pad || k == OpKind::Concat || k == OpKind::Gather;
}

class IndexedEmitter {
 public:
  IndexedEmitter(const OpGraph &g, const LoweringOptions &o) : g_(g), opt_(o) {}

  LoweredKernel run() {
    analyse();
    emit();
    LoweredKernel k;
    k.kernelName = g_.name + "_kernel";
    k.source = src_.str();
    k.family = KernelFamily::Indexed;
    k.grid[0] = static_cast<unsigned>(grid_);
    k.block[0] = kBlock;
    k.algorithmicBytes = lowering::countAlgorithmicBytes(g_);
    k.shapeArgs = lowering::buildShapeArgs(g_);
    if (chunksArg_) k.scalarArgs.push_back(chunksTotal_);
    std::ostringstream note;
    note << "indexed vec=" << vec_ << " block=" << kBlock << " grid=" << grid_ << " rank=" << space_.size();
    if (!staged_.empty()) note << " lds_tiles=" << staged_.size() << " tile=" << kTile << "x" << kTile << " axis=" << tDim_;
    k.scheduleNote = note.str();
    return k;
  }

 private:
  static constexpr int kBlock = 256;
  // A description with open extents: nothing in an index map depends on the outermost extent of the outputs unless an
  // op works on that axis (every stride is a product of the extents to its right), so the number of chunks is a kernel
  // argument instead of a constant and the workgroup numbering of the tiled transposes does not name it: batches of
  // any size then share one code object wherever the ops leave the batch axis alone.
  bool chunksArg_ = false;
  int64_t chunksTotal_ = 0;
  // One component of a tensor index at the element a thread is working on.
  struct Ix {
    std::string s;         // C expression for the current element
    int kind = 0;          // 0: same for all V elements of the chunk; 1: u + e; 2: anything else
    std::string u;         // kind 1: the chunk-uniform part
    bool aligned = false;  // kind 1: u is known to be a multiple of V
    bool early = true;     // kind 0 (s) / kind 1 (u): only uses variables that exist in front of the element loop
    Ix() : s("0") {}
    Ix(const std::string &text, bool isEarly = true) : s(text), early(isEarly) {}  // NOLINT(runtime/explicit)
    Ix(const char *text) : s(text) {}                                             // NOLINT(runtime/explicit)
    bool operator==(const Ix &o) const { return s == o.s; }
    bool operator!=(const Ix &o) const { return s != o.s; }
  };
  typedef std::vector<Ix> Index;  // one component per dimension
  static Ix affine(const std::string &u, bool aligned, bool early) {
    Ix x("(" + u + " + e)", early);
    x.kind = 1;
    x.u = u;
    x.aligned = aligned;
    return x;
  }
  static Ix perElement(const std::string &text) {
    Ix x(text, false);
    x.kind = 2;
    return x;
  }

  const OpGraph &g_;
  LoweringOptions opt_;
  std::ostringstream src_;
  std::vector<int64_t> space_;  // iteration space: the shape of the outputs
  int vec_ = 1;
  std::vector<bool> streamedInput_;  // per kernel input: read at most once per element by the whole grid
  bool overlapTail_ = false;   // V does not divide the innermost extent: the last chunk of a row overlaps its neighbour
  int64_t chunksPerRow_ = 1;
  int64_t grid_ = 1;
  // tiled mode (LDS-staged transposed inputs)
  static constexpr int kTile = 64;
  struct Staged {
    int transposed;  // tensor id of the Transpose result
    int input;       // tensor id of the kernel input it reads
    int xRowDim;     // dimension of the input that follows the outputs' innermost axis
    int vecX;        // elements per staging load
  };
  std::vector<Staged> staged_;
  int tDim_ = -1;               // output dimension the staged inputs' innermost axis lands on
  Index canonical_;             // index of the current output element, by dimension
  std::vector<bool> assignedInput_;   // per kernel input: overwritten by an Assign of this kernel (empty: none is)
  std::vector<bool> relaxed_;
  int nextTemp_ = 0;
  int indent_ = 2;
  // values already computed in the scopes that are open: (tensor id, index text) -> variable
  std::vector<std::map<std::string, std::string>> scopes_;
  // Statements go to `src_` until the element loop is opened; its body is collected in `body_` and statements that
  // belong in front of it (chunk-wide loads, chunk-uniform gather positions) in `hoist_`.
  std::ostringstream body_, hoist_;
  std::ostringstream *out_ = &src_;
  int hoistIndent_ = 1;
  bool inLoop_ = false;
  struct Cond {
    std::string chunkText;  // the condition for the whole chunk, if uniform
    bool uniformEarly;      // holds for all V elements or none, and can be evaluated in front of the loop
  };
  std::vector<Cond> conds_;
  std::map<std::string, std::string> hoistedLoads_;  // (input, chunk offset, guard) -> array

  std::string ctOf(int id) const { return computeTypeName(g_.tensor(id).dtype); }
  std::string tagOf(int id) const { return dtypeTag(g_.tensor(id).dtype); }
  void stmt(const std::string &s) { *out_ << std::string(static_cast<size_t>(indent_) * 2, ' ') << s << "\n"; }
  void hoisted(const std::string &s) { hoist_ << std::string(static_cast<size_t>(hoistIndent_) * 2, ' ') << s << "\n"; }
  std::string fresh(const char *prefix) { return prefix + std::to_string(nextTemp_++); }

  void analyse() {
    for (const OpNode &op : g_.ops) {
      if (op.kind == OpKind::Unknown) {
        throw LoweringError("op " + op.name + " is not in the op table (mindspore.unknown cannot be legalized)");
      }
      if (op.kind == OpKind::Unsupported) throw LoweringError("op " + op.name + " has no kernel family yet");
      if (op.kind == OpKind::Assign) {
        // The value is stored over the destination (a kernel input) besides being the op's result (linalg.copy
        // ins=value outs=destination, MindSporeToLinalg.cpp:495-524). The thread that computes an element of the result
        // stores it to the same position of the destination, so the result must be an output of the kernel, and no
        // thread may read the destination anywhere but at its own position (checked where inputs are read).
        const TensorValue &dst = g_.tensor(op.inputs[0]);
        const TensorValue &res = g_.tensor(op.outputs[0]);
        if (dst.inputIndex < 0 || res.outputIndex < 0 || dst.dtype != res.dtype) {
          throw LoweringError("op " + op.name + ": next to data-movement ops the destination must be a kernel input and the result an output of the kernel");
        }
        if (assignedInput_.empty()) assignedInput_.assign(g_.inputs.size(), false);
        assignedInput_[static_cast<size_t>(dst.inputIndex)] = true;
      }
      if (op.kind == OpKind::MatMul || lowering::isReduceKind(op.kind)) {
        throw LoweringError("op " + op.name + " cannot be fused with data-movement ops (Transpose, Tile, Slice, Pad, "
                            "Concat) in one kernel yet");
      }
      if (op.outputs.size() != 1) throw LoweringError("op " + op.name + ": multiple results are not supported");
      if (isViewKind(op.kind)) {
        for (int in : op.inputs) {
          if (op.kind == OpKind::Gather && in == op.inputs[1]) continue;  // the indices
          if (g_.tensor(in).dtype != g_.tensor(op.outputs[0]).dtype) {
            throw LoweringError("op " + op.name + ": operand and result element types differ");
          }
        }
      }
    }
    space_ = g_.tensor(g_.outputs[0]).shape;
    if (space_.empty()) space_.push_back(1);
    for (int id : g_.outputs) {
      std::vector<int64_t> s = g_.tensor(id).shape;
      if (s.empty()) s.push_back(1);
      if (s != space_) throw LoweringError("outputs of different shapes cannot share an indexed kernel yet");
      if (g_.tensor(id).producer < 0) throw LoweringError("output " + g_.tensor(id).name + " is a kernel input");
    }
    int64_t numel = 1;
    for (int64_t d : space_) numel *= d;
    for (const TensorValue &t : g_.tensors) {
      if (t.numel() >= (1LL << 31)) throw LoweringError("tensor " + t.name + " is too large for 32-bit indexing");
    }
    size_t widest = 1;
    for (int id : g_.outputs) widest = std::max(widest, dtypeSize(g_.tensor(id).dtype));
    int v = opt_.vec > 0 ? opt_.vec : static_cast<int>(16 / widest);
    v = std::max(1, std::min(v, 16));
    if ((v & (v - 1)) != 0) v = 1;
    // An innermost extent that V does not divide keeps the full chunk width: the last chunk of a row then starts
    // at extent - V and shares elements with its neighbour (both write the same values); such chunks are only
    // element-aligned in memory.
    // (not with an Assign: a thread would read elements of the destination that its neighbour has already overwritten)
    if (opt_.vec == 0 && (space_.back() % v) != 0 && space_.back() >= 2 * v && assignedInput_.empty()) {
      overlapTail_ = true;
    } else {
      while (v > 1 && (space_.back() % v) != 0) v >>= 1;
    }
    vec_ = v;
    chunksPerRow_ = (space_.back() + vec_ - 1) / vec_;
    const int64_t chunks = numel / space_.back() * chunksPerRow_;
    grid_ = std::max<int64_t>(1, (chunks + kBlock - 1) / kBlock);
    pickStaging();
    findStreamedInputs();
    if (!staged_.empty() && overlapTail_) {
      // the LDS-tiled transposes keep their own chunking: narrower chunks instead
      overlapTail_ = false;
      while (vec_ > 1 && (space_.back() % vec_) != 0) vec_ >>= 1;
      chunksPerRow_ = space_.back() / vec_;
    }
    if (!staged_.empty()) {
      grid_ = 1;
      for (size_t d = 0; d < space_.size(); ++d) {
        const bool tiledDim = static_cast<int>(d) == tDim_ || d + 1 == space_.size();
        grid_ *= tiledDim ? (space_[d] + kTile - 1) / kTile : space_[d];
      }
    }
    if (grid_ > 2147483647LL) throw LoweringError("grid too large");
  }

  // Kernel inputs every element of which is read at most once by the whole grid: they have one consumer, and from
  // there to a kernel output every op either maps elements one to one (Transpose, Slice, StridedSlice, Pad, Concat,
  // Reshape, Cast and other elementwise ops on operands of the result's size) or drops some (the slices). A Tile, a
  // broadcast, a Gather's data operand or a second consumer mean re-use, and such inputs keep ordinary loads.
  void findStreamedInputs() {
    streamedInput_.assign(g_.inputs.size(), false);
    if (opt_.nonTemporal == 0) return;
    std::vector<int> uses(g_.tensors.size(), 0);
    for (const OpNode &op : g_.ops) {
      for (int in : op.inputs) ++uses[static_cast<size_t>(in)];
    }
    for (size_t i = 0; i < g_.inputs.size(); ++i) {
      int id = g_.inputs[i];
      bool once = true;
      while (once) {
        if (uses[static_cast<size_t>(id)] != 1) {
          once = uses[static_cast<size_t>(id)] == 0 && g_.tensor(id).outputIndex >= 0;   // reached an output
          break;
        }
        const OpNode *consumer = nullptr;
        for (const OpNode &op : g_.ops) {
          for (int in : op.inputs) {
            if (in == id) consumer = &op;
          }
        }
        const TensorValue &from = g_.tensor(id), &to = g_.tensor(consumer->outputs[0]);
        switch (consumer->kind) {
          case OpKind::Transpose:
          case OpKind::Slice:
          case OpKind::StridedSlice:
          case OpKind::Pad:
          case OpKind::Concat:
          case OpKind::Reshape:
            break;
          case OpKind::Tile:
          case OpKind::BroadcastTo:
          case OpKind::Gather:
            once = false;
            break;
          default:
            once = lowering::isElementwiseKind(consumer->kind) && from.numel() == to.numel();
            break;
        }
        if (g_.tensor(consumer->outputs[0]).outputIndex >= 0 && uses[static_cast<size_t>(consumer->outputs[0])] == 0) {
          break;
        }
        id = consumer->outputs[0];
      }
      // whole 64-byte pieces only (see the result stores)
      const TensorValue &t = g_.tensor(g_.inputs[i]);
      const int64_t rowBytes = (t.shape.empty() ? 1 : t.shape.back()) * static_cast<int64_t>(dtypeSize(t.dtype));
      streamedInput_[i] = once && rowBytes % 64 == 0;
    }
  }

  // Transposes of kernel inputs that move the innermost axis and produce a tensor of the outputs' shape. All staged
  // inputs must agree on the output axis their innermost axis lands on (one tiling plane per kernel).
  void pickStaging() {
    if (opt_.variant == 1) return;  // AKG_HIP_VARIANT=1: pull everything (for comparisons)
    const size_t rank = space_.size();
    if (rank < 2 || space_.back() < 16) return;
    for (const OpNode &op : g_.ops) {
      if (op.kind != OpKind::Transpose || staged_.size() >= 3) continue;
      const TensorValue &x = g_.tensor(op.inputs[0]);
      const TensorValue &y = g_.tensor(op.outputs[0]);
      if (x.inputIndex < 0 || y.shape != space_ || x.shape.size() != rank) continue;
      if (op.perm[rank - 1] == static_cast<int64_t>(rank) - 1) continue;  // innermost axis stays: reads are contiguous
      int t = -1;
      for (size_t d = 0; d < rank; ++d) {
        if (op.perm[d] == static_cast<int64_t>(rank) - 1) t = static_cast<int>(d);
      }
      if (t < 0 || (tDim_ >= 0 && t != tDim_) || space_[static_cast<size_t>(t)] < 16) continue;
      tDim_ = t;
      Staged st;
      st.transposed = op.outputs[0];
      st.input = op.inputs[0];
      st.xRowDim = static_cast<int>(op.perm[rank - 1]);
      int vx = static_cast<int>(16 / dtypeSize(x.dtype));
      while (vx > 1 && (x.shape.back() % vx) != 0) vx >>= 1;
      st.vecX = vx;
      staged_.push_back(st);
    }
  }

  // ---- index helpers ------------------------------------------------------------------------------------
  static std::string linearize(const Index &idx, const std::vector<int64_t> &shape) {
    std::string e;
    for (size_t d = 0; d < shape.size(); ++d) {
      if (shape[d] == 1) continue;  // the index of a unit dimension is 0
      e = e.empty() ? idx[d].s : "(" + e + ") * " + std::to_string(shape[d]) + " + " + idx[d].s;
    }
    return e.empty() ? "0" : e;
  }

  // Index of `linear` (a C expression) in a dense tensor of `shape`. `early`: the expression only uses variables that
  // exist in front of the element loop, so the temporary can be defined there.
  Index delinearize(const std::string &linear, const std::vector<int64_t> &shape, bool uniform = true, bool early = true) {
    const std::string base = fresh("l");
    const bool hoist = inLoop_ && uniform && early;
    if (hoist) {
      hoisted("const int " + base + " = " + linear + ";");
    } else {
      stmt("const int " + base + " = " + linear + ";");
    }
    const bool resultEarly = !inLoop_ || hoist;
    Index out(shape.size());
    int64_t inner = 1;
    for (size_t d = shape.size(); d-- > 0;) {
      if (shape[d] != 1) {
        std::string e = inner == 1 ? base : "(" + base + " / " + std::to_string(inner) + ")";
        int64_t outer = 1;
        for (size_t k = 0; k < d; ++k) outer *= shape[k];
        if (outer != 1) e = "(" + e + " % " + std::to_string(shape[d]) + ")";
        out[d] = uniform ? Ix(e, resultEarly) : perElement(e);
      }
      inner *= shape[d];
    }
    return out;
  }

  // Index of an operand that numpy-broadcasts (right-aligned) into a result of `outShape`.
  Index broadcastIndex(const Index &idx, const std::vector<int64_t> &outShape, const std::vector<int64_t> &inShape,
                       const std::string &what) {
    std::vector<int64_t> in = inShape;
    while (in.size() > outShape.size() && in.front() == 1) in.erase(in.begin());
    if (in.size() > outShape.size()) throw LoweringError(what + ": operand rank exceeds the result's");
    const size_t off = outShape.size() - in.size();
    Index out(inShape.size());
    const size_t lead = inShape.size() - in.size();
    for (size_t d = 0; d < in.size(); ++d) {
      if (in[d] == 1) continue;
      if (in[d] != outShape[off + d]) throw LoweringError(what + ": operand does not broadcast to the result");
      out[lead + d] = idx[off + d];
    }
    return out;
  }

  // idx + delta (delta a compile-time constant), keeping the chunk form where it survives
  Ix shifted(const Ix &x, int64_t delta) const {
    if (delta == 0) return x;
    const std::string d = delta > 0 ? " + " + std::to_string(delta) : " - " + std::to_string(-delta);
    if (x.kind == 0) return Ix("(" + x.s + d + ")", x.early);
    if (x.kind == 1) return affine("(" + x.u + d + ")", x.aligned && (delta % vec_) == 0, x.early);
    return perElement("(" + x.s + d + ")");
  }

  // `x` compared against the half-open range [0, extent): per-element text, and whether it is one answer per chunk
  Cond rangeCond(const Ix &x, int64_t extent, std::string *text) const {
    *text = "static_cast<unsigned>(" + x.s + ") < " + std::to_string(extent) + "u";
    if (x.kind == 0) return Cond{*text, x.early};
    if (x.kind == 1 && x.aligned && (extent % vec_) == 0) {
      return Cond{"static_cast<unsigned>(" + x.u + ") < " + std::to_string(extent) + "u", x.early};
    }
    return Cond{"", false};
  }

  bool condsHoistable() const {
    for (const Cond &c : conds_) {
      if (!c.uniformEarly) return false;
    }
    return true;
  }
  std::string guardText() const {
    std::string g;
    for (const Cond &c : conds_) g = g.empty() ? "(" + c.chunkText + ")" : g + " && (" + c.chunkText + ")";
    return g;
  }

  static std::string keyOf(int id, const Index &idx) {
    std::string k = std::to_string(id) + "@";
    for (const Ix &x : idx) k += x.s + ",";
    return k;
  }

  const std::string *lookup(const std::string &key) const {
    for (size_t s = scopes_.size(); s-- > 0;) {
      auto it = scopes_[s].find(key);
      if (it != scopes_[s].end()) return &it->second;
    }
    return nullptr;
  }

  // ---- value of tensor `id` at `idx`: emits what is needed and returns a C expression of the compute type ----
  std::string valueAt(int id, Index idx) {
    const TensorValue &t = g_.tensor(id);
    if (t.isConst) return lowering::literalFor(t.dtype, t.constValue);
    if (idx.size() != std::max<size_t>(1, t.shape.size())) throw LoweringError("internal: index rank of " + t.name);
    for (size_t d = 0; d < t.shape.size(); ++d) {
      if (t.shape[d] == 1) idx[d] = Ix();
    }
    const std::string key = keyOf(id, idx);
    if (const std::string *known = lookup(key)) return *known;
    const std::string var = fresh("v");
    const std::string ct = ctOf(id);
    if (t.producer < 0) {
      if (t.inputIndex < 0) throw LoweringError("operand " + t.name + " is undefined");
      if (!assignedInput_.empty() && assignedInput_[static_cast<size_t>(t.inputIndex)]) {
        Index own = canonical_;
        for (size_t d = 0; d < t.shape.size() && d < own.size(); ++d) {
          if (t.shape[d] == 1) own[d] = Ix();
        }
        if (own.size() != idx.size() || idx != own) {
          throw LoweringError("input " + t.name + " is overwritten by an Assign of this kernel and read through an index map: "
                              "a thread would read positions that another thread writes");
        }
      }
      const std::string chunkLoad = inLoop_ ? tryChunkLoad(id, idx) : std::string();
      if (!chunkLoad.empty()) {
        scopes_.back()[key] = chunkLoad;
        return chunkLoad;
      }
      stmt("const " + ct + " " + var + " = " + tagOf(id) + "::load(in" + std::to_string(t.inputIndex) + "[" +
           linearize(idx, t.shape) + "]);");
      scopes_.back()[key] = var;
      return var;
    }
    for (size_t k = 0; k < staged_.size(); ++k) {
      if (staged_[k].transposed != id || idx != canonical_) continue;
      // the patch of the transposed input is in LDS: row = position along the outputs' innermost axis
      stmt("const " + ct + " " + var + " = " + tagOf(id) + "::load(akg_tile" + std::to_string(k) +
           "[ci * V + e][tt]);  // Transpose -> " + t.name + " (staged)");
      scopes_.back()[key] = var;
      return var;
    }
    const OpNode &op = g_.ops[static_cast<size_t>(t.producer)];
    const std::vector<int64_t> outShape = t.shape.empty() ? std::vector<int64_t>{1} : t.shape;
    auto inShapeOf = [&](size_t i) {
      const std::vector<int64_t> &s = g_.tensor(op.inputs[i]).shape;
      return s.empty() ? std::vector<int64_t>{1} : s;
    };
    const std::string note = "  // " + op.name + " -> " + t.name;
    switch (op.kind) {
      case OpKind::Reshape: {
        const std::vector<int64_t> in = inShapeOf(0);
        bool allUniform = true, allEarly = true, outerUniform = true, outerEarly = true;
        for (size_t d = 0; d < idx.size(); ++d) {
          const bool uni = idx[d].kind == 0;
          allUniform = allUniform && uni;
          allEarly = allEarly && idx[d].early;
          if (d + 1 < idx.size()) {
            outerUniform = outerUniform && uni;
            outerEarly = outerEarly && idx[d].early;
          }
        }
        Index src;
        if (allUniform) {
          src = delinearize(linearize(idx, outShape), in, true, allEarly);
        } else if (outerUniform && in.back() == outShape.back() && in.back() != 1) {
          // the innermost axis is untouched: re-derive the outer coordinates only, keep the innermost component
          Index outerIdx(idx.begin(), idx.end() - 1);
          const std::vector<int64_t> outerOut(outShape.begin(), outShape.end() - 1), outerIn(in.begin(), in.end() - 1);
          src = delinearize(linearize(outerIdx, outerOut), outerIn, true, outerEarly);
          src.push_back(idx.back());
        } else {
          src = delinearize(linearize(idx, outShape), in, false, false);
        }
        stmt("const " + ct + " " + var + " = " + valueAt(op.inputs[0], src) + ";" + note);
        break;
      }
      case OpKind::BroadcastTo: {
        const Index src = broadcastIndex(idx, outShape, inShapeOf(0), "op " + op.name);
        stmt("const " + ct + " " + var + " = " + valueAt(op.inputs[0], src) + ";" + note);
        break;
      }
      case OpKind::Transpose: {
        Index src(idx.size());
        for (size_t d = 0; d < idx.size(); ++d) src[static_cast<size_t>(op.perm[d])] = idx[d];
        stmt("const " + ct + " " + var + " = " + valueAt(op.inputs[0], src) + ";" + note);
        break;
      }
      case OpKind::Tile: {
        const std::vector<int64_t> in = inShapeOf(0);
        Index src(idx.size());
        for (size_t d = 0; d < idx.size(); ++d) {
          const Ix &x = idx[d];
          const std::string m = " % " + std::to_string(in[d]) + ")";
          if (in[d] == outShape[d]) {
            src[d] = x;
          } else if (x.kind == 0) {
            src[d] = Ix("(" + x.s + m, x.early);
          } else if (x.kind == 1 && x.aligned && (in[d] % vec_) == 0) {
            src[d] = affine("(" + x.u + m, true, x.early);  // a chunk never straddles a period that V divides
          } else {
            src[d] = perElement("(" + x.s + m);
          }
        }
        stmt("const " + ct + " " + var + " = " + valueAt(op.inputs[0], src) + ";" + note);
        break;
      }
      case OpKind::Slice:
      case OpKind::StridedSlice: {
        Index src(idx.size());
        for (size_t d = 0; d < idx.size(); ++d) {
          if (op.strides[d] == 1) {
            src[d] = shifted(idx[d], op.begin[d]);
            continue;
          }
          const std::string e = "(" + std::to_string(op.begin[d]) + " + " + idx[d].s + " * " + std::to_string(op.strides[d]) + ")";
          src[d] = idx[d].kind == 0 ? Ix(e, idx[d].early) : perElement(e);
        }
        stmt("const " + ct + " " + var + " = " + valueAt(op.inputs[0], src) + ";" + note);
        break;
      }
      case OpKind::Pad: {
        const std::vector<int64_t> in = inShapeOf(0);
        std::string cond;
        Cond chunk{"", true};
        Index src(idx.size());
        for (size_t d = 0; d < idx.size(); ++d) {
          src[d] = shifted(idx[d], -op.begin[d]);
          if (in[d] == outShape[d]) continue;
          std::string c;
          const Cond one = rangeCond(src[d], in[d], &c);
          cond = cond.empty() ? c : cond + " && " + c;
          chunk.uniformEarly = chunk.uniformEarly && one.uniformEarly;
          chunk.chunkText = chunk.chunkText.empty() ? one.chunkText : chunk.chunkText + " && " + one.chunkText;
        }
        const std::string fill = lowering::literalFor(t.dtype, static_cast<double>(op.padValue));
        if (cond.empty()) {
          stmt("const " + ct + " " + var + " = " + valueAt(op.inputs[0], src) + ";" + note);
        } else {
          stmt(ct + " " + var + " = " + fill + ";" + note);
          stmt("if (" + cond + ") {");
          openScope();
          conds_.push_back(chunk);
          stmt(var + " = " + valueAt(op.inputs[0], src) + ";");
          conds_.pop_back();
          closeScope();
          stmt("}");
        }
        break;
      }
      case OpKind::Gather: {
        // result index = data index with the gathered axis replaced by the indices' dimensions; the looked-up
        // position is clamped into the axis (the reference reads out of bounds there, which must not fault a GPU)
        const std::vector<int64_t> data = inShapeOf(0), ind = inShapeOf(1);
        const size_t a = static_cast<size_t>(op.concatAxis);
        const size_t indRank = g_.tensor(op.inputs[1]).shape.size();
        Index where(ind.size());
        bool uniform = true, early = true;
        for (size_t d = 0; d < indRank && d < ind.size(); ++d) {
          where[d] = idx[a + d];
          uniform = uniform && where[d].kind == 0;
          early = early && where[d].early;
        }
        const std::string pos = fresh("g");
        const std::string clampHi = std::to_string(data[a] - 1);
        // One position for the whole chunk, computable in front of the element loop: do it there, so that the data
        // read below can become a chunk-wide load (embedding lookups).
        const bool hoist = inLoop_ && uniform && early && conds_.empty();
        if (hoist) {
          // evaluate the position in the scope that encloses the element loop, writing in front of the loop
          std::ostringstream *savedOut = out_;
          const int savedIndent = indent_;
          std::vector<std::map<std::string, std::string>> inner(scopes_.begin() + static_cast<long>(loopScope_), scopes_.end());
          scopes_.resize(loopScope_);
          out_ = &hoist_;
          indent_ = hoistIndent_;
          inLoop_ = false;
          const std::string raw = valueAt(op.inputs[1], where);
          stmt("int " + pos + " = static_cast<int>(" + raw + ");");
          stmt(pos + " = " + pos + " < 0 ? 0 : (" + pos + " > " + clampHi + " ? " + clampHi + " : " + pos + ");");
          inLoop_ = true;
          scopes_.insert(scopes_.end(), inner.begin(), inner.end());
          out_ = savedOut;
          indent_ = savedIndent;
        } else {
          stmt("int " + pos + " = static_cast<int>(" + valueAt(op.inputs[1], where) + ");");
          stmt(pos + " = " + pos + " < 0 ? 0 : (" + pos + " > " + clampHi + " ? " + clampHi + " : " + pos + ");");
        }
        Index src(data.size());
        for (size_t d = 0; d < a; ++d) src[d] = idx[d];
        src[a] = uniform ? Ix(pos, hoist || !inLoop_) : perElement(pos);
        for (size_t d = a + 1; d < data.size(); ++d) src[d] = idx[d - 1 + indRank];
        stmt("const " + ct + " " + var + " = " + valueAt(op.inputs[0], src) + ";" + note);
        break;
      }
      case OpKind::Concat: {
        const std::vector<int64_t> first = inShapeOf(0);
        const size_t a = static_cast<size_t>(op.concatAxis);
        Index second = idx;
        second[a] = shifted(idx[a], -first[a]);
        Cond chunk{"", false};
        if (idx[a].kind == 0) {
          chunk = Cond{idx[a].s + " < " + std::to_string(first[a]), idx[a].early};
        } else if (idx[a].kind == 1 && idx[a].aligned && (first[a] % vec_) == 0) {
          chunk = Cond{idx[a].u + " < " + std::to_string(first[a]), idx[a].early};
        }
        stmt(ct + " " + var + ";" + note);
        stmt("if (" + idx[a].s + " < " + std::to_string(first[a]) + ") {");
        openScope();
        conds_.push_back(chunk);
        stmt(var + " = " + valueAt(op.inputs[0], idx) + ";");
        conds_.pop_back();
        closeScope();
        stmt("} else {");
        openScope();
        conds_.push_back(Cond{"!(" + chunk.chunkText + ")", chunk.uniformEarly});
        stmt(var + " = " + valueAt(op.inputs[1], second) + ";");
        conds_.pop_back();
        closeScope();
        stmt("}");
        break;
      }
      case OpKind::Assign: {
        const std::vector<std::string> operands = {
            "", valueAt(op.inputs[1], broadcastIndex(idx, outShape, inShapeOf(1), "op " + op.name))};
        stmt("const " + ct + " " + var + " = " + lowering::elementwiseExpr(g_, op, operands, false) + ";" + note);
        break;
      }
      default: {
        if (!lowering::isElementwiseKind(op.kind)) throw LoweringError("op " + op.name + " has no indexed lowering");
        std::vector<std::string> operands;
        for (size_t i = 0; i < op.inputs.size(); ++i) {
          const TensorValue &in = g_.tensor(op.inputs[i]);
          if (in.isConst) {
            operands.push_back(lowering::literalFor(in.dtype, in.constValue));
            continue;
          }
          operands.push_back(valueAt(op.inputs[i], broadcastIndex(idx, outShape, inShapeOf(i), "op " + op.name)));
        }
        const std::string expr = lowering::elementwiseExpr(g_, op, operands, relaxed_[static_cast<size_t>(id)]);
        stmt("const " + ct + " " + var + " = " + expr + ";" + note);
        break;
      }
    }
    scopes_.back()[key] = var;
    return var;
  }

  // A kernel input read at `idx`: if its V elements for this chunk are V consecutive elements in memory (aligned or
  // not) and the read happens for the whole chunk or not at all, load them once in front of the element loop and return the
  // expression of the current element; otherwise return "".
  std::string tryChunkLoad(int id, const Index &idx) {
    const TensorValue &t = g_.tensor(id);
    if (vec_ < 2 || t.shape.empty() || idx.empty() || opt_.variant == 2) return std::string();
    const Ix &last = idx.back();
    if (last.kind != 1 || !last.early || t.shape.back() < vec_) return std::string();
    const bool alignedAccess = last.aligned && (t.shape.back() % vec_) == 0;
    for (size_t d = 0; d + 1 < idx.size(); ++d) {
      if (idx[d].kind != 0 || !idx[d].early) return std::string();
    }
    if (!condsHoistable()) return std::string();
    Index first = idx;
    first.back() = Ix(last.u);
    const std::string offset = linearize(first, t.shape);
    const std::string guard = guardText();
    const std::string key = std::to_string(id) + "@" + offset + "?" + guard;
    auto it = hoistedLoads_.find(key);
    if (it == hoistedLoads_.end()) {
      const std::string arr = fresh("w");
      const std::string tag = tagOf(id);
      hoisted(ctOf(id) + " " + arr + "[V] = {};");
      hoisted(std::string(guard.empty() ? "" : "if (" + guard + ") ") +
              (alignedAccess ? "akg::load_chunk<" + tag + ", V, " +
                                   (streamedInput_[static_cast<size_t>(t.inputIndex)] ? "true" : "false") + ">(in"
                             : "akg::load_chunk_unaligned<" + tag + ", V>(in") +
              std::to_string(t.inputIndex) + " + " + offset + ", " + arr + ");");
      it = hoistedLoads_.emplace(key, arr).first;
    }
    return it->second + "[e]";
  }

  // Opens the element loop: what follows goes to the loop body until closeElementLoop writes hoisted statements,
  // loop header and body to `src_`.
  size_t loopScope_ = 0;
  void openElementLoop(int indentOfLoop) {
    body_.str(std::string());
    hoist_.str(std::string());
    hoistedLoads_.clear();
    conds_.clear();
    hoistIndent_ = indentOfLoop;
    indent_ = indentOfLoop;
    out_ = &body_;
    inLoop_ = true;
    loopScope_ = scopes_.size();
    openScope();
  }
  void closeElementLoop() {
    closeScope();
    inLoop_ = false;
    out_ = &src_;
    src_ << hoist_.str();
    stmt("#pragma unroll");
    stmt("for (int e = 0; e < V; ++e) {");
    src_ << body_.str();
    stmt("}");
  }

  void emitTiledBody() {
    const size_t rank = space_.size();
    const size_t td = static_cast<size_t>(tDim_);
    const int64_t extentI = space_.back(), extentT = space_[td];
    const int64_t tilesI = (extentI + kTile - 1) / kTile, tilesT = (extentT + kTile - 1) / kTile;
    src_ << "  constexpr int V = " << vec_ << ";\n";
    src_ << "  constexpr int TILE = " << kTile << ";\n";
    for (size_t k = 0; k < staged_.size(); ++k) {
      src_ << "  __shared__ " << tagOf(staged_[k].input) << "::storage akg_tile" << k << "[TILE][TILE + "
           << std::max<size_t>(1, 4 / dtypeSize(g_.tensor(staged_[k].input).dtype)) << "];\n";
    }
    src_ << "  const int tid = static_cast<int>(threadIdx.x);\n";
    // workgroup -> (other dims..., tile along t, tile along the innermost axis); the innermost tile index is fastest
    // output rows that are not whole cache lines: tiles that write parts of one line next to each other on one XCD
    // (64 x 1000 x 1024 -> 64 x 1024 x 1000 bf16: 33.5 % of the HBM peak in launch order)
    const int64_t outRowBytes = space_.back() * static_cast<int64_t>(dtypeSize(g_.tensor(g_.outputs[0]).dtype));
    if (outRowBytes % 64 != 0 && grid_ >= 64) {
      src_ << "  int akg_w = akg::xcd_contiguous_id(static_cast<int>(blockIdx.x), "
           << (opt_.extentAsArgument ? std::string("static_cast<int>(gridDim.x)") : std::to_string(grid_)) << ");\n";
    } else {
      src_ << "  int akg_w = static_cast<int>(blockIdx.x);\n";
    }
    src_ << "  const int i0 = (akg_w % " << tilesI << ") * TILE;\n  akg_w /= " << tilesI << ";\n";
    src_ << "  const int t0 = (akg_w % " << tilesT << ") * TILE;\n  akg_w /= " << tilesT << ";\n";
    canonical_.assign(rank, Ix());
    size_t lastSplit = rank;   // the outermost dim of the numbering: what is left of the workgroup id is its index
    for (size_t d = 0; d + 1 < rank; ++d) {
      if (d != td && space_[d] != 1) {
        lastSplit = d;
        break;
      }
    }
    for (size_t d = rank - 1; d-- > 0;) {
      if (d == td) continue;
      if (space_[d] == 1) continue;
      if (opt_.extentAsArgument && d == lastSplit) {
        src_ << "  const int g" << d << " = akg_w;\n";
      } else {
        src_ << "  const int g" << d << " = akg_w % " << space_[d] << ";\n  akg_w /= " << space_[d] << ";\n";
      }
      canonical_[d] = Ix("g" + std::to_string(d));
    }
    canonical_[td] = Ix("gt");
    canonical_[rank - 1] = affine("inner0", true, true);
    indent_ = 1;
    scopes_.clear();
    scopes_.emplace_back();
    // ---- stage: rows follow the outputs' innermost axis, columns the input's innermost axis (output axis t)
    for (size_t k = 0; k < staged_.size(); ++k) {
      const Staged &st = staged_[k];
      const TensorValue &x = g_.tensor(st.input);
      const OpNode &op = g_.ops[static_cast<size_t>(g_.tensor(st.transposed).producer)];
      const int chunksPerRow = kTile / st.vecX;
      stmt("for (int c = tid; c < TILE * " + std::to_string(chunksPerRow) + "; c += " + std::to_string(kBlock) + ") {");
      ++indent_;
      stmt("const int r = c / " + std::to_string(chunksPerRow) + ", q = (c % " + std::to_string(chunksPerRow) + ") * " +
           std::to_string(st.vecX) + ";");
      stmt("if (i0 + r < " + std::to_string(extentI) + " && t0 + q < " + std::to_string(extentT) + ") {");
      ++indent_;
      // input index: input dim perm[d] takes output index d
      Index xi(rank);
      for (size_t d = 0; d < rank; ++d) {
        Ix v = canonical_[d];
        if (d == td) v = Ix("(t0 + q)");
        if (d == rank - 1) v = Ix("(i0 + r)");
        xi[static_cast<size_t>(op.perm[d])] = v;
      }
      stmt("const " + tagOf(st.input) + "::storage *src = in" + std::to_string(x.inputIndex) + " + " +
           linearize(xi, x.shape) + ";");
      const size_t bytes = static_cast<size_t>(st.vecX) * dtypeSize(x.dtype);
      // the hint only where the tile rows are whole 64-byte pieces of a line (see the stores below)
      const bool ntIn = opt_.nonTemporal != 0 && (x.shape.back() * static_cast<int64_t>(dtypeSize(x.dtype))) % 64 == 0;
      stmt("akg::Raw<" + std::to_string(bytes) + ">::type raw = " +
           (ntIn ? "__builtin_nontemporal_load(" : "*(") + "reinterpret_cast<const akg::Raw<" +
           std::to_string(bytes) + ">::type *>(src));");
      stmt("__builtin_memcpy(&akg_tile" + std::to_string(k) + "[r][q], &raw, " + std::to_string(bytes) + ");");
      --indent_;
      stmt("}");
      --indent_;
      stmt("}");
    }
    stmt("__syncthreads();");
    // ---- compute: a thread takes V-element chunks of the 64 x 64 output patch
    const int chunksPerRow = kTile / vec_;
    stmt("for (int c = tid; c < TILE * " + std::to_string(chunksPerRow) + "; c += " + std::to_string(kBlock) + ") {");
    ++indent_;
    stmt("const int tt = c / " + std::to_string(chunksPerRow) + ", ci = c % " + std::to_string(chunksPerRow) + ";");
    stmt("const int gt = t0 + tt;");
    stmt("if (gt >= " + std::to_string(extentT) + " || i0 + ci * V >= " + std::to_string(extentI) + ") continue;");
    for (size_t i = 0; i < g_.outputs.size(); ++i) stmt(ctOf(g_.outputs[i]) + " o" + std::to_string(i) + "[V];");
    stmt("const int inner0 = i0 + ci * V;");
    openElementLoop(indent_);
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      const std::string v = valueAt(g_.outputs[i], canonical_);
      stmt("o" + std::to_string(i) + "[e] = " + v + ";");
    }
    closeElementLoop();
    Index first = canonical_;
    first[rank - 1] = Ix("inner0");
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      // Non-temporal stores leave L2 at once: fine for whole lines, but a row segment that ends inside a line would
      // reach memory as a partial write before the neighbouring tile adds the rest of the line.
      const bool ntOut = opt_.nonTemporal != 0 &&
                         (space_.back() * static_cast<int64_t>(dtypeSize(g_.tensor(g_.outputs[i]).dtype))) % 64 == 0;
      stmt("akg::store_chunk<" + tagOf(g_.outputs[i]) + ", V, " + (ntOut ? "true" : "false") + ">(out" + std::to_string(i) +
           " + " + linearize(first, space_) + ", o" + std::to_string(i) + ");");
    }
    --indent_;
    stmt("}");
  }

  void openScope() {
    scopes_.emplace_back();
    ++indent_;
  }
  void closeScope() {
    scopes_.pop_back();
    --indent_;
  }

  void emit() {
    relaxed_ = lowering::relaxedPrecisionTensors(g_);
    const std::string kname = g_.name + "_kernel";
    src_ << "// Generated by the akg HIP lowering for gfx950. Op description: " << g_.name << "\n";
    src_ << "// family: indexed, fusion class: " << operatorTemplateName(g_.operatorTemplate) << "\n";
    src_ << "#include \"akg_rt.hpp\"\n\n";
    src_ << "extern \"C\" __global__ __launch_bounds__(" << kBlock << ") void " << kname << "(";
    size_t argc = 0;
    for (size_t i = 0; i < g_.inputs.size(); ++i, ++argc) {
      const bool written = !assignedInput_.empty() && assignedInput_[i];
      src_ << (argc ? ", " : "") << (written ? "" : "const ") << tagOf(g_.inputs[i]) << "::storage *__restrict__ in" << i;
    }
    for (size_t i = 0; i < g_.outputs.size(); ++i, ++argc) {
      src_ << (argc ? ", " : "") << tagOf(g_.outputs[i]) << "::storage *__restrict__ out" << i;
    }
    chunksArg_ = opt_.extentAsArgument && staged_.empty();
    if (chunksArg_) src_ << ", const long akg_chunks_arg";
    src_ << ") {\n";
    if (!staged_.empty() && !assignedInput_.empty()) {
      throw LoweringError("an Assign next to a transpose that is staged through LDS tiles has no kernel yet");
    }
    if (!staged_.empty()) {
      emitTiledBody();
      src_ << "}\n";
      return;
    }
    int64_t numel = 1;
    for (int64_t d : space_) numel *= d;
    src_ << "  constexpr int V = " << vec_ << ";\n";
    src_ << "  const int chunk = static_cast<int>(blockIdx.x) * " << kBlock << " + static_cast<int>(threadIdx.x);\n";
    chunksTotal_ = numel / space_.back() * chunksPerRow_;
    if (chunksArg_) {
      src_ << "  if (chunk >= static_cast<int>(akg_chunks_arg)) return;\n";
    } else {
      src_ << "  if (chunk >= " << chunksTotal_ << ") return;\n";
    }
    if (overlapTail_) {
      src_ << "  int akg_inner = (chunk % " << chunksPerRow_ << ") * V;\n";
      src_ << "  if (akg_inner > " << space_.back() - vec_ << ") akg_inner = " << space_.back() - vec_ << ";\n";
      src_ << "  const int base = (chunk / " << chunksPerRow_ << ") * " << space_.back()
           << " + akg_inner;  // linear position of this thread's first element\n";
    } else {
      src_ << "  const int base = chunk * V;  // linear position of this thread's first element\n";
    }
    indent_ = 1;
    scopes_.clear();
    scopes_.emplace_back();
    // index of the chunk's first element; the innermost coordinate advances with e and never wraps
    Index start = delinearize("base", space_);
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      stmt(ctOf(g_.outputs[i]) + " o" + std::to_string(i) + "[V];");
    }
    Index idx = start;
    if (space_.back() != 1) {
      stmt("const int inner0 = " + start.back().s + ";" +
           (overlapTail_ ? "" : "  // a multiple of V: V divides the innermost extent"));
      idx.back() = affine("inner0", !overlapTail_, true);
    }
    canonical_ = idx;
    openElementLoop(indent_);
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      const std::string v = valueAt(g_.outputs[i], idx);
      stmt("o" + std::to_string(i) + "[e] = " + v + ";");
    }
    closeElementLoop();
    for (size_t i = 0; i < g_.outputs.size(); ++i) {
      // results are written once and never read by this kernel: non-temporal where whole 64-byte pieces are stored
      const bool ntOut = opt_.nonTemporal != 0 &&
                         (space_.back() * static_cast<int64_t>(dtypeSize(g_.tensor(g_.outputs[i]).dtype))) % 64 == 0;
      stmt(std::string("akg::store_chunk") + (overlapTail_ ? "_unaligned<" : "<") + tagOf(g_.outputs[i]) + ", V" +
           (overlapTail_ ? "" : (ntOut ? ", true" : ", false")) + ">(out" + std::to_string(i) + " + base, o" +
           std::to_string(i) + ");");
      // an output that is the result of an Assign: the same chunk goes over the destination
      const int producer = g_.tensor(g_.outputs[i]).producer;
      if (producer >= 0 && g_.ops[static_cast<size_t>(producer)].kind == OpKind::Assign) {
        const OpNode &as = g_.ops[static_cast<size_t>(producer)];
        stmt("akg::store_chunk<" + tagOf(g_.outputs[i]) + ", V, false>(in" + std::to_string(g_.tensor(as.inputs[0]).inputIndex) +
             " + base, o" + std::to_string(i) + ");  // " + as.name + " -> " + g_.tensor(as.inputs[0]).name);
      }
    }
    src_ << "}\n";
  }
};

}  // namespace

bool wantsIndexedKernel(const OpGraph &graph) {
  bool reshapes = false, contraction = false;
  for (const OpNode &op : graph.ops) {
    if (isViewKind(op.kind)) return true;
    if (op.kind == OpKind::MatMul || lowering::isReduceKind(op.kind)) contraction = true;
    if (op.kind == OpKind::Reshape) {
      // A Reshape that only adds or drops leading unit dimensions keeps every operand right-aligned with the
      // outputs, which is what the chunked elementwise kernel relies on; any other Reshape changes how the
      // dimensions of operands in front of it line up with the outputs' and needs real index arithmetic.
      std::vector<int64_t> a = graph.tensor(op.inputs[0]).shape, b = graph.tensor(op.outputs[0]).shape;
      while (a.size() > 1 && a.front() == 1) a.erase(a.begin());
      while (b.size() > 1 && b.front() == 1) b.erase(b.begin());
      if (a != b) reshapes = true;
    }
  }
  return reshapes && !contraction;
}

LoweredKernel lowerIndexedToHip(const OpGraph &graph, const LoweringOptions &options) {
  IndexedEmitter emitter(graph, options);
  return emitter.run();
}

}  // namespace akg
