/**
 * C-ABI layer: compile (translate -> identify -> lower -> hiprtc -> artifacts) and the runtime launch shim.
 *
 * The launch shim replaces the CUDA driver-API program that the reference generates per kernel from a Python
 * string template (akg-mlir/python/akg_mlir/utils/code_template.py:16-212, filled by gen_runtime_code.py:149-189).
 * Differences that matter on MI355X: the code object is loaded once per handle, launches go to a caller's
 * stream with device-resident buffers (akg_hip_launch), and the reference-style "host pointers in, host
 * pointers out" call (akg_hip_run_host) is kept as a separate, explicitly slower entry point.
 */
#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cerrno>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <fstream>
#include <map>
#include <memory>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/akg_hip.h"
#include "HipLowering.h"
#include "Staging.h"
#include "Json.h"
#include "OpGraph.h"
#include "Sha256.h"
#include "StaticScratch.h"

// Text of the device-side headers, generated at build time from kernels/*.hpp.
#include "KernelLibEmbed.inc"

#define AKG_HIP_VERSION_STRING "akg-hip 0.1 (gfx950)"

struct akg_hip_kernel {
  akg::OpGraph graph;
  akg::LoweredKernel lowered;
  // (shared between the handles that were made from one source: the specialisations of a dynamic description)
  std::shared_ptr<const std::vector<char>> codeObject;
  std::string codeSha256;
  bool cacheHit = false;
  double buildMs = 0.0;   // wall time of translation, lowering and (unless cached) device compilation of this handle
  std::mutex mu;
  // loaded lazily on first launch, per device
  struct Loaded {
    int device = -1;
    hipModule_t module = nullptr;
    hipFunction_t function = nullptr;
    std::vector<hipFunction_t> earlier;  // lowered.earlierPhases, in their order
    void *workspace = nullptr;  // lowered.workspaceBytes of zero-filled device memory, or NULL
    // Launches of one handle share its workspace. They are ordered on the device by the library: a launch that goes to
    // another stream than the last one first waits (through this event) for what that stream holds.
    hipEvent_t lastUse = nullptr;
    hipStream_t lastStream = nullptr;
    bool used = false;
    bool recorded = false;   // lastUse was recorded behind the previous launch already (AKG_HIP_SAFE_STREAMS=1)
    // a launch sequence that failed half way may have left arrival counters set: zero-fill before the next launch
    bool dirty = false;
  };
  std::deque<Loaded> loaded;   // (a deque: launches keep pointers to their entry while other devices are added)
  // A description run as a sequence of kernels (Staging.h): each stage is a handle of its own; this handle owns
  // them and the temporaries between them (its workspace), and has no code object itself.
  struct Stage {
    akg_hip_kernel *kernel = nullptr;
    std::vector<akg::StageArg> args;
  };
  std::vector<Stage> stages;
  std::vector<uint64_t> tempBytes, tempOffsets;
};

// Code objects compiled in this process, by the digest of their source (identical sources arise when a dynamic
// description is specialised to shape sets that its kernel takes as an argument, and when one description is compiled
// twice).
std::mutex g_codeCacheMutex;
std::map<std::string, std::shared_ptr<const std::vector<char>>> g_codeCache;

// Code objects loaded on a device, by the digest of the code object: handles made from one source (every token count
// of a dynamic MatMul is a handle of its own) share one module instead of loading a copy each.
struct SharedModule {
  hipModule_t module = nullptr;
  long refs = 0;
};
std::mutex g_moduleMutex;
std::map<std::pair<std::string, int>, SharedModule> g_modules;

// A dynamic-shape description and the kernels specialised from it so far, keyed by the bound input shapes.
struct akg_hip_dynamic {
  std::string jsonText;
  std::string outDir;
  bool hasOutDir = false;
  int numInputs = 0;
  std::vector<int> inputRanks;
  std::vector<int> outputRanks;   // declared ranks of the outputs (output_desc), for the packed launch form
  std::mutex mu;
  std::map<std::string, akg_hip_kernel_t *> specializations;
};

namespace {

thread_local std::string g_lastError;

int fail(int code, const std::string &msg) {
  g_lastError = msg;
  return code;
}

std::string hipErr(hipError_t e) { return std::string(hipGetErrorName(e)) + ": " + hipGetErrorString(e); }

const std::vector<std::string> &compileFlags() {
  // -ffp-contract=off: every op of the description is its own IEEE operation in the reference CPU pipeline;
  //   fusing a*b+c into an fma would change results (and break the bit-exact int8 quantisation).
  // packed-fp32-ops off: the compiler must not form v_pk_{add,mul,fma}_f32.
  static const std::vector<std::string> flags = [] {
    std::vector<std::string> f = {
      "--offload-arch=gfx950", "-O3",      "-std=c++17",     "-ffp-contract=off",
      "-Xclang",               "-target-feature", "-Xclang", "-packed-fp32-ops",
      // No SLP vectorisation: with packed float32 operations switched off, a two-lane float32 subtraction it forms
      // next to 16-bit conversions has ended instruction selection with a fatal error (which ends the calling
      // process), and the measured kernels run the same without it (every figure within its run-to-run spread).
      "-fno-slp-vectorize",
    };
    // AKG_HIP_EXTRA_FLAGS: space-separated extra device-compiler flags (experiments; part of the cache key)
    if (const char *extra = std::getenv("AKG_HIP_EXTRA_FLAGS")) {
      std::istringstream is(extra);
      std::string tok;
      while (is >> tok) f.push_back(tok);
    }
    return f;
  }();
  return flags;
}

std::string sourceDigest(const std::string &source) {
  akg::Sha256 h;
  h.update(source.data(), source.size());
  for (size_t i = 0; i < akg::kernel_lib::kNumHeaders; ++i) {
    h.update(akg::kernel_lib::kHeaderNames[i], std::strlen(akg::kernel_lib::kHeaderNames[i]));
    h.update(akg::kernel_lib::kHeaderTexts[i], std::strlen(akg::kernel_lib::kHeaderTexts[i]));
  }
  for (const auto &f : compileFlags()) h.update(f.data(), f.size());
  return h.hexDigest();
}

bool readFile(const std::string &path, std::string *out) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return false;
  std::ostringstream ss;
  ss << f.rdbuf();
  *out = ss.str();
  return true;
}

bool writeFile(const std::string &path, const void *data, size_t len) {
  // (a temporary name of this process and call: several processes may fill one artifact directory at once, and two
  // writers of one temporary file could publish it half written)
  static std::atomic<unsigned long> serial{0};
  std::string tmp = path + ".tmp." + std::to_string(static_cast<long>(getpid())) + "." + std::to_string(serial.fetch_add(1));
  {
    std::ofstream f(tmp, std::ios::binary | std::ios::trunc);
    if (!f) return false;
    f.write(static_cast<const char *>(data), static_cast<std::streamsize>(len));
    if (!f) return false;
  }
  if (std::rename(tmp.c_str(), path.c_str()) == 0) return true;
  (void)std::remove(tmp.c_str());
  return false;
}

bool makeDirs(const std::string &dir) {
  if (dir.empty()) return false;
  std::string cur;
  for (size_t i = 0; i <= dir.size(); ++i) {
    if (i == dir.size() || dir[i] == '/') {
      if (!cur.empty() && cur != "/") {
        if (mkdir(cur.c_str(), 0755) != 0 && errno != EEXIST) return false;
      }
    }
    if (i < dir.size()) cur.push_back(dir[i]);
  }
  struct stat st;
  return stat(dir.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}

int compileToCodeObject(const akg::LoweredKernel &k, std::vector<char> *code, std::string *log) {
  hiprtcProgram prog = nullptr;
  std::vector<const char *> headerTexts, headerNames;
  for (size_t i = 0; i < akg::kernel_lib::kNumHeaders; ++i) {
    headerTexts.push_back(akg::kernel_lib::kHeaderTexts[i]);
    headerNames.push_back(akg::kernel_lib::kHeaderNames[i]);
  }
  std::string progName = k.kernelName + ".hip";
  // AKG_HIP_DUMP_SOURCE=DIR: every source goes to DIR/<kernel>.hip before the device compiler sees it (the compiler
  // ends the process on an internal error; the source that did it is then on disk)
  if (const char *dumpDir = std::getenv("AKG_HIP_DUMP_SOURCE")) {
    if (dumpDir[0] != 0 && makeDirs(dumpDir)) writeFile(std::string(dumpDir) + "/" + progName, k.source.data(), k.source.size());
  }
  hiprtcResult r = hiprtcCreateProgram(&prog, k.source.c_str(), progName.c_str(), static_cast<int>(headerTexts.size()),
                                       headerTexts.data(), headerNames.data());
  if (r != HIPRTC_SUCCESS) {
    *log = std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r);
    return AKG_HIP_ERR_COMPILE;
  }
  std::vector<const char *> opts;
  for (const auto &f : compileFlags()) opts.push_back(f.c_str());
  r = hiprtcCompileProgram(prog, static_cast<int>(opts.size()), opts.data());
  size_t logSize = 0;
  if (hiprtcGetProgramLogSize(prog, &logSize) == HIPRTC_SUCCESS && logSize > 1) {
    log->resize(logSize);
    hiprtcGetProgramLog(prog, &(*log)[0]);
  }
  if (r != HIPRTC_SUCCESS) {
    *log = std::string("hiprtcCompileProgram: ") + hiprtcGetErrorString(r) + "\n" + *log;
    hiprtcDestroyProgram(&prog);
    return AKG_HIP_ERR_COMPILE;
  }
  size_t size = 0;
  r = hiprtcGetCodeSize(prog, &size);
  if (r != HIPRTC_SUCCESS || size == 0) {
    *log = "hiprtcGetCodeSize failed";
    hiprtcDestroyProgram(&prog);
    return AKG_HIP_ERR_COMPILE;
  }
  code->resize(size);
  r = hiprtcGetCode(prog, code->data());
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    *log = "hiprtcGetCode failed";
    return AKG_HIP_ERR_COMPILE;
  }
  return AKG_HIP_OK;
}

std::string jsonEscape(const std::string &s) {
  std::string o;
  for (char c : s) {
    if (c == '"' || c == '\\') {
      o.push_back('\\');
      o.push_back(c);
    } else if (c == '\n') {
      o += "\\n";
    } else {
      o.push_back(c);
    }
  }
  return o;
}

// <op>.json: mapping result (GPUMapping.cpp:645-665) + kernelName / is_dynamic / sha256 (mlir_driver.py:807-815),
// plus this backend's own bookkeeping keys.
std::string metaJson(const akg_hip_kernel &k, const std::string &srcDigest) {
  std::ostringstream os;
  os << "{";
  os << "\"blockIdx.x\": " << k.lowered.grid[0] << ", \"blockIdx.y\": " << k.lowered.grid[1]
     << ", \"blockIdx.z\": " << k.lowered.grid[2] << ", ";
  os << "\"threadIdx.x\": " << k.lowered.block[0] << ", \"threadIdx.y\": " << k.lowered.block[1]
     << ", \"threadIdx.z\": " << k.lowered.block[2] << ", ";
  os << "\"kernelName\": \"" << jsonEscape(k.lowered.kernelName) << "\", ";
  os << "\"is_dynamic\": false, ";
  os << "\"sha256\": \"" << k.codeSha256 << "\", ";
  os << "\"target_info\": {\"arch\": \"gfx950\"}, ";
  os << "\"family\": \"" << akg::kernelFamilyName(k.lowered.family) << "\", ";
  os << "\"OperatorType\": \"" << akg::operatorTemplateName(k.graph.operatorTemplate) << "\", ";
  os << "\"schedule\": \"" << jsonEscape(k.lowered.scheduleNote) << "\", ";
  os << "\"algorithmic_bytes\": " << k.lowered.algorithmicBytes << ", ";
  os << "\"algorithmic_ops\": " << k.lowered.algorithmicOps << ", ";
  os << "\"workspace_bytes\": " << k.lowered.workspaceBytes << ", ";
  if (!k.lowered.scalarArgs.empty()) {
    // a specialisation of a dynamic description whose kernel takes extents as arguments: these 64-bit values follow
    // the tensor pointers in the kernel's argument list (the workspace pointer, if any, comes last)
    os << "\"scalar_args\": [";
    for (size_t i = 0; i < k.lowered.scalarArgs.size(); ++i) os << (i ? ", " : "") << k.lowered.scalarArgs[i];
    os << "], ";
  }
  if (!k.stages.empty()) {
    // the description runs as these kernels, in this order, each with artifacts of its own under its name; "args" says
    // where each tensor of a stage's signature lives: input i / output j of this description, or temporary t at a byte
    // offset of the workspace
    os << "\"stages\": [";
    for (size_t i = 0; i < k.stages.size(); ++i) {
      const auto &st = k.stages[i];
      os << (i ? ", " : "") << "{\"kernelName\": \"" << jsonEscape(st.kernel->lowered.kernelName) << "\", \"args\": [";
      for (size_t a = 0; a < st.args.size(); ++a) {
        const akg::StageArg &sa = st.args[a];
        os << (a ? ", " : "");
        if (sa.kind == akg::StageArg::Kind::Input) {
          os << "{\"input\": " << sa.index << "}";
        } else if (sa.kind == akg::StageArg::Kind::Output) {
          os << "{\"output\": " << sa.index << "}";
        } else {
          os << "{\"workspace_offset\": " << k.tempOffsets[static_cast<size_t>(sa.index)] << "}";
        }
      }
      os << "]}";
    }
    os << "], ";
  }
  if (!k.lowered.earlierPhases.empty()) {
    // kernels of the same code object to launch before kernelName, in this order, with the same arguments
    os << "\"earlier_phases\": [";
    for (size_t i = 0; i < k.lowered.earlierPhases.size(); ++i) {
      const akg::KernelPhase &ph = k.lowered.earlierPhases[i];
      os << (i ? ", " : "") << "{\"kernelName\": \"" << jsonEscape(ph.kernelName) << "\", \"blockIdx.x\": " << ph.grid[0]
         << ", \"blockIdx.y\": " << ph.grid[1] << ", \"blockIdx.z\": " << ph.grid[2] << ", \"threadIdx.x\": " << ph.block[0]
         << ", \"threadIdx.y\": " << ph.block[1] << ", \"threadIdx.z\": " << ph.block[2] << "}";
    }
    os << "], ";
  }
  os << "\"source_sha256\": \"" << srcDigest << "\"";
  os << "}";
  return os.str();
}

std::string shapeArgText(const akg::LoweredKernel &k) {
  std::ostringstream os;
  os << "[";
  for (size_t i = 0; i < k.shapeArgs.size(); ++i) {
    os << (i ? "," : "") << "[";
    for (size_t j = 0; j < k.shapeArgs[i].size(); ++j) os << (j ? "," : "") << k.shapeArgs[i][j];
    os << "]";
  }
  os << "]";
  return os.str();
}

// <op>_shape_info.json (DumpShapeInfo.cpp:133-142): shapes as the caller sees them and as the kernel addresses them.
// Kernels here take bare pointers to the caller's dense row-major buffers and carry every extent as a compile-time
// constant, so both lists are the tensors' own shapes and there are no runtime variables.
std::string shapeInfoJson(const akg::OpGraph &g) {
  std::ostringstream shapes;
  shapes << "[";
  bool first = true;
  auto emitShape = [&](int id) {
    shapes << (first ? "" : ", ") << "[";
    const auto &s = g.tensor(id).shape;
    for (size_t i = 0; i < s.size(); ++i) shapes << (i ? ", " : "") << s[i];
    shapes << "]";
    first = false;
  };
  for (int id : g.inputs) emitShape(id);
  for (int id : g.outputs) emitShape(id);
  shapes << "]";
  return "{\"hostShapes\": " + shapes.str() + ", \"deviceShapes\": " + shapes.str() +
         ", \"runtimeVars\": [], \"SupportInfo\": {}}";
}

int doCompile(const std::string &jsonText, const char *outDir, akg_hip_kernel_t **outKernel,
              const akg::ShapeBinding *binding = nullptr, bool allowStages = true);

void destroyKernel(akg_hip_kernel *kernel);

// The description as a sequence of kernels. `k` holds the translated graph; `reason` is why no single kernel serves it.
int compileStaged(const std::string &jsonText, std::unique_ptr<akg_hip_kernel> k, const char *outDir,
                  akg_hip_kernel_t **outKernel, const std::string &reason, bool dynamic, const std::string &artifactSuffix) {
  const std::string refusal = std::string("kernel ") + k->graph.name + ": " + reason;
  akg::StagingPlan plan;
  std::string why;
  try {
    // first only behind contractions and data-movement ops (the pieces are compiled with staging allowed again, so a
    // piece that still needs it is cut at its reductions); if there is no such cut, at the reductions
    if (!akg::planStages(jsonText, k->graph, false, &plan, &why) && !akg::planStages(jsonText, k->graph, true, &plan, &why)) {
      return fail(AKG_HIP_ERR_UNSUPPORTED, refusal + " (and it cannot run as several kernels: " + why + ")");
    }
  } catch (const std::exception &e) {
    return fail(AKG_HIP_ERR_UNSUPPORTED, refusal);
  }
  k->tempBytes = plan.tempBytes;
  bool allHits = true;
  std::ostringstream source, note;
  note << "staged:";
  for (const akg::StagePlan &sp : plan.stages) {
    akg_hip_kernel_t *stage = nullptr;
    // a stage of a dynamic description is specialised to the shapes its tensors have in the bound graph (its op
    // entries still carry the open dimensions)
    akg::ShapeBinding stageBinding;
    if (dynamic) {
      stageBinding.inputShapes.assign(sp.shapes.begin(), sp.shapes.end() - static_cast<long>(sp.numOutputs));
    }
    const int rc = doCompile(sp.jsonText, outDir, &stage, dynamic ? &stageBinding : nullptr, true);
    if (rc != AKG_HIP_OK) {
      const std::string inner = g_lastError;
      for (auto &st : k->stages) destroyKernel(st.kernel);
      k->stages.clear();
      return fail(AKG_HIP_ERR_UNSUPPORTED, refusal + " (and as several kernels: " + inner + ")");
    }
    allHits = allHits && stage->cacheHit;
    std::vector<akg_hip_kernel::Stage> pieces;
    if (stage->stages.empty()) {
      akg_hip_kernel::Stage st;
      st.kernel = stage;
      st.args = sp.args;
      pieces.push_back(st);
    } else {
      // the piece needed stages of its own: they become stages of this handle, their tensors found through the piece's
      // bindings and their temporaries appended to this handle's
      const size_t pieceInputs = sp.args.size() - sp.numOutputs;
      const int tempBase = static_cast<int>(k->tempBytes.size());
      k->tempBytes.insert(k->tempBytes.end(), stage->tempBytes.begin(), stage->tempBytes.end());
      for (auto &inner : stage->stages) {
        akg_hip_kernel::Stage st;
        st.kernel = inner.kernel;
        for (const akg::StageArg &a : inner.args) {
          akg::StageArg m = a;
          if (a.kind == akg::StageArg::Kind::Input) {
            m = sp.args[static_cast<size_t>(a.index)];
          } else if (a.kind == akg::StageArg::Kind::Output) {
            m = sp.args[pieceInputs + static_cast<size_t>(a.index)];
          } else {
            m.index = tempBase + a.index;
          }
          st.args.push_back(m);
        }
        pieces.push_back(st);
      }
      stage->stages.clear();   // ownership moved
      destroyKernel(stage);
    }
    for (const auto &st : pieces) {
      k->stages.push_back(st);
      source << "// ---- " << st.kernel->lowered.kernelName << "\n" << st.kernel->lowered.source << "\n";
      note << " | " << st.kernel->lowered.kernelName << ": " << akg::kernelFamilyName(st.kernel->lowered.family) << " grid="
           << st.kernel->lowered.grid[0] << " block=" << st.kernel->lowered.block[0];
    }
  }
  uint64_t offset = 0;
  for (uint64_t bytes : k->tempBytes) {
    k->tempOffsets.push_back(offset);
    offset += (bytes + 255) / 256 * 256;
  }
  const akg_hip_kernel *last = k->stages.back().kernel;
  k->graph.name += artifactSuffix;
  k->lowered = akg::LoweredKernel();
  k->lowered.kernelName = last->lowered.kernelName;
  k->lowered.family = akg::KernelFamily::Staged;
  for (int d = 0; d < 3; ++d) {
    k->lowered.grid[d] = last->lowered.grid[d];
    k->lowered.block[d] = last->lowered.block[d];
  }
  k->lowered.source = source.str();
  k->lowered.scheduleNote = note.str();
  k->lowered.algorithmicBytes = akg::lowering::countAlgorithmicBytes(k->graph);
  k->lowered.shapeArgs = akg::lowering::buildShapeArgs(k->graph);
  k->lowered.workspaceBytes = offset;
  k->cacheHit = allHits;
  if (outDir != nullptr && outDir[0] != 0) {
    const std::string base = std::string(outDir) + "/" + k->graph.name;
    const std::string meta = metaJson(*k, sourceDigest(k->lowered.source));
    const std::string shapeArg = shapeArgText(k->lowered);
    const std::string shapeInfo = shapeInfoJson(k->graph);
    if (!writeFile(base + "_shape_info.json", shapeInfo.data(), shapeInfo.size()) ||
        !writeFile(base + "_shape_arg.txt", shapeArg.data(), shapeArg.size()) ||
        !writeFile(base + ".json", meta.data(), meta.size())) {
      for (auto &st : k->stages) destroyKernel(st.kernel);
      k->stages.clear();
      return fail(AKG_HIP_ERR_IO, std::string("cannot write artifacts under ") + outDir);
    }
  }
  *outKernel = k.release();
  g_lastError.clear();
  return AKG_HIP_OK;
}

int doCompileTimed(const std::string &jsonText, const char *outDir, akg_hip_kernel_t **outKernel,
                   const akg::ShapeBinding *binding, bool allowStages);

int doCompile(const std::string &jsonText, const char *outDir, akg_hip_kernel_t **outKernel,
              const akg::ShapeBinding *binding, bool allowStages) {
  const auto t0 = std::chrono::steady_clock::now();
  const int rc = doCompileTimed(jsonText, outDir, outKernel, binding, allowStages);
  if (rc == AKG_HIP_OK && outKernel != nullptr && *outKernel != nullptr) {
    (*outKernel)->buildMs = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  }
  return rc;
}

int doCompileTimed(const std::string &jsonText, const char *outDir, akg_hip_kernel_t **outKernel,
                   const akg::ShapeBinding *binding, bool allowStages) {
  if (outKernel == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "out_kernel is NULL");
  *outKernel = nullptr;
  std::unique_ptr<akg_hip_kernel> k(new akg_hip_kernel());
  std::string artifactSuffix;
  try {
    k->graph = akg::translateJsonToOpGraph(jsonText, binding);
    if (binding != nullptr) {
      // one artifact set per shape: the specialisation is named after a digest of the bound input shapes
      akg::Sha256 h;
      for (const auto &shape : binding->inputShapes) {
        for (int64_t d : shape) {
          const std::string t = std::to_string(d) + ",";
          h.update(t.data(), t.size());
        }
        h.update(";", 1);
      }
      artifactSuffix = "_s" + h.hexDigest().substr(0, 12);
    }
  } catch (const akg::json::ParseError &e) {
    return fail(AKG_HIP_ERR_JSON, e.what());
  } catch (const akg::TranslateError &e) {
    return fail(AKG_HIP_ERR_TRANSLATE, e.what());
  }
  if (binding == nullptr) {
    // ArgMax over an axis that is not the innermost one: respelled as Transpose + ArgMax over the last axis (+ Reshape)
    bool outerArgMax = false;
    for (const akg::OpNode &op : k->graph.ops) {
      if (op.kind != akg::OpKind::ArgMax || op.axes.size() != 1) continue;
      const std::vector<int64_t> &shape = k->graph.tensor(op.inputs[0]).shape;
      for (size_t d = static_cast<size_t>(op.axes[0]) + 1; d < shape.size(); ++d) outerArgMax = outerArgMax || shape[d] != 1;
    }
    std::string respelled;
    try {
      if (outerArgMax && akg::moveArgMaxToInnermostAxis(jsonText, &respelled)) {
        return doCompileTimed(respelled, outDir, outKernel, binding, allowStages);
      }
    } catch (const std::exception &) {
      // leave the description as it is: the lowering below says what it cannot do
    }
  }
  try {
    akg::LoweringOptions options = akg::LoweringOptions::fromEnvironment();
    options.extentAsArgument = binding != nullptr;
    k->lowered = akg::lowerToHip(k->graph, options);
    // the kernel keeps the description's name (shape sets may share its code object); the artifacts are per shape set
    k->graph.name += artifactSuffix;
  } catch (const akg::LoweringError &e) {
    if (allowStages) {
      return compileStaged(jsonText, std::move(k), outDir, outKernel, e.what(), binding != nullptr, artifactSuffix);
    }
    return fail(AKG_HIP_ERR_UNSUPPORTED, std::string("kernel ") + k->graph.name + ": " + e.what());
  }
  const std::string srcDigest = sourceDigest(k->lowered.source);
  bool fromMemory = false;

  std::string dir = outDir ? std::string(outDir) : std::string();
  std::string base;
  if (!dir.empty()) {
    if (!makeDirs(dir)) return fail(AKG_HIP_ERR_IO, "cannot create artifact directory " + dir);
    base = dir + "/" + k->graph.name;
    // cache probe (AKG_HIP_NO_CACHE=1 forces a fresh device compilation)
    const char *noCache = std::getenv("AKG_HIP_NO_CACHE");
    std::string meta, code;
    if (!(noCache && noCache[0] == '1') && readFile(base + ".json", &meta) && readFile(base + ".hsaco", &code) && !code.empty()) {
      try {
        akg::json::Value mv = akg::json::Value::parse(meta);
        if (mv.contains("source_sha256") && mv.at("source_sha256").asString() == srcDigest &&
            mv.contains("sha256") && mv.at("sha256").asString() == akg::Sha256::of(code)) {
          k->codeObject = std::make_shared<const std::vector<char>>(code.begin(), code.end());
          k->codeSha256 = mv.at("sha256").asString();
          k->cacheHit = true;
        }
      } catch (const std::exception &) {
        // unreadable meta: recompile
      }
    }
  }
  if (!k->cacheHit && !(std::getenv("AKG_HIP_NO_CACHE") && std::getenv("AKG_HIP_NO_CACHE")[0] == '1')) {
    // code objects compiled earlier in this process, by source digest
    std::lock_guard<std::mutex> lock(g_codeCacheMutex);
    auto it = g_codeCache.find(srcDigest);
    if (it != g_codeCache.end()) {
      k->codeObject = it->second;
      akg::Sha256 h;
      h.update(k->codeObject->data(), k->codeObject->size());
      k->codeSha256 = h.hexDigest();
      k->cacheHit = true;
      fromMemory = true;
    }
  }
  if (!k->cacheHit && !dir.empty() && !(std::getenv("AKG_HIP_NO_CACHE") && std::getenv("AKG_HIP_NO_CACHE")[0] == '1')) {
    // code objects compiled by any process that used this artifact directory, by source digest: a shape set this
    // process meets for the first time may share its source with one another process has compiled
    std::string code;
    if (readFile(dir + "/by_source/" + srcDigest + ".hsaco", &code) && !code.empty()) {
      k->codeObject = std::make_shared<const std::vector<char>>(code.begin(), code.end());
      k->codeSha256 = akg::Sha256::of(code);
      k->cacheHit = true;
      fromMemory = true;
      std::lock_guard<std::mutex> lock(g_codeCacheMutex);
      if (g_codeCache.size() < 1024) g_codeCache[srcDigest] = k->codeObject;
    }
  }
  if (!k->cacheHit || (fromMemory && !base.empty())) {
    std::string log;
    int rc = AKG_HIP_OK;
    if (!fromMemory) {
      std::vector<char> fresh;
      rc = compileToCodeObject(k->lowered, &fresh, &log);
      if (rc == AKG_HIP_OK) k->codeObject = std::make_shared<const std::vector<char>>(std::move(fresh));
    }
    if (rc != AKG_HIP_OK) {
      if (!base.empty()) (void)writeFile(base + ".hip", k->lowered.source.data(), k->lowered.source.size());
      if (k->lowered.family == akg::KernelFamily::ColumnReduce && allowStages) {
        // The column kernel is an optimisation over one kernel per reduction level (registers of two resident sets,
        // LDS of the widest strips): if its source does not compile, the description still runs the other way.
        if (!artifactSuffix.empty() && k->graph.name.size() > artifactSuffix.size()) {
          k->graph.name.erase(k->graph.name.size() - artifactSuffix.size());
        }
        return compileStaged(jsonText, std::move(k), outDir, outKernel,
                             "device compilation of the column kernel failed (" + log.substr(0, 200) + ")", binding != nullptr, artifactSuffix);
      }
      return fail(rc, "device compilation of " + k->lowered.kernelName + " failed:\n" + log);
    }
    akg::Sha256 h;
    h.update(k->codeObject->data(), k->codeObject->size());
    k->codeSha256 = h.hexDigest();
    if (!fromMemory) {
      {
        std::lock_guard<std::mutex> lock(g_codeCacheMutex);
        if (g_codeCache.size() < 1024) g_codeCache[srcDigest] = k->codeObject;   // bounded: some tens of MB at most
      }
      if (!dir.empty() && makeDirs(dir + "/by_source")) {
        (void)writeFile(dir + "/by_source/" + srcDigest + ".hsaco", k->codeObject->data(), k->codeObject->size());
      }
    }
    if (!base.empty()) {
      std::string meta = metaJson(*k, srcDigest);
      std::string shapeArg = shapeArgText(k->lowered);
      std::string shapeInfo = shapeInfoJson(k->graph);
      if (!writeFile(base + "_shape_info.json", shapeInfo.data(), shapeInfo.size()) ||
          !writeFile(base + ".hip", k->lowered.source.data(), k->lowered.source.size()) ||
          !writeFile(base + ".hsaco", k->codeObject->data(), k->codeObject->size()) ||
          !writeFile(base + "_shape_arg.txt", shapeArg.data(), shapeArg.size()) ||
          !writeFile(base + ".json", meta.data(), meta.size())) {
        return fail(AKG_HIP_ERR_IO, "cannot write artifacts under " + dir);
      }
    }
  }
  *outKernel = k.release();
  g_lastError.clear();
  return AKG_HIP_OK;
}

// The module of `k`'s code object on `device` (the current one): loaded once per process and device, counted per user.
hipError_t acquireModule(const akg_hip_kernel &k, int device, hipModule_t *out) {
  std::lock_guard<std::mutex> lock(g_moduleMutex);
  SharedModule &m = g_modules[std::make_pair(k.codeSha256, device)];
  if (m.module == nullptr) {
    const hipError_t e = hipModuleLoadData(&m.module, k.codeObject->data());
    if (e != hipSuccess) {
      g_modules.erase(std::make_pair(k.codeSha256, device));
      return e;
    }
  }
  ++m.refs;
  *out = m.module;
  return hipSuccess;
}

void releaseModule(const std::string &codeSha256, int device) {
  std::lock_guard<std::mutex> lock(g_moduleMutex);
  auto it = g_modules.find(std::make_pair(codeSha256, device));
  if (it == g_modules.end()) return;
  if (--it->second.refs <= 0) {
    (void)hipModuleUnload(it->second.module);
    g_modules.erase(it);
  }
}

// Code object and workspace of `k` on the current device, loaded / allocated on first use.
int ensureLoaded(akg_hip_kernel *k, akg_hip_kernel::Loaded **out) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipGetDevice: " + hipErr(e));
  std::lock_guard<std::mutex> lock(k->mu);
  for (auto &l : k->loaded) {
    if (l.device == device) {
      *out = &l;
      return AKG_HIP_OK;
    }
  }
  akg_hip_kernel::Loaded l;
  l.device = device;
  if (!k->stages.empty()) {
    for (auto &st : k->stages) {
      akg_hip_kernel::Loaded *ls = nullptr;
      const int rc = ensureLoaded(st.kernel, &ls);
      if (rc != AKG_HIP_OK) return rc;
    }
  } else {
    e = acquireModule(*k, device, &l.module);
    if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipModuleLoadData: " + hipErr(e));
    e = hipModuleGetFunction(&l.function, l.module, k->lowered.kernelName.c_str());
    if (e != hipSuccess) {
      releaseModule(k->codeSha256, device);
      return fail(AKG_HIP_ERR_RUNTIME, "hipModuleGetFunction(" + k->lowered.kernelName + "): " + hipErr(e));
    }
  }
  for (const akg::KernelPhase &ph : k->lowered.earlierPhases) {
    hipFunction_t f = nullptr;
    e = hipModuleGetFunction(&f, l.module, ph.kernelName.c_str());
    if (e != hipSuccess) {
      releaseModule(k->codeSha256, device);
      return fail(AKG_HIP_ERR_RUNTIME, "hipModuleGetFunction(" + ph.kernelName + "): " + hipErr(e));
    }
    l.earlier.push_back(f);
  }
  if (k->lowered.workspaceBytes > 0) {
    // Zero-filled once; every launch leaves the arrival counters at zero again. Launches of one handle share the
    // workspace, so they must not overlap on the device (launch them on one stream, or order the streams).
    e = hipMalloc(&l.workspace, k->lowered.workspaceBytes);
    if (e == hipSuccess) e = hipMemset(l.workspace, 0, k->lowered.workspaceBytes);
    // the fill runs on the null stream and may still be in flight when hipMemset returns; the first launch may go to
    // a stream that does not wait for the null stream
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&l.lastUse, hipEventDisableTiming);
    if (e != hipSuccess) {
      if (l.workspace) (void)hipFree(l.workspace);
      if (l.module) releaseModule(k->codeSha256, device);
      return fail(AKG_HIP_ERR_RUNTIME, "workspace of " + std::to_string(k->lowered.workspaceBytes) + " bytes: " + hipErr(e));
    }
  }
  k->loaded.push_back(l);
  *out = &k->loaded.back();
  return AKG_HIP_OK;
}

void destroyKernel(akg_hip_kernel *kernel) {
  if (kernel == nullptr) return;
  for (auto &st : kernel->stages) destroyKernel(st.kernel);
  for (auto &l : kernel->loaded) {
    if (l.lastUse) (void)hipEventDestroy(l.lastUse);
    if (l.workspace) (void)hipFree(l.workspace);
    if (l.module) releaseModule(kernel->codeSha256, l.device);
  }
  delete kernel;
}

int numTensors(const akg_hip_kernel *k) { return static_cast<int>(k->graph.inputs.size() + k->graph.outputs.size()); }

const akg::TensorValue &tensorAt(const akg_hip_kernel *k, int index) {
  size_t nin = k->graph.inputs.size();
  if (static_cast<size_t>(index) < nin) return k->graph.tensor(k->graph.inputs[static_cast<size_t>(index)]);
  return k->graph.tensor(k->graph.outputs[static_cast<size_t>(index) - nin]);
}

uint64_t alignScratch(uint64_t bytes) { return (bytes + 255) / 256 * 256; }

// Device memory beyond inputs and outputs that one launch of `k` uses: its own workspace (for a staged description the
// tensors between its kernels) followed by the workspaces of its stages, each piece a multiple of 256 bytes.
uint64_t scratchBytesNeeded(const akg_hip_kernel *k) {
  uint64_t total = alignScratch(k->lowered.workspaceBytes);
  for (const auto &st : k->stages) total += scratchBytesNeeded(st.kernel);
  return total;
}

// Code object of `k` (and of its stages) on `device`, if it has been loaded there; loads nothing.
bool findLoaded(akg_hip_kernel *k, int device, akg_hip_kernel::Loaded **out) {
  for (auto &st : k->stages) {
    akg_hip_kernel::Loaded *ls = nullptr;
    if (!findLoaded(st.kernel, device, &ls)) return false;
  }
  std::lock_guard<std::mutex> lock(k->mu);
  for (auto &l : k->loaded) {
    if (l.device == device) {
      *out = &l;
      return true;
    }
  }
  return false;
}

// Orders a launch that uses the handle's own workspace behind the handle's previous launch when that went to another
// stream, and zero-fills the workspace first if an earlier launch sequence broke off. Nothing of this is recorded into a
// stream capture (a captured launch is ordered by the graph it becomes part of).
struct WorkspaceTurn {
  akg_hip_kernel *k;
  akg_hip_kernel::Loaded *l;
  hipStream_t stream;
  bool active = false;      // the launch uses the handle's workspace and the stream is not capturing
  std::unique_lock<std::mutex> lock;
  WorkspaceTurn(akg_hip_kernel *kernel, akg_hip_kernel::Loaded *loaded, hipStream_t s, bool usesOwnWorkspace)
      : k(kernel), l(loaded), stream(s) {
    if (!usesOwnWorkspace || l->workspace == nullptr) return;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) (void)hipGetLastError();
    if (status != hipStreamCaptureStatusNone) return;
    lock = std::unique_lock<std::mutex>(k->mu);
    active = true;
  }
  int begin() {
    if (!active) return AKG_HIP_OK;
    if (l->used && l->lastStream != stream && l->recorded) {
      // the previous launch left its event behind itself: the stream it went to is not touched again
      const hipError_t e = hipStreamWaitEvent(stream, l->lastUse, 0);
      if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipStreamWaitEvent: " + hipErr(e));
    } else if (l->used && l->lastStream != stream) {
      // The event is recorded only now, at the switch of streams, behind everything enqueued on the previous stream so
      // far (an event after every launch would put a marker between back-to-back launches of the common one-stream
      // caller: 3 us on a 45 us reduction).
      hipStreamCaptureStatus prev = hipStreamCaptureStatusNone;
      hipError_t e = hipStreamIsCapturing(l->lastStream, &prev);
      if (e == hipSuccess && prev != hipStreamCaptureStatusNone) {
        return fail(AKG_HIP_ERR_RUNTIME, "kernel " + k->graph.name + ": its previous launch went to a stream that is being "
                                         "captured now; launches of one handle share its workspace and cannot be ordered across that");
      }
      if (e == hipSuccess) e = hipEventRecord(l->lastUse, l->lastStream);
      if (e == hipSuccess) {
        e = hipStreamWaitEvent(stream, l->lastUse, 0);
        if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipStreamWaitEvent: " + hipErr(e));
      } else {
        // the previous stream is gone (destroyed by the caller): wait for the device instead
        (void)hipGetLastError();
        e = hipDeviceSynchronize();
        if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipDeviceSynchronize: " + hipErr(e));
      }
    }
    if (l->dirty) {
      const hipError_t e = hipMemsetAsync(l->workspace, 0, k->lowered.workspaceBytes, stream);
      if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "clearing the workspace: " + hipErr(e));
      l->dirty = false;
    }
    return AKG_HIP_OK;
  }
  int end(int rc) {
    if (!active) return rc;
    if (rc != AKG_HIP_OK) {
      l->dirty = true;   // some launches of the sequence may have run: the counters cannot be trusted
    }
    // also after a failure: what did get enqueued still uses the workspace
    l->lastStream = stream;
    l->used = true;
    // AKG_HIP_SAFE_STREAMS=1: for callers that destroy streams between launches of one handle. The event goes behind
    // every launch (≈3 us between back-to-back launches), and the next launch on another stream waits for it without
    // ever touching this stream's handle again (which may be gone by then, or be another stream at the same address).
    const char *safe = std::getenv("AKG_HIP_SAFE_STREAMS");
    const bool safeStreams = safe != nullptr && safe[0] == '1';
    l->recorded = false;
    if (safeStreams && hipEventRecord(l->lastUse, stream) == hipSuccess) l->recorded = true;
    return rc;
  }
};

// Enqueues the kernel(s) of `k`. With `scratchBase` NULL the handle's own workspaces are used; otherwise the launch
// takes its scratchBytesNeeded(k) bytes from `scratchBase` (laid out as that function says) and nothing is loaded or
// allocated: every code object must be on the device already.
int launchSequence(akg_hip_kernel *k, akg_hip_kernel::Loaded &l, void *const *devicePtrs, hipStream_t stream,
                   char *scratchBase);

int launchOn(akg_hip_kernel *k, akg_hip_kernel::Loaded *l, void *const *devicePtrs, hipStream_t stream,
             char *scratchBase = nullptr) {
  WorkspaceTurn turn(k, l, stream, scratchBase == nullptr);
  int rc = turn.begin();
  if (rc == AKG_HIP_OK) rc = launchSequence(k, *l, devicePtrs, stream, scratchBase);
  return turn.end(rc);
}

int launchSequence(akg_hip_kernel *k, akg_hip_kernel::Loaded &l, void *const *devicePtrs, hipStream_t stream,
                   char *scratchBase) {
  void *const workspace = scratchBase != nullptr ? (k->lowered.workspaceBytes > 0 ? scratchBase : nullptr) : l.workspace;
  if (!k->stages.empty()) {
    const size_t nin = k->graph.inputs.size();
    char *stageScratch = scratchBase != nullptr ? scratchBase + alignScratch(k->lowered.workspaceBytes) : nullptr;
    for (auto &st : k->stages) {
      akg_hip_kernel::Loaded *ls = nullptr;
      int rc = AKG_HIP_OK;
      if (scratchBase != nullptr) {
        if (!findLoaded(st.kernel, l.device, &ls)) return fail(AKG_HIP_ERR_INTERNAL, "stage not loaded");
      } else {
        rc = ensureLoaded(st.kernel, &ls);
      }
      if (rc != AKG_HIP_OK) return rc;
      std::vector<void *> ptrs(st.args.size());
      for (size_t a = 0; a < st.args.size(); ++a) {
        const akg::StageArg &sa = st.args[a];
        if (sa.kind == akg::StageArg::Kind::Input) {
          ptrs[a] = devicePtrs[sa.index];
        } else if (sa.kind == akg::StageArg::Kind::Output) {
          ptrs[a] = devicePtrs[nin + static_cast<size_t>(sa.index)];
        } else {
          ptrs[a] = static_cast<char *>(workspace) + k->tempOffsets[static_cast<size_t>(sa.index)];
        }
      }
      rc = launchOn(st.kernel, ls, ptrs.data(), stream, stageScratch);
      if (rc != AKG_HIP_OK) return rc;
      if (stageScratch != nullptr) stageScratch += scratchBytesNeeded(st.kernel);
    }
    return AKG_HIP_OK;
  }
  // kernel arguments: the tensor pointers, then the 64-bit scalars of the lowering, then the workspace
  const int n = numTensors(k);
  const int nscalar = static_cast<int>(k->lowered.scalarArgs.size());
  const int nargs = n + nscalar + (workspace ? 1 : 0);
  std::vector<void *> slots(static_cast<size_t>(nargs));
  std::vector<void *> params(static_cast<size_t>(nargs));
  for (int i = 0; i < nargs; ++i) {
    if (i < n) {
      slots[static_cast<size_t>(i)] = devicePtrs[i];
      params[static_cast<size_t>(i)] = &slots[static_cast<size_t>(i)];
    } else if (i < n + nscalar) {
      params[static_cast<size_t>(i)] = const_cast<int64_t *>(&k->lowered.scalarArgs[static_cast<size_t>(i - n)]);
    } else {
      slots[static_cast<size_t>(i)] = workspace;
      params[static_cast<size_t>(i)] = &slots[static_cast<size_t>(i)];
    }
  }
  for (size_t i = 0; i < l.earlier.size(); ++i) {
    const akg::KernelPhase &ph = k->lowered.earlierPhases[i];
    hipError_t pe = hipModuleLaunchKernel(l.earlier[i], ph.grid[0], ph.grid[1], ph.grid[2], ph.block[0], ph.block[1],
                                          ph.block[2], 0, stream, params.data(), nullptr);
    if (pe != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipModuleLaunchKernel(" + ph.kernelName + "): " + hipErr(pe));
  }
  hipError_t e = hipModuleLaunchKernel(l.function, k->lowered.grid[0], k->lowered.grid[1], k->lowered.grid[2],
                                       k->lowered.block[0], k->lowered.block[1], k->lowered.block[2], 0, stream,
                                       params.data(), nullptr);
  if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipModuleLaunchKernel: " + hipErr(e));
  return AKG_HIP_OK;
}

int checkPtrs(const akg_hip_kernel *k, void *const *ptrs, int n) {
  if (k == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "kernel is NULL");
  if (ptrs == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "pointer array is NULL");
  if (n != numTensors(k)) {
    return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "kernel " + k->graph.name + " takes " + std::to_string(numTensors(k)) +
                                                " tensors, " + std::to_string(n) + " given");
  }
  for (int i = 0; i < n; ++i) {
    if (ptrs[i] == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "tensor pointer " + std::to_string(i) + " is NULL");
  }
  return AKG_HIP_OK;
}

}  // namespace

extern "C" {

int akg_hip_compile(const char *json_text, size_t json_len, const char *out_dir, akg_hip_kernel_t **out_kernel) {
  if (json_text == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "json_text is NULL");
  try {
    return doCompile(std::string(json_text, json_len), out_dir, out_kernel);
  } catch (const std::exception &e) {
    return fail(AKG_HIP_ERR_INTERNAL, std::string("internal error: ") + e.what());
  }
}

int akg_hip_compile_file(const char *info_path, const char *out_dir, akg_hip_kernel_t **out_kernel) {
  if (info_path == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "info_path is NULL");
  std::string path(info_path);
  if (path.find("..") != std::string::npos) {
    return fail(AKG_HIP_ERR_IO, "path " + path + " must not contain '..'");
  }
  std::string text;
  if (!readFile(path, &text)) return fail(AKG_HIP_ERR_IO, "cannot read " + path);
  try {
    return doCompile(text, out_dir, out_kernel);
  } catch (const std::exception &e) {
    return fail(AKG_HIP_ERR_INTERNAL, std::string("internal error: ") + e.what());
  }
}

int akg_hip_kernel_num_tensors(const akg_hip_kernel_t *kernel, int *n_tensors) {
  if (kernel == nullptr || n_tensors == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  *n_tensors = numTensors(kernel);
  return AKG_HIP_OK;
}

int akg_hip_kernel_tensor(const akg_hip_kernel_t *kernel, int index, akg_hip_tensor_desc *desc) {
  if (kernel == nullptr || desc == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  if (index < 0 || index >= numTensors(kernel)) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "tensor index out of range");
  const akg::TensorValue &t = tensorAt(kernel, index);
  std::memset(desc, 0, sizeof(*desc));
  desc->dtype = static_cast<int32_t>(t.dtype);
  if (t.shape.size() > AKG_HIP_MAX_RANK) return fail(AKG_HIP_ERR_UNSUPPORTED, "tensor rank exceeds AKG_HIP_MAX_RANK");
  desc->rank = static_cast<int32_t>(t.shape.size());
  for (size_t i = 0; i < t.shape.size(); ++i) desc->shape[i] = t.shape[i];
  desc->bytes = t.numel() * static_cast<int64_t>(akg::dtypeSize(t.dtype));
  desc->is_output = static_cast<size_t>(index) >= kernel->graph.inputs.size() ? 1 : 0;
  std::snprintf(desc->name, sizeof(desc->name), "%s", t.name.c_str());
  return AKG_HIP_OK;
}

int akg_hip_kernel_get_info(const akg_hip_kernel_t *kernel, akg_hip_kernel_info *info) {
  if (kernel == nullptr || info == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  std::memset(info, 0, sizeof(*info));
  std::snprintf(info->kernel_name, sizeof(info->kernel_name), "%s", kernel->lowered.kernelName.c_str());
  std::snprintf(info->family, sizeof(info->family), "%s", akg::kernelFamilyName(kernel->lowered.family));
  std::snprintf(info->operator_type, sizeof(info->operator_type), "%s",
                akg::operatorTemplateName(kernel->graph.operatorTemplate));
  for (int i = 0; i < 3; ++i) {
    info->grid[i] = kernel->lowered.grid[i];
    info->block[i] = kernel->lowered.block[i];
  }
  info->algorithmic_bytes = kernel->lowered.algorithmicBytes;
  info->algorithmic_ops = kernel->lowered.algorithmicOps;
  info->cache_hit = kernel->cacheHit ? 1 : 0;
  info->workspace_bytes = kernel->lowered.workspaceBytes;
  info->build_ms = kernel->buildMs;
  return AKG_HIP_OK;
}

int akg_hip_kernel_source(const akg_hip_kernel_t *kernel, const char **source) {
  if (kernel == nullptr || source == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  *source = kernel->lowered.source.c_str();
  return AKG_HIP_OK;
}

int akg_hip_launch(akg_hip_kernel_t *kernel, void *const *device_ptrs, int n_ptrs, void *stream) {
  int rc = checkPtrs(kernel, device_ptrs, n_ptrs);
  if (rc != AKG_HIP_OK) return rc;
  akg_hip_kernel::Loaded *fn = nullptr;
  rc = ensureLoaded(kernel, &fn);
  if (rc != AKG_HIP_OK) return rc;
  return launchOn(kernel, fn, device_ptrs, static_cast<hipStream_t>(stream));
}

int akg_hip_launch_static_scratch(akg_hip_kernel_t *kernel, void *const *device_ptrs, int n_ptrs, void *stream) {
  int rc = checkPtrs(kernel, device_ptrs, n_ptrs);
  if (rc != AKG_HIP_OK) return rc;
  const uint64_t need = scratchBytesNeeded(kernel);
  if (need > AKG_HIP_STATIC_SCRATCH_BYTES) {
    return fail(AKG_HIP_ERR_UNSUPPORTED, "kernel " + kernel->graph.name + " needs " + std::to_string(need) +
                                           " bytes of scratch, the static array holds " +
                                           std::to_string(AKG_HIP_STATIC_SCRATCH_BYTES) + ": use akg_hip_launch");
  }
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipGetDevice: " + hipErr(e));
  akg_hip_kernel::Loaded *fn = nullptr;
  if (!findLoaded(kernel, device, &fn)) {
    return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "kernel " + kernel->graph.name + " is not loaded on device " +
                                                std::to_string(device) +
                                                ": call akg_hip_kernel_prepare once before the launches that must not allocate");
  }
  char *base = nullptr;
  if (need > 0) {
    void *p = nullptr;
    e = akg::staticScratchOnCurrentDevice(&p);
    if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "address of the static scratch array: " + hipErr(e));
    base = static_cast<char *>(p);
    // The array keeps whatever the last launch on this device left (another handle's partial results, or counters of
    // a launch that failed half way), and the kernels expect their arrival counters at zero: clear the part used.
    e = akg::staticScratchClear(base, need, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "clearing the static scratch array: " + hipErr(e));
  } else {
    // no kernel of this handle uses scratch; a non-NULL base only tells launchOn to load and allocate nothing
    static char unused;
    base = &unused;
  }
  return launchOn(kernel, fn, device_ptrs, static_cast<hipStream_t>(stream), base);
}

static_assert(AKG_HIP_STATIC_SCRATCH_MAX == AKG_HIP_STATIC_SCRATCH_BYTES,
              "the limit the header states and the size of the array are one number");

int akg_hip_kernel_prepare(akg_hip_kernel_t *kernel) {
  if (kernel == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "kernel is NULL");
  akg_hip_kernel::Loaded *l = nullptr;
  const int rc = ensureLoaded(kernel, &l);
  if (rc != AKG_HIP_OK) return rc;
  // A handle that akg_hip_launch_static_scratch can serve: look the array's address up now. The first look-up on a
  // device makes the runtime load the library's own code object there and materialise the array, which a launch that
  // must not allocate (or that is being captured into a graph) cannot afford; afterwards it is a table read.
  const uint64_t need = scratchBytesNeeded(kernel);
  if (need > 0 && need <= AKG_HIP_STATIC_SCRATCH_BYTES) {
    void *p = nullptr;
    const hipError_t e = akg::staticScratchOnCurrentDevice(&p);
    if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "address of the static scratch array: " + hipErr(e));
  }
  return AKG_HIP_OK;
}

int akg_hip_run_host(akg_hip_kernel_t *kernel, void *const *host_ptrs, int n_ptrs) {
  int rc = checkPtrs(kernel, host_ptrs, n_ptrs);
  if (rc != AKG_HIP_OK) return rc;
  akg_hip_kernel::Loaded *fn = nullptr;
  rc = ensureLoaded(kernel, &fn);
  if (rc != AKG_HIP_OK) return rc;
  const int n = numTensors(kernel);
  std::vector<void *> dev(static_cast<size_t>(n), nullptr);
  auto release = [&]() {
    for (void *p : dev) {
      if (p) (void)hipFree(p);
    }
  };
  for (int i = 0; i < n; ++i) {
    const akg::TensorValue &t = tensorAt(kernel, i);
    size_t bytes = static_cast<size_t>(t.numel()) * akg::dtypeSize(t.dtype);
    hipError_t e = hipMalloc(&dev[static_cast<size_t>(i)], bytes ? bytes : 1);
    if (e != hipSuccess) {
      release();
      return fail(AKG_HIP_ERR_RUNTIME, "hipMalloc(" + std::to_string(bytes) + "): " + hipErr(e));
    }
    // Every tensor is copied in, outputs included: callers pre-fill outputs (with NaN in the reference
    // harness) so that elements a kernel fails to write are detected.
    e = hipMemcpy(dev[static_cast<size_t>(i)], host_ptrs[i], bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      release();
      return fail(AKG_HIP_ERR_RUNTIME, "hipMemcpy H2D: " + hipErr(e));
    }
  }
  rc = launchOn(kernel, fn, dev.data(), nullptr);
  if (rc == AKG_HIP_OK) {
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) rc = fail(AKG_HIP_ERR_RUNTIME, "kernel execution: " + hipErr(e));
  }
  if (rc == AKG_HIP_OK) {
    const size_t nin = kernel->graph.inputs.size();
    for (int i = static_cast<int>(nin); i < n; ++i) {
      const akg::TensorValue &t = tensorAt(kernel, i);
      size_t bytes = static_cast<size_t>(t.numel()) * akg::dtypeSize(t.dtype);
      hipError_t e = hipMemcpy(host_ptrs[i], dev[static_cast<size_t>(i)], bytes, hipMemcpyDeviceToHost);
      if (e != hipSuccess) {
        rc = fail(AKG_HIP_ERR_RUNTIME, "hipMemcpy D2H: " + hipErr(e));
        break;
      }
    }
  }
  release();
  return rc;
}

int akg_hip_profile(akg_hip_kernel_t *kernel, void *const *device_ptrs, int n_ptrs, int number, int repeat,
                    double *avg_ms) {
  int rc = checkPtrs(kernel, device_ptrs, n_ptrs);
  if (rc != AKG_HIP_OK) return rc;
  if (avg_ms == nullptr || number <= 0 || repeat <= 0) {
    return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "number and repeat must be positive and avg_ms non-NULL");
  }
  akg_hip_kernel::Loaded *fn = nullptr;
  rc = ensureLoaded(kernel, &fn);
  if (rc != AKG_HIP_OK) return rc;
  hipStream_t stream = nullptr;
  hipEvent_t start = nullptr, stop = nullptr;
  hipError_t e = hipStreamCreate(&stream);
  if (e != hipSuccess) return fail(AKG_HIP_ERR_RUNTIME, "hipStreamCreate: " + hipErr(e));
  (void)hipEventCreate(&start);
  (void)hipEventCreate(&stop);
  auto cleanup = [&]() {
    if (start) (void)hipEventDestroy(start);
    if (stop) (void)hipEventDestroy(stop);
    (void)hipStreamDestroy(stream);
  };
  // one untimed launch first, as the reference shim does
  rc = launchOn(kernel, fn, device_ptrs, stream);
  if (rc == AKG_HIP_OK && (e = hipStreamSynchronize(stream)) != hipSuccess) {
    rc = fail(AKG_HIP_ERR_RUNTIME, "warm-up launch: " + hipErr(e));
  }
  double totalMs = 0.0;
  for (int r = 0; r < repeat && rc == AKG_HIP_OK; ++r) {
    (void)hipEventRecord(start, stream);
    for (int i = 0; i < number && rc == AKG_HIP_OK; ++i) rc = launchOn(kernel, fn, device_ptrs, stream);
    (void)hipEventRecord(stop, stream);
    e = hipEventSynchronize(stop);
    if (rc == AKG_HIP_OK && e != hipSuccess) rc = fail(AKG_HIP_ERR_RUNTIME, "timed launches: " + hipErr(e));
    float ms = 0.0f;
    if (rc == AKG_HIP_OK) {
      (void)hipEventElapsedTime(&ms, start, stop);
      totalMs += static_cast<double>(ms) / number;
    }
  }
  cleanup();
  if (rc == AKG_HIP_OK) *avg_ms = totalMs / repeat;
  return rc;
}

void akg_hip_kernel_destroy(akg_hip_kernel_t *kernel) { destroyKernel(kernel); }

const char *akg_hip_last_error(void) { return g_lastError.c_str(); }

int akg_hip_translate(const char *json_text, size_t json_len, char **out_text) {
  if (json_text == nullptr || out_text == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  *out_text = nullptr;
  try {
    akg::OpGraph g = akg::translateJsonToOpGraph(std::string(json_text, json_len));
    std::string text = akg::printOpGraph(g);
    char *buf = static_cast<char *>(std::malloc(text.size() + 1));
    if (buf == nullptr) return fail(AKG_HIP_ERR_INTERNAL, "out of memory");
    std::memcpy(buf, text.c_str(), text.size() + 1);
    *out_text = buf;
    return AKG_HIP_OK;
  } catch (const akg::json::ParseError &e) {
    return fail(AKG_HIP_ERR_JSON, e.what());
  } catch (const akg::TranslateError &e) {
    return fail(AKG_HIP_ERR_TRANSLATE, e.what());
  } catch (const std::exception &e) {
    return fail(AKG_HIP_ERR_INTERNAL, e.what());
  }
}

void akg_hip_free_string(char *text) { std::free(text); }

int akg_hip_dynamic_create(const char *json_text, size_t json_len, const char *out_dir, akg_hip_dynamic_t **out) {
  if (json_text == nullptr || out == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  *out = nullptr;
  try {
    std::unique_ptr<akg_hip_dynamic> d(new akg_hip_dynamic());
    d->jsonText.assign(json_text, json_len);
    if (out_dir != nullptr) {
      d->outDir = out_dir;
      d->hasOutDir = true;
    }
    const akg::json::Value root = akg::json::Value::parse(d->jsonText);
    if (!root.isObject() || !root.contains("input_desc") || !root.contains("op_desc") || !root.contains("output_desc")) {
      return fail(AKG_HIP_ERR_TRANSLATE, "not an op description");
    }
    d->numInputs = static_cast<int>(root.at("input_desc").size());
    for (size_t i = 0; i < root.at("input_desc").size(); ++i) {
      const akg::json::Value &desc = root.at("input_desc")[i][0];
      d->inputRanks.push_back(desc.contains("shape") ? static_cast<int>(desc.at("shape").size()) : 1);
    }
    for (size_t i = 0; i < root.at("output_desc").size(); ++i) {
      const akg::json::Value &desc = root.at("output_desc")[i];
      d->outputRanks.push_back(desc.contains("shape") ? static_cast<int>(desc.at("shape").size()) : 1);
    }
    *out = d.release();
    g_lastError.clear();
    return AKG_HIP_OK;
  } catch (const akg::json::ParseError &e) {
    return fail(AKG_HIP_ERR_JSON, e.what());
  } catch (const std::exception &e) {
    return fail(AKG_HIP_ERR_TRANSLATE, e.what());
  }
}

int akg_hip_dynamic_num_inputs(const akg_hip_dynamic_t *dyn, int *n_inputs) {
  if (dyn == nullptr || n_inputs == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  *n_inputs = dyn->numInputs;
  return AKG_HIP_OK;
}

int akg_hip_dynamic_specialize(akg_hip_dynamic_t *dyn, const int64_t *const *input_shapes, const int32_t *input_ranks,
                               int n_inputs, akg_hip_kernel_t **out_kernel) {
  if (dyn == nullptr || input_shapes == nullptr || input_ranks == nullptr || out_kernel == nullptr) {
    return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  }
  *out_kernel = nullptr;
  if (n_inputs != dyn->numInputs) {
    return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "the description has " + std::to_string(dyn->numInputs) + " inputs, " +
                                                std::to_string(n_inputs) + " shapes given");
  }
  akg::ShapeBinding binding;
  std::string key;
  for (int i = 0; i < n_inputs; ++i) {
    if (input_ranks[i] < 0 || input_ranks[i] > AKG_HIP_MAX_RANK || input_shapes[i] == nullptr) {
      return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "bad rank or NULL shape for input " + std::to_string(i));
    }
    std::vector<int64_t> shape(input_shapes[i], input_shapes[i] + input_ranks[i]);
    for (int64_t d : shape) key += std::to_string(d) + ",";
    key += ";";
    binding.inputShapes.push_back(std::move(shape));
  }
  std::lock_guard<std::mutex> lock(dyn->mu);
  auto it = dyn->specializations.find(key);
  if (it != dyn->specializations.end()) {
    *out_kernel = it->second;
    return AKG_HIP_OK;
  }
  akg_hip_kernel_t *k = nullptr;
  int rc;
  try {
    rc = doCompile(dyn->jsonText, dyn->hasOutDir ? dyn->outDir.c_str() : nullptr, &k, &binding);
  } catch (const std::exception &e) {
    return fail(AKG_HIP_ERR_INTERNAL, std::string("internal error: ") + e.what());
  }
  if (rc != AKG_HIP_OK) return rc;
  dyn->specializations[key] = k;
  *out_kernel = k;
  return AKG_HIP_OK;
}

int akg_hip_dynamic_launch_packed(akg_hip_dynamic_t *dyn, void *const *tensor_ptrs, const int64_t *const *shape_lists,
                                  int n_tensors, void *stream, akg_hip_kernel_t **used_kernel) {
  if (dyn == nullptr || tensor_ptrs == nullptr || shape_lists == nullptr) {
    return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "NULL argument");
  }
  const int nin = dyn->numInputs, nout = static_cast<int>(dyn->outputRanks.size());
  if (n_tensors != nin + nout) {
    return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "the description has " + std::to_string(nin) + " inputs and " +
                                                std::to_string(nout) + " outputs, " + std::to_string(n_tensors) + " tensors given");
  }
  // per tensor: [offset, sizes..., strides...] (the integer fields of its memref descriptor)
  auto readDense = [&](int i, int rank, std::vector<int64_t> *shape) -> int {
    const int64_t *list = shape_lists[i];
    if (list == nullptr) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "shape list " + std::to_string(i) + " is NULL");
    if (list[0] != 0) return fail(AKG_HIP_ERR_UNSUPPORTED, "tensor " + std::to_string(i) + ": a non-zero offset is not supported");
    shape->assign(list + 1, list + 1 + rank);
    int64_t expect = 1;
    for (int d = rank; d-- > 0;) {
      const int64_t extent = (*shape)[static_cast<size_t>(d)];
      if (extent < 0) return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "tensor " + std::to_string(i) + ": negative extent");
      if (extent != 1 && list[1 + rank + d] != expect) {
        return fail(AKG_HIP_ERR_UNSUPPORTED, "tensor " + std::to_string(i) + ": only dense row-major tensors are supported");
      }
      expect *= extent;
    }
    return AKG_HIP_OK;
  };
  std::vector<std::vector<int64_t>> inShapes(static_cast<size_t>(nin));
  std::vector<const int64_t *> shapePtrs(static_cast<size_t>(nin));
  for (int i = 0; i < nin; ++i) {
    const int rc = readDense(i, dyn->inputRanks[static_cast<size_t>(i)], &inShapes[static_cast<size_t>(i)]);
    if (rc != AKG_HIP_OK) return rc;
    shapePtrs[static_cast<size_t>(i)] = inShapes[static_cast<size_t>(i)].data();
  }
  std::vector<int32_t> ranks(dyn->inputRanks.begin(), dyn->inputRanks.end());
  akg_hip_kernel_t *kernel = nullptr;
  int rc = akg_hip_dynamic_specialize(dyn, shapePtrs.data(), ranks.data(), nin, &kernel);
  if (rc != AKG_HIP_OK) return rc;
  for (int j = 0; j < nout; ++j) {
    std::vector<int64_t> given;
    rc = readDense(nin + j, dyn->outputRanks[static_cast<size_t>(j)], &given);
    if (rc != AKG_HIP_OK) return rc;
    const akg::TensorValue &t = tensorAt(kernel, nin + j);
    int64_t n = 1;
    for (int64_t e : given) n *= e;
    if (n != t.numel()) {
      return fail(AKG_HIP_ERR_INVALID_ARGUMENT, "output " + std::to_string(j) + ": the shape given does not follow from the input shapes");
    }
  }
  if (used_kernel != nullptr) *used_kernel = kernel;
  return akg_hip_launch(kernel, tensor_ptrs, n_tensors, stream);
}

void akg_hip_dynamic_destroy(akg_hip_dynamic_t *dyn) {
  if (dyn == nullptr) return;
  for (auto &kv : dyn->specializations) akg_hip_kernel_destroy(kv.second);
  delete dyn;
}

const char *akg_hip_version(void) { return AKG_HIP_VERSION_STRING; }

}  // extern "C"
