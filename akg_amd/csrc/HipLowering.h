/**
 * GPU lowering of an op graph for gfx950: picks a kernel family and a launch shape, and emits the HIP source
 * of one kernel `<op>_kernel(inputs..., outputs...)`.
 *
 * Replaces the reference's generic GPU pipeline (akg-mlir/lib/Pipelines/GPUPipelines/GPUOpt.cpp:45-132:
 * bufferize -> affine/scf loops -> AKGGPUMapping -> gpu.launch outlining -> NVVM). There a polyhedral
 * scheduler maps one scalar element per thread per step; here each fusion class of the reference's own
 * lattice (OperatorIdentify.cpp:51-93) has a hand-written skeleton for CDNA4 and the lowering only fills in
 * the per-element chain:
 *   Elementwise / Broadcast / Reshape  -> streaming kernel, 128-bit accesses, whole chain in registers
 *   Reduction (direction X)            -> one row per thread group, row resident in registers across all
 *                                         reductions of the fusion, wave64 butterfly + LDS reductions
 *   Matmul (+ elementwise epilogue)    -> int8 MFMA tile kernel, epilogue applied to the int32 accumulators
 * The kernel signature contract is the reference's: bare pointers, inputs then outputs
 * (KernelOutliningExt.cpp:175-213, GPUCodegen.cpp:49-51).
 */
#ifndef AKG_HIP_HIPLOWERING_H_
#define AKG_HIP_HIPLOWERING_H_

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "OpGraph.h"

namespace akg {

class LoweringError : public std::runtime_error {
 public:
  explicit LoweringError(const std::string &msg) : std::runtime_error(msg) {}
};

enum class KernelFamily { Elementwise, RowReduce, GemmEpilogue, StreamReduce, Indexed, SegmentSum, Staged, ColumnReduce };
const char *kernelFamilyName(KernelFamily f);

// Tuning knobs; 0 means "let the heuristic decide". They can be set through the environment
// (AKG_HIP_VEC, AKG_HIP_TPR, AKG_HIP_CHUNKS, AKG_HIP_BLOCK, AKG_HIP_SPLIT) for sweeps.
struct LoweringOptions {
  int vec = 0;          // elements per chunk
  int threadsPerRow = 0;
  int chunks = 0;       // chunks per thread
  int block = 0;        // threads per workgroup
  int split = 0;        // streaming reductions: workgroups sharing one group of outputs (AKG_HIP_SPLIT)
  // Experiment switch (AKG_HIP_VARIANT), read by whichever family lowers the kernel; 0 = the measured default.
  //   gemm_epilogue  bit 3: no skinny kernel for M <= 64 (the tile kernel with K split instead),
  //                  bit 5: the other arrangement of the tile kernel's wavefronts (2 x 4 for 4 x 2 and back)
  //   row_reduce     1: keep the row in registers, 2: walk the row (no packing), 4: walk it, packed if possible
  //   stream_reduce  7: no column kernel (several kernels instead)
  //   column_reduce  5: one strip per workgroup (no second set of resident registers)
  //   segment_sum    1: every workgroup scans all ids, 2: positions grouped by segment first (whatever the size),
  //                  3: grouped by bucket of segments first (whatever the number of buckets)
  //   indexed        1: no LDS-tiled transposes, 2: no chunk-wide loads
  int variant = 0;
  int nonTemporal = 1;  // stream once-touched tensors with non-temporal accesses (AKG_HIP_NT=0 turns it off)
  // Compute units of the part the kernels are made for (MI355X / MI350X: 256; AKG_HIP_CUS for another gfx950 part):
  // what persistent grids are sized by. The lowering runs without a device, so this is not asked of one.
  int computeUnits = 256;
  // A MatMul whose declared result is float16 / bfloat16 accumulates in that type in the reference (product and sum
  // rounded at every k), which only the serial kernel on the vector ALUs reproduces. AKG_HIP_MATMUL_F32_ACC=1 is the
  // caller's explicit consent to the matrix units instead: float32 accumulation, ONE rounding to the declared type - more
  // accurate than the reference's value and different from it (outside rtol 1e-2 from K = 64 on for N(0,1) data).
  bool matmulF32Acc = false;
  // Dynamic-shape descriptions: the elementwise / row-reduction kernels take their row count (or, when everything
  // folds into one dimension, their element count) as a kernel argument instead of a constant, so that shape sets
  // that differ only there share one code object (the source no longer depends on them). Likewise the rows of A of
  // a MatMul, the outermost reduced extent of a streaming reduction and the batch of the column kernel.
  bool extentAsArgument = false;
  static LoweringOptions fromEnvironment();
};

// A launch that precedes the kernel proper (same arguments, same stream, in order).
struct KernelPhase {
  std::string kernelName;
  unsigned grid[3] = {1, 1, 1};
  unsigned block[3] = {1, 1, 1};
};

struct LoweredKernel {
  std::string kernelName;  // "<op>_kernel", as the reference names its outlined gpu.func
  // Kernels of the same code object that run before `kernelName`, in this order (empty for all families but the
  // grouped segment sum). Grid, block and name of the kernel proper stay in the fields below.
  std::vector<KernelPhase> earlierPhases;
  std::string source;      // HIP translation unit
  KernelFamily family = KernelFamily::Elementwise;
  unsigned grid[3] = {1, 1, 1};
  unsigned block[3] = {1, 1, 1};
  uint64_t algorithmicBytes = 0;  // bytes of all kernel inputs and outputs, each counted once
  uint64_t algorithmicOps = 0;    // 2*M*N*K for a contraction, 0 otherwise
  std::string scheduleNote;       // human-readable schedule summary (vec, threads per row, ...)
  // per kernel argument: [offset, sizes..., strides...] as in `<k>_shape_arg.txt`
  std::vector<std::vector<int64_t>> shapeArgs;
  // 64-bit scalar kernel arguments that follow the tensor pointers (before the workspace pointer, if any)
  std::vector<int64_t> scalarArgs;
  // Device workspace the kernel takes as one extra trailing pointer argument (0: none). The runtime allocates it
  // per kernel handle and device and zero-fills it once; the kernel leaves it zeroed where it must be.
  uint64_t workspaceBytes = 0;
};

LoweredKernel lowerToHip(const OpGraph &graph, const LoweringOptions &options);

// Family-specific entries used by lowerToHip (HipLoweringGemm.cpp, HipLoweringReduce.cpp, HipLoweringIndexed.cpp).
LoweredKernel lowerGemmToHip(const OpGraph &graph, const LoweringOptions &options);
LoweredKernel lowerStreamReduceToHip(const OpGraph &graph, const LoweringOptions &options);
// One reduced axis that is not the innermost one, reduction results used against the unreduced tensor (HipLoweringColumn.cpp).
LoweredKernel lowerColumnToHip(const OpGraph &graph, const LoweringOptions &options);
LoweredKernel lowerTileToHip(const OpGraph &graph, const LoweringOptions &options);      // elementwise, row_reduce
LoweredKernel lowerIndexedToHip(const OpGraph &graph, const LoweringOptions &options);
LoweredKernel lowerSegmentSumToHip(const OpGraph &graph, const LoweringOptions &options);
// True when the graph contains a data-movement op (Transpose, Tile, Slice, StridedSlice, Pad, Concat).
bool wantsIndexedKernel(const OpGraph &graph);
// True when the reductions of `graph` belong to the streaming family: some reduced axis is not the innermost one
// (direction Y / ALL), or the rows are too long or too few for the register-resident row kernel.
bool wantsStreamReduce(const OpGraph &graph);

// Shared helpers for the emitters.
namespace lowering {
const char *dtypeTag(DType t);          // "akg::f32", ...
const char *computeTypeName(DType t);   // "float", "int", ...
std::string literalFor(DType t, double value);  // constant of the compute type, already rounded to t
uint64_t countAlgorithmicBytes(const OpGraph &g);
std::vector<std::vector<int64_t>> buildShapeArgs(const OpGraph &g);
// Expression of one elementwise op in terms of operand expressions (already in their compute types).
// `relaxed` selects hardware-approximate transcendental / reciprocal sequences (see precisionDemand).
std::string elementwiseExpr(const OpGraph &g, const OpNode &op, const std::vector<std::string> &operands,
                            bool relaxed = false);
// Backward precision-demand analysis. Returns, per tensor, true when every path from it to a kernel output
// passes through a Cast to float16 / bfloat16 before anything that needs exact values (integer casts,
// comparisons, Floor, float32 / float64 / integer outputs). Such values only need about 3 decimal digits, so
// the lowering may compute them with ~1 ulp float32 hardware approximations (AKG_HIP_PRECISE=1 disables this).
std::vector<bool> relaxedPrecisionTensors(const OpGraph &g);
bool isElementwiseKind(OpKind k);
bool isReduceKind(OpKind k);
// Combiner functor, initial value and rounding rule of a reduction whose result type is `od`
// (createInitValueForReduce / createCombinerForReduce, MindSporeToLinalg.cpp:791-901).
struct ReduceSpec {
  std::string combiner;        // "akg::RedSum", ...
  std::string init;            // literal of the compute type
  bool roundEachStep = false;  // narrow result types accumulate in that type: round after every step
  // A float16 / bfloat16 sum or product: rounding after every step makes the order of the steps part of the result, and
  // the reference's is one serial loop per result element in index order. (Integer sums and products wrap around and
  // are the same in any order; a maximum is one of its operands.)
  bool ordered = false;
};
ReduceSpec reduceSpec(const OpNode &op, DType od);
}  // namespace lowering

}  // namespace akg

#endif  // AKG_HIP_HIPLOWERING_H_
