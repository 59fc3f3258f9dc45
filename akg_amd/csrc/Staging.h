/**
 * Descriptions that no single kernel serves because a reduced value meets an unreduced one where the kernel families
 * cannot bring them together (a softmax or a normalisation over an outer axis, statistics and their use in one
 * description) are run as a sequence of kernels instead. The reference leaves such cuts to MindSpore's graph-kernel
 * splitter, which hands AKG one description per piece (the "_split_" descriptions of its test tree, e.g.
 * Fused_Sub_Exp_ReduceSum_split + Fused_RealDiv_split for a softmax); here a description that arrives uncut is cut the
 * same way: at the results of its reductions.
 *
 * Every tensor gets a level: inputs 0, an elementwise result the greatest level of its operands, a reduction's result
 * one more than its operand; so does the result of a data-movement op (Transpose, Slice, Pad, Concat, Tile, Gather,
 * Reshape), which no kernel that reduces takes in: it gets a kernel of its own (with the elementwise ops in front of
 * it) and the reduction reads its result from memory. A MatMul that a reduction depends on (attention scores and their
 * softmax) is cut the same way: the contraction leaves its result in memory, the ops behind it run in the next kernel;
 * operands of a contraction that are computed in the description are cut too (the GEMM kernel reads memory). The kernels of level s compute the reductions whose operands have level s (from the
 * description's inputs and the reduction results of earlier levels, recomputing the elementwise ops in between) and
 * the description's outputs of level s. Reduction results that are not outputs of the description live in a temporary
 * buffer the handle owns. Each kernel is an ordinary description made of the original's op entries and goes through
 * the ordinary pipeline.
 */
#ifndef AKG_HIP_STAGING_H_
#define AKG_HIP_STAGING_H_

#include <cstdint>
#include <string>
#include <vector>

#include "OpGraph.h"

namespace akg {

struct StageArg {
  enum class Kind { Input, Output, Temp };
  Kind kind = Kind::Input;
  int index = 0;  // position among the description's inputs / outputs, or temporary number
};

struct StagePlan {
  std::string jsonText;        // the stage as a description of its own, named "<op>_stage<k>"
  std::vector<StageArg> args;  // where each tensor of its signature lives (its inputs, then its outputs)
  std::vector<std::vector<int64_t>> shapes;  // shape of each of them in the translated graph
  size_t numOutputs = 0;
};

struct StagingPlan {
  std::vector<StagePlan> stages;     // in launch order
  std::vector<uint64_t> tempBytes;   // size of every temporary
};

// False (with the reason in *why) when the description cannot be cut: fewer than two kernels would result, its op
// entries do not match the translated graph one to one, or it holds an Assign whose write could
// not be ordered behind every other kernel's reads of the input it overwrites.
// `reductionsToo` false: cut only behind contractions and data-movement ops (what is left between two cuts may still be
// one kernel: a softmax behind a MatMul); true: at reduction results as well.
bool planStages(const std::string &jsonText, const OpGraph &g, bool reductionsToo, StagingPlan *plan, std::string *why);

// ArgMax over an axis that is not the innermost one. The row family finds the position of the greatest element along
// the innermost axis only, so such an op is respelled in the description itself: Transpose (the reduced axis moved to
// the back), ArgMax over the last axis, and a Reshape where keep_dims put a 1 in the middle of the result shape. The
// respelled description then runs as two kernels (the transpose gets one of its own). Returns true and the new text
// when something was respelled; descriptions with open (-1) extents are left alone.
bool moveArgMaxToInnermostAxis(const std::string &jsonText, std::string *rewritten);

}  // namespace akg

#endif  // AKG_HIP_STAGING_H_
