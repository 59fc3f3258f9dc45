/**
 * akg_hip.h - C ABI of the MI355X (gfx950) backend for AKG-MLIR fused operators.
 *
 * Drop-in boundary: a MindSpore graph-kernel JSON op description goes in, a callable kernel with the same
 * tensor signature (inputs in `input_desc` order, then outputs in `output_desc` order) comes out.
 * Plain C types only; every function returns 0 on success or a negative akg_hip_status code and never
 * terminates the process (the reference's tools exit non-zero and its launch shim calls exit(1),
 * akg-mlir/python/akg_mlir/utils/code_template.py:47-56).
 *
 * Each entry point names the reference interface it replaces.
 */
#ifndef AKG_HIP_H_
#define AKG_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum akg_hip_status {
  AKG_HIP_OK = 0,
  AKG_HIP_ERR_INVALID_ARGUMENT = -1,
  AKG_HIP_ERR_JSON = -2,          /* malformed JSON text */
  AKG_HIP_ERR_TRANSLATE = -3,     /* well-formed JSON that is not a valid op description (also: a tensor with an extent
                                     of 0 or more than 2^40 elements, an op with the wrong number of operands) */
  AKG_HIP_ERR_UNSUPPORTED = -4,   /* valid description with no gfx950 kernel family (or an unknown op) */
  AKG_HIP_ERR_COMPILE = -5,       /* device compilation failed */
  AKG_HIP_ERR_IO = -6,            /* artifact directory / file access */
  AKG_HIP_ERR_RUNTIME = -7,       /* HIP runtime error (no device, launch failure, out of memory) */
  AKG_HIP_ERR_INTERNAL = -8
} akg_hip_status;

/* Element types of the op-description format (TranslateToMindsporeDialect.cpp:488-502). */
typedef enum akg_hip_dtype {
  AKG_HIP_BOOL = 0,
  AKG_HIP_INT8 = 1,
  AKG_HIP_INT16 = 2,
  AKG_HIP_INT32 = 3,
  AKG_HIP_INT64 = 4,
  AKG_HIP_FLOAT16 = 5,
  AKG_HIP_BFLOAT16 = 6,
  AKG_HIP_FLOAT32 = 7,
  AKG_HIP_FLOAT64 = 8
} akg_hip_dtype;

#define AKG_HIP_MAX_RANK 8

typedef struct akg_hip_tensor_desc {
  int32_t dtype;                      /* akg_hip_dtype */
  int32_t rank;
  int64_t shape[AKG_HIP_MAX_RANK];
  int64_t bytes;                      /* dense row-major size */
  int32_t is_output;                  /* 0: kernel input, 1: kernel output */
  char name[64];                      /* tensor_name of the description */
} akg_hip_tensor_desc;

typedef struct akg_hip_kernel_info {
  char kernel_name[256];              /* "<op>_kernel" (KernelOutliningExt.cpp:433) */
  char family[32];                    /* "elementwise" | "row_reduce" | "stream_reduce" | "gemm_epilogue" | "indexed" | "segment_sum" |
                                         "staged" (a sequence of kernels of the other families; kernel_name, grid and
                                         block are those of the last one) */
  char operator_type[32];             /* fusion class, OperatorIdentify.cpp:51-93 */
  uint32_t grid[3];                   /* blockIdx.x/y/z extents, as written to <k>.json (of the kernel proper when
                                         earlier launches precede it: segment sums over many positions) */
  uint32_t block[3];                  /* threadIdx.x/y/z extents */
  uint64_t algorithmic_bytes;         /* bytes of every input and output, each counted once (an input that is only
                                         sliced or gathered from: the bytes taken out of it) */
  uint64_t algorithmic_ops;           /* 2*M*N*K of the contraction, 0 for bandwidth-bound families */
  int32_t cache_hit;                  /* 1 if no device compilation was needed: the code object came from the
                                         artifact directory or from this process's memory (same source digest) */
  uint64_t workspace_bytes;           /* device scratch the handle owns per device (streaming reductions, GEMMs
                                         with K split over workgroups, grouped segment sums), else 0 */
  double build_ms;                    /* wall time it took to make this handle: translation, lowering and, unless
                                         cache_hit, device compilation (a new shape set of a dynamic description that
                                         shares a code object costs about a millisecond, a device compilation ~0.5 s) */
} akg_hip_kernel_info;

typedef struct akg_hip_kernel akg_hip_kernel_t;

/**
 * Compile one op description to a gfx950 code object and return a kernel handle. Needs no GPU.
 * Replaces the compile half of MlirDriver.compile_gpu (akg-mlir/python/akg_mlir/mlir_driver.py:337-374):
 * mindspore-translate -json-to-mindspore (TranslateToMindsporeDialect.cpp:1461) -> akg-opt --gpu-opt
 * (GPUOpt.cpp:45-132) -> akg-opt --gpu-codegen (GPUCodegen.cpp:34-55) -> akg-translate -gen-ptx
 * (TranslateToPTX.cpp:67-103).
 * If out_dir is non-NULL the reference's artifact set is written there: <op>.hsaco (in place of <op>.ptx),
 * <op>.json {blockIdx.*, threadIdx.*, kernelName, is_dynamic, sha256} (GPUMapping.cpp:645-665,
 * mlir_driver.py:776-815), <op>_shape_arg.txt (KernelOutliningExt.cpp:384-423), <op>_shape_info.json {hostShapes,
 * deviceShapes, runtimeVars, SupportInfo} (DumpShapeInfo.cpp:133-142), <op>.hip (the emitted
 * source, the counterpart of the <op>_gpu.mlir dump); a matching artifact found there is reused instead
 * of compiling (the reference's KERNEL_META_DIR cache, mlir_driver.py:47-53).
 */
int akg_hip_compile(const char *json_text, size_t json_len, const char *out_dir, akg_hip_kernel_t **out_kernel);

/** Same, reading the description from a file (the `-f x.info` of akg_benchmark, benchmark.py:249-328).
 *  Paths containing ".." are rejected as in checkAndReadJson (akg/Utils/IOHelper.hpp:44-61). */
int akg_hip_compile_file(const char *info_path, const char *out_dir, akg_hip_kernel_t **out_kernel);

/** Number of kernel arguments (inputs + outputs). Replaces reading `input_desc`/`output_desc` on the Python
 *  side (composite_op_helper.py:833-902). */
int akg_hip_kernel_num_tensors(const akg_hip_kernel_t *kernel, int *n_tensors);

/** Descriptor of argument `index` (inputs first, then outputs: BufferResultsToOutParams, GPUOpt.cpp:78). */
int akg_hip_kernel_tensor(const akg_hip_kernel_t *kernel, int index, akg_hip_tensor_desc *desc);

/** Launch shape, family, algorithmic work. Replaces get_gpu_setting_by_input (dynamic_utils.py:564-577). */
int akg_hip_kernel_get_info(const akg_hip_kernel_t *kernel, akg_hip_kernel_info *info);

/** Emitted HIP source of the kernel (NUL-terminated, owned by the handle); for a description that runs as several
 *  kernels, their sources one after the other. */
int akg_hip_kernel_source(const akg_hip_kernel_t *kernel, const char **source);

/**
 * Load the code object on the current device and allocate the handle's workspace there (workspace_bytes of
 * kernel_info: partial results of streaming reductions and split-K GEMMs, the sorted positions of large segment
 * sums, the tensors between the kernels of a staged description), so that later launches on this device
 * allocate nothing. Optional: the first akg_hip_launch on a device does the same. Replaces the cuModuleLoadData /
 * cuModuleGetFunction prologue of the generated shim (code_template.py:180-203).
 */
int akg_hip_kernel_prepare(akg_hip_kernel_t *kernel);

/**
 * The hot call: enqueue the kernel (or, for a description that needs several, its kernels in order) on `stream`
 * (a hipStream_t, NULL for the default stream) with one DEVICE
 * pointer per argument, inputs then outputs. Asynchronous; after the first call on a device (or
 * akg_hip_kernel_prepare) it allocates nothing. Launches of one handle whose workspace_bytes is non-zero share
 * that workspace: the library keeps them apart on the device (a launch that goes to another stream than the handle's
 * previous one first waits, through an event recorded on that previous stream at the switch, for what it holds - so a
 * stream must outlive the handle's next launch on another stream, or AKG_HIP_SAFE_STREAMS=1 must be set, which records
 * the event behind every launch instead and never touches a stream after its launch), and zero-fills the workspace again
 * in front of the next launch if a launch sequence broke off half way. Launches recorded into a stream capture are ordered by
 * the graph they become part of; two graphs replaying one handle at the same time are the caller's to keep apart.
 * Replaces the cuLaunchKernel
 * step of the generated shim (code_template.py:204) without its per-call context creation, module load,
 * cuMemAlloc and copies.
 */
int akg_hip_launch(akg_hip_kernel_t *kernel, void *const *device_ptrs, int n_ptrs, void *stream);

/**
 * akg_hip_launch for callers that cannot allocate device memory: code under HIP graph capture, serving loops with a
 * frozen memory plan, harnesses that forbid hipMalloc. It has no counterpart in the reference (whose shim allocates
 * and frees every tensor on every call, code_template.py:160-211). Same arguments and results as akg_hip_launch, but
 * the device memory that the kernels use beyond inputs and outputs (arrival counters and partial results of streaming
 * reductions and split-K GEMMs, grouped segment sums, the tensors between the kernels of a staged description) is a
 * fixed array of AKG_HIP_STATIC_SCRATCH_MAX bytes inside the library's own code object instead of the handle's
 * workspace, and the call allocates, loads and frees nothing:
 *  - akg_hip_kernel_prepare must have been called for this handle on the current device (it loads the code objects);
 *    otherwise AKG_HIP_ERR_INVALID_ARGUMENT;
 *  - a handle that needs more than AKG_HIP_STATIC_SCRATCH_MAX bytes is refused with AKG_HIP_ERR_UNSUPPORTED;
 *  - the part of the array the handle uses is cleared by a fill kernel on `stream` in front of the launch;
 *  - every call on a device shares that device's array, whatever the handle: calls that overlap on one device race.
 *    Order them on one stream or with events.
 * Each device holds the array (16 MiB) from the first such call until the process ends.
 */
#define AKG_HIP_STATIC_SCRATCH_MAX (16u << 20)
int akg_hip_launch_static_scratch(akg_hip_kernel_t *kernel, void *const *device_ptrs, int n_ptrs, void *stream);

/**
 * Reference-style execution with HOST pointers: allocate device buffers, copy every tensor in (outputs
 * too, as the reference does, gen_runtime_code.py:95-97), launch, copy the outputs back, free. Replaces
 * `extern "C" cuda_runtime_exec(T0* data_0, ...)` (code_template.py:160-211) called from MlirDriver.run_gpu
 * (mlir_driver.py:426-447).
 */
int akg_hip_run_host(akg_hip_kernel_t *kernel, void *const *host_ptrs, int n_ptrs);

/**
 * Time `repeat` batches of `number` back-to-back launches on device-resident buffers with HIP events and
 * return the mean milliseconds per launch. Replaces `cuda_runtime_profiling(..., number, repeat,
 * min_repeat_ms)` (code_template.py:68-155), which timed with std::chrono around a stream synchronize.
 */
int akg_hip_profile(akg_hip_kernel_t *kernel, void *const *device_ptrs, int n_ptrs, int number, int repeat,
                    double *avg_ms);

/** Release the handle (and its loaded module, if any). */
void akg_hip_kernel_destroy(akg_hip_kernel_t *kernel);

/** Message of the last failure on the calling thread ("" if none). */
const char *akg_hip_last_error(void);

/** Translate only: render the typed op graph (the `mindspore-translate -json-to-mindspore` output,
 *  TranslateRegistration.cpp:42-50) into a malloc'ed string the caller frees with akg_hip_free_string. */
int akg_hip_translate(const char *json_text, size_t json_len, char **out_text);
void akg_hip_free_string(char *text);

/**
 * Dynamic shapes: a description whose tensors carry -1 dimensions (MindSpore's dynamic-shape graph kernels). The
 * reference compiles such a description once (`akg-opt --gpu-dyn-opt`), passes sizes and strides as kernel arguments
 * ([ptrs[], shape/stride[][]] packing, LLVMParameterPacking.cpp:91-194) and solves the launch shape per call in Python
 * (dynamic_utils.py:269-526). Here a dynamic description is kept as text and specialised on demand:
 * akg_hip_dynamic_specialize binds the -1s to the given input shapes, derives every op's result shape, lowers the
 * kernel for these shapes and returns its handle. Elementwise and row-reduction kernels take the product of their
 * leading dimensions and their row length as kernel arguments (the schedule is made for the power-of-two bucket of
 * 16-byte chunks the row falls into), MatMul fusions the rows of A and their K split, streaming reductions over the
 * outermost extent that extent and their split, the column kernel the batch in front of its reduced axis: shape sets
 * that differ only there share one code object and the second one needs no device compilation; anything else compiles
 * once per shape set (or is found in the artifact directory). The handle is owned by the dynamic object (do not destroy it); it is
 * launched with akg_hip_launch like any other, and akg_hip_kernel_tensor reports the concrete output shapes.
 */
typedef struct akg_hip_dynamic akg_hip_dynamic_t;
int akg_hip_dynamic_create(const char *json_text, size_t json_len, const char *out_dir, akg_hip_dynamic_t **out);
int akg_hip_dynamic_num_inputs(const akg_hip_dynamic_t *dyn, int *n_inputs);
/** input_shapes[i] points at input_ranks[i] extents of kernel input i (input_desc order). */
int akg_hip_dynamic_specialize(akg_hip_dynamic_t *dyn, const int64_t *const *input_shapes, const int32_t *input_ranks,
                               int n_inputs, akg_hip_kernel_t **out_kernel);
/**
 * The reference's calling form for dynamic-shape kernels (packParamsDynamicShape, LLVMParameterPacking.cpp:91-194, as
 * filled by transform_data_to_ctypes, mlir_driver.py:186-252): one array with the data pointer of every tensor, inputs
 * then outputs, and one array with, per tensor, a pointer to its int64 list [offset, sizes..., strides...] (the integer
 * fields of its memref descriptor; trailing padding is ignored). Reads the input shapes from the lists, finds or makes
 * the specialisation for them (akg_hip_dynamic_specialize), checks the output shapes given against the derived ones,
 * and enqueues the launch on `stream` with the pointers as DEVICE pointers. Tensors must be dense row-major with offset
 * 0 (anything else: AKG_HIP_ERR_UNSUPPORTED). `used_kernel`, if non-NULL, receives the handle that ran (owned by `dyn`).
 */
int akg_hip_dynamic_launch_packed(akg_hip_dynamic_t *dyn, void *const *tensor_ptrs, const int64_t *const *shape_lists,
                                  int n_tensors, void *stream, akg_hip_kernel_t **used_kernel);
void akg_hip_dynamic_destroy(akg_hip_dynamic_t *dyn);

/** Library version string. */
const char *akg_hip_version(void);

#ifdef __cplusplus
}
#endif

#endif /* AKG_HIP_H_ */
