"""Python host-side mirror of the reference's driver over the C ABI (ctypes, no compute in Python).

`HipDriver` follows `MlirDriver` of the reference (akg-mlir/python/akg_mlir/mlir_driver.py:255-322):
`HipDriver(kernel_name, input_file, output_dir).compile()` then `.run(input_for_mod, output_indexes)` with host
arrays in signature order (inputs then outputs; outputs are overwritten in place), where the reference's
`backend="gpu"` spawned five tools and an nvcc-built shim. `HipKernel` is the thin handle underneath and also offers
the device-pointer launch that the hot path uses.
"""
import ctypes
import json
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libakg_hip.so")
DEFAULT_META_DIR = os.path.join(_HERE, "kernel_meta")

AKG_HIP_MAX_RANK = 8
DTYPE_NAMES = ["bool", "int8", "int16", "int32", "int64", "float16", "bfloat16", "float32", "float64"]
# numpy view of each element type on the host; bfloat16 travels as uint16 bit patterns
NP_HOST_DTYPE = {"bool": np.bool_, "int8": np.int8, "int16": np.int16, "int32": np.int32, "int64": np.int64,
                 "float16": np.float16, "bfloat16": np.uint16, "float32": np.float32, "float64": np.float64}


class AkgHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("akg_hip error %d: %s" % (code, message))
        self.code = code


class _TensorDesc(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("rank", ctypes.c_int32), ("shape", ctypes.c_int64 * AKG_HIP_MAX_RANK),
                ("bytes", ctypes.c_int64), ("is_output", ctypes.c_int32), ("name", ctypes.c_char * 64)]


class _KernelInfo(ctypes.Structure):
    _fields_ = [("kernel_name", ctypes.c_char * 256), ("family", ctypes.c_char * 32),
                ("operator_type", ctypes.c_char * 32), ("grid", ctypes.c_uint32 * 3), ("block", ctypes.c_uint32 * 3),
                ("algorithmic_bytes", ctypes.c_uint64), ("algorithmic_ops", ctypes.c_uint64),
                ("cache_hit", ctypes.c_int32), ("workspace_bytes", ctypes.c_uint64), ("build_ms", ctypes.c_double)]


_lib = None


def load_library():
    """Load libakg_hip.so from the package directory. There is no fallback: without the native library nothing runs."""
    global _lib
    if _lib is not None:
        return _lib
    # torch wheels bundle their own HIP runtime. Two HIP runtimes in one process cannot both own the GPU, so when
    # torch is installed it is imported first and libakg_hip.so then binds to the runtime torch already loaded.
    try:
        import torch  # noqa: F401  pylint: disable=unused-import,import-outside-toplevel
    except ImportError:
        pass
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `make -C akg_amd/csrc` (or __graft_entry__.build())" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    vp, cp, ci = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int
    lib.akg_hip_compile.argtypes = [cp, ctypes.c_size_t, cp, ctypes.POINTER(vp)]
    lib.akg_hip_compile_file.argtypes = [cp, cp, ctypes.POINTER(vp)]
    lib.akg_hip_kernel_num_tensors.argtypes = [vp, ctypes.POINTER(ci)]
    lib.akg_hip_kernel_tensor.argtypes = [vp, ci, ctypes.POINTER(_TensorDesc)]
    lib.akg_hip_kernel_get_info.argtypes = [vp, ctypes.POINTER(_KernelInfo)]
    lib.akg_hip_kernel_source.argtypes = [vp, ctypes.POINTER(cp)]
    lib.akg_hip_kernel_prepare.argtypes = [vp]
    lib.akg_hip_launch.argtypes = [vp, ctypes.POINTER(vp), ci, vp]
    lib.akg_hip_launch_static_scratch.argtypes = [vp, ctypes.POINTER(vp), ci, vp]
    lib.akg_hip_run_host.argtypes = [vp, ctypes.POINTER(vp), ci]
    lib.akg_hip_profile.argtypes = [vp, ctypes.POINTER(vp), ci, ci, ci, ctypes.POINTER(ctypes.c_double)]
    lib.akg_hip_kernel_destroy.argtypes = [vp]
    lib.akg_hip_kernel_destroy.restype = None
    lib.akg_hip_last_error.restype = cp
    lib.akg_hip_translate.argtypes = [cp, ctypes.c_size_t, ctypes.POINTER(vp)]
    lib.akg_hip_free_string.argtypes = [vp]
    lib.akg_hip_free_string.restype = None
    lib.akg_hip_version.restype = cp
    lib.akg_hip_dynamic_create.argtypes = [cp, ctypes.c_size_t, cp, ctypes.POINTER(vp)]
    lib.akg_hip_dynamic_num_inputs.argtypes = [vp, ctypes.POINTER(ci)]
    lib.akg_hip_dynamic_specialize.argtypes = [vp, ctypes.POINTER(ctypes.POINTER(ctypes.c_int64)),
                                               ctypes.POINTER(ctypes.c_int32), ci, ctypes.POINTER(vp)]
    lib.akg_hip_dynamic_launch_packed.argtypes = [vp, ctypes.POINTER(vp), ctypes.POINTER(ctypes.POINTER(ctypes.c_int64)), ci, vp,
                                                  ctypes.POINTER(vp)]
    lib.akg_hip_dynamic_destroy.argtypes = [vp]
    lib.akg_hip_dynamic_destroy.restype = None
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        raise AkgHipError(rc, load_library().akg_hip_last_error().decode("utf-8", "replace"))


def translate(json_text):
    """Typed op graph of a description as text (what `mindspore-translate -json-to-mindspore` prints)."""
    lib = load_library()
    raw = json_text.encode("utf-8") if isinstance(json_text, str) else json_text
    out = ctypes.c_void_p()
    _check(lib.akg_hip_translate(raw, len(raw), ctypes.byref(out)))
    try:
        return ctypes.string_at(out).decode("utf-8")
    finally:
        lib.akg_hip_free_string(out)


class HipDynamicKernel:
    """A dynamic-shape description (-1 dimensions), specialised per set of input shapes on demand."""

    def __init__(self, json_text, out_dir=DEFAULT_META_DIR):
        self._lib = load_library()
        self._handle = ctypes.c_void_p()
        raw = json_text.encode("utf-8") if isinstance(json_text, str) else json_text
        od = out_dir.encode("utf-8") if out_dir else None
        _check(self._lib.akg_hip_dynamic_create(raw, len(raw), od, ctypes.byref(self._handle)))
        self._kernels = {}
        self._by_handle = {}

    def specialize(self, input_shapes):
        """HipKernel for exactly these input shapes (list of lists, input_desc order); cached per shape set."""
        key = tuple(tuple(int(d) for d in s) for s in input_shapes)
        if key in self._kernels:
            return self._kernels[key]
        n = len(key)
        arrays = [(ctypes.c_int64 * max(1, len(s)))(*s) for s in key]
        ptrs = (ctypes.POINTER(ctypes.c_int64) * n)(*[ctypes.cast(a, ctypes.POINTER(ctypes.c_int64)) for a in arrays])
        ranks = (ctypes.c_int32 * n)(*[len(s) for s in key])
        out = ctypes.c_void_p()
        _check(self._lib.akg_hip_dynamic_specialize(self._handle, ptrs, ranks, n, ctypes.byref(out)))
        k = HipKernel(None, _borrowed=out)
        k._keepalive = self
        self._kernels[key] = k
        return k

    def launch_packed(self, device_ptrs, shapes, stream=None):
        """The reference's dynamic calling form (LLVMParameterPacking.cpp:91-194): `device_ptrs` for inputs then outputs,
        `shapes` their concrete shapes; packs [0, sizes, strides] per tensor like transform_data_to_ctypes
        (mlir_driver.py:186-252) and returns the HipKernel that ran."""
        n = len(device_ptrs)
        width = 1 + 2 * max([len(s) for s in shapes] + [1])
        lists = []
        for s in shapes:
            strides = [1] * len(s)
            for d in range(len(s) - 2, -1, -1):
                strides[d] = strides[d + 1] * s[d + 1]
            row = [0] + list(s) + strides
            lists.append((ctypes.c_int64 * width)(*(row + [0] * (width - len(row)))))
        lptrs = (ctypes.POINTER(ctypes.c_int64) * n)(*[ctypes.cast(a, ctypes.POINTER(ctypes.c_int64)) for a in lists])
        ptrs = (ctypes.c_void_p * n)(*device_ptrs)
        used = ctypes.c_void_p()
        _check(self._lib.akg_hip_dynamic_launch_packed(self._handle, ptrs, lptrs, n, ctypes.c_void_p(stream or 0),
                                                       ctypes.byref(used)))
        key = used.value
        if key not in self._by_handle:
            k = HipKernel(None, _borrowed=used)
            k._keepalive = self
            self._by_handle[key] = k
        return self._by_handle[key]

    def __del__(self):
        h = getattr(self, "_handle", None)
        if h:
            self._kernels = {}
            self._by_handle = {}
            self._lib.akg_hip_dynamic_destroy(h)
            self._handle = None


class TensorDesc:
    def __init__(self, raw):
        self.dtype = DTYPE_NAMES[raw.dtype]
        self.shape = [int(raw.shape[i]) for i in range(raw.rank)]
        self.nbytes = int(raw.bytes)
        self.is_output = bool(raw.is_output)
        self.name = raw.name.decode("utf-8")

    def __repr__(self):
        return "TensorDesc(%s %s %s%s)" % (self.name, self.dtype, self.shape, " out" if self.is_output else "")


class HipKernel:
    """A compiled fused kernel. Construct from JSON text or with `HipKernel.from_file`."""

    def __init__(self, json_text, out_dir=DEFAULT_META_DIR, _path=None, _borrowed=None):
        self._lib = load_library()
        self._handle = ctypes.c_void_p()
        self._owned = _borrowed is None
        od = out_dir.encode("utf-8") if out_dir else None
        if _borrowed is not None:
            self._handle = _borrowed      # owned by a HipDynamicKernel
        elif _path is not None:
            _check(self._lib.akg_hip_compile_file(_path.encode("utf-8"), od, ctypes.byref(self._handle)))
        else:
            raw = json_text.encode("utf-8") if isinstance(json_text, str) else json_text
            _check(self._lib.akg_hip_compile(raw, len(raw), od, ctypes.byref(self._handle)))
        n = ctypes.c_int()
        _check(self._lib.akg_hip_kernel_num_tensors(self._handle, ctypes.byref(n)))
        self.tensors = []
        for i in range(n.value):
            raw_desc = _TensorDesc()
            _check(self._lib.akg_hip_kernel_tensor(self._handle, i, ctypes.byref(raw_desc)))
            self.tensors.append(TensorDesc(raw_desc))
        info = _KernelInfo()
        _check(self._lib.akg_hip_kernel_get_info(self._handle, ctypes.byref(info)))
        self.kernel_name = info.kernel_name.decode("utf-8")
        self.family = info.family.decode("utf-8")
        self.operator_type = info.operator_type.decode("utf-8")
        self.grid = tuple(int(x) for x in info.grid)
        self.block = tuple(int(x) for x in info.block)
        self.algorithmic_bytes = int(info.algorithmic_bytes)
        self.algorithmic_ops = int(info.algorithmic_ops)
        self.cache_hit = bool(info.cache_hit)
        self.workspace_bytes = int(info.workspace_bytes)
        self.build_ms = float(info.build_ms)

    @classmethod
    def from_file(cls, info_path, out_dir=DEFAULT_META_DIR):
        return cls(None, out_dir=out_dir, _path=info_path)

    def close(self):
        """Destroy the handle now (akg_hip_kernel_destroy) instead of when the object is collected."""
        h = getattr(self, "_handle", None)
        if h and getattr(self, "_owned", True):
            self._lib.akg_hip_kernel_destroy(h)
        self._handle = None

    def __del__(self):
        self.close()

    @property
    def inputs(self):
        return [t for t in self.tensors if not t.is_output]

    @property
    def outputs(self):
        return [t for t in self.tensors if t.is_output]

    @property
    def source(self):
        out = ctypes.c_char_p()
        _check(self._lib.akg_hip_kernel_source(self._handle, ctypes.byref(out)))
        return out.value.decode("utf-8")

    def _ptr_array(self, ptrs):
        if len(ptrs) != len(self.tensors):
            raise ValueError("kernel %s takes %d tensors, %d given" % (self.kernel_name, len(self.tensors), len(ptrs)))
        return (ctypes.c_void_p * len(ptrs))(*ptrs)

    def prepare(self):
        """Load the code object and allocate the workspace on the current device (later launches allocate nothing)."""
        _check(self._lib.akg_hip_kernel_prepare(self._handle))

    # -- device-resident path (the hot call) -------------------------------------------------------------
    def launch_ptrs(self, device_ptrs, stream=None):
        arr = self._ptr_array(device_ptrs)
        _check(self._lib.akg_hip_launch(self._handle, arr, len(device_ptrs), ctypes.c_void_p(stream or 0)))

    def launch_static_scratch_ptrs(self, device_ptrs, stream=None):
        """`launch_ptrs` through the entry point that allocates nothing (needs `prepare()` on the device first)."""
        arr = self._ptr_array(device_ptrs)
        _check(self._lib.akg_hip_launch_static_scratch(self._handle, arr, len(device_ptrs), ctypes.c_void_p(stream or 0)))

    def launch(self, tensors, stream=None):
        """Launch on torch device tensors (inputs then outputs), on `stream` (a torch stream) or the current one."""
        import torch
        for t, d in zip(tensors, self.tensors):
            if not t.is_cuda or not t.is_contiguous():
                raise ValueError("tensor %s must be a contiguous device tensor" % d.name)
            if t.numel() * t.element_size() != d.nbytes:
                raise ValueError("tensor %s has %d bytes, kernel expects %d" % (d.name, t.numel() * t.element_size(), d.nbytes))
        s = stream if stream is not None else torch.cuda.current_stream()
        self.launch_ptrs([t.data_ptr() for t in tensors], s.cuda_stream)

    def profile_ptrs(self, device_ptrs, number=10, repeat=5):
        arr = self._ptr_array(device_ptrs)
        avg = ctypes.c_double()
        _check(self._lib.akg_hip_profile(self._handle, arr, len(device_ptrs), number, repeat, ctypes.byref(avg)))
        return avg.value

    # -- reference-style path: host arrays in, outputs overwritten in place ---------------------------------
    def run_host(self, arrays):
        keep = []
        for a, d in zip(arrays, self.tensors):
            if not isinstance(a, np.ndarray) or not a.flags["C_CONTIGUOUS"]:
                raise ValueError("tensor %s must be a C-contiguous numpy array" % d.name)
            if a.nbytes != d.nbytes:
                raise ValueError("tensor %s has %d bytes, kernel expects %d" % (d.name, a.nbytes, d.nbytes))
            if d.is_output and not a.flags["WRITEABLE"]:
                raise ValueError("output %s is not writeable" % d.name)
            keep.append(a)
        arr = self._ptr_array([a.ctypes.data for a in keep])
        _check(self._lib.akg_hip_run_host(self._handle, arr, len(keep)))

    def empty_outputs(self, fill_nan=True):
        """Host output arrays, NaN-prefilled like the reference harness does (composite_op_helper.py:702)."""
        outs = []
        for d in self.outputs:
            a = np.zeros(d.shape, dtype=NP_HOST_DTYPE[d.dtype])
            if fill_nan:
                if d.dtype in ("float16", "float32", "float64"):
                    a.fill(np.nan)
                elif d.dtype == "bfloat16":
                    a.fill(0x7FC0)
            outs.append(a)
        return outs


class HipDriver:
    """Counterpart of the reference's MlirDriver for backend "hip" (mlir_driver.py:255-322)."""

    def __init__(self, kernel_name=None, input_file=None, output_dir=None, backend="hip", profiling_trails=0):
        if backend != "hip":
            raise ValueError("HipDriver only drives the hip backend")
        if input_file is None:
            raise ValueError("input_file (an .info op description) is required")
        self.input_file = input_file
        self.output_dir = output_dir or os.environ.get("KERNEL_META_DIR") or DEFAULT_META_DIR
        self.profiling_trails = profiling_trails
        with open(input_file, "r", encoding="utf-8") as f:
            self.desc = json.load(f)
        self.kernel_name = kernel_name or self.desc["op"]
        self.kernel = None

    def compile(self):
        self.kernel = HipKernel.from_file(self.input_file, out_dir=self.output_dir)
        return self.kernel

    def run(self, input_for_mod, output_indexes=None):
        """`input_for_mod`: host arrays, inputs then outputs (as gen_json_data builds them,
        composite_op_helper.py:833-902). Outputs are overwritten in place and also returned, selected by
        `output_indexes` (negative indices from the end, as the reference harness passes them)."""
        if self.kernel is None:
            self.compile()
        self.kernel.run_host(list(input_for_mod))
        if output_indexes is None:
            output_indexes = list(range(-len(self.kernel.outputs), 0))
        return [input_for_mod[i] for i in output_indexes]
