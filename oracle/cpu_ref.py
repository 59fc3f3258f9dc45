"""TEST INFRASTRUCTURE - CPU oracle, part 3: build and call the C restatement through the reference's CPU ABI.

This is the checker, not the product: only tests, the smoke check and the CPU-baseline leg of the benchmark may import
it. The compiled restatement exports `void <op>(void **packed)` - one bare pointer per tensor, inputs then outputs -
exactly how the reference calls its CPU kernels (mlir_driver.py:403-424, transform_data_to_ctypes :186-252,
LLVMParameterPacking.cpp:57-89). Libraries are built into oracle/_build/ (kept out of version control).
"""
import ctypes
import json
import os
import time

import numpy as np

from . import gen_cpu

HERE = os.path.dirname(os.path.abspath(__file__))
BUILD_DIR = os.path.join(HERE, "_build")

NP_EXTERNAL = {"bool": np.bool_, "int8": np.int8, "uint8": np.int8, "int16": np.int16, "int32": np.int32,
               "int64": np.int64, "float16": np.float16, "bfloat16": np.uint16, "float32": np.float32,
               "float64": np.float64}


class CpuKernel:
    """One compiled restatement."""

    def __init__(self, info_path, openmp=False, matmul_order="ijk", rebuild=False):
        with open(info_path, "r", encoding="utf-8") as f:
            self.desc = json.load(f)
        self.name = self.desc["op"]
        stem = self.name + ("_omp" if openmp else "") + ("" if matmul_order == "ijk" else "_" + matmul_order)
        self.so_path = os.path.join(BUILD_DIR, stem + ".so")
        if rebuild or not os.path.exists(self.so_path) or \
                os.path.getmtime(self.so_path) < os.path.getmtime(gen_cpu.__file__):
            gen_cpu.build(info_path, BUILD_DIR, openmp=openmp, matmul_order=matmul_order)
        self.lib = ctypes.CDLL(self.so_path)
        self.fn = getattr(self.lib, self.name)
        self.fn.restype = None
        self.fn.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.openmp = openmp

    def output_arrays(self, fill_nan=True):
        outs = []
        for d in self.desc["output_desc"]:
            dt = NP_EXTERNAL[d["data_type"]]
            a = np.zeros(d.get("shape", [1]), dtype=dt)
            if fill_nan:
                # NaN-prefilled outputs expose elements a kernel fails to write (composite_op_helper.py:702)
                if d["data_type"] in ("float16", "float32", "float64"):
                    a.fill(np.nan)
                elif d["data_type"] == "bfloat16":
                    a.fill(0x7FC0)
            outs.append(a)
        return outs

    def pack(self, inputs, outputs):
        arrays = []
        for entry, arr in zip(self.desc["input_desc"], inputs):
            d = entry[0]
            a = np.ascontiguousarray(arr, dtype=NP_EXTERNAL[d["data_type"]])
            if a.size != int(np.prod(d.get("shape", [1]))):
                raise ValueError("input %s has the wrong number of elements" % d["tensor_name"])
            arrays.append(a)
        arrays.extend(outputs)
        packed = (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
        return packed, arrays

    def __call__(self, inputs):
        outputs = self.output_arrays()
        packed, keep = self.pack(inputs, outputs)
        self.fn(packed)
        del keep
        return outputs

    def time(self, inputs, warmup=1, iters=3):
        """Mean seconds per call: warm-up calls, then timed calls (the reference's timing wrapper does the same with
        1000 warm-ups, code_template.py:219-254; calls here take long enough that a few suffice)."""
        outputs = self.output_arrays(fill_nan=False)
        packed, keep = self.pack(inputs, outputs)
        for _ in range(warmup):
            self.fn(packed)
        t0 = time.perf_counter()
        for _ in range(iters):
            self.fn(packed)
        dt = (time.perf_counter() - t0) / iters
        del keep
        return dt
