#!/usr/bin/env python3
"""TEST INFRASTRUCTURE - CPU oracle, part 1: op description -> C restatement of the reference CPU pipeline.

This is the checker, not the product: only tests, the smoke check and the CPU-baseline leg of the benchmark may use
it. It restates, for one MindSpore graph-kernel JSON description, what the reference's `--cpu-opt` pipeline
(akg-mlir/lib/Pipelines/CPUOpt.cpp:185-216, default `cpu-fast=false`) compiles to:

  * every op computes in its declared result element type (MindSporeToTosa.cpp:475-504 + upstream tosa-to-linalg:
    arith.addf/mulf/divf..., tosa.cast = round-to-nearest-even truncf for float->float, roundeven + clamp + fptosi for
    float->int); math ops go to libm (`convert-math-to-libm`, CPUOpt.cpp:162): tanhf, expf, logf, ...; math.rsqrt
    reaches LLVM as 1/sqrt(x);
  * elementwise producers with a single use are fused into their consumer's loop nest
    (`linalg-fuse-elementwise-ops`, CPUOpt.cpp:89-92); everything else is a buffer in memory;
  * a reduction is its own loop nest accumulating serially, in the result element type, from the init value of
    createInitValueForReduce (MindSporeToLinalg.cpp:791-843: sum 0, prod 1, max = -largest finite, min = +largest
    finite) with the combiner of createCombinerForReduce (:845-901: addf, mulf, maxnumf, minnumf);
  * MatMul is linalg.matmul into a zero-filled accumulator of the OUTPUT element type (MindSporeToLinalg.cpp:1453-1546),
    i.e. int8 x int8 -> int32 is sign-extend + i32 multiply-accumulate, loops in (i, j, k) order
    (`convert-linalg-to-loops`, CPUOpt.cpp:199-205);
  * the function is `void <op>(void **packed)`: one bare pointer per tensor, inputs then outputs
    (ParameterPacking, akg-mlir/lib/Dialect/LLVMIR/Transforms/LLVMParameterPacking.cpp:57-89).

Scalar, single-threaded, like the reference default. With --openmp the outermost parallel loop of every nest gets
`#pragma omp parallel for` (what cpu-fast + enable-parallel would allow, LoopParallelize.cpp:83-141).

Parity status of the individual rules is listed in oracle/README.md ("pinned by" column).
"""
import argparse
import json
import math
import os
import struct
import subprocess
import sys

try:
    from oracle.view_attrs import VIEW_OPS, view_params, expand_split
except ImportError:  # run as a script from inside oracle/
    from view_attrs import VIEW_OPS, view_params, expand_split

FLOATS = ("float16", "bfloat16", "float32", "float64")
INTS = ("int8", "int16", "int32", "int64")

C_STORAGE = {
    "bool": "uint8_t", "int8": "int8_t", "int16": "int16_t", "int32": "int32_t", "int64": "int64_t",
    "float16": "uint16_t", "bfloat16": "uint16_t", "float32": "float", "float64": "double",
}
C_COMPUTE = {
    "bool": "int", "int8": "int32_t", "int16": "int32_t", "int32": "int32_t", "int64": "int64_t",
    "float16": "float", "bfloat16": "float", "float32": "float", "float64": "double",
}
INT_RANGE = {"int8": (-128, 127), "int16": (-32768, 32767), "int32": (-2147483648, 2147483647),
             "int64": (-9223372036854775808, 9223372036854775807)}

# Exp / Log / Tanh / Floor come through tosa (MindSporeToTosa.cpp:490-497) and end in libm (`convert-math-to-libm`), Sin / Cos /
# Sqrt through math.sin / cos / sqrt (MindSporeToLinalg.cpp:182-193,248-259). ASin, ACos and Atan are in the op table but
# have no lowering in the reference (createLinalgBodyCalculationForElementwiseOp, MindSporeToLinalg.cpp:341-375, returns
# nothing for them and its conversion fails): they are restated as the functions their names say.
UNARY_MATH = {"Exp": "exp", "Log": "log", "Tanh": "tanh", "Sqrt": "sqrt", "Floor": "floor", "Sin": "sin", "Cos": "cos",
              "ASin": "asin", "ACos": "acos", "Atan": "atan"}
COMPARE = {"Equal": "==", "NotEqual": "!=", "Greater": ">", "GreaterEqual": ">=", "Less": "<", "LessEqual": "<="}
MATMULS = ("MatMul", "BatchMatMul")
# Assign / InplaceAssign: linalg.copy ins=input1 outs=input0 (MindSporeToLinalg.cpp:495-524): the value is written over
# the first operand's buffer (a kernel input) and is also the op's result; the result has the destination's shape
# (TranslateToMindsporeDialect.cpp:359-364,398-404)
ASSIGNS = ("Assign", "InplaceAssign")
SEGMENTS = ("UnsortedSegmentSum",)
REDUCES = ("ReduceSum", "ReduceMax", "ReduceMin", "ReducePrd", "ReduceAll", "ReduceAny")
ATTR_AS_INPUT = ("Reshape", "BroadcastTo", "ReduceMax", "ReduceMin", "ReduceSum", "ReducePrd", "ReduceAll", "ReduceAny",
                 "ArgMax", "Transpose", "Tile")

PRELUDE = r"""
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- element type helpers (software conversions: no _Float16/__bf16 in this compiler) ---- */
static inline float akg_bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t akg_f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float akg_bf16_load(uint16_t b) { return akg_bits_to_f32((uint32_t)b << 16); }
static inline uint16_t akg_bf16_store(float f) {              /* arith.truncf f32->bf16: round to nearest even */
  uint32_t u = akg_f32_to_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static inline float akg_rnd_bf16(float f) { return akg_bf16_load(akg_bf16_store(f)); }

static inline float akg_f16_load(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return akg_bits_to_f32(sign);
    float v = (float)man * 5.9604644775390625e-08f;             /* man * 2^-24, exact */
    return sign ? -v : v;
  }
  if (exp == 31) return akg_bits_to_f32(sign | 0x7f800000u | (man << 13));
  return akg_bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}
static inline uint16_t akg_f16_store(float f) {               /* arith.truncf f32->f16: round to nearest even */
  uint32_t u = akg_f32_to_bits(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);                  /* NaN */
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                 /* >= 65520 -> inf */
  if (a < 0x33000001u) return sign;                                        /* <= 2^-25 -> 0 (tie to even) */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;                                /* 24-bit significand */
  int shift = (e < -14) ? (13 + (-14 - e)) : 13;                           /* bits to drop */
  uint32_t kept = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) kept += 1u;
  uint32_t out;
  if (e < -14) {
    out = kept;                                                            /* subnormal (may carry into normal) */
  } else {
    out = ((uint32_t)(e + 15) << 10) + (kept - 0x400u);                    /* carry propagates into exponent */
  }
  return (uint16_t)(sign | out);
}
static inline float akg_rnd_f16(float f) { return akg_f16_load(akg_f16_store(f)); }

/* arith.maximumf / minimumf (NaN-propagating), used by tosa.maximum / tosa.minimum */
static inline float akg_maximumf(float a, float b) { return (a != a) ? a : ((b != b) ? b : (a > b ? a : (b > a ? b : (signbit(a) ? b : a)))); }
static inline float akg_minimumf(float a, float b) { return (a != a) ? a : ((b != b) ? b : (a < b ? a : (b < a ? b : (signbit(a) ? a : b)))); }
static inline double akg_maximumd(double a, double b) { return (a != a) ? a : ((b != b) ? b : (a > b ? a : (b > a ? b : (signbit(a) ? b : a)))); }
static inline double akg_minimumd(double a, double b) { return (a != a) ? a : ((b != b) ? b : (a < b ? a : (b < a ? b : (signbit(a) ? a : b)))); }

/* tosa.cast float -> signed int: math.roundeven, clamp to the destination range, fptosi */
static inline int64_t akg_cast_f2i(double x, double lo, double hi) {
  double r = nearbyint(x);                                   /* default rounding mode: half to even */
  if (r != r) return 0;
  if (r <= lo) return (int64_t)lo;
  if (r >= hi) return (hi >= 9223372036854775807.0) ? INT64_MAX : (int64_t)hi;
  return (int64_t)r;
}
static inline int64_t akg_clamp_i(int64_t v, int64_t lo, int64_t hi) { return v < lo ? lo : (v > hi ? hi : v); }
static inline int32_t akg_divsi32(int32_t a, int32_t b) { return b == 0 ? 0 : ((a == INT32_MIN && b == -1) ? a : a / b); }
static inline int64_t akg_divsi64(int64_t a, int64_t b) { return b == 0 ? 0 : ((a == INT64_MIN && b == -1) ? a : a / b); }
"""


class OracleError(Exception):
    pass


def canon_dtype(name):
    if name in ("uint8", "sint8"):
        return "int8"  # TranslateToMindsporeDialect.cpp:331-333
    if name == "int1":
        return "bool"
    if name not in C_STORAGE:
        raise OracleError("data type %s is not supported" % name)
    return name


class T:
    """One tensor of the description."""

    def __init__(self, name, shape, dtype):
        self.name = name
        self.shape = list(shape) if shape else [1]
        self.dtype = canon_dtype(dtype)
        self.const = None      # python number for scalar constants
        self.producer = None   # Op
        self.uses = 0
        self.is_input = False
        self.is_output = False
        self.buffer = None     # C identifier of the memory holding it, if materialised
        self.alias_of = None   # Reshape views

    @property
    def numel(self):
        return int(math.prod(self.shape))


class Op:
    def __init__(self, name, inputs, output, attrs):
        self.name = name
        self.inputs = inputs
        self.output = output
        self.attrs = attrs
        self.axes = []
        self.keep_dims = False


def parse(desc):
    """JSON document -> (name, inputs, ops, outputs); same reading rules as the reference translator
    (TranslateToMindsporeDialect.cpp:295-415, 793-808, 1273-1318)."""
    desc = expand_split(desc)
    tensors = {}
    inputs = []
    for entry in desc["input_desc"]:
        d = entry[0]
        t = T(d["tensor_name"], d.get("shape", [1]), d["data_type"])
        t.is_input = True
        tensors[t.name] = t
        inputs.append(t)
    ops = []
    for od in desc["op_desc"]:
        name = od["name"]
        if name == "ElemAny":  # same mindspore op as ReduceAny (TranslateToMindsporeDialect.cpp:463)
            name = "ReduceAny"
        attrs = {a["name"]: a["value"] for a in (od.get("attr") or [])}
        ins = []
        entries = od["input_desc"]
        if name == "Concat":  # one entry holding the list of operands (TranslateToMindsporeDialect.cpp:772-791)
            entries = [[d] for entry in entries for d in entry]
        for idx, entry in enumerate(entries):
            if idx == 1 and name in ATTR_AS_INPUT:
                continue
            if name == "Cast" and idx > 0:
                continue
            if name == "StridedSlice" and idx > 0:
                continue
            if name == "Gather" and idx > 1:
                continue
            if name in ASSIGNS and idx > 1:
                continue
            if name in SEGMENTS and idx > 1:
                continue
            d = entry[0]
            if d["tensor_name"] in tensors:
                ins.append(tensors[d["tensor_name"]])
                continue
            if "value" not in d:
                raise OracleError("op %s: operand %s is undefined" % (name, d["tensor_name"]))
            v = d["value"]
            if isinstance(v, list):
                if len(v) != 1:
                    raise OracleError("array constants are not supported")
                v = v[0]
            c = T(d["tensor_name"], d.get("shape", [1]), d["data_type"])
            c.const = v if c.dtype in FLOATS else int(v)
            tensors[c.name] = c
            ins.append(c)
        o = od["output_desc"][0]
        out = T(o["tensor_name"], ins[0].shape if name in ASSIGNS else o.get("shape", [1]), o["data_type"])
        op = Op(name, ins, out, attrs)
        if name in VIEW_OPS:
            op.view = view_params(od, ins[0].shape)
        out.producer = op
        if name in REDUCES + ("ArgMax",):
            if len(od["input_desc"]) == 2:
                axes = od["input_desc"][1][0]["value"]
            else:
                axes = attrs["axis"]
            if not isinstance(axes, list):
                axes = [axes]
            if not axes:
                axes = [1]
            rank = len(ins[0].shape)
            op.axes = sorted(set(a + rank if a < 0 else a for a in axes))
            op.keep_dims = bool(attrs.get("keep_dims", False))
        tensors[out.name] = out
        ops.append(op)
    outputs = []
    for d in desc["output_desc"]:
        t = tensors[d["tensor_name"]]
        t.is_output = True
        outputs.append(t)
    for op in ops:
        for t in op.inputs:
            t.uses += 1
    return desc["op"], inputs, ops, outputs


def float_literal(dtype, v):
    """C literal of constant `v` rounded to `dtype`, in the compute type."""
    if dtype == "float64":
        return "(%s)" % float(v).hex() if math.isfinite(v) else ("NAN" if v != v else ("INFINITY" if v > 0 else "-INFINITY"))
    f = struct.unpack("f", struct.pack("f", float(v)))[0]
    if not math.isfinite(f):
        return "NAN" if f != f else ("INFINITY" if f > 0 else "-INFINITY")
    lit = "%sf" % float(f).hex()
    if dtype == "float16":
        return "akg_rnd_f16(%s)" % lit
    if dtype == "bfloat16":
        return "akg_rnd_bf16(%s)" % lit
    return "(%s)" % lit


class Emitter:
    def __init__(self, desc, openmp=False, matmul_order="ijk"):
        self.name, self.inputs, self.ops, self.outputs = parse(desc)
        self.openmp = openmp
        self.matmul_order = matmul_order
        self.lines = []
        self.temps = []

    # -- which values live in memory --------------------------------------------------------------------
    def is_elementwise(self, op):
        return op.name not in REDUCES + MATMULS + ("Reshape", "ArgMax") + VIEW_OPS + ASSIGNS + SEGMENTS

    def plan(self):
        consumers = {}
        for op in self.ops:
            for t in op.inputs:
                consumers.setdefault(t.name, []).append(op)
        for op in self.ops:
            out = op.output
            if op.name == "Reshape":
                out.alias_of = op.inputs[0]
                continue
            inline = (self.is_elementwise(op) and out.uses == 1 and not out.is_output
                      and consumers[out.name][0].name not in MATMULS + ("Reshape",) + VIEW_OPS + SEGMENTS)
            out.inline = inline
        # the source of a Reshape view and MatMul operands must be in memory
        for op in self.ops:
            if op.name in MATMULS + ("Reshape",) + VIEW_OPS + SEGMENTS:
                for t in op.inputs:
                    if t.producer is not None and t.producer.name != "Reshape":
                        t.inline = False

    # -- expressions ------------------------------------------------------------------------------------
    @staticmethod
    def index_expr(t, iter_shape):
        """Linear index of `t` for the iteration point (i0..in-1), numpy broadcasting, right-aligned."""
        shape = list(t.shape)
        while len(shape) > len(iter_shape) and shape[0] == 1:
            shape = shape[1:]
        if len(shape) > len(iter_shape):
            raise OracleError("tensor %s does not broadcast into the loop nest" % t.name)
        off = len(iter_shape) - len(shape)
        expr = None
        for d, extent in enumerate(shape):
            if extent != 1 and extent != iter_shape[off + d]:
                raise OracleError("tensor %s (shape %s) does not broadcast to %s" % (t.name, t.shape, iter_shape))
            term = "i%d" % (off + d) if extent != 1 else "0"
            expr = term if expr is None else "(%s) * %dL + %s" % (expr, extent, term)
        return expr or "0"

    def root(self, t):
        while t.alias_of is not None:
            t = t.alias_of
        return t

    def value_expr(self, t, iter_shape):
        """C expression (compute type) of tensor `t` at the current iteration point."""
        if t.const is not None:
            if t.dtype in FLOATS:
                return float_literal(t.dtype, t.const)
            if t.dtype == "bool":
                return "1" if t.const else "0"
            return "((%s)%dLL)" % (C_COMPUTE[t.dtype], int(t.const))
        if t.alias_of is not None:
            # a reshape view: same linear position in the source buffer (shapes are dense row-major)
            src = self.root(t)
            return self.load_expr(src, self.index_expr(t, iter_shape))
        if t.producer is not None and getattr(t, "inline", False):
            return self.op_expr(t.producer, iter_shape)
        return self.load_expr(t, self.index_expr(t, iter_shape))

    def load_expr(self, t, idx):
        ref = "%s[%s]" % (t.buffer, idx)
        if t.dtype == "float16":
            return "akg_f16_load(%s)" % ref
        if t.dtype == "bfloat16":
            return "akg_bf16_load(%s)" % ref
        if t.dtype == "bool":
            return "(%s != 0)" % ref
        return "((%s)%s)" % (C_COMPUTE[t.dtype], ref)

    @staticmethod
    def store_expr(dtype, value):
        if dtype == "float16":
            return "akg_f16_store(%s)" % value
        if dtype == "bfloat16":
            return "akg_bf16_store(%s)" % value
        if dtype == "bool":
            return "(uint8_t)((%s) ? 1 : 0)" % value
        return "(%s)(%s)" % (C_STORAGE[dtype], value)

    @staticmethod
    def rnd(dtype, e):
        if dtype == "float16":
            return "akg_rnd_f16(%s)" % e
        if dtype == "bfloat16":
            return "akg_rnd_bf16(%s)" % e
        if dtype in ("int8", "int16"):
            return "((int32_t)(%s)(%s))" % (C_STORAGE[dtype], e)
        return e

    def op_expr(self, op, iter_shape):
        od = op.output.dtype
        ct = C_COMPUTE[od]
        ins = [self.value_expr(t, iter_shape) for t in op.inputs]
        conv = ["((%s)%s)" % (ct, e) if C_COMPUTE[t.dtype] != ct else e for e, t in zip(ins, op.inputs)]
        suffix = "" if od == "float64" else "f"
        n = op.name
        if n in ("Add", "Sub", "Mul"):
            sym = {"Add": "+", "Sub": "-", "Mul": "*"}[n]
            if od in INTS:
                ut = "uint64_t" if od == "int64" else "uint32_t"
                return self.rnd(od, "((%s)((%s)%s %s (%s)%s))" % (ct, ut, conv[0], sym, ut, conv[1]))
            return self.rnd(od, "(%s %s %s)" % (conv[0], sym, conv[1]))
        if n in ("Div", "RealDiv"):
            if od in INTS:
                return self.rnd(od, "%s(%s, %s)" % ("akg_divsi64" if od == "int64" else "akg_divsi32", conv[0], conv[1]))
            return self.rnd(od, "(%s / %s)" % (conv[0], conv[1]))
        if n in ("Maximum", "Minimum"):
            if od in INTS:
                sym = ">" if n == "Maximum" else "<"
                return "((%s) %s (%s) ? (%s) : (%s))" % (conv[0], sym, conv[1], conv[0], conv[1])
            fn = ("akg_maximum" if n == "Maximum" else "akg_minimum") + ("d" if od == "float64" else "f")
            return "%s(%s, %s)" % (fn, conv[0], conv[1])
        if n == "Neg":
            return self.rnd(od, "(-%s)" % conv[0]) if od in FLOATS else self.rnd(od, "((%s)(0u - (uint64_t)%s))" % (ct, conv[0]))
        if n == "Abs":
            if od in FLOATS:
                return "fabs%s(%s)" % (suffix, conv[0])
            return self.rnd(od, "((%s) < 0 ? (%s)(0u - (uint64_t)%s) : (%s))" % (conv[0], ct, conv[0], conv[0]))
        if n == "Square":
            return self.rnd(od, "(%s * %s)" % (conv[0], conv[0]))
        if n in UNARY_MATH:
            if od not in FLOATS:
                raise OracleError("%s needs a float tensor" % n)
            return self.rnd(od, "%s%s(%s)" % (UNARY_MATH[n], suffix, conv[0]))
        if n in ("Asinh", "Acosh"):
            # not libm: log(x + sqrt(1 + x*x)) and log(x + sqrt(x*x - 1)), one arith / math op of the result type each
            # (createAsinhOp / createAcoshOp, MindSporeToLinalg.cpp:156-180)
            if od not in FLOATS:
                raise OracleError("%s needs a float tensor" % n)
            one = "1.0" if od == "float64" else "1.0f"
            sq = self.rnd(od, "(%s * %s)" % (conv[0], conv[0]))
            inner = self.rnd(od, "(%s + %s)" % (one, sq)) if n == "Asinh" else self.rnd(od, "(%s - %s)" % (sq, one))
            root = self.rnd(od, "sqrt%s(%s)" % (suffix, inner))
            return self.rnd(od, "log%s(%s)" % (suffix, self.rnd(od, "(%s + %s)" % (conv[0], root))))
        if n == "Rsqrt":
            one = "1.0" if od == "float64" else "1.0f"
            return self.rnd(od, "(%s / sqrt%s(%s))" % (one, suffix, conv[0]))
        if n == "Reciprocal":
            one = "1.0" if od == "float64" else "1.0f"
            return self.rnd(od, "(%s / %s)" % (one, conv[0]))
        if n == "Pow":
            return self.rnd(od, "pow%s(%s, %s)" % (suffix, conv[0], conv[1]))
        if n == "Atan2":
            return self.rnd(od, "atan2%s(%s, %s)" % (suffix, conv[0], conv[1]))
        if n in COMPARE:
            a, b = ins
            if C_COMPUTE[op.inputs[0].dtype] != C_COMPUTE[op.inputs[1].dtype]:
                a, b = "((double)%s)" % a, "((double)%s)" % b
            return "((%s)(%s %s %s))" % (ct, a, COMPARE[n], b)
        if n == "IsNan":
            return "((%s)(%s != %s))" % (ct, ins[0], ins[0])
        if n == "IsInf":
            return "((%s)(isinf(%s) != 0))" % (ct, ins[0])
        if n == "IsFinite":
            return "((%s)(isfinite(%s) != 0))" % (ct, ins[0])
        if n == "LogicalNot":
            return "((%s)(!(%s != 0)))" % (ct, ins[0])
        if n == "LogicalAnd":
            return "((%s)((%s != 0) && (%s != 0)))" % (ct, ins[0], ins[1])
        if n == "LogicalOr":
            return "((%s)((%s != 0) || (%s != 0)))" % (ct, ins[0], ins[1])
        if n == "Select":
            return "((%s != 0) ? %s : %s)" % (ins[0], conv[1], conv[2])
        if n == "AddN":
            e = conv[0]
            for c in conv[1:]:
                e = self.rnd(od, "(%s + %s)" % (e, c))
            return e
        if n == "BroadcastTo":
            return conv[0]
        if n == "Cast":
            return self.cast_expr(op.inputs[0].dtype, od, ins[0])
        raise OracleError("op %s is not supported by the CPU restatement" % n)

    def cast_expr(self, src, dst, e):
        if dst == "bool":
            return "(%s != 0)" % e
        if dst in FLOATS:
            return self.rnd(dst, "((%s)%s)" % (C_COMPUTE[dst], e))
        lo, hi = INT_RANGE[dst]
        if src in FLOATS:
            return "((%s)akg_cast_f2i((double)%s, %s.0, %s.0))" % (C_COMPUTE[dst], e, lo, hi)
        if src == "bool":
            return "((%s)(%s ? 1 : 0))" % (C_COMPUTE[dst], e)
        lo_lit = "INT64_MIN" if lo == INT_RANGE["int64"][0] else "%dLL" % lo
        return "((%s)akg_clamp_i((int64_t)%s, %s, %dLL))" % (C_COMPUTE[dst], e, lo_lit, hi)

    # -- statements -------------------------------------------------------------------------------------
    def emit(self, s, depth=1):
        self.lines.append("  " * depth + s)

    def open_loops(self, shape, parallel_outer, first_index=0, depth=1):
        for d, extent in enumerate(shape):
            if d == 0 and parallel_outer and self.openmp:
                self.emit("#pragma omp parallel for schedule(static)", depth)
            self.emit("for (int64_t i%d = 0; i%d < %dL; ++i%d) {" % (first_index + d, first_index + d, extent, first_index + d),
                      depth + d)
        return depth + len(shape)

    def close_loops(self, count, depth):
        for d in range(count):
            self.emit("}", depth - 1 - d)

    def emit_elementwise(self, op):
        out = op.output
        shape = out.shape
        depth = self.open_loops(shape, True)
        expr = self.op_expr(op, shape)
        self.emit("%s[%s] = %s;" % (out.buffer, self.index_expr(out, shape), self.store_expr(out.dtype, expr)), depth)
        self.close_loops(len(shape), depth)

    def emit_assign(self, op):
        dst, src, out = op.inputs[0], op.inputs[1], op.output
        if not dst.is_input or dst.dtype != out.dtype:
            raise OracleError("%s: the destination must be a kernel input of the value's type" % op.name)
        shape = dst.shape
        depth = self.open_loops(shape, True)
        value = self.value_expr(src, shape)
        self.emit("const %s v = %s;" % (C_STORAGE[out.dtype], self.store_expr(out.dtype, value)), depth)
        idx = self.index_expr(dst, shape)
        self.emit("((%s *)%s)[%s] = v;" % (C_STORAGE[dst.dtype], dst.buffer, idx), depth)
        self.emit("%s[%s] = v;" % (out.buffer, idx), depth)
        self.close_loops(len(shape), depth)

    def emit_segment_sum(self, op):
        """UnsortedSegmentSum (MindSporeToLinalg.cpp:596-745): the index dimensions collapse into one, the result is
        zero-filled, and ONE serial loop over the index positions adds data[i, :] to result[ids[i], :], rounding to the
        result's type after every addition. The reference indexes the result with the id as it is; ids outside
        [0, segments) are dropped here (parity unpinned for those: the reference's access would be out of bounds)."""
        data, ids, out = op.inputs[0], op.inputs[1], op.output
        if data.const is not None or ids.const is not None or data.dtype != out.dtype or ids.dtype in FLOATS + ("bool",):
            raise OracleError("UnsortedSegmentSum: needs a data tensor of the result's type and integer segment ids")
        if list(data.shape[:len(ids.shape)]) != list(ids.shape):
            raise OracleError("UnsortedSegmentSum: the ids must have the leading dimensions of the data")
        positions = max(1, ids.numel)
        slice_ = data.numel // positions
        segments = out.numel // slice_
        want = op.attrs.get("numSegments", op.attrs.get("num_segments", segments))
        if isinstance(want, list):
            want = want[0]
        if int(want) != segments:
            raise OracleError("UnsortedSegmentSum: the result shape does not follow from the segment count")
        rd, ri = self.root(data), self.root(ids)
        od = out.dtype
        self.emit("memset(%s, 0, sizeof(%s) * %dL);" % (out.buffer, C_STORAGE[od], out.numel))
        self.emit("for (int64_t i = 0; i < %dL; ++i) {" % positions)
        self.emit("const int64_t id = (int64_t)%s[i];" % ri.buffer, 2)
        self.emit("if (id < 0 || id >= %dL) continue;" % segments, 2)
        self.emit("for (int64_t j = 0; j < %dL; ++j) {" % slice_, 2)
        x = self.load_expr(rd, "i * %dL + j" % slice_)
        acc = self.load_expr(out, "id * %dL + j" % slice_)
        if od in FLOATS:
            step = self.rnd(od, "(%s + %s)" % (x, acc))
        else:
            step = self.rnd(od, "((%s)((uint64_t)%s + (uint64_t)%s))" % (C_COMPUTE[od], x, acc))
        self.emit("%s[id * %dL + j] = %s;" % (out.buffer, slice_, self.store_expr(od, step)), 3)
        self.emit("}", 2)
        self.emit("}")

    def emit_view(self, op):
        """Data-movement op: a loop nest over the result that copies the operand element its index map names."""
        out, src, vp = op.output, op.inputs[0], op.view
        if src.const is not None or out.dtype != src.dtype:
            raise OracleError("%s: operand must be a tensor of the result's type" % op.name)
        shape = out.shape
        rank = len(shape)
        depth = self.open_loops(shape, True)
        idx = ["i%d" % d for d in range(rank)]

        def lin(t, terms):
            expr = None
            for term, extent in zip(terms, t.shape):
                expr = term if expr is None else "(%s) * %dL + %s" % (expr, extent, term)
            return expr or "0"

        def load(t, terms):
            return self.load_expr(self.root(t), lin(t, terms))

        n = op.name
        if n == "Transpose":
            terms = [None] * rank
            for d, p in enumerate(vp["perm"]):
                terms[p] = idx[d]
            value = load(src, terms)
        elif n == "Tile":
            value = load(src, ["(%s %% %dL)" % (idx[d], src.shape[d]) for d in range(rank)])
        elif n in ("Slice", "StridedSlice"):
            value = load(src, ["(%dL + %s * %dL)" % (vp["begin"][d], idx[d], vp["strides"][d]) for d in range(rank)])
        elif n == "Pad":
            cond = " && ".join("%s >= %dL && %s < %dL" % (idx[d], vp["low"][d], idx[d], vp["low"][d] + src.shape[d])
                               for d in range(rank))
            inner = load(src, ["(%s - %dL)" % (idx[d], vp["low"][d]) for d in range(rank)])
            if out.dtype in FLOATS:
                fill = float_literal(out.dtype, float(vp["value"]))
            else:
                fill = "((%s)%dLL)" % (C_COMPUTE[out.dtype], vp["value"])
            value = "((%s) ? %s : %s)" % (cond, inner, fill)
        elif n == "Gather":
            ind, a = op.inputs[1], vp["axis"]
            nind = len(ind.shape)
            pos = load(ind, idx[a:a + nind])
            hi = src.shape[a] - 1
            clamped = "((%s) < 0 ? 0 : ((%s) > %dL ? %dL : (int64_t)(%s)))" % (pos, pos, hi, hi, pos)
            value = load(src, idx[:a] + [clamped] + idx[a + nind:])
        else:
            other, a = op.inputs[1], vp["axis"]
            if other.const is not None or other.dtype != out.dtype:
                raise OracleError("Concat: operands must be tensors of the result's type")
            second = list(idx)
            second[a] = "(%s - %dL)" % (idx[a], src.shape[a])
            value = "((%s < %dL) ? %s : %s)" % (idx[a], src.shape[a], load(src, idx), load(other, second))
        self.emit("%s[%s] = %s;" % (out.buffer, lin(out, idx), self.store_expr(out.dtype, value)), depth)
        self.close_loops(rank, depth)

    def emit_argmax(self, op):
        """ArgMax over one axis. The reference hands it to tosa.argmax (MindSporeToTosa.cpp:497) with attributes that op
        does not have, so what is restated is upstream's lowering of tosa.argmax itself (LLVM 19.1.7, TosaToLinalg
        ArgMaxConverter): index 0 and the lowest finite value to start with, a later element replaces them only if
        it is greater under an ordered comparison (so the first of equal maxima wins and NaN never does)."""
        src, out = op.inputs[0], op.output
        if len(op.axes) != 1 or out.dtype not in INTS or src.dtype == "bool":
            raise OracleError("ArgMax: one axis, an integer result and a non-bool operand are required")
        axis = op.axes[0]
        in_shape = src.shape
        par = [d for d in range(len(in_shape)) if d != axis]
        sd = src.dtype
        if sd in FLOATS:
            big = {"float16": 65504.0, "bfloat16": 3.3895313892515355e38, "float32": 3.4028234663852886e38,
                   "float64": 1.7976931348623157e308}[sd]
            lowest = float_literal(sd, -big)
        else:
            lo = INT_RANGE[sd][0]
            lowest = "INT64_MIN" if sd == "int64" else ("INT32_MIN" if lo <= -2147483648 else "%d" % lo)
        depth = 1
        for k, d in enumerate(par):
            self.emit("for (int64_t i%d = 0; i%d < %dL; ++i%d) {" % (d, d, in_shape[d], d), depth + k)
        depth += len(par)
        self.emit("{", depth)
        self.emit("%s best = %s;" % (C_COMPUTE[sd], lowest), depth + 1)
        self.emit("int64_t where = 0;", depth + 1)
        self.emit("for (int64_t i%d = 0; i%d < %dL; ++i%d) {" % (axis, axis, in_shape[axis], axis), depth + 1)
        x = self.value_expr(src, in_shape)
        self.emit("const %s v = %s;" % (C_COMPUTE[sd], x), depth + 2)
        self.emit("if (v > best) { best = v; where = i%d; }" % axis, depth + 2)
        self.emit("}", depth + 1)
        expr = None
        for d in par:
            expr = "i%d" % d if expr is None else "(%s) * %dL + i%d" % (expr, in_shape[d], d)
        self.emit("%s[%s] = (%s)where;" % (out.buffer, expr or "0", C_STORAGE[out.dtype]), depth + 1)
        self.emit("}", depth)
        for k in range(len(par)):
            self.emit("}", depth - 1 - k)

    def emit_reduce(self, op):
        src, out = op.inputs[0], op.output
        od = out.dtype
        ct = C_COMPUTE[od]
        in_shape = src.shape
        axes = op.axes
        par = [d for d in range(len(in_shape)) if d not in axes]
        if od in FLOATS:
            big = {"float16": 65504.0, "bfloat16": 3.3895313892515355e38, "float32": 3.4028234663852886e38,
                   "float64": 1.7976931348623157e308}[od]
            inits = {"ReduceSum": float_literal(od, 0.0), "ReducePrd": float_literal(od, 1.0),
                     "ReduceMax": float_literal(od, -big), "ReduceMin": float_literal(od, big)}
        elif od in INTS:
            lo, hi = INT_RANGE[od]
            lo_lit = "INT64_MIN" if od == "int64" else "%d" % lo if lo > -2147483648 else "INT32_MIN"
            hi_lit = "INT64_MAX" if od == "int64" else "%d" % hi
            inits = {"ReduceSum": "0", "ReducePrd": "1", "ReduceMax": lo_lit, "ReduceMin": hi_lit}
        else:
            inits = {"ReduceAll": "1", "ReduceAny": "0"}
        if op.name not in inits:
            raise OracleError("%s on %s is not supported" % (op.name, od))
        # loops over the kept dims (in order), then over the reduced dims (in order): per output element the
        # reduced indices are visited in increasing order, as in the loop nest linalg produces.
        order = par + axes
        depth = 1
        if par and self.openmp:
            self.emit("#pragma omp parallel for schedule(static)", depth)
        for k, d in enumerate(par):
            self.emit("for (int64_t i%d = 0; i%d < %dL; ++i%d) {" % (d, d, in_shape[d], d), depth + k)
        depth += len(par)
        if not par:
            self.emit("{", depth)  # a reduction over every axis: its accumulator gets a scope of its own
            depth += 1
        self.emit("%s acc = %s;" % (ct, inits[op.name]), depth)
        for k, d in enumerate(axes):
            self.emit("for (int64_t i%d = 0; i%d < %dL; ++i%d) {" % (d, d, in_shape[d], d), depth + k)
        inner = depth + len(axes)
        x = self.value_expr(src, in_shape)
        suffix = "" if od == "float64" else "f"
        if op.name == "ReduceSum":
            step = self.rnd(od, "(acc + %s)" % x) if od in FLOATS else self.rnd(od, "((%s)((uint64_t)acc + (uint64_t)%s))" % (ct, x))
        elif op.name == "ReducePrd":
            step = self.rnd(od, "(acc * %s)" % x) if od in FLOATS else self.rnd(od, "((%s)((uint64_t)acc * (uint64_t)%s))" % (ct, x))
        elif op.name == "ReduceMax":
            step = "fmax%s(acc, %s)" % (suffix, x) if od in FLOATS else "(acc > %s ? acc : %s)" % (x, x)
        elif op.name == "ReduceMin":
            step = "fmin%s(acc, %s)" % (suffix, x) if od in FLOATS else "(acc < %s ? acc : %s)" % (x, x)
        elif op.name == "ReduceAll":
            step = "(acc && (%s != 0))" % x
        else:
            step = "(acc || (%s != 0))" % x
        self.emit("acc = %s;" % step, inner)
        for k in range(len(axes)):
            self.emit("}", inner - 1 - k)
        # linear index of the output: kept dims in order (keep_dims only inserts 1s)
        expr = None
        for d in par:
            expr = "i%d" % d if expr is None else "(%s) * %dL + i%d" % (expr, in_shape[d], d)
        self.emit("%s[%s] = %s;" % (out.buffer, expr or "0", self.store_expr(od, "acc")), depth)
        if not par:
            self.emit("}", depth - 1)
        for k in range(len(par)):
            self.emit("}", depth - 1 - k)
        _ = order

    def emit_matmul(self, op):
        a, b, out = op.inputs[0], op.inputs[1], op.output
        if op.attrs.get("transpose_a", False):
            raise OracleError("TransposeA is not supported (MindSporeToLinalg.cpp:1508-1510)")
        tb = bool(op.attrs.get("transpose_b", False))
        if len(a.shape) not in (2, 3) or len(b.shape) != len(a.shape):
            raise OracleError("MatMul operands must both be rank 2, or both rank 3 with one batch dimension")
        # BatchMatMul (linalg.batch_matmul, MindSporeToLinalg.cpp:1511-1530): the same loop nest per batch index
        batch = a.shape[0] if len(a.shape) == 3 else 1
        if len(a.shape) == 3 and b.shape[0] != batch:
            raise OracleError("batch extents differ")
        m, k = a.shape[-2], a.shape[-1]
        n = b.shape[-2] if tb else b.shape[-1]
        od = out.dtype
        ct = C_COMPUTE[od]
        ra, rb = self.root(a), self.root(b)
        aidx = "(bt * %dL + i) * %dL + k" % (m, k)
        bidx = ("(bt * %dL + j) * %dL + k" % (n, k)) if tb else ("(bt * %dL + k) * %dL + j" % (k, n))
        prod = "(%s)%s * (%s)%s" % (ct, self.load_expr(ra, aidx), ct, self.load_expr(rb, bidx))
        cidx = "(bt * %dL + i) * %dL + j" % (m, n)
        # zero-filled accumulator of the output type
        self.emit("memset(%s, 0, sizeof(%s) * %dL);" % (out.buffer, C_STORAGE[od], batch * m * n))
        self.emit("for (int64_t bt = 0; bt < %dL; ++bt) {" % batch)
        if self.openmp:
            self.emit("#pragma omp parallel for schedule(static)", 2)
        self.emit("for (int64_t i = 0; i < %dL; ++i) {" % m, 2)
        if self.matmul_order == "ijk":
            self.emit("for (int64_t j = 0; j < %dL; ++j) {" % n, 3)
            self.emit("for (int64_t k = 0; k < %dL; ++k) {" % k, 4)
        else:
            self.emit("for (int64_t k = 0; k < %dL; ++k) {" % k, 3)
            self.emit("for (int64_t j = 0; j < %dL; ++j) {" % n, 4)
        if od in INTS:
            ut = "uint64_t" if od == "int64" else "uint32_t"
            self.emit("%s[%s] = (%s)((%s)%s[%s] + (%s)(%s));" % (out.buffer, cidx, C_STORAGE[od], ut, out.buffer, cidx, ut, prod), 5)
        elif od in ("float16", "bfloat16"):
            # linalg.matmul casts both operands to the accumulator's element type, multiplies and adds in it: a product
            # rounded to the 16-bit type, then a sum rounded to it, every step (the accumulator lives in the result buffer)
            step = self.rnd(od, "(%s + %s)" % (self.load_expr(out, cidx), self.rnd(od, "(%s)" % prod)))
            self.emit("%s[%s] = %s;" % (out.buffer, cidx, self.store_expr(od, step)), 5)
        else:
            self.emit("%s[%s] = %s[%s] + %s;" % (out.buffer, cidx, out.buffer, cidx, prod), 5)
        self.emit("}", 4)
        self.emit("}", 3)
        self.emit("}", 2)
        self.emit("}")

    def generate(self):
        self.plan()
        L = self.lines
        L.append("/* Generated by oracle/gen_cpu.py from op description %s. TEST INFRASTRUCTURE (CPU oracle). */" % self.name)
        L.append(PRELUDE)
        L.append("void %s(void **packed) {" % self.name)
        arg = 0
        for t in self.inputs:
            t.buffer = "in%d" % arg
            self.emit("const %s *%s = (const %s *)packed[%d];" % (C_STORAGE[t.dtype], t.buffer, C_STORAGE[t.dtype], arg))
            arg += 1
        copies = []  # a value listed more than once among the outputs: the later listings are copies of the first
        for k, t in enumerate(self.outputs):
            if t in self.outputs[:k]:
                self.emit("%s *dup%d = (%s *)packed[%d];" % (C_STORAGE[t.dtype], k, C_STORAGE[t.dtype], arg))
                copies.append((k, t))
            else:
                t.buffer = "out%d" % k
                self.emit("%s *%s = (%s *)packed[%d];" % (C_STORAGE[t.dtype], t.buffer, C_STORAGE[t.dtype], arg))
            arg += 1
        for op in self.ops:
            out = op.output
            if op.name == "Reshape":
                src = self.root(out)
                if src.numel != out.numel:
                    raise OracleError("Reshape changes the element count")
                if out.is_output:
                    # a reshaped graph output is a copy of its source
                    self.emit("memcpy(%s, %s, sizeof(%s) * %dL);" % (out.buffer, src.buffer, C_STORAGE[out.dtype], out.numel))
                    out.alias_of = None
                continue
            if getattr(out, "inline", False):
                continue
            if out.buffer is None:
                out.buffer = "tmp_%s" % out.name
                self.temps.append(out.buffer)
                self.emit("%s *%s = (%s *)malloc(sizeof(%s) * %dL);" % (C_STORAGE[out.dtype], out.buffer, C_STORAGE[out.dtype],
                                                                       C_STORAGE[out.dtype], max(1, out.numel)))
            self.emit("/* %s -> %s */" % (op.name, out.name))
            if op.name in REDUCES:
                self.emit_reduce(op)
            elif op.name == "ArgMax":
                self.emit_argmax(op)
            elif op.name in MATMULS:
                self.emit_matmul(op)
            elif op.name in VIEW_OPS:
                self.emit_view(op)
            elif op.name in ASSIGNS:
                self.emit_assign(op)
            elif op.name in SEGMENTS:
                self.emit_segment_sum(op)
            else:
                self.emit_elementwise(op)
        for k, t in copies:
            self.emit("memcpy(dup%d, %s, sizeof(%s) * %dL);" % (k, t.buffer, C_STORAGE[t.dtype], max(1, t.numel)))
        for b in self.temps:
            self.emit("free(%s);" % b)
        L.append("}")
        return "\n".join(L) + "\n"


def generate_c(desc, openmp=False, matmul_order="ijk"):
    return Emitter(desc, openmp=openmp, matmul_order=matmul_order).generate()


def build(info_path, out_dir, openmp=False, matmul_order="ijk", cc="gcc"):
    """Compile the restatement of one description to `<out_dir>/<op>[_omp].so`; returns (path, op name)."""
    with open(info_path, "r", encoding="utf-8") as f:
        desc = json.load(f)
    src = generate_c(desc, openmp=openmp, matmul_order=matmul_order)
    os.makedirs(out_dir, exist_ok=True)
    stem = desc["op"] + ("_omp" if openmp else "") + ("" if matmul_order == "ijk" else "_" + matmul_order)
    c_path = os.path.join(out_dir, stem + ".c")
    so_path = os.path.join(out_dir, stem + ".so")
    with open(c_path, "w", encoding="utf-8") as f:
        f.write(src)
    # Scalar code like the reference's llc output (no loop vectoriser there); no contraction, no fast-math.
    cmd = [cc, "-O3", "-fno-tree-vectorize", "-fno-unroll-loops", "-ffp-contract=off", "-fno-fast-math", "-fPIC", "-shared",
           "-o", so_path, c_path, "-lm"]
    if openmp:
        cmd.insert(1, "-fopenmp")
    subprocess.run(cmd, check=True)
    return so_path, desc["op"]


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("info", nargs="+")
    ap.add_argument("-o", "--out-dir", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "_build"))
    ap.add_argument("--openmp", action="store_true")
    ap.add_argument("--matmul-order", default="ijk", choices=["ijk", "ikj"])
    ap.add_argument("--emit-only", action="store_true", help="print the C source instead of compiling")
    args = ap.parse_args()
    for path in args.info:
        if args.emit_only:
            with open(path, "r", encoding="utf-8") as f:
                sys.stdout.write(generate_c(json.load(f), args.openmp, args.matmul_order))
        else:
            so, _ = build(path, args.out_dir, args.openmp, args.matmul_order)
            print(so)


if __name__ == "__main__":
    main()
