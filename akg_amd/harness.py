"""Harness semantics shared by the parity tests and the benchmark: seeded synthetic inputs and result comparison.

The reference harness draws unseeded N(mu, 0.1) inputs and compares with np.allclose at a per-dtype tolerance
(akg-mlir/python/akg_mlir/utils/composite_op_helper.py:833-902, gen_random.py:84-136, result_analysis.py:424-462,
benchmark.py:57-71). Here inputs are seeded (so runs are repeatable and the CPU oracle and the GPU see the same
bytes) and the tolerances are the stricter ones this backend is held to: integer / bool outputs bit-exact, float32
rtol 1e-5, float16 / bfloat16 rtol 1e-2 and atol 1e-3.
"""
import json

import numpy as np

BASE_SEED = 20260000


def f32_to_bf16_bits(x):
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    out = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    if np.any(nan):
        out = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), out)
    return out


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _as_dtype(x, dtype):
    if dtype == "bfloat16":
        return f32_to_bf16_bits(x)
    return x.astype({"float16": np.float16, "float32": np.float32, "float64": np.float64}[dtype])


def load_desc(path):
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


def pattern_of(desc):
    """Which of the five measured fusion patterns a description is, judged from its ops (None if neither)."""
    names = [o["name"] for o in desc["op_desc"]]
    if "MatMul" in names:
        return "gemm"
    if "Gather" in names:
        return "gather"
    if "ReduceMax" in names and "Exp" in names:
        return "softmax"
    if "Rsqrt" in names and "ReduceSum" in names:
        return "layernorm"
    if "ReduceMax" in names and "Abs" in names:
        return "quant"
    if not any(n.startswith("Reduce") for n in names):
        return "elementwise"
    return None


def make_inputs(desc, seed=BASE_SEED, pattern=None):
    """Seeded inputs in `input_desc` order, as host arrays (bfloat16 as uint16 bit patterns).

    elementwise: N(0,1).  softmax: N(0, sigma=2).  layernorm: x, r ~ N(0,1), gamma ~ U(0.5,1.5), beta ~ N(0,0.1).
    quant: x, r ~ N(0,1) with 0.1 % of the positions overwritten by +-50.  gemm: int8 ~ U[-127,127], float scales
    ~ U(0.001,0.02), bias ~ N(0,0.1), 16-bit float matrix operands ~ N(0, 0.25).  Anything else: N(0,1) floats, small integers."""
    rng = np.random.default_rng(seed)
    pattern = pattern or pattern_of(desc)
    specs = [(e[0]["data_type"], e[0].get("shape", [1])) for e in desc["input_desc"]]
    out = []
    for idx, (dt, shape) in enumerate(specs):
        if dt in ("int8", "uint8"):
            out.append(rng.integers(-127, 128, size=shape, dtype=np.int8))
            continue
        if dt in ("int16", "int32", "int64") and pattern == "gather":
            # positions along the gathered axis, a few of them just outside it (those are clamped)
            op = next(o for o in desc["op_desc"] if o["name"] == "Gather")
            attrs = {a["name"]: a["value"] for a in (op.get("attr") or [])}
            extent = op["input_desc"][0][0]["shape"][int(attrs.get("axis", 0))]
            out.append(rng.integers(-2, extent + 2, size=shape).astype(dt))
            continue
        if dt in ("int16", "int32", "int64") and any(o["name"] == "UnsortedSegmentSum" for o in desc["op_desc"]):
            op = next(o for o in desc["op_desc"] if o["name"] == "UnsortedSegmentSum")
            out.append(rng.integers(0, op["output_desc"][0]["shape"][0], size=shape).astype(dt))
            continue
        if dt in ("int16", "int32", "int64"):
            out.append(rng.integers(-100, 101, size=shape).astype(dt))
            continue
        if dt == "bool":
            if any(o["name"] == "ReduceAll" for o in desc["op_desc"]):
                out.append(rng.random(size=shape) < 0.999)      # mostly true, so that some results are true
            else:
                out.append(rng.integers(0, 2, size=shape).astype(np.bool_))
            continue
        if pattern == "softmax":
            x = rng.standard_normal(shape, dtype=np.float32) * 2.0
        elif pattern == "layernorm":
            if idx == 1:
                x = rng.uniform(0.5, 1.5, size=shape).astype(np.float32)
            elif idx == 2:
                x = (rng.standard_normal(shape, dtype=np.float32) * 0.1).astype(np.float32)
            else:
                x = rng.standard_normal(shape, dtype=np.float32)
        elif pattern == "quant":
            x = rng.standard_normal(shape, dtype=np.float32)
            mask = rng.random(size=shape, dtype=np.float32) < 0.001
            sign = np.where(rng.random(size=shape, dtype=np.float32) < 0.5, -50.0, 50.0).astype(np.float32)
            x = np.where(mask, sign, x)
        elif pattern == "gemm" and len(shape) == 2 and min(shape) > 1 and dt in ("float16", "bfloat16"):
            x = (rng.standard_normal(shape, dtype=np.float32) * 0.25).astype(np.float32)       # float operands
        elif pattern == "gemm":
            if len(shape) == 1 and dt != "float32":
                x = (rng.standard_normal(shape, dtype=np.float32) * 0.1).astype(np.float32)   # bias
            else:
                x = rng.uniform(0.001, 0.02, size=shape).astype(np.float32)                    # scales
        else:
            x = rng.standard_normal(shape, dtype=np.float32)
        out.append(_as_dtype(x, dt))
    return out


def to_float(arr, dtype):
    """Host array -> float64 values for comparison."""
    if dtype == "bfloat16":
        return bf16_bits_to_f32(arr).astype(np.float64)
    return np.asarray(arr).astype(np.float64)


def tolerance(dtype):
    if dtype == "float32":
        return 1e-5, 1e-8
    if dtype == "float64":
        return 1e-12, 1e-14
    if dtype in ("float16", "bfloat16"):
        return 1e-2, 1e-3
    return 0.0, 0.0


def compare(actual, expected, dtype):
    """Returns (ok, message). Integer and bool tensors must be identical; floats within the dtype's tolerance;
    NaN only where the expectation has NaN."""
    if actual.shape != expected.shape:
        return False, "shape %s != %s" % (actual.shape, expected.shape)
    if dtype in ("int8", "int16", "int32", "int64", "bool", "uint8"):
        bad = np.count_nonzero(actual != expected)
        if bad:
            idx = np.argwhere(actual != expected)[0]
            return False, "%d of %d elements differ; first at %s: %s != %s" % (
                bad, actual.size, tuple(idx), actual[tuple(idx)], expected[tuple(idx)])
        return True, "bit-exact"
    a, e = to_float(actual, dtype), to_float(expected, dtype)
    rtol, atol = tolerance(dtype)
    with np.errstate(invalid="ignore"):
        close = np.isclose(a, e, rtol=rtol, atol=atol, equal_nan=True)
    if not close.all():
        bad = np.count_nonzero(~close)
        idx = tuple(np.argwhere(~close)[0])
        return False, "%d of %d elements outside rtol=%g atol=%g; first at %s: %r vs %r" % (
            bad, a.size, rtol, atol, idx, a[idx], e[idx])
    with np.errstate(invalid="ignore", divide="ignore"):
        err = np.abs(a - e)
        rel = np.nanmax(np.where(np.abs(e) > 0, err / np.abs(e), 0.0)) if a.size else 0.0
    return True, "max abs err %.3g, max rel err %.3g" % (float(np.nanmax(err)) if a.size else 0.0, float(rel))


def compare_bits(actual, expected, dtype):
    """Returns (ok, message): the two tensors must hold the same bit patterns, whatever the element type (the bar for
    results the workload states as bit-exact, e.g. the float32 scales of the per-token quantisation)."""
    a, e = np.ascontiguousarray(actual), np.ascontiguousarray(expected)
    if a.shape != e.shape:
        return False, "shape %s != %s" % (a.shape, e.shape)
    if a.dtype.itemsize != e.dtype.itemsize:
        return False, "element size %d != %d" % (a.dtype.itemsize, e.dtype.itemsize)
    raw = np.dtype("u%d" % a.dtype.itemsize)
    ab, eb = a.view(raw), e.view(raw)
    bad = int(np.count_nonzero(ab != eb))
    if bad:
        idx = tuple(np.argwhere(ab != eb)[0])
        return False, "%d of %d %s elements differ in their bits; first at %s: %r vs %r" % (
            bad, ab.size, dtype, idx, a[idx], e[idx])
    return True, "bit-exact"


def widen_to_float64(desc):
    """The same description with every float32 tensor, cast target and constant declared float64: evaluated by the
    oracle it gives the fused expression with (nearly) exact accumulation, whatever the order of a summation."""
    text = json.dumps(desc).replace('"float32"', '"float64"')
    return json.loads(text)


def compare_reassociated(actual, exact64, dtype, terms):
    """Bar for a float32 result that went through a reduction of `terms` values in another order than the serial
    loop: rtol 1e-5 against the float64-accumulated value, plus an absolute allowance of 1e-6 * sqrt(terms) for
    sums of O(1) terms that cancel (the float32 rounding of the partial sums, which no order avoids)."""
    if dtype != "float32":
        return compare(actual, exact64, dtype)
    a, e = np.asarray(actual, dtype=np.float64), np.asarray(exact64, dtype=np.float64).reshape(np.shape(actual))
    atol = 1e-6 * float(np.sqrt(max(1, terms)))
    close = np.isclose(a, e, rtol=1e-5, atol=atol, equal_nan=True)
    if not close.all():
        idx = tuple(np.argwhere(~close)[0])
        return False, "%d of %d elements outside rtol=1e-5 atol=%g of the float64 value; first at %s: %r vs %r" % (
            np.count_nonzero(~close), a.size, atol, idx, a[idx], e[idx])
    err = np.abs(a - e)
    with np.errstate(invalid="ignore", divide="ignore"):
        rel = np.nanmax(np.where(np.abs(e) > 0, err / np.abs(e), 0.0)) if a.size else 0.0
    return True, "vs float64: max abs err %.3g, max rel err %.3g" % (float(err.max()) if a.size else 0.0, float(rel))
