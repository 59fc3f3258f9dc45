"""TEST INFRASTRUCTURE - CPU oracle, part 2: op-by-op numpy restatement of the same semantics.

This is the checker, not the product: only tests, the smoke check and the CPU-baseline leg of the benchmark may import
it. It evaluates a MindSpore graph-kernel JSON description one op at a time with numpy, every op in its declared
result element type, and is deliberately written independently of oracle/gen_cpu.py (different language, no fusion,
vectorised) so that the two can be checked against each other.

Rules restated (reference file:line):
  * op vocabulary and reading rules of the description: TranslateToMindsporeDialect.cpp:295-415,417-486,793-808,1273-1360
  * elementwise ops in the result type; Cast = tosa.cast: MindSporeToTosa.cpp:475-504
  * reductions: init value and combiner, accumulation in the result type, increasing index order:
    MindSporeToLinalg.cpp:791-901,1333-1451
  * MatMul accumulates in the output type from zero: MindSporeToLinalg.cpp:1453-1546
  * numpy spelling of the expected values in the reference harness: python/akg_mlir/utils/op_dsl.py:126-168,295-327,747-809
    (two of its rules are NOT followed because they contradict the compiled pipeline: `astype` truncation for
    float->int casts, and int8 products without widening)

bfloat16 tensors are numpy uint16 arrays holding the bit patterns; internally they are float32 arrays whose values are
bfloat16-representable.
"""
import json

import numpy as np

from oracle.view_attrs import VIEW_OPS, view_params, expand_split

FLOATS = ("float16", "bfloat16", "float32", "float64")
NP_DTYPE = {"bool": np.bool_, "int8": np.int8, "int16": np.int16, "int32": np.int32, "int64": np.int64,
            "float16": np.float16, "bfloat16": np.float32, "float32": np.float32, "float64": np.float64}
ATTR_AS_INPUT = ("Reshape", "BroadcastTo", "ReduceMax", "ReduceMin", "ReduceSum", "ReducePrd", "ReduceAll", "ReduceAny",
                 "ArgMax", "Transpose", "Tile")
LARGEST = {"float16": 65504.0, "bfloat16": 3.3895313892515355e38, "float32": 3.4028234663852886e38,
           "float64": 1.7976931348623157e308}


# ---------------------------------------------------------------------------------------------------------
# bfloat16 <-> float32 (round to nearest even, arith.truncf)
# ---------------------------------------------------------------------------------------------------------
def bf16_bits_to_f32(bits):
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = (u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16
    out = rounded.astype(np.uint16)
    if np.any(nan):
        out = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), out)
    return out


def round_to_bf16(x):
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


def canon_dtype(name):
    if name in ("uint8", "sint8"):
        return "int8"
    if name == "int1":
        return "bool"
    if name not in NP_DTYPE:
        raise ValueError("data type %s is not supported" % name)
    return name


def to_internal(arr, dtype):
    """External array (bf16 as uint16 bits) -> internal array."""
    if dtype == "bfloat16":
        return bf16_bits_to_f32(arr)
    return np.asarray(arr, dtype=NP_DTYPE[dtype])


def to_external(arr, dtype):
    if dtype == "bfloat16":
        return f32_to_bf16_bits(arr)
    return np.ascontiguousarray(arr, dtype=NP_DTYPE[dtype])


def finish(x, dtype):
    """Round a freshly computed array to the declared result type."""
    if dtype == "bfloat16":
        return round_to_bf16(np.asarray(x, dtype=np.float32))
    return np.asarray(x).astype(NP_DTYPE[dtype], copy=False)


def compute_view(x, dtype):
    """Array to do arithmetic on: float16 computes in float32 and is rounded once per op."""
    if dtype == "float16":
        return x.astype(np.float32)
    return x


def cast(x, src, dst):
    """tosa.cast."""
    if dst == "bool":
        return x != 0
    if dst in FLOATS:
        if src == "bool":
            x = x.astype(np.float32)
        if dst == "bfloat16":
            return round_to_bf16(x.astype(np.float32))
        return x.astype(NP_DTYPE[dst])
    info = np.iinfo(NP_DTYPE[dst])
    if src in FLOATS:
        r = np.rint(x.astype(np.float64))            # round half to even
        r = np.where(np.isnan(r), 0.0, r)
        r = np.clip(r, float(info.min), float(info.max))
        if dst == "int64":
            r = np.where(r >= 9.223372036854775807e18, np.nextafter(9.223372036854775807e18, 0), r)
        return r.astype(NP_DTYPE[dst])
    if src == "bool":
        return x.astype(NP_DTYPE[dst])
    return np.clip(x.astype(np.int64), info.min, info.max).astype(NP_DTYPE[dst])   # saturating narrowing


def maximum_nan(a, b):
    """arith.maximumf: NaN propagates (numpy's maximum does that too) and -0 is less than +0 (numpy returns either)."""
    r = np.maximum(a, b)
    if np.asarray(r).dtype.kind != "f":
        return r
    zeros = (np.asarray(a) == 0) & (np.asarray(b) == 0)
    return np.where(zeros, np.where(np.signbit(a) & np.signbit(b), -0.0, 0.0).astype(r.dtype), r)


def minimum_nan(a, b):
    """arith.minimumf: NaN propagates, -0 is less than +0."""
    r = np.minimum(a, b)
    if np.asarray(r).dtype.kind != "f":
        return r
    zeros = (np.asarray(a) == 0) & (np.asarray(b) == 0)
    return np.where(zeros, np.where(np.signbit(a) | np.signbit(b), -0.0, 0.0).astype(r.dtype), r)


def serial_reduce(x, axes, combine, init, dtype, keep_dims):
    """Reduce `axes` of x visiting the reduced indices in increasing order, rounding to `dtype` after every step."""
    rank = x.ndim
    kept = [d for d in range(rank) if d not in axes]
    xt = np.transpose(x, kept + list(axes))
    kept_shape = [x.shape[d] for d in kept]
    xt = xt.reshape(kept_shape + [-1])
    acc = np.full(kept_shape, init, dtype=xt.dtype)
    for k in range(xt.shape[-1]):
        acc = finish(combine(compute_view(acc, dtype), compute_view(xt[..., k], dtype)), dtype)
    if keep_dims:
        acc = acc.reshape([1 if d in axes else x.shape[d] for d in range(rank)])
    return acc


def matmul_exact_i32(a, b):
    """int8 x int8 -> int32 with exact accumulation: float32 BLAS on K-blocks small enough that every partial sum
    is an integer below 2**24 (127*127*1024 < 2**24), summed in int64 and wrapped to int32."""
    m, k = a.shape
    n = b.shape[1]
    acc = np.zeros((m, n), dtype=np.int64)
    step = 1024
    for k0 in range(0, k, step):
        pa = a[:, k0:k0 + step].astype(np.float32)
        pb = b[k0:k0 + step, :].astype(np.float32)
        acc += (pa @ pb).astype(np.int64)
    return acc.astype(np.int32)   # two's complement wrap, as i32 accumulation would


def evaluate(desc, inputs, updates=None):
    """Evaluate the description on `inputs` (list of external arrays in input_desc order); returns the list of
    external output arrays in output_desc order. Assign / InplaceAssign overwrite a kernel input: pass a dict as
    `updates` to receive {input position: new external array} (the caller's arrays are left alone)."""
    if isinstance(desc, str):
        desc = json.loads(desc)
    desc = expand_split(desc)
    env = {}
    dtypes = {}
    shapes = {}
    if len(inputs) != len(desc["input_desc"]):
        raise ValueError("expected %d inputs" % len(desc["input_desc"]))
    for entry, arr in zip(desc["input_desc"], inputs):
        d = entry[0]
        dt = canon_dtype(d["data_type"])
        shape = d.get("shape", [1])
        env[d["tensor_name"]] = to_internal(arr, dt).reshape(shape)
        dtypes[d["tensor_name"]] = dt
    for od in desc["op_desc"]:
        name = od["name"]
        if name == "ElemAny":  # same mindspore op as ReduceAny (TranslateToMindsporeDialect.cpp:463)
            name = "ReduceAny"
        attrs = {a["name"]: a["value"] for a in (od.get("attr") or [])}
        ins, in_dt = [], []
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
            if name in ("Assign", "InplaceAssign") and idx > 1:
                continue
            if name == "UnsortedSegmentSum" and idx > 1:
                continue
            d = entry[0]
            tn = d["tensor_name"]
            if tn not in env:
                v = d["value"]
                dt = canon_dtype(d["data_type"])
                if isinstance(v, list):
                    v = v[0]
                if dt not in FLOATS and dt != "bool":
                    v = int(v)
                c = np.array([v]).astype(np.float32 if dt == "bfloat16" else NP_DTYPE[dt])
                env[tn] = finish(c, dt) if dt in FLOATS else c
                dtypes[tn] = dt
            ins.append(env[tn])
            in_dt.append(dtypes[tn])
        o = od["output_desc"][0]
        odt = canon_dtype(o["data_type"])
        oshape = o.get("shape", [1])
        cv = [compute_view(x, dt) for x, dt in zip(ins, in_dt)]

        def same(x, dt=odt):
            # operands of arithmetic ops are converted to the result's compute type if they differ
            target = np.float32 if dt in ("float16", "bfloat16") else NP_DTYPE[dt]
            return x.astype(target, copy=False)

        with np.errstate(all="ignore"):
            if name in ("Add", "Sub", "Mul"):
                f = {"Add": np.add, "Sub": np.subtract, "Mul": np.multiply}[name]
                res = f(same(cv[0]), same(cv[1]))
            elif name in ("Div", "RealDiv"):
                if odt in FLOATS:
                    res = same(cv[0]) / same(cv[1])
                else:
                    a, b = same(cv[0]).astype(np.int64), same(cv[1]).astype(np.int64)
                    q = np.where(b == 0, 0, np.trunc(a / np.where(b == 0, 1, b))).astype(np.int64)
                    res = q
            elif name == "Maximum":
                res = maximum_nan(same(cv[0]), same(cv[1]))
            elif name == "Minimum":
                res = minimum_nan(same(cv[0]), same(cv[1]))
            elif name == "Neg":
                res = -same(cv[0])
            elif name == "Abs":
                res = np.abs(same(cv[0]))
            elif name == "Square":
                res = same(cv[0]) * same(cv[0])
            elif name == "Exp":
                res = np.exp(same(cv[0]))
            elif name == "Log":
                res = np.log(same(cv[0]))
            elif name == "Tanh":
                res = np.tanh(same(cv[0]))
            elif name == "Sqrt":
                res = np.sqrt(same(cv[0]))
            elif name == "Rsqrt":
                x = same(cv[0])
                res = x.dtype.type(1) / np.sqrt(x)
            elif name == "Reciprocal":
                x = same(cv[0])
                res = x.dtype.type(1) / x
            elif name == "Floor":
                res = np.floor(same(cv[0]))
            elif name in ("Sin", "Cos", "ASin", "ACos", "Atan"):
                f = {"Sin": np.sin, "Cos": np.cos, "ASin": np.arcsin, "ACos": np.arccos, "Atan": np.arctan}[name]
                res = f(same(cv[0]))
            elif name in ("Asinh", "Acosh"):
                # createAsinhOp / createAcoshOp (MindSporeToLinalg.cpp:156-180): log(x + sqrt(1 + x*x)) and
                # log(x + sqrt(x*x - 1)) spelled as single ops of the result type, not the libm functions
                x = same(cv[0])
                step = lambda v: compute_view(finish(v, odt), odt)
                sq = step(x * x)
                inner = step(x.dtype.type(1) + sq) if name == "Asinh" else step(sq - x.dtype.type(1))
                res = np.log(step(x + step(np.sqrt(inner))))
            elif name == "Pow":
                res = np.power(same(cv[0]), same(cv[1]))
            elif name == "Atan2":
                res = np.arctan2(same(cv[0]), same(cv[1]))
            elif name in ("Equal", "NotEqual", "Greater", "GreaterEqual", "Less", "LessEqual"):
                f = {"Equal": np.equal, "NotEqual": np.not_equal, "Greater": np.greater,
                     "GreaterEqual": np.greater_equal, "Less": np.less, "LessEqual": np.less_equal}[name]
                res = f(cv[0], cv[1])
            elif name == "IsNan":
                res = np.isnan(cv[0])
            elif name == "IsInf":
                res = np.isinf(cv[0])
            elif name == "IsFinite":
                res = np.isfinite(cv[0])
            elif name == "LogicalNot":
                res = np.logical_not(cv[0] != 0)
            elif name == "LogicalAnd":
                res = np.logical_and(cv[0] != 0, cv[1] != 0)
            elif name == "LogicalOr":
                res = np.logical_or(cv[0] != 0, cv[1] != 0)
            elif name == "Select":
                res = np.where(cv[0] != 0, same(cv[1]), same(cv[2]))
            elif name == "AddN":
                res = same(cv[0])
                for x in cv[1:]:
                    res = compute_view(finish(res + same(x), odt), odt)
            elif name == "Cast":
                res = cast(ins[0], in_dt[0], odt)
            elif name == "Reshape":
                res = ins[0].reshape(oshape)
            elif name == "BroadcastTo":
                res = np.broadcast_to(ins[0], oshape)
            elif name == "ArgMax":
                # upstream tosa.argmax lowering (LLVM 19.1.7): start at index 0 with the lowest finite value, a later
                # element wins only if it is greater (ordered comparison: never a NaN, never an equal one)
                axes = od["input_desc"][1][0]["value"] if len(od["input_desc"]) == 2 else attrs["axis"]
                axes = axes if isinstance(axes, list) else [axes]
                assert len(axes) == 1, "ArgMax: one axis"
                axis = axes[0] + ins[0].ndim if axes[0] < 0 else axes[0]
                x = np.moveaxis(cv[0], axis, -1)
                if in_dt[0] in FLOATS:
                    best = np.full(x.shape[:-1], -LARGEST[in_dt[0]], dtype=x.dtype)
                else:
                    best = np.full(x.shape[:-1], np.iinfo(x.dtype).min, dtype=x.dtype)
                where = np.zeros(x.shape[:-1], dtype=np.int64)
                for k in range(x.shape[-1]):
                    v = x[..., k]
                    hit = v > best
                    best = np.where(hit, v, best)
                    where = np.where(hit, k, where)
                res = where.reshape(oshape)
            elif name in ("ReduceSum", "ReduceMax", "ReduceMin", "ReducePrd", "ReduceAll", "ReduceAny"):
                if len(od["input_desc"]) == 2:
                    axes = od["input_desc"][1][0]["value"]
                else:
                    axes = attrs["axis"]
                if not isinstance(axes, list):
                    axes = [axes]
                if not axes:
                    axes = [1]
                rank = ins[0].ndim
                axes = sorted(set(a + rank if a < 0 else a for a in axes))
                keep = bool(attrs.get("keep_dims", False))
                x = ins[0]
                if name in ("ReduceSum", "ReducePrd"):
                    comb = np.add if name == "ReduceSum" else np.multiply
                    init = 0 if name == "ReduceSum" else 1
                    res = serial_reduce(x, axes, comb, init, odt, keep)
                elif name in ("ReduceMax", "ReduceMin"):
                    # maxnumf / minnumf are associative and ignore NaN: order does not matter
                    f = np.fmax if name == "ReduceMax" else np.fmin
                    if odt in FLOATS:
                        init = -LARGEST[odt] if name == "ReduceMax" else LARGEST[odt]
                    else:
                        info = np.iinfo(NP_DTYPE[odt])
                        init = info.min if name == "ReduceMax" else info.max
                    res = f.reduce(x, axis=tuple(axes), keepdims=keep)
                    res = f(res, np.asarray(init, dtype=res.dtype))
                else:
                    f = np.logical_and if name == "ReduceAll" else np.logical_or
                    res = f.reduce(x != 0, axis=tuple(axes), keepdims=keep)
            elif name in VIEW_OPS:
                x = ins[0]
                vp = view_params(od, list(x.shape))
                if name == "Transpose":
                    res = np.transpose(x, vp["perm"])
                elif name == "Tile":
                    res = np.tile(x, vp["multiples"])
                elif name in ("Slice", "StridedSlice"):
                    res = x[tuple(slice(b, b + n * st, st) for b, n, st in zip(vp["begin"], vp["size"], vp["strides"]))]
                elif name == "Pad":
                    fill = np.asarray(vp["value"]).astype(x.dtype)
                    res = np.pad(x, list(zip(vp["low"], vp["high"])), mode="constant", constant_values=fill)
                elif name == "Gather":
                    res = np.take(x, ins[1].astype(np.int64), axis=vp["axis"], mode="clip")
                else:
                    res = np.concatenate([x, ins[1]], axis=vp["axis"])
                res = np.ascontiguousarray(res)
            elif name == "UnsortedSegmentSum":
                # serial loop over the collapsed index positions, accumulating in the result's type
                # (MindSporeToLinalg.cpp:596-745); ids outside [0, segments) are dropped
                ids_flat = np.asarray(ins[1]).astype(np.int64).reshape(-1)
                rows = cv[0].reshape(ids_flat.size, -1)
                segments = int(np.prod(oshape)) // max(1, rows.shape[1])
                res = np.zeros((segments, rows.shape[1]), dtype=rows.dtype)
                if odt in ("float16", "bfloat16", "int8", "int16"):
                    for i, sid in enumerate(ids_flat):     # rounds after every addition
                        if 0 <= sid < segments:
                            res[sid] = compute_view(finish(rows[i] + res[sid], odt), odt)
                else:
                    ok = (ids_flat >= 0) & (ids_flat < segments)
                    np.add.at(res, ids_flat[ok], rows[ok])  # unbuffered: applied in index order
                res = res.reshape(oshape)
            elif name in ("Assign", "InplaceAssign"):
                # linalg.copy ins=input1 outs=input0 (MindSporeToLinalg.cpp:495-524)
                dst_name = od["input_desc"][0][0]["tensor_name"]
                res = np.array(ins[1]).reshape(ins[0].shape)
                env[dst_name] = res
                oshape = list(ins[0].shape)
                if updates is not None:
                    pos = [e[0]["tensor_name"] for e in desc["input_desc"]].index(dst_name)
                    updates[pos] = to_external(res, odt).reshape(ins[0].shape)
            elif name in ("MatMul", "BatchMatMul"):
                if attrs.get("transpose_a", False):
                    raise ValueError("TransposeA is not supported")
                a, b = ins[0], ins[1]
                if a.ndim == 2:
                    a, b = a[None], b[None]
                if attrs.get("transpose_b", False):
                    b = np.swapaxes(b, 1, 2)
                slices = []
                for a2, b2 in zip(a, b):      # one matrix product per batch index
                    if odt == "int32" and in_dt[0] == "int8" and in_dt[1] == "int8":
                        slices.append(matmul_exact_i32(a2, b2))
                    elif odt in ("float32", "float64"):
                        # serial k order in the output type
                        acc = np.zeros((a2.shape[0], b2.shape[1]), dtype=NP_DTYPE[odt])
                        for k in range(a2.shape[1]):
                            acc = acc + np.outer(a2[:, k].astype(acc.dtype), b2[k, :].astype(acc.dtype))
                        slices.append(acc)
                    elif odt in ("float16", "bfloat16") and in_dt[0] == odt and in_dt[1] == odt:
                        # accumulator of the 16-bit result type (MindSporeToLinalg.cpp:1453-1546): the product and the
                        # sum are each rounded to it, step by step in k order
                        rnd = lambda v: compute_view(finish(v, odt), odt)
                        acc = np.zeros((a2.shape[0], b2.shape[1]), dtype=np.float32)
                        a32, b32 = compute_view(a2, odt), compute_view(b2, odt)
                        for k in range(a2.shape[1]):
                            acc = rnd(acc + rnd(np.outer(a32[:, k], b32[k, :])))
                        slices.append(acc)
                    else:
                        raise ValueError("MatMul %s x %s -> %s is not restated" % (in_dt[0], in_dt[1], odt))
                res = np.stack(slices)
                if ins[0].ndim == 2:
                    res = res[0]
            else:
                raise ValueError("op %s is not supported by the numpy restatement" % name)
        res = finish(res, odt) if name not in ("Cast",) else res
        res = np.asarray(res)
        if res.size == int(np.prod(oshape)):
            res = res.reshape(oshape)
        else:
            res = np.broadcast_to(res, oshape)
        env[o["tensor_name"]] = res
        dtypes[o["tensor_name"]] = odt
        shapes[o["tensor_name"]] = oshape
    outs = []
    for d in desc["output_desc"]:
        tn = d["tensor_name"]
        outs.append(to_external(env[tn], dtypes[tn]).reshape(d.get("shape", [1])))
    return outs
