"""Author MindSpore graph-kernel op descriptions (`.info` JSON) programmatically.

The document layout is the one the reference's translator reads
(akg-mlir/lib/Target/MindsporeDialect/TranslateToMindsporeDialect.cpp:55-75,295-415): top-level `op`, `process`,
`input_desc` (a list of single-element lists), `op_desc` (each with `name`, `attr`, `input_desc`, `output_desc`)
and `output_desc`. Scalar constants are op inputs of shape [1] that carry a numeric `value` (:650-658).
Only op names of the reference's op table (:417-486) are emitted.
"""
import json
import re

_IDENT = re.compile(r"^[A-Za-z_][A-Za-z0-9_]*$")


class Tensor:
    def __init__(self, name, shape, dtype, value=None):
        self.name = name
        self.shape = list(shape)
        self.dtype = dtype
        self.value = value

    def desc(self, with_value=True):
        d = {"data_type": self.dtype, "format": "DefaultFormat", "shape": list(self.shape), "tensor_name": self.name}
        if with_value and self.value is not None:
            d["value"] = self.value
        return d


class DescBuilder:
    """Builds one fused-op description; tensors are created through `input`, `const` and the op methods."""

    def __init__(self, name, process="hip", arch="gfx950"):
        if not _IDENT.match(name):
            raise ValueError("op name must be a C identifier: %r" % name)
        self.name = name
        self.process = process
        self.arch = arch
        self.inputs = []
        self.ops = []
        self._n_const = 0
        self._n_out = 0

    # -- tensors ---------------------------------------------------------------------------------------
    def input(self, shape, dtype):
        t = Tensor("input_%d" % len(self.inputs), shape, dtype)
        self.inputs.append(t)
        return t

    def const(self, value, dtype):
        self._n_const += 1
        return Tensor("const_%d" % self._n_const, [1], dtype, value=value)

    # -- generic op ------------------------------------------------------------------------------------
    def op(self, name, inputs, shape, dtype, attrs=None):
        out = Tensor("output_0_%d" % self._n_out, shape, dtype)
        self._n_out += 1
        self.ops.append({
            "attr": attrs,
            "impl_path": "",
            "input_desc": [[t.desc()] for t in inputs],
            "name": name,
            "output_desc": [out.desc(with_value=False)],
        })
        return out

    # -- shape helpers ---------------------------------------------------------------------------------
    @staticmethod
    def _broadcast(a, b):
        ra, rb = list(a)[::-1], list(b)[::-1]
        out = []
        for i in range(max(len(ra), len(rb))):
            da = ra[i] if i < len(ra) else 1
            db = rb[i] if i < len(rb) else 1
            if da != db and da != 1 and db != 1:
                raise ValueError("shapes %s and %s do not broadcast" % (a, b))
            out.append(max(da, db))
        return out[::-1]

    # -- op vocabulary used by the fused patterns ----------------------------------------------------------
    def unary(self, name, x, dtype=None):
        return self.op(name, [x], x.shape, dtype or x.dtype)

    def binary(self, name, a, b, dtype=None):
        return self.op(name, [a, b], self._broadcast(a.shape, b.shape), dtype or (a.dtype if a.value is None else b.dtype))

    def add(self, a, b):
        return self.binary("Add", a, b)

    def sub(self, a, b):
        return self.binary("Sub", a, b)

    def mul(self, a, b):
        return self.binary("Mul", a, b)

    def div(self, a, b):
        return self.binary("RealDiv", a, b)

    def maximum(self, a, b):
        return self.binary("Maximum", a, b)

    def minimum(self, a, b):
        return self.binary("Minimum", a, b)

    def cast(self, x, dtype):
        return self.op("Cast", [x], x.shape, dtype, attrs=[{"data_type": "str", "name": "dst_type", "value": dtype}])

    def reduce(self, name, x, axis, keep_dims):
        axes = [a % len(x.shape) for a in axis]
        shape = [1 if i in axes else d for i, d in enumerate(x.shape)] if keep_dims else \
                [d for i, d in enumerate(x.shape) if i not in axes]
        if not shape:
            shape = [1]
        attrs = [{"data_type": "listInt", "name": "axis", "value": list(axis)},
                 {"data_type": "bool", "name": "keep_dims", "value": bool(keep_dims)}]
        return self.op(name, [x], shape, x.dtype, attrs=attrs)

    def reshape(self, x, shape):
        return self.op("Reshape", [x], shape, x.dtype, attrs=[{"data_type": "listInt", "name": "shape", "value": list(shape)}])

    def matmul(self, a, b, dtype, transpose_b=False):
        m, k = a.shape
        n = b.shape[0] if transpose_b else b.shape[1]
        attrs = [{"data_type": "bool", "name": "transpose_a", "value": False},
                 {"data_type": "bool", "name": "transpose_b", "value": bool(transpose_b)}]
        return self.op("MatMul", [a, b], [m, n], dtype, attrs=attrs)

    # -- document --------------------------------------------------------------------------------------
    def build(self, outputs):
        return {
            "composite": True,
            "composite_graph": "akg_amd",
            "id": 0,
            "input_desc": [[t.desc()] for t in self.inputs],
            "op": self.name,
            "op_desc": self.ops,
            "output_desc": [t.desc(with_value=False) for t in outputs],
            "platform": "AKG",
            "process": self.process,
            "target_info": {"arch": self.arch},
            "version": 2,
        }

    def dumps(self, outputs):
        return json.dumps(self.build(outputs), indent=1, sort_keys=True)


# ---------------------------------------------------------------------------------------------------------
# The five fused patterns, parameterised by shape.
# ---------------------------------------------------------------------------------------------------------
def elementwise_tanh_add_mul(rows, cols, name=None):
    """out = tanh((a + b) * c), float32."""
    b = DescBuilder(name or "Fused_Add_Mul_Tanh_f32_%dx%d" % (rows, cols))
    x, y, z = (b.input([rows, cols], "float32") for _ in range(3))
    out = b.unary("Tanh", b.mul(b.add(x, y), z))
    return b.dumps([out])


def softmax_last_axis(rows, cols, dtype="float16", name=None):
    """Softmax over the last axis; internals in float32 behind explicit casts, as MindSpore emits them."""
    b = DescBuilder(name or "Fused_Cast_ReduceMax_Sub_Exp_ReduceSum_RealDiv_Cast_softmax_%s_%dx%d" % (
        {"float16": "f16", "bfloat16": "bf16", "float32": "f32"}[dtype], rows, cols))
    x = b.input([rows, cols], dtype)
    xf = b.cast(x, "float32") if dtype != "float32" else x
    mx = b.reduce("ReduceMax", xf, [1], True)
    e = b.unary("Exp", b.sub(xf, mx))
    s = b.reduce("ReduceSum", e, [1], True)
    p = b.div(e, s)
    out = b.cast(p, dtype) if dtype != "float32" else p
    return b.dumps([out])


def softmax_over_axis(shape, axis, dtype="float32", name=None):
    """Softmax over any one axis of `shape` (the channel axis of an NCHW tensor, say). Over an axis that is not the last
    one no single kernel serves it: the max, the sum and the quotient each need a pass of their own."""
    b = DescBuilder(name or "Fused_ReduceMax_Sub_Exp_ReduceSum_RealDiv_softmax_%s_%s_axis%d" % (
        _SHORT[dtype], "x".join(str(d) for d in shape), axis))
    x = b.input(list(shape), dtype)
    xf = b.cast(x, "float32") if dtype != "float32" else x
    mx = b.reduce("ReduceMax", xf, [axis], True)
    e = b.unary("Exp", b.sub(xf, mx))
    p = b.div(e, b.reduce("ReduceSum", e, [axis], True))
    return b.dumps([b.cast(p, dtype) if dtype != "float32" else p])


def batchnorm_train_forward(n, c, h, w, dtype="float32", eps=1e-5, name=None):
    """Training batch norm in one description: per-channel mean and variance of x[N,C,H,W] over N, H, W (keep_dims),
    y = (x - mean) * rsqrt(var + eps) * gamma + beta. Outputs: y, mean, variance."""
    b = DescBuilder(name or "Fused_bn_train_forward_%s_%dx%dx%dx%d" % (_SHORT[dtype], n, c, h, w))
    x = b.input([n, c, h, w], dtype)
    gamma = b.input([1, c, 1, 1], "float32")
    beta = b.input([1, c, 1, 1], "float32")
    xf = b.cast(x, "float32") if dtype != "float32" else x
    inv = b.const(1.0 / (n * h * w), "float32")
    mean = b.mul(b.reduce("ReduceSum", xf, [0, 2, 3], True), inv)
    xc = b.sub(xf, mean)
    var = b.mul(b.reduce("ReduceSum", b.mul(xc, xc), [0, 2, 3], True), inv)
    y = b.add(b.mul(b.mul(xc, b.unary("Rsqrt", b.add(var, b.const(eps, "float32")))), gamma), beta)
    return b.dumps([b.cast(y, dtype) if dtype != "float32" else y, mean, var])


def layernorm_over_axis1(outer, width, inner, dtype="bfloat16", eps=1e-5, name=None):
    """LayerNorm over the middle axis of [outer, width, inner] (channels-first activations) with gamma / beta
    [width, 1]."""
    b = DescBuilder(name or "Fused_LayerNorm_axis1_%s_%dx%dx%d" % (_SHORT[dtype], outer, width, inner))
    x = b.input([outer, width, inner], dtype)
    gamma = b.input([width, 1], dtype)
    beta = b.input([width, 1], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    xf = f(x)
    inv = b.const(1.0 / width, "float32")
    mean = b.mul(b.reduce("ReduceSum", xf, [1], True), inv)
    xc = b.sub(xf, mean)
    var = b.mul(b.reduce("ReduceSum", b.mul(xc, xc), [1], True), inv)
    y = b.add(b.mul(b.mul(xc, b.unary("Rsqrt", b.add(var, b.const(eps, "float32")))), f(gamma)), f(beta))
    return b.dumps([b.cast(y, dtype) if dtype != "float32" else y])


def layernorm_residual(rows, cols, dtype="bfloat16", eps=1e-5, name=None):
    """out = LayerNorm(x) * gamma + beta + r over the last axis, float32 internals."""
    b = DescBuilder(name or "Fused_LayerNorm_Residual_%s_%dx%d" % (
        {"float16": "f16", "bfloat16": "bf16", "float32": "f32"}[dtype], rows, cols))
    x = b.input([rows, cols], dtype)
    gamma = b.input([cols], dtype)
    beta = b.input([cols], dtype)
    r = b.input([rows, cols], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    xf, gf, bf, rf = f(x), f(gamma), f(beta), f(r)
    inv_n = b.const(1.0 / cols, "float32")
    mean = b.mul(b.reduce("ReduceSum", xf, [1], True), inv_n)
    xc = b.sub(xf, mean)
    var = b.mul(b.reduce("ReduceSum", b.mul(xc, xc), [1], True), inv_n)
    rstd = b.unary("Rsqrt", b.add(var, b.const(eps, "float32")))
    y = b.add(b.add(b.mul(b.mul(xc, rstd), gf), bf), rf)
    out = b.cast(y, dtype) if dtype != "float32" else y
    return b.dumps([out])


def rmsnorm(rows, cols, dtype="bfloat16", eps=1e-6, residual=False, name=None):
    """out = x * rsqrt(mean(x * x) + eps) * gamma over the last axis, float32 internals. With `residual` the normalised
    tensor is h = x + r (rounded to the storage type, as the next layer reads it) and h is the first output."""
    tag = {"float16": "f16", "bfloat16": "bf16", "float32": "f32"}[dtype]
    b = DescBuilder(name or "Fused_%sRMSNorm_%s_%dx%d" % ("Add_" if residual else "", tag, rows, cols))
    x = b.input([rows, cols], dtype)
    gamma = b.input([cols], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    outs = []
    if residual:
        r = b.input([rows, cols], dtype)
        h = b.add(f(x), f(r))
        h = b.cast(h, dtype) if dtype != "float32" else h
        outs.append(h)
        xf = f(h)
    else:
        xf = f(x)
    ms = b.mul(b.reduce("ReduceSum", b.mul(xf, xf), [1], True), b.const(1.0 / cols, "float32"))
    rstd = b.unary("Rsqrt", b.add(ms, b.const(eps, "float32")))
    y = b.mul(b.mul(xf, rstd), f(gamma))
    outs.append(b.cast(y, dtype) if dtype != "float32" else y)
    return b.dumps(outs)


def quant_int8_residual(rows, cols, dtype="bfloat16", name=None):
    """Per-token symmetric int8 quantisation of s = x + r: scale = absmax(s) / 127 per row,
    q = cast_int8(clamp(s / scale, -127, 127)) with the cast rounding half to even. Outputs: q, scale."""
    b = DescBuilder(name or "Fused_Add_Abs_ReduceMax_RealDiv_Cast_quant_%s_%dx%d" % (
        {"float16": "f16", "bfloat16": "bf16", "float32": "f32"}[dtype], rows, cols))
    x = b.input([rows, cols], dtype)
    r = b.input([rows, cols], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    s = b.add(f(x), f(r))
    amax = b.reduce("ReduceMax", b.unary("Abs", s), [1], False)
    scale = b.div(amax, b.const(127.0, "float32"))
    q = b.div(s, b.reshape(scale, [rows, 1]))
    q = b.minimum(b.maximum(q, b.const(-127.0, "float32")), b.const(127.0, "float32"))
    q8 = b.cast(q, "int8")
    return b.dumps([q8, scale])


def gemm_int8_dequant_bias_gelu(m, k, n, out_dtype="bfloat16", transpose_b=False, name=None):
    """out = GELU_tanh(dequant(A @ B) + bias): int8 x int8 -> int32, times per-row and per-column float32 scales,
    plus bias, GELU spelled with Mul/Add/Tanh (no Erf/Gelu in the op table)."""
    b = DescBuilder(name or "Fused_MatMul_Cast_Mul_Mul_Add_GeluTanh_Cast_i8_%dx%dx%d%s" % (
        m, k, n, "_tb" if transpose_b else ""))
    a = b.input([m, k], "int8")
    sa = b.input([m, 1], "float32")
    w = b.input([n, k] if transpose_b else [k, n], "int8")
    sb = b.input([n], "float32")
    bias = b.input([n], out_dtype)
    acc = b.matmul(a, w, "int32", transpose_b=transpose_b)
    x = b.mul(b.mul(b.cast(acc, "float32"), sa), sb)
    x = b.add(x, b.cast(bias, "float32") if out_dtype != "float32" else bias)
    x3 = b.mul(b.mul(x, x), x)
    inner = b.mul(b.add(x, b.mul(x3, b.const(0.044715, "float32"))), b.const(0.7978845608028654, "float32"))
    g = b.mul(b.mul(x, b.add(b.unary("Tanh", inner), b.const(1.0, "float32"))), b.const(0.5, "float32"))
    out = b.cast(g, out_dtype) if out_dtype != "float32" else g
    return b.dumps([out])


# ---------------------------------------------------------------------------------------------------------
# Streaming-reduction patterns (reduce direction Y and ALL, multi-output fusions).
# ---------------------------------------------------------------------------------------------------------
_SHORT = {"float16": "f16", "bfloat16": "bf16", "float32": "f32", "int32": "i32"}


def square_reduce(shape, axes, dtype="float32", keep_dims=False, op="ReduceSum", name=None):
    """out = Reduce(x * x) over `axes`, e.g. [1,5100,3072] over axis 1 (reduce direction Y) or [768,512] over
    both axes (direction ALL). 16-bit inputs are cast to float32 first and the result is cast back."""
    b = DescBuilder(name or "Fused_Mul_%s_%s_%s_axes%s" % (
        op, _SHORT[dtype], "x".join(str(d) for d in shape), "_".join(str(a) for a in axes)))
    x = b.input(list(shape), dtype)
    wide = dtype in ("float16", "bfloat16")
    v = b.cast(x, "float32") if wide else x
    r = b.reduce(op, b.mul(v, v), list(axes), keep_dims)
    return b.dumps([b.cast(r, dtype) if wide else r])


def bias_grad(rows, cols, dtype="bfloat16", name=None):
    """Gradients of `y = x * gamma + beta` for dy [rows, cols]: dgamma = sum_rows(dy * x), dbeta = sum_rows(dy),
    both [cols] float32. Two column reductions (direction Y) of one pass over dy and x."""
    b = DescBuilder(name or "Fused_Mul_ReduceSum_ReduceSum_biasgrad_%s_%dx%d" % (_SHORT[dtype], rows, cols))
    dy = b.input([rows, cols], dtype)
    x = b.input([rows, cols], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    dyf = f(dy)
    dgamma = b.reduce("ReduceSum", b.mul(dyf, f(x)), [0], False)
    dbeta = b.reduce("ReduceSum", dyf, [0], False)
    return b.dumps([dgamma, dbeta])


def batchnorm_stats(n, c, h, w, dtype="bfloat16", name=None):
    """Per-channel sum and sum of squares of x[N,C,H,W] over N, H and W (the statistics pass of a training batch norm):
    the kept axis lies between the reduced ones."""
    b = DescBuilder(name or "Fused_Cast_ReduceSum_Mul_ReduceSum_bnstats_%s_%dx%dx%dx%d" % (_SHORT[dtype], n, c, h, w))
    x = b.input([n, c, h, w], dtype)
    xf = b.cast(x, "float32") if dtype != "float32" else x
    s1 = b.reduce("ReduceSum", xf, [0, 2, 3], False)
    s2 = b.reduce("ReduceSum", b.mul(xf, xf), [0, 2, 3], False)
    return b.dumps([s1, s2])


def batchnorm_stats_update(n, c, h, w, dtype="float32", momentum=0.9, name=None):
    """Training batch norm, statistics half: per-channel mean and variance of x[N,C,H,W] over N, H, W, and the running
    statistics updated in place from them (two Assigns on [C] inputs). Outputs: mean, variance, and the two assigned
    values."""
    b = DescBuilder(name or "Fused_bnstats_update_%s_%dx%dx%dx%d" % (_SHORT[dtype], n, c, h, w))
    x = b.input([n, c, h, w], dtype)
    run_mean = b.input([c], "float32")
    run_var = b.input([c], "float32")
    xf = b.cast(x, "float32") if dtype != "float32" else x
    inv = b.const(1.0 / (n * h * w), "float32")
    mean = b.mul(b.reduce("ReduceSum", xf, [0, 2, 3], False), inv)
    sq = b.mul(b.reduce("ReduceSum", b.mul(xf, xf), [0, 2, 3], False), inv)
    var = b.sub(sq, b.mul(mean, mean))
    keep, take = b.const(momentum, "float32"), b.const(1.0 - momentum, "float32")
    new_mean = b.add(b.mul(run_mean, keep), b.mul(mean, take))
    new_var = b.add(b.mul(run_var, keep), b.mul(var, take))
    a0 = b.op("Assign", [run_mean, new_mean], [c], "float32")
    a1 = b.op("Assign", [run_var, new_var], [c], "float32")
    return b.dumps([mean, var, a0, a1])


def sub_exp_reduce_y(outer, reduced, inner, dtype="float32", name=None):
    """Two outputs, as the reference's Fused_Sub_Exp_ReduceSum_split: e = exp(x - m) (full shape, stored while
    streaming) and s = sum over the middle axis of e, with m broadcast along the reduced axis."""
    b = DescBuilder(name or "Fused_Sub_Exp_ReduceSum_split_%s_%dx%dx%d" % (_SHORT[dtype], outer, reduced, inner))
    x = b.input([outer, reduced, inner], dtype)
    m = b.input([outer, 1, inner], dtype)
    e = b.unary("Exp", b.sub(x, m))
    s = b.reduce("ReduceSum", e, [1], True)
    return b.dumps([e, s])


def mean_absmax_all(rows, cols, dtype="float32", name=None):
    """Two reductions over every axis with ops after them: mean = sum(x) / N and amax = max(|x|), both [1]."""
    b = DescBuilder(name or "Fused_ReduceSum_Abs_ReduceMax_all_%s_%dx%d" % (_SHORT[dtype], rows, cols))
    x = b.input([rows, cols], dtype)
    mean = b.mul(b.reduce("ReduceSum", x, [0, 1], False), b.const(1.0 / (rows * cols), dtype))
    amax = b.reduce("ReduceMax", b.unary("Abs", x), [0, 1], False)
    return b.dumps([mean, amax])


def gemm_bias_act(m, k, n, dtype="bfloat16", act="gelu", transpose_b=False, acc_dtype="float32", name=None):
    """out = act(A @ B + bias): `dtype` operands (bfloat16 / float16), MatMul result declared `acc_dtype`, bias
    [n] in `dtype`, activation "gelu" (tanh form, spelled with Mul/Add/Tanh), "relu" (Maximum with 0) or "none"."""
    b = DescBuilder(name or "Fused_MatMul_Add_%s_%s_%dx%dx%d%s" % (act, _SHORT[dtype], m, k, n, "_tb" if transpose_b else ""))
    a = b.input([m, k], dtype)
    w = b.input([n, k] if transpose_b else [k, n], dtype)
    bias = b.input([n], dtype)
    x = b.matmul(a, w, acc_dtype, transpose_b=transpose_b)
    if acc_dtype != "float32":
        x = b.cast(x, "float32")
    x = b.add(x, b.cast(bias, "float32"))
    if act == "gelu":
        x3 = b.mul(b.mul(x, x), x)
        inner = b.mul(b.add(x, b.mul(x3, b.const(0.044715, "float32"))), b.const(0.7978845608028654, "float32"))
        x = b.mul(b.mul(x, b.add(b.unary("Tanh", inner), b.const(1.0, "float32"))), b.const(0.5, "float32"))
    elif act == "relu":
        x = b.maximum(x, b.const(0.0, "float32"))
    return b.dumps([b.cast(x, dtype)])


# ---------------------------------------------------------------------------------------------------------
# Data-movement ops (Transpose, Tile, Slice, StridedSlice, Pad, Concat) on DescBuilder values.
# ---------------------------------------------------------------------------------------------------------
def _listint(name, value):
    return {"data_type": "listInt", "name": name, "value": [int(v) for v in value]}


def transpose(b, x, perm):
    shape = [x.shape[p] for p in perm]
    return b.op("Transpose", [x], shape, x.dtype, attrs=[_listint("perm", perm)])


def tile(b, x, multiples):
    shape = [d * m for d, m in zip(x.shape, multiples)]
    return b.op("Tile", [x], shape, x.dtype, attrs=[_listint("multiples", multiples)])


def slice_(b, x, begin, size):
    shape = [x.shape[d] - begin[d] if s == -1 else s for d, s in enumerate(size)]
    return b.op("Slice", [x], shape, x.dtype, attrs=[_listint("begin", begin), _listint("size", size)])


def strided_slice(b, x, begin, end, strides):
    e = [v + x.shape[d] if v < 0 else v for d, v in enumerate(end)]
    shape = [(e[d] - begin[d] + strides[d] - 1) // strides[d] for d in range(len(begin))]
    return b.op("StridedSlice", [x], shape, x.dtype,
                attrs=[_listint("begin", begin), _listint("end", end), _listint("strides", strides)])


def pad(b, x, padding, value=0):
    """`padding` = (before, after) pairs, the first pair for the last dimension."""
    shape = list(x.shape)
    for i in range(len(padding) // 2):
        shape[len(shape) - 1 - i] += padding[2 * i] + padding[2 * i + 1]
    return b.op("Pad", [x], shape, x.dtype, attrs=[_listint("padding", padding),
                                                   {"data_type": "int", "name": "value", "value": int(value)},
                                                   {"data_type": "str", "name": "mode", "value": "constant"}])


def concat(b, x, y, axis):
    """The operands of a Concat travel as ONE input entry holding the list of tensors (TranslateToMindsporeDialect.cpp
    :772-791), unlike every other op, where each operand is an entry of its own."""
    shape = list(x.shape)
    shape[axis] += y.shape[axis]
    out = b.op("Concat", [x, y], shape, x.dtype, attrs=[{"data_type": "int", "name": "axis", "value": int(axis)},
                                                         {"data_type": "int", "name": "inputNums", "value": 2}])
    b.ops[-1]["input_desc"] = [[x.desc(), y.desc()]]
    return out


def split(b, x, sizes, axis):
    """One Split op with len(sizes) results: consecutive pieces of `x` along `axis`."""
    outs = []
    for n in sizes:
        shape = list(x.shape)
        shape[axis] = int(n)
        outs.append(Tensor("output_0_%d" % b._n_out, shape, x.dtype))
        b._n_out += 1
    b.ops.append({
        "attr": [{"data_type": "int", "name": "output_num", "value": len(sizes)},
                 {"data_type": "listInt", "name": "size_splits", "value": [int(n) for n in sizes]},
                 {"data_type": "int", "name": "axis", "value": int(axis)}],
        "impl_path": "", "input_desc": [[x.desc()]], "name": "Split",
        "output_desc": [t.desc(with_value=False) for t in outs]})
    return outs


def split_swiglu(rows, width, dtype="bfloat16", name=None):
    """SwiGLU on a fused projection: x[rows, 2*width] is split into gate and up halves along the last axis,
    out = gate * sigmoid(gate) * up."""
    b = DescBuilder(name or "Fused_Split_SwiGLU_%s_%dx%d" % (_SHORT[dtype], rows, width))
    x = b.input([rows, 2 * width], dtype)
    gate, up = split(b, x, [width, width], 1)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    gf, uf = f(gate), f(up)
    sig = b.unary("Reciprocal", b.add(b.unary("Exp", b.unary("Neg", gf)), b.const(1.0, "float32")))
    y = b.mul(b.mul(gf, sig), uf)
    return b.dumps([b.cast(y, dtype) if dtype != "float32" else y])


def transpose_bias_add(batch, rows, cols, dtype="bfloat16", name=None):
    """out[b, c, r] = x[b, r, c] + bias[r] (bias broadcast along the new innermost axis is [rows]): the layout change
    in front of an attention score product, fused with an elementwise op."""
    b = DescBuilder(name or "Fused_Transpose_Add_%s_%dx%dx%d" % (_SHORT[dtype], batch, rows, cols))
    x = b.input([batch, rows, cols], dtype)
    bias = b.input([rows], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    y = b.add(f(transpose(b, x, [0, 2, 1])), f(bias))
    return b.dumps([b.cast(y, dtype) if dtype != "float32" else y])


def view_chain(name=None):
    """Every data-movement op once, on small ragged shapes: pad -> tile -> strided slice -> transpose, a slice of a
    second input concatenated on, then an elementwise op."""
    b = DescBuilder(name or "Fused_Pad_Tile_StridedSlice_Transpose_Slice_Concat_Mul_f32")
    x = b.input([5, 7], "float32")
    y = b.input([9, 30], "float32")
    p = pad(b, x, [1, 2, 3, 0], value=2)            # [8, 10]
    t = tile(b, p, [2, 3])                          # [16, 30]
    s = strided_slice(b, t, [1, 0], [-1, 30], [2, 1])  # [7, 30]
    tr = transpose(b, s, [1, 0])                    # [30, 7]
    ys = slice_(b, y, [2, 0], [4, -1])              # [4, 30]
    c = concat(b, tr, transpose(b, ys, [1, 0]), 1)  # [30, 11]
    return b.dumps([b.mul(c, b.const(0.5, "float32"))])


def transpose_0213_neg(shape, dtype="float16", name=None):
    """out = -transpose(x, [0, 2, 1, 3]): the innermost axis stays innermost (head / sequence swap of attention)."""
    b = DescBuilder(name or "Fused_Transpose_Neg_%s_%s" % (_SHORT[dtype], "x".join(str(d) for d in shape)))
    x = b.input(list(shape), dtype)
    return b.dumps([b.unary("Neg", transpose(b, x, [0, 2, 1, 3]))])


def slice_concat_int(name=None):
    """int32: two slices of one input concatenated in swapped order along axis 0, plus a padded second input."""
    b = DescBuilder(name or "Fused_Slice_Slice_Concat_Pad_Add_i32")
    x = b.input([12, 16], "int32")
    y = b.input([10, 12], "int32")
    top = slice_(b, x, [0, 0], [5, -1])
    bottom = slice_(b, x, [5, 0], [-1, -1])
    swapped = concat(b, bottom, top, 0)                 # [12, 16]
    return b.dumps([b.add(swapped, pad(b, y, [3, 1, 0, 2], value=-7))])


def transpose_reshape_add(name=None):
    """x [4,6,10] -> transpose [1,0,2] -> reshape [24,10] -> + y [24,10]: a Reshape between data-movement ops."""
    b = DescBuilder(name or "Fused_Transpose_Reshape_Add_f32_4x6x10")
    x = b.input([4, 6, 10], "float32")
    y = b.input([24, 10], "float32")
    t = b.reshape(transpose(b, x, [1, 0, 2]), [24, 10])
    return b.dumps([b.add(t, y)])


def transpose_sum(shape, perm, dtype="float32", name=None):
    """out = transpose(x, perm) + transpose(y, perm) * 2: two kernel inputs read through the same permutation."""
    b = DescBuilder(name or "Fused_Transpose_Transpose_Mul_Add_%s_%s_perm%s" % (
        _SHORT[dtype], "x".join(str(d) for d in shape), "".join(str(p) for p in perm)))
    x = b.input(list(shape), dtype)
    y = b.input(list(shape), dtype)
    return b.dumps([b.add(transpose(b, x, perm), b.mul(transpose(b, y, perm), b.const(2.0, dtype)))])


def batch_matmul_scale_mask(batch, m, k, n, dtype="bfloat16", transpose_b=True, name=None):
    """Attention scores: out[b] = (Q[b] @ K[b]^T) * scale + mask, Q [batch,m,k], K [batch,n,k] (transpose_b) or
    [batch,k,n], mask [batch,m,n] in float32, result in `dtype`."""
    b = DescBuilder(name or "Fused_BatchMatMul_Mul_Add_%s_%dx%dx%dx%d%s" % (_SHORT[dtype], batch, m, k, n, "_tb" if transpose_b else ""))
    q = b.input([batch, m, k], dtype)
    kk = b.input([batch, n, k] if transpose_b else [batch, k, n], dtype)
    mask = b.input([batch, m, n], "float32")
    attrs = [{"data_type": "bool", "name": "transpose_a", "value": False},
             {"data_type": "bool", "name": "transpose_b", "value": bool(transpose_b)}]
    s = b.op("BatchMatMul", [q, kk], [batch, m, n], "float32", attrs=attrs)
    s = b.add(b.mul(s, b.const(1.0 / (k ** 0.5), "float32")), mask)
    return b.dumps([b.cast(s, dtype)])


def attention_probabilities(batch, m, k, n, dtype="bfloat16", name=None):
    """softmax((Q[b] @ K[b]^T) * scale + mask) over the last axis in one description: Q [batch,m,k], K [batch,n,k],
    mask [batch,m,n] float32, probabilities in `dtype`."""
    b = DescBuilder(name or "Fused_BatchMatMul_Mul_Add_softmax_%s_%dx%dx%dx%d" % (_SHORT[dtype], batch, m, k, n))
    q = b.input([batch, m, k], dtype)
    kk = b.input([batch, n, k], dtype)
    mask = b.input([batch, m, n], "float32")
    attrs = [{"data_type": "bool", "name": "transpose_a", "value": False},
             {"data_type": "bool", "name": "transpose_b", "value": True}]
    s = b.op("BatchMatMul", [q, kk], [batch, m, n], "float32", attrs=attrs)
    s = b.add(b.mul(s, b.const(1.0 / (k ** 0.5), "float32")), mask)
    e = b.unary("Exp", b.sub(s, b.reduce("ReduceMax", s, [2], True)))
    p = b.div(e, b.reduce("ReduceSum", e, [2], True))
    return b.dumps([b.cast(p, dtype)])


def sgd_clip_by_global_norm(rows, cols, dtype="float32", lr=0.01, clip=1.0, name=None):
    """p <- p - lr * g * min(1, clip / ||g||): the norm is a reduction over the whole gradient, the update an Assign over
    the parameter. Outputs: the assigned parameter and the norm."""
    b = DescBuilder(name or "Fused_sgd_clip_global_norm_%s_%dx%d" % (_SHORT[dtype], rows, cols))
    p = b.input([rows, cols], dtype)
    g = b.input([rows, cols], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    gf = f(g)
    norm = b.unary("Sqrt", b.reduce("ReduceSum", b.mul(gf, gf), [0, 1], True))
    scale = b.minimum(b.div(b.const(clip, "float32"), b.add(norm, b.const(1e-6, "float32"))), b.const(1.0, "float32"))
    new_p = b.sub(f(p), b.mul(b.mul(gf, scale), b.const(lr, "float32")))
    new_p = b.cast(new_p, dtype) if dtype != "float32" else new_p
    a = b.op("Assign", [p, new_p], [rows, cols], dtype)
    return b.dumps([a, norm])


def transposed_a_matmul_bias_relu(m, k, n, dtype="bfloat16", name=None):
    """relu(A^T @ B + bias) with A stored [k, m]: the reference's MatMul refuses transpose_a
    (MindSporeToLinalg.cpp:1508-1510), so the description spells the transpose as an op of its own."""
    b = DescBuilder(name or "Fused_Transpose_MatMul_Add_relu_%s_%dx%dx%d" % (_SHORT[dtype], m, k, n))
    a = b.input([k, m], dtype)
    w = b.input([k, n], dtype)
    bias = b.input([n], dtype)
    acc = b.matmul(transpose(b, a, [1, 0]), w, "float32")
    y = b.maximum(b.add(acc, b.cast(bias, "float32")), b.const(0.0, "float32"))
    return b.dumps([b.cast(y, dtype)])


def gather(b, data, indices, axis):
    shape = list(data.shape[:axis]) + list(indices.shape) + list(data.shape[axis + 1:])
    return b.op("Gather", [data, indices], shape, data.dtype,
                attrs=[{"data_type": "int", "name": "axis", "value": int(axis)},
                       {"data_type": "int", "name": "batch_dims", "value": 0}])


def embedding_lookup_scale(vocab, width, batch, seq, dtype="bfloat16", name=None):
    """out[b, s, :] = table[ids[b, s], :] * scale + pos[s, :]: an embedding gather fused with its scale and the
    positional term."""
    b = DescBuilder(name or "Fused_Gather_Mul_Add_%s_%dx%d_ids%dx%d" % (_SHORT[dtype], vocab, width, batch, seq))
    table = b.input([vocab, width], dtype)
    ids = b.input([batch, seq], "int32")
    pos = b.input([seq, width], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    x = b.add(b.mul(f(gather(b, table, ids, 0)), b.const(float(width) ** 0.5, "float32")), f(pos))
    return b.dumps([b.cast(x, dtype) if dtype != "float32" else x])


def unsorted_segment_sum(index_shape, slice_shape, segments, dtype="float32", ids_dtype="int32", name=None):
    """out[ids[i...], :] += data[i..., :] over the index positions in row-major order (an embedding-table gradient, a
    graph-network aggregation). The segment count is carried as the attribute the reference's test descriptions use."""
    b = DescBuilder(name or "Fused_UnsortedSegmentSum_%s_%s_seg%d" % (
        _SHORT[dtype], "x".join(str(d) for d in list(index_shape) + list(slice_shape)), segments))
    data = b.input(list(index_shape) + list(slice_shape), dtype)
    ids = b.input(list(index_shape), ids_dtype)
    out = b.op("UnsortedSegmentSum", [data, ids], [segments] + list(slice_shape), dtype,
               attrs=[{"data_type": "int", "name": "num_segments", "value": int(segments)}])
    return b.dumps([out])


def argmax(b, x, axis, keep_dims=False, dtype="int32"):
    axis = axis % len(x.shape)
    shape = [1 if i == axis else d for i, d in enumerate(x.shape)] if keep_dims else \
            [d for i, d in enumerate(x.shape) if i != axis] or [1]
    return b.op("ArgMax", [x], shape, dtype, attrs=[{"data_type": "listInt", "name": "axis", "value": [int(axis)]},
                                                    {"data_type": "bool", "name": "keep_dims", "value": bool(keep_dims)}])


def argmax_last_axis(shape, dtype="float32", keep_dims=False, index_dtype="int32", scale=None, name=None):
    """Greedy decoding step: index of the greatest logit per row (optionally after a scale, so that an elementwise op
    is fused in front)."""
    b = DescBuilder(name or "Fused_ArgMax_%s_%s" % (_SHORT[dtype], "x".join(str(d) for d in shape)))
    x = b.input(list(shape), dtype)
    y = x
    if scale is not None:
        y = b.mul(b.cast(x, "float32") if dtype != "float32" else x, b.const(float(scale), "float32"))
    return b.dumps([argmax(b, y, len(shape) - 1, keep_dims, index_dtype)])


def any_greater(rows, cols, threshold=2.5, op="ElemAny", name=None):
    """out[r] = any(x[r, :] > threshold), spelled with `ElemAny` (the reference maps it to its ReduceAny op)."""
    b = DescBuilder(name or "Fused_Greater_%s_f32_%dx%d" % (op, rows, cols))
    x = b.input([rows, cols], "float32")
    hit = b.binary("Greater", x, b.const(threshold, "float32"), dtype="bool")
    return b.dumps([b.reduce(op, hit, [1], False)])


def momentum_update(rows, cols, dtype="float32", lr=0.01, mu=0.9, name=None):
    """SGD with momentum, in place: v <- mu * v + g (Assign), p <- p - lr * v (Assign). Kernel inputs p, v, g; the two
    Assign results are the (fake) outputs."""
    b = DescBuilder(name or "Fused_Mul_Add_Assign_Mul_Sub_Assign_%s_%dx%d" % (_SHORT[dtype], rows, cols))
    p = b.input([rows, cols], dtype)
    v = b.input([rows, cols], dtype)
    g = b.input([rows, cols], dtype)
    f = (lambda t: b.cast(t, "float32")) if dtype != "float32" else (lambda t: t)
    back = (lambda t: b.cast(t, dtype)) if dtype != "float32" else (lambda t: t)
    v_new = b.add(b.mul(f(v), b.const(mu, "float32")), f(g))
    v_out = b.op("Assign", [v, back(v_new)], [rows, cols], dtype)
    p_new = b.sub(f(p), b.mul(v_new, b.const(lr, "float32")))
    p_out = b.op("InplaceAssign", [p, back(p_new), back(v_new)], [rows, cols], dtype,
                 attrs=[{"data_type": "bool", "name": "fake_output", "value": True}])
    return b.dumps([v_out, p_out])


# ---------------------------------------------------------------------------------------------------------
# Op-table rows outside the measured fusions, grouped so that each group is one small kernel.
# ---------------------------------------------------------------------------------------------------------
def optable_unary_math(rows, cols, dtype="float32", name=None):
    """Log, Sin, Cos, ASin, ACos, Atan, Asinh, Acosh and Floor of one input, each on the part of its domain where an ulp
    of the function is an ulp of the answer; nine outputs of the input's type (computed in float32 for 16-bit inputs)."""
    b = DescBuilder(name or "Fused_optable_unary_math_%s_%dx%d" % (dtype, rows, cols))
    x = b.input([rows, cols], dtype)
    xf = b.cast(x, "float32") if dtype != "float32" else x
    c = lambda v: b.const(float(v), "float32")  # noqa: E731
    mag = b.unary("Abs", xf)
    unit = b.minimum(b.maximum(xf, c(-0.9)), c(0.9))
    outs = [b.unary("Log", b.add(mag, c(0.5))), b.unary("Sin", xf), b.unary("Cos", xf), b.unary("ASin", unit),
            b.unary("ACos", unit), b.unary("Atan", xf), b.unary("Asinh", b.add(mag, c(0.5))),
            b.unary("Acosh", b.add(mag, c(1.5))), b.unary("Floor", b.mul(xf, c(3.0)))]
    return b.dumps([b.cast(t, dtype) if dtype != "float32" else t for t in outs])


def optable_predicates_logic(rows, cols, name=None):
    """IsNan / IsInf / IsFinite on values that are NaN (Sqrt of a negative) or -inf (Log of zero) for about half of the
    elements, LogicalNot / And / Or over them, GreaterEqual and Less, and a Select steered by the result."""
    b = DescBuilder(name or "Fused_optable_predicates_logic_%dx%d" % (rows, cols))
    x = b.input([rows, cols], "float32")
    y = b.input([rows, cols], "float32")
    zero = b.const(0.0, "float32")
    nan_ = b.unary("IsNan", b.unary("Sqrt", x), "bool")
    inf_ = b.unary("IsInf", b.unary("Log", b.maximum(y, zero)), "bool")
    fin_ = b.unary("IsFinite", b.unary("Log", b.maximum(x, zero)), "bool")
    q = b.binary("LogicalAnd", b.unary("LogicalNot", nan_), b.binary("LogicalOr", inf_, fin_, "bool"), "bool")
    ge = b.binary("GreaterEqual", x, y, "bool")
    lt = b.binary("Less", x, y, "bool")
    pick = b.op("Select", [b.binary("LogicalAnd", ge, q, "bool"), x, y], [rows, cols], "float32")
    return b.dumps([q, lt, pick])


def optable_pow_atan2_addn(rows, cols, dtype="float32", name=None):
    """Pow with a positive base and with a whole exponent on a base of either sign, Atan2 over all four quadrants, AddN
    of four operands."""
    b = DescBuilder(name or "Fused_optable_pow_atan2_addn_%s_%dx%d" % (dtype, rows, cols))
    ins = [b.input([rows, cols], dtype) for _ in range(3)]
    x, y, z = [b.cast(t, "float32") if dtype != "float32" else t for t in ins]
    c = lambda v: b.const(float(v), "float32")  # noqa: E731
    clip2 = lambda t: b.minimum(b.maximum(t, c(-2.0)), c(2.0))  # noqa: E731
    outs = [b.binary("Pow", b.add(b.minimum(b.unary("Abs", x), c(1.5)), c(0.5)), clip2(y)),
            b.binary("Pow", clip2(x), c(3.0)),
            b.binary("Atan2", x, y),
            b.op("AddN", [x, y, z, x], [rows, cols], "float32")]
    return b.dumps([b.cast(t, dtype) if dtype != "float32" else t for t in outs])


def optable_int_div(rows, cols, name=None):
    """Integer Div (truncating; zero divisors occur) and a comparison of an integer with a float tensor."""
    b = DescBuilder(name or "Fused_optable_int_div_%dx%d" % (rows, cols))
    n = b.input([rows, cols], "int32")
    d = b.input([rows, cols], "int32")
    f = b.input([rows, cols], "float32")
    q = b.binary("Div", b.mul(n, b.const(37, "int32")), d, "int32")
    return b.dumps([q, b.binary("Less", d, b.mul(f, b.const(50.0, "float32")), "bool")])
