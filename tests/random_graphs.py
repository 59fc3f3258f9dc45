"""Seeded random fused-op descriptions for differential tests (product kernel against the CPU oracle).

A description is grown op by op from two to four kernel inputs of broadcast-compatible shapes. Every value carries two
facts the generator respects: its value range is tame (inputs are N(0,1); Exp / Reciprocal / RealDiv get bounded
operands), and whether it is `exact`, i.e. computed only through correctly rounded operations. Ops that are
discontinuous in their operand (comparisons, Select conditions, rounding to a narrower type) are only applied to exact
values: two correct implementations may differ by an ulp after tanh or exp, and a discontinuity would turn that ulp
into a different result.
"""
import numpy as np

from akg_amd import op_desc

FLOATS = ("float32", "float16", "bfloat16")


class Val:
    def __init__(self, t, exact=True, positive=False, bounded=True):
        self.t = t
        self.exact = exact
        self.positive = positive   # values >= some margin above zero
        self.bounded = bounded     # |values| small enough for Exp


def _variant_shape(rng, base):
    """A shape that broadcasts to `base`: some extents set to 1, leading dims possibly dropped."""
    s = [d if rng.random() < 0.7 else 1 for d in base]
    drop = int(rng.integers(0, len(s)))
    if rng.random() < 0.3:
        s = s[drop:] or [1]
    return s


def random_description(seed, allow_views=True, allow_reduce=True):
    """Returns (json_text, notes). Deterministic in `seed`."""
    rng = np.random.default_rng(seed)
    rank = int(rng.integers(1, 5))
    extents = [1, 2, 3, 4, 5, 7, 8, 9, 16, 33]
    base = [int(rng.choice(extents)) for _ in range(rank)]
    if rng.random() < 0.5:
        base[-1] = int(rng.choice([8, 16, 32, 40, 64, 100]))
    dtype = str(rng.choice(FLOATS))
    b = op_desc.DescBuilder("Fused_random_%d" % seed)
    f32 = lambda v: b.cast(v.t, "float32") if v.t.dtype != "float32" else v.t  # noqa: E731

    vals = [Val(b.input(base, dtype))]
    for _ in range(int(rng.integers(1, 4))):
        vals.append(Val(b.input(_variant_shape(rng, base), dtype)))
    # compute in float32 like the measured fusions do
    work = [Val(f32(v), True) for v in vals]
    notes = []
    used_view = False

    def pick(pred=lambda v: True):
        cands = [v for v in work if pred(v)]
        return cands[int(rng.integers(0, len(cands)))] if cands else None

    n_ops = int(rng.integers(3, 10))
    for _ in range(n_ops):
        kind = rng.random()
        x = pick()
        if kind < 0.30:      # binary arithmetic with broadcasting
            y = pick()
            name = str(rng.choice(["Add", "Sub", "Mul", "Maximum", "Minimum"]))
            try:
                t = b.binary(name, x.t, y.t)
            except ValueError:
                continue
            work.append(Val(t, x.exact and y.exact, bounded=False if name == "Mul" else x.bounded and y.bounded))
            notes.append(name)
        elif kind < 0.45:    # unary, correctly rounded
            name = str(rng.choice(["Abs", "Neg", "Square"]))
            work.append(Val(b.unary(name, x.t), x.exact, bounded=x.bounded and name != "Square"))
            notes.append(name)
        elif kind < 0.58:    # transcendental on a bounded operand
            xb = pick(lambda v: v.bounded)
            if xb is None:
                continue
            clipped = b.minimum(b.maximum(xb.t, b.const(-6.0, "float32")), b.const(6.0, "float32"))
            name = str(rng.choice(["Tanh", "Exp"]))
            work.append(Val(b.unary(name, clipped), False, positive=name == "Exp", bounded=name == "Tanh"))
            notes.append(name)
        elif kind < 0.66:    # division / reciprocal / sqrt with a safe operand
            safe = b.add(b.unary("Abs", x.t), b.const(0.5, "float32"))
            name = str(rng.choice(["RealDiv", "Reciprocal", "Sqrt", "Rsqrt"]))
            if name == "RealDiv":
                y = pick()
                try:
                    t = b.binary("RealDiv", y.t, safe)
                except ValueError:
                    continue
                work.append(Val(t, x.exact and y.exact, bounded=False))
            else:
                work.append(Val(b.unary(name, safe), x.exact, positive=True, bounded=x.bounded))
            notes.append(name)
        elif kind < 0.76:    # comparison + Select on exact operands
            xe, ye = pick(lambda v: v.exact), pick(lambda v: v.exact)
            if xe is None or ye is None:
                continue
            try:
                cmp_ = b.binary(str(rng.choice(["Greater", "LessEqual", "Equal", "NotEqual"])), xe.t, ye.t, dtype="bool")
                a2, b2 = pick(), pick()
                shape = b._broadcast(b._broadcast(cmp_.shape, a2.t.shape), b2.t.shape)
            except ValueError:
                continue
            t = b.op("Select", [cmp_, a2.t, b2.t], shape, "float32")
            work.append(Val(t, a2.exact and b2.exact, bounded=a2.bounded and b2.bounded))
            notes.append("Select")
        elif kind < 0.82:    # round trip through a narrow type (a rounding step: exact operands only)
            x = pick(lambda v: v.exact)
            if x is None:
                continue
            nt = str(rng.choice(["float16", "bfloat16"]))
            work.append(Val(b.cast(b.cast(x.t, nt), "float32"), x.exact, bounded=x.bounded))
            notes.append("Cast-" + nt)
        elif allow_views and len(x.t.shape) >= 1 and kind < 1.0:
            t = x.t
            which = str(rng.choice(["Transpose", "Slice", "StridedSlice", "Pad", "Tile", "Concat", "Reshape", "Split"]))
            r = len(t.shape)
            if which == "Transpose" and r >= 2:
                t = op_desc.transpose(b, t, [int(p) for p in rng.permutation(r)])
            elif which == "Slice" and max(t.shape) >= 2:
                begin = [int(rng.integers(0, d)) for d in t.shape]
                size = [int(rng.integers(1, d - s + 1)) for d, s in zip(t.shape, begin)]
                t = op_desc.slice_(b, t, begin, size)
            elif which == "StridedSlice" and max(t.shape) >= 3:
                begin = [int(rng.integers(0, max(1, d // 2))) for d in t.shape]
                end = [int(rng.integers(s + 1, d + 1)) for d, s in zip(t.shape, begin)]
                strides = [int(rng.integers(1, 4)) for _ in t.shape]
                t = op_desc.strided_slice(b, t, begin, end, strides)
            elif which == "Pad":
                pairs = int(rng.integers(1, r + 1))
                t = op_desc.pad(b, t, [int(rng.integers(0, 4)) for _ in range(2 * pairs)], value=int(rng.integers(-3, 4)))
            elif which == "Tile" and int(np.prod(t.shape)) <= 4096:
                t = op_desc.tile(b, t, [int(rng.integers(1, 3)) for _ in t.shape])
            elif which == "Concat":
                y = pick(lambda v: v.t.shape == x.t.shape)
                t = op_desc.concat(b, t, y.t, int(rng.integers(0, r)))
                x = Val(t, x.exact and y.exact, bounded=x.bounded and y.bounded)
            elif which == "Split" and max(t.shape) >= 2:
                ax = int(rng.choice([d for d in range(r) if t.shape[d] >= 2]))
                if t.shape[ax] % 2 == 0 and rng.random() < 0.5:     # two equal pieces, both used
                    lo, hi = op_desc.split(b, t, [t.shape[ax] // 2] * 2, ax)
                    t = b.sub(lo, hi)
                else:                                               # unequal pieces, one of them used
                    cut = int(rng.integers(1, t.shape[ax]))
                    t = op_desc.split(b, t, [cut, t.shape[ax] - cut], ax)[int(rng.integers(0, 2))]
            elif which == "Reshape" and int(np.prod(t.shape)) > 1:
                n = int(np.prod(t.shape))
                divs = [d for d in range(1, n + 1) if n % d == 0]
                d0 = int(rng.choice(divs))
                t = b.reshape(t, [d0, n // d0])
            else:
                continue
            work.append(Val(t, x.exact, x.positive, x.bounded))
            used_view = True
            notes.append(which)
    out = work[-1]
    outs = [out.t]
    if allow_reduce and rng.random() < 0.5 and len(out.t.shape) >= 1:
        r = len(out.t.shape)
        pick_axes = rng.random()
        if pick_axes < 0.5:
            axis = [r - 1]
        elif pick_axes < 0.8 or r < 2:
            axis = [int(rng.integers(0, r))]
        else:   # several axes, possibly with kept ones in between ([N,C,HW] over N and HW)
            axis = sorted(int(a) for a in rng.choice(r, size=int(rng.integers(2, r + 1)), replace=False))
        name = str(rng.choice(["ReduceSum", "ReduceMax", "ReduceMin"]))
        notes.append("%s%s" % (name, axis))
        # A sum declared in the 16-bit type of the description: rounded after every step, so its steps must come in the
        # reference's serial order. Only of exactly computed values (an ulp of difference in one term would round the
        # chain differently); drawn from a generator of its own so that the other descriptions stay what they were.
        if name == "ReduceSum" and dtype != "float32" and out.exact and np.random.default_rng(seed + 7_000_000).random() < 0.6:
            out = Val(b.cast(out.t, dtype), True, out.positive, out.bounded)
            notes.append("declared-" + dtype)
        if rng.random() < 0.4 and (axis == [len(out.t.shape) - 1] or name != "ReduceSum"):
            # use the reduced value again on the elements it came from (softmax-like): the row kernel serves the last
            # axis, other axes need a kernel per pass (max / min only there: they do not depend on the order)
            outs = [b.sub(out.t, b.reduce(name, out.t, axis, True))]
            notes.append("Sub-after-reduce")
        else:
            outs = [b.reduce(name, out.t, axis, bool(rng.random() < 0.5))]
    if allow_reduce and not used_view and len(outs) == 1 and outs[0] is out.t and out.exact and out.t.shape[-1] >= 2 \
            and rng.random() < 0.15:
        # position of the greatest element of every row; only on exactly computed values (a tie broken by an ulp
        # would name another position), ties themselves are welcome: the first one wins
        notes.append("ArgMax")
        return b.dumps([op_desc.argmax(b, out.t, len(out.t.shape) - 1, bool(rng.random() < 0.5),
                                       str(rng.choice(["int32", "int64"])))]), notes
    final = []
    for t in outs:
        final.append(b.cast(t, dtype) if dtype != "float32" and rng.random() < 0.7 else t)
    return b.dumps(final), notes


def random_matmul_description(seed):
    """A MatMul in the middle of a random description: an optional Cast or Transpose in front of its first operand,
    bias and activation behind it, and optionally a softmax over the rows, column sums or a row maximum of the result,
    so that the contraction's neighbours are sometimes its epilogue and sometimes kernels of their own. 16-bit results
    (the accumulation order of the matrix units differs from the serial loop's). Returns (json_text, notes)."""
    rng = np.random.default_rng(100000 + seed)
    m = int(rng.choice([1, 7, 40, 64, 130]))
    k = int(rng.choice([32, 64, 256]))
    n = int(rng.choice([8, 136, 256]))
    dtype = str(rng.choice(["bfloat16", "float16"]))
    tb = bool(rng.integers(0, 2))
    b = op_desc.DescBuilder("Fused_random_matmul_%d" % seed)
    notes = ["%dx%dx%d" % (m, k, n), dtype]
    front = str(rng.choice(["none", "cast", "transpose"]))
    if front == "cast":
        a = b.cast(b.input([m, k], "float32"), dtype)
    elif front == "transpose":
        a = op_desc.transpose(b, b.input([k, m], dtype), [1, 0])
    else:
        a = b.input([m, k], dtype)
    notes.append("front-" + front)
    w = b.input([n, k] if tb else [k, n], dtype)
    acc = b.matmul(a, w, "float32", transpose_b=tb)
    notes.append("tb" if tb else "nt")
    y = acc
    if rng.random() < 0.7:
        y = b.add(y, b.cast(b.input([n], dtype), "float32"))
        notes.append("bias")
    act = str(rng.choice(["none", "relu", "tanh"]))
    if act == "relu":
        y = b.maximum(y, b.const(0.0, "float32"))
    elif act == "tanh":
        y = b.unary("Tanh", b.mul(y, b.const(0.125, "float32")))
    notes.append(act)
    outs = []
    tail = str(rng.choice(["none", "none", "softmax", "colsum", "rowmax"]))
    notes.append("tail-" + tail)
    if tail == "softmax":
        s = b.mul(y, b.const(1.0 / (k ** 0.5), "float32"))
        e = b.unary("Exp", b.sub(s, b.reduce("ReduceMax", s, [1], True)))
        outs.append(b.div(e, b.reduce("ReduceSum", e, [1], True)))
    elif tail == "colsum":
        outs += [y, b.mul(b.reduce("ReduceSum", y, [0], True), b.const(1.0 / m, "float32"))]
    elif tail == "rowmax":
        outs += [y, b.reduce("ReduceMax", y, [1], False)]
    else:
        outs.append(y)
    return b.dumps([b.cast(t, dtype) for t in outs]), notes


def random_int8_matmul_description(seed):
    """An int8 x int8 -> int32 MatMul (the quantised contraction): the bare int32 accumulators as an output (held to their
    bits), and / or a dequantising epilogue (per-row and per-column float32 scales, bias, activation) cast to a float
    type. Shapes cover whole and ragged MFMA tiles, skinny A, K that is not a whole number of 16-byte pieces (the
    serial kernel) and both layouts of B. Returns (json_text, notes)."""
    rng = np.random.default_rng(300000 + seed)
    m = int(rng.choice([1, 7, 40, 64, 130, 300]))
    k = int(rng.choice([32, 64, 256, 100, 1040]))
    n = int(rng.choice([8, 36, 136, 256, 520]))
    tb = bool(rng.integers(0, 2))
    b = op_desc.DescBuilder("Fused_random_int8_matmul_%d" % seed)
    notes = ["%dx%dx%d" % (m, k, n), "tb" if tb else "nt"]
    a = b.input([m, k], "int8")
    w = b.input([n, k] if tb else [k, n], "int8")
    acc = b.matmul(a, w, "int32", transpose_b=tb)
    outs = []
    shape = str(rng.choice(["bare", "dequant", "both"]))
    notes.append(shape)
    if shape in ("bare", "both"):
        outs.append(acc)
    if shape in ("dequant", "both"):
        y = b.cast(acc, "float32")
        y = b.mul(y, b.input([m, 1], "float32"))
        y = b.mul(y, b.input([n], "float32"))
        if rng.random() < 0.6:
            y = b.add(y, b.cast(b.input([n], "bfloat16"), "float32"))
            notes.append("bias")
        act = str(rng.choice(["none", "relu", "tanh"]))
        if act == "relu":
            y = b.maximum(y, b.const(0.0, "float32"))
        elif act == "tanh":
            y = b.unary("Tanh", y)
        notes.append(act)
        out_dtype = str(rng.choice(["bfloat16", "float16", "float32"]))
        notes.append(out_dtype)
        outs.append(b.cast(y, out_dtype) if out_dtype != "float32" else y)
    return b.dumps(outs), notes


def random_optable_description(seed):
    """The rows of the op table that `random_description` does not draw: Log, Sin, Cos, ASin, ACos, Atan, Asinh, Acosh,
    Floor, IsNan / IsInf / IsFinite, LogicalNot / And / Or, Pow, Atan2, AddN, GreaterEqual, Less, integer Div, a
    comparison of an integer with a float tensor, ReduceAny / ReduceAll. Same discipline as above: discontinuous ops see
    exactly computed operands only (the predicates excepted: whether Sqrt or Log of an exact value is NaN / infinite does
    not depend on the last bit), transcendental ops see operands from the part of their domain where an ulp of their
    result is an ulp of the answer. Returns (json_text, notes)."""
    rng = np.random.default_rng(500000 + seed)
    rank = int(rng.integers(1, 4))
    base = [int(rng.choice([1, 2, 3, 5, 8, 9, 33])) for _ in range(rank)]
    base[-1] = int(rng.choice([7, 16, 40, 64, 100, 257]))
    dtype = str(rng.choice(FLOATS))
    b = op_desc.DescBuilder("Fused_random_optable_%d" % seed)
    c = lambda v: b.const(float(v), "float32")  # noqa: E731
    ins = [b.input(base, dtype)] + [b.input(_variant_shape(rng, base), dtype) for _ in range(int(rng.integers(1, 3)))]
    work = [Val(b.cast(t, "float32") if dtype != "float32" else t, True) for t in ins]
    bools = []
    notes = []

    def pick(pred=lambda v: True):
        cands = [v for v in work if pred(v)]
        return cands[int(rng.integers(0, len(cands)))] if cands else None

    def clip(t, lo, hi):
        return b.minimum(b.maximum(t, c(lo)), c(hi))

    for _ in range(int(rng.integers(3, 9))):
        kind = str(rng.choice(["trig", "inverse", "hyper", "log", "pow", "atan2", "addn", "floor", "predicate", "logic",
                               "compare", "intdiv", "mixed"]))
        x = pick()
        try:
            if kind == "trig":
                name = str(rng.choice(["Sin", "Cos", "Atan"]))
                work.append(Val(b.unary(name, clip(x.t, -6.0, 6.0)), False))
            elif kind == "inverse":
                name = str(rng.choice(["ASin", "ACos"]))
                work.append(Val(b.unary(name, clip(x.t, -0.9, 0.9)), False))
            elif kind == "hyper":
                name = str(rng.choice(["Asinh", "Acosh"]))
                arg = b.add(clip(b.unary("Abs", x.t), 0.0, 40.0), c(0.5 if name == "Asinh" else 1.5))
                work.append(Val(b.unary(name, arg), False, positive=True))
            elif kind == "log":
                name = "Log"
                work.append(Val(b.unary("Log", b.add(clip(b.unary("Abs", x.t), 0.0, 40.0), c(0.5))), False))
            elif kind == "pow":
                name = "Pow"
                if rng.random() < 0.5:     # any sign of the base, a whole exponent
                    t = b.binary("Pow", clip(x.t, -2.0, 2.0), c(int(rng.choice([2, 3]))))
                else:
                    y = pick()
                    t = b.binary("Pow", b.add(clip(b.unary("Abs", x.t), 0.0, 1.5), c(0.5)), clip(y.t, -2.0, 2.0))
                work.append(Val(t, False))
            elif kind == "atan2":
                name = "Atan2"
                xe, ye = pick(lambda v: v.exact), pick(lambda v: v.exact)
                work.append(Val(b.binary("Atan2", ye.t, xe.t), False))
            elif kind == "addn":
                name = "AddN"
                terms = [pick() for _ in range(int(rng.integers(3, 5)))]
                shape = terms[0].t.shape
                for t in terms[1:]:
                    shape = b._broadcast(shape, t.t.shape)
                if any(list(t.t.shape) != list(shape) for t in terms):
                    continue     # linalg's AddN takes operands of one shape
                work.append(Val(b.op("AddN", [t.t for t in terms], shape, "float32"), all(t.exact for t in terms), bounded=False))
            elif kind == "floor":
                name = "Floor"
                xe = pick(lambda v: v.exact)
                work.append(Val(b.unary("Floor", b.mul(xe.t, c(3.0))), True))
            elif kind == "predicate":
                name = str(rng.choice(["IsNan", "IsInf", "IsFinite"]))
                xe = pick(lambda v: v.exact)
                # Sqrt of a negative value is NaN, Log of zero is -inf: both whatever the last bit of the function says
                src = b.unary("Sqrt", xe.t) if name == "IsNan" else b.unary("Log", b.maximum(xe.t, c(0.0)))
                bools.append(b.unary(name, src, "bool"))
            elif kind == "logic":
                if len(bools) < 1:
                    continue
                name = str(rng.choice(["LogicalNot", "LogicalAnd", "LogicalOr"]))
                p = bools[int(rng.integers(0, len(bools)))]
                if name == "LogicalNot":
                    bools.append(b.unary(name, p))
                else:
                    q = bools[int(rng.integers(0, len(bools)))]
                    bools.append(b.binary(name, p, q, "bool"))
            elif kind == "compare":
                name = str(rng.choice(["GreaterEqual", "Less"]))
                xe, ye = pick(lambda v: v.exact), pick(lambda v: v.exact)
                bools.append(b.binary(name, xe.t, ye.t, "bool"))
            elif kind == "intdiv":
                name = "Div"
                xe, ye = pick(lambda v: v.exact), pick(lambda v: v.exact)
                num = b.cast(b.mul(xe.t, c(100.0)), "int32")
                den = b.cast(b.mul(ye.t, c(3.0)), "int32")        # zero now and then: the agreed x / 0 = 0
                work.append(Val(b.cast(b.binary("Div", num, den, "int32"), "float32"), True, bounded=False))
            else:
                name = "Less-mixed"
                xe, ye = pick(lambda v: v.exact), pick(lambda v: v.exact)
                bools.append(b.binary("Less", b.cast(b.mul(xe.t, c(2.0)), "int32"), ye.t, "bool"))
        except ValueError:
            continue
        notes.append(name)
    outs = []
    if bools:
        p = bools[-1]
        a2, b2 = pick(), pick()
        try:
            shape = b._broadcast(b._broadcast(p.shape, a2.t.shape), b2.t.shape)
            work.append(Val(b.op("Select", [p, a2.t, b2.t], shape, "float32"), a2.exact and b2.exact))
            notes.append("Select")
        except ValueError:
            pass
        if rng.random() < 0.6 and len(p.shape) >= 1:
            name = str(rng.choice(["ReduceAny", "ElemAny", "ReduceAll"]))
            axis = [len(p.shape) - 1] if rng.random() < 0.6 else list(range(len(p.shape)))
            outs.append(b.reduce(name, p, axis, bool(rng.random() < 0.5)))
            notes.append("%s%s" % (name, axis))
        else:
            outs.append(p)
    y = work[-1].t
    outs.append(b.cast(y, dtype) if dtype != "float32" and rng.random() < 0.7 else y)
    return b.dumps(outs), notes
