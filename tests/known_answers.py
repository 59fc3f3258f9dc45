"""Known-answer vectors at the points the numeric rules are about: ties and saturation of float -> int8, bfloat16 /
float16 rounding, a row of -inf under ReduceMax, NaN / +-inf / +-0 through the math ops, ordered comparisons, signed
integer compares and division (with the two corner values the reference leaves undefined), AddN's order, Pow / Atan2
operand order and special cases, Asinh / Acosh in the reference's spelling, the predicates and the logical ops, and a
per-token quantisation whose quotients are exact .5 ties.

Every case is (name, description text, inputs, wanted outputs, mode). The wanted values come from IEEE-754 tables, Python's
`math` and exact arithmetic, not from the oracle: the CPU suite holds both oracle restatements to them, the GPU suite
holds the HIP kernels to them and to the oracle's outputs. Modes:
  "bits"   same bit patterns (NaN anywhere the wanted value is NaN, any payload)
  "ulp"    NaN exactly where wanted; zeros and infinities exact with their sign; finite values within `ulps` units in the
           last place of the wanted value (float32)
"""
import math

import numpy as np

from akg_amd import harness, op_desc

F32 = np.float32
NAN, INF = float("nan"), float("inf")


def _unary(op, n, dtype="float32", out_dtype=None):
    b = op_desc.DescBuilder("kat_%s_%s_%d" % (op.lower(), dtype, n))
    return b.dumps([b.unary(op, b.input([n], dtype), out_dtype)])


def _binary(op, n, dtype="float32", out_dtype=None):
    b = op_desc.DescBuilder("kat_%s_%s_%d" % (op.lower(), dtype, n))
    x = b.input([n], dtype)
    y = b.input([n], dtype)
    return b.dumps([b.binary(op, x, y, out_dtype)])


def _f32(values):
    return np.array(values, dtype=np.float64).astype(F32)


def cases():
    out = []

    def add(name, text, inputs, want, mode="bits", ulps=1.0):
        out.append({"name": name, "text": text, "inputs": inputs, "want": want, "mode": mode, "ulps": ulps})

    # ---- casts
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 3.4999, 3.5001, -128.5, -129.5, 1e9, -1e9, 0.49999997,
                  INF, -INF], dtype=F32)
    want = np.array([0, 2, 2, 0, -2, -2, 126, 127, 3, 4, -128, -128, 127, -128, 0, 127, -128], dtype=np.int8)
    b = op_desc.DescBuilder("kat_cast_f32_i8")
    add("cast_f32_to_int8_ties_and_saturation", b.dumps([b.cast(b.input([x.size], "float32"), "int8")]), [x], [want])

    bf = [(0x3F800000, 0x3F80), (0x3F808000, 0x3F80), (0x3F818000, 0x3F82), (0x3F808001, 0x3F81), (0x3F807FFF, 0x3F80),
          (0x7F7FFFFF, 0x7F80), (0xBF818000, 0xBF82), (0x00000001, 0x0000), (0x7F800000, 0x7F80), (0x80000000, 0x8000)]
    b = op_desc.DescBuilder("kat_cast_f32_bf16")
    add("cast_f32_to_bfloat16_round_to_nearest_even", b.dumps([b.cast(b.input([len(bf)], "float32"), "bfloat16")]),
        [np.array([v for v, _ in bf], dtype=np.uint32).view(F32)], [np.array([w for _, w in bf], dtype=np.uint16)])

    h = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 5.9604645e-08, 2.9802322e-08, 2.98023224e-08 * 1.0000001,
                  6.097555e-05, 6.1035156e-05, 1.0009765625, 1.00048828125, 1.00146484375, INF, -INF], dtype=F32)
    with np.errstate(over="ignore"):
        want = h.astype(np.float16)
    b = op_desc.DescBuilder("kat_cast_f32_f16")
    add("cast_f32_to_float16_ieee", b.dumps([b.cast(b.input([h.size], "float32"), "float16")]), [h], [want])

    # ---- reductions
    b = op_desc.DescBuilder("kat_reduce_max_init")
    text = b.dumps([b.reduce("ReduceMax", b.input([2, 4], "float32"), [1], True)])
    add("reduce_max_of_minus_inf_row_is_minus_largest_finite", text,
        [np.array([[-INF] * 4, [1.0, 5.0, -2.0, 3.0]], dtype=F32)], [np.array([[-np.finfo(F32).max], [5.0]], dtype=F32)])
    m = np.zeros((4, 5), dtype=np.bool_)
    m[1, 4] = True
    m[3, :] = True
    for spelling, want in (("ReduceAny", [False, True, False, True]), ("ElemAny", [False, True, False, True]),
                           ("ReduceAll", [False, False, False, True])):
        b = op_desc.DescBuilder("kat_%s" % spelling.lower())
        add(spelling.lower() + "_truth", b.dumps([b.reduce(spelling, b.input([4, 5], "bool"), [1], False)]), [m], [np.array(want)])

    # ---- unary math at the special values
    pi = math.pi
    table = {
        "Log": ([0.0, -0.0, 1.0, -1.0, INF, NAN, 4.0], [-INF, -INF, 0.0, NAN, INF, NAN, math.log(4.0)]),
        "Sin": ([0.0, -0.0, INF, NAN, 1.0], [0.0, -0.0, NAN, NAN, math.sin(1.0)]),
        "Cos": ([0.0, -0.0, INF, NAN, 1.0], [1.0, 1.0, NAN, NAN, math.cos(1.0)]),
        "ASin": ([0.0, -0.0, 1.0, -1.0, 1.5, NAN], [0.0, -0.0, pi / 2, -pi / 2, NAN, NAN]),
        "ACos": ([1.0, -1.0, 0.0, 1.5, NAN], [0.0, pi, pi / 2, NAN, NAN]),
        "Atan": ([0.0, -0.0, INF, -INF, 1.0, NAN], [0.0, -0.0, pi / 2, -pi / 2, pi / 4, NAN]),
        "Exp": ([0.0, -0.0, INF, -INF, NAN, 1.0, 100.0, -110.0], [1.0, 1.0, INF, 0.0, NAN, math.e, INF, 0.0]),
        "Tanh": ([0.0, -0.0, INF, -INF, NAN, 100.0, -100.0, 0.5], [0.0, -0.0, 1.0, -1.0, NAN, 1.0, -1.0, math.tanh(0.5)]),
        "Sqrt": ([0.0, -0.0, 4.0, -1.0, INF, NAN, 2.0], [0.0, -0.0, 2.0, NAN, INF, NAN, math.sqrt(2.0)]),
        "Rsqrt": ([4.0, 0.0, INF, -1.0, NAN, 0.25], [0.5, INF, 0.0, NAN, NAN, 2.0]),
        "Reciprocal": ([4.0, 0.0, -0.0, INF, -INF, NAN, 3.0], [0.25, INF, -INF, 0.0, -0.0, NAN, 1.0 / 3.0]),
        "Abs": ([0.0, -0.0, -INF, NAN, -2.5], [0.0, 0.0, INF, NAN, 2.5]),
        "Neg": ([0.0, -0.0, INF, NAN, 2.5], [-0.0, 0.0, -INF, NAN, -2.5]),
    }
    for op, (xs, wants) in table.items():
        # the largest finite results that a float32 exp overflows past are not in the table: 100 and -110 are far outside
        add("special_values_" + op.lower(), _unary(op, len(xs)), [_f32(xs)], [_f32(wants)], "ulp", 2.0)

    xs = [0.0, -0.0, 0.5, -0.5, 1.0, -1.0, 2.9999998, -2.0000002, 8388607.5, -8388607.5, 16777216.0, 1e30, -1e30, INF, -INF,
          1e-45, -1e-45, NAN]
    x = _f32(xs)
    want = np.array([float(math.floor(float(v))) if math.isfinite(float(v)) else float(v) for v in x], dtype=F32)
    want[1] = -0.0
    add("floor_toward_minus_infinity", _unary("Floor", x.size), [x], [want])

    # ---- Asinh / Acosh in the reference's spelling: log(x + sqrt(1 + x*x)), log(x + sqrt(x*x - 1)), one op of the type per step
    k = _f32([-1.0e4, 2.0e19, 0.0, 1.0])
    add("asinh_spelled_out_cancels_and_overflows", _unary("Asinh", 4), [k], [_f32([-INF, INF, 0.0, math.asinh(1.0)])], "ulp", 4.0)
    k = _f32([1.0, 0.5, 2.0, 2.0e19])
    add("acosh_spelled_out", _unary("Acosh", 4), [k], [_f32([0.0, NAN, math.acosh(2.0), INF])], "ulp", 4.0)
    # float16: 300 * 300 overflows the type, so the result is +inf; 0.01 + 1 rounds to 1.009765625
    k16 = np.array([300.0, 0.01], dtype=np.float16)
    add("asinh_float16_rounds_every_step", _unary("Asinh", 2, "float16"), [k16],
        [np.array([INF, math.log(1.009765625)], dtype=np.float64).astype(np.float16)], "half")

    # ---- predicates, logic, comparisons
    x = np.array([NAN, INF, -INF, 0.0, -0.0, 1.0, 3.4028235e38, 1e-45, -NAN], dtype=F32)
    for op, bits in {"IsNan": [1, 0, 0, 0, 0, 0, 0, 0, 1], "IsInf": [0, 1, 1, 0, 0, 0, 0, 0, 0],
                     "IsFinite": [0, 0, 0, 1, 1, 1, 1, 1, 0]}.items():
        add("predicate_" + op.lower(), _unary(op, x.size, "float32", "bool"), [x], [np.array(bits, dtype=np.bool_)])
    hh = np.array([NAN, INF, -INF, 65504.0, 6e-8], dtype=np.float16)
    add("predicate_isfinite_float16", _unary("IsFinite", hh.size, "float16", "bool"), [hh], [np.array([0, 0, 0, 1, 1], dtype=np.bool_)])
    a = np.array([False, False, True, True])
    bb = np.array([False, True, False, True])
    add("logical_and", _binary("LogicalAnd", 4, "bool"), [a, bb], [np.array([False, False, False, True])])
    add("logical_or", _binary("LogicalOr", 4, "bool"), [a, bb], [np.array([False, True, True, True])])
    add("logical_not", _unary("LogicalNot", 4, "bool"), [a], [np.array([True, True, False, False])])
    fa = np.array([1.0, 2.0, 2.0, NAN, 1.0, NAN, 0.0, -INF, INF], dtype=F32)
    fb = np.array([2.0, 1.0, 2.0, 1.0, NAN, NAN, -0.0, INF, INF], dtype=F32)
    for op, bits in {"Less": [1, 0, 0, 0, 0, 0, 0, 1, 0], "LessEqual": [1, 0, 1, 0, 0, 0, 1, 1, 1],
                     "Greater": [0, 1, 0, 0, 0, 0, 0, 0, 0], "GreaterEqual": [0, 1, 1, 0, 0, 0, 1, 0, 1],
                     "Equal": [0, 0, 1, 0, 0, 0, 1, 0, 1], "NotEqual": [1, 1, 0, 1, 1, 1, 0, 1, 0]}.items():
        add("ordered_compare_" + op.lower(), _binary(op, fa.size, "float32", "bool"), [fa, fb], [np.array(bits, dtype=np.bool_)])
    ia = np.array([-1, 1, -2147483648, 5, 2147483647], dtype=np.int32)
    ib = np.array([1, -1, 2147483647, 5, -2147483648], dtype=np.int32)
    for op, bits in {"Less": [1, 0, 1, 0, 0], "GreaterEqual": [0, 1, 0, 1, 1]}.items():
        add("signed_compare_" + op.lower(), _binary(op, ia.size, "int32", "bool"), [ia, ib], [np.array(bits, dtype=np.bool_)])

    # ---- Maximum / Minimum propagate NaN (arith.maximumf / minimumf)
    ma = _f32([1.0, NAN, 2.0, -0.0, INF])
    mb = _f32([2.0, 1.0, NAN, 0.0, -INF])
    add("maximum_propagates_nan", _binary("Maximum", 5), [ma, mb], [_f32([2.0, NAN, NAN, 0.0, INF])])
    add("minimum_propagates_nan", _binary("Minimum", 5), [ma, mb], [_f32([1.0, NAN, NAN, -0.0, -INF])])

    # ---- Pow, Atan2
    base = [2.0, -2.0, -2.0, -8.0, 0.0, 5.0, NAN, 1.0, 0.0, -0.0, INF, 3.0, 9.0, -INF]
    expo = [3.0, 3.0, 2.0, 1 / 3, 0.0, 0.0, 0.0, NAN, -1.0, -1.0, -1.0, 2.0, 0.5, 3.0]
    want = [8.0, -8.0, 4.0, NAN, 1.0, 1.0, 1.0, 1.0, INF, -INF, 0.0, 9.0, 3.0, -INF]
    add("pow_operand_order_and_special_cases", _binary("Pow", len(base)), [_f32(base), _f32(expo)], [_f32(want)], "ulp", 2.0)
    y = [1.0, 1.0, -1.0, -1.0, 0.0, -0.0, 0.0, 1.0, -1.0, 0.0, -0.0, INF, NAN]
    xx = [1.0, -1.0, -1.0, 1.0, -1.0, -1.0, 1.0, 0.0, 0.0, 0.0, 0.0, INF, 1.0]
    want = [pi / 4, 3 * pi / 4, -3 * pi / 4, -pi / 4, pi, -pi, 0.0, pi / 2, -pi / 2, 0.0, -0.0, pi / 4, NAN]
    add("atan2_quadrants_and_operand_order", _binary("Atan2", len(y)), [_f32(y), _f32(xx)], [_f32(want)], "ulp", 2.0)

    # ---- AddN: left to right in the declared type
    b = op_desc.DescBuilder("kat_addn_4_float32")
    xs = [b.input([2], "float32") for _ in range(4)]
    add("addn_left_to_right_float32", b.dumps([b.op("AddN", xs, [2], "float32")]),
        [_f32([1e8, 1.0]), _f32([-1e8, 2.0]), _f32([1.0, 3.0]), _f32([0.5, 4.0])], [_f32([1.5, 10.0])])
    b = op_desc.DescBuilder("kat_addn_3_float16")
    xs = [b.input([1], "float16") for _ in range(3)]
    add("addn_rounds_every_step_float16", b.dumps([b.op("AddN", xs, [1], "float16")]),
        [np.array([2048.0], dtype=np.float16), np.array([1.0], dtype=np.float16), np.array([1.0], dtype=np.float16)],
        [np.array([2048.0], dtype=np.float16)])

    # ---- integer division: truncates toward zero; x / 0 = 0 and INT_MIN / -1 = INT_MIN are this backend's choice where
    # arith.divsi is undefined
    da = np.array([7, -7, 7, -7, 0, 2147483647, -2147483647, 5, -5, 0, -2147483648], dtype=np.int32)
    db = np.array([2, 2, -2, -2, 5, -1, 2, 0, 0, 0, -1], dtype=np.int32)
    add("integer_division_truncates_and_corner_values", _binary("Div", da.size, "int32"), [da, db],
        [np.array([3, -3, -3, 3, 0, -2147483647, -1073741823, 0, 0, 0, -2147483648], dtype=np.int32)])

    # ---- per-token int8 quantisation on exact ties: absmax 127 makes the scale 1, so x / scale is x itself and the
    # fused clamp + cast sees 0.5, 1.5, 2.5, 126.5 (all exact in bfloat16) -> 0, 2, 2, 126; the residual is zero
    cols = 16
    row = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, -126.5, 3.5, 4.5, -127.0, 0.0, 64.5, 65.5, 1.0]
    qwant = [127, 0, 2, 2, 0, -2, -2, 126, -126, 4, 4, -127, 0, 64, 66, 1]
    row2 = [v * 2 for v in row]              # absmax 254 -> scale 2: the same quotients
    row3 = [0.0] * cols                      # absmax 0 -> scale 0 -> 0 / 0 = NaN -> cast gives 0
    xq = harness.f32_to_bf16_bits(np.array([row, row2, row3], dtype=F32))
    rq = harness.f32_to_bf16_bits(np.zeros((3, cols), dtype=F32))
    add("quantisation_on_exact_ties", op_desc.quant_int8_residual(3, cols, "bfloat16", "kat_quant_ties"), [xq, rq],
        [np.array([qwant, qwant, [0] * cols], dtype=np.int8), np.array([1.0, 2.0, 0.0], dtype=F32)])
    return out


def check(case, got):
    """(ok, message) for the outputs `got` of one case against its wanted values."""
    for k, (g, w) in enumerate(zip(got, case["want"])):
        g = np.asarray(g)
        w = np.asarray(w).reshape(g.shape)
        if w.dtype.kind in "biu" or case["mode"] == "bits" and w.dtype.kind != "f":
            if not np.array_equal(g.view(w.dtype) if g.dtype.itemsize == w.dtype.itemsize else g, w):
                return False, "output %d: got %s, want %s" % (k, g.ravel().tolist(), w.ravel().tolist())
            continue
        gf = g.astype(np.float64) if g.dtype.kind == "f" else harness.bf16_bits_to_f32(g).astype(np.float64)
        wf = w.astype(np.float64) if w.dtype.kind == "f" else harness.bf16_bits_to_f32(w).astype(np.float64)
        if not np.array_equal(np.isnan(gf), np.isnan(wf)):
            return False, "output %d: NaN at other places: got %s, want %s" % (k, gf.ravel().tolist(), wf.ravel().tolist())
        ok = ~np.isnan(wf)
        if not np.array_equal(np.signbit(gf[ok]), np.signbit(wf[ok])):
            return False, "output %d: signs differ (zeros included): got %s, want %s" % (k, gf.ravel().tolist(), wf.ravel().tolist())
        if case["mode"] == "bits":
            if not np.array_equal(gf[ok], wf[ok]):
                return False, "output %d: got %s, want %s" % (k, gf.ravel().tolist(), wf.ravel().tolist())
            continue
        exact = ok & (~np.isfinite(wf) | (wf == 0))
        if not np.array_equal(gf[exact], wf[exact]):
            return False, "output %d: zeros / infinities differ: got %s, want %s" % (k, gf.ravel().tolist(), wf.ravel().tolist())
        fin = ok & ~exact
        if case["mode"] == "half":
            close = np.abs(gf[fin] - wf[fin]) <= 1e-3 + 1e-2 * np.abs(wf[fin])
        else:
            spacing = np.spacing(np.abs(wf[fin]).astype(F32)).astype(np.float64)
            close = np.abs(gf[fin] - wf[fin]) <= case["ulps"] * spacing
        if not close.all():
            return False, "output %d: got %s, want %s" % (k, gf.ravel().tolist(), wf.ravel().tolist())
    return True, "as wanted"
