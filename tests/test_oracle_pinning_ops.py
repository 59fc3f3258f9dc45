"""Pins the op-table rows of the CPU oracle that no fused pattern of the measured configurations exercises: Log, Sin, Cos,
ASin, ACos, Atan, Asinh, Acosh, Floor, IsNan / IsInf / IsFinite, LogicalNot / And / Or, Pow, Atan2, AddN, the six
comparisons, integer Div, ReduceAny under both of its names, and MatMul with a 16-bit declared result.

Nothing here retypes the oracle's expressions. Expected values come from Python's `math` module and exact float64 /
rational arithmetic (correctly rounded to the declared type), from IEEE-754 special-case tables, and from known-answer
vectors chosen so that a plausible mistake fails: a libm asinh where the reference spells log(x + sqrt(1 + x*x)), swapped
atan2 / pow operands, AddN summed from the right, an unordered comparison, a float32 accumulator where the declared type is
float16, floor as truncation.
"""
import json
import math
import os

import numpy as np
import pytest

from akg_amd import op_desc
from oracle import cpu_ref, np_ref

F32 = np.float32
NAN, INF = float("nan"), float("inf")


def run_both(text, inputs, tmp_path):
    desc = json.loads(text)
    path = os.path.join(str(tmp_path), desc["op"] + ".info")
    with open(path, "w", encoding="utf-8") as f:
        f.write(text)
    return cpu_ref.CpuKernel(path, rebuild=True)(inputs), np_ref.evaluate(desc, inputs)


def unary_desc(op, n, dtype="float32", out_dtype=None):
    b = op_desc.DescBuilder("pin_%s_%s_%d" % (op.lower(), dtype, n))
    x = b.input([n], dtype)
    return b.dumps([b.unary(op, x, out_dtype)])


def binary_desc(op, n, dtype="float32", out_dtype=None):
    b = op_desc.DescBuilder("pin_%s_%s_%d" % (op.lower(), dtype, n))
    x = b.input([n], dtype)
    y = b.input([n], dtype)
    return b.dumps([b.binary(op, x, y, out_dtype)])


def ulps_f32(got, want64):
    """Distance of float32 `got` from the float64 values `want64`, in units of the float32 spacing at the target."""
    want32 = want64.astype(F32)
    spacing = np.spacing(np.abs(want32)).astype(np.float64)
    return np.abs(got.astype(np.float64) - want64) / spacing


def same_bits(a, b):
    return np.array_equal(np.asarray(a).view(np.uint32), np.asarray(b, dtype=F32).view(np.uint32))


# ---------------------------------------------------------------------------------------------------------
# unary math against float64 `math`
# ---------------------------------------------------------------------------------------------------------
UNARY_CASES = {
    # op: (math function, sampler of the domain)
    "Log": (math.log, lambda r, n: np.exp(r.uniform(-80, 80, n))),
    "Sin": (math.sin, lambda r, n: r.uniform(-20, 20, n)),
    "Cos": (math.cos, lambda r, n: r.uniform(-20, 20, n)),
    "ASin": (math.asin, lambda r, n: r.uniform(-1, 1, n)),
    "ACos": (math.acos, lambda r, n: r.uniform(-1, 1, n)),
    "Atan": (math.atan, lambda r, n: r.standard_normal(n) * 10 ** r.uniform(-3, 3, n)),
}


@pytest.mark.parametrize("op", sorted(UNARY_CASES))
def test_unary_math_ops_agree_with_float64_math(op, tmp_path):
    fn, sample = UNARY_CASES[op]
    x = sample(np.random.default_rng(11), 4000).astype(F32)
    c_out, n_out = run_both(unary_desc(op, x.size), [x], tmp_path)
    want = np.array([fn(float(v)) for v in x], dtype=np.float64)
    assert ulps_f32(c_out[0], want).max() <= 1.0      # glibc's float functions are within one unit in the last place
    assert ulps_f32(n_out[0], want).max() <= 4.0      # numpy's vectorised float32 loops are a little looser


def test_unary_math_special_values(tmp_path):
    pi = math.pi
    table = {
        "Log": ([0.0, -0.0, 1.0, -1.0, INF, NAN, 4.0], [-INF, -INF, 0.0, NAN, INF, NAN, math.log(4.0)]),
        "Sin": ([0.0, -0.0, INF, NAN], [0.0, -0.0, NAN, NAN]),
        "Cos": ([0.0, -0.0, INF, NAN], [1.0, 1.0, NAN, NAN]),
        "ASin": ([0.0, -0.0, 1.0, -1.0, 1.5, NAN], [0.0, -0.0, pi / 2, -pi / 2, NAN, NAN]),
        "ACos": ([1.0, -1.0, 0.0, 1.5, NAN], [0.0, pi, pi / 2, NAN, NAN]),
        "Atan": ([0.0, -0.0, INF, -INF, 1.0, NAN], [0.0, -0.0, pi / 2, -pi / 2, pi / 4, NAN]),
    }
    for op, (xs, wants) in table.items():
        x = np.array(xs, dtype=F32)
        want = np.array(wants, dtype=np.float64).astype(F32)
        for out in run_both(unary_desc(op, x.size), [x], tmp_path):
            got = out[0]
            assert np.array_equal(np.isnan(got), np.isnan(want)), op
            ok = ~np.isnan(want)
            # exact where the answer is exact (zeros keep their sign, infinities), one unit otherwise
            fin = ok & np.isfinite(want)
            assert np.array_equal(got[ok & ~fin], want[ok & ~fin]), (op, got, want)
            assert np.all(np.abs(got[fin].astype(np.float64) - want[fin]) <= np.spacing(np.abs(want[fin]))), (op, got, want)
            assert np.array_equal(np.signbit(got[ok]), np.signbit(want[ok])), op


def test_floor_rounds_toward_minus_infinity(tmp_path):
    xs = [0.0, -0.0, 0.5, -0.5, 1.0, -1.0, 2.9999998, -2.0000002, 8388607.5, -8388607.5, 16777216.0, 1e30, -1e30, INF, -INF,
          1e-45, -1e-45]
    x = np.array(xs, dtype=F32)
    want = np.array([float(math.floor(float(v))) if math.isfinite(float(v)) else float(v) for v in x], dtype=F32)
    want[1] = -0.0                                   # floor(-0) keeps the sign
    for out in run_both(unary_desc("Floor", x.size), [x], tmp_path):
        assert same_bits(out[0], want)               # truncation would turn -0.5 into -0 and -2.0000002 into -2
    nan_in = np.array([NAN], dtype=F32)
    for out in run_both(unary_desc("Floor", 1), [nan_in], tmp_path):
        assert np.isnan(out[0][0])


# ---------------------------------------------------------------------------------------------------------
# Asinh / Acosh: the reference spells them out in single ops of the result type (MindSporeToLinalg.cpp:156-180)
# ---------------------------------------------------------------------------------------------------------
def test_asinh_and_acosh_follow_the_reference_spelling(tmp_path):
    # Where the spelled-out form is well conditioned it is the function itself ...
    x = np.random.default_rng(5).uniform(1.0, 1000.0, 3000).astype(F32)
    want = np.array([math.asinh(float(v)) for v in x])
    for out in run_both(unary_desc("Asinh", x.size), [x], tmp_path):
        assert ulps_f32(out[0], want).max() <= 4.0
    y = np.random.default_rng(6).uniform(1.5, 1000.0, 3000).astype(F32)
    want = np.array([math.acosh(float(v)) for v in y])
    for out in run_both(unary_desc("Acosh", y.size), [y], tmp_path):
        assert ulps_f32(out[0], want).max() <= 4.0
    # ... and where it is not, the spelling shows: for x = -1e4, 1 + x*x rounds to 1e8, its root to 1e4, x + 1e4 is 0 and
    # the result is log(0) = -inf, where asinh(-1e4) = -9.9035. x*x overflows float32 at 2e19 (asinh = 45.1).
    k = np.array([-1.0e4, 2.0e19, 0.0, 1.0], dtype=F32)
    for out in run_both(unary_desc("Asinh", k.size), [k], tmp_path):
        assert out[0][0] == -INF and out[0][1] == INF and out[0][2] == 0.0
        assert abs(float(out[0][3]) - math.asinh(1.0)) < 2e-7
    k = np.array([1.0, 0.5, 2.0, 2.0e19], dtype=F32)
    for out in run_both(unary_desc("Acosh", k.size), [k], tmp_path):
        assert out[0][0] == 0.0 and np.isnan(out[0][1]) and out[0][3] == INF
        assert abs(float(out[0][2]) - math.acosh(2.0)) < 3e-7


def test_asinh_in_float16_rounds_every_step(tmp_path):
    # 300 * 300 overflows float16, so the square is +inf and so is the result; evaluated in float32 and rounded at the
    # end it would be 6.3984. At 0.01 the square vanishes against 1, the root is 1, and 0.01 + 1 rounds to the float16
    # neighbour 1.009765625 of 1.01: the result is log(1.009765625) = 0.0097183, where asinh(0.01) = 0.0099998.
    x = np.array([300.0, 0.01, 2.0], dtype=np.float16)
    for out in run_both(unary_desc("Asinh", x.size, "float16"), [x], tmp_path):
        got = out[0].astype(np.float64)
        assert got[0] == INF
        assert abs(got[1] - math.log(1.009765625)) < 8e-6
        assert abs(got[2] - math.asinh(2.0)) < 2e-3


# ---------------------------------------------------------------------------------------------------------
# predicates, logic, comparisons: truth tables
# ---------------------------------------------------------------------------------------------------------
def test_float_predicates_known_answers(tmp_path):
    x = np.array([NAN, INF, -INF, 0.0, -0.0, 1.0, 3.4028235e38, 1e-45, -NAN], dtype=F32)
    want = {"IsNan": [1, 0, 0, 0, 0, 0, 0, 0, 1], "IsInf": [0, 1, 1, 0, 0, 0, 0, 0, 0], "IsFinite": [0, 0, 0, 1, 1, 1, 1, 1, 0]}
    for op, bits in want.items():
        for out in run_both(unary_desc(op, x.size, "float32", "bool"), [x], tmp_path):
            assert out[0].dtype == np.bool_ and out[0].tolist() == [bool(v) for v in bits], op
    h = np.array([NAN, INF, -INF, 65504.0, 6e-8], dtype=np.float16)
    for out in run_both(unary_desc("IsFinite", h.size, "float16", "bool"), [h], tmp_path):
        assert out[0].tolist() == [False, False, False, True, True]


def test_logical_ops_truth_tables(tmp_path):
    a = np.array([False, False, True, True])
    b = np.array([False, True, False, True])
    for out in run_both(binary_desc("LogicalAnd", 4, "bool"), [a, b], tmp_path):
        assert out[0].tolist() == [False, False, False, True]
    for out in run_both(binary_desc("LogicalOr", 4, "bool"), [a, b], tmp_path):
        assert out[0].tolist() == [False, True, True, True]
    for out in run_both(unary_desc("LogicalNot", 4, "bool"), [a], tmp_path):
        assert out[0].tolist() == [True, True, False, False]


def test_float_comparisons_are_ordered(tmp_path):
    # arith.cmpf OGT / OGE / OLT / OLE / OEQ: false whenever an operand is NaN; NotEqual is the negation of OEQ
    # (ConvertMindSporeNotBinaryOp, MindSporeToTosa.cpp:499), so it is true there. -0 equals +0.
    a = np.array([1.0, 2.0, 2.0, NAN, 1.0, NAN, 0.0, -INF, INF], dtype=F32)
    b = np.array([2.0, 1.0, 2.0, 1.0, NAN, NAN, -0.0, INF, INF], dtype=F32)
    want = {
        "Less": [1, 0, 0, 0, 0, 0, 0, 1, 0], "LessEqual": [1, 0, 1, 0, 0, 0, 1, 1, 1],
        "Greater": [0, 1, 0, 0, 0, 0, 0, 0, 0], "GreaterEqual": [0, 1, 1, 0, 0, 0, 1, 0, 1],
        "Equal": [0, 0, 1, 0, 0, 0, 1, 0, 1], "NotEqual": [1, 1, 0, 1, 1, 1, 0, 1, 0],
    }
    for op, bits in want.items():
        for out in run_both(binary_desc(op, a.size, "float32", "bool"), [a, b], tmp_path):
            assert out[0].tolist() == [bool(v) for v in bits], op


def test_integer_comparisons_are_signed(tmp_path):
    a = np.array([-1, 1, -2147483648, 5, 2147483647], dtype=np.int32)
    b = np.array([1, -1, 2147483647, 5, -2147483648], dtype=np.int32)
    for op, bits in {"Less": [1, 0, 1, 0, 0], "GreaterEqual": [0, 1, 0, 1, 1]}.items():
        for out in run_both(binary_desc(op, a.size, "int32", "bool"), [a, b], tmp_path):
            assert out[0].tolist() == [bool(v) for v in bits], op      # an unsigned compare would call -1 the largest


# ---------------------------------------------------------------------------------------------------------
# Pow, Atan2: operand order and the IEEE special cases
# ---------------------------------------------------------------------------------------------------------
def test_pow_operand_order_and_special_cases(tmp_path):
    base = [2.0, -2.0, -2.0, -8.0, 0.0, 5.0, NAN, 1.0, 0.0, -0.0, INF, 3.0, 9.0, -INF]
    expo = [3.0, 3.0, 2.0, 1 / 3, 0.0, 0.0, 0.0, NAN, -1.0, -1.0, -1.0, 2.0, 0.5, 3.0]
    want = [8.0, -8.0, 4.0, NAN, 1.0, 1.0, 1.0, 1.0, INF, -INF, 0.0, 9.0, 3.0, -INF]
    a, b = np.array(base, dtype=F32), np.array(expo, dtype=F32)
    for out in run_both(binary_desc("Pow", a.size), [a, b], tmp_path):
        got = out[0]
        w = np.array(want, dtype=F32)
        assert np.array_equal(np.isnan(got), np.isnan(w)), got       # a negative base with a fractional exponent: NaN
        assert np.array_equal(got[~np.isnan(w)], w[~np.isnan(w)]), got   # 2^3 = 8, not 3^2 = 9: base first
    r = np.random.default_rng(3)
    a = r.uniform(0.1, 30.0, 3000).astype(F32)
    b = r.uniform(-6.0, 6.0, 3000).astype(F32)
    want = np.array([math.pow(float(x), float(y)) for x, y in zip(a, b)])
    c_out, n_out = run_both(binary_desc("Pow", a.size), [a, b], tmp_path)
    assert ulps_f32(c_out[0], want).max() <= 1.0
    assert ulps_f32(n_out[0], want).max() <= 4.0


def test_atan2_quadrants_and_operand_order(tmp_path):
    pi = math.pi
    y = [1.0, 1.0, -1.0, -1.0, 0.0, -0.0, 0.0, 1.0, -1.0, 0.0, -0.0, INF, NAN]
    x = [1.0, -1.0, -1.0, 1.0, -1.0, -1.0, 1.0, 0.0, 0.0, 0.0, 0.0, INF, 1.0]
    want = [pi / 4, 3 * pi / 4, -3 * pi / 4, -pi / 4, pi, -pi, 0.0, pi / 2, -pi / 2, 0.0, -0.0, pi / 4, NAN]
    a, b = np.array(y, dtype=F32), np.array(x, dtype=F32)
    w = np.array(want, dtype=np.float64)
    for out in run_both(binary_desc("Atan2", a.size), [a, b], tmp_path):
        got = out[0]
        assert np.isnan(got[-1])
        assert np.all(ulps_f32(got[:-1], w[:-1]) <= 1.0), got        # (y, x): atan2(1, -1) is 3pi/4, atan2(-1, 1) is -pi/4
        assert np.array_equal(np.signbit(got[:-1]), np.signbit(w[:-1].astype(F32)))


# ---------------------------------------------------------------------------------------------------------
# AddN: left to right, rounding to the declared type after every addition (createAddNOpBody, :209-221)
# ---------------------------------------------------------------------------------------------------------
def addn_desc(n_operands, n, dtype):
    b = op_desc.DescBuilder("pin_addn_%d_%s" % (n_operands, dtype))
    xs = [b.input([n], dtype) for _ in range(n_operands)]
    return b.dumps([b.op("AddN", xs, [n], dtype)])


def test_addn_adds_left_to_right_in_the_declared_type(tmp_path):
    # (1e8 + -1e8) + 1 = 1, but 1e8 + (-1e8 + 1) = 0 in float32
    ins = [np.array([1e8, 1.0], dtype=F32), np.array([-1e8, 2.0], dtype=F32), np.array([1.0, 3.0], dtype=F32),
           np.array([0.5, 4.0], dtype=F32)]
    for out in run_both(addn_desc(4, 2, "float32"), ins, tmp_path):
        assert out[0].tolist() == [1.5, 10.0]
    # float16: 2048 + 1 + 1 stays 2048 when every step rounds; summed wide and rounded once it is 2050
    h = [np.array([2048.0], dtype=np.float16), np.array([1.0], dtype=np.float16), np.array([1.0], dtype=np.float16)]
    for out in run_both(addn_desc(3, 1, "float16"), h, tmp_path):
        assert float(out[0][0]) == 2048.0


# ---------------------------------------------------------------------------------------------------------
# integer Div: arith.divsi truncates toward zero (createDivOpBody, MindSporeToLinalg.cpp:229-246)
# ---------------------------------------------------------------------------------------------------------
def test_integer_division_truncates_toward_zero(tmp_path):
    a = np.array([7, -7, 7, -7, 0, 2147483647, -2147483647], dtype=np.int32)
    b = np.array([2, 2, -2, -2, 5, -1, 2], dtype=np.int32)
    want = [3, -3, -3, 3, 0, -2147483647, -1073741823]          # floor division would give -4 for -7 / 2
    for out in run_both(binary_desc("Div", a.size, "int32"), [a, b], tmp_path):
        assert out[0].tolist() == want


def test_integer_division_corner_values_chosen_where_the_reference_is_undefined(tmp_path):
    # arith.divsi is undefined for a zero divisor and for INT_MIN / -1 (the reference's compiled loop traps on x86).
    # The oracle and the kernel agree on: x / 0 = 0, INT_MIN / -1 = INT_MIN (the wrapped quotient).
    a = np.array([5, -5, 0, -2147483648], dtype=np.int32)
    b = np.array([0, 0, 0, -1], dtype=np.int32)
    for out in run_both(binary_desc("Div", a.size, "int32"), [a, b], tmp_path):
        assert out[0].tolist() == [0, 0, 0, -2147483648]


# ---------------------------------------------------------------------------------------------------------
# ReduceAny (also spelled ElemAny in descriptions, TranslateToMindsporeDialect.cpp:463)
# ---------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("spelling", ["ReduceAny", "ElemAny"])
def test_reduce_any_is_true_where_some_element_is(spelling, tmp_path):
    b = op_desc.DescBuilder("pin_%s" % spelling.lower())
    x = b.input([4, 5], "bool")
    text = b.dumps([b.reduce(spelling, x, [1], False)])
    m = np.zeros((4, 5), dtype=np.bool_)
    m[1, 4] = True
    m[3, :] = True
    for out in run_both(text, [m], tmp_path):
        assert out[0].tolist() == [False, True, False, True]
    ball = op_desc.DescBuilder("pin_reduceall")
    x = ball.input([4, 5], "bool")
    text = ball.dumps([ball.reduce("ReduceAll", x, [1], False)])
    for out in run_both(text, [m], tmp_path):
        assert out[0].tolist() == [False, False, False, True]


# ---------------------------------------------------------------------------------------------------------
# MatMul with a 16-bit declared result: zero-filled accumulator of that type (MindSporeToLinalg.cpp:1453-1546)
# ---------------------------------------------------------------------------------------------------------
def matmul_desc(m, k, n, dtype, transpose_b=False):
    b = op_desc.DescBuilder("pin_matmul_%s_%dx%dx%d%s" % (dtype, m, k, n, "_tb" if transpose_b else ""))
    a = b.input([m, k], dtype)
    w = b.input([n, k] if transpose_b else [k, n], dtype)
    return b.dumps([b.matmul(a, w, dtype, transpose_b=transpose_b)])


def test_float16_matmul_accumulator_stalls_like_a_float16_sum(tmp_path):
    # 4096 products of 1: a float16 running sum stops at 2048; a float32 accumulator rounded at the end gives 4096
    a = np.ones((2, 4096), dtype=np.float16)
    w = np.ones((4096, 3), dtype=np.float16)
    for out in run_both(matmul_desc(2, 4096, 3, "float16"), [a, w], tmp_path):
        assert np.all(out[0].astype(np.float32) == 2048.0)


def _round_to(dtype, v):
    """Correctly rounded value of the Python float `v` in `dtype`, as a Python float."""
    if dtype == "float16":
        with np.errstate(over="ignore"):
            return float(np.float16(v))
    bits = np.array([v], dtype=np.float64).astype(F32)      # exact inputs here are sums / products of 8-bit significands
    return float(np_ref.bf16_bits_to_f32(np_ref.f32_to_bf16_bits(bits))[0])


@pytest.mark.parametrize("dtype,transpose_b", [("float16", False), ("bfloat16", False), ("float16", True)])
def test_sixteen_bit_matmul_rounds_product_and_sum_every_step(dtype, transpose_b, tmp_path):
    """Brute force in Python floats: products and sums of two 16-bit values are exact in float64, so rounding each of
    them once to the 16-bit type is the correctly rounded step the reference's arith.mulf / arith.addf perform."""
    rng = np.random.default_rng(17)
    m, k, n = 5, 37, 4
    a32 = (rng.standard_normal((m, k)) * 3).astype(F32)
    w32 = (rng.standard_normal((k, n)) * 3).astype(F32)
    if dtype == "float16":
        a, w = a32.astype(np.float16), w32.astype(np.float16)
        af, wf = a.astype(np.float64), w.astype(np.float64)
    else:
        a, w = np_ref.f32_to_bf16_bits(a32), np_ref.f32_to_bf16_bits(w32)
        af, wf = np_ref.bf16_bits_to_f32(a).astype(np.float64), np_ref.bf16_bits_to_f32(w).astype(np.float64)
    want = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            acc = 0.0
            for kk in range(k):
                acc = _round_to(dtype, acc + _round_to(dtype, float(af[i, kk]) * float(wf[kk, j])))
            want[i, j] = acc
    w_in = np.ascontiguousarray(w.T) if transpose_b else w
    for out in run_both(matmul_desc(m, k, n, dtype, transpose_b), [a, w_in], tmp_path):
        got = out[0].astype(np.float64) if dtype == "float16" else np_ref.bf16_bits_to_f32(out[0]).astype(np.float64)
        assert np.array_equal(got, want)


# ---------------------------------------------------------------------------------------------------------
# the shared known-answer table (tests/known_answers.py): both restatements against it; the GPU suite pushes the same
# vectors through the HIP kernels
# ---------------------------------------------------------------------------------------------------------
import known_answers  # noqa: E402

_KAT = {c["name"]: c for c in known_answers.cases()}


@pytest.mark.parametrize("name", sorted(_KAT))
def test_known_answer_table_holds_for_both_restatements(name, tmp_path):
    case = _KAT[name]
    c_out, n_out = run_both(case["text"], case["inputs"], tmp_path)
    for which, outs in (("C restatement", c_out), ("numpy restatement", n_out)):
        ok, msg = known_answers.check(case, outs)
        assert ok, "%s, %s: %s" % (name, which, msg)
