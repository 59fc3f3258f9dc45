"""Pins the CPU oracle (oracle/gen_cpu.py C restatement and oracle/np_ref.py) WITHOUT restating its formulas:
known-answer vectors for the rounding rules, closed forms and library routines for the fused patterns (scipy / torch in
float64), brute force with exact rational arithmetic on tiny inputs, invariants, and the two independently written
restatements against each other. The reference repository holds no numeric golden vectors for this path, so these are
what the mathematics fixes; each check is chosen so that a plausible mistake (truncation instead of round-half-even, a
dropped epsilon, a transposed operand, int8 products without widening, -inf instead of -FLT_MAX) fails it.
"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest

from akg_amd import harness, op_desc
from oracle import cpu_ref, gen_cpu, np_ref

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FIXTURES = os.path.join(ROOT, "akg_amd", "fixtures")


def build_and_run(desc_text, inputs, tmp_path, name=None):
    """Compile a description with the C restatement and run it; also evaluate the numpy restatement."""
    desc = json.loads(desc_text)
    path = os.path.join(str(tmp_path), (name or desc["op"]) + ".info")
    with open(path, "w", encoding="utf-8") as f:
        f.write(desc_text)
    c_out = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    n_out = np_ref.evaluate(desc, inputs)
    return desc, c_out, n_out


# ---------------------------------------------------------------------------------------------------------
# rounding rules: known-answer vectors
# ---------------------------------------------------------------------------------------------------------
BF16_KAT = [  # float32 bits -> bfloat16 bits under round-to-nearest-even
    (0x3F800000, 0x3F80),  # 1.0
    (0x3F808000, 0x3F80),  # tie, even mantissa below -> stays
    (0x3F818000, 0x3F82),  # tie, odd mantissa below -> rounds up to even
    (0x3F808001, 0x3F81),  # just above the tie
    (0x3F807FFF, 0x3F80),  # just below the tie
    (0x7F7FFFFF, 0x7F80),  # FLT_MAX rounds to +inf
    (0xBF818000, 0xBF82),  # negative tie
    (0x00000001, 0x0000),  # smallest subnormal -> 0
    (0x7F800000, 0x7F80),  # inf
]


def test_bf16_round_to_nearest_even_known_answers():
    bits = np.array([b for b, _ in BF16_KAT], dtype=np.uint32)
    want = np.array([w for _, w in BF16_KAT], dtype=np.uint16)
    got_np = np_ref.f32_to_bf16_bits(bits.view(np.float32))
    got_h = harness.f32_to_bf16_bits(bits.view(np.float32))
    assert np.array_equal(got_np, want)
    assert np.array_equal(got_h, want)


def test_bf16_cast_in_c_restatement_known_answers(tmp_path):
    b = op_desc.DescBuilder("kat_cast_bf16")
    x = b.input([len(BF16_KAT)], "float32")
    text = b.dumps([b.cast(x, "bfloat16")])
    bits = np.array([v for v, _ in BF16_KAT], dtype=np.uint32).view(np.float32)
    _, c_out, n_out = build_and_run(text, [bits], tmp_path)
    want = np.array([w for _, w in BF16_KAT], dtype=np.uint16)
    assert np.array_equal(c_out[0], want)
    assert np.array_equal(n_out[0], want)


def test_f16_cast_matches_ieee_half_conversion(tmp_path):
    # numpy's float32 -> float16 conversion is IEEE round-to-nearest-even; the C restatement converts in software.
    rng = np.random.default_rng(7)
    special = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e6, -1e6, 5.9604645e-08, 2.9802322e-08, 2.98023224e-08 * 1.0000001,
                        6.097555e-05, 6.1035156e-05, 1.0009765625, 1.00048828125, 1.00146484375, np.inf, -np.inf], dtype=np.float32)
    x = np.concatenate([special, (rng.standard_normal(4000) * 10 ** rng.uniform(-9, 5, 4000)).astype(np.float32)])
    b = op_desc.DescBuilder("kat_cast_f16")
    t = b.input([x.size], "float32")
    text = b.dumps([b.cast(t, "float16")])
    _, c_out, n_out = build_and_run(text, [x], tmp_path)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    assert np.array_equal(c_out[0].view(np.uint16), want.view(np.uint16))
    assert np.array_equal(n_out[0].view(np.uint16), want.view(np.uint16))


def test_float_to_int8_cast_rounds_half_to_even_and_saturates(tmp_path):
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 3.4999, 3.5001, -128.5, -129.5, 1e9, -1e9, 0.49999997],
                 dtype=np.float32)
    want = np.array([0, 2, 2, 0, -2, -2, 126, 127, 3, 4, -128, -128, 127, -128, 0], dtype=np.int8)
    b = op_desc.DescBuilder("kat_cast_i8")
    t = b.input([x.size], "float32")
    text = b.dumps([b.cast(t, "int8")])
    _, c_out, n_out = build_and_run(text, [x], tmp_path)
    assert np.array_equal(c_out[0], want)      # truncation toward zero would give 0,1,2,0,-1,-2,126,127,...
    assert np.array_equal(n_out[0], want)


def test_reduce_max_starts_from_minus_largest_finite_not_minus_inf(tmp_path):
    # a row of -inf must reduce to -FLT_MAX (maxnumf(-FLT_MAX, -inf)), not to -inf
    b = op_desc.DescBuilder("kat_reduce_max_init")
    t = b.input([2, 4], "float32")
    text = b.dumps([b.reduce("ReduceMax", t, [1], True)])
    x = np.array([[-np.inf] * 4, [1.0, 5.0, -2.0, 3.0]], dtype=np.float32)
    _, c_out, n_out = build_and_run(text, [x], tmp_path)
    want = np.array([[-np.finfo(np.float32).max], [5.0]], dtype=np.float32)
    assert np.array_equal(c_out[0], want)
    assert np.array_equal(n_out[0], want)


def test_reduce_sum_accumulates_in_the_declared_narrow_type(tmp_path):
    # 4096 ones in float16: a float16 accumulator stalls at 2048 (2048 + 1 rounds back to 2048); an accumulator that is
    # silently widened to float32 would return 4096.
    b = op_desc.DescBuilder("kat_reduce_sum_f16")
    t = b.input([1, 4096], "float16")
    text = b.dumps([b.reduce("ReduceSum", t, [1], True)])
    x = np.ones((1, 4096), dtype=np.float16)
    _, c_out, n_out = build_and_run(text, [x], tmp_path)
    assert float(c_out[0][0, 0]) == 2048.0
    assert float(n_out[0][0, 0]) == 2048.0


# ---------------------------------------------------------------------------------------------------------
# fused patterns against closed forms / library routines
# ---------------------------------------------------------------------------------------------------------
def run_fixture_both(name, seed):
    path = os.path.join(FIXTURES, name + ".info")
    desc = harness.load_desc(path)
    inputs = harness.make_inputs(desc, seed=seed)
    c_out = cpu_ref.CpuKernel(path)([a.copy() for a in inputs])   # Assign ops overwrite their destination input
    n_out = np_ref.evaluate(desc, inputs)
    return desc, inputs, c_out, n_out


def test_elementwise_chain_matches_float64_closed_form():
    desc, (a, b, c), c_out, n_out = run_fixture_both("small_ew_tanh_add_mul_f32_7x33", 11)
    want = np.tanh((a.astype(np.float64) + b) * c)
    for got in (c_out[0], n_out[0]):
        assert np.allclose(got, want, rtol=1e-6, atol=1e-7)
    # a dropped or reordered term is far outside this tolerance
    assert not np.allclose(np.tanh(a.astype(np.float64) + b * c), want, rtol=1e-3, atol=1e-3)


def test_softmax_matches_scipy_and_its_invariants():
    from scipy.special import softmax
    desc, (x,), c_out, n_out = run_fixture_both("small_softmax_f16_33x1000", 12)
    want = softmax(x.astype(np.float64), axis=1)
    for got in (c_out[0], n_out[0]):
        g = got.astype(np.float64)
        assert np.allclose(g, want, rtol=2e-3, atol=1e-6)          # float16 output: 2^-11 relative
        assert np.allclose(g.sum(axis=1), 1.0, atol=2e-3)
        assert (g >= 0).all()
    # shift invariance: adding a per-row constant that is exact in float16 changes nothing but rounding
    shifted = (x.astype(np.float32) + np.float32(2.0)).astype(np.float16)
    path = os.path.join(FIXTURES, "small_softmax_f16_33x1000.info")
    again = cpu_ref.CpuKernel(path)([shifted])[0].astype(np.float64)
    assert np.allclose(again, want, rtol=6e-3, atol=1e-5)


def test_softmax_f32_matches_torch_float64():
    import torch
    desc, (x,), c_out, n_out = run_fixture_both("small_softmax_f32_5x77", 13)
    want = torch.softmax(torch.from_numpy(x).double(), dim=1).numpy()
    assert np.allclose(c_out[0], want, rtol=1e-5, atol=1e-9)
    assert np.allclose(n_out[0], want, rtol=1e-5, atol=1e-9)


def test_layernorm_residual_matches_torch_float64_and_invariants():
    import torch
    desc, (x, g, be, r), c_out, n_out = run_fixture_both("small_layernorm_residual_bf16_19x520", 14)
    xf, gf, bf, rf = (torch.from_numpy(harness.bf16_bits_to_f32(t)).double() for t in (x, g, be, r))
    want = (torch.nn.functional.layer_norm(xf, (520,), gf, bf, eps=1e-5) + rf).numpy()
    for got in (c_out[0], n_out[0]):
        gotf = harness.bf16_bits_to_f32(got).astype(np.float64)
        assert np.allclose(gotf, want, rtol=8e-3, atol=1e-6)        # bfloat16 output: 2^-8 relative
        # undo the affine part: rows must have mean ~0 and variance ~1
        z = (gotf - rf.numpy() - bf.numpy()) / gf.numpy()
        assert np.abs(z.mean(axis=1)).max() < 2e-2
        assert np.abs(z.var(axis=1) - 1.0).max() < 3e-2
    wrong_unbiased = torch.nn.functional.layer_norm(xf, (520,), gf, bf, eps=1e-5)
    assert not np.allclose(wrong_unbiased.numpy(), want, rtol=1e-2, atol=1e-2)   # dropping the residual is visible


def test_layernorm_float32_against_float64_tight(tmp_path):
    # the same pattern in float32 end to end, where a wrong epsilon or an N-1 divisor shows at 1e-6
    import torch
    text = op_desc.layernorm_residual(6, 64, "float32", eps=1e-5, name="ln_f32_6x64")
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6, 64)).astype(np.float32) * 1e-2     # small variance: epsilon matters
    g = rng.uniform(0.5, 1.5, 64).astype(np.float32)
    be = (rng.standard_normal(64) * 0.1).astype(np.float32)
    r = rng.standard_normal((6, 64)).astype(np.float32)
    _, c_out, n_out = build_and_run(text, [x, g, be, r], tmp_path)
    t = lambda a: torch.from_numpy(a).double()
    want = (torch.nn.functional.layer_norm(t(x), (64,), t(g), t(be), eps=1e-5) + t(r)).numpy()
    assert np.allclose(c_out[0], want, rtol=2e-6, atol=2e-6)
    assert np.allclose(n_out[0], want, rtol=2e-6, atol=2e-6)
    no_eps = (torch.nn.functional.layer_norm(t(x), (64,), t(g), t(be), eps=0.0) + t(r)).numpy()
    assert not np.allclose(no_eps, want, rtol=1e-4, atol=1e-4)
    unbiased = ((t(x) - t(x).mean(1, keepdim=True)) / (t(x).var(1, unbiased=True, keepdim=True) + 1e-5).sqrt() * t(g) + t(be) + t(r)).numpy()
    assert not np.allclose(unbiased, want, rtol=1e-4, atol=1e-4)


def test_rmsnorm_matches_float64_closed_form(tmp_path):
    # x * rsqrt(mean(x^2) + eps) * gamma in float32 end to end against float64: a mean subtracted by mistake (LayerNorm), a
    # sum in place of the mean, or epsilon outside the root all show at 1e-4 on small-variance rows
    text = op_desc.rmsnorm(6, 64, "float32", eps=1e-6, name="rms_f32_6x64")
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((6, 64)) * 1e-3 + 2e-3).astype(np.float32)      # small, not centred: epsilon and the mean matter
    g = rng.uniform(0.5, 1.5, 64).astype(np.float32)
    _, c_out, n_out = build_and_run(text, [x, g], tmp_path)
    xd, gd = x.astype(np.float64), g.astype(np.float64)
    want = xd / np.sqrt((xd * xd).mean(axis=1, keepdims=True) + 1e-6) * gd
    assert np.allclose(c_out[0], want, rtol=3e-6, atol=1e-9)
    assert np.allclose(n_out[0], want, rtol=3e-6, atol=1e-9)
    centred = (xd - xd.mean(1, keepdims=True)) / np.sqrt(xd.var(1, keepdims=True) + 1e-6) * gd
    no_eps = xd / np.sqrt((xd * xd).mean(axis=1, keepdims=True)) * gd
    summed = xd / np.sqrt((xd * xd).sum(axis=1, keepdims=True) + 1e-6) * gd
    for wrong in (centred, no_eps, summed):
        assert not np.allclose(wrong, want, rtol=1e-4, atol=1e-9)


def test_rmsnorm_fixtures_match_torch_float64_and_invariants():
    import torch
    desc, (x, g), c_out, n_out = run_fixture_both("small_rmsnorm_bf16_19x520", 15)
    xf, gf = (torch.from_numpy(harness.bf16_bits_to_f32(t)).double() for t in (x, g))
    want = torch.nn.functional.rms_norm(xf, (520,), gf, eps=1e-6).numpy()
    for got in (c_out[0], n_out[0]):
        gotf = harness.bf16_bits_to_f32(got).astype(np.float64)
        assert np.allclose(gotf, want, rtol=8e-3, atol=1e-6)              # bfloat16 output: 2^-8 relative
        z = gotf / gf.numpy()
        assert np.abs((z * z).mean(axis=1) - 1.0).max() < 2e-2           # rows have unit mean square
    # with the residual add in front: h = bf16(x + r) is an output and is what gets normalised
    desc, (x, g, r), c_out, n_out = run_fixture_both("small_rmsnorm_add_bf16_64x4096", 16)
    xf, gf, rf = (harness.bf16_bits_to_f32(t) for t in (x, g, r))
    h_bits = harness.f32_to_bf16_bits(xf + rf)
    hd = torch.from_numpy(harness.bf16_bits_to_f32(h_bits)).double()
    want = torch.nn.functional.rms_norm(hd, (4096,), torch.from_numpy(gf).double(), eps=1e-6).numpy()
    for outs in (c_out, n_out):
        assert np.array_equal(outs[0], h_bits)
        assert np.allclose(harness.bf16_bits_to_f32(outs[1]).astype(np.float64), want, rtol=8e-3, atol=1e-6)


def correctly_rounded_f32(fr):
    """Nearest float32 (ties to even) of an exact Fraction, by comparing against the neighbours' midpoints."""
    approx = np.float32(float(fr))
    cands = [np.nextafter(approx, np.float32(-np.inf)), approx, np.nextafter(approx, np.float32(np.inf))]
    best = min(cands, key=lambda c: (abs(Fraction(float(c)) - fr), int(np.float32(c).view(np.uint32)) & 1))
    return np.float32(best)


def test_quant_brute_force_with_exact_rationals(tmp_path):
    # tiny case, every quantity recomputed with exact rational arithmetic + explicit correct rounding
    rows, cols = 3, 8
    text = op_desc.quant_int8_residual(rows, cols, "bfloat16", name="quant_tiny")
    rng = np.random.default_rng(5)
    x = harness.f32_to_bf16_bits(rng.standard_normal((rows, cols)).astype(np.float32) * 3)
    r = harness.f32_to_bf16_bits(rng.standard_normal((rows, cols)).astype(np.float32))
    x[0, 0] = harness.f32_to_bf16_bits(np.array([50.0], dtype=np.float32))[0]        # an outlier
    _, c_out, n_out = build_and_run(text, [x, r], tmp_path)
    xf, rf = harness.bf16_bits_to_f32(x), harness.bf16_bits_to_f32(r)
    for i in range(rows):
        s = [correctly_rounded_f32(Fraction(float(xf[i, j])) + Fraction(float(rf[i, j]))) for j in range(cols)]
        amax = max(abs(Fraction(float(v))) for v in s)
        scale = correctly_rounded_f32(amax / 127)
        assert c_out[1][i] == scale and n_out[1][i] == scale
        for j in range(cols):
            q = correctly_rounded_f32(Fraction(float(s[j])) / Fraction(float(scale)))
            q = min(max(Fraction(float(q)), Fraction(-127)), Fraction(127))
            fl = q.numerator // q.denominator
            rem = q - fl
            n = fl + 1 if (rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1)) else fl
            assert int(c_out[0][i, j]) == n, (i, j)
            assert int(n_out[0][i, j]) == n, (i, j)


def test_quant_invariants_full_row_width():
    desc, (x, r), c_out, n_out = run_fixture_both("small_quant_int8_residual_bf16_64x8192", 15)
    assert np.array_equal(c_out[0], n_out[0]) and np.array_equal(c_out[1], n_out[1])
    q, scale = c_out
    s = harness.bf16_bits_to_f32(x) + harness.bf16_bits_to_f32(r)
    assert np.array_equal(np.abs(q.astype(np.int32)).max(axis=1), np.full(64, 127))      # absmax maps to +-127
    assert np.allclose(scale, np.abs(s).max(axis=1) / np.float32(127.0), rtol=1e-7)
    # dequantised value within half a step (plus division rounding) of the source
    assert (np.abs(q.astype(np.float64) * scale[:, None] - s) <= scale[:, None] * 0.5000001).all()


def test_int8_matmul_is_exact_integer_arithmetic(tmp_path):
    # brute force with Python integers on a tiny case whose products overflow int8 and int16
    b = op_desc.DescBuilder("mm_tiny")
    a_t = b.input([3, 5], "int8")
    b_t = b.input([5, 4], "int8")
    text = b.dumps([b.matmul(a_t, b_t, "int32")])
    a = np.array([[127, -127, 100, -100, 77], [1, 2, 3, 4, 5], [-128, -128, -128, -128, -128]], dtype=np.int8)
    bm = np.array([[127, 1, -1, 0], [-127, 2, -2, 0], [100, 3, -3, 0], [-100, 4, -4, 0], [77, 5, -5, 127]], dtype=np.int8)
    _, c_out, n_out = build_and_run(text, [a, bm], tmp_path)
    want = [[sum(int(a[i, k]) * int(bm[k, j]) for k in range(5)) for j in range(4)] for i in range(3)]
    assert c_out[0].tolist() == want
    assert n_out[0].tolist() == want
    assert want[0][0] == 127 * 127 + 127 * 127 + 100 * 100 + 100 * 100 + 77 * 77     # no narrow-type wraparound


def test_matmul_transpose_b_reads_b_as_n_by_k(tmp_path):
    b = op_desc.DescBuilder("mm_tb")
    a_t = b.input([2, 3], "int8")
    b_t = b.input([4, 3], "int8")
    text = b.dumps([b.matmul(a_t, b_t, "int32", transpose_b=True)])
    a = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.int8)
    bt = np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1]], dtype=np.int8)
    _, c_out, n_out = build_and_run(text, [a, bt], tmp_path)
    want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.int32)
    assert np.array_equal(c_out[0], want) and np.array_equal(n_out[0], want)


def test_gemm_dequant_bias_gelu_matches_torch_float64():
    import torch
    desc, (a, sa, w, sb, bias), c_out, n_out = run_fixture_both("small_gemm_i8_dequant_bias_gelu_256x512x256", 16)
    acc = torch.from_numpy(a).long() @ torch.from_numpy(w).long()
    x = acc.double() * torch.from_numpy(sa).double() * torch.from_numpy(sb).double() + \
        torch.from_numpy(harness.bf16_bits_to_f32(bias)).double()
    want = torch.nn.functional.gelu(x, approximate="tanh").numpy()
    for got in (c_out[0], n_out[0]):
        g = harness.bf16_bits_to_f32(got).astype(np.float64)
        assert np.allclose(g, want, rtol=8e-3, atol=1e-3)
    # per-row vs per-column scale mix-up would be visible
    wrong = torch.nn.functional.gelu(acc.double() * torch.from_numpy(sa).double().T * torch.from_numpy(sb).double()[:, None]
                                     + torch.from_numpy(harness.bf16_bits_to_f32(bias)).double(), approximate="tanh").numpy()
    assert not np.allclose(wrong, want, rtol=5e-2, atol=5e-2)


# ---------------------------------------------------------------------------------------------------------
# data-movement ops, outer-axis reductions, float MatMul
# ---------------------------------------------------------------------------------------------------------
def test_data_movement_chain_matches_plain_numpy(tmp_path):
    """pad -> tile -> strided slice (negative end) -> transpose, slice -> transpose, concat: written out with numpy's
    own pad / tile / slicing / concatenate. A padding pair applied to the wrong dimension, a perm read as its inverse,
    an `end` not counted from the back or a swapped concat order changes the result."""
    text = op_desc.view_chain("pin_view_chain")
    x = np.arange(35, dtype=np.float32).reshape(5, 7) + 1
    y = -(np.arange(270, dtype=np.float32).reshape(9, 30) + 1)
    _, c_out, n_out = build_and_run(text, [x, y], tmp_path)
    p = np.pad(x, ((3, 0), (1, 2)), constant_values=2)      # padding [1,2,3,0]: (1,2) on the last axis, (3,0) before it
    t = np.tile(p, (2, 3))
    s = t[1:15:2, :]                                        # begin 1, end -1 -> 15, stride 2
    expect = np.concatenate([s.T, y[2:6, :].T], axis=1) * np.float32(0.5)
    assert expect.shape == (30, 11)
    assert np.array_equal(c_out[0], expect) and np.array_equal(n_out[0], expect)


def test_transpose_perm_is_result_dim_from_operand_dim(tmp_path):
    """perm [2,0,1]: result dim d has the extent (and the index) of operand dim perm[d] (tosa.transpose), not the inverse."""
    b = op_desc.DescBuilder("pin_transpose_201")
    x = b.input([2, 3, 4], "int32")
    text = b.dumps([op_desc.transpose(b, x, [2, 0, 1])])
    data = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    _, c_out, n_out = build_and_run(text, [data], tmp_path)
    assert c_out[0].shape == (4, 2, 3)
    for i in range(4):
        for j in range(2):
            for k in range(3):
                assert c_out[0][i, j, k] == data[j, k, i] == n_out[0][i, j, k]


def test_outer_axis_reduction_visits_the_reduced_index_in_order(tmp_path):
    """ReduceSum over axis 0 in float16: per column, the running sum is rounded after every row (same rule as the row
    reduction, now with the reduced axis outermost). 4096 ones per column stall at 2048; a float32 accumulator or a
    pairwise order would give 4096."""
    b = op_desc.DescBuilder("pin_colsum_f16")
    x = b.input([4096, 3], "float16")
    text = b.dumps([b.reduce("ReduceSum", x, [0], False)])
    _, c_out, n_out = build_and_run(text, [np.ones((4096, 3), dtype=np.float16)], tmp_path)
    assert np.all(c_out[0] == 2048) and np.all(n_out[0] == 2048)
    # float32, all axes: the serial order is the row-major order of the operand
    b = op_desc.DescBuilder("pin_allsum_f32")
    x = b.input([3, 5], "float32")
    text = b.dumps([b.reduce("ReduceSum", x, [0, 1], False)])
    data = np.array([1e8, 1.0, -1e8, 1.0, 1.0] * 3, dtype=np.float32).reshape(3, 5)
    _, c_out, n_out = build_and_run(text, [data], tmp_path)
    acc = np.float32(0)
    for v in data.reshape(-1):
        acc = np.float32(acc + v)
    assert c_out[0][0] == acc == n_out[0][0] and acc != np.float32(data.astype(np.float64).sum())


def test_bf16_matmul_bias_gelu_matches_torch_float64():
    import torch
    name = "small_gemm_bf16_bias_gelu_256x512x256"
    desc, inputs, c_out, n_out = run_fixture_both(name, 23)
    a, w, bias = [torch.from_numpy(harness.bf16_bits_to_f32(x).astype(np.float64)) for x in inputs]
    ref = torch.nn.functional.gelu(a @ w + bias, approximate="tanh").numpy()
    for out in (c_out[0], n_out[0]):
        got = harness.bf16_bits_to_f32(out).astype(np.float64)
        assert np.allclose(got, ref, rtol=1e-2, atol=1e-3)
    # transposed B: the same numbers read as [N, K]
    desc, inputs, c_out, _ = run_fixture_both(name + "_tb", 23)
    a, w, bias = [torch.from_numpy(harness.bf16_bits_to_f32(x).astype(np.float64)) for x in inputs]
    ref = torch.nn.functional.gelu(a @ w.T + bias, approximate="tanh").numpy()
    assert np.allclose(harness.bf16_bits_to_f32(c_out[0]).astype(np.float64), ref, rtol=1e-2, atol=1e-3)


def test_gather_takes_rows_by_index_and_clamps(tmp_path):
    """Gather along axis 1 of a rank-3 tensor with rank-2 indices: result shape data[:1] + indices + data[2:], written
    out element by element; positions outside the axis are clamped (undefined in the reference)."""
    b = op_desc.DescBuilder("pin_gather_axis1")
    data = b.input([2, 5, 3], "int32")
    ind = b.input([2, 2], "int32")
    text = b.dumps([op_desc.gather(b, data, ind, 1)])
    x = np.arange(30, dtype=np.int32).reshape(2, 5, 3)
    idx = np.array([[4, 0], [7, -1]], dtype=np.int32)
    _, c_out, n_out = build_and_run(text, [x, idx], tmp_path)
    assert c_out[0].shape == (2, 2, 2, 3)
    for i in range(2):
        for j in range(2):
            for k in range(2):
                row = min(max(int(idx[j, k]), 0), 4)
                assert np.array_equal(c_out[0][i, j, k], x[i, row]) and np.array_equal(n_out[0][i, j, k], x[i, row])


def test_unsorted_segment_sum_adds_slices_in_index_order(tmp_path):
    """UnsortedSegmentSum against a dictionary of Python lists: every slice lands in the row its id names, rows no id
    names stay zero, and the additions happen in index order in the result's type. The order is pinned by a row that
    receives 1, 2^24 and -2^24 in that order: float32 gives 0 (1 + 2^24 rounds to 2^24), any other order gives 1.
    Ids outside [0, segments) are dropped (undefined in the reference)."""
    text = op_desc.unsorted_segment_sum([3, 2], [2], 5, "float32", name="pin_segment_sum")
    data = np.array([[[1, 10], [5, 50]], [[2.0 ** 24, 20], [7, 70]], [[-2.0 ** 24, 30], [9, 90]]], dtype=np.float32)
    ids = np.array([[2, 0], [2, 7], [2, -1]], dtype=np.int32)
    _, c_out, n_out = build_and_run(text, [data, ids], tmp_path)
    rows = {}
    for pos in range(6):
        sid = int(ids.reshape(-1)[pos])
        if 0 <= sid < 5:
            rows.setdefault(sid, []).append(data.reshape(6, 2)[pos])
    expect = np.zeros((5, 2), dtype=np.float32)
    for sid, parts in rows.items():
        acc = np.zeros(2, dtype=np.float32)
        for part in parts:
            acc = (acc + part).astype(np.float32)
        expect[sid] = acc
    assert expect[2, 0] == 0.0 and expect[2, 1] == 60.0 and expect[0, 0] == 5.0
    assert np.array_equal(c_out[0], expect) and np.array_equal(np.asarray(n_out[0]).reshape(5, 2), expect)
    # bfloat16 accumulates in bfloat16: 256 ones in one row stop growing at 256 (257 is not representable)
    text = op_desc.unsorted_segment_sum([300], [1], 2, "bfloat16", name="pin_segment_sum_bf16")
    ones = harness.f32_to_bf16_bits(np.ones((300, 1), dtype=np.float32))
    _, c_out, n_out = build_and_run(text, [ones, np.zeros(300, dtype=np.int32)], tmp_path)
    assert harness.bf16_bits_to_f32(c_out[0]).reshape(-1).tolist() == [256.0, 0.0]
    assert harness.bf16_bits_to_f32(n_out[0]).reshape(-1).tolist() == [256.0, 0.0]


def test_split_gives_consecutive_pieces_along_the_axis(tmp_path):
    """Split into three unequal pieces along axis 1 against numpy's split; each piece goes through an op of its own so
    that a swapped or shifted piece shows. (The reference translates Split but has no lowering for it.)"""
    b = op_desc.DescBuilder("pin_split")
    x = b.input([3, 10, 2], "float32")
    p0, p1, p2 = op_desc.split(b, x, [2, 5, 3], 1)
    text = b.dumps([b.unary("Neg", p0), b.mul(p1, b.const(3.0, "float32")), b.unary("Abs", p2)])
    data = np.arange(60, dtype=np.float32).reshape(3, 10, 2) - 17.0
    _, c_out, n_out = build_and_run(text, [data], tmp_path)
    a0, a1, a2 = np.split(data, [2, 7], axis=1)
    for got in (c_out, n_out):
        assert np.array_equal(np.asarray(got[0]).reshape(a0.shape), -a0)
        assert np.array_equal(np.asarray(got[1]).reshape(a1.shape), a1 * 3.0)
        assert np.array_equal(np.asarray(got[2]).reshape(a2.shape), np.abs(a2))


def test_argmax_takes_the_first_greatest_element_and_never_a_nan(tmp_path):
    """ArgMax against numpy.argmax on rows without NaN (numpy also takes the first of equal maxima), and the cases
    upstream's lowering of tosa.argmax fixes: NaN is never taken, a row of -inf or of NaN only gives 0 (nothing is
    greater than the lowest finite value it starts with)."""
    b = op_desc.DescBuilder("pin_argmax")
    x = b.input([6, 7], "float32")
    text = b.dumps([op_desc.argmax(b, x, 1)])
    inf, nan = np.inf, np.nan
    data = np.array([[1, 5, 3, 5, 0, -2, 5],            # three equal maxima: the first
                     [nan, 2, 9, nan, 9, 1, 0],         # NaN skipped, first 9
                     [-inf] * 7,                        # nothing above the lowest finite value
                     [nan] * 7,
                     [-3, -2, -1, -0.5, -7, -0.5, -9],  # negative values
                     [0, 0, 0, 0, 0, 0, inf]], dtype=np.float32)
    _, c_out, n_out = build_and_run(text, [data], tmp_path)
    expect = [1, 2, 0, 0, 3, 6]
    assert c_out[0].tolist() == expect and np.asarray(n_out[0]).reshape(-1).tolist() == expect
    rng = np.random.default_rng(9)
    b = op_desc.DescBuilder("pin_argmax_axis0")
    x = b.input([50, 4, 9], "float32")
    text = b.dumps([op_desc.argmax(b, x, 0, keep_dims=True, dtype="int64")])
    data = rng.integers(-5, 6, size=(50, 4, 9)).astype(np.float32)       # many ties
    _, c_out, n_out = build_and_run(text, [data], tmp_path)
    want = np.argmax(data, axis=0).reshape(1, 4, 9)
    assert np.array_equal(c_out[0], want) and np.array_equal(np.asarray(n_out[0]).reshape(1, 4, 9), want)


def test_assign_writes_the_value_over_its_first_operand(tmp_path):
    """Momentum step in float32 against the formula written out in numpy: v <- 0.9 v + g, p <- p - 0.01 v. The C
    restatement updates the caller's input arrays in place, the numpy one reports the updates."""
    text = op_desc.momentum_update(5, 9, "float32", name="pin_momentum")
    rng = np.random.default_rng(5)
    p0, v0, g0 = (rng.standard_normal((5, 9), dtype=np.float32) for _ in range(3))
    ins = [p0.copy(), v0.copy(), g0.copy()]
    updates = {}
    n_out = np_ref.evaluate(json.loads(text), [p0, v0, g0], updates)
    _, c_out, _ = build_and_run(text, ins, tmp_path)
    v1 = (np.float32(0.9) * v0 + g0).astype(np.float32)
    p1 = (p0 - np.float32(0.01) * v1).astype(np.float32)
    assert np.array_equal(ins[1], v1) and np.array_equal(ins[0], p1) and np.array_equal(ins[2], g0)
    assert np.array_equal(updates[1], v1) and np.array_equal(updates[0], p1) and sorted(updates) == [0, 1]
    assert np.array_equal(c_out[0], v1) and np.array_equal(c_out[1], p1)
    assert np.array_equal(n_out[0], v1) and np.array_equal(n_out[1], p1)


def test_assign_after_a_reduction_updates_running_statistics(tmp_path):
    """Batch-norm statistics with the running mean and variance assigned from them, against numpy's own mean and var
    over (N, H, W) in float64: a reduction over the wrong axes, a biased/unbiased mix-up or swapped momentum weights
    would each show."""
    text = op_desc.batchnorm_stats_update(6, 5, 4, 7, "float32", momentum=0.9, name="pin_bn_update")
    rng = np.random.default_rng(17)
    x = rng.standard_normal((6, 5, 4, 7), dtype=np.float32) * 2 + 1
    rm, rv = rng.standard_normal(5, dtype=np.float32), rng.random(5, dtype=np.float32) + 0.5
    ins = [x.copy(), rm.copy(), rv.copy()]
    updates = {}
    n_out = np_ref.evaluate(json.loads(text), [x, rm, rv], updates)
    _, c_out, _ = build_and_run(text, ins, tmp_path)
    mean, var = x.astype(np.float64).mean(axis=(0, 2, 3)), x.astype(np.float64).var(axis=(0, 2, 3))
    want = [mean, var, 0.9 * rm + 0.1 * mean, 0.9 * rv + 0.1 * var]
    for got_c, got_n, w in zip(c_out, n_out, want):
        assert np.allclose(got_c, w, rtol=2e-5, atol=2e-5) and np.allclose(np.asarray(got_n), w, rtol=2e-5, atol=2e-5)
    assert np.array_equal(ins[1], c_out[2]) and np.array_equal(ins[2], c_out[3]) and np.array_equal(ins[0], x)
    assert sorted(updates) == [1, 2] and np.allclose(updates[1], want[2], rtol=2e-5, atol=2e-5)


def test_batch_matmul_is_one_product_per_batch_index():
    """BatchMatMul against torch float64 bmm: batches must not mix and transpose_b must read [batch, n, k]."""
    import torch
    for name, tb, dt in (("small_batchmatmul_scale_mask_bf16_3x200x64x136_tb", True, "bfloat16"),
                         ("small_batchmatmul_scale_mask_f16_2x256x128x256", False, "float16")):
        desc, inputs, c_out, n_out = run_fixture_both(name, 24)
        q, k, mask = (torch.from_numpy(harness.to_float(x, d)) for x, d in zip(inputs, (dt, dt, "float32")))
        ref = (torch.bmm(q, k.transpose(1, 2) if tb else k) / (q.shape[-1] ** 0.5) + mask).numpy()
        for out in (c_out[0], n_out[0]):
            assert np.allclose(harness.to_float(out, dt), ref, rtol=1e-2, atol=1e-3)


# ---------------------------------------------------------------------------------------------------------
# the two restatements against each other on every small fixture
# ---------------------------------------------------------------------------------------------------------
SMALL = sorted(f[:-5] for f in os.listdir(FIXTURES) if f.startswith("small_") and f.endswith(".info"))


@pytest.mark.parametrize("name", SMALL)
def test_c_and_numpy_restatements_agree(name):
    desc, inputs, c_out, n_out = run_fixture_both(name, 21)
    for d, a, b in zip(desc["output_desc"], c_out, n_out):
        ok, msg = harness.compare(a, b, d["data_type"])
        assert ok, "%s %s: %s" % (name, d["tensor_name"], msg)
        if name.startswith("small_quant") or name.startswith("small_layernorm"):
            # no transcendental function involved: the two must agree bit for bit
            assert np.array_equal(a, b)


def test_openmp_build_is_bit_identical_to_serial():
    path = os.path.join(FIXTURES, "small_layernorm_residual_bf16_64x4096.info")
    inputs = harness.make_inputs(harness.load_desc(path), seed=22)
    serial = cpu_ref.CpuKernel(path)(inputs)
    par = cpu_ref.CpuKernel(path, openmp=True)(inputs)
    assert np.array_equal(serial[0], par[0])


def test_generated_c_uses_the_packed_pointer_abi():
    with open(os.path.join(FIXTURES, "small_quant_int8_residual_bf16_37x1544.info"), "r", encoding="utf-8") as f:
        src = gen_cpu.generate_c(json.load(f))
    assert "void small_quant_int8_residual_bf16_37x1544(void **packed)" in src
    # inputs first, then outputs
    assert src.index("packed[0]") < src.index("packed[1]") < src.index("packed[2]") < src.index("packed[3]")
