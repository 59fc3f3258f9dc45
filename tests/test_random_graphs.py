"""Differential tests on seeded random fused-op descriptions (tests/random_graphs.py).

CPU half: every description translates, lowers and compiles for gfx950 (no GPU needed), and the two oracle
restatements agree on it. GPU half: the kernel's results against the C oracle, to the usual bars.
"""
import json
import os

import numpy as np
import pytest

from akg_amd import driver, harness
from oracle import cpu_ref, np_ref
from random_graphs import random_description, random_int8_matmul_description, random_matmul_description, random_optable_description

# AKG_RANDOM_GRAPHS=N widens the sweep for a one-off soak on the CPU oracle / a GPU box
SEEDS = list(range(1, 1 + int(os.environ.get("AKG_RANDOM_GRAPHS", "40"))))


def _write(tmp_path, text):
    desc = json.loads(text)
    path = os.path.join(str(tmp_path), desc["op"] + ".info")
    with open(path, "w", encoding="utf-8") as f:
        f.write(text)
    return desc, path


def _terms(desc):
    """Largest number of elements a reduction of the description folds into one result (1 if none)."""
    shapes = {e[0]["tensor_name"]: e[0].get("shape", [1]) for e in desc["input_desc"]}
    worst = 1
    for od in desc["op_desc"]:
        out = od["output_desc"][0]
        shapes[out["tensor_name"]] = out.get("shape", [1])
        if od["name"].startswith("Reduce"):
            src = od["input_desc"][0][0].get("shape", [1])
            worst = max(worst, int(np.prod(src)) // max(1, int(np.prod(out.get("shape", [1])))))
    return worst


@pytest.mark.parametrize("seed", SEEDS[:16])
def test_random_description_compiles_and_oracles_agree(seed, tmp_path):
    text, notes = random_description(seed)
    desc, path = _write(tmp_path, text)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family in ("elementwise", "row_reduce", "stream_reduce", "indexed", "staged"), notes
    inputs = harness.make_inputs(desc, seed=seed)
    c_out = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    n_out = np_ref.evaluate(desc, inputs)
    for d, a, b in zip(desc["output_desc"], c_out, n_out):
        ok, msg = harness.compare(a, b, d["data_type"])
        assert ok, "seed %d %s (%s): %s" % (seed, d["tensor_name"], " ".join(notes), msg)


INEXACT = ("Exp", "Tanh", "Sqrt", "Rsqrt", "Reciprocal", "RealDiv", "Log", "Sin", "Cos", "ASin", "ACos", "Atan", "Asinh",
           "Acosh", "Pow", "Atan2")


def compare_with_oracle(kernel, desc, notes, inputs, got, expect, seed):
    """Bars of the GPU half: bool / integer / 16-bit outputs by `harness.compare`; float32 outputs to rtol 1e-5 plus what
    the conditioning of the description itself allows (see the comments inside)."""
    terms = _terms(desc)
    wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
    exact = np_ref.evaluate(harness.widen_to_float64(desc), wide)
    for d, g, e, x in zip(kernel.outputs, got, expect, exact):
        if d.dtype == "float32" and terms > 1 and any(n.startswith("ReduceSum") for n in notes):
            # float32 sums are reassociated on the GPU: hold them to the float64 value instead of the serial order
            ok, msg = harness.compare_reassociated(g, x, d.dtype, terms)
        elif d.dtype == "float32":
            # rtol 1e-5, plus what the float32 oracle itself loses against the float64 evaluation at that element:
            # after a subtraction of nearly equal tanh / exp values two correct float32 evaluations differ by that much
            e64 = np.asarray(x, dtype=np.float64).reshape(e.shape)
            slack = 16.0 * np.abs(e.astype(np.float64) - e64)
            if any(n in INEXACT for n in notes):
                # the device's transcendental functions (and its hardware square roots and reciprocals where relaxed)
                # are good to an ulp or two of their own results, which here are of the inputs' order of magnitude
                # (operands are clipped in front of them); a subtraction of two such values keeps that absolute
                # error however small its result is, and the oracle may happen to be exact at that element
                scale = max([1.0] + [float(np.max(np.abs(a.astype(np.float64)))) for a in inputs if a.dtype.kind == "f" and a.size])
                slack = slack + 2.0 * float(np.finfo(np.float32).eps) * scale
            with np.errstate(invalid="ignore"):
                bad = np.abs(g.astype(np.float64) - e.astype(np.float64)) > 1e-5 * np.abs(e) + 1e-8 + slack
            bad &= ~(np.isnan(g) & np.isnan(e))
            bad &= ~(np.isinf(g) & (g == e))
            ok, msg = not bad.any(), "%d of %d elements outside rtol 1e-5 + conditioning slack" % (bad.sum(), bad.size)
        else:
            ok, msg = harness.compare(g, e, d.dtype)
        print("  %s %s %s: %s" % (kernel.family, d.name, d.dtype, msg), flush=True)
        assert ok, "seed %d (%s) output %s: %s" % (seed, " ".join(notes), d.name, msg)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", SEEDS)
def test_random_description_matches_oracle_on_gpu(seed, tmp_path):
    from test_gpu_parity import run_on_gpu
    text, notes = random_description(seed)
    desc, path = _write(tmp_path, text)
    print("seed %d: %s" % (seed, " ".join(notes)), flush=True)
    kernel = driver.HipKernel(text, out_dir=None)
    inputs = harness.make_inputs(desc, seed=seed)
    got = run_on_gpu(kernel, inputs)
    expect = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    compare_with_oracle(kernel, desc, notes, inputs, got, expect, seed)


MATMUL_SEEDS = list(range(1, 1 + int(os.environ.get("AKG_RANDOM_MATMULS", "40"))))


@pytest.mark.parametrize("seed", MATMUL_SEEDS[:12])
def test_random_matmul_description_compiles(seed):
    text, notes = random_matmul_description(seed)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family in ("gemm_epilogue", "staged"), notes
    assert "gemm_" in kernel.source


@pytest.mark.gpu
@pytest.mark.parametrize("seed", MATMUL_SEEDS)
def test_random_matmul_description_matches_oracle_on_gpu(seed, tmp_path):
    from test_gpu_parity import run_on_gpu
    text, notes = random_matmul_description(seed)
    desc, path = _write(tmp_path, text)
    print("seed %d: %s" % (seed, " ".join(notes)), flush=True)
    kernel = driver.HipKernel(text, out_dir=None)
    inputs = harness.make_inputs(desc, seed=seed)
    got = run_on_gpu(kernel, inputs)
    expect = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    for d, g, e in zip(kernel.outputs, got, expect):
        ok, msg = harness.compare(g, e, d.dtype)
        print("  %s %s %s: %s" % (kernel.family, d.name, d.dtype, msg), flush=True)
        assert ok, "seed %d (%s) output %s: %s" % (seed, " ".join(notes), d.name, msg)


INT8_MATMUL_SEEDS = list(range(1, 1 + int(os.environ.get("AKG_RANDOM_INT8_MATMULS", "30"))))


@pytest.mark.parametrize("seed", INT8_MATMUL_SEEDS[:12])
def test_random_int8_matmul_description_compiles_and_oracles_agree(seed, tmp_path):
    text, notes = random_int8_matmul_description(seed)
    desc, path = _write(tmp_path, text)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family in ("gemm_epilogue", "staged"), notes
    inputs = harness.make_inputs(desc, seed=seed)
    c_out = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    n_out = np_ref.evaluate(desc, inputs)
    for d, a, b in zip(desc["output_desc"], c_out, n_out):
        ok, msg = harness.compare(a, b, d["data_type"])
        assert ok, "seed %d (%s) output %s: the two oracles disagree: %s" % (seed, " ".join(notes), d["tensor_name"], msg)
    if notes[2] in ("bare", "both"):
        # the accumulators against Python integers on a few elements: exact, whatever the machine arithmetic
        a, w = inputs[0].astype(object), inputs[1].astype(object)
        if notes[1] == "tb":
            w = w.T
        for (i, j) in [(0, 0), (a.shape[0] - 1, w.shape[1] - 1), (a.shape[0] // 2, w.shape[1] // 3)]:
            assert int(c_out[0][i, j]) == int(sum(a[i, :] * w[:, j]))


@pytest.mark.gpu
@pytest.mark.parametrize("seed", INT8_MATMUL_SEEDS)
def test_random_int8_matmul_description_matches_oracle_on_gpu(seed, tmp_path):
    """int32 accumulators bit for bit (harness.compare holds integer outputs to equality), the dequantised results to the
    bar of their type."""
    from test_gpu_parity import run_on_gpu
    text, notes = random_int8_matmul_description(seed)
    desc, path = _write(tmp_path, text)
    print("seed %d: %s" % (seed, " ".join(notes)), flush=True)
    kernel = driver.HipKernel(text, out_dir=None)
    inputs = harness.make_inputs(desc, seed=seed)
    got = run_on_gpu(kernel, inputs)
    expect = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    for d, g, e in zip(kernel.outputs, got, expect):
        ok, msg = harness.compare(g, e, d.dtype)
        print("  %s %s %s: %s" % (kernel.family, d.name, d.dtype, msg), flush=True)
        assert ok, "seed %d (%s) output %s: %s" % (seed, " ".join(notes), d.name, msg)


OPTABLE_SEEDS = list(range(1, 1 + int(os.environ.get("AKG_RANDOM_OPTABLE", "40"))))


@pytest.mark.parametrize("seed", OPTABLE_SEEDS[:16])
def test_random_optable_description_compiles_and_oracles_agree(seed, tmp_path):
    text, notes = random_optable_description(seed)
    desc, path = _write(tmp_path, text)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family in ("elementwise", "row_reduce", "stream_reduce", "staged"), notes
    inputs = harness.make_inputs(desc, seed=seed)
    c_out = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    n_out = np_ref.evaluate(desc, inputs)
    for d, a, b in zip(desc["output_desc"], c_out, n_out):
        if d["data_type"] == "float32":
            # libm against numpy's vectorised float32 functions: an ulp or two of values of the operands' magnitude
            with np.errstate(invalid="ignore"):
                bad = np.abs(a.astype(np.float64) - b.astype(np.float64)) > 1e-5 * np.abs(b) + 4e-6
            bad &= ~(np.isnan(a) & np.isnan(b)) & ~(np.isinf(a) & (a == b))
            ok, msg = not bad.any(), "%d of %d elements apart" % (bad.sum(), bad.size)
        else:
            ok, msg = harness.compare(a, b, d["data_type"])
        assert ok, "seed %d %s (%s): %s" % (seed, d["tensor_name"], " ".join(notes), msg)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", OPTABLE_SEEDS)
def test_random_optable_description_matches_oracle_on_gpu(seed, tmp_path):
    from test_gpu_parity import run_on_gpu
    text, notes = random_optable_description(seed)
    desc, path = _write(tmp_path, text)
    print("seed %d: %s" % (seed, " ".join(notes)), flush=True)
    kernel = driver.HipKernel(text, out_dir=None)
    inputs = harness.make_inputs(desc, seed=seed)
    got = run_on_gpu(kernel, inputs)
    expect = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    compare_with_oracle(kernel, desc, notes, inputs, got, expect, seed)
