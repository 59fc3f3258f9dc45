"""The known-answer vectors of tests/known_answers.py through the HIP kernels (launched through the C ABI): ties and
saturation of float -> int8 (also inside the fused clamp + cast of the per-token quantisation), 16-bit rounding, a row of
-inf under ReduceMax, NaN / +-inf / +-0 through the math ops, ordered and signed comparisons, integer division and its two
corner values, AddN's order, Pow / Atan2, Asinh / Acosh in the reference's spelling. Seeded N(0,1) data almost never lands
on these points, so they are pushed through the device code one by one and held to the table and to the oracle."""
import json
import os

import numpy as np
import pytest

import known_answers
from akg_amd import driver, harness
from oracle import cpu_ref

pytestmark = pytest.mark.gpu

_KAT = {c["name"]: c for c in known_answers.cases()}


@pytest.mark.parametrize("name", sorted(_KAT))
def test_known_answer_vectors_through_the_hip_kernels(name, tmp_path):
    from test_gpu_parity import run_on_gpu
    case = _KAT[name]
    desc = json.loads(case["text"])
    path = os.path.join(str(tmp_path), desc["op"] + ".info")
    with open(path, "w", encoding="utf-8") as f:
        f.write(case["text"])
    kernel = driver.HipKernel(case["text"], out_dir=None)
    print("case %s: %s grid %d block %d" % (name, kernel.family, kernel.grid[0], kernel.block[0]), flush=True)
    got = run_on_gpu(kernel, case["inputs"])
    ok, msg = known_answers.check(case, got)
    print("  against the table: %s" % msg, flush=True)
    assert ok, "%s: %s" % (name, msg)
    # and against the oracle on the same vectors: NaN in the same places, everything else to the bar of its type
    expect = cpu_ref.CpuKernel(path, rebuild=True)(case["inputs"])
    for d, g, e in zip(kernel.outputs, got, expect):
        ok, msg = harness.compare(g, e, d.dtype)
        print("  %s %s against the oracle: %s" % (d.name, d.dtype, msg), flush=True)
        assert ok, "%s output %s: %s" % (name, d.name, msg)
