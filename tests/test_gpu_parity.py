"""GPU parity: every fused kernel, launched through the C ABI on device-resident buffers, against the CPU oracle
(the C restatement of the reference CPU pipeline) on the same seeded inputs.

Bars: int8 / integer outputs bit-exact; float32 rtol 1e-5 (atol 1e-8); float16 / bfloat16 rtol 1e-2, atol 1e-3.
Outputs are NaN-prefilled on the device so that an element the kernel does not write fails the comparison.
"""
import glob
import os

import numpy as np
import pytest

from akg_amd import driver, harness, op_desc
from dynamic_cases import DYNAMIC_COLUMNS, DYNAMIC_POOLS, DYNAMIC_STATS, DYNAMIC_STREAMS, DYNAMIC_VIEWS, open_extent
from oracle import cpu_ref

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FIXTURES = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "akg_amd", "fixtures")
STREAM_MARKS = ("reducey", "reduceall", "reducex_long", "biasgrad", "sub_exp_reducesum", "mean_absmax_all", "bnstats")
ALL_SMALL = sorted(os.path.basename(p) for p in glob.glob(os.path.join(FIXTURES, "small_*.info")))
STAGED = [n for n in ALL_SMALL if "_staged_" in n]
SMALL = [n for n in ALL_SMALL if not any(m in n for m in STREAM_MARKS) and "segment_sum" not in n and n not in STAGED
         and "sgdclip" not in n]
STREAM = [n for n in ALL_SMALL if any(m in n for m in STREAM_MARKS) and "bnstats_update" not in n and n not in STAGED]
FULL = ["c1_ew_tanh_add_mul_f32_1024x4096.info", "c2_softmax_f16_8192x4096.info",
        "c3_layernorm_residual_bf16_16384x4096.info", "c4_quant_int8_residual_bf16_32768x8192.info",
        "n10_rmsnorm_bf16_16384x4096.info", "n11_rmsnorm_add_bf16_16384x4096.info"]


def _torch_view(a):
    import torch
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16))
    return torch.from_numpy(a)


def run_on_gpu(kernel, inputs):
    """Upload, launch through akg_hip_launch, download. Outputs start as NaN / 0x7F bytes."""
    import torch
    dev = torch.device("cuda:0")
    ins = [_torch_view(a).to(dev) for a in inputs]
    outs = []
    for d in kernel.outputs:
        t = torch.empty(d.nbytes, dtype=torch.uint8, device=dev)
        t.fill_(0xFF if d.dtype in ("float16", "bfloat16", "float32", "float64") else 0x7B)
        outs.append(t)
    kernel.launch(ins + outs)
    torch.cuda.synchronize()
    return [o.cpu().numpy().view(driver.NP_HOST_DTYPE[d.dtype]).reshape(d.shape) for d, o in zip(kernel.outputs, outs)]


def check_fixture(name, seed, openmp):
    path = os.path.join(FIXTURES, name)
    print("case %s seed %d" % (name, seed), flush=True)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    inputs = harness.make_inputs(desc, seed=seed)
    got = run_on_gpu(kernel, inputs)
    expect = cpu_ref.CpuKernel(path, openmp=openmp)(inputs)
    # the per-token quantisation states both of its outputs as bit-exact: the int8 values and the float32 scales
    bits = "quant_int8" in name
    for d, g, e in zip(kernel.outputs, got, expect):
        ok, msg = harness.compare_bits(g, e, d.dtype) if bits else harness.compare(g, e, d.dtype)
        print("  %s %s: %s" % (d.name, d.dtype, msg), flush=True)
        assert ok, "%s output %s: %s" % (name, d.name, msg)


@pytest.mark.parametrize("name", SMALL)
def test_small_fixture_matches_oracle(name):
    check_fixture(name, seed=harness.BASE_SEED + 100, openmp=False)


def check_stream_reduction(path, seed, repeats=1, family="stream_reduce"):
    """Streaming reductions (direction Y / ALL, long rows) combine partial results of many workgroups, so float sums
    are reassociated. Outputs that do not come from a float sum (max / min, the unreduced outputs, 16-bit results)
    are held to the usual bars against the serial oracle; float32 sums are held to rtol 1e-5 against the float64
    evaluation of the same description, and the serial float32 oracle is shown for scale. The kernel is launched
    `repeats` times on the same handle: every launch must leave the workspace ready for the next."""
    from oracle import np_ref
    print("case %s seed %d" % (os.path.basename(path), seed), flush=True)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    assert family is None or kernel.family == family
    inputs = harness.make_inputs(desc, seed=seed)
    serial = cpu_ref.CpuKernel(path)(inputs)
    wide_inputs = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
    exact = np_ref.evaluate(harness.widen_to_float64(desc), wide_inputs)
    in_numel = max(int(np.prod(e[0].get("shape", [1]))) for e in desc["input_desc"])
    has_sum = any(o["name"] in ("ReduceSum", "ReducePrd") for o in desc["op_desc"])
    for rep in range(repeats):
        got = run_on_gpu(kernel, inputs)
        for d, g, e, x in zip(kernel.outputs, got, serial, exact):
            terms = max(1, in_numel // max(1, g.size))
            if d.dtype == "float32" and has_sum and g.size < in_numel:
                ok, msg = harness.compare_reassociated(g, x, d.dtype, terms)
                gap = float(np.max(np.abs(np.asarray(e, dtype=np.float64) - np.asarray(x).reshape(e.shape))))
                msg += " (serial float32 oracle is %.3g away from float64)" % gap
            else:
                ok, msg = harness.compare(g, e, d.dtype)
            print("  launch %d %s %s: %s" % (rep, d.name, d.dtype, msg), flush=True)
            assert ok, "%s output %s: %s" % (os.path.basename(path), d.name, msg)


# a softmax / LayerNorm over ONE outer axis: the column kernel keeps the reduced run in registers (one kernel, one read)
COLUMN = [n for n in STAGED if "softmax" in n or "layernorm" in n]


@pytest.mark.parametrize("name,schedule", [(n, "default") for n in STAGED] + [(n, "several_kernels") for n in COLUMN])
def test_descriptions_cut_into_several_kernels_match_the_oracle(name, schedule, monkeypatch, tmp_path):
    """A softmax or a normalisation over an outer axis, batch-norm statistics and their use in one description: the
    streaming reductions cannot serve them. One reduced axis whose run fits a workgroup's registers goes to the column
    kernel (one kernel); otherwise, or when asked for, the handle runs one kernel per reduction level (temporaries in
    its workspace). float32 results against the float64 evaluation (the sums are reassociated), 16-bit ones against the
    serial oracle; three launches of one handle."""
    from oracle import np_ref
    path = os.path.join(FIXTURES, name)
    desc = harness.load_desc(path)
    if schedule == "several_kernels":
        monkeypatch.setenv("AKG_HIP_VARIANT", "7")
    kernel = driver.HipKernel.from_file(path, out_dir=str(tmp_path))
    print("case %s %s: %s grid %d block %d" % (name, schedule, kernel.family, kernel.grid[0], kernel.block[0]), flush=True)
    if name in COLUMN and schedule == "default":
        assert kernel.family == "column_reduce" and kernel.source.count("extern \"C\" __global__") == 1 and kernel.workspace_bytes == 0
    else:
        assert kernel.family == "staged" and kernel.source.count("extern \"C\" __global__") >= 2
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 730)
    serial = cpu_ref.CpuKernel(path)(inputs)
    wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
    exact = np_ref.evaluate(harness.widen_to_float64(desc), wide)
    in_numel = max(int(np.prod(e[0].get("shape", [1]))) for e in desc["input_desc"])
    terms = max(1, in_numel // min(int(np.prod(d.shape)) for d in kernel.outputs))
    for launch in range(3):
        got = run_on_gpu(kernel, inputs)
        for d, g, e, x in zip(kernel.outputs, got, serial, exact):
            if d.dtype == "float32":
                ok, msg = harness.compare_reassociated(g, x, d.dtype, max(terms, 64))
            else:
                ok, msg = harness.compare(g, e, d.dtype)
            print("  launch %d %s %s: %s" % (launch, d.name, d.dtype, msg), flush=True)
            assert ok, "%s output %s: %s" % (name, d.name, msg)
    # the reference-style call on host buffers and the timing call go through the same sequence of kernels
    host_outs = kernel.empty_outputs()
    kernel.run_host([np.ascontiguousarray(a) for a in inputs] + host_outs)
    for g, h in zip(got, host_outs):
        assert np.array_equal(np.ascontiguousarray(g).view(np.uint8), h.view(np.uint8))


def _column_cases():
    """name -> (builder function, family expected)"""
    def l2_normalise_no_keep(b):
        # x / sqrt(sum(x * x) over axis 1): the reduction drops its axis and a Reshape puts it back
        x = b.input([6, 37, 50], "float32")
        ss = b.reduce("ReduceSum", b.mul(x, x), [1], False)
        return [b.div(x, b.unary("Sqrt", b.reshape(ss, [6, 1, 50])))]

    def centred_with_statistics(b):
        # three outputs: the centred tensor, the mean [4,1,9,8] and the greatest centred value per column
        x = b.input([4, 23, 9, 8], "float16")
        xf = b.cast(x, "float32")
        mean = b.mul(b.reduce("ReduceSum", xf, [1], True), b.const(1.0 / 23, "float32"))
        xc = b.sub(xf, mean)
        return [b.cast(xc, "float16"), mean, b.reduce("ReduceMax", xc, [1], True)]

    def scaled_by_a_shared_plane(b):
        # an operand [1, 19, 6] that every outer index shares, one value per outer index [7,1,1], an inner axis of 6
        x = b.input([7, 19, 6], "float32")
        w = b.input([1, 19, 6], "float32")
        g = b.input([7, 1, 1], "float32")
        y = b.mul(b.mul(x, w), g)
        return [b.sub(y, b.reduce("ReduceMin", y, [1], True))]

    def integer_range(b):
        x = b.input([3, 130, 20], "int32")
        lo, hi = b.reduce("ReduceMin", x, [1], True), b.reduce("ReduceMax", x, [1], True)
        return [b.sub(x, lo), b.sub(hi, lo)]

    def narrow_columns(b):
        # two columns only: the threads of a wavefront that share a column are 2, 4, ... 32 lanes apart
        x = b.input([5, 300, 2], "float32")
        return [b.div(x, b.reduce("ReduceSum", b.unary("Abs", x), [1], True))]

    def half_sums(b):
        # the sum is declared float16: rounded after every addition, in index order, as the oracle's serial loop
        x = b.input([2, 40, 24], "float16")
        return [b.sub(x, b.reduce("ReduceMax", x, [1], True)), b.reduce("ReduceSum", x, [1], True)]

    def no_keep_meets_the_tensor_unreshaped(b):
        # the [5,5] result of a reduction over the middle axis used directly against [5,5,5]: broadcasting aligns it on
        # the right (as rows and columns of every outer index), which is not the column kernel's business
        x = b.input([5, 5, 5], "float32")
        return [b.sub(x, b.reduce("ReduceMax", x, [1], False))]

    def run_too_long_for_registers(b):
        x = b.input([2, 20000, 64], "float32")
        return [b.sub(x, b.reduce("ReduceMax", x, [1], True))]

    def several_strips_per_workgroup(b):
        # 16 x 35 strips of 44 resident registers a thread: 256 workgroups stay and take two or three strips each, the
        # next one's chunks on their way while this one is worked on; 1101 columns end inside a chunk, 700 rows inside
        # the last round of a thread's rows. Softmax over the middle axis, a weight per row of the run beside it.
        x = b.input([16, 700, 1101], "float32")
        w = b.input([700, 1], "float32")
        e = b.unary("Exp", b.sub(x, b.reduce("ReduceMax", x, [1], True)))
        return [b.mul(b.div(e, b.reduce("ReduceSum", e, [1], True)), w)]

    return {"l2_normalise_no_keep": (l2_normalise_no_keep, "column_reduce"), "centred_with_statistics": (centred_with_statistics, "column_reduce"),
            "several_strips_per_workgroup": (several_strips_per_workgroup, "column_reduce"),
            "scaled_by_a_shared_plane": (scaled_by_a_shared_plane, "column_reduce"), "integer_range": (integer_range, "column_reduce"),
            "narrow_columns": (narrow_columns, "column_reduce"), "half_sums": (half_sums, "column_reduce"),
            "no_keep_meets_the_tensor_unreshaped": (no_keep_meets_the_tensor_unreshaped, "staged"),
            "run_too_long_for_registers": (run_too_long_for_registers, "staged")}


@pytest.mark.parametrize("case", sorted(_column_cases()))
def test_reductions_over_a_middle_axis_whose_results_meet_the_tensor_again(case):
    """The column kernel on shapes that stress its layout: a reduction without keep_dims and the Reshape that follows,
    outputs of the reduced shape next to full ones, operands that broadcast over the outer or the inner axes, integer
    data, two columns only, a 16-bit sum (bit for bit the oracle's serial sum), and a run too long for a workgroup's
    registers (several kernels instead). float32 sums against the float64 evaluation, everything else against the oracle
    bit for bit or to its tolerance."""
    from oracle import np_ref
    build, family = _column_cases()[case]
    b = op_desc.DescBuilder("column_" + case)
    text = b.dumps(build(b))
    desc = json_loads(text)
    kernel = driver.HipKernel(text, out_dir=None)
    print("case %s: %s grid %d block %d" % (case, kernel.family, kernel.grid[0], kernel.block[0]), flush=True)
    assert kernel.family == family
    if case == "several_strips_per_workgroup":
        assert kernel.grid[0] == 256 and "constexpr long TOTAL = 560;" in kernel.source and "load_packed_partial" in kernel.source
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 790)
    expect = np_ref.evaluate(desc, inputs)
    wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
    exact = np_ref.evaluate(harness.widen_to_float64(desc), wide)
    run = max(e[0]["shape"][1] for e in desc["input_desc"])
    sums = any(o["name"] == "ReduceSum" for o in desc["op_desc"])
    for launch in range(2):
        got = run_on_gpu(kernel, inputs)
        for d, g, e, x in zip(kernel.outputs, got, expect, exact):
            if d.dtype == "float32" and sums:
                ok, msg = harness.compare_reassociated(g, x, d.dtype, run)
            elif case == "half_sums":
                # a float16 sum takes its steps in the serial loop's order: the oracle's bits
                ok = bool(np.array_equal(np.asarray(g).view(np.uint16), np.asarray(e).view(np.uint16)))
                msg = "bit-identical" if ok else "differs from the serial float16 sum in %d elements" % int(
                    (np.asarray(g).view(np.uint16) != np.asarray(e).view(np.uint16)).sum())
            else:
                ok, msg = harness.compare(g, e, d.dtype)
            print("  launch %d %s %s: %s" % (launch, d.name, d.dtype, msg), flush=True)
            assert ok, "%s output %s: %s" % (case, d.name, msg)


def _ordered_cases():
    """Descriptions with a float16 / bfloat16 ReduceSum or ReducePrd, (builder, kernel family, exact): every family
    that reduces. `exact` is False where a transcendental sits in front of the sum (its last bit may differ from libm's,
    and the chain then rounds differently): those are held to the 16-bit tolerance."""
    def red(name, shape, dtype, axes, keep):
        return lambda b: [b.reduce(name, b.input(shape, dtype), axes, keep)]

    def softmax16(b):
        x = b.input([33, 777], "float16")
        e = b.unary("Exp", b.sub(x, b.reduce("ReduceMax", x, [1], True)))
        return [b.div(e, b.reduce("ReduceSum", e, [1], True))]

    def prod_and_sum(b):
        x = b.input([19, 300], "bfloat16")
        return [b.reduce("ReducePrd", x, [1], True), b.reduce("ReduceSum", x, [1], True)]

    def centred_columns(b):
        x = b.input([2, 4096, 24], "float16")
        return [b.sub(x, b.reduce("ReduceSum", x, [1], True))]

    def scaled_columns(b):
        x = b.input([3, 301, 130], "bfloat16")
        return [b.mul(x, b.reduce("ReduceSum", x, [1], True)), b.reduce("ReduceMax", x, [1], True)]

    def two_accumulators(b):
        x = b.input([100, 77], "float16")
        return [b.reduce("ReduceSum", x, [0, 1], False), b.reduce("ReduceSum", b.cast(x, "float32"), [0, 1], False)]

    return {
        "row_f16_64x4096": (red("ReduceSum", [64, 4096], "float16", [1], True), "row_reduce", True),
        "row_bf16_37x1000": (red("ReduceSum", [37, 1000], "bfloat16", [1], False), "row_reduce", True),
        "row_softmax_f16_33x777": (softmax16, "row_reduce", False),
        "row_512_threads_f16_5x20000": (red("ReduceSum", [5, 20000], "float16", [1], True), "row_reduce", True),
        "row_walked_f16_64x70001": (red("ReduceSum", [64, 70001], "float16", [1], True), "row_reduce", True),
        "row_prod_sum_bf16_19x300": (prod_and_sum, "row_reduce", True),
        "column_f16_2x4096x24": (centred_columns, "column_reduce", True),
        "column_bf16_3x301x130": (scaled_columns, "column_reduce", True),
        "stream_y_f16_4096x520": (red("ReduceSum", [4096, 520], "float16", [0], False), "stream_reduce", True),
        "stream_y_bf16_7x300x33": (red("ReduceSum", [7, 300, 33], "bfloat16", [1], True), "stream_reduce", True),
        "stream_all_bf16_768x512": (red("ReduceSum", [768, 512], "bfloat16", [0, 1], False), "stream_reduce", True),
        "stream_all_two_accumulators_f16_100x77": (two_accumulators, "stream_reduce", True),
        "stream_x_long_f16_3x70000": (red("ReduceSum", [3, 70000], "float16", [1], True), "stream_reduce", True),
        "stream_kept_between_f16_8x6x7x12": (red("ReduceSum", [8, 6, 7, 12], "float16", [0, 2, 3], False), "stream_reduce", True),
    }


@pytest.mark.parametrize("case", sorted(_ordered_cases()))
def test_sixteen_bit_sums_take_their_steps_in_the_reference_order(case):
    """A ReduceSum / ReducePrd whose declared result is float16 or bfloat16 rounds after every step, so the order of the
    steps is part of the result; the reference's is one serial loop per result element in index order
    (MindSporeToLinalg.cpp:845-901,1333-1451). Every reducing family must give the oracle's bits (the 16-bit tolerance
    where a transcendental in front of the sum may differ from libm in its last bit)."""
    from oracle import np_ref
    build, family, exact = _ordered_cases()[case]
    b = op_desc.DescBuilder("ordered_" + case)
    text = b.dumps(build(b))
    desc = json_loads(text)
    kernel = driver.HipKernel(text, out_dir=None)
    print("case %s: %s grid %d block %d" % (case, kernel.family, kernel.grid[0], kernel.block[0]), flush=True)
    assert kernel.family == family
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 4242)
    expect = np_ref.evaluate(desc, inputs)
    wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
    in_numel = max(int(np.prod(e[0]["shape"])) for e in desc["input_desc"])
    for launch in range(2):
        got = run_on_gpu(kernel, inputs)
        for d, g, e in zip(kernel.outputs, got, expect):
            if d.dtype == "float32":
                x = np_ref.evaluate(harness.widen_to_float64(desc), wide)[list(kernel.outputs).index(d)]
                ok, msg = harness.compare_reassociated(g, x, d.dtype, max(1, in_numel // max(1, g.size)))
            elif exact:
                gb, eb = np.asarray(g).view(np.uint16), np.asarray(e).view(np.uint16)
                ok = bool(np.array_equal(gb, eb))
                msg = "bit-identical" if ok else "%d of %d elements differ from the serial sum" % (int((gb != eb).sum()), gb.size)
            else:
                ok, msg = harness.compare(g, e, d.dtype)
            print("  launch %d %s %s: %s" % (launch, d.name, d.dtype, msg), flush=True)
            assert ok, "%s output %s: %s" % (case, d.name, msg)


@pytest.mark.parametrize("family", ["row_reduce", "column_reduce", "stream_reduce"])
def test_4096_float16_ones_sum_to_2048_on_the_device(family):
    """The known answer of the reference's rule: a float16 accumulator stalls at 2048 (2048 + 1 rounds back to 2048). A
    tree of partial sums gives 4096."""
    shape, axes = {"row_reduce": ([3, 4096], [1]), "column_reduce": ([2, 4096, 16], [1]), "stream_reduce": ([4096, 40], [0])}[family]
    b = op_desc.DescBuilder("kat_ones_" + family)
    x = b.input(shape, "float16")
    s = b.reduce("ReduceSum", x, axes, True)
    text = b.dumps([b.add(x, s)] if family == "column_reduce" else [s])
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family == family
    got = run_on_gpu(kernel, [np.ones(shape, dtype=np.float16)])[0]
    want = 2049.0 if family == "column_reduce" else 2048.0   # (2048 + 1 in float16 is 2048 again; 2049 is not representable)
    want = float(np.float16(want))
    assert np.all(got.astype(np.float32) == want), "got %s, want %s everywhere" % (np.unique(got), want)



@pytest.mark.parametrize("schedule", ["column_reduce", "staged"])
def test_dynamic_description_that_needs_several_kernels(schedule, tmp_path, monkeypatch):
    """A softmax over axis 1 with an open leading dimension: every shape set is specialised into its own column kernel
    or, with that kernel switched off, its own sequence of kernels (stage artifacts carry the shape digest); results
    against the oracle of the same description written with the bound shape."""
    if schedule == "staged":
        monkeypatch.setenv("AKG_HIP_VARIANT", "7")
    text = op_desc.softmax_over_axis([32, 12, 24, 40], 1, "float32", "dyn_softmax_axis1")
    d = json_loads(text)

    def open_leading(e):
        if isinstance(e, dict):
            if e.get("shape") and e["shape"][0] == 32:
                e["shape"][0] = -1
            for v in e.values():
                open_leading(v)
        elif isinstance(e, list):
            for v in e:
                open_leading(v)
    open_leading(d)
    dyn = driver.HipDynamicKernel(__import__("json").dumps(d), out_dir=str(tmp_path))
    for lead in (32, 7, 32):
        kernel = dyn.specialize([[lead, 12, 24, 40]])
        assert kernel.family == schedule and [t.shape for t in kernel.tensors] == [[lead, 12, 24, 40]] * 2
        static = op_desc.softmax_over_axis([lead, 12, 24, 40], 1, "float32", "static_softmax_axis1_%d" % lead)
        path = os.path.join(str(tmp_path), "static_%d.info" % lead)
        open(path, "w").write(static)
        inputs = harness.make_inputs(json_loads(static), seed=harness.BASE_SEED + 740 + lead)
        got = run_on_gpu(kernel, inputs)
        expect = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
        ok, msg = harness.compare(got[0], expect[0], "float32")
        assert ok, "leading dimension %d: %s" % (lead, msg)
    stem = "dyn_softmax_axis1_stage0_s" if schedule == "staged" else "dyn_softmax_axis1_s"
    assert len([f for f in os.listdir(str(tmp_path)) if f.startswith(stem) and f.endswith(".hsaco")]) == 2


@pytest.mark.parametrize("name", STREAM)
def test_streaming_reduction_matches_oracle(name):
    check_stream_reduction(os.path.join(FIXTURES, name), seed=harness.BASE_SEED + 400, repeats=3)


def test_full_size_bias_gradient_column_sums():
    check_stream_reduction(os.path.join(FIXTURES, "n1_biasgrad_bf16_16384x4096.info"), seed=harness.BASE_SEED + 11)


def test_full_size_long_row_softmax():
    """f16 [512, 131072]: the row is kept packed in registers across the three walks."""
    check_fixture("n4_softmax_f16_512x131072.info", seed=harness.BASE_SEED + 13, openmp=True)


def test_full_size_batchnorm_statistics():
    check_stream_reduction(os.path.join(FIXTURES, "n5_bnstats_bf16_256x64x56x56.info"), seed=harness.BASE_SEED + 14)


def test_full_size_skinny_matmul_with_split_k():
    check_fixture("n6_gemm_bf16_bias_gelu_16x8192x8192.info", seed=harness.BASE_SEED + 15, openmp=True)


def test_full_size_batched_transpose_bias_add():
    """[32,2048,1024] -> [32,1024,2048] bfloat16 transpose fused with a bias add (indexed family), every element."""
    check_fixture("n3_transpose_bias_add_bf16_32x2048x1024.info", seed=harness.BASE_SEED + 12, openmp=True)


def test_tensors_of_two_gib_and_more_are_addressed_with_64_bit_offsets(tmp_path):
    """float32 [34000, 16384] is 2.08 GiB: beyond what a buffer descriptor with 32-bit offsets reaches, so the kernels
    address it through plain pointers. Elementwise (bias add, every element against the oracle's OpenMP build), column
    sums (against float64 numpy) and a softmax over f16 [34000, 32768] (first and last rows against the oracle of a
    64-row description: rows are independent, and a wrapped offset would show at the far end)."""
    rows, cols = 34000, 16384
    b = op_desc.DescBuilder("big_bias_add_f32_%dx%d" % (rows, cols))
    x, v = b.input([rows, cols], "float32"), b.input([cols], "float32")
    text = b.dumps([b.add(x, v)])
    path = os.path.join(str(tmp_path), "big_bias_add.info")
    open(path, "w").write(text)
    rng = np.random.default_rng(7)
    xs = rng.standard_normal((rows, cols), dtype=np.float32)
    vs = rng.standard_normal(cols, dtype=np.float32)
    kernel = driver.HipKernel(text, out_dir=None)
    assert "make_buffer" not in kernel.source
    print("case big bias add", flush=True)
    got = run_on_gpu(kernel, [xs, vs])[0]
    expect = cpu_ref.CpuKernel(path, openmp=True, rebuild=True)([xs, vs])[0]
    assert np.array_equal(got, expect)
    del got
    # the same description with its row count open: the row count is a kernel argument, the addressing stays 64-bit
    print("case big bias add, rows open", flush=True)
    b = op_desc.DescBuilder("big_bias_add_rows_open_f32")
    x, v = b.input([7777, cols], "float32"), b.input([cols], "float32")
    dyn = driver.HipDynamicKernel(open_extent(b.dumps([b.add(x, v)]), 7777), out_dir=None)
    kernel = dyn.specialize([[rows, cols], [cols]])
    assert "make_buffer" not in kernel.source and "akg_extent" in kernel.source
    got = run_on_gpu(kernel, [xs, vs])[0]
    assert np.array_equal(got, expect)
    del got, expect
    print("case big column sum", flush=True)
    text = op_desc.square_reduce([rows, cols], [0], "float32", False, "ReduceSum", name="big_colsum_f32_%dx%d" % (rows, cols))
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family == "stream_reduce" and "make_buffer(in0" not in kernel.source
    got = run_on_gpu(kernel, [xs])[0]
    exact = np.einsum("rc,rc->c", xs, xs, dtype=np.float64)
    ok, msg = harness.compare_reassociated(got, exact, "float32", rows)
    print("  column sums: %s" % msg, flush=True)
    assert ok, msg
    del xs
    print("case big softmax", flush=True)
    rows, cols = 34000, 32768
    kernel = driver.HipKernel(op_desc.softmax_last_axis(rows, cols, "float16"), out_dir=None)
    assert "make_buffer" not in kernel.source
    xh = (rng.standard_normal((rows, cols), dtype=np.float32) * 2.0).astype(np.float16)
    got = run_on_gpu(kernel, [xh])[0]
    small = op_desc.softmax_last_axis(64, cols, "float16", name="big_softmax_rows_sample")
    spath = os.path.join(str(tmp_path), "big_softmax_rows_sample.info")
    open(spath, "w").write(small)
    ref = cpu_ref.CpuKernel(spath, openmp=True, rebuild=True)
    for first in (0, rows // 2, rows - 64):
        expect = ref([np.ascontiguousarray(xh[first:first + 64])])[0]
        ok, msg = harness.compare(got[first:first + 64], expect, "float16")
        print("  rows %d..%d: %s" % (first, first + 63, msg), flush=True)
        assert ok, msg
    sums = got[::997].astype(np.float64).sum(axis=1)
    assert np.all(np.abs(sums - 1.0) < 2e-2)      # every sampled row is a distribution


ODD_LONG_ROWS = {
    "softmax_f16_3x70001": lambda n: op_desc.softmax_last_axis(3, 70001, "float16", n),
    "layernorm_bf16_2x57001": lambda n: op_desc.layernorm_residual(2, 57001, "bfloat16", 1e-5, n),
    "quant_bf16_2x131081": lambda n: op_desc.quant_int8_residual(2, 131081, "bfloat16", n),
    "argmax_f16_2x100003": lambda n: op_desc.argmax_last_axis([2, 100003], "float16", False, "int32", None, n),
    "softmax_f32_2x300001": lambda n: op_desc.softmax_last_axis(2, 300001, "float32", n),
    "layernorm_bf16_3x16391": lambda n: op_desc.layernorm_residual(3, 16391, "bfloat16", 1e-5, n),
}


@pytest.mark.parametrize("case", sorted(ODD_LONG_ROWS))
def test_rows_that_are_long_and_odd_at_once(case, tmp_path):
    """Row kernels where the walks over a long row, the packed row and the overlapping last chunk meet."""
    name = "odd_long_" + case
    text = ODD_LONG_ROWS[case](name)
    path = os.path.join(str(tmp_path), name + ".info")
    open(path, "w").write(text)
    print("case %s" % name, flush=True)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family == "row_reduce" and "akg_tail" in kernel.source
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 800)
    got = run_on_gpu(kernel, inputs)
    expect = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    cols = desc["input_desc"][0][0]["shape"][-1]
    for d, g, e in zip(kernel.outputs, got, expect):
        if d.dtype == "float32":
            # a serial float32 sum of 300 001 terms is itself 1e-4 away from the exact one: float32 results are held
            # to rtol 1e-5 against the float64 evaluation of the same description instead
            from oracle import np_ref
            wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
            exact = np_ref.evaluate(harness.widen_to_float64(desc), wide)[kernel.outputs.index(d)]
            ok, msg = harness.compare_reassociated(g, exact, d.dtype, cols)
            gap = float(np.max(np.abs(np.asarray(e, dtype=np.float64) - np.asarray(exact).reshape(e.shape))))
            msg += " (serial float32 oracle is %.3g away from float64)" % gap
        else:
            ok, msg = harness.compare(g, e, d.dtype)
        print("  %s %s: %s" % (d.name, d.dtype, msg), flush=True)
        assert ok, "%s output %s: %s" % (name, d.name, msg)


SKINNY_CASES = [("bf16", 1, 1024, 520, False), ("bf16", 16, 4096, 1024, False), ("f16", 16, 2048, 264, True),
                ("i8", 32, 4096, 260, False), ("i8", 7, 64, 128, True), ("i8", 1, 32, 4, False), ("f16", 5, 16, 136, False),
                ("bf16", 32, 8192, 136, True), ("batch_bf16", 3, 256, 520, True), ("batch_bf16", 32, 2048, 260, False),
                ("bf16", 33, 2048, 264, False), ("i8", 64, 4096, 520, False), ("f16", 48, 1024, 136, True),
                ("i8", 50, 8192, 128, True), ("batch_bf16", 64, 512, 260, False)]


@pytest.mark.parametrize("case", SKINNY_CASES, ids=lambda c: "%s_%dx%dx%d%s" % (c[0], c[1], c[2], c[3], "_tb" if c[4] else ""))
def test_skinny_matmul_streams_b_into_mfma_operands(case, tmp_path):
    """At most 64 rows of A: strips of 128 columns, B loaded straight into MFMA operands (transposed in registers when
    row-major), K split over wavefronts and workgroups. One row to 64, one K step to 256, ragged N, both layouts, all
    three element types, batched; against the oracle, and twice (the workspace must be left ready)."""
    kind, m, k, n, tb = case
    name = "skinny_gemm_%s_%dx%dx%d%s" % (kind, m, k, n, "_tb" if tb else "")
    if kind == "i8":
        text = op_desc.gemm_int8_dequant_bias_gelu(m, k, n, "bfloat16", tb, name)
    elif kind == "batch_bf16":
        text = op_desc.batch_matmul_scale_mask(5, m, k, n, "bfloat16", tb, name)
    else:
        text = op_desc.gemm_bias_act(m, k, n, "bfloat16" if kind == "bf16" else "float16", "gelu", tb, "float32", name)
    path = os.path.join(str(tmp_path), name + ".info")
    open(path, "w").write(text)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel(text, out_dir=None)
    assert "gemm_skinny" in kernel.source
    print("case %s grid %d x %d workspace %d" % (name, kernel.grid[0], kernel.grid[1], kernel.workspace_bytes), flush=True)
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 720)
    expect = cpu_ref.CpuKernel(path, openmp=True, rebuild=True)(inputs)
    for launch in range(2):
        got = run_on_gpu(kernel, inputs)
        ok, msg = harness.compare(got[0], expect[0], kernel.outputs[0].dtype)
        assert ok, "%s launch %d: %s" % (name, launch, msg)


def _random_gemm_cases(count, seed=123):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(count):
        kind = str(rng.choice(["i8", "bf16", "f16"]))
        m = int(rng.choice([1, 3, 16, 33, 64, 100, 200, 256, 257, 300, 511]))
        n = int(rng.choice([4, 8, 136, 256, 260, 520, 776]))
        k = int(rng.choice([16, 64, 272, 512, 1008, 2048, 3008, 4096, 8192] if kind == "i8" else
                           [16, 64, 264, 512, 1000, 2048, 3000, 4096, 8192]))
        cases.append((kind, m, k, n, bool(rng.integers(0, 2)), str(rng.choice(["gelu", "relu", "none"]))))
    return cases


@pytest.mark.parametrize("case", _random_gemm_cases(20), ids=lambda c: "%s_%dx%dx%d%s" % (c[0], c[1], c[2], c[3], "_tb" if c[4] else ""))
def test_gemm_family_on_ragged_shapes_with_and_without_split_k(case, tmp_path):
    """MatMul fusions on shapes that are no multiple of the tile in any direction, K from one step to 64 (split over up
    to 16 workgroups per tile when K is long and the tiles are few), both operand layouts."""
    kind, m, k, n, tb, act = case
    name = "ragged_gemm_%s_%dx%dx%d%s" % (kind, m, k, n, "_tb" if tb else "")
    if kind == "i8":
        text = op_desc.gemm_int8_dequant_bias_gelu(m, k, n, "bfloat16", tb, name)
    else:
        text = op_desc.gemm_bias_act(m, k, n, "bfloat16" if kind == "bf16" else "float16", act, tb, "float32", name)
    path = os.path.join(str(tmp_path), name + ".info")
    open(path, "w").write(text)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel(text, out_dir=None)
    print("case %s grid %d workspace %d" % (name, kernel.grid[0], kernel.workspace_bytes), flush=True)
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 700)
    got = run_on_gpu(kernel, inputs)
    expect = cpu_ref.CpuKernel(path, openmp=True, rebuild=True)(inputs)
    ok, msg = harness.compare(got[0], expect[0], kernel.outputs[0].dtype)
    assert ok, "%s: %s" % (name, msg)


def test_launches_can_be_captured_in_a_hip_graph_and_replayed():
    """After `prepare` a launch allocates nothing and records no memset, so a serving loop can capture a chain of
    kernels once and replay it: a softmax, a column reduction (workspace + arrival counters), a split-K GEMM
    (workspace), a grouped segment sum (five launches over one workspace) and a softmax over an outer axis (three
    kernels with temporaries between them) are captured in one graph and replayed four times on fresh inputs, with eager work and
    synchronisations in between; every replay must equal the eager launches bit for bit (the counters and partials
    of one replay must be ready for the next)."""
    import torch
    dev = torch.device("cuda:0")
    names = ["small_softmax_f16_64x4096", "small_biasgrad_bf16_2048x1024", "small_gemm_bf16_bias_gelu_100x2048x520",
             "small_segment_sum_f16_150001_by_4_seg300", "small_staged_softmax_f32_32x12x24x40_axis1"]
    kernels, descs = [], []
    for n in names:
        path = os.path.join(FIXTURES, n + ".info")
        k = driver.HipKernel.from_file(path)
        k.prepare()
        kernels.append(k)
        descs.append(harness.load_desc(path))
    assert kernels[1].workspace_bytes > 0 and kernels[2].workspace_bytes > 0 and kernels[3].workspace_bytes > 0

    def buffers(k):
        return [torch.zeros(t.nbytes, dtype=torch.uint8, device=dev) for t in k.tensors]
    static = [buffers(k) for k in kernels]          # the graph's own buffers
    eager = [buffers(k) for k in kernels]

    def upload(bufs, k, inputs):
        for b, a in zip(bufs, inputs):
            b.copy_(torch.from_numpy(a.view(np.uint8).reshape(-1)))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                   # warm-up launches outside the capture
        for k, bufs in zip(kernels, static):
            k.launch(bufs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for k, bufs in zip(kernels, static):
            k.launch(bufs)
    for replay in range(4):
        print("replay %d" % replay, flush=True)
        for k, d, sb, eb in zip(kernels, descs, static, eager):
            inputs = harness.make_inputs(d, seed=harness.BASE_SEED + 900 + replay)
            upload(sb, k, inputs)
            upload(eb, k, inputs)
            for b in sb[len(inputs):]:
                b.fill_(0x7B)                        # stale results of the previous replay must not survive
        graph.replay()
        torch.cuda.synchronize()
        for k, eb in zip(kernels, eager):            # the program's own eager work between replays
            k.launch(eb)
        torch.cuda.synchronize()
        for k, sb, eb in zip(kernels, static, eager):
            n_in = len(k.tensors) - len(k.outputs)
            for a, b in zip(sb[n_in:], eb[n_in:]):
                assert torch.equal(a, b), "replay %d of %s differs from the eager launch" % (replay, k.kernel_name)


def test_handles_launched_from_several_threads_on_their_own_streams():
    """Four threads, each with a handle and a stream of its own (one of them with a workspace, one with five launches
    per step), launch 40 times at once; every thread's result must equal what the same handle gives alone."""
    import threading
    import torch
    dev = torch.device("cuda:0")
    names = ["small_softmax_f16_64x4096", "small_biasgrad_bf16_2048x1024", "small_segment_sum_f16_150001_by_4_seg300",
             "small_gemm_bf16_bias_gelu_100x2048x520"]
    jobs = []
    for i, n in enumerate(names):
        path = os.path.join(FIXTURES, n + ".info")
        k = driver.HipKernel.from_file(path)
        k.prepare()
        inputs = harness.make_inputs(harness.load_desc(path), seed=harness.BASE_SEED + 950 + i)
        alone = run_on_gpu(k, inputs)
        ins = [_torch_view(a).to(dev) for a in inputs]
        outs = [torch.zeros(d.nbytes, dtype=torch.uint8, device=dev) for d in k.outputs]
        jobs.append((k, ins, outs, alone, torch.cuda.Stream()))
    torch.cuda.synchronize()
    failures = []

    def work(job):
        k, ins, outs, _, stream = job
        try:
            for _ in range(40):
                k.launch(ins + outs, stream=stream)
            stream.synchronize()
        except Exception as exc:                                  # noqa: BLE001 - reported by the main thread
            failures.append((k.kernel_name, repr(exc)))
    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not failures, failures
    for k, _, outs, alone, _ in jobs:
        for d, o, a in zip(k.outputs, outs, alone):
            got = o.cpu().numpy().view(driver.NP_HOST_DTYPE[d.dtype]).reshape(d.shape)
            assert np.array_equal(got.view(np.uint8), np.ascontiguousarray(a).view(np.uint8)), k.kernel_name


def test_handles_of_one_source_share_their_module_and_outlive_each_other():
    """Handles made from one source (two compilations of one description; the specialisations of a dynamic description)
    share the loaded code object. Destroying one of them must leave the others launchable, and the last one to go
    unloads it: a third handle made afterwards loads it afresh."""
    path = os.path.join(FIXTURES, "small_softmax_f16_64x4096.info")
    desc = harness.load_desc(path)
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 5)
    a, b = driver.HipKernel.from_file(path, out_dir=None), driver.HipKernel.from_file(path, out_dir=None)
    want = run_on_gpu(a, inputs)
    assert np.array_equal(run_on_gpu(b, inputs)[0].view(np.uint8), want[0].view(np.uint8))
    a.close()
    for _ in range(2):
        assert np.array_equal(run_on_gpu(b, inputs)[0].view(np.uint8), want[0].view(np.uint8))
    b.close()
    c = driver.HipKernel.from_file(path, out_dir=None)
    assert np.array_equal(run_on_gpu(c, inputs)[0].view(np.uint8), want[0].view(np.uint8))


def test_cli_runs_a_description_on_the_gpu():
    """`akg-hip run X.info`: seeded inputs, NaN-prefilled outputs, a call on host buffers and timed launches. Two runs
    give the same checksums (one kernel, a sequence of kernels, and a kernel that must leave unnamed rows zero) and no NaN
    is left in the outputs."""
    import subprocess
    tool = os.path.join(ROOT, "akg_amd", "akg-hip")
    for fixture in ("small_softmax_f16_64x4096.info", "small_staged_softmax_f32_32x12x24x40_axis1.info",
                    "small_segment_sum_f32_700x3_by_1x3_seg50.info"):
        runs = []
        for _ in range(2):
            p = subprocess.run([tool, "run", os.path.join(FIXTURES, fixture), "-n", "5", "-r", "2"], capture_output=True,
                               text=True, timeout=120)
            assert p.returncode == 0, p.stderr
            runs.append(p.stdout)
        lines = [l for l in runs[0].splitlines() if l.startswith("output ")]
        assert lines and lines == [l for l in runs[1].splitlines() if l.startswith("output ")]
        assert all(l.split()[-1] in ("0", "-1") for l in lines), runs[0]
        ms = float([l for l in runs[0].splitlines() if l.startswith("time")][0].split()[1])
        assert 0.0 < ms < 50.0
    p = subprocess.run([tool, "run", os.path.join(FIXTURES, "no_such.info")], capture_output=True, text=True, timeout=60)
    assert p.returncode == 1 and "cannot read" in p.stderr


def test_cli_compares_against_expectations_made_elsewhere(tmp_path):
    """`akg-hip run --dump / --inputs / --expect`: the numeric compare of the reference's akg_benchmark
    (benchmark.py:94-130) with the expectation computed outside the tool. The tool's own seeded inputs are dumped,
    the oracle evaluates the description on them, and the tool, given those inputs again, accepts the oracle's
    outputs and rejects them once one element is changed."""
    import subprocess
    tool = os.path.join(ROOT, "akg_amd", "akg-hip")
    for fixture in ("small_softmax_f16_64x4096.info", "small_quant_int8_residual_bf16_37x1544.info",
                    "small_ew_tanh_add_mul_f32_7x33.info"):
        path = os.path.join(FIXTURES, fixture)
        dump, want = tmp_path / (fixture + ".dump"), tmp_path / (fixture + ".want")
        dump.mkdir()
        want.mkdir()
        p = subprocess.run([tool, "run", path, "-n", "1", "-r", "1", "--dump", str(dump)], capture_output=True, text=True,
                           timeout=120)
        assert p.returncode == 0, p.stderr
        kernel = driver.HipKernel.from_file(path)
        n_in = len(kernel.inputs)
        inputs = [np.fromfile(str(dump / ("arg%d.bin" % i)), dtype=driver.NP_HOST_DTYPE[d.dtype]).reshape(d.shape)
                  for i, d in enumerate(kernel.inputs)]
        expect = cpu_ref.CpuKernel(path, openmp=False)(inputs)
        for j, e in enumerate(expect):
            np.ascontiguousarray(e).tofile(str(want / ("arg%d.bin" % (n_in + j))))
        cmd = [tool, "run", path, "-n", "1", "-r", "1", "--inputs", str(dump), "--expect", str(want)]
        p = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
        assert p.returncode == 0, p.stdout + p.stderr
        assert p.stdout.count("compare ") == len(expect) and "MISMATCH" not in p.stdout, p.stdout
        # one element off by far more than any bar (the top exponent bit of a float, bit 6 of an int8): the tool
        # counts it and exits 1
        raw = bytearray((want / ("arg%d.bin" % n_in)).read_bytes())
        esize = np.dtype(driver.NP_HOST_DTYPE[kernel.outputs[0].dtype]).itemsize
        raw[(len(raw) // esize // 2) * esize + esize - 1] ^= 0x40
        (want / ("arg%d.bin" % n_in)).write_bytes(bytes(raw))
        p = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
        assert p.returncode == 1 and "MISMATCH in 1 elements" in p.stdout, p.stdout + p.stderr
    p = subprocess.run([tool, "run", os.path.join(FIXTURES, "small_softmax_f16_64x4096.info"), "--inputs",
                        str(tmp_path / "nowhere")], capture_output=True, text=True, timeout=60)
    assert p.returncode == 1 and "must hold" in p.stderr


@pytest.mark.parametrize("name", FULL)
def test_full_size_config_matches_oracle(name):
    # the full sizes of the measured configurations; the oracle runs its OpenMP build (same per-row arithmetic, rows in parallel)
    check_fixture(name, seed=harness.BASE_SEED + 1 + FULL.index(name), openmp=True)


REF_INFO = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_info")
# Every op description of the reference's own test tree (akg-mlir/tests/st/**), copied as data under their own names
# (".info_failed" / ".info.failed" are the reference's markers for cases its CPU pipeline does not pass).
REF_SKIPPED = ()


def _is_dynamic(path):
    d = harness.load_desc(path)
    return any(x < 0 for e in d["input_desc"] for x in e[0].get("shape", [1]))


REF_ALL = sorted(f for f in os.listdir(REF_INFO) if ".info" in f and not (REF_SKIPPED and f.startswith(REF_SKIPPED)))
REF_DYNAMIC = [f for f in REF_ALL if _is_dynamic(os.path.join(REF_INFO, f))]
REF_STREAM = [f for f in REF_ALL if f not in REF_DYNAMIC and "ReduceSum_split" in f]
REF_SEGMENT = [f for f in REF_ALL if f.startswith("Fused_UnsortedSegmentSum_")]
REF_STATIC = [f for f in REF_ALL if f not in REF_DYNAMIC and f not in REF_STREAM and f not in REF_SEGMENT]


@pytest.mark.parametrize("name", REF_STREAM)
def test_reference_repository_all_reduce_descriptions(name):
    """Fused_Mul_ReduceSum_split_*: the reference's own all-reduce system-test descriptions ([768,512] -> [1] and
    [3072] -> [1]), unchanged."""
    check_stream_reduction(os.path.join(REF_INFO, name), seed=harness.BASE_SEED + 200, repeats=2, family=None)



@pytest.mark.parametrize("name", REF_STATIC)
def test_reference_repository_descriptions_match_oracle(name):
    """Op descriptions taken unchanged from the reference's own system-test data (static-shape ones)."""
    path = os.path.join(REF_INFO, name)
    print("case %s" % name, flush=True)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 200)
    got = run_on_gpu(kernel, inputs)
    expect = cpu_ref.CpuKernel(path)(inputs)
    for d, g, e in zip(kernel.outputs, got, expect):
        ok, msg = harness.compare(g, e, d.dtype)
        print("  %s %s: %s" % (d.name, d.dtype, msg), flush=True)
        assert ok, "%s output %s: %s" % (name, d.name, msg)


@pytest.mark.parametrize("shape,axes,split", [([8192, 1024], [0], 64), ([2048, 4096], [0, 1], 128), ([64, 32, 4096], [0, 2], 32)])
def test_workspace_launches_from_two_streams_are_ordered_and_repeat_bit_for_bit(shape, axes, split, monkeypatch):
    """Many workgroups per output group (the split is forced up) leave partial results and arrival counters in the
    handle's workspace; the last one to arrive finishes in slot order. 300 launches of ONE handle, alternating between
    two streams with no host synchronisation in between, each into an output buffer of its own: the library orders
    them on the device (they share the workspace), and every result must equal the first bit for bit - a lost
    partial, a counter left set or two launches inside the workspace at once would show as a different sum."""
    import torch
    monkeypatch.setenv("AKG_HIP_SPLIT", str(split))
    name = "ws_order_%s_%s" % ("x".join(map(str, shape)), "".join(map(str, axes)))
    text = op_desc.square_reduce(shape, axes, "float32", False, "ReduceSum", name)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family == "stream_reduce" and kernel.workspace_bytes > 0
    print("case %s grid %d workspace %d" % (name, kernel.grid[0], kernel.workspace_bytes), flush=True)
    desc = json_loads(text)
    x = harness.make_inputs(desc, seed=harness.BASE_SEED + 99)[0]
    dev = torch.device("cuda:0")
    xin = torch.from_numpy(x).to(dev)
    launches = 300
    nbytes = kernel.outputs[0].nbytes
    outs = torch.full((launches, nbytes), 0xFF, dtype=torch.uint8, device=dev)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for i in range(launches):
        kernel.launch_ptrs([xin.data_ptr(), outs[i].data_ptr()], streams[i % 2].cuda_stream)
    torch.cuda.synchronize()
    host = outs.cpu().numpy()
    for i in range(1, launches):
        assert np.array_equal(host[i], host[0]), "launch %d differs from launch 0" % i
    got = host[0].view(np.float32).reshape(kernel.outputs[0].shape)
    exact = np.sum(x.astype(np.float64) ** 2, axis=tuple(axes))
    ok, msg = harness.compare_reassociated(got, exact, "float32", int(np.prod(shape)) // max(1, got.size))
    assert ok, msg


def test_a_stream_destroyed_between_launches_of_one_handle(monkeypatch):
    """AKG_HIP_SAFE_STREAMS=1: the event that orders launches of a handle with a workspace is recorded behind every
    launch, so the library never touches a stream again after launching on it - the caller may destroy it. Launch on a
    stream, destroy it while the work may still be running, launch on a second one: both results equal the first launch
    of all (made on the default stream)."""
    import ctypes
    import torch
    monkeypatch.setenv("AKG_HIP_SAFE_STREAMS", "1")
    monkeypatch.setenv("AKG_HIP_SPLIT", "64")
    hip = ctypes.CDLL("libamdhip64.so")
    text = op_desc.square_reduce([8192, 1024], [0], "float32", False, "ReduceSum", "ws_stream_gone")
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.workspace_bytes > 0
    x = harness.make_inputs(json_loads(text), seed=harness.BASE_SEED + 98)[0]
    dev = torch.device("cuda:0")
    xin = torch.from_numpy(x).to(dev)
    outs = torch.full((5, kernel.outputs[0].nbytes), 0xFF, dtype=torch.uint8, device=dev)
    kernel.launch_ptrs([xin.data_ptr(), outs[0].data_ptr()], torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for i in range(1, 5):
        stream = ctypes.c_void_p()
        assert hip.hipStreamCreate(ctypes.byref(stream)) == 0
        kernel.launch_ptrs([xin.data_ptr(), outs[i].data_ptr()], stream.value)
        assert hip.hipStreamDestroy(stream) == 0      # asynchronous: the stream goes once its work has drained
    torch.cuda.synchronize()
    host = outs.cpu().numpy()
    for i in range(1, 5):
        assert np.array_equal(host[i], host[0]), "launch %d differs" % i


def _run_with_inputs_back(kernel, inputs):
    """Like run_on_gpu, but also returns the device copies of the inputs after the launch (Assign writes over them)."""
    import torch
    dev = torch.device("cuda:0")
    ins = [_torch_view(a).to(dev) for a in inputs]
    outs = []
    for d in kernel.outputs:
        t = torch.empty(d.nbytes, dtype=torch.uint8, device=dev)
        t.fill_(0xFF if d.dtype in ("float16", "bfloat16", "float32", "float64") else 0x7B)
        outs.append(t)
    kernel.launch(ins + outs)
    torch.cuda.synchronize()
    got = [o.cpu().numpy().view(driver.NP_HOST_DTYPE[d.dtype]).reshape(d.shape) for d, o in zip(kernel.outputs, outs)]
    back = [t.cpu().numpy().view(a.dtype).reshape(a.shape) for t, a in zip(ins, inputs)]
    return got, back


def _gemm_assign(m, k, n, dtype, name):
    """Accumulator update behind a MatMul: acc <- 0.9 acc + 0.1 (A @ B), the product also returned in 16 bits."""
    b = op_desc.DescBuilder(name)
    a, w, acc = b.input([m, k], dtype), b.input([k, n], dtype), b.input([m, n], "float32")
    y = b.matmul(a, w, "float32")
    upd = b.add(b.mul(acc, b.const(0.9, "float32")), b.mul(y, b.const(0.1, "float32")))
    return b.dumps([b.op("Assign", [acc, upd], [m, n], "float32"), b.cast(y, dtype if dtype != "float32" else "float32")])


def _slice_assign(name):
    """momentum <- 0.9 momentum + grad[:, 8:72]: an in-place update whose value comes through a Slice."""
    b = op_desc.DescBuilder(name)
    mom, grad = b.input([37, 64], "float32"), b.input([37, 100], "float32")
    upd = b.add(b.mul(mom, b.const(0.9, "float32")), op_desc.slice_(b, grad, [0, 8], [37, 64]))
    return b.dumps([b.op("Assign", [mom, upd], [37, 64], "float32")])


def _transposed_self_assign(name):
    """p <- p + p^T: the destination is read through a Transpose, so the transposed copy must be made before the update."""
    b = op_desc.DescBuilder(name)
    p = b.input([48, 48], "float32")
    return b.dumps([b.op("Assign", [p, b.add(p, op_desc.transpose(b, p, [1, 0]))], [48, 48], "float32")])


@pytest.mark.parametrize("case", ["gemm_bf16_256x512x256", "gemm_f16_100x264x136", "gemm_f32_70x100x36", "slice", "transposed_self"])
def test_assign_next_to_a_matmul_or_a_data_movement_op(case, tmp_path):
    """Assign in the GEMM epilogue (the destination is a kernel input of the result's shape; also on the split-K and the
    serial kernels) and in the indexed family (the thread that computes an element stores it over the destination too);
    a destination that is read through an index map makes the description run as two kernels. The destination's device
    copy must hold the oracle's updated values afterwards, the other inputs must be untouched."""
    from oracle import np_ref
    if case.startswith("gemm"):
        _, dt, dims = case.split("_")
        m, k, n = [int(x) for x in dims.split("x")]
        text = _gemm_assign(m, k, n, {"bf16": "bfloat16", "f16": "float16", "f32": "float32"}[dt], "assign_" + case)
    elif case == "slice":
        text = _slice_assign("assign_slice")
    else:
        text = _transposed_self_assign("assign_transposed_self")
    desc = json_loads(text)
    kernel = driver.HipKernel(text, out_dir=None)
    print("case %s: %s grid %d" % (case, kernel.family, kernel.grid[0]), flush=True)
    if case == "transposed_self":
        assert kernel.family == "staged"
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 77)
    updates = {}
    expect = np_ref.evaluate(desc, inputs, updates=updates)
    got, back = _run_with_inputs_back(kernel, [a.copy() for a in inputs])
    # float32 results of the matrix units add the same products in another order than the oracle's k loop
    # and are held against the float64 evaluation of the same description instead
    mfma_terms = k if case.startswith("gemm") and "gemm_serial" not in kernel.source else 0
    exact, exact_updates = expect, updates
    if mfma_terms:
        exact_updates = {}
        wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
        exact = np_ref.evaluate(harness.widen_to_float64(desc), wide, updates=exact_updates)

    def check(g, e, x, dt, what):
        if dt == "float32" and mfma_terms:
            ok, msg = harness.compare_reassociated(g, np.asarray(x, dtype=np.float64), dt, mfma_terms)
        else:
            ok, msg = harness.compare(g, e, dt)
        assert ok, "%s %s: %s" % (case, what, msg)

    for d, g, e, x in zip(kernel.outputs, got, expect, exact):
        check(g, e, x, d.dtype, "output " + d.name)
    assert updates, "the description overwrites no input"
    for pos, a in enumerate(inputs):
        check(back[pos], updates.get(pos, a), exact_updates.get(pos, a), desc["input_desc"][pos][0]["data_type"],
              "input %d after the launch" % pos)
        if pos not in updates:
            assert np.array_equal(back[pos].view(np.uint8), a.view(np.uint8)), "%s: input %d was modified" % (case, pos)


@pytest.mark.parametrize("shape,axis,keep,dtype", [([5, 7, 9], 1, False, "float32"), ([5, 7, 9], 0, True, "float16"),
                                                   ([40, 300], 0, False, "bfloat16"), ([3, 4, 5, 6], 2, True, "float32"),
                                                   ([64, 1000, 2], 1, False, "float32")])
def test_argmax_over_an_axis_that_is_not_the_innermost(shape, axis, keep, dtype):
    """ArgMax over an outer axis is respelled as Transpose + ArgMax over the last axis (+ Reshape for keep_dims) and runs
    as two kernels; positions must equal the oracle's (first of equal maxima: the inputs are rounded to a coarse grid so
    that ties occur)."""
    from oracle import np_ref
    b = op_desc.DescBuilder("argmax_axis%d_%s_%s" % (axis, dtype, "x".join(map(str, shape))))
    x = b.input(shape, dtype)
    text = b.dumps([op_desc.argmax(b, x, axis, keep, "int32")])
    desc = json_loads(text)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family == "staged" and kernel.source.count('extern "C" __global__') == 2
    x_in = harness.make_inputs(desc, seed=harness.BASE_SEED + 5)[0]
    as_f32 = harness.bf16_bits_to_f32(x_in) if dtype == "bfloat16" else x_in.astype(np.float32)
    coarse = (np.round(as_f32 * 4) / 4).astype(np.float32)          # ties
    x_in = harness.f32_to_bf16_bits(coarse) if dtype == "bfloat16" else coarse.astype(x_in.dtype)
    got = run_on_gpu(kernel, [x_in])[0]
    expect = np_ref.evaluate(desc, [x_in])[0]
    assert np.array_equal(got, expect)
    assert np.array_equal(got.reshape(-1), np.argmax(coarse, axis=axis).reshape(-1))


def check_segment_sum(path, seed, repeats=2):
    """UnsortedSegmentSum keeps the serial order of the additions per output element: bit-exact against the oracle,
    float types included, and on every launch (nothing may be left over from the one before)."""
    print("case %s seed %d" % (os.path.basename(path), seed), flush=True)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    assert kernel.family == "segment_sum"
    inputs = harness.make_inputs(desc, seed=seed)
    expect = cpu_ref.CpuKernel(path)(inputs)
    for rep in range(repeats):
        got = run_on_gpu(kernel, inputs)
        assert len(got) == 1 and got[0].shape == expect[0].shape
        same = np.array_equal(np.ascontiguousarray(got[0]).view(np.uint8), np.ascontiguousarray(expect[0]).view(np.uint8))
        print("  launch %d: %s" % (rep, "bit-exact" if same else "DIFFERS"), flush=True)
        assert same, os.path.basename(path)
    return inputs, expect


@pytest.mark.parametrize("name", REF_SEGMENT)
def test_reference_repository_segment_sum_descriptions(name):
    """Fused_UnsortedSegmentSum_split_*: the reference's own descriptions (marked failed for its CPU pipeline), up to
    24.5 million index positions scattered into [4954, 1, 3]."""
    check_segment_sum(os.path.join(REF_INFO, name), seed=harness.BASE_SEED + 300)


@pytest.mark.parametrize("name", [n for n in ALL_SMALL if "segment_sum" in n])
def test_segment_sum_is_bit_exact(name):
    check_segment_sum(os.path.join(FIXTURES, name), seed=harness.BASE_SEED + 301)


@pytest.mark.parametrize("dtype,slice_,segments,positions,ids", [
    ("float16", 2, 2000, 200000, "int32"),      # 4-byte rows, 16 segments a bucket, 16-bit additions rounded per step
    ("int32", 3, 1600, 150000, "int64"),        # 12-byte integer rows, 64-bit ids
    ("bfloat16", 6, 800, 131077, "int32"),      # 12-byte rows of six elements, 4 segments a bucket, a ragged last chunk
    ("float32", 1, 4000, 100000, "int32"),      # one column
])
def test_bucketed_segment_sum_in_other_types(dtype, slice_, segments, positions, ids, tmp_path):
    """The schedule by bucket of segments for rows of 4, 8 and 12 bytes in 16-bit, integer and float32 data: bit-exact
    against the serial loop (16-bit sums included: every addition is rounded, in position order)."""
    name = "bucketed_%s_x%d_seg%d_%d" % (dtype, slice_, segments, positions)
    text = op_desc.unsorted_segment_sum([positions], [slice_], segments, dtype, ids, name)
    path = os.path.join(str(tmp_path), name + ".info")
    open(path, "w").write(text)
    kernel = driver.HipKernel(text, out_dir=None)
    assert "grouped by bucket" in kernel.source, kernel.source[:200]
    check_segment_sum(path, seed=harness.BASE_SEED + 770)


@pytest.mark.parametrize("schedule", ["scan", "grouped", "bucketed"])
def test_segment_sum_drops_ids_outside_the_range_and_leaves_unnamed_rows_zero(schedule, monkeypatch, tmp_path):
    """The three schedules (every workgroup scanning all ids; positions grouped by segment first; grouped by bucket of
    eight segments first and by segment in LDS) on the same small case."""
    monkeypatch.setenv("AKG_HIP_VARIANT", {"scan": "1", "grouped": "2", "bucketed": "3"}[schedule])
    path = os.path.join(FIXTURES, "small_segment_sum_f32_700x3_by_1x3_seg50.info")
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path, out_dir=str(tmp_path))
    assert ("grouped by segment" in kernel.source) == (schedule == "grouped")
    assert ("grouped by bucket" in kernel.source) == (schedule == "bucketed")
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 302)
    ids = inputs[1]
    ids[ids == 17] = 50          # nobody names row 17; 50 and -3 are outside [0, 50)
    ids[::7] = -3
    expect = cpu_ref.CpuKernel(path)(inputs)
    got = run_on_gpu(kernel, inputs)
    assert np.array_equal(got[0], expect[0]) and not got[0][17].any() and got[0].any()


def test_segment_sum_with_neighbours_runs_as_stages_and_stays_bit_exact(tmp_path):
    """out = -UnsortedSegmentSum(2 * data, ids): the scaling, the segment sum and the negation are three kernels; the
    additions keep their serial order, so the result equals the oracle's bit for bit (scaling by two and negation are
    exact)."""
    b = op_desc.DescBuilder("Fused_Mul_UnsortedSegmentSum_Neg")
    data, ids = b.input([70000, 3], "float32"), b.input([70000], "int32")
    seg = b.op("UnsortedSegmentSum", [b.mul(data, b.const(2.0, "float32")), ids], [500, 3], "float32",
               attrs=[{"data_type": "int", "name": "num_segments", "value": 500}])
    text = b.dumps([b.unary("Neg", seg)])
    path = os.path.join(str(tmp_path), "Fused_Mul_UnsortedSegmentSum_Neg.info")
    open(path, "w").write(text)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family == "staged" and "grouped by segment" in kernel.source
    inputs = harness.make_inputs(json_loads(text), seed=harness.BASE_SEED + 780)
    expect = cpu_ref.CpuKernel(path, rebuild=True)(inputs)
    for launch in range(2):
        got = run_on_gpu(kernel, inputs)
        assert np.array_equal(got[0].view(np.uint8), expect[0].view(np.uint8)), "launch %d" % launch


@pytest.mark.parametrize("schedule", ["by_segment", "by_bucket"])
@pytest.mark.parametrize("pattern", ["one_segment", "sorted", "runs_of_64", "mostly_outside", "one_bucket"])
def test_grouped_segment_sum_on_skewed_ids(pattern, schedule, monkeypatch, tmp_path):
    """The grouped schedules where the ids are far from uniform: every position in one segment (every lane of a tile
    ranks behind its neighbours, one chain of 300000 additions), ids already sorted (a run touches few segments), whole
    tiles of equal ids, nine ids in ten outside [0, segments), and every id within one bucket of eight segments.
    Bit-exact against the serial loop."""
    monkeypatch.setenv("AKG_HIP_VARIANT", "2" if schedule == "by_segment" else "3")
    path = os.path.join(FIXTURES, "small_segment_sum_f32_300000_by_3_seg5000.info")
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path, out_dir=str(tmp_path))
    assert ("grouped by segment" if schedule == "by_segment" else "grouped by bucket") in kernel.source
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 760)
    ids = inputs[1]
    rng = np.random.default_rng(harness.BASE_SEED + 761)
    if pattern == "one_segment":
        ids[...] = 4999
    elif pattern == "sorted":
        ids[...] = np.sort(ids.reshape(-1)).reshape(ids.shape)
    elif pattern == "runs_of_64":
        ids[...] = np.repeat(rng.integers(0, 5000, size=(ids.size + 63) // 64), 64)[:ids.size].reshape(ids.shape)
    elif pattern == "one_bucket":
        ids[...] = rng.integers(4992, 5000, size=ids.shape)
    else:
        outside = rng.random(ids.shape) < 0.9
        ids[outside] = rng.choice(np.array([-1, -70000, 5000, 2 ** 31 - 1], dtype=ids.dtype), size=int(outside.sum()))
    expect = cpu_ref.CpuKernel(path)(inputs)
    for launch in range(2):
        got = run_on_gpu(kernel, inputs)
        assert np.array_equal(got[0].view(np.uint8), expect[0].view(np.uint8)), "%s launch %d" % (pattern, launch)


# Shapes the dynamic descriptions of the reference's test tree are specialised to (input_desc order).
REF_DYNAMIC_SHAPES = {
    "Fused_Cast_Sub_Mul_split_14802837530264465372": [[[32, 1, 48, 48]], [[32, 1, 5, 1000]], [[32, 1, 48, 40]]],
    "Fused_Mul_Add_ReduceMax_split_8454462579718005500": [[[32, 1, 40, 72], [32, 12, 40, 72]], [[1, 1, 16, 520], [32, 12, 16, 520]],
                                                          [[32, 1, 9, 72], [32, 12, 9, 72]]],
    "Fused_RealDiv_split_4177286244677596212": [[[32, 12, 24, 40], [32, 12, 24, 1]], [[32, 12, 7, 40], [32, 12, 7, 1]],
                                                [[32, 12, 24, 136], [32, 12, 24, 1]]],
    "Fused_ReduceMax_fusion_2054638663855723468": [[[100, 768]], [[3, 768]], [[2048, 768]]],
    "Fused_ReduceMax_fusion_234578345729057892345": [[[4096, 33]], [[4096, 4096]], [[4096, 40]]],
    "Fused_Sub_Exp_ReduceSum_split_7283368012049929718": [[[32, 12, 24, 40], [32, 12, 24, 1]], [[32, 12, 5, 40], [32, 12, 5, 1]],
                                                          [[32, 12, 24, 1000], [32, 12, 24, 1]]],
    "Fused_Sub_Mul_Cast_fusion_4217325526348104075": [[[32, 16, 20, 64], [32, 16, 20, 1], [32, 16, 20, 64]],
                                                      [[32, 16, 3, 64], [32, 16, 3, 1], [32, 16, 3, 64]],
                                                      [[32, 16, 20, 72], [32, 16, 20, 1], [32, 16, 20, 72]]],
    "Fused_Sub_Mul_split_1454621004286351279": [[[32, 1, 48, 48]], [[32, 1, 6, 48]], [[32, 1, 48, 520]]],
    "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957.dynamic": [[[32, 1, 48, 48], [32, 12, 48, 48]], [[1, 1, 40, 72], [32, 12, 40, 72]],
                                                                          [[32, 1, 7, 1000], [32, 12, 7, 1000]]],
    "elem_dyn_fuse_broadcast": [[[4096, 96], [96], [1, 96]], [[4096, 7], [7], [1, 7]], [[4096, 1000], [1000], [1, 1000]]],
}


def _bind_description(desc, shapes):
    """The test's own shape derivation for the dynamic reference descriptions (written apart from the product's):
    numpy broadcasting for elementwise ops, the axis attribute for reductions, element count for a Reshape."""
    d = json_loads(__import__("json").dumps(desc))
    env = {}
    for entry, shape in zip(d["input_desc"], shapes):
        entry[0]["shape"] = list(shape)
        env[entry[0]["tensor_name"]] = list(shape)
    for od in d["op_desc"]:
        attrs = {a["name"]: a["value"] for a in (od.get("attr") or [])}
        ins = []
        for entry in od["input_desc"]:
            if entry[0]["tensor_name"] in env:
                entry[0]["shape"] = env[entry[0]["tensor_name"]]
            if "value" not in entry[0] or entry[0]["tensor_name"] in env:
                ins.append(tuple(entry[0]["shape"]))
        declared = od["output_desc"][0]["shape"]
        if od["name"].startswith("Reduce"):
            axes = attrs["axis"] if "axis" in attrs else od["input_desc"][1][0]["value"]
            axes = [a % len(ins[0]) for a in (axes if isinstance(axes, list) else [axes])]
            keep = bool(attrs.get("keep_dims", False))
            out = [1 if i in axes else n for i, n in enumerate(ins[0]) if keep or i not in axes] or [1]
        elif od["name"] == "Reshape":
            known = int(np.prod([n for n in declared if n >= 0]))
            out = [n if n >= 0 else int(np.prod(ins[0])) // known for n in declared]
        else:
            out = list(np.broadcast_shapes(*ins))
            out = [1] * (len(declared) - len(out)) + out
        od["output_desc"][0]["shape"] = out
        env[od["output_desc"][0]["tensor_name"]] = out
    for o in d["output_desc"]:
        o["shape"] = env[o["tensor_name"]]
    return d


@pytest.mark.parametrize("name", [n for n in REF_DYNAMIC if "Softmax_fusion" not in n])
def test_reference_dynamic_descriptions_specialised(name):
    """Every other dynamic-shape description of the reference's test tree, specialised to one or two shape sets."""
    from oracle import np_ref
    path = os.path.join(REF_INFO, name)
    desc = harness.load_desc(path)
    dyn = driver.HipDynamicKernel(open(path, encoding="utf-8").read())
    for shapes in REF_DYNAMIC_SHAPES[name.split(".info")[0]]:
        kernel = dyn.specialize(shapes)
        bound = _bind_description(desc, shapes)
        assert [t.shape for t in kernel.outputs] == [o["shape"] for o in bound["output_desc"]]
        inputs = harness.make_inputs(bound, seed=harness.BASE_SEED + 650)
        got = run_on_gpu(kernel, inputs)
        expect = np_ref.evaluate(bound, inputs)
        wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
        exact = np_ref.evaluate(harness.widen_to_float64(bound), wide)
        full = max(int(np.prod(s)) for s in shapes)
        for d, g, e, x in zip(kernel.outputs, got, expect, exact):
            terms = max(1, full // max(1, g.size))
            if d.dtype == "float32" and terms > 1 and any(o["name"] == "ReduceSum" for o in desc["op_desc"]):
                ok, msg = harness.compare_reassociated(g, x, d.dtype, terms)
            else:
                ok, msg = harness.compare(g, e, d.dtype)
            print("  %s %s %s %s: %s" % (kernel.family, shapes, d.name, d.dtype, msg), flush=True)
            assert ok, "%s %s output %s: %s" % (name, shapes, d.name, msg)


@pytest.mark.parametrize("name", REF_DYNAMIC)
def test_reference_dynamic_descriptions_through_the_packed_calling_form(name):
    """All ten dynamic-shape descriptions of the reference's test tree, three shape sets each, called the way the
    reference calls a dynamic kernel: one array of data pointers and one of [offset, sizes, strides] lists
    (LLVMParameterPacking.cpp:91-194); the library reads the shapes from the lists and finds or makes the
    specialisation. The first set is launched again at the end: it must come from the cache (same handle)."""
    import torch
    from oracle import np_ref
    path = os.path.join(REF_INFO, name)
    desc = harness.load_desc(path)
    dyn = driver.HipDynamicKernel(open(path, encoding="utf-8").read())
    sets = REF_DYNAMIC_SHAPES[name.split(".info")[0]]
    assert len(sets) >= 3
    dev = torch.device("cuda:0")
    seen = []
    for shapes in sets + sets[:1]:
        bound = _bind_description(desc, shapes)
        inputs = harness.make_inputs(bound, seed=harness.BASE_SEED + 651)
        ins = [_torch_view(a).to(dev) for a in inputs]
        out_shapes = [o["shape"] for o in bound["output_desc"]]
        out_dtypes = [o["data_type"] for o in bound["output_desc"]]
        outs = []
        for shp, dt in zip(out_shapes, out_dtypes):
            t = torch.empty(int(np.prod(shp)) * np.dtype(driver.NP_HOST_DTYPE[dt]).itemsize, dtype=torch.uint8, device=dev)
            t.fill_(0xFF if dt in ("float16", "bfloat16", "float32", "float64") else 0x7B)
            outs.append(t)
        kernel = dyn.launch_packed([t.data_ptr() for t in ins + outs], list(shapes) + out_shapes,
                                   torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        seen.append(kernel)
        print("  %s %s: %s, made in %.1f ms%s" % (name[:40], shapes, kernel.family, kernel.build_ms,
                                                 " (no device compilation)" if kernel.cache_hit else ""), flush=True)
        got = [o.cpu().numpy().view(driver.NP_HOST_DTYPE[dt]).reshape(shp) for o, dt, shp in zip(outs, out_dtypes, out_shapes)]
        expect = np_ref.evaluate(bound, inputs)
        wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
        exact = np_ref.evaluate(harness.widen_to_float64(bound), wide)
        full = max(int(np.prod(s)) for s in shapes)
        for dt, g, e, x in zip(out_dtypes, got, expect, exact):
            terms = max(1, full // max(1, g.size))
            if dt == "float32" and terms > 1 and any(o["name"] == "ReduceSum" for o in desc["op_desc"]):
                ok, msg = harness.compare_reassociated(g, x, dt, terms)
            else:
                ok, msg = harness.compare(g, e, dt)
            assert ok, "%s %s: %s" % (name, shapes, msg)
    assert seen[-1] is seen[0]
    # a wrong output shape and a strided tensor are refused, not launched
    shapes = sets[0]
    bound = _bind_description(desc, shapes)
    out_shapes = [o["shape"] for o in bound["output_desc"]]
    bad = [list(s) for s in out_shapes]
    bad[0][-1] += 1
    with pytest.raises(driver.AkgHipError) as e:
        dyn.launch_packed([ins[0].data_ptr()] * (len(shapes) + len(out_shapes)), list(shapes) + bad)
    assert e.value.code == -1


def _open_dims(text, rows, cols):
    """Turns the extents `rows` and `cols` of a description built for those sentinel sizes into open (-1) dimensions."""
    d = json_loads(text)

    def walk(x):
        if isinstance(x, dict):
            if "shape" in x:
                x["shape"] = [-1 if n in (rows, cols) else n for n in x["shape"]]
            for v in x.values():
                walk(v)
        elif isinstance(x, list):
            for v in x:
                walk(v)
    walk(d)
    return d


@pytest.mark.parametrize("pattern", ["softmax_f16", "layernorm_bf16", "quant_bf16", "bias_gelu_f32"])
def test_row_lengths_of_one_bucket_share_a_code_object_and_stay_correct(pattern):
    """Dynamic descriptions take the row length as a kernel argument: the schedule is made for a power-of-two bucket of
    chunk counts, chunks are element-aligned and the last one overlaps its neighbour by a run-time amount; rows that are
    whole 64-byte pieces in every tensor have a source of their own (no overlap, whole lines streamed). Row lengths
    across a bucket (odd ones, the bucket's ends, one chunk short of it, two whole-line ones), with different row counts:
    the first of its kind makes the code object, the others must reuse it (no device compilation) and all must match
    the oracle."""
    from oracle import np_ref
    R, C = 7777, 9999
    if pattern == "softmax_f16":
        text, v, lengths = op_desc.softmax_last_axis(R, C, "float16", "dyn_softmax_f16"), 8, [520, 1000, 1024, 513, 777, 768]
    elif pattern == "layernorm_bf16":
        text, v, lengths = op_desc.layernorm_residual(R, C, "bfloat16", 1e-5, "dyn_layernorm_bf16"), 8, [4096, 2056, 3001, 4095, 3072]
    elif pattern == "quant_bf16":
        text, v, lengths = op_desc.quant_int8_residual(R, C, "bfloat16", "dyn_quant_bf16"), 8, [300, 264, 511, 512, 320]
    else:
        b = op_desc.DescBuilder("dyn_bias_gelu_f32")
        x, bias = b.input([R, C], "float32"), b.input([C], "float32")
        y = b.add(x, bias)
        text, v, lengths = b.dumps([b.mul(y, b.unary("Tanh", y))]), 4, [72, 100, 128, 68]
    desc = _open_dims(text, R, C)
    dyn = driver.HipDynamicKernel(__import__("json").dumps(desc), out_dir=None)
    narrowest = min(np.dtype(driver.NP_HOST_DTYPE[e[0]["data_type"]]).itemsize for e in desc["input_desc"] + [desc["output_desc"][:1]])
    first = {}
    for n, cols in enumerate(lengths):
        rows = [37, 5, 130, 64, 2][n % 5]
        # the description's open dims are (rows, cols) for matrices and (cols) for vectors
        shapes = [[cols] if len(e[0]["shape"]) == 1 else [rows, cols] for e in desc["input_desc"]]
        kernel = dyn.specialize(shapes)
        bound = _bind_description(desc, shapes)
        inputs = harness.make_inputs(bound, seed=harness.BASE_SEED + 41 + n)
        got = run_on_gpu(kernel, inputs)
        expect = np_ref.evaluate(bound, inputs)
        for d, g, e in zip(kernel.outputs, got, expect):
            ok, msg = harness.compare(g, e, d.dtype)
            print("  %s rows %d cols %d %s: %s (made in %.1f ms, cache_hit %s)" % (pattern, rows, cols, d.name, msg, kernel.build_ms,
                                                                                 kernel.cache_hit), flush=True)
            assert ok, "%s cols %d output %s: %s" % (pattern, cols, d.name, msg)
        # rows of the row kernels that are whole 64-byte pieces in every tensor have a source of their own in the bucket
        whole = pattern != "bias_gelu_f32" and (cols * narrowest) % 64 == 0
        assert ("akg_overlap" not in kernel.source) == (whole or pattern == "bias_gelu_f32")
        if whole not in first:
            first[whole] = kernel
        elif pattern != "bias_gelu_f32" or cols % v == 0:
            assert kernel.cache_hit, "%s: row length %d compiled anew" % (pattern, cols)


def _bind_softmax_description(desc, shapes):
    """The test's own reading of the dynamic description: numpy broadcasting for the elementwise ops, axis 3 kept as 1
    for the two reductions. Written apart from the product's shape derivation on purpose."""
    d = json_loads(__import__("json").dumps(desc))
    env = {}
    for entry, shape in zip(d["input_desc"], shapes):
        entry[0]["shape"] = list(shape)
        env[entry[0]["tensor_name"]] = list(shape)
    for od in d["op_desc"]:
        ins = []
        for entry in od["input_desc"]:
            if entry[0]["tensor_name"] in env:
                entry[0]["shape"] = env[entry[0]["tensor_name"]]
            ins.append(tuple(entry[0]["shape"]))
        if od["name"].startswith("Reduce"):
            out = list(ins[0])
            out[3] = 1
        else:
            out = list(np.broadcast_shapes(*ins))
        od["output_desc"][0]["shape"] = out
        env[od["output_desc"][0]["tensor_name"]] = out
    for o in d["output_desc"]:
        o["shape"] = env[o["tensor_name"]]
    return d


@pytest.mark.parametrize("shapes", [[[32, 1, 48, 48], [32, 12, 48, 48]], [[1, 1, 40, 72], [32, 12, 40, 72]],
                                    [[32, 1, 7, 1000], [32, 12, 7, 1000]]])
def test_reference_dynamic_shape_softmax_specialised_per_shape(shapes):
    """The reference's dynamic-shape system-test description (masked attention softmax, every extent but 32 x 12 open),
    specialised to three shape sets through akg_hip_dynamic_specialize and checked against the oracle evaluated on the
    description with the same shapes written in."""
    from oracle import np_ref
    path = os.path.join(REF_INFO, "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957.dynamic.info")
    desc = harness.load_desc(path)
    dyn = driver.HipDynamicKernel(open(path, encoding="utf-8").read())
    kernel = dyn.specialize(shapes)
    bound = _bind_softmax_description(desc, shapes)
    assert [t.shape for t in kernel.outputs] == [bound["output_desc"][0]["shape"]]
    rng = np.random.default_rng(harness.BASE_SEED + 600)
    mask = (rng.random(shapes[0]) < 0.8).astype(np.float32)          # 1 = keep, 0 = masked out by -10000
    scores = (rng.standard_normal(shapes[1], dtype=np.float32) * 4).astype(np.float32)
    got = run_on_gpu(kernel, [mask, scores])[0]
    expect = np_ref.evaluate(bound, [mask, scores])[0]
    ok, msg = harness.compare(got, expect, "float32")
    print("  shapes %s: %s" % (shapes, msg), flush=True)
    assert ok, msg
    assert np.allclose(got.sum(axis=3), 1.0, atol=1e-5)


@pytest.mark.parametrize("name", ["small_momentum_update_f32_37x130", "small_momentum_update_bf16_64x256"])
def test_assign_overwrites_its_destination_inputs(name):
    """Assign / InplaceAssign write their value over a kernel INPUT (the momentum and the parameter of an optimizer
    step) besides returning it: the device copies of those inputs must hold the oracle's updated values afterwards, the
    untouched input must be unchanged, and a second launch must apply a second step."""
    import torch
    path = os.path.join(FIXTURES, name + ".info")
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 700)
    dev = torch.device("cuda:0")
    ins = [_torch_view(a.copy()).to(dev) for a in inputs]
    outs = [torch.empty(d.nbytes, dtype=torch.uint8, device=dev) for d in kernel.outputs]
    oracle = cpu_ref.CpuKernel(path)
    host = [a.copy() for a in inputs]
    for step in range(2):
        kernel.launch(ins + outs)
        torch.cuda.synchronize()
        expect_out = oracle(host)                       # updates host[0] (parameter) and host[1] (momentum) in place
        for d, o, e in zip(kernel.outputs, outs, expect_out):
            got = o.cpu().numpy().view(driver.NP_HOST_DTYPE[d.dtype]).reshape(d.shape)
            ok, msg = harness.compare(got, e, d.dtype)
            assert ok, "step %d output %s: %s" % (step, d.name, msg)
        for i, (t, h) in enumerate(zip(ins, host)):
            got = t.cpu().numpy().view(h.dtype).reshape(h.shape)
            ok, msg = harness.compare(got, h, desc["input_desc"][i][0]["data_type"])
            print("  step %d input %d: %s" % (step, i, msg), flush=True)
            assert ok, "step %d input %d: %s" % (step, i, msg)
        assert np.array_equal(host[2], inputs[2])       # the gradient is only read
    assert not np.array_equal(host[0], inputs[0]) and not np.array_equal(host[1], inputs[1])


@pytest.mark.parametrize("name", ["small_sgdclip_update_f32_300x130", "small_sgdclip_update_bf16_64x256"])
def test_assign_in_a_description_that_runs_as_several_kernels(name):
    """SGD with clipping by the global gradient norm: the norm is a reduction over the whole gradient (first kernel),
    the update an Assign over the parameter (last kernel, after every read of the parameter). Two steps: the norm
    against the float64 evaluation, the parameter on the device against the oracle's updated copy, the gradient
    untouched."""
    import torch
    from oracle import np_ref
    path = os.path.join(FIXTURES, name + ".info")
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    assert kernel.family == "staged"
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 770)
    dev = torch.device("cuda:0")
    ins = [_torch_view(a.copy()).to(dev) for a in inputs]
    outs = [torch.empty(d.nbytes, dtype=torch.uint8, device=dev) for d in kernel.outputs]
    oracle = cpu_ref.CpuKernel(path)
    host = [a.copy() for a in inputs]
    for step in range(2):
        wide = [a.astype(np.float64) if a.dtype == np.float32 else a.copy() for a in host]
        exact = np_ref.evaluate(harness.widen_to_float64(desc), wide, {})
        kernel.launch(ins + outs)
        torch.cuda.synchronize()
        expect_out = oracle(host)                       # updates host[0] (the parameter) in place
        got = [o.cpu().numpy().view(driver.NP_HOST_DTYPE[d.dtype]).reshape(d.shape) for d, o in zip(kernel.outputs, outs)]
        ok, msg = harness.compare(got[0], expect_out[0], kernel.outputs[0].dtype)
        assert ok, "step %d parameter output: %s" % (step, msg)
        ok, msg = harness.compare_reassociated(got[1], exact[1], "float32", inputs[1].size)
        assert ok, "step %d norm: %s" % (step, msg)
        on_device = ins[0].cpu().numpy().view(host[0].dtype).reshape(host[0].shape)
        ok, msg = harness.compare(on_device, host[0], desc["input_desc"][0][0]["data_type"])
        assert ok, "step %d parameter on the device: %s" % (step, msg)
        assert np.array_equal(ins[1].cpu().numpy().view(inputs[1].dtype).reshape(inputs[1].shape), inputs[1])
    assert not np.array_equal(host[0], inputs[0])


@pytest.mark.parametrize("name", ["small_bnstats_update_f32_32x16x28x28", "small_bnstats_update_bf16_8x6x7x12"])
def test_running_statistics_are_assigned_after_the_reduction(name):
    """Batch-norm statistics with the running mean and variance updated in place (Assign after a streaming reduction):
    mean, variance and the updated running statistics against the float64 evaluation; two launches apply two updates;
    the activations are only read."""
    import torch
    from oracle import np_ref
    path = os.path.join(FIXTURES, name + ".info")
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    assert kernel.family == "stream_reduce"
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 710)
    inputs[2] = np.abs(inputs[2]) + 0.5                               # a running variance
    dev = torch.device("cuda:0")
    ins = [_torch_view(a.copy()).to(dev) for a in inputs]
    outs = [torch.empty(d.nbytes, dtype=torch.uint8, device=dev) for d in kernel.outputs]
    host = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
    terms = int(np.prod(desc["input_desc"][0][0]["shape"])) // host[1].size
    for step in range(2):
        kernel.launch(ins + outs)
        torch.cuda.synchronize()
        updates = {}
        exact = np_ref.evaluate(harness.widen_to_float64(desc), host, updates)
        for d, o, e in zip(kernel.outputs, outs, exact):
            got = o.cpu().numpy().view(driver.NP_HOST_DTYPE[d.dtype]).reshape(d.shape)
            ok, msg = harness.compare_reassociated(got, e, d.dtype, terms)
            print("  step %d %s: %s" % (step, d.name, msg), flush=True)
            assert ok, "step %d output %s: %s" % (step, d.name, msg)
        assert sorted(updates) == [1, 2]
        for i, new in updates.items():
            host[i] = np.asarray(new, dtype=np.float64)
            got = ins[i].cpu().numpy().view(np.float32).reshape(host[i].shape)
            ok, msg = harness.compare_reassociated(got, host[i], "float32", terms)
            assert ok, "step %d running statistic %d: %s" % (step, i, msg)
        assert np.array_equal(ins[0].cpu().numpy().view(inputs[0].dtype).reshape(inputs[0].shape), inputs[0])
    assert not np.allclose(host[1], inputs[1])


def test_float32_tanh_accuracy_over_the_whole_range():
    """The float32 tanh of the device op library is an own implementation (series below 0.25, hardware exp2 and
    reciprocal above): its error against the float64 value is measured on 8M arguments, dense around the branch
    point and log-spaced over every magnitude, and must stay an order of magnitude inside the 1e-5 bar."""
    from akg_amd import op_desc
    rows, cols = 2048, 4096
    b = op_desc.DescBuilder("Fused_Tanh_accuracy_f32_%dx%d" % (rows, cols))
    x = b.input([rows, cols], "float32")
    kernel = driver.HipKernel(b.dumps([b.unary("Tanh", x)]))
    rng = np.random.default_rng(harness.BASE_SEED + 500)
    n = rows * cols
    mag = np.concatenate([
        np.exp(rng.uniform(np.log(1e-30), np.log(100.0), n // 2)),      # every magnitude
        rng.uniform(0.0, 12.0, n // 4),                                  # where tanh bends and saturates
        rng.uniform(0.2, 0.3, n // 4 - 16),                              # around the branch point
        [0.0, 0.25, np.nextafter(np.float32(0.25), np.float32(0)), 1e-45, 1e-38, 44.0, 45.0, 88.0, 1e30, np.inf,
         np.nan, 9.0, 9.5, 10.0, 0.5, 1.0]]).astype(np.float32)
    sign = np.where(rng.random(n) < 0.5, -1.0, 1.0).astype(np.float32)
    xs = (mag * sign).reshape(rows, cols)
    got = run_on_gpu(kernel, [xs])[0].astype(np.float64)
    ref = np.tanh(xs.astype(np.float64))
    finite = np.isfinite(ref) & (ref != 0)
    rel = np.abs(got[finite] - ref[finite]) / np.abs(ref[finite])
    print("  tanh float32: max relative error %.3g over %d arguments" % (rel.max(), rel.size), flush=True)
    assert rel.max() < 2e-6
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    zero = xs == 0
    assert np.all(got[zero] == 0) and np.array_equal(np.signbit(got[zero]), np.signbit(xs[zero]))
    assert np.all(np.abs(got[np.isfinite(got)]) <= 1.0)


def test_run_host_reference_style_call_and_driver():
    """Host pointers in, outputs overwritten in place (the reference shim's calling convention), through HipDriver."""
    path = os.path.join(FIXTURES, "small_layernorm_residual_bf16_19x520.info")
    desc = harness.load_desc(path)
    d = driver.HipDriver(input_file=path)
    kernel = d.compile()
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 300)
    outs = kernel.empty_outputs(fill_nan=True)
    res = d.run(inputs + outs, output_indexes=[-1])
    assert res[0] is outs[0]
    expect = cpu_ref.CpuKernel(path)(inputs)
    ok, msg = harness.compare(outs[0], expect[0], "bfloat16")
    assert ok, msg
    # wrong tensor count is an error, not a crash
    with pytest.raises(ValueError):
        kernel.run_host(inputs)


def test_profile_entry_point_returns_a_plausible_time():
    import torch
    path = os.path.join(FIXTURES, "small_softmax_f16_64x4096.info")
    kernel = driver.HipKernel.from_file(path)
    bufs = [torch.zeros(t.nbytes, dtype=torch.uint8, device="cuda:0") for t in kernel.tensors]
    ms = kernel.profile_ptrs([b.data_ptr() for b in bufs], number=5, repeat=3)
    assert 0.0 < ms < 50.0


@pytest.mark.parametrize("kind", sorted(DYNAMIC_STREAMS))
def test_dynamic_streaming_reductions_share_one_code_object_across_reduced_extents(kind):
    """A reduction over the outermost extent of its operand (column sums over the tokens, a whole tensor into one number)
    with that extent open: the reference compiles such a kernel once and passes sizes at call time
    (LLVMParameterPacking.cpp:91-194). Here the reduced extent, the share of it a workgroup walks and the number of
    workgroups that share a result are kernel arguments: one code object for every extent, the split chosen per call
    (one workgroup per result for the short extents, several hundred for the long ones). Float32 sums against
    the float64 evaluation (they are reassociated), everything else against the oracle; 16-bit declared sums bit for
    bit. Every handle is launched twice (the arrival counters must be left at zero)."""
    from oracle import np_ref
    make = DYNAMIC_STREAMS[kind]
    sentinel = 7777
    dyn = driver.HipDynamicKernel(open_extent(make(sentinel, "dyn_" + kind), sentinel), out_dir=None)
    first = None
    for t in (6000, 40, 16384, 7, 1000, 2):
        bound = json_loads(make(t, "dyn_" + kind))
        shapes = [e[0]["shape"] for e in bound["input_desc"]]
        kernel = dyn.specialize(shapes)
        print("  %s T=%d: %s grid %d block %d, made in %.1f ms%s" % (kind, t, kernel.family, kernel.grid[0], kernel.block[0], kernel.build_ms,
                                                                      " (no device compilation)" if kernel.cache_hit else ""), flush=True)
        assert kernel.family == "stream_reduce" and "akg_r_arg" in kernel.source
        if first is None:
            first = kernel.source
        else:
            assert kernel.cache_hit and kernel.source == first, "T=%d made a new source" % t
        inputs = harness.make_inputs(bound, seed=harness.BASE_SEED + 77 + t)
        expect = np_ref.evaluate(bound, inputs)
        wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
        exact = np_ref.evaluate(harness.widen_to_float64(bound), wide)
        in_numel = max(int(np.prod(s)) for s in shapes)
        for launch in range(2):
            got = run_on_gpu(kernel, inputs)
            for j, (d, g, e, x) in enumerate(zip(kernel.outputs, got, expect, exact)):
                float_sum = kind in ("biasgrad_bf16", "sqsum_all_f32") or (kind == "norm_absmax_all_f32" and j == 0)
                if kind.startswith("declared"):
                    ok, msg = harness.compare_bits(g, e, d.dtype)
                elif float_sum:
                    ok, msg = harness.compare_reassociated(g, x, d.dtype, max(1, in_numel // max(1, g.size)))
                else:
                    ok, msg = harness.compare(g, e, d.dtype)
                print("    launch %d %s %s: %s" % (launch, d.name, d.dtype, msg), flush=True)
                assert ok, "%s T=%d output %s: %s" % (kind, t, d.name, msg)


@pytest.mark.parametrize("kind", sorted(DYNAMIC_POOLS) + sorted(DYNAMIC_STATS))
def test_dynamic_streaming_reductions_behind_an_open_batch(kind):
    """[batch, tokens, hidden] reduced over the tokens with batch and tokens both open (what a batch index advances by is
    then computed from the token count in the kernel), also with operands that span only some of the extents; and the
    per-channel statistics of [N,C,H,W] with the batch open (the reduced extent N * H * W is the argument, the channels
    lie between the reduced extents; 7 x 7 images keep their overlapping chunks). One code object per description, up to
    the choice of the workgroup numbering for small grids. Float32 sums against the float64 evaluation, the maxima
    against the oracle; two launches per handle."""
    from oracle import np_ref
    sources = set()
    if kind in DYNAMIC_POOLS:
        make = DYNAMIC_POOLS[kind]
        dyn = driver.HipDynamicKernel(open_extent(make(7777, 5555, "dyn_" + kind), (7777, 5555)), out_dir=None)
        bounds = [json_loads(make(b, t, "dyn_" + kind)) for b, t in ((4, 300), (32, 64), (2, 5000), (7, 9), (1, 700))]
        arg = "akg_o_arg"
    else:
        make = DYNAMIC_STATS[kind]
        dyn = driver.HipDynamicKernel(open_extent(make(7777, "dyn_" + kind), 7777), out_dir=None)
        bounds = [json_loads(make(n, "dyn_" + kind)) for n in (8, 256, 3, 64)]
        arg = "akg_r_arg"
    for bound in bounds:
        shapes = [e[0]["shape"] for e in bound["input_desc"]]
        kernel = dyn.specialize(shapes)
        print("  %s %s: %s grid %d block %d, made in %.1f ms%s" % (kind, shapes[0], kernel.family, kernel.grid[0], kernel.block[0], kernel.build_ms,
                                                                    " (no device compilation)" if kernel.cache_hit else ""), flush=True)
        assert kernel.family == "stream_reduce"
        if shapes[0][0] > 1:
            assert arg in kernel.source
            sources.add(kernel.source)
        inputs = harness.make_inputs(bound, seed=harness.BASE_SEED + 99 + shapes[0][0])
        expect = np_ref.evaluate(bound, inputs)
        wide = [a.astype(np.float64) if a.dtype == np.float32 else a for a in inputs]
        exact = np_ref.evaluate(harness.widen_to_float64(bound), wide)
        in_numel = max(int(np.prod(sh)) for sh in shapes)
        is_max = [o["name"] == "ReduceMax" for o in bound["op_desc"] if o["output_desc"][0]["tensor_name"] in
                  [x["tensor_name"] for x in bound["output_desc"]]]
        for launch in range(2):
            got = run_on_gpu(kernel, inputs)
            for j, (d, g, e, x) in enumerate(zip(kernel.outputs, got, expect, exact)):
                if j < len(is_max) and is_max[j]:
                    ok, msg = harness.compare(g, e, d.dtype)
                else:
                    ok, msg = harness.compare_reassociated(g, x, d.dtype, max(1, in_numel // max(1, g.size)))
                print("    launch %d %s %s: %s" % (launch, d.name, d.dtype, msg), flush=True)
                assert ok, "%s %s output %s: %s" % (kind, shapes[0], d.name, msg)
    # (the statistics change their workgroup numbering for small grids; 7 x 9 x 7 has a reduced extent no chunk divides)
    assert len(sources) <= (2 if kind in DYNAMIC_STATS or kind == "rowmax_equal_extents_bf16" else 1), "%d sources" % len(sources)


@pytest.mark.parametrize("kind", sorted(DYNAMIC_VIEWS))
def test_dynamic_data_movement_with_an_open_batch(kind):
    """Transposes (through index maps and through LDS tiles) with the batch open share one code object: the number of
    chunks is a kernel argument and the workgroup numbering does not name the outermost extent. Ops that work on the
    open axis itself (a Concat or a Tile along the batch) keep its extent in their index maps: every batch size is its
    own source there, and every result is still right. Data movement is exact: bit for bit against the oracle."""
    from oracle import np_ref
    make, sentinels, shared = DYNAMIC_VIEWS[kind]
    dyn = driver.HipDynamicKernel(open_extent(make(7777, "dyn_" + kind), sentinels), out_dir=None)
    sources = set()
    for n in (4, 32, 3):
        bound = json_loads(make(n, "dyn_" + kind))
        shapes = [e[0]["shape"] for e in bound["input_desc"]]
        kernel = dyn.specialize(shapes)
        print("  %s N=%d: %s grid %d, made in %.1f ms%s" % (kind, n, kernel.family, kernel.grid[0], kernel.build_ms,
                                                          " (no device compilation)" if kernel.cache_hit else ""), flush=True)
        assert kernel.family == "indexed"
        assert [t.shape for t in kernel.outputs] == [o["shape"] for o in bound["output_desc"]]
        sources.add(kernel.source)
        inputs = harness.make_inputs(bound, seed=harness.BASE_SEED + 111 + n)
        expect = np_ref.evaluate(bound, inputs)
        got = run_on_gpu(kernel, inputs)
        for d, g, e in zip(kernel.outputs, got, expect):
            ok, msg = harness.compare_bits(g, e, d.dtype)
            print("    %s %s: %s" % (d.name, d.dtype, msg), flush=True)
            assert ok, "%s N=%d output %s: %s" % (kind, n, d.name, msg)
    assert (len(sources) == 1) == shared, "%d sources" % len(sources)


@pytest.mark.parametrize("kind", sorted(DYNAMIC_COLUMNS))
def test_dynamic_column_kernels_share_one_code_object_across_batch_sizes(kind):
    """A softmax over the classes of [N,21,H,W] and a LayerNorm over the channels of [N,C,HW] with the batch open: the
    extent in front of the reduced axis is a kernel argument of the column kernel, so every batch size above one runs
    on one code object (LLVMParameterPacking.cpp:91-194: the reference passes sizes at call time). 16-bit results
    against the oracle."""
    from oracle import np_ref
    make = DYNAMIC_COLUMNS[kind]
    sentinel = 7777
    dyn = driver.HipDynamicKernel(open_extent(make(sentinel, "dyn_" + kind), sentinel), out_dir=None)
    first = None
    for n in (6, 2, 40, 3):
        bound = json_loads(make(n, "dyn_" + kind))
        shapes = [e[0]["shape"] for e in bound["input_desc"]]
        kernel = dyn.specialize(shapes)
        print("  %s N=%d: %s grid %d block %d, made in %.1f ms%s" % (kind, n, kernel.family, kernel.grid[0], kernel.block[0], kernel.build_ms,
                                                                      " (no device compilation)" if kernel.cache_hit else ""), flush=True)
        assert kernel.family == "column_reduce" and "akg_outer_arg" in kernel.source
        if first is None:
            first = kernel.source
        else:
            assert kernel.cache_hit and kernel.source == first, "N=%d made a new source" % n
        inputs = harness.make_inputs(bound, seed=harness.BASE_SEED + 88 + n)
        expect = np_ref.evaluate(bound, inputs)
        got = run_on_gpu(kernel, inputs)
        for d, g, e in zip(kernel.outputs, got, expect):
            ok, msg = harness.compare(g, e, d.dtype)
            print("    %s %s: %s" % (d.name, d.dtype, msg), flush=True)
            assert ok, "%s N=%d output %s: %s" % (kind, n, d.name, msg)


def test_sixteen_bit_matmul_on_the_matrix_units_by_switch(monkeypatch):
    """AKG_HIP_MATMUL_F32_ACC=1: a MatMul declared bfloat16 runs on the MFMA kernel with a float32 sum rounded once. That is
    not the reference's value (16-bit accumulation, which the default serial kernel reproduces bit for bit), so it is held
    to the float64 product of the same bfloat16 operands within the bfloat16 bar."""
    import torch
    monkeypatch.setenv("AKG_HIP_MATMUL_F32_ACC", "1")
    b = op_desc.DescBuilder("mm_bf16_f32acc")
    a_t = b.input([300, 1024], "bfloat16")
    w_t = b.input([1024, 520], "bfloat16")
    kernel = driver.HipKernel(b.dumps([b.matmul(a_t, w_t, "bfloat16")]), out_dir=None)
    assert "gemm_256x256" in kernel.source
    rng = np.random.default_rng(5)
    a = harness.f32_to_bf16_bits((rng.standard_normal((300, 1024)) * 0.25).astype(np.float32))
    w = harness.f32_to_bf16_bits((rng.standard_normal((1024, 520)) * 0.25).astype(np.float32))
    got = run_on_gpu(kernel, [a, w])[0]
    want = torch.from_numpy(harness.bf16_bits_to_f32(a)).double() @ torch.from_numpy(harness.bf16_bits_to_f32(w)).double()
    ok, msg = harness.compare(got, harness.f32_to_bf16_bits(want.float().numpy()), "bfloat16")
    print("  float32 accumulation rounded once vs float64: %s" % msg, flush=True)
    assert ok, msg


@pytest.mark.parametrize("kind", ["int8_dequant_bias_gelu", "bf16_bias_gelu_tb"])
def test_dynamic_matmul_shares_code_objects_across_token_counts(kind):
    """A MatMul fusion whose row count (the token count) is open: the reference compiles such a kernel once and passes
    sizes at call time (LLVMParameterPacking.cpp:91-194). Here M and the K split are kernel arguments of the tile kernel
    (every M above 64: one code object, the split chosen per call) and of the skinny kernel (three sizes: up to 16, 32
    and 64 rows), so a new token count costs a lowering and no device compilation. Results against the oracle of the
    same description written with the bound M: int8 fusions to the bf16 bar with exact accumulators behind them, bf16 to
    its bar."""
    from oracle import np_ref
    sentinel = 777
    if kind == "int8_dequant_bias_gelu":
        make = lambda m, name: op_desc.gemm_int8_dequant_bias_gelu(m, 2048, 1024, "bfloat16", False, name)   # noqa: E731
    else:
        make = lambda m, name: op_desc.gemm_bias_act(m, 2048, 1024, "bfloat16", "gelu", True, "float32", name)  # noqa: E731
    open_desc = json_loads(make(sentinel, "dyn_" + kind))

    def walk(x):
        if isinstance(x, dict):
            if "shape" in x:
                x["shape"] = [-1 if n == sentinel else n for n in x["shape"]]
            for v in x.values():
                walk(v)
        elif isinstance(x, list):
            for v in x:
                walk(v)
    walk(open_desc)
    dyn = driver.HipDynamicKernel(__import__("json").dumps(open_desc), out_dir=None)
    compiled = {}
    for m in (1000, 300, 2304, 65, 64, 48, 33, 32, 20, 16, 7, 2):
        bound = json_loads(make(m, "dyn_" + kind))
        shapes = [e[0]["shape"] for e in bound["input_desc"]]
        kernel = dyn.specialize(shapes)
        bucket = "tile" if m > 64 else ("skinny%d" % (16 if m <= 16 else 32 if m <= 32 else 64))
        print("  M=%d: %s grid %d block %d, made in %.1f ms%s" % (m, bucket, kernel.grid[0], kernel.block[0], kernel.build_ms,
                                                                " (no device compilation)" if kernel.cache_hit else ""), flush=True)
        if bucket in compiled:
            assert kernel.cache_hit and kernel.build_ms < 20.0, "M=%d compiled again (%s was built for M=%d)" % (m, bucket, compiled[bucket])
        else:
            compiled[bucket] = m
        inputs = harness.make_inputs(bound, seed=harness.BASE_SEED + 31 + m)
        got = run_on_gpu(kernel, inputs)
        expect = np_ref.evaluate(bound, inputs)
        for d, g, e in zip(kernel.outputs, got, expect):
            ok, msg = harness.compare(g, e, d.dtype)
            print("    %s %s: %s" % (d.name, d.dtype, msg), flush=True)
            assert ok, "M=%d output %s: %s" % (m, d.name, msg)
        if m in (1000, 300):
            # the kernel of the static description with this ragged M (rows clamped in front of the loop as well):
            # the same bits as the specialisation of the dynamic one
            fixed = run_on_gpu(driver.HipKernel(make(m, "dyn_" + kind), out_dir=None), inputs)
            for d, g, f, e in zip(kernel.outputs, got, fixed, expect):
                if kind == "int8_dequant_bias_gelu":   # exact accumulators: the same bits whatever the K split
                    assert np.array_equal(g.view(np.uint8), f.view(np.uint8)), "M=%d: static and dynamic kernels differ" % m
                ok, msg = harness.compare(f, e, d.dtype)
                assert ok, "M=%d (static) output %s: %s" % (m, d.name, msg)
    assert sorted(compiled) == ["skinny16", "skinny32", "skinny64", "tile"]


@pytest.mark.parametrize("m,k,n,tb", [(512, 8192, 512, False), (4096, 8192, 8192, False), (4096, 8192, 8192, True),
                                      (1000, 4112, 1032, False), (48, 8192, 4096, False)])
def test_bare_int8_matmul_accumulators_are_exact(m, k, n, tb):
    """MatMul int8 x int8 -> int32 with the accumulators themselves as the output (no epilogue to hide a dropped or doubled
    product behind a 16-bit tolerance), at the shape of the measured fusion and on ragged, split-K and skinny ones:
    every element equal to torch._int_mm's exact integer product, and sampled rows (spread over every row tile) equal
    to the oracle's exact accumulation."""
    import torch
    from oracle import np_ref
    b = op_desc.DescBuilder("bare_mm_i8_%dx%dx%d%s" % (m, k, n, "_tb" if tb else ""))
    a_t = b.input([m, k], "int8")
    w_t = b.input([n, k] if tb else [k, n], "int8")
    text = b.dumps([b.matmul(a_t, w_t, "int32", transpose_b=tb)])
    kernel = driver.HipKernel(text, out_dir=None)
    print("case %s: %s grid %d block %d" % (kernel.kernel_name, kernel.family, kernel.grid[0], kernel.block[0]), flush=True)
    assert kernel.family == "gemm_epilogue" and "mfma" in kernel.source
    rng = np.random.default_rng(harness.BASE_SEED + 55)
    a = rng.integers(-127, 128, size=(m, k), dtype=np.int8)
    w = rng.integers(-127, 128, size=(n, k) if tb else (k, n), dtype=np.int8)
    got = run_on_gpu(kernel, [a, w])[0]
    assert got.dtype == np.int32 and got.shape == (m, n)
    wk = np.ascontiguousarray(w.T) if tb else w
    rows = np.unique(np.concatenate([np.arange(0, m, max(1, m // 16)), rng.integers(0, m, 16), [m - 1]]))
    expect_rows = np_ref.matmul_exact_i32(a[rows], wk)
    bad = int(np.count_nonzero(got[rows] != expect_rows))
    print("  %d sampled rows vs exact accumulation: %d elements differ" % (len(rows), bad), flush=True)
    assert bad == 0
    dev = torch.device("cuda:0")
    # torch._int_mm wants at least 17 rows and extents that are multiples of 8: pad A with zero rows, compare the real ones
    pad_m = max(32, (m + 7) // 8 * 8)
    a_pad = np.zeros((pad_m, k), dtype=np.int8)
    a_pad[:m] = a
    ref = torch._int_mm(torch.from_numpy(a_pad).to(dev), torch.from_numpy(wk).to(dev))[:m].cpu().numpy()
    bad = int(np.count_nonzero(got != ref))
    print("  all %d accumulators vs torch._int_mm: %d differ" % (got.size, bad), flush=True)
    assert bad == 0


def test_c5_full_size_gemm_fusion():
    """Full configuration: 4096 x 8192 x 8192. The CPU oracle cannot run 2.7e11 MACs in a test, so:
    (1) 96 sampled rows (all 8192 columns each, rows spread over every 256-row tile) against the oracle evaluated on
        exactly those rows of A (exact int32 accumulation, same epilogue);
    (2) every output against an independent computation of the same formula with torch on the GPU
        (torch._int_mm for the exact int32 product), within the bfloat16 tolerance."""
    import torch
    from oracle import np_ref
    from akg_amd import op_desc
    name = "c5_gemm_i8_dequant_bias_gelu_4096x8192x8192.info"
    path = os.path.join(FIXTURES, name)
    print("case %s" % name, flush=True)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 5)
    got = run_on_gpu(kernel, inputs)[0]
    a, sa, w, sb, bias = inputs
    rng = np.random.default_rng(99)
    rows = np.sort(np.concatenate([np.arange(16) * 256 + rng.integers(0, 256, 16), rng.integers(0, 4096, 80)]))
    sub = json_loads(op_desc.gemm_int8_dequant_bias_gelu(len(rows), 8192, 8192, "bfloat16", False, "c5_rows"))
    expect_rows = np_ref.evaluate(sub, [a[rows], sa[rows], w, sb, bias])[0]
    ok, msg = harness.compare(got[rows], expect_rows, "bfloat16")
    print("  sampled rows vs oracle: %s" % msg, flush=True)
    assert ok, msg
    dev = torch.device("cuda:0")
    acc = torch._int_mm(torch.from_numpy(a).to(dev), torch.from_numpy(w).to(dev))
    x = acc.float() * torch.from_numpy(sa).to(dev) * torch.from_numpy(sb).to(dev)
    x = x + torch.from_numpy(harness.bf16_bits_to_f32(bias)).to(dev)
    ref = torch.nn.functional.gelu(x, approximate="tanh").to(torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)
    ok, msg = harness.compare(got, ref, "bfloat16")
    print("  all outputs vs torch: %s" % msg, flush=True)
    assert ok, msg


def test_full_size_bf16_gemm_bias_gelu_fusion():
    """bfloat16 MatMul + bias + GELU at 4096 x 8192 x 8192 (float32 accumulation on the MFMA units):
    (1) 48 sampled rows against the oracle (float32 products summed serially in k) evaluated on those rows of A;
    (2) every output against torch on the GPU (float32 matmul of the same bfloat16 values), bfloat16 tolerance."""
    import torch
    from oracle import np_ref
    from akg_amd import op_desc
    name = "n2_gemm_bf16_bias_gelu_4096x8192x8192.info"
    path = os.path.join(FIXTURES, name)
    print("case %s" % name, flush=True)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 6)
    got = run_on_gpu(kernel, inputs)[0]
    a, w, bias = inputs
    rng = np.random.default_rng(98)
    rows = np.sort(np.concatenate([np.arange(16) * 256 + rng.integers(0, 256, 16), rng.integers(0, 4096, 32)]))
    sub = json_loads(op_desc.gemm_bias_act(len(rows), 8192, 8192, "bfloat16", "gelu", False, "float32", "n2_rows"))
    expect_rows = np_ref.evaluate(sub, [a[rows], w, bias])[0]
    ok, msg = harness.compare(got[rows], expect_rows, "bfloat16")
    print("  sampled rows vs oracle: %s" % msg, flush=True)
    assert ok, msg
    dev = torch.device("cuda:0")
    as_f32 = lambda bits: torch.from_numpy(harness.bf16_bits_to_f32(bits)).to(dev)
    allow = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        x = as_f32(a) @ as_f32(w) + as_f32(bias)
    finally:
        torch.backends.cuda.matmul.allow_tf32 = allow
    ref = torch.nn.functional.gelu(x, approximate="tanh").to(torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)
    ok, msg = harness.compare(got, ref, "bfloat16")
    print("  all outputs vs torch: %s" % msg, flush=True)
    assert ok, msg


@pytest.mark.parametrize("m,transpose_b", [(147456, True), (139264, False)])
def test_matmul_whose_first_operand_is_larger_than_two_gib(m, transpose_b):
    """A of [147456, 8192] bfloat16 is 2.25 GiB: the rows beyond 131072 lie at byte offsets no 32-bit buffer offset
    reaches from the start of A, so the descriptor of A starts at each tile's first row. 64 sampled rows (every
    region of A, the last tile and the rows either side of the 2 GiB line among them) against the oracle evaluated on
    those rows, and the rest of the result must hold no NaN prefill."""
    from oracle import np_ref
    from akg_amd import op_desc
    k, n = 8192, 256
    name = "big_a_gemm_%dx%dx%d%s" % (m, k, n, "_tb" if transpose_b else "")
    print("case %s" % name, flush=True)
    text = op_desc.gemm_bias_act(m, k, n, "bfloat16", "gelu", transpose_b, "float32", name)
    desc = json_loads(text)
    kernel = driver.HipKernel(text, out_dir=None)
    assert kernel.family == "gemm_epilogue"
    rng = np.random.default_rng(4)
    small = harness.make_inputs(json_loads(op_desc.gemm_bias_act(4096, k, n, "bfloat16", "gelu", transpose_b, "float32", "p")), seed=harness.BASE_SEED + 8)
    a = np.tile(small[0], (m // 4096, 1))
    # every row its own: the row index into a few elements, so that a wrong row cannot pass for the right one
    a[:, 0] = harness.f32_to_bf16_bits((np.arange(m) % 251).astype(np.float32) / 64.0 - 2.0)
    a[:, 4097] = harness.f32_to_bf16_bits((np.arange(m) // 251 % 241).astype(np.float32) / 64.0 - 2.0)
    inputs = [a, small[1], small[2]]
    got = run_on_gpu(kernel, inputs)[0]
    line = (1 << 31) // (k * 2)   # first row beyond 2 GiB
    rows = np.unique(np.concatenate([[0, 255, 256, line - 2, line - 1, line, line + 1, line + 255, line + 256, m - 257, m - 256, m - 1],
                                     rng.integers(0, m, 52)]))
    sub = json_loads(op_desc.gemm_bias_act(len(rows), k, n, "bfloat16", "gelu", transpose_b, "float32", "rows"))
    expect_rows = np_ref.evaluate(sub, [a[rows], inputs[1], inputs[2]])[0]
    ok, msg = harness.compare(got[rows], expect_rows, "bfloat16")
    print("  sampled rows vs oracle: %s" % msg, flush=True)
    assert ok, msg
    assert not np.isnan(harness.bf16_bits_to_f32(got)).any()


SERIAL_GEMMS = ["small_gemm_f16_result_f16_bias_relu_70x200x36.info", "small_gemm_bf16_result_bf16_bias_none_33x129x5_tb.info",
                "small_gemm_f32_bias_gelu_70x100x36.info", "small_gemm_bf16_bias_gelu_65x30x10.info"]


@pytest.mark.parametrize("name", SERIAL_GEMMS)
def test_matmul_in_the_reference_arithmetic_is_bit_identical_to_the_oracle(name):
    """A MatMul whose declared result type is float16 / bfloat16 (the reference rounds the product and the sum to it at
    every k), or whose shape or element type the MFMA kernels do not take, runs as one serial chain over k per result
    element: the same additions in the same order as the oracle's loop nest, so the accumulators are identical. The
    fixtures without a transcendental epilogue are compared bit for bit, the GELU ones to the 16-bit / float32 bars."""
    path = os.path.join(FIXTURES, name)
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    assert kernel.family == "gemm_epilogue" and "gemm_serial" in kernel.source
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 16)
    got = run_on_gpu(kernel, inputs)[0]
    expect = cpu_ref.CpuKernel(path)(inputs)[0]
    if "gelu" in name:
        ok, msg = harness.compare(got, expect, kernel.outputs[0].dtype)
        assert ok, msg
    else:
        assert np.array_equal(got.view(np.uint16), expect.view(np.uint16))


def test_sixteen_bit_matmul_result_follows_the_declared_type_on_a_long_k():
    """4096 products of 1 in float16: the running sum stalls at 2048 as the reference's does; an accumulator that is
    silently float32 returns 4096."""
    from akg_amd import op_desc
    b = op_desc.DescBuilder("Fused_MatMul_f16_result_ones_8x4096x12")
    a = b.input([8, 4096], "float16")
    w = b.input([4096, 12], "float16")
    kernel = driver.HipKernel(b.dumps([b.matmul(a, w, "float16")]))
    got = run_on_gpu(kernel, [np.ones((8, 4096), np.float16), np.ones((4096, 12), np.float16)])[0]
    assert np.all(got.astype(np.float32) == 2048.0)


def json_loads(text):
    import json
    return json.loads(text)
