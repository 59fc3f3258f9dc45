"""Host-side logic, runnable without a GPU: the C-ABI library loads and exports every declared symbol, the JSON
translator reads descriptions the way the reference's does (checked against Python's own JSON reader on the reference's
own fixture files), error conventions, artifact formats, and the lowering decisions (family, schedule, math selection).
No kernel is launched here.
"""
import ctypes
import hashlib
import json
import os
import re
import subprocess

import numpy as np
import pytest

from akg_amd import driver, harness, op_desc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FIXTURES = os.path.join(ROOT, "akg_amd", "fixtures")
REF_INFO = os.path.join(ROOT, "tests", "golden", "ref_info")
HEADER = os.path.join(ROOT, "include", "akg_hip.h")


# ---------------------------------------------------------------------------------------------------------
# C ABI
# ---------------------------------------------------------------------------------------------------------
def declared_symbols():
    with open(HEADER, "r", encoding="utf-8") as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(akg_hip_[a-z_]+)\s*\(", text)))


def test_library_exports_every_symbol_the_header_declares():
    lib = driver.load_library()
    names = declared_symbols()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), "libakg_hip.so does not export %s" % n
    # and nothing in the signatures is a C++ / torch type: the header compiles as plain C
    r = subprocess.run(["gcc", "-std=c99", "-fsyntax-only", "-x", "c", HEADER], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_version_and_last_error():
    lib = driver.load_library()
    assert b"gfx950" in lib.akg_hip_version()
    h = ctypes.c_void_p()
    rc = lib.akg_hip_compile(b"{", 1, None, ctypes.byref(h))
    assert rc == -2 and not h.value
    assert b"json" in lib.akg_hip_last_error()


def test_null_arguments_are_rejected_not_crashed_on():
    lib = driver.load_library()
    h = ctypes.c_void_p()
    assert lib.akg_hip_compile(None, 0, None, ctypes.byref(h)) == -1
    assert lib.akg_hip_compile(b"{}", 2, None, None) == -1
    n = ctypes.c_int()
    assert lib.akg_hip_kernel_num_tensors(None, ctypes.byref(n)) == -1
    assert lib.akg_hip_launch(None, None, 0, None) == -1
    lib.akg_hip_kernel_destroy(None)


# ---------------------------------------------------------------------------------------------------------
# translator vs an independent JSON reader, on the reference's own fixture files
# ---------------------------------------------------------------------------------------------------------
def _static(name):
    d = harness.load_desc(os.path.join(REF_INFO, name))
    return not any(x < 0 for e in d["input_desc"] for x in e[0].get("shape", [1]))


# every static description of the reference's test tree
STATIC_REF = sorted(f for f in os.listdir(REF_INFO) if ".info" in f and _static(f))


@pytest.mark.parametrize("name", STATIC_REF)
def test_signature_of_reference_fixture_matches_python_json(name):
    path = os.path.join(REF_INFO, name)
    desc = harness.load_desc(path)
    text = driver.translate(open(path, "r", encoding="utf-8").read())
    # function name and attributes
    assert text.startswith("func.func @%s(" % desc["op"])
    assert 'process = "%s"' % desc["process"] in text
    arch = desc.get("target_info", {}).get("arch", "")
    assert 'arch = "%s"' % arch in text
    # inputs in input_desc order, outputs in output_desc order, uint8 read as int8
    head = text.split("\n", 1)[0]
    args = re.findall(r"%(\w+): tensor<([0-9x]*)(\w+)>", head)
    assert [a[0] for a in args] == [e[0]["tensor_name"] for e in desc["input_desc"]]
    for (nm, dims, dt), e in zip(args, desc["input_desc"]):
        want_dt = "int8" if e[0]["data_type"] == "uint8" else e[0]["data_type"]
        assert dt == want_dt
        assert [int(d) for d in dims.split("x") if d] == e[0].get("shape", [1])
    ret = re.search(r"return (.*)", text).group(1)
    assert [r.strip().lstrip("%") for r in ret.split(",")] == [o["tensor_name"] for o in desc["output_desc"]]
    # one mindspore op per op_desc entry, in order
    ops = re.findall(r'= "mindspore\.(\w+)"', text)
    ops = [o for o in ops if o != "const"]
    assert len(ops) == len(desc["op_desc"])


def test_scalar_constant_inputs_become_constants():
    path = os.path.join(REF_INFO, "Fused_Mul_RealDiv_Exp_fusion_2550894545544229730.info")
    text = driver.translate(open(path, "r", encoding="utf-8").read())
    assert '"mindspore.const"() {value = -0.00599632' in text     # "value" on a shape-[1] operand, attr: null
    assert text.count('"mindspore.mul"') == 1 and text.count('"mindspore.exp"') == 1


def test_dynamic_shapes_are_a_translate_error():
    path = os.path.join(REF_INFO, "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957.dynamic.info")
    with pytest.raises(driver.AkgHipError) as e:
        driver.translate(open(path, "r", encoding="utf-8").read())
    assert e.value.code == -3 and "dynamic" in str(e.value)


def _desc(mutate):
    d = json.loads(op_desc.elementwise_tanh_add_mul(4, 8, "t"))
    mutate(d)
    return json.dumps(d)


def test_error_conventions():
    # malformed JSON -> -2
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel('{"op": ', out_dir=None)
    assert e.value.code == -2
    # missing required key -> json error naming the key (the reference's .at() throws as well)
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(_desc(lambda d: d.pop("process")), out_dir=None)
    assert "process" in str(e.value)
    # an empty tensor -> translate error, for every family (no schedule divides by an extent of 0)
    for make in (lambda: op_desc.elementwise_tanh_add_mul(7, 128, "z_ew"), lambda: op_desc.softmax_last_axis(7, 128, "float16", "z_sm"),
                 lambda: op_desc.square_reduce([7, 128], [0], "float32", False, "ReduceSum", "z_red"),
                 lambda: op_desc.transpose_bias_add(2, 7, 128, "bfloat16", "z_tr"),
                 lambda: op_desc.gemm_bias_act(7, 128, 64, "bfloat16", "gelu", False, "float32", "z_gemm"),
                 lambda: op_desc.gemm_bias_act(8, 7, 64, "bfloat16", "gelu", False, "float32", "z_gemm_k")):
        desc = json.loads(make())

        def empty(node):
            if isinstance(node, dict):
                if isinstance(node.get("shape"), list):
                    node["shape"] = [0 if d == 7 else d for d in node["shape"]]
                for v in node.values():
                    empty(v)
            elif isinstance(node, list):
                for v in node:
                    empty(v)
        empty(desc)
        text = json.dumps(desc)
        assert any(0 in e[0]["shape"] for e in desc["input_desc"])
        with pytest.raises(driver.AkgHipError) as e:
            driver.HipKernel(text, out_dir=None)
        assert e.value.code == -3 and "extent of 0" in str(e.value)
    # an op with fewer operands than its kind reads, and a tensor no device holds -> translate errors
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(_desc(lambda d: d["op_desc"][0].update(name="MatMul", input_desc=d["op_desc"][0]["input_desc"][:1])), out_dir=None)
    assert e.value.code == -3 and "operands" in str(e.value)
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(_desc(lambda d: d["input_desc"][0][0].update(shape=[2 ** 31, 2 ** 31])), out_dir=None)
    assert e.value.code == -3 and "2^40" in str(e.value)
    # dtype outside the type table -> translate error
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(_desc(lambda d: d["input_desc"][0][0].update(data_type="complex64")), out_dir=None)
    assert e.value.code == -3
    # op name outside the op table: translator accepts it (mindspore.unknown), lowering rejects it -> -4
    unknown = _desc(lambda d: d["op_desc"][2].update(name="Erf"))
    assert '"mindspore.unknown"' in driver.translate(unknown) and 'ori_op = "Erf"' in driver.translate(unknown)
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(unknown, out_dir=None)
    assert e.value.code == -4 and "Erf" in str(e.value)
    # attribute with an unsupported data_type is fatal
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(_desc(lambda d: d["op_desc"][0].update(attr=[{"name": "x", "data_type": "tensor", "value": 1}])),
                         out_dir=None)
    assert e.value.code == -3
    # operand that is neither defined nor a constant
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(_desc(lambda d: d["op_desc"][0]["input_desc"][0][0].update(tensor_name="nowhere")), out_dir=None)
    assert e.value.code == -3 and "nowhere" in str(e.value)
    # a reduced value that meets an unreduced one along an outer axis: the column kernel keeps the reduced run in
    # registers; what it does not take (a run too long, an Assign) needs a second pass and runs as several kernels,
    # unless it also holds an op that is not cut, and then both reasons are given
    b = op_desc.DescBuilder("Fused_ReduceMax_Sub_axis0")
    x = b.input([64, 128], "float32")
    text = b.dumps([b.sub(x, b.reduce("ReduceMax", x, [0], True))])
    assert driver.HipKernel(text, out_dir=None).family == "column_reduce"
    b = op_desc.DescBuilder("Fused_ReduceMax_Sub_axis0_long")
    x = b.input([40000, 128], "float32")
    assert driver.HipKernel(b.dumps([b.sub(x, b.reduce("ReduceMax", x, [0], True))]), out_dir=None).family == "staged"
    b = op_desc.DescBuilder("Fused_ReduceMax_Sub_Assign_axis0")
    x = b.input([64, 128], "float32")
    a = b.op("Assign", [x, b.sub(x, b.reduce("ReduceMax", x, [0], True))], [64, 128], "float32")
    # the Assign runs in the last kernel, behind the reduction's reads of x: allowed
    assert driver.HipKernel(b.dumps([a]), out_dir=None).family == "staged"
    # ... but not when a later kernel would read the input again after it was overwritten (the second reduction
    # recomputes from x), nor when the Assign's result is no output (its kernel would never run)
    b = op_desc.DescBuilder("Fused_Assign_then_reduce_again")
    x = b.input([64, 128], "float32")
    a = b.op("Assign", [x, b.sub(x, b.reduce("ReduceMax", x, [0], True))], [64, 128], "float32")
    s2 = b.reduce("ReduceSum", b.unary("Abs", a), [0], True)
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(b.dumps([a, b.sub(x, s2)]), out_dir=None)
    assert e.value.code == -4 and "second pass" in str(e.value) and "Assign" in str(e.value)
    # path with '..' is refused (checkAndReadJson)
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel.from_file(os.path.join(FIXTURES, "..", "fixtures", "small_softmax_f32_5x77.info"), out_dir=None)
    assert e.value.code == -6


def test_uint8_is_read_as_int8_and_missing_shape_is_one():
    def mut(d):
        d["input_desc"][0][0]["data_type"] = "uint8"
        d["op_desc"][0]["input_desc"][0][0]["data_type"] = "uint8"
    text = driver.translate(_desc(mut))
    assert "%input_0: tensor<4x8xint8>" in text

    def drop(d):
        d["input_desc"] = [[{"tensor_name": "input_0", "data_type": "float32"}]]
        d["op_desc"] = [{"name": "Neg", "attr": None, "input_desc": [[{"tensor_name": "input_0", "data_type": "float32"}]],
                         "output_desc": [{"tensor_name": "o", "data_type": "float32"}]}]
        d["output_desc"] = [{"tensor_name": "o", "data_type": "float32"}]
    text = driver.translate(_desc(drop))
    assert "%input_0: tensor<1xfloat32>" in text


def test_reduce_axis_from_second_input_and_negative_axis():
    b = op_desc.DescBuilder("r")
    x = b.input([4, 6], "float32")
    out = b.reduce("ReduceSum", x, [-1], True)
    d = b.build([out])
    d["op_desc"][0]["attr"] = [{"name": "keep_dims", "data_type": "bool", "value": True}]
    d["op_desc"][0]["input_desc"].append([{"tensor_name": "axis", "data_type": "int64", "shape": [1], "value": -1}])
    text = driver.translate(json.dumps(d))
    assert "axis = [1], keepdims = true" in text


# ---------------------------------------------------------------------------------------------------------
# lowering decisions and artifacts
# ---------------------------------------------------------------------------------------------------------
def test_fusion_class_and_family_per_configuration():
    want = {
        "c1_ew_tanh_add_mul_f32_1024x4096": ("Elementwise", "elementwise"),
        "c2_softmax_f16_8192x4096": ("Reduction", "row_reduce"),
        "c3_layernorm_residual_bf16_16384x4096": ("Reduction", "row_reduce"),
        "c4_quant_int8_residual_bf16_32768x8192": ("Reduction", "row_reduce"),
        "c5_gemm_i8_dequant_bias_gelu_4096x8192x8192": ("Matmul", "gemm_epilogue"),
    }
    bytes_want = {"c1_ew_tanh_add_mul_f32_1024x4096": 67108864, "c2_softmax_f16_8192x4096": 134217728,
                  "c3_layernorm_residual_bf16_16384x4096": 402669568,
                  "c4_quant_int8_residual_bf16_32768x8192": 1342308352,
                  "c5_gemm_i8_dequant_bias_gelu_4096x8192x8192": 167837696}
    for name, (cls, fam) in want.items():
        k = driver.HipKernel.from_file(os.path.join(FIXTURES, name + ".info"))
        assert (k.operator_type, k.family) == (cls, fam)
        assert k.kernel_name == name + "_kernel"
        assert k.algorithmic_bytes == bytes_want[name]
        assert [t.is_output for t in k.tensors] == sorted(t.is_output for t in k.tensors)   # inputs first
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "c5_gemm_i8_dequant_bias_gelu_4096x8192x8192.info"))
    assert k.algorithmic_ops == 2 * 4096 * 8192 * 8192


def test_streaming_reduction_family_and_schedule():
    """Reduce direction Y / ALL and over-long rows go to the streaming family; its workspace holds one arrival
    counter per output group plus SPLIT partials per reduction, and is absent when one workgroup owns a group."""
    k = driver.HipKernel.from_file(os.path.join(REF_INFO, "Fused_Mul_ReduceSum_split_13305325157517622155.info"))
    assert (k.operator_type, k.family) == ("Reduction", "stream_reduce")
    assert "direction=X" in _meta_schedule(k) and k.workspace_bytes > 0 and k.grid[0] > 1
    assert "akg_ws" in k.source and "last_workgroup" in k.source
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_reducey_sqsum_f32_1x5100x3072.info"))
    assert k.family == "stream_reduce" and "direction=Y" in _meta_schedule(k)
    assert "outer=1 reduced=5100 inner=3072" in _meta_schedule(k)
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_reducey_sqsum_f32_3x37x50.info"))
    assert k.workspace_bytes == 0 and "akg_ws" not in k.source      # too little work to split
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "n1_biasgrad_bf16_16384x4096.info"))
    assert k.family == "stream_reduce" and k.algorithmic_bytes == 2 * 16384 * 4096 * 2 + 2 * 4096 * 4
    assert len(k.outputs) == 2
    # the same reduction along the innermost axis with rows that fit in registers stays in the row family
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_softmax_f32_5x77.info"))
    assert k.family == "row_reduce" and k.workspace_bytes == 0
    # The streaming loop issues a trip's loads together, conditions as operands, before the work on any of them; the
    # depth of a trip is picked so that the last one is full (49 chunks per thread: 7 trips of 7, not 13 of 4).
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "n5_bnstats_bf16_256x64x56x56.info"))
    assert "constexpr int U = 7;" in k.source and "t_in0[U][V]" in k.source
    loads, work = k.source.index("load_chunk_if<akg::bf16, V, true>(b_in0, akg_in"), k.source.index("if (akg_in) acc0 =")
    assert loads < work and k.source.count("for (int u = 0; u < U; ++u)") == 2


def test_assign_after_a_streaming_reduction_stores_over_its_input():
    """Running statistics of a batch norm: the Assigns take values that exist only after the reduction, so their stores
    sit in the kernel's last phase, over parameters that are not const; the activations stay read-only. An Assign
    over the streamed tensor itself with a value built from the reduced result needs a second pass: that description runs
    as two kernels, the Assign in the second."""
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_bnstats_update_f32_32x16x28x28.info"))
    assert k.family == "stream_reduce" and len(k.outputs) == 4
    params = re.search(r"void\s+\w+_kernel\((.*?)\)\s*\{", k.source, flags=re.S).group(1)
    assert "const akg::f32::storage *__restrict__ in0" in params
    assert ", akg::f32::storage *__restrict__ in1" in params
    assert ", akg::f32::storage *__restrict__ in2" in params
    post = k.source[k.source.rindex("last_workgroup"):] if "last_workgroup" in k.source else k.source
    assert "akg::store_one<akg::f32>(b_in1," in post and "akg::store_one<akg::f32>(b_in2," in post
    b = op_desc.DescBuilder("assign_over_streamed")
    x = b.input([64, 4096], "float32")
    s = b.reduce("ReduceSum", x, [0], True)
    a = b.op("Assign", [x, b.add(x, s)], [64, 4096], "float32")
    two = driver.HipKernel(b.dumps([a]), out_dir=None)
    assert two.family == "staged" and two.source.count('extern "C" __global__') == 2


def test_unsorted_segment_sum_translates_and_gets_its_own_family():
    path = os.path.join(REF_INFO, "Fused_UnsortedSegmentSum_split_11686736348673473318.info_failed")
    k = driver.HipKernel.from_file(path)
    assert k.family == "segment_sum" and k.workspace_bytes == 0
    assert [t.shape for t in k.outputs] == [[4954, 1, 3]]
    assert "mindspore.unsorted_segment_sum" in driver.translate(open(path, encoding="utf-8").read())
    # the kernel scans ids 64 at a time and keeps the accumulators of its segments in LDS
    assert "__ballot" in k.source and "__shared__" in k.source and "atomic" not in k.source
    d = json.loads(op_desc.unsorted_segment_sum([12], [5], 4, "float32"))
    d["op_desc"][0]["attr"] = None              # no segment count anywhere: the reference's own message
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(json.dumps(d), out_dir=None)
    assert e.value.code == -3 and "numSegments" in str(e.value)
    d = json.loads(op_desc.unsorted_segment_sum([12], [5], 4, "float32"))
    d["op_desc"][0]["attr"][0]["name"] = "numSegments"      # the spelling the reference's translator reads
    assert driver.HipKernel(json.dumps(d), out_dir=None).family == "segment_sum"
    d["op_desc"][0]["input_desc"][1][0]["shape"] = [6]      # ids must cover the leading dimensions of the data
    d["input_desc"][1][0]["shape"] = [6]
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(json.dumps(d), out_dir=None)
    assert e.value.code == -3 and "leading dimensions" in str(e.value)
    # fused with neighbours: the segment sum keeps a kernel of its own, the neighbours get theirs
    b = op_desc.DescBuilder("Fused_UnsortedSegmentSum_Neg")
    data, ids = b.input([12, 5], "float32"), b.input([12], "int32")
    seg = b.op("UnsortedSegmentSum", [data, ids], [4, 5], "float32", attrs=[{"data_type": "int", "name": "num_segments", "value": 4}])
    k = driver.HipKernel(b.dumps([b.unary("Neg", seg)]), out_dir=None)
    assert k.family == "staged" and "_stage0_kernel" in k.source and "_stage1_kernel" in k.source


def test_segment_sum_over_many_positions_is_grouped_by_segment_first(tmp_path, monkeypatch):
    """From 65536 positions on: four launches that sort the positions by segment (integer counters only) precede the
    kernel proper; they are listed in the artifact's JSON in launch order, and the handle owns the workspace they
    share. Short rows are moved into segment order, wide ones stay where they are."""
    monkeypatch.setenv("AKG_HIP_VARIANT", "2")
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_segment_sum_f32_300000_by_3_seg5000.info"), out_dir=str(tmp_path))
    meta = json.load(open(os.path.join(str(tmp_path), k.kernel_name[:-len("_kernel")] + ".json")))
    assert k.family == "segment_sum" and "grouped by segment" in meta["schedule"]
    runs = 300000 // 1024
    run_length = -(-(-(-300000 // runs)) // 64) * 64
    runs = -(-300000 // run_length)
    words = runs * 5000 + 5000 + 5000 + 1
    words = -(-words // 4) * 4 + 300000 * 3
    assert k.workspace_bytes == 4 * words
    names = [p["kernelName"] for p in meta["earlier_phases"]]
    stem = k.kernel_name[:-len("_kernel")]
    assert names == [stem + "_count", stem + "_offsets", stem + "_starts", stem + "_place"]
    assert [p["blockIdx.x"] for p in meta["earlier_phases"]] == [runs, -(-(-(-5000 // 16)) // 8) * 8, 1, runs]
    assert meta["kernelName"] == k.kernel_name and meta["workspace_bytes"] == k.workspace_bytes
    for n in names + [k.kernel_name]:
        assert 'void %s(' % n in k.source
    assert "placed[static_cast<long>(at + rank) * UNITS + c] = row[u][c]" in k.source
    # no float atomics anywhere: the only atomic is the integer count in LDS
    assert k.source.count("atomicAdd(&akg_cnt[key_of(id)], 1u)") == 1 and k.source.count("atomic") == 1
    monkeypatch.delenv("AKG_HIP_VARIANT")
    wide = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_segment_sum_f32_140000_by_40_seg129.info"), out_dir=None)
    assert "akg_ws[W_SORTED + at + rank] = " in wide.source and "placed" not in wide.source
    small = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_segment_sum_f32_700x3_by_1x3_seg50.info"), out_dir=None)
    assert small.workspace_bytes == 0 and "grouped" not in small.source


def test_short_rows_into_many_segments_are_grouped_by_bucket_first(tmp_path):
    """Rows of 4, 8 or 12 bytes into enough segments for 96 buckets: the positions are sorted by bucket of eight
    segments, chunk by chunk in LDS, into 16-byte entries {row, segment}; the last launch has one workgroup per bucket
    and sorts by segment in LDS. Same launch names, integer counters only."""
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_segment_sum_f32_300000_by_3_seg5000.info"), out_dir=str(tmp_path))
    meta = json.load(open(os.path.join(str(tmp_path), k.kernel_name[:-len("_kernel")] + ".json")))
    assert k.family == "segment_sum" and "grouped by bucket of 8 segments: 625 buckets" in meta["schedule"]
    chunks = -(-300000 // 4096)
    words = chunks * 625 + 625 + 625 + 1
    words = -(-words // 4) * 4 + 300000 * 4
    assert k.workspace_bytes == 4 * words
    stem = k.kernel_name[:-len("_kernel")]
    assert [p["kernelName"] for p in meta["earlier_phases"]] == [stem + "_count", stem + "_offsets", stem + "_starts", stem + "_place"]
    assert [p["blockIdx.x"] for p in meta["earlier_phases"]] == [chunks, -(-(-(-625 // 4)) // 8) * 8, 1, -(-chunks // 8) * 8]
    assert meta["blockIdx.x"] == 625 and meta["threadIdx.x"] == 512
    assert k.source.count("chunk_sort<NW, KEYS, KEY_BITS, TILES, 1>") == 1 and k.source.count("chunk_sort<NW, S, BUCKET_BITS, TILES, 4>") == 1
    assert k.source.count("atomic") == 1
    # few segments, 16-byte rows, 8-byte arithmetic: grouped by segment as before
    for name in ("small_segment_sum_f16_150001_by_4_seg300.info",):
        other = driver.HipKernel.from_file(os.path.join(FIXTURES, name), out_dir=None)
        assert "grouped by segment" in other.source


def test_argmax_becomes_a_max_and_a_least_position_in_the_row_family():
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_argmax_f32_37x1000.info"))
    assert k.family == "row_reduce" and [t.dtype for t in k.outputs] == ["int32"]
    assert "mindspore.argmax" in driver.translate(open(os.path.join(FIXTURES, "small_argmax_f32_37x1000.info")).read())
    assert k.source.count("group_reduce<akg::RedMax") == 1 and k.source.count("group_reduce<akg::RedMin") == 1
    assert "static_cast<int>(akg_cols[j] + e)" in k.source
    # a row too long for registers: the position pass is one more walk over the (packed) row
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_argmax_bf16_scaled_4x70000.info"))
    assert k.source.count("for (int akg_g = 0; akg_g < GROUPS") == 3 and "RawChunk" in k.source
    # an outer axis: respelled as Transpose + ArgMax over the last axis, two kernels
    b = op_desc.DescBuilder("Fused_ArgMax_axis0")
    k = driver.HipKernel(b.dumps([op_desc.argmax(b, b.input([8, 16], "float32"), 0)]), out_dir=None)
    assert k.family == "staged" and k.source.count('extern "C" __global__') == 2 and [t.shape for t in k.outputs] == [[16]]
    b = op_desc.DescBuilder("Fused_ArgMax_axis1_keep")
    k = driver.HipKernel(b.dumps([op_desc.argmax(b, b.input([4, 8, 16], "float32"), 1, True)]), out_dir=None)
    assert k.family == "staged" and [t.shape for t in k.outputs] == [[4, 1, 16]]
    b = op_desc.DescBuilder("Fused_ArgMax_float_result")
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(b.dumps([op_desc.argmax(b, b.input([8, 16], "float32"), 1, dtype="float32")]), out_dir=None)
    assert "integer" in str(e.value)


def test_data_movement_ops_translate_and_go_to_the_indexed_family():
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_view_chain_f32.info"))
    assert (k.operator_type, k.family) == ("Transpose", "indexed")
    text = driver.translate(open(os.path.join(FIXTURES, "small_view_chain_f32.info"), encoding="utf-8").read())
    for needle in ("mindspore.pad", "mindspore.tile", "mindspore.strided_slice", "mindspore.transpose", "mindspore.slice",
                   "mindspore.concat", "perm = [1, 0]", "low = [3, 1], value = 2"):
        assert needle in text, needle
    # a Tile alone is a Broadcast-class kernel, a Slice alone is unclassified (Default), as in the reference
    b = op_desc.DescBuilder("Fused_Tile_only")
    assert driver.HipKernel(b.dumps([op_desc.tile(b, b.input([3, 4], "float32"), [2, 2])]), out_dir=None).operator_type == "Broadcast"
    b = op_desc.DescBuilder("Fused_Slice_only")
    assert driver.HipKernel(b.dumps([op_desc.slice_(b, b.input([8, 8], "float32"), [1, 2], [3, -1])]), out_dir=None).operator_type == "Default"

    def broken(mutate):
        b = op_desc.DescBuilder("Fused_broken")
        x = b.input([4, 6], "float32")
        d = b.build([op_desc.transpose(b, x, [1, 0])])
        mutate(d)
        return json.dumps(d)
    with pytest.raises(driver.AkgHipError) as e:   # not a permutation
        driver.HipKernel(broken(lambda d: d["op_desc"][0]["attr"][0].update(value=[1, 1])), out_dir=None)
    assert e.value.code == -3 and "permutation" in str(e.value)
    with pytest.raises(driver.AkgHipError) as e:   # declared shape does not follow from the attributes
        driver.HipKernel(broken(lambda d: d["op_desc"][0]["output_desc"][0].update(shape=[4, 6])), out_dir=None)
    assert e.value.code == -3 and "declared result shape" in str(e.value)
    # the mask attributes of a strided slice are ignored, as the reference's lowering ignores them
    # (MindSporeFinalizingLower.cpp:117-124 reads begin / end / strides only): same kernel source with and without
    b = op_desc.DescBuilder("Fused_masked_slice")
    x = b.input([8, 8], "float32")
    d = b.build([op_desc.strided_slice(b, x, [1, 0], [4, 8], [1, 2])])
    plain = driver.HipKernel(json.dumps(d), out_dir=None).source
    for mask in ("beginMask", "endMask", "shrinkAxisMask"):
        d["op_desc"][0]["attr"].append({"data_type": "int", "name": mask, "value": 1})
    assert driver.HipKernel(json.dumps(d), out_dir=None).source == plain
    from oracle import np_ref
    grid = np.arange(64, dtype=np.float32).reshape(8, 8)
    assert np.array_equal(np_ref.evaluate(d, [grid])[0], grid[1:4, 0:8:2])
    # ... but a declared result that drops the unit dimension a shrink mask stands for is not what begin / end / strides
    # give, and is refused
    d["op_desc"][0]["attr"][1]["value"] = [2, 8]     # end: rows 1..2, one row
    d["op_desc"][0]["output_desc"][0]["shape"] = [4]
    d["output_desc"][0]["shape"] = [4]
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(json.dumps(d), out_dir=None)
    assert e.value.code == -3 and "declared result shape" in str(e.value)
    # a reduction or a MatMul next to a transpose has no single kernel: the transpose gets a kernel of its own and the
    # other reads its result from the handle's workspace
    b = op_desc.DescBuilder("Fused_Transpose_ReduceSum")
    x = b.input([4, 6], "float32")
    k = driver.HipKernel(b.dumps([b.reduce("ReduceSum", op_desc.transpose(b, x, [1, 0]), [1], False)]), out_dir=None)
    assert k.family == "staged" and k.workspace_bytes == 256 and k.source.count('extern "C" __global__') == 2
    b = op_desc.DescBuilder("Fused_Transpose_MatMul")
    x, w = b.input([64, 32], "bfloat16"), b.input([64, 128], "bfloat16")
    k = driver.HipKernel(b.dumps([b.matmul(op_desc.transpose(b, x, [1, 0]), w, "float32")]), out_dir=None)
    assert k.family == "staged" and "gemm_skinny" in k.source and "stage0_kernel" in k.source


def test_shape_sets_that_differ_in_the_leading_dimensions_share_one_code_object(tmp_path):
    """The elementwise / row kernels of a dynamic description take their row count as a kernel argument, so their
    source does not depend on it: a second shape set with the same row length is served by the code object of the first
    (no device compilation), with its own grid."""
    text = open(os.path.join(REF_INFO, "Fused_ReduceMax_fusion_2054638663855723468.info_failed"), encoding="utf-8").read()
    dyn = driver.HipDynamicKernel(text, out_dir=str(tmp_path))
    a = dyn.specialize([[100, 768]])
    b = dyn.specialize([[3, 768]])
    c = dyn.specialize([[5000, 768]])
    assert a.source == b.source == c.source
    assert "const long akg_extent" in a.source and "const long ROWS = akg_extent;" in a.source
    assert (a.cache_hit, b.cache_hit, c.cache_hit) == (False, True, True)
    assert len({a.grid, b.grid, c.grid}) == 3 and a.family == "row_reduce"
    # the static entry point keeps constants
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_softmax_f16_33x1000.info"), out_dir=None)
    assert "akg_extent" not in k.source and "constexpr long ROWS = 33L;" in k.source
    # everything folds into one dimension: the element count is the argument
    text = open(os.path.join(REF_INFO, "Fused_Sub_Mul_split_1454621004286351279.info_failed"), encoding="utf-8").read()
    dyn = driver.HipDynamicKernel(text, out_dir=None)
    a, b = dyn.specialize([[32, 1, 48, 48]]), dyn.specialize([[32, 1, 7, 100]])
    assert a.source == b.source and "const long COLS = akg_extent;" in a.source and b.cache_hit


def test_dynamic_description_is_specialised_per_shape(tmp_path):
    text = open(os.path.join(REF_INFO, "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957.dynamic.info"),
                encoding="utf-8").read()
    dyn = driver.HipDynamicKernel(text, out_dir=str(tmp_path))
    a = dyn.specialize([[32, 1, 48, 48], [32, 12, 48, 48]])
    b = dyn.specialize([[1, 1, 40, 72], [32, 12, 40, 72]])       # the mask may also broadcast along the batch
    assert a.family == b.family == "row_reduce"
    assert [t.shape for t in a.tensors] == [[32, 1, 48, 48], [32, 12, 48, 48], [32, 12, 48, 48]]
    assert [t.shape for t in b.tensors] == [[1, 1, 40, 72], [32, 12, 40, 72], [32, 12, 40, 72]]
    assert a.kernel_name == b.kernel_name == "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957_kernel"
    assert a.source != b.source                                                     # 48 and 72 columns: two kernels
    assert dyn.specialize([[32, 1, 48, 48], [32, 12, 48, 48]]) is a                 # cached per shape set
    made = sorted(f for f in os.listdir(str(tmp_path)) if f.endswith(".hsaco"))     # one artifact set per shape set
    assert len(made) == 2 and all(re.match(r"Fused_Sub_Mul_Mul_Add_Softmax_fusion_\d+_s[0-9a-f]{12}\.hsaco$", f) for f in made)
    with pytest.raises(driver.AkgHipError) as e:    # a static extent of the description cannot be rebound
        dyn.specialize([[32, 1, 48, 48], [31, 12, 48, 48]])
    assert e.value.code == -3 and "contradicts" in str(e.value)
    with pytest.raises(driver.AkgHipError) as e:    # operands that do not broadcast under the binding
        dyn.specialize([[32, 1, 48, 48], [32, 12, 48, 47]])
    assert e.value.code == -3
    with pytest.raises(driver.AkgHipError) as e:    # wrong number of shapes
        dyn.specialize([[32, 1, 48, 48]])
    assert e.value.code == -1
    # a dynamic Reshape may leave one extent open; reductions and MatMul derive their result shapes
    b2 = op_desc.DescBuilder("Fused_dyn_matmul")
    x = b2.input([-1, 64], "bfloat16")
    w = b2.input([64, 32], "bfloat16")
    d = b2.build([b2.cast(b2.matmul(x, w, "float32"), "bfloat16")])
    k = driver.HipDynamicKernel(json.dumps(d), out_dir=None).specialize([[128, 64], [64, 32]])
    assert k.family == "gemm_epilogue" and k.outputs[0].shape == [128, 32]


def _meta_schedule(kernel):
    with open(os.path.join(driver.DEFAULT_META_DIR, kernel.kernel_name[:-len("_kernel")] + ".json"), encoding="utf-8") as f:
        return json.load(f)["schedule"]


def test_artifacts_have_the_reference_layout(tmp_path):
    # under a name of its own: code objects are also remembered per process, by the digest of their source
    name = "artifact_layout_quant_int8_residual_bf16_37x1544"
    info = str(tmp_path / (name + ".info"))
    with open(info, "w", encoding="utf-8") as f:
        f.write(op_desc.quant_int8_residual(37, 1544, "bfloat16", name))
    out = str(tmp_path / "meta")
    k = driver.HipKernel.from_file(info, out_dir=out)
    assert not k.cache_hit
    for ext in (".hsaco", ".json", "_shape_arg.txt", "_shape_info.json", ".hip"):
        assert os.path.exists(os.path.join(out, name + ext))
    shape_info = json.load(open(os.path.join(out, name + "_shape_info.json")))
    assert shape_info["hostShapes"] == shape_info["deviceShapes"] == [[37, 1544], [37, 1544], [37, 1544], [37]]
    assert shape_info["runtimeVars"] == [] and "SupportInfo" in shape_info
    meta = json.load(open(os.path.join(out, name + ".json")))
    for key in ("blockIdx.x", "blockIdx.y", "blockIdx.z", "threadIdx.x", "threadIdx.y", "threadIdx.z"):
        assert isinstance(meta[key], int)
    assert meta["kernelName"] == name + "_kernel" and meta["is_dynamic"] is False
    assert (meta["blockIdx.x"], meta["threadIdx.x"]) == (k.grid[0], k.block[0])
    code = open(os.path.join(out, name + ".hsaco"), "rb").read()
    assert code[:4] == b"\x7fELF"
    assert meta["sha256"] == hashlib.sha256(code).hexdigest()          # hashlib as the independent digest
    # [offset, sizes..., strides...] per kernel argument, inputs then outputs
    shape_arg = json.load(open(os.path.join(out, name + "_shape_arg.txt")))
    assert shape_arg == [[0, 37, 1544, 1544, 1], [0, 37, 1544, 1544, 1], [0, 37, 1544, 1544, 1], [0, 37, 1]]
    # second compile reuses the artifact; a corrupted code object is detected and replaced
    assert driver.HipKernel.from_file(info, out_dir=out).cache_hit
    with open(os.path.join(out, name + ".hsaco"), "ab") as f:
        f.write(b"x")
    os.environ["AKG_HIP_NO_CACHE"] = "1"      # no artifact probe and no per-process memory: a device compilation
    try:
        assert not driver.HipKernel.from_file(info, out_dir=out).cache_hit
    finally:
        del os.environ["AKG_HIP_NO_CACHE"]
    assert open(os.path.join(out, name + ".hsaco"), "rb").read() == code
    with open(os.path.join(out, name + ".hsaco"), "ab") as f:
        f.write(b"x")
    assert driver.HipKernel.from_file(info, out_dir=out).cache_hit      # served from memory, the file repaired
    assert open(os.path.join(out, name + ".hsaco"), "rb").read() == code


def test_math_selection_follows_the_precision_demand():
    # float16 output: exp and the division by the row sum may use hardware approximations
    src = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_softmax_f16_33x1000.info")).source
    assert "akg::fast_exp(" in src and "akg::fast_rcp(" in src and "akg::op_exp(" not in src
    # float32 output: library-grade exp and exact division (hoisted reciprocal + FMA correction)
    src = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_softmax_f32_5x77.info")).source
    assert "akg::op_exp(" in src and "akg::div_uniform(" in src and "fast_" not in src
    # int8 output: the path into the integer cast is exact
    src = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_quant_int8_residual_bf16_37x1544.info")).source
    assert "akg::div_uniform(" in src and "fast_" not in src
    # float32 elementwise chain: device-library tanh
    src = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_ew_tanh_add_mul_f32_8x128.info")).source
    assert "akg::op_tanh(" in src and "fast_" not in src
    # a constant factor of 1024 and more between an approximation and the 16-bit cast would carry its absolute error
    # (1.2e-7 for the hardware tanh form) towards the tolerance: the operands behind such a factor are exact
    for factor, fast in ((4.0, True), (4096.0, False)):
        b = op_desc.DescBuilder("scaled_tanh_f16_%d" % int(factor))
        x = b.input([64, 128], "float32")
        src = driver.HipKernel(b.dumps([b.cast(b.mul(b.unary("Tanh", x), b.const(factor, "float32")), "float16")]), out_dir=None).source
        assert ("akg::fast_tanh(" in src) == fast and ("akg::op_tanh(" in src) != fast
    # AKG_HIP_PRECISE=1 switches every relaxation off
    os.environ["AKG_HIP_PRECISE"] = "1"
    try:
        src = driver.HipKernel(open(os.path.join(FIXTURES, "small_softmax_f16_33x1000.info")).read(), out_dir=None).source
        assert "fast_" not in src
    finally:
        del os.environ["AKG_HIP_PRECISE"]


def test_streamed_tensors_use_non_temporal_accesses_broadcast_vectors_do_not():
    src = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_layernorm_residual_bf16_64x4096.info")).source
    loads = re.findall(r"load_chunk<akg::bf16, V, (true|false)>\(b_in(\d)", src)
    assert dict((i, nt) for nt, i in loads) == {"0": "true", "1": "false", "2": "false", "3": "true"}
    assert "store_chunk<akg::bf16, V, true>" in src
    # rows of 1040 bytes share cache lines with their neighbours: no hint
    src = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_layernorm_residual_bf16_19x520.info")).source
    assert "V, true>" not in src


def test_ragged_shapes_get_guards_and_aligned_shapes_do_not():
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_softmax_f32_5x77.info"))
    assert "akg_row_ok" in k.source
    src = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_softmax_f16_33x1000.info")).source
    assert "akg_ok[j] = akg_cols[j] < COLS;" in src          # 125 chunks on 128 threads
    # 77 is not a multiple of the 4-element chunk: chunks stay 4 wide, the last one starts at COLS - V and the three
    # elements it shares with its neighbour are left out of the reductions
    assert "constexpr int V = 4;" in k.source and "if (akg_tail[j]) akg_cols[j] = COLS - V;" in k.source
    assert "(!akg_tail[j] || e >= 3)" in k.source
    src = driver.HipKernel.from_file(os.path.join(FIXTURES, "c2_softmax_f16_8192x4096.info")).source
    assert "akg_ok[j] = true;" in src and "akg_row_ok" not in src and "akg_tail" not in src


def test_row_schedules_for_odd_and_long_rows():
    def consts(name):
        src = driver.HipKernel.from_file(os.path.join(FIXTURES, name + ".info")).source
        return {m[0]: int(m[1]) for m in re.findall(r"constexpr int (\w+) = (\d+);", src)}, src
    c, _ = consts("small_softmax_f16_9x768")                  # 96 chunks: 32 threads x 3, no idle slot
    assert (c["TPR"], c["NCHUNK"], c["V"]) == (32, 3, 8)
    c, _ = consts("small_layernorm_residual_bf16_5x5120")     # 640 chunks: 128 x 5
    assert (c["TPR"], c["NCHUNK"]) == (128, 5)
    # a LayerNorm (a reduction waiting for another, gamma and beta behind them) takes at most 256 threads a row, four
    # to eight chunks each: 1376 chunks as 256 x 6 (10 % idle, like 512 x 3; 1024 x 2 idles 33 %)
    c, _ = consts("small_layernorm_residual_bf16_3x11008")
    assert (c["TPR"], c["NCHUNK"]) == (256, 6)
    c, _ = consts("c3_layernorm_residual_bf16_16384x4096")
    assert (c["TPR"], c["NCHUNK"]) == (128, 4)
    c, _ = consts("n10_rmsnorm_bf16_16384x4096")              # one reduction: the general rule
    assert (c["TPR"], c["NCHUNK"]) == (512, 1)
    c, _ = consts("c2_softmax_f16_8192x4096")
    assert (c["TPR"], c["NCHUNK"]) == (512, 1)
    # rows beyond 64 values per thread are walked in groups: one walk per reduction and one for the outputs. A row of
    # 16-bit inputs that fits 64 registers per thread in its memory image is loaded once and kept packed ...
    c, src = consts("small_softmax_f16_3x70000")
    assert (c["TPR"], c["NCHUNK"], c["GROUPS"]) == (1024, 2, 5) and src.count("for (int akg_g = 0; akg_g < GROUPS") == 4
    # (the last group of the row is ragged: the chunks' conditions are operands of the accesses, not branches around them)
    assert src.count("load_raw_chunk_if<akg::f16, V, true>(b_in0, akg_ok[j], ") == 1 and src.count("unpack_chunk<akg::f16, V>(r_in0") == 3
    assert "load_chunk<akg::f16" not in src and src.count("forget_unpacked") == 2
    c, src = consts("small_layernorm_residual_bf16_2x57000")
    assert c["GROUPS"] == 4 and "r_in0[GROUPS * NCHUNK]" in src and "r_in3[GROUPS * NCHUNK]" in src and "r_in1" not in src
    # ... a longer one is re-read by every walk, with the non-temporal hint only in the last walk that reads it
    c, src = consts("small_layernorm_residual_bf16_2x66000")
    assert c["GROUPS"] == 3 and src.count("for (int akg_g = 0; akg_g < GROUPS") == 3 and "RawChunk" not in src
    assert re.findall(r"load_chunk_if<akg::bf16, V, (true|false)>\(b_in0", src) == ["false", "false", "true"]


def test_elementwise_dimension_folding():
    # all operands full-size: folded to one flat dimension; a broadcast operand keeps a [rows, cols] view
    k = driver.HipKernel.from_file(os.path.join(REF_INFO, "fused_sub_add.info"), out_dir=None)
    assert "constexpr long ROWS = 1L;" in k.source
    k = driver.HipKernel.from_file(os.path.join(REF_INFO, "Fused_Cast_Mul_fusion_11325474031898152154.info"), out_dir=None)
    assert k.operator_type == "Broadcast" and k.family == "elementwise"


def test_hip_driver_mirrors_the_reference_driver_interface(tmp_path):
    info = os.path.join(FIXTURES, "small_softmax_f32_5x77.info")
    d = driver.HipDriver(input_file=info, output_dir=str(tmp_path))
    assert d.kernel_name == "small_softmax_f32_5x77"
    k = d.compile()
    assert os.path.exists(os.path.join(str(tmp_path), "small_softmax_f32_5x77.json"))
    assert [t.dtype for t in k.tensors] == ["float32", "float32"]
    with pytest.raises(ValueError):
        driver.HipDriver(input_file=info, backend="cuda")


def test_description_no_single_kernel_serves_is_cut_at_its_reduction_results(tmp_path):
    """Training batch norm in one description: mean (level 1), variance (level 2, it needs x - mean) and the normalised
    tensor (level 2). The handle runs a kernel per reduction level plus one per output shape; every stage is a
    description of its own made of the original op entries, compiled through the ordinary pipeline into artifacts of
    its own; reduction results that are no outputs live in the handle's workspace."""
    path = os.path.join(FIXTURES, "small_staged_bn_train_forward_f32_16x8x14x14.info")
    k = driver.HipKernel.from_file(path, out_dir=str(tmp_path))
    name = "small_staged_bn_train_forward_f32_16x8x14x14"
    meta = json.load(open(os.path.join(str(tmp_path), name + ".json")))
    assert k.family == "staged" and meta["family"] == "staged"
    stages = meta["stages"]
    assert [s["kernelName"] for s in stages] == ["%s_stage%d_kernel" % (name, i) for i in range(5)]
    assert meta["kernelName"] == stages[-1]["kernelName"] == k.kernel_name
    # two temporaries (the raw sums, [1,8,1,1] float32 each, 256-byte slots); stage 0 reads x and writes the first sum
    assert k.workspace_bytes == 512
    assert stages[0]["args"] == [{"input": 0}, {"workspace_offset": 0}]
    assert stages[1]["args"] == [{"input": 0}, {"workspace_offset": 0}, {"workspace_offset": 256}]
    written = sorted(a["output"] for s in stages for a in s["args"][-1:] if "output" in a)
    assert written == [0, 1, 2]
    for i in range(5):
        stage_meta = json.load(open(os.path.join(str(tmp_path), "%s_stage%d.json" % (name, i))))
        assert stage_meta["family"] in ("stream_reduce", "elementwise")
        assert os.path.exists(os.path.join(str(tmp_path), "%s_stage%d.hsaco" % (name, i)))
    assert not os.path.exists(os.path.join(str(tmp_path), name + ".hsaco"))      # the handle itself has no code object
    assert k.source.count('extern "C" __global__') == 5
    # the last axis needs no cut: one row kernel
    one = driver.HipKernel(op_desc.softmax_over_axis([32, 12, 24, 40], 3, "float32", "sm_last"), out_dir=None)
    assert one.family == "row_reduce"


def test_descriptions_that_cannot_be_cut_say_both_reasons(monkeypatch):
    """Staging refuses what it cannot order or name: an output listed twice (two kernels would write one buffer) keeps the
    single-kernel refusal and adds its own reason; nothing crashes. (The column kernel serves this description - it
    stores the value to both buffers - so it is switched off here.)"""
    b = op_desc.DescBuilder("twice_listed_outer_softmax")
    x = b.input([64, 128], "float32")
    y = b.sub(x, b.reduce("ReduceMax", x, [0], True))
    k = driver.HipKernel(b.dumps([y, y]), out_dir=None)
    assert k.family == "column_reduce" and "out0 + " in k.source and "out1 + " in k.source
    monkeypatch.setenv("AKG_HIP_VARIANT", "7")
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(b.dumps([y, y]), out_dir=None)
    assert e.value.code == -4 and "second pass" in str(e.value) and "listed twice" in str(e.value)
    monkeypatch.delenv("AKG_HIP_VARIANT")
    # an op outside the op table is refused before any cut is tried
    d = json.loads(op_desc.softmax_over_axis([8, 16], 0, "float32", "unknown_op_outer"))
    d["op_desc"][1]["name"] = "Frobnicate"
    with pytest.raises(driver.AkgHipError) as e:
        driver.HipKernel(json.dumps(d), out_dir=None)
    assert e.value.code in (-3, -4) and "Frobnicate" in str(e.value)


def test_matmul_next_to_a_softmax_is_cut_behind_the_contraction(tmp_path, monkeypatch):
    """Attention probabilities in one description: the contraction (with nothing fused behind it) leaves the float32
    scores in the workspace, and everything behind it, scale, mask and softmax, is ONE row kernel: the cut is made
    behind contractions and data-movement ops first, and at reductions only where a piece still needs it."""
    text = op_desc.attention_probabilities(4, 128, 64, 256, "bfloat16", "attn_probs")
    k = driver.HipKernel(text, out_dir=str(tmp_path))
    meta = json.load(open(os.path.join(str(tmp_path), "attn_probs.json")))
    assert k.family == "staged" and [s["kernelName"] for s in meta["stages"]] == ["attn_probs_stage0_kernel", "attn_probs_stage1_kernel"]
    assert k.workspace_bytes == 4 * 128 * 256 * 4
    fams = [json.load(open(os.path.join(str(tmp_path), "attn_probs_stage%d.json" % i)))["family"] for i in range(2)]
    assert fams == ["gemm_epilogue", "row_reduce"]
    assert meta["stages"][1]["args"] == [{"input": 2}, {"workspace_offset": 0}, {"output": 0}]
    # a piece that needs cuts of its own: its stages are spliced in, temporaries appended
    b = op_desc.DescBuilder("transpose_then_softmax_axis0")
    x = b.input([64, 96], "float32")
    t = op_desc.transpose(b, x, [1, 0])
    e = b.unary("Exp", b.sub(t, b.reduce("ReduceMax", t, [0], True)))
    text = b.dumps([b.div(e, b.reduce("ReduceSum", e, [0], True))])
    k = driver.HipKernel(text, out_dir=str(tmp_path))
    meta = json.load(open(os.path.join(str(tmp_path), "transpose_then_softmax_axis0.json")))
    # the softmax over axis 0 of the transposed tensor is one column kernel ...
    assert [s["kernelName"] for s in meta["stages"]] == ["transpose_then_softmax_axis0_stage%d_kernel" % i for i in range(2)]
    assert json.load(open(os.path.join(str(tmp_path), "transpose_then_softmax_axis0_stage1.json")))["family"] == "column_reduce"
    assert k.workspace_bytes == 96 * 64 * 4
    # ... and three kernels without it
    monkeypatch.setenv("AKG_HIP_VARIANT", "7")
    other = os.path.join(str(tmp_path), "several")
    os.makedirs(other)
    k = driver.HipKernel(text, out_dir=other)
    meta = json.load(open(os.path.join(other, "transpose_then_softmax_axis0.json")))
    assert [s["kernelName"] for s in meta["stages"]] == ["transpose_then_softmax_axis0_stage0_kernel"] + [
        "transpose_then_softmax_axis0_stage1_stage%d_kernel" % i for i in range(3)]
    assert k.workspace_bytes == 96 * 64 * 4 + 256 + 256


def test_column_kernel_schedule():
    """One reduced axis that is not the innermost one, results used against the tensor: [O, R, I] with a workgroup per
    strip of columns; the chunks of a thread's rows stay in registers as loaded (the workgroup grows until they fit), one
    walk per reduction level, no workspace. Strips with a large footprint: one workgroup per CU walks several of them, the
    next strip's chunks on their way into a second set of registers while this one is worked on."""
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "n9_layernorm_axis1_bf16_64x768x1024.info"), out_dir=None)
    assert k.family == "column_reduce" and k.workspace_bytes == 0 and (k.grid[0], k.block[0]) == (512, 512)   # 1024 strips: two workgroups a CU, two strips each
    assert "constexpr int V = 8, LX = 8, LY = 64, CH = 12, BLOCK = 512;" in k.source and "// ---- walk 2 ----" in k.source
    assert "constexpr long TOTAL = 1024;" in k.source
    assert k.source.count("akg::column_reduce<akg::RedSum, akg::f32, false, LX, BLOCK, V>") == 2
    assert "akg::PackedChunk<akg::bf16, V> akg_a0[CH];" in k.source and "akg::PackedChunk<akg::bf16, V> akg_b_set0[CH];" in k.source
    assert k.source.count("global__") == 1 and k.source.count("akg::forget_derived(p_in0[j]);") == 2
    assert "[&] { if (akg_next < TOTAL) akg_load(akg_next, akg_b_set0); }" in k.source
    os.environ["AKG_HIP_VARIANT"] = "5"   # one strip per workgroup
    try:
        k = driver.HipKernel.from_file(os.path.join(FIXTURES, "n9_layernorm_axis1_bf16_64x768x1024.info"), out_dir=None)
    finally:
        del os.environ["AKG_HIP_VARIANT"]
    assert (k.grid[0], k.block[0]) == (64 * 16, 512) and "akg_b_set0" not in k.source and "forget_derived" not in k.source
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "n8_softmax_axis1_f16_32x21x512x512.info"), out_dir=None)
    assert (k.grid[0], k.block[0]) == (32 * 512, 256) and "LX = 64, LY = 4, CH = 6" in k.source and "akg_b_set0" not in k.source
    # rows that are not a multiple of the chunk: element-aligned accesses, the last chunk partly outside
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_staged_layernorm_axis1_bf16_8x64x49.info"), out_dir=None)
    assert "load_packed_partial<akg::bf16, V>(akg_p, akg_row_ok[j] ? akg_cols : 0" in k.source and "store_chunk_partial" in k.source
    # a 16-bit sum keeps its rounding per step and the serial order of the steps (one chain per column through LDS), a
    # maximum needs neither; a 16-bit integer sum wraps around and is the same in any order
    b = op_desc.DescBuilder("column_half")
    x = b.input([2, 40, 24], "float16")
    k = driver.HipKernel(b.dumps([b.sub(x, b.reduce("ReduceMax", x, [1], True)), b.reduce("ReduceSum", x, [1], True)]), out_dir=None)
    assert "column_chain_step<akg::RedSum, akg::f16, LX, BLOCK, V, NOWN>" in k.source and "column_chain_finish<akg::f16," in k.source
    assert "column_reduce<akg::RedMax, akg::f16, false," in k.source and "column_reduce<akg::RedSum" not in k.source
    b = op_desc.DescBuilder("column_short")
    x = b.input([2, 40, 24], "int16")
    k = driver.HipKernel(b.dumps([b.sub(x, b.reduce("ReduceSum", x, [1], True))]), out_dir=None)
    assert "column_reduce<akg::RedSum, akg::i16, true," in k.source and "column_chain" not in k.source
    # two reduced axes around a kept one (batch-norm statistics and their use) are not for this kernel
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "small_staged_bn_train_forward_f32_16x8x14x14.info"), out_dir=None)
    assert k.family == "staged"


def test_streaming_schedules_follow_what_was_measured():
    """The grid and the loads in flight of streaming reductions, and the K splits of MatMuls with few tiles: one
    workgroup per CU with eight loads in flight per thread in both directions, fewer workgroups and whole groups for
    small inputs, the loads divided by the workgroups a CU holds where the grid is larger, partials of at most 1 MiB
    per tile."""
    def red(shape, axes, dtype, name, op="ReduceSum"):
        return driver.HipKernel(op_desc.square_reduce(shape, axes, dtype, False, op, name), out_dir=None)
    k = driver.HipKernel.from_file(os.path.join(FIXTURES, "n1_biasgrad_bf16_16384x4096.info"))
    assert k.grid[0] == 256 and "constexpr int U = 4;" in k.source and "RSTEP" in k.source     # two operands x four chunks
    k = red([1, 65536, 1024], [1], "float32", "sched_tall")
    assert k.grid[0] == 256 and "constexpr int U = 8;" in k.source
    k = red([16, 4096, 1536], [1], "bfloat16", "sched_192_groups")        # 192 groups: 768 workgroups, two loads each
    assert k.grid[0] == 768 and "constexpr int U = 2;" in k.source
    k = red([4, 16384, 768], [1], "float32", "sched_48_groups")           # 48 groups: 240 workgroups, not 288
    assert k.grid[0] == 240
    k = red([1, 1024, 1024], [1], "float32", "sched_small_y")             # 4 MiB: 128 workgroups
    assert k.grid[0] == 128 and k.workspace_bytes > 0
    k = red([16, 256, 256], [1], "float32", "sched_small_whole_groups")   # 64 groups: each left whole, no partials
    assert k.grid[0] == 64 and k.workspace_bytes == 0
    k = driver.HipKernel(op_desc.batchnorm_stats(32, 64, 28, 28, "bfloat16", "sched_small_bn"), out_dir=None)
    assert k.grid[0] == 64 and k.workspace_bytes == 0
    k = red([1024, 4096], [0, 1], "float32", "sched_small_all")           # 16 MiB into one number: 128 workgroups
    assert k.grid[0] == 128
    k = red([64, 262143], [1], "float16", "sched_long_odd_rows")          # chunk slots with an overlapping last one, batched
    assert "RUN_CHUNKS" in k.source and "constexpr int U = 8;" in k.source and "load_chunk_if" in k.source
    k = driver.HipKernel(op_desc.gemm_bias_act(256, 8192, 8192, "bfloat16", "gelu", False, "float32", "sched_split_256"))
    assert "k_splits=4" in _meta_schedule(k)
    k = driver.HipKernel(op_desc.gemm_bias_act(128, 8192, 8192, "bfloat16", "gelu", False, "float32", "sched_split_128"))
    assert "k_splits=8" in _meta_schedule(k)
    k = driver.HipKernel(op_desc.gemm_bias_act(16, 8192, 1024, "bfloat16", "gelu", False, "float32", "sched_split_skinny"))
    assert "k_splits=16" in _meta_schedule(k)
    # a [N,K] weight is loaded without the non-temporal hint, a row-major one with it
    k = driver.HipKernel(op_desc.gemm_bias_act(16, 8192, 8192, "bfloat16", "gelu", True, "float32", "sched_skinny_nk"), out_dir=None)
    assert "true, Epilogue, 4, 4, 2, false>" in k.source


def test_skinny_matmul_gets_the_streaming_kernel():
    """At most 64 rows of A and K a multiple of 32 bytes: B goes straight into MFMA operands (no 256 x 256 tile), strips
    of 128 columns times K splits make about 256 workgroups, and the workspace holds a counter per strip plus M x 128
    partials per strip and split. Other shapes keep the tile kernel."""
    k = driver.HipKernel(op_desc.gemm_bias_act(16, 8192, 8192, "bfloat16", "gelu", False, "float32", "skinny_a"), out_dir=None)
    assert "akg::gemm_skinny<akg::MmaBF16, 16L, 8192L, 8192L, false, Epilogue, 4, 4, 2, true>" in k.source
    assert (k.grid[0], k.block[0]) == (64 * 4, 256) and k.workspace_bytes == 256 + 64 * 4 * 16 * 128 * 4
    k = driver.HipKernel(op_desc.gemm_int8_dequant_bias_gelu(1, 64, 128, "bfloat16", True, "skinny_b"), out_dir=None)
    assert "akg::gemm_skinny<akg::MmaI8, 1L, 128L, 64L, true, Epilogue, 1, " in k.source and k.workspace_bytes == 0
    k = driver.HipKernel(op_desc.gemm_bias_act(65, 1024, 256, "bfloat16", "gelu", False, "float32", "not_skinny_rows"), out_dir=None)
    assert "gemm_skinny" not in k.source and "gemm_256x256" in k.source
    k = driver.HipKernel(op_desc.gemm_bias_act(16, 3000, 264, "float16", "relu", True, "float32", "not_skinny_k"), out_dir=None)
    assert "gemm_skinny" not in k.source                    # 6000 bytes of K: not a multiple of 32


def test_tile_kernel_arranges_its_wavefronts_by_operand_type():
    """The 256 x 256 tile kernel: int8 with a row-major B runs 2 x 4 wavefronts of 128 x 64 (half the transposing reads of
    B), the 16-bit types and a B given as [N,K] keep 4 x 2 wavefronts of 64 x 128; AKG_HIP_VARIANT bit 5 swaps the two."""
    tall = "akg::gemm_256x256<akg::MmaI8, 512L, 768L, 1024L, false, Epilogue, 1, 2>("
    k = driver.HipKernel(op_desc.gemm_int8_dequant_bias_gelu(512, 1024, 768, "bfloat16", False, "tall_tiles"), out_dir=None)
    assert tall in k.source
    k = driver.HipKernel(op_desc.gemm_int8_dequant_bias_gelu(512, 1024, 768, "bfloat16", True, "wide_tiles_tb"), out_dir=None)
    assert "akg::gemm_256x256<akg::MmaI8, 512L, 768L, 1024L, true, Epilogue, 1>(" in k.source
    k = driver.HipKernel(op_desc.gemm_bias_act(512, 1024, 768, "bfloat16", "gelu", False, "float32", "wide_tiles_bf16"), out_dir=None)
    assert "akg::gemm_256x256<akg::MmaBF16, 512L, 768L, 1024L, false, Epilogue, 3>(" in k.source
    os.environ["AKG_HIP_VARIANT"] = "32"
    try:
        k = driver.HipKernel(op_desc.gemm_int8_dequant_bias_gelu(512, 1024, 768, "bfloat16", False, "tall_tiles"), out_dir=None)
        assert tall not in k.source
        k = driver.HipKernel(op_desc.gemm_bias_act(512, 1024, 768, "bfloat16", "gelu", False, "float32", "wide_tiles_bf16"), out_dir=None)
        assert "akg::gemm_256x256<akg::MmaBF16, 512L, 768L, 1024L, false, Epilogue, 3, 2>(" in k.source
    finally:
        del os.environ["AKG_HIP_VARIANT"]


def test_compiling_from_several_threads_gives_the_serial_results(tmp_path, monkeypatch):
    """The reference compiles one kernel per process (its schedule tools are process-wide singletons,
    GlobalVars.hpp:129-132) and forks workers over a directory (benchmark.py:304-317). This library is called from
    threads instead: eight threads compile different descriptions at once, twice each, into one artifact directory;
    every code object must equal the one a single thread produces, and errors stay with the thread that made them."""
    import threading
    monkeypatch.setenv("AKG_HIP_NO_CACHE", "1")
    names = ["small_softmax_f16_64x4096", "small_biasgrad_bf16_2048x1024", "small_segment_sum_f32_700x3_by_1x3_seg50",
             "small_reducey_sqsum_f32_3x37x50", "small_softmax_f32_5x77", "small_gemm_bf16_bias_gelu_100x2048x520",
             "small_segment_sum_f32_300000_by_3_seg5000", "small_bnstats_update_f32_32x16x28x28"]
    texts = [open(os.path.join(FIXTURES, n + ".info"), encoding="utf-8").read() for n in names]
    serial_dir, threaded_dir = str(tmp_path / "serial"), str(tmp_path / "threaded")
    os.makedirs(serial_dir), os.makedirs(threaded_dir)

    def digest(d, n):
        return json.load(open(os.path.join(d, n + ".json")))["sha256"]
    for t in texts:
        driver.HipKernel(t, out_dir=serial_dir)
    want = [digest(serial_dir, n) for n in names]
    failures = []

    def work(i):
        try:
            for _ in range(2):
                k = driver.HipKernel(texts[i], out_dir=threaded_dir)
                assert k.kernel_name == names[i] + "_kernel"
                with pytest.raises(driver.AkgHipError) as e:      # this thread's own error text
                    driver.HipKernel('{"op": "broken_%d"' % i, out_dir=None)
                assert "broken" in str(e.value) or e.value.code < 0
        except Exception as exc:                                  # noqa: BLE001 - reported by the main thread
            failures.append((names[i], repr(exc)))
    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(names))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures
    assert [digest(threaded_dir, n) for n in names] == want


def test_cli_tool():
    tool = os.path.join(ROOT, "akg_amd", "akg-hip")
    info = os.path.join(FIXTURES, "small_softmax_f32_5x77.info")
    r = subprocess.run([tool, "translate", info], capture_output=True, text=True)
    assert r.returncode == 0 and "mindspore.reduce_max" in r.stdout
    r = subprocess.run([tool, "info", info], capture_output=True, text=True)
    assert r.returncode == 0 and "row_reduce" in r.stdout
    r = subprocess.run([tool, "emit", os.path.join(REF_INFO, "Fused_Mul_ReduceSum_split_13305325157517622155.info")],
                       capture_output=True, text=True)
    assert r.returncode == 0 and "last_workgroup" in r.stdout
    # a dynamic-shape description is an error with a non-zero exit, never a crash
    r = subprocess.run([tool, "emit", os.path.join(
        REF_INFO, "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957.dynamic.info")], capture_output=True, text=True)
    assert r.returncode == 1 and "error -3" in r.stderr and "--shapes" in r.stderr
    # ... unless the shapes of a call come with it: then it is specialised to them first
    dynamic = os.path.join(REF_INFO, "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957.dynamic.info")
    r = subprocess.run([tool, "info", dynamic, "--shapes", "32,1,48,48;32,12,48,48"], capture_output=True, text=True)
    assert r.returncode == 0 and "row_reduce" in r.stdout and "[32,12,48,48]" in r.stdout, r.stderr
    r = subprocess.run([tool, "emit", dynamic, "--shapes", "32,1,40,40;32,12,40,40"], capture_output=True, text=True)
    assert r.returncode == 0 and "akg_dim_arg0" in r.stdout
    r = subprocess.run([tool, "emit", dynamic, "--shapes", "32,1,40,40"], capture_output=True, text=True)
    assert r.returncode == 1 and "2 inputs" in r.stderr


def test_code_objects_are_found_by_source_digest_across_processes(tmp_path):
    """The artifact directory also keeps every code object under the digest of its source (by_source/): a process that
    meets a shape set for the first time finds the code another process compiled for a different shape set with the
    same source, and compiles nothing. Two runs of the command line tool; AKG_HIP_NO_CACHE=1 still compiles."""
    tool = os.path.join(ROOT, "akg_amd", "akg-hip")
    dynamic = os.path.join(REF_INFO, "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957.dynamic.info")
    env = {k: v for k, v in os.environ.items() if k != "AKG_HIP_NO_CACHE"}
    out = str(tmp_path / "meta")

    def hit(shapes, extra_env=None):
        r = subprocess.run([tool, "compile", dynamic, "--shapes", shapes, "-o", out], capture_output=True, text=True,
                           env=dict(env, **(extra_env or {})))
        assert r.returncode == 0, r.stderr
        return [l for l in r.stdout.splitlines() if l.startswith("cache hit")][0].split()[-1]
    assert hit("32,1,48,48;32,12,48,48") == "0"
    # the artifacts of a specialisation say which extents its kernel takes as arguments behind the tensor pointers
    metas = [json.load(open(os.path.join(out, f))) for f in os.listdir(out) if f.endswith(".json") and "shape_info" not in f]
    assert len(metas) == 1 and metas[0]["scalar_args"] == [32 * 12 * 48, 48, 32, 12, 48]
    assert hit("32,1,9,48;32,12,9,48") == "1"           # another shape set, another process, the same source
    assert len(os.listdir(os.path.join(out, "by_source"))) == 1
    assert hit("32,1,7,48;32,12,7,48", {"AKG_HIP_NO_CACHE": "1"}) == "0"


def test_dynamic_descriptions_share_code_objects_across_shape_sets(monkeypatch):
    """What a new shape set of a dynamic description costs: a device compilation only when the source changes. The leading
    extents (also of operands that span only some of them: a mask shared by the heads), the row count, the row length
    inside its power-of-two bucket of chunk counts, the rows of A of a MatMul and its K split are kernel arguments; what
    still makes a new source is a row length in another bucket, rows that are whole 64-byte pieces against rows that are
    not, and a chunk width that stops dividing the rows. Counted
    on the shape sets the GPU tests use for the reference's ten dynamic descriptions (three each)."""
    monkeypatch.setenv("AKG_HIP_NO_CACHE", "0")
    shape_sets = {
        "Fused_Cast_Sub_Mul_split_14802837530264465372": ([[[32, 1, 48, 48]], [[32, 1, 5, 1000]], [[32, 1, 48, 40]]], 1),
        "Fused_RealDiv_split_4177286244677596212": ([[[32, 12, 24, 40], [32, 12, 24, 1]], [[32, 12, 7, 40], [32, 12, 7, 1]],
                                                    [[32, 12, 24, 136], [32, 12, 24, 1]]], 1),
        "Fused_ReduceMax_fusion_2054638663855723468": ([[[100, 768]], [[3, 768]], [[2048, 768]]], 1),
        "Fused_ReduceMax_fusion_234578345729057892345": ([[[4096, 33]], [[4096, 4096]], [[4096, 40]]], 2),       # 33 / 40 and 4096: two buckets
        "Fused_Sub_Mul_Cast_fusion_4217325526348104075": ([[[32, 16, 20, 64], [32, 16, 20, 1], [32, 16, 20, 64]],
                                                          [[32, 16, 3, 64], [32, 16, 3, 1], [32, 16, 3, 64]],
                                                          [[32, 16, 20, 72], [32, 16, 20, 1], [32, 16, 20, 72]]], 1),
        "Fused_Sub_Mul_split_1454621004286351279": ([[[32, 1, 48, 48]], [[32, 1, 6, 48]], [[32, 1, 48, 520]]], 1),
    }
    for f in sorted(os.listdir(REF_INFO)):
        stem = f.split(".info")[0]
        if stem not in shape_sets:
            continue
        sets, allowed = shape_sets[stem]
        dyn = driver.HipDynamicKernel(open(os.path.join(REF_INFO, f), encoding="utf-8").read(), out_dir=None)
        compiled = sum(0 if dyn.specialize(shapes).cache_hit else 1 for shapes in sets)
        assert compiled <= allowed, "%s: %d device compilations for three shape sets (%d allowed)" % (stem, compiled, allowed)
    # an attention mask [32,1,S,T] against scores [32,12,S,T] with S and T open: one code object
    # as long as the rows stay in one bucket (40 and 48 columns: 5 and 6 chunks of 8)
    path = os.path.join(REF_INFO, "Fused_Sub_Mul_Mul_Add_Softmax_fusion_13911402818667958957.dynamic.info")
    dyn = driver.HipDynamicKernel(open(path, encoding="utf-8").read(), out_dir=None)
    first = dyn.specialize([[32, 1, 48, 48], [32, 12, 48, 48]])
    assert "akg_dim_arg0" in first.source and "akg_dim_arg2" in first.source
    # rows that are whole 64-byte pieces (48 and 64 float32) have a source of their own inside the bucket: no chunk
    # overlaps its neighbour there and whole lines are streamed
    assert "akg_overlap" not in first.source
    for shapes in ([[32, 1, 64, 64], [32, 12, 64, 64]], [[32, 1, 9, 48], [32, 12, 9, 48]]):
        k = dyn.specialize(shapes)
        assert k.cache_hit and k.source == first.source, shapes
    ragged = dyn.specialize([[32, 1, 40, 40], [32, 12, 40, 40]])
    assert not ragged.cache_hit and "akg_overlap" in ragged.source
    k = dyn.specialize([[32, 1, 44, 44], [32, 12, 44, 44]])
    assert k.cache_hit and k.source == ragged.source


def test_streaming_and_column_kernels_take_their_open_extent_as_an_argument(monkeypatch):
    """Reductions over the outermost extent of their operand (column sums over the tokens, a whole tensor into one number)
    and reductions over one inner axis with the batch in front of it: that extent is a kernel argument (with the split
    of the streaming kernel, which the host chooses per call), so a new extent costs a lowering and no device
    compilation. The grid and the workspace still follow the extent."""
    import json
    from dynamic_cases import DYNAMIC_COLUMNS, DYNAMIC_STREAMS, open_extent
    monkeypatch.setenv("AKG_HIP_NO_CACHE", "0")
    for cases, family, arg, extents in ((DYNAMIC_STREAMS, "stream_reduce", "akg_r_arg", (6000, 40, 16384, 7)),
                                        (DYNAMIC_COLUMNS, "column_reduce", "akg_outer_arg", (6, 2, 40))):
        for kind, make in sorted(cases.items()):
            dyn = driver.HipDynamicKernel(open_extent(make(7777, "dynhost_" + kind), 7777), out_dir=None)
            seen = []
            for t in extents:
                bound = json.loads(make(t, "dynhost_" + kind))
                k = dyn.specialize([e[0]["shape"] for e in bound["input_desc"]])
                assert k.family == family and arg in k.source, (kind, t, k.family)
                seen.append(k)
            assert all(k.source == seen[0].source for k in seen), kind
            assert all(k.cache_hit for k in seen[1:]), kind
            if family == "stream_reduce" and not kind.startswith("declared"):
                # one workgroup per strip of columns for the short extent, hundreds for the long one
                assert seen[2].grid[0] > seen[1].grid[0], (kind, seen[1].grid, seen[2].grid)
                assert seen[2].workspace_bytes > seen[1].workspace_bytes >= 256
            if family == "column_reduce":
                assert seen[2].grid[0] == 20 * seen[1].grid[0]
    # batch and tokens of [batch, tokens, hidden] both open: the batch is a fourth argument and the stride of a batch
    # index is computed from the token count
    from dynamic_cases import DYNAMIC_POOLS, DYNAMIC_STATS
    for kind, make in sorted(DYNAMIC_POOLS.items()):
        dyn = driver.HipDynamicKernel(open_extent(make(7777, 5555, "dynhost_" + kind), (7777, 5555)), out_dir=None)
        seen = [dyn.specialize([e[0]["shape"] for e in json.loads(make(b, t, "dynhost_" + kind))["input_desc"]])
                for b, t in ((4, 300), (32, 64), (2, 5000))]
        assert all(k.family == "stream_reduce" and "akg_o_arg" in k.source and "akg_o * (R * " in k.source for k in seen), kind
        # a result with the shape of the reduced value is as many bytes as the kept extent says
        assert all("make_buffer(out0, akg_o_arg * " in k.source for k in seen), kind
        assert all(k.source == seen[0].source for k in seen) and all(k.cache_hit for k in seen[1:]), kind
    # data movement with the batch open: the number of chunks is an argument; ops on the batch axis keep its extent
    from dynamic_cases import DYNAMIC_VIEWS
    for kind, (make, sentinels, shared) in sorted(DYNAMIC_VIEWS.items()):
        dyn = driver.HipDynamicKernel(open_extent(make(7777, "dynhost_" + kind), sentinels), out_dir=None)
        seen = [dyn.specialize([e[0]["shape"] for e in json.loads(make(n, "dynhost_" + kind))["input_desc"]]) for n in (4, 32, 3)]
        assert all(k.family == "indexed" for k in seen), kind
        assert (len({k.source for k in seen}) == 1) == shared, kind
        assert all(k.cache_hit for k in seen[1:]) == shared, kind
    # the batch of [N,C,H,W] statistics: N * H * W is the argument, the buffer sizes follow N
    for kind, make in sorted(DYNAMIC_STATS.items()):
        dyn = driver.HipDynamicKernel(open_extent(make(7777, "dynhost_" + kind), 7777), out_dir=None)
        seen = [dyn.specialize([e[0]["shape"] for e in json.loads(make(n, "dynhost_" + kind))["input_desc"]]) for n in (8, 3, 32)]
        assert all(k.family == "stream_reduce" and "akg_r_arg" in k.source for k in seen), kind
        assert all(k.source == seen[0].source for k in seen) and all(k.cache_hit for k in seen[1:]), kind


def test_description_that_ended_the_device_compiler_with_slp_vectorisation(tmp_path, monkeypatch):
    """A random description (bf16 operands, a Sub, casts through float16, a column sum with its reduced extent open) whose
    kernel ended instruction selection with a fatal error - and the process with it - while the SLP vectoriser was on: it
    formed a two-lane float32 subtraction that the backend cannot select with packed float32 operations switched off.
    Device compiles run without that vectoriser; here the description must compile, and AKG_HIP_DUMP_SOURCE must leave
    the source of what was compiled on disk (what names the culprit when a compiler does end the process)."""
    import json
    monkeypatch.setenv("AKG_HIP_DUMP_SOURCE", str(tmp_path))
    monkeypatch.setenv("AKG_HIP_NO_CACHE", "1")
    path = os.path.join(os.path.dirname(REF_INFO), "regress", "two_lane_float_sub_next_to_half_casts.dynamic.info")
    dyn = driver.HipDynamicKernel(open(path, encoding="utf-8").read(), out_dir=None)
    k = dyn.specialize([[8, 16, 33, 7], [1, 16, 33, 7]])
    assert k.family == "stream_reduce" and not k.cache_hit
    dumped = os.path.join(str(tmp_path), k.kernel_name + ".hip")
    assert os.path.exists(dumped) and open(dumped, encoding="utf-8").read() == k.source


def test_hardware_tanh_form_only_where_its_absolute_error_cannot_grow():
    """Values that only reach 16-bit outputs may use hardware approximations. The tanh form 1 - 2 / (e^2x + 1) is the one
    whose error is absolute (1.2e-7 near zero): it stays only where nothing can blow that up - GELU, whose factor x is what
    the tanh's own argument is made of (a large x saturates the tanh exactly) - and gives way to the series-near-zero
    implementation (relative error) behind a constant of 1024 and more or an unrelated computed factor."""
    gelu = driver.HipKernel(op_desc.gemm_bias_act(64, 64, 64, "bfloat16", "gelu", False, "float32", "tanh_gelu"), out_dir=None)
    assert "akg::fast_tanh(" in gelu.source and "akg::op_tanh(" not in gelu.source

    def scaled(factor_is_input, constant):
        b = op_desc.DescBuilder("tanh_scaled_%d_%d" % (int(factor_is_input), int(constant)))
        x = b.cast(b.input([64, 256], "bfloat16"), "float32")
        t = b.unary("Tanh", x)
        f = b.cast(b.input([64, 256], "bfloat16"), "float32") if factor_is_input else b.const(constant, "float32")
        return driver.HipKernel(b.dumps([b.cast(b.mul(t, f), "bfloat16")]), out_dir=None).source
    assert "akg::fast_tanh(" in scaled(False, 8.0)
    assert "akg::op_tanh(" in scaled(False, 4096.0) and "akg::fast_tanh(" not in scaled(False, 4096.0)
    assert "akg::op_tanh(" in scaled(True, 0.0) and "akg::fast_tanh(" not in scaled(True, 0.0)
    # a float32 output never sees an approximation
    b = op_desc.DescBuilder("tanh_f32")
    assert "akg::fast_tanh(" not in driver.HipKernel(b.dumps([b.unary("Tanh", b.input([64, 256], "float32"))]), out_dir=None).source


def test_sixteen_bit_matmul_runs_on_the_matrix_units_only_by_explicit_switch(monkeypatch, tmp_path):
    """A MatMul declared float16 / bfloat16 means 16-bit accumulation in the reference: the serial kernel by default (bit
    for bit, slow). AKG_HIP_MATMUL_F32_ACC=1 is the caller's consent to float32 accumulation rounded once; the `schedule`
    entry of `<k>.json` says which one runs."""
    text = op_desc.gemm_bias_act(256, 512, 256, "bfloat16", "gelu", False, "bfloat16", "mm_declared_bf16")
    k = driver.HipKernel(text, out_dir=str(tmp_path / "serial"))
    meta = json.load(open(tmp_path / "serial" / "mm_declared_bf16.json"))
    assert "akg::gemm_serial<" in k.source and "serial" in meta["schedule"]
    monkeypatch.setenv("AKG_HIP_MATMUL_F32_ACC", "1")
    k = driver.HipKernel(text, out_dir=str(tmp_path / "mfma"))
    meta = json.load(open(tmp_path / "mfma" / "mm_declared_bf16.json"))
    assert "akg::gemm_256x256<akg::MmaBF16" in k.source and "accr[e] = akg::bf16::rnd(acc[e])" in k.source
    assert "AKG_HIP_MATMUL_F32_ACC" in meta["schedule"]
