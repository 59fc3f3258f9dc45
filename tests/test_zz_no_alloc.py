"""The launch entry point that allocates nothing (akg_hip_launch_static_scratch) against akg_hip_launch.

Kernels that need device memory beyond inputs and outputs take it from a fixed array inside the library instead of the
handle's workspace. Both entry points run the same kernels in the same order and the partial results are combined in a
fixed order, so the outputs must be identical bit for bit (which is inside every bar of the parity tests). Calls follow
each other on one stream; the second description of each sequence is smaller than the first, so it finds the array
holding the first one's leftovers.
"""
import os

import numpy as np
import pytest

from akg_amd import driver, harness

pytestmark = pytest.mark.gpu

FIXTURES = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "akg_amd", "fixtures")

# (larger first, smaller second) - streaming reductions, a GEMM with K split over workgroups, descriptions that run as
# several kernels, a grouped segment sum (several launches of one code object sharing the scratch)
SEQUENCES = [
    ("small_biasgrad_bf16_1000x4095.info", "small_biasgrad_bf16_2048x1024.info"),
    ("small_reducey_sqsum_f32_1x5100x3072.info", "small_reduceall_sqsum_f32_768x512.info"),
    ("small_gemm_i8_dequant_bias_gelu_300x2064x520_tb.info", "small_gemm_bf16_bias_gelu_256x512x256.info"),
    ("small_staged_bn_train_forward_f32_16x8x14x14.info", "small_staged_bn_train_forward_bf16_8x6x7x12.info"),
    ("small_segment_sum_f16_150001_by_4_seg300.info", "small_bnstats_f32_32x16x28x28.info"),
]


def _device_buffers(kernel, inputs):
    import torch
    dev = torch.device("cuda:0")
    ins = [torch.from_numpy(a.view(np.int16) if a.dtype == np.uint16 else a).to(dev) for a in inputs]
    outs = []
    for d in kernel.outputs:
        t = torch.empty(d.nbytes, dtype=torch.uint8, device=dev)
        t.fill_(0xFF if d.dtype in ("float16", "bfloat16", "float32", "float64") else 0x7B)
        outs.append(t)
    return ins, outs


def _run(kernel, inputs, static):
    import torch
    ins, outs = _device_buffers(kernel, inputs)
    ptrs = [t.data_ptr() for t in ins + outs]
    stream = torch.cuda.current_stream().cuda_stream
    if static:
        kernel.launch_static_scratch_ptrs(ptrs, stream)
    else:
        kernel.launch_ptrs(ptrs, stream)
    torch.cuda.synchronize()
    # Assign / InplaceAssign descriptions also write an input: compare those too
    return [t.cpu().numpy().view(np.uint8).copy() for t in outs + ins]


def test_first_static_scratch_launch_is_captured_into_a_graph_and_allocates_nothing():
    """The callers this entry point is for: the FIRST launch through it in the process (when this file runs alone) is
    recorded into a HIP graph - `prepare` has looked the array's address up, so nothing is loaded or materialised under
    capture -, the graph is replayed three times on fresh inputs with the program's own eager launches and
    synchronisations in between, every replay equal to akg_hip_launch bit for bit; and an eager call leaves the
    device's free memory exactly as it found it."""
    import torch
    dev = torch.device("cuda:0")
    path = os.path.join(FIXTURES, "small_biasgrad_bf16_2048x1024.info")
    kernel = driver.HipKernel.from_file(path)
    assert kernel.workspace_bytes > 0
    desc = harness.load_desc(path)
    kernel.prepare()
    static = [torch.zeros(t.nbytes, dtype=torch.uint8, device=dev) for t in kernel.tensors]
    eager = [torch.zeros(t.nbytes, dtype=torch.uint8, device=dev) for t in kernel.tensors]
    n_in = len(kernel.tensors) - len(kernel.outputs)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        kernel.launch_static_scratch_ptrs([b.data_ptr() for b in static], torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        print("replay %d" % replay, flush=True)
        inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 77 + replay)
        for bufs in (static, eager):
            for b, a in zip(bufs, inputs):
                b.copy_(torch.from_numpy(a.view(np.uint8).reshape(-1)))
            for b in bufs[n_in:]:
                b.fill_(0x7B)
        graph.replay()
        torch.cuda.synchronize()
        kernel.launch(eager)                      # the allocating entry point, eagerly, between the replays
        torch.cuda.synchronize()
        for a, b in zip(static[n_in:], eager[n_in:]):
            assert torch.equal(a, b), "replay %d differs from akg_hip_launch" % replay
    free_before = torch.cuda.mem_get_info()[0]
    kernel.launch_static_scratch_ptrs([b.data_ptr() for b in static], torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_after == free_before, "an eager static-scratch launch changed the free device memory by %d bytes" % (free_before - free_after)
    for a, b in zip(static[n_in:], eager[n_in:]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("first,second", SEQUENCES)
def test_static_scratch_launch_equals_the_allocating_launch(first, second):
    cases = []
    for name in (first, second):
        path = os.path.join(FIXTURES, name)
        kernel = driver.HipKernel.from_file(path)
        assert kernel.workspace_bytes > 0, "%s uses no scratch: it proves nothing here" % name
        inputs = harness.make_inputs(harness.load_desc(path), seed=harness.BASE_SEED + 4242)
        kernel.prepare()
        cases.append((name, kernel, inputs))
    expected = [_run(k, i, static=False) for _, k, i in cases]
    # twice through the sequence: the second round starts on an array that every kernel of the first has used
    for round_no in range(2):
        for (name, kernel, inputs), want in zip(cases, expected):
            print("case %s round %d" % (name, round_no), flush=True)
            got = _run(kernel, inputs, static=True)
            for idx, (g, w) in enumerate(zip(got, want)):
                assert np.array_equal(g, w), "%s round %d: buffer %d differs from akg_hip_launch's" % (name, round_no, idx)


def test_static_scratch_launch_of_kernels_that_take_their_extents_as_arguments():
    """Specialisations of a dynamic description: the streaming reduction's kernel takes its reduced extent and its split
    as arguments behind the tensor pointers and always takes the scratch pointer, also when one workgroup per result
    needs no exchange (the second, smaller shape set). Same outputs through both entry points, two rounds."""
    import json
    from dynamic_cases import DYNAMIC_STREAMS, open_extent
    make = DYNAMIC_STREAMS["biasgrad_bf16"]
    dyn = driver.HipDynamicKernel(open_extent(make(7777, "dyn_noalloc"), 7777), out_dir=None)
    cases = []
    for t in (6000, 40):
        bound = json.loads(make(t, "dyn_noalloc"))
        kernel = dyn.specialize([e[0]["shape"] for e in bound["input_desc"]])
        assert kernel.workspace_bytes > 0 and "akg_r_arg" in kernel.source
        kernel.prepare()
        cases.append((t, kernel, harness.make_inputs(bound, seed=harness.BASE_SEED + 4300 + t)))
    expected = [_run(k, i, static=False) for _, k, i in cases]
    for round_no in range(2):
        for (t, kernel, inputs), want in zip(cases, expected):
            print("case T=%d round %d" % (t, round_no), flush=True)
            got = _run(kernel, inputs, static=True)
            for idx, (g, w) in enumerate(zip(got, want)):
                assert np.array_equal(g, w), "T=%d round %d: buffer %d differs from akg_hip_launch's" % (t, round_no, idx)


def test_static_scratch_launch_needs_a_prepared_handle_and_refuses_oversized_scratch():
    path = os.path.join(FIXTURES, "small_reduceall_sqsum_f32_768x512.info")
    kernel = driver.HipKernel.from_file(path)
    inputs = harness.make_inputs(harness.load_desc(path), seed=harness.BASE_SEED)
    ins, outs = _device_buffers(kernel, inputs)
    ptrs = [t.data_ptr() for t in ins + outs]
    with pytest.raises(driver.AkgHipError) as not_loaded:
        kernel.launch_static_scratch_ptrs(ptrs)
    assert not_loaded.value.code == -1 and "akg_hip_kernel_prepare" in str(not_loaded.value)
    # 335 MB of grouped rows: beyond the 16 MiB array
    big = driver.HipKernel.from_file(os.path.join(FIXTURES, "n7_segment_sum_f32_4954x4953_by_1x3_seg4954.info"))
    assert big.workspace_bytes > (16 << 20)
    fake = [ptrs[0]] * len(big.tensors)
    with pytest.raises(driver.AkgHipError) as too_big:
        big.launch_static_scratch_ptrs(fake)
    assert too_big.value.code == -4 and "scratch" in str(too_big.value)


def test_static_scratch_launch_serves_kernels_without_scratch():
    import torch
    path = os.path.join(FIXTURES, "small_softmax_f16_64x4096.info")
    if not os.path.exists(path):
        pytest.skip("fixture missing")
    kernel = driver.HipKernel.from_file(path)
    assert kernel.workspace_bytes == 0
    kernel.prepare()
    inputs = harness.make_inputs(harness.load_desc(path), seed=harness.BASE_SEED + 7)
    want = _run(kernel, inputs, static=False)
    got = _run(kernel, inputs, static=True)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)
    torch.cuda.synchronize()
