#!/usr/bin/env python3
"""Benchmark of the fused-operator hot path on one MI355X.

A "step" is one launch of the fused kernel of one op description through the C ABI (akg_hip_launch) on buffers that
are already resident in HBM. The headline workload is the fused softmax fp16 [8192,4096]; the other measured
configurations are reported in `per_config`. Inputs are synthetic (seeded); several distinct buffer sets are rotated so
that a launch reads from HBM and not from the 256 MB last-level cache.

Prints ONE JSON line:
  value / ms_per_step  host-clock throughput of K back-to-back steps (algorithmic bytes / wall time)
  roofline             achieved = algorithmic bytes per launch / mean launch duration from HIP events recorded on the
                       launch stream around the same K launches; peak = 8 TB/s HBM3E (or the dense int8 MFMA peak)
  cpu_baseline         the CPU oracle (C restatement of the reference CPU pipeline, 1 thread, like the reference's
                       default) timed on this host on the same workload
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FIXTURES = os.path.join(ROOT, "akg_amd", "fixtures")
HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA, published (no sparsity)
BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 / fp16 MFMA, published (no sparsity)

WORKLOADS = {
    "c1_ew_tanh_add_mul_f32_1024x4096": "f32",
    "c2_softmax_f16_8192x4096": "f32",
    "c3_layernorm_residual_bf16_16384x4096": "f32",
    "c4_quant_int8_residual_bf16_32768x8192": "f32",
    "c5_gemm_i8_dequant_bias_gelu_4096x8192x8192": "int8",
    # the row next to the five: two column sums (reduce direction Y) of one pass over two bf16 [16384,4096] tensors
    "n1_biasgrad_bf16_16384x4096": "f32",
    # batched transpose [32,2048,1024] -> [32,1024,2048] fused with a bias add (indexed family)
    "n3_transpose_bias_add_bf16_32x2048x1024": "f32",
    # bfloat16 MatMul + bias + GELU on the same shape as the int8 fusion (float32 accumulation)
    "n2_gemm_bf16_bias_gelu_4096x8192x8192": "bf16",
    # shapes off the measured ones: a softmax row of 131072 (kept packed in registers across three walks), batch-norm
    # statistics (kept axis between reduced ones), a skinny MatMul (B streamed straight into MFMA operands: bound by the weight stream)
    "n4_softmax_f16_512x131072": "f32",
    "n5_bnstats_bf16_256x64x56x56": "f32",
    "n6_gemm_bf16_bias_gelu_16x8192x8192": "bf16",
    # 24.5 million index positions of 3 floats added into 4954 rows in the serial order (five launches per step)
    "n7_segment_sum_f32_4954x4953_by_1x3_seg4954": "f32",
}
DEFAULT_WORKLOAD = "c2_softmax_f16_8192x4096"
# plain streaming kernel of known size (out = -x, 256 MiB in + 256 MiB out): calibrates the HBM traffic counters
CALIBRATION = "calib_neg_f32_16384x4096"

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE; scaled by the same counters' reading
# for a plain copy of known size: FETCH_SIZE reads half the bytes, scale 2.0; WRITE_SIZE scale 1.0). Values are the
# ones of the summaries under profiles/; None = not measured yet.
CLOCK_RAMP_MS = 120.0
MEASURED_TRAFFIC_BYTES = {
    "c1_ew_tanh_add_mul_f32_1024x4096": 67142582,
    "c2_softmax_f16_8192x4096": 134243913,
    "c3_layernorm_residual_bf16_16384x4096": 402797563,
    "c4_quant_int8_residual_bf16_32768x8192": 1343173505,
    "c5_gemm_i8_dequant_bias_gelu_4096x8192x8192": 470254548,
    "n1_biasgrad_bf16_16384x4096": 270924759,
    "n2_gemm_bf16_bias_gelu_4096x8192x8192": 872910920,
    "n3_transpose_bias_add_bf16_32x2048x1024": 268462651,
    "n4_softmax_f16_512x131072": 268593234,
    "n5_bnstats_bf16_256x64x56x56": 102898801,
    "n6_gemm_bf16_bias_gelu_16x8192x8192": 140865236,
    "n7_segment_sum_f32_4954x4953_by_1x3_seg4954": 2127240577,
}


def gpu_measure(name, steps, warmup, torch, driver, harness, np):
    path = os.path.join(FIXTURES, name + ".info")
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 1)
    dev = torch.device("cuda:0")
    per_set = sum(t.nbytes for t in kernel.tensors)
    nsets = max(2, min(12, int(1.2e9 // per_set) + 1))
    sets = []
    for _ in range(nsets):
        bufs = []
        for t, a in zip(kernel.tensors, inputs + [None] * len(kernel.outputs)):
            b = torch.empty(t.nbytes, dtype=torch.uint8, device=dev)
            if a is not None:
                b.copy_(torch.from_numpy(a.view(np.uint8).reshape(-1)))
            bufs.append(b)
        sets.append(bufs)
    ptrs = [[b.data_ptr() for b in bufs] for bufs in sets]
    stream = torch.cuda.current_stream()
    st = stream.cuda_stream
    # Clock ramp: an idle MI355X sits at a few hundred MHz and needs some tens of milliseconds of sustained work
    # to reach its steady clocks (the first ~15 ms of launches after idle run 10-25 % slower). The figures reported
    # are steady-state ones, so the device is kept busy for CLOCK_RAMP_MS before the W warm-up steps.
    t_ramp = time.perf_counter()
    i = 0
    while (time.perf_counter() - t_ramp) * 1e3 < CLOCK_RAMP_MS:
        for _ in range(16):
            kernel.launch_ptrs(ptrs[i % nsets], st)
            i += 1
        torch.cuda.synchronize()
    for i in range(warmup):
        kernel.launch_ptrs(ptrs[i % nsets], st)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for i in range(steps):
        kernel.launch_ptrs(ptrs[i % nsets], st)
    e1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / steps
    kernel_ms = e0.elapsed_time(e1) / steps
    return kernel, inputs, wall_ms, kernel_ms, nsets


def roofline_of(kernel, kernel_ms, name):
    int8 = WORKLOADS.get(name) == "int8"
    mfma_peak = INT8_MFMA_PEAK_TOPS if int8 else BF16_MFMA_PEAK_TFLOPS
    # the bound that takes longer at its peak decides: a contraction with a skinny operand is bound by its operand stream
    mfma_bound = kernel.algorithmic_ops / (mfma_peak * 1e12) > kernel.algorithmic_bytes / (HBM_PEAK_GBS * 1e9)
    if kernel.algorithmic_ops and mfma_bound:
        achieved = kernel.algorithmic_ops / (kernel_ms * 1e-3) / 1e12
        peak = mfma_peak
        return {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TOP/s" if int8 else "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(name)}
    achieved = kernel.algorithmic_bytes / (kernel_ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(name)}


def cpu_baseline(name, inputs, kernel):
    """Time the CPU oracle (checker code; used here only as the reported CPU baseline)."""
    from oracle import cpu_ref
    path = os.path.join(FIXTURES, name + ".info")
    serial = cpu_ref.CpuKernel(path, openmp=False)
    # bounded sample: the full workload, called a few times (a call of the largest configuration takes seconds)
    t = serial.time(inputs, warmup=1, iters=3)
    out = {"value": round(kernel.algorithmic_bytes / t / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
           "sample": "full %s workload, 1 warm-up + 3 timed calls of the serial C restatement (%.3f s per call)" % (name, t)}
    try:
        par = cpu_ref.CpuKernel(path, openmp=True)
        tp = par.time(inputs, warmup=1, iters=3)
        out["all_cores_value"] = round(kernel.algorithmic_bytes / tp / 1e9, 3)
        out["all_cores"] = int(os.environ.get("OMP_NUM_THREADS", 0)) or (os.cpu_count() or 1)
    except Exception as e:  # the OpenMP build is optional
        out["all_cores_error"] = str(e)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS) + [CALIBRATION])
    ap.add_argument("--only", action="store_true", help="measure only --workload (no per_config sweep)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every fused operator here is a single-device kernel (rows shard with no "
                 "exchange); run with --gpus 1")

    import numpy as np
    import torch
    from akg_amd import driver, harness
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")

    name = args.workload
    kernel, inputs, wall_ms, kernel_ms, nsets = gpu_measure(name, args.steps, args.warmup, torch, driver, harness, np)
    is_gemm = roofline_of(kernel, kernel_ms, name)["bound"] == "mfma"
    if is_gemm:
        value = kernel.algorithmic_ops / (wall_ms * 1e-3) / 1e12
        if WORKLOADS.get(name) == "int8":
            unit, metric = "TOP/s", "achieved int8 TOP/s of the fused GEMM (2*M*N*K ops per launch / time)"
        else:
            unit, metric = "TFLOP/s", "achieved TFLOP/s of the fused GEMM (2*M*N*K flops per launch / time)"
    else:
        value = kernel.algorithmic_bytes / (wall_ms * 1e-3) / 1e9
        unit, metric = "GB/s", "achieved HBM GB/s of the fused op (algorithmic bytes per launch / time)"
    line = {
        "metric": metric, "value": round(value, 2), "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": WORKLOADS.get(name, "f32"), "data": "synthetic",
        "config": {"workload": name, "family": kernel.family, "grid": kernel.grid[0], "block": kernel.block[0],
                   "algorithmic_bytes": kernel.algorithmic_bytes, "algorithmic_ops": kernel.algorithmic_ops,
                   "buffer_sets_rotated": nsets, "clock_ramp_ms": CLOCK_RAMP_MS},
        "roofline": roofline_of(kernel, kernel_ms, name),
        "kernel_ms": round(kernel_ms, 5),
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(name, inputs, kernel)
    if not args.only:
        per = {}
        for other in sorted(WORKLOADS):
            if other == name:
                per[other] = dict(line["roofline"], kernel_ms=line["kernel_ms"])
                continue
            try:
                k2, _, _, kms, _ = gpu_measure(other, max(20, args.steps // 4), max(5, args.warmup // 2), torch, driver,
                                               harness, np)
                per[other] = dict(roofline_of(k2, kms, other), kernel_ms=round(kms, 5))
            except driver.AkgHipError as e:
                per[other] = {"error": str(e)}
        line["per_config"] = per
    print(json.dumps(line))


if __name__ == "__main__":
    main()
