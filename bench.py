#!/usr/bin/env python3
"""Benchmark of the fused-operator hot path on one MI355X.

A "step" is one launch of the fused kernel of one op description through the C ABI (akg_hip_launch) on buffers that
are already resident in HBM. The headline workload is the fused softmax fp16 [8192,4096]; every measured configuration
is reported under `per_config`. Inputs are synthetic (seeded); several distinct buffer sets are rotated so that a launch
reads from HBM and not from the 256 MB last-level cache.

Prints ONE JSON line on stdout (kept short, so that a stored tail holds all of it); the long per-workload and
calibration records go to stderr as one line that starts with "detail: ":
  value / ms_per_step  host-clock throughput of K back-to-back steps (algorithmic bytes / wall time)
  roofline             achieved = algorithmic bytes (or ops) per launch / mean launch duration from HIP events recorded
                       on the launch stream around the same K launches; peak = 8 TB/s HBM3E (or the dense MFMA peak);
                       traffic = HBM bytes per launch as the rocprofv3 summary under profiles/ holds them (null if the
                       summary is missing)
  cpu_baseline         the CPU oracle (C restatement of the reference CPU pipeline, 1 thread like the reference's
                       default, and its OpenMP build on all host cores) timed on this host on a bounded sample
  roofline.by_config   {short name: {bound, frac, kernel_ms}} for every measured workload (c1 .. c5 are the five of
                       BASELINE.json), from the same run
  cpu_by_config        the CPU baseline of the other BASELINE configurations, in short
  calibration          {name: fraction of the peak} of what the box itself allows (below), and socket power / shader clock
                       sampled while C5 and the register-only MFMA loop run (outside any timed region)
  per_config (detail)  the same roofline object per workload, with kernel_ms (mean of the K launches), kernel_ms_median
                       and kernel_ms_min (over groups of 10 launches), a cache-resident figure for the two configurations
                       that fit the last-level cache, and a cpu_baseline for each of the five measured configurations
  calibration (detail) what the box itself allows, measured in the same run: streaming kernels of exactly the sizes of
                       C1 and C2 (this backend's own minimal kernels and the vendor's device-to-device copy), register-only
                       MFMA loops on zero and on random operands (the part is power limited), and the vendor library's
                       GEMM on the shapes of C5 and N2
"""
import argparse
import ctypes
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FIXTURES = os.path.join(ROOT, "akg_amd", "fixtures")
PROFILES = os.path.join(ROOT, "profiles")
PROBE_LIB = os.path.join(ROOT, "bench_probe", "libakg_bench_probe.so")
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
    # reductions over an axis that is not the innermost one whose results meet the tensor again: the column kernel keeps
    # the reduced run in registers (one read, one write); per_config also times the same description as one kernel per
    # reduction level (three reads)
    "n8_softmax_axis1_f16_32x21x512x512": "f32",
    "n9_layernorm_axis1_bf16_64x768x1024": "f32",
    # RMSNorm over the last axis (row family), alone and with the residual add in front (two outputs)
    "n10_rmsnorm_bf16_16384x4096": "f32",
    "n11_rmsnorm_add_bf16_16384x4096": "f32",
    # a MatMul DECLARED bfloat16: the reference rounds product and sum to 16 bits at every k, which only a serial chain
    # per result on the vector ALUs reproduces (bit-exact); this row shows what that rule costs against n2's float32 spelling
    "n12_gemm_serial_bf16_declared_bf16_1024x1024x1024": "bf16",
}
# workloads also measured on the schedule of several kernels (AKG_HIP_VARIANT=7 while the handle is built)
SEVERAL_KERNELS = ("n8_softmax_axis1_f16_32x21x512x512", "n9_layernorm_axis1_bf16_64x768x1024")
DEFAULT_WORKLOAD = "c2_softmax_f16_8192x4096"
# plain streaming kernel of known size (out = -x, 256 MiB in + 256 MiB out): calibrates the HBM traffic counters
CALIBRATION = "calib_neg_f32_16384x4096"
# streaming kernels with next to no arithmetic, of exactly the tensor sizes of C1 (3 reads + 1 write of 16 MiB) and C2
# (1 read + 1 write of 64 MiB): what a kernel of that size can reach on this box
SIZE_MATCHED = {"calib_add3_f32_1024x4096": "c1_ew_tanh_add_mul_f32_1024x4096",
                "calib_neg_f16_8192x4096": "c2_softmax_f16_8192x4096"}
# bounded CPU samples: the description the CPU leg runs, and how it relates to the workload
CPU_SAMPLES = {
    "c1_ew_tanh_add_mul_f32_1024x4096": ("c1_ew_tanh_add_mul_f32_1024x4096", "the full workload", 1.0),
    "c2_softmax_f16_8192x4096": ("c2_softmax_f16_8192x4096", "the full workload", 1.0),
    "c3_layernorm_residual_bf16_16384x4096": ("c3_layernorm_residual_bf16_16384x4096", "the full workload", 1.0),
    "c4_quant_int8_residual_bf16_32768x8192": ("c4_quant_int8_residual_bf16_32768x8192", "the full workload", 1.0),
    "c5_gemm_i8_dequant_bias_gelu_4096x8192x8192": ("c5_mslice64_gemm_i8_dequant_bias_gelu_64x8192x8192",
                                                    "an M-slice of 64 of the 4096 rows of A (1/64 of the ops, the whole of B)", 1.0 / 64),
}
CACHE_RESIDENT = ("c1_ew_tanh_add_mul_f32_1024x4096", "c2_softmax_f16_8192x4096")
CLOCK_RAMP_MS = 120.0
GROUP = 10   # launches per timed group of the median / min pass


def traffic_from_profile(name):
    """HBM bytes per launch from the rocprofv3 summary of this workload (profiles/<name>.md), or None."""
    try:
        with open(os.path.join(PROFILES, name + ".md"), "r", encoding="utf-8") as f:
            m = re.search(r"Traffic per launch = (\d+) bytes", f.read())
        return int(m.group(1)) if m else None
    except OSError:
        return None


def ramp(launch, torch):
    """An idle MI355X sits at a few hundred MHz and needs some tens of milliseconds of sustained work to reach its
    steady clocks (the first ~15 ms of launches after idle run 10-25 % slower). The figures reported are steady-state
    ones, so the device is kept busy for CLOCK_RAMP_MS before the warm-up steps."""
    t_ramp = time.perf_counter()
    i = 0
    while (time.perf_counter() - t_ramp) * 1e3 < CLOCK_RAMP_MS:
        for _ in range(16):
            launch(i)
            i += 1
        torch.cuda.synchronize()


def timed(launch, steps, warmup, torch, groups=True):
    """(wall ms, mean event ms, median ms, min ms) per step of `launch(i)`. The K steps of the contract are one region
    bracketed by two events on the launch stream; median and min come from a second pass in groups of GROUP launches."""
    stream = torch.cuda.current_stream()
    ramp(launch, torch)
    for i in range(warmup):
        launch(i)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for i in range(steps):
        launch(i)
    e1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / steps
    mean_ms = e0.elapsed_time(e1) / steps
    if not groups:
        return wall_ms, mean_ms, None, None
    n_groups = max(3, steps // GROUP)
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(n_groups + 1)]
    marks[0].record(stream)
    for g in range(n_groups):
        for i in range(GROUP):
            launch(g * GROUP + i)
        marks[g + 1].record(stream)
    torch.cuda.synchronize()
    per = [marks[g].elapsed_time(marks[g + 1]) / GROUP for g in range(n_groups)]
    return wall_ms, mean_ms, statistics.median(per), min(per)


def gpu_measure(name, steps, warmup, torch, driver, harness, np, resident=False, variant=None, text=None):
    path = os.path.join(FIXTURES, name + ".info")
    desc = json.loads(text) if text is not None else harness.load_desc(path)
    if text is not None:
        kernel = driver.HipKernel(text, out_dir=None)      # a description made for this run (the size sweep)
    elif variant is None:
        kernel = driver.HipKernel.from_file(path)
    else:
        # another schedule of the same description: built without artifacts, so that the cached default stays
        before = os.environ.get("AKG_HIP_VARIANT")
        os.environ["AKG_HIP_VARIANT"] = str(variant)
        try:
            kernel = driver.HipKernel.from_file(path, out_dir=None)
        finally:
            if before is None:
                del os.environ["AKG_HIP_VARIANT"]
            else:
                os.environ["AKG_HIP_VARIANT"] = before
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 1)
    dev = torch.device("cuda:0")
    per_set = sum(t.nbytes for t in kernel.tensors)
    nsets = 1 if resident else max(2, min(12, int(1.2e9 // per_set) + 1))
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
    st = torch.cuda.current_stream().cuda_stream
    wall_ms, mean_ms, med_ms, min_ms = timed(lambda i: kernel.launch_ptrs(ptrs[i % nsets], st), steps, warmup, torch)
    return kernel, inputs, wall_ms, mean_ms, med_ms, min_ms, nsets


def roofline_of(kernel, kernel_ms, name):
    int8 = WORKLOADS.get(name) == "int8"
    mfma_peak = INT8_MFMA_PEAK_TOPS if int8 else BF16_MFMA_PEAK_TFLOPS
    # the bound that takes longer at its peak decides: a contraction with a skinny operand is bound by its operand stream
    mfma_bound = kernel.algorithmic_ops / (mfma_peak * 1e12) > kernel.algorithmic_bytes / (HBM_PEAK_GBS * 1e9)
    if kernel.algorithmic_ops and mfma_bound:
        achieved = kernel.algorithmic_ops / (kernel_ms * 1e-3) / 1e12
        peak = mfma_peak
        return {"bound": "mfma", "achieved": round(achieved, 2), "peak": peak, "unit": "TOP/s" if int8 else "TFLOP/s",
                "frac": round(achieved / peak, 4), "traffic": traffic_from_profile(name)}
    achieved = kernel.algorithmic_bytes / (kernel_ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic_from_profile(name)}


def cpu_baseline(name, harness, driver):
    """Time the CPU oracle (checker code; used here only as the reported CPU baseline) on the bounded sample of `name`."""
    from oracle import cpu_ref
    sample, what, share = CPU_SAMPLES[name]
    path = os.path.join(FIXTURES, sample + ".info")
    desc = harness.load_desc(path)
    kernel = driver.HipKernel.from_file(path)       # algorithmic work of the sample, from the same accounting
    inputs = harness.make_inputs(desc, seed=harness.BASE_SEED + 1)
    is_gemm = kernel.algorithmic_ops > 0
    work = kernel.algorithmic_ops / 1e12 if is_gemm else kernel.algorithmic_bytes / 1e9
    unit = ("TOP/s" if WORKLOADS.get(name) == "int8" else "TFLOP/s") if is_gemm else "GB/s"
    serial = cpu_ref.CpuKernel(path, openmp=False)
    slow = is_gemm or kernel.algorithmic_bytes > 1e9
    t = serial.time(inputs, warmup=0 if slow else 1, iters=1 if slow else 3)
    out = {"value": round(work / t, 6 if is_gemm else 3), "unit": unit, "cores": 1, "kind": "port",
           "sample": "%s: %s, serial C restatement, %.3f s per call%s" %
                     (sample, what, t, "" if share == 1.0 else " (the rate is that of the slice; the full workload is %d slices)" % round(1 / share))}
    try:
        par = cpu_ref.CpuKernel(path, openmp=True)
        tp = par.time(inputs, warmup=1, iters=2)
        out["all_cores_value"] = round(work / tp, 6 if is_gemm else 3)
        out["all_cores"] = int(os.environ.get("OMP_NUM_THREADS", 0)) or (os.cpu_count() or 1)
    except Exception as e:  # the OpenMP build is optional
        out["all_cores_error"] = str(e)
    return out


class PowerSampler:
    """Socket power (W) and shader clock (MHz) of GPU 0 read through amdsmi while a callable keeps the device busy (2.6 s, the
    readings of the last second: they refresh about once a second); never inside a timed region. Every field is None where the library or the permission to read is missing."""

    def __init__(self):
        self.smi = None
        self.handle = None
        try:
            import amdsmi
            amdsmi.amdsmi_init()
            self.smi = amdsmi
            self.handle = amdsmi.amdsmi_get_processor_handles()[0]
        except Exception:  # no library, no device node, no permission
            self.smi = None

    def read(self):
        if self.smi is None:
            return None, None
        power = clock = None
        try:
            info = self.smi.amdsmi_get_power_info(self.handle)
            for key in ("current_socket_power", "average_socket_power", "socket_power"):
                v = info.get(key)
                if isinstance(v, (int, float)) and v > 0:
                    power = float(v)
                    break
        except Exception:
            pass
        try:
            info = self.smi.amdsmi_get_clock_info(self.handle, self.smi.AmdSmiClkType.GFX)
            v = info.get("clk", info.get("cur_clk"))
            if isinstance(v, (int, float)) and v > 0:
                clock = float(v)
        except Exception:
            pass
        return power, clock

    def during(self, launch, torch, busy_ms=2600.0):
        """Keeps the device busy with `launch(i)` for busy_ms and samples between batches of launches."""
        if self.smi is None:
            return {"socket_power_w": None, "shader_clock_mhz": None, "samples": 0}
        powers, clocks = [], []
        t0 = time.perf_counter()
        i = 0
        while (time.perf_counter() - t0) * 1e3 < busy_ms:
            for _ in range(8):
                launch(i)
                i += 1
            if (time.perf_counter() - t0) * 1e3 > busy_ms * 0.6:   # the library's readings refresh about once a second
                p, c = self.read()
                if p is not None:
                    powers.append(p)
                if c is not None:
                    clocks.append(c)
            torch.cuda.synchronize()
        cap = None
        try:
            cap = round(float(self.smi.amdsmi_get_power_cap_info(self.handle).get("power_cap", 0)) / 1e6, 0) or None
        except Exception:
            pass
        return {"socket_power_w": round(statistics.median(powers), 1) if powers else None, "power_cap_w": cap,
                "shader_clock_mhz": round(statistics.median(clocks), 0) if clocks else None, "samples": max(len(powers), len(clocks))}


def vendor_gemm(kind, torch, steps):
    """The vendor library's GEMM on the shape and layout of C5 (int8) / N2 (bf16): no epilogue, same buffers reused."""
    dev = torch.device("cuda:0")
    m, k, n = 4096, 8192, 8192
    if kind == "int8":
        a = torch.randint(-127, 128, (m, k), dtype=torch.int8, device=dev)
        b = torch.randint(-127, 128, (k, n), dtype=torch.int8, device=dev)
        call, peak, unit = (lambda i: torch._int_mm(a, b)), INT8_MFMA_PEAK_TOPS, "TOP/s"
        what = "torch._int_mm, B row-major as in C5, int32 result, no epilogue, same buffers reused"
    else:
        a = (torch.randn((m, k), device=dev) * 0.25).to(torch.bfloat16)
        b = (torch.randn((k, n), device=dev) * 0.25).to(torch.bfloat16)
        call, peak, unit = (lambda i: torch.matmul(a, b)), BF16_MFMA_PEAK_TFLOPS, "TFLOP/s"
        what = "torch.matmul, B row-major as in N2, bf16 result, no epilogue, same buffers reused"
    _, mean_ms, med_ms, min_ms = timed(call, steps, 3, torch)
    rate = 2.0 * m * n * k / (mean_ms * 1e-3) / 1e12
    return {"kernel_ms": round(mean_ms, 5), "kernel_ms_median": round(med_ms, 5), "kernel_ms_min": round(min_ms, 5),
            "achieved": round(rate, 1), "unit": unit, "frac": round(rate / peak, 4), "what": what}


def size_sweep(torch, driver, harness, np, steps, warmup):
    """C1's and C2's kernels at half to eight times their rows: kernel time = fixed + bytes / rate fitted by least
    squares. `fixed_us` is what a launch of this kind costs whatever its size (ramp of the first loads, drain of the
    last stores), `asymptote_frac` the fraction of the HBM peak the same kernel streams at once that cost is amortised;
    `frac_at_size` is what the fit gives at the configuration's own size."""
    from akg_amd import op_desc
    out = {}
    patterns = {
        "c1": (lambda r: op_desc.elementwise_tanh_add_mul(r, 4096, name="sweep_c1_%d" % r), 1024),
        "c2": (lambda r: op_desc.softmax_last_axis(r, 4096, "float16", name="sweep_c2_%d" % r), 8192),
    }
    for key, (make, base_rows) in patterns.items():
        xs, ys, points = [], [], {}
        for factor in (0.5, 1, 2, 4, 8):
            rows = int(base_rows * factor)
            k, _, _, mean_ms, _, _, _ = gpu_measure("sweep", steps, warmup, torch, driver, harness, np, text=make(rows))
            xs.append(float(k.algorithmic_bytes))
            ys.append(mean_ms * 1e-3)
            points["%dx4096" % rows] = round(mean_ms * 1e3, 2)
            del k
        a = np.vstack([np.ones(len(xs)), np.array(xs)]).T
        (fixed_s, per_byte), *_ = np.linalg.lstsq(a, np.array(ys), rcond=None)
        base_bytes = xs[1]
        out[key] = {"kernel_us_by_shape": points, "fixed_us": round(fixed_s * 1e6, 2),
                    "asymptote_frac": round(1.0 / per_byte / 1e9 / HBM_PEAK_GBS, 4),
                    "frac_at_size": round(base_bytes / (fixed_s + per_byte * base_bytes) / 1e9 / HBM_PEAK_GBS, 4)}
    return out


def calibration(torch, driver, harness, np, steps, warmup, sampler=None, power=None):
    """Ceilings of this box, measured in this run."""
    out = {}
    power = {} if power is None else power
    dev = torch.device("cuda:0")
    # 1. streaming kernels of exactly C1's and C2's sizes: this backend's own minimal kernels ...
    for calib, twin in SIZE_MATCHED.items():
        try:
            k, _, _, mean_ms, med_ms, min_ms, _ = gpu_measure(calib, steps, warmup, torch, driver, harness, np)
            gbs = k.algorithmic_bytes / (mean_ms * 1e-3) / 1e9
            out[calib] = {"size_of": twin, "bytes": k.algorithmic_bytes, "kernel_ms": round(mean_ms, 5),
                          "kernel_ms_median": round(med_ms, 5), "kernel_ms_min": round(min_ms, 5),
                          "achieved": round(gbs, 1), "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4)}
        except Exception as e:
            out[calib] = {"error": str(e)}
    # ... and the vendor's device-to-device copy moving the same number of bytes (half read, half written)
    for label, total in (("vendor_copy_64MiB_moved", 64 << 20), ("vendor_copy_128MiB_moved", 128 << 20)):
        half = total // 2
        nsets = max(2, int(1.2e9 // total) + 1)
        src = [torch.randint(0, 255, (half,), dtype=torch.uint8, device=dev) for _ in range(nsets)]
        dst = [torch.empty(half, dtype=torch.uint8, device=dev) for _ in range(nsets)]
        _, mean_ms, med_ms, min_ms = timed(lambda i: dst[i % nsets].copy_(src[i % nsets]), steps, warmup, torch)
        gbs = total / (mean_ms * 1e-3) / 1e9
        out[label] = {"bytes": total, "kernel_ms": round(mean_ms, 5), "kernel_ms_median": round(med_ms, 5),
                      "kernel_ms_min": round(min_ms, 5), "achieved": round(gbs, 1), "unit": "GB/s",
                      "frac": round(gbs / HBM_PEAK_GBS, 4), "what": "torch Tensor.copy_ between two device buffers"}
        del src, dst
    # 2. register-only MFMA loops (no memory traffic in the loop) on zero and on random operands
    try:
        probe = ctypes.CDLL(PROBE_LIB)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        fns = {"i8": probe.akg_probe_mfma_i8, "bf16": probe.akg_probe_mfma_bf16,
               "i8_32x32": probe.akg_probe_mfma_i8_32x32, "bf16_32x32": probe.akg_probe_mfma_bf16_32x32}
        for fn in fns.values():
            fn.argtypes = [vp, vp, ci, ci, vp]
        rng = np.random.default_rng(7)
        workgroups, iterations = 512, 500
        sink = torch.empty(workgroups * 512, dtype=torch.int32, device=dev)
        st = torch.cuda.current_stream().cuda_stream
        zeros = np.zeros(32 * 1024, np.uint8)
        random_i8 = rng.integers(-127, 128, 32 * 1024, dtype=np.int8).view(np.uint8)
        random_bf16 = harness.f32_to_bf16_bits((rng.standard_normal(16 * 1024) * 0.25).astype(np.float32)).view(np.uint8)
        for kind, peak, unit, per_iteration in (("i8", INT8_MFMA_PEAK_TOPS, "TOP/s", 2097152), ("bf16", BF16_MFMA_PEAK_TFLOPS, "TFLOP/s", 1048576)):
            for shape, suffix in (("16x16 tiles, 64 bytes of K per MFMA (the GEMM kernel's shape)", ""), ("32x32 tiles, 32 bytes of K per MFMA", "_32x32")):
                for operands, host in (("zero", zeros), ("random", random_i8 if kind == "i8" else random_bf16)):
                    label = "mfma_%s%s_register_loop_%s_operands" % (kind, suffix, operands)
                    fn = fns[kind + suffix]
                    ops = workgroups * 8 * iterations * per_iteration
                    buf = torch.from_numpy(np.ascontiguousarray(host)).to(dev)
                    _, mean_ms, med_ms, min_ms = timed(lambda i: fn(st, buf.data_ptr(), iterations, workgroups, sink.data_ptr()),
                                                       max(10, steps // 10), 2, torch)
                    rate = ops / (mean_ms * 1e-3) / 1e12
                    if sampler is not None and kind == "i8" and suffix == "":
                        power[label] = sampler.during(lambda i: fn(st, buf.data_ptr(), iterations, workgroups, sink.data_ptr()), torch)
                    out[label] = {"ops": ops, "kernel_ms": round(mean_ms, 4), "kernel_ms_median": round(med_ms, 4),
                                  "kernel_ms_min": round(min_ms, 4), "achieved": round(rate, 1), "unit": unit, "peak": peak,
                                  "frac": round(rate / peak, 4),
                                  "what": "512 workgroups x 8 wavefronts, nothing but MFMAs on register operands, " + shape}
    except OSError as e:
        out["mfma_register_loops"] = {"error": str(e)}
    # 3. the vendor library on the GEMM shapes (no epilogue: plain int32 / bf16 result)
    try:
        for kind in ("int8", "bf16"):
            out["vendor_%s_gemm_4096x8192x8192" % kind] = vendor_gemm(kind, torch, max(20, steps // 4))
    except Exception as e:  # a torch build without these routines
        out["vendor_gemm"] = {"error": str(e)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS) + [CALIBRATION] + sorted(SIZE_MATCHED))
    ap.add_argument("--only", action="store_true", help="measure only --workload (no per_config sweep, no calibration)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--vendor-gemm", choices=("int8", "bf16"),
                    help="run only the vendor library's GEMM of the calibration (for a profiler) and print its figures")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every fused operator here is a single-device kernel (rows shard with no "
                 "exchange); run with --gpus 1")

    import numpy as np
    import torch
    from akg_amd import driver, harness
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")

    if args.vendor_gemm:
        print(json.dumps({"vendor_%s_gemm_4096x8192x8192" % args.vendor_gemm: vendor_gemm(args.vendor_gemm, torch, args.steps)}))
        return
    name = args.workload
    kernel, _, wall_ms, kernel_ms, med_ms, min_ms, nsets = gpu_measure(name, args.steps, args.warmup, torch, driver, harness, np)
    roof = roofline_of(kernel, kernel_ms, name)
    if roof["bound"] == "mfma":
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
        "roofline": roof,
        "kernel_ms": round(kernel_ms, 5), "kernel_ms_median": round(med_ms, 5), "kernel_ms_min": round(min_ms, 5),
    }
    if not args.no_cpu_baseline and name in CPU_SAMPLES:
        line["cpu_baseline"] = cpu_baseline(name, harness, driver)
    short = lambda w: w.split("_", 1)[0]   # noqa: E731  "c5_gemm_..." -> "c5"
    line["config"]["why_this_workload"] = ("configs[1] of BASELINE.json, the configuration the contract names for N=1; all five "
                                           "configurations are under roofline.by_config" if name == DEFAULT_WORKLOAD else "--workload")
    if not args.only:
        per = {}
        by_config = {}
        cpu_by_config = {}
        power = {}
        sampler = PowerSampler()
        for other in sorted(WORKLOADS):
            try:
                if other == name:
                    k2, entry = kernel, dict(roof, kernel_ms=line["kernel_ms"], kernel_ms_median=line["kernel_ms_median"],
                                             kernel_ms_min=line["kernel_ms_min"])
                else:
                    k2, _, _, kms, kmed, kmin, _ = gpu_measure(other, max(20, args.steps // 4), max(5, args.warmup // 2), torch,
                                                               driver, harness, np)
                    entry = dict(roofline_of(k2, kms, other), kernel_ms=round(kms, 5), kernel_ms_median=round(kmed, 5),
                                 kernel_ms_min=round(kmin, 5))
                by_config[short(other)] = {"bound": entry["bound"], "frac": entry["frac"], "kernel_ms": entry["kernel_ms"]}
                if other in CACHE_RESIDENT:
                    # the same buffers launch after launch: reads come from the 256 MB last-level cache
                    _, _, _, rms, _, rmin, _ = gpu_measure(other, max(20, args.steps // 4), max(5, args.warmup // 2), torch,
                                                           driver, harness, np, resident=True)
                    r = roofline_of(k2, rms, other)
                    entry["cache_resident"] = {"kernel_ms": round(rms, 5), "kernel_ms_min": round(rmin, 5),
                                               "achieved": r["achieved"], "unit": r["unit"], "frac_of_hbm_peak": r["frac"]}
                if other in SEVERAL_KERNELS:
                    k3, _, _, sms, smed, smin, _ = gpu_measure(other, max(20, args.steps // 4), max(5, args.warmup // 2), torch,
                                                               driver, harness, np, variant=7)
                    r = roofline_of(k3, sms, other)
                    entry["several_kernels"] = {"family": k3.family, "kernel_ms": round(sms, 5), "kernel_ms_median": round(smed, 5),
                                                "kernel_ms_min": round(smin, 5), "achieved": r["achieved"], "unit": r["unit"],
                                                "frac": r["frac"]}
                if other in CPU_SAMPLES and not args.no_cpu_baseline:
                    entry["cpu_baseline"] = line["cpu_baseline"] if other == name else cpu_baseline(other, harness, driver)
                    c = entry["cpu_baseline"]
                    cpu_by_config[short(other)] = {"value": c["value"], "unit": c["unit"], "cores": c["cores"],
                                                   "all_cores_value": c.get("all_cores_value"), "all_cores": c.get("all_cores")}
                if other.startswith("c5_") and sampler.smi is not None:
                    # power and clock while the int8 GEMM runs (its own buffers, outside any timed region)
                    dev = torch.device("cuda:0")
                    bufs = [torch.zeros(t.nbytes, dtype=torch.uint8, device=dev) for t in k2.tensors]
                    for b, a in zip(bufs, harness.make_inputs(harness.load_desc(os.path.join(FIXTURES, other + ".info")), seed=harness.BASE_SEED + 1)):
                        b.copy_(torch.from_numpy(a.view(np.uint8).reshape(-1)))
                    ptrs = [b.data_ptr() for b in bufs]
                    st = torch.cuda.current_stream().cuda_stream
                    power[short(other)] = sampler.during(lambda i: k2.launch_ptrs(ptrs, st), torch)
                    del bufs
                per[other] = entry
            except driver.AkgHipError as e:
                per[other] = {"error": str(e)}
                by_config[short(other)] = {"error": str(e)[:80]}
        detail = {"per_config": per,
                  "calibration": calibration(torch, driver, harness, np, max(20, args.steps // 4), max(5, args.warmup // 2), sampler, power)}
        detail["power"] = power
        try:
            detail["size_sweep"] = size_sweep(torch, driver, harness, np, max(20, args.steps // 4), max(5, args.warmup // 2))
        except driver.AkgHipError as e:
            detail["size_sweep"] = {"error": str(e)}
        line["roofline"]["by_config"] = by_config
        if cpu_by_config:
            line["cpu_by_config"] = cpu_by_config
        line["calibration"] = dict({k: v.get("frac") for k, v in detail["calibration"].items() if isinstance(v, dict) and "frac" in v},
                                   power=power, size_sweep={k: {x: v[x] for x in ("fixed_us", "asymptote_frac", "frac_at_size")}
                                                            for k, v in detail["size_sweep"].items() if isinstance(v, dict) and "fixed_us" in v})
        sys.stderr.write("detail: " + json.dumps(detail) + "\n")
        sys.stderr.flush()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
