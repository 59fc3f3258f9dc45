"""GPU parity: every fused kernel, launched through the C ABI on device-resident buffers, against the CPU oracle
(the C restatement of the reference CPU pipeline) on the same seeded inputs.

Bars: int8 / integer outputs bit-exact; float32 rtol 1e-5 (atol 1e-8); float16 / bfloat16 rtol 1e-2, atol 1e-3.
Outputs are NaN-prefilled on the device so that an element the kernel does not write fails the comparison.
"""
import glob
import os

import numpy as np
import pytest

from akg_amd import driver, harness
from oracle import cpu_ref

pytestmark = pytest.mark.gpu

FIXTURES = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "akg_amd", "fixtures")
SMALL = sorted(os.path.basename(p) for p in glob.glob(os.path.join(FIXTURES, "small_*.info")))
FULL = ["c1_ew_tanh_add_mul_f32_1024x4096.info", "c2_softmax_f16_8192x4096.info",
        "c3_layernorm_residual_bf16_16384x4096.info", "c4_quant_int8_residual_bf16_32768x8192.info"]


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
    for d, g, e in zip(kernel.outputs, got, expect):
        ok, msg = harness.compare(g, e, d.dtype)
        print("  %s %s: %s" % (d.name, d.dtype, msg), flush=True)
        assert ok, "%s output %s: %s" % (name, d.name, msg)


@pytest.mark.parametrize("name", SMALL)
def test_small_fixture_matches_oracle(name):
    check_fixture(name, seed=harness.BASE_SEED + 100, openmp=False)


@pytest.mark.parametrize("name", FULL)
def test_full_size_config_matches_oracle(name):
    # full BASELINE sizes; the oracle runs its OpenMP build (same per-row arithmetic, rows in parallel)
    check_fixture(name, seed=harness.BASE_SEED + 1 + FULL.index(name), openmp=True)
