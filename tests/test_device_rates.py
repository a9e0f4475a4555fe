"""The stand-alone yardsticks beside the library (csrc/mfma_rate.hip, csrc/hbm_rate.hip): they are built with the
library, refuse bad arguments before touching a device, and on a GPU print the JSON lines bench.py reads."""

import json
import os
import subprocess

import pytest

LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tensor-product-attention-jax_amd", "lib")
EXE = os.path.join(LIB, "mfma_rate")
HBM = os.path.join(LIB, "hbm_rate")


def test_built_and_refuses_bad_arguments():
    assert os.access(EXE, os.X_OK), f"{EXE} missing: run make in tensor-product-attention-jax_amd/csrc"
    for argv in (["3"], ["2", "0", "0"], ["1", "0", "256", "0"], ["2", "0", "70000"]):
        r = subprocess.run([EXE, *argv], capture_output=True, text=True, timeout=30)
        assert r.returncode == 2 and "usage" in r.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("waves,zeros", [(1, 1), (2, 0)])
def test_reports_a_rate(gpu, waves, zeros):
    r = subprocess.run([EXE, str(waves), str(zeros), "64", "256"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert line["waves_per_simd"] == waves and line["zeros"] == zeros and line["workgroups"] == 64
    # 64 of 256 CUs cannot exceed a quarter of the device's peak
    assert 0 < line["tflops"] <= 2516.6 / 4 * 1.05


def test_hbm_rate_built_and_refuses_bad_arguments():
    assert os.access(HBM, os.X_OK), f"{HBM} missing: run make in tensor-product-attention-jax_amd/csrc"
    for argv in (["1"], ["100000"], ["x"]):
        r = subprocess.run([HBM, *argv], capture_output=True, text=True, timeout=30)
        assert r.returncode == 2 and "usage" in r.stderr


@pytest.mark.gpu
def test_hbm_rate_reports_rates(gpu):
    r = subprocess.run([HBM, "512"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert line["mib"] == 512
    assert 0 < line["read_gbs"] <= 8000 * 1.05 and 0 < line["copy_gbs"] <= 8000 * 1.05
