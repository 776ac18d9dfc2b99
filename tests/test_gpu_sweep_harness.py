"""The reference's perf harness (performance/output.log:1-13, test/test.cc:37-61) as
`bench.py --sweep matmul`, run on the GPU: its log is parsed field by field, and sampled
rows of every C it computed are checked against the oracle on the same seeded operands
(the harness's own correctness column compares with the ROCm library only)."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from conftest import rel_err
from kernelcodegen_amd import inputs, sweeps

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

BLOCK = re.compile(
    r"Matrix size : \n --- M --- : (\d+)\n --- N --- : (\d+)\n --- K --- : (\d+)\n\n"
    r"Occupancy: (\d+)%  \(computed from the launch geometry: (\S+), grid (\d+) x (\d+) threads, (\d+) B LDS[^\n]*\)\n"
    r"My Matmul Latency = ([0-9.e+-]+) ms  \(([0-9.]+) TFLOP/s, ([0-9.]+)% of fp32 MFMA peak\)\n\n"
    r"rocm-lib Latency\(NN\) = ([0-9.e+-]+) ms\nrocm-lib Ratio\(NN\) = ([0-9.e+-]+)%\n\n"
    r"rocm-lib Latency\(TT\) = ([0-9.e+-]+) ms\nrocm-lib Ratio\(TT\) = ([0-9.e+-]+)%\n\n"
    r"max \|C - library\| / max \|C\| on sampled rows = ([0-9.e+-]+)\n")


@pytest.mark.parametrize("relu", [False, True])
def test_output_log_fields_and_rows_against_the_oracle(oracle, dev, tmp_path, relu):
    series_file = os.path.join(str(tmp_path), "series.json")
    cmd = [sys.executable, os.path.join(ROOT, "bench.py"), "--sweep", "matmul", "--max-dim", "1024", "--seeded",
           "--dump", str(tmp_path), "--series", series_file] + (["--relu"] if relu else [])
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    blocks = BLOCK.findall(res.stdout)
    want = [(4096, 2048, 1024)] + [(d, d, d) for d in (256, 512, 768, 1024)]
    assert [(int(b[0]), int(b[1]), int(b[2])) for b in blocks] == want
    for b, (M, N, K) in zip(blocks, want):
        occ, kernel, grid, threads, lds = int(b[3]), b[4], int(b[5]), int(b[6]), int(b[7])
        mine, tflops, pct, nn, ratio_nn, tt, ratio_tt, err_lib = (float(x) for x in b[8:16])
        assert kernel.startswith("gemm_f32_") and grid >= 1 and threads in (256, 512) and 0 < lds <= 160 * 1024
        assert occ in (25, 50)                       # 2 waves per SIMD of 8, once or twice per CU
        assert 0 < mine < 5 and 0 < nn < 5 and 0 < tt < 5
        assert abs(tflops - 2.0 * M * N * K / mine / 1e9) <= 0.02 * tflops + 0.01
        assert abs(pct - 100 * tflops / 157.3) < 0.2
        assert abs(ratio_nn - 100 * nn / mine) < 0.01 * ratio_nn
        assert abs(ratio_tt - 100 * tt / mine) < 0.01 * ratio_tt
        assert err_lib < 1e-4
        # the rows the harness computed, against the oracle on the same operands
        A = inputs.uniform((M, K), sweeps.MATMUL_SEED, 0)
        B = inputs.uniform((K, N), sweeps.MATMUL_SEED, 1)
        got = np.load(os.path.join(str(tmp_path), "C_%dx%dx%d.npy" % (M, N, K)))
        ref = np.concatenate([oracle.matmul(np.ascontiguousarray(A[a:c]), B) for a, c in sweeps.row_bands(M)])
        if relu:
            ref = oracle.relu(ref)
        assert got.shape == ref.shape
        assert max(rel_err(got, ref)) < 1e-4, (M, N, K)
    # the series performance/plot.py draws (latency, throughput, ratio to peak; four methods)
    import json
    with open(series_file) as fp:
        series = json.load(fp)
    assert series["dims"] == ["4096x2048x1024", 256, 512, 768, 1024] and len(series["methods"]) == 4
    for key in ("latency_ms", "throughput_tflops", "peak_ratio_percent"):
        assert len(series[key]) == 4 and all(len(line) == 5 for line in series[key])
    for i, b in enumerate(blocks):
        assert abs(series["latency_ms"][0][i] - float(b[8])) <= 1e-5 * float(b[8]) + 1e-9
        assert abs(series["latency_ms"][1][i] - float(b[11])) <= 1e-5 * float(b[11]) + 1e-9
        assert abs(series["throughput_tflops"][0][i] - float(b[9])) < 0.02
        assert abs(series["peak_ratio_percent"][3][i] - 100.0) < 1e-9
    # the summary table carries one row per size
    assert res.stdout.count("\n| %dx%dx%d |" % want[0]) == 1 and res.stdout.count("\n| 1024x1024x1024 |") == 1


def test_chosen_sizes_with_a_workspace_against_the_oracle(oracle, dev, tmp_path):
    """`--dims` (a square size and an M x N x K one) with `--workspace`: 1152^3 runs its
    K-split plan (the log says so), 512 x 384 x 256 has none; sampled rows of both against
    the oracle on the same seeded operands."""
    cmd = [sys.executable, os.path.join(ROOT, "bench.py"), "--sweep", "matmul", "--dims", "1152,512x384x256",
           "--workspace", "--relu", "--seeded", "--dump", str(tmp_path)]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-2000:]
    blocks = BLOCK.findall(res.stdout)
    want = [(1152, 1152, 1152), (512, 384, 256)]
    assert [(int(b[0]), int(b[1]), int(b[2])) for b in blocks] == want
    assert res.stdout.count("K-split plan") == 1
    for (M, N, K) in want:
        A = inputs.uniform((M, K), sweeps.MATMUL_SEED, 0)
        B = inputs.uniform((K, N), sweeps.MATMUL_SEED, 1)
        got = np.load(os.path.join(str(tmp_path), "C_%dx%dx%d.npy" % (M, N, K)))
        ref = np.concatenate([oracle.relu(oracle.matmul(np.ascontiguousarray(A[a:c]), B)) for a, c in sweeps.row_bands(M)])
        assert max(rel_err(got, ref)) < 1e-4, (M, N, K)
