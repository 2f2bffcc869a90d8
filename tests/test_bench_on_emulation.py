"""``bench.py`` run against the CPU emulation of the kernels (tests/emu/run_bench.py): the
script's whole flow on a small batch, on a host without a GPU.  The times it prints mean
nothing there; what is checked is that it runs through, that its JSON line carries what the
benchmark contract asks for, and that the output it timed agrees with the oracle."""

import json
import os
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    if torch.cuda.is_available():
        pytest.skip("a GPU is here: bench.py itself runs on it")
    sys.path.insert(0, os.path.join(ROOT, "tests", "emu"))
    import build as emu_build

    if emu_build.compiler() is None:
        pytest.skip("no clang++ to build the emulation with")
    res = subprocess.run(
        [sys.executable, os.path.join(ROOT, "tests", "emu", "run_bench.py"), *args, "--steps", "4", "--warmup", "2", "--layers", "2", "--kv-copies", "2"],
        cwd=ROOT, capture_output=True, text=True, timeout=1200,
    )
    assert res.returncode == 0, res.stdout[-1500:] + res.stderr[-2500:]
    lines = [l for l in res.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1, res.stdout[-2000:]  # one JSON line
    return json.loads(lines[0])


def _check_contract(line, steps=4, warmup=2):
    assert line["unit"] == "us/step" and line["value"] > 0 and line["higher_is_better"] is False
    assert (line["n_gpus"], line["steps"], line["warmup"]) == (1, steps, warmup)
    assert line["vs_baseline"] is None and line["data"] == "synthetic" and "workload" in line["config"]
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s" and "traffic" in roof
    assert roof["launches_timed"] >= 1 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    cpu = line["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    return cpu


def test_decode_step_at_a_small_qwen3_4b_shape():
    line = _bench("--config", "2", "--shrink", "32", "--cpu-seqs", "8")
    cpu = _check_contract(line)
    assert line["config"]["num_seqs"] == 16 and "divided by 32" in line["config"]["workload"]
    assert line["roofline"]["kernel"] == "fca_attend32_kernel" and line["roofline"]["traffic"] is None and line["mfma_util"] is None
    assert line["breakdown_us"]["merge_kernel"] > 0 and line["breakdown_us"]["metadata_update"] > 0
    assert set(line["noncascade"]) >= {"us_per_step", "speedup_of_cascade"}
    assert cpu["max_abs_err_of_timed_output"] <= 2e-2  # the timed path's rows against the oracle, bf16 tolerance


def test_fp32_configuration():
    line = _bench("--config", "1", "--cpu-seqs", "4", "--skip-noncascade")
    cpu = _check_contract(line)
    assert line["dtype"] == "f32" and line["roofline"]["kernel"] == "fca_attend_f32_kernel"
    assert line["breakdown_us"]["merge_kernel"] is None
    assert cpu["max_abs_err_of_timed_output"] <= 2e-5
