"""Tests marked gpu, run as they are against the CPU emulation of the kernels.

``--on-emulation`` (tests/conftest.py) puts the library of tests/emu in the place of
libzorro_fca.so and lets host tensors pose as device tensors, in a process of its own.  The
test bodies, the Python host code they drive and the C ABI are the ones of the GPU run; the
kernels are the same sources compiled for the CPU.  A host without a GPU then still executes
what those tests say: a wrong argument order in a ctypes call, a tolerance that does not hold
or a misspelt name shows here and not only on the GPU box.

Here: a selection that takes about half a minute (the files of the kernels that are launched
on request or were added last: fp32, three tile buffers for fp8, sliding window and dropout in
split attention, row gather and sum).  The whole files, and the other files marked gpu except
their HIP-graph tests, run the same way:

    python -m pytest tests/test_zt_fp8_three_buffers.py ... -m gpu --on-emulation -k "not graph" -n 6
"""

import os
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

FILES = [
    "tests/test_zt_fp8_three_buffers.py",
    "tests/test_zv_split_window_dropout.py",
    "tests/test_zw_reconstruct.py",
    "tests/test_zy_fp32.py",
]
SELECTION = (
    "test_configuration_1_in_fp32 or fp32_cache_writer or fp32_tensors_are_refused or test_zw_reconstruct "
    "or through_autograd or other_caches_and_shapes or (test_zt and test_random_forests)"
)


def test_a_selection_of_the_gpu_tests_passes_on_the_emulation():
    if torch.cuda.is_available():
        pytest.skip("a GPU is here: the tests marked gpu run on it")
    sys.path.insert(0, os.path.join(ROOT, "tests", "emu"))
    import build as emu_build

    if emu_build.compiler() is None:
        pytest.skip("no clang++ to build the emulation with")
    emu_build.build()  # once, before the workers ask for it
    import importlib.util

    workers = ["-n", "4"] if importlib.util.find_spec("xdist") else []  # (one process takes about two minutes)
    res = subprocess.run(
        [sys.executable, "-m", "pytest", *FILES, "-m", "gpu", "--on-emulation", "-x", "-q", *workers, "-p", "no:cacheprovider", "-k", SELECTION],
        cwd=ROOT, capture_output=True, text=True, timeout=1500,
    )
    tail = res.stdout[-3000:] + res.stderr[-1000:]
    assert res.returncode == 0, tail
    assert " passed" in res.stdout and "skipped" not in res.stdout.splitlines()[-1], tail
