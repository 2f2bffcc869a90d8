"""Runs ``bench.py`` against the CPU emulation of the kernels, in a process of its own: the
script's own flow (workload, metadata, warm-up, timed steps, breakdown, the check against the
oracle, the JSON line) with the library of this folder in the place of libzorro_fca.so.  Times
read from it mean nothing; what it shows is that the script runs and that what it prints holds
together.  usage: python tests/emu/run_bench.py <arguments of bench.py> (--device cpu is added)."""

import os
import runpy
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

from tests.conftest import _emulated_device  # noqa: E402


class _Event:
    """torch.cuda.Event for a host without a GPU: the host's clock at ``record``."""

    cuda_event = None  # (the library's launch timing takes NULL for "none")

    def __init__(self, enable_timing=False):
        self.at = 0.0

    def record(self, stream=None):
        self.at = time.perf_counter()

    def elapsed_time(self, other):
        return max((other.at - self.at) * 1e3, 1e-6)


if __name__ == "__main__":
    if torch.cuda.is_available():
        sys.exit("a GPU is here: run bench.py itself")
    _emulated_device()
    torch.cuda.Event = _Event
    sys.argv = [os.path.join(ROOT, "bench.py"), *sys.argv[1:], "--device", "cpu"]
    runpy.run_path(sys.argv[0], run_name="__main__")
