"""Split attention of the trainer at head size 256 (the reference's in-tree Qwen3.5:
arctic_platform/model/implementations/qwen35/models/qwen3_5_moe/configuration_qwen3_5_moe.py:35).
Only the kernels that share their operands through LDS have an instance of that size, one
workgroup per CU, so the query heads per KV head must be a multiple of four.

Kept in a file of its own behind the other split attention tests: these instances have been
checked by the CPU emulation (tests/test_emulated_kernels.py) and compile without scratch
(tests/test_kernel_codegen.py); this file is their test on the GPU."""

import ctypes
import random

import pytest
import torch

from arctic_platform_amd import _lib
from oracle.split_attention import total_tokens
from tests.test_split_attention import LAYOUTS, _random_layout, _run_case


def test_plans_at_head_size_256():
    lib = _lib.load_library()
    fwd, bwd = ctypes.c_size_t(), ctypes.c_size_t()
    plan = _lib.FcaSplitPlan(32 * 1024, 32, 8, 256)
    assert lib.fca_split_workspace_bytes(ctypes.byref(plan), ctypes.byref(fwd), ctypes.byref(bwd)) == 0
    assert fwd.value == 2 * (32768 * 8 * 256 * 2)
    assert bwd.value == 3 * (32768 * 8 * 256 * 2) + 4 * (32768 * 32 * 256 * 2) + 2 * 32768 * 32 * 4
    for hq, hkv in ((6, 2), (2, 2), (14, 2)):  # three, one and seven query heads per KV head
        plan = _lib.FcaSplitPlan(100, hq, hkv, 256)
        assert lib.fca_split_workspace_bytes(ctypes.byref(plan), None, None) == -2
        assert b"multiple of 4" in lib.fca_last_error()


@pytest.mark.gpu
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("heads", [(8, 2, 256), (4, 1, 256)])
def test_forward_and_backward_match_the_oracle(layout, heads):
    _run_case(layout, *heads, seed=21)


@pytest.mark.gpu
def test_random_and_smallest_layouts():
    rng = random.Random(256)
    layouts = [[(1, [0])], [(0, [1])], [(31, [1])], [(32, [1])], [(3, []), (2, [4])], [(127, [1]), (1, [127])]]
    while len(layouts) < 12:
        layout = _random_layout(rng)
        if total_tokens(layout):
            layouts.append(layout)
    for i, layout in enumerate(layouts):
        print("layout", layout, flush=True)
        _run_case(layout, 8, 2, 256, seed=i)


@pytest.mark.gpu
def test_sharp_scores_and_strided_inputs():
    _run_case([(150, [90, 40]), (64, [33])], 16, 2, 256, seed=17, q_gain=8.0)
    _run_case([(70, [40, 33, 12])], 8, 2, 256, seed=4, strided=True)
