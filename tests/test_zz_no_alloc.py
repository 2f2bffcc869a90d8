"""The decode entry point that allocates nothing (``fca_decode_step_static``: partial rows
in a device array inside the library) against ``fca_decode_step`` on caller-owned
buffers, through the C ABI: same kernels, so the results must agree bit for bit."""

import ctypes

import pytest
import torch

from arctic_platform_amd.workloads import make_config

pytestmark = pytest.mark.gpu


def _both(w, chunk, rows=32):
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode, forest_cascade_decode_static

    md = build_forest_metadata(
        w.block_table, w.seq_lens, num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim,
        chunk_tokens=chunk, rows_per_item=rows,
    )
    ref_out, ref_lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
    # the caller-owned partial buffers must play no part in the static call
    md.partial_out.fill_(float("nan"))
    md.partial_lse.fill_(float("nan"))
    out = torch.full_like(ref_out, float("nan"))
    lse = torch.full_like(ref_lse, float("nan"))
    forest_cascade_decode_static(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale, out=out, lse=lse)
    torch.cuda.synchronize()
    md.check()
    return ref_out, ref_lse, out, lse


def test_static_scratch_matches_decode_step_twice(gpu):
    """Two calls in a row, the second on a smaller batch: what the first call left in the
    library's array must not reach the second call's result."""
    from tests.helpers import assert_matches_oracle, oracle_for

    big = make_config(2, device=gpu, shrink=4, poison_unused=True)
    small = make_config(1, device=gpu, dtype=torch.bfloat16, poison_unused=True)
    for w, chunk in ((big, 256), (small, 64)):
        ref_out, ref_lse, out, lse = _both(w, chunk)
        assert torch.equal(out.view(torch.int16), ref_out.view(torch.int16)), w.name
        assert torch.equal(lse.view(torch.int32), ref_lse.view(torch.int32)), w.name
        o_ref, l_ref = oracle_for(w)
        assert_matches_oracle(out, lse, o_ref, l_ref, what=f"static scratch, {w.name}")


def test_static_scratch_fp8_and_64_row_tiles(gpu):
    w = make_config(5, device=gpu, shrink=8, poison_unused=True)
    ref_out, ref_lse, out, lse = _both(w, 128, rows=64)
    assert torch.equal(out.view(torch.int16), ref_out.view(torch.int16))
    assert torch.equal(lse.view(torch.int32), ref_lse.view(torch.int32))


def test_static_scratch_refuses_plans_beyond_its_size(gpu):
    from arctic_platform_amd import _lib
    from arctic_platform_amd.forest import make_plan

    lib = _lib.load_library()
    plan = make_plan(4096, 2048, 32, 8, 128, chunk_tokens=512)
    po, pl = ctypes.c_size_t(), ctypes.c_size_t()
    _lib.check(lib.fca_workspace_bytes(ctypes.byref(plan), None, ctypes.byref(po), ctypes.byref(pl)))
    assert po.value + pl.value > _lib.FCA_STATIC_SCRATCH_BYTES
    t = _lib.FcaTensors()
    rc = lib.fca_decode_step_static(ctypes.byref(plan), ctypes.byref(t), None, None, 0, 0, 0, None, None)
    assert rc == -2 and b"static scratch" in lib.fca_last_error()
