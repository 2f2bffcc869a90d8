"""Attention on an fp8 cache with three register tile buffers per wave (``fca_tensors.tile_buffers
= 3``, head size 128, 32-row items) on the GPU, against the CPU oracle and against the same
step on the two-buffer kernel.  The instance is launched only where a caller asks for it; its
file is collected after the tests of the kernels every caller gets."""

import random

import pytest
import torch

from arctic_platform_amd.workloads import make_config, make_forest_workload, two_level_forest
from tests.helpers import assert_matches_oracle, oracle_for
from tests.test_gpu_random_forests import random_forest

pytestmark = pytest.mark.gpu


def _run(w, fp8_tile_buffers, max_workgroups=0, reproducible=False, **kw):
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    md = build_forest_metadata(
        w.block_table, w.seq_lens, num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, **kw
    )
    md.fp8_tile_buffers, md.max_workgroups, md.reproducible = fp8_tile_buffers, max_workgroups, reproducible
    out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
    torch.cuda.synchronize()
    md.check()
    return md, out, lse


@pytest.mark.parametrize(
    "seed,hq,hkv,depth,fanout,len_range,leaf_range,chunk",
    [
        (17, 24, 4, 3, 4, (1, 150), (1, 100), 128),
        (41, 32, 8, 3, 3, (1, 400), (1, 200), 512),  # items of one to sixteen tiles: every remainder of three
        (42, 8, 8, 2, 4, (1, 260), (1, 70), 96),  # chunks of exactly one group of tiles
        (43, 64, 2, 2, 3, (30, 700), (1, 40), 1024),
    ],
)
def test_random_forests(gpu, seed, hq, hkv, depth, fanout, len_range, leaf_range, chunk):
    seg_len, paths = random_forest(random.Random(seed), depth, fanout, len_range, leaf_range)
    w = make_forest_workload(
        "random", seg_len, paths, torch.Generator().manual_seed(seed), num_q_heads=hq, num_kv_heads=hkv, head_dim=128,
        kv_dtype=torch.float8_e4m3fn, device=gpu, poison_unused=True,
    )
    ref_out, ref_lse = oracle_for(w)
    md, out, lse = _run(w, 3, chunk_tokens=chunk)
    assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"seed {seed}, three tile buffers")
    # With no item cut between two waves both kernels attend the same tiles in the same order,
    # whatever buffer a tile travels through: the same bits.
    _, out3, lse3 = _run(w, 3, reproducible=True, chunk_tokens=chunk)
    _, out2, lse2 = _run(w, 0, reproducible=True, chunk_tokens=chunk)
    assert torch.equal(out3, out2) and torch.equal(lse3, lse2)


@pytest.mark.parametrize("workgroups,chunk", [(8, 512), (8, 1024)])
def test_items_shared_by_pairs_of_waves(gpu, workgroups, chunk):
    """A small grid on the fp8 configuration: the largest items are set aside, one per pair of
    waves, and attended from both ends in groups of three tiles until the claims meet."""
    w = make_config(5, device=gpu, shrink=4, poison_unused=True)
    ref_out, ref_lse = oracle_for(w)
    md, out, lse = _run(w, 3, max_workgroups=workgroups, chunk_tokens=chunk)
    assert max(it["tok_len"] for it in md.items()) >= 10 * 32, "no item of four groups of three tiles"
    assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"C5/4, {workgroups} workgroups, three tile buffers")
    ctr = md.meta[md.layout.coop_ctr : md.layout.coop_ctr + 1024]
    assert int(ctr.abs().max()) == 0
    rows = md.plan.num_seqs * md.layout.max_partials * md.plan.num_q_heads
    scales = md.partial_lse[: 2 * rows].view(torch.int32)[1::2]
    assert int(((scales & 0x007FFFFF) != 0).sum()) > 0, "no pair of waves met on an item"
    _, out_b, lse_b = _run(w, 3, max_workgroups=workgroups, chunk_tokens=chunk)
    assert_matches_oracle(out_b, lse_b, ref_out, ref_lse, what="second launch")


def test_whole_gpu_on_long_prompts(gpu):
    """The lengths of the fp8 configuration on the whole GPU (fewer prompt groups)."""
    gen = torch.Generator().manual_seed(55)
    seg_len, paths = two_level_forest(gen, 8, 8, (1024, 4096), (1, 1024))
    w = make_forest_workload(
        "long prompts", seg_len, paths, gen, num_q_heads=32, num_kv_heads=8, head_dim=128, kv_dtype=torch.float8_e4m3fn,
        device=gpu, poison_unused=True,
    )
    md, out, lse = _run(w, 3, chunk_tokens=1024)
    assert_matches_oracle(out, lse, *oracle_for(w), what="8 x 8, three tile buffers")


def test_other_caches_and_shapes_are_not_affected(gpu):
    """The option is the metadata's; a bf16 cache, another head size or 64-row items run their own
    kernels under it, and the C ABI refuses the value where no such instance exists."""
    import ctypes

    from arctic_platform_amd import _lib

    w = make_config(2, device=gpu, shrink=16)
    md, out, lse = _run(w, 3, chunk_tokens=512)
    assert_matches_oracle(out, lse, *oracle_for(w), what="bf16 under fp8_tile_buffers")
    lib = _lib.load_library()
    kv = w.kv_cache
    t = _lib.FcaTensors(
        w.q.data_ptr(), w.q.stride(0), w.q.stride(1), kv.data_ptr(), kv.data_ptr() + kv.stride(0) * 2, kv.stride(1), kv.stride(2),
        _lib.FCA_BF16, 0, md.block_table.data_ptr(), md.block_table.stride(0), None, None, float(w.scale), 0, 0, 3,
    )
    rc = lib.fca_prefix_pass(ctypes.byref(md.plan), ctypes.byref(t), md.meta.data_ptr(), md.partial_out.data_ptr(), md.partial_lse.data_ptr(), None)
    assert rc == -2 and b"tile_buffers 3" in lib.fca_last_error()  # FCA_ERR_UNSUPPORTED


def test_decode_loop_through_the_adapter(gpu):
    """The adapter's ``fp8_tile_buffers`` key reaches the launches of a decode loop on an fp8 cache
    (three steps, every step appends a token per sequence and attends; checked against the oracle)."""
    from tests.test_backend import decode_loop

    meta = decode_loop(gpu, 5, '{"chunk_tokens": 256, "fp8_tile_buffers": 3}')
    assert meta.forest.fp8_tile_buffers == 3
