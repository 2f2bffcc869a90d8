"""The HIP kernels on the CPU: the sources of ``csrc/`` are built against ``tests/emu/emu.h`` (a
workgroup as cooperative fibers, cross-lane operations as rendezvous, MFMA and the other
GPU-only instructions by their definition) and called through the same C ABI as the real
library, with host pointers.  Every buffer a kernel is handed ends flush against an inaccessible
page, so an access past its end stops the test with a segmentation fault, as it would raise a
memory access fault on the GPU.

This checks the logic of the kernels (work dealing, tile schedules, rings, masks, merges) and their
addresses against the same oracle as the GPU tests, on small inputs.  It does not replace those
tests: it runs none of the compiled GPU code and knows nothing of the GPU's memory model."""

import ctypes
import mmap
import os
import random
import sys

import pytest
import torch

from arctic_platform_amd import _lib
from arctic_platform_amd.forest import ForestMetadata, make_plan
from arctic_platform_amd.workloads import make_forest_workload, two_level_forest
from oracle.cache import append_kv_reference
from oracle.forest import canonical_nodes, discover_forest
from oracle.split_attention import split_attention as oracle_split
from oracle.split_attention import total_tokens
from tests.helpers import assert_matches_oracle, oracle_for
from tests.test_gpu_random_forests import CASES, random_forest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "emu"))
import build as emu_build  # noqa: E402

EMU_WORKGROUPS = 8  # fca_tensors.max_workgroups: a grid the fibers get through in seconds
_libc = ctypes.CDLL(None, use_errno=True)
_mappings = []


def guarded(t: torch.Tensor) -> torch.Tensor:
    """A copy of ``t`` whose bytes end flush against an inaccessible page and start behind one."""
    page = mmap.PAGESIZE
    t = t.contiguous()
    nbytes = t.numel() * t.element_size()
    n16 = max(16, (nbytes + 15) // 16 * 16)
    total = (n16 + page - 1) // page * page + 2 * page
    m = mmap.mmap(-1, total)
    base = ctypes.addressof(ctypes.c_char.from_buffer(m))
    assert _libc.mprotect(ctypes.c_void_p(base), ctypes.c_size_t(page), 0) == 0
    assert _libc.mprotect(ctypes.c_void_p(base + total - page), ctypes.c_size_t(page), 0) == 0
    raw = torch.frombuffer(m, dtype=torch.uint8, count=n16, offset=total - page - n16)
    g = raw[:nbytes].view(t.dtype).view(t.shape)
    g.copy_(t)
    _mappings.append(m)
    return g


@pytest.fixture(scope="module")
def emu():
    if emu_build.compiler() is None:
        pytest.skip("no clang++ to build the emulation with")
    lib = _lib.declare_signatures(ctypes.CDLL(emu_build.build()))
    lib.emu_set_dma_late.argtypes = [ctypes.c_int]
    lib.emu_set_dma_late.restype = None
    # FCA_EMU_RUN_ORDER runs the same tests with the waves of a workgroup (bit 0), the workgroups of a launch
    # (bit 1) or the lanes of a wave (bit 2) taken from the last to the first: no kernel may care
    lib.emu_set_run_order(int(os.environ.get("FCA_EMU_RUN_ORDER", "0")))
    # FCA_EMU_THREADS = n runs n workgroups of a launch at the same time on host threads of their own
    # (default: one after the other, which repeats bit for bit)
    lib.emu_set_host_threads(int(os.environ.get("FCA_EMU_THREADS", "1")))
    yield lib
    lib.emu_set_dma_late(0)


@pytest.fixture(params=[1, 8], ids=["one-after-the-other", "eight-at-a-time"])
def workgroups_at_a_time(emu, request):
    """Workgroups of a launch one after the other, or eight at a time on host threads of their own:
    then the waves of different workgroups really do draw tickets and claim tiles against each other."""
    emu.emu_set_host_threads(request.param)
    yield request.param
    emu.emu_set_host_threads(int(os.environ.get("FCA_EMU_THREADS", "1")))


def _ok(lib, rc):
    assert rc == 0, lib.fca_last_error().decode()


# ---- decode attention: builder, attention kernels, merge ---------------------------------------
# (seed, Hq, Hkv, D, kv dtype, samples per prompt, prefix range, suffix range, chunk, rows): six prompts,
# long enough for the waves of eight workgroups to end on items they share
SHARED_LAST_ITEMS = [
    (101, 24, 4, 128, torch.float8_e4m3fn, 5, (700, 2500), (40, 700), 512, 32),
    (102, 16, 4, 128, torch.bfloat16, 5, (700, 2500), (40, 700), 512, 32),
    (108, 4, 1, 64, torch.bfloat16, 16, (1000, 3000), (1, 1100), 1024, 64),  # 64-row tiles, chunks of 64 blocks
]


def _decode(lib, w, chunk, rows, max_levels=4, tile_buffers=0, reproducible=0):
    S, mb = w.block_table.shape
    plan = make_plan(S, mb, w.num_q_heads, w.num_kv_heads, w.head_dim, chunk_tokens=chunk, rows_per_item=rows, max_levels=max_levels)
    layout = _lib.FcaMetaLayout()
    _ok(lib, lib.fca_meta_describe(ctypes.byref(plan), ctypes.byref(layout)))
    nm, no, nl = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    _ok(lib, lib.fca_workspace_bytes(ctypes.byref(plan), ctypes.byref(nm), ctypes.byref(no), ctypes.byref(nl)))
    meta = guarded(torch.zeros(nm.value // 4, dtype=torch.int32))
    po = guarded(torch.full((no.value // 2,), float("nan"), dtype=torch.float16))
    pl = guarded(torch.full((nl.value // 4,), float("nan"), dtype=torch.float32))
    bt, sl = guarded(w.block_table), guarded(w.seq_lens)
    q = guarded(w.q)
    kv = guarded(w.kv_cache.view(torch.uint8)).view(w.kv_cache.dtype)
    ks = None if w.k_scale is None else guarded(w.k_scale)
    vs = None if w.v_scale is None else guarded(w.v_scale)
    _ok(lib, lib.fca_build_metadata(ctypes.byref(plan), bt.data_ptr(), bt.stride(0), sl.data_ptr(), meta.data_ptr(), None))
    md = ForestMetadata(plan=plan, layout=layout, meta=meta, partial_out=po, partial_lse=pl, block_table=bt, seq_lens=sl)
    md.check()
    esz = kv.element_size()
    t = _lib.FcaTensors(
        q.data_ptr(), q.stride(0), q.stride(1), kv.data_ptr(), kv.data_ptr() + kv.stride(0) * esz, kv.stride(1), kv.stride(2),
        _lib.FCA_FP8_E4M3 if kv.dtype == torch.float8_e4m3fn else _lib.FCA_BF16, 0, bt.data_ptr(), bt.stride(0),
        None if ks is None else ks.data_ptr(), None if vs is None else vs.data_ptr(), float(w.scale), reproducible, EMU_WORKGROUPS,
        tile_buffers,
    )
    out = guarded(torch.full((S, w.num_q_heads, w.head_dim), float("nan")).bfloat16())
    lse = guarded(torch.full((S, w.num_q_heads), float("nan"), dtype=torch.float32))
    _ok(
        lib,
        lib.fca_decode_step(
            ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), out.data_ptr(), out.stride(0),
            out.stride(1), _lib.FCA_BF16, lse.data_ptr(), None,
        ),
    )
    # the launch leaves its work ticket and its claim counters at zero for the next one
    assert int(meta[layout.header + 3]) == 0
    assert int(meta[layout.coop_ctr : layout.coop_ctr + 1024].abs().sum()) == 0
    md.emu_call = (plan, t, (q, kv, ks, vs))  # for a test that launches on the same tensors again
    return md, out, lse


def _second_partials(md):
    """Partial rows of the launch that point at a second partial, written by the other wave of a
    pair (the row's stored scale carries the pointer in its mantissa)."""
    rows = md.plan.num_seqs * md.layout.max_partials * md.plan.num_q_heads
    scales = md.partial_lse[: 2 * rows].view(torch.int32)[1::2]
    return int(((scales & 0x007FFFFF) != 0).sum())


def _check_nodes(md, w):
    nodes, leaves = discover_forest(w.block_table.tolist(), w.seq_lens.tolist(), max_levels=md.plan.max_levels)
    assert canonical_nodes(md.nodes()) == canonical_nodes(nodes)
    assert [(l["blk_start"], l["tokens"]) for l in md.leaves()] == [(l["blk_start"], l["tokens"]) for l in leaves]
    assert md.header()["unique_tokens"] == w.unique_tokens


@pytest.mark.parametrize("case", [c for c in CASES if c[0] in (2, 5, 10, 12, 15, 21, 24)], ids=lambda c: f"seed{c[0]}")
def test_random_forests_decode(emu, case):
    seed, hq, hkv, d, kv_dtype, depth, fanout, len_range, leaf_range, chunk, rows = case
    seg_len, paths = random_forest(random.Random(seed), depth, fanout, len_range, leaf_range)
    w = make_forest_workload(
        "random", seg_len, paths, torch.Generator().manual_seed(seed), num_q_heads=hq, num_kv_heads=hkv, head_dim=d,
        kv_dtype=kv_dtype, device="cpu", poison_unused=True,
    )
    md, out, lse = _decode(emu, w, chunk, rows)
    _check_nodes(md, w)
    assert_matches_oracle(out, lse, *oracle_for(w), what=f"seed {seed}")


@pytest.mark.parametrize("case", SHARED_LAST_ITEMS, ids=lambda c: f"seed{c[0]}")
def test_long_items_shared_by_two_waves(emu, case, workgroups_at_a_time):
    seed, hq, hkv, d, kv_dtype, samples, prefix_range, suffix_range, chunk, rows = case
    gen = torch.Generator().manual_seed(seed)
    seg_len, paths = two_level_forest(gen, 6, samples, prefix_range, suffix_range)
    w = make_forest_workload(
        "two-level", seg_len, paths, gen, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, kv_dtype=kv_dtype, device="cpu",
        poison_unused=True,
    )
    md, out, lse = _decode(emu, w, chunk, rows)
    # enough items for the 32-row kernel to set the largest ones aside, one per pair of waves
    if rows == 32:
        assert md.header()["items"] * hkv >= 16 + 3 * 32
        assert _second_partials(md) > 0  # some pair of waves did meet on its last item
    _check_nodes(md, w)
    ref = oracle_for(w)
    assert_matches_oracle(out, lse, *ref, what=f"seed {seed}")
    for again in range(4 if workgroups_at_a_time > 1 else 0):  # (where the claims of a pair meet differs from run to run)
        md, out, lse = _decode(emu, w, chunk, rows)
        assert_matches_oracle(out, lse, *ref, what=f"seed {seed}, run {again + 2}")


# ---- three register tile buffers for fp8 tiles at head size 128 (fca_tensors.tile_buffers = 3) -------
@pytest.mark.parametrize(
    "seed,hq,hkv,depth,fanout,len_range,leaf_range,chunk",
    [
        (17, 24, 4, 3, 4, (1, 150), (1, 100), 128),  # GQA 6: chunks of four tiles, a group and a tile
        (41, 32, 8, 3, 3, (1, 400), (1, 200), 512),  # items of one to sixteen tiles: every remainder of three
        (42, 8, 8, 2, 4, (1, 260), (1, 70), 96),  # no GQA: chunks of exactly one group
        (43, 64, 2, 2, 3, (30, 700), (1, 40), 1024),  # one member per item, items of up to 22 tiles
    ],
)
def test_three_tile_buffers_on_random_forests(emu, seed, hq, hkv, depth, fanout, len_range, leaf_range, chunk):
    seg_len, paths = random_forest(random.Random(seed), depth, fanout, len_range, leaf_range)
    w = make_forest_workload(
        "random", seg_len, paths, torch.Generator().manual_seed(seed), num_q_heads=hq, num_kv_heads=hkv, head_dim=128,
        kv_dtype=torch.float8_e4m3fn, device="cpu", poison_unused=True,
    )
    md, out, lse = _decode(emu, w, chunk, 32, tile_buffers=3)
    _check_nodes(md, w)
    assert_matches_oracle(out, lse, *oracle_for(w), what=f"seed {seed}, three tile buffers")
    # With no item cut between two waves both kernels attend the same tiles in the same order,
    # whatever buffer a tile travels through: the same bits.
    _, out3, lse3 = _decode(emu, w, chunk, 32, tile_buffers=3, reproducible=1)
    _, out2, lse2 = _decode(emu, w, chunk, 32, reproducible=1)
    assert torch.equal(out3, out2) and torch.equal(lse3, lse2)


@pytest.mark.parametrize("seed,samples,prefix_range,suffix_range,chunk", [(101, 5, (700, 2500), (40, 700), 512)])
def test_three_tile_buffers_on_items_shared_by_two_waves(emu, seed, samples, prefix_range, suffix_range, chunk, workgroups_at_a_time):
    """Last items long enough (four groups of three tiles) are attended by the two waves of a pair from
    both ends, in groups of three."""
    gen = torch.Generator().manual_seed(seed)
    seg_len, paths = two_level_forest(gen, 6, samples, prefix_range, suffix_range)
    w = make_forest_workload(
        "two-level", seg_len, paths, gen, num_q_heads=24, num_kv_heads=4, head_dim=128, kv_dtype=torch.float8_e4m3fn, device="cpu",
        poison_unused=True,
    )
    md, out, lse = _decode(emu, w, chunk, 32, tile_buffers=3)
    assert md.header()["items"] * 4 >= 16 + 3 * 32
    assert _second_partials(md) > 0  # some pair of waves did meet on its last item
    _check_nodes(md, w)
    ref = oracle_for(w)
    assert_matches_oracle(out, lse, *ref, what=f"seed {seed}, three tile buffers")
    for again in range(4 if workgroups_at_a_time > 1 else 0):  # (where the claims of a pair meet differs from run to run)
        md, out, lse = _decode(emu, w, chunk, 32, tile_buffers=3)
        assert_matches_oracle(out, lse, *ref, what=f"seed {seed}, three tile buffers, run {again + 2}")


def test_three_tile_buffers_are_refused_where_there_is_no_such_kernel(emu):
    gen = torch.Generator().manual_seed(1)
    seg_len, paths = two_level_forest(gen, 2, 2, (40, 80), (1, 30))
    for kw, rows in (
        (dict(head_dim=128, kv_dtype=torch.bfloat16), 32),
        (dict(head_dim=64, kv_dtype=torch.float8_e4m3fn), 32),
        (dict(head_dim=128, kv_dtype=torch.float8_e4m3fn), 64),
        (dict(head_dim=256, kv_dtype=torch.float8_e4m3fn), 32),
    ):
        w = make_forest_workload("small", seg_len, paths, gen, num_q_heads=8, num_kv_heads=2, device="cpu", **kw)
        with pytest.raises(AssertionError, match="tile_buffers 3"):
            _decode(emu, w, 64, rows, tile_buffers=3)
    w = make_forest_workload("small", seg_len, paths, gen, num_q_heads=8, num_kv_heads=2, head_dim=128, kv_dtype=torch.float8_e4m3fn, device="cpu")
    with pytest.raises(AssertionError, match="tile_buffers 2"):
        _decode(emu, w, 64, 32, tile_buffers=2)


def test_entry_points_agree(emu):
    """Shared and private items as launches of their own plus the merge, the decode step on the
    library's own partial buffers, sharing switched off, fp32 output into a strided tensor: all
    give the decode step's result (the first three bit for bit)."""
    seed, hq, hkv, d, kv_dtype, samples, prefix_range, suffix_range, chunk, rows = SHARED_LAST_ITEMS[1]
    gen = torch.Generator().manual_seed(seed)
    seg_len, paths = two_level_forest(gen, 3, 4, (200, 900), (10, 300))
    w = make_forest_workload("two-level", seg_len, paths, gen, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, kv_dtype=kv_dtype, device="cpu", poison_unused=True)
    md, out, lse = _decode(emu, w, 128, 32)
    S = w.block_table.shape[0]
    plan, meta = md.plan, md.meta
    q, kv, bt = guarded(w.q), guarded(w.kv_cache), md.block_table
    t = _lib.FcaTensors(
        q.data_ptr(), q.stride(0), q.stride(1), kv.data_ptr(), kv.data_ptr() + kv.stride(0) * 2, kv.stride(1), kv.stride(2), _lib.FCA_BF16, 0,
        bt.data_ptr(), bt.stride(0), None, None, float(w.scale), 0, EMU_WORKGROUPS,
    )
    fresh = lambda: (guarded(torch.full((S, hq, d), float("nan")).bfloat16()), guarded(torch.full((S, hq), float("nan"), dtype=torch.float32)))
    # 1. two passes and the merge
    po = guarded(torch.full_like(md.partial_out, float("nan")))
    pl = guarded(torch.full_like(md.partial_lse, float("nan")))
    o1, l1 = fresh()
    _ok(emu, emu.fca_prefix_pass(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), None))
    _ok(emu, emu.fca_suffix_pass(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), None))
    _ok(emu, emu.fca_merge(ctypes.byref(plan), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), o1.data_ptr(), o1.stride(0), o1.stride(1), _lib.FCA_BF16, l1.data_ptr(), None))
    assert torch.equal(o1.view(torch.int16), out.view(torch.int16)) and torch.equal(l1, lse)
    # 2. the library's own partial buffers
    o2, l2 = fresh()
    _ok(emu, emu.fca_decode_step_static(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), o2.data_ptr(), o2.stride(0), o2.stride(1), _lib.FCA_BF16, l2.data_ptr(), None))
    assert torch.equal(o2.view(torch.int16), out.view(torch.int16)) and torch.equal(l2, lse)
    # 3. fp32 output into every second row of a wider tensor
    wide = guarded(torch.full((S, 2, hq, d), float("nan"), dtype=torch.float32))
    o3 = wide[:, 1]
    _ok(emu, emu.fca_decode_step(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), o3.data_ptr(), o3.stride(0), o3.stride(1), _lib.FCA_F32, None, None))
    assert torch.isnan(wide[:, 0]).all()
    torch.testing.assert_close(o3.bfloat16().float(), out.float(), rtol=1e-2, atol=1e-2)
    # 4. sharing off: the same kernels as a plain paged decode attention
    md0, out0, lse0 = _decode(emu, w, 128, 32, max_levels=0)
    assert md0.header()["shared_items"] == 0
    assert_matches_oracle(out0, lse0, *oracle_for(w), what="sharing off")
    torch.testing.assert_close(lse0, lse, rtol=0, atol=1e-4)


def test_separate_passes_with_shared_items_equal_the_fused_step(emu):
    """Shared and private items as launches of their own, on a batch where either launch has
    enough long items for pairs of waves to attend some together: the launch over the private
    items shares none, so the second partials that the launch over the shared items left are
    still there when the merge follows them."""
    hq, hkv, d, chunk = 16, 4, 128, 256
    gen = torch.Generator().manual_seed(311)
    seg_len, paths = two_level_forest(gen, 10, 4, (400, 1200), (230, 500))
    w = make_forest_workload("two-level", seg_len, paths, gen, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, device="cpu", poison_unused=True)
    md, out, lse = _decode(emu, w, chunk, 32)
    waves = 4 * EMU_WORKGROUPS
    items = md.items()
    for shared in (True, False):
        own = [it for it in items if it["shared"] == shared]
        assert len(own) * hkv >= waves // 2 + 3 * waves, "too few items for the launch to set some aside"
        assert max(it["tok_len"] for it in own[: waves // 2 // hkv + 1]) >= 7 * 32 - 31, "no item long enough to be shared"
    S = w.block_table.shape[0]
    plan, meta, bt = md.plan, md.meta, md.block_table
    q, kv = guarded(w.q), guarded(w.kv_cache)
    t = _lib.FcaTensors(
        q.data_ptr(), q.stride(0), q.stride(1), kv.data_ptr(), kv.data_ptr() + kv.stride(0) * 2, kv.stride(1), kv.stride(2), _lib.FCA_BF16, 0,
        bt.data_ptr(), bt.stride(0), None, None, float(w.scale), 0, EMU_WORKGROUPS,
    )
    po = guarded(torch.full_like(md.partial_out, float("nan")))
    pl = guarded(torch.full_like(md.partial_lse, float("nan")))
    o1 = guarded(torch.full((S, hq, d), float("nan")).bfloat16())
    l1 = guarded(torch.full((S, hq), float("nan"), dtype=torch.float32))
    _ok(emu, emu.fca_prefix_pass(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), None))
    S_rows = S * md.layout.max_partials * hq
    back = pl.view(-1, 2)[S_rows:].clone()
    assert bool((~torch.isnan(back[:, 0])).any()), "the launch over the shared items left no second partial"
    _ok(emu, emu.fca_suffix_pass(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), None))
    assert torch.equal(pl.view(-1, 2)[S_rows:].view(torch.int32), back.view(torch.int32)), "the suffix launch wrote second partials"
    _ok(emu, emu.fca_merge(ctypes.byref(plan), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), o1.data_ptr(), o1.stride(0), o1.stride(1), _lib.FCA_BF16, l1.data_ptr(), None))
    ref_out, ref_lse = oracle_for(w)
    assert_matches_oracle(o1, l1, ref_out, ref_lse, what="prefix + suffix + merge")
    assert_matches_oracle(out, lse, ref_out, ref_lse, what="fused step")
    # where the waves of a pair meet is the one thing the launches may differ in
    torch.testing.assert_close(l1, lse, rtol=0, atol=2e-3)
    # reproducible: no item is shared, nothing is written behind the ordinary rows, and the step equals itself
    t.reproducible = 1
    res = []
    for _ in range(2):
        po.fill_(float("nan")), pl.fill_(float("nan"))
        o2 = guarded(torch.full((S, hq, d), float("nan")).bfloat16())
        l2 = guarded(torch.full((S, hq), float("nan"), dtype=torch.float32))
        _ok(emu, emu.fca_decode_step(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), o2.data_ptr(), o2.stride(0), o2.stride(1), _lib.FCA_BF16, l2.data_ptr(), None))
        assert bool(torch.isnan(pl.view(-1, 2)[S_rows:]).all())
        res.append((o2, l2))
    assert torch.equal(res[0][0].view(torch.int16), res[1][0].view(torch.int16)) and torch.equal(res[0][1], res[1][1])
    assert_matches_oracle(res[0][0], res[0][1], ref_out, ref_lse, what="reproducible step")


# ---- KV bytes requested per launch ------------------------------------------------------------------
@pytest.mark.parametrize(
    "name,forest,kv_dtype,rows,bound",
    [
        # prompts and suffixes as long as the benchmark configurations draw them (fewer groups): items of up to 32 tiles
        ("Qwen3-4B lengths", lambda g: two_level_forest(g, 4, 8, (1024, 4096), (1, 1024)), torch.bfloat16, 32, 1.13),
        ("the same with an fp8 cache", lambda g: two_level_forest(g, 4, 8, (1024, 4096), (1, 1024)), torch.float8_e4m3fn, 32, 1.13),
        ("a 16k-token prompt, 64-row tiles", lambda g: two_level_forest(g, 1, 16, (16384, 16384), (256, 2048)), torch.bfloat16, 64, 1.08),
        # three tile buffers: a refill past an item's end repeats up to two tiles, and a wave ends on three
        ("an fp8 cache, three tile buffers", lambda g: two_level_forest(g, 4, 8, (1024, 4096), (1, 1024)), torch.float8_e4m3fn, 32, 1.22),
    ],
    ids=["c2-lengths", "c5-lengths", "c3-lengths", "c5-lengths-3buf"],
)
def test_a_launch_requests_every_kv_block_about_once(emu, name, forest, kv_dtype, rows, bound):
    """The streaming kernels read their KV tiles with non-temporal loads, which the emulation counts:
    the bytes the attention launch of a decode step requests stay within a
    few per cent of the unique KV bytes of the batch (the roofline's algorithmic bytes).  What lies
    above 1 is by design: a refill past an item's end repeats its last tile so that the number of
    loads in flight never varies, a ragged last tile is fetched whole, and each wave ends on two
    tiles nobody uses.  On the GPU most of those repeats are served by the caches (the traffic
    counters read 1.04 x the unique bytes at the Qwen3-4B shape); a kernel change that read a
    shared prefix once per sample, or a tile twice, would show here as 2 x and more."""
    emu.emu_take_streamed_bytes.restype = ctypes.c_ulonglong
    gen = torch.Generator().manual_seed(7)
    seg_len, paths = forest(gen)
    w = make_forest_workload(name, seg_len, paths, gen, num_q_heads=8, num_kv_heads=2, head_dim=128, kv_dtype=kv_dtype, device="cpu")
    md, out, lse = _decode(emu, w, 1024, rows, tile_buffers=3 if "three tile buffers" in name else 0)
    assert_matches_oracle(out, lse, *oracle_for(w), what=name)
    # the attention launch once more, on its own (the merge streams the partial rows it reads back)
    plan, t, _ = md.emu_call
    emu.emu_take_streamed_bytes()
    _ok(emu, emu.fca_forest_pass(ctypes.byref(plan), ctypes.byref(t), md.meta.data_ptr(), md.partial_out.data_ptr(), md.partial_lse.data_ptr(), None))
    ratio = emu.emu_take_streamed_bytes() / w.unique_kv_bytes
    assert 1.0 <= ratio <= bound, f"{name}: {ratio:.3f} x the unique KV bytes"


# ---- the all-fp32 path --------------------------------------------------------------------------------
def _decode_f32(lib, w, chunk, max_levels=4, static=False):
    """fca_decode_step on fp32 queries and an fp32 cache; returns (metadata, out fp32, lse)."""
    S, mb = w.block_table.shape
    plan = make_plan(S, mb, w.num_q_heads, w.num_kv_heads, w.head_dim, chunk_tokens=chunk, rows_per_item=32, max_levels=max_levels)
    layout = _lib.FcaMetaLayout()
    _ok(lib, lib.fca_meta_describe(ctypes.byref(plan), ctypes.byref(layout)))
    nm, no, nl = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    _ok(lib, lib.fca_workspace_bytes_dtype(ctypes.byref(plan), _lib.FCA_F32, ctypes.byref(nm), ctypes.byref(no), ctypes.byref(nl)))
    half = ctypes.c_size_t()
    _ok(lib, lib.fca_workspace_bytes(ctypes.byref(plan), None, ctypes.byref(half), None))
    assert no.value == 2 * half.value
    meta = guarded(torch.zeros(nm.value // 4, dtype=torch.int32))
    po = guarded(torch.full((no.value // 4,), float("nan"), dtype=torch.float32))
    pl = guarded(torch.full((nl.value // 4,), float("nan"), dtype=torch.float32))
    bt, sl = guarded(w.block_table), guarded(w.seq_lens)
    q, kv = guarded(w.q), guarded(w.kv_cache)
    assert q.dtype == torch.float32 and kv.dtype == torch.float32
    _ok(lib, lib.fca_build_metadata(ctypes.byref(plan), bt.data_ptr(), bt.stride(0), sl.data_ptr(), meta.data_ptr(), None))
    md = ForestMetadata(plan=plan, layout=layout, meta=meta, partial_out=po, partial_lse=pl, block_table=bt, seq_lens=sl)
    md.check()
    t = _lib.FcaTensors(
        q.data_ptr(), q.stride(0), q.stride(1), kv.data_ptr(), kv.data_ptr() + kv.stride(0) * 4, kv.stride(1), kv.stride(2),
        _lib.FCA_F32, 0, bt.data_ptr(), bt.stride(0), None, None, float(w.scale), 0, EMU_WORKGROUPS,
    )
    out = guarded(torch.full((S, w.num_q_heads, w.head_dim), float("nan"), dtype=torch.float32))
    lse = guarded(torch.full((S, w.num_q_heads), float("nan"), dtype=torch.float32))
    if static:
        _ok(lib, lib.fca_decode_step_static(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1), _lib.FCA_F32, lse.data_ptr(), None))
    else:
        _ok(lib, lib.fca_decode_step(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1), _lib.FCA_F32, lse.data_ptr(), None))
    assert int(meta[layout.header + 3]) == 0
    # the other entry points that take tensors have no fp32 path and say so
    assert lib.fca_forest_pass(ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), None) == -2
    assert b"fca_decode_step" in lib.fca_last_error()
    return md, out, lse


def _assert_fp32_close(out, lse, w, what):
    """fp32 arithmetic on fp32 inputs against the fp64 oracle on the same inputs: 2e-5."""
    ref_out, ref_lse = oracle_for(w)
    err = (out.double() - ref_out).abs()
    assert bool((err <= 2e-5 + 2e-5 * ref_out.abs()).all()), f"{what}: out max |err| {err.max():.3g}"
    lerr = (lse.double() - ref_lse).abs().max()
    assert lerr <= 2e-5, f"{what}: lse max |err| {lerr:.3g}"


@pytest.mark.parametrize("chunk", [32, 96, 512])
def test_fp32_configuration_1(emu, chunk):
    """The small fp32 configuration as it is defined (fp32 q, K, V): outputs and log-sum-exp to
    fp32 accuracy, and the committed golden result of the fp64 oracle on the same values."""
    import numpy as np

    from arctic_platform_amd.workloads import make_config

    w = make_config(1, device="cpu", poison_unused=True)
    assert w.q.dtype == torch.float32 and w.kv_cache.dtype == torch.float32
    md, out, lse = _decode_f32(emu, w, chunk)
    _check_nodes(md, w)
    _assert_fp32_close(out, lse, w, f"C1 fp32, chunk {chunk}")
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1.npz"))
    assert float(np.abs(out.numpy() - gold["out"]).max()) <= 2e-5
    assert float(np.abs(lse.numpy() - gold["lse"]).max()) <= 2e-5


@pytest.mark.parametrize("case", [c for c in CASES if c[0] in (2, 5, 7, 12, 15)], ids=lambda c: f"seed{c[0]}")
def test_fp32_random_forests(emu, case):
    """Random forests (several levels, ragged lengths, GQA groups that do not fill a tile) in fp32,
    head sizes 64 and 128, on caller-owned partial buffers and on the library's own."""
    seed, hq, hkv, d, kv_dtype, depth, fanout, len_range, leaf_range, chunk, rows = case
    if d == 256:
        pytest.skip("the fp32 path has head sizes 64 and 128")
    seg_len, paths = random_forest(random.Random(seed), depth, fanout, len_range, leaf_range)
    w = make_forest_workload(
        "random", seg_len, paths, torch.Generator().manual_seed(seed), num_q_heads=hq, num_kv_heads=hkv, head_dim=d,
        dtype=torch.float32, device="cpu", poison_unused=True,
    )
    md, out, lse = _decode_f32(emu, w, chunk)
    _check_nodes(md, w)
    _assert_fp32_close(out, lse, w, f"seed {seed}")
    _, out2, lse2 = _decode_f32(emu, w, chunk, static=True)
    assert torch.equal(out2, out) and torch.equal(lse2, lse)
    # sharing off: the same kernel as a plain paged decode attention
    md0, out0, lse0 = _decode_f32(emu, w, chunk, max_levels=0)
    assert md0.header()["shared_items"] == 0
    _assert_fp32_close(out0, lse0, w, f"seed {seed}, sharing off")


@pytest.mark.parametrize("rows,d", [(32, 128), (64, 128), (32, 64), (32, 256)])
def test_merge_stays_inside_buffers_of_random_bits(emu, rows, d):
    """fca_merge on partial buffers nothing has written: whatever bits they hold, every load stays
    inside them (the buffers end against inaccessible pages), and a row whose scale points
    outside the rows set aside for second partials comes out as NaN."""
    hq, hkv = 8, 2
    gen = torch.Generator().manual_seed(rows + d)
    seg_len, paths = two_level_forest(gen, 3, 4, (2000, 2600), (10, 300))
    w = make_forest_workload("two-level", seg_len, paths, gen, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, device="cpu")
    S, mb = w.block_table.shape
    plan = make_plan(S, mb, hq, hkv, d, chunk_tokens=128, rows_per_item=rows, max_levels=4)
    layout = _lib.FcaMetaLayout()
    _ok(emu, emu.fca_meta_describe(ctypes.byref(plan), ctypes.byref(layout)))
    assert layout.max_partials >= 16  # the merge with several lane groups per row
    nm, no, nl = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    _ok(emu, emu.fca_workspace_bytes(ctypes.byref(plan), ctypes.byref(nm), ctypes.byref(no), ctypes.byref(nl)))
    meta = guarded(torch.zeros(nm.value // 4, dtype=torch.int32))
    bt, sl = guarded(w.block_table), guarded(w.seq_lens)
    _ok(emu, emu.fca_build_metadata(ctypes.byref(plan), bt.data_ptr(), bt.stride(0), sl.data_ptr(), meta.data_ptr(), None))
    npart = meta[layout.seq_npart : layout.seq_npart + S]
    assert int(npart.min()) >= 16
    out = guarded(torch.zeros(S, hq, d).bfloat16())
    lse = guarded(torch.zeros(S, hq, dtype=torch.float32))
    merge = lambda po, pl: _ok(emu, emu.fca_merge(ctypes.byref(plan), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1), _lib.FCA_BF16, lse.data_ptr(), None))
    # 1. random bits everywhere
    po = guarded(torch.randint(-(2**15), 2**15, (no.value // 2,), generator=gen, dtype=torch.int16))
    pl = guarded(torch.randint(-(2**31), 2**31, (nl.value // 4,), generator=gen, dtype=torch.int64).to(torch.int32))
    merge(po, pl)
    # 2. plausible values: finite log-sum-exps, and scales whose mantissa bits point anywhere in their 23 bits
    plf = pl.view(torch.float32).view(-1, 2)
    plf[:, 0] = torch.randn(plf.shape[0], generator=gen)
    scale_bits = torch.randint(0, 2**23, (plf.shape[0],), generator=gen, dtype=torch.int32) | 0x3F800000
    plf[:, 1] = scale_bits.view(torch.float32)
    po.view(torch.float16).copy_(torch.randn(po.shape[0], generator=gen).half())
    merge(po, pl)
    stray = (scale_bits & 0x7FFFFF) - 32
    back_rows = plf.shape[0] - S * layout.max_partials * hq
    assert back_rows == 32 * min(1024, (layout.max_items * hkv + 3) // 2)
    bad = ((stray < 0) & (scale_bits & 0x7FFFFF != 0)) | (stray >= back_rows)
    for s in range(S):
        for h in range(hq):
            first = (s * layout.max_partials) * hq + h
            rows_of = [first + i * hq for i in range(int(npart[s]))]
            assert bool(torch.isnan(lse[s, h])) == bool(bad[rows_of].any()), (s, h)
    # 3. a buffer of zeros (what the Python side allocates): empty rows, no NaN
    po.zero_(), pl.zero_()
    merge(po, pl)
    assert not bool(torch.isnan(out.float()).any())


# ---- query runs: rows over table rows, declared groups, causal nodes ------------------------------
def _decode_rows(lib, table, row_table, row_lens, row_group, q, cache, k_scale, v_scale, *, chunk, rows, levels):
    """Build with a row table and attend; returns (metadata, out, lse)."""
    i32 = lambda v: guarded(torch.tensor(v, dtype=torch.int32))
    hq, d = q.shape[1], q.shape[2]
    hkv = cache.shape[2]
    R = len(row_table)
    plan = make_plan(R, table.shape[1], hq, hkv, d, chunk_tokens=chunk, rows_per_item=rows, max_levels=levels)
    layout = _lib.FcaMetaLayout()
    _ok(lib, lib.fca_meta_describe(ctypes.byref(plan), ctypes.byref(layout)))
    nm, no, nl = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    _ok(lib, lib.fca_workspace_bytes(ctypes.byref(plan), ctypes.byref(nm), ctypes.byref(no), ctypes.byref(nl)))
    meta = guarded(torch.zeros(nm.value // 4, dtype=torch.int32))
    po = guarded(torch.full((no.value // 2,), float("nan"), dtype=torch.float16))
    pl = guarded(torch.full((nl.value // 4,), float("nan"), dtype=torch.float32))
    bt, rt, rl = guarded(table), i32(row_table), i32(row_lens)
    rg = None if row_group is None else i32(row_group)
    _ok(
        lib,
        lib.fca_build_metadata_rows(
            ctypes.byref(plan), bt.data_ptr(), bt.stride(0), bt.shape[0], rt.data_ptr(), None if rg is None else rg.data_ptr(),
            rl.data_ptr(), meta.data_ptr(), 0, None,
        ),
    )
    md = ForestMetadata(plan=plan, layout=layout, meta=meta, partial_out=po, partial_lse=pl, block_table=bt, seq_lens=rl, row_table=rt, row_group=rg)
    md.check()
    qg = guarded(q)
    kv = guarded(cache.view(torch.uint8)).view(cache.dtype)
    ks = None if k_scale is None else guarded(k_scale)
    vs = None if v_scale is None else guarded(v_scale)
    esz = kv.element_size()
    t = _lib.FcaTensors(
        qg.data_ptr(), qg.stride(0), qg.stride(1), kv.data_ptr(), kv.data_ptr() + kv.stride(0) * esz, kv.stride(1), kv.stride(2),
        _lib.FCA_FP8_E4M3 if kv.dtype == torch.float8_e4m3fn else _lib.FCA_BF16, 1, bt.data_ptr(), bt.stride(0),
        None if ks is None else ks.data_ptr(), None if vs is None else vs.data_ptr(), float(d**-0.5), 0, EMU_WORKGROUPS,
    )
    out = guarded(torch.full((R, hq, d), float("nan")).bfloat16())
    lse = guarded(torch.full((R, hq), float("nan"), dtype=torch.float32))
    _ok(
        lib,
        lib.fca_decode_step(
            ctypes.byref(plan), ctypes.byref(t), meta.data_ptr(), po.data_ptr(), pl.data_ptr(), out.data_ptr(), out.stride(0),
            out.stride(1), _lib.FCA_BF16, lse.data_ptr(), None,
        ),
    )
    return md, out, lse


def _check_rows(md, out, lse, table, row_table, row_lens, row_group, q, cache, k_scale, v_scale, levels, what):
    from oracle.attention import flat_decode_attention

    nodes, leaves = discover_forest(table.tolist(), row_lens, max_levels=levels, row_table=row_table, row_group=row_group)
    assert canonical_nodes(md.nodes()) == canonical_nodes(nodes), what
    key = lambda ns: sorted((tuple(sorted(n["members"])), n["tokens"], n["causal"]) for n in ns)
    assert key(md.nodes()) == key(nodes), what
    assert [l["tokens"] for l in md.leaves()] == [l["tokens"] for l in leaves], what
    ref_out, ref_lse = flat_decode_attention(
        q, cache, table[torch.tensor(row_table)], torch.tensor(row_lens), q.shape[2] ** -0.5, k_scale, v_scale
    )
    assert_matches_oracle(out, lse, ref_out, ref_lse, what=what)


def test_query_runs_and_speculative_verify(emu):
    from tests.test_query_runs import CASES as RUN_CASES
    from tests.test_query_runs import _batch_on_gpu, run_rows

    for n, (seed, hq, hkv, d, kv_dtype, rows, chunk, batch, share) in enumerate(RUN_CASES):
        table, cache, q, k_scale, v_scale, max_blocks = _batch_on_gpu("cpu", seed, batch, hq, hkv, d, kv_dtype, share)
        row_table, row_lens, row_group = run_rows(batch, max_blocks)
        for levels in (4, 0) if n % 3 == 0 else (4,):  # (sharing off on every third case)
            md, out, lse = _decode_rows(emu, table, row_table, row_lens, row_group, q, cache, k_scale, v_scale, chunk=chunk, rows=rows, levels=levels)
            _check_rows(md, out, lse, table, row_table, row_lens, row_group, q, cache, k_scale, v_scale, levels, f"query runs {seed}, levels {levels}")


def test_random_batches_of_query_rows(emu):
    """Random head sizes, GQA groups (7 among them), tile heights, fp8, chunks, level caps, prefix
    sharing between sequences, runs tiled per block, no declarations, arbitrary declarations across
    sequences, rows in shuffled order."""
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from tests.test_query_runs import run_rows

    for seed in range(25):
        rng = random.Random(seed)
        gen = torch.Generator().manual_seed(seed)
        d, hkv, g = rng.choice([64, 128]), rng.choice([1, 2, 4]), rng.choice([1, 2, 4, 7, 8, 16])
        hq, rows_per_item, fp8 = hkv * g, rng.choice([32, 64]), rng.random() < 0.3
        chunk, levels = rng.choice([32, 64, 128, 1024]), rng.choice([0, 1, 2, 4, 8])
        nseq, max_blocks = rng.randint(1, 10), rng.randint(2, 14)
        nblocks = nseq * max_blocks + 2
        table = torch.randperm(nblocks, generator=gen).to(torch.int32)[: nseq * max_blocks].view(nseq, max_blocks).clone()
        for s in range(1, nseq):  # a sequence may start with the blocks of an earlier one
            if rng.random() < 0.6:
                t, k = rng.randrange(s), rng.randint(1, max_blocks)
                table[s, :k] = table[t, :k]
        batch = []
        for s in range(nseq):
            ql = min(rng.choice([1, 1, 1, 2, 3, 5, 16, 17, 33]), max_blocks * 16)
            batch.append((rng.randint(0, max_blocks * 16 - ql), ql))
        mode = rng.choice(["tiles", "tiles", "none", "odd"])
        row_table, row_lens, row_group = run_rows(batch, max_blocks)
        if mode == "odd":  # arbitrary declarations, across sequences too
            row_group = [rng.randrange(3) for _ in row_group]
        if rng.random() < 0.3:  # rows in any order: declared tiles then are not runs of adjacent rows
            perm = list(range(len(row_table)))
            rng.shuffle(perm)
            row_table, row_lens, row_group = ([v[i] for i in perm] for v in (row_table, row_lens, row_group))
        groups = None if mode == "none" else row_group
        cache = torch.randn(kv_cache_shape(nblocks, 16, hkv, d), generator=gen)
        k_scale = v_scale = None
        if fp8:
            k_scale = torch.rand(hkv, generator=gen) * 0.09 + 0.01
            v_scale = torch.rand(hkv, generator=gen) * 0.09 + 0.01
            cache = (cache * 20).clamp(-448, 448).to(torch.float8_e4m3fn)
        else:
            cache = cache.to(torch.bfloat16)
        q = torch.randn(len(row_table), hq, d, generator=gen).to(torch.bfloat16)
        what = f"seed {seed}: D {d}, Hq {hq} / Hkv {hkv}, rows {rows_per_item}, fp8 {fp8}, chunk {chunk}, levels {levels}, {mode}"
        md, out, lse = _decode_rows(emu, table, row_table, row_lens, groups, q, cache, k_scale, v_scale, chunk=chunk, rows=rows_per_item, levels=levels)
        _check_rows(md, out, lse, table, row_table, row_lens, groups, q, cache, k_scale, v_scale, levels, what)


def test_row_arrays_from_query_start_loc(emu):
    from tests.test_query_runs import run_rows

    rng = random.Random(9)
    for max_blocks in (7, 64):
        batch = []
        for _ in range(rng.randint(1, 40)):
            ql = rng.choice([1, 1, 1, 2, 5, 16, 17, 40])
            batch.append((rng.randint(0, max_blocks * 16 - ql), ql))
        want = run_rows(batch, max_blocks)
        n = len(want[0])
        starts = guarded(torch.tensor([0] + [q for _, q in batch]).cumsum(0).to(torch.int32))
        seq_lens = guarded(torch.tensor([c + q for c, q in batch], dtype=torch.int32))
        got = [guarded(torch.full((n,), -7, dtype=torch.int32)) for _ in range(3)]
        _ok(emu, emu.fca_rows_from_query_runs(starts.data_ptr(), seq_lens.data_ptr(), len(batch), n, max_blocks, got[0].data_ptr(), got[1].data_ptr(), got[2].data_ptr(), None))
        for g, w in zip(got, want):
            assert g.tolist() == w


# ---- metadata updates between the steps of a decode loop ------------------------------------------
def test_update_keeps_the_forest_and_detects_a_changed_batch(emu):
    from arctic_platform_amd.workloads import make_config
    from tests.test_metadata_update import _grown, _semantics

    w = make_config(2, device="cpu", shrink=8)
    S = w.block_table.shape[0]
    wide = torch.zeros(S, w.block_table.shape[1] + 8, dtype=torch.int32)
    wide[:, : w.block_table.shape[1]] = w.block_table
    w.block_table = wide
    plan = make_plan(S, wide.shape[1], w.num_q_heads, w.num_kv_heads, w.head_dim, chunk_tokens=64, rows_per_item=32, max_levels=4)
    layout = _lib.FcaMetaLayout()
    _ok(emu, emu.fca_meta_describe(ctypes.byref(plan), ctypes.byref(layout)))
    nm = ctypes.c_size_t()
    _ok(emu, emu.fca_workspace_bytes(ctypes.byref(plan), ctypes.byref(nm), None, None))

    def build(bt, sl, meta=None, update=False):
        bt, sl = guarded(bt), guarded(sl)
        if meta is None:
            meta = guarded(torch.zeros(nm.value // 4, dtype=torch.int32))
        entry = emu.fca_update_metadata if update else emu.fca_build_metadata
        _ok(emu, entry(ctypes.byref(plan), bt.data_ptr(), bt.stride(0), sl.data_ptr(), meta.data_ptr(), None))
        md = ForestMetadata(plan=plan, layout=layout, meta=meta, partial_out=None, partial_lse=None, block_table=bt, seq_lens=sl)
        md.check()
        return md

    md = build(w.block_table, w.seq_lens)
    assert md.header()["updates"] == 0
    gen = torch.Generator().manual_seed(5)
    # 1 token (most rows stay inside their block), 17 (every row crosses a block), 70 (chunk counts change)
    for n, steps in enumerate((1, 17, 70)):
        bt, sl = _grown(w, steps, gen)
        md = build(bt, sl, md.meta, update=True)
        assert md.header()["updates"] == n + 1, "the update fell back to a full build"
        assert _semantics(md) == _semantics(build(bt, sl))
        w.block_table, w.seq_lens = bt, sl
    # sequence 3 leaves its group: one of its shared blocks becomes a private copy
    bt = w.block_table.clone()
    bt[3, 2] = int(bt.max()) + 1
    md = build(bt, w.seq_lens, md.meta, update=True)
    assert md.header()["updates"] == 0
    assert _semantics(md) == _semantics(build(bt, w.seq_lens))
    # a new request in an old slot: shorter than the prefix its row shared
    sl = w.seq_lens.clone()
    sl[5] = 20
    md = build(bt, sl, md.meta, update=True)
    assert md.header()["updates"] == 0
    assert _semantics(md) == _semantics(build(bt, sl))


# ---- KV-cache append and the way back -----------------------------------------------------------
@pytest.mark.parametrize("kv_dtype", [torch.bfloat16, torch.float8_e4m3fn, torch.float32])
@pytest.mark.parametrize("d", [64, 128])
def test_cache_append_and_gather(emu, kv_dtype, d):
    gen = torch.Generator().manual_seed(d)
    hkv, nblocks = 2, 9
    # a prefill run that starts off a block boundary, single decode tokens, a padding slot
    slots = list(range(21, 75)) + [3, 130, -1, 100]
    tkn = len(slots)
    rows_dtype = torch.float32 if kv_dtype == torch.float32 else torch.bfloat16  # fp32 rows go with an fp32 cache
    key = guarded((torch.randn(tkn, hkv, d, generator=gen) * 3).to(rows_dtype))
    value = guarded((torch.randn(tkn, hkv, d, generator=gen) * 3).to(rows_dtype))
    slot_mapping = guarded(torch.tensor(slots, dtype=torch.int64))
    cache0 = torch.zeros(2, nblocks, hkv, 16 * d, dtype=torch.bfloat16).to(kv_dtype)
    cache = guarded(cache0.view(torch.uint8)).view(kv_dtype)
    fp8 = kv_dtype == torch.float8_e4m3fn
    ks = guarded(torch.tensor([0.5, 2.0])) if fp8 else None
    vs = guarded(torch.tensor([1.0, 0.25])) if fp8 else None
    esz = cache.element_size()
    args = [
        key.stride(0), key.stride(1), tkn, hkv, d, slot_mapping.data_ptr(), cache.data_ptr(), cache.data_ptr() + cache.stride(0) * esz,
        cache.stride(1), cache.stride(2), {torch.bfloat16: _lib.FCA_BF16, torch.float8_e4m3fn: _lib.FCA_FP8_E4M3, torch.float32: _lib.FCA_F32}[kv_dtype],
        None if ks is None else ks.data_ptr(),
        None if vs is None else vs.data_ptr(), None,
    ]
    _ok(emu, emu.fca_append_kv(key.data_ptr(), value.data_ptr(), *args))
    want = append_kv_reference(cache0, key, value, slot_mapping, ks, vs)
    assert torch.equal(cache.view(torch.uint8), want.view(torch.uint8))
    back_k, back_v = guarded(torch.full_like(key, float("nan"))), guarded(torch.full_like(value, float("nan")))
    _ok(emu, emu.fca_gather_kv(back_k.data_ptr(), back_v.data_ptr(), *args))
    live = torch.tensor([s >= 0 for s in slots])
    assert not back_k[~live].any() and not back_v[~live].any()  # a padding slot reads as zeros
    if not fp8:
        assert torch.equal(back_k[live], key[live]) and torch.equal(back_v[live], value[live])
    else:  # what decode attention sees: the stored value times the scale
        step = torch.tensor([0.5, 2.0]).view(1, 2, 1) * 32 + 1e-3  # spacing of e4m3 below 448, times the scale
        assert ((back_k.float() - key.float()).abs()[live] <= step).all()


# ---- whole samples from a deduplicated tensor and back ----------------------------------------------
@pytest.mark.parametrize("dtype,channels", [(torch.bfloat16, 64), (torch.float32, 8), (torch.bfloat16, 2560)])
def test_row_gather_and_row_sum(emu, dtype, channels):
    """fca_gather_rows with the index of a reconstruction and of a deduplication (negative entries give
    zero rows; strided sources), and fca_sum_rows as the gradient of a reconstruction, against plain
    indexing.  Guard pages sit behind every buffer."""
    from arctic_platform_amd.reconstruct import SampleIndex
    from arctic_platform_amd.split_attention import SplitLayout
    from oracle.split_attention import deduplicate_packed, reconstruct_packed

    layout, ids = [(40, [20, 33, 7]), (7, [5]), (3, [])], [[3, 0, 2], [1], []]
    ix = SampleIndex(SplitLayout(layout, device="cpu"), ids)
    t, esz = ix.num_dedup, torch.empty((), dtype=dtype).element_size()
    gen = torch.Generator().manual_seed(channels)
    wide = guarded((torch.randn(t, 2 * channels, generator=gen) * 10).to(dtype))
    x = wide[:, channels:]  # every second half row: a strided source
    full = guarded(torch.full((ix.num_full, channels), float("nan")).to(dtype))
    index = guarded(torch.from_numpy(ix.full_from))
    _ok(emu, emu.fca_gather_rows(x.data_ptr(), x.stride(0) * esz, index.data_ptr(), ix.num_full, channels * esz, full.data_ptr(), full.stride(0) * esz, None))
    assert torch.equal(full, reconstruct_packed(x, layout, ids))
    back = guarded(torch.full((t, channels), float("nan")).to(dtype))
    index2 = guarded(torch.from_numpy(ix.dedup_from))
    _ok(emu, emu.fca_gather_rows(full.data_ptr(), full.stride(0) * esz, index2.data_ptr(), t, channels * esz, back.data_ptr(), back.stride(0) * esz, None))
    assert torch.equal(back, deduplicate_packed(full, layout, ids))
    assert not back[-3:].any()  # the prompt of the group without samples
    # the gradient of the reconstruction: every deduplicated row sums its copies
    grad_full = guarded(torch.randn(ix.num_full, channels, generator=gen).to(dtype))
    grad = guarded(torch.full((t, channels), float("nan")).to(dtype))
    offs, rows = guarded(torch.from_numpy(ix.copies_offsets)), guarded(torch.from_numpy(ix.copies_rows))
    code = _lib.FCA_F32 if dtype == torch.float32 else _lib.FCA_BF16
    _ok(emu, emu.fca_sum_rows(grad_full.data_ptr(), grad_full.stride(0) * esz, offs.data_ptr(), rows.data_ptr(), t, channels, code, grad.data_ptr(), grad.stride(0) * esz, None))
    want = torch.zeros(t, channels, dtype=torch.float64).index_add_(0, torch.from_numpy(ix.full_from).long(), grad_full.double())
    torch.testing.assert_close(grad.double(), want, rtol=1e-2 if dtype == torch.bfloat16 else 1e-6, atol=1e-2 if dtype == torch.bfloat16 else 1e-6)
    # argument checks
    assert emu.fca_gather_rows(x.data_ptr(), x.stride(0) * esz, index.data_ptr(), ix.num_full, channels * esz - 8, full.data_ptr(), full.stride(0) * esz, None) == -1
    assert emu.fca_sum_rows(grad_full.data_ptr(), grad_full.stride(0) * esz, offs.data_ptr(), rows.data_ptr(), t, channels, _lib.FCA_FP8_E4M3, grad.data_ptr(), grad.stride(0) * esz, None) == -2


# ---- split attention of the trainer --------------------------------------------------------------
def _close(name, got, ref, scale_tol):
    got, ref = got.detach().double(), ref.detach().double()
    bound = scale_tol * ref.abs().max() + 2e-2 * ref.abs() + 1e-5
    err = (got - ref).abs()
    assert bool((err <= bound).all()), f"{name}: max |err| {err.max():.4g}, largest reference {ref.abs().max():.4g}"


SPLIT_LAYOUTS = [
    [(40, [20, 3])],
    [(0, [5]), (33, [0, 64, 1])],
    [(100, [30, 30, 30, 30])],
    [(33, [32, 100, 1, 32]), (31, [17, 0, 45])],
]


@pytest.mark.parametrize("late", [False, True], ids=["loads-land-at-once", "loads-land-at-their-wait"])
# (with as many KV heads as query heads dK and dV are stored straight from the accumulators; a small batch
# with fewer KV heads forms them per query head and sums the slices)
@pytest.mark.parametrize("heads", [(8, 2, 128), (4, 1, 64), (6, 2, 64), (8, 2, 256), (2, 2, 64)], ids=lambda h: "Hq%d-Hkv%d-D%d" % h)
def test_split_attention_forward_and_backward(emu, heads, late):
    """``late``: a direct-to-LDS load lands only when a wait covers it, the latest the hardware allows
    (a missing or miscounted wait then shows as stale operands); otherwise at once, the earliest (a
    buffer refilled while it is still being read then shows)."""
    _split_cases(emu, heads, late, None)


@pytest.mark.parametrize(
    "heads,window,late",
    [((8, 2, 128), 1, False), ((8, 2, 128), 45, True), ((8, 2, 128), 200, False), ((6, 2, 64), 7, True), ((6, 2, 64), 32, False), ((4, 1, 256), 45, True)],
    ids=lambda x: "Hq%d-Hkv%d-D%d" % x if isinstance(x, tuple) else f"{x}",
)
def test_split_attention_with_a_sliding_window(emu, heads, window, late):
    """The instances for a sliding window: a row sees the last ``window`` positions of its own
    sample's sequence (the prompt's tokens, then the response's), itself included.  Windows
    shorter than a tile, of exactly a tile, across tiles, and longer than every sample."""
    _split_cases(emu, heads, late, window)


@pytest.mark.parametrize(
    "heads,window,dropout,late",
    [((8, 2, 128), None, 0.1, True), ((6, 2, 64), None, 0.5, False), ((8, 2, 128), 45, 0.25, False), ((4, 1, 256), None, 0.3, True)],
    ids=lambda x: "Hq%d-Hkv%d-D%d" % x if isinstance(x, tuple) else f"{x}",
)
def test_split_attention_with_attention_dropout(emu, heads, window, dropout, late):
    """Attention dropout in the general instances: the four kernels draw the fate of a probability
    from the same hash of (seed, query head, row, key), which the host restates for the oracle."""
    _split_cases(emu, heads, late, window, dropout)


def _split_cases(emu, heads, late, window, dropout=0.0):
    from arctic_platform_amd.split_attention import SplitLayout, dropout_keep_mask

    hq, hkv, d = heads
    emu.emu_set_dma_late(1 if late else 0)
    for ci, layout in enumerate(SPLIT_LAYOUTS):
        t = total_tokens(layout)
        g = torch.Generator().manual_seed(ci)
        q = guarded(torch.randn(t, hq, d, generator=g).bfloat16())
        k = guarded(torch.randn(t, hkv, d, generator=g).bfloat16())
        v = guarded(torch.randn(t, hkv, d, generator=g).bfloat16())
        scale = d**-0.5
        lay = guarded(torch.from_numpy(SplitLayout(layout, device="cpu", sliding_window=window).host))
        nt = (t + 31) // 32
        plan = _lib.FcaSplitPlan(t, hq, hkv, d, window or 0, dropout, 4000 + ci)
        keep = dropout_keep_mask(4000 + ci, dropout, hq, t) if dropout > 0 else None
        fwd, bwd = ctypes.c_size_t(), ctypes.c_size_t()
        _ok(emu, emu.fca_split_workspace_bytes(ctypes.byref(plan), ctypes.byref(fwd), ctypes.byref(bwd)))
        ws_f, ws_b = guarded(torch.zeros(fwd.value, dtype=torch.uint8)), guarded(torch.zeros(bwd.value, dtype=torch.uint8))
        out = guarded(torch.full((t, hq, d), float("nan")).bfloat16())
        lse = guarded(torch.full((hq, 32 * nt), float("nan"), dtype=torch.float32))
        _ok(
            emu,
            emu.fca_split_attention_forward(
                ctypes.byref(plan), q.data_ptr(), hq * d, k.data_ptr(), hkv * d, v.data_ptr(), hkv * d, lay.data_ptr(), scale,
                ws_f.data_ptr(), out.data_ptr(), hq * d, lse.data_ptr(), None,
            ),
        )
        q64, k64, v64 = (x.double().requires_grad_() for x in (q, k, v))
        ro, rl = oracle_split(q64, k64, v64, layout, scale, window=window, keep=keep, dropout=dropout)
        _close("out", out, ro, 2e-2 / max(1.0, float(ro.detach().abs().max())))
        torch.testing.assert_close(lse[:, :t].T.double(), rl.detach(), rtol=1e-3, atol=1e-3)
        dout = guarded(torch.randn(t, hq, d, generator=torch.Generator().manual_seed(ci + 1)).bfloat16())
        ro.backward(dout.double())
        dq, dk, dv = (guarded(torch.full_like(x, float("nan"))) for x in (q, k, v))
        _ok(
            emu,
            emu.fca_split_attention_backward(
                ctypes.byref(plan), q.data_ptr(), hq * d, k.data_ptr(), hkv * d, v.data_ptr(), hkv * d, out.data_ptr(), hq * d,
                dout.data_ptr(), hq * d, lse.data_ptr(), lay.data_ptr(), scale, ws_b.data_ptr(), dq.data_ptr(), hq * d,
                dk.data_ptr(), hkv * d, dv.data_ptr(), hkv * d, None,
            ),
        )
        _close("dq", dq, q64.grad, 1e-2)
        _close("dk", dk, k64.grad, 1e-2)
        _close("dv", dv, v64.grad, 1e-2)
