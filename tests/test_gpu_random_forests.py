"""Randomised forests and shapes on the GPU against the CPU oracle, plus graph replay."""

import dataclasses
import random

import pytest
import torch

from arctic_platform_amd.workloads import make_forest_workload
from oracle.forest import canonical_nodes, discover_forest
from tests.helpers import assert_matches_oracle, oracle_for

pytestmark = pytest.mark.gpu


def random_forest(rng, max_depth, fanout, len_range, leaf_range):
    """A random tree of segments; every leaf is one sequence.  Lengths are drawn so that
    shared segments end inside blocks, on block boundaries and below one block."""
    seg_len, paths = [], []

    def grow(path, depth):
        if depth == max_depth or (depth > 0 and rng.random() < 0.3):
            seg_len.append(rng.choice([0, 1, 15, 16, 17]) if rng.random() < 0.3 else rng.randint(*leaf_range))
            paths.append(path + [len(seg_len) - 1])
            return
        for _ in range(rng.randint(1, fanout)):
            seg_len.append(rng.choice([3, 16, 32, 33]) if rng.random() < 0.3 else rng.randint(*len_range))
            grow(path + [len(seg_len) - 1], depth + 1)

    grow([], 0)
    return seg_len, paths


CASES = [
    # (seed, Hq, Hkv, D, kv dtype, depth, fanout, shared len range, leaf len range, chunk, rows)
    (1, 8, 2, 64, torch.bfloat16, 3, 3, (1, 90), (1, 70), 32, 32),
    (2, 32, 8, 128, torch.bfloat16, 4, 3, (1, 200), (1, 100), 64, 32),
    (3, 16, 16, 128, torch.bfloat16, 2, 5, (20, 300), (1, 50), 128, 32),  # MHA, one row per member
    (4, 32, 4, 128, torch.bfloat16, 3, 4, (1, 150), (1, 150), 96, 64),  # GQA 8, 64-row tiles
    (5, 8, 1, 64, torch.float8_e4m3fn, 3, 3, (1, 120), (1, 90), 64, 32),  # one KV head, fp8, D 64
    (6, 32, 8, 128, torch.float8_e4m3fn, 5, 2, (1, 80), (1, 60), 32, 64),  # deep tree, fp8, 64 rows
    (7, 64, 2, 128, torch.bfloat16, 2, 3, (1, 100), (1, 40), 1024, 32),  # GQA 32: one member per 32-row tile
    (8, 4, 4, 64, torch.bfloat16, 6, 2, (1, 40), (0, 20), 32, 32),  # deeper than the default level cap
    (9, 32, 2, 64, torch.bfloat16, 3, 4, (1, 120), (1, 80), 64, 64),  # GQA 16, D 64, four members per 64-row tile
    (10, 16, 2, 64, torch.float8_e4m3fn, 4, 3, (1, 100), (1, 60), 32, 64),  # fp8, D 64, 64 rows
    # query heads per KV head that are no power of two: a tile then ends in dead rows (32 = 4 * 7 + 4)
    (11, 28, 4, 128, torch.bfloat16, 3, 4, (1, 150), (1, 100), 64, 32),  # GQA 7
    (12, 28, 4, 128, torch.float8_e4m3fn, 3, 4, (1, 150), (1, 100), 64, 64),  # GQA 7, fp8, 64 rows
    (13, 12, 4, 128, torch.bfloat16, 4, 3, (1, 120), (1, 80), 32, 64),  # GQA 3, 64 rows
    (14, 12, 4, 64, torch.float8_e4m3fn, 4, 3, (1, 120), (1, 80), 32, 32),  # GQA 3, fp8, D 64
    (15, 10, 2, 128, torch.bfloat16, 3, 5, (1, 200), (1, 60), 96, 32),  # GQA 5: six members per 32-row tile, two dead rows
    (16, 10, 2, 64, torch.bfloat16, 3, 5, (1, 200), (1, 60), 96, 64),  # GQA 5, D 64, 64 rows
    (17, 24, 4, 128, torch.float8_e4m3fn, 3, 4, (1, 150), (1, 100), 128, 32),  # GQA 6, fp8
    (18, 24, 4, 128, torch.bfloat16, 3, 4, (1, 150), (1, 100), 128, 64),  # GQA 6, 64 rows
    # more than 32 query heads per KV head: only the 64-row tiles hold a member
    (19, 64, 1, 128, torch.bfloat16, 2, 3, (1, 100), (1, 40), 64, 64),  # GQA 64: one member fills a tile
    (20, 96, 2, 64, torch.float8_e4m3fn, 3, 3, (1, 100), (1, 60), 32, 64),  # GQA 48, fp8, D 64: sixteen dead rows
    # head size 256 (the reference's in-tree Qwen3.5: configuration_qwen3_5_moe.py:35), 32-row tiles only
    (21, 16, 2, 256, torch.bfloat16, 3, 3, (1, 150), (1, 100), 64, 32),  # GQA 8
    (22, 16, 4, 256, torch.float8_e4m3fn, 3, 4, (1, 150), (1, 100), 96, 32),  # GQA 4, fp8
    (23, 4, 4, 256, torch.bfloat16, 4, 3, (1, 200), (1, 60), 1024, 32),  # MHA, one chunk per node
    (24, 32, 2, 256, torch.float8_e4m3fn, 2, 4, (1, 300), (1, 80), 128, 32),  # GQA 16: two members per tile
]


@pytest.mark.parametrize("case", CASES, ids=[f"seed{c[0]}" for c in CASES])
def test_random_forest(gpu, case):
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    seed, hq, hkv, d, kv_dtype, depth, fanout, len_range, leaf_range, chunk, rows = case
    rng = random.Random(seed)
    seg_len, paths = random_forest(rng, depth, fanout, len_range, leaf_range)
    gen = torch.Generator().manual_seed(seed)
    w = make_forest_workload("random", seg_len, paths, gen, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, kv_dtype=kv_dtype, device=gpu, poison_unused=True)
    # shuffle the rows so that group members are not adjacent
    perm = torch.randperm(w.num_seqs, generator=gen).to(gpu)
    w = dataclasses.replace(w, q=w.q[perm].contiguous(), block_table=w.block_table[perm].contiguous(), seq_lens=w.seq_lens[perm].contiguous())
    for max_levels in (4, 8):
        md = build_forest_metadata(w.block_table, w.seq_lens, num_q_heads=hq, num_kv_heads=hkv, head_dim=d, chunk_tokens=chunk, rows_per_item=rows, max_levels=max_levels)
        out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
        torch.cuda.synchronize()
        md.check()
        nodes, leaves = discover_forest(w.block_table.cpu().tolist(), w.seq_lens.cpu().tolist(), max_levels=max_levels)
        assert canonical_nodes(md.nodes()) == canonical_nodes(nodes)
        assert [l["tokens"] for l in md.leaves()] == [l["tokens"] for l in leaves]
        ref_out, ref_lse = oracle_for(w)
        empty = w.seq_lens.cpu() == 0
        if empty.any():  # a sequence without any KV: out = 0, lse = -inf by definition
            assert (out.cpu()[empty] == 0).all() and torch.isinf(lse.cpu()[empty]).all()
            keep = (~empty).nonzero().squeeze(1).tolist()
            assert_matches_oracle(out, lse, ref_out, ref_lse, seqs=keep, what=f"random forest {seed}")
        else:
            assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"random forest {seed}")


def test_many_sequences(gpu):
    """More sequences than builder threads (its scans and loops wrap) and a single group
    spanning all of them at level 0."""
    from arctic_platform_amd.workloads import three_level_forest

    gen = torch.Generator().manual_seed(9)
    seg_len, paths = three_level_forest(gen, 48, 150, 10, (1, 60), (1, 40))  # 1500 sequences
    w = make_forest_workload("many", seg_len, paths, gen, num_q_heads=8, num_kv_heads=2, head_dim=64, device=gpu)
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    md = build_forest_metadata(w.block_table, w.seq_lens, num_q_heads=8, num_kv_heads=2, head_dim=64, chunk_tokens=64, rows_per_item=64)
    out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale)
    torch.cuda.synchronize()
    md.check()
    nodes, _ = discover_forest(w.block_table.cpu().tolist(), w.seq_lens.cpu().tolist(), max_levels=4)
    assert canonical_nodes(md.nodes()) == canonical_nodes(nodes)
    assert max(len(n["members"]) for n in md.nodes()) == 1500
    sample = list(range(0, 1500, 97))
    from tests.helpers import oracle_for_sample

    ref_out, ref_lse = oracle_for_sample(w, sample)
    assert_matches_oracle(out[sample], lse[sample], ref_out, ref_lse, what="1500 sequences")


def test_graph_capture_and_replay(gpu):
    """Build + decode captured in a HIP graph: no allocation or host sync inside, and every
    replay (with fresh inputs in the same buffers) equals the eager result."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode
    from arctic_platform_amd.workloads import make_config

    w = make_config(2, device=gpu, shrink=8)
    kw = dict(num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=128)
    q = w.q.clone()
    bt, sl = w.block_table.clone(), w.seq_lens.clone()
    out = torch.empty_like(q)
    md = build_forest_metadata(bt, sl, **kw)
    forest_cascade_decode(q, w.kv_cache, md, w.scale, out=out, return_lse=False)  # warm-up outside the graph
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            build_forest_metadata(bt, sl, out=md, **kw)
            forest_cascade_decode(q, w.kv_cache, md, w.scale, out=out, return_lse=False)
    gen = torch.Generator(device=gpu).manual_seed(3)
    for replay in range(4):
        q.copy_(torch.randn(q.shape, generator=gen, device=gpu).to(q.dtype))
        if replay == 2:  # a different batch: every sequence one token shorter
            sl.copy_(w.seq_lens - 1)
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        md_e = build_forest_metadata(bt, sl, **kw)
        want = forest_cascade_decode(q, w.kv_cache, md_e, w.scale, return_lse=False)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {replay} differs from eager"


def test_empty_sequence_in_batch(gpu):
    """A row with no KV at all (length 0) between ordinary rows: out = 0, lse = -inf."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    gen = torch.Generator().manual_seed(4)
    seg_len = [40, 0, 25, 7]
    paths = [[0, 2], [1], [0, 3]]  # the middle sequence consists of one empty segment
    w = make_forest_workload("empty", seg_len, paths, gen, num_q_heads=8, num_kv_heads=2, head_dim=64, device=gpu, poison_unused=True)
    assert w.seq_lens.tolist() == [65, 0, 47]
    md = build_forest_metadata(w.block_table, w.seq_lens, num_q_heads=8, num_kv_heads=2, head_dim=64, chunk_tokens=32)
    out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale)
    torch.cuda.synchronize()
    md.check()
    assert md.seq_num_partials()[1] == 0
    assert (out[1] == 0).all() and torch.isinf(lse[1]).all() and (lse[1] < 0).all()
    ref_out, ref_lse = oracle_for(w)
    assert_matches_oracle(out, lse, ref_out, ref_lse, seqs=[0, 2], what="batch with an empty row")


@pytest.mark.parametrize("rows,dtype", [(32, torch.bfloat16), (64, torch.bfloat16), (32, torch.float8_e4m3fn)])
def test_many_small_items_drawn_from_the_counter(gpu, rows, dtype):
    """More work items than five per wavefront of the device, all tiny: the tail of the work
    list is then drawn from the counter in the metadata header, one- and two-tile items
    follow each other without a gap, and the counter must be back at zero after every
    launch so that the same metadata serves the next one."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode
    from arctic_platform_amd.workloads import three_level_forest

    gen = torch.Generator().manual_seed(21)
    # 840 sequences in 168 small groups under one root: ~1000 items x 8 KV heads
    seg_len, paths = three_level_forest(gen, 20, 168, 5, (1, 70), (1, 45))
    w = make_forest_workload("small-items", seg_len, paths, gen, num_q_heads=32, num_kv_heads=8, head_dim=128,
                             kv_dtype=dtype, device=gpu)
    kw = dict(num_q_heads=32, num_kv_heads=8, head_dim=128, chunk_tokens=32, rows_per_item=rows)
    md = build_forest_metadata(w.block_table, w.seq_lens, **kw)
    torch.cuda.synchronize()
    tickets = md.header()["items"] * 8
    waves = 4 * torch.cuda.get_device_properties(gpu).multi_processor_count
    assert tickets > 5 * waves, f"the case is meant to exceed five items per wave ({tickets} tickets, {waves} waves)"
    ref_out, ref_lse = oracle_for(w)
    first = None
    for launch in range(3):
        out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
        torch.cuda.synchronize()
        assert int(md.meta[md.layout.header + 3]) == 0, f"ticket counter not back at zero after launch {launch}"
        assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"small items, launch {launch}")
        if first is None:
            first = (out.clone(), lse.clone())
        else:
            assert torch.equal(out, first[0]) and torch.equal(lse, first[1]), "launches on one metadata differ"
    # the same under graph replay: the counter has to re-arm itself, nothing clears it
    out_g = torch.empty_like(first[0])
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale, out=out_g, return_lse=False)
    for replay in range(3):
        out_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, first[0]), f"replay {replay} differs from the eager launch"
        assert int(md.meta[md.layout.header + 3]) == 0
