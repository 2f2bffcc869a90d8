"""Query runs: several query tokens per sequence (prefill chunks, mixed batches).

One query row per token over the sequence's block-table row; long runs are tiled by
declaring the tokens of one cache block a group, which becomes a causal node: the group
reads its KV once and every row stops at its own token.  CPU tests pin the forest oracle's
handling of declared groups by coverage invariants and hand-built cases; GPU tests
compare the kernels with the flat fp64 oracle row by row.
"""

import random

import pytest
import torch

from oracle.forest import canonical_nodes, discover_forest

BLOCK = 16


def run_rows(ctx_and_query, max_blocks, tile_min=2):
    """Row arrays of a batch given (context tokens, query tokens) per sequence: the table
    row, the causal length and the declared group of every query row.  Runs of at least
    ``tile_min`` tokens are tiled per cache block; shorter ones are left to discovery."""
    row_table, row_lens, row_group = [], [], []
    for s, (ctx, ql) in enumerate(ctx_and_query):
        for i in range(ql):
            n = ctx + i + 1
            row_table.append(s)
            row_lens.append(n)
            row_group.append(s * max_blocks + (n - 1) // BLOCK if ql >= tile_min else -1)
    return row_table, row_lens, row_group


def covered_tokens(nodes, leaves, row, row_len):
    """Token ranges a row reads through its shared nodes and its leaf, as a sorted list.  A
    causal node ends, for each member, at the member's own last token."""
    spans = []
    for n in nodes:
        if row in n["members"]:
            end = n["blk_start"] * BLOCK + n["tokens"]
            if n["parent"] >= 0:  # a node starts where its parent ends
                up = nodes[n["parent"]]
                assert row in up["members"] and n["blk_start"] == up["blk_start"] + up["num_blocks"]
            assert n["causal"] or n["tokens"] == n["num_blocks"] * BLOCK
            assert not n["causal"] or (n["num_blocks"] - 1) * BLOCK < n["tokens"] <= n["num_blocks"] * BLOCK
            spans.append((n["blk_start"] * BLOCK, min(end, row_len) if n["causal"] else end))
    leaf = leaves[row]
    spans.append((leaf["blk_start"] * BLOCK, leaf["blk_start"] * BLOCK + leaf["tokens"]))
    return sorted(spans)


def assert_exact_cover(nodes, leaves, row_lens):
    for r, n in enumerate(row_lens):
        at = 0
        for lo, hi in covered_tokens(nodes, leaves, r, n):
            if hi == lo:
                continue
            assert lo == at, f"row {r}: gap or overlap at token {at} (next span starts at {lo})"
            at = hi
        assert at == n, f"row {r}: covered {at} tokens of {n}"


def test_fresh_prefill_is_tiled_per_block():
    # one sequence, 40 prompt tokens, nothing cached: blocks 0, 1 and half of block 2
    table = [[7, 3, 9, 0]]
    row_table, row_lens, row_group = run_rows([(0, 40)], max_blocks=4)
    nodes, leaves = discover_forest(table, row_lens, row_table=row_table, row_group=row_group)
    # one causal node per block of the run, holding everything up to the tile's last token
    assert canonical_nodes(nodes) == sorted(
        [(tuple(range(0, 16)), 0, 1), (tuple(range(16, 32)), 0, 2), (tuple(range(32, 40)), 0, 3)]
    )
    assert sorted(n["tokens"] for n in nodes) == [16, 32, 40] and all(n["causal"] for n in nodes)
    assert [l["tokens"] for l in leaves] == [0] * 40
    assert_exact_cover(nodes, leaves, row_lens)


def test_chunked_prefill_continues_inside_a_block():
    # 23 tokens cached, 30 more arrive: first tile is the rest of block 1 (tokens 23..31)
    table = [[4, 5, 6, 8]]
    row_table, row_lens, row_group = run_rows([(23, 30)], max_blocks=4)
    nodes, leaves = discover_forest(table, row_lens, row_table=row_table, row_group=row_group)
    assert canonical_nodes(nodes) == sorted(
        [(tuple(range(0, 9)), 0, 2), (tuple(range(9, 25)), 0, 3), (tuple(range(25, 30)), 0, 4)]
    )
    assert sorted(n["tokens"] for n in nodes) == [32, 48, 53]
    assert_exact_cover(nodes, leaves, row_lens)


def test_declared_group_that_is_no_tile_keeps_private_leaves():
    # two sequences over one cached prompt of three blocks, declared a group by the caller
    table = [[1, 2, 3, 10], [1, 2, 3, 11]]
    nodes, leaves = discover_forest(table, [52, 60], row_table=[0, 1], row_group=[5, 5])
    assert canonical_nodes(nodes) == [((0, 1), 0, 3)] and not nodes[0]["causal"] and nodes[0]["tokens"] == 48
    assert [l["tokens"] for l in leaves] == [4, 12]
    # same rows, but the shorter one ends inside the third block: that block stays private
    nodes, leaves = discover_forest(table, [40, 60], row_table=[0, 1], row_group=[5, 5])
    assert canonical_nodes(nodes) == [((0, 1), 0, 2)]
    assert [l["tokens"] for l in leaves] == [8, 28]
    # one table row, lengths that are not successive: no tile either
    nodes, leaves = discover_forest([[1, 2, 3, 4]], [50, 52], row_table=[0, 0], row_group=[0, 0])
    assert canonical_nodes(nodes) == [((0, 1), 0, 3)] and not nodes[0]["causal"]
    assert_exact_cover(nodes, leaves, [50, 52])


def test_mixed_batch_keeps_discovery_for_single_tokens():
    # sequences 0 and 1 decode one token each over a shared two-block prompt; sequence 2 is a prefill
    table = [[1, 2, 10, 0], [1, 2, 11, 0], [20, 21, 22, 23]]
    row_table, row_lens, row_group = run_rows([(36, 1), (40, 1), (0, 50)], max_blocks=4)
    nodes, leaves = discover_forest(table, row_lens, row_table=row_table, row_group=row_group)
    got = canonical_nodes(nodes)
    assert ((0, 1), 0, 2) in got  # the decode rows share their prompt as before
    assert (tuple(range(2 + 16, 2 + 32)), 0, 2) in got and (tuple(range(2 + 48, 2 + 50)), 0, 4) in got
    assert_exact_cover(nodes, leaves, row_lens)


def test_runs_below_a_prompt_shared_between_sequences():
    # two samples of one prompt (blocks 1, 2, 3 cached and shared), each verifying three
    # speculated tokens at lengths 50..52 and 58..60; a third sequence alone
    table = [[1, 2, 3, 10], [1, 2, 3, 11], [7, 8, 9, 0]]
    row_table, row_lens, row_group = run_rows([(49, 3), (57, 3), (20, 1)], max_blocks=4)
    nodes, leaves = discover_forest(table, row_lens, row_table=row_table, row_group=row_group)
    by_members = {tuple(n["members"]): n for n in nodes}
    # all six rows read the prompt once ...
    shared = by_members[(0, 1, 2, 3, 4, 5)]
    assert (shared["blk_start"], shared["num_blocks"], shared["causal"]) == (0, 3, False)
    # ... and below it each sequence's rows form one causal tile over its fourth block
    for members, last_len in (((0, 1, 2), 52), ((3, 4, 5), 60)):
        n = by_members[members]
        assert n["causal"] and (n["blk_start"], n["num_blocks"], n["tokens"]) == (3, 1, last_len - 48)
        assert nodes[n["parent"]] is shared and n["level"] == 1
    assert len(nodes) == 3 and [l["tokens"] for l in leaves] == [0] * 6 + [21]
    assert_exact_cover(nodes, leaves, row_lens)


def test_cover_invariant_on_random_batches():
    rng = random.Random(5)
    for _ in range(30):
        nseq = rng.randint(1, 5)
        max_blocks = 12
        table = [[rng.randrange(1000) for _ in range(max_blocks)] for _ in range(nseq)]
        if nseq > 1 and rng.random() < 0.5:  # two sequences with a common cached prompt
            table[1][:3] = table[0][:3]
        batch = []
        for _ in range(nseq):
            ql = rng.choice([1, 1, 2, 15, 16, 17, 33, 60])
            ctx = rng.randint(48 if ql == 1 else 0, max_blocks * BLOCK - ql)
            batch.append((ctx, ql))
        row_table, row_lens, row_group = run_rows(batch, max_blocks, tile_min=rng.choice([2, 17]))
        for levels in (1, 4):
            nodes, leaves = discover_forest(table, row_lens, max_levels=levels, row_table=row_table, row_group=row_group)
            assert_exact_cover(nodes, leaves, row_lens)
            for n in nodes:  # the members of a node really hold the same blocks there
                ids = {tuple(table[row_table[r]][n["blk_start"] : n["blk_start"] + n["num_blocks"]]) for r in n["members"]}
                assert len(ids) == 1


def test_cpu_cascade_with_causal_nodes_equals_flat_attention():
    """The decomposition the kernels run (shared nodes, causal tiles with every member
    stopping at its own token, leaves, log-sum-exp merge), restated on the CPU in fp64,
    equals flat attention row by row."""
    from arctic_platform_amd.kv_layout import pack_blocks
    from oracle.attention import flat_decode_attention
    from oracle.cascade import cascade_decode_attention

    rng = random.Random(3)
    gen = torch.Generator().manual_seed(3)
    hq, hkv, d, max_blocks = 4, 2, 64, 6
    for trial in range(6):
        nseq = rng.randint(2, 4)
        nblocks = nseq * max_blocks
        table = torch.randperm(nblocks, generator=gen).to(torch.int32).view(nseq, max_blocks)
        if trial % 2:
            table[1, :2] = table[0, :2]  # a cached prompt shared by the first two sequences
        k = torch.randn(nblocks, BLOCK, hkv, d, generator=gen, dtype=torch.float64)
        v = torch.randn(nblocks, BLOCK, hkv, d, generator=gen, dtype=torch.float64)
        cache = pack_blocks(k, v, torch.float64)
        batch = []
        for s in range(nseq):
            ql = rng.choice([1, 2, 5, 17, 30])
            batch.append((rng.randint(32 if trial % 2 and s < 2 else 0, max_blocks * BLOCK - ql), ql))
        row_table, row_lens, row_group = run_rows(batch, max_blocks)
        q = torch.randn(len(row_table), hq, d, generator=gen, dtype=torch.float64)
        lens = torch.tensor(row_lens, dtype=torch.int32)
        ref_out, ref_lse = flat_decode_attention(q, cache, table[torch.tensor(row_table)], lens, 0.125)
        for chunk in (None, 32):
            out, lse, nodes, _ = cascade_decode_attention(
                q, cache, table, lens, 0.125, chunk_tokens=chunk, row_table=row_table, row_group=row_group
            )
            assert torch.allclose(out, ref_out, rtol=0, atol=1e-10) and torch.allclose(lse, ref_lse, rtol=0, atol=1e-10)
        assert any(n["causal"] for n in nodes) or all(ql == 1 for _, ql in batch)


# ---------------------------------------------------------------------------------- GPU


def _batch_on_gpu(gpu, seed, batch, hq, hkv, d, kv_dtype, share=()):
    """Random cache and block tables for (context, query) pairs; ``share`` lists pairs of
    sequences (a, b, blocks) whose first blocks are the same physical blocks."""
    from arctic_platform_amd.kv_layout import kv_cache_shape

    gen = torch.Generator().manual_seed(seed)
    max_blocks = max((c + q + BLOCK - 1) // BLOCK for c, q in batch) + 1
    nblocks = len(batch) * max_blocks + 3
    perm = torch.randperm(nblocks, generator=gen).to(torch.int32)
    table = perm[: len(batch) * max_blocks].view(len(batch), max_blocks).clone()
    for a, b, n in share:
        table[b, :n] = table[a, :n]
    shape = kv_cache_shape(nblocks, BLOCK, hkv, d)
    cache = torch.randn(shape, generator=gen)
    k_scale = v_scale = None
    if kv_dtype == torch.float8_e4m3fn:
        k_scale = torch.rand(hkv, generator=gen) * 0.09 + 0.01
        v_scale = torch.rand(hkv, generator=gen) * 0.09 + 0.01
        cache = (cache * 20).clamp(-448, 448)
    cache = cache.to(kv_dtype)
    rows = sum(q for _, q in batch)
    q = torch.randn(rows, hq, d, generator=gen).to(torch.bfloat16)
    dev = lambda t: None if t is None else t.to(gpu)
    return dev(table), dev(cache), dev(q), dev(k_scale), dev(v_scale), max_blocks


CASES = [
    # (seed, Hq, Hkv, D, kv dtype, rows per item, chunk, [(context, query)], shared prompts)
    (1, 8, 2, 64, torch.bfloat16, 32, 64, [(0, 1), (0, 37), (0, 300), (23, 50), (100, 1), (64, 16)], ()),
    (2, 32, 8, 128, torch.bfloat16, 64, 128, [(0, 200), (130, 70), (77, 1), (90, 1), (5, 3)], ((2, 3, 4),)),
    (3, 16, 4, 128, torch.float8_e4m3fn, 64, 256, [(0, 129), (511, 33), (40, 1)], ()),
    (4, 32, 4, 64, torch.bfloat16, 64, 32, [(16, 48), (0, 16), (15, 2)], ()),  # GQA 8: two row tiles per group
    # speculative verify: four samples of one 100-token prompt and two of another, 2 to 5 query tokens each
    (5, 32, 8, 128, torch.bfloat16, 64, 64, [(130, 4), (141, 4), (97, 5), (163, 2), (80, 3), (95, 3), (40, 1)], ((0, 1, 6), (0, 2, 6), (0, 3, 6), (4, 5, 4))),
    (6, 8, 2, 64, torch.float8_e4m3fn, 32, 32, [(130, 4), (141, 4), (97, 5), (70, 20)], ((0, 1, 6), (0, 2, 6), (0, 3, 3))),
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[f"seed{c[0]}" for c in CASES])
def test_query_runs_match_oracle(gpu, case):
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode
    from oracle.attention import flat_decode_attention
    from tests.helpers import assert_matches_oracle

    seed, hq, hkv, d, kv_dtype, rows, chunk, batch, share = case
    table, cache, q, k_scale, v_scale, max_blocks = _batch_on_gpu(gpu, seed, batch, hq, hkv, d, kv_dtype, share)
    row_table, row_lens, row_group = run_rows(batch, max_blocks)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu)
    scale = d**-0.5
    for levels in (4, 0):
        md = build_forest_metadata(
            table, i32(row_lens), num_q_heads=hq, num_kv_heads=hkv, head_dim=d, chunk_tokens=chunk, rows_per_item=rows,
            max_levels=levels, row_table=i32(row_table), row_group=i32(row_group),
        )
        out, lse = forest_cascade_decode(q, cache, md, scale, k_scale, v_scale)
        torch.cuda.synchronize()
        md.check()
        nodes, leaves = discover_forest(table.cpu().tolist(), row_lens, max_levels=levels, row_table=row_table, row_group=row_group)
        assert canonical_nodes(md.nodes()) == canonical_nodes(nodes)
        by_members = lambda ns: sorted((tuple(n["members"]), n["tokens"], n["causal"]) for n in ns)
        assert by_members(md.nodes()) == by_members(nodes)
        assert [l["tokens"] for l in md.leaves()] == [l["tokens"] for l in leaves]
        # every item addresses the block table by table row
        assert all(0 <= it["rep"] < len(batch) for it in md.items())
        ref_out, ref_lse = flat_decode_attention(
            q.cpu(), cache.cpu(), table.cpu()[torch.tensor(row_table)], torch.tensor(row_lens), scale,
            None if k_scale is None else k_scale.cpu(), None if v_scale is None else v_scale.cpu(),
        )
        assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"query runs {seed}, levels {levels}")


@pytest.mark.gpu
def test_random_batches_of_query_rows(gpu):
    """Random shapes (head size, GQA group incl. 7, tile height, fp8, chunk, level cap),
    random prefix sharing between sequences, random runs, tiles declared per block, no
    declarations, arbitrary declarations across sequences, rows in shuffled order: the node
    lists equal the oracle's and every row equals flat attention."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from arctic_platform_amd.ops import forest_cascade_decode
    from oracle.attention import flat_decode_attention
    from tests.helpers import assert_matches_oracle

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu)
    for seed in range(60):
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
            ql = min(rng.choice([1, 1, 1, 2, 3, 5, 16, 17, 33]), max_blocks * BLOCK)
            batch.append((rng.randint(0, max_blocks * BLOCK - ql), ql))
        mode = rng.choice(["tiles", "tiles", "none", "odd"])
        row_table, row_lens, row_group = run_rows(batch, max_blocks)
        if mode == "odd":  # arbitrary declarations, across sequences too
            row_group = [rng.randrange(3) for _ in row_group]
        if rng.random() < 0.3:  # rows in any order: declared tiles then are not runs of adjacent rows
            perm = list(range(len(row_table)))
            rng.shuffle(perm)
            row_table, row_lens, row_group = ([v[i] for i in perm] for v in (row_table, row_lens, row_group))
        groups = None if mode == "none" else row_group
        cache = torch.randn(kv_cache_shape(nblocks, BLOCK, hkv, d), generator=gen)
        k_scale = v_scale = None
        if fp8:
            k_scale = (torch.rand(hkv, generator=gen) * 0.09 + 0.01).to(gpu)
            v_scale = (torch.rand(hkv, generator=gen) * 0.09 + 0.01).to(gpu)
            cache = (cache * 20).clamp(-448, 448).to(torch.float8_e4m3fn).to(gpu)
        else:
            cache = cache.to(torch.bfloat16).to(gpu)
        q = torch.randn(len(row_table), hq, d, generator=gen).to(torch.bfloat16).to(gpu)
        what = f"seed {seed}: D {d}, Hq {hq} / Hkv {hkv}, rows {rows_per_item}, fp8 {fp8}, chunk {chunk}, levels {levels}, {mode}"
        md = build_forest_metadata(
            table.to(gpu), i32(row_lens), num_q_heads=hq, num_kv_heads=hkv, head_dim=d, chunk_tokens=chunk, rows_per_item=rows_per_item,
            max_levels=levels, row_table=i32(row_table), row_group=None if groups is None else i32(groups),
        )
        out, lse = forest_cascade_decode(q, cache, md, d**-0.5, k_scale, v_scale)
        torch.cuda.synchronize()
        md.check()
        nodes, leaves = discover_forest(table.tolist(), row_lens, max_levels=levels, row_table=row_table, row_group=groups)
        assert canonical_nodes(md.nodes()) == canonical_nodes(nodes), what
        key = lambda ns: sorted((tuple(sorted(n["members"])), n["tokens"], n["causal"]) for n in ns)
        assert key(md.nodes()) == key(nodes), what
        assert [l["tokens"] for l in md.leaves()] == [l["tokens"] for l in leaves], what
        ref_out, ref_lse = flat_decode_attention(
            q.cpu(), cache.cpu(), table[torch.tensor(row_table)], torch.tensor(row_lens), d**-0.5,
            None if k_scale is None else k_scale.cpu(), None if v_scale is None else v_scale.cpu(),
        )
        assert_matches_oracle(out, lse, ref_out, ref_lse, what=what)


@pytest.mark.gpu
def test_declared_groups_that_are_no_tiles(gpu):
    """Groups the caller declares across table rows (an explicit tree spec) and groups whose
    lengths do not form a run: shared node before the members' own blocks, private leaves."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode
    from oracle.attention import flat_decode_attention
    from tests.helpers import assert_matches_oracle

    hq, hkv, d = 8, 2, 64
    batch = [(50, 1), (70, 1), (90, 1), (10, 9)]
    table, cache, q, _, _, max_blocks = _batch_on_gpu(gpu, 21, batch, hq, hkv, d, torch.bfloat16, share=((0, 1, 3), (0, 2, 3)))
    row_table = [0, 1, 2] + [3] * 9
    row_lens = [51, 71, 91] + [11, 13, 12, 14, 15, 16, 17, 18, 19]  # two rows of the run swapped
    row_group = [4, 4, 4] + [9] * 9
    q = q[: len(row_table)]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu)
    md = build_forest_metadata(table, i32(row_lens), num_q_heads=hq, num_kv_heads=hkv, head_dim=d, chunk_tokens=32, row_table=i32(row_table), row_group=i32(row_group))
    out, lse = forest_cascade_decode(q, cache, md, d**-0.5)
    torch.cuda.synchronize()
    md.check()
    nodes, leaves = discover_forest(table.cpu().tolist(), row_lens, max_levels=4, row_table=row_table, row_group=row_group)
    assert canonical_nodes(md.nodes()) == canonical_nodes(nodes)
    assert ((0, 1, 2), 0, 3) in canonical_nodes(nodes) and not any(n["causal"] for n in md.nodes())
    assert [l["tokens"] for l in md.leaves()] == [l["tokens"] for l in leaves]
    ref_out, ref_lse = flat_decode_attention(q.cpu(), cache.cpu(), table.cpu()[torch.tensor(row_table)], torch.tensor(row_lens), d**-0.5)
    assert_matches_oracle(out, lse, ref_out, ref_lse, what="declared groups that are no tiles")


@pytest.mark.gpu
def test_longest_path_fills_the_partial_slots_exactly(gpu):
    """Two discovered levels, a node of a declared group below them and a leaf, every one a
    chunk of its own: the rows use every partial slot the plan reserves."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode
    from oracle.attention import flat_decode_attention
    from tests.helpers import assert_matches_oracle

    hq, hkv, d = 8, 2, 64
    batch = [(59, 1), (62, 1), (40, 1), (33, 1)]  # four single-token rows over four-block tables
    table, cache, q, _, _, max_blocks = _batch_on_gpu(gpu, 41, batch, hq, hkv, d, torch.bfloat16)
    table = table[:, :4].contiguous()
    table[1:, 0] = table[0, 0]  # everybody shares the first block,
    table[1:3, 1] = table[0, 1]  # rows 0, 1 and 2 the second,
    table[1, 2] = table[0, 2]  # rows 0 and 1 the third: one level more than discovery may take
    row_lens = [60, 63, 41, 34]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=gpu)
    md = build_forest_metadata(
        table, i32(row_lens), num_q_heads=hq, num_kv_heads=hkv, head_dim=d, chunk_tokens=1024, max_levels=2,
        row_table=i32([0, 1, 2, 3]), row_group=i32([7, 7, -1, -1]),
    )
    out, lse = forest_cascade_decode(q, cache, md, d**-0.5)
    torch.cuda.synchronize()
    md.check()
    nodes, leaves = discover_forest(table.cpu().tolist(), row_lens, max_levels=2, row_table=[0, 1, 2, 3], row_group=[7, 7, -1, -1])
    assert canonical_nodes(md.nodes()) == canonical_nodes(nodes)
    assert canonical_nodes(nodes) == sorted([((0, 1, 2, 3), 0, 1), ((0, 1, 2), 1, 1), ((0, 1), 2, 1)])
    assert [l["tokens"] for l in md.leaves()] == [12, 15, 9, 18]
    assert md.seq_num_partials()[:2] == [md.layout.max_partials] * 2 == [4, 4]
    ref_out, ref_lse = flat_decode_attention(q.cpu(), cache.cpu(), table.cpu(), torch.tensor(row_lens), d**-0.5)
    assert_matches_oracle(out, lse, ref_out, ref_lse, what="longest path")


@pytest.mark.gpu
def test_row_arrays_from_query_start_loc(gpu):
    """The device-side bookkeeping (request, causal length and tile id of every query token)
    against the plain loops of run_rows, bit for bit."""
    from arctic_platform_amd.forest import rows_from_query_runs

    rng = random.Random(9)
    for max_blocks in (7, 64):
        batch = []
        for _ in range(rng.randint(1, 40)):
            ql = rng.choice([1, 1, 1, 2, 5, 16, 17, 40])
            batch.append((rng.randint(0, max_blocks * BLOCK - ql), ql))
        want = run_rows(batch, max_blocks)
        starts = torch.tensor([0] + [q for _, q in batch]).cumsum(0).to(torch.int32).to(gpu)
        seq_lens = torch.tensor([c + q for c, q in batch], dtype=torch.int32, device=gpu)
        got = rows_from_query_runs(starts, seq_lens, len(want[0]), max_blocks)
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert g.cpu().tolist() == w


@pytest.mark.gpu
def test_query_runs_under_graph_replay(gpu):
    """Row arrays + build + attention of a mixed step captured in a HIP graph: nothing in it
    allocates or waits for the host, and every replay on changed inputs (same buffers)
    equals the eager result."""
    from arctic_platform_amd.forest import build_forest_metadata, rows_from_query_runs
    from arctic_platform_amd.ops import forest_cascade_decode

    hq, hkv, d = 16, 4, 64
    batch = [(40, 50), (100, 1), (7, 3), (64, 1), (0, 33)]
    table, cache, q, _, _, max_blocks = _batch_on_gpu(gpu, 31, batch, hq, hkv, d, torch.bfloat16, share=((1, 3, 3),))
    rows = q.shape[0]
    starts = torch.tensor([0] + [n for _, n in batch]).cumsum(0).to(torch.int32).to(gpu)
    seq_lens = torch.tensor([c + n for c, n in batch], dtype=torch.int32, device=gpu)
    kw = dict(num_q_heads=hq, num_kv_heads=hkv, head_dim=d, chunk_tokens=32, rows_per_item=64)
    bufs = tuple(torch.empty(rows, dtype=torch.int32, device=gpu) for _ in range(3))
    out = torch.empty_like(q)

    def step(md):
        rt, rl, rg = rows_from_query_runs(starts, seq_lens, rows, max_blocks, out=bufs)
        md = build_forest_metadata(table, rl, out=md, row_table=rt, row_group=rg, **kw)
        forest_cascade_decode(q, cache, md, d**-0.5, out=out, return_lse=False)
        return md

    md = step(None)  # allocates the workspaces, outside the graph
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            step(md)
    gen = torch.Generator(device=gpu).manual_seed(5)
    for replay in range(4):
        q.copy_(torch.randn(q.shape, generator=gen, device=gpu).to(q.dtype))
        if replay >= 2:  # the same runs one token further back in their sequences
            seq_lens.copy_(torch.tensor([c + n - 1 for c, n in batch], dtype=torch.int32, device=gpu))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        rt, rl, rg = rows_from_query_runs(starts, seq_lens, rows, max_blocks)
        md_e = build_forest_metadata(table, rl, row_table=rt, row_group=rg, **kw)
        want = forest_cascade_decode(q, cache, md_e, d**-0.5, return_lse=False)
        torch.cuda.synchronize()
        md_e.check()
        assert torch.equal(got, want), f"replay {replay} differs from eager"


@pytest.mark.gpu
def test_bad_row_table_is_flagged_not_followed(gpu):
    from arctic_platform_amd.forest import build_forest_metadata

    table = torch.arange(8, dtype=torch.int32, device=gpu).view(2, 4)
    lens = torch.tensor([5, 9, 20], dtype=torch.int32, device=gpu)
    rows = torch.tensor([0, 7, 1], dtype=torch.int32, device=gpu)  # 7 is not a row of the table
    md = build_forest_metadata(table, lens, num_q_heads=8, num_kv_heads=2, head_dim=64, row_table=rows)
    torch.cuda.synchronize()
    with pytest.raises(ValueError, match="row_table"):
        md.check()


@pytest.mark.gpu
def test_prefill_and_decode_through_backend(gpu):
    """A mixed step through the adapter: one sequence prefills 150 tokens, one continues a
    chunked prefill, two decode; forward() writes the new K/V and attends."""
    import types

    from arctic_platform_amd.backend import CommonAttentionMetadata, ForestCascadeAttentionBackend
    from oracle.attention import flat_decode_attention
    from tests.helpers import assert_matches_oracle

    hq, hkv, d = 16, 4, 128
    batch = [(0, 150), (70, 40), (300, 1), (33, 1)]
    table, cache, q, _, _, max_blocks = _batch_on_gpu(gpu, 11, batch, hq, hkv, d, torch.bfloat16)
    builder = ForestCascadeAttentionBackend.get_builder_cls()(hq, hkv, d, device=gpu, forest_cascade_attn_configs='{"chunk_tokens": 64}')
    impl = ForestCascadeAttentionBackend.get_impl_cls()(hq, d, d**-0.5, hkv)
    qlens = torch.tensor([b[1] for b in batch])
    starts = torch.cat([torch.zeros(1, dtype=torch.long), qlens.cumsum(0)]).to(torch.int32).to(gpu)
    seq_lens = torch.tensor([c + n for c, n in batch], dtype=torch.int32, device=gpu)
    row_table, row_lens, _ = run_rows(batch, max_blocks)
    pos = torch.tensor(row_lens) - 1
    slots = (table.cpu()[torch.tensor(row_table), pos // BLOCK].long() * BLOCK + pos % BLOCK).to(gpu)
    gen = torch.Generator().manual_seed(12)
    t = q.shape[0]
    key = torch.randn(t, hkv * d, generator=gen).to(torch.bfloat16).to(gpu)
    value = torch.randn(t, hkv * d, generator=gen).to(torch.bfloat16).to(gpu)
    meta = builder.build(0, CommonAttentionMetadata(starts, seq_lens, table, slots, num_reqs=len(batch), max_query_len=150, num_actual_tokens=t))
    out = impl.forward(types.SimpleNamespace(), q.view(t, hq * d), key, value, cache, meta)
    torch.cuda.synchronize()
    meta.forest.check()
    ref_out, ref_lse = flat_decode_attention(q.cpu(), cache.cpu(), table.cpu()[torch.tensor(row_table)], torch.tensor(row_lens), d**-0.5)
    got = out.view(t, hq, d)
    assert_matches_oracle(got, ref_lse, ref_out, ref_lse, what="mixed step through the backend")
