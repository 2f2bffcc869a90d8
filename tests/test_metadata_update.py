"""Length-only updates of the forest metadata (the next step of a running decode loop)
against fresh builds and the CPU oracle."""

import pytest
import torch

from arctic_platform_amd.workloads import make_config
from tests.helpers import assert_matches_oracle, oracle_for

pytestmark = pytest.mark.gpu


def _semantics(md):
    """What a metadata workspace means, independent of the order of its arrays."""
    nodes = sorted((tuple(n["members"]), n["rep"], n["blk_start"], n["num_blocks"], n["level"], n["ord"]) for n in md.nodes())
    leaves = [(l["blk_start"], l["tokens"]) for l in md.leaves()]
    items = sorted((i["rep"], i["blk_start"], i["tok_len"], tuple(i["members"]), i["ord"], i["shared"]) for i in md.items())
    h = md.header()
    return nodes, leaves, items, md.seq_num_partials(), (h["items"], h["shared_items"], h["shared_nodes"], h["unique_tokens"], h["levels"])


def _grown(w, steps, gen):
    """Block table and lengths after every sequence has decoded `steps` more tokens: new
    private blocks are taken from ids no row uses yet."""
    bt, sl = w.block_table.clone(), w.seq_lens.clone()
    next_free = int(bt.max()) + 1
    for s in range(bt.shape[0]):
        old, new = int(sl[s]), int(sl[s]) + steps
        for b in range((old + 15) // 16, (new + 15) // 16):
            bt[s, b] = next_free
            next_free += 1
        sl[s] = new
    return bt, sl


@pytest.mark.parametrize("index,rows", [(2, 32), (4, 32), (3, 64)])
def test_update_equals_fresh_build(gpu, index, rows):
    from arctic_platform_amd.forest import build_forest_metadata

    w = make_config(index, device=gpu, shrink=8)
    kw = dict(num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=64, rows_per_item=rows)
    # room for growth in the table
    wide = torch.zeros(w.block_table.shape[0], w.block_table.shape[1] + 8, dtype=torch.int32, device=gpu)
    wide[:, : w.block_table.shape[1]] = w.block_table
    w.block_table = wide
    md = build_forest_metadata(w.block_table, w.seq_lens, **kw)
    torch.cuda.synchronize()
    assert md.header()["updates"] == 0
    gen = torch.Generator().manual_seed(5)
    # 1 token (most rows stay inside their block), 17 (every row crosses a block), 70 (chunk counts change)
    for n, steps in enumerate((1, 17, 70)):
        bt, sl = _grown(w, steps, gen)
        md = build_forest_metadata(bt, sl, out=md, update=True, **kw)
        fresh = build_forest_metadata(bt, sl, **kw)
        torch.cuda.synchronize()
        md.check()
        assert md.header()["updates"] == n + 1, "the update fell back to a full build"
        assert _semantics(md) == _semantics(fresh)
        w.block_table, w.seq_lens = bt, sl


def test_update_detects_a_changed_batch(gpu):
    """A row whose shared blocks changed, a sequence shorter than its shared prefix, another
    plan: each is found on the device and answered with a full build."""
    from arctic_platform_amd.forest import build_forest_metadata

    w = make_config(2, device=gpu, shrink=8)
    kw = dict(num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=64)
    md = build_forest_metadata(w.block_table, w.seq_lens, **kw)
    md = build_forest_metadata(w.block_table, w.seq_lens, out=md, update=True, **kw)
    torch.cuda.synchronize()
    assert md.header()["updates"] == 1

    # sequence 3 leaves its group: one of its shared blocks becomes a private copy
    bt = w.block_table.clone()
    bt[3, 2] = int(bt.max()) + 1
    md = build_forest_metadata(bt, w.seq_lens, out=md, update=True, **kw)
    fresh = build_forest_metadata(bt, w.seq_lens, **kw)
    torch.cuda.synchronize()
    assert md.header()["updates"] == 0
    assert _semantics(md) == _semantics(fresh)
    assert all(n["blk_start"] + n["num_blocks"] <= 2 for n in md.nodes() if 3 in n["members"])

    # a slot reused by a short new request: shorter than the shared prefix of the old one
    sl = w.seq_lens.clone()
    sl[5] = 20
    md = build_forest_metadata(bt, sl, out=md, update=True, **kw)
    fresh = build_forest_metadata(bt, sl, **kw)
    torch.cuda.synchronize()
    assert md.header()["updates"] == 0
    assert _semantics(md) == _semantics(fresh)

    # a slot reused by a new request that is shorter than its predecessor but longer than the
    # predecessor's shared prefix: still a full build (the newcomer may share more)
    sl1 = sl.clone()
    sl1[7] = int(sl[7]) - 1
    md = build_forest_metadata(bt, sl1, out=md, update=True, **kw)
    torch.cuda.synchronize()
    assert md.header()["updates"] == 0
    md = build_forest_metadata(bt, sl1, out=md, update=True, **kw)
    torch.cuda.synchronize()
    assert md.header()["updates"] == 1
    sl = sl1

    # bad length: the full build flags it
    sl2 = sl.clone()
    sl2[0] = -4
    md = build_forest_metadata(bt, sl2, out=md, update=True, **kw)
    torch.cuda.synchronize()
    with pytest.raises(ValueError):
        md.check()


@pytest.mark.parametrize("index", [2, 5])
def test_decode_loop_with_updates(gpu, index):
    """Five decode steps: append the step's K/V, update the metadata, attend; every step is
    checked against the oracle on the cache as it then stands."""
    from arctic_platform_amd.cache import append_kv
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    w = make_config(index, device=gpu, shrink=8)
    kw = dict(num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=128)
    S = w.num_seqs
    wide = torch.zeros(S, w.block_table.shape[1] + 2, dtype=torch.int32, device=gpu)
    wide[:, : w.block_table.shape[1]] = w.block_table
    # spare physical blocks for the new tokens
    spare = torch.zeros(2, S * 2, *w.kv_cache.shape[2:], dtype=torch.uint8 if w.kv_cache.dtype != torch.bfloat16 else torch.bfloat16, device=gpu).view(w.kv_cache.dtype)
    first_spare = w.kv_cache.shape[1]
    w.kv_cache = torch.cat([w.kv_cache, spare], dim=1).contiguous()
    w.block_table = wide
    md = build_forest_metadata(w.block_table, w.seq_lens, **kw)
    gen = torch.Generator(device=gpu).manual_seed(11)
    next_free = first_spare
    for step in range(5):
        lens = w.seq_lens.cpu()
        slots = torch.empty(S, dtype=torch.int64)
        for s in range(S):
            pos = int(lens[s])
            if pos % 16 == 0:
                w.block_table[s, pos // 16] = next_free
                next_free += 1
            slots[s] = int(w.block_table[s, pos // 16]) * 16 + pos % 16
        k = torch.randn(S, w.num_kv_heads, w.head_dim, generator=gen, device=gpu).to(torch.bfloat16)
        v = torch.randn(S, w.num_kv_heads, w.head_dim, generator=gen, device=gpu).to(torch.bfloat16)
        if w.k_scale is not None:
            k, v = k * 0.05, v * 0.05
        append_kv(k, v, w.kv_cache, slots.to(gpu), w.k_scale, w.v_scale)
        w.seq_lens = w.seq_lens + 1
        w.q = torch.randn(w.q.shape, generator=gen, device=gpu).to(w.q.dtype)
        md = build_forest_metadata(w.block_table, w.seq_lens, out=md, update=True, **kw)
        out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
        torch.cuda.synchronize()
        md.check()
        assert md.header()["updates"] == step + 1
        ref_out, ref_lse = oracle_for(w)
        assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"decode step {step}")


def test_update_with_a_row_table_and_none_with_declared_groups(gpu):
    """Query rows over a row table keep their forest across an update like plain rows (the
    fingerprints follow the row table).  The kept forest may share less than a fresh build
    would (two rows of one sequence gain a common block when they cross a block boundary),
    so the check is the attention result.  A build with declared groups leaves nothing to
    keep, so an update on it is a full build with the same result."""
    import dataclasses

    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    w = make_config(2, device=gpu, shrink=8)
    kw = dict(num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=64, rows_per_item=64)
    S = w.num_seqs
    # two query rows per sequence: the sequence without its last token, and all of it
    row_table = torch.arange(S, device=gpu).repeat_interleave(2).to(torch.int32)
    lens = torch.stack([w.seq_lens - 1, w.seq_lens], 1).reshape(-1).contiguous()
    lens = (lens - 2).clamp_(min=1).contiguous()  # start two tokens back, then step forward
    q = torch.randn(2 * S, w.num_q_heads, w.head_dim, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(gpu)
    md = build_forest_metadata(w.block_table, lens, row_table=row_table, **kw)
    for n in range(2):
        lens = (lens + 1).contiguous()  # the next step: both rows one token further
        md = build_forest_metadata(w.block_table.clone(), lens, out=md, update=True, row_table=row_table, **kw)  # (the table may move; ids stay)
        out, lse = forest_cascade_decode(q, w.kv_cache, md, w.scale)
        torch.cuda.synchronize()
        md.check()
        assert md.header()["updates"] == n + 1, "the update fell back to a full build"
        rows = dataclasses.replace(w, q=q, block_table=w.block_table[row_table.long()], seq_lens=lens)
        ref_out, ref_lse = oracle_for(rows)
        assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"row-table update {n}")
    groups = (row_table * w.block_table.shape[1] + (lens - 1) // 16).to(torch.int32)
    md2 = build_forest_metadata(w.block_table, lens, row_table=row_table, row_group=groups, **kw)
    again = build_forest_metadata(w.block_table, lens, out=md2, update=True, row_table=row_table, row_group=groups, **kw)
    fresh = build_forest_metadata(w.block_table, lens, row_table=row_table, row_group=groups, **kw)
    torch.cuda.synchronize()
    again.check()
    assert again.header()["updates"] == 0 and _semantics(again) == _semantics(fresh)
    assert any(n["causal"] for n in again.nodes())
