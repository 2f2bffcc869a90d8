"""Attention-backend surface: set-up checks on the CPU, a decode loop on the GPU."""

import types

import pytest
import torch

from arctic_platform_amd.backend import (
    CommonAttentionMetadata,
    ForestCascadeAttentionBackend,
    ForestCascadeAttentionImpl,
    ForestCascadeMetadataBuilder,
    parse_forest_cascade_configs,
)


def test_backend_surface():
    b = ForestCascadeAttentionBackend
    assert b.get_name() == "FOREST_CASCADE_ATTN"
    assert b.get_kv_cache_shape(100, 16, 8, 128) == (2, 100, 8, 2048)
    with pytest.raises(ValueError):
        b.get_kv_cache_shape(100, 32, 8, 128)
    assert b.get_impl_cls() is ForestCascadeAttentionImpl and b.get_builder_cls() is ForestCascadeMetadataBuilder


def test_default_chunk_follows_the_head_size():
    """1024-token chunks; 512 at head size 256, whose work list is short (two KV heads) and whose
    kernel holds one tile buffer; a configured value wins."""
    cls = ForestCascadeAttentionBackend.get_builder_cls()
    assert cls(32, 8, 128, device="cpu").chunk_tokens == 1024
    assert cls(16, 2, 256, device="cpu").chunk_tokens == 512
    assert cls(16, 2, 256, device="cpu", forest_cascade_attn_configs='{"chunk_tokens": 2048}').chunk_tokens == 2048
    assert cls(32, 8, 128, device="cpu").fp8_tile_buffers == 0
    assert cls(32, 8, 128, device="cpu", forest_cascade_attn_configs='{"fp8_tile_buffers": 3}').fp8_tile_buffers == 3
    with pytest.raises(ValueError, match="fp8_tile_buffers"):
        cls(32, 8, 128, device="cpu", forest_cascade_attn_configs='{"fp8_tile_buffers": 2}')


def test_config_string_and_rejections():
    assert parse_forest_cascade_configs("{}") == {} and parse_forest_cascade_configs(None) == {}
    assert parse_forest_cascade_configs('{"chunk_tokens": 512}') == {"chunk_tokens": 512}
    assert parse_forest_cascade_configs('{"kv_reread": true}') == {"kv_reread": True}
    assert ForestCascadeMetadataBuilder(32, 8, 128, device="cpu", forest_cascade_attn_configs={"kv_reread": False}).kv_reread is False
    assert ForestCascadeMetadataBuilder(32, 8, 128, device="cpu").kv_reread is None
    with pytest.raises(ValueError):
        parse_forest_cascade_configs({"bogus": 1})
    with pytest.raises(NotImplementedError):
        ForestCascadeAttentionImpl(32, 128, 0.088, 8, sliding_window=4096)
    with pytest.raises(ValueError):
        ForestCascadeAttentionImpl(32, 96, 0.1, 8)
    with pytest.raises(ValueError):
        ForestCascadeMetadataBuilder(30, 8, 128, device="cpu")
    builder = ForestCascadeMetadataBuilder(32, 8, 128, device="cpu", forest_cascade_attn_configs="{}")
    meta = CommonAttentionMetadata(None, None, None, None, num_reqs=4, max_query_len=0)
    with pytest.raises(ValueError, match="max_query_len"):
        builder.build(0, meta)
    assert builder.reproducible is False
    assert ForestCascadeMetadataBuilder(32, 8, 128, device="cpu", forest_cascade_attn_configs='{"reproducible": true}').reproducible is True


def test_query_runs_need_the_token_count_from_the_host():
    """A step with query runs sizes its row arrays by the number of query tokens; that number comes
    from the host side (num_actual_tokens, or the engine's host copy of query_start_loc), never from
    reading the device tensor back."""
    builder = ForestCascadeMetadataBuilder(32, 8, 128, device="cpu")
    starts = torch.tensor([0, 3, 5], dtype=torch.int32)
    lens = torch.tensor([40, 50], dtype=torch.int32)
    table = torch.zeros(2, 8, dtype=torch.int32)
    meta = CommonAttentionMetadata(starts, lens, table, torch.zeros(5, dtype=torch.int64), num_reqs=2, max_query_len=3)
    with pytest.raises(ValueError, match="num_actual_tokens"):
        builder.build(0, meta)


def test_workspace_cache_is_bounded():
    b = ForestCascadeMetadataBuilder(32, 8, 128, device="cpu")
    for shape in range(3 * b.MAX_KEPT_WORKSPACES):
        b._steps_since_build[shape] = 0
        b._keep(shape, object())
    assert len(b._workspaces) == b.MAX_KEPT_WORKSPACES and len(b._steps_since_build) == b.MAX_KEPT_WORKSPACES
    assert list(b._workspaces)[0] == 2 * b.MAX_KEPT_WORKSPACES  # the oldest went first


def test_workspace_cache_is_bounded_by_bytes():
    from arctic_platform_amd.forest import ForestMetadata

    b = ForestCascadeMetadataBuilder(32, 8, 128, device="cpu")
    b.MAX_KEPT_BYTES = 3000

    def fake(n):
        return ForestMetadata(None, None, torch.zeros(n, dtype=torch.int32), torch.zeros(0), torch.zeros(0), None, None)

    for i in range(5):
        b._keep(i, fake(250))  # 1000 bytes each
    assert list(b._workspaces) == [2, 3, 4]
    b._keep("big", fake(5000))  # beyond the cap on its own: everything else goes, it stays
    assert list(b._workspaces) == ["big"]


def test_prompt_layouts_never_evict_forest_workspaces(monkeypatch):
    import arctic_platform_amd.backend as backend

    b = ForestCascadeMetadataBuilder(8, 2, 128, device="cpu")
    b._keep("decode-shape", object())
    for n in range(300, 300 + 3 * b.MAX_KEPT_LAYOUTS):
        starts = torch.tensor([0, n], dtype=torch.int32)
        lens = torch.tensor([n], dtype=torch.int32)
        common = CommonAttentionMetadata(
            starts, lens, torch.zeros(1, 64, dtype=torch.int32), torch.zeros(n, dtype=torch.int64), num_reqs=1, max_query_len=n,
            num_actual_tokens=n, query_start_loc_cpu=starts, seq_lens_cpu=lens,
        )
        assert b.build(0, common).fresh_prefill is not None
    assert "decode-shape" in b._workspaces and len(b._layouts) == b.MAX_KEPT_LAYOUTS


def test_cached_prompt_layout_follows_the_number_of_decodes_in_front(monkeypatch):
    """Two steps with the same (query, context) lengths of their prompts but a different
    number of decode requests in front: the cache slots of the context must come from the
    prompt's own block-table row both times."""
    import arctic_platform_amd.backend as backend

    monkeypatch.setattr(backend, "build_forest_metadata", lambda *a, **k: None)
    monkeypatch.setattr(backend, "rows_from_query_runs", lambda *a, **k: (None, None, None))
    b = ForestCascadeMetadataBuilder(8, 2, 128, device="cpu")
    max_blocks = 128
    table = torch.arange(2 * max_blocks, dtype=torch.int32).view(2, max_blocks)

    def step(q_lens, s_lens):
        n = len(q_lens)
        starts = torch.tensor([0] + q_lens, dtype=torch.int32).cumsum(0).to(torch.int32)
        lens = torch.tensor(s_lens, dtype=torch.int32)
        common = CommonAttentionMetadata(
            starts, lens, table[:n], torch.zeros(sum(q_lens), dtype=torch.int64), num_reqs=n, max_query_len=max(q_lens),
            num_actual_tokens=sum(q_lens), query_start_loc_cpu=starts, seq_lens_cpu=lens,
        )
        return b.build(0, common)

    for q_lens, s_lens in (([512], [1536]), ([1, 512], [40, 1536]), ([512], [1536])):
        meta = step(q_lens, s_lens)
        first = len(q_lens) - 1
        assert meta.fresh_start == sum(q_lens[:first])
        pos = torch.arange(1536)
        want = table[first, pos // 16].long() * 16 + pos % 16
        assert torch.equal(meta.context_slots, want), q_lens
    assert len(b._layouts) == 1  # one layout served all three steps


def test_lengths_beyond_the_block_table_are_refused_on_the_host():
    b = ForestCascadeMetadataBuilder(8, 2, 128, device="cpu")
    starts = torch.tensor([0, 1, 2], dtype=torch.int32)
    table = torch.zeros(2, 4, dtype=torch.int32)
    for lens in ([10, 65], [-1, 5]):
        lens = torch.tensor(lens, dtype=torch.int32)
        common = CommonAttentionMetadata(
            starts, lens, table, torch.zeros(2, dtype=torch.int64), num_reqs=2, max_query_len=1,
            query_start_loc_cpu=starts, seq_lens_cpu=lens,
        )
        with pytest.raises(ValueError, match="seq_lens must lie in"):
            b.build(0, common)
    lens = torch.tensor([10, 20], dtype=torch.int32)
    starts = torch.tensor([0, 11, 12], dtype=torch.int32)
    common = CommonAttentionMetadata(
        starts, lens, table, torch.zeros(12, dtype=torch.int64), num_reqs=2, max_query_len=11,
        query_start_loc_cpu=starts, seq_lens_cpu=lens,
    )
    with pytest.raises(ValueError, match="query length"):
        b.build(0, common)


@pytest.mark.gpu
@pytest.mark.parametrize("index", [2, 5])
def test_decode_loop_through_backend(gpu, index):
    """Three decode steps: every step appends one token per sequence through forward()
    and attends; outputs are checked against the oracle on the cache as written."""
    decode_loop(gpu, index, '{"chunk_tokens": 128}')


def decode_loop(gpu, index, configs):
    from arctic_platform_amd.workloads import make_config
    from tests.helpers import assert_matches_oracle, oracle_for
    import dataclasses

    w = make_config(index, device=gpu, shrink=8)
    hq, hkv, d = w.num_q_heads, w.num_kv_heads, w.head_dim
    builder = ForestCascadeAttentionBackend.get_builder_cls()(hq, hkv, d, device=gpu, forest_cascade_attn_configs=configs)
    impl = ForestCascadeAttentionBackend.get_impl_cls()(hq, d, w.scale, hkv, kv_cache_dtype="fp8" if index == 5 else "auto")
    layer = types.SimpleNamespace(k_scale=w.k_scale, v_scale=w.v_scale)
    # room for growth: spare blocks of the pool become the next private blocks
    used = set(w.block_table.flatten().tolist())
    spare = [b for b in range(w.kv_cache.shape[1]) if b not in used]
    table = torch.cat([w.block_table, torch.zeros(w.num_seqs, 1, dtype=torch.int32, device=gpu)], 1).contiguous()
    lens = w.seq_lens.clone()
    gen = torch.Generator(device=gpu).manual_seed(8)
    workspace = None
    for step in range(3):
        lens += 1
        pos = (lens - 1).long()
        need_new = (pos % 16 == 0).nonzero().squeeze(1).tolist()
        for s in need_new:
            if pos[s] // 16 < table.shape[1] and spare:
                table[s, pos[s] // 16] = spare.pop()
        slots = table.gather(1, (pos // 16)[:, None]).squeeze(1).long() * 16 + pos % 16
        qkv = torch.randn(w.num_seqs, (hq + 2 * hkv) * d, generator=gen, device=gpu).to(torch.bfloat16)
        q, k, v = qkv.split([hq * d, hkv * d, hkv * d], dim=1)
        common = CommonAttentionMetadata(
            query_start_loc=torch.arange(w.num_seqs + 1, dtype=torch.int32, device=gpu),
            seq_lens=lens,
            block_table_tensor=table,
            slot_mapping=slots,
            num_reqs=w.num_seqs,
            max_query_len=1,
        )
        meta = builder.build(0, common)
        if workspace is None:
            workspace = meta.forest.meta.data_ptr()
        assert meta.forest.meta.data_ptr() == workspace, "metadata workspace was reallocated"
        out = torch.empty(w.num_seqs, hq * d, dtype=torch.bfloat16, device=gpu)
        res = impl.forward(layer, q.contiguous(), k.contiguous(), v.contiguous(), w.kv_cache, meta, output=out)
        torch.cuda.synchronize()
        meta.forest.check()
        assert res.data_ptr() == out.data_ptr()
        now = dataclasses.replace(w, q=q.reshape(w.num_seqs, hq, d), block_table=table, seq_lens=lens)
        ref_out, ref_lse = oracle_for(now)
        lse = torch.zeros(w.num_seqs, hq, device=gpu)  # forward() returns no lse; compare outputs only
        assert_matches_oracle(out.view(w.num_seqs, hq, d), ref_lse.float(), ref_out, ref_lse, what=f"C{index} step {step}")
        assert meta.forest.header()["shared_nodes"] == 8
        assert meta.forest.header()["updates"] == step, "steps after the first are length-only updates"
    return meta


@pytest.mark.gpu
@pytest.mark.parametrize("q_lens_kind", ["uniform3", "mixed"])
def test_several_query_tokens_per_sequence(gpu, q_lens_kind):
    """The verify step of speculative decoding: a sequence brings several query tokens, each
    seeing the cache up to and including itself.  The adapter turns every query token into a
    row of its own over the sequence's block table; outputs are checked against the oracle
    run on exactly those rows."""
    from arctic_platform_amd.workloads import make_config
    from tests.helpers import assert_matches_oracle, oracle_for
    import dataclasses

    w = make_config(2, device=gpu, shrink=8)
    hq, hkv, d = w.num_q_heads, w.num_kv_heads, w.head_dim
    builder = ForestCascadeAttentionBackend.get_builder_cls()(hq, hkv, d, device=gpu, forest_cascade_attn_configs='{"chunk_tokens": 128}')
    impl = ForestCascadeAttentionBackend.get_impl_cls()(hq, d, w.scale, hkv)
    gen = torch.Generator().manual_seed(4)
    S = w.num_seqs
    if q_lens_kind == "uniform3":
        q_lens = torch.full((S,), 3, dtype=torch.int64)
    else:
        q_lens = torch.randint(1, 6, (S,), generator=gen)
    q_lens = torch.minimum(q_lens, w.seq_lens.cpu().long())  # a sequence cannot bring more tokens than it has
    starts = torch.cat([torch.zeros(1, dtype=torch.int64), q_lens.cumsum(0)])
    T = int(starts[-1])
    q = torch.randn(T, hq * d, generator=gen).to(torch.bfloat16).to(gpu)
    common = CommonAttentionMetadata(
        query_start_loc=starts.to(torch.int32).to(gpu),
        seq_lens=w.seq_lens,
        block_table_tensor=w.block_table,
        slot_mapping=torch.zeros(T, dtype=torch.int64, device=gpu),
        num_reqs=S,
        max_query_len=int(q_lens.max()),
        num_actual_tokens=T,
    )
    layer = types.SimpleNamespace(k_scale=None, v_scale=None)
    for step in range(2):  # the second call builds into the same workspace
        meta = builder.build(0, common)
        out = impl.forward(layer, q, None, None, w.kv_cache, meta)
        torch.cuda.synchronize()
        meta.forest.check()
        # (steps with query runs are always full builds: their rows move on with every step)
        assert meta.forest.header()["updates"] == 0
        # the oracle on one row per query token
        req = torch.repeat_interleave(torch.arange(S), q_lens)
        ahead = starts[1:][req] - 1 - torch.arange(T)
        rows = dataclasses.replace(
            w,
            q=q.view(T, hq, d),
            block_table=w.block_table[req.to(gpu)],
            seq_lens=(w.seq_lens.cpu().long()[req] - ahead).to(torch.int32).to(gpu),
        )
        ref_out, ref_lse = oracle_for(rows)
        assert_matches_oracle(out.view(T, hq, d), ref_lse.float(), ref_out, ref_lse, what=f"{q_lens_kind} step {step}")
    # below the prompt nodes, the query tokens of a sequence form causal tiles over its
    # private blocks: more shared nodes than groups, and no row has a leaf of its own
    nodes = meta.forest.nodes()
    assert len(nodes) > 8 and any(n["causal"] for n in nodes) and any(not n["causal"] for n in nodes)
    tiled = {r for n in nodes if n["causal"] for r in n["members"]}
    assert all(leaf["tokens"] == 0 for r, leaf in enumerate(meta.forest.leaves()) if r in tiled)



@pytest.mark.gpu
def test_fresh_prompts_take_the_split_attention_kernels(gpu):
    """A step that brings only fresh prompts (no cached context) and host copies of the
    lengths: the adapter attends straight from the step's K and V on the split-attention
    kernels, still fills the cache, and a following decode step reads it.  With a cached
    context, or without the host copies, the same call goes the query-run way."""
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from oracle.attention import flat_decode_attention

    hq, hkv, d = 8, 2, 128
    scale = d**-0.5
    lens = [300, 77, 512]
    T, S = sum(lens), len(lens)
    gen = torch.Generator().manual_seed(9)
    max_blocks = 40
    table = torch.randperm(S * max_blocks, generator=gen).to(torch.int32).view(S, max_blocks).to(gpu)
    cache = torch.zeros(kv_cache_shape(S * max_blocks, 16, hkv, d), dtype=torch.bfloat16, device=gpu)
    q, k, v = (torch.randn(T, h * d, generator=gen).to(torch.bfloat16).to(gpu) for h in (hq, hkv, hkv))
    starts = torch.tensor([0] + lens).cumsum(0)
    seq = torch.repeat_interleave(torch.arange(S), torch.tensor(lens))
    pos = torch.cat([torch.arange(n) for n in lens])
    slots = (table.cpu().long()[seq, pos // 16] * 16 + pos % 16).to(gpu)
    builder = ForestCascadeAttentionBackend.get_builder_cls()(hq, hkv, d, device=gpu)
    impl = ForestCascadeAttentionBackend.get_impl_cls()(hq, d, scale, hkv)
    layer = types.SimpleNamespace(k_scale=None, v_scale=None)
    common = CommonAttentionMetadata(
        query_start_loc=starts.to(torch.int32).to(gpu), seq_lens=torch.tensor(lens, dtype=torch.int32, device=gpu),
        block_table_tensor=table, slot_mapping=slots, num_reqs=S, max_query_len=max(lens), num_actual_tokens=T,
        query_start_loc_cpu=starts.to(torch.int32), seq_lens_cpu=torch.tensor(lens, dtype=torch.int32),
    )
    meta = builder.build(0, common)
    assert meta.fresh_prefill is not None and meta.forest is None
    out = impl.forward(layer, q, k, v, cache, meta)
    # the oracle reads the cache the call has just filled: one row per token, cut off behind it
    ref, _ = flat_decode_attention(
        q.view(T, hq, d).cpu(), cache.cpu(), table.cpu()[seq], (pos + 1).to(torch.int32), scale, dtype=torch.float32
    )
    torch.testing.assert_close(out.view(T, hq, d).cpu().float(), ref, rtol=2e-2, atol=2e-2)
    assert builder.build(0, common).fresh_prefill is meta.fresh_prefill  # the layout is kept with the workspaces
    # the query-run way on the same step (no host copies): same rows
    import dataclasses
    slow = builder.build(0, dataclasses.replace(common, query_start_loc_cpu=None, seq_lens_cpu=None))
    assert slow.fresh_prefill is None
    out2 = impl.forward(layer, q, None, None, cache, slow)
    torch.testing.assert_close(out2.view(T, hq, d).cpu().float(), ref, rtol=2e-2, atol=2e-2)
    # a cached context in front of the last sequence: no fresh prompts at the end of the batch
    # (a chunk behind a context only joins them when it is long; ruled out here)
    builder.CONTEXT_PREFILL_MIN_QUERY = 10**9
    longer = dataclasses.replace(common, seq_lens_cpu=torch.tensor([lens[0], lens[1], lens[2] + 16], dtype=torch.int32))
    assert builder.build(0, longer).fresh_prefill is None
    # in front of the first one: the two behind it are still taken as fresh prompts
    longer = dataclasses.replace(common, seq_lens_cpu=torch.tensor([lens[0] + 16, lens[1], lens[2]], dtype=torch.int32))
    assert builder.build(0, longer).fresh_start == lens[0]


@pytest.mark.gpu
def test_decodes_followed_by_fresh_prompts_in_one_step(gpu):
    """The usual serving step: running sequences bring one token each, and two new prompts
    arrive behind them.  The decodes go through the forest, the prompts through the
    split-attention kernels, every row is checked against the oracle on the filled cache."""
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from oracle.attention import flat_decode_attention

    hq, hkv, d = 8, 2, 128
    scale = d**-0.5
    gen = torch.Generator().manual_seed(21)
    context = [70, 33, 128, 5, 200, 64]  # tokens already cached of the running sequences
    q_lens = [1] * len(context) + [300, 150]
    s_lens = [c + 1 for c in context] + [300, 150]
    S, T = len(q_lens), sum(q_lens)
    max_blocks = 24
    table = torch.randperm(S * max_blocks, generator=gen).to(torch.int32).view(S, max_blocks).to(gpu)
    cache = torch.randn(kv_cache_shape(S * max_blocks, 16, hkv, d), generator=gen).to(torch.bfloat16).to(gpu)
    q, k, v = (torch.randn(T, h * d, generator=gen).to(torch.bfloat16).to(gpu) for h in (hq, hkv, hkv))
    starts = torch.tensor([0] + q_lens).cumsum(0)
    seq = torch.repeat_interleave(torch.arange(S), torch.tensor(q_lens))
    pos = torch.cat([torch.arange(s - n, s) for n, s in zip(q_lens, s_lens)])
    slots = (table.cpu().long()[seq, pos // 16] * 16 + pos % 16).to(gpu)
    builder = ForestCascadeAttentionBackend.get_builder_cls()(hq, hkv, d, device=gpu)
    impl = ForestCascadeAttentionBackend.get_impl_cls()(hq, d, scale, hkv)
    layer = types.SimpleNamespace(k_scale=None, v_scale=None)
    common = CommonAttentionMetadata(
        query_start_loc=starts.to(torch.int32).to(gpu), seq_lens=torch.tensor(s_lens, dtype=torch.int32, device=gpu),
        block_table_tensor=table, slot_mapping=slots, num_reqs=S, max_query_len=max(q_lens), num_actual_tokens=T,
        query_start_loc_cpu=starts.to(torch.int32), seq_lens_cpu=torch.tensor(s_lens, dtype=torch.int32),
    )
    meta = builder.build(0, common)
    assert meta.fresh_prefill is not None and meta.fresh_start == len(context) and meta.forest is not None
    assert meta.forest.plan.num_seqs == len(context)
    out = impl.forward(layer, q, k, v, cache, meta)
    torch.cuda.synchronize()
    meta.forest.check()
    ref, _ = flat_decode_attention(
        q.view(T, hq, d).cpu(), cache.cpu(), table.cpu()[seq], (pos + 1).to(torch.int32), scale, dtype=torch.float32
    )
    torch.testing.assert_close(out.view(T, hq, d).cpu().float(), ref, rtol=2e-2, atol=2e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("kv_dtype", [torch.bfloat16, torch.float8_e4m3fn])
def test_long_chunk_behind_a_cached_context(gpu, kv_dtype):
    """Decodes, then a long prefill chunk whose sequence already has 130 tokens in the cache
    (a cached prefix or an earlier chunk), then a fresh prompt: the two prompts attend on the
    split-attention kernels with K and V gathered from the cache, context included."""
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from oracle.attention import flat_decode_attention

    hq, hkv, d = 8, 2, 128
    scale = d**-0.5
    gen = torch.Generator().manual_seed(22)
    q_lens = [1, 1, 1, 600, 300]
    s_lens = [50, 17, 200, 730, 300]
    S, T = len(q_lens), sum(q_lens)
    max_blocks = 48
    table = torch.randperm(S * max_blocks, generator=gen).to(torch.int32).view(S, max_blocks).to(gpu)
    cache = torch.randn(kv_cache_shape(S * max_blocks, 16, hkv, d), generator=gen).to(kv_dtype).to(gpu)
    q, k, v = (torch.randn(T, h * d, generator=gen).to(torch.bfloat16).to(gpu) for h in (hq, hkv, hkv))
    starts = torch.tensor([0] + q_lens).cumsum(0)
    seq = torch.repeat_interleave(torch.arange(S), torch.tensor(q_lens))
    pos = torch.cat([torch.arange(s - n, s) for n, s in zip(q_lens, s_lens)])
    slots = (table.cpu().long()[seq, pos // 16] * 16 + pos % 16).to(gpu)
    builder = ForestCascadeAttentionBackend.get_builder_cls()(hq, hkv, d, device=gpu)
    fp8 = kv_dtype == torch.float8_e4m3fn
    impl = ForestCascadeAttentionBackend.get_impl_cls()(hq, d, scale, hkv, kv_cache_dtype="fp8" if fp8 else "auto")
    ks = torch.tensor([0.9, 1.3], device=gpu) if fp8 else None
    vs = torch.tensor([1.1, 0.7], device=gpu) if fp8 else None
    layer = types.SimpleNamespace(k_scale=ks, v_scale=vs)
    common = CommonAttentionMetadata(
        query_start_loc=starts.to(torch.int32).to(gpu), seq_lens=torch.tensor(s_lens, dtype=torch.int32, device=gpu),
        block_table_tensor=table, slot_mapping=slots, num_reqs=S, max_query_len=max(q_lens), num_actual_tokens=T,
        query_start_loc_cpu=starts.to(torch.int32), seq_lens_cpu=torch.tensor(s_lens, dtype=torch.int32),
    )
    meta = builder.build(0, common)
    assert meta.fresh_start == 3 and meta.context_slots is not None and meta.context_slots.numel() == 730 + 300
    assert meta.fresh_prefill.responses_only and meta.fresh_prefill.num_query_rows == 900
    out = impl.forward(layer, q, k, v, cache, meta)
    torch.cuda.synchronize()
    ref, _ = flat_decode_attention(
        q.view(T, hq, d).cpu(), cache.cpu(), table.cpu()[seq], (pos + 1).to(torch.int32), scale,
        None if ks is None else ks.cpu(), None if vs is None else vs.cpu(), dtype=torch.float32,
    )
    torch.testing.assert_close(out.view(T, hq, d).cpu().float(), ref, rtol=2e-2, atol=2e-2)
    # a short chunk behind a context stays on the query-run path
    short = CommonAttentionMetadata(
        query_start_loc=torch.tensor([0, 100], dtype=torch.int32, device=gpu), seq_lens=torch.tensor([730], dtype=torch.int32, device=gpu),
        block_table_tensor=table[3:4], slot_mapping=slots[:100], num_reqs=1, max_query_len=100, num_actual_tokens=100,
        query_start_loc_cpu=torch.tensor([0, 100], dtype=torch.int32), seq_lens_cpu=torch.tensor([730], dtype=torch.int32),
    )
    assert builder.build(0, short).fresh_prefill is None
