"""GPU parity: HIP kernels, called through the C ABI, against the CPU oracle."""

import pytest
import torch

from arctic_platform_amd.workloads import make_config
from oracle.forest import canonical_nodes, discover_forest
from tests.helpers import assert_matches_oracle, oracle_for

pytestmark = pytest.mark.gpu


def _run(w, max_workgroups=0, reproducible=False, **kw):
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    md = build_forest_metadata(
        w.block_table, w.seq_lens, num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, **kw
    )
    md.max_workgroups, md.reproducible = max_workgroups, reproducible
    out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
    torch.cuda.synchronize()
    md.check()
    return md, out, lse


def _check_forest(md, w):
    nodes, leaves = discover_forest(w.block_table.cpu().tolist(), w.seq_lens.cpu().tolist(), max_levels=md.plan.max_levels)
    assert canonical_nodes(md.nodes()) == canonical_nodes(nodes)
    got = md.leaves()
    assert [(l["blk_start"], l["tokens"]) for l in got] == [(l["blk_start"], l["tokens"]) for l in leaves]
    hdr = md.header()
    assert hdr["unique_tokens"] == w.unique_tokens
    # every (sequence, token) is covered exactly once by the items on its path
    cover = {}
    for it in md.items():
        for s in it["members"]:
            cover.setdefault(s, []).append((it["blk_start"] * 16, it["tok_len"], it["ord"]))
    lens = w.seq_lens.cpu().tolist()
    npart = md.seq_num_partials()
    for s, n in enumerate(lens):
        spans = sorted(cover.get(s, []))
        pos = 0
        for start, length, _ in spans:
            assert start == pos, f"seq {s}: gap or overlap at token {pos}"
            pos += length
        assert pos == n
        assert sorted(o for _, _, o in spans) == list(range(npart[s]))


@pytest.mark.parametrize("chunk", [32, 96, 512])
def test_config1_bf16(gpu, chunk):
    w = make_config(1, device=gpu, dtype=torch.bfloat16, poison_unused=True)
    md, out, lse = _run(w, chunk_tokens=chunk)
    _check_forest(md, w)
    ref_out, ref_lse = oracle_for(w)
    assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"C1 chunk={chunk}")


@pytest.mark.parametrize("index", [2, 3, 4, 5])
@pytest.mark.parametrize("rows", [32, 64])
def test_shrunk_configs(gpu, index, rows):
    w = make_config(index, device=gpu, shrink=8, poison_unused=True)
    md, out, lse = _run(w, chunk_tokens=128, rows_per_item=rows)
    _check_forest(md, w)
    ref_out, ref_lse = oracle_for(w)
    assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"C{index}/8 rows={rows}")


def test_non_cascade_equals_cascade(gpu):
    w = make_config(2, device=gpu, shrink=8, poison_unused=True)
    md0, out0, lse0 = _run(w, chunk_tokens=128, cascade=False)
    assert md0.header()["shared_nodes"] == 0 and md0.header()["unique_tokens"] == w.flat_tokens
    ref_out, ref_lse = oracle_for(w)
    assert_matches_oracle(out0, lse0, ref_out, ref_lse, what="non-cascade")


def test_golden_micro_cases(gpu):
    """Committed inputs and expected outputs (bf16-exact values) through the kernels."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.kv_layout import pack_blocks
    from arctic_platform_amd.ops import forest_cascade_decode
    from tests.test_golden import micro_cases

    for name, c in micro_cases():
        hq, d = c["q"].shape[1], c["q"].shape[2]
        hkv = c["k_blocks"].shape[2]
        cache = pack_blocks(c["k_blocks"], c["v_blocks"], torch.bfloat16).to(gpu)
        q = c["q"].to(torch.bfloat16).to(gpu)
        for chunk in (32, 512):
            md = build_forest_metadata(
                c["block_table"].to(gpu), c["seq_lens"].to(gpu), num_q_heads=hq, num_kv_heads=hkv, head_dim=d, chunk_tokens=chunk
            )
            out, lse = forest_cascade_decode(q, cache, md, d**-0.5, out_dtype=torch.float32)
            torch.cuda.synchronize()
            md.check()
            assert_matches_oracle(out, lse, c["out"], c["lse"], what=f"{name} chunk={chunk}")
            if name == "fully_shared":
                assert md.header()["shared_nodes"] == 1 and all(l["tokens"] == 0 for l in md.leaves())
            if name == "interleaved_groups":
                assert sorted(n["members"] for n in md.nodes()) == [[0, 2], [1, 3]]


def test_config1_golden(gpu):
    import os

    import numpy as np

    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1.npz"))
    # the fixture is for the CPU generator's fp32 values: draw them on the CPU, round to bf16
    import dataclasses

    from arctic_platform_amd.kv_layout import convert_cache

    w32 = make_config(1)
    w = dataclasses.replace(
        w32,
        q=w32.q.to(torch.bfloat16).to(gpu),
        kv_cache=convert_cache(w32.kv_cache, w32.head_dim, torch.bfloat16).to(gpu),
        block_table=w32.block_table.to(gpu),
        seq_lens=w32.seq_lens.to(gpu),
    )
    md, out, lse = _run(w, chunk_tokens=256)
    # The fixture holds the exact result for the generator's fp32 values; the kernels take
    # bf16 inputs, so what they can be held to is the fixture moved by that rounding alone
    # (the fp64 oracle on the rounded inputs says by how much: about 1e-2 on the log-sum-exp)
    # plus the tolerance of the path on equal inputs.
    ref_out, ref_lse = oracle_for(w)
    gold_out, gold_lse = torch.from_numpy(z["out"]), torch.from_numpy(z["lse"])
    moved_out = (ref_out - gold_out).abs().max()
    moved_lse = (ref_lse - gold_lse).abs().max()
    assert moved_lse <= 2e-2 and moved_out <= 1e-2, (moved_out, moved_lse)
    err = (out.cpu().double() - gold_out).abs().max()
    lerr = (lse.cpu().double() - gold_lse).abs().max()
    assert err <= moved_out + 1e-2 and lerr <= moved_lse + 1e-3, (err, lerr, moved_out, moved_lse)


@pytest.mark.parametrize("index", [2, 3, 4, 5])
def test_full_size_configs(gpu, index):
    """The benchmark shapes at full size: oracle on a sample of rows, and properties that
    need no oracle on every row (non-cascade kernel agrees with the cascade; the split-K
    chunking and the row-tile height do not change the result beyond fp32 noise)."""
    from tests.helpers import oracle_for_sample

    w = make_config(index, device=gpu)
    rows = 64 if index == 3 else 32
    md, out, lse = _run(w, chunk_tokens=1024, rows_per_item=rows)
    hdr = md.header()
    assert hdr["unique_tokens"] == w.unique_tokens
    assert hdr["shared_nodes"] == {2: 64, 3: 16, 4: 33, 5: 64}[index]
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()

    step = w.num_seqs // 8
    sample = sorted({0, w.num_seqs - 1, *range(3, w.num_seqs, step)})
    ref_out, ref_lse = oracle_for_sample(w, sample)
    assert_matches_oracle(out[sample], lse[sample], ref_out, ref_lse, what=f"C{index} sample")

    # same batch through the non-cascade kernel (every sequence private over its whole row)
    _, out_nc, lse_nc = _run(w, chunk_tokens=512, rows_per_item=32, cascade=False)
    assert (lse - lse_nc).abs().max() <= 2e-4
    assert (out.float() - out_nc.float()).abs().max() <= 1.6e-2  # two bf16 roundings of values < 1
    # different chunking and row-tile height
    _, out2, lse2 = _run(w, chunk_tokens=256, rows_per_item=96 - rows)
    assert (lse - lse2).abs().max() <= 2e-4
    assert (out.float() - out2.float()).abs().max() <= 1.6e-2
    assert_matches_oracle(out2[sample], lse2[sample], ref_out, ref_lse, what=f"C{index} sample, {96 - rows}-row tiles")


def test_interleaved_group_order(gpu):
    """Rows of a group scattered over the batch: outputs must come back in row order."""
    import dataclasses

    w = make_config(2, device=gpu, shrink=8, poison_unused=True)
    perm = torch.randperm(w.num_seqs, generator=torch.Generator().manual_seed(3)).to(gpu)
    w2 = dataclasses.replace(w, q=w.q[perm].contiguous(), block_table=w.block_table[perm].contiguous(), seq_lens=w.seq_lens[perm].contiguous())
    md, out, lse = _run(w2, chunk_tokens=128)
    _check_forest(md, w2)
    assert md.header()["shared_nodes"] == 8
    ref_out, ref_lse = oracle_for(w2)
    assert_matches_oracle(out, lse, ref_out, ref_lse, what="interleaved groups")


def test_split_passes_equal_fused(gpu):
    """prefix pass + suffix pass + merge through their own entry points == decode_step."""
    from arctic_platform_amd import ops
    from arctic_platform_amd.forest import build_forest_metadata

    w = make_config(4, device=gpu, shrink=8)
    md, out, lse = _run(w, chunk_tokens=128)
    md2 = build_forest_metadata(w.block_table, w.seq_lens, num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=128)
    md2.partial_out.fill_(float("nan"))
    md2.partial_lse.fill_(float("nan"))
    ops.prefix_pass(w.q, w.kv_cache, md2, w.scale)
    ops.suffix_pass(w.q, w.kv_cache, md2, w.scale)
    out2, lse2 = ops.merge_partials(md2, w.q)
    torch.cuda.synchronize()
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


def test_strided_q_and_out_and_reuse(gpu):
    """q and out as views of wider buffers (a fused QKV projection output), metadata
    rebuilt in place, and the fp32 output type."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    w = make_config(2, device=gpu, shrink=8)
    kw = dict(num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=256)
    md = build_forest_metadata(w.block_table, w.seq_lens, **kw)
    ref_out, ref_lse = oracle_for(w)
    wide = torch.zeros(w.num_seqs, w.num_q_heads + 16, w.head_dim, dtype=torch.bfloat16, device=gpu)
    wide[:, : w.num_q_heads] = w.q
    dst = torch.full((w.num_seqs, w.num_q_heads * 2, w.head_dim), 7.0, dtype=torch.float32, device=gpu)
    out, lse = forest_cascade_decode(wide[:, : w.num_q_heads], w.kv_cache, md, w.scale, out=dst[:, ::2])
    torch.cuda.synchronize()
    assert_matches_oracle(out, lse, ref_out, ref_lse, what="strided q / fp32 out")
    assert (dst[:, 1::2] == 7.0).all()
    md_b = build_forest_metadata(w.block_table, w.seq_lens, out=md, **kw)
    assert md_b.meta.data_ptr() == md.meta.data_ptr()
    out_b, lse_b = forest_cascade_decode(w.q, w.kv_cache, md_b, w.scale)
    torch.cuda.synchronize()
    assert_matches_oracle(out_b, lse_b, ref_out, ref_lse, what="rebuilt metadata")


def test_bad_lengths_are_flagged(gpu):
    from arctic_platform_amd.forest import build_forest_metadata

    bt = torch.zeros(2, 4, dtype=torch.int32, device=gpu)
    sl = torch.tensor([65, 3], dtype=torch.int32, device=gpu)  # 65 tokens need 5 blocks, the table has 4
    md = build_forest_metadata(bt, sl, num_q_heads=8, num_kv_heads=2, head_dim=64)
    torch.cuda.synchronize()
    with pytest.raises(ValueError):
        md.check()
    # a caller that never looks at the flag still cannot mistake the result for attention
    # over the clamped sequence: the merge turns every output of such metadata into NaN
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from arctic_platform_amd.ops import forest_cascade_decode

    q = torch.randn(2, 8, 64, device=gpu).to(torch.bfloat16)
    cache = torch.randn(kv_cache_shape(4, 16, 2, 64), device=gpu).to(torch.bfloat16)
    out, lse = forest_cascade_decode(q, cache, md, 0.125)
    torch.cuda.synchronize()
    assert torch.isnan(out.float()).all() and torch.isnan(lse).all()


def test_error_budget_of_fp32_outputs(gpu):
    """Outputs asked for in fp32 show what the arithmetic itself loses: the probabilities
    enter the value product as bf16 (as in the reference's eager path, which casts them to
    the query dtype), about 1.5e-3 relative in the root mean square.  The half-precision
    partial rows with their per-row power-of-two scale sit well below that, whatever the
    magnitude of V: one KV head's values are scaled by 2^12, another's by 2^-12."""
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    w = make_config(2, device=gpu, shrink=8)
    w.kv_cache[1, :, 0] *= 4096.0
    w.kv_cache[1, :, 1] *= 1.0 / 4096.0
    md = build_forest_metadata(w.block_table, w.seq_lens, num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads,
                               head_dim=w.head_dim, chunk_tokens=128)
    out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, out_dtype=torch.float32)
    torch.cuda.synchronize()
    ref_out, ref_lse = oracle_for(w)
    group = w.num_q_heads // w.num_kv_heads
    for kvh in range(w.num_kv_heads):
        heads = slice(kvh * group, (kvh + 1) * group)
        got, want = out[:, heads].cpu().double(), ref_out[:, heads]
        rel = float((got - want).norm() / want.norm())
        assert rel < 2.5e-3, f"KV head {kvh}: relative rms error {rel:.2e}"
    assert float((lse.cpu().double() - ref_lse).abs().max()) < 1e-5


@pytest.mark.parametrize("index,workgroups,chunk", [(2, 8, 512), (2, 8, 1024), (5, 8, 512), (4, 16, 256)])
def test_items_shared_by_pairs_of_waves(gpu, index, workgroups, chunk):
    """With many items per wave the 32-row kernel sets the largest items aside, one per pair of
    waves, and both waves of a pair attend it from either end until their claims meet.  A
    small grid brings that schedule to a small batch.  Items long enough (four pairs of tiles)
    are shared, shorter ones go to the front wave alone; either way the result is the oracle's,
    the claim counters are zero again after every launch, and a second launch agrees."""
    from arctic_platform_amd.ops import forest_cascade_decode

    w = make_config(index, device=gpu, shrink=4, poison_unused=True)
    md, out, lse = _run(w, max_workgroups=workgroups, chunk_tokens=chunk)
    items = md.items()
    waves = 4 * workgroups
    tickets = len(items) * w.num_kv_heads
    assert tickets >= waves // 2 + 3 * waves, "the batch is too small to set items aside"
    set_aside = [it["tok_len"] for it in items[: waves // 2 // w.num_kv_heads + 1]]
    assert max(set_aside) >= 7 * 32 - 31, "no item long enough to be shared"
    ref_out, ref_lse = oracle_for(w)
    assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"C{index}/4, {workgroups} workgroups")
    ctr = md.meta[md.layout.coop_ctr : md.layout.coop_ctr + 1024]
    assert int(ctr.abs().max()) == 0
    out2, lse2 = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
    torch.cuda.synchronize()
    assert_matches_oracle(out2, lse2, ref_out, ref_lse, what="second launch")
    assert int(ctr.abs().max()) == 0


def test_reproducible_launches_share_no_item_and_repeat_bit_for_bit(gpu):
    """fca_tensors.reproducible: on a batch and grid where the default launch lets pairs of waves
    attend their last items together, no second partial is written, two launches agree in every
    bit, and the result is the oracle's."""
    from arctic_platform_amd.ops import forest_cascade_decode

    w = make_config(2, device=gpu, shrink=4, poison_unused=True)
    md, out, lse = _run(w, max_workgroups=8, reproducible=True, chunk_tokens=512)
    rows = md.plan.num_seqs * md.layout.max_partials * w.num_q_heads
    md.partial_lse.view(-1, 2)[rows:].fill_(float("nan"))
    out2, lse2 = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
    torch.cuda.synchronize()
    assert torch.equal(out2.view(torch.int16), out.view(torch.int16)) and torch.equal(lse2.view(torch.int32), lse.view(torch.int32))
    assert bool(torch.isnan(md.partial_lse.view(-1, 2)[rows:]).all()), "a second partial was written"
    ref_out, ref_lse = oracle_for(w)
    assert_matches_oracle(out, lse, ref_out, ref_lse, what="reproducible launch")
    # the same batch with sharing: second partials appear
    md.reproducible = False
    forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
    torch.cuda.synchronize()
    assert bool((~torch.isnan(md.partial_lse.view(-1, 2)[rows:, 0])).any())

