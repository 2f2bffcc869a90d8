"""GPU parity: HIP kernels, called through the C ABI, against the CPU oracle."""

import pytest
import torch

from arctic_platform_amd.workloads import make_config
from oracle.forest import canonical_nodes, discover_forest
from tests.helpers import assert_matches_oracle, oracle_for

pytestmark = pytest.mark.gpu


def _run(w, **kw):
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    md = build_forest_metadata(
        w.block_table, w.seq_lens, num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, **kw
    )
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
    assert hdr["ticket"] == 0 and hdr["done"] == 0, "work queue was not re-armed"
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
