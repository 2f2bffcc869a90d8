"""Pins for the CPU oracle: independent routes, closed forms and invariants chosen so a
dropped term, a wrong sign or index, or a transposed operand fails at least one."""

import math

import pytest
import torch

from arctic_platform_amd.kv_layout import pack_blocks, unpack_blocks
from arctic_platform_amd.workloads import make_config
from oracle.attention import dense_attention, flat_decode_attention, gather_kv, sdpa_decode_attention
from oracle.cascade import cascade_decode_attention
from oracle.merge import merge_partials


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def test_brute_force_matches_library_sdpa_and_logsumexp():
    # independent route: torch's SDPA kernel with repeated KV heads, and torch.logsumexp
    q, k, v = _rand(1, 8, 64, seed=1), _rand(77, 2, 64, seed=2), _rand(77, 2, 64, seed=3)
    out, lse = dense_attention(q, k, v, 0.125)
    ref_out, ref_lse = sdpa_decode_attention(q[0], k, v, 0.125)
    assert torch.allclose(out[0].float(), ref_out, rtol=1e-5, atol=1e-6)
    assert torch.allclose(lse[0].float(), ref_lse, rtol=1e-5, atol=1e-5)


def test_explicit_loops_tiny():
    # brute force with Python loops on a tiny case: catches transposed einsum operands
    q, k, v = _rand(2, 4, 8, seed=4), _rand(5, 2, 8, seed=5), _rand(5, 2, 8, seed=6)
    out, lse = dense_attention(q, k, v, 0.3)
    for r in range(2):
        for h in range(4):
            kvh = h // 2
            scores = [0.3 * sum(float(q[r, h, d]) * float(k[t, kvh, d]) for d in range(8)) for t in range(5)]
            mx = max(scores)
            ws = [math.exp(s - mx) for s in scores]
            tot = sum(ws)
            assert abs(float(lse[r, h]) - (mx + math.log(tot))) < 1e-12
            for d in range(8):
                want = sum(ws[t] * float(v[t, kvh, d]) for t in range(5)) / tot
                assert abs(float(out[r, h, d]) - want) < 1e-12


def test_single_token_closed_form():
    q, k, v = _rand(3, 4, 16, seed=7), _rand(1, 2, 16, seed=8), _rand(1, 2, 16, seed=9)
    out, lse = dense_attention(q, k, v, 0.25)
    for h in range(4):
        assert torch.allclose(out[:, h], v[0, h // 2].expand(3, 16))
        assert torch.allclose(lse[:, h], 0.25 * (q[:, h] @ k[0, h // 2]))


def test_gqa_mapping_distinct_constant_v_per_kv_head():
    # each KV head carries its own constant V: output of query head h must be head h // rep
    q, k = _rand(2, 8, 16, seed=10), _rand(9, 2, 16, seed=11)
    v = torch.stack([torch.full((9, 16), 3.0), torch.full((9, 16), -5.0)], dim=1).double()
    out, _ = dense_attention(q, k, v, 0.25)
    assert torch.allclose(out[:, :4], torch.full((2, 4, 16), 3.0, dtype=torch.float64))
    assert torch.allclose(out[:, 4:], torch.full((2, 4, 16), -5.0, dtype=torch.float64))


def test_score_shift_moves_lse_only():
    # appending a constant channel to q and k adds c * scale to every score
    q, k, v = _rand(1, 2, 8, seed=12), _rand(6, 2, 8, seed=13), _rand(6, 2, 8, seed=14)
    out0, lse0 = dense_attention(q, k, v, 0.5)
    q1 = torch.cat([q, torch.ones(1, 2, 1, dtype=torch.float64)], -1)
    k1 = torch.cat([k, torch.full((6, 2, 1), 3.0, dtype=torch.float64)], -1)
    v1 = torch.cat([v, torch.zeros(6, 2, 1, dtype=torch.float64)], -1)
    out1, lse1 = dense_attention(q1, k1, v1, 0.5)
    assert torch.allclose(out1[..., :8], out0)
    assert torch.allclose(lse1, lse0 + 1.5)


def test_empty_token_set():
    out, lse = dense_attention(_rand(2, 4, 8), torch.zeros(0, 2, 8), torch.zeros(0, 2, 8), 1.0)
    assert (out == 0).all() and torch.isinf(lse).all() and (lse < 0).all()


def test_merge_partition_independence_and_order():
    q, k, v = _rand(2, 4, 8, seed=20), _rand(40, 2, 8, seed=21), _rand(40, 2, 8, seed=22)
    full_out, full_lse = dense_attention(q, k, v, 0.35)
    for cuts in ([0, 40], [0, 1, 40], [0, 7, 19, 40], [0, 13, 13, 40]):
        parts = [dense_attention(q, k[a:b], v[a:b], 0.35) for a, b in zip(cuts[:-1], cuts[1:])]
        for order in (parts, parts[::-1]):
            out, lse = merge_partials(torch.stack([p[0] for p in order]), torch.stack([p[1] for p in order]))
            assert torch.allclose(out, full_out, atol=1e-12) and torch.allclose(lse, full_lse, atol=1e-12)


def test_merge_is_associative():
    q, k, v = _rand(1, 2, 8, seed=23), _rand(30, 2, 8, seed=24), _rand(30, 2, 8, seed=25)
    a, b, c = (dense_attention(q, k[i : i + 10], v[i : i + 10], 1.0) for i in (0, 10, 20))
    ab = merge_partials(torch.stack([a[0], b[0]]), torch.stack([a[1], b[1]]))
    left = merge_partials(torch.stack([ab[0], c[0]]), torch.stack([ab[1], c[1]]))
    bc = merge_partials(torch.stack([b[0], c[0]]), torch.stack([b[1], c[1]]))
    right = merge_partials(torch.stack([a[0], bc[0]]), torch.stack([a[1], bc[1]]))
    assert torch.allclose(left[0], right[0], atol=1e-12) and torch.allclose(left[1], right[1], atol=1e-12)


def test_merge_empty_partial_is_identity_and_all_empty():
    o, l = _rand(3, 4, seed=26), _rand(3, seed=27)
    junk = torch.full((3, 4), float("nan"), dtype=torch.float64)  # an empty partial's output must never be read
    ninf = torch.full((3,), float("-inf"), dtype=torch.float64)
    out, lse = merge_partials(torch.stack([junk, o, junk]), torch.stack([ninf, l, ninf]))
    assert torch.equal(out, o) and torch.equal(lse, l)
    out, lse = merge_partials(torch.stack([junk, junk]), torch.stack([ninf, ninf]))
    assert (out == 0).all() and torch.isinf(lse).all()


def test_merge_two_partials_textbook_weights():
    # out = (e^l1 o1 + e^l2 o2) / (e^l1 + e^l2), lse = log(e^l1 + e^l2)
    o = torch.tensor([[1.0, 2.0], [5.0, -2.0]], dtype=torch.float64)[:, None, :]
    l = torch.tensor([0.3, -1.2], dtype=torch.float64)[:, None]
    out, lse = merge_partials(o, l)
    w = torch.exp(l[:, 0])
    assert torch.allclose(out[0], (w[0] * o[0, 0] + w[1] * o[1, 0]) / w.sum())
    assert torch.allclose(lse[0], torch.log(w.sum()))


def test_layout_round_trip_and_gather():
    g = torch.Generator().manual_seed(5)
    for dtype in (torch.float32, torch.bfloat16, torch.float8_e4m3fn):
        k = torch.randn(6, 16, 2, 64, generator=g).to(dtype)
        v = torch.randn(6, 16, 2, 64, generator=g).to(dtype)
        cache = pack_blocks(k, v, dtype)
        k2, v2 = unpack_blocks(cache, 64)
        assert torch.equal(k2.float(), k.float()) and torch.equal(v2.float(), v.float())
        # the oracle's own reader agrees with the package's packer, element by element
        kk, vv = gather_kv(cache, [4, 1], 23, 64, torch.float64)
        want_k = torch.cat([k[4], k[1]])[:23].double()
        want_v = torch.cat([v[4], v[1]])[:23].double()
        assert torch.equal(kk, want_k) and torch.equal(vv, want_v)
        # raw element order of one tile, straight from the layout definition
        x = 16 // cache.element_size()
        tile = cache[0, 3, 1].float()
        assert float(tile[(5 // x) * 16 * x + 9 * x + 5 % x]) == float(k[3, 9, 1, 5].float())
        assert float(cache[1, 3, 1].float()[37 * 16 + 9]) == float(v[3, 9, 1, 37].float())


@pytest.mark.parametrize("index,shrink", [(1, 1), (2, 16), (4, 16), (5, 16)])
def test_cascade_equals_flat(index, shrink):
    w = make_config(index, shrink=shrink, poison_unused=True)
    flat = flat_decode_attention(w.q, w.kv_cache, w.block_table, w.seq_lens, w.scale, w.k_scale, w.v_scale)
    for chunk in (None, 48):
        out, lse, nodes, leaves = cascade_decode_attention(
            w.q, w.kv_cache, w.block_table, w.seq_lens, w.scale, w.k_scale, w.v_scale, chunk_tokens=chunk
        )
        assert torch.allclose(out, flat[0], atol=1e-10) and torch.allclose(lse, flat[1], atol=1e-10)
    assert not torch.isnan(flat[0]).any(), "oracle read a poisoned slot"
    assert len(nodes) >= 1


def test_fp8_dequantises_first():
    w = make_config(5, shrink=32)
    out, lse = flat_decode_attention(w.q, w.kv_cache, w.block_table, w.seq_lens, w.scale, w.k_scale, w.v_scale, seqs=[0])
    n = int(w.seq_lens[0])
    k, v = gather_kv(w.kv_cache, w.block_table[0, : (n + 15) // 16], n, 128, torch.float64)
    k = k * w.k_scale.double()[None, :, None]
    v = v * w.v_scale.double()[None, :, None]
    ref_out, ref_lse = dense_attention(w.q[:1], k, v, w.scale)
    assert torch.equal(out[0], ref_out[0]) and torch.equal(lse[0], ref_lse[0])
