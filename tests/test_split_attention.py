"""Split attention of the trainer over a deduplicated batch: the oracle's pins, the layout
array (host code of the library, no GPU needed) and, on the GPU, forward and backward of
the HIP kernels against the oracle."""

import ctypes
import math
import random

import numpy as np
import pytest
import torch

from arctic_platform_amd import _lib
from arctic_platform_amd.split_attention import (
    SplitLayout,
    dropout_keep_mask,
    split_attention,
    split_attention_padded,
    split_attention_backward,
    split_attention_forward,
)
from oracle.split_attention import (
    full_attention_of_samples,
    reconstruct,
    segments,
    split_attention as oracle_split,
    total_tokens,
    visible,
)

LAYOUTS = [
    [(40, [20, 33]), (7, [5])],
    [(100, [64, 1, 70]), (0, [40]), (33, [0, 31])],
    [(5, [3]), (1, [1, 1, 1, 1, 1, 1, 1, 1])],
    [(64, [32, 32]), (32, [64])],
]


def _random_layout(rng):
    return [
        (rng.choice([0, 1, 5, 31, 32, 33, 70, 130]), [rng.choice([0, 1, 3, 17, 32, 40, 64, 90]) for _ in range(rng.randint(1, 4))])
        for _ in range(rng.randint(1, 4))
    ]


def _inputs(layout, hq, hkv, d, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    t = total_tokens(layout)
    return (
        torch.randn(t, hq, d, generator=g).to(dtype),
        torch.randn(t, hkv, d, generator=g).to(dtype),
        torch.randn(t, hkv, d, generator=g).to(dtype),
    )


# ---- the oracle's pins (CPU) ----------------------------------------------------------------
@pytest.mark.parametrize("layout", LAYOUTS)
def test_oracle_equals_full_attention_of_every_sample(layout):
    """What the reference's own test asserts of the patched model
    (tests/zorro_train/test_once_patcher.py:189-206): the deduplicated forward gives every
    sample the rows that plain causal attention over its whole sequence gives, and the
    prompt rows once.  Gradients: a prompt's K and V collect all samples of the group."""
    q, k, v = _inputs(layout, 4, 2, 16, 3)
    q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
    out, lse = oracle_split(q, k, v, layout, 0.25)
    full = full_attention_of_samples(q, k, v, layout, 0.25)
    # rows of the split result, sample by sample
    outs, lses = reconstruct(out, layout), reconstruct(lse, layout)
    for (fo, fl), so, sl in zip(full, outs, lses):
        torch.testing.assert_close(so, fo, rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(sl, fl, rtol=1e-12, atol=1e-12)
    # a loss that weighs every deduplicated row once; the same loss on the full
    # computation takes a prompt row from the group's first sample only
    w = torch.randn(out.shape, generator=torch.Generator().manual_seed(5), dtype=torch.float64)
    gs = torch.autograd.grad((out * w).sum(), (q, k, v))
    loss = 0.0
    sample = 0
    seen = set()
    for g, kind, start, n in segments(layout):
        if kind == "p":
            prompt = (start, n)
            continue
        fo = full[sample][0]
        ps, pn = prompt
        if g not in seen:
            loss = loss + (fo[:pn] * w[ps : ps + pn]).sum()
            seen.add(g)
        loss = loss + (fo[pn:] * w[start : start + n]).sum()
        sample += 1
    # prompts of groups whose samples are all empty still count
    gf = torch.autograd.grad(loss, (q, k, v))
    for a, b in zip(gs, gf):
        torch.testing.assert_close(a, b, rtol=1e-10, atol=1e-10)


def test_oracle_against_the_brute_force_mask_and_closed_forms():
    layout = LAYOUTS[1]
    q, k, v = _inputs(layout, 4, 2, 8, 11)
    out, lse = oracle_split(q, k, v, layout, 0.3)
    vis = visible(layout)
    s = torch.einsum("qhd,khd->hqk", q, k.repeat_interleave(2, 1)) * 0.3
    s = s.masked_fill(~vis[None], -math.inf)
    torch.testing.assert_close(lse, torch.logsumexp(s, -1).T, rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(out, torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), v.repeat_interleave(2, 1)), rtol=1e-12, atol=1e-12)
    # constant values: every output row is that constant; zero queries: lse = log(keys seen)
    vc = torch.ones_like(v) * 0.75
    oc, lz = oracle_split(torch.zeros_like(q), k, vc, layout, 0.3)
    assert torch.allclose(oc, torch.full_like(oc, 0.75), atol=1e-14)
    torch.testing.assert_close(lz, vis.sum(1).double().log()[:, None].expand(-1, 4), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("window", [1, 5, 40, 1000])
def test_oracle_with_a_sliding_window(window):
    """The window of the two reference calls (qwen_attention_patcher.py:1206, :1226), pinned
    three ways: against scaled_dot_product_attention under a boolean mask written with plain
    loops over positions; split == every sample's whole sequence under the same window; and the
    special cases that need no arithmetic."""
    layout = LAYOUTS[1]
    q, k, v = _inputs(layout, 4, 2, 8, 13)
    out, lse = oracle_split(q, k, v, layout, 0.3, window=window)
    vis = visible(layout, window)
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), attn_mask=vis[None], scale=0.3
    ).transpose(0, 1)
    torch.testing.assert_close(out, ref, rtol=1e-10, atol=1e-10)
    s = (torch.einsum("qhd,khd->hqk", q, kk) * 0.3).masked_fill(~vis[None], -math.inf)
    torch.testing.assert_close(lse, torch.logsumexp(s, -1).T, rtol=1e-12, atol=1e-12)
    # every sample on its own, its whole sequence under the same window
    full = full_attention_of_samples(q, k, v, layout, 0.3, window=window)
    for (fo, fl), so, sl in zip(full, reconstruct(out, layout), reconstruct(lse, layout)):
        torch.testing.assert_close(so, fo, rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(sl, fl, rtol=1e-12, atol=1e-12)
    # the number of keys a row sees: min(window, its position + 1)
    seen = []
    for g, kind, start, n in segments(layout):
        base = 0 if kind == "p" else layout[g][0]
        seen += [min(window, base + i + 1) for i in range(n)]
    assert vis.sum(1).tolist() == seen
    if window == 1:  # a row sees itself only: its own V row, and lse = its own score
        torch.testing.assert_close(out, vv, rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(lse, torch.einsum("qhd,qhd->qh", q, kk) * 0.3, rtol=1e-12, atol=1e-12)
    if window == 1000:  # longer than every sample: no window at all
        o2, l2 = oracle_split(q, k, v, layout, 0.3)
        assert torch.equal(out, o2) and torch.equal(lse, l2)
        assert torch.equal(vis, visible(layout))


def test_oracle_with_attention_dropout():
    """Dropout on the attention weights (after the softmax, before the product with V), the
    way the eager interface the reference resolves applies it.  Pinned by what needs no
    second implementation: nothing dropped = no dropout at all; a constant V gives back the
    surviving probability mass over 1 - p; over many seeds the mean output tends to the
    undropped one; the log-sum-exp does not move; and the mask itself drops a share p,
    with no visible tie between neighbouring heads, rows or keys."""
    layout = LAYOUTS[0]
    hq, t = 4, total_tokens(layout)
    q, k, v = _inputs(layout, hq, 2, 8, 17)
    plain_out, plain_lse = oracle_split(q, k, v, layout, 0.3)
    everything = torch.ones(hq, t, t, dtype=torch.bool)
    out, lse = oracle_split(q, k, v, layout, 0.3, keep=everything, dropout=0.0)
    assert torch.equal(out, plain_out) and torch.equal(lse, plain_lse)
    p = 0.25
    keep = dropout_keep_mask(99, p, hq, t)
    vc = torch.ones_like(v) * 0.5
    out, lse = oracle_split(q, k, vc, layout, 0.3, keep=keep, dropout=p)
    assert torch.equal(lse, plain_lse)
    vis = visible(layout)
    s = (torch.einsum("qhd,khd->hqk", q, k.repeat_interleave(2, 1)) * 0.3).masked_fill(~vis[None], -math.inf)
    mass = (torch.softmax(s, -1) * keep).sum(-1) / (1 - p)  # [Hq, T]
    torch.testing.assert_close(out, 0.5 * mass.T[:, :, None].expand(-1, -1, 8), rtol=1e-12, atol=1e-12)
    mean = torch.zeros_like(plain_out)
    seeds = 400
    for seed in range(seeds):
        mean += oracle_split(q, k, v, layout, 0.3, keep=dropout_keep_mask(seed, p, hq, t), dropout=p)[0]
    # a row that sees n keys has variance ~ p / (1 - p) * sum(prob^2 v^2) per seed
    assert float((mean / seeds - plain_out).abs().max()) < 0.25
    assert float((mean / seeds - plain_out).abs().mean()) < 0.03
    # the mask: share dropped, and no tie between neighbours along any of its three axes
    big = dropout_keep_mask(7, p, 8, 300).float()
    assert abs(float(big.mean()) - (1 - p)) < 3 * math.sqrt(p * (1 - p) / big.numel()) + 1e-4
    centred = big - big.mean()
    for a, b in ((centred[1:], centred[:-1]), (centred[:, 1:], centred[:, :-1]), (centred[:, :, 1:], centred[:, :, :-1])):
        corr = float((a * b).mean() / centred.var())
        assert abs(corr) < 0.01, corr
    assert not torch.equal(dropout_keep_mask(7, p, 2, 64), dropout_keep_mask(8, p, 2, 64))
    assert bool(dropout_keep_mask(7, 0.0, 2, 64).all())


# ---- the layout array (host code of the library) -------------------------------------------------
@pytest.mark.parametrize("window", [None, 1, 9, 32, 50, 200])
def test_layout_array_against_brute_force(window):
    rng = random.Random(7)
    layouts = LAYOUTS + [_random_layout(rng) for _ in range(120 if window is None else 40)]
    for layout in layouts:
        if total_tokens(layout) == 0:
            continue
        L = SplitLayout(layout, device="cpu", sliding_window=window)
        t, nt = L.num_tokens, L.num_tiles
        vis = visible(layout, window).numpy()
        lim = L.kv_lim()
        r, c = np.arange(t)[:, None], np.arange(t)[None, :]
        pos = L.pos()
        seen = (c <= r) & (r < lim[:t][None, :])
        if window is not None:  # what the kernels test element by element
            seen &= pos[:t][:, None] - pos[:t][None, :] < window
        assert (seen == vis).all(), layout
        assert (lim[t:] == 0).all() and (pos[t:] == 0).all()
        want_pos = []
        for g, kind, start, n in segments(layout):
            want_pos += [(0 if kind == "p" else layout[g][0]) + i for i in range(n)]
        assert pos[:t].tolist() == want_pos
        padded = np.zeros((32 * nt, 32 * nt), bool)
        padded[:t, :t] = vis
        tiles = padded.reshape(nt, 32, nt, 32).any(axis=(1, 3))  # [query tile, key tile]
        for i, (a0, a1, b0, _) in enumerate(L.q_tiles()):
            assert a0 <= a1 <= b0 <= i
            covered = set(range(a0, a1)) | set(range(b0, i + 1))
            assert set(np.nonzero(tiles[i])[0].tolist()) <= covered, (layout, i)
        for j, qend in enumerate(L.kv_qend()):
            need = np.nonzero(tiles[:, j])[0]
            assert need.min() >= j and need.max() == qend - 1, (layout, j)
        assert sorted(L.q_order().tolist()) == list(range(nt))
        assert (L.kv_limmin() == lim.reshape(nt, 32).min(axis=1)).all()
        assert sorted(L.kv_order().tolist()) == list(range((nt + 3) // 4))


def test_layout_walks_only_what_is_needed():
    """Eight long responses over one prompt: a query tile of the last response walks the
    prompt's tiles and its own, not the seven responses in between."""
    L = SplitLayout([(1024, [512] * 8)], device="cpu")
    a0, a1, b0, _ = L.q_tiles()[L.num_tiles - 1]
    assert (a0, a1) == (0, 32) and b0 == (1024 + 7 * 512) // 32
    assert L.kv_qend()[0] == L.num_tiles and L.kv_qend()[40] == (1024 + 512) // 32
    # within a group the longest walks first; groups one after the other
    cost = [(a1 - a0) + (i - b0 + 1) for i, (a0, a1, b0, _) in enumerate(L.q_tiles())]
    assert [cost[i] for i in L.q_order()] == sorted(cost, reverse=True)
    two = SplitLayout([(64, [64]), (128, [32])], device="cpu")
    assert sorted(two.q_order()[:4].tolist()) == [0, 1, 2, 3] and two.q_order()[4] == 8
    # key tiles go four to a workgroup, the longest walks first: the prompt's, front to back
    assert L.kv_order()[:8].tolist() == list(range(8))
    # a tile inside a prompt needs no element-wise test against later query tiles of the group
    assert L.kv_limmin()[0] == 1024 + 8 * 512 and L.kv_limmin()[L.num_tiles - 1] == 1024 + 8 * 512


def test_layout_from_the_trainers_reconstruction_info():
    """segment_info as ZoRRoTrain._dedup_input_ids leaves it (zorro_train.py:311-356: the prompt
    segment recorded once per sample of the group, then one response segment per sample) and as
    unpad_deduplicated_batch updates it (:646-672, num_valid_tokens).  Groups as in the
    reference's own grouping test (tests/zorro_train/test_dedup.py:76-88): [[0, 2], [1, 3]]."""
    groups = [[0, 2], [1, 3]]
    prompt_len, response_len = 6, 4
    valid = {("prompt", 0): 5, ("prompt", 2): 5, ("prompt", 1): 6, ("prompt", 3): 6,
             ("response", 0): 4, ("response", 2): 1, ("response", 1): 0, ("response", 3): 3}
    segment_info, pos = [], 0
    for g, members in enumerate(groups):
        for m in members:
            segment_info.append(dict(start=pos, end=pos + prompt_len, original_idx=m, type="prompt", group_idx=g))
        pos += prompt_len
        for m in members:
            segment_info.append(dict(start=pos, end=pos + response_len, original_idx=m, type="response", group_idx=g))
            pos += response_len
    info = dict(prompt_groups=groups, segment_info=segment_info)
    padded = SplitLayout.from_reconstruction_info(info, device="cpu")
    assert padded.groups == [(6, [4, 4]), (6, [4, 4])] and padded.num_tokens == 28
    for seg in segment_info:
        seg["num_valid_tokens"] = valid[(seg["type"], seg["original_idx"])]
    unpadded = SplitLayout.from_reconstruction_info(info, device="cpu")
    assert unpadded.groups == [(5, [4, 1]), (6, [0, 3])] and unpadded.num_tokens == 19
    assert unpadded.kv_lim()[:19].tolist() == [10] * 5 + [9] * 4 + [10] + [19] * 6 + [19] * 3


def test_layout_for_response_rows_only():
    """A prefill chunk behind a cached context: the context is the prompt, q and out hold the
    chunk's rows only, numbered in packed order; tiles of nothing but context rows are skipped."""
    L = SplitLayout([(70, [5]), (0, [3]), (33, [40])], device="cpu", responses_only=True)
    assert L.num_tokens == 151 and L.num_query_rows == 48
    qi = L.q_index()
    assert qi[:70].tolist() == [-1] * 70 and qi[70:78].tolist() == list(range(8))
    assert qi[78:111].tolist() == [-1] * 33 and qi[111:151].tolist() == list(range(8, 48)) and (qi[151:] == -1).all()
    assert [int(rec[3]) for rec in L.q_tiles()] == [0, 0, 1, 1, 1]
    full = SplitLayout([(70, [5]), (0, [3]), (33, [40])], device="cpu")
    assert full.q_index()[:151].tolist() == list(range(151)) and all(rec[3] == 1 for rec in full.q_tiles())
    assert (full.kv_lim() == L.kv_lim()).all()


def test_dropout_range_and_the_window_must_be_the_layouts():
    """The trainer passes both on every call (qwen_attention_patcher.py:1204-1206).  A dropout
    outside [0, 1) raises before a tensor is looked at; so does a window that is not the one
    the layout was made for (its walks are cut to it)."""
    from arctic_platform_amd.split_attention import split_attention, split_attention_padded

    plain = SplitLayout([(4, [3])], device="cpu")
    windowed = SplitLayout([(4, [3])], device="cpu", sliding_window=128)
    for fn, args in ((split_attention, (None, None, None)), (split_attention_padded, (None, None, None, None))):
        with pytest.raises(ValueError, match="dropout"):
            fn(*args, plain, 1.0, dropout=1.0)
        with pytest.raises(ValueError, match="dropout"):
            fn(*args, plain, 1.0, dropout=-0.1)
        with pytest.raises(ValueError, match="sliding_window"):
            fn(*args, plain, 1.0, sliding_window=4096)
        with pytest.raises(ValueError, match="sliding_window"):
            fn(*args, windowed, 1.0, dropout=0.0, sliding_window=64)
        with pytest.raises(ValueError, match="sliding_window"):
            fn(*args, windowed, 1.0)
    with pytest.raises(ValueError, match="positive"):
        SplitLayout([(4, [3])], device="cpu", sliding_window=0)


def test_layout_with_a_window_walks_only_what_the_window_leaves():
    """One prompt of 1024 tokens, eight responses of 512, window 256: a query tile deep inside a
    response walks eight key tiles of its own response and nothing of the prompt; the first tile
    of a response walks the prompt's last eight tiles; a prompt key tile is walked by the query
    tiles up to the start of the last response and no further."""
    L = SplitLayout([(1024, [512] * 8)], device="cpu", sliding_window=256)
    last = L.num_tiles - 1
    a0, a1, b0, _ = L.q_tiles()[last]
    assert a0 == a1 and b0 == last - 8
    first_of_last = (1024 + 7 * 512) // 32
    a0, a1, b0, _ = L.q_tiles()[first_of_last]
    assert (a0, a1) == (32 - 8, 32) and b0 == first_of_last
    # the prompt's last key tile: seen by the first 255 rows of every response, the last of which starts at tile first_of_last
    assert L.kv_qend()[31] == first_of_last + 8
    # the prompt's first key tile: positions 0..31 are seen by prompt rows up to position 286 only
    assert L.kv_qend()[0] == (31 + 256 - 1) // 32 + 1


def test_layout_arguments_are_checked():
    lib = _lib.load_library()
    prompt = np.asarray([4], dtype=np.int32)
    sizes = np.asarray([2], dtype=np.int32)
    resp = np.asarray([3, 2], dtype=np.int32)
    out = np.zeros(128, dtype=np.int32)
    assert lib.fca_split_layout_build(1, prompt.ctypes.data, sizes.ctypes.data, resp.ctypes.data, 9, 0, 0, out.ctypes.data) == 0
    assert lib.fca_split_layout_build(1, prompt.ctypes.data, sizes.ctypes.data, resp.ctypes.data, 10, 0, 0, out.ctypes.data) < 0
    assert b"holds 9 tokens" in lib.fca_last_error()
    resp[1] = -1
    assert lib.fca_split_layout_build(1, prompt.ctypes.data, sizes.ctypes.data, resp.ctypes.data, 6, 0, 0, out.ctypes.data) < 0
    plan = _lib.FcaSplitPlan(100, 6, 4, 128)
    assert lib.fca_split_workspace_bytes(ctypes.byref(plan), None, None) < 0
    plan = _lib.FcaSplitPlan(100, 8, 2, 128)
    fwd, bwd = ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.fca_split_workspace_bytes(ctypes.byref(plan), ctypes.byref(fwd), ctypes.byref(bwd)) == 0
    kv, qq = 128 * 2 * 128 * 2, 128 * 8 * 128 * 2
    # a batch this small forms dk and dv per query head: two sets of fp32 slices [Hq / Hkv][T][Hkv][D] on top
    assert fwd.value == 2 * kv and bwd.value == 3 * kv + 4 * qq + 2 * 128 * 8 * 4 + 2 * 4 * 100 * 2 * 128 * 4
    big = _lib.FcaSplitPlan(32 * 1024, 32, 8, 128)
    assert lib.fca_split_workspace_bytes(ctypes.byref(big), ctypes.byref(fwd), ctypes.byref(bwd)) == 0
    assert bwd.value == 3 * (32768 * 8 * 256) + 4 * (32768 * 32 * 256) + 2 * 32768 * 32 * 4
    with pytest.raises(RuntimeError, match="GPU"):
        L = SplitLayout([(4, [3, 2])], device="cpu")
        x = torch.zeros(9, 4, 64, dtype=torch.bfloat16)
        split_attention_forward(x, x, x, L, 0.125)


# ---- the kernels (GPU) ----------------------------------------------------------------------
def _close(name, got, ref, scale_tol):
    """bf16 results of fp32 accumulations over bf16 probabilities: 2e-2 relative plus
    ``scale_tol`` of the tensor's largest magnitude (plus 1e-5: a gradient that is exactly zero,
    such as dq of a row that sees a single key, comes out as rounding noise of that size)."""
    got, ref = got.detach().cpu().double(), ref.detach().double()
    bound = scale_tol * ref.abs().max() + 2e-2 * ref.abs() + 1e-5
    err = (got - ref).abs()
    assert bool((err <= bound).all()), f"{name}: max |err| {err.max():.4g}, largest reference {ref.abs().max():.4g}"


def _run_case(layout, hq, hkv, d, seed, strided=False, q_gain=1.0, window=None, dropout=0.0):
    q, k, v = _inputs(layout, hq, hkv, d, seed, torch.bfloat16)
    q = (q.float() * q_gain).bfloat16()
    t = q.shape[0]
    scale = d**-0.5
    L = SplitLayout(layout, sliding_window=window)
    if strided:
        # slices of one projection output [T, (Hq + 2 Hkv) * D], the way a fused QKV arrives
        fused = torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], dim=1).cuda()
        qd = fused[:, : hq * d].view(t, hq, d)
        kd = fused[:, hq * d : (hq + hkv) * d].view(t, hkv, d)
        vd = fused[:, (hq + hkv) * d :].view(t, hkv, d)
        assert t == 1 or qd.stride(0) == (hq + 2 * hkv) * d
    else:
        qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    out, lse = split_attention_forward(qd, kd, vd, L, scale, dropout=dropout, seed=seed + 5)
    q64, k64, v64 = (x.double().requires_grad_() for x in (q, k, v))
    keep = dropout_keep_mask(seed + 5, dropout, hq, t) if dropout > 0 else None
    ro, rl = oracle_split(q64, k64, v64, layout, scale, window=window, keep=keep, dropout=dropout)
    # Dropout scales the kept probabilities, and with them their gradients, by 1 / (1 - p) before
    # they are rounded to bf16 for the matrix cores: the rounding noise grows by that factor, and
    # so do the bounds (found on a single element of one layout that lay 10 % over the plain bound).
    grow = 1.0 / (1.0 - dropout)
    _close("out", out, ro, grow * 2e-2 / max(1.0, float(ro.detach().abs().max())))
    torch.testing.assert_close(lse[:, :t].T.cpu().double(), rl.detach(), rtol=1e-3, atol=1e-3)
    dout = torch.randn(t, hq, d, generator=torch.Generator().manual_seed(seed + 1)).bfloat16()
    ro.backward(dout.double())
    dq, dk, dv = split_attention_backward(dout.cuda(), qd, kd, vd, out, lse, L, scale, dropout=dropout, seed=seed + 5)
    _close("dq", dq, q64.grad, grow * 1e-2)
    _close("dk", dk, k64.grad, grow * 1e-2)
    _close("dv", dv, v64.grad, grow * 1e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("layout", LAYOUTS)
@pytest.mark.parametrize("heads", [(4, 2, 128), (8, 1, 64), (2, 2, 128)])
def test_forward_and_backward_match_the_oracle(layout, heads):
    _run_case(layout, *heads, seed=21)


@pytest.mark.gpu
def test_random_layouts_match_the_oracle():
    rng = random.Random(99)
    done = 0
    while done < 12:
        layout = _random_layout(rng)
        if total_tokens(layout) == 0:
            continue
        print("layout", layout, flush=True)
        _run_case(layout, 4, 2, rng.choice([64, 128]), seed=done)
        done += 1


@pytest.mark.gpu
@pytest.mark.parametrize(
    "layout",
    [
        [(1, [0])],  # one token in all
        [(0, [1])],
        [(31, [1])],  # exactly one tile
        [(32, [1])],  # one token into the second tile
        [(0, [2, 0, 3])],  # no prompt at all
        [(3, []), (2, [4])],  # a group without samples
        [(127, [1]), (1, [127])],
    ],
)
@pytest.mark.parametrize("heads", [(4, 1, 128), (6, 2, 64)])
def test_smallest_and_odd_layouts(layout, heads):
    """Fewer steps than ring stages, a single tile, empty prompts and responses; four query
    heads per KV head take the LDS-shared kernels, three the per-wave ones."""
    _run_case(layout, *heads, seed=33)


@pytest.mark.gpu
@pytest.mark.parametrize("q_gain", [8.0, 1 / 64])
def test_sharp_and_flat_score_distributions(q_gain):
    """Scores of magnitude ~100 (softmax close to one-hot, row maxima that jump from tile to
    tile, so the running reference of the forward is rescaled often) and scores near zero."""
    _run_case([(150, [90, 40]), (64, [33])], 8, 2, 128, seed=17, q_gain=q_gain)


@pytest.mark.gpu
def test_strided_inputs_of_a_fused_projection():
    _run_case([(70, [40, 33, 12])], 8, 2, 128, seed=4, strided=True)


@pytest.mark.gpu
def test_training_shape_through_autograd():
    """One group of a GRPO batch at real head counts: 8 responses over a prompt, Hq 32 /
    Hkv 8 / D 128, through torch.autograd (what the trainer's layer would call)."""
    layout = [(600, [300, 420, 150, 512, 64, 333, 200, 97])]
    q, k, v = _inputs(layout, 32, 8, 128, 2, torch.bfloat16)
    scale = 128**-0.5
    L = SplitLayout.from_group_token_layout([{"prompt_tokens": 600, "response_tokens": layout[0][1]}])
    qd, kd, vd = (x.cuda().requires_grad_() for x in (q, k, v))
    out = split_attention(qd, kd, vd, L, scale)
    w = torch.randn(out.shape, generator=torch.Generator().manual_seed(8)).bfloat16()
    (out.float() * w.cuda().float()).sum().backward()
    q64, k64, v64 = (x.double().requires_grad_() for x in (q, k, v))
    ro, _ = oracle_split(q64, k64, v64, layout, scale)
    (ro * w.double()).sum().backward()
    _close("out", out, ro, 2e-2 / max(1.0, float(ro.detach().abs().max())))
    _close("dq", qd.grad, q64.grad, 1e-2)
    _close("dk", kd.grad, k64.grad, 1e-2)
    _close("dv", vd.grad, v64.grad, 1e-2)
    # the layout serves a second layer without new scratch
    before = {k_: b.data_ptr() for k_, b in L._scratch.items()}
    split_attention(qd, kd, vd, L, scale).sum().backward()
    assert before == {k_: b.data_ptr() for k_, b in L._scratch.items()}


@pytest.mark.gpu
def test_large_batch_is_invariant_under_group_order():
    """110k tokens at Hq 32 / Hkv 8 / D 128: a size the oracle cannot cover whole.  Groups do
    not see each other, so running the batch with its groups in reverse order must give every
    group the same rows (tiles fall differently, so equal up to rounding); one group is also
    checked against the oracle, forward and backward."""
    rng = random.Random(3)
    groups = [(rng.randint(1024, 4096), [rng.randint(1, 1024) for _ in range(8)]) for _ in range(16)]
    hq, hkv, d = 32, 8, 128
    scale = d**-0.5
    q, k, v = _inputs(groups, hq, hkv, d, 12, torch.bfloat16)
    dout = torch.randn(q.shape, generator=torch.Generator().manual_seed(13)).bfloat16()
    sizes = [p + sum(rs) for p, rs in groups]
    starts = [sum(sizes[:g]) for g in range(len(groups))]

    def run(order):
        idx = torch.cat([torch.arange(starts[g], starts[g] + sizes[g]) for g in order])
        L = SplitLayout([groups[g] for g in order])
        qd, kd, vd, dd = (x[idx].cuda() for x in (q, k, v, dout))
        out, lse = split_attention_forward(qd, kd, vd, L, scale)
        grads = split_attention_backward(dd, qd, kd, vd, out, lse, L, scale)
        inverse = torch.empty_like(idx)
        inverse[idx] = torch.arange(idx.numel())
        return [x.cpu()[inverse] for x in (out, *grads)]

    forward_order = run(list(range(len(groups))))
    reverse_order = run(list(reversed(range(len(groups)))))
    for name, a, b in zip(("out", "dq", "dk", "dv"), forward_order, reverse_order):
        _close(name, a, b.double(), 1e-2)
    g = min(range(len(groups)), key=lambda i: sizes[i])
    sl = slice(starts[g], starts[g] + sizes[g])
    q64, k64, v64 = (x[sl].double().requires_grad_() for x in (q, k, v))
    ro, _ = oracle_split(q64, k64, v64, [groups[g]], scale, dtype=torch.float32)
    ro.backward(dout[sl].float())
    _close("out", forward_order[0][sl], ro, 2e-2 / max(1.0, float(ro.detach().abs().max())))
    for name, got, ref in zip(("dq", "dk", "dv"), forward_order[1:], (q64.grad, k64.grad, v64.grad)):
        _close(name, got[sl], ref, 1e-2)


@pytest.mark.gpu
def test_padded_batch_is_gathered_attended_and_scattered():
    """Prompts padded on the left, responses on the right, as the trainer's padded batches are:
    the valid rows get the oracle's values, padding rows zeros, and gradients reach only valid
    rows."""
    layout = [(5, [4, 1]), (6, [0, 3])]
    prompt_len, response_len = 6, 4
    valid = []
    for p, rs in layout:
        valid += [False] * (prompt_len - p) + [True] * p
        for r in rs:
            valid += [True] * r + [False] * (response_len - r)
    valid = torch.tensor(valid)
    tp, t = valid.numel(), int(valid.sum())
    assert t == total_tokens(layout)
    gen = torch.Generator().manual_seed(6)
    hq, hkv, d = 4, 2, 64
    qp, kp, vp = (torch.randn(tp, h, d, generator=gen).bfloat16() for h in (hq, hkv, hkv))
    qd, kd, vd = (x.cuda().requires_grad_() for x in (qp, kp, vp))
    out = split_attention_padded(qd, kd, vd, valid.cuda(), SplitLayout(layout), d**-0.5)
    w = torch.randn(tp, hq, d, generator=gen).bfloat16()
    (out.float() * w.cuda().float()).sum().backward()
    q64, k64, v64 = (x[valid].double().requires_grad_() for x in (qp, kp, vp))
    ro, _ = oracle_split(q64, k64, v64, layout, d**-0.5)
    (ro * w[valid].double()).sum().backward()
    assert float(out.detach()[~valid.cuda()].abs().max()) == 0.0
    _close("out", out[valid.cuda()], ro, 2e-2)
    for name, got, ref in (("dq", qd.grad, q64.grad), ("dk", kd.grad, k64.grad), ("dv", vd.grad, v64.grad)):
        assert float(got[~valid.cuda()].abs().max()) == 0.0, name
        _close(name, got[valid.cuda()], ref, 1e-2)
    with pytest.raises(ValueError, match="valid tokens"):
        split_attention_padded(qd, kd, vd, torch.ones(tp, dtype=torch.bool).cuda(), SplitLayout(layout), 0.125)


@pytest.mark.gpu
def test_chunks_behind_a_context_attend_as_responses():
    """responses_only: k and v hold context + chunk of every sequence, q only the chunks.
    The rows equal the response rows of the full computation (the oracle), the context's own
    attention is never formed."""
    layout = [(70, [45]), (0, [33]), (200, [64]), (16, [1])]
    hq, hkv, d = 8, 2, 128
    scale = d**-0.5
    q_all, k, v = _inputs(layout, hq, hkv, d, 5, torch.bfloat16)
    ro, _ = oracle_split(q_all.double(), k.double(), v.double(), layout, scale)
    L = SplitLayout(layout, responses_only=True)
    rows = torch.tensor(L.q_index()[: L.num_tokens] >= 0)
    assert int(rows.sum()) == L.num_query_rows == 143
    out, _ = split_attention_forward(q_all[rows].cuda(), k.cuda(), v.cuda(), L, scale)
    _close("out", out, ro[rows], 2e-2 / max(1.0, float(ro.abs().max())))
    with pytest.raises(ValueError, match="forward only"):
        split_attention_backward(out, out, k.cuda(), v.cuda(), out, out, L, scale)


@pytest.mark.gpu
def test_forward_and_backward_replay_from_a_graph():
    """The calls launch kernels only (no memsets, no host round trips), so a layer's forward
    and backward can be captured once and replayed; every replay, with new inputs and eager
    work in between, equals the eager result bit for bit."""
    layout = [(90, [40, 70]), (33, [64])]
    hq, hkv, d = 8, 2, 128
    scale = d**-0.5
    L = SplitLayout(layout)
    t = L.num_tokens
    gen = torch.Generator().manual_seed(31)
    q, k, v, dout = (torch.empty(t, h, d, dtype=torch.bfloat16, device="cuda") for h in (hq, hkv, hkv, hq))

    def refill():
        for x in (q, k, v, dout):
            x.copy_(torch.randn(x.shape, generator=gen).bfloat16())

    refill()
    out, lse = split_attention_forward(q, k, v, L, scale)  # warm-up: scratch buffers exist before the capture
    split_attention_backward(dout, q, k, v, out, lse, L, scale)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            g_out, g_lse = split_attention_forward(q, k, v, L, scale)
            g_grads = split_attention_backward(dout, q, k, v, g_out, g_lse, L, scale)
    for _ in range(3):
        refill()
        graph.replay()
        torch.cuda.synchronize()
        e_out, e_lse = split_attention_forward(q, k, v, L, scale)
        e_grads = split_attention_backward(dout, q, k, v, e_out, e_lse, L, scale)
        torch.cuda.synchronize()
        assert torch.equal(g_out, e_out) and torch.equal(g_lse[:, :t], e_lse[:, :t])
        for a, b in zip(g_grads, e_grads):
            assert torch.equal(a, b)
