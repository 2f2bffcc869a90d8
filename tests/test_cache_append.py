"""KV-cache append: oracle against the layout helpers on the CPU, kernel against the
oracle bit for bit on the GPU."""

import pytest
import torch

from arctic_platform_amd.kv_layout import pack_blocks, unpack_blocks
from oracle.cache import append_kv_reference


def _case(dtype, d, seed):
    g = torch.Generator().manual_seed(seed)
    nb, hkv, t = 7, 2, 21
    cache = pack_blocks(torch.zeros(nb, 16, hkv, d), torch.zeros(nb, 16, hkv, d), dtype)
    key = (torch.randn(t, hkv, d, generator=g) * 3).to(torch.bfloat16)
    value = (torch.randn(t, hkv, d, generator=g) * 3).to(torch.bfloat16)
    slots = torch.randperm(nb * 16, generator=g)[:t].to(torch.int64)
    slots[5] = -1  # a padding token
    ks = torch.tensor([0.013, 0.4]) if dtype == torch.float8_e4m3fn else None
    vs = torch.tensor([0.05, 0.021]) if dtype == torch.float8_e4m3fn else None
    return cache, key, value, slots, ks, vs


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.bfloat16, 128), (torch.float8_e4m3fn, 128)])
def test_oracle_agrees_with_layout_helpers(dtype, d):
    cache, key, value, slots, ks, vs = _case(dtype, d, 11)
    got = append_kv_reference(cache, key, value, slots, ks, vs)
    k, v = unpack_blocks(got, d)
    for t, slot in enumerate(slots.tolist()):
        if slot < 0:
            continue
        b, o = divmod(slot, 16)
        want_k, want_v = key[t].float(), value[t].float()
        if dtype == torch.float8_e4m3fn:
            want_k = (want_k / ks[:, None]).clamp(-448, 448).to(dtype).float()
            want_v = (want_v / vs[:, None]).clamp(-448, 448).to(dtype).float()
        assert torch.equal(k[b, o].float(), want_k) and torch.equal(v[b, o].float(), want_v)
    written = {divmod(s, 16) for s in slots.tolist() if s >= 0}
    for b in range(k.shape[0]):
        for o in range(16):
            if (b, o) not in written:
                assert (k[b, o].float() == 0).all() and (v[b, o].float() == 0).all()


def test_fp8_saturates_and_keeps_nan():
    cache = pack_blocks(torch.zeros(1, 16, 1, 64), torch.zeros(1, 16, 1, 64), torch.float8_e4m3fn)
    key = torch.zeros(1, 1, 64, dtype=torch.bfloat16)
    key[0, 0, 0], key[0, 0, 1], key[0, 0, 2] = 1e4, -1e4, float("nan")
    got = append_kv_reference(cache, key, key, torch.tensor([3]), torch.tensor([1.0]), torch.tensor([1.0]))
    k, _ = unpack_blocks(got, 64)
    assert float(k[0, 3, 0, 0].float()) == 448.0 and float(k[0, 3, 0, 1].float()) == -448.0
    assert torch.isnan(k[0, 3, 0, 2].float())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.bfloat16, 128), (torch.float8_e4m3fn, 64), (torch.float8_e4m3fn, 128)])
def test_kernel_is_bit_exact(gpu, dtype, d):
    from arctic_platform_amd.cache import append_kv

    cache, key, value, slots, ks, vs = _case(dtype, d, 12)
    if dtype == torch.float8_e4m3fn:
        key[2, 0, 0], key[2, 0, 1], value[2, 1, 3] = 1e4, -1e4, float("nan")
    want = append_kv_reference(cache, key, value, slots, ks, vs)
    dev_cache = cache.to(gpu)
    # key/value as views of a fused projection output: [T, Hq + 2 Hkv, D]
    fused = torch.zeros(key.shape[0], 4 + 2 * key.shape[1], d, dtype=torch.bfloat16, device=gpu)
    fused[:, 4:6], fused[:, 6:8] = key.to(gpu), value.to(gpu)
    append_kv(fused[:, 4:6], fused[:, 6:8], dev_cache, slots.to(gpu), None if ks is None else ks.to(gpu), None if vs is None else vs.to(gpu))
    torch.cuda.synchronize()
    a = dev_cache.cpu().view(torch.uint8) if dtype == torch.float8_e4m3fn else dev_cache.cpu().view(torch.int16)
    b = want.view(torch.uint8) if dtype == torch.float8_e4m3fn else want.view(torch.int16)
    assert torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 64), (torch.bfloat16, 128), (torch.float8_e4m3fn, 64), (torch.float8_e4m3fn, 128)])
def test_gather_is_the_way_back(gpu, dtype, d):
    """Rows gathered from the cache are, bit for bit, what the oracle's cache holds at those
    slots (times the per-head scales for fp8, rounded to bf16); a negative slot gives zeros."""
    from arctic_platform_amd.cache import gather_kv

    cache, key, value, slots, ks, vs = _case(dtype, d, 12)
    want_cache = append_kv_reference(cache, key, value, slots, ks, vs)
    k_blocks, v_blocks = unpack_blocks(want_cache, d)  # [blocks, 16, Hkv, D]
    pick = slots.clone()
    pick[1] = -1
    got_k, got_v = gather_kv(want_cache.to(gpu), pick.to(gpu), d, None if ks is None else ks.to(gpu), None if vs is None else vs.to(gpu))
    for got, blocks, scale in ((got_k, k_blocks, ks), (got_v, v_blocks, vs)):
        rows = blocks[pick.clamp(min=0) // 16, pick.clamp(min=0) % 16].float()
        if dtype == torch.float8_e4m3fn:
            rows = rows * scale[None, :, None]
        rows = rows.to(torch.bfloat16)
        rows[pick < 0] = 0
        assert torch.equal(got.cpu().view(torch.int16), rows.view(torch.int16))


@pytest.mark.gpu
def test_append_then_attend(gpu):
    """Decode step end to end: append the new token of every sequence, then attend."""
    from arctic_platform_amd.cache import append_kv
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode
    from arctic_platform_amd.workloads import make_config
    from tests.helpers import assert_matches_oracle, oracle_for

    for index in (2, 5):
        w = make_config(index, device=gpu, shrink=8)
        lens = w.seq_lens.long()
        last = lens - 1  # position of the newest token
        blk = w.block_table.gather(1, (last // 16)[:, None]).squeeze(1).long()
        slots = blk * 16 + last % 16
        g = torch.Generator(device=gpu).manual_seed(5)
        key = torch.randn(w.num_seqs, w.num_kv_heads, w.head_dim, generator=g, device=gpu).to(torch.bfloat16)
        value = torch.randn(w.num_seqs, w.num_kv_heads, w.head_dim, generator=g, device=gpu).to(torch.bfloat16)
        append_kv(key, value, w.kv_cache, slots, w.k_scale, w.v_scale)
        md = build_forest_metadata(w.block_table, w.seq_lens, num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim, chunk_tokens=256)
        out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale, w.k_scale, w.v_scale)
        torch.cuda.synchronize()
        # the oracle reads the cache the kernel wrote; the write itself is checked bit-exactly above
        ref_cache = append_kv_reference(w.kv_cache.cpu(), key.cpu(), value.cpu(), slots.cpu(),
                                        None if w.k_scale is None else w.k_scale.cpu(), None if w.v_scale is None else w.v_scale.cpu())
        assert torch.equal(ref_cache.view(torch.uint8), w.kv_cache.cpu().view(torch.uint8))
        ref_out, ref_lse = oracle_for(w)
        assert_matches_oracle(out, lse, ref_out, ref_lse, what=f"append+attend C{index}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 128), (torch.float8_e4m3fn, 128), (torch.bfloat16, 64), (torch.float8_e4m3fn, 64), (torch.bfloat16, 256), (torch.float8_e4m3fn, 256)])
@pytest.mark.parametrize("start", [0, 8, 5])
def test_prefill_runs_take_packed_stores(gpu, dtype, d, start):
    """Runs of consecutive tokens (a prefill chunk that starts at a block boundary, in the
    middle of a block, and off any 8-token boundary), a padding token inside a run, and a
    token count that is no multiple of 16: the packed V stores and the element stores must
    leave the same bytes as the plain loops of the oracle, and the gather must read them back."""
    from arctic_platform_amd.cache import append_kv, gather_kv
    from arctic_platform_amd.kv_layout import kv_cache_shape

    gen = torch.Generator().manual_seed(11 + start)
    hkv, nblocks, t = 2, 12, 75
    table = torch.randperm(nblocks, generator=gen)
    pos = start + torch.arange(t)
    slots = table[pos // 16].to(torch.int64) * 16 + pos % 16
    slots[37] = -1  # padding in the middle of a run
    key = torch.randn(t, hkv, d, generator=gen).to(torch.bfloat16)
    value = torch.randn(t, hkv, d, generator=gen).to(torch.bfloat16)
    fp8 = dtype == torch.float8_e4m3fn
    ks = torch.tensor([0.02, 0.03]) if fp8 else None
    vs = torch.tensor([0.015, 0.04]) if fp8 else None
    base = (torch.randn(kv_cache_shape(nblocks, 16, hkv, d), generator=gen) * 0.1).to(torch.bfloat16).to(dtype)
    want = append_kv_reference(base, key, value, slots, ks, vs)
    cache = base.clone().to(gpu)
    append_kv(key.to(gpu), value.to(gpu), cache, slots.to(gpu), None if ks is None else ks.to(gpu), None if vs is None else vs.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(cache.cpu().view(torch.uint8), want.view(torch.uint8))
    gk, gv = gather_kv(cache, slots.to(gpu), d, None if ks is None else ks.to(gpu), None if vs is None else vs.to(gpu))
    torch.cuda.synchronize()
    live = slots >= 0
    assert (gk.cpu()[~live] == 0).all() and (gv.cpu()[~live] == 0).all()
    if not fp8:
        assert torch.equal(gk.cpu()[live], key[live]) and torch.equal(gv.cpu()[live], value[live])
    else:
        x = 16
        for tok in (0, 1, 36, 38, t - 1):
            blk, off = divmod(int(slots[tok]), 16)
            for h in range(hkv):
                raw_k = want[0, blk, h].view(d // x, 16, x)[:, off].reshape(d)
                raw_v = want[1, blk, h].view(d, 16)[:, off]
                assert torch.equal(gk.cpu()[tok, h], (raw_k.float() * ks[h]).to(torch.bfloat16))
                assert torch.equal(gv.cpu()[tok, h], (raw_v.float() * vs[h]).to(torch.bfloat16))

