"""The all-fp32 path on the GPU: fp32 queries on an fp32 paged cache, fp32 products and
partial rows (``fca_decode_step`` with ``kv_dtype = FCA_F32``), against the fp64 oracle on
the same fp32 values.  Tolerance: 2e-5 absolute plus 2e-5 relative on ``out``, 2e-5 on the
log-sum-exp (fp32 rounding of sums over a few thousand terms; the bf16 path's stated
tolerance is a thousand times that)."""

import os
import random

import numpy as np
import pytest
import torch

from arctic_platform_amd.workloads import make_config, make_forest_workload
from tests.helpers import oracle_for
from tests.test_gpu_random_forests import random_forest

pytestmark = pytest.mark.gpu


def _run(w, **kw):
    from arctic_platform_amd.forest import build_forest_metadata
    from arctic_platform_amd.ops import forest_cascade_decode

    md = build_forest_metadata(
        w.block_table, w.seq_lens, num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim,
        partial_dtype=torch.float32, **kw,
    )
    out, lse = forest_cascade_decode(w.q, w.kv_cache, md, w.scale)
    torch.cuda.synchronize()
    md.check()
    assert out.dtype == torch.float32
    return md, out, lse


def _assert_close(out, lse, w, what):
    ref_out, ref_lse = oracle_for(w)
    err = (out.cpu().double() - ref_out).abs()
    assert bool((err <= 2e-5 + 2e-5 * ref_out.abs()).all()), f"{what}: out max |err| {err.max():.3g}"
    lerr = (lse.cpu().double() - ref_lse).abs().max()
    assert lerr <= 2e-5, f"{what}: lse max |err| {lerr:.3g}"


@pytest.mark.parametrize("chunk", [32, 96, 512])
def test_configuration_1_in_fp32(gpu, chunk):
    """Configuration 1 as it is defined: 1 group, prefix 512, 4 samples x 64 suffix tokens, Hq 8 /
    Hkv 2 / D 64, fp32.  Checked against the oracle and against the committed golden result."""
    w = make_config(1, device=gpu, poison_unused=True)
    assert w.q.dtype == torch.float32 and w.kv_cache.dtype == torch.float32
    md, out, lse = _run(w, chunk_tokens=chunk)
    assert md.header()["shared_nodes"] == 1
    _assert_close(out, lse, w, f"C1 fp32, chunk {chunk}")
    # the golden file holds the fp64 result for the CPU generator's values
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config1.npz"))
    import dataclasses

    w_cpu = make_config(1)
    w_gold = dataclasses.replace(w_cpu, q=w_cpu.q.to(gpu), kv_cache=w_cpu.kv_cache.to(gpu), block_table=w_cpu.block_table.to(gpu), seq_lens=w_cpu.seq_lens.to(gpu))
    _, out_g, lse_g = _run(w_gold, chunk_tokens=chunk)
    assert float(np.abs(out_g.cpu().numpy() - z["out"]).max()) <= 2e-5
    assert float(np.abs(lse_g.cpu().numpy() - z["lse"]).max()) <= 2e-5


@pytest.mark.parametrize(
    "seed,hq,hkv,d,depth,fanout,shared,leaf,chunk",
    [
        (2, 32, 8, 128, 4, 3, (1, 200), (1, 100), 64),
        (5, 8, 1, 64, 3, 3, (1, 120), (1, 90), 64),
        (7, 64, 2, 128, 2, 3, (1, 100), (1, 40), 1024),  # 32 query heads per KV head: one member per item
        (15, 10, 2, 128, 3, 5, (1, 200), (1, 60), 96),  # five heads per KV head: two dead rows per item
        (31, 16, 4, 64, 3, 4, (300, 1500), (1, 700), 512),  # chunks of many 64-token steps
    ],
)
def test_random_forests_in_fp32(gpu, seed, hq, hkv, d, depth, fanout, shared, leaf, chunk):
    seg_len, paths = random_forest(random.Random(seed), depth, fanout, shared, leaf)
    w = make_forest_workload(
        "random", seg_len, paths, torch.Generator().manual_seed(seed), num_q_heads=hq, num_kv_heads=hkv, head_dim=d,
        dtype=torch.float32, device=gpu, poison_unused=True,
    )
    md, out, lse = _run(w, chunk_tokens=chunk)
    _assert_close(out, lse, w, f"seed {seed}")
    # sharing off: the same kernel as a plain paged decode attention
    md0, out0, lse0 = _run(w, chunk_tokens=chunk, cascade=False)
    assert md0.header()["shared_items"] == 0
    _assert_close(out0, lse0, w, f"seed {seed}, sharing off")
    # the library's own partial buffers
    from arctic_platform_amd.ops import forest_cascade_decode_static

    out2, lse2 = torch.full_like(out, float("nan")), torch.full_like(lse, float("nan"))
    forest_cascade_decode_static(w.q, w.kv_cache, md, w.scale, out=out2, lse=lse2)
    torch.cuda.synchronize()
    assert torch.equal(out2, out) and torch.equal(lse2, lse)


def test_fp32_cache_writer_and_reader(gpu):
    """fp32 rows into an fp32 cache and back, bit-exact against the CPU restatement's plain loops."""
    from arctic_platform_amd.cache import append_kv, gather_kv
    from arctic_platform_amd.kv_layout import kv_cache_shape
    from oracle.cache import append_kv_reference

    gen = torch.Generator().manual_seed(3)
    hkv, d, nblocks = 2, 64, 9
    slots = list(range(21, 75)) + [3, 130, -1, 100]
    key = torch.randn(len(slots), hkv, d, generator=gen)
    value = torch.randn(len(slots), hkv, d, generator=gen)
    slot_mapping = torch.tensor(slots, dtype=torch.int64)
    cache = torch.zeros(kv_cache_shape(nblocks, 16, hkv, d), dtype=torch.float32, device=gpu)
    append_kv(key.to(gpu), value.to(gpu), cache, slot_mapping.to(gpu))
    want = append_kv_reference(torch.zeros(kv_cache_shape(nblocks, 16, hkv, d)), key, value, slot_mapping)
    assert torch.equal(cache.cpu(), want)
    back_k, back_v = gather_kv(cache, slot_mapping.to(gpu), d)
    live = torch.tensor([s >= 0 for s in slots])
    assert back_k.dtype == torch.float32 and torch.equal(back_k.cpu()[live], key[live]) and torch.equal(back_v.cpu()[live], value[live])
    assert not back_k.cpu()[~live].any() and not back_v.cpu()[~live].any()
    with pytest.raises(TypeError, match="float32"):
        append_kv(key.to(gpu).bfloat16(), value.to(gpu).bfloat16(), cache, slot_mapping.to(gpu))


def test_fp32_tensors_are_refused_where_there_is_no_fp32_path(gpu):
    from arctic_platform_amd import ops
    from arctic_platform_amd.forest import build_forest_metadata

    w = make_config(1, device=gpu)
    kw = dict(num_q_heads=w.num_q_heads, num_kv_heads=w.num_kv_heads, head_dim=w.head_dim)
    half_rows = build_forest_metadata(w.block_table, w.seq_lens, **kw)
    with pytest.raises(ValueError, match="partial_dtype"):
        ops.forest_cascade_decode(w.q, w.kv_cache, half_rows, w.scale)
    md = build_forest_metadata(w.block_table, w.seq_lens, partial_dtype=torch.float32, **kw)
    with pytest.raises(TypeError, match="forest_cascade_decode"):
        ops.prefix_pass(w.q, w.kv_cache, md, w.scale)
    with pytest.raises(TypeError, match="both in float32"):
        ops.forest_cascade_decode(w.q.bfloat16(), w.kv_cache, md, w.scale)
    with pytest.raises(ValueError, match="partial_dtype"):
        ops.forest_cascade_decode(w.q.bfloat16(), w.kv_cache.bfloat16(), md, w.scale)
