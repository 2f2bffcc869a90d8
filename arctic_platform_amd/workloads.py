"""Seeded synthetic decode-step workloads for forest cascade attention.

A workload is a forest of token segments (shared prompt segments and per-sample
suffixes), paged into 16-token physical blocks.  Two sequences point at the same
physical block exactly when the whole block lies inside their common token prefix,
which is how a block-granular prefix cache behaves: a shared prefix whose length is
not a multiple of 16 leaves its last few tokens in every sample's first private block.

Draw order (one ``torch.Generator`` per workload, seed = 1000 + configuration number):
segment lengths, then the physical block permutation, then q, then K and V.
"""

from __future__ import annotations

import dataclasses
import math

import numpy as np
import torch

from .kv_layout import BLOCK_SIZE, pack_blocks

FP8_MAX = 448.0


@dataclasses.dataclass
class ForestWorkload:
    name: str
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    q: torch.Tensor  # [S, Hq, D]
    kv_cache: torch.Tensor  # [2, num_blocks, Hkv, 16 * D]
    block_table: torch.Tensor  # [S, max_blocks] int32
    seq_lens: torch.Tensor  # [S] int32
    scale: float
    k_scale: torch.Tensor | None  # [Hkv] fp32 (fp8 caches only)
    v_scale: torch.Tensor | None
    seg_len: list  # tokens per segment
    seq_paths: list  # per sequence: segment ids, root first
    unique_tokens: int  # valid tokens summed over distinct physical blocks
    flat_tokens: int  # sum of seq_lens

    @property
    def num_seqs(self) -> int:
        return self.q.shape[0]

    @property
    def kv_bytes_per_token(self) -> int:
        return 2 * self.num_kv_heads * self.head_dim * self.kv_cache.element_size()

    @property
    def unique_kv_bytes(self) -> int:
        return self.unique_tokens * self.kv_bytes_per_token

    @property
    def flat_kv_bytes(self) -> int:
        return self.flat_tokens * self.kv_bytes_per_token


def _randint(gen, lo, hi, n):
    """n integers uniform on [lo, hi] inclusive."""
    return torch.randint(lo, hi + 1, (n,), generator=gen).tolist()


def two_level_forest(gen, groups, samples, prefix_range, suffix_range):
    seg_len, paths = [], []
    prefix = _randint(gen, prefix_range[0], prefix_range[1], groups)
    suffix = _randint(gen, suffix_range[0], suffix_range[1], groups * samples)
    for g in range(groups):
        seg_len.append(prefix[g])
    for g in range(groups):
        for i in range(samples):
            seg_len.append(suffix[g * samples + i])
            paths.append([g, len(seg_len) - 1])
    return seg_len, paths


def three_level_forest(gen, system_len, segments, samples, segment_range, suffix_range):
    seg_len, paths = [system_len], []
    mid = _randint(gen, segment_range[0], segment_range[1], segments)
    suffix = _randint(gen, suffix_range[0], suffix_range[1], segments * samples)
    for g in range(segments):
        seg_len.append(mid[g])
    for g in range(segments):
        for i in range(samples):
            seg_len.append(suffix[g * samples + i])
            paths.append([0, 1 + g, len(seg_len) - 1])
    return seg_len, paths


def page_forest(seg_len, paths, gen, spare_blocks=0.125, shuffle_blocks=True):
    """Assign physical blocks.  Returns (block_table, seq_lens, slot_src, num_blocks).

    ``slot_src[b * 16 + t]`` is the index of the logical token (position in the
    concatenation of all segments) stored in slot ``t`` of physical block ``b``,
    or -1 for a slot no sequence reads.
    """
    seg_base = np.concatenate([[0], np.cumsum(seg_len)]).astype(np.int64)
    key_to_block: dict = {}
    rows, lens, fills = [], [], []
    for s, path in enumerate(paths):
        tok_src = np.concatenate([seg_base[g] + np.arange(seg_len[g], dtype=np.int64) for g in path])
        ends = np.cumsum([seg_len[g] for g in path])
        n = int(ends[-1])
        row = []
        for j in range(math.ceil(n / BLOCK_SIZE)):
            last = j * BLOCK_SIZE + BLOCK_SIZE - 1
            if last < n:
                owner = path[int(np.searchsorted(ends, last, side="right"))]
                key = (owner, j)
            else:
                key = ("tail", s, j)
            blk = key_to_block.get(key)
            if blk is None:
                blk = len(key_to_block)
                key_to_block[key] = blk
                fills.append((blk, tok_src[j * BLOCK_SIZE : min(n, (j + 1) * BLOCK_SIZE)]))
            row.append(blk)
        rows.append(row)
        lens.append(n)
    used = len(key_to_block)
    num_blocks = used + max(1, int(used * spare_blocks))
    perm = torch.randperm(num_blocks, generator=gen).numpy()  # drawn even if unused: keeps later draws in place
    if not shuffle_blocks:
        perm = np.arange(num_blocks)
    slot_src = np.full(num_blocks * BLOCK_SIZE, -1, dtype=np.int64)
    for blk, src in fills:
        base = int(perm[blk]) * BLOCK_SIZE
        slot_src[base : base + len(src)] = src
    max_blocks = max(len(r) for r in rows)
    table = np.zeros((len(rows), max_blocks), dtype=np.int32)
    for s, row in enumerate(rows):
        table[s, : len(row)] = perm[np.asarray(row, dtype=np.int64)]
    return table, np.asarray(lens, dtype=np.int32), slot_src, num_blocks


def make_forest_workload(
    name,
    seg_len,
    paths,
    gen,
    *,
    num_q_heads,
    num_kv_heads,
    head_dim,
    dtype=torch.bfloat16,
    kv_dtype=None,
    device="cpu",
    poison_unused=False,
    shuffle_blocks=True,
):
    """Build q, the paged cache and the block table for a forest of segments."""
    kv_dtype = kv_dtype or dtype
    table, lens, slot_src, num_blocks = page_forest(seg_len, paths, gen, shuffle_blocks=shuffle_blocks)
    total = int(sum(seg_len))
    dev_gen = gen
    if torch.device(device).type != "cpu":
        dev_gen = torch.Generator(device=device)
        dev_gen.manual_seed(gen.initial_seed())
    num_seqs = len(paths)
    q = torch.randn(num_seqs, num_q_heads, head_dim, generator=dev_gen, device=device, dtype=torch.float32).to(dtype)
    pool_k = torch.randn(total, num_kv_heads, head_dim, generator=dev_gen, device=device, dtype=torch.float32)
    pool_v = torch.randn(total, num_kv_heads, head_dim, generator=dev_gen, device=device, dtype=torch.float32)
    k_scale = v_scale = None
    if kv_dtype == torch.float8_e4m3fn:
        k_scale = (0.01 + 0.09 * torch.rand(num_kv_heads, generator=gen)).to(device)
        v_scale = (0.01 + 0.09 * torch.rand(num_kv_heads, generator=gen)).to(device)
        pool_k = (pool_k / k_scale[None, :, None]).clamp_(-FP8_MAX, FP8_MAX)
        pool_v = (pool_v / v_scale[None, :, None]).clamp_(-FP8_MAX, FP8_MAX)
    pool_k = pool_k.to(kv_dtype)
    pool_v = pool_v.to(kv_dtype)
    src = torch.from_numpy(slot_src).to(device)
    unused = src < 0
    idx = src.clamp(min=0)
    shape = (num_blocks, BLOCK_SIZE, num_kv_heads, head_dim)
    # index_select on raw bytes keeps fp8 payloads intact
    def spread(pool):
        raw = pool.view(torch.uint8) if pool.element_size() == 1 else pool
        out = raw.index_select(0, idx)
        return out.view(kv_dtype) if pool.element_size() == 1 else out

    k_blocks = spread(pool_k)
    v_blocks = spread(pool_v)
    del pool_k, pool_v
    if poison_unused:
        # NaN in every slot no sequence reads (0x7f is NaN in e4m3)
        for blocks in (k_blocks, v_blocks):
            if kv_dtype == torch.float8_e4m3fn:
                blocks.view(torch.uint8)[unused] = 0x7F
            else:
                blocks[unused] = float("nan")
    cache = pack_blocks(k_blocks.view(shape), v_blocks.view(shape), kv_dtype)
    return ForestWorkload(
        name=name,
        num_q_heads=num_q_heads,
        num_kv_heads=num_kv_heads,
        head_dim=head_dim,
        q=q,
        kv_cache=cache,
        block_table=torch.from_numpy(table).to(device),
        seq_lens=torch.from_numpy(lens).to(device),
        scale=1.0 / math.sqrt(head_dim),
        k_scale=k_scale,
        v_scale=v_scale,
        seg_len=list(seg_len),
        seq_paths=[list(p) for p in paths],
        unique_tokens=int((slot_src >= 0).sum()),
        flat_tokens=int(lens.sum()),
    )


CONFIG_NAMES = {
    1: "C1 tiny fp32: 1 group, prefix 512, 4 samples x 64 suffix, Hq 8 / Hkv 2 / D 64",
    2: "C2 Qwen3-4B decode: 64 groups x 8 samples, prefix U[1024,4096], suffix U[1,1024], Hq 32 / Hkv 8 / D 128, bf16",
    3: "C3 long-context rollout: 16 groups x 16 samples, prefix 32768, suffix U[256,4096], Hq 32 / Hkv 8 / D 128, bf16",
    4: "C4 three-level forest: system 1024, 32 segments U[2048,6144] x 8 samples, suffix U[1,2048], Hq 32 / Hkv 8 / D 128, bf16",
    5: "C5 fp8 KV Qwen3-4B decode: C2 shape, K/V fp8 e4m3 with per-KV-head scales U[0.01,0.1]",
    # beyond the five benchmark configurations: the forest of C2 with the attention heads of the
    # in-tree Qwen3.5 (configuration_qwen3_5_moe.py:23-35)
    6: "C2 forest with Qwen3.5 heads: 64 groups x 8 samples, prefix U[1024,4096], suffix U[1,1024], Hq 16 / Hkv 2 / D 256, bf16",
}


def make_config(index: int, device="cpu", *, shrink: int = 1, dtype=None, poison_unused=False, seed=None, shuffle_blocks=True):
    """The five benchmark configurations.  ``shrink`` divides group counts and lengths
    (for CPU-sized variants of the same shape); ``dtype`` overrides the q/KV element type
    of configuration 1 (fp32 by definition) so the bf16 kernels can run it.
    """
    gen = torch.Generator()
    gen.manual_seed(1000 + index if seed is None else seed)
    d = lambda v: max(1, v // shrink)
    if index == 1:
        seg_len, paths = two_level_forest(gen, 1, 4, (512, 512), (64, 64))
        kw = dict(num_q_heads=8, num_kv_heads=2, head_dim=64, dtype=dtype or torch.float32)
    elif index in (2, 5):
        seg_len, paths = two_level_forest(gen, d(64), 8, (d(1024), d(4096)), (1, d(1024)))
        kw = dict(num_q_heads=32, num_kv_heads=8, head_dim=128, dtype=torch.bfloat16)
        if index == 5:
            kw["kv_dtype"] = torch.float8_e4m3fn
    elif index == 6:
        seg_len, paths = two_level_forest(gen, d(64), 8, (d(1024), d(4096)), (1, d(1024)))
        kw = dict(num_q_heads=16, num_kv_heads=2, head_dim=256, dtype=torch.bfloat16)
    elif index == 3:
        seg_len, paths = two_level_forest(gen, d(16), 16, (d(32768), d(32768)), (d(256), d(4096)))
        kw = dict(num_q_heads=32, num_kv_heads=8, head_dim=128, dtype=torch.bfloat16)
    elif index == 4:
        seg_len, paths = three_level_forest(gen, d(1024), d(32), 8, (d(2048), d(6144)), (1, d(2048)))
        kw = dict(num_q_heads=32, num_kv_heads=8, head_dim=128, dtype=torch.bfloat16)
    else:
        raise ValueError(f"unknown configuration {index}")
    name = CONFIG_NAMES[index] + (f" (lengths and groups / {shrink})" if shrink > 1 else "")
    return make_forest_workload(
        name, seg_len, paths, gen, device=device, poison_unused=poison_unused, shuffle_blocks=shuffle_blocks, **kw
    )
