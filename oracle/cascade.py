"""Forest cascade decode attention on the CPU: discovery, one stacked pass per shared
node, one pass per private leaf, log-sum-exp merge.  Proves the decomposition the
kernels implement equals flat attention (oracle.attention.flat_decode_attention).

The stacking of every member's query rows against one copy of the shared KV mirrors the
grouped response pass of the trainer (``_compute_response_attention_grouped_unpacked``,
arctic_platform/rl/zorro_train/qwen_attention_patcher.py:409-462).
"""

from __future__ import annotations

import torch

from .attention import BLOCK, dense_attention, gather_kv
from .forest import discover_forest
from .merge import merge_partials


def cascade_decode_attention(
    q, kv_cache, block_table, seq_lens, scale, k_scale=None, v_scale=None, dtype=torch.float64, max_levels=8, chunk_tokens=None,
    row_table=None, row_group=None,
):
    """Returns (out ``[S, Hq, D]``, lse ``[S, Hq]``, nodes, leaves).

    With ``row_table`` / ``row_group`` the rows are query rows over table rows (query runs,
    see oracle.forest); a causal node is attended to by each member up to the member's own
    last token, chunk by chunk like any other node.
    """
    s_all, hq, d = q.shape
    lens = [int(n) for n in seq_lens.tolist()]
    trow = list(range(s_all)) if row_table is None else [int(r) for r in row_table]
    nodes, leaves = discover_forest(block_table.tolist(), lens, BLOCK, max_levels, row_table=row_table, row_group=row_group)
    partial_out = [[] for _ in range(s_all)]
    partial_lse = [[] for _ in range(s_all)]

    def run(members, rep, blk_start, tokens, causal=False):
        nb = (tokens + BLOCK - 1) // BLOCK
        k, v = gather_kv(kv_cache, block_table[trow[rep], blk_start : blk_start + nb], tokens, d, dtype)
        if k_scale is not None:
            k = k * k_scale.to(dtype).cpu()[None, :, None]
        if v_scale is not None:
            v = v * v_scale.to(dtype).cpu()[None, :, None]
        step = chunk_tokens or max(tokens, 1)
        for lo in range(0, tokens, step):
            hi = min(lo + step, tokens)
            if not causal:
                o, l = dense_attention(q[members], k[lo:hi], v[lo:hi], scale, dtype)
            for i, s in enumerate(members):
                if causal:  # this member's tokens of the chunk: up to its own
                    sees = min(hi, lens[s] - blk_start * BLOCK)
                    oi, li = dense_attention(q[s : s + 1], k[lo:sees], v[lo:sees], scale, dtype)
                    partial_out[s].append(oi[0])
                    partial_lse[s].append(li[0])
                else:
                    partial_out[s].append(o[i])
                    partial_lse[s].append(l[i])

    for n in nodes:
        run(n["members"], n["members"][0], n["blk_start"], n["tokens"], n["causal"])
    for s, leaf in enumerate(leaves):
        run([s], s, leaf["blk_start"], leaf["tokens"])

    out = torch.zeros(s_all, hq, d, dtype=dtype)
    lse = torch.full((s_all, hq), float("-inf"), dtype=dtype)
    for s in range(s_all):
        if partial_out[s]:
            out[s], lse[s] = merge_partials(torch.stack(partial_out[s]), torch.stack(partial_lse[s]))
    return out, lse, nodes, leaves
