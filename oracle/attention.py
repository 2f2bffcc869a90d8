"""Flat (non-cascade) decode attention over a paged cache: the value oracle.

Restates, for one query token per sequence:
* grouped-query head mapping, query head h reads KV head h // (Hq / Hkv)
  (``_repeat_kv`` expands each KV head n_rep times in place:
  arctic_platform/model/implementations/qwen35/models/qwen3_5_moe/modeling_qwen3_5_moe.py:368-373);
* scores scaled by head_dim ** -0.5 (same file :385), softmax over every cached token
  with no mask (the decode token sees its whole history), probabilities times V
  (``_attention_core`` :440-454; the eager interface the trainer resolves at
  arctic_platform/rl/zorro_train/qwen_attention_patcher.py:55-61 and calls at :511-527);
* the natural-log log-sum-exp of the scaled scores, as ``torch.logsumexp`` is used at
  arctic_platform/common/utils/tiled_logits.py:129.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

BLOCK = 16


def gather_kv(kv_cache, block_ids, num_tokens, head_dim, dtype=torch.float64):
    """Read ``num_tokens`` tokens through a list of physical block ids.

    Cache layout (stated independently of the package code): plane 0 holds K tiles
    ``[head_dim / x, 16, x]`` per (block, kv head) with x = 16 bytes / element size;
    plane 1 holds V tiles ``[head_dim, 16]``.  Returns k, v as ``[tokens, Hkv, D]``.
    """
    ids = torch.as_tensor(block_ids, dtype=torch.long, device=kv_cache.device)
    x = 16 // kv_cache.element_size()
    hkv = kv_cache.shape[2]
    kt = kv_cache[0].index_select(0, ids).to(dtype).view(len(ids), hkv, head_dim // x, BLOCK, x)
    vt = kv_cache[1].index_select(0, ids).to(dtype).view(len(ids), hkv, head_dim, BLOCK)
    k = kt.permute(0, 3, 1, 2, 4).reshape(len(ids) * BLOCK, hkv, head_dim)[:num_tokens]
    v = vt.permute(0, 3, 1, 2).reshape(len(ids) * BLOCK, hkv, head_dim)[:num_tokens]
    return k, v


def dense_attention(q, k, v, scale, dtype=torch.float64):
    """q ``[R, Hq, D]`` against one shared token set k, v ``[T, Hkv, D]``.

    Returns (out ``[R, Hq, D]``, lse ``[R, Hq]``).  T == 0 gives out = 0, lse = -inf.
    """
    r, hq, d = q.shape
    t, hkv, _ = k.shape
    rep = hq // hkv
    if t == 0:
        return torch.zeros(r, hq, d, dtype=dtype), torch.full((r, hq), float("-inf"), dtype=dtype)
    kk = k.to(dtype).repeat_interleave(rep, dim=1)  # [T, Hq, D]
    vv = v.to(dtype).repeat_interleave(rep, dim=1)
    s = torch.einsum("rhd,thd->rht", q.to(dtype), kk) * scale
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    return torch.einsum("rht,thd->rhd", p, vv), lse


def flat_decode_attention(q, kv_cache, block_table, seq_lens, scale, k_scale=None, v_scale=None, dtype=torch.float64, seqs=None):
    """Every sequence attends to its own full block-table row, no sharing exploited.

    fp8 caches are dequantised first: value = fp8 -> float, times the per-KV-head scale.
    ``seqs`` restricts the computation to a subset of rows (same output shape, other
    rows left at zero / -inf).
    """
    s_all, hq, d = q.shape
    out = torch.zeros(s_all, hq, d, dtype=dtype)
    lse = torch.full((s_all, hq), float("-inf"), dtype=dtype)
    lens = seq_lens.tolist()
    for s in range(s_all) if seqs is None else seqs:
        n = lens[s]
        nb = (n + BLOCK - 1) // BLOCK
        k, v = gather_kv(kv_cache, block_table[s, :nb], n, d, dtype)
        if k_scale is not None:
            k = k * k_scale.to(dtype).cpu()[None, :, None]
        if v_scale is not None:
            v = v * v_scale.to(dtype).cpu()[None, :, None]
        o, l = dense_attention(q[s : s + 1], k, v, scale, dtype)
        out[s], lse[s] = o[0], l[0]
    return out, lse


def sdpa_decode_attention(q_row, k, v, scale):
    """Second, independent route for one sequence: the library kernel the reference
    calls (modeling_qwen3_5_moe.py:448-454) with KV heads repeated, fp32, no causal
    mask (a one-row causal mask in torch is top-left aligned and would hide all but
    the first key).  q_row ``[Hq, D]``, k, v ``[T, Hkv, D]``.
    """
    hq = q_row.shape[0]
    rep = hq // k.shape[1]
    kk = k.float().repeat_interleave(rep, dim=1).permute(1, 0, 2)[None]  # [1, Hq, T, D]
    vv = v.float().repeat_interleave(rep, dim=1).permute(1, 0, 2)[None]
    qq = q_row.float()[None, :, None, :]
    out = F.scaled_dot_product_attention(qq, kk, vv, is_causal=False, scale=scale)[0, :, 0]
    lse = torch.logsumexp(torch.einsum("hd,htd->ht", q_row.float(), kk[0]) * scale, dim=-1)
    return out, lse
