"""Test infrastructure only: CPU restatement of the trainer's split attention over a
deduplicated, unpadded batch.  Nothing in the product imports it.

Deduplicated order of the tokens (``ZoRRoTrain._dedup_input_ids``,
arctic_platform/rl/zorro_train/zorro_train.py:311-356; read back by
``get_group_token_layout``, :2413-2436): for every prompt group the prompt once, then the
response of every sample of the group.  A layout here is that function's result reduced
to what attention needs: a list of ``(prompt_tokens, [response_tokens, ...])``.

The patched attention forward makes two attention calls per layer
(``patched_forward_split_unpadded``, arctic_platform/rl/zorro_train/
qwen_attention_patcher.py:1117-1259): causal attention of every unique prompt over itself
(:1198-1208), and attention of every response over its prompt followed by itself, causal
with the mask aligned bottom-right (:1211-1228: K and V are the prompt's rows followed by
the response's, one copy per sample), and puts the outputs back in deduplicated order
(:1229-1231).  ``split_attention`` below follows those two calls with plain tensor
algebra in the given dtype; autograd through it is the backward the kernels are checked
against.  ``full_attention_of_samples`` is the computation the split replaces, every
sample's whole sequence attended causally on its own, which is what the reference's own
test compares the patched model with (tests/zorro_train/test_once_patcher.py:189-206).

Both calls also receive ``sliding_window`` (:1206, :1226), which the attention interface
turns into "key index > query index - sliding_window" on top of the causal mask, indices
counted in the call's own key sequence (transformers ``sliding_window_overlay``,
masking_utils.py:92-101; the flash path's ``window_size = (sliding_window - 1, ...)``,
modeling_flash_attention_utils.py:650-655).  ``window`` below is that argument.

Pins (tests/test_split_attention.py): split == full on the rows both produce, for outputs
and for gradients (prompt rows of a group receive the sum over its samples), a closed form
(constant V), and the row sums of the probabilities implied by the log-sum-exp; with a
window: the same against ``scaled_dot_product_attention`` under an explicit boolean mask
built with plain loops, a window of 1 (every row returns its own V row), and a window at
least as long as the longest sample (equal to no window).
"""

from __future__ import annotations

import math

import torch


def segments(layout):
    """[(group, kind, start, length)] in deduplicated order; kind 'p' or 'r'."""
    out, t = [], 0
    for g, (prompt, responses) in enumerate(layout):
        out.append((g, "p", t, int(prompt)))
        t += int(prompt)
        for n in responses:
            out.append((g, "r", t, int(n)))
            t += int(n)
    return out


def total_tokens(layout) -> int:
    return sum(int(p) + sum(int(n) for n in rs) for p, rs in layout)


def _attend(q, k, v, scale, first_key_offset, window=None, keep=None, dropout=0.0):
    """q [Lq, Hq, D], k/v [Lk, Hkv, D]; query i sees keys 0 .. first_key_offset + i
    (bottom-right aligned causal mask when first_key_offset = Lk - Lq), with ``window`` only
    the last ``window`` of them.  ``keep`` (bool [Hq, Lq, Lk]) with ``dropout`` = p: the
    probabilities where it is false are dropped and the others divided by 1 - p, after the
    softmax and before the product with V, as the eager attention interface applies
    ``nn.functional.dropout`` to the attention weights (transformers
    models/qwen3/modeling_qwen3.py:173-207).  Returns out and the natural-log log-sum-exp
    [Lq, Hq] (of the scores, untouched by dropout)."""
    lq, hq, _ = q.shape
    lk, hkv, _ = k.shape
    rep = hq // hkv
    kk = k.repeat_interleave(rep, dim=1)
    vv = v.repeat_interleave(rep, dim=1)
    s = torch.einsum("qhd,khd->hqk", q, kk) * scale
    keys = torch.arange(lk)[None, :]
    rows = torch.arange(lq)[:, None]
    s = s.masked_fill(keys > rows + first_key_offset, -math.inf)
    if window is not None:
        s = s.masked_fill(keys <= rows + first_key_offset - int(window), -math.inf)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    if keep is not None:
        p = p * keep.to(p.dtype) / (1.0 - dropout)
    return torch.einsum("hqk,khd->qhd", p, vv), lse.transpose(0, 1)


def split_attention(q, k, v, layout, scale, dtype=torch.float64, window=None, keep=None, dropout=0.0):
    """q [T, Hq, D], k/v [T, Hkv, D] in deduplicated order.  Returns (out [T, Hq, D],
    lse [T, Hq]) in ``dtype``.  Differentiable.  ``keep``: bool [Hq, T, T] over places in the
    deduplicated order (row, key), the dropout mask of attention dropout ``dropout``."""
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)

    def sub(rows, keys):  # the mask of a call: its rows against its key sequence
        return None if keep is None else keep[:, rows][:, :, keys]

    outs, lses = [], []
    prompt_of = {}
    for g, kind, start, n in segments(layout):
        if kind == "p":
            prompt_of[g] = (start, n)
            own = torch.arange(start, start + n)
            o, l = _attend(q[start : start + n], k[start : start + n], v[start : start + n], scale, 0, window, sub(own, own), dropout)
        else:
            ps, pn = prompt_of[g]
            kk = torch.cat([k[ps : ps + pn], k[start : start + n]])
            vv = torch.cat([v[ps : ps + pn], v[start : start + n]])
            own = torch.arange(start, start + n)
            o, l = _attend(q[start : start + n], kk, vv, scale, pn, window, sub(own, torch.cat([torch.arange(ps, ps + pn), own])), dropout)
        outs.append(o)
        lses.append(l)
    return torch.cat(outs), torch.cat(lses)


def reconstruct(x, layout):
    """Deduplicated rows -> one tensor per sample: the prompt's rows followed by the
    response's (the packed reconstruction, zorro_train.py:1071-1159)."""
    samples = []
    prompt = None
    for g, kind, start, n in segments(layout):
        if kind == "p":
            prompt = x[start : start + n]
        else:
            samples.append(torch.cat([prompt, x[start : start + n]]))
    return samples


def reconstruct_packed(x, layout, sample_ids=None):
    """Deduplicated rows -> every sample's prompt rows followed by its response rows, samples in
    the order of their batch indices, one packed tensor (the loops of
    ``ZoRRoTrain._reconstruct_sequences_packed``, zorro_train.py:1071-1159).  ``sample_ids[g]``:
    batch indices of group g's samples in layout order (default: numbered in layout order)."""
    per_sample = reconstruct(x, layout)
    if sample_ids is None:
        order = list(range(len(per_sample)))
    else:
        flat = [s for ids in sample_ids for s in ids]
        order = sorted(range(len(flat)), key=lambda k: flat[k])
    return torch.cat([per_sample[k] for k in order]) if per_sample else x[:0]


def deduplicate_packed(full, layout, sample_ids=None):
    """The way back (``ZoRRoTrain.deduplicate_sequences`` for an unpadded batch, zorro_train.py:
    1162-1179 and the packed variant behind it): a group's prompt rows from its first sample,
    every response from its own sample.  A group without samples gets zero prompt rows."""
    lens = [p + r for p, rs in layout for r in rs]
    flat = list(range(len(lens))) if sample_ids is None else [s for ids in sample_ids for s in ids]
    # where every sample starts in the packed tensor (samples lie in batch order)
    by_batch = sorted(range(len(flat)), key=lambda k: flat[k])
    start, at = {}, 0
    for k in by_batch:
        start[k] = at
        at += lens[k]
    out, k = [], 0
    for p, rs in layout:
        if rs:
            out.append(full[start[k] : start[k] + p])
        else:
            out.append(torch.zeros((p,) + tuple(full.shape[1:]), dtype=full.dtype))
        for r in rs:
            out.append(full[start[k] + p : start[k] + p + r])
            k += 1
    return torch.cat(out) if out else full[:0]


def full_attention_of_samples(q, k, v, layout, scale, dtype=torch.float64, window=None):
    """Every sample's whole sequence attended causally on its own, from the deduplicated
    tensors; returns per sample (out, lse) of prompt + response rows."""
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    return [
        _attend(qs, ks, vs, scale, 0, window)
        for qs, ks, vs in zip(reconstruct(q, layout), reconstruct(k, layout), reconstruct(v, layout))
    ]


def visible(layout, window=None):
    """Brute force: boolean [T, T], entry (r, t) true when query row r attends to key t.
    With ``window``, positions count along the sample's own sequence (prompt, then response)."""
    n = total_tokens(layout)
    vis = torch.zeros(n, n, dtype=torch.bool)
    prompt_of = {}
    for g, kind, start, length in segments(layout):
        if kind == "p":
            prompt_of[g] = (start, length)
        for i in range(length):
            r = start + i
            row_pos = i if kind == "p" else prompt_of[g][1] + i
            for j in range(i + 1):  # the row's own segment
                key_pos = j if kind == "p" else prompt_of[g][1] + j
                if window is None or row_pos - key_pos < window:
                    vis[r, start + j] = True
            if kind == "r":
                ps, pn = prompt_of[g]
                for j in range(pn):
                    if window is None or row_pos - j < window:
                        vis[r, ps + j] = True
    return vis
