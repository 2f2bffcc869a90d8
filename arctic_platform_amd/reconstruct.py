"""Whole samples from a deduplicated training tensor, and back.

The trainer keeps every prompt group's prompt once, followed by the response of each of its
samples (``ZoRRoTrain._dedup_input_ids``, arctic_platform/rl/zorro_train/zorro_train.py:311-356).
Where it wants whole samples again (the embeddings the patched model forward hands on,
rl/zorro_train/qwen_model_patcher.py:394; the attention modes that attend every sample on its
own, rl/zorro_train/qwen_attention_patcher.py:801-811) it calls
``ZoRRoTrain.reconstruct_sequences`` (zorro_train.py:725-745), whose packed form is Python loops
over slices and ``torch.cat`` (:1071-1159; the Triton kernel at :160-235 copies a row per
program), and ``deduplicate_sequences`` (:1162-1179) for the way back.

Here both are one gather of whole rows through an index made once per batch
(``fca_gather_rows``), in the packed (unpadded) form: every sample's valid tokens, prompt then
response, samples in the order of their indices in the original batch.  Both are
differentiable: the gradient of a reconstruction sums, for every deduplicated row, the rows of
its copies (``fca_sum_rows``; a prompt row collects all samples of its group), the gradient of
a deduplication is a gather the other way with zeros where a row was not taken.
"""

from __future__ import annotations

import numpy as np
import torch

from . import _lib
from .split_attention import SplitLayout, _stream_ptr


class SampleIndex:
    """Index arrays between the deduplicated order of a ``SplitLayout`` and the packed order of
    whole samples.  ``sample_ids[g]`` lists the original batch indices of group ``g``'s samples in
    the order of the layout's responses (``reconstruction_info["prompt_groups"]``); the default
    numbers the samples in layout order."""

    def __init__(self, layout: SplitLayout, sample_ids=None):
        groups = layout.groups
        if sample_ids is None:
            sample_ids, n = [], 0
            for _, responses in groups:
                sample_ids.append(list(range(n, n + len(responses))))
                n += len(responses)
        if len(sample_ids) != len(groups) or any(len(ids) != len(rs) for ids, (_, rs) in zip(sample_ids, groups)):
            raise ValueError("sample_ids must list one batch index per response of every group")
        flat = sorted(i for ids in sample_ids for i in ids)
        if flat != list(range(len(flat))):
            raise ValueError("sample_ids must be a permutation of 0 .. number of samples - 1")
        # place of every segment in the deduplicated order
        where = {}  # sample -> (prompt start, prompt tokens, response start, response tokens, first of its group)
        t = 0
        for (prompt, responses), ids in zip(groups, sample_ids):
            p0 = t
            t += prompt
            for k, (n, s) in enumerate(zip(responses, ids)):
                where[s] = (p0, prompt, t, n, k == 0)
                t += n
        self.num_dedup = t
        full_from, dedup_from = [], np.full(t, -1, dtype=np.int32)
        at = 0
        for s in range(len(flat)):
            p0, pn, r0, rn, first = where[s]
            full_from.append(np.arange(p0, p0 + pn, dtype=np.int32))
            full_from.append(np.arange(r0, r0 + rn, dtype=np.int32))
            if first:  # the group's first sample lends its prompt rows to the deduplicated tensor
                dedup_from[p0 : p0 + pn] = np.arange(at, at + pn, dtype=np.int32)
            dedup_from[r0 : r0 + rn] = np.arange(at + pn, at + pn + rn, dtype=np.int32)
            at += pn + rn
        self.num_full = at
        self.full_from = np.concatenate(full_from) if full_from else np.zeros(0, np.int32)  # [num_full] -> dedup row
        self.dedup_from = dedup_from  # [num_dedup] -> full row (a prompt of a group without samples: -1)
        # the copies of every deduplicated row, for the gradient of a reconstruction
        order = np.argsort(self.full_from, kind="stable").astype(np.int32)
        counts = np.bincount(self.full_from, minlength=t) if at else np.zeros(t, np.int64)
        self.copies_offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
        self.copies_rows = order
        # where a full row went in a deduplication (-1: not taken), for its gradient
        taken = np.full(at, -1, dtype=np.int32)
        live = dedup_from >= 0
        taken[dedup_from[live]] = np.nonzero(live)[0].astype(np.int32)
        self.full_taken = taken
        self._dev = {}

    def on(self, device, name):
        key = (str(device), name)
        if key not in self._dev:
            self._dev[key] = torch.from_numpy(np.ascontiguousarray(getattr(self, name))).to(device)
        return self._dev[key]


def sample_index(layout: SplitLayout, sample_ids=None) -> SampleIndex:
    """The index of a layout, kept with it (one per ``sample_ids``; the default is the layout's
    own, which ``SplitLayout.from_reconstruction_info`` takes from ``prompt_groups``)."""
    if sample_ids is None:
        sample_ids = layout.sample_ids
    store = layout.__dict__.setdefault("_sample_index", {})
    key = None if sample_ids is None else tuple(tuple(ids) for ids in sample_ids)
    if key not in store:
        store[key] = SampleIndex(layout, sample_ids)
    return store[key]


def _rows(x, tokens, what):
    """[T, ...] or [1, T, ...] -> (2-D view [T, C], had a batch dimension)."""
    if x.dim() >= 3 and x.shape[0] == 1 and x.shape[1] == tokens:
        batched, x2 = True, x[0]
    elif x.shape[0] == tokens:
        batched, x2 = False, x
    else:
        raise ValueError(f"{what} must be [T, ...] or [1, T, ...] with T = {tokens}, got {tuple(x.shape)}")
    if not x2.is_cuda:
        raise RuntimeError(f"rows are gathered on the GPU; {what} must be a device tensor")
    width = 1
    for n in x2.shape[1:]:
        width *= int(n)
    x2 = (x2 if x2.is_contiguous() else x2.contiguous()).reshape(tokens, width)  # (an explicit width: no rows is a legal batch)
    if (x2.shape[1] * x2.element_size()) % 16 or x2.data_ptr() % 16:
        raise ValueError(f"a row of {what} must be a multiple of 16 bytes and 16-byte aligned")
    return x2, batched


def _gather(src, index, num_rows):
    if src.shape[0] == 0:  # nothing to take rows from: every index is "none"
        return torch.zeros((num_rows, src.shape[1]), dtype=src.dtype, device=src.device)
    out = torch.empty((num_rows, src.shape[1]), dtype=src.dtype, device=src.device)
    _lib.check(
        _lib.load_library().fca_gather_rows(
            src.data_ptr(), src.stride(0) * src.element_size(), index.data_ptr(), num_rows, src.shape[1] * src.element_size(),
            out.data_ptr(), out.stride(0) * out.element_size(), _stream_ptr(src.device),
        )
    )
    return out


def _sum_copies(src, offsets, rows, num_dst):
    if src.dtype == torch.bfloat16:
        code = _lib.FCA_BF16
    elif src.dtype == torch.float32:
        code = _lib.FCA_F32
    else:
        raise TypeError(f"gradients of a reconstruction are summed in bfloat16 or float32, got {src.dtype}")
    if src.shape[1] % 8:
        raise ValueError("a row must hold a multiple of 8 values")
    out = torch.empty((num_dst, src.shape[1]), dtype=src.dtype, device=src.device)
    _lib.check(
        _lib.load_library().fca_sum_rows(
            src.data_ptr(), src.stride(0) * src.element_size(), offsets.data_ptr(), rows.data_ptr(), num_dst, src.shape[1], code,
            out.data_ptr(), out.stride(0) * out.element_size(), _stream_ptr(src.device),
        )
    )
    return out


class _Reconstruct(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x2, index: SampleIndex):
        ctx.index = index
        return _gather(x2, index.on(x2.device, "full_from"), index.num_full)

    @staticmethod
    def backward(ctx, grad):
        ix = ctx.index
        g = grad if grad.is_contiguous() else grad.contiguous()
        return _sum_copies(g, ix.on(g.device, "copies_offsets"), ix.on(g.device, "copies_rows"), ix.num_dedup), None


class _Deduplicate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x2, index: SampleIndex):
        ctx.index = index
        return _gather(x2, index.on(x2.device, "dedup_from"), index.num_dedup)

    @staticmethod
    def backward(ctx, grad):
        ix = ctx.index
        g = grad if grad.is_contiguous() else grad.contiguous()
        return _gather(g, ix.on(g.device, "full_taken"), ix.num_full), None


def reconstruct_sequences(dedup_hidden: torch.Tensor, layout: SplitLayout, sample_ids=None) -> torch.Tensor:
    """``[T, ...]`` (or ``[1, T, ...]``) in deduplicated order -> ``[T_full, ...]`` (``[1, T_full, ...]``):
    every sample's prompt rows followed by its response rows, samples in batch order, no padding
    (``ZoRRoTrain.reconstruct_sequences`` for an unpadded batch).  Differentiable."""
    ix = sample_index(layout, sample_ids)
    x2, batched = _rows(dedup_hidden, ix.num_dedup, "dedup_hidden")
    out = _Reconstruct.apply(x2, ix).reshape((ix.num_full,) + tuple(dedup_hidden.shape[2 if batched else 1 :]))
    return out.unsqueeze(0) if batched else out


def deduplicate_sequences(full_hidden: torch.Tensor, layout: SplitLayout, sample_ids=None) -> torch.Tensor:
    """The way back (``ZoRRoTrain.deduplicate_sequences`` for an unpadded batch): a group's prompt
    rows from its first sample, every response from its own sample.  Differentiable; the prompt
    rows of the other samples of a group receive no gradient."""
    ix = sample_index(layout, sample_ids)
    x2, batched = _rows(full_hidden, ix.num_full, "full_hidden")
    out = _Deduplicate.apply(x2, ix).reshape((ix.num_dedup,) + tuple(full_hidden.shape[2 if batched else 1 :]))
    return out.unsqueeze(0) if batched else out
