"""Split attention of the trainer over a deduplicated, unpadded batch, forward and backward.

Host-side face of ``fca_split_attention_forward`` / ``fca_split_attention_backward``.  It
stands where the trainer's patched attention forward makes its two ``attention_interface``
calls and regroups their outputs (``patched_forward_split_unpadded``,
arctic_platform/rl/zorro_train/qwen_attention_patcher.py:1186-1231): prompt rows attend
causally to their prompt, response rows to the whole prompt of their group and causally to
their own response.  The tensors stay in deduplicated order (for every prompt group the
prompt once, then the response of every sample, zorro_train.py:311-356); nothing is copied
per sample, and in the backward a prompt's dK and dV collect all samples of its group.

``SplitLayout.from_group_token_layout`` takes what ``ZoRRoTrain.get_group_token_layout``
returns (zorro_train.py:2413-2436): a list of dicts with ``prompt_tokens`` and
``response_tokens``.  A layout is made once per batch and serves every layer.
"""

from __future__ import annotations

import ctypes

import numpy as np
import torch

from . import _lib


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class SplitLayout:
    """Token layout of one deduplicated batch: ``[(prompt_tokens, [response_tokens, ...]), ...]``."""

    def __init__(self, groups, device="cuda", responses_only=False, scratch_pool=None, sliding_window=None):
        """``scratch_pool``: a dict shared by layouts whose calls run one after the other on one
        stream (the adapter makes a layout per step), so that they share their scratch buffers.
        ``responses_only`` (forward only): ``k`` and ``v`` hold every token, ``q`` and ``out`` only
        the response rows, in packed order, and the prompts' own attention is not computed (a
        prefill chunk behind a cached context, with the context as the prompt).
        ``sliding_window`` (the argument of the trainer's attention calls,
        qwen_attention_patcher.py:1206, :1226; None = no window): a row sees only the keys fewer
        than that many positions before it in its own sample's sequence, itself included."""
        self.groups = [(int(p), [int(n) for n in rs]) for p, rs in groups]
        self.responses_only = bool(responses_only)
        if sliding_window is not None and int(sliding_window) < 1:
            raise ValueError(f"sliding_window must be a positive number of tokens or None, got {sliding_window}")
        self.window = 0 if sliding_window is None else int(sliding_window)
        prompt = np.asarray([p for p, _ in self.groups], dtype=np.int32)
        sizes = np.asarray([len(rs) for _, rs in self.groups], dtype=np.int32)
        resp = np.asarray([n for _, rs in self.groups for n in rs], dtype=np.int32)
        self.num_tokens = int(prompt.sum()) + int(resp.sum())
        self.num_query_rows = int(resp.sum()) if self.responses_only else self.num_tokens
        self.num_tiles = (self.num_tokens + 31) // 32
        lib = _lib.load_library()
        n = ctypes.c_int64()
        _lib.check(lib.fca_split_layout_ints(self.num_tokens, ctypes.byref(n)))
        self.host = np.zeros(max(int(n.value), 1), dtype=np.int32)
        _lib.check(
            lib.fca_split_layout_build(
                len(self.groups), prompt.ctypes.data, sizes.ctypes.data, resp.ctypes.data, self.num_tokens,
                1 if self.responses_only else 0, self.window, self.host.ctypes.data,
            )
        )
        self.device = torch.device(device)
        self.dev = torch.from_numpy(self.host).to(self.device) if self.device.type == "cuda" else None
        # original batch index of every sample, group by group (None: numbered in layout order)
        self.sample_ids = None
        self._scratch = {} if scratch_pool is None else scratch_pool

    @classmethod
    def from_group_token_layout(cls, layout, device="cuda", sliding_window=None):
        return cls([(g["prompt_tokens"], g["response_tokens"]) for g in layout], device=device, sliding_window=sliding_window)

    @classmethod
    def from_reconstruction_info(cls, reconstruction_info, device="cuda", sliding_window=None):
        """From the trainer's ``reconstruction_info`` itself: ``prompt_groups`` (lists of sample
        indices) and ``segment_info`` (dicts with ``group_idx``, ``type`` "prompt" / "response",
        ``original_idx`` and ``num_valid_tokens``, or ``start`` / ``end`` before unpadding), read the
        way ``ZoRRoTrain.get_group_token_layout`` reads them (zorro_train.py:2409-2436): the
        prompt's count from the group's first sample, one response count per sample in group order."""

        def valid(seg):
            return int(seg["num_valid_tokens"] if "num_valid_tokens" in seg else seg["end"] - seg["start"])

        segs = {(s["group_idx"], s["type"], s["original_idx"]): s for s in reconstruction_info["segment_info"]}
        groups = []
        for g, members in enumerate(reconstruction_info["prompt_groups"]):
            prompt = valid(segs[(g, "prompt", members[0])])
            groups.append((prompt, [valid(segs[(g, "response", m)]) for m in members]))
        layout = cls(groups, device=device, sliding_window=sliding_window)
        layout.sample_ids = [[int(m) for m in members] for members in reconstruction_info["prompt_groups"]]
        return layout

    # views of the layout array (tests, inspection)
    def kv_lim(self):
        return self.host[: 32 * self.num_tiles]

    def q_tiles(self):
        o = 32 * self.num_tiles
        return self.host[o : o + 4 * self.num_tiles].reshape(-1, 4)

    def kv_qend(self):
        o = 36 * self.num_tiles
        return self.host[o : o + self.num_tiles]

    def q_order(self):
        o = 37 * self.num_tiles
        return self.host[o : o + self.num_tiles]

    def kv_limmin(self):
        o = 38 * self.num_tiles
        return self.host[o : o + self.num_tiles]

    def kv_order(self):
        o = 39 * self.num_tiles
        return self.host[o : o + (self.num_tiles + 3) // 4]

    def q_index(self):
        o = 40 * self.num_tiles
        return self.host[o : o + 32 * self.num_tiles]

    def pos(self):
        o = 72 * self.num_tiles
        return self.host[o : o + 32 * self.num_tiles]

    def scratch(self, plan, backward: bool) -> torch.Tensor:
        """Scratch of a call, kept with the layout: layers run one after the other on a stream."""
        fwd, bwd = ctypes.c_size_t(), ctypes.c_size_t()
        _lib.check(_lib.load_library().fca_split_workspace_bytes(ctypes.byref(plan), ctypes.byref(fwd), ctypes.byref(bwd)))
        need = bwd.value if backward else fwd.value
        key = "bwd" if backward else "fwd"
        buf = self._scratch.get(key)
        if buf is None or buf.numel() < need:
            buf = self._scratch[key] = torch.empty(max(need, 16), dtype=torch.uint8, device=self.device)
        return buf


def _check_rows(name, x, tokens):
    if x.dtype != torch.bfloat16 or x.dim() != 3 or x.shape[0] != tokens:
        raise ValueError(f"{name} must be bfloat16 [T, H, D] with T = {tokens}, got {tuple(x.shape)} {x.dtype}")
    if not x.is_cuda:
        raise RuntimeError(f"split attention runs on the GPU; {name} must be a device tensor")
    if x.stride(2) != 1 or x.stride(1) != x.shape[2]:
        raise ValueError(f"the heads of a token of {name} must be contiguous")


def _check_heads(q, k, v):
    if k.shape != v.shape or k.shape[2] != q.shape[2]:
        raise ValueError(f"k and v must have one shape and the head size of q, got q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")


def _plan(q, k, layout, dropout=0.0, seed=0):
    dropout = float(dropout or 0.0)
    if not 0.0 <= dropout < 1.0:
        raise ValueError(f"attention dropout must lie in [0, 1), got {dropout}")
    return _lib.FcaSplitPlan(layout.num_tokens, q.shape[1], k.shape[1], q.shape[2], layout.window, dropout, int(seed) & 0xFFFFFFFF)


def dropout_keep_mask(seed: int, dropout: float, num_q_heads: int, num_tokens: int) -> torch.Tensor:
    """The mask the kernels apply for ``dropout`` and ``seed``: bool ``[Hq, T, T]``, entry
    (h, r, t) true when the probability of row r and key t (places in the deduplicated order)
    survives in query head h.  The hash of include/zorro_fca.h restated on the host, for
    callers that want to see or reproduce what a step dropped."""
    thr = min(int(float(dropout) * 4294967296.0), 4294967295) if dropout > 0 else 0
    if dropout > 0:
        thr = max(thr, 1)
    m = 0xFFFFFFFF
    h = np.arange(num_q_heads, dtype=np.uint64)[:, None, None]
    r = np.arange(num_tokens, dtype=np.uint64)[None, :, None]
    t = np.arange(num_tokens, dtype=np.uint64)[None, None, :]
    x = ((int(seed) & m) + h * 0xC2B2AE3D + r * 0x9E3779B1 + t * 0x85EBCA77) & m
    x ^= x >> 16
    x = (x * 0x7FEB352D) & m
    x ^= x >> 15
    x = (x * 0x846CA68B) & m
    x ^= x >> 16
    return torch.from_numpy(x >= thr)


def split_attention_forward(q, k, v, layout: SplitLayout, scale: float, out=None, dropout: float = 0.0, seed: int = 0):
    """q ``[T, Hq, D]``, k, v ``[T, Hkv, D]`` bf16 in deduplicated order.  Returns
    ``(out [T, Hq, D] bf16, lse fp32 [Hq, 32 * ceil(T / 32)])``; ``lse[:, :T]`` is the
    natural-log log-sum-exp of every row's scores.  ``out`` may be given to write into.
    ``dropout`` > 0 drops attention probabilities after the softmax (``seed`` decides which;
    the backward needs the same two values)."""
    t, rows = layout.num_tokens, layout.num_query_rows
    _check_rows("q", q, rows)
    for name, x in (("k", k), ("v", v)):
        _check_rows(name, x, t)
    _check_heads(q, k, v)
    plan = _plan(q, k, layout, dropout, seed)
    if out is None:
        out = torch.empty((rows, q.shape[1], q.shape[2]), dtype=torch.bfloat16, device=q.device)
    else:
        _check_rows("out", out, rows)
        if out.shape != q.shape:
            raise ValueError(f"out must have the shape of q, got {tuple(out.shape)} against {tuple(q.shape)}")
    lse = torch.empty((q.shape[1], 32 * layout.num_tiles), dtype=torch.float32, device=q.device)
    if t == 0:
        return out, lse
    _lib.check(
        _lib.load_library().fca_split_attention_forward(
            ctypes.byref(plan), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
            layout.dev.data_ptr(), float(scale), layout.scratch(plan, False).data_ptr(), out.data_ptr(), out.stride(0),
            lse.data_ptr(), _stream_ptr(q.device),
        )
    )
    return out, lse


def split_attention_backward(dout, q, k, v, out, lse, layout: SplitLayout, scale: float, dropout: float = 0.0, seed: int = 0):
    """Gradients ``(dq, dk, dv)`` of ``split_attention_forward``'s ``out`` with respect to
    its inputs, for the upstream gradient ``dout`` (``dropout`` and ``seed`` as in the forward)."""
    if layout.responses_only:
        raise ValueError("a layout with responses_only serves the forward only")
    t = layout.num_tokens
    for name, x in (("q", q), ("k", k), ("v", v), ("out", out), ("dout", dout)):
        _check_rows(name, x, t)
    _check_heads(q, k, v)
    if out.shape != q.shape or dout.shape != q.shape:
        raise ValueError("out and dout must have the shape of q")
    plan = _plan(q, k, layout, dropout, seed)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    for name, x in (("dq", dq), ("dk", dk), ("dv", dv)):
        _check_rows(name, x, t)
    if t == 0:
        return dq, dk, dv
    _lib.check(
        _lib.load_library().fca_split_attention_backward(
            ctypes.byref(plan), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
            out.data_ptr(), out.stride(0), dout.data_ptr(), dout.stride(0), lse.data_ptr(), layout.dev.data_ptr(),
            float(scale), layout.scratch(plan, True).data_ptr(), dq.data_ptr(), dq.stride(0), dk.data_ptr(), dk.stride(0),
            dv.data_ptr(), dv.stride(0), _stream_ptr(q.device),
        )
    )
    return dq, dk, dv


class _SplitAttention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, layout, scale, dropout=0.0, seed=0):
        out, lse = split_attention_forward(q, k, v, layout, scale, dropout=dropout, seed=seed)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.layout, ctx.scale, ctx.dropout, ctx.seed = layout, scale, dropout, seed
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse = ctx.saved_tensors
        if dout.stride(2) != 1 or dout.stride(1) != dout.shape[2]:
            dout = dout.contiguous()
        dq, dk, dv = split_attention_backward(dout, q, k, v, out, lse, ctx.layout, ctx.scale, ctx.dropout, ctx.seed)
        return dq, dk, dv, None, None, None, None


def _check_call_arguments(dropout, sliding_window, layout):
    """The trainer hands both to its attention calls on every step
    (qwen_attention_patcher.py:1204-1206, :1224-1226).  The window is a property of the layout
    (its walks are cut to it), so the call's value must be the one the layout was made for."""
    if dropout is not None and not 0.0 <= float(dropout) < 1.0:
        raise ValueError(f"attention dropout must lie in [0, 1), got {dropout}")
    want = 0 if sliding_window is None else int(sliding_window)
    if want != layout.window:
        raise ValueError(
            f"sliding_window={sliding_window} but the layout was made for "
            f"{layout.window or None}: pass sliding_window to SplitLayout as well"
        )


def split_attention(q, k, v, layout: SplitLayout, scale: float, dropout: float = 0.0, sliding_window=None, seed=None):
    """Differentiable split attention: ``out [T, Hq, D]`` in deduplicated order.  ``dropout``
    and ``sliding_window`` are the arguments of the trainer's attention calls
    (``0.0 if not module.training else module.attention_dropout``; the window must be the one
    ``layout`` was made for).  With dropout, ``seed`` decides which probabilities fall (drawn
    from torch's CPU generator when not given, so ``torch.manual_seed`` makes a run repeatable);
    the backward reuses it."""
    _check_call_arguments(dropout, sliding_window, layout)
    dropout = float(dropout or 0.0)
    if dropout > 0.0 and seed is None:
        seed = int(torch.randint(0, 2**31 - 1, (1,)).item())
    return _SplitAttention.apply(q, k, v, layout, scale, dropout, int(seed or 0))


def split_attention_padded(q, k, v, valid, layout: SplitLayout, scale: float, dropout: float = 0.0, sliding_window=None, seed=None):
    """The same attention for a deduplicated batch that still carries its padding (the
    trainer's padded variant, qwen_attention_patcher.py:881-1040, which masks the padding inside
    its two attention calls): ``q``, ``k``, ``v`` are ``[T_padded, H, D]``, ``valid`` a bool
    ``[T_padded]`` (the deduplicated attention mask, zorro_train.py:359-372), ``layout`` counts
    the valid tokens.  The valid rows are gathered, attended, and scattered back; padding rows
    of the result are zero and receive no gradient.  Differentiable."""
    _check_call_arguments(dropout, sliding_window, layout)
    index = torch.nonzero(valid, as_tuple=False).squeeze(-1)
    if index.numel() != layout.num_tokens:
        raise ValueError(f"{index.numel()} valid tokens, the layout counts {layout.num_tokens}")
    out = split_attention(q.index_select(0, index), k.index_select(0, index), v.index_select(0, index), layout, scale, dropout, sliding_window, seed)
    return torch.zeros_like(q).index_copy(0, index, out)
