"""Forest cascade decode attention operator.

``forest_cascade_decode`` is what an attention backend's per-layer ``forward`` calls for a
decode batch: one query token per sequence against the paged KV cache, using metadata
built once per scheduler step by ``build_forest_metadata``.  It sits where the platform's
sampling engine runs attention after ``ReplicaPool.generate``
(arctic_platform/common/ray_server.py:921-933) when the job was started with
``zorro_inference.enable`` (arctic_platform/common/utils/server_models.py:123-140).

Semantics: plain softmax attention with grouped KV heads, scale passed in, no mask
(arctic_platform/model/implementations/qwen35/models/qwen3_5_moe/modeling_qwen3_5_moe.py:
368-373, :385, :440-454); ``lse`` is the natural-log sum of exponentiated scaled scores.
"""

from __future__ import annotations

import ctypes

import torch

from . import _lib
from .forest import ForestMetadata, _stream_ptr
from .kv_layout import BLOCK_SIZE


def _tensors(q, kv_cache, meta: ForestMetadata, scale, k_scale, v_scale, f32_ok=False) -> _lib.FcaTensors:
    plan = meta.plan
    if q.dtype == torch.float32 or kv_cache.dtype == torch.float32:
        # the all-fp32 path: fp32 queries on an fp32 cache, fp32 partial rows
        if q.dtype != kv_cache.dtype:
            raise TypeError(f"the fp32 path takes q and the KV cache both in float32, got {q.dtype} and {kv_cache.dtype}")
        if not f32_ok:
            raise TypeError("float32 tensors run through forest_cascade_decode (and its static variant) only")
        kv_dtype = _lib.FCA_F32
    elif q.dtype != torch.bfloat16:
        raise TypeError("q must be bfloat16 (or float32 with a float32 KV cache)")
    elif kv_cache.dtype == torch.bfloat16:
        kv_dtype = _lib.FCA_BF16
    elif kv_cache.dtype == torch.float8_e4m3fn:
        kv_dtype = _lib.FCA_FP8_E4M3
    else:
        raise TypeError(f"unsupported KV cache dtype {kv_cache.dtype} (bfloat16, float8_e4m3fn, or float32 with a float32 q)")
    if q.shape != (plan.num_seqs, plan.num_q_heads, plan.head_dim) or q.stride(2) != 1:
        raise ValueError(f"q must be [{plan.num_seqs}, {plan.num_q_heads}, {plan.head_dim}] with contiguous head_dim")
    if (
        kv_cache.dim() != 4
        or kv_cache.shape[0] != 2
        or kv_cache.shape[2] != plan.num_kv_heads
        or kv_cache.shape[3] != BLOCK_SIZE * plan.head_dim
        or kv_cache.stride(3) != 1
    ):
        raise ValueError("kv_cache must be [2, num_blocks, num_kv_heads, 16 * head_dim] (see kv_layout)")
    if not (q.is_cuda and kv_cache.is_cuda):
        raise RuntimeError("forest cascade attention runs on the GPU only; q and kv_cache must be device tensors")
    for name, sc in (("k_scale", k_scale), ("v_scale", v_scale)):
        if sc is not None and (sc.dtype != torch.float32 or sc.shape != (plan.num_kv_heads,) or not sc.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous fp32 tensor of shape [{plan.num_kv_heads}]")
    esz = kv_cache.element_size()
    return _lib.FcaTensors(
        q.data_ptr(),
        q.stride(0),
        q.stride(1),
        kv_cache.data_ptr(),
        kv_cache.data_ptr() + kv_cache.stride(0) * esz,
        kv_cache.stride(1),
        kv_cache.stride(2),
        kv_dtype,
        1 if meta.kv_reread else 0,
        meta.block_table.data_ptr(),
        meta.block_table.stride(0),
        k_scale.data_ptr() if k_scale is not None else None,
        v_scale.data_ptr() if v_scale is not None else None,
        float(scale),
        1 if meta.reproducible else 0,
        int(meta.max_workgroups),
        int(meta.fp8_tile_buffers) if kv_dtype == _lib.FCA_FP8_E4M3 and plan.head_dim == 128 and plan.rows_per_item == 32 else 0,
    )


def _check_partials(meta: ForestMetadata, t) -> None:
    """fp32 tensors write fp32 partial rows: the workspace must have been sized for them."""
    want = torch.float32 if t.kv_dtype == _lib.FCA_F32 else torch.float16
    if meta.partial_out.dtype != want:
        raise ValueError(
            f"the metadata's partial rows are {meta.partial_out.dtype}, these tensors need {want}: "
            "build the metadata with partial_dtype=torch.float32 for float32 tensors (and without for the others)"
        )


def _out_args(q, meta, out, out_dtype):
    plan = meta.plan
    if out is None:
        out = torch.empty(plan.num_seqs, plan.num_q_heads, plan.head_dim, dtype=out_dtype or torch.bfloat16, device=q.device)
    if out.dtype == torch.bfloat16:
        code = _lib.FCA_BF16
    elif out.dtype == torch.float32:
        code = _lib.FCA_F32
    else:
        raise TypeError("out must be bfloat16 or float32")
    if out.shape != (plan.num_seqs, plan.num_q_heads, plan.head_dim) or out.stride(2) != 1:
        raise ValueError("out must be [num_seqs, num_q_heads, head_dim] with contiguous head_dim")
    return out, code


def forest_cascade_decode(
    q, kv_cache, meta: ForestMetadata, scale, k_scale=None, v_scale=None, out=None, return_lse=True, out_dtype=None
):
    """One layer's decode attention.  Returns ``out`` or ``(out, lse)``.  ``q`` and ``kv_cache``
    in float32 take the all-fp32 path (fp32 products and partial rows; ``out`` then defaults to
    float32): the metadata must have been built with ``partial_dtype=torch.float32``."""
    lib = _lib.load_library()
    t = _tensors(q, kv_cache, meta, scale, k_scale, v_scale, f32_ok=True)
    _check_partials(meta, t)
    out, code = _out_args(q, meta, out, out_dtype or (torch.float32 if t.kv_dtype == _lib.FCA_F32 else None))
    lse = torch.empty(meta.plan.num_seqs, meta.plan.num_q_heads, dtype=torch.float32, device=q.device) if return_lse else None
    _lib.check(
        lib.fca_decode_step(
            ctypes.byref(meta.plan),
            ctypes.byref(t),
            meta.meta.data_ptr(),
            meta.partial_out.data_ptr(),
            meta.partial_lse.data_ptr(),
            out.data_ptr(),
            out.stride(0),
            out.stride(1),
            code,
            lse.data_ptr() if lse is not None else None,
            _stream_ptr(q.device),
        )
    )
    return (out, lse) if return_lse else out


def forest_cascade_decode_static(q, kv_cache, meta: ForestMetadata, scale, k_scale=None, v_scale=None, *, out, lse=None):
    """``forest_cascade_decode`` on the library's own partial buffers
    (``fca_decode_step_static``): nothing is allocated, so ``out`` (and ``lse`` if wanted)
    must be passed in, and ``meta.partial_out`` / ``meta.partial_lse`` are not touched.
    Plans whose partial rows exceed ``_lib.FCA_STATIC_SCRATCH_BYTES`` raise.  All calls on
    one GPU share the buffers: keep them in stream order."""
    lib = _lib.load_library()
    t = _tensors(q, kv_cache, meta, scale, k_scale, v_scale, f32_ok=True)
    out, code = _out_args(q, meta, out, None)
    if lse is not None and (lse.dtype != torch.float32 or lse.shape != (meta.plan.num_seqs, meta.plan.num_q_heads) or not lse.is_contiguous()):
        raise ValueError("lse must be a contiguous fp32 tensor [num_seqs, num_q_heads]")
    _lib.check(
        lib.fca_decode_step_static(
            ctypes.byref(meta.plan), ctypes.byref(t), meta.meta.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1),
            code, lse.data_ptr() if lse is not None else None, _stream_ptr(q.device),
        )
    )
    return out if lse is None else (out, lse)


def prefix_pass(q, kv_cache, meta: ForestMetadata, scale, k_scale=None, v_scale=None):
    """Shared-node work items only; fills their slots of the partial buffers."""
    lib = _lib.load_library()
    t = _tensors(q, kv_cache, meta, scale, k_scale, v_scale)
    _lib.check(
        lib.fca_prefix_pass(
            ctypes.byref(meta.plan), ctypes.byref(t), meta.meta.data_ptr(), meta.partial_out.data_ptr(),
            meta.partial_lse.data_ptr(), _stream_ptr(q.device),
        )
    )


def suffix_pass(q, kv_cache, meta: ForestMetadata, scale, k_scale=None, v_scale=None):
    """Private-leaf work items only; fills their slots of the partial buffers."""
    lib = _lib.load_library()
    t = _tensors(q, kv_cache, meta, scale, k_scale, v_scale)
    _lib.check(
        lib.fca_suffix_pass(
            ctypes.byref(meta.plan), ctypes.byref(t), meta.meta.data_ptr(), meta.partial_out.data_ptr(),
            meta.partial_lse.data_ptr(), _stream_ptr(q.device),
        )
    )


def forest_pass(q, kv_cache, meta: ForestMetadata, scale, k_scale=None, v_scale=None):
    """Shared and private work items in one launch; fills every live partial slot."""
    lib = _lib.load_library()
    t = _tensors(q, kv_cache, meta, scale, k_scale, v_scale)
    _lib.check(
        lib.fca_forest_pass(
            ctypes.byref(meta.plan), ctypes.byref(t), meta.meta.data_ptr(), meta.partial_out.data_ptr(),
            meta.partial_lse.data_ptr(), _stream_ptr(q.device),
        )
    )


def merge_partials(meta: ForestMetadata, q_like, out=None, return_lse=True, out_dtype=None):
    """Log-sum-exp merge of the partial buffers into ``out`` (and ``lse``)."""
    if meta.partial_out.dtype != torch.float16:
        raise TypeError("merge_partials reads the half-precision partial rows of the bf16 / fp8 passes; fp32 rows are merged inside forest_cascade_decode")
    lib = _lib.load_library()
    out, code = _out_args(q_like, meta, out, out_dtype)
    lse = torch.empty(meta.plan.num_seqs, meta.plan.num_q_heads, dtype=torch.float32, device=out.device) if return_lse else None
    _lib.check(
        lib.fca_merge(
            ctypes.byref(meta.plan), meta.meta.data_ptr(), meta.partial_out.data_ptr(), meta.partial_lse.data_ptr(),
            out.data_ptr(), out.stride(0), out.stride(1), code, lse.data_ptr() if lse is not None else None,
            _stream_ptr(out.device),
        )
    )
    return (out, lse) if return_lse else out
