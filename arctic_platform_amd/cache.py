"""KV-cache writer for the forest cascade layout.

``append_kv`` is the per-layer step that precedes decode attention: it scatters the new
tokens' K and V into the paged cache at the slots the scheduler assigned
(slot = physical_block * 16 + offset, negative = padding), in the tile order the
attention kernel reads, quantising to fp8 e4m3 when the cache is fp8.  The platform only
forwards the cache dtype to its engine (``vllm_config`` through ``build_model_config``,
arctic_platform/common/utils/server_models.py:143-165); the write itself happens in the
engine's attention backend, which is what this call replaces.
"""

from __future__ import annotations

import torch

from . import _lib
from .forest import _stream_ptr
from .kv_layout import BLOCK_SIZE


def gather_kv(kv_cache, slot_mapping, head_dim, k_scale=None, v_scale=None, out=None):
    """The way back: bf16 ``(key, value)`` rows ``[T, Hkv, D]`` of the tokens at ``slot_mapping``
    (fp8 caches times their scales: the values decode attention sees; negative slot = zeros)."""
    hkv = kv_cache.shape[2]
    t = slot_mapping.shape[0]
    if out is None:
        rows_dtype = torch.float32 if kv_cache.dtype == torch.float32 else torch.bfloat16
        out = tuple(torch.empty(t, hkv, head_dim, dtype=rows_dtype, device=kv_cache.device) for _ in range(2))
    _cache_rows(True, out[0], out[1], kv_cache, slot_mapping, k_scale, v_scale)
    return out


def append_kv(key, value, kv_cache, slot_mapping, k_scale=None, v_scale=None) -> None:
    """key, value: bf16 ``[T, Hkv, D]`` (float32 for a float32 cache); slot_mapping: int64 ``[T]``;
    kv_cache as in kv_layout."""
    _cache_rows(False, key, value, kv_cache, slot_mapping, k_scale, v_scale)


def _cache_rows(gather, key, value, kv_cache, slot_mapping, k_scale, v_scale) -> None:
    f32 = kv_cache.dtype == torch.float32
    rows_dtype = torch.float32 if f32 else torch.bfloat16
    if key.dtype != rows_dtype or value.dtype != rows_dtype or key.shape != value.shape or key.dim() != 3:
        raise TypeError(f"key and value must be {rows_dtype} tensors of the same shape [tokens, kv_heads, head_dim] for a {kv_cache.dtype} cache")
    if key.stride() != value.stride() or key.stride(2) != 1:
        raise ValueError("key and value must share strides and have a contiguous head_dim")
    t, hkv, d = key.shape
    if slot_mapping.dtype != torch.int64 or slot_mapping.shape != (t,) or not slot_mapping.is_contiguous():
        raise ValueError("slot_mapping must be a contiguous int64 tensor of shape [tokens]")
    if (
        kv_cache.dim() != 4
        or kv_cache.shape[0] != 2
        or kv_cache.shape[2] != hkv
        or kv_cache.shape[3] != BLOCK_SIZE * d
        or kv_cache.stride(3) != 1
    ):
        raise ValueError("kv_cache must be [2, num_blocks, num_kv_heads, 16 * head_dim] with contiguous tiles")
    if kv_cache.dtype == torch.bfloat16:
        code = _lib.FCA_BF16
    elif kv_cache.dtype == torch.float8_e4m3fn:
        code = _lib.FCA_FP8_E4M3
    elif f32:
        code = _lib.FCA_F32  # the all-fp32 path: fp32 rows, fp32 cache
    else:
        raise TypeError(f"unsupported KV cache dtype {kv_cache.dtype}")
    if not (key.is_cuda and kv_cache.is_cuda and slot_mapping.is_cuda):
        raise RuntimeError("append_kv runs on the GPU only")
    for name, sc in (("k_scale", k_scale), ("v_scale", v_scale)):
        if sc is not None and (sc.dtype != torch.float32 or sc.shape != (hkv,) or not sc.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous fp32 tensor of shape [{hkv}]")
    lib = _lib.load_library()
    esz = kv_cache.element_size()
    _lib.check(
        (lib.fca_gather_kv if gather else lib.fca_append_kv)(
            key.data_ptr(), value.data_ptr(), key.stride(0), key.stride(1), t, hkv, d, slot_mapping.data_ptr(),
            kv_cache.data_ptr(), kv_cache.data_ptr() + kv_cache.stride(0) * esz, kv_cache.stride(1), kv_cache.stride(2),
            code, k_scale.data_ptr() if k_scale is not None else None, v_scale.data_ptr() if v_scale is not None else None,
            _stream_ptr(key.device),
        )
    )
