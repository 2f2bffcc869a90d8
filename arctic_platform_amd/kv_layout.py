"""Paged KV-cache layout read by the forest cascade kernels.

One cache tensor per layer, shape ``[2, num_blocks, num_kv_heads, block_size * head_dim]``
(plane 0 = K, plane 1 = V), block_size fixed at 16 tokens.  Inside one (block, kv head)
tile the element order is the MFMA operand order of gfx950, so a wavefront can load its
operands with one contiguous 16-byte read per lane and no shuffle:

* K tile: ``[head_dim / x, 16 tokens, x]`` with ``x = 16 bytes / element size`` (8 for bf16,
  16 for fp8).  For one 16-byte slice of the head dimension the 16 tokens are adjacent.
* V tile: ``[head_dim, 16 tokens]``.  For one channel the 16 tokens are adjacent, which is
  the contraction order of the ``P @ V`` product.

This is the split layout the vLLM ROCm paged-attention path uses for its cache, so a
stock ROCm backend can serve the prefill side of the same cache.

The attention-backend hook ``get_kv_cache_shape`` of the engine that the platform starts
(``arctic_platform/common/ray_server.py:395-404``) is where this shape is announced.
"""

from __future__ import annotations

import torch

BLOCK_SIZE = 16


def x_width(dtype: torch.dtype) -> int:
    """Elements per 16-byte slice of the head dimension in a K tile."""
    return 16 // torch.empty((), dtype=dtype).element_size()


def kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_dim: int):
    if block_size != BLOCK_SIZE:
        raise ValueError(f"forest cascade attention supports block_size={BLOCK_SIZE} only, got {block_size}")
    return (2, num_blocks, num_kv_heads, block_size * head_dim)


def pack_blocks(k: torch.Tensor, v: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
    """Token-major blocks ``[num_blocks, 16, num_kv_heads, head_dim]`` -> cache tensor."""
    if k.shape != v.shape or k.dim() != 4 or k.shape[1] != BLOCK_SIZE:
        raise ValueError("k and v must both be [num_blocks, 16, num_kv_heads, head_dim]")
    dtype = dtype or k.dtype
    nb, bs, hkv, d = k.shape
    x = x_width(dtype)
    if d % x:
        raise ValueError(f"head_dim {d} is not a multiple of {x}")
    cache = torch.empty(kv_cache_shape(nb, bs, hkv, d), dtype=dtype, device=k.device)
    # K: [nb, tok, h, d/x, x] -> [nb, h, d/x, tok, x]
    cache[0].view(nb, hkv, d // x, bs, x).copy_(k.view(nb, bs, hkv, d // x, x).permute(0, 2, 3, 1, 4))
    # V: [nb, tok, h, d] -> [nb, h, d, tok]
    cache[1].view(nb, hkv, d, bs).copy_(v.permute(0, 2, 3, 1))
    return cache


def unpack_blocks(cache: torch.Tensor, head_dim: int):
    """Cache tensor -> token-major ``(k, v)`` blocks ``[num_blocks, 16, num_kv_heads, head_dim]``."""
    two, nb, hkv, tile = cache.shape
    if two != 2 or tile != BLOCK_SIZE * head_dim:
        raise ValueError("not a forest-cascade KV cache tensor")
    x = x_width(cache.dtype)
    k = cache[0].view(nb, hkv, head_dim // x, BLOCK_SIZE, x).permute(0, 3, 1, 2, 4).reshape(nb, BLOCK_SIZE, hkv, head_dim)
    v = cache[1].view(nb, hkv, head_dim, BLOCK_SIZE).permute(0, 3, 1, 2)
    return k, v


def convert_cache(cache: torch.Tensor, head_dim: int, dtype: torch.dtype) -> torch.Tensor:
    """Re-pack a cache for another element type (the slice width ``x`` depends on it)."""
    k, v = unpack_blocks(cache, head_dim)
    return pack_blocks(k.to(dtype), v.to(dtype), dtype)
