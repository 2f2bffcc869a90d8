"""CPU restatement of the KV-cache append: token-major write into 16-token blocks, then
the tile order of the cache; fp8 caches store clamp(x / scale, +-448) rounded to the
nearest e4m3 value (ties to even), which is what ``torch.Tensor.to(float8_e4m3fn)`` does.

The reference holds no cache writer (the engine that owns the paged cache is external,
arctic_platform/common/ray_server.py:395-404); the layout is this build's own and the
expected bytes follow from its definition, so the check is bit-exact.
"""

from __future__ import annotations

import torch

BLOCK = 16
FP8_MAX = 448.0


def append_kv_reference(kv_cache, key, value, slot_mapping, k_scale=None, v_scale=None):
    """Returns a new cache tensor with the tokens written.  Written independently of the
    package's pack/unpack helpers: element offsets come straight from the layout."""
    out = kv_cache.clone()
    raw = out.view(torch.uint8) if out.element_size() == 1 else out
    d = key.shape[2]
    x = 16 // out.element_size()
    fp8 = out.dtype == torch.float8_e4m3fn
    for t, slot in enumerate(slot_mapping.tolist()):
        if slot < 0:
            continue
        blk, off = divmod(slot, BLOCK)
        for h in range(key.shape[1]):
            k, v = key[t, h].float(), value[t, h].float()
            if fp8:
                ks = 1.0 if k_scale is None else float(k_scale[h])
                vs = 1.0 if v_scale is None else float(v_scale[h])
                k = (k / torch.tensor(ks, dtype=torch.float32)).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn).view(torch.uint8)
                v = (v / torch.tensor(vs, dtype=torch.float32)).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn).view(torch.uint8)
            else:
                k, v = k.to(out.dtype), v.to(out.dtype)
            ktile, vtile = raw[0, blk, h], raw[1, blk, h]
            for ch in range(d):
                ktile[(ch // x) * BLOCK * x + off * x + ch % x] = k[ch]
                vtile[ch * BLOCK + off] = v[ch]
    return out
