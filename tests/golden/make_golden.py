"""Regenerates the golden fixtures in this directory from the CPU oracle.

    python tests/golden/make_golden.py

config1.npz  - benchmark configuration 1 (fp32): lengths, block table, SHA-256 of the
               generated q and cache bytes, oracle out [4, 8, 64] and lse [4, 8].
micro.npz    - small hand-shaped cases with all inputs stored (values are exactly
               representable in bf16, so the GPU kernels can be fed the same numbers):
               single token, ragged private sequences, a three-level forest with ragged
               tails, fully shared sequences with empty leaves, interleaved groups.
Nothing here comes from the reference: the expected values are this repository's own
fp64 oracle, which tests/test_oracle.py pins against independent routes.
"""

import hashlib
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from arctic_platform_amd.kv_layout import pack_blocks  # noqa: E402
from arctic_platform_amd.workloads import make_config  # noqa: E402
from oracle.attention import flat_decode_attention  # noqa: E402


def sha(t):
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def config1():
    w = make_config(1)
    out, lse = flat_decode_attention(w.q, w.kv_cache, w.block_table, w.seq_lens, w.scale)
    np.savez(
        os.path.join(HERE, "config1.npz"),
        seed=1001,
        seq_lens=w.seq_lens.numpy(),
        block_table=w.block_table.numpy(),
        q_sha256=sha(w.q),
        cache_sha256=sha(w.kv_cache),
        out=out.numpy(),
        lse=lse.numpy(),
    )


MICRO = {
    # name: (Hq, Hkv, D, rows of block ids, lengths)
    "single_token": (4, 1, 64, [[3]], [1]),
    "ragged_private": (8, 2, 64, [[0, 9, 9], [1, 9, 9], [2, 4, 7]], [1, 16, 33]),
    "three_level": (
        8,
        2,
        128,
        [[1, 2, 10, 11, 12, 5, 6], [1, 2, 10, 11, 12, 7, 0], [1, 2, 3, 4, 16, 8, 0], [1, 2, 3, 4, 16, 9, 13], [1, 2, 14, 15, 0, 0, 0]],
        [16 * 7 - 1, 16 * 6, 16 * 5 + 1, 16 * 7, 16 * 3 + 5],
    ),
    "fully_shared": (8, 2, 64, [[4, 5], [4, 5], [4, 5]], [32, 32, 32]),
    "interleaved_groups": (4, 2, 64, [[1, 2, 3], [5, 6, 7], [1, 2, 8], [5, 6, 9]], [40, 47, 48, 33]),
}


def micro():
    store = {}
    for i, (name, (hq, hkv, d, rows, lens)) in enumerate(MICRO.items()):
        g = torch.Generator().manual_seed(7000 + i)
        nb = max(max(r) for r in rows) + 2
        bf = lambda t: t.to(torch.bfloat16).float()
        k = bf(torch.randn(nb, 16, hkv, d, generator=g))
        v = bf(torch.randn(nb, 16, hkv, d, generator=g))
        q = bf(torch.randn(len(rows), hq, d, generator=g))
        cache = pack_blocks(k, v, torch.float32)
        table = torch.tensor(rows, dtype=torch.int32)
        sl = torch.tensor(lens, dtype=torch.int32)
        out, lse = flat_decode_attention(q, cache, table, sl, d**-0.5)
        store.update(
            {
                f"{name}.q": q.numpy(),
                # bf16 bit patterns: half the size, and exactly what the kernels are fed
                f"{name}.k_blocks_bf16": k.to(torch.bfloat16).view(torch.int16).numpy(),
                f"{name}.v_blocks_bf16": v.to(torch.bfloat16).view(torch.int16).numpy(),
                f"{name}.block_table": table.numpy(),
                f"{name}.seq_lens": sl.numpy(),
                f"{name}.out": out.numpy(),
                f"{name}.lse": lse.numpy(),
            }
        )
    np.savez_compressed(os.path.join(HERE, "micro.npz"), **store)


if __name__ == "__main__":
    config1()
    micro()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
