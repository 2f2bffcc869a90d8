"""Committed golden vectors: the oracle and the generator must keep reproducing them."""

import hashlib
import os

import numpy as np
import torch

from arctic_platform_amd.kv_layout import pack_blocks
from arctic_platform_amd.workloads import make_config
from oracle.attention import flat_decode_attention
from oracle.cascade import cascade_decode_attention

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _sha(t):
    return hashlib.sha256(t.contiguous().view(torch.uint8).numpy().tobytes()).hexdigest()


def micro_cases():
    z = np.load(os.path.join(HERE, "micro.npz"))
    names = sorted({k.split(".")[0] for k in z.files})
    for name in names:
        c = {k.split(".", 1)[1]: torch.from_numpy(z[k]) for k in z.files if k.startswith(name + ".")}
        for kv in ("k_blocks", "v_blocks"):
            c[kv] = c.pop(kv + "_bf16").view(torch.bfloat16).float()
        yield name, c


def test_config1_generator_is_reproducible():
    z = np.load(os.path.join(HERE, "config1.npz"))
    w = make_config(1)
    assert w.seq_lens.tolist() == z["seq_lens"].tolist() == [576] * 4
    assert np.array_equal(w.block_table.numpy(), z["block_table"])
    assert _sha(w.q) == str(z["q_sha256"]) and _sha(w.kv_cache) == str(z["cache_sha256"])
    assert w.unique_tokens == 512 + 4 * 64 and w.flat_tokens == 4 * 576


def test_config1_oracle_matches_golden():
    z = np.load(os.path.join(HERE, "config1.npz"))
    w = make_config(1)
    out, lse = flat_decode_attention(w.q, w.kv_cache, w.block_table, w.seq_lens, w.scale)
    assert np.allclose(out.numpy(), z["out"], rtol=0, atol=1e-12) and np.allclose(lse.numpy(), z["lse"], rtol=0, atol=1e-12)
    cout, clse, nodes, _ = cascade_decode_attention(w.q, w.kv_cache, w.block_table, w.seq_lens, w.scale, chunk_tokens=80)
    assert np.allclose(cout.numpy(), z["out"], atol=1e-10) and np.allclose(clse.numpy(), z["lse"], atol=1e-10)
    assert len(nodes) == 1 and nodes[0]["num_blocks"] == 32


def test_micro_cases_oracle_matches_golden():
    seen = 0
    for name, c in micro_cases():
        d = c["q"].shape[-1]
        cache = pack_blocks(c["k_blocks"], c["v_blocks"], torch.float32)
        out, lse = flat_decode_attention(c["q"], cache, c["block_table"], c["seq_lens"], d**-0.5)
        assert torch.allclose(out, c["out"], rtol=0, atol=1e-12), name
        assert torch.allclose(lse, c["lse"], rtol=0, atol=1e-12), name
        cout, clse, _, _ = cascade_decode_attention(c["q"], cache, c["block_table"], c["seq_lens"], d**-0.5)
        assert torch.allclose(cout, c["out"], atol=1e-10) and torch.allclose(clse, c["lse"], atol=1e-10), name
        seen += 1
    assert seen == 5
