"""Shared helpers of the parity tests: tolerances and oracle adapters."""

import torch

from oracle.attention import flat_decode_attention

# Stated tolerances of this path: bf16 outputs within rtol 2e-2 / atol 2e-2 of the fp64
# oracle on the same (already rounded) inputs, fp32 log-sum-exp within 1e-3.
OUT_RTOL = 2e-2
OUT_ATOL = 2e-2
LSE_ATOL = 1e-3


def oracle_for(w, seqs=None):
    """fp64 flat attention on a workload's own tensors (moved to the CPU)."""
    return flat_decode_attention(
        w.q.cpu(),
        w.kv_cache.cpu(),
        w.block_table.cpu(),
        w.seq_lens.cpu(),
        w.scale,
        None if w.k_scale is None else w.k_scale.cpu(),
        None if w.v_scale is None else w.v_scale.cpu(),
        seqs=seqs,
    )


def assert_matches_oracle(out, lse, ref_out, ref_lse, seqs=None, what=""):
    out = out.detach().cpu().double()
    lse = lse.detach().cpu().double()
    if seqs is not None:
        idx = torch.as_tensor(list(seqs))
        out, lse, ref_out, ref_lse = out[idx], lse[idx], ref_out[idx], ref_lse[idx]
    assert torch.isfinite(out).all(), f"{what}: non-finite output"
    err = (out - ref_out).abs()
    tol = OUT_ATOL + OUT_RTOL * ref_out.abs()
    assert (err <= tol).all(), f"{what}: out max abs err {err.max():.4g} (worst excess {(err - tol).max():.4g})"
    lerr = (lse - ref_lse).abs().max()
    assert lerr <= LSE_ATOL, f"{what}: lse max abs err {lerr:.4g}"
    return float(err.max()), float(lerr)


def oracle_for_sample(w, seqs):
    """Oracle on a few rows of a large workload: only the blocks those rows use are
    brought to the CPU (block ids are renumbered; values are untouched)."""
    seqs = list(seqs)
    lens = w.seq_lens.cpu()
    table = w.block_table.cpu()
    need = sorted({int(b) for s in seqs for b in table[s, : (int(lens[s]) + 15) // 16].tolist()})
    remap = torch.zeros(w.kv_cache.shape[1], dtype=torch.long)
    remap[need] = torch.arange(len(need))
    cache = w.kv_cache[:, torch.as_tensor(need, device=w.kv_cache.device)].cpu()
    sub_table = remap[table[seqs].long()].to(torch.int32)
    return flat_decode_attention(
        w.q[seqs].cpu(),
        cache,
        sub_table,
        lens[seqs],
        w.scale,
        None if w.k_scale is None else w.k_scale.cpu(),
        None if w.v_scale is None else w.v_scale.cpu(),
    )
