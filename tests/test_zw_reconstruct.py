"""Whole samples from a deduplicated tensor and back: the index arrays (host code, no GPU
needed) against the CPU restatement of the reference's loops and against the properties the
reference's own tests assert, then the HIP gather and row-sum kernels on the GPU."""

import random

import numpy as np
import pytest
import torch

from arctic_platform_amd.split_attention import SplitLayout
from oracle.split_attention import deduplicate_packed, reconstruct_packed, total_tokens

LAYOUTS = [
    ([(6, [4, 4]), (6, [4, 4])], [[0, 2], [1, 3]]),  # the grouping of tests/zorro_train/test_dedup.py:76-88
    ([(5, [4, 1]), (6, [0, 3])], [[0, 2], [1, 3]]),  # the same after unpadding
    ([(40, [20, 33]), (7, [5])], None),
    ([(3, []), (2, [4])], None),  # a group without samples
    ([(0, [2, 0, 3])], [[2, 0, 1]]),  # no prompt, samples listed out of order
]


def _index(layout, ids):
    from arctic_platform_amd.reconstruct import SampleIndex

    return SampleIndex(SplitLayout(layout, device="cpu"), ids)


def _random_case(rng):
    layout = [(rng.choice([0, 1, 5, 33]), [rng.choice([0, 1, 3, 17]) for _ in range(rng.randint(0, 4))]) for _ in range(rng.randint(1, 4))]
    n = sum(len(rs) for _, rs in layout)
    perm = list(range(n))
    rng.shuffle(perm)
    ids, k = [], 0
    for _, rs in layout:
        ids.append(sorted(perm[k : k + len(rs)]))  # members of a group ascending, groups interleaved
        k += len(rs)
    return layout, ids


def test_index_arrays_against_the_reference_loops():
    rng = random.Random(3)
    cases = LAYOUTS + [_random_case(rng) for _ in range(60)]
    for layout, ids in cases:
        t = total_tokens(layout)
        if t == 0:
            continue
        ix = _index(layout, ids)
        x = torch.arange(t * 3, dtype=torch.float32).view(t, 3)
        want = reconstruct_packed(x, layout, ids)
        assert ix.num_dedup == t and ix.num_full == want.shape[0]
        assert torch.equal(x[torch.from_numpy(ix.full_from).long()], want), layout
        full = torch.randn(ix.num_full, 3, generator=torch.Generator().manual_seed(1))
        back = deduplicate_packed(full, layout, ids)
        src = torch.from_numpy(ix.dedup_from).long()
        padded = torch.cat([full, torch.zeros(1, 3)])  # -1: a row of zeros
        got = padded[torch.where(src >= 0, src, torch.tensor(ix.num_full))]
        assert torch.equal(got, back), layout
        # deduplicate is a left inverse of reconstruct (tests/zorro_train/test_dedup.py:138-156), where every group has a sample
        if all(rs for _, rs in layout):
            assert torch.equal(deduplicate_packed(want, layout, ids), x)
        # the copies of a deduplicated row are exactly the full rows that came from it
        for j in range(t):
            rows = ix.copies_rows[ix.copies_offsets[j] : ix.copies_offsets[j + 1]]
            assert sorted(rows.tolist()) == np.nonzero(ix.full_from == j)[0].tolist()
        # and a full row was taken by a deduplication exactly where dedup_from says so
        for i in range(ix.num_full):
            assert (ix.full_taken[i] >= 0) == bool((ix.dedup_from == i).any())
            if ix.full_taken[i] >= 0:
                assert ix.dedup_from[ix.full_taken[i]] == i


def test_reconstructed_embeddings_are_those_of_the_original_batch():
    """The reference's round trip (tests/zorro_train/test_dedup.py:108-136, unpadded): embedding the
    deduplicated ids and reconstructing gives, sample by sample, the embeddings of the sample's
    own prompt and response ids."""
    gen = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, 100, (6,), generator=gen) for _ in range(2)]
    groups = [[0, 2, 5], [1, 3, 4]]
    responses = {s: torch.randint(0, 100, (int(torch.randint(1, 5, (1,), generator=gen)),), generator=gen) for s in range(6)}
    layout = [(6, [len(responses[s]) for s in members]) for members in groups]
    dedup_ids = torch.cat([torch.cat([prompts[g]] + [responses[s] for s in members]) for g, members in enumerate(groups)])
    embedding = torch.randn(100, 4, generator=gen)
    ix = _index(layout, groups)
    got = embedding[dedup_ids][torch.from_numpy(ix.full_from).long()]
    group_of = {s: g for g, members in enumerate(groups) for s in members}
    want = torch.cat([embedding[torch.cat([prompts[group_of[s]], responses[s]])] for s in range(6)])
    assert torch.equal(got, want)


def test_layout_from_reconstruction_info_keeps_the_sample_indices():
    info = dict(
        prompt_groups=[[0, 2], [1, 3]],
        segment_info=[dict(group_idx=g, type=kind, original_idx=m, num_valid_tokens=n) for g, members in enumerate([[0, 2], [1, 3]])
                      for kind, n in (("prompt", 5), ("response", 3)) for m in members],
    )
    layout = SplitLayout.from_reconstruction_info(info, device="cpu")
    assert layout.sample_ids == [[0, 2], [1, 3]]
    from arctic_platform_amd.reconstruct import sample_index

    ix = sample_index(layout)
    # samples in batch order 0, 1, 2, 3: group 0's prompt, sample 0's response, group 1's prompt, sample 1's response, ...
    assert ix.full_from[:8].tolist() == [0, 1, 2, 3, 4, 5, 6, 7] and ix.full_from[8:16].tolist() == [11, 12, 13, 14, 15, 16, 17, 18]
    assert sample_index(layout) is ix
    with pytest.raises(ValueError, match="permutation"):
        _index([(2, [1, 1])], [[0, 2]])


# ---- the kernels (GPU) -----------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("dtype,shape", [(torch.bfloat16, (32, 128)), (torch.float32, (8,)), (torch.bfloat16, (2560,)), (torch.int32, (4,))])
def test_reconstruct_and_deduplicate_on_the_gpu(gpu, dtype, shape):
    from arctic_platform_amd.reconstruct import deduplicate_sequences, reconstruct_sequences

    rng = random.Random(11)
    for layout, ids in LAYOUTS + [_random_case(rng) for _ in range(6)]:
        t = total_tokens(layout)
        L = SplitLayout(layout)
        x = (torch.randn((t,) + shape, generator=torch.Generator().manual_seed(t)) * 100).to(dtype)
        got = reconstruct_sequences(x.to(gpu), L, ids)
        assert torch.equal(got.cpu(), reconstruct_packed(x, layout, ids)), layout
        batched = reconstruct_sequences(x.to(gpu).unsqueeze(0), L, ids)
        assert batched.shape[0] == 1 and torch.equal(batched[0], got)
        full = (torch.randn((got.shape[0],) + shape, generator=torch.Generator().manual_seed(t + 1)) * 100).to(dtype)
        back = deduplicate_sequences(full.to(gpu), L, ids)
        assert torch.equal(back.cpu(), deduplicate_packed(full, layout, ids)), layout


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_gradients_sum_over_the_copies_of_a_row(gpu, dtype):
    from arctic_platform_amd.reconstruct import deduplicate_sequences, reconstruct_sequences, sample_index

    layout, ids = [(40, [20, 33, 7]), (7, [5]), (3, [])], [[3, 0, 2], [1], []]
    L = SplitLayout(layout)
    ix = sample_index(L, ids)
    t = total_tokens(layout)
    x = torch.randn(t, 4, 16, generator=torch.Generator().manual_seed(2)).to(dtype).to(gpu).requires_grad_()
    full = reconstruct_sequences(x, L, ids)
    w = torch.randn(full.shape, generator=torch.Generator().manual_seed(3)).to(dtype).to(gpu)
    (full.float() * w.float()).sum().backward()
    # the same through torch's own indexing, summed in fp32 in the same order
    src = torch.from_numpy(ix.full_from).long().to(gpu)
    want = torch.zeros(t, 4, 16, dtype=torch.float32, device=gpu).index_add_(0, src, w.float())
    tol = dict(rtol=0, atol=0) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(x.grad.float(), want.to(dtype).float(), **tol)
    # deduplication: rows that were not taken get no gradient
    y = torch.randn(ix.num_full, 8, generator=torch.Generator().manual_seed(4)).to(dtype).to(gpu).requires_grad_()
    d = deduplicate_sequences(y, L, ids)
    g = torch.randn(d.shape, generator=torch.Generator().manual_seed(5)).to(dtype).to(gpu)
    d.backward(g)
    taken = torch.from_numpy(ix.full_taken).long().to(gpu)
    want = torch.where((taken >= 0)[:, None], g[taken.clamp(min=0)], torch.zeros(1, dtype=dtype, device=gpu))
    assert torch.equal(y.grad, want)
