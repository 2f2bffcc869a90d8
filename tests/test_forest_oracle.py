"""Shared-prefix discovery oracle: literal groupings from the reference's own tests,
hand-built forests, and invariants on generated workloads."""

import random

import torch

from arctic_platform_amd.workloads import make_config, page_forest, three_level_forest, two_level_forest
from oracle.forest import canonical_nodes, discover_forest, prompt_groups, unique_tokens


def _table(prompts, suffix_blocks=2, prompt_blocks=4):
    """Block tables for sequences given by prompt id: equal prompts share their blocks."""
    next_id = [100]
    shared = {}
    rows, lens = [], []
    for p in prompts:
        if p not in shared:
            shared[p] = list(range(next_id[0], next_id[0] + prompt_blocks))
            next_id[0] += prompt_blocks
        private = list(range(next_id[0], next_id[0] + suffix_blocks))
        next_id[0] += suffix_blocks
        rows.append(shared[p] + private)
        lens.append((prompt_blocks + suffix_blocks) * 16 - 3)
    return rows, lens


def test_reference_grouping_literals():
    # the three expectations of tests/zorro_train/test_dedup.py:76-104
    assert prompt_groups(*_table([0, 0, 0, 1, 1, 1])) == [[0, 1, 2], [3, 4, 5]]
    assert prompt_groups(*_table([0, 1, 2, 3])) == [[0], [1], [2], [3]]
    assert prompt_groups(*_table([0, 0, 0, 0, 0])) == [[0, 1, 2, 3, 4]]


def test_non_contiguous_groups_keep_first_seen_order():
    # samples 0,2 share one prompt and 1,3 another (tests/zorro_train/test_dedup.py:226-229)
    assert prompt_groups(*_table([7, 9, 7, 9])) == [[0, 2], [1, 3]]


def test_hand_built_three_level():
    #      blocks:  sys(2)  seg(3)   private
    rows = [
        [1, 2, 10, 11, 12, 50, 51],
        [1, 2, 10, 11, 12, 60],
        [1, 2, 20, 21, 22, 70],
        [1, 2, 20, 21, 22, 80, 81],
        [1, 2, 30, 31],
    ]
    lens = [16 * 7 - 1, 16 * 6, 16 * 5 + 1, 16 * 7, 16 * 3 + 5]
    nodes, leaves = discover_forest(rows, lens)
    assert canonical_nodes(nodes) == sorted([((0, 1, 2, 3, 4), 0, 2), ((0, 1), 2, 3), ((2, 3), 2, 3)])
    assert [l["blk_start"] for l in leaves] == [5, 5, 5, 5, 2]
    assert [l["tokens"] for l in leaves] == [31, 16, 1, 32, 21]
    for n in nodes:
        assert n["level"] == (0 if len(n["members"]) == 5 else 1)


def test_partial_block_is_never_shared_and_short_member_limits_run():
    rows = [[5, 6, 7, 8], [5, 6, 7, 9], [5, 6, 0, 0]]
    lens = [64, 60, 31]  # sequence 2 has one full block only
    nodes, leaves = discover_forest(rows, lens)
    assert canonical_nodes(nodes) == sorted([((0, 1, 2), 0, 1), ((0, 1), 1, 2)])
    assert [l["tokens"] for l in leaves] == [16, 12, 15]


def test_level_cap_and_no_sharing():
    rows, lens = _table([0, 0, 1, 1])
    nodes, leaves = discover_forest(rows, lens, max_levels=0)
    assert nodes == [] and [l["blk_start"] for l in leaves] == [0, 0, 0, 0]
    assert unique_tokens(nodes, leaves) == sum(lens)


def test_invariants_on_generated_forests():
    for seed in range(6):
        gen = torch.Generator().manual_seed(seed)
        if seed % 2:
            seg, paths = three_level_forest(gen, 40, 3, 3, (17, 90), (1, 70))
        else:
            seg, paths = two_level_forest(gen, 4, 3, (5, 120), (1, 50))
        table, lens, slot_src, _ = page_forest(seg, paths, gen)
        nodes, leaves = discover_forest(table.tolist(), lens.tolist())
        # path concatenation reproduces every block-table row; lengths add up
        on_path = {s: [] for s in range(len(lens))}
        for n in nodes:
            for s in n["members"]:
                on_path[s].append((n["blk_start"], n["num_blocks"]))
        for s, n_tok in enumerate(lens.tolist()):
            pos = 0
            for start, count in sorted(on_path[s]):
                assert start == pos
                pos += count
            assert leaves[s]["blk_start"] == pos and leaves[s]["tokens"] == n_tok - 16 * pos
        assert unique_tokens(nodes, leaves) == int((slot_src >= 0).sum())
        # invariant under a permutation of the sequences and a relabelling of block ids
        order = list(range(len(lens)))
        random.Random(seed).shuffle(order)
        relabel = random.Random(seed + 1).sample(range(10000), int(table.max()) + 1)
        t2 = [[relabel[b] for b in table[s].tolist()] for s in order]
        nodes2, _ = discover_forest(t2, [int(lens[s]) for s in order])
        back = [(tuple(sorted(order[m] for m in n["members"])), n["blk_start"], n["num_blocks"]) for n in nodes2]
        assert sorted(back) == canonical_nodes(nodes)


def test_workload_unique_tokens_match_definition():
    w = make_config(4, shrink=16)
    nodes, leaves = discover_forest(w.block_table.tolist(), w.seq_lens.tolist())
    assert unique_tokens(nodes, leaves) == w.unique_tokens
    assert max(n["level"] for n in nodes) == 1 and len([n for n in nodes if n["level"] == 0]) == 1
