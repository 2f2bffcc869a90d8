"""Shared-prefix discovery over block tables, by brute force with Python containers.

Grouping semantics follow the reference's prompt-group discovery: rows are compared with
the first member of each existing group, groups appear in first-seen order and members in
ascending row order (``ZoRRoTrain.find_prompt_groups``,
arctic_platform/rl/zorro_train/zorro_train.py:242-285; the hash-map variant
``create_prompt_groups``, arctic_platform/rl/zorro_train/seqlen_balancing.py:437-486).
Here the compared rows are leading runs of physical block ids instead of prompt tokens,
and the comparison is applied recursively, which turns the flat groups into a forest.

A node is a maximal run of leading block-table positions whose physical ids are identical
for a fixed set of two or more sequences.  Only full blocks can be shared.  What is left
of a sequence below its deepest shared node is its private leaf.

Query rows need not be block-table rows: with ``row_table`` query row r reads table row
``row_table[r]`` up to ``seq_lens[r]`` tokens (the tokens of a query run).  ``row_group``
declares groups among such rows.  A declared row takes part in the discovery above, but
the last block it may share there is the one before the block that holds its last token,
and a group made of nothing but declared rows of one table row is left alone.  After
discovery the declared rows meet under (node they ended in, group id).  A group whose
members are successive rows over one table row, each one token longer than the one before
it and all ending in one block, is a tile of a query run: its node runs from where
discovery left the rows to the last member's last token (``tokens``), is marked ``causal``
(each member attends only up to its own token) and leaves its members no leaf.  Any other
declared group gets a plain node over what its members still have in common.  The trainer's counterpart is the
response-over-shared-prompt attention, which reads each unique prompt once for all its
responses (arctic_platform/rl/zorro_train/qwen_attention_patcher.py:1117-1262).
"""

from __future__ import annotations

from collections import OrderedDict

BLOCK = 16


def discover_forest(block_table, seq_lens, block_size=BLOCK, max_levels=8, row_table=None, row_group=None):
    """Returns (nodes, leaves).

    nodes: list of dict(members, blk_start, num_blocks, tokens, causal, level, parent) for
    shared runs.  leaves: per sequence dict(blk_start, tokens, parent): the private remainder.
    """
    table = [list(map(int, row)) for row in block_table]
    lens = [int(n) for n in seq_lens]
    trow = list(range(len(lens))) if row_table is None else [int(r) for r in row_table]
    bt = [table[r] for r in trow]
    group_of = [-1] * len(lens) if row_group is None else [int(g) for g in row_group]
    nfull = [(max(n - 1, 0) if g >= 0 else n) // block_size for n, g in zip(lens, group_of)]
    nodes = []
    leaf_start = [0] * len(lens)
    leaf_parent = [-1] * len(lens)

    def common_run(group, pos):
        limit = min(nfull[s] for s in group) - pos
        first = group[0]
        run = 0
        while run < limit and all(bt[s][pos + run] == bt[first][pos + run] for s in group):
            run += 1
        return run

    def add_node(group, pos, run, tokens, causal, level, parent):
        nodes.append(dict(members=list(group), blk_start=pos, num_blocks=run, tokens=tokens, causal=causal, level=level, parent=parent))
        for s in group:
            leaf_start[s] = pos + run
            leaf_parent[s] = len(nodes) - 1
        return len(nodes) - 1

    def descend(members, pos, level, parent):
        if level >= max_levels:
            return
        groups = OrderedDict()
        for s in members:
            if pos < nfull[s]:
                groups.setdefault(bt[s][pos], []).append(s)
        for group in groups.values():
            if len(group) < 2:
                continue
            if all(group_of[s] >= 0 and trow[s] == trow[group[0]] for s in group):
                continue  # the rows of one query run: tiled by their declared groups below
            run = common_run(group, pos)
            node_id = add_node(group, pos, run, run * block_size, False, level, parent)
            descend(group, pos + run, level + 1, node_id)

    descend(list(range(len(lens))), 0, 0, -1)

    # declared groups, below whatever discovery found
    if max_levels > 0:
        declared = OrderedDict()
        for s in range(len(lens)):
            if group_of[s] >= 0 and lens[s] >= 1:
                declared.setdefault((leaf_parent[s], group_of[s]), []).append(s)
        for (parent, _), group in declared.items():
            if len(group) < 2:
                continue
            first, pos = group[0], leaf_start[group[0]]
            level = nodes[parent]["level"] + 1 if parent >= 0 else 0
            tile = all(
                s == first + i
                and trow[s] == trow[first]
                and lens[s] == lens[first] + i
                and (lens[s] - 1) // block_size == (lens[first] - 1) // block_size
                for i, s in enumerate(group)
            )
            run = common_run(group, pos)
            if tile:
                add_node(group, pos, run + 1, lens[group[-1]] - pos * block_size, True, level, parent)
            elif run > 0:
                add_node(group, pos, run, run * block_size, False, level, parent)

    leaves = [
        dict(blk_start=leaf_start[s], tokens=max(0, lens[s] - leaf_start[s] * block_size), parent=leaf_parent[s])
        for s in range(len(lens))
    ]
    return nodes, leaves


def prompt_groups(block_table, seq_lens, block_size=BLOCK):
    """Top-level groups only, in first-seen order with ascending members: the shape of
    the reference's ``prompt_groups`` result (zorro_train.py:262-283)."""
    nodes, _ = discover_forest(block_table, seq_lens, block_size, max_levels=1)
    group_of = {}
    for node in nodes:
        for s in node["members"]:
            group_of[s] = node["members"]
    out = []
    for s in range(len(seq_lens)):
        g = group_of.get(s, [s])
        if g[0] == s:  # a group is emitted when its first member comes up
            out.append(list(g))
    return out


def canonical_nodes(nodes):
    """Order-free form of a node list for comparisons."""
    return sorted((tuple(sorted(n["members"])), n["blk_start"], n["num_blocks"]) for n in nodes)


def unique_tokens(nodes, leaves, block_size=BLOCK):
    return sum(n.get("tokens", n["num_blocks"] * block_size) for n in nodes) + sum(l["tokens"] for l in leaves)
