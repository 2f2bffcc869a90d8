"""Forest metadata: block tables -> shared nodes, member lists and the work list.

Host-side face of ``fca_build_metadata``.  The discovery runs on the device with no
host synchronisation; this module only sizes the workspaces and, for inspection and
tests, decodes a built workspace back into Python lists.

The grouping rule mirrors the trainer's prompt-group discovery
(arctic_platform/rl/zorro_train/zorro_train.py:242-285): rows are compared with the first
member of a group, groups come out in first-seen order, members ascending.  Here the rows
are leading runs of physical block ids and the rule is applied level by level.
"""

from __future__ import annotations

import ctypes
import dataclasses

import torch

from . import _lib
from .kv_layout import BLOCK_SIZE

ITEM_INTS = 8


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


@dataclasses.dataclass
class ForestMetadata:
    plan: _lib.FcaPlan
    layout: _lib.FcaMetaLayout
    meta: torch.Tensor  # int32 workspace on the device
    partial_out: torch.Tensor  # half, fca_workspace_bytes: [S * max_partials * Hq + shared-item rows, D], rows scaled by a power of two
    partial_lse: torch.Tensor  # fp32, fca_workspace_bytes: {lse, row scale} per row
    block_table: torch.Tensor
    seq_lens: torch.Tensor  # per query row
    row_table: torch.Tensor | None = None  # block-table row of every query row (None: the row itself)
    row_group: torch.Tensor | None = None  # declared groups of query rows
    # The tiles of a long query run read the same blocks one after the other: the attention
    # calls then keep their KV loads cacheable (fca_tensors.kv_reread).
    kv_reread: bool = False
    # Attention launches never let two waves attend one item together (fca_tensors.reproducible):
    # the same bits from every launch on the same inputs, at a few per cent of the speed.
    reproducible: bool = False
    # Cap of the attention grid in workgroups, 0 = the whole GPU (fca_tensors.max_workgroups).
    max_workgroups: int = 0
    # Register tile buffers per wave for attention on an fp8 cache: 0 = the kernel's own (two), 3 =
    # three where that instance exists (head size 128, 32-row items; fca_tensors.tile_buffers).
    # Calls on a bf16 cache, or with another head size or tile height, are not affected.
    fp8_tile_buffers: int = 0

    # ---- inspection (synchronises; not for the decode loop) -------------------------
    def header(self) -> dict:
        h = self.meta[self.layout.header : self.layout.header + 16].tolist()
        return dict(
            items=h[0],
            shared_items=h[1],
            shared_nodes=h[2],
            error=h[5],
            unique_tokens=(h[6] & 0xFFFFFFFF) | (h[7] << 32),
            levels=h[8],
            updates=h[14],
        )

    def check(self) -> None:
        err = self.header()["error"]
        if err & 1:
            raise ValueError("a sequence length is negative or exceeds max_blocks * block_size")
        if err & 2:
            raise RuntimeError("work list overflowed its reserved size")
        if err & 4:
            raise ValueError("a row_table entry is outside the block table")
        if err & 8:
            raise RuntimeError("a row needs more partial slots than the plan reserves")

    def nodes(self) -> list:
        L, m = self.layout, self.meta.cpu()
        n = int(m[L.header + 2])
        members = m[L.members :]
        out = []
        for i in range(n):
            off, cnt = int(m[L.node_moff + i]), int(m[L.node_mcnt + i])
            out.append(
                dict(
                    members=members[off : off + cnt].tolist(),
                    rep=int(m[L.node_rep + i]),
                    blk_start=int(m[L.node_blk + i]),
                    num_blocks=int(m[L.node_nblk + i]),
                    tokens=int(m[L.node_tok + i]),
                    causal=bool(m[L.node_causal + i]),
                    level=int(m[L.node_level + i]),
                    ord=int(m[L.node_ord + i]),
                )
            )
        return out

    def leaves(self) -> list:
        L, m = self.layout, self.meta.cpu()
        s = self.plan.num_seqs
        lens = self.seq_lens.cpu().tolist()
        blk = m[L.seq_leaf_blk : L.seq_leaf_blk + s].tolist()
        return [dict(blk_start=blk[i], tokens=max(0, lens[i] - blk[i] * BLOCK_SIZE)) for i in range(s)]

    def seq_num_partials(self) -> list:
        L = self.layout
        return self.meta[L.seq_npart : L.seq_npart + self.plan.num_seqs].tolist()

    def items(self) -> list:
        L, m = self.layout, self.meta.cpu()
        n = int(m[L.header])
        shared = int(m[L.header + 1])
        rec = m[L.items : L.items + n * ITEM_INTS].view(n, ITEM_INTS).tolist()
        members = m[L.members :]
        out = []
        for i, r in enumerate(rec):
            out.append(
                dict(
                    rep=r[0],
                    blk_start=r[1],
                    tok_len=r[2],
                    members=members[r[3] : r[3] + r[4]].tolist(),
                    ord=r[5],
                    node=r[6],
                    sees=r[7],
                    shared=i < shared,
                )
            )
        return out


def rows_from_query_runs(query_start_loc: torch.Tensor, seq_lens: torch.Tensor, num_rows: int, max_blocks: int, out=None):
    """Row table, row lengths and tile group ids of a step with query runs, one entry per
    query token (``fca_rows_from_query_runs``; one launch, no synchronisation).  ``out`` may
    hold three int32 tensors of at least ``num_rows`` entries to write into."""
    num_reqs = seq_lens.shape[0]
    if query_start_loc.dtype != torch.int32 or seq_lens.dtype != torch.int32:
        raise TypeError("query_start_loc and seq_lens must be int32")
    if query_start_loc.shape[0] < num_reqs + 1 or not (query_start_loc.is_contiguous() and seq_lens.is_contiguous()):
        raise ValueError("query_start_loc must be contiguous with num_reqs + 1 entries, seq_lens contiguous")
    if not seq_lens.is_cuda:
        raise RuntimeError("query rows are made on the GPU; seq_lens must be a device tensor")
    if out is None:
        out = tuple(torch.empty(num_rows, dtype=torch.int32, device=seq_lens.device) for _ in range(3))
    row_table, row_lens, row_group = (t[:num_rows] for t in out)
    _lib.check(
        _lib.load_library().fca_rows_from_query_runs(
            query_start_loc.data_ptr(), seq_lens.data_ptr(), num_reqs, num_rows, max_blocks,
            row_table.data_ptr(), row_lens.data_ptr(), row_group.data_ptr(), _stream_ptr(seq_lens.device),
        )
    )
    return row_table, row_lens, row_group


def make_plan(
    num_seqs, max_blocks, num_q_heads, num_kv_heads, head_dim, *, chunk_tokens=512, rows_per_item=32, max_levels=4
) -> _lib.FcaPlan:
    return _lib.FcaPlan(
        num_seqs, max_blocks, num_q_heads, num_kv_heads, head_dim, BLOCK_SIZE, chunk_tokens, rows_per_item, max_levels
    )


def build_forest_metadata(
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    *,
    num_q_heads: int,
    num_kv_heads: int,
    head_dim: int,
    block_size: int = BLOCK_SIZE,
    chunk_tokens: int = 512,
    rows_per_item: int = 32,
    cascade: bool = True,
    max_levels: int = 4,
    out: ForestMetadata | None = None,
    update: bool = False,
    row_table: torch.Tensor | None = None,
    row_group: torch.Tensor | None = None,
    kv_reread: bool | None = None,
    partial_dtype: torch.dtype | None = None,
) -> ForestMetadata:
    """Discover the shared-prefix forest of a decode batch on the device.

    With ``row_table`` (int32 ``[R]``) the query rows are not the block-table rows: query row
    ``r`` attends to the first ``seq_lens[r]`` tokens of table row ``row_table[r]`` (the tokens
    of a query run: one row per token, each one token longer), ``seq_lens`` is ``[R]`` and
    the result serves ``q`` of ``R`` rows.  ``row_group`` (int32 ``[R]``, -1 = none) declares
    groups of rows that share their leading blocks (``fca_build_metadata_rows``).
    ``kv_reread`` says whether a launch reads KV blocks again and again (long query runs,
    many tiles per sequence); the default assumes so when groups are declared.
    ``partial_dtype=torch.float32`` sizes the partial rows for the all-fp32 path (fp32 queries on
    an fp32 cache); the default is the scaled half-precision rows of the bf16 / fp8 kernels.

    ``cascade=False`` turns sharing off: every sequence becomes one private node over its
    whole block-table row, which makes the same kernels a plain paged decode attention.
    Pass a previous result as ``out`` to rebuild into the same workspaces (no allocation).
    With ``update=True`` and such an ``out``, the forest found by the last build is kept if
    the rows still carry it (``fca_update_metadata``: the next step of a decode loop, where
    sequences only grew); any other change is detected on the device and built anew.
    """
    if block_size != BLOCK_SIZE:
        raise ValueError(f"block_size must be {BLOCK_SIZE}")
    if block_table.dtype != torch.int32 or seq_lens.dtype != torch.int32:
        raise TypeError("block_table and seq_lens must be int32")
    if row_table is None and row_group is not None:
        raise ValueError("row_group needs a row_table")
    num_rows = block_table.shape[0] if row_table is None else row_table.shape[0]
    if block_table.dim() != 2 or block_table.stride(1) != 1 or seq_lens.shape != (num_rows,):
        raise ValueError("block_table must be [num_seqs, max_blocks] with contiguous rows and seq_lens one per query row")
    if not seq_lens.is_contiguous() or seq_lens.device != block_table.device:
        raise ValueError("seq_lens must be contiguous and on the device of block_table")
    for name, t in (("row_table", row_table), ("row_group", row_group)):
        if t is not None and (t.dtype != torch.int32 or t.shape != (num_rows,) or not t.is_contiguous() or not t.is_cuda):
            raise ValueError(f"{name} must be a contiguous int32 device tensor with one entry per query row")
    if not block_table.is_cuda:
        raise RuntimeError("forest metadata is built on the GPU; block_table must be a device tensor")
    lib = _lib.load_library()
    plan = make_plan(
        num_rows,
        block_table.shape[1],
        num_q_heads,
        num_kv_heads,
        head_dim,
        chunk_tokens=chunk_tokens,
        rows_per_item=rows_per_item,
        max_levels=max_levels if cascade else 0,
    )
    if partial_dtype not in (None, torch.float16, torch.float32):
        raise ValueError(f"partial_dtype must be torch.float32 or None, got {partial_dtype}")
    partial_dtype = partial_dtype or torch.float16
    same_workspace = out is not None and bytes(out.plan) == bytes(plan) and out.partial_out.dtype == partial_dtype
    if same_workspace:
        md = dataclasses.replace(out, block_table=block_table, seq_lens=seq_lens, row_table=row_table, row_group=row_group)
        md.kv_reread = row_group is not None if kv_reread is None else bool(kv_reread)
    else:
        layout = _lib.FcaMetaLayout()
        _lib.check(lib.fca_meta_describe(ctypes.byref(plan), ctypes.byref(layout)))
        nm, no, nl = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
        kv_dtype = _lib.FCA_F32 if partial_dtype == torch.float32 else _lib.FCA_BF16
        _lib.check(lib.fca_workspace_bytes_dtype(ctypes.byref(plan), kv_dtype, ctypes.byref(nm), ctypes.byref(no), ctypes.byref(nl)))
        dev = block_table.device
        md = ForestMetadata(
            plan=plan,
            layout=layout,
            meta=torch.zeros(nm.value // 4, dtype=torch.int32, device=dev),
            partial_out=torch.empty(no.value // (4 if partial_dtype == torch.float32 else 2), dtype=partial_dtype, device=dev),
            # (zeros: a merge that runs before any attention pass has written the buffers then
            # finds plain empty rows, not row scales that point somewhere)
            partial_lse=torch.zeros(nl.value // 4, dtype=torch.float32, device=dev),
            block_table=block_table,
            seq_lens=seq_lens,
            row_table=row_table,
            row_group=row_group,
            kv_reread=row_group is not None if kv_reread is None else bool(kv_reread),
        )
    if row_table is not None:
        _lib.check(
            lib.fca_build_metadata_rows(
                ctypes.byref(md.plan),
                block_table.data_ptr(),
                block_table.stride(0),
                block_table.shape[0],
                row_table.data_ptr(),
                row_group.data_ptr() if row_group is not None else None,
                seq_lens.data_ptr(),
                md.meta.data_ptr(),
                1 if update and same_workspace else 0,
                _stream_ptr(block_table.device),
            )
        )
        return md
    entry = lib.fca_update_metadata if update and same_workspace else lib.fca_build_metadata
    _lib.check(
        entry(
            ctypes.byref(md.plan),
            block_table.data_ptr(),
            block_table.stride(0),
            seq_lens.data_ptr(),
            md.meta.data_ptr(),
            _stream_ptr(block_table.device),
        )
    )
    return md
