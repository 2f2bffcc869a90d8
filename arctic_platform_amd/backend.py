"""Attention-backend surface of forest cascade attention.

The platform's sampling job hands attention to its engine's backend plug-in: the engine
asks the backend for the KV-cache shape, calls a metadata builder once per scheduler
step and the implementation's ``forward`` once per attention layer
(engine start-up: arctic_platform/common/ray_server.py:395-404; the feature switch that
selects this backend: arctic_platform/common/utils/server_models.py:123-140 and the raw
engine kwarg ``forest_cascade_attn_configs`` used by
recipes/rl/skyrl/txt2sql/run_qwen3_8b_bird_grpo_arl.sh:98-111).  The engine itself is
not part of the reference tree, so the class and argument names below follow the engine's
public plug-in convention from its documentation, not from code in the reference.

Decode batches: one query token per sequence, or a few (the verify step of speculative
decoding, ``spec_model`` in the platform's config), prefill chunks and mixed batches.  A
sequence with several query tokens is handed to the kernels as that many query rows over
the same block-table row, each one token longer than the one before it
(``fca_build_metadata_rows``).  The run is cut into tiles, one per 16-token block of the
cache, by declaring the rows of a tile a group.  The forest builder first finds what the
sequence shares with other sequences (a cached prompt): all rows of all those sequences
read that once.  Below it every tile becomes a causal node: its rows read the rest of
the sequence, up to and including their own block, once for all of them, and the kernels
hide from each row the tokens behind its own.  The response-over-shared-prompt attention of
the trainer is the in-tree counterpart
(arctic_platform/rl/zorro_train/qwen_attention_patcher.py:1117-1262).
"""

from __future__ import annotations

import collections
import dataclasses
import json

import torch

from .cache import append_kv, gather_kv
from .config import ModelConfig, validate_fca_support
from .forest import ForestMetadata, build_forest_metadata, rows_from_query_runs
from .kv_layout import BLOCK_SIZE, kv_cache_shape
from .ops import forest_cascade_decode
from .split_attention import SplitLayout, split_attention_forward


@dataclasses.dataclass
class CommonAttentionMetadata:
    """The per-step fields of the engine's common metadata that this backend reads."""

    query_start_loc: torch.Tensor  # [num_reqs + 1] int32, cumulative query tokens
    seq_lens: torch.Tensor  # [num_reqs] int32, tokens in the cache incl. the new one
    block_table_tensor: torch.Tensor  # [num_reqs, max_blocks] int32
    slot_mapping: torch.Tensor  # [num_tokens] int64
    num_reqs: int
    max_query_len: int
    num_actual_tokens: int | None = None
    # host copies, as the engine keeps them; with them a step of fresh prompts only is recognised
    # without a device round trip
    query_start_loc_cpu: torch.Tensor | None = None
    seq_lens_cpu: torch.Tensor | None = None


@dataclasses.dataclass
class ForestCascadeMetadata:
    forest: ForestMetadata | None
    slot_mapping: torch.Tensor
    num_decode_tokens: int
    # set when the batch ends in fresh prompts: causal attention of every such prompt over
    # itself, straight from the step's own K and V
    fresh_prefill: SplitLayout | None = None
    fresh_start: int = 0  # first token of the fresh prompts; the tokens before it go through ``forest``
    # when some of those prompts have a cached context: cache slots of context + chunk of each,
    # in the layout's packed order; K and V are then gathered from the cache per layer
    context_slots: torch.Tensor | None = None


def parse_forest_cascade_configs(value) -> dict:
    """``forest_cascade_attn_configs`` arrives as a JSON string (``"{}"`` in the recipes)
    or a dict.  Known keys: chunk_tokens, rows_per_item, max_levels, enable, rebuild_every,
    kv_reread (true: keep KV loads cacheable, for batches whose shared prompts carry more
    query rows than one row tile holds, e.g. more than rows_per_item / (Hq / Hkv) samples per
    prompt; false: stream; absent: decided per step from the query lengths), reproducible
    (true: no work item is cut between two waves at a point that depends on timing, so equal
    inputs give equal bits, at a few per cent of the speed), fp8_tile_buffers (3: attention on an
    fp8 cache at head size 128 keeps three tiles in flight per wave instead of two)."""
    if value is None or value == "":
        return {}
    cfg = json.loads(value) if isinstance(value, str) else dict(value)
    unknown = set(cfg) - {"chunk_tokens", "rows_per_item", "max_levels", "enable", "rebuild_every", "kv_reread", "reproducible", "fp8_tile_buffers"}
    if unknown:
        raise ValueError(f"unknown forest_cascade_attn_configs keys: {sorted(unknown)}")
    return cfg


class ForestCascadeAttentionBackend:
    accept_output_buffer = True

    @staticmethod
    def get_name() -> str:
        return "FOREST_CASCADE_ATTN"

    @staticmethod
    def get_impl_cls():
        return ForestCascadeAttentionImpl

    @staticmethod
    def get_metadata_cls():
        return ForestCascadeMetadata

    @staticmethod
    def get_builder_cls():
        return ForestCascadeMetadataBuilder

    @staticmethod
    def get_supported_head_sizes():
        return [64, 128, 256]

    @staticmethod
    def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int):
        return kv_cache_shape(num_blocks, block_size, num_kv_heads, head_size)


class ForestCascadeMetadataBuilder:
    """Makes the forest metadata once per scheduler step.  Workspaces are kept per batch
    shape (num_reqs, max_blocks), so a steady decode loop allocates nothing; the least
    recently used ones are dropped beyond ``MAX_KEPT_WORKSPACES`` shapes.  A step on a
    shape seen before asks for an update: the device keeps the forest of the last build when
    the rows still carry it (sequences only grew) and builds anew otherwise.  Every
    ``rebuild_every``-th step is a full build regardless, so sharing that appeared since
    (a new request with a cached prompt) is picked up."""

    MAX_KEPT_WORKSPACES = 16
    MAX_KEPT_BYTES = 8 << 30  # device memory of the kept forest workspaces (partial rows dominate)
    # layouts of prompt steps are keyed by the exact token counts of a step, so nearly every
    # prefill step makes a new one: they live in a small store of their own and never push a
    # decode shape's workspaces out
    MAX_KEPT_LAYOUTS = 8
    # a step of fresh prompts with at least this many tokens runs on the trainer's split
    # attention kernels (each prompt a group of its own): operands shared through LDS, about
    # twice the rate of the query-run path, which stays for everything that reads the cache
    FRESH_PREFILL_MIN_TOKENS = 256
    # a prefill chunk behind a cached context joins them when it is at least this long: its
    # context has to be gathered from the cache into packed rows first (several passes over
    # the context's KV per layer), which only a long chunk pays back
    CONTEXT_PREFILL_MIN_QUERY = 512

    def __init__(self, num_q_heads, num_kv_heads, head_dim, device="cuda", forest_cascade_attn_configs=None):
        cfg = parse_forest_cascade_configs(forest_cascade_attn_configs)
        validate_fca_support(
            ModelConfig(use_fca=True), head_dim=head_dim, num_q_heads=num_q_heads, num_kv_heads=num_kv_heads
        )
        self.num_q_heads, self.num_kv_heads, self.head_dim = num_q_heads, num_kv_heads, head_dim
        self.device = torch.device(device)
        self.enabled = bool(cfg.get("enable", True))
        # split-K chunk: 1024 tokens; head size 256 has few KV heads and a single-buffer kernel, so
        # its work list is cut finer to give every wave something to do (measured: 238 against 257 us
        # at 512 sequences of Hq 16 / Hkv 2)
        self.chunk_tokens = int(cfg.get("chunk_tokens", 512 if head_dim == 256 else 1024))
        self.max_levels = int(cfg.get("max_levels", 4))
        self.rebuild_every = max(1, int(cfg.get("rebuild_every", 32)))
        self.kv_reread = None if cfg.get("kv_reread") is None else bool(cfg["kv_reread"])
        # the same bits from every launch on the same inputs (no item attended by two waves together)
        self.reproducible = bool(cfg.get("reproducible", False))
        self.fp8_tile_buffers = int(cfg.get("fp8_tile_buffers", 0))
        if self.fp8_tile_buffers not in (0, 3):
            raise ValueError(f"fp8_tile_buffers must be 0 or 3, got {self.fp8_tile_buffers}")
        group = num_q_heads // num_kv_heads
        self.rows_per_item = int(cfg.get("rows_per_item", 64 if group > 32 else 32))
        # several query tokens per sequence multiply the rows of every shared node: unless the
        # configuration fixes the tile height, such steps use 64-row tiles (head size 256 has
        # 32-row tiles only)
        self.rows_multi_token = int(cfg.get("rows_per_item", 32 if head_dim == 256 else 64))
        if head_dim == 256 and (self.rows_per_item != 32 or self.rows_multi_token != 32):
            raise ValueError("head_dim 256 takes rows_per_item 32 only")
        # long prompts go to the split attention kernels at head sizes 64 and 128 (at 256 those
        # kernels run one workgroup per CU and the route has not been measured against the query-run path)
        self.prompts_on_split_kernels = head_dim in (64, 128)
        if group > self.rows_per_item:
            raise ValueError(f"{group} query heads per KV head do not fit rows_per_item={self.rows_per_item}")
        self._workspaces: collections.OrderedDict = collections.OrderedDict()
        self._layouts: collections.OrderedDict = collections.OrderedDict()
        self._split_scratch: dict = {}  # shared by the layouts of prompt steps, which change every step
        self._steps_since_build: dict = {}

    @staticmethod
    def _bytes_of(value) -> int:
        if isinstance(value, ForestMetadata):
            return sum(t.numel() * t.element_size() for t in (value.meta, value.partial_out, value.partial_lse))
        return 0

    def _keep(self, key, value):
        """Remember a workspace; forget the least recently used ones beyond the cap on their
        number and on the device memory they hold (the one just stored always stays)."""
        self._workspaces[key] = value
        self._workspaces.move_to_end(key)
        held = sum(self._bytes_of(v) for v in self._workspaces.values())
        while len(self._workspaces) > 1 and (len(self._workspaces) > self.MAX_KEPT_WORKSPACES or held > self.MAX_KEPT_BYTES):
            old, gone = self._workspaces.popitem(last=False)
            held -= self._bytes_of(gone)
            self._steps_since_build.pop(old, None)

    def build(self, common_prefix_len: int, common_attn_metadata: CommonAttentionMetadata) -> ForestCascadeMetadata:
        m = common_attn_metadata
        if m.max_query_len < 1:
            raise ValueError(f"max_query_len must be at least 1, got {m.max_query_len}")
        bt, sl = m.block_table_tensor[: m.num_reqs], m.seq_lens[: m.num_reqs]
        num_tokens = m.num_reqs
        if m.seq_lens_cpu is not None:
            # the device builder can only flag bad lengths in its header; with the engine's host
            # copy at hand they are refused here, before anything is launched
            lens = m.seq_lens_cpu[: m.num_reqs]
            if int(lens.min()) < 0 or int(lens.max()) > bt.shape[1] * BLOCK_SIZE:
                raise ValueError(
                    f"seq_lens must lie in [0, max_blocks * {BLOCK_SIZE} = {bt.shape[1] * BLOCK_SIZE}], got [{int(lens.min())}, {int(lens.max())}]"
                )
            if m.query_start_loc_cpu is not None:
                ql = m.query_start_loc_cpu[1 : m.num_reqs + 1] - m.query_start_loc_cpu[: m.num_reqs]
                if int(ql.min()) < 0 or bool((ql > lens).any()):
                    raise ValueError("every request's query length must lie in [0, seq_len]")
        row_table = row_group = None
        if m.max_query_len > 1 and m.query_start_loc_cpu is not None and m.seq_lens_cpu is not None and self.enabled and self.prompts_on_split_kernels:
            # The requests at the end of the batch that are fresh prompts (the engine puts decodes
            # first): they attend on the split-attention kernels, the requests before them go on
            # as a step of their own.
            q_lens = (m.query_start_loc_cpu[1 : m.num_reqs + 1] - m.query_start_loc_cpu[: m.num_reqs]).tolist()
            s_lens = m.seq_lens_cpu[: m.num_reqs].tolist()
            first = m.num_reqs
            while first > 0 and q_lens[first - 1] > 1 and (
                q_lens[first - 1] == s_lens[first - 1] or q_lens[first - 1] >= self.CONTEXT_PREFILL_MIN_QUERY
            ):
                first -= 1
            fresh = q_lens[first:]
            context = [s - q for s, q in zip(s_lens[first:], fresh)]
            if sum(fresh) >= self.FRESH_PREFILL_MIN_TOKENS:
                # Kept per (query, context) lengths: the layout and, for prompts behind a context,
                # the position of every packed token and its request counted from the first of
                # these prompts.  The number of requests in front of them is not part of the key,
                # so it is added when the slots are computed.
                key = (tuple(fresh), tuple(context))
                if key not in self._layouts:
                    if any(context):
                        layout = SplitLayout(
                            [(c, [n]) for c, n in zip(context, fresh)], device=self.device, responses_only=True,
                            scratch_pool=self._split_scratch,
                        )
                        rel = torch.repeat_interleave(torch.arange(len(fresh)), torch.tensor(s_lens[first:]))
                        pos = torch.cat([torch.arange(n) for n in s_lens[first:]])
                        entry = (layout, rel.to(self.device), pos.to(self.device))
                    else:
                        entry = (SplitLayout([(0, [n]) for n in fresh], device=self.device, scratch_pool=self._split_scratch), None, None)
                    self._layouts[key] = entry
                    while len(self._layouts) > self.MAX_KEPT_LAYOUTS:
                        self._layouts.popitem(last=False)
                self._layouts.move_to_end(key)
                layout, rel, pos = self._layouts[key]
                slots = None
                if rel is not None:
                    slots = m.block_table_tensor[rel + first, pos // BLOCK_SIZE].to(torch.int64) * BLOCK_SIZE + pos % BLOCK_SIZE
                total, before = sum(q_lens), sum(q_lens[:first])
                rest = None
                if first > 0:
                    rest = self.build(
                        common_prefix_len,
                        dataclasses.replace(
                            m, num_reqs=first, max_query_len=max(q_lens[:first]), num_actual_tokens=before,
                            query_start_loc_cpu=None, seq_lens_cpu=None,
                        ),
                    ).forest
                return ForestCascadeMetadata(
                    forest=rest, slot_mapping=m.slot_mapping[:total], num_decode_tokens=total, fresh_prefill=layout, fresh_start=before,
                    context_slots=slots,
                )
        if m.max_query_len > 1:
            # one row per query token: the row of its sequence, cut off behind the token itself;
            # the tokens of a run that fall into one cache block form a tile
            starts = m.query_start_loc[: m.num_reqs + 1]
            # (the count comes from the host side: reading it off the device tensor would stall
            # the scheduler step on a device -> host copy and cannot be captured in a graph)
            if m.num_actual_tokens is not None:
                num_tokens = int(m.num_actual_tokens)
            elif m.query_start_loc_cpu is not None:
                num_tokens = int(m.query_start_loc_cpu[m.num_reqs])
            else:
                raise ValueError("a step with query runs needs num_actual_tokens or query_start_loc_cpu (the number of query tokens)")
            rows_key = (num_tokens, "rows")
            if rows_key not in self._workspaces:
                self._keep(rows_key, tuple(torch.empty(num_tokens, dtype=torch.int32, device=bt.device) for _ in range(3)))
            self._workspaces.move_to_end(rows_key)
            row_table, sl, row_group = rows_from_query_runs(
                starts.to(torch.int32).contiguous(), sl.contiguous(), num_tokens, bt.shape[1], out=self._workspaces[rows_key]
            )
        key = (num_tokens, bt.shape[1], m.max_query_len > 1, row_group is not None)
        since = self._steps_since_build.get(key, self.rebuild_every)
        update = key in self._workspaces and since + 1 < self.rebuild_every
        self._steps_since_build[key] = since + 1 if update else 0
        forest = build_forest_metadata(
            bt,
            sl,
            num_q_heads=self.num_q_heads,
            num_kv_heads=self.num_kv_heads,
            head_dim=self.head_dim,
            block_size=BLOCK_SIZE,
            chunk_tokens=self.chunk_tokens,
            rows_per_item=self.rows_multi_token if m.max_query_len > 1 else self.rows_per_item,
            cascade=self.enabled,
            max_levels=self.max_levels,
            out=self._workspaces.get(key),
            update=update and row_group is None,
            row_table=row_table,
            row_group=row_group,
            # With three or more query tokens per sequence the rows of a shared prompt usually
            # fill more than one row tile, and every tile reads the prompt again: loads that
            # stay in the caches then win (q = 4: 578 -> 516 us per layer at the 512-sequence
            # shape, q = 8: 948 -> 742 us); one or two tokens read a block about once, like
            # plain decode, and stream.
            kv_reread=m.max_query_len > 2 if self.kv_reread is None else self.kv_reread,
        )
        if forest is not None:  # (a test double of the builder returns none)
            forest.reproducible = self.reproducible
            forest.fp8_tile_buffers = self.fp8_tile_buffers
        self._keep(key, forest)
        return ForestCascadeMetadata(forest=forest, slot_mapping=m.slot_mapping[:num_tokens], num_decode_tokens=num_tokens)


class ForestCascadeAttentionImpl:
    def __init__(
        self,
        num_heads: int,
        head_size: int,
        scale: float,
        num_kv_heads: int | None = None,
        alibi_slopes=None,
        sliding_window=None,
        kv_cache_dtype: str = "auto",
        logits_soft_cap=None,
        attn_type: str = "decoder",
    ):
        if alibi_slopes is not None or sliding_window is not None or logits_soft_cap is not None:
            raise NotImplementedError("forest cascade attention supports plain softmax attention only (no ALiBi, sliding window or soft cap)")
        if attn_type != "decoder":
            raise NotImplementedError(f"attention type {attn_type!r} is not supported")
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads or num_heads
        self.head_size = head_size
        self.scale = float(scale)
        self.kv_cache_dtype = kv_cache_dtype
        validate_fca_support(
            ModelConfig(use_fca=True, kv_cache_dtype=kv_cache_dtype),
            head_dim=head_size,
            num_q_heads=num_heads,
            num_kv_heads=self.num_kv_heads,
        )

    def forward(self, layer, query, key, value, kv_cache, attn_metadata: ForestCascadeMetadata, output=None):
        """query ``[T, Hq*D]`` or ``[T, Hq, D]``; key/value ``[T, Hkv*D]`` / ``[T, Hkv, D]`` or
        None when the cache already holds the step's tokens; returns ``output`` shaped like
        ``query``.  Per-KV-head fp8 scales are read from ``layer.k_scale`` / ``layer.v_scale``."""
        t = attn_metadata.num_decode_tokens
        q = query[:t].view(t, self.num_heads, self.head_size)
        k_scale = getattr(layer, "k_scale", None)
        v_scale = getattr(layer, "v_scale", None)
        if key is not None:
            append_kv(
                key[:t].view(t, self.num_kv_heads, self.head_size),
                value[:t].view(t, self.num_kv_heads, self.head_size),
                kv_cache,
                attn_metadata.slot_mapping,
                k_scale,
                v_scale,
            )
        if output is None:
            output = torch.empty_like(query)
        if attn_metadata.fresh_prefill is not None:
            if key is None and attn_metadata.context_slots is None:
                raise ValueError("a step with fresh prompts needs the step's key and value")
            f = attn_metadata.fresh_start
            if attn_metadata.context_slots is not None:  # context and chunk alike, from the cache just filled
                k_rows, v_rows = gather_kv(kv_cache, attn_metadata.context_slots, self.head_size, k_scale, v_scale)
            else:
                k_rows = key[f:t].view(t - f, self.num_kv_heads, self.head_size)
                v_rows = value[f:t].view(t - f, self.num_kv_heads, self.head_size)
            split_attention_forward(
                q[f:], k_rows, v_rows, attn_metadata.fresh_prefill, self.scale,
                out=output[f:t].view(t - f, self.num_heads, self.head_size),
            )
            if f == 0:
                return output
            t, q = f, q[:f]
        forest_cascade_decode(
            q, kv_cache, attn_metadata.forest, self.scale, k_scale, v_scale,
            out=output[:t].view(t, self.num_heads, self.head_size), return_lse=False,
        )
        return output
