/*
 * zorro_fca.h - C ABI of libzorro_fca.so: forest cascade decode attention for gfx950.
 *
 * The platform switches this path on per sampling job with
 * arctic_inference_config = {"zorro_inference": {"enable": true}}
 * (arctic_platform/common/utils/server_models.py:123-140) and the engine it starts
 * (arctic_platform/common/ray_server.py:395-404, :921-933) runs it once per attention
 * layer per decode step.  The reference binds the path through an external Python
 * package, not through an in-tree FFI, so the entry points below are what a ctypes /
 * nanobind stub of that package's attention backend binds:
 *
 *   metadata build   <- the backend's per-scheduler-step metadata builder
 *   prefix / suffix / merge / decode_step <- the backend's per-layer forward()
 *
 * Conventions
 *   - every function returns 0 on success or a negative fca_status; fca_last_error()
 *     returns a thread-local message for the last failure on the calling thread;
 *   - all pointers named *_dev are device pointers; strides are in ELEMENTS;
 *   - `stream` is a hipStream_t passed as void*; every call is asynchronous on it,
 *     performs no host<->device synchronisation and allocates nothing;
 *   - the caller owns every buffer, including the metadata and partial workspaces whose
 *     sizes fca_workspace_bytes() reports;
 *   - the attention and merge calls read the metadata workspace; the attention call also
 *     uses one self-resetting work counter in its header (zero before and after every
 *     launch), and the partial workspaces are written by the attention call and read by
 *     the merge.  Calls that use one set of workspaces must therefore not overlap in
 *     time: stream order is enough; layers running concurrently on different streams need
 *     their own metadata and partial workspaces.
 */
#ifndef ZORRO_FCA_H
#define ZORRO_FCA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FCA_VERSION 105
#define FCA_BLOCK_SIZE 16
#define FCA_MAX_LEVELS 8

typedef enum fca_status {
  FCA_OK = 0,
  FCA_ERR_INVALID_ARG = -1,
  FCA_ERR_UNSUPPORTED = -2,
  FCA_ERR_HIP = -3
} fca_status;

/* q is bf16 and the KV cache bf16 or fp8: the products run on the bf16 matrix cores with
 * fp32 accumulation.  kv_dtype FCA_F32 is the all-fp32 path of the small fp32 configuration:
 * q, the KV cache and the partial rows are fp32 and so is every product (vector units; the
 * chip has no more fp32 rate in its matrix cores), at the precision of the reference's
 * softmax-in-fp32 attention (arctic_platform/rl/zorro_train/qwen_attention_patcher.py:55-61).
 * It runs through fca_decode_step and fca_decode_step_static only, at head sizes 64 and 128
 * with rows_per_item 32; the separate passes and the merge refuse it.  fca_append_kv and
 * fca_gather_kv with kv_dtype FCA_F32 move fp32 rows to and from an fp32 cache. */
typedef enum fca_dtype {
  FCA_BF16 = 0,     /* q, out, KV cache */
  FCA_FP8_E4M3 = 1, /* KV cache only (OCP e4m3fn) */
  FCA_F32 = 2       /* out; as kv_dtype: q and the KV cache are fp32 */
} fca_dtype;

/* Shape of one decode batch and the tiling the metadata is built for. */
typedef struct fca_plan {
  int32_t num_seqs;      /* S: rows of q and of the block table */
  int32_t max_blocks;    /* columns of the block table */
  int32_t num_q_heads;   /* Hq, multiple of num_kv_heads, Hq / Hkv <= rows_per_item */
  int32_t num_kv_heads;  /* Hkv */
  int32_t head_dim;      /* 64, 128 or 256 (256: rows_per_item 32 only) */
  int32_t block_size;    /* must be FCA_BLOCK_SIZE */
  int32_t chunk_tokens;  /* split-K chunk, multiple of 32 in [32, 1024] */
  int32_t rows_per_item; /* query rows stacked per work item: 32 or 64 */
  int32_t max_levels;    /* shared tree levels to discover, 0 = non-cascade, <= FCA_MAX_LEVELS */
} fca_plan;

/* Tensors of one attention layer. */
typedef struct fca_tensors {
  const void* q_dev;           /* bf16 (fp32 when kv_dtype is FCA_F32) [S, Hq, D], D contiguous */
  int64_t q_seq_stride;
  int64_t q_head_stride;
  const void* k_cache_dev;     /* K plane: [num_blocks, Hkv, D/x, 16, x], x = 16 bytes / elem size */
  const void* v_cache_dev;     /* V plane: [num_blocks, Hkv, D, 16] */
  int64_t kv_block_stride;     /* elements between blocks of one plane */
  int64_t kv_head_stride;      /* elements between KV heads of one block */
  int32_t kv_dtype;            /* FCA_BF16, FCA_FP8_E4M3, or FCA_F32 (then q is fp32 as well) */
  int32_t kv_reread;           /* 0: a launch reads every KV block about once (decode), loads bypass
                                  the caches; non-zero: blocks are read again and again (query runs
                                  built with fca_build_metadata_rows), loads stay cacheable */
  const int32_t* block_table_dev; /* [S, max_blocks] physical block ids ([table_rows, max_blocks]
                                  for metadata built with fca_build_metadata_rows) */
  int64_t block_table_stride;
  const float* k_scale_dev;    /* [Hkv] dequant scales for fp8 caches, or NULL (= 1) */
  const float* v_scale_dev;
  float softmax_scale;         /* usually head_dim ** -0.5 */
  int32_t reproducible;        /* non-zero: no work item is attended by two waves together, so where an
                                  item is cut, and with it the last bit of a few outputs, never depends
                                  on timing: two launches on the same inputs give the same bits */
  int32_t max_workgroups;      /* > 0: the attention launch uses at most this many workgroups (four waves
                                  each; two in the fp32 path), leaving the rest of the GPU to work on
                                  other streams; 0: all */
  int32_t tile_buffers;        /* 0: the kernel's own choice (two register tile buffers per wave in the
                                  32-row kernel).  3: three, for fp8 caches at head_dim 128 with
                                  rows_per_item 32 only (an fp8 tile is half the bytes of a bf16 one, so
                                  two of them keep half as many bytes in flight): tiles are attended in
                                  groups of three.  Any other value, or 3 elsewhere: FCA_ERR_UNSUPPORTED */
} fca_tensors;

/* Offsets (in int32 units) of the arrays inside a built metadata workspace, for
 * inspection and tests.  Item records are 8 x int32:
 * {rep_row, blk_start, tok_len, member_off, member_cnt, ord, node, sees}; rep_row is the
 * block-table row the item reads, sees is 0 except in the last chunk of a causal node,
 * where member i of the item attends to the first sees + i tokens of the chunk. */
typedef struct fca_meta_layout {
  int64_t header;        /* [16]: 0 items, 1 shared items, 2 nodes (shared), 3 work ticket
                            (self-resetting, owned by the attention kernel), 4 reserved,
                            5 error flags (1 bad length, 2 work list overflow, 4 bad row table
                            entry, 8 partial slots of a row overflow), 6/7 unique tokens lo/hi,
                            8 levels found,
                            10-13 and 15 state for fca_update_metadata, 14 updates since the
                            last full build */
  int64_t seq_npart;     /* [S] partial slots used per sequence */
  int64_t seq_leaf_blk;  /* [S] first block position of the private leaf */
  int64_t node_rep;      /* [S] shared nodes: representative sequence */
  int64_t node_blk;      /* [S] first block position */
  int64_t node_nblk;     /* [S] number of blocks */
  int64_t node_level;    /* [S] */
  int64_t node_moff;     /* [S] offset into members */
  int64_t node_mcnt;     /* [S] number of members */
  int64_t node_ord;      /* [S] partial ordinal of the node's first chunk */
  int64_t members;       /* [S * (FCA_MAX_LEVELS + 2)] sequence ids; leaves last */
  int64_t items;         /* [max_items * 8] */
  int64_t max_items;
  int64_t max_partials;  /* partial slots reserved per sequence */
  int64_t total_int32;
  int64_t node_tok;      /* [S] KV tokens of the node: num blocks * 16, or, for a causal node, up to
                            the last token of its last member */
  int64_t node_causal;   /* [S] 1: the node is a tile of a query run (fca_build_metadata_rows) */
  int64_t coop_ctr;      /* [1024] claim counters of the attention kernel (pairs of waves that attend
                            an item together), zero between launches */
} fca_meta_layout;

int fca_version(void);
const char* fca_last_error(void);

/* Workspace sizes for a plan: metadata (int32 arrays) and the two partial buffers.  A
 * partial output row is D half-precision values times one power-of-two scale per row:
 * partial_out is half [rows, D], partial_lse is fp32 [rows, 2] = {natural-log lse, scale},
 * rows = S * max_partials * Hq plus 32 for each pair of waves that may attend an item
 * together (at most 1024 pairs; the second wave of a pair writes there, and the scale of
 * the first wave's row carries the place in its mantissa bits; fca_suffix_pass shares no
 * item, so that it leaves alone what fca_prefix_pass wrote there for the same merge).  Both
 * are opaque to the caller: written by the passes, read by the merge. */
int fca_workspace_bytes(const fca_plan* plan, size_t* meta_bytes, size_t* partial_out_bytes, size_t* partial_lse_bytes);
/* The same for a given kv_dtype: with FCA_F32 the partial rows are fp32 (partial_out twice the
 * bytes); FCA_BF16 and FCA_FP8_E4M3 give what fca_workspace_bytes gives. */
int fca_workspace_bytes_dtype(const fca_plan* plan, int32_t kv_dtype, size_t* meta_bytes, size_t* partial_out_bytes,
                              size_t* partial_lse_bytes);
int fca_meta_describe(const fca_plan* plan, fca_meta_layout* layout);

/* Forest metadata builder: block tables + lengths -> flat node / member / work-item arrays.
 * Analog of the host-side prompt-group discovery of the trainer
 * (arctic_platform/rl/zorro_train/zorro_train.py:242-285, seqlen_balancing.py:437-486). */
int fca_build_metadata(const fca_plan* plan, const int32_t* block_table_dev, int64_t block_table_stride,
                       const int32_t* seq_lens_dev, void* meta_dev, void* stream);

/* The same for the next scheduler step of a running decode loop, into a workspace that a
 * build (or an earlier update) has filled: sequences have grown and may have taken new
 * private blocks.  The forest is kept if every row still starts with the blocks its shared
 * nodes were built from (compared through a per-row fingerprint), those are still full
 * blocks of the row and no sequence got shorter; then only the private leaves and the work list are made again, at a
 * fraction of the cost.  Otherwise, or on a workspace never built or built for another
 * plan, this is fca_build_metadata.  Either way the result is valid for the given rows; a
 * kept forest may miss sharing that only a new build would find.  The comparison is by a
 * 64-bit fingerprint of the shared block ids of each row (a sum of (id xor c) * w_j with odd
 * weights per position): one changed id, or two ids exchanged, always change it; an arbitrary
 * rewrite of several ids of a row goes unnoticed with probability about 2^-64 per row, in
 * which case the row would attend to the blocks its shared nodes were built from, not the
 * new ones.  Callers that rewrite the shared part of a row (rather than append to it) and
 * cannot accept that call fca_build_metadata.  Header slot 14 counts
 * the updates since the last full build.  This replaces the per-step rebuild of the host-side
 * group discovery (arctic_platform/rl/zorro_train/zorro_train.py:242-285 runs once per batch). */
int fca_update_metadata(const fca_plan* plan, const int32_t* block_table_dev, int64_t block_table_stride,
                        const int32_t* seq_lens_dev, void* meta_dev, void* stream);

/* Metadata for query rows that are not one per block-table row: a sequence that brings a
 * run of query tokens (a prefill or a chunk of one, the verify step of speculative
 * decoding) contributes one query row per token.  plan->num_seqs is the number of query
 * rows R (rows of q and out); row r attends to the first row_lens_dev[r] tokens of
 * block-table row row_table_dev[r] (< table_rows), which for token i of a sequence is the
 * sequence's length up to and including that token, so causal order needs no mask.
 * row_group_dev may be NULL.  A value >= 0 declares a group, which is how a run is cut
 * into tiles: give the tokens of one 16-token cache block of one sequence one id.
 * All rows first go through the discovery of fca_build_metadata (rows with -1 exactly as
 * there).  A declared row never shares the block its own token is in through discovery,
 * and a group that discovery finds among declared rows of one table row alone is left
 * alone, so what discovery keeps is what a sequence shares with other sequences (a
 * cached prompt): all rows of all those sequences read it once.  Then the declared rows
 * meet under (node they ended in, group id).  When the members of a group are successive
 * rows over one table row, each one token longer than the one before it and all ending in
 * one block, the group becomes a causal node from there to its last token: it reads the
 * rest of its KV, its own block included, once, the kernels hide from every row the
 * tokens behind its own, and the rows have no private part.  Any other declared group
 * (rows over different table rows: an explicit tree) becomes a plain node over the blocks
 * its members still have in common (rows of one table row are not compared, others are,
 * so a wrong declaration costs sharing, never correctness), and each row reads the rest
 * alone.  A build with declared groups leaves nothing for an update to keep, so an update
 * on such a workspace is a full build; update != 0 otherwise asks for the update of
 * fca_update_metadata.  The attention calls take the [table_rows, max_blocks] block
 * table, and kv_reread = 1 when runs are long (many tiles read the same blocks).
 * Counterpart in the reference: the response-over-shared-prompt attention of the trainer,
 * which rebuilds full sequences from de-duplicated prompts
 * (arctic_platform/rl/zorro_train/zorro_train.py:160-235) and runs
 * a varlen attention over them (rl/zorro_train/qwen_attention_patcher.py:1117-1262). */
int fca_build_metadata_rows(const fca_plan* plan, const int32_t* block_table_dev, int64_t block_table_stride,
                            int32_t table_rows, const int32_t* row_table_dev, const int32_t* row_group_dev,
                            const int32_t* row_lens_dev, void* meta_dev, int32_t update, void* stream);

/* The three row arrays of fca_build_metadata_rows from what an engine keeps per request:
 * query_start_loc_dev [num_reqs + 1] (cumulative query tokens, num_rows at the end) and
 * seq_lens_dev [num_reqs] (tokens in the cache including the whole run).  Token i of a run
 * of q tokens gets its request as table row, length seq_len - (q - 1 - i), and, for
 * q >= 2, the group id request * max_blocks + (block its own token is in); single tokens
 * get -1.  One launch, no host synchronisation.  In the reference this bookkeeping is
 * host code on the trainer's side (cu_seqlens per response and per unique prompt,
 * arctic_platform/rl/zorro_train/zorro_train.py:2059-2127). */
int fca_rows_from_query_runs(const int32_t* query_start_loc_dev, const int32_t* seq_lens_dev, int32_t num_reqs,
                             int32_t num_rows, int32_t max_blocks, int32_t* row_table_dev, int32_t* row_lens_dev,
                             int32_t* row_group_dev, void* stream);

/* Shared-prefix pass: work items of shared nodes only.  Writes normalised partial
 * outputs and natural-log LSEs into the slots the metadata assigns. */
int fca_prefix_pass(const fca_plan* plan, const fca_tensors* t, void* meta_dev,
                    void* partial_out_dev, float* partial_lse_dev, void* stream);
/* Per-sequence suffix pass: work items of private leaves only (with max_levels = 0 this
 * is the non-cascade paged decode kernel). */
int fca_suffix_pass(const fca_plan* plan, const fca_tensors* t, void* meta_dev,
                    void* partial_out_dev, float* partial_lse_dev, void* stream);
/* Both classes of work items in one launch (what fca_decode_step runs before its merge). */
int fca_forest_pass(const fca_plan* plan, const fca_tensors* t, void* meta_dev,
                    void* partial_out_dev, float* partial_lse_dev, void* stream);
/* Log-sum-exp merge of each sequence's partials (online max / rescaled sum as in
 * arctic_platform/model/implementations/qwen35/models/layers/lm_head.py:190-202).
 * out: [S, Hq, D] bf16 or f32; lse: fp32 [S, Hq], natural log, may be NULL.
 * Precondition: since the metadata was last built or updated, fca_forest_pass, or both
 * fca_prefix_pass and fca_suffix_pass, have run on these partial buffers, so that every slot
 * the metadata counts for a row has been written.  On buffers that hold anything else the
 * merge stays inside the buffers (a row scale whose mantissa bits point past the rows set
 * aside for second partials is not followed, and that output row becomes NaN) but its
 * results mean nothing. */
int fca_merge(const fca_plan* plan, const void* meta_dev, const void* partial_out_dev,
              const float* partial_lse_dev, void* out_dev, int64_t out_seq_stride, int64_t out_head_stride,
              int32_t out_dtype, float* lse_dev, void* stream);
/* One layer's decode attention: prefix and suffix items in one launch, then the merge. */
int fca_decode_step(const fca_plan* plan, const fca_tensors* t, void* meta_dev,
                    void* partial_out_dev, float* partial_lse_dev, void* out_dev, int64_t out_seq_stride,
                    int64_t out_head_stride, int32_t out_dtype, float* lse_dev, void* stream);

/* fca_decode_step for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the partial rows live in
 * a file-scope device array of FCA_STATIC_SCRATCH_BYTES inside the library instead of
 * caller-owned partial buffers, and the call allocates nothing.  No counterpart in the
 * reference.  The caller still passes q, the cache, the built metadata workspace and out.
 * Plans whose partial buffers (fca_workspace_bytes) do not fit are refused with
 * FCA_ERR_UNSUPPORTED.  Results are those of fca_decode_step bit for bit.  Each GPU holds
 * one such array from the first call on it until the process ends, and every call on a GPU
 * uses it: calls that overlap in time on one GPU (two streams, two threads) race; stream
 * order is enough.  The first call on a device looks the array's address up
 * (hipGetSymbolAddress); make that call outside graph capture. */
#define FCA_STATIC_SCRATCH_BYTES (48u << 20)
int fca_decode_step_static(const fca_plan* plan, const fca_tensors* t, void* meta_dev, void* out_dev,
                           int64_t out_seq_stride, int64_t out_head_stride, int32_t out_dtype, float* lse_dev,
                           void* stream);

/* KV-cache append, the step before decode attention in every layer: scatter the new
 * tokens' K and V (bf16 [T, Hkv, D]; fp32 when kv_dtype is FCA_F32) into the cache tiles at slot = block * 16 + offset
 * (negative slot = padding, skipped), quantising to fp8 e4m3 with per-KV-head scales
 * (stored = clamp(x / scale, +-448) rounded to nearest even) when kv_dtype says so.
 * Replaces the external engine's cache-write op on this layout; in-tree the reference only
 * names the cache dtype it forwards to that engine (vllm_config, server_models.py:143-165). */
int fca_append_kv(const void* key_dev, const void* value_dev, int64_t token_stride, int64_t head_stride,
                  int32_t num_tokens, int32_t num_kv_heads, int32_t head_dim, const int64_t* slot_mapping_dev,
                  void* k_cache_dev, void* v_cache_dev, int64_t kv_block_stride, int64_t kv_head_stride, int32_t kv_dtype,
                  const float* k_scale_dev, const float* v_scale_dev, void* stream);
/* The way back: the tokens at slot_mapping[t] leave the cache as bf16 rows key[t], value[t]
 * ([T, Hkv, D]; fp8 tiles times their per-head scales, i.e. the values decode attention
 * sees; a negative slot gives zeros).  Used by the adapter to hand a prompt's cached context
 * to the split-attention kernels; like fca_append_kv it stands for an op of the external
 * engine and has no in-tree counterpart in the reference. */
int fca_gather_kv(void* key_dev, void* value_dev, int64_t token_stride, int64_t head_stride, int32_t num_tokens,
                  int32_t num_kv_heads, int32_t head_dim, const int64_t* slot_mapping_dev, const void* k_cache_dev,
                  const void* v_cache_dev, int64_t kv_block_stride, int64_t kv_head_stride, int32_t kv_dtype,
                  const float* k_scale_dev, const float* v_scale_dev, void* stream);

/* ---- split attention of the trainer (forward and backward) ---------------------------
 * Attention over a deduplicated, unpadded training batch: q [T, Hq, D], k and v
 * [T, Hkv, D], bf16, tokens in deduplicated order (for every prompt group the prompt once,
 * then the response of every sample: ZoRRoTrain._dedup_input_ids,
 * arctic_platform/rl/zorro_train/zorro_train.py:311-356).  Replaces the two
 * attention_interface calls of patched_forward_split_unpadded and the regrouping around
 * them (arctic_platform/rl/zorro_train/qwen_attention_patcher.py:1186-1231): prompt rows
 * attend causally to their prompt, response rows to their group's whole prompt and causally
 * to their own response.  Row strides are in elements; the heads of a token are contiguous
 * ([H, D]); every pointer 16-byte aligned, strides multiples of 8.
 * window > 0 is the sliding_window both reference calls receive (:1206, :1226): a row also
 * sees only the keys fewer than `window` positions before it, its own included, positions
 * counted in the sample's own sequence (the prompt's tokens, then the response's), i.e.
 * key position > row position - window.  The layout must have been built for a window at
 * least as wide (or for none): its walks leave out the tiles no row sees any more.
 * dropout_p > 0 is the dropout both calls receive while training (:1204, :1224): after the
 * softmax each probability is dropped with that probability and the others are scaled by
 * 1 / (1 - dropout_p), as the attention interface does (dropout on the attention weights,
 * then the product with V); the log-sum-exp is that of the undropped scores.  Which
 * probabilities fall is a function of (dropout_seed, query head, row, key) alone:
 *   x = seed + head * 0xC2B2AE3D + row * 0x9E3779B1 + key * 0x85EBCA77   (mod 2^32; row and
 *       key are places in the deduplicated order)
 *   x ^= x >> 16; x *= 0x7FEB352D; x ^= x >> 15; x *= 0x846CA68B; x ^= x >> 16;
 *   dropped  <=>  x < floor(dropout_p * 2^32)
 * so the forward and the three gradients agree without a stored mask, and a caller can
 * reproduce it.  The backward must be given the plan (seed included) of its forward. */
typedef struct fca_split_plan {
  int32_t num_tokens; /* T: tokens of the deduplicated batch */
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t head_dim; /* 64, 128 or 256 (256: num_q_heads / num_kv_heads a multiple of 4) */
  int32_t window;   /* 0 = none */
  float dropout_p;  /* in [0, 1); 0 = none */
  uint32_t dropout_seed;
} fca_split_plan;

/* int32 entries of the layout array of a batch of num_tokens tokens. */
int fca_split_layout_ints(int32_t num_tokens, int64_t* num_ints);
/* Host function: fills the layout array (host memory, fca_split_layout_ints entries) from
 * the token layout of ZoRRoTrain.get_group_token_layout (zorro_train.py:2413-2436):
 * prompt_tokens[g], group_sizes[g] samples per group, response_tokens one per sample in
 * group order.  The counts must add up to num_tokens.  The caller copies the array to the
 * device once per batch; every layer's forward and backward reads it.
 * responses_only != 0 (forward only, no counterpart in the reference): k and v still hold
 * all num_tokens rows, but q and out hold the response rows only, in packed order, and the
 * prompts' own attention is not computed -- a prefill chunk behind a cached context, with
 * the context as the prompt.
 * window > 0: the walks of the layout skip what a sliding window of that width hides from
 * every row of a tile; such a layout serves plans with 0 < plan->window <= window only. */
int fca_split_layout_build(int32_t num_groups, const int32_t* prompt_tokens, const int32_t* group_sizes,
                           const int32_t* response_tokens, int32_t num_tokens, int32_t responses_only, int32_t window,
                           int32_t* layout_host);
/* Bytes of device scratch a forward / a backward call needs: operand tiles in MFMA order,
 * per-row sums, and for small batches fp32 slices of dk and dv per query head of a KV head. */
int fca_split_workspace_bytes(const fca_split_plan* plan, size_t* forward_bytes, size_t* backward_bytes);
/* out [T, Hq, D] bf16; lse fp32 [Hq][32 * ceil(T / 32)], natural log (kept for backward). */
int fca_split_attention_forward(const fca_split_plan* plan, const void* q_dev, int64_t q_stride, const void* k_dev,
                                int64_t k_stride, const void* v_dev, int64_t v_stride, const int32_t* layout_dev,
                                float scale, void* workspace_dev, void* out_dev, int64_t out_stride, float* lse_dev,
                                void* stream);
/* Gradients dq [T, Hq, D], dk, dv [T, Hkv, D] (bf16, fp32 accumulation; a prompt's dk and
 * dv sum over the samples of its group) from dout, the forward's inputs, out and lse. */
int fca_split_attention_backward(const fca_split_plan* plan, const void* q_dev, int64_t q_stride, const void* k_dev,
                                 int64_t k_stride, const void* v_dev, int64_t v_stride, const void* out_dev,
                                 int64_t out_stride, const void* dout_dev, int64_t dout_stride, const float* lse_dev,
                                 const int32_t* layout_dev, float scale, void* workspace_dev, void* dq_dev,
                                 int64_t dq_stride, void* dk_dev, int64_t dk_stride, void* dv_dev, int64_t dv_stride,
                                 void* stream);

/* ---- whole samples from a deduplicated tensor, and back ---------------------------------
 * dst[i] = src[index[i]] for rows of row_bytes bytes (a multiple of 16; strides in bytes,
 * multiples of 16; index < 0 gives a row of zeros).  With the index of every sample's prompt
 * rows followed by its response rows this is ZoRRoTrain.reconstruct_sequences in its packed
 * form (arctic_platform/rl/zorro_train/zorro_train.py:1071-1159, and the row-per-program
 * Triton kernel at :160-235); with the index of each group's first sample's prompt rows and
 * every sample's response rows it is deduplicate_sequences (:1162-1179).  The index arrays
 * are made on the host once per batch. */
int fca_gather_rows(const void* src_dev, int64_t src_stride_bytes, const int32_t* index_dev, int64_t num_rows, int64_t row_bytes,
                    void* dst_dev, int64_t dst_stride_bytes, void* stream);
/* The transpose of a gather, for its gradient: dst[j] = sum over k in [offsets[j],
 * offsets[j + 1]) of src[rows[k]], channels (a multiple of 8) of bf16 or fp32 per row, added
 * up in fp32 in the order given (no atomics: the result does not depend on timing).  The
 * gradient of a reconstructed tensor with respect to the deduplicated one: a prompt row sums
 * the rows of its copies in all samples of its group. */
int fca_sum_rows(const void* src_dev, int64_t src_stride_bytes, const int32_t* offsets_dev, const int32_t* rows_dev,
                 int64_t num_dst_rows, int64_t channels, int32_t dtype, void* dst_dev, int64_t dst_stride_bytes, void* stream);

/* Plain device-to-device copy with 16-byte loads and stores.  No counterpart in the
 * reference: it is the known-size yardstick for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE
 * readings of the kernels above. */
int fca_calibration_copy(const void* src_dev, void* dst_dev, size_t bytes, void* stream);

/* Measurement hook, no counterpart in the reference: the next attention launch this thread
 * makes (fca_prefix_pass, fca_suffix_pass, fca_forest_pass, or the attention launch inside
 * fca_decode_step) records its own begin and end in the two HIP events (hipEvent_t, created
 * by the caller with timing enabled), taken from the kernel's dispatch itself, so that
 * hipEventElapsedTime(start, stop) is the kernel's duration and the launch is not fenced in
 * by event records on the stream (those cost about 3 us each here).  One launch consumes the
 * pair; NULL, NULL withdraws it.  Not for use under a profiler that intercepts dispatches:
 * it keeps its own hold on every dispatch's completion signal.  Under rocprofv3 (recognised
 * by ROCP_TOOL_LIBRARIES in the environment) a non-NULL pair is refused with
 * FCA_ERR_UNSUPPORTED and the next launch is an ordinary one. */
int fca_time_next_attention(void* start_event, void* stop_event);

#ifdef __cplusplus
}
#endif
#endif /* ZORRO_FCA_H */
