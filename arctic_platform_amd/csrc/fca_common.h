// Shared definitions of the forest-cascade kernels: metadata workspace layout and
// launch parameter blocks.  Internal to libzorro_fca.so; the public ABI is zorro_fca.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/zorro_fca.h"

namespace fca {

constexpr int kBlock = FCA_BLOCK_SIZE;   // tokens per physical KV block
constexpr int kTile = 32;                // tokens per MFMA tile (two blocks)
constexpr int kMaxChunk = 1024;          // one lane of a wave holds one block id of a chunk
constexpr int kItemInts = 8;             // int32 per work-item record
constexpr int kSizeBuckets = 32;         // size classes for the descending work-list order
constexpr int kHeaderInts = 16;
// Items that two waves of the 32-row attention kernel attend together (one from either end):
// at most this many pairs of waves, one claim counter each in the metadata workspace, and 32
// partial rows each behind the ordinary partial rows for the wave that comes from the back.
// A launch over the private items alone (fca_suffix_pass) shares no item: it would write the
// same 32 rows per pair as the launch over the shared items that precedes the same merge.
constexpr int kCoopMaxPairs = 1024;
constexpr int kCoopMinPairs = 4;  // groups of tiles (pairs; threes with three tile buffers) an item needs to be shared

enum HeaderSlot {
  H_ITEMS = 0,
  H_SHARED_ITEMS = 1,
  H_NODES = 2,
  H_TICKET = 3,
  H_RESERVED1 = 4,
  H_ERROR = 5,
  H_TOKENS_LO = 6,
  H_TOKENS_HI = 7,
  H_LEVELS = 8,
  // state a later update of the same workspace starts from
  H_LEAF_MEMBERS = 10,   // offset of the leaf entries in the member list
  H_SHARED_TOK_LO = 11,  // KV tokens held by shared nodes
  H_SHARED_TOK_HI = 12,
  H_BUILT = 13,          // kBuiltMagic once a build has completed on this workspace
  H_UPDATES = 14,        // length-only updates since the last full build
  H_PLAN_SIG = 15        // fingerprint of the plan the workspace was built for
};
constexpr int kBuiltMagic = 0x46434131;

// Offsets in int32 units from the start of the metadata workspace.
struct MetaLayout {
  int64_t header;
  int64_t seq_npart, seq_leaf_blk;
  int64_t node_rep, node_blk, node_nblk, node_level, node_moff, node_mcnt, node_ord;
  int64_t node_tok;     // KV tokens of the node: blocks * 16, or up to its last member's token (causal node)
  int64_t node_causal;  // 1: the members are successive tokens of one query run and the node includes their own block
  int64_t members;
  int64_t items;
  // builder scratch
  int64_t s_pos, s_par, s_ord, s_nfull, s_leader, s_lcp, s_run, s_cnt, s_node, s_slot, s_tmp0, s_tmp1, s_nitems;
  int64_t s_sig;  // 64-bit fingerprint of each row's shared blocks, 2 int32 each
  int64_t hash_keys;  // 64-bit keys, 2 int32 each
  int64_t hash_min;
  int64_t hash_size;  // entries (power of two)
  int64_t coop_ctr;   // [kCoopMaxPairs] claim counters of the attention kernel, zero between launches
  int64_t max_items;
  int64_t max_partials;
  int64_t total;
};

inline __host__ __device__ int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

inline __host__ MetaLayout make_layout(const fca_plan& p) {
  MetaLayout L{};
  const int64_t S = p.num_seqs;
  int64_t off = 0;
  auto take = [&](int64_t n) {
    int64_t at = off;
    off = align_up(off + n, 4);  // keep every array 16-byte aligned
    return at;
  };
  // chunks of the nodes on a row's path: at most tokens / chunk plus one per node, and a path
  // holds at most max_levels discovered nodes, one node of a declared group and the leaf
  L.max_partials = (int64_t)p.max_blocks * kBlock / p.chunk_tokens + p.max_levels + 2;
  L.max_items = S * L.max_partials;
  L.header = take(kHeaderInts);
  L.seq_npart = take(S);
  L.seq_leaf_blk = take(S);
  L.node_rep = take(S);
  L.node_blk = take(S);
  L.node_nblk = take(S);
  L.node_level = take(S);
  L.node_moff = take(S);
  L.node_mcnt = take(S);
  L.node_ord = take(S);
  L.node_tok = take(S);
  L.node_causal = take(S);
  L.members = take(S * (FCA_MAX_LEVELS + 2));  // discovery levels, the pass for declared groups, leaves
  L.items = take(L.max_items * kItemInts);
  L.s_pos = take(S);
  L.s_par = take(S);
  L.s_ord = take(S);
  L.s_nfull = take(S);
  L.s_leader = take(S);
  L.s_lcp = take(S);
  L.s_run = take(S);
  L.s_cnt = take(S);
  L.s_node = take(S);
  L.s_slot = take(S);
  L.s_tmp0 = take(S);
  L.s_tmp1 = take(S);
  L.s_nitems = take(2 * S);
  L.s_sig = take(2 * S);
  int64_t hs = 64;
  while (hs < 4 * S) hs <<= 1;
  L.hash_size = hs;
  L.hash_keys = take(2 * hs);
  L.hash_min = take(hs);
  L.coop_ctr = take(kCoopMaxPairs);
  L.total = off;
  return L;
}

// Chunks a node of `tokens` KV tokens is split into, and their common length: an even
// split rounded up to whole MFMA tiles, so no chunk is a sliver.
inline __host__ __device__ int chunk_len_for(int tokens, int chunk_tokens) {
  if (tokens <= 0) return 0;
  int n = (tokens + chunk_tokens - 1) / chunk_tokens;
  int len = (tokens + n - 1) / n;
  return (len + kTile - 1) / kTile * kTile;
}
// Pairs of waves that can share an item under a plan: the attention grid never has more
// than one wave per possible ticket.
inline __host__ int64_t coop_pairs_for(const fca_plan& p, const MetaLayout& L) {
  const int64_t waves = L.max_items * p.num_kv_heads + 3;
  return waves / 2 < kCoopMaxPairs ? waves / 2 : kCoopMaxPairs;
}
inline __host__ __device__ int num_chunks_for(int tokens, int chunk_tokens) {
  if (tokens <= 0) return 0;
  int len = chunk_len_for(tokens, chunk_tokens);
  return (tokens + len - 1) / len;
}

// Device-scope 8-byte accesses: a store that is written through to memory, a load that does
// not trust the L2 of the XCD it runs on.
__device__ inline void store8_coherent(void* ptr, uint64_t v) {
  __hip_atomic_store(reinterpret_cast<uint64_t*>(ptr), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline uint64_t load8_coherent(const void* ptr) {
  return __hip_atomic_load(reinterpret_cast<const uint64_t*>(ptr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct BuildParams {
  fca_plan plan;
  const int32_t* block_table;
  int64_t bt_stride;
  const int32_t* seq_lens;
  int32_t* meta;
  MetaLayout L;
  int32_t try_update;  // keep the forest of the last build if the rows still carry it
  // Query rows that are not one per block-table row (all NULL / 0 for the plain case):
  const int32_t* row_table;  // block-table row of every query row, NULL = the row itself
  const int32_t* row_group;  // >= 0: rows with the same value form one declared group, NULL = none
  int32_t table_rows;        // rows of the block table, bounds row_table
};

struct AttendParams {
  const void* q;
  int64_t q_seq_stride, q_head_stride;  // elements
  const char* k_cache;
  const char* v_cache;
  int64_t kv_block_bytes, kv_head_bytes;
  const int32_t* block_table;
  int64_t bt_stride;
  const float* k_scale;
  const float* v_scale;
  float scale;
  int32_t* meta;
  int64_t off_header, off_items, off_members;
  void* partial_out;   // half [rows, Hq, D], each row times its scale
  float* partial_lse;  // [rows, Hq, 2]: natural-log lse, scale of the row
  int32_t num_q_heads, num_kv_heads, group;  // group = Hq / Hkv
  int32_t max_partials;
  int32_t select;  // 0 all items, 1 shared only, 2 leaves only
  int32_t kv_reread;  // a launch reads KV blocks more than once (query runs): keep the loads cacheable
  // items attended by two waves (32-row kernel): claim counters, how many pairs the partial
  // buffers have rows for, and the first of those rows
  int32_t* coop_ctr;
  int32_t coop_pairs;
  int64_t coop_row0;
};

struct MergeParams {
  const int32_t* header;  // metadata header: a non-zero error slot turns every output into NaN
  const int32_t* seq_npart;
  const void* partial_out;
  const float* partial_lse;
  void* out;
  int64_t out_seq_stride, out_head_stride;
  float* lse;
  int32_t num_seqs, num_q_heads, head_dim, max_partials, out_dtype;
  int32_t vector_out;  // out rows allow 16-byte stores
  int64_t coop_row0;   // first of the partial rows written by waves that took a shared item from the back
  int64_t coop_rows;   // how many such rows the partial buffers hold: a tag that points past them is not followed
  int32_t partial_f32; // the partial rows are fp32 (written by the fp32 attention pass), not scaled halves
};

struct AppendParams {
  const void* key;    // bf16 [T, Hkv, D]
  const void* value;
  int64_t token_stride, head_stride;  // elements
  const int64_t* slot_mapping;        // [T]
  void* k_cache;
  void* v_cache;
  int64_t cache_block_stride, cache_head_stride;  // elements
  const float* k_scale;
  const float* v_scale;
  int32_t num_tokens, num_kv_heads, head_dim;
};

// Split attention over packed training tensors (fca_split.hip).  Tensors are [T, H, D]
// bf16 with a token stride; `t` tensors are transposed tile copies [H][tiles][D][32].
struct SplitParams {
  const void *q, *k, *v, *out_in, *dout;
  int64_t q_stride, k_stride, v_stride, o_stride, do_stride;  // token strides, elements
  // operand images of 32-token tiles, [H][tiles][slot][64 lanes][8]: `n` = rows as the first
  // product of a chain takes them, `r` = transposed as the second product takes them
  const void *kn, *kr, *vn, *vr, *qn, *qr, *don, *dor;
  void* out;
  float* lse;    // [Hq][tiles * 32] natural log
  float* delta;  // [Hq][tiles * 32] rowsum(dout * out)
  float* lse2;   // [Hq][tiles * 32] lse * log2(e), made by the backward's first pass
  void *dq, *dk, *dv;
  int64_t dq_stride, dk_stride, dv_stride;
  const int32_t* layout;
  int32_t num_tokens, num_tiles, num_q_heads, num_kv_heads;
  float scale;
  // small batches: dk and dv are formed per query head (fp32 slices [Hq / Hkv][T][Hkv][D]) and summed afterwards
  int32_t head_split;
  float *dk_part, *dv_part;
  // The general instances of the kernels (chosen when a window or dropout is asked for):
  // window > 0: a row sees only the keys fewer than `window` positions before it in its own
  // sequence (prompt followed by the sample's response); none = a window no sequence reaches.
  int32_t window;
  // Attention dropout: the probability of (query head, row, key) is dropped when
  // split_dropout_hash(...) < drop_thr and scaled by drop_scale = 1 / (1 - p) otherwise.
  uint32_t drop_thr, drop_seed;
  float drop_scale;
};
// The hash that decides dropout, the same for all four kernels and for the tests' restatement:
// one 32-bit mix (two multiplications) of a linear combination of the three indices and the seed.
__host__ __device__ inline uint32_t split_dropout_hash(uint32_t seed, uint32_t head, uint32_t row, uint32_t key) {
  uint32_t x = seed + head * 0xC2B2AE3Du + row * 0x9E3779B1u + key * 0x85EBCA77u;
  x ^= x >> 16;
  x *= 0x7FEB352Du;
  x ^= x >> 15;
  x *= 0x846CA68Bu;
  x ^= x >> 16;
  return x;
}
// A batch with few key tiles leaves most of the chip idle behind its longest walks (a prompt's
// key tiles are seen by the whole group): then every query head of a KV head gets a workgroup
// of its own, which shortens the longest walk by Hq / Hkv.
inline bool split_by_head(int64_t tiles, int num_q_heads, int num_kv_heads) {
  return num_q_heads > num_kv_heads && ((tiles + 3) / 4) * num_kv_heads < 1024;
}
// Offsets into the int32 layout array of a batch of `tiles` 32-token tiles.
struct SplitLayout {
  int64_t kv_lim, q_tiles, kv_qend, q_order, kv_limmin, kv_order, q_index, pos, total;
};
__host__ __device__ inline SplitLayout make_split_layout(int64_t tiles) {
  SplitLayout L;
  L.kv_lim = 0;
  L.q_tiles = 32 * tiles;
  L.kv_qend = L.q_tiles + 4 * tiles;
  L.q_order = L.kv_qend + tiles;
  L.kv_limmin = L.q_order + tiles;
  L.kv_order = L.kv_limmin + tiles;  // ceil(tiles / 4) entries used
  L.q_index = L.kv_order + tiles;  // row of q and out that belongs to a packed token, -1 = none
  L.pos = L.q_index + 32 * tiles;  // position of a packed token in its sample's sequence (prompt, then response)
  L.total = L.pos + 32 * tiles;
  return L;
}
void build_split_layout(int num_groups, const int32_t* prompt_tokens, const int32_t* group_sizes,
                        const int32_t* response_tokens, int64_t tiles, bool responses_only, int32_t window, int32_t* out);
hipError_t launch_split_forward(const SplitParams& p, int head_dim, hipStream_t stream);
hipError_t launch_split_backward(const SplitParams& p, int head_dim, hipStream_t stream);

hipError_t launch_build(const BuildParams& p, hipStream_t stream);
hipError_t launch_rows(const int32_t* query_start_loc, const int32_t* seq_lens, int num_reqs, int num_rows, int max_blocks,
                       int32_t* row_table, int32_t* row_lens, int32_t* row_group, hipStream_t stream);
hipError_t launch_append(const AppendParams& p, int kv_dtype, hipStream_t stream);
hipError_t launch_gather(const AppendParams& p, int kv_dtype, hipStream_t stream);  // key / value are written
// max_workgroups > 0 caps the grid
hipError_t launch_attend(const AttendParams& p, const fca_plan& plan, int kv_dtype, int max_workgroups, int tile_buffers, hipStream_t stream);
// Events the next attention launch of this thread records its begin and end in (NULL: none).
void set_attend_timing(hipEvent_t start, hipEvent_t stop);
void take_attend_timing(hipEvent_t* start, hipEvent_t* stop);
hipError_t launch_attend_f32(const AttendParams& p, const fca_plan& plan, int max_workgroups, hipStream_t stream);
hipError_t launch_attend32(const AttendParams& p, const fca_plan& plan, int kv_dtype, int tile_buffers, int grid, hipStream_t stream);
hipError_t launch_merge(const MergeParams& p, hipStream_t stream);
hipError_t launch_copy(const void* src, void* dst, size_t bytes, hipStream_t stream);
hipError_t launch_gather_rows(const void* src, int64_t src_stride, const int32_t* index, int64_t num_rows, int64_t row_bytes,
                              void* dst, int64_t dst_stride, hipStream_t stream);  // strides in bytes
hipError_t launch_sum_rows(const void* src, int64_t src_stride, const int32_t* offsets, const int32_t* rows, int64_t num_dst_rows,
                           int64_t channels, bool f32, void* dst, int64_t dst_stride, hipStream_t stream);

}  // namespace fca
