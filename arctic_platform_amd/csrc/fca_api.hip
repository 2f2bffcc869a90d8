// C ABI of libzorro_fca.so (declared in include/zorro_fca.h): argument checks and launches.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "fca_common.h"

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(FCA_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int check_plan(const fca_plan* p) {
  if (!p) return fail(FCA_ERR_INVALID_ARG, "plan is NULL");
  if (p->num_seqs < 1) return fail(FCA_ERR_INVALID_ARG, "num_seqs must be >= 1, got %d", p->num_seqs);
  if (p->max_blocks < 1) return fail(FCA_ERR_INVALID_ARG, "max_blocks must be >= 1, got %d", p->max_blocks);
  if (p->block_size != FCA_BLOCK_SIZE)
    return fail(FCA_ERR_UNSUPPORTED, "block_size %d is not supported (only %d)", p->block_size, FCA_BLOCK_SIZE);
  if (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256)
    return fail(FCA_ERR_UNSUPPORTED, "head_dim %d is not supported (64, 128 or 256)", p->head_dim);
  if (p->num_kv_heads < 1 || p->num_q_heads < p->num_kv_heads || p->num_q_heads % p->num_kv_heads)
    return fail(FCA_ERR_INVALID_ARG, "num_q_heads %d must be a positive multiple of num_kv_heads %d", p->num_q_heads,
                p->num_kv_heads);
  if (p->rows_per_item != 32 && p->rows_per_item != 64)
    return fail(FCA_ERR_UNSUPPORTED, "rows_per_item %d is not supported (32 or 64)", p->rows_per_item);
  if (p->head_dim == 256 && p->rows_per_item != 32)
    return fail(FCA_ERR_UNSUPPORTED, "head_dim 256 takes rows_per_item 32 only (two row tiles of accumulators do not fit)");
  if (p->num_q_heads / p->num_kv_heads > p->rows_per_item)
    return fail(FCA_ERR_UNSUPPORTED, "GQA group %d exceeds rows_per_item %d", p->num_q_heads / p->num_kv_heads,
                p->rows_per_item);
  if (p->chunk_tokens < fca::kTile || p->chunk_tokens > fca::kMaxChunk || p->chunk_tokens % fca::kTile)
    return fail(FCA_ERR_INVALID_ARG, "chunk_tokens %d must be a multiple of %d in [%d, %d]", p->chunk_tokens, fca::kTile,
                fca::kTile, fca::kMaxChunk);
  if (p->max_levels < 0 || p->max_levels > FCA_MAX_LEVELS)
    return fail(FCA_ERR_INVALID_ARG, "max_levels %d must be in [0, %d]", p->max_levels, FCA_MAX_LEVELS);
  const fca::MetaLayout L = fca::make_layout(*p);
  if (L.max_items * p->num_kv_heads > 0x7fffffffLL || L.total > 0x7fffffffLL)
    return fail(FCA_ERR_UNSUPPORTED, "batch too large for 32-bit work indices");
  return FCA_OK;
}

int kv_elem_bytes(int kv_dtype) { return kv_dtype == FCA_FP8_E4M3 ? 1 : kv_dtype == FCA_F32 ? 4 : 2; }

// f32_ok: the entry point has an fp32 path (fca_decode_step and fca_decode_step_static)
int check_tensors(const fca_plan* p, const fca_tensors* t, bool f32_ok = false) {
  if (!t) return fail(FCA_ERR_INVALID_ARG, "tensors is NULL");
  if (!t->q_dev || !t->k_cache_dev || !t->v_cache_dev || !t->block_table_dev)
    return fail(FCA_ERR_INVALID_ARG, "q, k_cache, v_cache and block_table must be non-NULL");
  if (t->kv_dtype == FCA_F32) {
    if (!f32_ok)
      return fail(FCA_ERR_UNSUPPORTED, "fp32 tensors (kv_dtype FCA_F32) run through fca_decode_step and fca_decode_step_static only");
    if (p->head_dim != 64 && p->head_dim != 128)
      return fail(FCA_ERR_UNSUPPORTED, "the fp32 path takes head_dim 64 or 128, got %d", p->head_dim);
    if (p->rows_per_item != 32)
      return fail(FCA_ERR_UNSUPPORTED, "the fp32 path takes rows_per_item 32, got %d", p->rows_per_item);
  } else if (t->kv_dtype != FCA_BF16 && t->kv_dtype != FCA_FP8_E4M3) {
    return fail(FCA_ERR_UNSUPPORTED, "kv_dtype %d is not supported (bf16, fp8 e4m3, or fp32 with an fp32 q)", t->kv_dtype);
  }
  const int esz = kv_elem_bytes(t->kv_dtype);
  if ((reinterpret_cast<uintptr_t>(t->q_dev) & 15) || (t->q_seq_stride % 8) || (t->q_head_stride % 8))
    return fail(FCA_ERR_INVALID_ARG, "q must be 16-byte aligned with strides that are multiples of 8 elements");
  if ((reinterpret_cast<uintptr_t>(t->k_cache_dev) & 15) || (reinterpret_cast<uintptr_t>(t->v_cache_dev) & 15) ||
      (t->kv_block_stride * esz) % 16 || (t->kv_head_stride * esz) % 16)
    return fail(FCA_ERR_INVALID_ARG, "KV cache planes must be 16-byte aligned with 16-byte-multiple strides");
  if (t->kv_head_stride < (int64_t)FCA_BLOCK_SIZE * p->head_dim)
    return fail(FCA_ERR_INVALID_ARG, "kv_head_stride %lld is smaller than one tile (%d elements)",
                (long long)t->kv_head_stride, FCA_BLOCK_SIZE * p->head_dim);
  if (t->block_table_stride < p->max_blocks)
    return fail(FCA_ERR_INVALID_ARG, "block_table_stride %lld is smaller than max_blocks %d",
                (long long)t->block_table_stride, p->max_blocks);
  if (t->max_workgroups < 0) return fail(FCA_ERR_INVALID_ARG, "max_workgroups must be >= 0, got %d", t->max_workgroups);
  if (t->tile_buffers != 0 &&
      !(t->tile_buffers == 3 && t->kv_dtype == FCA_FP8_E4M3 && p->head_dim == 128 && p->rows_per_item == 32))
    return fail(FCA_ERR_UNSUPPORTED,
                "tile_buffers %d: 0, or 3 for an fp8 cache at head_dim 128 with rows_per_item 32 (got kv_dtype %d, head_dim %d, rows_per_item %d)",
                t->tile_buffers, t->kv_dtype, p->head_dim, p->rows_per_item);
  return FCA_OK;
}

fca::AttendParams attend_params(const fca_plan* p, const fca_tensors* t, void* meta, void* po, float* pl, int select) {
  const fca::MetaLayout L = fca::make_layout(*p);
  const int esz = kv_elem_bytes(t->kv_dtype);
  fca::AttendParams a{};
  a.q = t->q_dev;
  a.q_seq_stride = t->q_seq_stride;
  a.q_head_stride = t->q_head_stride;
  a.k_cache = static_cast<const char*>(t->k_cache_dev);
  a.v_cache = static_cast<const char*>(t->v_cache_dev);
  a.kv_block_bytes = t->kv_block_stride * esz;
  a.kv_head_bytes = t->kv_head_stride * esz;
  a.block_table = t->block_table_dev;
  a.bt_stride = t->block_table_stride;
  a.k_scale = t->k_scale_dev;
  a.v_scale = t->v_scale_dev;
  a.scale = t->softmax_scale;
  a.meta = static_cast<int32_t*>(meta);
  a.off_header = L.header;
  a.off_items = L.items;
  a.off_members = L.members;
  a.partial_out = po;
  a.partial_lse = pl;
  a.num_q_heads = p->num_q_heads;
  a.num_kv_heads = p->num_kv_heads;
  a.group = p->num_q_heads / p->num_kv_heads;
  a.max_partials = (int32_t)L.max_partials;
  a.select = select;
  a.kv_reread = t->kv_reread;
  // Items attended by two waves together: not when the caller wants the same bits from every
  // launch, and not in a launch over the private items alone, whose second partials would land
  // in the rows the launch over the shared items has just written for the same merge.
  a.coop_ctr = t->reproducible || select == 2 ? nullptr : a.meta + L.coop_ctr;
  a.coop_pairs = (int32_t)fca::coop_pairs_for(*p, L);
  a.coop_row0 = (int64_t)p->num_seqs * L.max_partials * p->num_q_heads;
  return a;
}

int run_attend(const fca_plan* p, const fca_tensors* t, void* meta, void* po, float* pl, int select, void* stream,
               bool f32_ok = false) {
  if (int rc = check_plan(p)) return rc;
  if (int rc = check_tensors(p, t, f32_ok)) return rc;
  if (!meta || !po || !pl) return fail(FCA_ERR_INVALID_ARG, "metadata and partial workspaces must be non-NULL");
  if ((reinterpret_cast<uintptr_t>(po) & 15) || (reinterpret_cast<uintptr_t>(pl) & 15))
    return fail(FCA_ERR_INVALID_ARG, "partial workspaces must be 16-byte aligned");
  const fca::AttendParams a = attend_params(p, t, meta, po, pl, select);
  hipError_t e = t->kv_dtype == FCA_F32
                     ? fca::launch_attend_f32(a, *p, t->max_workgroups, static_cast<hipStream_t>(stream))
                     : fca::launch_attend(a, *p, t->kv_dtype, t->max_workgroups, t->tile_buffers, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "attention pass launch");
}

int run_merge(const fca_plan* p, const void* meta, const void* po, const float* pl, void* out, int64_t oss, int64_t ohs,
              int32_t out_dtype, float* lse, void* stream, bool partial_f32 = false) {
  if (int rc = check_plan(p)) return rc;
  if (!meta || !po || !pl || !out) return fail(FCA_ERR_INVALID_ARG, "metadata, partials and out must be non-NULL");
  if (out_dtype != FCA_BF16 && out_dtype != FCA_F32)
    return fail(FCA_ERR_UNSUPPORTED, "out dtype %d is not supported (bf16 or f32)", out_dtype);
  if ((reinterpret_cast<uintptr_t>(po) & 15) || (reinterpret_cast<uintptr_t>(pl) & 15))
    return fail(FCA_ERR_INVALID_ARG, "partial workspaces must be 16-byte aligned");
  const fca::MetaLayout L = fca::make_layout(*p);
  fca::MergeParams m{};
  m.header = static_cast<const int32_t*>(meta) + L.header;
  m.seq_npart = static_cast<const int32_t*>(meta) + L.seq_npart;
  m.partial_out = po;
  m.partial_lse = pl;
  m.out = out;
  m.out_seq_stride = oss;
  m.out_head_stride = ohs;
  m.lse = lse;
  m.num_seqs = p->num_seqs;
  m.num_q_heads = p->num_q_heads;
  m.head_dim = p->head_dim;
  m.max_partials = (int32_t)L.max_partials;
  m.coop_row0 = (int64_t)p->num_seqs * L.max_partials * p->num_q_heads;
  m.coop_rows = 32 * fca::coop_pairs_for(*p, L);
  m.partial_f32 = partial_f32;
  m.out_dtype = out_dtype;
  // whole 16-byte stores when every 8-channel group of out is 16-byte aligned
  const int64_t esz = out_dtype == FCA_F32 ? 4 : 2;
  m.vector_out = !(reinterpret_cast<uintptr_t>(out) & 15) && (oss * esz) % 16 == 0 && (ohs * esz) % 16 == 0;
  hipError_t e = fca::launch_merge(m, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "merge launch");
}

}  // namespace

extern "C" {

int fca_version(void) { return FCA_VERSION; }

const char* fca_last_error(void) { return g_error; }

int fca_workspace_bytes(const fca_plan* plan, size_t* meta_bytes, size_t* partial_out_bytes, size_t* partial_lse_bytes) {
  return fca_workspace_bytes_dtype(plan, FCA_BF16, meta_bytes, partial_out_bytes, partial_lse_bytes);
}

int fca_workspace_bytes_dtype(const fca_plan* plan, int32_t kv_dtype, size_t* meta_bytes, size_t* partial_out_bytes,
                              size_t* partial_lse_bytes) {
  if (int rc = check_plan(plan)) return rc;
  if (kv_dtype != FCA_BF16 && kv_dtype != FCA_FP8_E4M3 && kv_dtype != FCA_F32)
    return fail(FCA_ERR_UNSUPPORTED, "kv_dtype %d is not supported (bf16, fp8 e4m3 or fp32)", kv_dtype);
  const fca::MetaLayout L = fca::make_layout(*plan);
  // one row per (partial slot, query head), then 32 rows per pair of waves that may share an item
  const size_t rows = (size_t)plan->num_seqs * (size_t)L.max_partials * plan->num_q_heads + 32 * (size_t)fca::coop_pairs_for(*plan, L);
  if (meta_bytes) *meta_bytes = (size_t)L.total * sizeof(int32_t);
  if (partial_out_bytes) *partial_out_bytes = rows * plan->head_dim * (kv_dtype == FCA_F32 ? 4 : 2);  // fp32 or half
  if (partial_lse_bytes) *partial_lse_bytes = rows * 2 * sizeof(float);    // {lse, scale}
  return FCA_OK;
}

int fca_meta_describe(const fca_plan* plan, fca_meta_layout* out) {
  if (int rc = check_plan(plan)) return rc;
  if (!out) return fail(FCA_ERR_INVALID_ARG, "layout is NULL");
  const fca::MetaLayout L = fca::make_layout(*plan);
  out->header = L.header;
  out->seq_npart = L.seq_npart;
  out->seq_leaf_blk = L.seq_leaf_blk;
  out->node_rep = L.node_rep;
  out->node_blk = L.node_blk;
  out->node_nblk = L.node_nblk;
  out->node_level = L.node_level;
  out->node_moff = L.node_moff;
  out->node_mcnt = L.node_mcnt;
  out->node_ord = L.node_ord;
  out->members = L.members;
  out->items = L.items;
  out->max_items = L.max_items;
  out->max_partials = L.max_partials;
  out->total_int32 = L.total;
  out->node_tok = L.node_tok;
  out->node_causal = L.node_causal;
  out->coop_ctr = L.coop_ctr;
  return FCA_OK;
}

static int run_build(const fca_plan* plan, const int32_t* block_table_dev, int64_t block_table_stride,
                     const int32_t* seq_lens_dev, void* meta_dev, int try_update, void* stream,
                     int32_t table_rows = 0, const int32_t* row_table_dev = nullptr,
                     const int32_t* row_group_dev = nullptr) {
  if (int rc = check_plan(plan)) return rc;
  if (row_table_dev && table_rows < 1)
    return fail(FCA_ERR_INVALID_ARG, "table_rows must be >= 1 when a row table is given, got %d", table_rows);
  if (!block_table_dev || !seq_lens_dev || !meta_dev)
    return fail(FCA_ERR_INVALID_ARG, "block_table, seq_lens and metadata workspace must be non-NULL");
  if (block_table_stride < plan->max_blocks)
    return fail(FCA_ERR_INVALID_ARG, "block_table_stride %lld is smaller than max_blocks %d",
                (long long)block_table_stride, plan->max_blocks);
  if (reinterpret_cast<uintptr_t>(meta_dev) & 15)
    return fail(FCA_ERR_INVALID_ARG, "metadata workspace must be 16-byte aligned");
  fca::BuildParams b{};
  b.plan = *plan;
  b.block_table = block_table_dev;
  b.bt_stride = block_table_stride;
  b.seq_lens = seq_lens_dev;
  b.meta = static_cast<int32_t*>(meta_dev);
  b.L = fca::make_layout(*plan);
  b.try_update = try_update;
  b.row_table = row_table_dev;
  b.row_group = row_group_dev;
  b.table_rows = table_rows;
  hipError_t e = fca::launch_build(b, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "metadata builder launch");
}

int fca_build_metadata(const fca_plan* plan, const int32_t* block_table_dev, int64_t block_table_stride,
                       const int32_t* seq_lens_dev, void* meta_dev, void* stream) {
  return run_build(plan, block_table_dev, block_table_stride, seq_lens_dev, meta_dev, 0, stream);
}

int fca_update_metadata(const fca_plan* plan, const int32_t* block_table_dev, int64_t block_table_stride,
                        const int32_t* seq_lens_dev, void* meta_dev, void* stream) {
  return run_build(plan, block_table_dev, block_table_stride, seq_lens_dev, meta_dev, 1, stream);
}

int fca_build_metadata_rows(const fca_plan* plan, const int32_t* block_table_dev, int64_t block_table_stride,
                            int32_t table_rows, const int32_t* row_table_dev, const int32_t* row_group_dev,
                            const int32_t* row_lens_dev, void* meta_dev, int32_t update, void* stream) {
  return run_build(plan, block_table_dev, block_table_stride, row_lens_dev, meta_dev, update ? 1 : 0, stream, table_rows,
                   row_table_dev, row_group_dev);
}

int fca_rows_from_query_runs(const int32_t* query_start_loc_dev, const int32_t* seq_lens_dev, int32_t num_reqs,
                             int32_t num_rows, int32_t max_blocks, int32_t* row_table_dev, int32_t* row_lens_dev,
                             int32_t* row_group_dev, void* stream) {
  if (num_reqs < 1 || num_rows < 0 || max_blocks < 1)
    return fail(FCA_ERR_INVALID_ARG, "num_reqs and max_blocks must be >= 1 and num_rows >= 0");
  if ((int64_t)num_reqs * max_blocks > 0x7fffffffLL)
    return fail(FCA_ERR_UNSUPPORTED, "num_reqs * max_blocks exceeds 32-bit group ids");
  if (num_rows == 0) return FCA_OK;
  if (!query_start_loc_dev || !seq_lens_dev || !row_table_dev || !row_lens_dev || !row_group_dev)
    return fail(FCA_ERR_INVALID_ARG, "query_start_loc, seq_lens and the three row arrays must be non-NULL");
  hipError_t e = fca::launch_rows(query_start_loc_dev, seq_lens_dev, num_reqs, num_rows, max_blocks, row_table_dev,
                                  row_lens_dev, row_group_dev, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "query-row kernel launch");
}

int fca_prefix_pass(const fca_plan* plan, const fca_tensors* t, void* meta_dev, void* partial_out_dev,
                    float* partial_lse_dev, void* stream) {
  return run_attend(plan, t, meta_dev, partial_out_dev, partial_lse_dev, 1, stream);
}

int fca_suffix_pass(const fca_plan* plan, const fca_tensors* t, void* meta_dev, void* partial_out_dev,
                    float* partial_lse_dev, void* stream) {
  return run_attend(plan, t, meta_dev, partial_out_dev, partial_lse_dev, 2, stream);
}

int fca_forest_pass(const fca_plan* plan, const fca_tensors* t, void* meta_dev, void* partial_out_dev,
                    float* partial_lse_dev, void* stream) {
  return run_attend(plan, t, meta_dev, partial_out_dev, partial_lse_dev, 0, stream);
}

int fca_merge(const fca_plan* plan, const void* meta_dev, const void* partial_out_dev, const float* partial_lse_dev,
              void* out_dev, int64_t out_seq_stride, int64_t out_head_stride, int32_t out_dtype, float* lse_dev,
              void* stream) {
  return run_merge(plan, meta_dev, partial_out_dev, partial_lse_dev, out_dev, out_seq_stride, out_head_stride, out_dtype,
                   lse_dev, stream);
}

int fca_decode_step(const fca_plan* plan, const fca_tensors* t, void* meta_dev, void* partial_out_dev,
                    float* partial_lse_dev, void* out_dev, int64_t out_seq_stride, int64_t out_head_stride,
                    int32_t out_dtype, float* lse_dev, void* stream) {
  if (int rc = run_attend(plan, t, meta_dev, partial_out_dev, partial_lse_dev, 0, stream, true)) return rc;
  return run_merge(plan, meta_dev, partial_out_dev, partial_lse_dev, out_dev, out_seq_stride, out_head_stride, out_dtype,
                   lse_dev, stream, t->kv_dtype == FCA_F32);
}

}  // extern "C"

// ---- decode step on the library's own partial buffers ----------------------------------
// The partial rows of fca_decode_step_static live in this array instead of caller memory.
// Every GPU the library runs on holds its own copy at its own address; host code may only
// use the address hipGetSymbolAddress reports for the current device, never the name.
static __device__ __align__(256) unsigned char scratch[FCA_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];  // device address of `scratch`, per device, once looked up
std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch` (looked up on the first call per device).
int static_scratch(unsigned char** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return fail(FCA_ERR_UNSUPPORTED, "device ordinal %d is beyond %d", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (!p || (reinterpret_cast<uintptr_t>(p) & 255)) return fail(FCA_ERR_HIP, "static scratch has no usable device address");
    g_scratch_ptr[dev] = p;
  }
  *ptr = static_cast<unsigned char*>(g_scratch_ptr[dev]);
  return FCA_OK;
}
}  // namespace

extern "C" {

int fca_decode_step_static(const fca_plan* plan, const fca_tensors* t, void* meta_dev, void* out_dev,
                           int64_t out_seq_stride, int64_t out_head_stride, int32_t out_dtype, float* lse_dev,
                           void* stream) {
  size_t po = 0, pl = 0;
  if (!t) return fail(FCA_ERR_INVALID_ARG, "tensors is NULL");
  if (int rc = fca_workspace_bytes_dtype(plan, t->kv_dtype, nullptr, &po, &pl)) return rc;
  const size_t lse_at = (po + 255) / 256 * 256;
  if (lse_at + pl > (size_t)FCA_STATIC_SCRATCH_BYTES)
    return fail(FCA_ERR_UNSUPPORTED,
                "the partial rows of this plan need %zu bytes, the static scratch holds %zu: use fca_decode_step with "
                "caller-owned partial buffers (or a larger chunk_tokens / fewer sequences)",
                lse_at + pl, (size_t)FCA_STATIC_SCRATCH_BYTES);
  unsigned char* base = nullptr;
  if (int rc = static_scratch(&base)) return rc;
  // Every partial slot the merge reads (ord < partial count of its sequence) is written by
  // the attention launch of the same call, so nothing of the last call's contents is read.
  void* partial_out = base;
  float* partial_lse = reinterpret_cast<float*>(base + lse_at);
  if (int rc = run_attend(plan, t, meta_dev, partial_out, partial_lse, 0, stream, true)) return rc;
  return run_merge(plan, meta_dev, partial_out, partial_lse, out_dev, out_seq_stride, out_head_stride, out_dtype, lse_dev,
                   stream, t->kv_dtype == FCA_F32);
}

static int cache_rows(bool gather, const void* key_dev, const void* value_dev, int64_t token_stride, int64_t head_stride,
                      int32_t num_tokens, int32_t num_kv_heads, int32_t head_dim, const int64_t* slot_mapping_dev,
                      void* k_cache_dev, void* v_cache_dev, int64_t kv_block_stride, int64_t kv_head_stride, int32_t kv_dtype,
                      const float* k_scale_dev, const float* v_scale_dev, void* stream) {
  if (num_tokens < 0 || num_kv_heads < 1) return fail(FCA_ERR_INVALID_ARG, "num_tokens must be >= 0 and num_kv_heads >= 1");
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail(FCA_ERR_UNSUPPORTED, "head_dim %d is not supported (64, 128 or 256)", head_dim);
  if (kv_dtype != FCA_BF16 && kv_dtype != FCA_FP8_E4M3 && kv_dtype != FCA_F32)
    return fail(FCA_ERR_UNSUPPORTED, "kv_dtype %d is not supported (bf16, fp8 e4m3, or fp32 with fp32 rows)", kv_dtype);
  if (num_tokens == 0) return FCA_OK;
  if (!key_dev || !value_dev || !slot_mapping_dev || !k_cache_dev || !v_cache_dev)
    return fail(FCA_ERR_INVALID_ARG, "key, value, slot_mapping and the cache planes must be non-NULL");
  const int esz = kv_elem_bytes(kv_dtype);
  if ((reinterpret_cast<uintptr_t>(key_dev) & 15) || (reinterpret_cast<uintptr_t>(value_dev) & 15) || token_stride % 8 ||
      head_stride % 8)
    return fail(FCA_ERR_INVALID_ARG, "key and value must be 16-byte aligned with strides that are multiples of 8 elements");
  if ((reinterpret_cast<uintptr_t>(k_cache_dev) & 15) || (reinterpret_cast<uintptr_t>(v_cache_dev) & 15) ||
      (kv_block_stride * esz) % 16 || (kv_head_stride * esz) % 16 || kv_head_stride < (int64_t)FCA_BLOCK_SIZE * head_dim)
    return fail(FCA_ERR_INVALID_ARG, "KV cache planes must be 16-byte aligned with 16-byte-multiple strides of at least one tile");
  fca::AppendParams a{};
  a.key = key_dev;
  a.value = value_dev;
  a.token_stride = token_stride;
  a.head_stride = head_stride;
  a.slot_mapping = slot_mapping_dev;
  a.k_cache = k_cache_dev;
  a.v_cache = v_cache_dev;
  a.cache_block_stride = kv_block_stride;
  a.cache_head_stride = kv_head_stride;
  a.k_scale = k_scale_dev;
  a.v_scale = v_scale_dev;
  a.num_tokens = num_tokens;
  a.num_kv_heads = num_kv_heads;
  a.head_dim = head_dim;
  hipError_t e = gather ? fca::launch_gather(a, kv_dtype, static_cast<hipStream_t>(stream))
                        : fca::launch_append(a, kv_dtype, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, gather ? "cache gather launch" : "cache append launch");
}

int fca_append_kv(const void* key_dev, const void* value_dev, int64_t token_stride, int64_t head_stride,
                  int32_t num_tokens, int32_t num_kv_heads, int32_t head_dim, const int64_t* slot_mapping_dev,
                  void* k_cache_dev, void* v_cache_dev, int64_t kv_block_stride, int64_t kv_head_stride, int32_t kv_dtype,
                  const float* k_scale_dev, const float* v_scale_dev, void* stream) {
  return cache_rows(false, key_dev, value_dev, token_stride, head_stride, num_tokens, num_kv_heads, head_dim, slot_mapping_dev,
                    k_cache_dev, v_cache_dev, kv_block_stride, kv_head_stride, kv_dtype, k_scale_dev, v_scale_dev, stream);
}

int fca_gather_kv(void* key_dev, void* value_dev, int64_t token_stride, int64_t head_stride, int32_t num_tokens,
                  int32_t num_kv_heads, int32_t head_dim, const int64_t* slot_mapping_dev, const void* k_cache_dev,
                  const void* v_cache_dev, int64_t kv_block_stride, int64_t kv_head_stride, int32_t kv_dtype,
                  const float* k_scale_dev, const float* v_scale_dev, void* stream) {
  return cache_rows(true, key_dev, value_dev, token_stride, head_stride, num_tokens, num_kv_heads, head_dim, slot_mapping_dev,
                    const_cast<void*>(k_cache_dev), const_cast<void*>(v_cache_dev), kv_block_stride, kv_head_stride, kv_dtype,
                    k_scale_dev, v_scale_dev, stream);
}

int fca_time_next_attention(void* start_event, void* stop_event) {
  if ((start_event == nullptr) != (stop_event == nullptr))
    return fail(FCA_ERR_INVALID_ARG, "start and stop events come as a pair (both or neither)");
  // A profiler that intercepts dispatches (rocprofv3 announces its tool library in the
  // environment of the program it starts) holds every dispatch's completion signal itself:
  // a launch that also carries events is refused there, not tried.
  static const bool profiled = [] {
    const char* tool = getenv("ROCP_TOOL_LIBRARIES");
    return tool != nullptr && tool[0] != 0;
  }();
  if (profiled && start_event)
    return fail(FCA_ERR_UNSUPPORTED, "launches are not timed with events under a profiler (ROCP_TOOL_LIBRARIES is set): "
                                     "take the kernel durations from its trace");
  fca::set_attend_timing(static_cast<hipEvent_t>(start_event), static_cast<hipEvent_t>(stop_event));
  return FCA_OK;
}

int fca_calibration_copy(const void* src_dev, void* dst_dev, size_t bytes, void* stream) {
  if (!src_dev || !dst_dev || (bytes & 15) || (reinterpret_cast<uintptr_t>(src_dev) & 15) ||
      (reinterpret_cast<uintptr_t>(dst_dev) & 15))
    return fail(FCA_ERR_INVALID_ARG, "calibration copy needs 16-byte aligned pointers and a multiple of 16 bytes");
  hipError_t e = fca::launch_copy(src_dev, dst_dev, bytes, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "calibration copy launch");
}

}  // extern "C"

namespace {
int check_split(const fca_split_plan* p) {
  if (!p) return fail(FCA_ERR_INVALID_ARG, "plan is NULL");
  if (p->num_tokens < 0 || p->num_tokens > (1 << 30)) return fail(FCA_ERR_INVALID_ARG, "num_tokens %d is out of range", p->num_tokens);
  if (p->head_dim != 64 && p->head_dim != 128 && p->head_dim != 256)
    return fail(FCA_ERR_UNSUPPORTED, "head_dim %d is not supported (64, 128 or 256)", p->head_dim);
  if (p->num_kv_heads < 1 || p->num_q_heads < p->num_kv_heads || p->num_q_heads % p->num_kv_heads)
    return fail(FCA_ERR_INVALID_ARG, "num_q_heads %d must be a positive multiple of num_kv_heads %d", p->num_q_heads,
                p->num_kv_heads);
  if (p->head_dim == 256 && (p->num_q_heads / p->num_kv_heads) % 4)
    return fail(FCA_ERR_UNSUPPORTED,
                "head_dim 256 takes a multiple of 4 query heads per KV head (got %d): only the kernels that share "
                "their operands through LDS have an instance of that size",
                p->num_q_heads / p->num_kv_heads);
  if (p->window < 0) return fail(FCA_ERR_INVALID_ARG, "window must be >= 0 (0 = none), got %d", p->window);
  if (!(p->dropout_p >= 0.f && p->dropout_p < 1.f))
    return fail(FCA_ERR_INVALID_ARG, "dropout_p must lie in [0, 1), got %g", (double)p->dropout_p);
  return FCA_OK;
}
// window, dropout threshold, scale and seed of a plan, as the kernels take them
void split_options(const fca_split_plan* plan, fca::SplitParams* p) {
  p->window = plan->window;
  p->drop_thr = 0, p->drop_scale = 1.f, p->drop_seed = 0;
  if (plan->dropout_p > 0.f) {
    const double thr = (double)plan->dropout_p * 4294967296.0;
    p->drop_thr = thr >= 4294967295.0 ? 4294967295u : thr < 1.0 ? 1u : (uint32_t)thr;
    p->drop_scale = 1.f / (1.f - plan->dropout_p);
    p->drop_seed = plan->dropout_seed;
    // the general instances test a window too: one that no sequence reaches
    if (p->window == 0) p->window = 0x3fffffff;
  }
}
int check_rows(const char* name, const void* ptr, int64_t stride, int heads, int head_dim) {
  if (!ptr) return fail(FCA_ERR_INVALID_ARG, "%s is NULL", name);
  if ((reinterpret_cast<uintptr_t>(ptr) & 15) || stride % 8 || stride < (int64_t)heads * head_dim)
    return fail(FCA_ERR_INVALID_ARG, "%s must be 16-byte aligned with a row stride that is a multiple of 8 and at least heads * head_dim", name);
  return FCA_OK;
}
struct SplitScratch {
  size_t kv_tiles, q_tiles, delta, head_slices;  // bytes
};
SplitScratch split_scratch(const fca_split_plan* p) {
  const size_t tiles = (p->num_tokens + 31) / 32, padded = 32 * tiles;
  const size_t slices = fca::split_by_head(tiles, p->num_q_heads, p->num_kv_heads)
                            ? (size_t)(p->num_q_heads / p->num_kv_heads) * p->num_tokens * p->num_kv_heads * p->head_dim * 4
                            : 0;
  return {padded * p->num_kv_heads * p->head_dim * 2, padded * p->num_q_heads * p->head_dim * 2, padded * p->num_q_heads * 4,
          (slices + 15) / 16 * 16};
}
}  // namespace

extern "C" {

int fca_split_layout_ints(int32_t num_tokens, int64_t* num_ints) {
  if (num_tokens < 0 || !num_ints) return fail(FCA_ERR_INVALID_ARG, "num_tokens must be >= 0 and num_ints non-NULL");
  *num_ints = fca::make_split_layout((num_tokens + 31) / 32).total;
  return FCA_OK;
}

int fca_split_layout_build(int32_t num_groups, const int32_t* prompt_tokens, const int32_t* group_sizes,
                           const int32_t* response_tokens, int32_t num_tokens, int32_t responses_only, int32_t window,
                           int32_t* layout_host) {
  if (num_groups < 0 || num_tokens < 0) return fail(FCA_ERR_INVALID_ARG, "num_groups and num_tokens must be >= 0");
  if (window < 0) return fail(FCA_ERR_INVALID_ARG, "window must be >= 0 (0 = none), got %d", window);
  if (num_groups > 0 && (!prompt_tokens || !group_sizes)) return fail(FCA_ERR_INVALID_ARG, "prompt_tokens and group_sizes must be non-NULL");
  int64_t total = 0, samples = 0;
  for (int g = 0; g < num_groups; ++g) {
    if (prompt_tokens[g] < 0 || group_sizes[g] < 0) return fail(FCA_ERR_INVALID_ARG, "group %d has a negative count", g);
    total += prompt_tokens[g];
    for (int s = 0; s < group_sizes[g]; ++s) {
      if (!response_tokens || response_tokens[samples + s] < 0)
        return fail(FCA_ERR_INVALID_ARG, "response_tokens is NULL or negative for sample %lld", (long long)(samples + s));
      total += response_tokens[samples + s];
    }
    samples += group_sizes[g];
  }
  if (total != num_tokens)
    return fail(FCA_ERR_INVALID_ARG, "the layout holds %lld tokens, num_tokens says %d", (long long)total, num_tokens);
  if (num_tokens == 0) return FCA_OK;
  if (!layout_host) return fail(FCA_ERR_INVALID_ARG, "layout_host is NULL");
  fca::build_split_layout(num_groups, prompt_tokens, group_sizes, response_tokens, (num_tokens + 31) / 32, responses_only != 0,
                          window, layout_host);
  return FCA_OK;
}

int fca_split_workspace_bytes(const fca_split_plan* plan, size_t* forward_bytes, size_t* backward_bytes) {
  if (int rc = check_split(plan)) return rc;
  const SplitScratch s = split_scratch(plan);
  if (forward_bytes) *forward_bytes = 2 * s.kv_tiles;
  if (backward_bytes) *backward_bytes = 3 * s.kv_tiles + 4 * s.q_tiles + 2 * s.delta + 2 * s.head_slices;
  return FCA_OK;
}

int fca_split_attention_forward(const fca_split_plan* plan, const void* q_dev, int64_t q_stride, const void* k_dev,
                                int64_t k_stride, const void* v_dev, int64_t v_stride, const int32_t* layout_dev,
                                float scale, void* workspace_dev, void* out_dev, int64_t out_stride, float* lse_dev,
                                void* stream) {
  if (int rc = check_split(plan)) return rc;
  if (plan->num_tokens == 0) return FCA_OK;
  if (!(scale > 0.f)) return fail(FCA_ERR_INVALID_ARG, "scale must be positive");
  if (int rc = check_rows("q", q_dev, q_stride, plan->num_q_heads, plan->head_dim)) return rc;
  if (int rc = check_rows("k", k_dev, k_stride, plan->num_kv_heads, plan->head_dim)) return rc;
  if (int rc = check_rows("v", v_dev, v_stride, plan->num_kv_heads, plan->head_dim)) return rc;
  if (int rc = check_rows("out", out_dev, out_stride, plan->num_q_heads, plan->head_dim)) return rc;
  if (!layout_dev || !workspace_dev || !lse_dev || (reinterpret_cast<uintptr_t>(layout_dev) & 15) ||
      (reinterpret_cast<uintptr_t>(workspace_dev) & 15) || (reinterpret_cast<uintptr_t>(lse_dev) & 15))
    return fail(FCA_ERR_INVALID_ARG, "layout, workspace and lse must be non-NULL and 16-byte aligned");
  fca::SplitParams p{};
  p.q = q_dev, p.k = k_dev, p.v = v_dev;
  p.q_stride = q_stride, p.k_stride = k_stride, p.v_stride = v_stride, p.o_stride = out_stride;
  p.kn = workspace_dev;
  p.vr = static_cast<char*>(workspace_dev) + split_scratch(plan).kv_tiles;
  p.out = out_dev;
  p.lse = lse_dev;
  p.layout = layout_dev;
  p.num_tokens = plan->num_tokens;
  p.num_tiles = (plan->num_tokens + 31) / 32;
  p.num_q_heads = plan->num_q_heads;
  p.num_kv_heads = plan->num_kv_heads;
  p.scale = scale;
  split_options(plan, &p);
  hipError_t e = fca::launch_split_forward(p, plan->head_dim, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "split attention forward launch");
}

int fca_split_attention_backward(const fca_split_plan* plan, const void* q_dev, int64_t q_stride, const void* k_dev,
                                 int64_t k_stride, const void* v_dev, int64_t v_stride, const void* out_dev,
                                 int64_t out_stride, const void* dout_dev, int64_t dout_stride, const float* lse_dev,
                                 const int32_t* layout_dev, float scale, void* workspace_dev, void* dq_dev,
                                 int64_t dq_stride, void* dk_dev, int64_t dk_stride, void* dv_dev, int64_t dv_stride,
                                 void* stream) {
  if (int rc = check_split(plan)) return rc;
  if (plan->num_tokens == 0) return FCA_OK;
  if (!(scale > 0.f)) return fail(FCA_ERR_INVALID_ARG, "scale must be positive");
  const int hq = plan->num_q_heads, hkv = plan->num_kv_heads, d = plan->head_dim;
  if (int rc = check_rows("q", q_dev, q_stride, hq, d)) return rc;
  if (int rc = check_rows("k", k_dev, k_stride, hkv, d)) return rc;
  if (int rc = check_rows("v", v_dev, v_stride, hkv, d)) return rc;
  if (int rc = check_rows("out", out_dev, out_stride, hq, d)) return rc;
  if (int rc = check_rows("dout", dout_dev, dout_stride, hq, d)) return rc;
  if (int rc = check_rows("dq", dq_dev, dq_stride, hq, d)) return rc;
  if (int rc = check_rows("dk", dk_dev, dk_stride, hkv, d)) return rc;
  if (int rc = check_rows("dv", dv_dev, dv_stride, hkv, d)) return rc;
  if (!layout_dev || !workspace_dev || !lse_dev || (reinterpret_cast<uintptr_t>(layout_dev) & 15) ||
      (reinterpret_cast<uintptr_t>(workspace_dev) & 15) || (reinterpret_cast<uintptr_t>(lse_dev) & 15))
    return fail(FCA_ERR_INVALID_ARG, "layout, workspace and lse must be non-NULL and 16-byte aligned");
  const SplitScratch s = split_scratch(plan);
  char* ws = static_cast<char*>(workspace_dev);
  fca::SplitParams p{};
  p.q = q_dev, p.k = k_dev, p.v = v_dev, p.out_in = out_dev, p.dout = dout_dev;
  p.q_stride = q_stride, p.k_stride = k_stride, p.v_stride = v_stride, p.o_stride = out_stride, p.do_stride = dout_stride;
  p.kn = ws;
  p.kr = ws + s.kv_tiles;
  p.vn = ws + 2 * s.kv_tiles;
  p.qn = ws + 3 * s.kv_tiles;
  p.qr = ws + 3 * s.kv_tiles + s.q_tiles;
  p.don = ws + 3 * s.kv_tiles + 2 * s.q_tiles;
  p.dor = ws + 3 * s.kv_tiles + 3 * s.q_tiles;
  p.delta = reinterpret_cast<float*>(ws + 3 * s.kv_tiles + 4 * s.q_tiles);
  p.lse2 = reinterpret_cast<float*>(ws + 3 * s.kv_tiles + 4 * s.q_tiles + s.delta);
  p.head_split = s.head_slices > 0;
  p.dk_part = reinterpret_cast<float*>(ws + 3 * s.kv_tiles + 4 * s.q_tiles + 2 * s.delta);
  p.dv_part = reinterpret_cast<float*>(ws + 3 * s.kv_tiles + 4 * s.q_tiles + 2 * s.delta + s.head_slices);
  p.lse = const_cast<float*>(lse_dev);
  p.dq = dq_dev, p.dk = dk_dev, p.dv = dv_dev;
  p.dq_stride = dq_stride, p.dk_stride = dk_stride, p.dv_stride = dv_stride;
  p.layout = layout_dev;
  p.num_tokens = plan->num_tokens;
  p.num_tiles = (plan->num_tokens + 31) / 32;
  p.num_q_heads = hq;
  p.num_kv_heads = hkv;
  p.scale = scale;
  split_options(plan, &p);
  hipError_t e = fca::launch_split_backward(p, d, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "split attention backward launch");
}

}  // extern "C"

// ---- rows of a deduplicated tensor to whole samples and back -----------------------------
extern "C" {

int fca_gather_rows(const void* src_dev, int64_t src_stride_bytes, const int32_t* index_dev, int64_t num_rows, int64_t row_bytes,
                    void* dst_dev, int64_t dst_stride_bytes, void* stream) {
  if (num_rows < 0 || row_bytes < 0) return fail(FCA_ERR_INVALID_ARG, "num_rows and row_bytes must be >= 0");
  if (num_rows == 0 || row_bytes == 0) return FCA_OK;
  if (num_rows > 0x7fffffffLL) return fail(FCA_ERR_UNSUPPORTED, "more than 2^31 - 1 rows");
  if (!src_dev || !index_dev || !dst_dev) return fail(FCA_ERR_INVALID_ARG, "src, index and dst must be non-NULL");
  if (row_bytes % 16 || src_stride_bytes % 16 || dst_stride_bytes % 16 || (reinterpret_cast<uintptr_t>(src_dev) & 15) ||
      (reinterpret_cast<uintptr_t>(dst_dev) & 15))
    return fail(FCA_ERR_INVALID_ARG, "rows must be 16-byte aligned: pointers, strides and row_bytes multiples of 16");
  if (src_stride_bytes < row_bytes || dst_stride_bytes < row_bytes)
    return fail(FCA_ERR_INVALID_ARG, "row strides must be at least row_bytes");
  hipError_t e = fca::launch_gather_rows(src_dev, src_stride_bytes, index_dev, num_rows, row_bytes, dst_dev, dst_stride_bytes,
                                         static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "row gather launch");
}

int fca_sum_rows(const void* src_dev, int64_t src_stride_bytes, const int32_t* offsets_dev, const int32_t* rows_dev,
                 int64_t num_dst_rows, int64_t channels, int32_t dtype, void* dst_dev, int64_t dst_stride_bytes, void* stream) {
  if (num_dst_rows < 0 || channels < 0) return fail(FCA_ERR_INVALID_ARG, "num_dst_rows and channels must be >= 0");
  if (dtype != FCA_BF16 && dtype != FCA_F32) return fail(FCA_ERR_UNSUPPORTED, "dtype %d is not supported (bf16 or f32)", dtype);
  if (num_dst_rows == 0 || channels == 0) return FCA_OK;
  if (num_dst_rows > 0x7fffffffLL) return fail(FCA_ERR_UNSUPPORTED, "more than 2^31 - 1 rows");
  if (!src_dev || !offsets_dev || !rows_dev || !dst_dev) return fail(FCA_ERR_INVALID_ARG, "src, offsets, rows and dst must be non-NULL");
  const int64_t row_bytes = channels * (dtype == FCA_F32 ? 4 : 2);
  if (channels % 8 || src_stride_bytes % 16 || dst_stride_bytes % 16 || (reinterpret_cast<uintptr_t>(src_dev) & 15) ||
      (reinterpret_cast<uintptr_t>(dst_dev) & 15))
    return fail(FCA_ERR_INVALID_ARG, "channels must be a multiple of 8 and rows 16-byte aligned");
  if (src_stride_bytes < row_bytes || dst_stride_bytes < row_bytes)
    return fail(FCA_ERR_INVALID_ARG, "row strides must be at least one row");
  hipError_t e = fca::launch_sum_rows(src_dev, src_stride_bytes, offsets_dev, rows_dev, num_dst_rows, channels, dtype == FCA_F32,
                                      dst_dev, dst_stride_bytes, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? FCA_OK : hip_fail(e, "row sum launch");
}

}  // extern "C"
