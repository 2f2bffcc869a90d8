// Log-sum-exp merge of the per-sequence partial results (tree levels x split-K chunks).
// Running-max formulation with guards for empty partials, as the online log-sum-exp of
// arctic_platform/model/implementations/qwen35/models/layers/lm_head.py:190-202.
#include <hip/hip_bf16.h>

#include <type_traits>

#include "fca_common.h"

namespace fca {

constexpr int kMergeThreads = 256;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x8 __attribute__((ext_vector_type(8)));

// D / 8 lanes per (sequence, query head) row and share; each lane owns 8 adjacent channels
// (16 bytes of a half-precision partial row).  A partial row is its stored halves times the
// row's scale; {lse, scale} sit side by side.  With SPLIT > 1 (plans with many partials per
// row: long contexts cut into many chunks) SPLIT such lane groups take every SPLIT-th
// partial of the row each and combine their running results at the end, which puts SPLIT
// times the loads in flight.  F32: the partial rows are fp32 (the fp32 attention pass), 32 bytes
// per lane, with scale 1.
template <int D, int SPLIT, bool F32 = false>
__global__ __launch_bounds__(kMergeThreads) void fca_merge_kernel(MergeParams p) {
  using RowElem = std::conditional_t<F32, float, _Float16>;
  using Row8 = std::conditional_t<F32, f32x8, f16x8>;
  constexpr int V = 8;
  constexpr int kLanesPerShare = D / V;
  constexpr int kLanesPerRow = kLanesPerShare * SPLIT;
  static_assert(kLanesPerRow <= 64, "the shares of a row combine inside one wave");
  const int row = blockIdx.x * (kMergeThreads / kLanesPerRow) + threadIdx.x / kLanesPerRow;
  const int sub = threadIdx.x % kLanesPerShare;
  const int share = (threadIdx.x / kLanesPerShare) % SPLIT;
  // (rows past the end keep running with no partials: the shares of a row exchange registers below)
  const bool live_row = row < p.num_seqs * p.num_q_heads;
  const int s = live_row ? row / p.num_q_heads : 0, hq = live_row ? row - s * p.num_q_heads : 0;
  const int np = live_row ? p.seq_npart[s] : 0;
  const int64_t base = (int64_t)s * p.max_partials;
  const RowElem* rows = static_cast<const RowElem*>(p.partial_out);
  const float2* lse_scale = reinterpret_cast<const float2*>(p.partial_lse);

  // One online pass (running maximum, rescaled sum).  The partials are taken in batches of B:
  // first every load of the batch is issued, none under a condition (the {lse, scale} pairs,
  // then the rows: none depends on another), then comes the arithmetic, which has no branch in
  // it, and only then the second partials that some row scales of the batch point at, again
  // all loads first.  Written as a loop of load-and-accumulate with the empty partials skipped,
  // the compiler puts every load behind the test of the value loaded before it, and a row pays
  // two memory round trips per partial, one after the other; this way it pays one per batch
  // and one more where the batch has a second partial.  A batch is six partials (a row of the
  // 512-sequence batch has two to six), four where SPLIT lane groups share a row.  One size only:
  // with a second, smaller one for the last partials of a row the compiler lifts what the two
  // have in common, the first load, above the choice between them and waits for it there.  The
  // kernel stays well below 128 registers, i.e. at least four waves per SIMD: the 4096 waves that
  // merge 512 sequences of 32 query heads are resident at once.
  constexpr int B = F32 || SPLIT > 1 ? 4 : 6;
  float m = -INFINITY, wsum = 0.f;
  int stray = 0;  // a row scale pointed outside the rows set aside for second partials
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = 0.f;
  // (an empty partial, lse = -inf, has weight 0 whatever its output holds, NaN included)
  auto take = [&](float l, float scale, const Row8& o) {
    const bool live = l > -INFINITY;
    const float m_new = fmaxf(m, l);
    const float keep = m > -INFINITY ? __expf(m - m_new) : 0.f;
    const float w = live ? __expf(l - m_new) : 0.f;
    wsum = wsum * keep + w;
    const float ws = w * scale;
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = acc[e] * keep + (live ? ws * (float)o[e] : 0.f);
    m = m_new;
  };
  typedef float f2v __attribute__((ext_vector_type(2)));
  for (int i0 = share; i0 < np; i0 += B * SPLIT) {
    f2v ls[B];
    Row8 o[B];
    // A partial past the row's last one reads the last one again (the same lines, requested a
    // moment earlier) and gets the weight of an empty partial below.
    // (read once: non-temporal, about 1 us per step at the Qwen3-4B shape)
#pragma unroll
    for (int j = 0; j < B; ++j) {
      const int64_t pr = (base + min(i0 + j * SPLIT, np - 1)) * p.num_q_heads + hq;
      ls[j] = __builtin_nontemporal_load(reinterpret_cast<const f2v*>(lse_scale + pr));
    }
#pragma unroll
    for (int j = 0; j < B; ++j) {
      const int64_t pr = (base + min(i0 + j * SPLIT, np - 1)) * p.num_q_heads + hq;
      o[j] = __builtin_nontemporal_load(reinterpret_cast<const Row8*>(rows + pr * D + sub * V));
    }
    // (nothing that looks at a loaded value moves up between the loads of the batch)
    __builtin_amdgcn_sched_barrier(0);
    // The scale is a power of two; its mantissa bits say where a second partial of the same
    // chunk is (an item attended by two waves of the attention kernel), 0 = nowhere:
    // tag = 32 * (pair + 1) + row of the tile.  Only a buffer no attention launch has written
    // (or one written for another plan) holds a tag that points anywhere else: it is not
    // followed, and the output row leaves as NaN.
    int rel[B];  // row among the second partials, -1 = none
    bool any = false;
#pragma unroll
    for (int j = 0; j < B; ++j) {
      if (i0 + j * SPLIT >= np) ls[j] = f2v{-INFINITY, 1.f};
      const unsigned tag = __float_as_uint(ls[j][1]) & 0x007fffffu;
      const bool follow = tag >= 32 && (int64_t)tag - 32 < p.coop_rows;
      if (tag != 0 && !follow) stray = 1;
      rel[j] = follow ? (int)tag - 32 : -1;
      any |= follow;
      take(ls[j][0], __uint_as_float(__float_as_uint(ls[j][1]) & 0xff800000u), o[j]);
    }
    // Second partials: about a quarter of the rows of a large batch have one.  Where a batch
    // has any, all B are loaded (a partial without one reads its own row again, at weight 0: a
    // row of its own, so that no single line is asked for by every wave) so that these loads too
    // stand in a row with nothing between them.
    if (any) {
      f2v bls[B];
      Row8 bo[B];
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const int64_t pr = (base + min(i0 + j * SPLIT, np - 1)) * p.num_q_heads + hq;
        const int64_t br = rel[j] >= 0 ? p.coop_row0 + rel[j] : pr;
        bls[j] = *reinterpret_cast<const f2v*>(lse_scale + br);
        bo[j] = *reinterpret_cast<const Row8*>(rows + br * D + sub * V);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < B; ++j)
        take(rel[j] >= 0 ? bls[j][0] : -INFINITY, __uint_as_float(__float_as_uint(bls[j][1]) & 0xff800000u), bo[j]);
    }
  }
  // combine the shares: the same update with a whole running result in place of one partial
#pragma unroll
  for (int off = kLanesPerShare; off < kLanesPerRow; off <<= 1) {
    const float m_o = __shfl_xor(m, off), wsum_o = __shfl_xor(wsum, off);
    const float m_new = fmaxf(m, m_o);
    const float keep = m > -INFINITY ? __expf(m - m_new) : 0.f;
    const float take = m_o > -INFINITY ? __expf(m_o - m_new) : 0.f;
    wsum = wsum * keep + wsum_o * take;
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = acc[e] * keep + __shfl_xor(acc[e], off) * take;
    m = m_new;
    stray |= __shfl_xor(stray, off);
  }
  if (!live_row || share != 0) return;
  // The builder records input it had to clamp (a length beyond the block table, a row-table
  // entry out of range, overflowing lists) in the header and carries on; results made from
  // such metadata leave as NaN so that they cannot pass for attention over a cut-off sequence.
  const bool flagged = p.header[H_ERROR] != 0 || stray != 0;
  const float inv = flagged ? __builtin_nanf("") : (wsum > 0.f ? 1.f / wsum : 0.f);
  const int64_t o = (int64_t)s * p.out_seq_stride + (int64_t)hq * p.out_head_stride + sub * V;
  if (p.out_dtype == FCA_F32) {
    float* dst = reinterpret_cast<float*>(p.out) + o;
    if (p.vector_out) {
      reinterpret_cast<float4*>(dst)[0] = make_float4(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv);
      reinterpret_cast<float4*>(dst)[1] = make_float4(acc[4] * inv, acc[5] * inv, acc[6] * inv, acc[7] * inv);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) dst[e] = acc[e] * inv;
    }
  } else {
    __hip_bfloat16* dst = reinterpret_cast<__hip_bfloat16*>(p.out) + o;
    if (p.vector_out) {
      union {
        __hip_bfloat16 h[V];
        uint4 u;
      } pack;
#pragma unroll
      for (int e = 0; e < V; ++e) pack.h[e] = __float2bfloat16(acc[e] * inv);
      *reinterpret_cast<uint4*>(dst) = pack.u;
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) dst[e] = __float2bfloat16(acc[e] * inv);
    }
  }
  if (p.lse && sub == 0) p.lse[row] = flagged ? __builtin_nanf("") : (wsum > 0.f ? m + __logf(wsum) : -INFINITY);
}

// Plain 16-bytes-per-lane copy, the yardstick the hardware traffic counters are scaled by.
__global__ __launch_bounds__(256) void fca_copy_kernel(const int4* __restrict__ src, int4* __restrict__ dst, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

hipError_t launch_copy(const void* src, void* dst, size_t bytes, hipStream_t stream) {
  hipLaunchKernelGGL(fca_copy_kernel, dim3(2048), dim3(256), 0, stream, static_cast<const int4*>(src),
                     static_cast<int4*>(dst), bytes / 16);
  return hipGetLastError();
}

hipError_t launch_merge(const MergeParams& p, hipStream_t stream) {
  const int rows = p.num_seqs * p.num_q_heads;
  if (rows == 0) return hipSuccess;
  // rows that can have many partials are merged by four lane groups each (two at head size
  // 256, where four would not fit a wave)
  const int split = p.max_partials >= 16 ? (p.head_dim == 256 ? 2 : 4) : 1;
  const int per_block = kMergeThreads / (p.head_dim / 8 * split);
  const int grid = (rows + per_block - 1) / per_block;
#define FCA_MERGE(D_, S_) hipLaunchKernelGGL((fca_merge_kernel<D_, S_>), dim3(grid), dim3(kMergeThreads), 0, stream, p)
  if (p.partial_f32) {  // head sizes 64 and 128 (checked with the tensors)
    if (p.head_dim == 128) {
      if (split == 4) hipLaunchKernelGGL((fca_merge_kernel<128, 4, true>), dim3(grid), dim3(kMergeThreads), 0, stream, p);
      else hipLaunchKernelGGL((fca_merge_kernel<128, 1, true>), dim3(grid), dim3(kMergeThreads), 0, stream, p);
    } else {
      if (split == 4) hipLaunchKernelGGL((fca_merge_kernel<64, 4, true>), dim3(grid), dim3(kMergeThreads), 0, stream, p);
      else hipLaunchKernelGGL((fca_merge_kernel<64, 1, true>), dim3(grid), dim3(kMergeThreads), 0, stream, p);
    }
  } else if (p.head_dim == 256) {
    if (split == 2) FCA_MERGE(256, 2); else FCA_MERGE(256, 1);
  } else if (p.head_dim == 128) {
    if (split == 4) FCA_MERGE(128, 4); else FCA_MERGE(128, 1);
  } else {
    if (split == 4) FCA_MERGE(64, 4); else FCA_MERGE(64, 1);
  }
#undef FCA_MERGE
  return hipGetLastError();
}

}  // namespace fca
