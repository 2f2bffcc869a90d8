// Forest cascade attention pass in fp32: fp32 queries, an fp32 paged cache, fp32 arithmetic
// throughout, fp32 partial rows.  It serves the small fp32 configuration (one prompt group,
// head size 64) at the precision of the reference's own CPU path (softmax in fp32:
// arctic_platform/rl/zorro_train/qwen_attention_patcher.py:55-61; scale and grouped heads:
// model/implementations/qwen35/models/qwen3_5_moe/modeling_qwen3_5_moe.py:368-373, :385).
//
// Same work items, metadata and partial slots as the bf16 kernels; what differs is how an
// item is attended.  gfx950 has no more fp32 rate in its matrix cores than in its vector
// units, so this kernel is plain vector code with wavefront reductions, one wave per item:
//   scores   lane = one of 64 tokens of a step; the lane holds its token's K row in
//            registers (16-byte loads: the K tile keeps 4 channels of a token together)
//            and reads the query rows from LDS, where every lane reads the same address;
//   softmax  per query row the maximum and the sum over the 64 tokens are wave reductions;
//            the probabilities go to LDS;
//   values   lane = channel; the lane holds the 64 tokens of its channel in registers
//            (the V tile keeps the 16 tokens of a channel together) and reads the
//            probabilities from LDS, again one address for all lanes.
// Items are dealt round-robin over the waves; nothing here draws from the work counter of
// the metadata header, which therefore stays zero.
#include <hip/hip_ext.h>

#include "fca_attend_common.h"

namespace fca {

namespace {

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

constexpr int kStepTokens = 64;  // tokens per step: one per lane
constexpr int kMaxRows = 32;     // query rows of an item (rows_per_item = 32)
// Two waves to a workgroup, two workgroups to a CU: every wave still has a SIMD and its whole
// register file to itself, and a workgroup's LDS (the query rows and the probabilities of its
// waves: 48 KB at head size 128) stays below 64 KB.
constexpr int kF32Waves = 2;
constexpr int kF32Threads = 64 * kF32Waves;

}  // namespace

template <int D>
__global__ __launch_bounds__(kF32Threads, 1) void fca_attend_f32_kernel(AttendParams p) {
  constexpr int CPL = D / 64;  // channels per lane in the value product
  __shared__ __attribute__((aligned(16))) float q_lds[kF32Waves][kMaxRows][D];
  __shared__ __attribute__((aligned(16))) float p_lds[kF32Waves][kMaxRows][kStepTokens];

  const int32_t* hdr = p.meta + p.off_header;
  const int total = hdr[H_ITEMS], shared = hdr[H_SHARED_ITEMS];
  const int first = p.select == 2 ? shared : 0;
  const int last_item = p.select == 1 ? shared : total;
  const int ntickets = (last_item - first) * p.num_kv_heads;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int G = p.group, Hkv = p.num_kv_heads;
  const int nwaves = (int)gridDim.x * kF32Waves;
  const float* qbase = static_cast<const float*>(p.q);
  float* pout = static_cast<float*>(p.partial_out);
  const float sc = p.scale * kLog2e;
  float(*qw)[D] = q_lds[wave];
  float(*pw)[kStepTokens] = p_lds[wave];

  for (int t = (int)blockIdx.x * kF32Waves + wave; t < ntickets; t += nwaves) {
    const int it = t / Hkv, kvh = t - it * Hkv;
    const int32_t* rec = p.meta + p.off_items + (int64_t)(first + it) * kItemInts;
    const int rep = __builtin_amdgcn_readfirstlane(rec[0]);
    const int blk_start = __builtin_amdgcn_readfirstlane(rec[1]);
    const int tok_len = __builtin_amdgcn_readfirstlane(rec[2]);
    const int member_off = __builtin_amdgcn_readfirstlane(rec[3]);
    const int mcnt = __builtin_amdgcn_readfirstlane(rec[4]);
    const int ord = __builtin_amdgcn_readfirstlane(rec[5]);
    const int sees = __builtin_amdgcn_readfirstlane(rec[7]);
    const int rows = mcnt * G;  // <= kMaxRows: checked with the plan
    const int nblk = (tok_len + kBlock - 1) / kBlock;
    const int32_t* members = p.meta + p.off_members + member_off;

    // query rows of the item into LDS: row = member * G + head of the KV head's group
    __builtin_amdgcn_wave_barrier();  // (the previous item's reads of these arrays are done)
    for (int idx = lane; idx < rows * (D / 4); idx += 64) {
      const int row = idx / (D / 4), c4 = idx - row * (D / 4);
      const int member = row / G, head = row - member * G;
      const float* src = qbase + (int64_t)members[member] * p.q_seq_stride + (int64_t)(kvh * G + head) * p.q_head_stride;
      *reinterpret_cast<f32x4*>(&qw[row][4 * c4]) = *reinterpret_cast<const f32x4*>(src + 4 * c4);
    }
    __builtin_amdgcn_wave_barrier();

    // running maximum (log2 domain) and sum of every row, the same in all lanes; output
    // accumulators: row r, channels lane + 64 * c
    float mrow[kMaxRows], lrow[kMaxRows], acc[kMaxRows][CPL];
#pragma unroll
    for (int r = 0; r < kMaxRows; ++r) {
      mrow[r] = -INFINITY, lrow[r] = 0.f;
#pragma unroll
      for (int c = 0; c < CPL; ++c) acc[r][c] = 0.f;
    }

    for (int tok0 = 0; tok0 < tok_len; tok0 += kStepTokens) {
      // ---- scores: this lane's token against every query row
      const int tok = tok0 + lane;
      const int my_blk = p.block_table[(int64_t)rep * p.bt_stride + blk_start + min(tok / kBlock, nblk - 1)];
      const char* kp = p.k_cache + (int64_t)kvh * p.kv_head_bytes + (int64_t)my_blk * p.kv_block_bytes + (tok % kBlock) * 16;
      f32x4 k[D / 4];
#pragma unroll
      for (int g = 0; g < D / 4; ++g) k[g] = *reinterpret_cast<const f32x4*>(kp + g * (kBlock * 16));
      float alpha[kMaxRows];
#pragma unroll
      for (int r = 0; r < kMaxRows; ++r) {
        alpha[r] = 1.f;
        if (r < rows) {
          float s = 0.f;
#pragma unroll
          for (int g = 0; g < D / 4; ++g) {
            const f32x4 qv = *reinterpret_cast<const f32x4*>(&qw[r][4 * g]);
            s = __builtin_fmaf(qv[0], k[g][0], s);
            s = __builtin_fmaf(qv[1], k[g][1], s);
            s = __builtin_fmaf(qv[2], k[g][2], s);
            s = __builtin_fmaf(qv[3], k[g][3], s);
          }
          // the tokens a row sees: the chunk, or, in the last chunk of a run of query tokens,
          // up to the row's own token (member i sees the first sees + i tokens)
          const int row_lim = sees > 0 ? min(tok_len, sees + r / G) : tok_len;
          const float s2 = tok < row_lim ? s * sc : -INFINITY;
          const float mnew = fmaxf(mrow[r], wave_max(s2));
          // (every row sees the chunk's first token, so mnew is finite from the first step on)
          const float e = fast_exp2(s2 - mnew);
          alpha[r] = fast_exp2(mrow[r] - mnew);
          lrow[r] = lrow[r] * alpha[r] + wave_sum(e);
          mrow[r] = mnew;
          pw[r][lane] = e;
        }
      }
      __builtin_amdgcn_wave_barrier();

      // ---- values: this lane's channels against the probabilities of every row
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        const int ch = lane + 64 * c;
        f32x4 v[kStepTokens / 4];
#pragma unroll
        for (int b = 0; b < kStepTokens / kBlock; ++b) {
          const int blk = __builtin_amdgcn_readlane(my_blk, b * kBlock);
          const char* vp = p.v_cache + (int64_t)kvh * p.kv_head_bytes + (int64_t)blk * p.kv_block_bytes + ch * (kBlock * 4);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            f32x4 w = *reinterpret_cast<const f32x4*>(vp + j * 16);
            // what lies behind the chunk's last token is not the chunk's (it may be anything,
            // NaN included): it must not meet even a zero probability
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (tok0 + b * kBlock + 4 * j + e >= tok_len) w[e] = 0.f;
            v[b * 4 + j] = w;
          }
        }
#pragma unroll
        for (int r = 0; r < kMaxRows; ++r) {
          if (r < rows) {
            float a = acc[r][c] * alpha[r];
#pragma unroll
            for (int j = 0; j < kStepTokens / 4; ++j) {
              const f32x4 pv = *reinterpret_cast<const f32x4*>(&pw[r][4 * j]);
              a = __builtin_fmaf(pv[0], v[j][0], a);
              a = __builtin_fmaf(pv[1], v[j][1], a);
              a = __builtin_fmaf(pv[2], v[j][2], a);
              a = __builtin_fmaf(pv[3], v[j][3], a);
            }
            acc[r][c] = a;
          }
        }
      }
      __builtin_amdgcn_wave_barrier();  // (the next step overwrites the probabilities)
    }

    // ---- the partial of the item: normalised rows and their log-sum-exp (natural log)
#pragma unroll
    for (int r = 0; r < kMaxRows; ++r) {
      if (r < rows) {
        const int member = r / G, head = r - member * G;
        const int64_t prow = ((int64_t)members[member] * p.max_partials + ord) * p.num_q_heads + kvh * G + head;
        const float inv = lrow[r] > 0.f ? 1.f / lrow[r] : 0.f;
#pragma unroll
        for (int c = 0; c < CPL; ++c) pout[prow * D + lane + 64 * c] = acc[r][c] * inv;
        if (lane == 0) {
          const f32x2 ls = {lrow[r] > 0.f ? (mrow[r] + fast_log2(lrow[r])) * kLn2 : -INFINITY, 1.f};
          *reinterpret_cast<f32x2*>(p.partial_lse + 2 * prow) = ls;
        }
      }
    }
  }
}

hipError_t launch_attend_f32(const AttendParams& p, const fca_plan& plan, int max_workgroups, hipStream_t stream) {
  const int64_t max_tickets = (int64_t)plan.num_seqs *
                              ((int64_t)plan.max_blocks * kBlock / plan.chunk_tokens + plan.max_levels + 2) * plan.num_kv_heads;
  int dev = 0, grid = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0) grid = cus;
  }
  grid *= 2;  // two workgroups of two waves per CU
  if (max_workgroups > 0 && max_workgroups < grid) grid = max_workgroups;
  if ((int64_t)grid * kF32Waves > max_tickets) grid = (int)((max_tickets + kF32Waves - 1) / kF32Waves);
  if (grid < 1) grid = 1;
  // (a pending pair of timing events is this launch's, as for the other attention kernels)
  hipEvent_t ev_start, ev_stop;
  take_attend_timing(&ev_start, &ev_stop);
#define FCA_LAUNCH_F32(D_) \
  if (ev_start) hipExtLaunchKernelGGL((fca_attend_f32_kernel<D_>), dim3(grid), dim3(kF32Threads), 0, stream, ev_start, ev_stop, 0, p); \
  else hipLaunchKernelGGL((fca_attend_f32_kernel<D_>), dim3(grid), dim3(kF32Threads), 0, stream, p)
  if (plan.head_dim == 128) {
    FCA_LAUNCH_F32(128);
  } else if (plan.head_dim == 64) {
    FCA_LAUNCH_F32(64);
  } else {
    return hipErrorInvalidValue;
  }
#undef FCA_LAUNCH_F32
  return hipGetLastError();
}

}  // namespace fca
