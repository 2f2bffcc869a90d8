// KV-cache append: writes the new tokens' K and V into the paged cache in the tile order
// the attention kernel reads (K tile [D/x][16 tokens][x], V tile [D][16 tokens]), with
// optional quantisation to fp8 e4m3 by per-KV-head scales.  This is the step that runs
// right before decode attention in every layer; slot_mapping follows the paged-cache
// convention slot = physical_block * 16 + offset, negative = padding token, skipped.
#include <hip/hip_bf16.h>

#include "fca_common.h"

namespace fca {

constexpr float kFp8Max = 448.f;

__device__ inline unsigned char to_fp8(float x) {
  // saturate (clamp, then round to nearest even); NaN is stored as the canonical 0x7f
  if (x != x) return 0x7f;
  x = fminf(fmaxf(x, -kFp8Max), kFp8Max);
  return (unsigned char)(__builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false) & 0xff);
}

// Both directions move 16 tokens of one KV head per workgroup through LDS, so that global
// memory sees whole pieces on either side: the token rows [T, Hkv, D] in 16-byte pieces of
// adjacent lanes, the K tile in 16-byte slices whose 16 tokens are adjacent lanes (256
// contiguous bytes per slice when the tokens fill a block in order, as a prefill's do), and
// the V tile, where a channel's 16 tokens are adjacent, in one packed store or load per
// channel and aligned run of eight tokens.  Tokens that do not form such a run (a decode
// step's single tokens, padding, a run that starts off an 8-token boundary) take element
// accesses for the V tile; the result is the same either way.
constexpr int kGroup = 16;      // tokens per workgroup
constexpr int kRowPieces = 33;  // 16-byte pieces per staged row: D / 8 <= 32, and one of padding

struct CacheStage {
  int4 k[kGroup][kRowPieces];
  int4 v[kGroup][kRowPieces];
  int64_t slot[kGroup];
  int run[2];  // tokens 8 * r .. 8 * r + 7 lie in consecutive slots from a multiple of eight on
};

__device__ inline void stage_slots(CacheStage& st, const AppendParams& p, int t0, int tid) {
  if (tid < kGroup) st.slot[tid] = t0 + tid < p.num_tokens ? p.slot_mapping[t0 + tid] : -1;
  __syncthreads();
  if (tid < 2) {
    const int64_t first = st.slot[8 * tid];
    bool ok = first >= 0 && first % 8 == 0;
    for (int k = 1; k < 8; ++k) ok = ok && st.slot[8 * tid + k] == first + k;
    st.run[tid] = ok ? 1 : 0;
  }
}

template <bool FP8>
__global__ __launch_bounds__(256) void fca_append_kernel(AppendParams p) {
  constexpr int XW = FP8 ? 16 : 8;  // channels per 16-byte slice of the K tile
  const int D = p.head_dim, pieces = D / 8, slices = D / XW;
  const int h = blockIdx.x % p.num_kv_heads, t0 = (blockIdx.x / p.num_kv_heads) * kGroup;
  const int tid = threadIdx.x;
  __shared__ CacheStage st;
  stage_slots(st, p, t0, tid);
  for (int j = tid; j < kGroup * pieces; j += 256) {
    const int i = j / pieces, c = j - i * pieces;
    if (t0 + i < p.num_tokens) {
      const int64_t at = (int64_t)(t0 + i) * p.token_stride + (int64_t)h * p.head_stride + c * 8;
      st.k[i][c] = *reinterpret_cast<const int4*>(reinterpret_cast<const __hip_bfloat16*>(p.key) + at);
      st.v[i][c] = *reinterpret_cast<const int4*>(reinterpret_cast<const __hip_bfloat16*>(p.value) + at);
    }
  }
  __syncthreads();
  const float ks = FP8 && p.k_scale ? p.k_scale[h] : 1.f;
  const float vs = FP8 && p.v_scale ? p.v_scale[h] : 1.f;
  const int64_t head_at = (int64_t)h * p.cache_head_stride;  // elements
  // K tile: slice c of token i
  for (int j = tid; j < kGroup * slices; j += 256) {
    const int c = j / kGroup, i = j - c * kGroup;
    const int64_t slot = st.slot[i];
    if (slot < 0) continue;
    const int64_t blk = slot / kBlock;
    const int off = (int)(slot - blk * kBlock);
    const int64_t at = blk * p.cache_block_stride + head_at + ((int64_t)c * kBlock + off) * XW;
    if constexpr (FP8) {
      const __hip_bfloat16* src = reinterpret_cast<const __hip_bfloat16*>(&st.k[i][2 * c]);
      unsigned char q[XW];
#pragma unroll
      for (int e = 0; e < XW; ++e) q[e] = to_fp8(__bfloat162float(src[e]) / ks);
      *reinterpret_cast<int4*>(reinterpret_cast<unsigned char*>(p.k_cache) + at) = *reinterpret_cast<const int4*>(q);
    } else {
      *reinterpret_cast<int4*>(reinterpret_cast<__hip_bfloat16*>(p.k_cache) + at) = st.k[i][c];
    }
  }
  // V tile: channel d, tokens 8 * half .. 8 * half + 7
  for (int j = tid; j < 2 * D; j += 256) {
    const int d = j >> 1, half = j & 1;
    __hip_bfloat16 x[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) x[k] = reinterpret_cast<const __hip_bfloat16*>(&st.v[8 * half + k][0])[d];
    if (st.run[half]) {
      const int64_t slot = st.slot[8 * half];
      const int64_t blk = slot / kBlock;
      const int off = (int)(slot - blk * kBlock);
      const int64_t at = blk * p.cache_block_stride + head_at + (int64_t)d * kBlock + off;
      if constexpr (FP8) {
        unsigned char q[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) q[k] = to_fp8(__bfloat162float(x[k]) / vs);
        *reinterpret_cast<uint2*>(reinterpret_cast<unsigned char*>(p.v_cache) + at) = *reinterpret_cast<const uint2*>(q);
      } else {
        *reinterpret_cast<int4*>(reinterpret_cast<__hip_bfloat16*>(p.v_cache) + at) = *reinterpret_cast<const int4*>(x);
      }
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int64_t slot = st.slot[8 * half + k];
        if (slot < 0) continue;
        const int64_t blk = slot / kBlock;
        const int off = (int)(slot - blk * kBlock);
        const int64_t at = blk * p.cache_block_stride + head_at + (int64_t)d * kBlock + off;
        if constexpr (FP8)
          reinterpret_cast<unsigned char*>(p.v_cache)[at] = to_fp8(__bfloat162float(x[k]) / vs);
        else
          reinterpret_cast<__hip_bfloat16*>(p.v_cache)[at] = x[k];
      }
    }
  }
}

// The way back: the tokens at the given slots leave the cache as bf16 rows [T, Hkv, D] (fp8
// tiles are multiplied by their per-head scales, i.e. the values decode attention sees).  A
// negative slot gives a row of zeros.
template <bool FP8>
__global__ __launch_bounds__(256) void fca_gather_kernel(AppendParams p) {
  constexpr int XW = FP8 ? 16 : 8;
  const int D = p.head_dim, pieces = D / 8, slices = D / XW;
  const int h = blockIdx.x % p.num_kv_heads, t0 = (blockIdx.x / p.num_kv_heads) * kGroup;
  const int tid = threadIdx.x;
  __shared__ CacheStage st;
  stage_slots(st, p, t0, tid);
  __syncthreads();
  const float ks = FP8 && p.k_scale ? p.k_scale[h] : 1.f;
  const float vs = FP8 && p.v_scale ? p.v_scale[h] : 1.f;
  const int64_t head_at = (int64_t)h * p.cache_head_stride;  // elements
  const __hip_bfloat16 zero = __float2bfloat16(0.f);
  for (int j = tid; j < kGroup * slices; j += 256) {
    const int c = j / kGroup, i = j - c * kGroup;
    const int64_t slot = st.slot[i];
    __hip_bfloat16 x[XW];
    if (slot < 0) {
#pragma unroll
      for (int e = 0; e < XW; ++e) x[e] = zero;
    } else {
      const int64_t blk = slot / kBlock;
      const int off = (int)(slot - blk * kBlock);
      const int64_t at = blk * p.cache_block_stride + head_at + ((int64_t)c * kBlock + off) * XW;
      if constexpr (FP8) {
        unsigned char q[XW];
        *reinterpret_cast<int4*>(q) = *reinterpret_cast<const int4*>(reinterpret_cast<const unsigned char*>(p.k_cache) + at);
#pragma unroll
        for (int e = 0; e < XW; ++e) x[e] = __float2bfloat16(__builtin_amdgcn_cvt_f32_fp8((int)q[e], 0) * ks);
      } else {
        *reinterpret_cast<int4*>(x) = *reinterpret_cast<const int4*>(reinterpret_cast<const __hip_bfloat16*>(p.k_cache) + at);
      }
    }
#pragma unroll
    for (int e = 0; e < XW; e += 8) st.k[i][(XW / 8) * c + e / 8] = *reinterpret_cast<const int4*>(x + e);
  }
  for (int j = tid; j < 2 * D; j += 256) {
    const int d = j >> 1, half = j & 1;
    __hip_bfloat16 x[8];
    if (st.run[half]) {
      const int64_t slot = st.slot[8 * half];
      const int64_t blk = slot / kBlock;
      const int off = (int)(slot - blk * kBlock);
      const int64_t at = blk * p.cache_block_stride + head_at + (int64_t)d * kBlock + off;
      if constexpr (FP8) {
        unsigned char q[8];
        *reinterpret_cast<uint2*>(q) = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned char*>(p.v_cache) + at);
#pragma unroll
        for (int k = 0; k < 8; ++k) x[k] = __float2bfloat16(__builtin_amdgcn_cvt_f32_fp8((int)q[k], 0) * vs);
      } else {
        *reinterpret_cast<int4*>(x) = *reinterpret_cast<const int4*>(reinterpret_cast<const __hip_bfloat16*>(p.v_cache) + at);
      }
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int64_t slot = st.slot[8 * half + k];
        x[k] = zero;
        if (slot < 0) continue;
        const int64_t blk = slot / kBlock;
        const int off = (int)(slot - blk * kBlock);
        const int64_t at = blk * p.cache_block_stride + head_at + (int64_t)d * kBlock + off;
        if constexpr (FP8)
          x[k] = __float2bfloat16(__builtin_amdgcn_cvt_f32_fp8((int)reinterpret_cast<const unsigned char*>(p.v_cache)[at], 0) * vs);
        else
          x[k] = reinterpret_cast<const __hip_bfloat16*>(p.v_cache)[at];
      }
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) reinterpret_cast<__hip_bfloat16*>(&st.v[8 * half + k][0])[d] = x[k];
  }
  __syncthreads();
  for (int j = tid; j < kGroup * pieces; j += 256) {
    const int i = j / pieces, c = j - i * pieces;
    if (t0 + i < p.num_tokens) {
      const int64_t at = (int64_t)(t0 + i) * p.token_stride + (int64_t)h * p.head_stride + c * 8;
      *reinterpret_cast<int4*>(reinterpret_cast<__hip_bfloat16*>(const_cast<void*>(p.key)) + at) = st.k[i][c];
      *reinterpret_cast<int4*>(reinterpret_cast<__hip_bfloat16*>(const_cast<void*>(p.value)) + at) = st.v[i][c];
    }
  }
}

// fp32 rows and an fp32 cache (the all-fp32 path): one thread per (token, KV head, four
// channels).  The K tile keeps four channels of a token together ([D / 4][16 tokens][4]), so
// that side is one 16-byte access; the V tile ([D][16 tokens]) takes one element per channel.
// A small-configuration path: no staging through LDS.
template <bool GATHER>
__global__ __launch_bounds__(256) void fca_cache_f32_kernel(AppendParams p) {
  const int groups = p.head_dim / 4;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)p.num_tokens * p.num_kv_heads * groups) return;
  const int g = (int)(idx % groups);
  const int h = (int)(idx / groups % p.num_kv_heads);
  const int64_t t = idx / groups / p.num_kv_heads;
  const int64_t slot = p.slot_mapping[t];
  const int64_t row = t * p.token_stride + (int64_t)h * p.head_stride + 4 * g;
  typedef float f4 __attribute__((ext_vector_type(4)));
  f4* krow = reinterpret_cast<f4*>(reinterpret_cast<float*>(const_cast<void*>(p.key)) + row);
  f4* vrow = reinterpret_cast<f4*>(reinterpret_cast<float*>(const_cast<void*>(p.value)) + row);
  if (slot < 0) {  // padding: nothing to write; the way back gives zeros
    if (GATHER) *krow = f4{0.f, 0.f, 0.f, 0.f}, *vrow = f4{0.f, 0.f, 0.f, 0.f};
    return;
  }
  const int64_t blk = slot / kBlock;
  const int off = (int)(slot - blk * kBlock);
  const int64_t tile = blk * p.cache_block_stride + (int64_t)h * p.cache_head_stride;  // elements
  f4* kc = reinterpret_cast<f4*>(reinterpret_cast<float*>(p.k_cache) + tile + ((int64_t)g * kBlock + off) * 4);
  float* vc = reinterpret_cast<float*>(p.v_cache) + tile + (int64_t)(4 * g) * kBlock + off;
  if (GATHER) {
    *krow = *kc;
    *vrow = f4{vc[0], vc[kBlock], vc[2 * kBlock], vc[3 * kBlock]};
  } else {
    *kc = *krow;
    const f4 v = *vrow;
    vc[0] = v[0], vc[kBlock] = v[1], vc[2 * kBlock] = v[2], vc[3 * kBlock] = v[3];
  }
}

static hipError_t launch_cache_f32(const AppendParams& p, bool gather, hipStream_t stream) {
  const int64_t threads = (int64_t)p.num_tokens * p.num_kv_heads * (p.head_dim / 4);
  const unsigned grid = (unsigned)((threads + 255) / 256);
  if (gather)
    hipLaunchKernelGGL(fca_cache_f32_kernel<true>, dim3(grid), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(fca_cache_f32_kernel<false>, dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}

hipError_t launch_gather(const AppendParams& p, int kv_dtype, hipStream_t stream) {
  const bool fp8 = kv_dtype == FCA_FP8_E4M3;
  if (p.num_tokens == 0) return hipSuccess;
  if (kv_dtype == FCA_F32) return launch_cache_f32(p, true, stream);
  const int grid = (p.num_tokens + kGroup - 1) / kGroup * p.num_kv_heads;
  if (fp8)
    hipLaunchKernelGGL(fca_gather_kernel<true>, dim3(grid), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(fca_gather_kernel<false>, dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}

hipError_t launch_append(const AppendParams& p, int kv_dtype, hipStream_t stream) {
  const bool fp8 = kv_dtype == FCA_FP8_E4M3;
  if (p.num_tokens == 0) return hipSuccess;
  if (kv_dtype == FCA_F32) return launch_cache_f32(p, false, stream);
  const int grid = (p.num_tokens + kGroup - 1) / kGroup * p.num_kv_heads;
  if (fp8)
    hipLaunchKernelGGL(fca_append_kernel<true>, dim3(grid), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(fca_append_kernel<false>, dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace fca
