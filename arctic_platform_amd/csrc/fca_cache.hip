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

// One thread per (token, kv head, group of XW channels), XW = channels per 16-byte K slice.
template <bool FP8>
__global__ __launch_bounds__(256) void fca_append_kernel(AppendParams p) {
  constexpr int XW = FP8 ? 16 : 8;
  const int groups = p.head_dim / XW;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)p.num_tokens * p.num_kv_heads * groups;
  if (idx >= total) return;
  const int c = (int)(idx % groups);
  const int h = (int)((idx / groups) % p.num_kv_heads);
  const int t = (int)(idx / ((int64_t)groups * p.num_kv_heads));
  const int64_t slot = p.slot_mapping[t];
  if (slot < 0) return;
  const int64_t blk = slot / kBlock;
  const int off = (int)(slot - blk * kBlock);

  const __hip_bfloat16* ksrc = reinterpret_cast<const __hip_bfloat16*>(p.key) + (int64_t)t * p.token_stride +
                               (int64_t)h * p.head_stride + c * XW;
  const __hip_bfloat16* vsrc = reinterpret_cast<const __hip_bfloat16*>(p.value) + (int64_t)t * p.token_stride +
                               (int64_t)h * p.head_stride + c * XW;
  const int64_t tile = blk * p.cache_block_stride + (int64_t)h * p.cache_head_stride;  // elements
  if constexpr (FP8) {
    const float ks = p.k_scale ? p.k_scale[h] : 1.f;
    const float vs = p.v_scale ? p.v_scale[h] : 1.f;
    unsigned char* kdst = reinterpret_cast<unsigned char*>(p.k_cache) + tile + ((int64_t)c * kBlock + off) * XW;
    unsigned char* vdst = reinterpret_cast<unsigned char*>(p.v_cache) + tile + (int64_t)c * XW * kBlock + off;
    unsigned char kq[XW];
#pragma unroll
    for (int e = 0; e < XW; ++e) kq[e] = to_fp8(__bfloat162float(ksrc[e]) / ks);
    *reinterpret_cast<int4*>(kdst) = *reinterpret_cast<const int4*>(kq);
#pragma unroll
    for (int e = 0; e < XW; ++e) vdst[e * kBlock] = to_fp8(__bfloat162float(vsrc[e]) / vs);
  } else {
    __hip_bfloat16* kdst = reinterpret_cast<__hip_bfloat16*>(p.k_cache) + tile + ((int64_t)c * kBlock + off) * XW;
    __hip_bfloat16* vdst = reinterpret_cast<__hip_bfloat16*>(p.v_cache) + tile + (int64_t)c * XW * kBlock + off;
    *reinterpret_cast<int4*>(kdst) = *reinterpret_cast<const int4*>(ksrc);
#pragma unroll
    for (int e = 0; e < XW; ++e) vdst[e * kBlock] = vsrc[e];
  }
}

// The way back: the tokens at the given slots leave the cache as bf16 rows [T, Hkv, D] (fp8
// tiles are multiplied by their per-head scales, i.e. the values decode attention sees).  A
// negative slot gives a row of zeros.  Same thread mapping as the append.
template <bool FP8>
__global__ __launch_bounds__(256) void fca_gather_kernel(AppendParams p) {
  constexpr int XW = FP8 ? 16 : 8;
  const int groups = p.head_dim / XW;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)p.num_tokens * p.num_kv_heads * groups;
  if (idx >= total) return;
  const int c = (int)(idx % groups);
  const int h = (int)((idx / groups) % p.num_kv_heads);
  const int t = (int)(idx / ((int64_t)groups * p.num_kv_heads));
  const int64_t slot = p.slot_mapping[t];
  __hip_bfloat16* kdst = reinterpret_cast<__hip_bfloat16*>(const_cast<void*>(p.key)) + (int64_t)t * p.token_stride +
                         (int64_t)h * p.head_stride + c * XW;
  __hip_bfloat16* vdst = reinterpret_cast<__hip_bfloat16*>(const_cast<void*>(p.value)) + (int64_t)t * p.token_stride +
                         (int64_t)h * p.head_stride + c * XW;
  __hip_bfloat16 kv[XW], vv[XW];
  if (slot < 0) {
#pragma unroll
    for (int e = 0; e < XW; ++e) kv[e] = vv[e] = __float2bfloat16(0.f);
  } else {
    const int64_t blk = slot / kBlock;
    const int off = (int)(slot - blk * kBlock);
    const int64_t tile = blk * p.cache_block_stride + (int64_t)h * p.cache_head_stride;  // elements
    if constexpr (FP8) {
      const float ks = p.k_scale ? p.k_scale[h] : 1.f;
      const float vs = p.v_scale ? p.v_scale[h] : 1.f;
      const unsigned char* ksrc = reinterpret_cast<const unsigned char*>(p.k_cache) + tile + ((int64_t)c * kBlock + off) * XW;
      const unsigned char* vsrc = reinterpret_cast<const unsigned char*>(p.v_cache) + tile + (int64_t)c * XW * kBlock + off;
      unsigned char kq[XW];
      *reinterpret_cast<int4*>(kq) = *reinterpret_cast<const int4*>(ksrc);
#pragma unroll
      for (int e = 0; e < XW; ++e) {
        kv[e] = __float2bfloat16(__builtin_amdgcn_cvt_f32_fp8((int)kq[e], 0) * ks);
        vv[e] = __float2bfloat16(__builtin_amdgcn_cvt_f32_fp8((int)vsrc[e * kBlock], 0) * vs);
      }
    } else {
      const __hip_bfloat16* ksrc = reinterpret_cast<const __hip_bfloat16*>(p.k_cache) + tile + ((int64_t)c * kBlock + off) * XW;
      const __hip_bfloat16* vsrc = reinterpret_cast<const __hip_bfloat16*>(p.v_cache) + tile + (int64_t)c * XW * kBlock + off;
      *reinterpret_cast<int4*>(kv) = *reinterpret_cast<const int4*>(ksrc);
#pragma unroll
      for (int e = 0; e < XW; ++e) vv[e] = vsrc[e * kBlock];
    }
  }
#pragma unroll
  for (int e = 0; e < XW; e += 8) {
    *reinterpret_cast<int4*>(kdst + e) = *reinterpret_cast<const int4*>(kv + e);
    *reinterpret_cast<int4*>(vdst + e) = *reinterpret_cast<const int4*>(vv + e);
  }
}

hipError_t launch_gather(const AppendParams& p, int kv_dtype, hipStream_t stream) {
  const bool fp8 = kv_dtype == FCA_FP8_E4M3;
  const int64_t total = (int64_t)p.num_tokens * p.num_kv_heads * (p.head_dim / (fp8 ? 16 : 8));
  if (total == 0) return hipSuccess;
  const int grid = (int)((total + 255) / 256);
  if (fp8)
    hipLaunchKernelGGL(fca_gather_kernel<true>, dim3(grid), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(fca_gather_kernel<false>, dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}

hipError_t launch_append(const AppendParams& p, int kv_dtype, hipStream_t stream) {
  const bool fp8 = kv_dtype == FCA_FP8_E4M3;
  const int64_t total = (int64_t)p.num_tokens * p.num_kv_heads * (p.head_dim / (fp8 ? 16 : 8));
  if (total == 0) return hipSuccess;
  const int grid = (int)((total + 255) / 256);
  if (fp8)
    hipLaunchKernelGGL(fca_append_kernel<true>, dim3(grid), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(fca_append_kernel<false>, dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError();
}

}  // namespace fca
