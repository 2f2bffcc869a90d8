// Rows of a deduplicated training tensor copied back into one sequence per sample, and the way
// back.  The trainer keeps a prompt group's prompt once and every sample's response behind it
// (arctic_platform/rl/zorro_train/zorro_train.py:311-356); where a layer wants whole samples
// again it rebuilds them with Python loops over slices and torch.cat
// (ZoRRoTrain._reconstruct_sequences_packed, zorro_train.py:1071-1159; the Triton kernel
// _triton_reconstruct_seq, :160-235, copies one row per program), and it picks the
// deduplicated rows out of whole samples the same way (_deduplicate_sequences_packed).  Both
// are the same kernel here: dst[i] = src[index[i]], whole rows in 16-byte pieces, with the
// index array made once per batch on the host.  The gradient of the first is a sum over the
// copies of a row (a prompt row collects every sample of its group): each destination row
// adds up the source rows listed for it, in fp32 and in a fixed order, so there are no atomics
// and the result does not depend on timing.
#include <hip/hip_bf16.h>

#include "fca_common.h"

namespace fca {

// One 16-byte piece per thread; a negative index gives a row of zeros.
__global__ __launch_bounds__(256) void fca_gather_rows_kernel(const char* __restrict__ src, int64_t src_stride,
                                                             const int32_t* __restrict__ index, int64_t num_rows, int pieces,
                                                             char* __restrict__ dst, int64_t dst_stride) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= num_rows * pieces) return;
  const int64_t row = idx / pieces;
  const int piece = (int)(idx - row * pieces);
  const int64_t from = index[row];
  int4 v = {0, 0, 0, 0};
  if (from >= 0) v = *reinterpret_cast<const int4*>(src + from * src_stride + 16 * (int64_t)piece);
  *reinterpret_cast<int4*>(dst + row * dst_stride + 16 * (int64_t)piece) = v;
}

// dst[j] = sum of src[rows[k]] for k in [offsets[j], offsets[j + 1]), eight channels per thread.
template <bool F32>
__global__ __launch_bounds__(256) void fca_sum_rows_kernel(const char* __restrict__ src, int64_t src_stride,
                                                          const int32_t* __restrict__ offsets, const int32_t* __restrict__ rows,
                                                          int64_t num_dst_rows, int groups, char* __restrict__ dst,
                                                          int64_t dst_stride) {
  constexpr int kBytes = F32 ? 32 : 16;  // eight channels
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= num_dst_rows * groups) return;
  const int64_t j = idx / groups;
  const int g = (int)(idx - j * groups);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // (unrolled: the rows of four copies are requested together; the sum keeps its order)
#pragma unroll 4
  for (int k = offsets[j]; k < offsets[j + 1]; ++k) {
    const char* p = src + (int64_t)rows[k] * src_stride + (int64_t)g * kBytes;
    if constexpr (F32) {
      const float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
      acc[0] += a.x, acc[1] += a.y, acc[2] += a.z, acc[3] += a.w, acc[4] += b.x, acc[5] += b.y, acc[6] += b.z, acc[7] += b.w;
    } else {
      union {
        int4 raw;
        __hip_bfloat16 h[8];
      } u;
      u.raw = *reinterpret_cast<const int4*>(p);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += __bfloat162float(u.h[e]);
    }
  }
  char* q = dst + j * dst_stride + (int64_t)g * kBytes;
  if constexpr (F32) {
    reinterpret_cast<float4*>(q)[0] = make_float4(acc[0], acc[1], acc[2], acc[3]);
    reinterpret_cast<float4*>(q)[1] = make_float4(acc[4], acc[5], acc[6], acc[7]);
  } else {
    union {
      int4 raw;
      __hip_bfloat16 h[8];
    } u;
#pragma unroll
    for (int e = 0; e < 8; ++e) u.h[e] = __float2bfloat16(acc[e]);
    *reinterpret_cast<int4*>(q) = u.raw;
  }
}

hipError_t launch_gather_rows(const void* src, int64_t src_stride, const int32_t* index, int64_t num_rows, int64_t row_bytes,
                              void* dst, int64_t dst_stride, hipStream_t stream) {
  if (num_rows == 0 || row_bytes == 0) return hipSuccess;
  const int pieces = (int)(row_bytes / 16);
  const unsigned grid = (unsigned)((num_rows * pieces + 255) / 256);
  hipLaunchKernelGGL(fca_gather_rows_kernel, dim3(grid), dim3(256), 0, stream, static_cast<const char*>(src), src_stride, index,
                     num_rows, pieces, static_cast<char*>(dst), dst_stride);
  return hipGetLastError();
}

hipError_t launch_sum_rows(const void* src, int64_t src_stride, const int32_t* offsets, const int32_t* rows, int64_t num_dst_rows,
                           int64_t channels, bool f32, void* dst, int64_t dst_stride, hipStream_t stream) {
  if (num_dst_rows == 0 || channels == 0) return hipSuccess;
  const int groups = (int)(channels / 8);
  const unsigned grid = (unsigned)((num_dst_rows * groups + 255) / 256);
  if (f32)
    hipLaunchKernelGGL(fca_sum_rows_kernel<true>, dim3(grid), dim3(256), 0, stream, static_cast<const char*>(src), src_stride,
                       offsets, rows, num_dst_rows, groups, static_cast<char*>(dst), dst_stride);
  else
    hipLaunchKernelGGL(fca_sum_rows_kernel<false>, dim3(grid), dim3(256), 0, stream, static_cast<const char*>(src), src_stride,
                       offsets, rows, num_dst_rows, groups, static_cast<char*>(dst), dst_stride);
  return hipGetLastError();
}

}  // namespace fca
