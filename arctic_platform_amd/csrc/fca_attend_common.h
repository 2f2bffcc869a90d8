// Pieces shared by the attention kernels: vector types, tile registers, fp8 conversion.
#pragma once

#include "fca_common.h"

namespace fca {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;
// Workgroups a CU holds at once: a wave's register budget is 512 / this.  Two where the
// kernel fits 256 registers without scratch and gains from the second wave per SIMD: head
// size 64 with 64-row tiles or fp8.  (The 32-row bf16 kernel at head size 64 would need two
// registers of scratch and gains under 2 %.)
constexpr int workgroups_per_cu(int head_dim, bool fp8, int rows_per_item) {
  return head_dim == 64 && (fp8 || rows_per_item == 64) ? 2 : 1;
}
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kRescaleSlack = 8.f;  // log2 units: rescale when a row maximum rises by more than 2^8

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ inline float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Raw operand registers of one 32-token tile.  bf16 V: one 16-byte load per 32-channel
// block and token block.  fp8 V: a lane fetches the whole 16-token row (16 bytes) of one
// channel, lane half h taking the channel blocks of parity h; the halves are exchanged
// with the lane 32 away just before use, so there is one load per pair of channel blocks.
template <int D, bool FP8>
struct KTile {
  static constexpr int NK = FP8 ? D / 32 : D / 16;  // 16-byte K loads per lane
  i32x4 k[NK];
};
template <int D, bool FP8>
struct VTile {
  static constexpr int NV = FP8 ? D / 64 : D / 32;  // 16-byte V loads per lane and token block
  i32x4 v[2][NV];
};

// 16-byte global accesses.  STREAM marks data that is touched once per launch (the KV
// tiles under prefix sharing, the partial rows): non-temporal, so it does not push the
// rest out of the caches and written rows leave for memory as whole bursts.  Measured on
// MI355X at the Qwen3-4B shape: 345 -> 323 us for the loads, -> 315 us with the stores.
template <bool STREAM>
__device__ inline i32x4 load16(const char* ptr) {
  const i32x4* q = reinterpret_cast<const i32x4*>(ptr);
  if constexpr (STREAM) return __builtin_nontemporal_load(q);
  return *q;
}
template <bool STREAM>
__device__ inline void store16(void* ptr, i32x4 v) {
  i32x4* q = reinterpret_cast<i32x4*>(ptr);
  if constexpr (STREAM) __builtin_nontemporal_store(v, q);
  else *q = v;
}

// ---- partial rows ------------------------------------------------------------------
// A partial output row is kept as D half-precision values times one power-of-two scale
// per row (the smallest power of two not below the row's largest magnitude), next to its
// fp32 log-sum-exp: {lse, scale} per row.  Every element keeps 11 significant bits
// whatever the magnitude of the row, eight times finer than the bf16 rounding of the
// probabilities inside the value product, at half the bytes of fp32 rows -- and writing
// the partials costs several times their share of a launch's bytes.
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));

// Bytes of one row in a wave's LDS strip: D halves + 16 bytes holding the row's index in
// the partial buffers.
template <int D>
constexpr int strip_row_bytes() { return D * 2 + 16; }

// Smallest power of two >= x for a positive, finite, normal x; 1 for anything else.
__device__ inline float pow2_ceil(float x) {
  const unsigned b = __float_as_uint(x);
  const unsigned e = (b + 0x007fffffu) & 0x7f800000u;
  return (x > 0.f && e != 0u && e != 0x7f800000u) ? __uint_as_float(e) : 1.f;
}

// Lane (m, h) holds, in acc[db][4 * q4 + e], channel 32 * db + 8 * q4 + 4 * h + e of query
// row `row` of the tile.  Normalises the row by `inv` (1 / softmax sum, times the V scale
// of an fp8 cache), stages it in the strip as scaled halves and, from the lanes with
// h == 0, writes {lse, scale} and leaves the destination row index in the strip.  `tag`
// (below 2^23) is stored in the mantissa bits of the scale, which is a power of two: the
// merge reads it as the place of a second partial of the same chunk (0 = none).
template <int D, bool THROUGH>
__device__ inline void stage_partial_row(char* strip, int row, int h, const f32x16 (&acc)[D / 32], float inv,
                                         int64_t prow, float lse, float* partial_lse, int tag = 0) {
  float amax = 0.f;
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) amax = fmaxf(amax, fabsf(acc[db][r]));
  amax = fmaxf(amax, __shfl_xor(amax, 32)) * fabsf(inv);
  const float scale = pow2_ceil(amax);
  const float k = inv / scale;  // exact: the scale is a power of two
  if (prow < 0) return;
  char* dst = strip + row * strip_row_bytes<D>();
  if (h == 0) {
    const f32x2 ls = {lse, __uint_as_float(__float_as_uint(scale) | (unsigned)tag)};
    if constexpr (THROUGH) store8_coherent(partial_lse + 2 * prow, __builtin_bit_cast(uint64_t, ls));
    else *reinterpret_cast<f32x2*>(partial_lse + 2 * prow) = ls;
    *reinterpret_cast<int64_t*>(dst + D * 2) = prow;
  }
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      f16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (_Float16)(acc[db][q4 * 4 + e] * k);
      *reinterpret_cast<f16x4*>(dst + (db * 32 + q4 * 8 + h * 4) * 2) = v;
    }
}

// The staged rows 0 .. rows-1 leave as whole rows, D / 8 lanes per row and 64 * 8 / D rows
// per pass, each lane with two 8-byte stores (one per half of the row, so that a store
// instruction covers a contiguous half row).  THROUGH (the kernels that stream their KV past
// the caches) makes them device-scope write-through stores: the rows are read once, by the
// merge, and written this way they do not linger in the L2 to be written back when the launch
// ends.  Measured at the Qwen3-4B shape against non-temporal 16-byte stores: 310.2 -> 304.2 us
// per step (the attention launch 3 us shorter, the merge behind it 3 us cheaper).  With
// sharing off the KV comes out of the memory-side cache, and ordinary stores are the faster
// ones there (921 against 943 us).
template <int D, bool THROUGH>
__device__ inline void store_partial_rows(const char* strip, int rows, int lane, void* partial_out) {
  constexpr int LPR = D / 8;     // lanes per row
  constexpr int RPS = 64 / LPR;  // rows per pass
  const int sub = lane / LPR, c = (lane % LPR) * 8;  // byte offset inside a half row
  for (int r0 = 0; r0 < rows; r0 += RPS) {
    const int r = r0 + sub;
    if (r < rows) {
      const char* src = strip + r * strip_row_bytes<D>();
      const int64_t pr = *reinterpret_cast<const int64_t*>(src + D * 2);
      char* dst = static_cast<char*>(partial_out) + pr * D * 2;
      const uint64_t lo = *reinterpret_cast<const uint64_t*>(src + c), hi = *reinterpret_cast<const uint64_t*>(src + D + c);
      if constexpr (THROUGH) {
        store8_coherent(dst + c, lo);
        store8_coherent(dst + D + c, hi);
      } else {
        *reinterpret_cast<uint64_t*>(dst + c) = lo;
        *reinterpret_cast<uint64_t*>(dst + D + c) = hi;
      }
    }
  }
}

// 8 fp8 e4m3 values (two dwords) -> 8 bf16 with the packed converter of gfx950 (scale 1:
// every e4m3 value is a bf16 value, so the conversion is exact).
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ inline bf16x8 fp8x8_to_bf16(int lo, int hi) {
  const bf16x2 a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
  const bf16x2 b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
  const bf16x2 c = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
  const bf16x2 d = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
  return bf16x8{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

}  // namespace fca
