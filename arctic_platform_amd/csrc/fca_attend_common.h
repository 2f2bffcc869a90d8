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
__device__ inline void store16(float* ptr, f32x4 v) {
  f32x4* q = reinterpret_cast<f32x4*>(ptr);
  if constexpr (STREAM) __builtin_nontemporal_store(v, q);
  else *q = v;
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
