// Forest cascade attention pass for gfx950: one persistent kernel serves both the
// shared-prefix pass (query rows of every member sequence x the GQA heads of one KV head
// stacked into a 32- or 64-row tile) and the per-sequence suffix pass (the same tile with
// only Hq/Hkv live rows).
//
// Work item = (node chunk, tile of members) x KV head.  Every wavefront is its own worker:
// it takes an item from a ticket queue, streams the chunk's 32-token tiles with private
// online-softmax state and writes one normalised partial.  There is no workgroup barrier
// anywhere.  The kernel runs one wave per SIMD with the whole 512-entry register file, so
// up to three tiles (48 KB per wave, 192 KB per CU) of K/V loads are in flight while a
// tile is consumed; registers, not LDS, are the staging buffer because the cache already
// stores tiles in MFMA operand order.  LDS only transposes the output tile so partial rows
// leave as whole 128-byte lines.
//
// Per tile and wave, with tokens on the MFMA M dimension (the transposed product):
//   St[32 tok x 32 rows] = K[32 x D] . Qt[D x 32]       D/16 x mfma_f32_32x32x16_bf16
//   online softmax over tokens = over the 16 accumulator registers of a lane plus one
//   exchange with the lane 32 away (both hold the same query row)
//   Ot[D x 32 rows]     += Vt[D x 32 tok] . Pt[32 x 32]  D/32 x 2 mfma
// The cache stores K as [D/x][16 tok][x] and V as [D][16 tok], which are the A-operand
// orders of these two products: every operand is one contiguous 16-byte (8-byte for fp8 V)
// global load per lane.  The K rows are fed in the token order that makes the softmax
// output registers line up with the B operand of the second product, so P never leaves
// registers.
//
// Semantics (softmax scale, GQA head mapping h -> h / (Hq/Hkv), no mask for the decode
// token) follow arctic_platform/model/implementations/qwen35/models/qwen3_5_moe/
// modeling_qwen3_5_moe.py:368-373, :385, :440-454.
#include <type_traits>

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
constexpr int kOutStride = 32 + 4;   // floats per row of the per-wave LDS transpose buffer (padded)

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ inline float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

template <bool FP8>
struct RawV {
  using type = i32x4;
};
template <>
struct RawV<true> {
  using type = i32x2;
};

// Raw operand registers of one 32-token tile.
template <int D, bool FP8>
struct KTile {
  static constexpr int NK = FP8 ? D / 32 : D / 16;  // 16-byte K loads per lane
  i32x4 k[NK];
};
template <int D, bool FP8>
struct VTile {
  static constexpr int NDB = D / 32;  // 32-channel blocks of V per token block
  typename RawV<FP8>::type v[2][NDB];
};

// 8 fp8 e4m3 values (two dwords) -> 8 bf16.  Exact: every e4m3 value is a bf16 value.
__device__ inline bf16x8 fp8x8_to_bf16(int lo, int hi) {
  f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(lo, false);
  f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(lo, true);
  f32x2 c = __builtin_amdgcn_cvt_pk_f32_fp8(hi, false);
  f32x2 d = __builtin_amdgcn_cvt_pk_f32_fp8(hi, true);
  bf16x8 r;
  r[0] = (__bf16)a[0];
  r[1] = (__bf16)a[1];
  r[2] = (__bf16)b[0];
  r[3] = (__bf16)b[1];
  r[4] = (__bf16)c[0];
  r[5] = (__bf16)c[1];
  r[6] = (__bf16)d[0];
  r[7] = (__bf16)d[1];
  return r;
}

template <int D, int NRT, bool FP8>
__device__ void process_item(const AttendParams& p, const int item, const int kvh, float* lds_out) {
  constexpr int KS = D / 16;   // MFMA steps of the score product
  constexpr int NDB = D / 32;  // 32-channel blocks of the output
  using KT = KTile<D, FP8>;
  using VT = VTile<D, FP8>;

  const int lane = threadIdx.x & 63;
  const int m = lane & 31, h = lane >> 5;

  const int32_t* meta = p.meta;
  const int4* rec = reinterpret_cast<const int4*>(meta + p.off_items + (int64_t)item * kItemInts);
  const int4 r0 = rec[0], r1 = rec[1];
  const int rep = __builtin_amdgcn_readfirstlane(r0.x);
  const int blk_start = __builtin_amdgcn_readfirstlane(r0.y);
  const int tok_len = __builtin_amdgcn_readfirstlane(r0.z);
  const int moff = __builtin_amdgcn_readfirstlane(r0.w);
  const int mcnt = __builtin_amdgcn_readfirstlane(r1.x);
  const int ord = __builtin_amdgcn_readfirstlane(r1.y);
  const int G = p.group;
  const int rows = mcnt * G;
  const int32_t* members = meta + p.off_members + moff;

  // Query rows as B operands.  Row n of the tile is (member n / G, head n % G of this KV head).
  bf16x8 qreg[NRT][KS];
  int64_t prow[NRT];  // partial row this lane's query row is written to
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    const int n = rt * 32 + m;
    const bool live = n < rows;
    const int mi = live ? n / G : 0;
    const int g = n - mi * G;
    const int seq = members[mi];
    prow[rt] = live ? ((int64_t)seq * p.max_partials + ord) * p.num_q_heads + kvh * G + g : -1;
    const __bf16* qp = reinterpret_cast<const __bf16*>(p.q) + (int64_t)seq * p.q_seq_stride +
                       (int64_t)(kvh * G + g) * p.q_head_stride;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      // channel offset of MFMA step i for this lane half: the K tile hands a lane
      // 16 bytes of one token, i.e. 8 channels (bf16) or 16 channels = two steps (fp8)
      const int dq = FP8 ? 32 * (i >> 1) + 16 * h + 8 * (i & 1) : 16 * i + 8 * h;
      bf16x8 v = *reinterpret_cast<const bf16x8*>(qp + dq);
      if (!live) v = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      qreg[rt][i] = v;
    }
  }
  const bool two_tiles = NRT > 1 && rows > 32;

  // Physical block ids of the chunk, one per lane (a chunk has at most 64 blocks).
  const int nblk = (tok_len + kBlock - 1) / kBlock;
  const int ntiles = (tok_len + kTile - 1) / kTile;
  const int my_blk = p.block_table[(int64_t)rep * p.bt_stride + blk_start + min(lane, nblk - 1)];

  const char* kbase = p.k_cache + (int64_t)kvh * p.kv_head_bytes;
  const char* vbase = p.v_cache + (int64_t)kvh * p.kv_head_bytes;
  // MFMA row m carries the token whose index has bits 2 and 3 of m swapped: the score
  // accumulator then holds, per lane half, tokens 8h..8h+7 of each block in register order.
  const int tok_of_m = (m & 3) | ((m & 4) << 1) | ((m & 8) >> 1);
  const int k_lane_off = h * 256 + tok_of_m * 16;
  const int v_lane_off = FP8 ? m * 16 + h * 8 : m * 32 + h * 16;
  constexpr int V_DB_STEP = FP8 ? 512 : 1024;

  auto load_tile = [&](KT& kt, VT& vt, int ti) {
    const int p0 = 2 * ti, p1 = min(2 * ti + 1, nblk - 1);
    const int b0 = __builtin_amdgcn_readlane(my_blk, p0);
    const int b1 = __builtin_amdgcn_readlane(my_blk, p1);
    const int kb = (m & 16) ? b1 : b0;
    const char* kp = kbase + (int64_t)kb * p.kv_block_bytes + k_lane_off;
#pragma unroll
    for (int i = 0; i < KT::NK; ++i) kt.k[i] = *reinterpret_cast<const i32x4*>(kp + i * 512);
    const char* vp0 = vbase + (int64_t)b0 * p.kv_block_bytes + v_lane_off;
    const char* vp1 = vbase + (int64_t)b1 * p.kv_block_bytes + v_lane_off;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      vt.v[0][db] = *reinterpret_cast<const typename RawV<FP8>::type*>(vp0 + db * V_DB_STEP);
      vt.v[1][db] = *reinterpret_cast<const typename RawV<FP8>::type*>(vp1 + db * V_DB_STEP);
    }
  };

  f32x16 acc[NRT][NDB];
  float mrow[NRT], lrow[NRT];
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    mrow[rt] = -INFINITY;
    lrow[rt] = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[rt][db][r] = 0.f;
  }

  float sc = p.scale * kLog2e;
  if (FP8 && p.k_scale) sc *= p.k_scale[kvh];

  auto compute_tile = [&](const KT& kt, const VT& vt, int ti) {
    const int tok0 = ti * kTile;
    const bool full = tok0 + kTile <= tok_len;
    f32x16 s[NRT];
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[rt][r] = 0.f;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      bf16x8 a;
      if constexpr (FP8) {
        const i32x4 w = kt.k[i >> 1];
        a = (i & 1) ? fp8x8_to_bf16(w[2], w[3]) : fp8x8_to_bf16(w[0], w[1]);
      } else {
        a = __builtin_bit_cast(bf16x8, kt.k[i]);
      }
      s[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[0][i], s[0], 0, 0, 0);
      if constexpr (NRT > 1) {
        if (two_tiles) s[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[1][i], s[1], 0, 0, 0);
      }
    }
    bf16x8 pb[NRT][2];
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      if (rt > 0 && !two_tiles) continue;
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float v = s[rt][r] * sc;
        // register r holds token 16 * (r / 8) + 8 * h + r % 8 of the tile
        if (!full && tok0 + 16 * (r >> 3) + 8 * h + (r & 7) >= tok_len) v = -INFINITY;
        s[rt][r] = v;
        mx = fmaxf(mx, v);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float mnew = fmaxf(mrow[rt], mx);
      const float alpha = fast_exp2(mrow[rt] - mnew);
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = fast_exp2(s[rt][r] - mnew);
        sum += e;
        pb[rt][r >> 3][r & 7] = (__bf16)e;
      }
      lrow[rt] = lrow[rt] * alpha + sum;
      mrow[rt] = mnew;
      // the running maximum settles after a few tiles; skip the rescale when no row moved
      if (__builtin_amdgcn_readfirstlane(__any(alpha != 1.f))) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[rt][db][r] *= alpha;
      }
    }
    auto pv = [&](auto ragged) {
#pragma unroll
      for (int blk = 0; blk < 2; ++blk) {
        // tokens this lane feeds for this block: 8h .. 8h+7; on a ragged tile zero the
        // ones past the end so stale cache contents (possibly NaN) cannot leak through 0 * x
        const int nv = tok_len - (tok0 + 16 * blk + 8 * h);
#pragma unroll
        for (int db = 0; db < NDB; ++db) {
          bf16x8 a;
          if constexpr (FP8) {
            i32x2 w = vt.v[blk][db];
            if constexpr (decltype(ragged)::value) {
#pragma unroll
              for (int j = 0; j < 2; ++j) {
                unsigned keep = 0;
#pragma unroll
                for (int b = 0; b < 4; ++b)
                  if (4 * j + b < nv) keep |= 0xffu << (8 * b);
                w[j] &= keep;
              }
            }
            a = fp8x8_to_bf16(w[0], w[1]);
          } else {
            i32x4 w = vt.v[blk][db];
            if constexpr (decltype(ragged)::value) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                unsigned keep = (2 * j < nv ? 0xffffu : 0u) | (2 * j + 1 < nv ? 0xffff0000u : 0u);
                w[j] &= keep;
              }
            }
            a = __builtin_bit_cast(bf16x8, w);
          }
          acc[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[0][blk], acc[0][db], 0, 0, 0);
          if constexpr (NRT > 1) {
            if (two_tiles)
              acc[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[1][blk], acc[1][db], 0, 0, 0);
          }
        }
      }
    };
    if (full)
      pv(std::false_type{});
    else
      pv(std::true_type{});
  };

  // Software pipeline over the chunk's tiles with rotating register buffers: two tiles of
  // loads (one when two row tiles need the registers) stay in flight while one is consumed.
  // Prefetches past the end are clamped to the last tile instead of being skipped, so the
  // outstanding-load count is the same on every path and each wait covers exactly the
  // tile about to be used; the repeated tile comes from L2.
  {
    const int last = ntiles - 1;
    if constexpr (NRT == 1) {
      KT k0, k1, k2;
      VT v0, v1, v2;
      load_tile(k0, v0, 0);
      load_tile(k1, v1, min(1, last));
      for (int ti = 0; ti < ntiles; ti += 3) {
        load_tile(k2, v2, min(ti + 2, last));
        compute_tile(k0, v0, ti);
        if (ti + 1 >= ntiles) break;
        load_tile(k0, v0, min(ti + 3, last));
        compute_tile(k1, v1, ti + 1);
        if (ti + 2 >= ntiles) break;
        load_tile(k1, v1, min(ti + 4, last));
        compute_tile(k2, v2, ti + 2);
      }
    } else {
      KT k0, k1;
      VT v0, v1;
      load_tile(k0, v0, 0);
      for (int ti = 0; ti < ntiles; ti += 2) {
        load_tile(k1, v1, min(ti + 1, last));
        compute_tile(k0, v0, ti);
        if (ti + 1 >= ntiles) break;
        load_tile(k0, v0, min(ti + 2, last));
        compute_tile(k1, v1, ti + 1);
      }
    }
  }

  // Normalise in registers (every accumulator register of a lane belongs to its own query
  // row), then transpose 32 channels at a time through this wave's LDS slab so each partial
  // row leaves as 128 contiguous bytes.  LDS operations of one wave execute in issue order;
  // the fences only keep the compiler from reordering them.
  float vs = 1.f;
  if (FP8 && p.v_scale) vs = p.v_scale[kvh];
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    if (rt > 0 && !two_tiles) continue;
    const float l = lrow[rt] + __shfl_xor(lrow[rt], 32);
    const float inv = vs / l;
    if (h == 0 && prow[rt] >= 0) p.partial_lse[prow[rt]] = (mrow[rt] + fast_log2(l)) * kLn2;
    const int orow = lane >> 3, opart = lane & 7;  // 8 rows per pass, 8 lanes x 16 bytes per row
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[rt][db][q4 * 4 + e] * inv;
        // accumulator register 4 * q4 + e holds channel 32 * db + 8 * q4 + 4 * h + e
        *reinterpret_cast<f32x4*>(&lds_out[m * kOutStride + q4 * 8 + h * 4]) = v;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int pass = 0; pass < 4; ++pass) {
        const int r = pass * 8 + orow;
        const f32x4 v = *reinterpret_cast<const f32x4*>(&lds_out[r * kOutStride + opart * 4]);
        const int64_t dst_row = __shfl(prow[rt], r);  // lanes 0..31 hold rows 0..31
        if (dst_row >= 0) *reinterpret_cast<f32x4*>(p.partial_out + dst_row * D + db * 32 + opart * 4) = v;
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }
}

template <int D, int NRT, bool FP8>
__global__ __launch_bounds__(kThreads, 1) void fca_attend_kernel(AttendParams p) {
  __shared__ __attribute__((aligned(16))) float lds_out[kWaves][32 * kOutStride];

  int32_t* hdr = p.meta + p.off_header;
  const int total = hdr[H_ITEMS], shared = hdr[H_SHARED_ITEMS];
  const int first = p.select == 2 ? shared : 0;
  const int last = p.select == 1 ? shared : total;
  const int ntickets = (last - first) * p.num_kv_heads;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;

  for (;;) {
    int t = 0;
    if (lane == 0) t = atomicAdd(&hdr[H_TICKET], 1);
    t = __builtin_amdgcn_readfirstlane(t);
    if (t >= ntickets) break;
    const int item = first + t / p.num_kv_heads;
    const int kvh = t - (t / p.num_kv_heads) * p.num_kv_heads;
    process_item<D, NRT, FP8>(p, item, kvh, lds_out[wave]);
  }
  // The last wave out re-arms the queue for the next launch on this metadata.
  if (lane == 0) {
    __threadfence();
    const int done = atomicAdd(&hdr[H_DONE], 1);
    if (done == (int)gridDim.x * kWaves - 1) {
      hdr[H_TICKET] = 0;
      hdr[H_DONE] = 0;
      __threadfence();
    }
  }
}

static int cached_cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

static int env_int(const char* name, int fallback) {
  const char* v = getenv(name);
  return v && *v ? atoi(v) : fallback;
}

hipError_t launch_attend(const AttendParams& p, const fca_plan& plan, int kv_dtype, hipStream_t stream) {
  static const int wgs_per_cu = env_int("FCA_WGS_PER_CU", 1);
  const int64_t max_tickets = (int64_t)plan.num_seqs *
                              ((int64_t)plan.max_blocks * kBlock / plan.chunk_tokens + plan.max_levels + 1) *
                              plan.num_kv_heads;
  int grid = cached_cu_count() * wgs_per_cu;
  if ((int64_t)grid * kWaves > max_tickets) grid = (int)((max_tickets + kWaves - 1) / kWaves);
  if (grid < 1) grid = 1;
  const bool fp8 = kv_dtype == FCA_FP8_E4M3;
  const int nrt = plan.rows_per_item / 32;
#define FCA_LAUNCH(D_, N_, F_) \
  hipLaunchKernelGGL((fca_attend_kernel<D_, N_, F_>), dim3(grid), dim3(kThreads), 0, stream, p)
  if (plan.head_dim == 128) {
    if (nrt == 1) {
      if (fp8) FCA_LAUNCH(128, 1, true); else FCA_LAUNCH(128, 1, false);
    } else {
      if (fp8) FCA_LAUNCH(128, 2, true); else FCA_LAUNCH(128, 2, false);
    }
  } else {
    if (nrt == 1) {
      if (fp8) FCA_LAUNCH(64, 1, true); else FCA_LAUNCH(64, 1, false);
    } else {
      if (fp8) FCA_LAUNCH(64, 2, true); else FCA_LAUNCH(64, 2, false);
    }
  }
#undef FCA_LAUNCH
  return hipGetLastError();
}

}  // namespace fca
