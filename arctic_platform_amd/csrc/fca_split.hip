// Split attention of the trainer over a deduplicated, unpadded batch, forward and backward,
// for gfx950.  Token order: for every prompt group the prompt once, then the response of
// every sample of the group (arctic_platform/rl/zorro_train/zorro_train.py:311-356).  A
// prompt row attends causally to its prompt; a response row attends to the whole prompt of
// its group and causally to its own response
// (arctic_platform/rl/zorro_train/qwen_attention_patcher.py:1198-1228, where the second
// call gets one copy of the prompt's K and V per sample).  Here nothing is copied per
// sample: since a group's responses follow its prompt, "row r attends to key t" is
//     t <= r < lim(t),   lim(t) = end of the group for a prompt token,
//                                 end of its own response for a response token,
// one int per key.  Work is cut into tiles of 32 consecutive tokens of the packed order; a
// tile may straddle segments, the per-element test above sorts that out.
//
// Kernels (mfma_f32_32x32x16_bf16, one wave per tile and head, four waves to a workgroup
// that share one stream of operands through LDS):
//   forward    per query tile, over the key tiles it can see (two ranges: the prompt's
//              tiles, then from the tile its own segment starts in up to its own):
//              St[tok x row] = K . Qt, online softmax per lane, Ot[d x row] += Vt . Pt
//   dq         per query tile, the same walk: Pt from the saved log-sum-exp,
//              dPt = V . dOt, dSt = Pt (dPt - delta), dQt[d x row] += Kt . dSt
//   dv, dk     per key tile, over the query tiles that can see it (one range) and the query
//              heads of its KV head: S[row x tok] = Q . Kt', P, dP = dO . Vt',
//              dVt[d x tok] += dOt . P, dKt[d x tok] += Qt . dS (two launches); a prompt's
//              dK and dV collect every sample of the group in registers and are written once
// A [T, H, D] tensor holds neither operand of these products contiguously for a 64-lane load:
// the first product of a chain wants 32 rows x 32 bytes per instruction, the second one
// contracts over tokens (or rows), which lie a row stride apart.  A first pass therefore
// writes every 32-token tile in operand order, 1 KB per operand slot ("images": rows as the
// first product takes them, and transposed as the second takes them; zero past the last
// token), and every operand load of the kernels is one contiguous kilobyte per wave.
// The first product feeds its rows in the order that makes its output registers the B
// operand of the second, so probabilities never leave registers.
#include <algorithm>
#include <cstdint>
#include <numeric>
#include <type_traits>
#include <vector>

#include "fca_attend_common.h"

namespace fca {

// ---- host: the layout array ------------------------------------------------------------
// With a window (> 0) row r sees key t only if pos(r) - pos(t) < window as well, pos = place of
// a token in its sample's own sequence (the prompt's tokens, then the response's): the walks
// of the query tiles start at the first tile any of their rows still sees, and a key tile's
// walk ends at the last query tile that still sees any of its keys.
void build_split_layout(int num_groups, const int32_t* prompt_tokens, const int32_t* group_sizes,
                        const int32_t* response_tokens, int64_t tiles, bool responses_only, int32_t window, int32_t* out) {
  const SplitLayout L = make_split_layout(tiles);
  const int64_t padded = 32 * tiles;
  std::vector<int32_t> own(padded, 0), pstart(padded, 0), pend(padded, 0), group_of(padded, 0);
  std::vector<int64_t> seen_end(padded, 0);  // one past the last row that sees key x
  int32_t* lim = out + L.kv_lim;
  int32_t* pos = out + L.pos;
  int64_t t = 0;
  int64_t ri = 0;
  int group = 0;
  int32_t* q_index = out + L.q_index;
  int32_t next_q = 0;
  bool in_prompt = false;
  auto fill = [&](int64_t from, int64_t to, int64_t limit, int64_t p0, int64_t p1) {
    for (int64_t x = from; x < to; ++x) {
      q_index[x] = responses_only && in_prompt ? -1 : next_q++;
      group_of[x] = group;
      lim[x] = (int32_t)limit;
      own[x] = (int32_t)from;
      pstart[x] = (int32_t)p0;
      pend[x] = (int32_t)p1;
      pos[x] = (int32_t)(in_prompt ? x - p0 : (p1 - p0) + (x - from));
      seen_end[x] = window > 0 ? std::min<int64_t>(to, x + window) : limit;
    }
  };
  for (int g = 0; g < num_groups; ++g) {
    group = g;
    const int64_t p0 = t, p1 = t + prompt_tokens[g];
    int64_t gend = p1;
    for (int s = 0; s < group_sizes[g]; ++s) gend += response_tokens[ri + s];
    in_prompt = true;
    fill(p0, p1, gend, p0, p1);
    in_prompt = false;
    t = p1;
    int64_t last_start = -1, last_len = 0;  // the group's last response that has tokens
    for (int s = 0; s < group_sizes[g]; ++s) {
      const int64_t s1 = t + response_tokens[ri + s];
      fill(t, s1, s1, p0, p1);
      if (s1 > t) last_start = t, last_len = s1 - t;
      t = s1;
    }
    if (window > 0 && last_start >= 0) {
      // a prompt key at position pt is seen by the first pt + window - (prompt length) rows of every response
      for (int64_t x = p0; x < p1; ++x) {
        const int64_t rows = (x - p0) + window - (p1 - p0);
        if (rows > 0) seen_end[x] = std::max(seen_end[x], last_start + std::min(last_len, rows));
      }
    }
    ri += group_sizes[g];
  }
  for (int64_t x = t; x < padded; ++x) lim[x] = 0, q_index[x] = -1, pos[x] = 0;
  const int64_t num_tokens = t;
  std::vector<int64_t> qcost(tiles);
  for (int64_t i = 0; i < tiles; ++i) {
    // The needs of a tile's first row cover those of the rows behind it: they belong to
    // later segments, whose own tokens and (if the group changes inside the tile) prompt
    // lie between the first row and themselves.
    const int64_t r0 = 32 * i;
    int32_t b0 = own[r0] / 32;
    int32_t a0 = pstart[r0] / 32;
    int32_t a1 = pend[r0] > pstart[r0] ? (pend[r0] + 31) / 32 : a0;
    a1 = std::max(a0, std::min(a1, b0));
    if (window > 0) {
      // the keys each row still sees, a range in its own segment and one in its prompt; the
      // part of a range inside the tiles [a0, a1) bounds that walk from the left, the rest
      // (a prompt's last tile may be the first of the other walk) the other one
      int64_t need_a = INT64_MAX, need_b = INT64_MAX;
      auto need = [&](int64_t lo, int64_t hi) {  // keys lo .. hi - 1
        if (lo / 32 >= a0 && lo / 32 < a1) need_a = std::min(need_a, lo);
        else need_b = std::min(need_b, lo);
        if (lo / 32 < a1 && (hi - 1) / 32 >= a1) need_b = std::min<int64_t>(need_b, 32 * (int64_t)a1);
      };
      for (int64_t r = r0; r < std::min<int64_t>(r0 + 32, num_tokens); ++r) {
        need(std::max<int64_t>(own[r], r - window + 1), r + 1);
        if (own[r] >= pend[r] && pend[r] > pstart[r]) {  // a response row behind a prompt
          const int64_t first = pstart[r] + std::max<int64_t>(0, (int64_t)pos[r] - window + 1);
          if (first < pend[r]) need(first, pend[r]);
        }
      }
      a0 = need_a == INT64_MAX ? a1 : std::max<int32_t>(a0, (int32_t)(need_a / 32));
      if (need_b != INT64_MAX) b0 = std::max<int32_t>(b0, (int32_t)(need_b / 32));
    }
    int32_t* rec = out + L.q_tiles + 4 * i;
    rec[0] = a0, rec[1] = a1, rec[2] = b0, rec[3] = 0;
    for (int x = 0; x < 32; ++x) rec[3] |= q_index[r0 + x] >= 0;  // any row of the tile that has a query
    qcost[i] = (a1 - a0) + (i - b0 + 1);
    int64_t mx = 0;
    for (int x = 0; x < 32; ++x) mx = std::max(mx, seen_end[r0 + x]);
    out[L.kv_qend + i] = (int32_t)((mx + 31) / 32);
    int32_t mn = lim[r0];
    for (int x = 1; x < 32; ++x) mn = std::min(mn, lim[r0 + x]);
    out[L.kv_limmin + i] = mn;
  }
  // Query tiles: group by group, so that the workgroups in flight read the same prompt, and
  // the longest walks of a group first.  Key tiles go four adjacent ones per workgroup; these
  // quads differ in length fifty-fold (a prompt's walk the whole group, a response's only
  // itself), so the longest go first.
  int32_t* qo = out + L.q_order;
  std::iota(qo, qo + tiles, 0);
  std::stable_sort(qo, qo + tiles, [&](int32_t a, int32_t b) {
    const int ga = group_of[32 * (int64_t)a], gb = group_of[32 * (int64_t)b];
    return ga != gb ? ga < gb : qcost[a] > qcost[b];
  });
  const int64_t quads = (tiles + 3) / 4;
  std::vector<int64_t> kcost(quads, 0);
  for (int64_t i = 0; i < tiles; ++i) kcost[i / 4] = std::max<int64_t>(kcost[i / 4], out[L.kv_qend + i] - 4 * (i / 4));
  int32_t* ko = out + L.kv_order;
  std::iota(ko, ko + tiles, 0);
  std::stable_sort(ko, ko + quads, [&](int32_t a, int32_t b) { return kcost[a] > kcost[b]; });
}

namespace {

// Row fed to lane m of the first product: bits 2 and 3 of m swapped.  Output register r of
// lane half h then belongs to row 16 * (r / 8) + 8 * h + r % 8, and registers 8 * blk ..
// 8 * blk + 7 are the B operand of the second product for the contiguous rows
// 16 * blk + 8 * h .. + 7.
__device__ inline int fed_row(int m) { return (m & ~12) | ((m & 4) << 1) | ((m & 8) >> 1); }

__device__ inline i32x4 ld16(const void* base, int64_t elem) {
  return *reinterpret_cast<const i32x4*>(static_cast<const __bf16*>(base) + elem);
}
__device__ inline bf16x8 as_bf16(i32x4 w) { return __builtin_bit_cast(bf16x8, w); }

typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

// acc[db][4 * q4 + e] of lane (n, h) is channel 32 * db + 8 * q4 + 4 * h + e of row/token n.
template <int D>
__device__ inline void store_rows(void* dst, int64_t row_elem, int h, const f32x16 (&acc)[D / 32], float mul) {
  __bf16* o = static_cast<__bf16*>(dst) + row_elem + 4 * h;
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      bf16x4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e) w[e] = (__bf16)(acc[db][4 * q4 + e] * mul);
      *reinterpret_cast<bf16x4*>(o + 32 * db + 8 * q4) = w;
    }
}

// ---- operand images --------------------------------------------------------------------------
// One workgroup per (tile, head): the tile's 32 rows go through LDS and leave in MFMA operand
// order, 16 bytes per lane and slot, so that every operand load of the attention kernels is
// one contiguous kilobyte per wave.
//   rows image        slot s, lane (m, h):        x[fed_row(m)][16 s + 8 h .. + 7]
//   transposed image  slot (blk, db), lane (m, h): x[16 blk + 8 h + i][32 db + m], i = 0 .. 7
// Rows past the last token are zero.
// With `other` (the images of dO are being made and `other` is O): also leaves, per row,
// delta = sum_d x * other and the log-sum-exp in log2 units, which the dk and dv kernels subtract.
template <int D>
__global__ __launch_bounds__(kThreads) void split_images_kernel(const __bf16* x, int64_t stride, int T, int nt,
                                                               __bf16* rows_image, __bf16* transposed_image,
                                                               const __bf16* other, int64_t other_stride, const float* lse,
                                                               float* delta, float* lse2) {
  __shared__ __attribute__((aligned(16))) __bf16 tile[32][D + 8];
  const int j = blockIdx.x, hh = blockIdx.y;
  for (int p = threadIdx.x; p < 32 * D / 8; p += kThreads) {
    const int tk = p / (D / 8), c = (p % (D / 8)) * 8;
    const int64_t t = 32 * (int64_t)j + tk;
    i32x4 w = {0, 0, 0, 0};
    if (t < T) w = ld16(x, t * stride + hh * D + c);
    *reinterpret_cast<i32x4*>(&tile[tk][c]) = w;
    if (other) {  // the D / 8 pieces of a row sit in adjacent lanes
      float sum = 0.f;
      if (t < T) {
        const bf16x8 a = as_bf16(w), b = as_bf16(ld16(other, t * other_stride + hh * D + c));
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += (float)a[i] * (float)b[i];
      }
#pragma unroll
      for (int m = 1; m < D / 8; m *= 2) sum += __shfl_xor(sum, m);
      if (c == 0) {
        const int64_t at = (int64_t)hh * 32 * nt + t;
        delta[at] = sum;
        lse2[at] = lse[at] * kLog2e;
      }
    }
  }
  __syncthreads();
  const int64_t base = ((int64_t)hh * nt + j) * (D / 16) * 512;
  for (int p = threadIdx.x; p < (D / 16) * 64; p += kThreads) {
    const int slot = p / 64, l = p % 64, m = l & 31, h = l >> 5;
    if (rows_image)
      *reinterpret_cast<i32x4*>(rows_image + base + p * 8) = *reinterpret_cast<const i32x4*>(&tile[fed_row(m)][16 * slot + 8 * h]);
    if (transposed_image) {
      const int blk = slot / (D / 32), db = slot % (D / 32);
      bf16x8 e;
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = tile[16 * blk + 8 * h + i][32 * db + m];
      *reinterpret_cast<bf16x8*>(transposed_image + base + p * 8) = e;
    }
  }
}

// ---- forward and dq: one wave per (query tile, query head) -----------------------------------
// Operand slots of one key tile, 1 KB each: K rows [0, KS), then (dq) V rows [KS, 2 KS), then
// the transposed image, V's (forward) or K's (dq).
// SHARED: the four waves of a workgroup are four query heads of one KV head on the same query
// tile, so they walk the same key tiles: each wave fetches a quarter of a tile's slots one
// tile ahead, the tile is passed around through LDS (two buffers, one barrier per tile) and
// the L1 sees a quarter of the operand traffic.  Without it (query heads per KV head not a
// multiple of four) every wave fetches its own tiles into two register buffers.  Head size
// 256 runs one workgroup per CU (its accumulators and query rows alone take 192 registers).
// WIN: the general instances, for a sliding window and for attention dropout.  Every pair of
// tiles is tested element by element there, with the positions of row and key in their own
// sequence beside the limits, and with dropout every probability draws its fate from a hash of
// (seed, query head, row, key), so that the four kernels agree on it without a stored mask.
template <int D, bool BWD, bool SHARED, bool WIN>
__global__ __launch_bounds__(kThreads, SHARED && D < 256 ? 2 : 1) void split_query_kernel(SplitParams p) {
  constexpr int KS = D / 16, NDB = D / 32, SLOTS = (BWD ? 3 : 2) * KS, PER = SLOTS / kWaves;
  __shared__ i32x4 lds[SHARED ? 2 : 1][SHARED ? SLOTS : 1][64];
  const SplitLayout L = make_split_layout(p.num_tiles);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
  // consecutive workgroups go to different XCDs: with the head quad running fastest an XCD
  // keeps to the same KV heads (when their number divides 8 or is a multiple of it) and its
  // L2 holds their K and V of the group in flight
  const int quads = (p.num_q_heads + kWaves - 1) / kWaves;
  const int hq = (blockIdx.x % quads) * kWaves + wave;
  if constexpr (!SHARED) {
    if (hq >= p.num_q_heads) return;
  }
  const int hkv = hq / (p.num_q_heads / p.num_kv_heads);
  const int nt = p.num_tiles;
  const int64_t padded = 32 * (int64_t)nt;
  const int i = __builtin_amdgcn_readfirstlane(p.layout[L.q_order + blockIdx.x / quads]);
  const int a0 = __builtin_amdgcn_readfirstlane(p.layout[L.q_tiles + 4 * i]);
  const int a1 = __builtin_amdgcn_readfirstlane(p.layout[L.q_tiles + 4 * i + 1]);
  const int b0 = __builtin_amdgcn_readfirstlane(p.layout[L.q_tiles + 4 * i + 2]);
  if (__builtin_amdgcn_readfirstlane(p.layout[L.q_tiles + 4 * i + 3]) == 0) return;  // a tile of rows without queries
  const int na = a1 - a0, ntile = na + i - b0 + 1;
  const int r = 32 * i + n;
  const int qi = p.layout[L.q_index + r];  // this lane's row of q and out, -1 = none
  const int64_t rc = max(qi, 0);
  // the first position this lane's row still sees: keys at positions pos_lo .. its own
  int pos_lo = 0;
  if constexpr (WIN) pos_lo = p.layout[L.pos + r] - p.window + 1;
  // dropout: the part of the hash argument that belongs to this lane's row and head
  const uint32_t drop_base = WIN ? p.drop_seed + (uint32_t)hq * 0xC2B2AE3Du + (uint32_t)r * 0x9E3779B1u : 0u;
  auto kept = [&](int j, int x) {  // register x of key tile j: key 32 j + 8 h + 16 (x / 8) + x % 8
    const uint32_t key = (uint32_t)(32 * j + 8 * h + 16 * (x >> 3) + (x & 7));
    uint32_t v = drop_base + key * 0x85EBCA77u;
    v ^= v >> 16, v *= 0x7FEB352Du, v ^= v >> 15, v *= 0x846CA68Bu, v ^= v >> 16;
    return v >= p.drop_thr;
  };

  bf16x8 qreg[KS], doreg[BWD ? KS : 1];
#pragma unroll
  for (int s = 0; s < KS; ++s) qreg[s] = as_bf16(ld16(p.q, rc * p.q_stride + hq * D + 16 * s + 8 * h));
  float lse2 = 0.f, delta = 0.f;
  if constexpr (BWD) {
#pragma unroll
    for (int s = 0; s < KS; ++s) doreg[s] = as_bf16(ld16(p.dout, rc * p.do_stride + hq * D + 16 * s + 8 * h));
    lse2 = p.lse[hq * padded + r] * kLog2e;
    delta = p.delta[hq * padded + r];
  }
  const float sc = p.scale * kLog2e;

  f32x16 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int x = 0; x < 16; ++x) acc[db][x] = 0.f;
  float mrow = -1e30f, lrow = 0.f;

  auto tile_of = [&](int idx) {
    idx = min(idx, ntile - 1);
    return idx < na ? a0 + idx : b0 + idx - na;
  };
  // slot of a tile -> its place in the images (every image holds KS slots per tile)
  auto slot_ptr = [&](int j, int slot) {
    const void* src = slot < KS ? p.kn : !BWD ? p.vr : slot < 2 * KS ? p.vn : p.kr;
    return static_cast<const __bf16*>(src) + (((int64_t)hkv * nt + j) * KS + slot % KS) * 512 + lane * 8;
  };

  // one key tile: `get(slot)` hands out operand registers; `limmin` = smallest lim of the tile
  auto compute = [&](int j, int limmin, auto&& get) {
    f32x16 sr;
#pragma unroll
    for (int x = 0; x < 16; ++x) sr[x] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) sr = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16(get(s)), qreg[s], sr, 0, 0, 0);
    // every row of this query tile sees every token of an earlier tile whose limits all lie
    // behind the query tile; anything else is tested element by element
    bool ok[16];
#pragma unroll
    for (int x = 0; x < 16; ++x) ok[x] = true;
    const bool masked = WIN || !(j < i && limmin >= 32 * i + 32);
    if constexpr (WIN) {
      // (four keys at a time, applied at once: sixteen tests kept side by side cost registers)
      const int tok0 = 32 * j + 8 * h;
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const i32x4 lim = *reinterpret_cast<const i32x4*>(p.layout + L.kv_lim + tok0 + 16 * blk + 4 * half);
          const i32x4 kpos = *reinterpret_cast<const i32x4*>(p.layout + L.pos + tok0 + 16 * blk + 4 * half);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int x = 8 * blk + 4 * half + e;
            const bool sees = tok0 + 16 * blk + 4 * half + e <= r && lim[e] > r && kpos[e] >= pos_lo;
            sr[x] = sees ? sr[x] : -INFINITY;
          }
          // (keeps the loads of the next four keys behind these tests: hoisted together, the
          // eight loads of a tile push the dq instance of head size 128 into scratch)
          __builtin_amdgcn_sched_barrier(0);
        }
    } else {
      if (masked) {
        const int tok0 = 32 * j + 8 * h;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const i32x4 lim = *reinterpret_cast<const i32x4*>(p.layout + L.kv_lim + tok0 + 16 * blk + 4 * half);
#pragma unroll
            for (int e = 0; e < 4; ++e) ok[8 * blk + 4 * half + e] = tok0 + 16 * blk + 4 * half + e <= r && lim[e] > r;
          }
      }
      // a hidden score becomes -inf, whose exponential is 0 (no branch around the exponentials)
      if (masked) {
#pragma unroll
        for (int x = 0; x < 16; ++x) sr[x] = ok[x] ? sr[x] : -INFINITY;
      }
    }
    bf16x8 pb[2];
    if constexpr (!BWD) {
      float mx = sr[0];
#pragma unroll
      for (int x = 1; x < 16; ++x) mx = fmaxf(mx, sr[x]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      // the reference point of the exponentials moves only when a row's maximum rises by
      // more than kRescaleSlack above it; the log-sum-exp does not depend on it
      const float mtile = mx * sc;
      if (__builtin_amdgcn_readfirstlane(__any(mtile > mrow + kRescaleSlack))) {
        const float mnew = fmaxf(mrow, mtile);
        const float alpha = fast_exp2(mrow - mnew);
        lrow *= alpha;
        mrow = mnew;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int x = 0; x < 16; ++x) acc[db][x] *= alpha;
      }
      float sum = 0.f;
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        float e = fast_exp2(__builtin_fmaf(sr[x], sc, -mrow));
        sum += e;  // (the row sum, and with it the log-sum-exp, is that of the probabilities before dropout)
        if constexpr (WIN) {
          if (p.drop_thr) e = kept(j, x) ? e * p.drop_scale : 0.f;
        }
        pb[x >> 3][x & 7] = (__bf16)e;
      }
      lrow += sum;
    } else {
      f32x16 dp;
#pragma unroll
      for (int x = 0; x < 16; ++x) dp[x] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16(get(KS + s)), doreg[s], dp, 0, 0, 0);
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const float e = fast_exp2(__builtin_fmaf(sr[x], sc, -lse2));
        float d = dp[x];
        if constexpr (WIN) {
          if (p.drop_thr) d = kept(j, x) ? d * p.drop_scale : 0.f;  // dP through the dropout of the forward
        }
        pb[x >> 3][x & 7] = (__bf16)(e * (d - delta));
      }
    }
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
      for (int db = 0; db < NDB; ++db)
        acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16(get(SLOTS - KS + blk * NDB + db)), pb[blk], acc[db], 0, 0, 0);
  };

  if constexpr (SHARED) {
    // requests past the end repeat the last tile, so every path issues the same loads
    i32x4 pf[PER];
    int pf_limmin;
    auto fetch = [&](int idx) {
      const int j = tile_of(idx);
#pragma unroll
      for (int x = 0; x < PER; ++x) pf[x] = ld16(slot_ptr(j, wave * PER + x), 0);
      pf_limmin = p.layout[L.kv_limmin + j];
    };
    auto publish = [&](int buf) {
#pragma unroll
      for (int x = 0; x < PER; ++x) lds[buf][wave * PER + x][lane] = pf[x];
    };
    fetch(0);
    publish(0);
    int limmin = __builtin_amdgcn_readfirstlane(pf_limmin);
    __syncthreads();
    for (int idx = 0; idx < ntile; ++idx) {
      const int buf = idx & 1;
      fetch(idx + 1);
      compute(tile_of(idx), limmin, [&](int slot) { return lds[buf][slot][lane]; });
      publish(buf ^ 1);
      limmin = __builtin_amdgcn_readfirstlane(pf_limmin);
      __syncthreads();
    }
  } else {
    struct Tile {
      i32x4 s[SLOTS];
      int j, limmin;
    };
    auto load = [&](Tile& t, int idx) {
      t.j = tile_of(idx);
#pragma unroll
      for (int x = 0; x < SLOTS; ++x) t.s[x] = ld16(slot_ptr(t.j, x), 0);
      t.limmin = p.layout[L.kv_limmin + t.j];
    };
    Tile ta, tb;
    load(ta, 0);
    for (int idx = 0; idx < ntile; idx += 2) {
      load(tb, idx + 1);
      compute(ta.j, __builtin_amdgcn_readfirstlane(ta.limmin), [&](int slot) { return ta.s[slot]; });
      load(ta, idx + 2);
      if (idx + 1 < ntile) compute(tb.j, __builtin_amdgcn_readfirstlane(tb.limmin), [&](int slot) { return tb.s[slot]; });
    }
  }

  if constexpr (!BWD) {
    const float l = lrow + __shfl_xor(lrow, 32);
    const float inv = l > 0.f ? 1.f / l : 0.f;
    if (qi >= 0) store_rows<D>(p.out, (int64_t)qi * p.o_stride + hq * D, h, acc, inv);
    if (h == 0) p.lse[hq * padded + r] = l > 0.f ? (mrow + fast_log2(l)) * kLn2 : 0.f;
  } else {
    if (qi >= 0) store_rows<D>(p.dq, (int64_t)qi * p.dq_stride + hq * D, h, acc, p.scale);
  }
}

// ---- dk, dv: one wave per (key tile, KV head) --------------------------------------------------
// A workgroup = four adjacent key tiles of one KV head.  Its waves need the same stream of
// query-side operands, one step per (query tile, query head of the KV head), and the stream
// is far larger than the L2, so a step's loads often take a trip to memory, several times
// the step's arithmetic.  The stream therefore goes through a ring of kRing LDS stages filled
// by direct-to-LDS loads (no landing registers): every wave requests a quarter of the slots
// of the step kRing - 1 ahead, waits only for its own requests of the step about to be used
// (loads complete in order, so "all but the newest kRing - 2 stages"), and one barrier per
// step both publishes that stage and frees the one just used.  A wave computes only the
// steps inside its own tile's range of query tiles.  dV and dK are two launches
// (DK = false / true): each keeps one set of accumulators, which leaves room for two
// workgroups per CU, at the price of forming the probabilities twice.
//   dV: slots Q rows [0, KS), dO transposed [KS, 2 KS):   P = exp(S - lse),  dVt += dOt . P
//   dK: slots Q rows, dO rows, Q transposed:   dS = P (dO . V - delta),      dKt += Qt . dS
constexpr int kRing = 3;

// Direct-to-LDS loads: every lane's 16 (4) bytes land at lds_slot + lane * 16 (4).  Written as
// assembly so that the compiler's wait insertion does not know of them: it would otherwise
// drain every outstanding request before each LDS read, and the ring below lives on requests
// that stay in flight across steps.  Loads the compiler does not know of can only make its
// own waits more conservative.  M0 (the LDS base of such a load) is restored.
__device__ inline unsigned lds_address(const void* p) {
  return __builtin_amdgcn_readfirstlane((unsigned)(size_t)((__attribute__((address_space(3))) void*)(p)));
}
__device__ inline void load_to_lds16(const void* src, unsigned lds_slot) {
  unsigned saved;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
               : "=&s"(saved)
               : "v"(src), "s"(lds_slot)
               : "memory");
}
__device__ inline void load_to_lds4(const void* src, unsigned lds_slot) {
  unsigned saved;
  asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\tglobal_load_lds_dword %1, off\n\ts_mov_b32 m0, %0"
               : "=&s"(saved)
               : "v"(src), "s"(lds_slot)
               : "memory");
}
// s_waitcnt that constrains only the vector-memory counter (gfx9 encoding)
#define FCA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0f70 | ((n) & 15) | (((n) >> 4) << 14))

// WIN: the instances for a sliding window; the positions of a step's 32 rows ride through the
// ring beside their log-sum-exp (requested by wave 1), and every step is tested element by element.
template <int D, bool DK, bool WIN>
__global__ __launch_bounds__(kThreads, D < 256 ? 2 : 1) void split_key_kernel(SplitParams p) {
  constexpr int KS = D / 16, NDB = D / 32, SLOTS = (DK ? 3 : 2) * KS, PER = SLOTS / kWaves;
  __shared__ i32x4 lds[kRing][SLOTS][64];
  __shared__ __attribute__((aligned(16))) float lds_stat[kRing][64];  // lse (in log2 units) of the step's 32 rows, then their delta
  __shared__ __attribute__((aligned(16))) int lds_pos[WIN ? kRing : 1][64];  // positions of the step's 32 rows (twice)
  const SplitLayout L = make_split_layout(p.num_tiles);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;
  const int hkv = blockIdx.x % p.num_kv_heads;
  const int ratio = p.num_q_heads / p.num_kv_heads;
  int rest = blockIdx.x / p.num_kv_heads;
  // the query heads this workgroup walks: all of the KV head, or (head_split) one of them
  int hq0 = hkv * ratio, group = ratio;
  if (p.head_split) hq0 += rest % ratio, rest /= ratio, group = 1;
  const int T = p.num_tokens, nt = p.num_tiles;
  const int64_t padded = 32 * (int64_t)nt;
  const int j0 = __builtin_amdgcn_readfirstlane(p.layout[L.kv_order + rest]) * kWaves;
  const int j = min(j0 + wave, nt - 1);  // a wave past the last tile repeats it and stores nothing
  const bool live = j0 + wave < nt;
  const int qend = live ? __builtin_amdgcn_readfirstlane(p.layout[L.kv_qend + j]) : 0;
  const int limmin = __builtin_amdgcn_readfirstlane(p.layout[L.kv_limmin + j]);
  int qend_all = 0;
  for (int w = 0; w < kWaves; ++w)
    if (j0 + w < nt) qend_all = max(qend_all, __builtin_amdgcn_readfirstlane(p.layout[L.kv_qend + j0 + w]));
  const int t = 32 * j + n;
  const int64_t tc = min(t, T - 1);
  const int lim_t = p.layout[L.kv_lim + t];
  // the last position that still sees this lane's key
  int pos_hi = 0;
  if constexpr (WIN) pos_hi = p.layout[L.pos + t] + p.window - 1;
  const uint32_t drop_base = WIN ? p.drop_seed + (uint32_t)t * 0x85EBCA77u : 0u;  // this lane's key in the dropout hash
  const float sc = p.scale * kLog2e;

  bf16x8 kreg[KS], vreg[DK ? KS : 1];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    kreg[s] = as_bf16(ld16(p.k, tc * p.k_stride + hkv * D + 16 * s + 8 * h));
    if constexpr (DK) vreg[s] = as_bf16(ld16(p.v, tc * p.v_stride + hkv * D + 16 * s + 8 * h));
  }
  f32x16 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int x = 0; x < 16; ++x) acc[db][x] = 0.f;

  // step = (query tile, query head of this KV head), head fastest, query tiles from the last
  // one down (the workgroups of a prompt's key tiles all end at the group's last query tile)
  const int steps = (qend_all - j0) * group;
  // Requests of one step: PER slots per wave, and from wave 0 the rows' lse (lanes 0-31) and
  // delta (lanes 32-63).  Steps past the end repeat the last one, so the count never changes.
  // (No division by the group size inside the loop: both walks are kept as counters.)
  int req_i = qend_all - 1, req_g = 0, req_buf = 0;  // the next request: query tile, head of the group, ring stage
  // what does not change from step to step: where this wave's slots start in their images
  // (per lane) and in a ring stage (LDS byte addresses)
  const __bf16* slot_src[PER];
#pragma unroll
  for (int x = 0; x < PER; ++x) {
    const int slot = wave * PER + x;
    const void* image = slot < KS ? p.qn : !DK ? p.dor : slot < 2 * KS ? p.don : p.qr;
    slot_src[x] = static_cast<const __bf16*>(image) + (slot % KS) * 512 + lane * 8;
  }
  const float* stat_src = (DK && h == 1 ? p.delta : p.lse2) + n;
  const unsigned slot_lds = lds_address(&lds[0][0][0]) + wave * PER * 1024;
  const unsigned stat_lds = lds_address(&lds_stat[0][0]);
  const int32_t* pos_src = p.layout + L.pos + n;
  const unsigned pos_lds = lds_address(&lds_pos[0][0]);
  auto request = [&]() {
    const int hq = hq0 + req_g;
    const int64_t at = ((int64_t)hq * nt + req_i) * KS * 512;
#pragma unroll
    for (int x = 0; x < PER; ++x) load_to_lds16(slot_src[x] + at, slot_lds + (req_buf * SLOTS + x) * 1024);
    if (wave == 0) load_to_lds4(stat_src + hq * padded + 32 * req_i, stat_lds + req_buf * 256);
    if constexpr (WIN) {
      if (wave == 1) load_to_lds4(pos_src + 32 * req_i, pos_lds + req_buf * 256);
    }
    req_buf = req_buf + 1 == kRing ? 0 : req_buf + 1;
    // past the last step the last one is requested again
    if (req_g + 1 < group)
      ++req_g;
    else if (req_i > j0)
      req_g = 0, --req_i;
  };

  // The loads above must have landed before the first request: a wait for them placed inside
  // the loop would also wait, every step, for the requests the compiler does not know of.
  FCA_WAIT_VMCNT(0);
  if (steps > 0) {
    for (int s = 0; s < kRing - 1; ++s) request();
    int i = qend_all - 1, g = 0, buf = 0;
    for (int step = 0; step < steps; ++step) {
      // this wave's requests of `step` have landed; after the barrier so have everyone's, and
      // everyone has finished with the stage of the step before, which the next request refills
      if (wave == 0 || (WIN && wave == 1))
        FCA_WAIT_VMCNT((kRing - 2) * (PER + 1));
      else
        FCA_WAIT_VMCNT((kRing - 2) * PER);
      __builtin_amdgcn_s_barrier();
      request();
      if (live && i >= j && i < qend) {
        f32x16 sr, dp;
#pragma unroll
        for (int x = 0; x < 16; ++x) sr[x] = 0.f, dp[x] = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          sr = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16(lds[buf][s][lane]), kreg[s], sr, 0, 0, 0);
          if constexpr (DK) dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16(lds[buf][KS + s][lane]), vreg[s], dp, 0, 0, 0);
        }
        bf16x8 pb[2];
        const int row0 = 32 * i + 8 * h;
        // a hidden score becomes -inf, whose exponential is 0 (no branch around the exponentials)
        if (WIN || !(i > j && limmin >= 32 * i + 32)) {
#pragma unroll
          for (int x = 0; x < 16; ++x) {
            const int qrow = row0 + 16 * (x >> 3) + (x & 7);
            bool sees = t <= qrow && qrow < lim_t;
            if constexpr (WIN) sees = sees && lds_pos[buf][8 * h + 16 * (x >> 3) + (x & 7)] <= pos_hi;
            sr[x] = sees ? sr[x] : -INFINITY;
          }
        }
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          // registers 4 q4 .. 4 q4 + 3 belong to rows 16 (q4 / 2) + 8 h + 4 (q4 % 2) + 0 .. 3 of the tile
          const int at = 16 * (q4 >> 1) + 8 * h + 4 * (q4 & 1);
          const f32x4 ls = *reinterpret_cast<const f32x4*>(&lds_stat[buf][at]);
          f32x4 dl = {0.f, 0.f, 0.f, 0.f};
          if constexpr (DK) dl = *reinterpret_cast<const f32x4*>(&lds_stat[buf][32 + at]);
#pragma unroll
          for (int e4 = 0; e4 < 4; ++e4) {
            const int x = 4 * q4 + e4;
            float e = fast_exp2(__builtin_fmaf(sr[x], sc, -ls[e4]));
            if constexpr (WIN) {
              float keep = 1.f;
              if (p.drop_thr) {  // row 32 i + 8 h + 16 (x / 8) + x % 8 of query head hq0 + g
                uint32_t v = drop_base + (uint32_t)(hq0 + g) * 0xC2B2AE3Du + (uint32_t)(row0 + 16 * (x >> 3) + (x & 7)) * 0x9E3779B1u;
                v ^= v >> 16, v *= 0x7FEB352Du, v ^= v >> 15, v *= 0x846CA68Bu, v ^= v >> 16;
                keep = v >= p.drop_thr ? p.drop_scale : 0.f;
              }
              if constexpr (DK) e *= dp[x] * keep - dl[e4];
              else e *= keep;
            } else {
              if constexpr (DK) e *= dp[x] - dl[e4];
            }
            pb[x >> 3][x & 7] = (__bf16)e;
          }
        }
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
          for (int db = 0; db < NDB; ++db)
            acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16(lds[buf][SLOTS - KS + blk * NDB + db][lane]), pb[blk],
                                                              acc[db], 0, 0, 0);
      }
      buf = buf + 1 == kRing ? 0 : buf + 1;
      if (++g == group) g = 0, --i;
    }
    FCA_WAIT_VMCNT(0);  // the repeated requests past the last step
  }
  if (live && t < T) {
    const float mul = DK ? p.scale : 1.f;
    if (p.head_split) {
      float* part = (DK ? p.dk_part : p.dv_part) + (((int64_t)(hq0 - hkv * ratio) * T + t) * p.num_kv_heads + hkv) * D + 4 * h;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          f32x4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = acc[db][4 * q4 + e] * mul;
          *reinterpret_cast<f32x4*>(part + 32 * db + 8 * q4) = w;
        }
    } else if constexpr (DK) {
      store_rows<D>(p.dk, (int64_t)t * p.dk_stride + hkv * D, h, acc, mul);
    } else {
      store_rows<D>(p.dv, (int64_t)t * p.dv_stride + hkv * D, h, acc, mul);
    }
  }
}

// out[t][c] = sum over the slices of part[slice][t][c], c over the Hkv * D values of a token.
__global__ __launch_bounds__(kThreads) void split_reduce_kernel(const float* part, int slices, int64_t tokens, int row,
                                                               __bf16* out, int64_t out_stride) {
  const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const int per_row = row / 4;
  if (idx >= tokens * per_row) return;
  const int64_t t = idx / per_row;
  const int c = (int)(idx % per_row) * 4;
  f32x4 sum = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < slices; ++s) sum += *reinterpret_cast<const f32x4*>(part + ((int64_t)s * tokens + t) * row + c);
  bf16x4 w;
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] = (__bf16)sum[e];
  *reinterpret_cast<bf16x4*>(out + t * out_stride + c) = w;
}

template <typename F>
hipError_t by_head_dim(int head_dim, F&& f) {
  if (head_dim == 128) return f(std::integral_constant<int, 128>{});
  if (head_dim == 256) return f(std::integral_constant<int, 256>{});
  if (head_dim == 64) return f(std::integral_constant<int, 64>{});
  return hipErrorInvalidValue;
}

}  // namespace

namespace {
hipError_t images(const void* x, int64_t stride, int heads, int head_dim, int num_tokens, int tiles, void* rows_image,
                  void* transposed_image, hipStream_t stream, const void* other = nullptr, int64_t other_stride = 0,
                  const float* lse = nullptr, float* delta = nullptr, float* lse2 = nullptr) {
  return by_head_dim(head_dim, [&](auto d) {
    constexpr int D = decltype(d)::value;
    split_images_kernel<D><<<dim3(tiles, heads), kThreads, 0, stream>>>(
        static_cast<const __bf16*>(x), stride, num_tokens, tiles, static_cast<__bf16*>(rows_image),
        static_cast<__bf16*>(transposed_image), static_cast<const __bf16*>(other), other_stride, lse, delta, lse2);
    return hipGetLastError();
  });
}
}  // namespace

hipError_t launch_split_forward(const SplitParams& p, int head_dim, hipStream_t stream) {
  const int T = p.num_tokens, nt = p.num_tiles;
  if (hipError_t e = images(p.k, p.k_stride, p.num_kv_heads, head_dim, T, nt, const_cast<void*>(p.kn), nullptr, stream)) return e;
  if (hipError_t e = images(p.v, p.v_stride, p.num_kv_heads, head_dim, T, nt, nullptr, const_cast<void*>(p.vr), stream)) return e;
  return by_head_dim(head_dim, [&](auto d) {
    constexpr int D = decltype(d)::value;
    const unsigned grid = (unsigned)p.num_tiles * ((p.num_q_heads + kWaves - 1) / kWaves);
    // (head size 256 has the LDS-shared kernels only: two register buffers of 32 operand slots
    // each do not fit a wave; such plans are refused when they are checked)
    const bool shared = (p.num_q_heads / p.num_kv_heads) % kWaves == 0;
    if (!shared && D == 256) return hipErrorInvalidValue;
    if (p.window > 0 || p.drop_thr) {
      if (shared) {
        split_query_kernel<D, false, true, true><<<grid, kThreads, 0, stream>>>(p);
      } else if constexpr (D < 256) {
        split_query_kernel<D, false, false, true><<<grid, kThreads, 0, stream>>>(p);
      }
    } else {
      if (shared) {
        split_query_kernel<D, false, true, false><<<grid, kThreads, 0, stream>>>(p);
      } else if constexpr (D < 256) {
        split_query_kernel<D, false, false, false><<<grid, kThreads, 0, stream>>>(p);
      }
    }
    return hipGetLastError();
  });
}

hipError_t launch_split_backward(const SplitParams& p, int head_dim, hipStream_t stream) {
  const int T = p.num_tokens, nt = p.num_tiles;
  auto V = [](const void* x) { return const_cast<void*>(x); };
  if (hipError_t e = images(p.k, p.k_stride, p.num_kv_heads, head_dim, T, nt, V(p.kn), V(p.kr), stream)) return e;
  if (hipError_t e = images(p.v, p.v_stride, p.num_kv_heads, head_dim, T, nt, V(p.vn), nullptr, stream)) return e;
  if (hipError_t e = images(p.q, p.q_stride, p.num_q_heads, head_dim, T, nt, V(p.qn), V(p.qr), stream)) return e;
  // the pass over dO also makes the per-row sums of dO * O and the log-sum-exp in log2 units
  if (hipError_t e = images(p.dout, p.do_stride, p.num_q_heads, head_dim, T, nt, V(p.don), V(p.dor), stream, p.out_in, p.o_stride,
                            p.lse, p.delta, p.lse2))
    return e;
  return by_head_dim(head_dim, [&](auto d) {
    constexpr int D = decltype(d)::value;
    const unsigned qgrid = (unsigned)nt * ((p.num_q_heads + kWaves - 1) / kWaves);
    const bool shared = (p.num_q_heads / p.num_kv_heads) % kWaves == 0;
    if (!shared && D == 256) return hipErrorInvalidValue;
    const int ratio = p.num_q_heads / p.num_kv_heads;
    const unsigned kgrid = (unsigned)((nt + kWaves - 1) / kWaves) * p.num_kv_heads * (p.head_split ? ratio : 1);
    if (p.window > 0 || p.drop_thr) {
      if (shared) {
        split_query_kernel<D, true, true, true><<<qgrid, kThreads, 0, stream>>>(p);
      } else if constexpr (D < 256) {
        split_query_kernel<D, true, false, true><<<qgrid, kThreads, 0, stream>>>(p);
      }
      if (hipError_t e = hipGetLastError()) return e;
      split_key_kernel<D, false, true><<<kgrid, kThreads, 0, stream>>>(p);
      if (hipError_t e = hipGetLastError()) return e;
      split_key_kernel<D, true, true><<<kgrid, kThreads, 0, stream>>>(p);
    } else {
      if (shared) {
        split_query_kernel<D, true, true, false><<<qgrid, kThreads, 0, stream>>>(p);
      } else if constexpr (D < 256) {
        split_query_kernel<D, true, false, false><<<qgrid, kThreads, 0, stream>>>(p);
      }
      if (hipError_t e = hipGetLastError()) return e;
      split_key_kernel<D, false, false><<<kgrid, kThreads, 0, stream>>>(p);
      if (hipError_t e = hipGetLastError()) return e;
      split_key_kernel<D, true, false><<<kgrid, kThreads, 0, stream>>>(p);
    }
    if (hipError_t e = hipGetLastError()) return e;
    if (p.head_split) {
      const int row = p.num_kv_heads * D;
      const unsigned rgrid = (unsigned)(((int64_t)T * (row / 4) + kThreads - 1) / kThreads);
      split_reduce_kernel<<<rgrid, kThreads, 0, stream>>>(p.dv_part, ratio, T, row, static_cast<__bf16*>(p.dv), p.dv_stride);
      if (hipError_t e = hipGetLastError()) return e;
      split_reduce_kernel<<<rgrid, kThreads, 0, stream>>>(p.dk_part, ratio, T, row, static_cast<__bf16*>(p.dk), p.dk_stride);
    }
    return hipGetLastError();
  });
}

}  // namespace fca
