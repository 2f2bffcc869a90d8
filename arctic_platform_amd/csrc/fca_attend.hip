// Forest cascade attention pass for gfx950: one persistent kernel per query-tile height
// serves both the shared-prefix pass (query rows of every member sequence x the GQA heads
// of one KV head stacked into a 32- or 64-row tile) and the per-sequence suffix pass (the
// same tile with only Hq/Hkv live rows).  This file holds the 64-row kernel and the launch
// dispatch; the 32-row kernel is in fca_attend32.hip.
//
// Work item = (node chunk, tile of members) x KV head.  Every wavefront is its own worker:
// it walks its share of the size-ordered work list, streams each chunk's 32-token tiles
// with private online-softmax state and writes one normalised partial per item.  There is
// no workgroup barrier.  At head size 128 the kernels run one wave per SIMD with the whole
// 512-entry register file (two waves where a smaller head leaves room): registers, not
// LDS, are the staging buffer for K and V, because the cache already stores tiles in MFMA
// operand order and a tile in flight needs a place to land either way.
//
// Per tile and wave, with tokens on the MFMA M dimension (the transposed product):
//   St[32 tok x 32 rows] = K[32 x D] . Qt[D x 32]       D/16 x mfma_f32_32x32x16_bf16
//   online softmax over tokens = over the 16 accumulator registers of a lane plus one
//   exchange with the lane 32 away (both hold the same query row)
//   Ot[D x 32 rows]     += Vt[D x 32 tok] . Pt[32 x 32]  D/32 x 2 mfma
// The cache stores K as [D/x][16 tok][x] and V as [D][16 tok], which are the A-operand
// orders of these two products: every operand is one contiguous 16-byte global load per
// lane.  The K rows are fed in the token order that makes the softmax output registers
// line up with the B operand of the second product, so P never leaves registers.
//
// Query runs (several query tokens of one sequence, one query row each) need a mask only
// where a tile of such rows meets its own tokens: the last tile of the last chunk of a
// causal node, where the item record says how many tokens the first member sees and every
// further member sees one more.  Everything else is the unmasked decode product.
//
// Semantics (softmax scale, GQA head mapping h -> h / (Hq/Hkv), no mask for the decode
// token) follow arctic_platform/model/implementations/qwen35/models/qwen3_5_moe/
// modeling_qwen3_5_moe.py:368-373, :385, :440-454.
#include <hip/hip_ext.h>

#include <cstring>
#include <cstdlib>
#include <type_traits>

#include "fca_attend_common.h"

namespace fca {


// The 64-row kernel: one persistent loop per wave that keeps loads in flight across work
// items.  Two 32-row tiles of accumulators and query registers leave room for one K/V
// tile buffer, refilled in halves, and for a one-item lookahead (the four-item lookahead
// of the 32-row kernel spills here).
//
// Dealing the work.  Most tickets are dealt statically, back and forth over the
// size-ordered list: in round r wave w of W takes ticket r * W + w (r even) or
// r * W + W - 1 - w (r odd), which evens out the descending sizes between waves at no
// cost.  A shared counter for everything would be expensive: device-wide atomics on one
// address serialise at roughly 20 ns each across the eight L2s, so 1024 waves asking at
// once wait tens of microseconds.  But waves do not run at the same speed (XCDs stream
// several percent apart on identical work), so the last full round and the remainder,
// the smallest items, come from a counter: each wave draws one item ahead, which hides
// the atomic's latency, and draws until the list is empty.  The draw that returns the
// last possible value re-arms the counter for the next launch.
//
// Hiding item boundaries.  While the tiles of the current item stream, the wave fetches
// the next item's record, block ids and member sequences; the next item's query rows and
// first tile are requested before the current item's partial is written out, so the
// memory pipe does not drain at item boundaries.
//
// NRT = row tiles of 32 query rows per item: 2 for the 64-row items; 1 makes this the 32-row
// kernel of head size 256, where two tile buffers and the deep lookahead of fca_attend32.hip
// do not fit the register file.
template <int D, bool FP8, bool STREAM, int NRT = 2>
__global__ __launch_bounds__(kThreads, workgroups_per_cu(D, FP8, 32 * NRT)) void fca_attend64_kernel(AttendParams p) {
  constexpr int KS = D / 16;   // MFMA steps of the score product
  constexpr int NDB = D / 32;  // 32-channel blocks of the output
  using KT = KTile<D, FP8>;
  using VT = VTile<D, FP8>;

  int32_t* hdr = p.meta + p.off_header;
  const int total = hdr[H_ITEMS], shared = hdr[H_SHARED_ITEMS];
  const int first = p.select == 2 ? shared : 0;
  const int last_item = p.select == 1 ? shared : total;
  const int ntickets = (last_item - first) * p.num_kv_heads;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const int m = lane & 31, h = lane >> 5;
  const int G = p.group, Hkv = p.num_kv_heads;
  const int32_t* meta = p.meta;

  // row n = rt * 32 + m of the stacked query tile is (member n / G, head n % G)
  int row_member[NRT], row_head[NRT];
#pragma unroll
  for (int rt = 0; rt < NRT; ++rt) {
    row_member[rt] = (rt * 32 + m) / G;
    row_head[rt] = (rt * 32 + m) - row_member[rt] * G;
  }
  // MFMA row m carries the token whose index has bits 2 and 3 of m swapped: the score
  // accumulator then holds, per lane half, tokens 8h..8h+7 of each block in register order.
  const int tok_of_m = (m & 3) | ((m & 4) << 1) | ((m & 8) >> 1);
  const int k_lane_off = h * 256 + tok_of_m * 16;
  // bf16: channel 32 * db + m, tokens 8h..8h+7; fp8: channel 32 * (2 * pair + h) + m, all 16 tokens
  const int v_lane_off = FP8 ? (h * 32 + m) * 16 : m * 32 + h * 16;
  constexpr int V_STEP = 1024;
  // wave-private strip of LDS for the output rows
  __shared__ __attribute__((aligned(16))) char strips[kWaves][NRT * 32 * strip_row_bytes<D>()];
  char* strip = strips[wave];

  const int nwaves = (int)gridDim.x * kWaves;
  const int static_tickets = min(ntickets, max(1, ntickets / nwaves - 1) * nwaves);
  // every wave that has work draws until it fails once
  const int dynamic_draws = ntickets - static_tickets + min(nwaves, ntickets);
  const int my_wave = (int)blockIdx.x * kWaves + wave;
  // A zero the compiler cannot see through.  Added to the record address it makes the
  // record look lane-dependent, which keeps the compiler from moving its fields into
  // scalar registers right behind the load: that move waits for every load in flight,
  // tiles included, while the fields are not needed before the next trip.
  int opaque_zero;
  asm volatile("v_mov_b32 %0, 0" : "=v"(opaque_zero));
  // Item record of a ticket (clamped, so a ticket past the end reads a valid record).
  auto load_record = [&](int t, int4& r0, int4& r1, int& kvh) {
    const int tc = min(t, ntickets - 1);
    const int it = tc / Hkv;
    kvh = tc - it * Hkv;
    const int4* rec =
        reinterpret_cast<const int4*>(meta + p.off_items + (int64_t)(first + it) * kItemInts + opaque_zero);
    r0 = rec[0];  // rep, blk_start, tok_len, member_off
    r1 = rec[1];  // member_cnt, ord, node, tokens the first member sees (causal last chunk) or 0
  };
  // Per-lane data that hangs off a record: one block id of the chunk per lane (a chunk has
  // at most 64 blocks) and the member sequence of this lane's query row(s).
  auto load_lane_meta = [&](const int4& r0, const int4& r1, int& my_blk, int (&seq)[NRT]) {
    const int nblk = (r0.z + kBlock - 1) / kBlock;
    my_blk = p.block_table[(int64_t)r0.x * p.bt_stride + r0.y + min(lane, nblk - 1)];
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) seq[rt] = meta[p.off_members + r0.w + (row_member[rt] < r1.x ? row_member[rt] : 0)];
  };
  bf16x8 qreg[NRT][KS];
  auto load_q = [&](const int (&seq)[NRT], int mcnt, int kvh) {
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
      const bool live = row_member[rt] < mcnt;
      const __bf16* qp = reinterpret_cast<const __bf16*>(p.q) + (int64_t)seq[rt] * p.q_seq_stride +
                         (int64_t)(kvh * G + row_head[rt]) * p.q_head_stride;
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
  };
  // The fences keep the compiler from sinking the loads below the arithmetic that follows,
  // which starts with a wait: a refill must be on its way before the wave blocks.
  auto load_k = [&](KT& kt, int my_blk, int nblk, int kvh, int ti) {
    __builtin_amdgcn_sched_barrier(0);
    const int p0 = 2 * ti, p1 = min(2 * ti + 1, nblk - 1);
    const int b0 = __builtin_amdgcn_readlane(my_blk, p0);
    const int b1 = __builtin_amdgcn_readlane(my_blk, p1);
    const int kb = (m & 16) ? b1 : b0;
    const char* kp = p.k_cache + (int64_t)kvh * p.kv_head_bytes + (int64_t)kb * p.kv_block_bytes + k_lane_off;
#pragma unroll
    for (int i = 0; i < KT::NK; ++i) kt.k[i] = load16<STREAM>(kp + i * 512);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto load_v = [&](VT& vt, int my_blk, int nblk, int kvh, int ti) {
    __builtin_amdgcn_sched_barrier(0);
    const int p0 = 2 * ti, p1 = min(2 * ti + 1, nblk - 1);
    const int b0 = __builtin_amdgcn_readlane(my_blk, p0);
    const int b1 = __builtin_amdgcn_readlane(my_blk, p1);
    const char* vbase = p.v_cache + (int64_t)kvh * p.kv_head_bytes + v_lane_off;
    const char* vp0 = vbase + (int64_t)b0 * p.kv_block_bytes;
    const char* vp1 = vbase + (int64_t)b1 * p.kv_block_bytes;
#pragma unroll
    for (int i = 0; i < VT::NV; ++i) {
      vt.v[0][i] = load16<STREAM>(vp0 + i * V_STEP);
      vt.v[1][i] = load16<STREAM>(vp1 + i * V_STEP);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto load_tile = [&](KT& kt, VT& vt, int my_blk, int nblk, int kvh, int ti) {
    load_k(kt, my_blk, nblk, kvh, ti);
    load_v(vt, my_blk, nblk, kvh, ti);
  };

  // ---- first item of this wave: fetched with the waits exposed
  int round = 0;
  if (my_wave < ntickets) {
    int4 r0, r1;
    int kvh, my_blk, seq[NRT];
    load_record(my_wave, r0, r1, kvh);
    load_lane_meta(r0, r1, my_blk, seq);
    load_q(seq, r1.x, kvh);
    // The tile buffer, refilled in halves.
    KT kb;
    VT vb;
    auto request_first_tiles = [&](int blk_ids, int len, int head) {
      load_tile(kb, vb, blk_ids, (len + kBlock - 1) / kBlock, head, 0);
    };
    request_first_tiles(my_blk, __builtin_amdgcn_readfirstlane(r0.z), kvh);

    for (;;) {
      const int tok_len = __builtin_amdgcn_readfirstlane(r0.z);
      const int mcnt = __builtin_amdgcn_readfirstlane(r1.x);
      const int ord = __builtin_amdgcn_readfirstlane(r1.y);
      const int rows = mcnt * G;
      const bool two_tiles = rows > 32;
      const int nblk = (tok_len + kBlock - 1) / kBlock;
      const int ntiles = (tok_len + kTile - 1) / kTile;
      // Last chunk of a query-run tile: member i sees the first `sees + i` tokens of the chunk
      // (its own token and what is before it).  All members end inside the last tile, which
      // then takes the masking path even when the chunk fills it.
      const int sees = __builtin_amdgcn_readfirstlane(r1.w);
      const int nfull = (tok_len - (sees > 0 ? 1 : 0)) / kTile;  // tiles without masking; at most one masked tile follows
      const int last = ntiles - 1;
      int64_t prow[NRT];  // partial row this lane's query row is written to, -1 for a dead row
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt)
        prow[rt] = row_member[rt] < mcnt
                       ? ((int64_t)seq[rt] * p.max_partials + ord) * p.num_q_heads + kvh * G + row_head[rt]
                       : -1;

      // next item: chase its record and per-lane data during the tile loop
      ++round;
      int t_next_v;  // meaningful in lane 0
      if (round * nwaves < static_tickets) {
        t_next_v = round * nwaves + ((round & 1) ? nwaves - 1 - my_wave : my_wave);
      } else {
        t_next_v = 0;
        if (lane == 0) {
          const int drawn = atomicAdd(&hdr[H_TICKET], 1);
          if (drawn == dynamic_draws - 1) hdr[H_TICKET] = 0;  // nobody draws after this one
          t_next_v = static_tickets + drawn;
        }
      }
      int4 n0 = r0, n1 = r1;  // harmless defaults for the first refresh below
      int nkvh = kvh, nmy_blk = my_blk, nseq[NRT];
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt) nseq[rt] = seq[rt];

      f32x16 acc[NRT][NDB];
      float mrow[NRT], lrow[NRT];  // reference maximum (scaled, log2 domain) and running sum
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

      // One 32-token tile.  RAGGED is the variant for the single tile that may run past the
      // end of the chunk: it masks scores and zeroes V there; full tiles carry no mask code.
      bf16x8 pb[NRT][2];  // probabilities of the current tile as B operands
      auto scores_softmax = [&](const KT& kt, int ti, auto ragged) {
        constexpr bool RAGGED = decltype(ragged)::value;
        const int tok0 = ti * kTile;
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt) {
          if (rt > 0 && !two_tiles) continue;
          // scores of one row tile at a time: the second tile reuses the score registers
          f32x16 sr;
#pragma unroll
          for (int r = 0; r < 16; ++r) sr[r] = 0.f;
#pragma unroll
          for (int i = 0; i < KS; ++i) {
            bf16x8 a;
            if constexpr (FP8) {
              const i32x4 w = kt.k[i >> 1];
              a = (i & 1) ? fp8x8_to_bf16(w[2], w[3]) : fp8x8_to_bf16(w[0], w[1]);
            } else {
              a = __builtin_bit_cast(bf16x8, kt.k[i]);
            }
            sr = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[rt][i], sr, 0, 0, 0);
          }
          // register r holds token 16 * (r / 8) + 8 * h + r % 8 of the tile
          if constexpr (RAGGED) {
            // every score register of a lane belongs to the lane's own query row
            const int row_lim = sees > 0 ? min(tok_len, sees + row_member[rt]) : tok_len;
#pragma unroll
            for (int r = 0; r < 16; ++r)
              if (tok0 + 16 * (r >> 3) + 8 * h + (r & 7) >= row_lim) sr[r] = -INFINITY;
          }
          float mx = sr[0];
#pragma unroll
          for (int r = 1; r < 16; ++r) mx = fmaxf(mx, sr[r]);
          mx = fmaxf(mx, __shfl_xor(mx, 32));
          // sc > 0, so the maximum of the scaled scores is the scaled maximum.  mrow is the
          // reference the exponentials are taken against, not the exact running maximum: it
          // moves (and the accumulators are rescaled) only when a row's maximum rises more
          // than kRescaleSlack above it, so probabilities stay below 2^kRescaleSlack and the
          // rescale, which touches every accumulator register, is rare.  The log-sum-exp
          // m + log2(l) does not depend on the reference.
          // The first tile sets the reference without a rescale (the accumulators are zero).
          const float mtile = mx * sc;
          if (ti == 0) mrow[rt] = mtile;
          if (__builtin_amdgcn_readfirstlane(__any(mtile > mrow[rt] + kRescaleSlack))) {
            const float mnew = fmaxf(mrow[rt], mtile);
            const float alpha = fast_exp2(mrow[rt] - mnew);
            lrow[rt] *= alpha;
            mrow[rt] = mnew;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
              for (int r = 0; r < 16; ++r) acc[rt][db][r] *= alpha;
          }
          const float mref = mrow[rt];
          float sum = 0.f;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float e = fast_exp2(__builtin_fmaf(sr[r], sc, -mref));
            sum += e;
            pb[rt][r >> 3][r & 7] = (__bf16)e;
          }
          lrow[rt] += sum;
        }
      };
      auto weighted_values = [&](const VT& vt, int ti, auto ragged) {
        constexpr bool RAGGED = decltype(ragged)::value;
        const int tok0 = ti * kTile;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
          // tokens this lane feeds for this block: 8h .. 8h+7; on the ragged tile zero the
          // ones past the end so stale cache contents (possibly NaN) cannot leak through 0 * x
          const int nv = tok_len - (tok0 + 16 * blk + 8 * h);
#pragma unroll
          for (int db = 0; db < NDB; ++db) {
            bf16x8 a;
            if constexpr (FP8) {
              // rows of channel blocks 2 * pair and 2 * pair + 1 sit in the lower and upper
              // lane halves; the swap hands every lane its tokens 8h..8h+7 of both blocks:
              // dwords 0,1 become the operand of block 2 * pair, dwords 2,3 of 2 * pair + 1
              const i32x4 raw = vt.v[blk][db >> 1];
              const auto s0 = __builtin_amdgcn_permlane32_swap((unsigned)raw[0], (unsigned)raw[2], false, false);
              const auto s1 = __builtin_amdgcn_permlane32_swap((unsigned)raw[1], (unsigned)raw[3], false, false);
              i32x2 w = {(int)s0[db & 1], (int)s1[db & 1]};
              if constexpr (RAGGED) {
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
              if constexpr (RAGGED) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  unsigned keep = (2 * j < nv ? 0xffffu : 0u) | (2 * j + 1 < nv ? 0xffff0000u : 0u);
                  w[j] &= keep;
                }
              }
              a = __builtin_bit_cast(bf16x8, w);
            }
            acc[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[0][blk], acc[0][db], 0, 0, 0);
            if (two_tiles) acc[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[1][blk], acc[1][db], 0, 0, 0);
          }
        }
      };

      auto compute_tile = [&](const KT& kt, const VT& vt, int ti, auto ragged) {
        scores_softmax(kt, ti, ragged);
        weighted_values(vt, ti, ragged);
      };

      // Tile pipeline; the first tiles are already requested.  Prefetches past the end are
      // clamped to the last tile instead of skipped, so the outstanding-load count is the
      // same on every path and every wait covers exactly the tile about to be used.  Each
      // trip also advances the next item's chain by one hop: the per-lane data is (re)read
      // from the record fetched one trip earlier, then the record is (re)read from the
      // ticket; both are idempotent, so no branch is needed.
      int ti = 0, trips = 0;
      // the next K as soon as the scores have issued, the next V as soon as the value
      // product has
      for (; ti < nfull; ++ti, ++trips) {
        scores_softmax(kb, ti, std::false_type{});
        load_k(kb, my_blk, nblk, kvh, min(ti + 1, last));
        weighted_values(vb, ti, std::false_type{});
        load_v(vb, my_blk, nblk, kvh, min(ti + 1, last));
        if (trips >= 1) {  // the first trip leaves a drawn ticket time to arrive
          load_lane_meta(n0, n1, nmy_blk, nseq);
          load_record(__builtin_amdgcn_readfirstlane(t_next_v), n0, n1, nkvh);
        }
      }
      if (ti < ntiles) compute_tile(kb, vb, ti, std::true_type{});

      // finish the chain for items too short to have done it on the way
      const int t_next = __builtin_amdgcn_readfirstlane(t_next_v);
      if (trips < 2) load_record(t_next, n0, n1, nkvh);
      if (trips < 3) load_lane_meta(n0, n1, nmy_blk, nseq);
      const bool more = t_next < ntickets;
      if (more) {
        // q registers and the tile buffer are dead now: request the next item's query rows
        // and first tile before writing this item's partial
        load_q(nseq, n1.x, nkvh);
        request_first_tiles(nmy_blk, __builtin_amdgcn_readfirstlane(n0.z), nkvh);
      }

      // Write the partial.  Every accumulator register of a lane belongs to the lane's own
      // query row, so normalisation is per lane.  The rows then pass through a wave-private
      // strip of LDS so that they leave as whole rows: stored straight from the accumulator
      // layout a row goes out in sixteen pieces, and partial writes of a cache line are slow.
      // (The fp8 scales are read where they are used: this kernel has no register to carry
      // them an item ahead, and its item boundaries wait for the loads in flight anyway.)
      float vs = 1.f;
      if (FP8 && p.v_scale) vs = p.v_scale[kvh];
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt) {
        if (rt > 0 && !two_tiles) continue;
        const float l = lrow[rt] + __shfl_xor(lrow[rt], 32);
        stage_partial_row<D, STREAM>(strip, rt * 32 + m, h, acc[rt], vs / l, prow[rt], (mrow[rt] + fast_log2(l)) * kLn2,
                             p.partial_lse);
      }
      __builtin_amdgcn_wave_barrier();
      store_partial_rows<D, STREAM>(strip, rows, lane, p.partial_out);
      __builtin_amdgcn_wave_barrier();
      if (!more) break;
      r0 = n0;
      r1 = n1;
      kvh = nkvh;
      my_blk = nmy_blk;
#pragma unroll
      for (int rt = 0; rt < NRT; ++rt) seq[rt] = nseq[rt];
    }
  }
}

static thread_local hipEvent_t g_time_start = nullptr, g_time_stop = nullptr;
void set_attend_timing(hipEvent_t start, hipEvent_t stop) { g_time_start = start, g_time_stop = stop; }
void take_attend_timing(hipEvent_t* start, hipEvent_t* stop) {
  *start = g_time_start, *stop = g_time_stop;
  g_time_start = g_time_stop = nullptr;
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

hipError_t launch_attend(const AttendParams& p, const fca_plan& plan, int kv_dtype, int max_workgroups, int tile_buffers, hipStream_t stream) {
  const bool fp8 = kv_dtype == FCA_FP8_E4M3;
  const int nrt = plan.rows_per_item / 32;
  // Four independent waves per workgroup.  At head size 128 a wave uses the whole register
  // file of its SIMD, so one workgroup per CU; at head size 64 two fit (32-row bf16 aside),
  // and the second wave per SIMD hides the arithmetic latency of a tile, which is what
  // limits a head that small (fp8 most of all).
  const int64_t max_tickets = (int64_t)plan.num_seqs *
                              ((int64_t)plan.max_blocks * kBlock / plan.chunk_tokens + plan.max_levels + 2) *
                              plan.num_kv_heads;
  int grid = cached_cu_count() * workgroups_per_cu(plan.head_dim, fp8, plan.rows_per_item);
  // the caller's cap: leaves CUs to other streams (and brings the many-items-per-wave
  // schedules of a large batch to a small one)
  if (max_workgroups > 0 && max_workgroups < grid) grid = max_workgroups;
  if ((int64_t)grid * kWaves > max_tickets) grid = (int)((max_tickets + kWaves - 1) / kWaves);
  if (grid < 1) grid = 1;
  if (nrt == 1 && plan.head_dim != 256) return launch_attend32(p, plan, kv_dtype, tile_buffers, grid, stream);
  // With sharing on, a launch reads every KV block once: stream it past the caches.  With
  // sharing off, sequences of a group read the same blocks again and again and the
  // memory-side cache serves the repeats, so the loads stay ordinary; likewise when query
  // runs make successive tiles of a sequence read the same blocks.
  const bool stream_kv = plan.max_levels > 0 && !p.kv_reread;
  hipEvent_t ev_start, ev_stop;
  take_attend_timing(&ev_start, &ev_stop);
#define FCA_LAUNCH(D_, F_, S_, N_) \
  if (ev_start) hipExtLaunchKernelGGL((fca_attend64_kernel<D_, F_, S_, N_>), dim3(grid), dim3(kThreads), 0, stream, ev_start, ev_stop, 0, p); \
  else hipLaunchKernelGGL((fca_attend64_kernel<D_, F_, S_, N_>), dim3(grid), dim3(kThreads), 0, stream, p)
#define FCA_PICK(D_, F_, N_) \
  if (stream_kv) { FCA_LAUNCH(D_, F_, true, N_); } else { FCA_LAUNCH(D_, F_, false, N_); }
  if (plan.head_dim == 256) {  // 32-row items only (checked with the plan)
    if (fp8) { FCA_PICK(256, true, 1); } else { FCA_PICK(256, false, 1); }
  } else if (plan.head_dim == 128) {
    if (fp8) { FCA_PICK(128, true, 2); } else { FCA_PICK(128, false, 2); }
  } else {
    if (fp8) { FCA_PICK(64, true, 2); } else { FCA_PICK(64, false, 2); }
  }
#undef FCA_PICK
#undef FCA_LAUNCH
  return hipGetLastError();
}

}  // namespace fca

