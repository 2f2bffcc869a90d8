// Forest cascade attention pass for query tiles of up to 32 rows: the tile stream of a
// wave never drains at an item boundary.
//
// Same work items, arithmetic and register-staged tiles as the kernel in fca_attend.hip;
// what differs is the schedule around the boundaries between items.  A wave looks four
// items ahead: at one fixed point of every item it takes one step for each of the
// following items -- query rows of item k+1, block ids and member sequences of item k+2,
// record of item k+3, ticket of item k+4 -- so every step reads what the step before it
// fetched one whole item earlier, and nothing is ever waited for at the place it was
// requested.  Tiles are attended in groups of as many as there are tile buffers (NB: two; three
// in the instance for fp8 at head size 128 that a caller can ask for, whose tiles are half the
// size).  Where an expression differs between the two it is picked by NB at compile time with
// the two-buffer form spelt as it always was: the two-buffer instances are the kernels that
// have been measured, and they compile to the same instructions as before NB existed.  With the next item's block ids
// at hand, the buffers are refilled with the next item's first tiles as soon as the current
// item's last tiles have been consumed, exactly as they are refilled inside an item.
//
// The last item of a wave is shared with a wave of another XCD.  XCDs stream at different
// speeds (the slowest takes about a sixth longer per tile than the fastest, and which is
// which differs from box to box), and with a handful of items per wave, drawn four items
// ahead of use, the draws come too early to tell a fast wave from a slow one.  So the
// largest items of the list are set aside, one per pair of waves (grids of a multiple of
// eight workgroups): both waves of a pair take
// the item as their last, one from its first group of tiles upwards, the other from its last
// group downwards, each claiming the next group of tiles from a counter of the pair until the
// claims meet.  Whichever wave arrives earlier or streams faster takes more of the item,
// and each wave writes a partial of its own (the second one into rows set aside behind the
// ordinary partial rows; the first one's row scale carries the second one's address).
//
// All loads sit at fixed places of the instruction stream (none inside a data-dependent
// branch): the hardware counts outstanding vector memory operations in order and the
// compiler picks each wait's count for the shortest path, so a load issued on only some
// paths would turn the waits behind it into full drains of the tile stream.
#include <hip/hip_ext.h>

#include <type_traits>

#include "fca_attend_common.h"

namespace fca {

template <int D, bool FP8, bool STREAM, int NB = 2>
__global__ __launch_bounds__(kThreads, workgroups_per_cu(D, FP8, 32)) void fca_attend32_kernel(AttendParams p) {
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
  const int nwaves = (int)gridDim.x * kWaves;
  const int my_wave = (int)blockIdx.x * kWaves + wave;
  if (my_wave >= ntickets) return;

  // row m of the stacked query tile is (member m / G, head m % G)
  const int row_member = m / G;
  const int row_head = m - row_member * G;
  // Query head of this lane's row under KV head kvh, for the three-buffer instance.  The sum is
  // formed in 32 bits, unsigned, at every use: written as a 64-bit sum the lane's share of it is
  // hoisted out of the item loop as a 64-bit register pair, and that instance has none to spare.
  auto q_head_of = [&](int kvh_) -> unsigned { return (unsigned)(kvh_ * G) + (unsigned)row_head; };
  // MFMA row m carries the token whose index has bits 2 and 3 of m swapped: the score
  // accumulator then holds, per lane half, tokens 8h..8h+7 of each block in register order.
  const int tok_of_m = (m & 3) | ((m & 4) << 1) | ((m & 8) >> 1);
  const int k_lane_off = h * 256 + tok_of_m * 16;
  // bf16: channel 32 * db + m, tokens 8h..8h+7; fp8: channel 32 * (2 * pair + h) + m, all 16 tokens
  const int v_lane_off = FP8 ? (h * 32 + m) * 16 : m * 32 + h * 16;
  constexpr int V_STEP = 1024;
  // wave-private strip of LDS for the output rows
  __shared__ __attribute__((aligned(16))) char strips[kWaves][32 * strip_row_bytes<D>()];
  char* strip = strips[wave];

  // Dealing the work.  Round r gives wave w of W ticket r * W + w (r even) or
  // r * W + W - 1 - w (r odd) over the size-ordered list, for all rounds but the last full
  // one and the remainder: those come from a counter in the metadata header, drawn four
  // items ahead of use, so a wave that streams faster takes more of the small items.  A
  // list shorter than five rounds is dealt statically as a whole.  Every wave draws until
  // its first failing draw; the draw that returns the last possible value resets the
  // counter for the next launch.
  // Cooperative last items: tickets [0, coop) are set aside, one per pair of waves; the rest
  // of the list (nmain tickets, numbered from coop upwards) is dealt as described above.
  // Workgroup b of the lower half of the grid pairs with workgroup (b + half the grid) ^ 3,
  // which the dispatcher places on another XCD (an even one with an odd one, an outer one
  // with an inner one) and whose place in every round of the dealing is half a round away,
  // so that the two bring complementary shares of the list (pairing neighbours, whose shares
  // are nearly the same, measured 1.4 % slower on the three-level forest and the same on the
  // Qwen3-4B shape); its wave w pairs with wave w there.  The lower half takes its items from
  // the front.
  const int half_grid = (int)gridDim.x >> 1;
  const bool coop_back = (int)blockIdx.x >= half_grid;
  const int pair_id = (coop_back ? (((int)blockIdx.x ^ 3) - half_grid) : (int)blockIdx.x) * kWaves + wave;
  // (not where two workgroups share a CU: the second wave per SIMD evens the speeds out, and
  // the kernel has no registers to spare there)
  constexpr bool COOP = workgroups_per_cu(D, FP8, 32) == 1;
  const bool coop_on = COOP && p.coop_ctr != nullptr && (gridDim.x & 7) == 0 && nwaves / 2 <= p.coop_pairs &&
                       ntickets >= nwaves / 2 + 3 * nwaves;
  const int coop = coop_on ? nwaves / 2 : 0;
  const int nmain = ntickets - coop;
  const int static_tickets = nmain < 5 * nwaves ? nmain : (nmain / nwaves - 1) * nwaves;
  const int dynamic_draws = nmain - static_tickets + nwaves;
  bool drawing = static_tickets < nmain;
  bool coop_pending = coop_on;
  // A zero the compiler cannot see through; it makes an address look lane-dependent.
  int opaque_zero;
  asm volatile("v_mov_b32 %0, 0" : "=v"(opaque_zero));
  // Tickets of static rounds are computed when they are resolved.  A drawn ticket lives
  // in lane 0 of tv_drawn from the draw to its resolution one item later; the static
  // rounds never touch that register, so they never wait for it.
  int tv_drawn = 0;
  auto issue_ticket = [&](int r) {
    // (behind a uniform address the compiler would read the result back on the spot to share
    // it between lanes, and wait for every load in flight)
    if (r * nwaves >= static_tickets && drawing && lane == 0)
      tv_drawn = atomicAdd(&hdr[H_TICKET + opaque_zero], 1);
  };
  // what follows a wave's last ticket of the main list: its pair's item, then nothing
  auto after_main = [&]() -> int {
    if (!coop_pending) return ntickets;
    coop_pending = false;
    return pair_id;
  };
  // ticket of round r; ntickets or more = none
  auto resolve_ticket = [&](int r) -> int {
    if (r * nwaves < static_tickets) {
      const int t = r * nwaves + ((r & 1) ? nwaves - 1 - my_wave : my_wave);
      return t < nmain ? coop + t : after_main();
    }
    if (!drawing) return after_main();
    const int drawn = __builtin_amdgcn_readfirstlane(tv_drawn);
    if (drawn == dynamic_draws - 1 && lane == 0) hdr[H_TICKET] = 0;  // nobody draws after this one
    const int t = static_tickets + drawn;
    if (t >= nmain) {
      drawing = false;
      return after_main();
    }
    return coop + t;
  };

  // The opaque zero in the record address keeps the compiler from moving the record's
  // fields into scalar registers right behind the load: that move would wait for every
  // load in flight.
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
  // at most 64 blocks) and the member sequence of this lane's query row.
  auto load_lane_meta = [&](const int4& r0, const int4& r1, int& my_blk, int& seq) {
    const int nblk = (r0.z + kBlock - 1) / kBlock;
    my_blk = p.block_table[(int64_t)r0.x * p.bt_stride + r0.y + min(lane, nblk - 1)];
    seq = meta[p.off_members + r0.w + (row_member < r1.x ? row_member : 0)];
  };
  auto load_q = [&](bf16x8 (&q)[KS], int seq, int mcnt, int kvh) {
    const bool live = row_member < mcnt;
    const __bf16* qp = reinterpret_cast<const __bf16*>(p.q) + (int64_t)seq * p.q_seq_stride +
                       (NB == 3 ? (int64_t)q_head_of(kvh) : (int64_t)(kvh * G + row_head)) * p.q_head_stride;
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      // channel offset of MFMA step i for this lane half: the K tile hands a lane 16 bytes
      // of one token, i.e. 8 channels (bf16) or 16 channels = two steps (fp8)
      const int dq = FP8 ? 32 * (i >> 1) + 16 * h + 8 * (i & 1) : 16 * i + 8 * h;
      bf16x8 v = *reinterpret_cast<const bf16x8*>(qp + dq);
      if (!live) v = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      q[i] = v;
    }
  };
  // The fences keep the compiler from sinking the loads below the first instructions of
  // the next tile's arithmetic, which start with a wait for that tile: a refill must be on
  // its way before the wave blocks.
  auto load_tile = [&](KT& kt, VT& vt, int my_blk, int nblk, int kvh, int ti) {
    __builtin_amdgcn_sched_barrier(0);
    const int p0 = 2 * ti, p1 = min(2 * ti + 1, nblk - 1);
    const int b0 = __builtin_amdgcn_readlane(my_blk, p0);
    const int b1 = __builtin_amdgcn_readlane(my_blk, p1);
    const int kb = (m & 16) ? b1 : b0;
    const char* kp = p.k_cache + (int64_t)kvh * p.kv_head_bytes + (int64_t)kb * p.kv_block_bytes + k_lane_off;
#pragma unroll
    for (int i = 0; i < KT::NK; ++i) kt.k[i] = load16<STREAM>(kp + i * 512);
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

  // ---- set-up: the first three items of this wave; their tickets are static
  int4 r0, r1, a0, a1, b0, b1;  // records of the current item and the two after it
  int kvh, akvh, bkvh;
  int my_blk, seq, a_blk, a_seq;  // per-lane data of the current and the next item
  int t_cur = resolve_ticket(0);  // rounds 0 to 3 are static, or the whole list is
  int ta = resolve_ticket(1);
  int tb = resolve_ticket(2);
  load_record(t_cur, r0, r1, kvh);
  load_record(ta, a0, a1, akvh);
  load_record(tb, b0, b1, bkvh);
  load_lane_meta(r0, r1, my_blk, seq);
  load_lane_meta(a0, a1, a_blk, a_seq);
  bf16x8 qreg[KS], nq[KS];
  load_q(qreg, seq, r1.x, kvh);
  // fp8 scales of an item's KV head: fetched one item ahead like the query rows (read at
  // the start of an item they would be waited for on the spot, with every tile in flight).
  // The loads are unconditional; without a scale array they read the query tensor and the
  // value is dropped.
  auto load_scales = [&](int head, float& ks, float& vs) {
    if constexpr (FP8) {
      const float* kp = p.k_scale ? p.k_scale + head : reinterpret_cast<const float*>(p.q);
      const float* vp = p.v_scale ? p.v_scale + head : reinterpret_cast<const float*>(p.q);
      if constexpr (NB == 3) {
        // scalar loads: their results live in scalar registers, which this instance has to
        // spare, and their counter is not the one the tile loads are waited for by
        const float k = *kp, v = *vp;
        ks = p.k_scale ? k : 1.f;
        vs = p.v_scale ? v : 1.f;
      } else {
        const float k = kp[opaque_zero], v = vp[opaque_zero];
        ks = p.k_scale ? k : 1.f;
        vs = p.v_scale ? v : 1.f;
      }
    }
  };
  float k_scale = 1.f, v_scale = 1.f, next_k_scale = 1.f, next_v_scale = 1.f;
  load_scales(kvh, k_scale, v_scale);
  // Tile buffers: two, or three where the registers allow it (an fp8 tile is half the size of a
  // bf16 one, and with two of them in flight the kernel runs at the latency of memory rather
  // than at its rate).  Tiles are attended in groups of NB; buffer b holds tile b of a group.
  KT kb0, kb1, kb2;
  VT vb0, vb1, vb2;
  {
    const int len = __builtin_amdgcn_readfirstlane(r0.z);
    const int nb = (len + kBlock - 1) / kBlock;
    const int lt = (len + kTile - 1) / kTile - 1;
    load_tile(kb0, vb0, my_blk, nb, kvh, 0);
    load_tile(kb1, vb1, my_blk, nb, kvh, min(1, lt));
    if constexpr (NB == 3) load_tile(kb2, vb2, my_blk, nb, kvh, min(2, lt));
  }

  // ---- state of the item being attended
  struct Item {
    int tok_len;  // KV tokens of the chunk
    // Last chunk of a query-run tile: member i sees the first `sees + i` tokens of the chunk
    // (its own token and what is before it).  All members end inside the last tile, which
    // then takes the masking path even when the chunk fills it.
    int sees;
    f32x16 acc[NDB];
    float mrow, lrow;  // reference maximum (scaled, log2 domain) and running sum
    float sc;
  };
  auto begin_item = [&](Item& it) {
    it.tok_len = __builtin_amdgcn_readfirstlane(r0.z);
    it.sees = __builtin_amdgcn_readfirstlane(r1.w);
    it.mrow = -INFINITY, it.lrow = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) it.acc[db][r] = 0.f;
    it.sc = p.scale * kLog2e;
    if (FP8) it.sc *= k_scale;
  };

  // One 32-token tile.  RAGGED is the variant for the single tile that may run past the
  // end of the chunk: it masks scores and zeroes V there; full tiles carry no mask code.
  auto compute_tile = [&](Item& it, const KT& kt, const VT& vt, int ti, auto ragged) {
    constexpr bool RAGGED = decltype(ragged)::value;
    f32x16(&acc)[NDB] = it.acc;
    float &mrow = it.mrow, &lrow = it.lrow;
    const float sc = it.sc;
    const int tok_len = it.tok_len, sees = it.sees;
    const int tok0 = ti * kTile;
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
      sr = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[i], sr, 0, 0, 0);
    }
    // register r holds token 16 * (r / 8) + 8 * h + r % 8 of the tile
    if constexpr (RAGGED) {
      // every score register of a lane belongs to the lane's own query row
      const int row_lim = sees > 0 ? min(tok_len, sees + row_member) : tok_len;
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
    // moves (and the accumulators are rescaled) only when a row's maximum rises more than
    // kRescaleSlack above it, so probabilities stay below 2^kRescaleSlack and the rescale,
    // which touches every accumulator register, is rare.  The log-sum-exp m + log2(l)
    // does not depend on the reference.
    // The first tile sets the reference without a rescale (the accumulators are zero).
    const float mtile = mx * sc;
    if (ti == 0) mrow = mtile;
    if (__builtin_amdgcn_readfirstlane(__any(mtile > mrow + kRescaleSlack))) {
      const float mnew = fmaxf(mrow, mtile);
      const float alpha = fast_exp2(mrow - mnew);
      lrow *= alpha;
      mrow = mnew;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[db][r] *= alpha;
    }
    const float mref = mrow;
    float sum = 0.f;
    bf16x8 pb[2];  // probabilities of the tile as B operands
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float e = fast_exp2(__builtin_fmaf(sr[r], sc, -mref));
      sum += e;
      pb[r >> 3][r & 7] = (__bf16)e;
    }
    lrow += sum;
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
        acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[blk], acc[db], 0, 0, 0);
      }
    }
  };

  // Write the partial of the item just attended: rows of a live member go to `prow` (-1: dead
  // row), `tag` rides in the mantissa of the stored row scale.  Every accumulator register of
  // a lane belongs to the lane's own query row, so normalisation is per lane.  The rows then
  // pass through a wave-private strip of LDS so that they leave as whole rows: stored
  // straight from the accumulator layout a row goes out in sixteen pieces, and back-to-back
  // partial writes to one cache line cost a wave several microseconds per item.
  auto write_partial = [&](Item& it, int64_t prow, int live_rows, int tag) {
    const float vs = FP8 ? v_scale : 1.f;
    const float l = it.lrow + __shfl_xor(it.lrow, 32);
    // an item half of which nobody attended here (the other wave of the pair took all of it)
    // leaves an empty partial: log-sum-exp -inf, weight 0 in the merge
    const float inv = l > 0.f ? vs / l : 0.f;
    stage_partial_row<D, STREAM>(strip, m, h, it.acc, inv, prow, (it.mrow + fast_log2(l)) * kLn2, p.partial_lse, tag);
    __builtin_amdgcn_wave_barrier();
    store_partial_rows<D, STREAM>(strip, live_rows, lane, p.partial_out);
    __builtin_amdgcn_wave_barrier();
  };

  bool to_pair_item = false;
  for (int round = 0;; ++round) {
    Item it;
    begin_item(it);
    const int tok_len = it.tok_len, sees = it.sees;
    const int mcnt = __builtin_amdgcn_readfirstlane(r1.x);
    const int ord = __builtin_amdgcn_readfirstlane(r1.y);
    const int nblk = (tok_len + kBlock - 1) / kBlock;
    const int ntiles = (tok_len + kTile - 1) / kTile;
    const int nfull = (tok_len - (sees > 0 ? 1 : 0)) / kTile;  // tiles without masking; at most one masked tile follows
    const int last = ntiles - 1;
    const int ngroups = NB == 2 ? (ntiles + 1) >> 1 : (ntiles + NB - 1) / NB;
    // partial row this lane's query row is written to, -1 for a dead row
    const int64_t prow = row_member < mcnt
                             ? (NB == 3 ? ((int64_t)seq * p.max_partials + ord) * p.num_q_heads + (int64_t)q_head_of(kvh)
                                        : ((int64_t)seq * p.max_partials + ord) * p.num_q_heads + kvh * G + row_head)
                             : -1;
    const int a_len = __builtin_amdgcn_readfirstlane(a0.z);
    const int a_nblk = (a_len + kBlock - 1) / kBlock;
    const int a_last = (a_len + kTile - 1) / kTile - 1;
    // first tiles of the next item: its first group, or, for the wave that takes its pair's
    // item from the back, its last group
    const bool a_from_back = COOP && coop_back && ta < coop && (NB == 2 ? a_last >= 2 * kCoopMinPairs - 2 : (a_last + NB) / NB >= kCoopMinPairs);
    const int a_t0 = a_from_back ? (NB == 2 ? (a_last & ~1) : NB * ((a_last + NB) / NB - 1)) : 0;
    const int a_t1 = min(a_t0 + 1, a_last);

    // ---- all groups of tiles but the last: every tile full, refills from this item.
    // Buffer b holds tile ti + b; a refill past the end (a last group that is not full)
    // repeats the last tile so that the number of loads in flight never varies.
    for (int gr = 0; gr < ngroups - 1; ++gr) {
      const int ti = NB * gr;
      compute_tile(it, kb0, vb0, ti, std::false_type{});
      load_tile(kb0, vb0, my_blk, nblk, kvh, ti + NB);
      compute_tile(it, kb1, vb1, ti + 1, std::false_type{});
      load_tile(kb1, vb1, my_blk, nblk, kvh, min(ti + NB + 1, last));
      if constexpr (NB == 3) {
        compute_tile(it, kb2, vb2, ti + 2, std::false_type{});
        load_tile(kb2, vb2, my_blk, nblk, kvh, min(ti + NB + 2, last));
      }
    }

    // ---- one step for each of the items ahead
    int b_blk, b_seq;
    load_lane_meta(b0, b1, b_blk, b_seq);
    const int tc = resolve_ticket(round + 3);
    int4 c0, c1;
    int ckvh;
    load_record(tc, c0, c1, ckvh);
    issue_ticket(round + 4);
    load_q(nq, a_seq, a1.x, akvh);
    load_scales(akvh, next_k_scale, next_v_scale);

    // ---- the last group: refills come from the next item (of a ticket past the end: from
    // the last record of the list, loads nobody uses)
    const int ti = NB * (ngroups - 1);
    if (ti < nfull)
      compute_tile(it, kb0, vb0, ti, std::false_type{});
    else
      compute_tile(it, kb0, vb0, ti, std::true_type{});
    load_tile(kb0, vb0, a_blk, a_nblk, akvh, a_t0);
    if (ti + 1 < nfull)
      compute_tile(it, kb1, vb1, ti + 1, std::false_type{});
    else if (ti + 1 <= last)
      compute_tile(it, kb1, vb1, ti + 1, std::true_type{});

    if constexpr (NB == 3) {
      load_tile(kb1, vb1, a_blk, a_nblk, akvh, a_t1);
      if (ti + 2 < nfull)
        compute_tile(it, kb2, vb2, ti + 2, std::false_type{});
      else if (ti + 2 <= last)
        compute_tile(it, kb2, vb2, ti + 2, std::true_type{});
    }

    // Write the partial (before the last refill: stores count as outstanding memory
    // operations too, and behind the refill they would be waited for together with it).
    write_partial(it, prow, mcnt * G, 0);
    if constexpr (NB == 3)
      load_tile(kb2, vb2, a_blk, a_nblk, akvh, min(a_t0 + 2, a_last));
    else
      load_tile(kb1, vb1, a_blk, a_nblk, akvh, a_t1);

    // ---- move on
    if (ta >= ntickets) break;
#pragma unroll
    for (int i = 0; i < KS; ++i) qreg[i] = nq[i];
    k_scale = next_k_scale, v_scale = next_v_scale;
    r0 = a0, r1 = a1, kvh = akvh, my_blk = a_blk, seq = a_seq;
    a0 = b0, a1 = b1, akvh = bkvh, a_blk = b_blk, a_seq = b_seq;
    b0 = c0, b1 = c1, bkvh = ckvh;
    t_cur = ta;
    ta = tb;
    tb = tc;
    if constexpr (COOP) {
      if (t_cur < coop) {
        to_pair_item = true;
        break;
      }
    }
  }

  // ---- the item shared with the other wave of the pair, the last one of both.  Groups of
  // tiles are claimed from a counter of the pair: bits 0-9 count the claims from the front,
  // bits 10-19 those from the back; the first two groups at either end are granted without a
  // claim.  A claim is good while the counts do not meet.  A wave that is through replaces its
  // own count by a marker (+2^20 from the front, -2^20 from the back) that makes every later
  // claim of the other wave fail, so that after both the counter is zero again for the next
  // launch.  Claims run two groups ahead of the arithmetic, refills one group ahead, so a claim
  // has a whole group of tiles to come back.  An item of fewer than four groups is attended by
  // its front wave alone.
  if (COOP && to_pair_item) {
    Item it;
    begin_item(it);
    const int tok_len = it.tok_len, sees = it.sees;
    const int mcnt = __builtin_amdgcn_readfirstlane(r1.x);
    const int ord = __builtin_amdgcn_readfirstlane(r1.y);
    const int nblk = (tok_len + kBlock - 1) / kBlock;
    const int ntiles = (tok_len + kTile - 1) / kTile;
    const int nfull = (tok_len - (sees > 0 ? 1 : 0)) / kTile;
    const int last = ntiles - 1;
    const int ngroups = NB == 2 ? (ntiles + 1) >> 1 : (ntiles + NB - 1) / NB;
    const bool shared_item = ngroups >= kCoopMinPairs;
    if (shared_item || !coop_back) {
      const bool from_back = shared_item && coop_back;
      const int64_t front_row = NB == 3 ? ((int64_t)seq * p.max_partials + ord) * p.num_q_heads + (int64_t)q_head_of(kvh)
                                        : ((int64_t)seq * p.max_partials + ord) * p.num_q_heads + kvh * G + row_head;
      const int64_t back_row = p.coop_row0 + (int64_t)pair_id * 32 + m;
      const int64_t prow = row_member < mcnt ? (from_back ? back_row : front_row) : -1;
      // the front partial says where the back partial of the same query row is
      const int tag = shared_item && !coop_back ? ((pair_id + 1) << 5) | m : 0;
      const int inc = shared_item ? (coop_back ? 1 << 10 : 1) : 0;
      int* ctr = p.coop_ctr + pair_id;
      int added = 0, claim_v = 0;
      auto issue_claim = [&](int by) {
        if (lane == 0) claim_v = atomicAdd(ctr + opaque_zero, by);
        added += by;
      };
      // the group of tiles after `cur`, or -1 when there is none left for this wave
      auto next_pair = [&](int cur) -> int {
        if (!shared_item) return cur + 1 < ngroups ? cur + 1 : -1;
        const int old = __builtin_amdgcn_readfirstlane(claim_v);
        const int f = old & 1023, b = (old >> 10) & 1023;
        if ((old >> 20) != 0 || 4 + f + b >= ngroups) return -1;
        return coop_back ? ngroups - 3 - b : 2 + f;
      };
      auto compute_any = [&](const KT& kt, const VT& vt, int ti) {
        if (ti > last) return;
        if (ti < nfull)
          compute_tile(it, kt, vt, ti, std::false_type{});
        else
          compute_tile(it, kt, vt, ti, std::true_type{});
      };
      int cur = from_back ? ngroups - 1 : 0;
      int nxt = from_back ? ngroups - 2 : (ngroups > 1 ? 1 : -1);  // granted
      issue_claim(inc);
      for (;;) {
        const int refill = nxt >= 0 ? nxt : cur;  // (past the end: loads nobody uses, as above)
        compute_any(kb0, vb0, NB * cur);
        load_tile(kb0, vb0, my_blk, nblk, kvh, NB * refill);
        compute_any(kb1, vb1, NB * cur + 1);
        load_tile(kb1, vb1, my_blk, nblk, kvh, min(NB * refill + 1, last));
        if constexpr (NB == 3) {
          compute_any(kb2, vb2, NB * cur + 2);
          load_tile(kb2, vb2, my_blk, nblk, kvh, min(NB * refill + 2, last));
        }
        if (nxt < 0) break;
        cur = nxt;
        nxt = next_pair(cur);
        issue_claim(nxt >= 0 ? inc : 0);
      }
      write_partial(it, prow, mcnt * G, tag);
      if (shared_item && lane == 0) atomicAdd(ctr, (coop_back ? -(1 << 20) : (1 << 20)) - added);
    }
  }
  // loads nobody uses are still in flight: let them land before the wave ends
  __builtin_amdgcn_s_waitcnt(0);
}

hipError_t launch_attend32(const AttendParams& p, const fca_plan& plan, int kv_dtype, int tile_buffers, int grid, hipStream_t stream) {
  const bool fp8 = kv_dtype == FCA_FP8_E4M3;
  // With sharing on, a launch reads every KV block once: stream it past the caches.  With
  // sharing off, sequences of a group read the same blocks again and again and the
  // memory-side cache serves the repeats, so the loads stay ordinary; likewise when query
  // runs make successive tiles of a sequence read the same blocks.
  const bool stream_kv = plan.max_levels > 0 && !p.kv_reread;
  hipEvent_t ev_start, ev_stop;
  take_attend_timing(&ev_start, &ev_stop);
#define FCA_LAUNCH(D_, F_, S_, N_) \
  if (ev_start) hipExtLaunchKernelGGL((fca_attend32_kernel<D_, F_, S_, N_>), dim3(grid), dim3(kThreads), 0, stream, ev_start, ev_stop, 0, p); \
  else hipLaunchKernelGGL((fca_attend32_kernel<D_, F_, S_, N_>), dim3(grid), dim3(kThreads), 0, stream, p)
#define FCA_PICK(D_, F_, N_) \
  if (stream_kv) { FCA_LAUNCH(D_, F_, true, N_); } else { FCA_LAUNCH(D_, F_, false, N_); }
  if (tile_buffers == 3) {  // fp8 at head size 128 only (checked with the tensors)
    FCA_PICK(128, true, 3);
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

