// Forest metadata builder: one workgroup turns (block_table, seq_lens) into shared
// nodes, member lists and a size-ordered work list, with no host round trip.
//
// Discovery is a level-by-level radix-tree construction.  At each level every still
// active sequence is keyed by (parent node, physical block id at its current position);
// sequences with equal keys elect the smallest index as leader, compare their rows
// against the leader's to find the common run, and the minimum run over the group
// becomes a shared node.  Members advance past the node and the next level regroups
// them; sequences left alone become private leaves.  Grouping semantics (compare with
// the group's first member, members ascending) follow the trainer's host-side discovery,
// arctic_platform/rl/zorro_train/zorro_train.py:242-285.
//
// Query rows need not be one per block-table row: with a row table, several rows (the
// tokens of a query run) read one table row up to different lengths.  The caller may
// declare groups among them.  Declared rows take part in discovery like any other row,
// except that their last block (the one their own token is in) is never shared there and
// that a group of nothing but declared rows of one table row is left alone.  After
// discovery the declared rows meet once more under (node they ended in, group id): a group
// that is a tile of a query run becomes a causal node from there to its last token, any
// other declared group a plain node over what its members have in common.  This is how a
// run is cut into tiles that each read their private KV once, below whatever its sequence
// shares with others.
//
// Between two scheduler steps of a decode loop only the lengths change: every sequence
// grows by a token and now and then takes a new private block.  The forest is a function
// of the shared blocks alone, so an update keeps it as long as every row still carries
// the blocks its shared nodes were built from (a 64-bit fingerprint per row, taken at
// build time, is compared) and those blocks are still full blocks of the row; only the
// leaves and the work list are made again.  Any mismatch falls back to the full build in
// the same launch, so an update is always safe to ask for.
#include "fca_common.h"

namespace fca {

constexpr int kBuildThreads = 1024;
constexpr unsigned long long kEmptyKey = ~0ull;

// Exclusive prefix sum of in[0..n) into out[0..n) by the whole workgroup; returns the
// total to every thread.  `in` may alias `out`.  Every thread sums a contiguous slice,
// the slice sums are scanned inside each wave with lane shuffles and across the sixteen
// waves through LDS: three barriers in all.
__device__ int block_exclusive_scan(const int* in, int* out, int n, int* lds) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per = (n + kBuildThreads - 1) / kBuildThreads;
  const int lo = min(tid * per, n), hi = min(lo + per, n);
  int sum = 0;
  for (int i = lo; i < hi; ++i) sum += in[i];
  int incl = sum;  // inclusive scan over the lanes of the wave
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int v = __shfl_up(incl, off);
    if (lane >= off) incl += v;
  }
  if (lane == 63) lds[wave] = incl;
  __syncthreads();
  int wave_base = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kBuildThreads / 64; ++w) {
    const int v = lds[w];
    if (w < wave) wave_base += v;
    total += v;
  }
  __syncthreads();  // lds is reused by the next call
  int run = wave_base + incl - sum;
  for (int i = lo; i < hi; ++i) {
    const int v = in[i];
    out[i] = run;
    run += v;
  }
  __syncthreads();
  return total;
}

__device__ inline unsigned hash_key(unsigned long long k) {
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdull;
  k ^= k >> 29;
  return (unsigned)k;
}

__device__ inline unsigned long long mix64(unsigned long long k) {
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdull;
  k ^= k >> 33;
  k *= 0xc4ceb9fe1a85ec53ull;
  k ^= k >> 33;
  return k;
}

// Lanes that work on one row together (row comparison, fingerprints).
constexpr int kRowLanes = 8;

// Fingerprint of the first n block ids of a row, computed by a group of kRowLanes lanes
// (every lane returns it): the sum over positions j of (id_j ^ c) * w_j in 64 bits, with an
// odd 32-bit weight per position.  A change of one id moves the sum by a non-zero multiple
// of an odd number, an exchange of two ids by a product of two non-zero numbers below 2^32:
// neither can be zero modulo 2^64.  One multiply-add per element.  A 16-byte aligned row is
// read four ids per load, eight loads in flight per lane (256 positions per round trip of
// the group); loads past the end are clamped and not counted.
__device__ inline unsigned long long row_fingerprint(const int32_t* row, int n, int glane) {
  unsigned long long acc = 0;
  constexpr int kUnroll = 8;
  auto term = [](int id, unsigned j) {
    return (unsigned long long)((unsigned)id ^ 0xa5a5a5a5u) * ((j * 0x9e3779b1u) | 1u);
  };
  int done = 0;  // positions covered by the vector part
  if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int4* row4 = reinterpret_cast<const int4*>(row);
    const int nv = n >> 2;
    for (int j0 = 0; j0 < nv; j0 += kRowLanes * kUnroll) {
      int4 v[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) v[u] = row4[min(j0 + u * kRowLanes + glane, nv - 1)];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int j = j0 + u * kRowLanes + glane;
        if (j < nv)
          acc += term(v[u].x, 4u * j) + term(v[u].y, 4u * j + 1) + term(v[u].z, 4u * j + 2) + term(v[u].w, 4u * j + 3);
      }
    }
    done = nv << 2;
  }
  for (int j0 = done; j0 < n; j0 += kRowLanes * kUnroll) {
    int v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) v[u] = row[min(j0 + u * kRowLanes + glane, n - 1)];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int j = j0 + u * kRowLanes + glane;
      if (j < n) acc += term(v[u], (unsigned)j);
    }
  }
  for (int off = kRowLanes / 2; off; off >>= 1) acc += __shfl_xor(acc, off, kRowLanes);
  return acc;
}

// First position below lim at which two rows differ (lim if none), found by a group of
// kRowLanes lanes; every lane returns it.  Where both rows are 16-byte aligned together
// they are compared four ids per load, eight loads per row in flight per lane (256
// positions per round trip of the group), and the scan stops at the first round that holds
// a difference.
__device__ inline int first_difference(const int32_t* a, const int32_t* b, int lim, int glane) {
  constexpr int kUnroll = 8;
  auto group_min = [](int v) {
    for (int off = kRowLanes / 2; off; off >>= 1) v = min(v, __shfl_xor(v, off, kRowLanes));
    return v;
  };
  // scalar compare of [lo, hi): a few positions at the ends, or everything for rows that
  // never reach a 16-byte boundary together
  auto scalar_part = [&](int lo, int hi) {
    int first = lim;
    for (int j0 = lo; j0 < hi && first == lim; j0 += kRowLanes * kUnroll) {
      int mine = lim;
#pragma unroll
      for (int u = kUnroll - 1; u >= 0; --u) {
        const int j = j0 + u * kRowLanes + glane;
        if (j < hi && a[j] != b[j]) mine = j;
      }
      first = group_min(mine);
    }
    return first;
  };
  const uintptr_t ua = reinterpret_cast<uintptr_t>(a), ub = reinterpret_cast<uintptr_t>(b);
  if ((ua & 15) != (ub & 15)) return scalar_part(0, lim);
  const int head = min(lim, (int)(((16 - (ua & 15)) & 15) >> 2));  // positions before the boundary
  int first = scalar_part(0, head);
  if (first != lim) return first;
  const int4* a4 = reinterpret_cast<const int4*>(a + head);
  const int4* b4 = reinterpret_cast<const int4*>(b + head);
  const int nv = (lim - head) >> 2;
  for (int j0 = 0; j0 < nv && first == lim; j0 += kRowLanes * kUnroll) {
    int mine = lim;
#pragma unroll
    for (int u = kUnroll - 1; u >= 0; --u) {
      const int j = j0 + u * kRowLanes + glane;
      if (j < nv) {
        const int4 x = a4[j], y = b4[j];
        const int at = head + 4 * j;
        if (x.w != y.w) mine = at + 3;
        if (x.z != y.z) mine = at + 2;
        if (x.y != y.y) mine = at + 1;
        if (x.x != y.x) mine = at;
      }
    }
    first = group_min(mine);
  }
  if (first != lim) return first;
  return scalar_part(head + 4 * nv, lim);
}

__device__ inline int plan_fingerprint(const fca_plan& pl) {
  unsigned long long k = mix64(((unsigned long long)(unsigned)pl.num_seqs << 32) | (unsigned)pl.max_blocks);
  k = mix64(k ^ (((unsigned long long)(unsigned)pl.num_q_heads << 32) | (unsigned)pl.num_kv_heads));
  k = mix64(k ^ (((unsigned long long)(unsigned)pl.chunk_tokens << 32) | (unsigned)pl.rows_per_item));
  k = mix64(k ^ (unsigned)pl.max_levels);
  return (int)(k & 0x7fffffff);
}

// Runs of equal keys over the adjacent lanes of a wave (adjacent lanes hold adjacent rows,
// and the rows of a group usually are adjacent): the lane a lane's run starts at.  One lane
// per run then speaks for all of them, which turns up to 64 atomics on one address into
// one.  Every lane of the wave must call this.
__device__ inline int run_head_lane(unsigned long long key, int lane) {
  const unsigned long long prev = __shfl_up(key, 1);
  const unsigned long long heads = __ballot(lane == 0 || prev != key);
  return 63 - __clzll((long long)(heads & ((2ull << lane) - 1)));
}

__global__ __launch_bounds__(kBuildThreads) void fca_build_kernel(BuildParams p) {
  __shared__ int lds_scan[kBuildThreads];
  __shared__ int lds_mismatch;
  __shared__ int lds_stale;  // the workspace holds no build of this plan (written before a barrier, read after it)
  __shared__ int lds_any;
  __shared__ int lds_listed;
  __shared__ int lds_hist[2 * kSizeBuckets];
  __shared__ int lds_cursor[2 * kSizeBuckets];
  __shared__ unsigned long long lds_tokens;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int S = p.plan.num_seqs;
  const int chunk = p.plan.chunk_tokens;
  const int group = p.plan.num_q_heads / p.plan.num_kv_heads;
  const int members_per_item = p.plan.rows_per_item / group;
  const MetaLayout& L = p.L;
  int32_t* meta = p.meta;
  int32_t* hdr = meta + L.header;
  int* pos = meta + L.s_pos;
  int* par = meta + L.s_par;
  int* ord = meta + L.s_ord;
  int* nfull = meta + L.s_nfull;
  int* leader = meta + L.s_leader;
  int* lcp = meta + L.s_lcp;
  int* run = meta + L.s_run;
  int* cnt = meta + L.s_cnt;
  int* nodeof = meta + L.s_node;
  int* slot = meta + L.s_slot;
  int* tmp0 = meta + L.s_tmp0;
  int* tmp1 = meta + L.s_tmp1;
  int* cbad = meta + L.s_nitems;  // per leader, raised by members: in discovery, the group is more than one query run;
                                  // in the pass for declared groups, the group is no tile of a query run
  int* cmax = cbad + S;           // per leader: largest member row minus the leader's row
  unsigned long long* hkeys = reinterpret_cast<unsigned long long*>(meta + L.hash_keys);
  int* hmin = meta + L.hash_min;
  const int hsize = (int)L.hash_size;
  int* members = meta + L.members;
  unsigned long long* sig = reinterpret_cast<unsigned long long*>(meta + L.s_sig);
  const int plan_sig = plan_fingerprint(p.plan);
  // block-table row of query row s
  auto table_row = [&](int s) -> int64_t {
    if (!p.row_table) return s;
    const int r = p.row_table[s];
    return r >= 0 && r < p.table_rows ? r : 0;  // (out of range: flagged by the full build)
  };
  // Rows the caller has grouped.  The common run of a declared group ends before the block
  // that holds the last token of its shortest row.  If the members are successive rows
  // reading one table row, each one token longer than the one before it, with their last
  // tokens in one block (a tile of a query run), the node takes that block in as well and
  // is marked causal: its last chunk tells the attention kernel how many of its tokens the
  // first member sees, and the kernel hides from every row the tokens behind its own.
  // Such members have no leaf.  Any other declared group keeps a private leaf per member
  // from that block on.
  auto declared = [&](int s) { return p.row_group && p.row_group[s] >= 0; };

  // claim counters of the attention kernel: zero before the first launch on this workspace
  // (every launch leaves them at zero again)
  for (int i = tid; i < kCoopMaxPairs; i += kBuildThreads) meta[L.coop_ctr + i] = 0;

  // ---- update: is the forest of the last build on this workspace still the forest of
  // these rows?  (pos = first private block of a row, ord = chunks of its shared nodes:
  // both are left in the workspace by the build.)
  bool reuse = false;
  if (p.try_update) {
    if (tid == 0) {
      lds_stale = (hdr[H_BUILT] != kBuiltMagic || hdr[H_PLAN_SIG] != plan_sig) ? 1 : 0;
      lds_mismatch = 0;
    }
    __syncthreads();
    // (a word of its own: lds_mismatch is raised inside the loop below, and a wave that looked at
    // it to decide whether to enter the loop would race with the waves already in it)
    if (!lds_stale) {
      const int gid = tid / kRowLanes, glane = tid % kRowLanes;
      for (int s = gid; s < S; s += kBuildThreads / kRowLanes) {
        const int len = p.seq_lens[s];
        const int shared_blocks = pos[s];
        // (a sequence that got shorter is a new request in an old slot: build anew, it may
        // share more than its predecessor did)
        bool ok = len >= tmp1[s] && len <= p.plan.max_blocks * kBlock && len / kBlock >= shared_blocks;
        if (ok) ok = row_fingerprint(p.block_table + table_row(s) * p.bt_stride, shared_blocks, glane) == sig[s];
        if (!ok && glane == 0) lds_mismatch = 1;
      }
    }
    __syncthreads();
    reuse = !lds_stale && !lds_mismatch;
  }

  int node_base = 0, member_base = 0, levels = 0;
  if (reuse) {
    node_base = hdr[H_NODES];
    member_base = hdr[H_LEAF_MEMBERS];
    levels = hdr[H_LEVELS];
    const int updates = hdr[H_UPDATES];
    const unsigned long long shared_tokens =
        (unsigned long long)(unsigned)hdr[H_SHARED_TOK_LO] | ((unsigned long long)(unsigned)hdr[H_SHARED_TOK_HI] << 32);
    __syncthreads();
    if (tid == 0) {
      lds_tokens = shared_tokens;
      hdr[H_ERROR] = 0;
      hdr[H_TICKET] = 0;
      hdr[H_UPDATES] = updates + 1;
    }
    for (int s = tid; s < S; s += kBuildThreads) tmp1[s] = p.seq_lens[s];
    __syncthreads();
  } else {
    if (tid < kHeaderInts) hdr[tid] = 0;
    if (tid == 0) lds_tokens = 0;
    // (the error flags set below must not be overtaken by the clearing of the header: other
    // waves would otherwise be free to flag a bad length before wave 0 has cleared the word)
    __syncthreads();
    for (int s = tid; s < S; s += kBuildThreads) {
      int len = p.seq_lens[s];
      if (len < 0 || len > p.plan.max_blocks * kBlock) {
        atomicOr(&hdr[H_ERROR], 1);
        len = max(0, min(len, p.plan.max_blocks * kBlock));
      }
      if (p.row_table && (p.row_table[s] < 0 || p.row_table[s] >= p.table_rows)) atomicOr(&hdr[H_ERROR], 4);
      tmp1[s] = len;  // validated length, kept for the leaf pass
      nfull[s] = p.plan.max_levels > 0 ? (declared(s) ? max(len - 1, 0) / kBlock : len / kBlock) : 0;
      pos[s] = 0;
      par[s] = -1;
      ord[s] = 0;
    }
    __syncthreads();

    // Discovery level by level; then, if the caller has declared groups, one more pass in
    // which the declared rows meet under (node they ended in, group id).  A row that drops
    // out of discovery keeps its parent in par as -(parent + 3), so -2 stands for "none".
    const bool have_groups = p.row_group != nullptr && p.plan.max_levels > 0;
    auto parent_of = [&](int s) { return par[s] <= -2 ? -par[s] - 3 : par[s]; };
    bool group_pass = false;
    for (int level = 0;; ++level) {
      if (!group_pass && level >= p.plan.max_levels) {
        if (!have_groups) break;
        group_pass = true;
      }
      if (tid == 0) lds_any = 0;
      for (int i = tid; i < hsize; i += kBuildThreads) {
        hkeys[i] = kEmptyKey;
        hmin[i] = 0x7fffffff;
      }
      for (int s = tid; s < S; s += kBuildThreads) {
        run[s] = 0x7fffffff;
        cnt[s] = 0;
        leader[s] = -1;
        slot[s] = -1;
        cbad[s] = 0;
        cmax[s] = 0;
      }
      __syncthreads();
      // Key every sequence that still has a full block at its position and has not dropped
      // out of sharing at an earlier level: rows meet under (parent node, physical block id
      // at the current position).  In the pass for declared groups: every declared row.
      // The first lane of every run of equal keys in a wave enters the key and its own row,
      // the smallest of the run, for all of them.
      for (int base = 0; base < S; base += kBuildThreads) {
        const int s = base + tid;
        const bool keyed =
            s < S && !(group_pass ? !declared(s) || tmp1[s] < 1 : par[s] <= -2 || pos[s] >= nfull[s]);
        unsigned long long key = kEmptyKey - 1 - (unsigned)lane;  // no key: a run of its own
        if (keyed) {
          if (group_pass) {
            key = (1ull << 63) | ((unsigned long long)(unsigned)(parent_of(s) + 1) << 32) | (unsigned)p.row_group[s];
          } else {
            const unsigned blk = (unsigned)p.block_table[table_row(s) * p.bt_stride + pos[s]];
            key = ((unsigned long long)(unsigned)(par[s] + 1) << 32) | blk;
          }
        }
        const int head = run_head_lane(key, lane);
        int h = -1;
        if (keyed && head == lane) {
          h = hash_key(key) & (hsize - 1);
          for (int probe = 0; probe < hsize; ++probe) {
            unsigned long long prev = atomicCAS(&hkeys[h], kEmptyKey, key);
            if (prev == kEmptyKey || prev == key) break;
            h = (h + 1) & (hsize - 1);
          }
          atomicMin(&hmin[h], s);
        }
        h = __shfl(h, head);
        if (keyed) slot[s] = h;
      }
      __syncthreads();
      for (int s = tid; s < S; s += kBuildThreads) {
        if (slot[s] >= 0) {
          leader[s] = hmin[slot[s]];
          lcp[s] = nfull[s] - pos[s];
          if (leader[s] != s) lds_any = 1;  // somebody follows a leader: a group of two or more
        }
      }
      __syncthreads();
      if (!lds_any) {  // every key is alone: no shared node at this level or below
        if (group_pass || !have_groups) break;
        group_pass = true;
        continue;
      }
      // Common run with the leader = first position where the two rows differ.  Followers
      // that read the leader's own table row (query rows of one sequence) have nothing to
      // compare; the others are listed (in a scratch array that is free here) and every group of
      // kRowLanes lanes takes one listed sequence at a time (128 in flight per pass).
      if (tid == 0) lds_listed = 0;
      __syncthreads();
      for (int s = tid; s < S; s += kBuildThreads) {
        const int t = leader[s];
        if (t < 0 || t == s) continue;
        if (table_row(s) == table_row(t))
          lcp[s] = min(lcp[s], min(nfull[s], nfull[t]) - pos[s]);
        else
          tmp0[atomicAdd(&lds_listed, 1)] = s;
      }
      __syncthreads();
      {
        const int gid = tid / kRowLanes, glane = tid % kRowLanes;
        const int listed = lds_listed;
        for (int i = gid; i < listed; i += kBuildThreads / kRowLanes) {
          const int s = tmp0[i], t = leader[s];
          const int lim = min(nfull[s], nfull[t]) - pos[s];
          const int32_t* row_s = p.block_table + table_row(s) * p.bt_stride + pos[s];
          const int32_t* row_t = p.block_table + table_row(t) * p.bt_stride + pos[s];
          const int first = first_difference(row_s, row_t, lim, glane);
          if (glane == 0) lcp[s] = min(lcp[s], first);
        }
      }
      __syncthreads();
      // Per leader: the shortest common run, the member count, the largest distance of a
      // member's row from the leader's, and a flag (below).  The last lane of every run of
      // equal leaders in a wave reports for the run.
      for (int base = 0; base < S; base += kBuildThreads) {
        const int s = base + tid;
        const int t = s < S ? leader[s] : -1;
        int shortest = 0x7fffffff, flag = 0;
        if (t >= 0) {
          shortest = lcp[s];
          if (group_pass) {
            // does the group look like a tile of a query run?
            flag = !(table_row(s) == table_row(t) && tmp1[s] == tmp1[t] + (s - t) &&
                     (tmp1[s] - 1) / kBlock == (tmp1[t] - 1) / kBlock);
          } else if (have_groups) {
            // does the group hold anything but declared rows of the leader's table row?
            flag = !declared(s) || table_row(s) != table_row(t);
          }
        }
        const unsigned long long key = t >= 0 ? (unsigned long long)(unsigned)t : kEmptyKey - 1 - (unsigned)lane;
        const int head = run_head_lane(key, lane);
        for (int off = 1; off < 64; off <<= 1) {  // minimum and flag from the run's first lane up to this one
          const int other_shortest = __shfl_up(shortest, off), other_flag = __shfl_up(flag, off);
          if (lane - off >= head) {
            shortest = min(shortest, other_shortest);
            flag |= other_flag;
          }
        }
        const int next_head = __shfl_down(head, 1);
        if (t >= 0 && (lane == 63 || next_head != head)) {
          atomicMin(&run[t], shortest);
          atomicAdd(&cnt[t], lane - head + 1);
          atomicMax(&cmax[t], s - t);
          if (flag) atomicOr(&cbad[t], 1);
        }
      }
      __syncthreads();
      // Which leaders make a node (kept in `slot`, which is free by now: 0 none, 1 plain, 2
      // causal).  Discovery leaves a group alone that is nothing but declared rows of one
      // table row, i.e. the rows of one query run: the pass for declared groups tiles them.
      // There, a group whose members are rows s, s + 1, ... without a gap, each one token
      // longer and all ending in one block, is such a tile and becomes a causal node.
      for (int s = tid; s < S; s += kBuildThreads) {
        int kind = 0;
        if (leader[s] == s && cnt[s] >= 2) {
          if (group_pass)
            kind = !cbad[s] && cmax[s] + 1 == cnt[s] ? 2 : (run[s] > 0 ? 1 : 0);
          else
            kind = !have_groups || cbad[s] ? 1 : 0;
        }
        if (leader[s] == s) slot[s] = kind;
        tmp0[s] = kind ? 1 : 0;
        nodeof[s] = kind ? cnt[s] : 0;
      }
      __syncthreads();
      const int new_nodes = block_exclusive_scan(tmp0, tmp0, S, lds_scan);
      if (new_nodes == 0) {
        if (group_pass || !have_groups) break;
        group_pass = true;
        continue;
      }
      const int new_members = block_exclusive_scan(nodeof, nodeof, S, lds_scan);
      ++levels;
      for (int s = tid; s < S; s += kBuildThreads) {
        if (leader[s] == s && slot[s]) {
          const int id = node_base + tmp0[s];
          // a causal node runs from the group's position to the last member's last token
          const bool causal = slot[s] == 2;
          const int ntok = causal ? tmp1[s] + cnt[s] - 1 - pos[s] * kBlock : run[s] * kBlock;
          meta[L.node_rep + id] = s;
          meta[L.node_blk + id] = pos[s];
          meta[L.node_nblk + id] = run[s] + (causal ? 1 : 0);
          meta[L.node_tok + id] = ntok;
          meta[L.node_causal + id] = causal ? 1 : 0;
          meta[L.node_level + id] = level;
          meta[L.node_moff + id] = member_base + nodeof[s];
          meta[L.node_mcnt + id] = cnt[s];
          meta[L.node_ord + id] = ord[s];
          tmp0[s] = id;
          atomicAdd(&lds_tokens, (unsigned long long)ntok);
        }
      }
      __syncthreads();
      // Member lists in ascending sequence order: rank = members of the same leader below s.
      // Where the members are not adjacent rows, one thread per sequence scans [leader, s).
      for (int s = tid; s < S; s += kBuildThreads) {
        const int t = leader[s];
        if (t < 0 || !slot[t]) continue;
        int below = s - t;  // members in adjacent rows (the usual case): the distance is the rank
        if (cmax[t] + 1 != cnt[t]) {
          below = 0;
          for (int j = t; j < s; ++j) below += leader[j] == t ? 1 : 0;
        }
        members[meta[L.node_moff + tmp0[t]] + below] = s;
      }
      __syncthreads();
      for (int s = tid; s < S; s += kBuildThreads) {
        const int t = leader[s];
        if (t >= 0 && slot[t]) {
          lcp[s] = 1;  // advances past the node, after the barrier (pos[t] is read by others)
          par[s] = tmp0[t];
        } else {
          lcp[s] = 0;
          if (par[s] > -2) par[s] = -(par[s] + 3);  // out of discovery from here on
        }
      }
      __syncthreads();
      for (int s = tid; s < S; s += kBuildThreads) {
        if (!lcp[s]) continue;
        pos[s] += meta[L.node_nblk + par[s]];
        ord[s] += num_chunks_for(meta[L.node_tok + par[s]], chunk);
      }
      node_base += new_nodes;
      member_base += new_members;
      __syncthreads();
      if (group_pass) break;
    }
    // What a later update starts from: fingerprints of the shared part of every row and
    // the totals of the shared nodes.  With declared groups there is nothing to keep: the
    // rows of a query run move on with every step, so the workspace stays marked as not
    // built and an update on it is a full build.
    if (!p.row_group) {
      const int gid = tid / kRowLanes, glane = tid % kRowLanes;
      for (int s = gid; s < S; s += kBuildThreads / kRowLanes) {
        const unsigned long long f = row_fingerprint(p.block_table + table_row(s) * p.bt_stride, pos[s], glane);
        if (glane == 0) sig[s] = f;
      }
      if (tid == 0) {
        hdr[H_LEAF_MEMBERS] = member_base;
        hdr[H_SHARED_TOK_LO] = (int)(lds_tokens & 0xffffffffull);
        hdr[H_SHARED_TOK_HI] = (int)(lds_tokens >> 32);
        hdr[H_PLAN_SIG] = plan_sig;
        hdr[H_BUILT] = kBuiltMagic;
      }
    }
  }  // full build
  __syncthreads();

  // Private leaves and per-sequence partial counts.  Node index space for the work list:
  // shared nodes [0, node_base), then leaf of sequence s at node_base + s.
  const int leaf_members = member_base;
  {
    unsigned long long leaf_tokens = 0;
    for (int s = tid; s < S; s += kBuildThreads) {
      const int tokens = max(0, tmp1[s] - pos[s] * kBlock);  // (none below a causal node)
      meta[L.seq_leaf_blk + s] = pos[s];
      const int npart = ord[s] + num_chunks_for(tokens, chunk);
      meta[L.seq_npart + s] = npart;
      if (npart > (int)L.max_partials) atomicOr(&hdr[H_ERROR], 8);  // (cannot happen: see make_layout)
      members[leaf_members + s] = s;
      leaf_tokens += (unsigned long long)tokens;
    }
    // one atomic per wave
    for (int off = 32; off; off >>= 1) leaf_tokens += __shfl_xor(leaf_tokens, off);
    if ((tid & 63) == 0 && leaf_tokens) atomicAdd(&lds_tokens, leaf_tokens);
  }
  if (tid < 2 * kSizeBuckets) {
    lds_hist[tid] = 0;
    lds_cursor[tid] = 0;
  }
  __syncthreads();

  // Work list: one item per (node chunk, tile of members), shared items first, each
  // class in descending size order: the attention kernel deals the list to its waves in
  // alternating directions, which balances a descending list well.
  const int total_nodes = node_base + S;
  // first_len: length of the first member of a causal node, 0 for any other node
  auto node_fields = [&](int n, int& rep, int& blk, int& tokens, int& moff, int& mcnt, int& o, int& first_len) {
    first_len = 0;
    // (rep is what the attention kernels index the block table with)
    if (n < node_base) {
      rep = (int)table_row(meta[L.node_rep + n]);
      blk = meta[L.node_blk + n];
      tokens = meta[L.node_tok + n];
      if (meta[L.node_causal + n]) first_len = tmp1[meta[L.node_rep + n]] - blk * kBlock;
      moff = meta[L.node_moff + n];
      mcnt = meta[L.node_mcnt + n];
      o = meta[L.node_ord + n];
    } else {
      const int s = n - node_base;
      rep = (int)table_row(s);
      blk = pos[s];
      tokens = max(0, tmp1[s] - pos[s] * kBlock);
      moff = leaf_members + s;
      mcnt = 1;
      o = ord[s];
    }
  };
  auto bucket_of = [&](int cls, int tok_len) {
    int sb = min(kSizeBuckets - 1, (tok_len * kSizeBuckets - 1) / chunk);
    return cls * kSizeBuckets + (kSizeBuckets - 1 - sb);
  };
  for (int n = tid; n < total_nodes; n += kBuildThreads) {
    int rep, blk, tokens, moff, mcnt, o, first_len;
    node_fields(n, rep, blk, tokens, moff, mcnt, o, first_len);
    const int clen = chunk_len_for(tokens, chunk);
    const int nch = num_chunks_for(tokens, chunk);
    const int ntile = (mcnt + members_per_item - 1) / members_per_item;
    const int cls = n < node_base ? 0 : 1;
    for (int c = 0; c < nch; ++c) {
      const int tl = min(clen, tokens - c * clen);
      atomicAdd(&lds_hist[bucket_of(cls, tl)], ntile);
    }
  }
  __syncthreads();
  if (tid == 0) {
    int acc = 0, shared_items = 0;
    for (int b = 0; b < 2 * kSizeBuckets; ++b) {
      if (b == kSizeBuckets) shared_items = acc;
      int v = lds_hist[b];
      lds_hist[b] = acc;
      acc += v;
    }
    hdr[H_ITEMS] = acc;
    hdr[H_SHARED_ITEMS] = shared_items;
    hdr[H_NODES] = node_base;
    hdr[H_LEVELS] = levels;
    hdr[H_TOKENS_LO] = (int)(lds_tokens & 0xffffffffull);
    hdr[H_TOKENS_HI] = (int)(lds_tokens >> 32);
    if (acc > (int)L.max_items) atomicOr(&hdr[H_ERROR], 2);
  }
  __syncthreads();
  int32_t* items = meta + L.items;
  for (int n = tid; n < total_nodes; n += kBuildThreads) {
    int rep, blk, tokens, moff, mcnt, o, first_len;
    node_fields(n, rep, blk, tokens, moff, mcnt, o, first_len);
    const int clen = chunk_len_for(tokens, chunk);
    const int nch = num_chunks_for(tokens, chunk);
    const int ntile = (mcnt + members_per_item - 1) / members_per_item;
    const int cls = n < node_base ? 0 : 1;
    for (int c = 0; c < nch; ++c) {
      const int tl = min(clen, tokens - c * clen);
      const int b = bucket_of(cls, tl);
      const int at = lds_hist[b] + atomicAdd(&lds_cursor[b], ntile);
      for (int r = 0; r < ntile; ++r) {
        if (at + r >= (int)L.max_items) break;
        int4* rec = reinterpret_cast<int4*>(items + (int64_t)(at + r) * kItemInts);
        // Last chunk of a causal node: tokens of the chunk the item's first member sees;
        // member i of the item sees i more.  Every member's own block lies in the last tile
        // of this chunk (chunks are whole tiles and a tile holds whole blocks).
        const int sees = first_len && c == nch - 1 ? first_len + r * members_per_item - c * clen : 0;
        rec[0] = make_int4(rep, blk + c * (clen / kBlock), tl, moff + r * members_per_item);
        rec[1] = make_int4(min(members_per_item, mcnt - r * members_per_item), o + c, n, sees);
      }
    }
  }
}

// Query rows of a step from the engine's per-request arrays: one thread per query token
// finds its request by bisection over the cumulative query lengths.
__global__ __launch_bounds__(256) void fca_rows_kernel(const int32_t* __restrict__ query_start_loc,
                                                       const int32_t* __restrict__ seq_lens, int num_reqs, int num_rows,
                                                       int max_blocks, int32_t* __restrict__ row_table,
                                                       int32_t* __restrict__ row_lens, int32_t* __restrict__ row_group) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= num_rows) return;
  int lo = 0, hi = num_reqs - 1;  // last request whose first token is at or before r
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (query_start_loc[mid] <= r) lo = mid; else hi = mid - 1;
  }
  const int first = query_start_loc[lo], end = query_start_loc[lo + 1];
  // the sequence length counts the whole run: this token sees all but the tokens after it
  const int len = seq_lens[lo] - (end - 1 - r);
  row_table[r] = lo;
  row_lens[r] = len;
  // a run of two or more tokens is tiled per cache block of the token
  row_group[r] = end - first > 1 ? lo * max_blocks + max(len - 1, 0) / kBlock : -1;
}

hipError_t launch_rows(const int32_t* query_start_loc, const int32_t* seq_lens, int num_reqs, int num_rows, int max_blocks,
                       int32_t* row_table, int32_t* row_lens, int32_t* row_group, hipStream_t stream) {
  hipLaunchKernelGGL(fca_rows_kernel, dim3((num_rows + 255) / 256), dim3(256), 0, stream, query_start_loc, seq_lens,
                     num_reqs, num_rows, max_blocks, row_table, row_lens, row_group);
  return hipGetLastError();
}

hipError_t launch_build(const BuildParams& p, hipStream_t stream) {
  hipLaunchKernelGGL(fca_build_kernel, dim3(1), dim3(kBuildThreads), 0, stream, p);
  return hipGetLastError();
}

}  // namespace fca
