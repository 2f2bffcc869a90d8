// CPU stand-in for the parts of HIP that the kernels of this library use, for tests without a GPU.
// A workgroup runs as cooperative fibers, one per thread, on one host thread; every cross-lane
// operation (shuffles, ballots, readfirstlane, MFMA, the wave barrier) and every workgroup barrier
// is a rendezvous of the lanes concerned; workgroups of a launch run one after the other, or, with
// emu::host_threads above 1, several at a time on host threads of their own (LDS is per host thread,
// atomics are the host's), which is how the workgroups of a persistent grid meet on a GPU.  What the
// kernels see of the GPU's data layouts (the operand and result registers of
// mfma_f32_32x32x16_bf16, v_permlane32_swap, the fp8 conversions, direct-to-LDS loads) follows
// the instruction set.  It checks kernel logic: indices, rings, masks, the dealing of work, and,
// with buffers placed against inaccessible pages by the caller, addresses.  It says nothing about
// speed, about the memory model between workgroups, or about what the compiler makes of the code.
// Test infrastructure only: nothing in the library includes it.
#pragma once
#include <sys/mman.h>
#include <ucontext.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <atomic>
#include <functional>
#include <thread>
#include <vector>

struct dim3 {
  unsigned x, y, z;
  dim3(unsigned a = 1, unsigned b = 1, unsigned c = 1) : x(a), y(b), z(c) {}
};
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0, hipErrorInvalidValue = 1;
typedef void* hipStream_t;
typedef void* hipEvent_t;
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emu"; }

#define __global__
#define __device__
#define __host__
#define __shared__ static thread_local
#define __launch_bounds__(...)

namespace emu {

constexpr int kStack = 512 * 1024;
struct WaveSync {
  int arrived = 0, active = 0;
  unsigned gen = 0;
  alignas(64) unsigned char stage[2][64][64];
};
// rendezvous of the lanes of one group of `width` lanes (shuffles with a width below 64 in code
// where the groups of a wave have gone different ways)
struct GroupSync {
  int arrived = 0;
  unsigned gen = 0;
};
struct DmaWrite {
  void* dst;
  unsigned char data[16];
  int bytes;
};
// a fiber's stack: mapped, not filled, so that only the pages a fiber touches cost anything
struct Stack {
  char* base = nullptr;
  Stack() {
    void* p = mmap(nullptr, kStack, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (p == MAP_FAILED) abort();
    base = static_cast<char*>(p);
  }
  Stack(const Stack&) = delete;
  Stack(Stack&& o) noexcept : base(o.base) { o.base = nullptr; }
  ~Stack() {
    if (base) munmap(base, kStack);
  }
  char* data() { return base; }
  size_t size() const { return kStack; }
};
struct Fiber {
  ucontext_t ctx;
  Stack stack;
  dim3 tid;
  int lane = 0, wave = 0;
  bool done = false;
  std::vector<DmaWrite> dma;  // direct-to-LDS loads issued and not yet landed (late mode)
};
struct Block {
  std::vector<Fiber> fibers;
  dim3 bid, gdim, bdim;
  std::vector<WaveSync> waves;
  std::vector<GroupSync> groups;  // [wave][log2 width][group]
  int b_arrived = 0, b_active = 0;
  unsigned b_gen = 0;
  ucontext_t sched;
  std::function<void()> body;
};
inline thread_local Block* B = nullptr;
inline thread_local Fiber* F = nullptr;
inline int host_threads = 1;  // workgroups of a launch that run at the same time
inline bool dma_late = false;  // direct-to-LDS loads land at the wait that covers them instead of at once
// Order in which the scheduler below takes what the hardware runs at the same time.  Bit 0: the waves of a
// workgroup from the last to the first in every round; bit 1: the workgroups of a launch from the last to the
// first; bit 2: the lanes of a wave from the last to the first between two rendezvous.  A kernel must not
// care: one that does relies on an order the hardware does not promise.
inline int run_order = 0;
inline std::atomic<unsigned long long> streamed_bytes{0};  // bytes requested by non-temporal loads (the kernels stream their KV tiles with them)
inline thread_local long n_progress = 0;  // rendezvous completed and fibers finished (deadlock detection)

inline void yield() {
  swapcontext(&F->ctx, &B->sched);
}

// Leave this lane's contribution and wait for the lanes of its group of `width`; returns the stage buffer.
// (The stage is the wave's: groups write disjoint entries; a group that runs ahead of the others
// could overwrite what a slower group still reads only if it lapped it twice, which the per-group
// generation count rules out for the entries of its own lanes.)
inline const unsigned char (*group_exchange(const void* mine, size_t n, int width))[64] {
  WaveSync& w = B->waves[F->wave];
  int lg = 0;
  while ((1 << lg) < width) ++lg;
  GroupSync& g = B->groups[(F->wave * 7 + lg) * 64 + F->lane / width];
  const unsigned gen = g.gen;
  const int par = gen & 1;
  if (n > 64) abort();
  memcpy(w.stage[par][F->lane], mine, n);
  ++g.arrived;
  while (g.gen == gen) {
    if (g.arrived >= width) {  // (lanes of a group leave a kernel together in the code this serves)
      g.arrived = 0;
      ++g.gen;
      ++n_progress;
      break;
    }
    yield();
  }
  return w.stage[par];
}

// Leave this lane's contribution and wait for the wave; returns the stage buffer to read.
inline const unsigned char (*wave_exchange(const void* mine, size_t n))[64] {
  WaveSync& w = B->waves[F->wave];
  const unsigned g = w.gen;
  const int par = g & 1;
  if (n > 64) abort();
  memcpy(w.stage[par][F->lane], mine, n);
  ++w.arrived;
  while (w.gen == g) {
    if (w.arrived >= w.active) {
      w.arrived = 0;
      ++w.gen;
      ++n_progress;
      break;
    }
    yield();
  }
  return w.stage[par];
}

inline void syncthreads() {
  const unsigned g = B->b_gen;
  ++B->b_arrived;
  while (B->b_gen == g) {
    if (B->b_arrived >= B->b_active) {
      B->b_arrived = 0;
      ++B->b_gen;
      ++n_progress;
      break;
    }
    yield();
  }
}

template <class T>
inline T shfl_idx(T v, int src) {
  auto st = wave_exchange(&v, sizeof(T));
  T r;
  memcpy(&r, st[src & 63], sizeof(T));
  return r;
}
template <class T>
inline T shfl_xor(T v, int mask, int width = 64) {
  if (width == 64) return shfl_idx(v, F->lane ^ mask);
  auto st = group_exchange(&v, sizeof(T), width);
  T r;
  memcpy(&r, st[(F->lane ^ mask) & 63], sizeof(T));
  return r;
}
template <class T>
inline T shfl_up(T v, int d, int width = 64) {
  const int base = F->lane / width * width, src = F->lane - d;
  auto st = wave_exchange(&v, sizeof(T));
  T r = v;
  if (src >= base) memcpy(&r, st[src], sizeof(T));
  return r;
}
template <class T>
inline T shfl_down(T v, int d, int width = 64) {
  const int base = F->lane / width * width, src = F->lane + d;
  auto st = wave_exchange(&v, sizeof(T));
  T r = v;
  if (src < base + width) memcpy(&r, st[src], sizeof(T));
  return r;
}
template <class T>
inline T shfl(T v, int src, int width = 64) {
  const int base = F->lane / width * width;
  return shfl_idx(v, base + (src & (width - 1)));
}
inline unsigned long long ballot(int pred) {
  int p = pred != 0;
  auto st = wave_exchange(&p, sizeof(p));
  unsigned long long m = 0;
  for (int l = 0; l < 64; ++l) {
    int q;
    memcpy(&q, st[l], sizeof(q));
    if (l < (int)B->bdim.x - 64 * F->wave && q) m |= 1ull << l;
  }
  return m;
}
inline int any(int pred) { return ballot(pred) != 0; }
template <class T>
inline T readfirstlane(T v) {
  return shfl_idx(v, 0);  // (every kernel here calls it with all lanes of the wave present)
}
template <class T>
inline T readlane(T v, int l) {
  return shfl_idx(v, l);
}

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
// D[i][j] += sum_k A[i][k] B[k][j], 32 x 32 x 16.  Lane (m, h): A row m, B column m, k = 8 h .. 8 h + 7;
// D register r of lane (j, h): row 8 (r / 4) + 4 h + r % 4, column j.
inline f32x16_t mfma_32x32x16_bf16(bf16x8_t a, bf16x8_t b, f32x16_t c, int, int, int) {
  struct {
    bf16x8_t a, b;
  } mine{a, b};
  auto st = wave_exchange(&mine, sizeof(mine));
  const int j = F->lane & 31, h = F->lane >> 5;
  for (int r = 0; r < 16; ++r) {
    const int i = 8 * (r / 4) + 4 * h + (r % 4);
    double s = 0;
    for (int k = 0; k < 16; ++k) {
      const __bf16* pa = reinterpret_cast<const __bf16*>(st[i + 32 * (k / 8)]);
      const __bf16* pb = reinterpret_cast<const __bf16*>(st[j + 32 * (k / 8)] + 16);
      s += (double)(float)pa[k % 8] * (double)(float)pb[k % 8];
    }
    c[r] += (float)s;
  }
  return c;
}

// ---- direct-to-LDS loads -------------------------------------------------------------------
inline thread_local char lds_anchor;  // LDS "addresses" are offsets from here (static storage lies within 2 GiB of it)
inline unsigned lds_address(const void* p) { return (unsigned)(int)((const char*)p - &lds_anchor); }
inline void dma_to_lds(const void* src, unsigned slot, int bytes) {
  char* dst = &lds_anchor + (int)slot + F->lane * bytes;
  if (!dma_late) {
    memcpy(dst, src, bytes);
    return;
  }
  DmaWrite w;
  w.dst = dst;
  w.bytes = bytes;
  memcpy(w.data, src, bytes);
  F->dma.push_back(w);
}
// all but the newest n of this lane's requests have landed
inline void wait_vmcnt(int n) {
  auto& q = F->dma;
  const int land = (int)q.size() - n;
  for (int k = 0; k < land; ++k) memcpy(q[k].dst, q[k].data, q[k].bytes);
  if (land > 0) q.erase(q.begin(), q.begin() + land);
}

// ---- launch ------------------------------------------------------------------------------------
inline void fiber_entry() {
  B->body();
  wait_vmcnt(0);
  F->done = true;
  ++n_progress;
  --B->waves[F->wave].active;
  --B->b_active;
  for (;;) yield();
}

// the workgroups of a launch that this host thread takes from `next`, one after the other
inline void run_blocks(dim3 grid, dim3 block, const std::function<void()>& kernel, std::atomic<unsigned>& next) {
  const int nthreads = block.x * block.y * block.z;
  const unsigned nblocks = grid.x * grid.y * grid.z;
  Block blk;
  blk.gdim = grid;
  blk.bdim = block;
  blk.body = kernel;
  blk.fibers.resize(nthreads);
  B = &blk;
  for (;;) {
    const unsigned taken = next.fetch_add(1);
    if (taken >= nblocks) break;
    const unsigned bi = (run_order & 2) ? nblocks - 1 - taken : taken;
    const unsigned bx = bi % grid.x, by = (bi / grid.x) % grid.y, bz = bi / (grid.x * grid.y);
    blk.bid = dim3(bx, by, bz);
    blk.waves.assign((nthreads + 63) / 64, WaveSync());
    blk.groups.assign((nthreads + 63) / 64 * 7 * 64, GroupSync());
    blk.b_arrived = 0, blk.b_gen = 0, blk.b_active = nthreads;
    for (int t = 0; t < nthreads; ++t) {
      Fiber& f = blk.fibers[t];
      f.tid = dim3(t % block.x, (t / block.x) % block.y, t / (block.x * block.y));
      f.lane = t & 63, f.wave = t >> 6, f.done = false;
      f.dma.clear();
      ++blk.waves[f.wave].active;
      getcontext(&f.ctx);
      f.ctx.uc_stack.ss_sp = f.stack.data();
      f.ctx.uc_stack.ss_size = f.stack.size();
      f.ctx.uc_link = &blk.sched;
      makecontext(&f.ctx, fiber_entry, 0);
    }
    int left = nthreads;
    while (left > 0) {
      const long before = n_progress;
      left = 0;
      const int nw = (nthreads + 63) / 64;
      for (int i = 0; i < nw * 64; ++i) {
        const int t = ((run_order & 1) ? nw - 1 - i / 64 : i / 64) * 64 + ((run_order & 4) ? 63 - i % 64 : i % 64);
        if (t >= nthreads) continue;
        Fiber& f = blk.fibers[t];
        if (f.done) continue;
        F = &f;
        swapcontext(&blk.sched, &f.ctx);
        if (!f.done) ++left;
      }
      if (left > 0 && n_progress == before) {
        // a full round in which nobody got anywhere: lanes wait for lanes that went another way
        fprintf(stderr, "emu: deadlock in block (%u, %u): %d threads wait at rendezvous that cannot complete\n", bx, by, left);
        for (size_t wv = 0; wv < blk.waves.size(); ++wv)
          fprintf(stderr, "  wave %zu: arrived %d of %d active\n", wv, blk.waves[wv].arrived, blk.waves[wv].active);
        fprintf(stderr, "  block barrier: arrived %d of %d\n", blk.b_arrived, blk.b_active);
        abort();
      }
    }
  }
  B = nullptr;
  F = nullptr;
}

template <class K>
inline void launch(dim3 grid, dim3 block, K&& kernel) {
  const std::function<void()> body = kernel;
  const unsigned nblocks = grid.x * grid.y * grid.z;
  std::atomic<unsigned> next{0};
  const unsigned helpers = host_threads > 1 ? std::min<unsigned>(host_threads, nblocks) - 1 : 0;
  std::vector<std::thread> pool;
  for (unsigned i = 0; i < helpers; ++i) pool.emplace_back([&] { run_blocks(grid, block, body, next); });
  run_blocks(grid, block, body, next);
  for (auto& t : pool) t.join();
}

}  // namespace emu

// device-library functions and builtins that the kernels use
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __hip_atomic_store(p, v, order, scope) __atomic_store_n(p, v, __ATOMIC_SEQ_CST)
#define __hip_atomic_load(p, order, scope) __atomic_load_n(p, __ATOMIC_SEQ_CST)
inline unsigned __float_as_uint(float f) { unsigned u; memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(unsigned u) { float f; memcpy(&f, &u, 4); return f; }
template <class T> inline T min(T a, T b) { return b < a ? b : a; }
template <class T> inline T max(T a, T b) { return a < b ? b : a; }
inline int64_t min(int64_t a, int b) { return a < b ? a : b; }
inline int64_t max(int64_t a, int b) { return a < b ? b : a; }
inline int64_t min(int a, int64_t b) { return a < b ? a : b; }
inline int64_t max(int a, int64_t b) { return a < b ? b : a; }
namespace emu {
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
[[noreturn]] inline void unsupported(const char* what) { fprintf(stderr, "emu: %s is not emulated\n", what); abort(); }
}  // namespace emu
#define __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8 emu::cvt_scalef32_pk_bf16_fp8_impl

struct alignas(16) int4 { int x, y, z, w; };
struct alignas(8) int2 { int x, y; };
struct alignas(8) float2 { float x, y; };
struct alignas(16) float4 { float x, y, z, w; };
struct alignas(16) uint4 { unsigned x, y, z, w; };
struct alignas(8) uint2 { unsigned x, y; };
inline float2 make_float2(float x, float y) { return float2{x, y}; }
inline float4 make_float4(float x, float y, float z, float w) { return float4{x, y, z, w}; }
inline uint4 make_uint4(unsigned x, unsigned y, unsigned z, unsigned w) { return uint4{x, y, z, w}; }
inline uint2 make_uint2(unsigned x, unsigned y) { return uint2{x, y}; }
inline int4 make_int4(int x, int y, int z, int w) { return int4{x, y, z, w}; }
inline int2 make_int2(int x, int y) { return int2{x, y}; }
typedef __bf16 __hip_bfloat16;
inline float __bfloat162float(__bf16 x) { return (float)x; }
inline __bf16 __float2bfloat16(float x) { return (__bf16)x; }
inline int __clzll(long long v) { return v == 0 ? 64 : __builtin_clzll((unsigned long long)v); }
inline int __clz(int v) { return v == 0 ? 32 : __builtin_clz((unsigned)v); }
inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
inline int __popc(unsigned v) { return __builtin_popcount(v); }
inline int __ffsll(unsigned long long v) { return __builtin_ffsll((long long)v); }
inline float __expf(float x) { return expf(x); }
inline float __logf(float x) { return logf(x); }
// (integers only: the kernels have no other atomics; the host's own, since workgroups may run on several host threads)
template <class T> inline T atomicAdd(T* p, T v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
template <class T> inline T atomicOr(T* p, T v) { return __atomic_fetch_or(p, v, __ATOMIC_SEQ_CST); }
template <class T> inline T atomicMin(T* p, T v) {
  T o = __atomic_load_n(p, __ATOMIC_SEQ_CST);
  while (v < o && !__atomic_compare_exchange_n(p, &o, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST)) {}
  return o;
}
template <class T> inline T atomicMax(T* p, T v) {
  T o = __atomic_load_n(p, __ATOMIC_SEQ_CST);
  while (o < v && !__atomic_compare_exchange_n(p, &o, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST)) {}
  return o;
}
template <class T> inline T atomicCAS(T* p, T c, T v) {
  __atomic_compare_exchange_n(p, &c, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST);
  return c;
}
inline int atomicAdd(int* p, unsigned v) { return atomicAdd<int>(p, (int)v); }
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&x)
inline hipError_t hipGetSymbolAddress(void** p, const void* sym) { *p = const_cast<void*>(sym); return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
enum { hipDeviceAttributeMultiprocessorCount = 1 };
inline hipError_t hipDeviceGetAttribute(int* v, int, int) { *v = 8; return hipSuccess; }
#define hipLaunchKernelGGL(k, g, b, sh, st, ...) emu::launch(g, b, [&] { k(__VA_ARGS__); })
#define hipExtLaunchKernelGGL(k, g, b, sh, st, e0, e1, fl, ...) emu::launch(g, b, [&] { k(__VA_ARGS__); })
namespace emu {
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
// v_permlane32_swap: the upper half of the first operand and the lower half of the second change places
inline u32x2_t permlane32_swap(unsigned a, unsigned b, bool, bool) {
  struct { unsigned a, b; } mine{a, b};
  auto st = wave_exchange(&mine, sizeof(mine));
  const int l = F->lane;
  unsigned oa, ob;
  memcpy(&oa, st[l ^ 32], 4);      // the partner's first operand
  memcpy(&ob, st[l ^ 32] + 4, 4);  // the partner's second operand
  u32x2_t r;
  r[0] = l < 32 ? a : ob;   // upper half of the first operand <- lower half of the second
  r[1] = l < 32 ? oa : b;   // lower half of the second operand <- upper half of the first
  return r;
}
inline float fp8_e4m3_to_float(unsigned char v) {
  const int sgn = v >> 7, ex = (v >> 3) & 15, man = v & 7;
  float f;
  if (ex == 15 && man == 7) f = NAN;
  else if (ex == 0) f = ldexpf((float)man, -9);
  else f = ldexpf(1.f + man / 8.f, ex - 7);
  return sgn ? -f : f;
}
inline unsigned char float_to_fp8_e4m3(float x) {  // round to nearest even, saturating (the caller clamps beforehand)
  if (x != x) return 0x7f;
  const unsigned char s = std::signbit(x) ? 0x80 : 0;
  float a = fabsf(x);
  if (a > 448.f) a = 448.f;
  if (a < ldexpf(1.f, -10)) return s;  // below half of the smallest subnormal
  int e;
  frexpf(a, &e);  // a = m * 2^e, m in [0.5, 1)
  int ex = e - 1 + 7;
  float q;
  if (ex <= 0) { q = nearbyintf(ldexpf(a, 9)); if (q >= 8) return s | 0x08; return s | (unsigned char)q; }
  q = nearbyintf(ldexpf(a, 3 - (e - 1)));  // 8 .. 16
  if (q >= 16) { q = 8; ++ex; }
  if (ex > 15 || (ex == 15 && q - 8 > 6)) return s | 0x7e;
  return s | (unsigned char)(ex << 3) | (unsigned char)(q - 8);
}
inline bf16x2_t cvt_scalef32_pk_bf16_fp8_impl(int src, float scale, bool hi) {
  const unsigned w = (unsigned)src >> (hi ? 16 : 0);
  bf16x2_t r;
  r[0] = (__bf16)(fp8_e4m3_to_float(w & 255) * scale);
  r[1] = (__bf16)(fp8_e4m3_to_float((w >> 8) & 255) * scale);
  return r;
}
inline float cvt_f32_fp8(int src, int sel) { return fp8_e4m3_to_float(((unsigned)src >> (8 * sel)) & 255); }
inline f32x2_t cvt_pk_f32_fp8(int src, bool hi) {
  const unsigned w = (unsigned)src >> (hi ? 16 : 0);
  f32x2_t r;
  r[0] = fp8_e4m3_to_float(w & 255), r[1] = fp8_e4m3_to_float((w >> 8) & 255);
  return r;
}
inline int cvt_pk_fp8_f32(float a, float b, int old, bool hi) {
  const unsigned two = float_to_fp8_e4m3(a) | (float_to_fp8_e4m3(b) << 8);
  return hi ? (int)(((unsigned)old & 0xffffu) | (two << 16)) : (int)(((unsigned)old & 0xffff0000u) | two);
}
}  // namespace emu
#define __builtin_amdgcn_permlane32_swap emu::permlane32_swap
#define __builtin_amdgcn_cvt_f32_fp8 emu::cvt_f32_fp8
#define __builtin_amdgcn_cvt_pk_f32_fp8 emu::cvt_pk_f32_fp8
#define __builtin_amdgcn_cvt_pk_fp8_f32 emu::cvt_pk_fp8_f32

#define threadIdx (emu::F->tid)
#define blockIdx (emu::B->bid)
#define gridDim (emu::B->gdim)
#define blockDim (emu::B->bdim)
#define __syncthreads() emu::syncthreads()
#define __shfl_xor(...) emu::shfl_xor(__VA_ARGS__)
#define __shfl_up(...) emu::shfl_up(__VA_ARGS__)
#define __shfl_down(...) emu::shfl_down(__VA_ARGS__)
#define __shfl(...) emu::shfl(__VA_ARGS__)
#define __any(p) emu::any(p)
#define __ballot(p) emu::ballot(p)
#define __builtin_amdgcn_readfirstlane(v) emu::readfirstlane(v)
#define __builtin_amdgcn_readlane(v, l) emu::readlane(v, l)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16 emu::mfma_32x32x16_bf16
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_logf(x) log2f(x)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_s_barrier() emu::syncthreads()
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
#define __builtin_amdgcn_sched_barrier(a) ((void)0)
// (a wave runs in lockstep on the GPU; here its lanes run one after the other, so wherever lanes read what
// other lanes of the wave wrote, the scheduling barrier that marks the place has to be a real rendezvous)
#define __builtin_amdgcn_wave_barrier() ((void)emu::wave_exchange("", 0))
#define __builtin_nontemporal_load(p) (emu::streamed_bytes += sizeof(*(p)), *(p))
#define __builtin_nontemporal_store(v, p) (*(p) = (v))
