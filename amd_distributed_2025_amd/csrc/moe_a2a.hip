// MoE dispatch/combine for one rank on MI355X (gfx950, wave64).
//
// Stages 1-3 are "ranked row moves". A workgroup owns a group of ROWS
// consecutive rows of its stage's input stream, one wave64 per row. Each wave
// first issues the 16-byte loads of its whole row (up to 16 vectors per lane
// in flight), then the workgroup finds the destination slot of all its rows
// with ONE pass over the stage's keys: a slot is the number of keys that
// precede the row in the stage's stable order, so every lane counts, for each
// of the group's rows, the keys it scanned that precede that row; the counts
// are reduced with a wave64 butterfly and a small LDS exchange; then each wave
// stores its row. The keys are a few KB and stay in L2. There are no atomics
// on global memory, no counters to clear and no dependencies between
// workgroups, so results do not depend on scheduling and nothing has to be
// zeroed between calls.
//
// Stage 4 (combine) gives a workgroup one token: it finds the rows addressed to
// the token, orders them by arrival, and accumulates them with the reference's
// per-addend rounding.
//
// Reference behaviour reproduced here: all2all/reference.py:68-148 (dispatch),
// :151-234 (combine), :262 (simulated expert).

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <limits.h>
#include <algorithm>
#include <cmath>
#include <mutex>
#include <type_traits>

#include "moe_a2a.h"

// Device memory of moe_a2a_dispatch_recv_static: the send-back plan of one call, held by the
// library so that the caller brings no buffer for it. Every GPU the library runs on has its own
// copy at its own address; host code reaches it only through the address that
// hipGetSymbolAddress returned for that GPU (static_plan_buffer below), never through this name.
#define MOE_A2A_STATIC_PLAN_EXPERTS 4096  /* world_size <= 64 times num_local_experts <= 64 */
static __device__ __align__(256) int32_t scratch[2 * MOE_A2A_STATIC_PLAN_EXPERTS];

namespace {

constexpr int META = MOE_A2A_META_DIM;
constexpr int BLOCK = 256;            // lanes of the block-per-row kernels and counting workgroups
constexpr int NWAVES = BLOCK / 64;
#ifndef MOE_A2A_ROWS
#define MOE_A2A_ROWS 4
#endif
constexpr int ROWS = MOE_A2A_ROWS;    // rows (= waves) per workgroup of a ranked row move
constexpr int COMBINE_CAP = 64;       // addends per token handled by the fast path
constexpr int COMBINE_WEIGHTS = 128;  // weights of one token staged in LDS
constexpr int COMBINE_BATCH = 8;      // addend rows loaded before accumulating
constexpr int MAX_LOCAL_EXPERTS = 4096;  // LDS prefix table of the expert-major walkers
constexpr int NUM_XCD = 8;

// 16 bytes as a native clang vector: loads and stores of it are single
// global_load/store_dwordx4 and the value lives in registers. (HIP's uint4 is a
// struct whose copies become memcpy calls that can pin a local in memory.)
typedef unsigned int b128 __attribute__((ext_vector_type(4)));

// Streaming (nontemporal) stores do not write-allocate in L2, which makes the
// writing kernel about a quarter faster, but a kernel that reads the rows right
// afterwards then fetches them from HBM and loses more than the writer gained.
// So they are used only for the two buffers whose next reader is the exchange
// (in a multi-GPU job: the fabric), not for expert_x / expert_y, which the
// expert computation reads next on the same device.
#ifndef MOE_A2A_NT_SEND   /* stage 1 -> send buffer */
#define MOE_A2A_NT_SEND 1
#endif
#ifndef MOE_A2A_NT_RECV   /* stage 2 -> expert_x */
#define MOE_A2A_NT_RECV 0
#endif
#ifndef MOE_A2A_NT_CSEND  /* stage 3 -> send-back buffer */
#define MOE_A2A_NT_CSEND 1
#endif
#ifndef MOE_A2A_NT_STANDIN /* expert and exchange stand-ins */
#define MOE_A2A_NT_STANDIN 0
#endif
#ifndef MOE_A2A_NT_LOAD
#define MOE_A2A_NT_LOAD 0
#endif
template <bool NT, typename V>
__device__ __forceinline__ void row_store(V* p, const V& v) {
  if constexpr (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}
template <typename P>
__device__ __forceinline__ auto stream_load(P p) {
#if MOE_A2A_NT_LOAD
  return __builtin_nontemporal_load(p);
#else
  return *p;
#endif
}

// ---------------------------------------------------------------- wave / block primitives

// Workgroup barrier that orders LDS traffic only. __syncthreads() also waits
// for every global load in flight, which would drain a row's prefetched payload
// in the middle of the slot computation; the waves here exchange data through
// LDS alone, so waiting for the LDS counter is enough.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Inclusive prefix sum across the 64 lanes of a wave, in the VALU's
// data-parallel-primitive (DPP) lane network: four row_shr steps scan each row
// of 16 lanes, row_bcast15 / row_bcast31 carry the row totals across rows.
// Six dependent VALU ops; a __shfl-based scan would take six round trips through
// the LDS crossbar, which is what dominates a slot computation of a few hundred
// cycles.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_add(int v) {
  // lanes whose source lies outside the row, or whose row is masked off, add 0
  return v + __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}

__device__ __forceinline__ int wave_inclusive_scan(int v) {
  v = dpp_add<0x111, 0xf>(v);  // row_shr:1
  v = dpp_add<0x112, 0xf>(v);  // row_shr:2
  v = dpp_add<0x114, 0xf>(v);  // row_shr:4
  v = dpp_add<0x118, 0xf>(v);  // row_shr:8
  v = dpp_add<0x142, 0xa>(v);  // row_bcast15 into rows 1 and 3
  v = dpp_add<0x143, 0xc>(v);  // row_bcast31 into rows 2 and 3
  return v;
}

// Sum over the wave, returned to every lane.
__device__ __forceinline__ int wave_sum(int v) {
  return __builtin_amdgcn_readlane(wave_inclusive_scan(v), 63);
}

// Sum over a workgroup of NW waves; every lane gets the total. `red` is NW ints
// of LDS and may be reused right after the call returns.
template <int NW>
__device__ __forceinline__ int block_sum(int v, int* red) {
  v = wave_sum(v);
  if (NW == 1) return v;
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  lds_barrier();
  int s = 0;
#pragma unroll
  for (int w = 0; w < NW; ++w) s += red[w];
  lds_barrier();
  return s;
}

// A value that was loaded early, handed on at the place where the program first needs it. The
// compiler moves arithmetic on a loaded value (a clamp, a compare) up to the load, out of loops
// and branches, and then waits for the load right there: a whole memory round trip ahead of
// everything issued after it. An empty volatile asm statement cannot be moved, so the wait lands
// where this is called.
__device__ __forceinline__ int first_use(int v) {
  asm volatile("" : "+v"(v));
  return v;
}

// A float32 value that counts as computed and rounded at this point: the compiler may not fuse the
// multiplication that made it with the conversion that follows. (Fused, a product rounded to fp16
// becomes v_fma_mixlo_f16 with an addend of +0, and -0 * scale + 0 is +0 where the product is -0.)
__device__ __forceinline__ float rounded_here(float v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Loads through a pointer that went through unknown_origin() and were issued before issued_here()
// stay before it. The compiler otherwise sinks a load whose value is only used under a condition
// into that condition's block, behind whatever the condition waits for; an asm statement that
// may write memory stops that only for pointers that it cannot prove untouched by the statement
// (a __restrict__ parameter is proven, the same address out of an asm statement is not).
// The pointer must be the same for every lane of the wave (it is kept in scalar registers).
template <typename T>
using global_ptr = const T __attribute__((address_space(1)))*;  // (still known to point into global memory)
template <typename T>
__device__ __forceinline__ global_ptr<T> unknown_origin(const T* p) {
  uint64_t a = (uint64_t)p;
  asm volatile("" : "+s"(a));
  return (global_ptr<T>)a;
}
__device__ __forceinline__ void issued_here() { asm volatile("" ::: "memory"); }

// Workgroups are handed to the 8 XCDs round-robin by blockIdx. This bijection
// on [0, grid) gives each XCD one contiguous run of logical items, so items
// that share a source row are served by the same L2.
__device__ __forceinline__ int xcd_contiguous(int b, int grid) {
  const int x = b % NUM_XCD;
  const int base = grid / NUM_XCD, rem = grid % NUM_XCD;
  return x * base + min(x, rem) + b / NUM_XCD;
}

// floor-mod (Python's %) by a positive divisor. `magic` = ceil(2^32 / d) gives
// an exact quotient for 0 <= e < 65536 and d <= 65536; other values take the
// slow path.
__device__ __forceinline__ int floormod(int e, int d, uint32_t magic) {
  if (d == 1) return 0;
  if ((uint32_t)e < 65536u) {
    uint32_t q = __umulhi((uint32_t)e, magic);
    return e - (int)q * d;
  }
  int m = e % d;
  return m < 0 ? m + d : m;
}

// Inclusive [lo, hi] range of expert ids owned by the same destination as `e`.
// Ids outside [0, E) name no destination: they form one class after all ranks
// (compared as unsigned numbers, a negative id is just a large one), so the
// classes still partition the integers, slots stay a permutation, the rows of
// the real destinations sit where the counts say, and the stray rows end up
// behind them, where no exchange looks.
__device__ __forceinline__ void dest_class(int e, int nle, int E, uint32_t magic, uint32_t& lo,
                                           uint32_t& hi) {
  if ((uint32_t)e >= (uint32_t)E) {
    lo = (uint32_t)E; hi = UINT_MAX;
  } else {
    const uint32_t d = (nle == 1) ? (uint32_t)e : __umulhi((uint32_t)e, magic);
    lo = d * nle; hi = lo + nle - 1;
  }
}

// NV vectors of one row chunk held in registers. Loads are unconditional
// (lanes past the end of the row re-read its last vector), so all of them are
// in flight at once; only the stores are predicated.
template <typename V, int NV>
struct Payload {
  V v[NV];
  __device__ __forceinline__ void load(const V* __restrict__ row, int base, int row_vecs) {
#pragma unroll
    for (int j = 0; j < NV; ++j) v[j] = stream_load(row + min(base + j * BLOCK + (int)threadIdx.x, row_vecs - 1));
  }
  template <bool NT>
  __device__ __forceinline__ void store_as(V* __restrict__ row, int base, int row_vecs) const {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int idx = base + j * BLOCK + threadIdx.x;
      if (idx < row_vecs) row_store<NT>(row + idx, v[j]);
    }
  }
  __device__ __forceinline__ void store(V* __restrict__ row, int base, int row_vecs) const {
    store_as<(MOE_A2A_NT_STANDIN != 0)>(row, base, row_vecs);
  }
  template <typename F>
  __device__ __forceinline__ void map(F f) {
#pragma unroll
    for (int j = 0; j < NV; ++j) v[j] = f(v[j]);
  }
};

// Sum of max(counts[i], 0) over i < n, computed by every wave on its own: the
// lanes load the counts side by side (one memory round trip instead of n
// dependent scalar loads) and reduce with the wave butterfly.
// Every count is also cut to `cap`; callers make sure n * cap fits an int, so
// the sum cannot wrap whatever the counts hold.
__device__ __forceinline__ int sum_counts(const int* __restrict__ counts, int n, int cap) {
  const int lane = threadIdx.x & 63;
  int s = 0;
  for (int i = lane; i < n; i += 64) s += min(max(counts[i], 0), cap);
  return __builtin_amdgcn_readfirstlane(wave_sum(s));
}

// Number of keys i in [0, n) that pass `test(key_i, i)`, summed over the lanes
// of this thread only (reduce with block_sum). `keys.fetch(idx, key)` loads
// SCAN_UNROLL keys at once (indices already clamped to [0, n)), so that all
// loads are in flight before the first compare; lanes past n are masked out.
#ifndef MOE_A2A_SCAN_UNROLL
#define MOE_A2A_SCAN_UNROLL 8
#endif
constexpr int SCAN_UNROLL = MOE_A2A_SCAN_UNROLL;
template <int BLK, typename Keys, typename Test>
__device__ __forceinline__ int count_keys(int n, const Keys& keys, Test test) {
  int cnt = 0;
  // the trip count is the same for every lane: fetch() may use wave shuffles
  for (int b = 0; b < n; b += SCAN_UNROLL * BLK) {
    const int i = b + threadIdx.x;
    int idx[SCAN_UNROLL], key[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) idx[u] = min(i + u * BLK, n - 1);
    keys.fetch(idx, key);
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u)
      cnt += (i + u * BLK < n) ? (int)test(key[u], i + u * BLK) : 0;
  }
  return cnt;
}

// Keys stored `stride` ints apart, key i at base[i * stride].
struct StridedKeys {
  const int* __restrict__ base;
  int stride;
  __device__ __forceinline__ void fetch(const int* idx, int* key) const {
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) key[u] = base[(size_t)idx[u] * stride];
  }
};

// One row chunk held by one wave: NVW vectors per lane, vector j of lane l is
// element base + j*64 + l of the row. Loads are unconditional and clamped, so
// all NVW of them are in flight at once; stores are predicated.
template <typename V, int NVW>
struct WavePayload {
  V v[NVW];
  template <typename P>  // const V* or global_ptr<V>
  __device__ __forceinline__ void load(P row, int base, int row_vecs, int lane) {
#pragma unroll
    for (int j = 0; j < NVW; ++j) v[j] = stream_load(row + min(base + j * 64 + lane, row_vecs - 1));
  }
  template <bool NT>
  __device__ __forceinline__ void store(V* __restrict__ row, int base, int row_vecs, int lane) const {
#pragma unroll
    for (int j = 0; j < NVW; ++j) {
      const int idx = base + j * 64 + lane;
      if (idx < row_vecs) row_store<NT>(row + idx, v[j]);
    }
  }
};

// For each of the ROWS rows r of a group: this lane's share of the number of
// keys i in [0, n) with test(r, key_i, i). Split in two so that the first
// batch of key loads can be issued BEFORE the row payload (loads return in
// issue order, so the keys arrive first and the slot is ready while the payload
// is still in flight):  RowsScan scan(n, keys);  ...issue payload...;
// scan.finish(keys, test, cnt);
template <typename Keys>
struct RowsScan {
  static constexpr int STEP = 64 * ROWS;
  int n, b;  // keys that may be loaded; first key of the batch in flight (same for every lane)
  int key[SCAN_UNROLL];
  // `n_load` keys are known to be readable; how many of them count is told to finish().
  __device__ __forceinline__ RowsScan(int n_load, const Keys& keys) : n(n_load), b(0) {
    if (n > 0) issue(keys);
  }
  // Every lane of the workgroup takes part (fetch() may use wave shuffles);
  // lanes whose keys fall past n load key n-1 and are masked in consume().
  __device__ __forceinline__ void issue(const Keys& keys) {
    const int i = b + threadIdx.x;
    int idx[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) idx[u] = min(i + u * STEP, n - 1);
    keys.fetch(idx, key);
  }
  template <typename Test>
  __device__ __forceinline__ void consume(Test test, int (&cnt)[ROWS]) const {
    const int i = b + threadIdx.x;
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) {
      const int i2 = i + u * STEP;
      if (i2 < n) {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) cnt[r] += (int)test(r, key[u], i2);
      }
    }
  }
  // Counts over keys [0, n_valid), n_valid <= n_load. The first batch is consumed
  // in straight-line code, apart from the loop over later batches: inside a loop
  // the compiler must assume the keys were the last loads issued and would wait
  // for the payload as well.
  template <typename Test>
  __device__ __forceinline__ void finish(const Keys& keys, int n_valid, Test test, int (&cnt)[ROWS]) {
#pragma unroll
    for (int r = 0; r < ROWS; ++r) cnt[r] = 0;
    const bool first = n > 0;
    n = min(n, n_valid);
    if (first) consume(test, cnt);
    for (b += SCAN_UNROLL * STEP; b < n; b += SCAN_UNROLL * STEP) {
      issue(keys);
      consume(test, cnt);
    }
  }
  // Adds the counts over keys [from, to): keys past the n_load the scan began with, readable now
  // that the caller knows the stream is that long (a stream longer than the hint it was launched with).
  template <typename Test>
  __device__ __forceinline__ void extend(const Keys& keys, int from, int to, Test test, int (&cnt)[ROWS]) {
    n = to;
    for (b = from; b < to; b += SCAN_UNROLL * STEP) {
      issue(keys);
      consume(test, cnt);
    }
  }
};

// Total of cnt[wave] over the workgroup, returned to the lanes of that wave:
// wave w gets the count that belongs to the group's row w. `part` is
// 2*ROWS*ROWS ints of LDS used in halves by alternate calls (`parity` flips per
// call), so one barrier per call is enough: a wave can only overwrite a half
// after every wave has passed the barrier of the call in between.
__device__ __forceinline__ int rows_reduce(const int (&cnt)[ROWS], int* part, int parity, int wave,
                                           int lane) {
  if (ROWS == 1) return wave_sum(cnt[0]);
  int* half = part + (parity & 1) * (ROWS * ROWS);
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int s = wave_sum(cnt[r]);
    if (lane == 0) half[wave * ROWS + r] = s;
  }
  lds_barrier();
  int mine = 0;
#pragma unroll
  for (int w = 0; w < ROWS; ++w) mine += half[w * ROWS + wave];
  return mine;
}

// ---------------------------------------------------------------- stage 1: dispatch, send side
//
// grid = W counting workgroups (rows per destination rank) followed by one
// workgroup per (group of ROWS entries, chunk). Entry i = t*K + k goes to slot
//   #{entries of a lower destination} + #{earlier entries of the same destination}.

template <typename V, int NVW>
__global__ __launch_bounds__(64 * ROWS) void dispatch_send_kernel(
    const V* __restrict__ x, const int* __restrict__ indices, int S, int K, int nle, int E, int W,
    uint32_t magic, int rank, int row_vecs, int chunks, V* __restrict__ send_buf,
    int* __restrict__ send_meta, int* __restrict__ send_counts, int* __restrict__ send_slot) {
  __shared__ int part[2 * ROWS * ROWS];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const StridedKeys key{indices, 1};

  if ((int)blockIdx.x < W) {
    const int lo = blockIdx.x * nle, hi = lo + nle - 1;
    int c = count_keys<64 * ROWS>(S, key, [lo, hi](int e, int) { return (e >= lo) & (e <= hi); });
    c = block_sum<ROWS>(c, part);
    if (tid == 0) send_counts[blockIdx.x] = c;
    return;
  }

  const int groups = (S + ROWS - 1) / ROWS;
  const int items = groups * chunks, movers = gridDim.x - W;
  int parity = 0;
  for (int q = xcd_contiguous(blockIdx.x - W, movers); q < items; q += movers, ++parity) {
    const int grp = chunks == 1 ? q : q / chunks, c = q - grp * chunks;
    const int i0 = grp * ROWS, i = i0 + wave;
    const bool valid = i < S;
    const int base = c * (64 * NVW);

    // every wave reads the expert ids of all rows of the group (the same few
    // words for every lane), so no exchange between the waves is needed
    int re[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) re[r] = indices[min(i0 + r, S - 1)];
    RowsScan<StridedKeys> scan(S, key);
    const int ic = min(i, S - 1);
    const int t = ic / K, k = ic - t * K;
    WavePayload<V, NVW> p;
    p.load(x + (size_t)t * row_vecs, base, row_vecs, lane);

    uint32_t rlo[ROWS], rhi[ROWS];
    int e = 0;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      dest_class(re[r], nle, E, magic, rlo[r], rhi[r]);
      if (r == wave) e = re[r];
    }
    int cnt[ROWS];
    scan.finish(key, S, [&](int r, int e2, int i2) {
      const uint32_t u2 = (uint32_t)e2;
      return (u2 < rlo[r]) | ((u2 <= rhi[r]) & (u2 >= rlo[r]) & (i2 < i0 + r));
    }, cnt);
    const int slot = rows_reduce(cnt, part, parity, wave, lane);

    if (valid) {
      p.template store<(MOE_A2A_NT_SEND != 0)>(send_buf + (size_t)slot * row_vecs, base, row_vecs, lane);
      if (c == 0) {
        if (lane < META) {
          int m = lane == 0 ? e : lane == 1 ? rank : lane == 2 ? t : lane == 3 ? k : 0;
          send_meta[(size_t)slot * META + lane] = m;
        }
        if (lane == 0 && send_slot) send_slot[i] = slot;
      }
    }
  }
}

// Stage 1 with one workgroup per (token, row chunk): the token's row is loaded
// once, its K entries are ranked together (FAN at a time) in one pass over the
// keys, and the row held in registers is stored to each of their slots. Compared
// with a wave per entry this reads every source row once instead of K times and
// issues an eighth of the key loads. The order is carried by one composite key
// per entry, class * S + i with class = destination, or W for an id outside
// [0, E): entry a precedes entry b exactly when its composite key is smaller.
// The host uses this kernel when (W + 2) * S fits an int.

// FAN: entries of a token that are ranked in one pass over the keys and then stored (2, 4 or 8).
// Fewer per pass means more passes over the keys and more barriers, but the first rows leave sooner
// and the ranking of the next entries runs while they drain; a compute unit has nothing else to
// do meanwhile, because all its workgroups rank at the same time. That pays while a pass is short.
// Measured at K = 8, H = 7168, the chain of four kernels (stage 1 alone in brackets), us, with
// 2 / 4 / 8: S = 2048 entries 36.5 / 36.9 / 37.4; S = 4096 73.9 / 75.4 / 74.5 (15.7 / 14.2 / 15.2);
// S = 8192 168.7 / 167.9 / 164.4 (31.6 / 31.8 / 29.0); S = 12288 233.2 / 230.5 / 222.6 (50.3 / 42.9 /
// 38.8); S = 32768 693.6 / 615.0 / 567.7 (245.4 / 169.4 / 130.6). The host takes 2 up to
// MOE_A2A_FAN2_MAX_ENTRIES entries and 8 above.
#ifndef MOE_A2A_FAN2_MAX_ENTRIES
#define MOE_A2A_FAN2_MAX_ENTRIES 4096
#endif
inline int fan_of(long long S) { return S <= MOE_A2A_FAN2_MAX_ENTRIES ? 2 : 8; }

template <typename V, int NV, int FAN>
__global__ __launch_bounds__(BLOCK) void dispatch_fanout_kernel(
    const V* __restrict__ x, const int* __restrict__ indices, int T, int K, int nle, int E, int W,
    uint32_t magic, int rank, int row_vecs, int chunks, V* __restrict__ send_buf,
    int* __restrict__ send_meta, int* __restrict__ send_counts, int* __restrict__ send_slot) {
  __shared__ int part[2 * NWAVES * FAN];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int S = T * K;
  // destination rank, or W for an id outside [0, E)
  auto klass = [&](int e) {
    return (uint32_t)e >= (uint32_t)E ? W : nle == 1 ? e : (int)__umulhi((uint32_t)e, magic);
  };

  if ((int)blockIdx.x < W) {
    const int want = blockIdx.x;
    int c = count_keys<BLOCK>(S, StridedKeys{indices, 1}, [&](int e, int) { return klass(e) == want; });
    c = block_sum<NWAVES>(c, part);
    if (tid == 0) send_counts[blockIdx.x] = c;
    return;
  }

  const int items = T * chunks, movers = gridDim.x - W;
  int parity = 0;
  for (int q = blockIdx.x - W; q < items; q += movers) {
    const int t = chunks == 1 ? q : q / chunks, c = q - t * chunks;
    const int base = c * (BLOCK * NV);
    const int i0 = t * K;

    // first batch of keys, then the row: the keys come back first
    int key[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) key[u] = indices[min(tid + u * BLOCK, S - 1)];
    Payload<V, NV> p;
    p.load(x + (size_t)t * row_vecs, base, row_vecs);

    for (int g0 = 0; g0 < K; g0 += FAN) {
      int mine[FAN];
#pragma unroll
      for (int g = 0; g < FAN; ++g) {
        const int i = i0 + min(g0 + g, K - 1);
        mine[g] = klass(indices[i]) * S + i;
      }
      int cnt[FAN];
#pragma unroll
      for (int g = 0; g < FAN; ++g) cnt[g] = 0;
      auto consume = [&](const int (&k)[SCAN_UNROLL], int b) {
#pragma unroll
        for (int u = 0; u < SCAN_UNROLL; ++u) {
          const int i2 = b + tid + u * BLOCK;
          const int ck = i2 < S ? klass(k[u]) * S + i2 : INT_MAX;
#pragma unroll
          for (int g = 0; g < FAN; ++g) cnt[g] += (int)(ck < mine[g]);
        }
      };
      consume(key, 0);
      for (int b = SCAN_UNROLL * BLOCK; b < S; b += SCAN_UNROLL * BLOCK) {
        int more[SCAN_UNROLL];
#pragma unroll
        for (int u = 0; u < SCAN_UNROLL; ++u) more[u] = indices[min(b + tid + u * BLOCK, S - 1)];
        consume(more, b);
      }

      int* half = part + (parity++ & 1) * (NWAVES * FAN);
#pragma unroll
      for (int g = 0; g < FAN; ++g) {
        const int sum = wave_sum(cnt[g]);
        if (lane == 0) half[wave * FAN + g] = sum;
      }
      lds_barrier();
      const int live = min(FAN, K - g0);
#pragma unroll
      for (int g = 0; g < FAN; ++g) {
        if (g < live) {
          int slot = 0;
#pragma unroll
          for (int w = 0; w < NWAVES; ++w) slot += half[w * FAN + g];
          p.template store_as<(MOE_A2A_NT_SEND != 0)>(send_buf + (size_t)slot * row_vecs, base, row_vecs);
        }
      }
      if (c == 0 && tid < live * META) {
        const int g = tid / META, f = tid - g * META;
        int slot = 0;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) slot += half[w * FAN + g];
        const int i = i0 + g0 + g;
        const int m = f == 0 ? indices[i] : f == 1 ? rank : f == 2 ? t : f == 3 ? g0 + g : 0;
        send_meta[(size_t)slot * META + f] = m;
        if (f == 0 && send_slot) send_slot[i] = slot;
      }
    }
  }
}

// The same fan-out for rows longer than 256 vectors: a workgroup of BLK = 512
// lanes holds NV vectors per lane (BLK lanes apart), so a row is cut into fewer
// chunks and its K entries are ranked less often. A lane compares 2048 / BLK keys per
// batch; the per-wave counts travel as 16-bit pairs (entry g with entry g + 4),
// are summed across the waves by the DPP row scan of one wave (a row of 16
// lanes per pair) and come back through LDS. Needs S < 65536 for the pairs not
// to carry into each other (a slot is below S). The composite key here is
// class << order_bits | i with S <= 1 << order_bits (no multiply per key). Measured at K = 8, H = 7168:
// the whole step 0.3 us shorter than with 256 lanes; 1024 lanes (one chunk per
// row) 0.5 us longer.

template <typename V, int BLK, int NV, bool POW2, int FAN>
__global__ __launch_bounds__(BLK) void dispatch_fanout_wide_kernel(
    const V* __restrict__ x, const int* __restrict__ indices, int T, int K, int nle, int E, int W,
    uint32_t magic, int nle_shift, int order_bits, int rank, int row_vecs, int chunks,
    V* __restrict__ send_buf, int* __restrict__ send_meta, int* __restrict__ send_counts,
    int* __restrict__ send_slot) {
  constexpr int NW = BLK / 64;
  constexpr int KEYS = SCAN_UNROLL * BLOCK / BLK;  // a batch stays SCAN_UNROLL * BLOCK keys
  constexpr int PAIRS = FAN / 2;
  static_assert(FAN == 2 || FAN == 4 || FAN == 8, "pairs of 16-bit counts, one DPP row of 16 lanes per pair");
  static_assert(NW <= 16 && KEYS >= 1, "one DPP row of 16 lanes sums the waves");
  __shared__ int part[NW * PAIRS];
  __shared__ int total[PAIRS];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int S = T * K;
  // destination rank, or W for an id outside [0, E). POW2: nle is a power of two and the division
  // is a shift (the multiply-high it replaces runs at a quarter of the rate)
  auto klass = [&](int e) {
    const int d = POW2 ? e >> nle_shift : (int)__umulhi((uint32_t)e, magic);
    return (uint32_t)e >= (uint32_t)E ? W : d;
  };
  // the composite key of entry i: class in the high bits, i below (S <= 1 << order_bits)
  auto composite = [&](int e, int i) { return (klass(e) << order_bits) | i; };

  if ((int)blockIdx.x < W) {
    const int want = blockIdx.x;
    int c = count_keys<BLK>(S, StridedKeys{indices, 1}, [&](int e, int) { return klass(e) == want; });
    c = block_sum<NW>(c, part);
    if (tid == 0) send_counts[blockIdx.x] = c;
    return;
  }

  const int items = T * chunks, movers = gridDim.x - W;
  for (int q = blockIdx.x - W; q < items; q += movers) {
    const int t = chunks == 1 ? q : q / chunks, c = q - t * chunks;
    const int col = c * (BLK * NV) + tid;  // this lane's first vector; the others BLK apart
    const int i0 = t * K;

    // the token's own expert ids, FAN at a time: lane l of every wave holds entry g0 + l % FAN. One
    // vector load issued ahead of the keys (as uniform loads they become scalar loads that are
    // waited for one by one in the middle of the ranking)
    const int own0 = indices[i0 + min(lane & (FAN - 1), K - 1)];
    int key[KEYS];
#pragma unroll
    for (int u = 0; u < KEYS; ++u) key[u] = indices[min(tid + u * BLK, S - 1)];
    V v[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) v[j] = stream_load(x + (size_t)t * row_vecs + min(col + j * BLK, row_vecs - 1));

    for (int g0 = 0; g0 < K; g0 += FAN) {
      // (a later group waits for its ids inside the branch: a wait at the place where the two paths
      // meet would cover the first group's row as well, which is requested behind its ids)
      int own = own0;
      if (g0 > 0) own = first_use(indices[i0 + min(g0 + (lane & (FAN - 1)), K - 1)]);
      int mine[FAN];
#pragma unroll
      for (int g = 0; g < FAN; ++g) {
        const int i = i0 + min(g0 + g, K - 1);
        mine[g] = composite(__builtin_amdgcn_readlane(own, g), i);
      }
      int cnt[FAN];
#pragma unroll
      for (int g = 0; g < FAN; ++g) cnt[g] = 0;
      auto consume = [&](const int (&k)[KEYS], int b) {
#pragma unroll
        for (int u = 0; u < KEYS; ++u) {
          const int i2 = b + tid + u * BLK;
          const int ck = i2 < S ? composite(k[u], i2) : INT_MAX;
#pragma unroll
          for (int g = 0; g < FAN; ++g) cnt[g] += (int)(ck < mine[g]);
        }
      };
      consume(key, 0);
      for (int b = KEYS * BLK; b < S; b += KEYS * BLK) {
        int more[KEYS];
#pragma unroll
        for (int u = 0; u < KEYS; ++u) more[u] = indices[min(b + tid + u * BLK, S - 1)];
        consume(more, b);
      }

#pragma unroll
      for (int h = 0; h < PAIRS; ++h) {
        const int sum = wave_sum(cnt[h] | (cnt[h + PAIRS] << 16));
        if (lane == 0) part[wave * PAIRS + h] = sum;
      }
      lds_barrier();
      if (wave == 0) {  // row h of 16 lanes adds up pair h of every wave
        const int h = lane >> 4, w = lane & 15;
        int sum = w < NW && h < PAIRS ? part[w * PAIRS + h] : 0;
        sum = dpp_add<0x111, 0xf>(sum);
        sum = dpp_add<0x112, 0xf>(sum);
        sum = dpp_add<0x114, 0xf>(sum);
        sum = dpp_add<0x118, 0xf>(sum);
        if (w == 15 && h < PAIRS) total[h] = sum;
      }
      lds_barrier();
      // no third barrier: `part` is next written before a barrier that wave 0 only reaches after
      // it has read `part`, and `total` after a barrier every wave reaches after reading it
      int slot[FAN];
#pragma unroll
      for (int h = 0; h < PAIRS; ++h) {
        const int both = total[h];
        slot[h] = both & 0xffff;
        slot[h + PAIRS] = (int)((unsigned)both >> 16);
      }
      const int live = min(FAN, K - g0);
#pragma unroll
      for (int g = 0; g < FAN; ++g) {
#pragma unroll
        for (int j = 0; j < NV; ++j)
          if (g < live && col + j * BLK < row_vecs)
            row_store<(MOE_A2A_NT_SEND != 0)>(send_buf + (size_t)slot[g] * row_vecs + col + j * BLK, v[j]);
      }
      if (c == 0 && tid < live * META) {
        const int g = tid / META, f = tid - g * META;
        int mine_slot = 0;
#pragma unroll
        for (int gg = 0; gg < FAN; ++gg) mine_slot = gg == g ? slot[gg] : mine_slot;
        const int i = i0 + g0 + g;
        const int e = __shfl(own, g, 64);  // (lanes 0 .. FAN-1 of wave 0 are among the active ones)
        const int m = f == 0 ? e : f == 1 ? rank : f == 2 ? t : f == 3 ? g0 + g : 0;
        send_meta[(size_t)mine_slot * META + f] = m;
        if (f == 0 && send_slot) send_slot[i] = mine_slot;
      }
    }
  }
}

// ---------------------------------------------------------------- send plan (counts, offsets, maps)
//
// The stable counting sort of stage 1 made explicit, for callers that want the
// plan without moving rows (a sender that writes into a peer's buffer, a
// debugger): rows per destination rank and per expert, the exclusive offsets
// of the destinations, and both index maps. One workgroup of 16 waves walks
// the (t, k) stream in tiles of 1024 entries:
//   pass 1  per-wave privatised LDS histograms of the destinations (no two
//           waves touch the same counters), one shared LDS histogram of the
//           expert ids; a wave64 exclusive scan turns the destination totals
//           into offsets;
//   pass 2  inside a wave, an entry's rank among the earlier lanes with the
//           same destination comes from a ballot per destination present in
//           the wave; the waves of a tile are ordered by a prefix over their
//           per-destination counts, tiles by a running base per destination.
// slot(i) = offset[d] + #earlier entries with destination d — the order of
// all2all/reference.py:79-86,93.

constexpr int PLAN_BLOCK = 1024;
constexpr int PLAN_WAVES = PLAN_BLOCK / 64;
constexpr int PLAN_MAX_RANKS = 64;      // destinations kept per wave in LDS
constexpr int PLAN_MAX_EXPERTS = 8192;  // shared expert histogram in LDS

__global__ __launch_bounds__(PLAN_BLOCK) void plan_send_kernel(
    const int* __restrict__ indices, int S, int nle, int E, int W, uint32_t magic,
    int* __restrict__ rank_counts, int* __restrict__ rank_offsets, int* __restrict__ expert_counts,
    int* __restrict__ dst_slot, int* __restrict__ src_entry) {
  __shared__ int wave_hist[PLAN_WAVES][PLAN_MAX_RANKS];
  __shared__ int base[PLAN_MAX_RANKS];        // next free slot of each destination
  __shared__ int expert_hist[PLAN_MAX_EXPERTS];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const unsigned long long lanes_below = lane == 0 ? 0ull : (~0ull >> (64 - lane));

  auto dest_of = [&](int e) { return nle == 1 ? e : (int)__umulhi((uint32_t)e, magic); };
  auto in_range = [&](int e) { return (e >= 0) & (e < E); };

  // ---- pass 1: histograms
  for (int i = tid; i < PLAN_WAVES * PLAN_MAX_RANKS; i += PLAN_BLOCK) (&wave_hist[0][0])[i] = 0;
  for (int i = tid; i < E; i += PLAN_BLOCK) expert_hist[i] = 0;
  lds_barrier();
  for (int b = 0; b < S; b += PLAN_BLOCK) {
    const int i = b + tid;
    const int e = i < S ? indices[i] : -1;
    if (in_range(e)) {
      atomicAdd(&expert_hist[e], 1);
      // lanes of one wave that share a destination add their count once
      const int d = dest_of(e);
      unsigned long long todo = __ballot(1);
      while (todo) {
        const int leader = __builtin_amdgcn_readfirstlane(d);
        const unsigned long long same = __ballot(d == leader);
        if (d == leader) {
          if ((same & lanes_below) == 0) wave_hist[wave][leader] += __popcll(same);
          break;
        }
        todo &= ~same;
      }
    }
  }
  lds_barrier();
  for (int i = tid; i < E; i += PLAN_BLOCK) expert_counts[i] = expert_hist[i];
  if (wave == 0) {  // destination totals -> exclusive offsets with a wave64 scan
    int total = 0;
    if (lane < W) {
#pragma unroll
      for (int w = 0; w < PLAN_WAVES; ++w) total += wave_hist[w][lane];
    }
    const int incl = wave_inclusive_scan(total);
    if (lane < W) {
      rank_counts[lane] = total;
      rank_offsets[lane] = incl - total;
      base[lane] = incl - total;
    }
    if (lane == W - 1 || (W == 64 && lane == 63)) rank_offsets[W] = incl;
  }
  lds_barrier();

  // ---- pass 2: stable slots, tile by tile
  for (int b = 0; b < S; b += PLAN_BLOCK) {
    for (int i = tid; i < PLAN_WAVES * PLAN_MAX_RANKS; i += PLAN_BLOCK) (&wave_hist[0][0])[i] = 0;
    lds_barrier();
    const int i = b + tid;
    const int e = i < S ? indices[i] : -1;
    const bool ok = in_range(e);
    const int d = ok ? dest_of(e) : -1;
    int rank_in_wave = 0;
    unsigned long long todo = __ballot(ok);
    while (todo) {  // every lane of the wave runs the same number of rounds
      const int first = __ffsll((long long)todo) - 1;
      const int leader = __builtin_amdgcn_readlane(d, first);
      const unsigned long long same = __ballot(ok && d == leader);
      if (ok && d == leader) {
        rank_in_wave = __popcll(same & lanes_below);
        if (rank_in_wave == 0) wave_hist[wave][leader] = __popcll(same);
      }
      todo &= ~same;
    }
    lds_barrier();
    if (ok) {
      int before = base[d];
      for (int w = 0; w < wave; ++w) before += wave_hist[w][d];
      const int slot = before + rank_in_wave;
      dst_slot[i] = slot;
      src_entry[slot] = i;
    }
    lds_barrier();
    if (tid < W) {
      int t = 0;
#pragma unroll
      for (int w = 0; w < PLAN_WAVES; ++w) t += wave_hist[w][tid];
      base[tid] += t;
    }
    lds_barrier();
  }
}

// ---------------------------------------------------------------- stage 2: dispatch, receive side
//
// grid = nle counting workgroups (rows per local expert) followed by one
// workgroup per (group of ROWS received rows, chunk). Row i goes to expert
// le = e % nle at position #{earlier rows of the same expert}.
//
// `hint_rows` rows of recv_buf / recv_meta are readable whatever the counts
// say. A workgroup whose rows lie below that bound issues all its loads before
// it knows the true row count R (the counts are loaded at the same time) and
// only the stores wait for R; rows at or past R are loaded and dropped. Counts
// that add up to more than `capacity_rows` (what the buffers hold) are cut off there.

//
// PLAN (W <= 64): the counting workgroup of expert le also splits its rows by
// source rank and writes, for every source s, two ints at plan[(le*W + s)*2]:
//   [0] the position inside expert le at which the rows from s start (inside an
//       expert, rows lie in arrival order, that is by source rank), and
//   [1] the row of the send-back stream of stage 3 that the first of them goes
//       to: #{rows from lower sources} + #{rows from s in lower experts}.
// Stage 3 then places a row without scanning any keys.

constexpr int PLAN_INTS = 2;  // ints per (local expert, source rank) of the send-back plan

// Long streams. The movers below rank a row by counting the keys ahead of it, and every
// workgroup of four rows repeats that pass: the key loads grow with the square of the row count
// (at 8192 rows they are two thirds of the payload). For long streams the positions are worked
// out by a launch of their own, one workgroup of 1024 lanes per tile of 1024 rows: an LDS
// histogram (atomics; the order of the adds does not matter) of the experts of all rows ahead of
// the tile, then inside the tile a row's rank among the earlier lanes of its wave with the same
// expert (the set of those lanes from one ballot per bit of the expert number), the waves ordered
// by a prefix over their per-expert counts. row_pos[i] = #{rows before i with the same local expert}, which is
// the slot the reference's running counter hands out (all2all/reference.py:140-146). The movers
// then read one int per row instead of scanning.
constexpr int RPLAN_BLOCK = 1024;
constexpr int RPLAN_WAVES = RPLAN_BLOCK / 64;
constexpr int RPLAN_MAX_EXPERTS = 256;  // local experts with a counter per wave in LDS

__global__ __launch_bounds__(RPLAN_BLOCK) void plan_recv_kernel(
    const int* __restrict__ recv_meta, const int* __restrict__ recv_counts, int W, int hint_rows,
    int capacity_rows, int nle, uint32_t magic, int expert_bits, int* __restrict__ row_pos) {
  __shared__ int ahead[RPLAN_MAX_EXPERTS];                  // rows of each expert before the tile
  __shared__ int in_wave[RPLAN_WAVES][RPLAN_MAX_EXPERTS];   // rows of each expert in each wave of the tile
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const unsigned long long lanes_below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int R = -1;  // not known yet
  auto rows = [&] { return min(sum_counts(recv_counts, W, capacity_rows), capacity_rows); };
  for (int first = blockIdx.x * RPLAN_BLOCK;; first += gridDim.x * RPLAN_BLOCK) {
    // A tile that lies wholly below the readable bound sends its loads off before the row
    // count is known: the counts travel at the same time (one round trip instead of three).
    const bool early = R < 0 && first + RPLAN_BLOCK <= hint_rows;
    if (!early) {
      if (R < 0) R = rows();
      if (first >= R) break;
    }
    const int last = early ? first + RPLAN_BLOCK - 1 : R - 1;  // last row that may be read
    const int i = first + tid;
    const int mine = recv_meta[(size_t)min(i, last) * META];
    int e2[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u)
      e2[u] = recv_meta[(size_t)min(tid + u * RPLAN_BLOCK, max(first - 1, 0)) * META];
    for (int j = tid; j < nle; j += RPLAN_BLOCK) ahead[j] = 0;
    for (int j = tid; j < RPLAN_WAVES * RPLAN_MAX_EXPERTS; j += RPLAN_BLOCK) (&in_wave[0][0])[j] = 0;
    if (R < 0) R = rows();
    lds_barrier();
    if (first >= R) break;  // (uniform over the workgroup)
    const bool ok = i < R;
    const int le = floormod(mine, nle, magic);
    for (int b = 0; b < first; b += SCAN_UNROLL * RPLAN_BLOCK) {
      if (b > 0) {
#pragma unroll
        for (int u = 0; u < SCAN_UNROLL; ++u)
          e2[u] = recv_meta[(size_t)min(b + tid + u * RPLAN_BLOCK, first - 1) * META];
      }
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u)
        if (b + tid + u * RPLAN_BLOCK < first) atomicAdd(&ahead[floormod(e2[u], nle, magic)], 1);
    }
    // the lanes of this wave with the same expert, from one ballot per bit of the expert number
    // (a loop over the experts present in the wave costs a round per expert: 3.8 us of issue
    // slots with 32 experts and four waves per SIMD)
    unsigned long long same = __ballot(ok);
    for (int b = 0; b < expert_bits; ++b) {
      const bool set = (le >> b) & 1;
      const unsigned long long with_bit = __ballot(set);
      same &= set ? with_bit : ~with_bit;
    }
    const int rank_in_wave = __popcll(same & lanes_below);
    if (ok && rank_in_wave == 0) in_wave[wave][le] = __popcll(same);
    lds_barrier();
    if (ok) {
      int pos = ahead[le] + rank_in_wave;
      for (int w = 0; w < wave; ++w) pos += in_wave[w][le];
      row_pos[i] = pos;
    }
    lds_barrier();  // the tables are cleared again by the next tile
  }
}

// How a mover finds the place of a row:
//   RECV_SCAN     by counting the earlier rows of the same expert (the padded layout of
//                 all2all/reference.py:127-136: row pos of expert le at le * max_recv + pos);
//   RECV_POS      from `row_pos` (plan_recv_kernel): the movers scan nothing (padded layout);
//   RECV_COMPACT  the compact layout: the experts' rows back to back, row pos of expert le at
//                 offset[le] + pos with offset = exclusive prefix of the rows per expert. A row's
//                 place is then the number of rows of lower experts anywhere in the stream plus
//                 the earlier rows of its own expert (one pass over all keys); `max_recv` is the
//                 number of rows the compact buffers hold, and the counting workgroups also write
//                 the offsets.
enum { RECV_SCAN = 0, RECV_POS = 1, RECV_COMPACT = 2 };

template <typename V, int NVW, bool PLAN, int MODE>
__global__ __launch_bounds__(64 * ROWS) void dispatch_recv_kernel(
    const V* __restrict__ recv_buf, const int* __restrict__ recv_meta,
    const int* __restrict__ recv_counts, int W, int hint_rows, int capacity_rows, int nle,
    uint32_t magic, int max_recv, int row_vecs, int chunks, int* __restrict__ expert_num_tokens,
    V* __restrict__ expert_x, int* __restrict__ expert_meta, int* __restrict__ plan,
    const int* __restrict__ row_pos, int* __restrict__ expert_offsets) {
  constexpr bool POS = MODE == RECV_POS, COMPACT = MODE == RECV_COMPACT;
  __shared__ int part[2 * ROWS * ROWS];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const StridedKeys key{recv_meta, META};

  if constexpr (PLAN) {
    if ((int)blockIdx.x < nle) {
      __shared__ int seg_end[64];  // rows received from sources 0..s
      __shared__ int hist[64][2];  // per source: rows of this expert, rows of lower experts
      const int me = blockIdx.x;
      const int mine = lane < W ? min(max(recv_counts[lane], 0), capacity_rows) : 0;
      const int incl = wave_inclusive_scan(mine);
      const int R = min(__builtin_amdgcn_readlane(incl, 63), capacity_rows);
      if (wave == 0 && lane < W) {
        seg_end[lane] = incl;
        hist[lane][0] = 0;
        hist[lane][1] = 0;
      }
      lds_barrier();
      constexpr int BLK = 64 * ROWS;
      for (int b = 0; b < R; b += SCAN_UNROLL * BLK) {
        int e2[SCAN_UNROLL];
#pragma unroll
        for (int u = 0; u < SCAN_UNROLL; ++u)
          e2[u] = recv_meta[(size_t)min(b + tid + u * BLK, R - 1) * META];
#pragma unroll
        for (int u = 0; u < SCAN_UNROLL; ++u) {
          const int i2 = b + tid + u * BLK;
          const int le2 = floormod(e2[u], nle, magic);
          if (i2 < R && le2 <= me) {
            int src = 0;
            for (int s = 0; s + 1 < W; ++s) src += (int)(seg_end[s] <= i2);
            atomicAdd(&hist[src][le2 < me ? 1 : 0], 1);
          }
        }
      }
      lds_barrier();
      if (wave == 0) {
        const int here = lane < W ? hist[lane][0] : 0;
        const int below = lane < W ? hist[lane][1] : 0;
        const int upto = wave_inclusive_scan(here);
        if (lane < W) {
          int* out = plan + ((size_t)me * W + lane) * PLAN_INTS;
          out[0] = upto - here;
          out[1] = (incl - mine) + below;
        }
        if (lane == 63) expert_num_tokens[me] = upto;
        if constexpr (COMPACT) {  // rows of lower experts, from every source: where this expert's rows start
          const int lower = wave_sum(below), mine_all = __builtin_amdgcn_readlane(upto, 63);
          if (lane == 0) {
            expert_offsets[me] = lower;
            if (me == nle - 1) expert_offsets[nle] = lower + mine_all;
          }
        }
      }
      return;
    }
  }

  if ((int)blockIdx.x < nle) {
    const int R = min(sum_counts(recv_counts, W, capacity_rows), capacity_rows);
    const int me = blockIdx.x;
    int c = count_keys<64 * ROWS>(R, key, [=](int e, int) { return floormod(e, nle, magic) == me; });
    c = block_sum<ROWS>(c, part);
    if (tid == 0) expert_num_tokens[me] = c;
    if constexpr (COMPACT) {
      int lower = count_keys<64 * ROWS>(R, key, [=](int e, int) { return floormod(e, nle, magic) < me; });
      lower = block_sum<ROWS>(lower, part);
      if (tid == 0) {
        expert_offsets[me] = lower;
        if (me == nle - 1) expert_offsets[nle] = lower + c;
      }
    }
    return;
  }

  const int movers = gridDim.x - nle;
  int parity = 0;
  // One (group, chunk) item. `limit` rows may be read; R is evaluated after the
  // loads are issued (it is already known on every pass but the first).
  auto move = [&](int q, int limit, auto&& rows_known) {
    const int grp = chunks == 1 ? q : q / chunks, c = q - grp * chunks;
    const int i0 = grp * ROWS, i = i0 + wave;
    const int ic = min(i, limit - 1);
    const int base = c * (64 * NVW);

    if constexpr (POS) {
      const int e = recv_meta[(size_t)ic * META];
      const int pos = row_pos[ic];
      int m = 0;
      if (c == 0 && lane < META) m = recv_meta[(size_t)ic * META + lane];
      WavePayload<V, NVW> p;
      p.load(recv_buf + (size_t)ic * row_vecs, base, row_vecs, lane);
      const int R = rows_known();
      if (i < R && (uint32_t)pos < (uint32_t)max_recv) {
        const size_t row = (size_t)floormod(e, nle, magic) * max_recv + pos;
        p.template store<(MOE_A2A_NT_RECV != 0)>(expert_x + row * row_vecs, base, row_vecs, lane);
        if (c == 0 && lane < META) expert_meta[row * META + lane] = m;
      }
      return R;
    }

    int re[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) re[r] = recv_meta[(size_t)min(i0 + r, limit - 1) * META];
    int m = 0;
    if (c == 0 && lane < META) m = recv_meta[(size_t)ic * META + lane];
    // only rows before the group's last row can precede any of its rows in its expert; the rows of
    // lower experts, which the compact layout puts ahead of it, lie anywhere in the stream
    RowsScan<StridedKeys> scan(COMPACT ? limit : min(i0 + ROWS - 1, limit), key);
    WavePayload<V, NVW> p;
    p.load(recv_buf + (size_t)ic * row_vecs, base, row_vecs, lane);

    const int R = rows_known();
    int rle[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) rle[r] = floormod(re[r], nle, magic);
    int cnt[ROWS];
    auto precedes = [&](int r, int e2, int i2) {
      const int le2 = floormod(e2, nle, magic);
      if constexpr (COMPACT) return (le2 < rle[r]) | ((le2 == rle[r]) & (i2 < i0 + r));
      else return (le2 == rle[r]) & (i2 < i0 + r);
    };
    scan.finish(key, COMPACT ? R : min(i0 + ROWS - 1, R), precedes, cnt);
    if constexpr (COMPACT) {
      // the scan began with the `limit` keys that were known to be readable; a stream longer than
      // that (a hint below the row count) has rows of lower experts behind them as well
      if (R > limit) scan.extend(key, limit, R, precedes, cnt);
    }
    const int pos = rows_reduce(cnt, part, parity++, wave, lane);

    if (i < R && pos < max_recv) {
      int le = 0;
#pragma unroll
      for (int r = 0; r < ROWS; ++r) le = r == wave ? rle[r] : le;
      const size_t row = COMPACT ? (size_t)pos : (size_t)le * max_recv + pos;
      p.template store<(MOE_A2A_NT_RECV != 0)>(expert_x + row * row_vecs, base, row_vecs, lane);
      if (c == 0 && lane < META) expert_meta[row * META + lane] = m;
    }
    return R;
  };

  // Back to front: the workgroups launched first take the last rows. A compute unit serves the
  // memory requests of its workgroups in launch order, and the later a row lies in the stream
  // the more keys its group scans; the workgroups a unit serves last should be the cheap ones
  // (measured at 2048 rows of 14 KB: 11.7 -> 11.1 us; with a few workgroups more than two per
  // unit, which are then the ones with next to nothing to scan, 13.2 -> 11.6 us).
  int q = movers - 1 - ((int)blockIdx.x - nle);
  int R;
  // only groups that lie wholly below the bound: their rows can be read as they are
  const int hint_items = hint_rows / ROWS * chunks;
  if (W <= 64 && q < hint_items) {
    // The count travels with the rows: nothing touches the loaded value before the key and row
    // loads have been issued (first_use).
    const int raw_count = recv_counts[min(lane, W - 1)];
    R = move(q, hint_rows, [&] {
      const int my_count = lane < W ? min(max(first_use(raw_count), 0), capacity_rows) : 0;
      return min(wave_sum(my_count), capacity_rows);
    });
    q += movers;
  } else {
    R = min(sum_counts(recv_counts, W, capacity_rows), capacity_rows);
  }
  const int items = (R + ROWS - 1) / ROWS * chunks;
  for (; q < items; q += movers) move(q, R, [&] { return R; });
}

// ---------------------------------------------------------------- expert-major stream helpers

// pre[0..nle] = exclusive prefix of value_of(le); returns the total. Each lane
// owns a contiguous run of experts; runs are combined by a wave64 scan and a
// scan over the wave totals.
template <int NW, class ValueOf>
__device__ __forceinline__ int expert_prefix_of(int nle, int* pre, int* red, ValueOf value_of) {
  const int tid = threadIdx.x;
  const int per = (nle + 64 * NW - 1) / (64 * NW);
  const int b = min(tid * per, nle), e = min(b + per, nle);
  int s = 0;
  for (int i = b; i < e; ++i) s += value_of(i);
  const int inc = wave_inclusive_scan(s);
  if ((tid & 63) == 63) red[tid >> 6] = inc;
  lds_barrier();
  int off = 0, total = 0;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    if (w < (tid >> 6)) off += red[w];
    total += red[w];
  }
  int run = off + inc - s;
  for (int i = b; i < e; ++i) {
    pre[i] = run;
    run += value_of(i);
  }
  if (tid == 0) pre[nle] = total;
  lds_barrier();
  return total;
}

// The prefix of the rows per expert, min(cnt[le], max_recv).
template <int NW>
__device__ __forceinline__ int expert_prefix(const int* __restrict__ cnt, int nle, int max_recv,
                                             int* pre, int* red) {
  return expert_prefix_of<NW>(nle, pre, red, [=](int le) { return min(max(cnt[le], 0), max_recv); });
}

// Largest le in [0, nle) with pre[le] <= g, for g < pre[nle] (so empty experts
// are skipped). Fixed-trip binary lifting: `top` is the largest power of two
// below nle (0 when nle == 1), so several searches can run interleaved.
__device__ __forceinline__ int expert_of(const int* pre, int nle, int top, int g) {
  int lo = 0;
  for (int step = top; step > 0; step >>= 1) {
    const int c = lo + step;
    if (c < nle && pre[c] <= g) lo = c;
  }
  return lo;
}

__device__ __forceinline__ int top_step(int nle) {
  int top = 0;
  for (int s = 1; s < nle; s <<= 1) top = s;
  return top;
}

// Keys (int FIELD of the meta row) of rows of the expert-major stream, row g
// being the g-th valid row in (le, j) order. The SCAN_UNROLL searches of one
// fetch advance in lock step, so their LDS reads overlap instead of chaining.
template <int FIELD>
struct ExpertStreamKeys {
  const int* pre;  // LDS, nle + 1 entries, pre[nle] = number of rows
  const int* __restrict__ meta;
  int nle, top, max_recv;
  bool compact;  // the experts' rows lie back to back: stream row g is buffer row g
  __device__ __forceinline__ void fetch(const int* g, int* key) const {
    if (compact) {
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) key[u] = meta[(size_t)g[u] * META + FIELD];
      return;
    }
    int le[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) le[u] = 0;
    for (int step = top; step > 0; step >>= 1) {
      // all reads of a step first, then all updates: the reads stay in flight together
      int c[SCAN_UNROLL], v[SCAN_UNROLL];
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) c[u] = min(le[u] + step, nle);  // pre[nle] > g: never taken
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) v[u] = pre[c[u]];
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) le[u] = v[u] <= g[u] ? c[u] : le[u];
    }
    int first[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) first[u] = pre[le[u]];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) {
      const size_t row = (size_t)le[u] * max_recv + (g[u] - first[u]);
      key[u] = meta[row * META + FIELD];
    }
  }
};

// The same stream when there are at most 64 local experts: lane l of every wave
// keeps the prefix of expert l in a register, so there is no LDS table, no
// barrier and the row a wave owns is found with one ballot. Lanes at or past
// nle hold the total, which no row index reaches.
struct WaveExpertPrefix {
  int excl, incl;  // rows before / up to and including expert `lane`
  int total;
  __device__ __forceinline__ WaveExpertPrefix(const int* __restrict__ cnt, int nle, int max_recv) {
    const int lane = threadIdx.x & 63;
    const int c = lane < nle ? min(max(cnt[lane], 0), max_recv) : 0;
    incl = wave_inclusive_scan(c);
    excl = incl - c;
    total = __builtin_amdgcn_readlane(incl, 63);
  }
  // expert holding row g (wave-uniform g < total) and the number of rows before it
  __device__ __forceinline__ void locate(int g, int& le, int& first) const {
    le = __popcll(__ballot(incl <= g));
    first = __builtin_amdgcn_readlane(excl, le);
  }
};

template <int FIELD>
struct WaveStreamKeys {
  int excl;  // this lane's WaveExpertPrefix::excl
  const int* __restrict__ meta;
  int nle, top, max_recv;
  bool compact;  // the experts' rows lie back to back: stream row g is buffer row g
  __device__ __forceinline__ void fetch(const int* g, int* key) const {
    if (compact) {  // (the same for every lane: no lane leaves the shuffles below behind)
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) key[u] = meta[(size_t)g[u] * META + FIELD];
      return;
    }
    int le[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) le[u] = 0;
    for (int step = top; step > 0; step >>= 1) {
      int c[SCAN_UNROLL], v[SCAN_UNROLL];
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) c[u] = le[u] + step;  // at most 32+16+...+1 = 63
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) v[u] = __shfl(excl, c[u], 64);
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) le[u] = v[u] <= g[u] ? c[u] : le[u];
    }
    int first[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) first[u] = __shfl(excl, le[u], 64);
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) {
      const size_t row = (size_t)le[u] * max_recv + (g[u] - first[u]);
      key[u] = meta[row * META + FIELD];
    }
  }
};

// ---------------------------------------------------------------- stage 3: combine, send side
//
// grid = W counting workgroups (rows per origin rank) followed by one workgroup
// per (group of ROWS valid expert rows, chunk), rows numbered g in (le, j)
// order. Row g with origin d goes to slot
//   #{rows of a lower origin} + #{earlier rows of origin d}.

//
// PLAN (needs SMALL and W <= 64): stage 2 left, for every (local expert, source
// rank), where that run of rows starts inside the expert and in the send-back
// stream (see dispatch_recv_kernel). A wave then finds the run its row lies in
// with one ballot over W lanes and needs no key scan and no exchange with the
// other waves. The plan counts every received row, so it only describes the
// buffers when no expert overflowed max_recv; if one did, every workgroup sees
// it in the counts and takes the scan instead.

template <typename V, int NVW, bool SMALL, bool PLAN>
__global__ __launch_bounds__(64 * ROWS) void combine_send_kernel(
    const V* __restrict__ expert_y, const int* __restrict__ expert_meta,
    const int* __restrict__ expert_num_tokens, int nle, int max_recv, int W, int row_vecs,
    int chunks, int capacity_rows, V* __restrict__ send_buf, int* __restrict__ send_meta,
    int* __restrict__ send_counts, const int* __restrict__ plan, int compact_rows) {
  static_assert(!PLAN || SMALL, "the planned path keeps the expert prefix in registers");
  __shared__ int part[2 * ROWS * ROWS];
  __shared__ int pre[SMALL ? 1 : MAX_LOCAL_EXPERTS + 1];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  // compact_rows > 0: expert_y / expert_meta hold the experts' rows back to back (stream row g is
  // buffer row g) in buffers of compact_rows rows, and max_recv is that number too
  const bool compact = compact_rows > 0;

  if constexpr (PLAN) {
    const int raw = lane < nle ? expert_num_tokens[lane] : 0;
    const int have = max(raw, 0);
    const int incl = wave_inclusive_scan(have), excl = incl - have;
    const int R = __builtin_amdgcn_readlane(incl, 63);
    // (the plan also counts rows that found no room; with such rows the scan below is taken)
    if (__ballot(raw > max_recv) == 0 && !(compact && R > compact_rows)) {

      if ((int)blockIdx.x < W) {
        // rows that go back to origin `me`: the lengths of its runs, one expert per lane
        const int me = blockIdx.x;
        int len = 0;
        if (lane < nle) {
          const int* run = plan + ((size_t)lane * W + me) * PLAN_INTS;
          len = (me + 1 < W ? run[PLAN_INTS] : have) - run[0];
        }
        const int total = wave_sum(len);
        if (tid == 0) send_counts[me] = total;
        return;
      }

      const int items = R * chunks, movers = (gridDim.x - W) * ROWS;
      for (int qv = (blockIdx.x - W) * ROWS + wave; qv < items; qv += movers) {
        const int q = __builtin_amdgcn_readfirstlane(qv);  // the same for every lane of a wave
        const int g = chunks == 1 ? q : q / chunks, c = q - g * chunks;
        const int base = c * (64 * NVW);
        const int le = __popcll(__ballot(incl <= g));
        const int j = g - __builtin_amdgcn_readlane(excl, le);
        const size_t row = compact ? (size_t)g : (size_t)le * max_recv + j;
        int run[PLAN_INTS] = {INT_MAX, 0};
        if (lane < W) __builtin_memcpy(run, plan + ((size_t)le * W + lane) * PLAN_INTS, sizeof(run));
        int m = 0;
        if (c == 0 && lane < META) m = expert_meta[row * META + lane];
        WavePayload<V, NVW> p;
        p.load(unknown_origin(expert_y + row * row_vecs), base, row_vecs, lane);
        // (the row is only used by the stores below, which depend on the slot: without this the
        // compiler moves the loads down behind the plan's round trip)
        issued_here();
        // the run starts are ascending in the source rank: the last one at or below j is ours
        const int src = max((int)__popcll(__ballot(run[0] <= j)) - 1, 0);
        const int slot = __builtin_amdgcn_readlane(run[1], src) + (j - __builtin_amdgcn_readlane(run[0], src));
        if (slot >= 0 && slot < capacity_rows) {
          p.template store<(MOE_A2A_NT_CSEND != 0)>(send_buf + (size_t)slot * row_vecs, base, row_vecs, lane);
          if (c == 0 && lane < META) send_meta[(size_t)slot * META + lane] = m;
        }
      }
      return;
    }
  }

  // SMALL (nle <= 64): prefix in registers; otherwise the LDS table
  using Keys = typename std::conditional<SMALL, WaveStreamKeys<1>, ExpertStreamKeys<1>>::type;
  int R, my_excl = 0, my_incl = 0;
  if constexpr (SMALL) {
    const WaveExpertPrefix wp(expert_num_tokens, nle, max_recv);
    R = wp.total; my_excl = wp.excl; my_incl = wp.incl;
  } else {
    R = expert_prefix<ROWS>(expert_num_tokens, nle, max_recv, pre, part);
  }
  if (compact) R = min(R, compact_rows);
  Keys key;
  if constexpr (SMALL) key = Keys{my_excl, expert_meta, nle, 32, max_recv, compact};
  else key = Keys{pre, expert_meta, nle, top_step(nle), max_recv, compact};
  // buffer row of stream row g (wave-uniform g < R)
  auto padded_row = [&](int g) -> size_t {
    if (compact) return (size_t)g;
    int le, first;
    if constexpr (SMALL) {
      le = __popcll(__ballot(my_incl <= g));
      first = __builtin_amdgcn_readlane(my_excl, le);
    } else {
      le = expert_of(pre, nle, key.top, g);
      first = pre[le];
    }
    return (size_t)le * max_recv + (g - first);
  };

  if ((int)blockIdx.x < W) {
    const int me = blockIdx.x;
    int c = count_keys<64 * ROWS>(R, key, [me](int d, int) { return d == me; });
    c = block_sum<ROWS>(c, part);
    if (tid == 0) send_counts[me] = c;
    return;
  }

  const int groups = (R + ROWS - 1) / ROWS;
  const int items = groups * chunks, movers = gridDim.x - W;
  int parity = 0;
  for (int q = blockIdx.x - W; q < items; q += movers, ++parity) {
    const int grp = chunks == 1 ? q : q / chunks, c = q - grp * chunks;
    const int g0 = grp * ROWS, g = g0 + wave;
    const bool valid = g < R;
    const int base = c * (64 * NVW);

    // origin rank of every row of the group, read by every wave (no exchange)
    int rd[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) rd[r] = expert_meta[padded_row(min(g0 + r, R - 1)) * META + 1];
    const size_t row = padded_row(min(g, R - 1));
    int m = 0;
    if (c == 0 && lane < META) m = expert_meta[row * META + lane];
    RowsScan<Keys> scan(R, key);
    WavePayload<V, NVW> p;
    p.load(expert_y + row * row_vecs, base, row_vecs, lane);

    int cnt[ROWS];
    // origins compared as unsigned numbers: a row whose meta names no rank (negative, or W and
    // above) sorts behind the rows of every real origin instead of shifting their segments
    scan.finish(key, R, [&](int r, int d2, int g2) {
      return ((uint32_t)d2 < (uint32_t)rd[r]) | ((d2 == rd[r]) & (g2 < g0 + r));
    }, cnt);
    const int slot = rows_reduce(cnt, part, parity, wave, lane);

    if (valid && slot < capacity_rows) {
      p.template store<(MOE_A2A_NT_CSEND != 0)>(send_buf + (size_t)slot * row_vecs, base, row_vecs, lane);
      if (c == 0 && lane < META) send_meta[(size_t)slot * META + lane] = m;
    }
  }
}

// ---------------------------------------------------------------- 16-bit float helpers
//
// Element arithmetic works on 32-bit words holding two 16-bit elements (low
// half = even element), so that the gfx950 pair conversion v_cvt_pk_bf16_f32
// (round to nearest even) does the rounding of both in one instruction.
// A NaN keeps whatever payload the hardware gives it while it is being
// accumulated; bf16 results are canonicalised to 0x7fc0 (what torch stores for
// any NaN) where they are written out.

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <int DT> struct Pair16;
template <> struct Pair16<MOE_A2A_BF16> {
  static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  static __device__ __forceinline__ uint32_t round(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
  }
  static __device__ __forceinline__ uint32_t canonical(uint32_t w) {
    if ((w & 0x7fffu) > 0x7f80u) w = (w & 0xffff0000u) | 0x7fc0u;
    if ((w & 0x7fff0000u) > 0x7f800000u) w = (w & 0x0000ffffu) | 0x7fc00000u;
    return w;
  }
};
template <> struct Pair16<MOE_A2A_F16> {
  static __device__ __forceinline__ float lo(uint32_t w) {
    return (float)__builtin_bit_cast(f16x2, w).x;
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return (float)__builtin_bit_cast(f16x2, w).y;
  }
  static __device__ __forceinline__ uint32_t round(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, f16x2));
  }
  static __device__ __forceinline__ uint32_t canonical(uint32_t w) { return w; }
};

template <typename V> struct Words;  // 32-bit words (element pairs) per vector
template <> struct Words<b128> { static constexpr int N = 4; };
template <> struct Words<uint16_t> { static constexpr int N = 1; };  // one element, high half unused

template <typename V>
__device__ __forceinline__ uint32_t get_word(const V& v, int i) {
  if constexpr (Words<V>::N == 1) return v;
  else return v[i];
}

template <typename V>
__device__ __forceinline__ V from_words(const uint32_t* w) {
  if constexpr (Words<V>::N == 1) {
    return (uint16_t)w[0];
  } else {
    b128 v;
    v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
    return v;
  }
}

// ---------------------------------------------------------------- stage 4: combine, receive side

// A running row sum: two floats per word, each always exactly representable in
// the 16-bit type. step() is one `out[t] += row.float() * w` of the reference:
//   p = RN32(f32(v) * w);  a = RN32(acc + p);  acc = RN16(a)
template <int DT>
struct PairAcc {
  float lo, hi;
  __device__ __forceinline__ void set(uint32_t w) { lo = Pair16<DT>::lo(w); hi = Pair16<DT>::hi(w); }
  __device__ __forceinline__ void step(uint32_t v, float w) {
    const float a = __fadd_rn(lo, __fmul_rn(Pair16<DT>::lo(v), w));
    const float b = __fadd_rn(hi, __fmul_rn(Pair16<DT>::hi(v), w));
    set(Pair16<DT>::round(a, b));
  }
  __device__ __forceinline__ uint32_t word() const {
    return Pair16<DT>::canonical(Pair16<DT>::round(lo, hi));
  }
};

// Workgroup of BLK lanes per (token, chunk); each lane owns NV vector columns.
// The workgroup finds the rows addressed to its token by scanning the src_token
// column of the arriving meta rows, orders them by arrival index, then walks
// them in that order with all rows of a batch loaded up front.
//
// `hint_rows` rows of recv_meta are readable whatever the counts say: the first
// batch of the scan is loaded before the true row count R is known (the counts
// are loaded at the same time); rows at or past R are ignored.

// Long streams: every workgroup of a token scanning the whole arriving stream makes the meta
// reads grow with tokens x rows. return_map_kernel turns the stream into a table first: one
// thread per arriving row writes its row number at entry_row[src_token * K + src_k]. A token's
// workgroup then looks its K entries up instead of scanning (MAPPED below). An entry is taken
// only if the meta row it points to names this token and this k NOW, so whatever an earlier
// call left in the table can never be mistaken for an arrival; the table needs no clearing.
// The one assumption is that no (token, k) pair arrives twice, which holds for every stream
// the dispatch produced: with duplicates the table keeps one of them.
__global__ __launch_bounds__(BLOCK) void return_map_kernel(
    const int* __restrict__ recv_meta, const int* __restrict__ recv_counts, int W, int hint_rows,
    int capacity_rows, int T, int K, int* __restrict__ entry_row) {
  // the first row of a thread is loaded before the row count is known when it lies below the
  // readable bound (the counts travel at the same time)
  int i = blockIdx.x * BLOCK + threadIdx.x;
  int tk[2] = {-1, -1};
  bool loaded = i < hint_rows;
  if (loaded) __builtin_memcpy(tk, recv_meta + (size_t)i * META + 2, 8);
  const int R = min(sum_counts(recv_counts, W, capacity_rows), capacity_rows);
  for (; i < R; i += gridDim.x * BLOCK) {
    if (!loaded) __builtin_memcpy(tk, recv_meta + (size_t)i * META + 2, 8);
    loaded = false;
    if ((uint32_t)tk[0] < (uint32_t)T && (uint32_t)tk[1] < (uint32_t)K) entry_row[(size_t)tk[0] * K + tk[1]] = i;
  }
}

template <typename V, int DT, int BLK, int NV, bool MAPPED>
__global__ __launch_bounds__(BLK) void combine_recv_kernel(
    const V* __restrict__ recv_buf, const int* __restrict__ recv_meta,
    const int* __restrict__ recv_counts, int W, int hint_rows, int capacity_rows,
    const float* __restrict__ weights, int T, int K, int row_vecs, int chunks, V* __restrict__ out, int accumulate,
    const int* __restrict__ entry_row) {
  constexpr int N = Words<V>::N;
  constexpr int FAST = 8;  // addends ordered in registers
  __shared__ int hit_row[COMBINE_CAP], hit_k[COMBINE_CAP];
  __shared__ int ord_row[COMBINE_CAP];
  __shared__ float ord_w[COMBINE_CAP];
  __shared__ float wts[COMBINE_WEIGHTS];
  __shared__ int nhit;
  const int tid = threadIdx.x, lane = tid & 63;
  const int kw = min(K, COMBINE_WEIGHTS);
  const bool lanes_hold_counts = W <= 64;
  // in flight with the first batch of the scan (first_use)
  const int raw_count = recv_counts[min(lane, W - 1)];
  int R = -1;  // not known yet
  auto rows_arrived = [&] {
    const int my_count = lane < W ? min(max(first_use(raw_count), 0), capacity_rows) : 0;
    return min(lanes_hold_counts ? wave_sum(my_count) : sum_counts(recv_counts, W, capacity_rows), capacity_rows);
  };

  // rows [lo, hi) of the arriving stream: note the ones addressed to token t
  auto scan = [&](int t, int lo, int hi) {
    for (int b = lo; b < hi; b += SCAN_UNROLL * BLK) {
      int key[SCAN_UNROLL], kk[SCAN_UNROLL];
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) {
        // src_token and src_k with one 8-byte load (4-byte aligned, which global loads accept);
        // fetching src_k for the hits alone with a dependent load costs more than it saves
        int tk[2];
        __builtin_memcpy(tk, recv_meta + (size_t)min(b + tid + u * BLK, hi - 1) * META + 2, 8);
        key[u] = tk[0];
        kk[u] = tk[1];
      }
      if (R < 0) R = rows_arrived();
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) {
        const int row = b + tid + u * BLK;
        // (an arriving row whose k names no weight of the token is not an addend)
        if (row < min(hi, R) && key[u] == t && (uint32_t)kk[u] < (uint32_t)K) {
          const int p = atomicAdd(&nhit, 1);
          if (p < COMBINE_CAP) {
            hit_row[p] = row;
            hit_k[p] = kk[u];
          }
        }
      }
    }
  };

  const int items = T * chunks;
  for (int q = blockIdx.x; q < items; q += gridDim.x) {
    const int t = chunks == 1 ? q : q / chunks, c = q - t * chunks;
    const int base = c * (BLK * NV);
    V* __restrict__ orow = out + (size_t)t * row_vecs;

    // the token's weights travel to LDS while the scan's loads are in flight
    float wreg = 0.0f;
    if (tid < kw) wreg = weights[(size_t)t * K + tid];

    PairAcc<DT> acc[NV][N];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      V o{};
      if (accumulate) o = orow[min(base + j * BLK + tid, row_vecs - 1)];
#pragma unroll
      for (int e = 0; e < N; ++e) acc[j][e].set(get_word(o, e));
    }

    if (tid == 0) nhit = 0;
    lds_barrier();
    if constexpr (MAPPED) {
      if (R < 0) R = rows_arrived();
      for (int k = tid; k < K; k += BLK) {
        const int i = entry_row[(size_t)t * K + k];
        if ((uint32_t)i < (uint32_t)R) {
          int tk[2];
          __builtin_memcpy(tk, recv_meta + (size_t)i * META + 2, 8);
          if (tk[0] == t && tk[1] == k) {
            const int p = atomicAdd(&nhit, 1);
            if (p < COMBINE_CAP) {
              hit_row[p] = i;
              hit_k[p] = k;
            }
          }
        }
      }
    } else if (R < 0) {
      // first item: one batch below the readable bound goes out before R is known
      const int spec = min(hint_rows, SCAN_UNROLL * BLK);
      scan(t, 0, spec);
      if (R < 0) R = rows_arrived();
      scan(t, spec, R);
    } else {
      scan(t, 0, R);
    }
    if (tid < kw) wts[tid] = wreg;
    lds_barrier();
    const int n = nhit;

    if (n <= FAST && K <= COMBINE_WEIGHTS) {  // (every weight of the token is in LDS)
      if (n > 0) {
        // Order the (at most 8) hits by arrival index. Lane l of every wave takes hit l % 8; its
        // place in the order is the number of hits that arrived earlier, counted with seven
        // rotations of a 16-lane DPP row (lanes 8..15 of a row hold the same eight hits again, so
        // rotating by 1..7 shows a lane every other hit once). Each lane then pushes its hit to
        // the lane of its place, and the ordered rows and weights are read lane by lane into
        // scalar registers. About 45 vector instructions per wave; a sorting network on the
        // hits as uniform values becomes some 150 scalar instructions, and the sixteen waves of a
        // compute unit share one scalar unit.
        const int p = lane & (FAST - 1);
        const int hr = p < n ? hit_row[p] : INT_MAX;
        const int hk = p < n ? hit_k[p] : 0;  // (0 <= k < K: checked when the hit was noted)
        const float hw = wts[hk];
        int place = 0;
#define MOE_A2A_ROT(S) place += (int)(__builtin_amdgcn_update_dpp(0, hr, 0x120 + S, 0xf, 0xf, false) < hr)
        MOE_A2A_ROT(1); MOE_A2A_ROT(2); MOE_A2A_ROT(3); MOE_A2A_ROT(4); MOE_A2A_ROT(5); MOE_A2A_ROT(6); MOE_A2A_ROT(7);
#undef MOE_A2A_ROT
        // (lanes without a hit all get place n, which nothing reads)
        const int to = ((lane & ~(FAST - 1)) | place) << 2;
        const int ordered_row = __builtin_amdgcn_ds_permute(to, hr);
        const int ordered_w = __builtin_amdgcn_ds_permute(to, __float_as_int(hw));
        V v[FAST][NV];
        float w[FAST];
#pragma unroll
        for (int u = 0; u < FAST; ++u) {
          // row 0 exists (n > 0): loaded for the places past n and not used
          const int row = u < n ? __builtin_amdgcn_readlane(ordered_row, u) : 0;
          w[u] = __int_as_float(__builtin_amdgcn_readlane(ordered_w, u));
#pragma unroll
          for (int j = 0; j < NV; ++j)
            v[u][j] = recv_buf[(size_t)row * row_vecs + min(base + j * BLK + tid, row_vecs - 1)];
        }
#pragma unroll
        for (int u = 0; u < FAST; ++u) {
          if (u < n) {
#pragma unroll
            for (int j = 0; j < NV; ++j)
#pragma unroll
              for (int e = 0; e < N; ++e) acc[j][e].step(get_word(v[u][j], e), w[u]);
          }
        }
      }
    } else if (n <= COMBINE_CAP) {
      if (tid < n) {  // order the hits by arrival index
        const int me = hit_row[tid];
        int r = 0;
        for (int b = 0; b < n; ++b) r += hit_row[b] < me;
        const int k = hit_k[tid];
        const bool ok = (k >= 0) & (k < K);
        ord_row[r] = ok ? me : -1;
        ord_w[r] = !ok ? 0.0f : k < kw ? wts[k] : weights[(size_t)t * K + k];
      }
      lds_barrier();
      for (int a0 = 0; a0 < n; a0 += COMBINE_BATCH) {
        V v[COMBINE_BATCH][NV];
#pragma unroll
        for (int u = 0; u < COMBINE_BATCH; ++u) {
          // clamped, unconditional loads keep the whole batch in flight
          const int row = max(ord_row[min(a0 + u, n - 1)], 0);
#pragma unroll
          for (int j = 0; j < NV; ++j)
            v[u][j] = recv_buf[(size_t)row * row_vecs + min(base + j * BLK + tid, row_vecs - 1)];
        }
#pragma unroll
        for (int u = 0; u < COMBINE_BATCH; ++u) {
          if (a0 + u < n && ord_row[a0 + u] >= 0) {
            const float w = ord_w[a0 + u];
#pragma unroll
            for (int j = 0; j < NV; ++j)
#pragma unroll
              for (int e = 0; e < N; ++e) acc[j][e].step(get_word(v[u][j], e), w);
          }
        }
      }
    } else {
      // More addends than the LDS list holds: walk the stream in order.
      for (int i = 0; i < R; ++i) {
        if (recv_meta[(size_t)i * META + 2] != t) continue;
        const int k = recv_meta[(size_t)i * META + 3];
        if (k < 0 || k >= K) continue;
        const float w = weights[(size_t)t * K + k];
#pragma unroll
        for (int j = 0; j < NV; ++j) {
          const int idx = base + j * BLK + tid;
          if (idx < row_vecs) {
            const V v = recv_buf[(size_t)i * row_vecs + idx];
#pragma unroll
            for (int e = 0; e < N; ++e) acc[j][e].step(get_word(v, e), w);
          }
        }
      }
    }

#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int idx = base + j * BLK + tid;
      if (idx < row_vecs) {
        uint32_t h[N];
#pragma unroll
        for (int e = 0; e < N; ++e) h[e] = acc[j][e].word();
        orow[idx] = from_words<V>(h);
      }
    }
    lds_barrier();  // the LDS lists are reused by the next item
  }
}

// ---------------------------------------------------------------- simulated expert

template <typename V, int NV, int DIN, int DOUT>
__global__ __launch_bounds__(BLOCK) void expert_scale_kernel(
    const V* __restrict__ expert_x, const int* __restrict__ expert_num_tokens, int nle,
    int max_recv, float scale, int row_vecs, int chunks, V* __restrict__ expert_y, int compact_rows) {
  __shared__ int red[NWAVES];
  __shared__ int pre[MAX_LOCAL_EXPERTS + 1];
  // compact_rows > 0: the experts' rows lie back to back in buffers of that many rows (= max_recv)
  int R = expert_prefix<NWAVES>(expert_num_tokens, nle, max_recv, pre, red);
  if (compact_rows > 0) R = min(R, compact_rows);
  const int top = top_step(nle);
  const int items = R * chunks;
  for (int q = blockIdx.x; q < items; q += gridDim.x) {
    const int g = chunks == 1 ? q : q / chunks, c = q - g * chunks;
    const int base = c * (BLOCK * NV);
    const int le = compact_rows > 0 ? 0 : expert_of(pre, nle, top, g);
    const size_t row = compact_rows > 0 ? (size_t)g : (size_t)le * max_recv + (g - pre[le]);
    Payload<V, NV> p;
    p.load(expert_x + row * row_vecs, base, row_vecs);
    p.map([scale](V v) {
      constexpr int N = Words<V>::N;
      uint32_t h[N];
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const uint32_t w = get_word(v, e);
        // .to(out_dtype), then times (1 + rank) in float32, rounded once
        const uint32_t o = Pair16<DOUT>::round(Pair16<DIN>::lo(w), Pair16<DIN>::hi(w));
        const float lo = rounded_here(__fmul_rn(Pair16<DOUT>::lo(o), scale));
        const float hi = rounded_here(__fmul_rn(Pair16<DOUT>::hi(o), scale));
        h[e] = Pair16<DOUT>::canonical(Pair16<DOUT>::round(lo, hi));
      }
      return from_words<V>(h);
    });
    p.store(expert_y + row * row_vecs, base, row_vecs);
  }
}

// The same for at most 64 local experts and 16-byte vectors: a wave per (row,
// chunk of 64 * NVW vectors), the expert prefix in one register per lane, the
// row found with one ballot. No LDS table, no barrier.
template <int NVW, int DIN, int DOUT>
__global__ __launch_bounds__(64 * ROWS) void expert_scale_wave_kernel(
    const b128* __restrict__ expert_x, const int* __restrict__ expert_num_tokens, int nle,
    int max_recv, float scale, int row_vecs, int chunks, b128* __restrict__ expert_y, int compact_rows) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const WaveExpertPrefix wp(expert_num_tokens, nle, max_recv);
  const int R = compact_rows > 0 ? min(wp.total, compact_rows) : wp.total;
  const int items = R * chunks, waves = gridDim.x * ROWS;
  for (int q = blockIdx.x * ROWS + wave; q < items; q += waves) {
    const int g = chunks == 1 ? q : q / chunks, c = q - g * chunks;
    const int base = c * (64 * NVW);
    int le, first;
    wp.locate(g, le, first);
    const size_t row = compact_rows > 0 ? (size_t)g : (size_t)le * max_recv + (g - first);
    WavePayload<b128, NVW> p;
    p.load(expert_x + row * row_vecs, base, row_vecs, lane);
#pragma unroll
    for (int j = 0; j < NVW; ++j) {
      uint32_t h[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t w = p.v[j][e];
        // .to(out_dtype), then times (1 + rank) in float32, rounded once
        const uint32_t o = Pair16<DOUT>::round(Pair16<DIN>::lo(w), Pair16<DIN>::hi(w));
        const float lo = rounded_here(__fmul_rn(Pair16<DOUT>::lo(o), scale));
        const float hi = rounded_here(__fmul_rn(Pair16<DOUT>::hi(o), scale));
        h[e] = Pair16<DOUT>::canonical(Pair16<DOUT>::round(lo, hi));
      }
      p.v[j] = from_words<b128>(h);
    }
    p.template store<(MOE_A2A_NT_STANDIN != 0)>(expert_y + row * row_vecs, base, row_vecs, lane);
  }
}

// ---------------------------------------------------------------- expert computation: grouped GEMM
//
// expert_y[le, j, :] = expert_x[le, j, :] @ W[le]^T for the valid rows j < expert_num_tokens[le] of
// the padded expert-major buffers: what stands where all2all/reference.py:262 has the simulated
// expert. W[le] is [H_out = H, H_in = H] with the input index contiguous (the layout of a linear
// layer's weight).
//
// With a few dozen rows per expert the problem is bound by streaming the weights (C4: 3.3 GB of
// them for 0.2 PFLOP), so the kernel is built to keep weight bytes in flight and to ask for them in
// whole cache lines. A workgroup of GW waves (4, or 5 to 8 for blocks of 128 tokens) owns GW * 32
// output columns x one block of TJ*32 tokens of one expert; a wave owns 32 of the columns for all
// tokens of the block (TJ tiles of
// v_mfma_f32_32x32x16, fp32 accumulators in registers) and walks the input dimension 64 elements
// (128 bytes of every row) at a time.
//
// Weights: the MFMA wants a lane to hold inputs of ONE output column, which read from memory as
// it lies makes every load instruction touch 32 different lines, a quarter of each (measured: 4.0
// TB/s against 5.6 with the same bytes requested line by line). So a wave loads its 32 x 128 bytes
// of a step with 8 lanes per line, drops them into 4 KB of LDS of its own, and picks the operands
// up from there in MFMA layout. No barrier is involved: a wave's LDS operations execute in order.
// Tokens: the rows of the block are what the waves share. Each step's 128 bytes of every token
// are loaded once per workgroup, parked in LDS and read from there by all of them: one LDS barrier per
// step. Both kinds of loads are issued DEPTH steps ahead of their use; the vector memory counter
// retires in order, so the token loads run one step ahead of the weights: waiting for the tokens
// that are parked next never waits for the weights issued after them.
// LDS layout of both: row-major 128-byte rows, the eight 16-byte vectors of a row XORed with bits
// 1..3 of the row number, which makes the parking writes (8 lanes per row) and the operand reads
// (16 rows, same vector) hit all 64 banks once per 16 lanes.
//
// The MFMA computes the tile transposed (weights as the A operand, tokens as B), which leaves a lane
// holding four consecutive output columns of one token: 8-byte stores. MFMA q of a step takes inputs
// 16 q .. 16 q + 15 of the step (a lane's half kb of them: the 16-byte vector 2 q + kb of the row), the
// order in which dense_gemm_kernel walks K too: which of the two kernels a row count selects changes no
// bit of the result.
//
// Tiles are numbered over (expert, block of tokens) by a prefix over the device-side counts, so a
// hot expert is spread over as many workgroups as it has blocks and an empty one costs nothing.
// Every block of an expert re-reads the expert's weights: TJ = 4 (128 tokens) is used when the
// caller's row count says blocks of 64 would not hold most experts.

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int DT> struct Mfma32x32x16;
template <> struct Mfma32x32x16<MOE_A2A_BF16> {
  static __device__ __forceinline__ f32x16 mma(b128 a, b128 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mfma32x32x16<MOE_A2A_F16> {
  static __device__ __forceinline__ f32x16 mma(b128 a, b128 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
};

#ifndef MOE_A2A_GEMM_OCC
#define MOE_A2A_GEMM_OCC 3
#endif
#ifndef MOE_A2A_GEMM_OCC4
#define MOE_A2A_GEMM_OCC4 2  // workgroups per compute unit with blocks of 128 tokens
#endif
#ifndef MOE_A2A_GEMM_DEPTH
#define MOE_A2A_GEMM_DEPTH 2
#endif
constexpr int BUFFER_RAW_32BIT = 0x00020000;  // word 3 of a gfx9 buffer descriptor: raw buffer of 32-bit data
constexpr int GEMM_COLS = 128;   // output columns per workgroup, 32 per wave
constexpr int GEMM_KSTEP = 64;   // input elements per step: 8 vectors of 16 bytes per row
#ifndef MOE_A2A_GEMM_DEPTH4
#define MOE_A2A_GEMM_DEPTH4 3  // with blocks of 128 tokens (two workgroups per unit: 655 against 675 us at C4)
#endif
constexpr int GEMM_DEPTH = MOE_A2A_GEMM_DEPTH;  // steps between a load and its use

// x [groups, max_rows, K], w [groups, N, K], bias [groups, N] or null, y [groups, max_rows, N];
// rows_of_group null: every group has max_rows rows (a plain dense product when groups == 1).
// GW waves per workgroup, 32 output columns each: every workgroup of an expert pulls the expert's
// token rows through its own L1, so wider workgroups halve that traffic (GW = 8: one workgroup of
// 512 lanes per compute unit instead of two of 256).
template <int DT, int TJ, int GW>
__global__ __launch_bounds__(64 * GW, GW > 4 ? 1 : TJ <= 2 ? MOE_A2A_GEMM_OCC : MOE_A2A_GEMM_OCC4) void expert_gemm_kernel(
    const b128* __restrict__ expert_x, const int* __restrict__ expert_num_tokens,
    const b128* __restrict__ weights, const uint16_t* __restrict__ bias, uint16_t* __restrict__ expert_y,
    int nle, int max_recv, int N, int K, int col_tiles, int compact) {
  constexpr int TOK = TJ * 32;               // tokens per block
  constexpr int D = TJ >= 4 ? MOE_A2A_GEMM_DEPTH4 : GEMM_DEPTH;
  __shared__ b128 xs[D][TOK * 8];            // D steps of TOK tokens x 8 vectors
  constexpr int THREADS = 64 * GW;
  // the token rows of a step are fetched and parked by all lanes when their number divides the
  // block's vectors, else by the first four waves
  constexpr int LOADERS = (TOK * 8) % THREADS == 0 ? THREADS : 256;
  constexpr int XL = TOK * 8 / LOADERS;       // token loads of a loading lane per step (LOADERS / 8 rows each)
  static_assert(XL >= 1 && XL * LOADERS == TOK * 8 && LOADERS <= THREADS, "whole loads");
  __shared__ b128 ws[GW][32 * 8];            // per wave: one step of its 32 weight rows x 8 vectors
  __shared__ int red[GW], red_rows[GW];
  __shared__ int home[4];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int row_vecs = K / 8, steps = (K + GEMM_KSTEP - 1) / GEMM_KSTEP;
  const int tail_vecs = row_vecs - (steps - 1) * 8;  // vectors of a row in the last step, 1..8
  auto rows_of = [=](int le) { return expert_num_tokens ? min(max(expert_num_tokens[le], 0), max_recv) : max_recv; };

  // Blocks of tokens per expert, summed over the run of experts this thread owns and scanned over
  // the workgroup: block number g of the launch belongs to the thread with begin <= g < begin + mine.
  const int per = (nle + THREADS - 1) / THREADS;
  const int run_b = min(tid * per, nle), run_e = min(run_b + per, nle);
  // compact: x and y hold the experts' rows back to back in buffers of max_recv rows. The rows
  // ahead of an expert are a prefix over the counts, and an expert only has the rows that still
  // fit the buffers (counts that add up to more never send a load or a store past their end).
  int mine_rows = 0;
  for (int le = run_b; le < run_e; ++le) mine_rows += rows_of(le);
  int rows_begin;
  {
    const int inc_rows = wave_inclusive_scan(mine_rows);
    if (lane == 63) red_rows[wave] = inc_rows;
    lds_barrier();
    int off_rows = 0;
#pragma unroll
    for (int w = 0; w < GW; ++w) off_rows += w < wave ? red_rows[w] : 0;
    rows_begin = off_rows + inc_rows - mine_rows;
  }
  // rows of expert le that are there: all of them in the padded layout
  auto kept_of = [=](int le, int ahead) {
    const int n = rows_of(le);
    return compact ? min(ahead + n, max_recv) - min(ahead, max_recv) : n;
  };
  auto blocks_for = [=](int rows) { return (rows + TOK - 1) / TOK; };
  int mine = 0;
  for (int le = run_b, ahead = rows_begin; le < run_e; ahead += rows_of(le), ++le) mine += blocks_for(kept_of(le, ahead));
  int begin, row_blocks;
  {
    const int inc = wave_inclusive_scan(mine);
    if (lane == 63) red[wave] = inc;
    lds_barrier();
    int off = 0, total = 0;
#pragma unroll
    for (int w = 0; w < GW; ++w) {
      off += w < wave ? red[w] : 0;
      total += red[w];
    }
    begin = off + inc - mine;
    row_blocks = total;
  }

  // Loads are 8 lanes per 128-byte row: lane l of a wave takes row l/8 (+ 8 per further load) and
  // the vector of that row that belongs in physical slot l%8.
  const int sub = lane >> 3, slot = lane & 7;
  // operand reads: row r of the tile, logical vector 2*q + kb of the step (q: the MFMA, kb: the lane's half)
  const int r = lane & 31, kb = lane >> 5, read_swz = (r >> 1) & 7;

  const int tiles = row_blocks * col_tiles, stride = gridDim.x;
  for (int tile = blockIdx.x; tile < tiles; tile += stride) {
    const int rb = tile / col_tiles, ct = tile - rb * col_tiles;
    if (begin <= rb && rb < begin + mine) {  // one thread: walk its run to the expert of block rb
      int le = run_b, first = begin, rows_ahead = rows_begin;
      for (;; ++le) {
        const int n = blocks_for(kept_of(le, rows_ahead));
        if (rb < first + n) break;
        first += n;
        rows_ahead += rows_of(le);
      }
      home[0] = le;
      home[1] = first;
      home[2] = min(rows_ahead, max_recv);
      home[3] = kept_of(le, rows_ahead);
    }
    lds_barrier();  // (the next write to `home` comes after the barriers of the steps below)
    // (uniform values are pinned to scalar registers: the bases below then cost no vector registers)
    const int le = __builtin_amdgcn_readfirstlane(home[0]);
    const int rows = __builtin_amdgcn_readfirstlane(home[3]);
    const int t0 = (rb - __builtin_amdgcn_readfirstlane(home[1])) * TOK;  // first token of the block (t0 < rows)
    // buffer row of the expert's first row
    const size_t row0 = compact ? (size_t)__builtin_amdgcn_readfirstlane(home[2]) : (size_t)le * max_recv;
    const int n0 = ct * (GW * 32) + __builtin_amdgcn_readfirstlane(wave) * 32;  // first output column of this wave
    const bool cols_valid = n0 < N;                      // the last tile of columns may be partly empty
    const int nw = min(n0, N - 32);                      // (a wave without columns reads valid memory)

    // weights: load i takes rows sub + 8*i of the wave's 32; tokens: load i takes tokens tid/8 + 32*i.
    // Both go through buffer descriptors (base and extent in scalar registers, a 32-bit byte offset
    // per lane, the step's offset as the scalar operand). The extent of the token buffer ends with
    // the expert's last valid row: lanes that would load tokens past it get zeros and cause no
    // traffic. Tiles of 32 tokens with no valid token are skipped altogether. When K is not a
    // multiple of 64, the lanes that hold vectors past the end of a row in the last step are sent
    // out of range there the same way (both operands: a zero times a stray NaN would not be zero).
    const int live = rows - t0;  // valid tokens of this block, > 0
    const int row_bytes = K * 2;
    const __amdgpu_buffer_rsrc_t wbuf = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(weights + ((size_t)le * N + nw) * row_vecs), 0, 32 * row_bytes, BUFFER_RAW_32BIT);
    const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(expert_x + (row0 + t0) * row_vecs), 0, min(live, TOK) * row_bytes, BUFFER_RAW_32BIT);
    constexpr int OUT_OF_RANGE = 0x40000000;
    int woff[4], wslot[4], xoff[XL], wpast[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = sub + 8 * i, vec = slot ^ ((row >> 1) & 7);
      woff[i] = row * row_bytes + vec * 16;
      wslot[i] = row * 8 + slot;
      if (i < 2) wpast[i] = vec >= tail_vecs ? OUT_OF_RANGE : 0;  // (loads i and i + 2 take the same vector)
    }
    constexpr int XROWS = LOADERS / 8;  // token rows one load of the workgroup covers: 32 or 64
    const bool loader = LOADERS == THREADS || tid < LOADERS;  // (whole waves)
    const int xrow = tid >> 3, xvec = slot ^ ((xrow >> 1) & 7);  // (XROWS * i does not change bits 1..3)
    const int xpast = xvec >= tail_vecs ? OUT_OF_RANGE : 0;
#pragma unroll
    for (int i = 0; i < XL; ++i) xoff[i] = (xrow + XROWS * i) * row_bytes + xvec * 16;

    f32x16 acc[TJ] = {};
    b128 wv[D][4], xv[D][XL];
    auto load_w = [&](int set, int step) {
      const int at = min(step, steps - 1);  // past the end: the last step again, unused
      const bool last = at == steps - 1;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        wv[set][i] = __builtin_amdgcn_raw_buffer_load_b128(wbuf, woff[i] + (last ? wpast[i & 1] : 0),
                                                           at * (GEMM_KSTEP * 2), 0);
    };
    auto load_x = [&](int set, int step) {
      const int at = min(step, steps - 1);
      const bool last = at == steps - 1;
      // (load i holds tokens XROWS * i .. of the block: a load without a valid token is neither
      // issued nor parked, and a tile of 32 tokens without one is not multiplied)
#pragma unroll
      for (int i = 0; i < XL; ++i)
        if (loader && i * XROWS < live)
          xv[set][i] = __builtin_amdgcn_raw_buffer_load_b128(xbuf, xoff[i] + (last ? xpast : 0),
                                                             at * (GEMM_KSTEP * 2), 0);
    };
    auto park_x = [&](int set) {
#pragma unroll
      for (int i = 0; i < XL; ++i)
        if (loader && i * XROWS < live) xs[set][tid + LOADERS * i] = xv[set][i];
    };
    auto compute = [&](int set) {
#pragma unroll
      for (int i = 0; i < 4; ++i) ws[wave][wslot[i]] = wv[set][i];
      b128 a[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) a[q] = ws[wave][r * 8 + ((q * 2 + kb) ^ read_swz)];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
          if (j * 32 < live) {
            const b128 tok = xs[set][(j * 32 + r) * 8 + ((q * 2 + kb) ^ read_swz)];
            acc[j] = Mfma32x32x16<DT>::mma(a[q], tok, acc[j]);
          }
        }
    };
    auto step = [&](int u, int at) {  // step `at`, which lives in register set and LDS buffer u = at % D
      compute(u);
      load_w(u, at + D);
      park_x((u + 1) % D);            // step at + 1, loaded one step before the weights now in flight
      load_x((u + 1) % D, at + 1 + D);
      lds_barrier();
    };

#pragma unroll
    for (int i = 0; i < D; ++i) {
      load_x(i, i);
      load_w(i, i);
    }
    park_x(0);
    load_x(0, D);
    lds_barrier();
    // D steps per trip, so that the register sets have fixed names in the loop body; the last
    // steps % D are peeled (inside the loop they would be paths on which set 0 follows set 0, and
    // the compiler would have to wait for the weights as if that happened)
    int at = 0;
    for (; at + D <= steps; at += D) {
#pragma unroll
      for (int u = 0; u < D; ++u) step(u, at + u);
    }
#pragma unroll
    for (int u = 0; u < D - 1; ++u)
      if (at + u < steps) step(u, at + u);

    // D[n][token] of a 32x32 tile: this lane holds token r and output columns g*8 + kb*4 + 0..3, g < 4.
    // With a bias the sum is rounded to the 16-bit type first and the bias added to that, as
    // `matmul(x, w.T) + bias` on 16-bit tensors does (gemm-rs/reference.py:54-57).
    if (cols_valid) {
      uint32_t bias2[4][2] = {};
      if (bias) {
#pragma unroll
        for (int g = 0; g < 4; ++g) __builtin_memcpy(bias2[g], bias + (size_t)le * N + n0 + kb * 4 + g * 8, 8);
      }
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
        const int token = t0 + j * 32 + r;
        if (token < rows) {
          uint16_t* out = expert_y + (row0 + token) * N + n0 + kb * 4;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x16& c = acc[j];
            uint32_t two[2] = {Pair16<DT>::canonical(Pair16<DT>::round(c[g * 4 + 0], c[g * 4 + 1])),
                               Pair16<DT>::canonical(Pair16<DT>::round(c[g * 4 + 2], c[g * 4 + 3]))};
            if (bias) {
#pragma unroll
              for (int h = 0; h < 2; ++h)
                two[h] = Pair16<DT>::canonical(Pair16<DT>::round(
                    __fadd_rn(Pair16<DT>::lo(two[h]), Pair16<DT>::lo(bias2[g][h])),
                    __fadd_rn(Pair16<DT>::hi(two[h]), Pair16<DT>::hi(bias2[g][h]))));
            }
            __builtin_memcpy(out + g * 8, two, 8);
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------- product with few rows
//
// Y[M, N] = X[M, K] @ W[N, K]^T for at most 64 rows: the weights are streamed once and no tile
// shape gives every compute unit work (M = 64, N = 7168: 56 tiles of 128 columns). Here a
// workgroup owns only 32 output columns x one block of 32 or 64 tokens, and its KW waves (four,
// eight for long K) split K: wave w takes steps w, w + KW, ... of 64 elements, streams
// its own slices of the 32 weight rows and of the token rows (both 8 lanes per 128-byte line,
// turned into MFMA layout through LDS private to the wave: no barrier in the loop), and keeps
// partial sums in registers. At the end the partial sums meet in LDS and are added in a fixed
// order (wave 0 + 1 + 2 + ...), so results do not depend on scheduling.

template <int DT, int TJ, int KW>
__global__ __launch_bounds__(64 * KW) void skinny_gemm_kernel(
    const b128* __restrict__ X, const b128* __restrict__ Wt, const uint16_t* __restrict__ bias,
    uint16_t* __restrict__ Y, int M, int N, int K, int col_units) {
  constexpr int TOK = TJ * 32;
  constexpr int XL = TJ * 4;  // token loads per lane and step: TOK rows x 8 vectors over 64 lanes
  extern __shared__ b128 skinny_lds[];  // per wave: 32 weight rows, then TOK token rows, of 8 vectors
  b128(*wsl)[32 * 8] = reinterpret_cast<b128(*)[32 * 8]>(skinny_lds);
  b128(*xsl)[TOK * 8] = reinterpret_cast<b128(*)[TOK * 8]>(skinny_lds + KW * 32 * 8);
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int row_vecs = K / 8, row_bytes = K * 2, steps = (K + GEMM_KSTEP - 1) / GEMM_KSTEP;
  const int tail_vecs = row_vecs - (steps - 1) * 8;
  const int rb = blockIdx.x / col_units, cu = blockIdx.x - rb * col_units;
  const int t0 = rb * TOK, n0 = cu * 32, live = M - t0;

  const __amdgpu_buffer_rsrc_t wbuf = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(Wt + (size_t)n0 * row_vecs), 0, 32 * row_bytes, BUFFER_RAW_32BIT);
  const __amdgpu_buffer_rsrc_t xbuf = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(X + (size_t)t0 * row_vecs), 0, min(live, TOK) * row_bytes, BUFFER_RAW_32BIT);
  constexpr int OUT_OF_RANGE = 0x40000000;
  // load i of a lane: row sub + 8 * i, the vector that belongs in physical slot `slot` of that row
  const int sub = lane >> 3, slot = lane & 7;
  auto vec_of = [&](int row) { return slot ^ ((row >> 1) & 7); };
  const int r = lane & 31, kb = lane >> 5, read_swz = (r >> 1) & 7;

  f32x16 acc[TJ] = {};
  b128 wv[2][4], xv[2][XL];
  auto load = [&](int set, int step) {
    const int at = min(step, steps - 1);  // past the end: the last step again, unused
    const bool last = at == steps - 1;
    const int soff = at * (GEMM_KSTEP * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = sub + 8 * i, vec = vec_of(row);
      wv[set][i] = __builtin_amdgcn_raw_buffer_load_b128(
          wbuf, row * row_bytes + vec * 16 + (last && vec >= tail_vecs ? OUT_OF_RANGE : 0), soff, 0);
    }
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      const int row = sub + 8 * i, vec = vec_of(row);
      xv[set][i] = __builtin_amdgcn_raw_buffer_load_b128(
          xbuf, row * row_bytes + vec * 16 + (last && vec >= tail_vecs ? OUT_OF_RANGE : 0), soff, 0);
    }
  };
  auto compute = [&](int set) {
#pragma unroll
    for (int i = 0; i < 4; ++i) wsl[wave][(sub + 8 * i) * 8 + slot] = wv[set][i];
#pragma unroll
    for (int i = 0; i < XL; ++i) xsl[wave][(sub + 8 * i) * 8 + slot] = xv[set][i];
    b128 a[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) a[q] = wsl[wave][r * 8 + ((kb * 4 + q) ^ read_swz)];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int j = 0; j < TJ; ++j) {
        if (j * 32 < live) {
          const b128 tok = xsl[wave][(j * 32 + r) * 8 + ((kb * 4 + q) ^ read_swz)];
          acc[j] = Mfma32x32x16<DT>::mma(a[q], tok, acc[j]);
        }
      }
  };

  load(0, wave);
  load(1, wave + KW);
  for (int s = wave; s < steps; s += 2 * KW) {
    compute(0);
    load(0, s + 2 * KW);
    if (s + KW < steps) compute(1);
    load(1, s + 3 * KW);
  }

  // partial sums to LDS (a wave's region holds exactly its TJ x 16 floats per lane), then wave j
  // adds up token tile j in the order of the waves and writes it out
  float* mine = reinterpret_cast<float*>(xsl[wave]);
#pragma unroll
  for (int j = 0; j < TJ; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) mine[(j * 16 + e) * 64 + lane] = acc[j][e];
  __syncthreads();
  if (wave < TJ && wave * 32 < live) {
    const int j = wave;
    float c[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      float sum = reinterpret_cast<const float*>(xsl[0])[(j * 16 + e) * 64 + lane];
#pragma unroll
      for (int w = 1; w < KW; ++w)
        sum = __fadd_rn(sum, reinterpret_cast<const float*>(xsl[w])[(j * 16 + e) * 64 + lane]);
      c[e] = sum;
    }
    // this lane: token r of tile j, output columns n0 + g*8 + kb*4 + 0..3, g < 4
    const int token = t0 + j * 32 + r;
    if (token < M) {
      uint16_t* out = Y + (size_t)token * N + n0 + kb * 4;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        uint32_t two[2] = {Pair16<DT>::canonical(Pair16<DT>::round(c[g * 4 + 0], c[g * 4 + 1])),
                           Pair16<DT>::canonical(Pair16<DT>::round(c[g * 4 + 2], c[g * 4 + 3]))};
        if (bias) {
          uint32_t b2[2];
          __builtin_memcpy(b2, bias + n0 + kb * 4 + g * 8, 8);
#pragma unroll
          for (int h = 0; h < 2; ++h)
            two[h] = Pair16<DT>::canonical(Pair16<DT>::round(
                __fadd_rn(Pair16<DT>::lo(two[h]), Pair16<DT>::lo(b2[h])),
                __fadd_rn(Pair16<DT>::hi(two[h]), Pair16<DT>::hi(b2[h]))));
        }
        __builtin_memcpy(out + g * 8, two, 8);
      }
    }
  }
}

// ---------------------------------------------------------------- dense product (many rows)
//
// C[M, N] = A[M, K] @ B[N, K]^T for thousands of rows: bound by the matrix cores, not by memory,
// so the kernel is built around operand reuse. A workgroup owns a BM x BN tile of C (256 x 256
// with four waves: a wave owns 128 x 128, sixteen 32 x 32 MFMA tiles, 256 accumulator registers,
// one wave per SIMD) and walks K in steps of 64 elements. Per step the workgroup copies BM + BN
// rows of 128 bytes into LDS once (through registers, two LDS buffers, one barrier per step), and
// every wave reads each operand fragment it needs once per 16-element slice of the step for a
// whole row or column of its MFMA tiles: 8 LDS reads for 16 MFMAs, issued one slice ahead.
// With one wave per SIMD nothing hides a wave's own stalls, so the loop body is laid out by hand
// (sched_group_barrier): exactly one memory instruction between two MFMAs, and every slice of a
// step carries the same mix (8 fragment reads, 4 LDS stores, 4 global loads). Sixteen loads or
// stores issued back to back make the wave wait for the queues of the memory pipes, which its
// three neighbours fill at the same moment, and the matrix core idles meanwhile (measured at
// 8192 x 8192 x 3584: 587 us -> 482 us with the interleaving, -> 466 us with the even mix).
// LDS rows are 128 bytes with the eight 16-byte vectors of a row XORed with bits 1..3 of the
// row number (reads of 32 rows at one vector hit every bank equally); a thread stores linearly and
// picks the global vector that belongs at its place, so the stores are conflict-free too.
// The tile is computed transposed (B rows as the first MFMA operand): a lane then holds four
// consecutive columns of one row of C.
// Tiles are numbered so that each XCD (blockIdx % 8) works on a run of consecutive tile numbers,
// and consecutive numbers walk GROUP_M tile rows down before they step to the next tile column:
// the 32 workgroups an XCD runs at a time share 4 row panels of A and 8 of B in its L2.

template <int DT, int WM, int WN, int TM, int TN, bool GROUPED>
__global__ __launch_bounds__(64 * WM * WN, TM * TN >= 16 ? 1 : 2) void dense_gemm_kernel(
    const b128* __restrict__ A, const b128* __restrict__ B, const uint16_t* __restrict__ bias,
    uint16_t* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
    const int* __restrict__ rows_of_group, int groups, int max_rows, int compact) {
  constexpr int NT = 64 * WM * WN, BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int LA = BM * 8 / NT, LB = BN * 8 / NT;  // 16-byte vectors a thread copies per step
  constexpr int GROUP_M = 4;
  extern __shared__ b128 tile_lds[];  // [2][(BM + BN) * 8]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = __builtin_amdgcn_readfirstlane(wave / WN), wn = __builtin_amdgcn_readfirstlane(wave % WN);
  const int row_vecs = K / 8, row_bytes = K * 2, steps = (K + GEMM_KSTEP - 1) / GEMM_KSTEP;
  const int tail_vecs = row_vecs - (steps - 1) * 8;

  // GROUPED: A is [groups, max_rows, K], B [groups, N, K], bias [groups, N] or null, C [groups,
  // max_rows, N], and group g has rows_of_group[g] rows (read here, clamped to max_rows). Row
  // tiles are numbered over the groups by a prefix over their counts: every thread sums the row
  // tiles of a run of groups, a scan over the workgroup places the runs, and the thread whose run
  // holds a row tile walks it to find the group. The launch strides over (row tile, column tile)
  // pairs, column tile fastest, so its size is a matter of speed only.
  __shared__ int grp_red[NT / 64], grp_red_rows[NT / 64];
  __shared__ int grp_home[4];
  [[maybe_unused]] auto rows_of = [=](int g) { return min(max(rows_of_group[g], 0), max_rows); };
  // compact: A and C hold the groups' rows back to back in buffers of max_rows rows. The rows
  // ahead of a group are a prefix over the counts, and a group only has the rows that still fit
  // the buffers (counts that add up to more never send a load or a store past their end).
  [[maybe_unused]] auto kept_of = [=](int g, int ahead) {
    const int n = rows_of(g);
    return compact ? min(ahead + n, max_rows) - min(ahead, max_rows) : n;
  };
  [[maybe_unused]] auto tiles_for = [=](int rows) { return (rows + BM - 1) / BM; };
  [[maybe_unused]] int run_first = 0, run_end = 0, run_begin = 0, run_tiles = 0, total_tiles = 0, run_rows_begin = 0;
  if constexpr (GROUPED) {
    const int per = (groups + NT - 1) / NT;
    run_first = min(tid * per, groups);
    run_end = min(run_first + per, groups);
    int run_rows = 0;
    for (int g = run_first; g < run_end; ++g) run_rows += rows_of(g);
    const int inc_rows = wave_inclusive_scan(run_rows);
    if (lane == 63) grp_red_rows[wave] = inc_rows;
    lds_barrier();
    int off_rows = 0;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) off_rows += w < wave ? grp_red_rows[w] : 0;
    run_rows_begin = off_rows + inc_rows - run_rows;
    for (int g = run_first, ahead = run_rows_begin; g < run_end; ahead += rows_of(g), ++g)
      run_tiles += tiles_for(kept_of(g, ahead));
    const int inc = wave_inclusive_scan(run_tiles);
    if (lane == 63) grp_red[wave] = inc;
    lds_barrier();
    int off = 0, total = 0;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) {
      off += w < wave ? grp_red[w] : 0;
      total += grp_red[w];
    }
    run_begin = off + inc - run_tiles;
    total_tiles = total * tiles_n;
    if ((int)blockIdx.x >= total_tiles) return;
  }
  int tile = blockIdx.x;
  do {  // (one pass unless GROUPED)
  int n0, rows_left;          // first column of the tile; rows of A and C from the tile's first row on
  const b128* a_tile;         // the tile's first row of A
  const b128* b_tile;         // the tile's first row of B (column n0 of the product)
  uint16_t* c_tile;           // the tile's first row of C
  const uint16_t* bias_row;   // the bias of the tile's group, or null
  if constexpr (GROUPED) {
    // whole rounds of the launch are renumbered so that an XCD works on consecutive pairs
    // (the column tiles of one row tile share its rows in that XCD's L2)
    const int round = tile / (int)gridDim.x;
    int logical = tile;
    if ((round + 1) * (int)gridDim.x <= total_tiles)
      logical = round * (int)gridDim.x + xcd_contiguous(blockIdx.x, gridDim.x);
    const int rb = logical / tiles_n, tn = logical - rb * tiles_n;
    lds_barrier();  // the tile before is out of LDS, and its grp_home has been read
    if (run_begin <= rb && rb < run_begin + run_tiles) {
      int g = run_first, first = run_begin, rows_ahead = run_rows_begin;
      for (;; ++g) {
        const int n = tiles_for(kept_of(g, rows_ahead));
        if (rb < first + n) break;
        first += n;
        rows_ahead += rows_of(g);
      }
      grp_home[0] = g;
      grp_home[1] = first;
      grp_home[2] = min(rows_ahead, max_rows);
      grp_home[3] = kept_of(g, rows_ahead);
    }
    lds_barrier();
    const int g = __builtin_amdgcn_readfirstlane(grp_home[0]);
    const int t0 = (rb - __builtin_amdgcn_readfirstlane(grp_home[1])) * BM;
    const size_t row0 = compact ? (size_t)__builtin_amdgcn_readfirstlane(grp_home[2]) : (size_t)g * max_rows;
    n0 = tn * BN;
    rows_left = __builtin_amdgcn_readfirstlane(grp_home[3]) - t0;
    a_tile = A + (row0 + t0) * row_vecs;
    b_tile = B + ((size_t)g * N + n0) * row_vecs;
    c_tile = C + (row0 + t0) * N;
    bias_row = bias ? bias + (size_t)g * N : nullptr;
  } else {
    const int logical = xcd_contiguous(blockIdx.x, gridDim.x);
    const int per_group = GROUP_M * tiles_n, group = logical / per_group, in = logical - group * per_group;
    const int rows = min(GROUP_M, tiles_m - group * GROUP_M);
    const int tn = in / rows, tm = group * GROUP_M + in - tn * rows;
    n0 = tn * BN;
    rows_left = M - tm * BM;
    a_tile = A + (size_t)tm * BM * row_vecs;
    b_tile = B + (size_t)n0 * row_vecs;
    c_tile = C + (size_t)tm * BM * N;
    bias_row = bias;
  }

  // Loads go through buffer descriptors whose extent ends with the last row of the matrix: rows of
  // a tile past it read as zeros. Vectors past the end of a row in the last step are sent out of
  // range the same way.
  const __amdgpu_buffer_rsrc_t abuf = __builtin_amdgcn_make_buffer_rsrc(
      (void*)a_tile, 0, min(BM, rows_left) * row_bytes, BUFFER_RAW_32BIT);
  const __amdgpu_buffer_rsrc_t bbuf = __builtin_amdgcn_make_buffer_rsrc(
      (void*)b_tile, 0, min(BN, N - n0) * row_bytes, BUFFER_RAW_32BIT);
  constexpr int OUT_OF_RANGE = 0x40000000;
  // copy i of a thread: LDS place p = tid + i * NT, that is row p / 8 (rows NT / 8 apart, which
  // leaves bits 1..3 of the row number alone) and the vector that belongs in physical slot p % 8
  const int crow = tid >> 3, cvec = (tid & 7) ^ ((crow >> 1) & 7);
  const int coff = crow * row_bytes + cvec * 16;
  const int cpast = cvec >= tail_vecs ? OUT_OF_RANGE : 0;
  const int rstep = (NT / 8) * row_bytes;

  b128 ga[LA], gb[LB];
  // A thread's LA + LB vectors of a step in four quarters: A[0..LA/2), A[LA/2..LA), B[0..LB/2), B[LB/2..LB)
  static_assert(LA % 2 == 0 && LB % 2 == 0, "quarters");
  auto load_quarter = [&](int q, int step) __attribute__((always_inline)) {
    const int at = min(step, steps - 1);  // (past the end: the last step again, never used)
    const int soff = at * (GEMM_KSTEP * 2), off = coff + (at == steps - 1 ? cpast : 0);
    if (q < 2) {
#pragma unroll
      for (int i = q * (LA / 2); i < (q + 1) * (LA / 2); ++i)
        ga[i] = __builtin_amdgcn_raw_buffer_load_b128(abuf, off + i * rstep, soff, 0);
    } else {
#pragma unroll
      for (int i = (q - 2) * (LB / 2); i < (q - 1) * (LB / 2); ++i)
        gb[i] = __builtin_amdgcn_raw_buffer_load_b128(bbuf, off + i * rstep, soff, 0);
    }
  };
  auto store_quarter = [&](int q, int buf) __attribute__((always_inline)) {
    b128* as = tile_lds + buf * ((BM + BN) * 8);
    b128* bs = as + BM * 8;
    if (q < 2) {
#pragma unroll
      for (int i = q * (LA / 2); i < (q + 1) * (LA / 2); ++i) as[tid + i * NT] = ga[i];
    } else {
#pragma unroll
      for (int i = (q - 2) * (LB / 2); i < (q - 1) * (LB / 2); ++i) bs[tid + i * NT] = gb[i];
    }
  };

  const int r = lane & 31, h = lane >> 5, swz = (r >> 1) & 7;
  f32x16 acc[TM][TN] = {};
  // Operand fragments of one 16-element slice of a step: two register sets, so that the reads of
  // the next slice are in flight while the matrix cores work on this one.
  b128 af[2][TM], bf[2][TN];
  auto read_frags = [&](int set, int buf, int kk) __attribute__((always_inline)) {
    const b128* as = tile_lds + buf * ((BM + BN) * 8) + (wm * TM * 32 + r) * 8;
    const b128* bs = tile_lds + buf * ((BM + BN) * 8) + BM * 8 + (wn * TN * 32 + r) * 8;
    const int v = (kk * 2 + h) ^ swz;
#pragma unroll
    for (int i = 0; i < TM; ++i) af[set][i] = as[i * 256 + v];
#pragma unroll
    for (int j = 0; j < TN; ++j) bf[set][j] = bs[j * 256 + v];
  };
  // (GROUPED) bands of 32 rows of this wave's part of the tile that hold rows of the group: the
  // last row tile of a group computes only those, in a copy of the loop with that one condition
  // (not for the 256 x 256 tile, whose registers have no room for the copy's state: it is used
  // where groups have many rows, and an empty band is a small part of them)
  constexpr bool SKIP_BANDS = GROUPED && TM * TN < 16;
  [[maybe_unused]] const int live_bands = min(max((rows_left - wm * TM * 32 + 31) / 32, 0), TM);
  auto mfmas = [&](int set, auto ragged) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if (decltype(ragged)::value && i >= live_bands) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = Mfma32x32x16<DT>::mma(bf[set][j], af[set][i], acc[i][j]);
    }
  };

  // Step s computes from LDS buffer s & 1. During it the rows of step s + 1 (in registers since
  // the step before) go to the other buffer, the rows of step s + 2 are requested from memory,
  // and the one barrier of the step sits before its last slice: behind it the first fragments
  // of step s + 1 are read while the matrix cores finish step s.
  // State at the start of step s: LDS buffer s & 1 holds the rows of step s; the other buffer
  // holds quarter 0 of step s + 1; the registers hold quarter 0 of step s + 2 and quarters 1..3
  // of step s + 1. Every slice of a step stores one quarter and requests its replacement, so
  // that the memory pipes see an even stream (four waves issuing all their loads in the same
  // slice oversubscribe the address unit while it idles in the others). Writes into a buffer
  // are legal from the barrier of the step that last read it to the barrier before the step that
  // reads it next: the last slice of step s - 1 and the first three of step s.
#pragma unroll
  for (int q = 0; q < 4; ++q) load_quarter(q, 0);
#pragma unroll
  for (int q = 0; q < 4; ++q) store_quarter(q, 0);
#pragma unroll
  for (int q = 0; q < 4; ++q) load_quarter(q, 1);
  store_quarter(0, 1);
  load_quarter(0, 2);
  __syncthreads();
  read_frags(0, 0, 0);
  // One memory instruction between two MFMAs: a wave that issues its loads or stores back to back
  // waits for the queues of the memory pipes and issues no MFMA meanwhile. A slice holds TM * TN
  // MFMAs, TM + TN fragment reads and one quarter's stores and loads; the 256 x 256 tile has its
  // measured order (read, store, read, load), smaller tiles spread theirs over the leading MFMAs.
  constexpr int N_MFMA = TM * TN, N_QUARTER = (LA > LB ? LA : LB) / 2;
  constexpr int READS_EACH = (TM + TN + N_MFMA - 1) / N_MFMA, MOVES_EACH = (N_QUARTER + N_MFMA - 1) / N_MFMA;
#define MOE_A2A_INTERLEAVE()                                            \
  if constexpr (N_MFMA == 16 && N_QUARTER == 4) {                       \
    _Pragma("unroll") for (int q = 0; q < 4; ++q) {                     \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                \
    }                                                                   \
  } else {                                                              \
    _Pragma("unroll") for (int q = 0; q < N_MFMA; ++q) {                \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                \
      __builtin_amdgcn_sched_group_barrier(0x100, READS_EACH, 0);       \
      __builtin_amdgcn_sched_group_barrier(0x200, MOVES_EACH, 0);       \
      __builtin_amdgcn_sched_group_barrier(0x020, MOVES_EACH, 0);       \
    }                                                                   \
  }                                                                     \
  __builtin_amdgcn_sched_barrier(0);
  auto one_step = [&](int step, int cur, auto ragged) __attribute__((always_inline)) {  // cur = step & 1, a constant where this is called
    read_frags(1, cur, 1);
    store_quarter(1, cur ^ 1);
    load_quarter(1, step + 2);
    mfmas(0, ragged);
    MOE_A2A_INTERLEAVE()
    read_frags(0, cur, 2);
    store_quarter(2, cur ^ 1);
    load_quarter(2, step + 2);
    mfmas(1, ragged);
    MOE_A2A_INTERLEAVE()
    read_frags(1, cur, 3);
    store_quarter(3, cur ^ 1);
    load_quarter(3, step + 2);
    mfmas(0, ragged);
    MOE_A2A_INTERLEAVE()
    lds_barrier();
    read_frags(0, cur ^ 1, 0);
    store_quarter(0, cur);
    load_quarter(0, step + 3);
    mfmas(1, ragged);
    MOE_A2A_INTERLEAVE()
  };
  auto walk_k = [&](auto ragged) __attribute__((always_inline)) {
    int step = 0;
    for (; step + 2 <= steps; step += 2) {
      one_step(step, 0, ragged);
      one_step(step + 1, 1, ragged);
    }
    if (step < steps) one_step(step, 0, ragged);
  };
  // (both copies hold the same barriers, so the waves of a workgroup may take different ones)
  if (!SKIP_BANDS || live_bands == TM) walk_k(std::false_type{});
  else if constexpr (SKIP_BANDS) walk_k(std::true_type{});

  // Results leave through LDS so that they reach memory in whole lines. acc[i][j] holds row
  // i*32 + r of the wave's tile and columns j*32 + g*8 + h*4 + 0..3 (g < 4): a lane's own values
  // are 8-byte pieces of 32 different rows. Each wave parks one band of 32 rows at a time in a
  // region of its own (rows padded by 16 bytes so that they start in different banks; a wave's
  // LDS operations execute in order, so no barrier is needed inside it) and reads it back with
  // 16 lanes per row: a store instruction then writes four 256-byte row segments.
  __syncthreads();  // every wave has read its last fragments: the operand tiles can be overwritten
  {
    constexpr int VR = TN * 4;            // 16-byte vectors per row of the wave's tile
    constexpr int PITCH = TN * 64 + 16;   // bytes per parked row
    constexpr int ROWS_PER_READ = 64 / VR;
    char* park = (char*)tile_lds + wave * (32 * PITCH);
    const int ncol = n0 + wn * TN * 32;
    uint32_t bias2[TN][4][2] = {};
    if (bias_row) {
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g)
          if (ncol + j * 32 < N) __builtin_memcpy(bias2[j][g], bias_row + ncol + j * 32 + g * 8 + h * 4, 8);
    }
    const int rrow = lane / VR, rvec = lane % VR;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if (SKIP_BANDS && i >= live_bands) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const f32x16& c = acc[i][j];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          uint32_t two[2] = {Pair16<DT>::canonical(Pair16<DT>::round(c[g * 4 + 0], c[g * 4 + 1])),
                             Pair16<DT>::canonical(Pair16<DT>::round(c[g * 4 + 2], c[g * 4 + 3]))};
          if (bias_row) {
#pragma unroll
            for (int e = 0; e < 2; ++e)
              two[e] = Pair16<DT>::canonical(Pair16<DT>::round(
                  __fadd_rn(Pair16<DT>::lo(two[e]), Pair16<DT>::lo(bias2[j][g][e])),
                  __fadd_rn(Pair16<DT>::hi(two[e]), Pair16<DT>::hi(bias2[j][g][e]))));
          }
          __builtin_memcpy(park + r * PITCH + (j * 32 + g * 8 + h * 4) * 2, two, 8);
        }
      }
#pragma unroll
      for (int p = 0; p < 32 / ROWS_PER_READ; ++p) {
        const int row = p * ROWS_PER_READ + rrow;
        const b128 v = *(const b128*)(park + row * PITCH + rvec * 16);
        const int m = (wm * TM + i) * 32 + row, n = ncol + rvec * 8;
        if (m < rows_left && n < N) *(b128*)(c_tile + (size_t)m * N + n) = v;
      }
    }
  }
  tile += gridDim.x;
  } while (GROUPED && tile < total_tiles);
}

#undef MOE_A2A_INTERLEAVE

// ---------------------------------------------------------------- exchange stand-in

template <typename V, int NV>
__global__ __launch_bounds__(BLOCK) void exchange_local_kernel(
    const V* __restrict__ send_buf, const int* __restrict__ send_meta,
    const int* __restrict__ send_counts, int dst_rank, V* __restrict__ recv_buf,
    int* __restrict__ recv_meta, const int* __restrict__ recv_counts, int src_rank, int row_vecs,
    int chunks, int send_capacity_rows, int recv_capacity_rows) {
  const int tid = threadIdx.x;
  const int src_off = sum_counts(send_counts, dst_rank, send_capacity_rows);
  const int dst_off = sum_counts(recv_counts, src_rank, recv_capacity_rows);
  int n = min(max(send_counts[dst_rank], 0), max(recv_counts[src_rank], 0));
  // never past what either buffer holds, whatever the counts claim
  n = max(min(n, min(send_capacity_rows - src_off, recv_capacity_rows - dst_off)), 0);
  const int items = n * chunks;
  for (int q = blockIdx.x; q < items; q += gridDim.x) {
    const int i = chunks == 1 ? q : q / chunks, c = q - i * chunks;
    const int base = c * (BLOCK * NV);
    Payload<V, NV> p;
    p.load(send_buf + (size_t)(src_off + i) * row_vecs, base, row_vecs);
    p.store(recv_buf + (size_t)(dst_off + i) * row_vecs, base, row_vecs);
    if (c == 0 && tid < META)
      recv_meta[(size_t)(dst_off + i) * META + tid] = send_meta[(size_t)(src_off + i) * META + tid];
  }
}

// All source legs of one destination in one launch: blockIdx.y is the source rank. The W source
// buffers are separate allocations (one per rank object), so their addresses travel by value in
// the kernel arguments. Every wave works out both offsets of its leg from the W counts the
// sources hold for this destination (one lane per source, a wave scan) and the kernel also
// writes those counts to recv_counts, which an exchange of counts would have delivered
// (all2all/reference.py:88-91,181-185).
constexpr int GATHER_MAX_RANKS = 64;
struct GatherSources {
  const void* buf[GATHER_MAX_RANKS];
  const int* meta[GATHER_MAX_RANKS];
  const int* counts[GATHER_MAX_RANKS];
};

template <typename V, int NV>
__global__ __launch_bounds__(BLOCK) void exchange_gather_kernel(
    GatherSources src, int W, int dst_rank, V* __restrict__ recv_buf, int* __restrict__ recv_meta,
    int* __restrict__ recv_counts, int row_vecs, int chunks, int send_capacity_rows,
    int recv_capacity_rows) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int s = blockIdx.y;
  // rows every source holds for this destination (lane l: source l)
  const int held = lane < W ? min(max(src.counts[lane][dst_rank], 0), send_capacity_rows) : 0;
  const int upto = wave_inclusive_scan(held);
  if (blockIdx.x == 0 && s == 0 && tid < W) recv_counts[tid] = held;
  const int dst_off = __builtin_amdgcn_readlane(upto - held, s);
  const int* __restrict__ my_counts = src.counts[s];
  const int src_off = sum_counts(my_counts, dst_rank, send_capacity_rows);
  int n = __builtin_amdgcn_readlane(held, s);
  // never past what either buffer holds, whatever the counts claim
  n = max(min(n, min(send_capacity_rows - src_off, recv_capacity_rows - dst_off)), 0);
  const V* __restrict__ send_buf = (const V*)src.buf[s];
  const int* __restrict__ send_meta = src.meta[s];
  const int items = n * chunks;
  for (int q = blockIdx.x; q < items; q += gridDim.x) {
    const int i = chunks == 1 ? q : q / chunks, c = q - i * chunks;
    const int base = c * (BLOCK * NV);
    Payload<V, NV> p;
    p.load(send_buf + (size_t)(src_off + i) * row_vecs, base, row_vecs);
    p.store(recv_buf + (size_t)(dst_off + i) * row_vecs, base, row_vecs);
    if (c == 0 && tid < META)
      recv_meta[(size_t)(dst_off + i) * META + tid] = send_meta[(size_t)(src_off + i) * META + tid];
  }
}

// ---------------------------------------------------------------- host side

struct Geometry {
  bool vec16;     // 16-byte vectors usable for every row buffer of the call
  int row_vecs;   // vectors (or 2-byte elements) per row
  int nv;         // block-per-row kernels: vectors per lane (1, 2 or 4)
  int chunks;     //   and workgroups per row = ceil(row_vecs / (BLOCK * nv))
  int nvw;        // wave-per-row kernels: vectors per lane of the row's wave
  int wchunks;    //   and chunks per row = ceil(row_vecs / (64 * nvw))
  int nle;
  int max_recv;
  uint32_t magic; // ceil(2^32 / nle)
};

bool shape_ok(const moe_a2a_shape* s) {
  return s && s->world_size >= 1 && s->rank >= 0 && s->rank < s->world_size &&
         s->num_experts >= s->world_size && s->num_experts <= 65536 &&
         s->num_experts % s->world_size == 0 && s->experts_per_token >= 1 && s->hidden_dim >= 1 &&
         s->max_num_tokens >= 1 &&
         (long long)s->max_num_tokens * s->world_size <= INT_MAX / 8;
}

bool aligned(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }

template <typename... P>
bool all_aligned(size_t a, P... ptrs) { return (aligned(ptrs, a) && ...); }

void row_geometry(Geometry& g, int hidden_dim, bool ptrs_16B) {
  const long long row_bytes = 2ll * hidden_dim;
  g.vec16 = (row_bytes % 16 == 0) && ptrs_16B;
  g.row_vecs = g.vec16 ? (int)(row_bytes / 16) : hidden_dim;
  g.nv = g.row_vecs <= BLOCK ? 1 : g.row_vecs <= 2 * BLOCK ? 2 : 4;
  g.chunks = (g.row_vecs + BLOCK * g.nv - 1) / (BLOCK * g.nv);
  g.nvw = 16;
  if (g.vec16) {
    const int need = (g.row_vecs + 63) / 64;
    for (int c : {14, 12, 8, 6, 4, 2, 1})
      if (need <= c) g.nvw = c;
  }
  g.wchunks = (g.row_vecs + 64 * g.nvw - 1) / (64 * g.nvw);
}

template <typename... P>
Geometry geometry(const moe_a2a_shape* s, P... row_ptrs) {
  Geometry g;
  row_geometry(g, s->hidden_dim, all_aligned(16, row_ptrs...));
  g.nle = s->num_experts / s->world_size;
  g.max_recv = s->max_num_tokens * s->world_size;
  g.magic = g.nle == 1 ? 0u : (uint32_t)(0xffffffffu / (uint32_t)g.nle) + 1u;
  return g;
}

// Workgroups that move rows: one per item up to a cap the kernels stride over.
// `items` beyond INT_MAX are rejected by the callers before this is reached.
int mover_blocks(long long items) {
  const long long cap = 1 << 20;
  long long g = items < cap ? items : cap;
  return (int)(g < 1 ? 1 : g);
}

bool items_fit(long long rows, int chunks) { return rows * chunks <= INT_MAX / 2; }

int launch_status() { return hipGetLastError() == hipSuccess ? MOE_A2A_OK : MOE_A2A_ELAUNCH; }

// Picks the <vector type, vectors per lane> instantiation for a geometry.
#define MOE_A2A_FOR_ROW_KERNEL(G, LAUNCH)                  \
  do {                                                     \
    if ((G).vec16) {                                       \
      if ((G).nv == 1) { LAUNCH(b128, 1); }                \
      else if ((G).nv == 2) { LAUNCH(b128, 2); }           \
      else { LAUNCH(b128, 4); }                            \
    } else {                                               \
      if ((G).nv == 1) { LAUNCH(uint16_t, 1); }            \
      else if ((G).nv == 2) { LAUNCH(uint16_t, 2); }       \
      else { LAUNCH(uint16_t, 4); }                        \
    }                                                      \
  } while (0)

// Same for the wave-per-row kernels: <vector type, vectors per lane of a wave>.
#define MOE_A2A_FOR_WAVE_KERNEL(G, LAUNCH)        \
  do {                                            \
    if ((G).vec16) {                              \
      switch ((G).nvw) {                          \
        case 1: LAUNCH(b128, 1); break;           \
        case 2: LAUNCH(b128, 2); break;           \
        case 4: LAUNCH(b128, 4); break;           \
        case 6: LAUNCH(b128, 6); break;           \
        case 8: LAUNCH(b128, 8); break;           \
        case 12: LAUNCH(b128, 12); break;         \
        case 14: LAUNCH(b128, 14); break;         \
        default: LAUNCH(b128, 16); break;         \
      }                                           \
    } else {                                      \
      LAUNCH(uint16_t, 16);                       \
    }                                             \
  } while (0)

#ifndef MOE_A2A_PLANNED_NVW
#define MOE_A2A_PLANNED_NVW 4  // vectors per lane of a mover that scans nothing
#endif

// The send-back plan is kept by the lanes of one wave: one lane per source rank
// in stage 2, one lane per local expert in stage 3.
bool plan_supported(const moe_a2a_shape* s) {
  return s->world_size <= 64 && s->num_experts / s->world_size <= 64;
}

// Address of `scratch` on the GPU that is current for the calling thread, looked up once per
// GPU with that GPU current and kept. Returns nullptr if the runtime cannot name it.
constexpr int MAX_GPUS = 64;
std::mutex static_plan_mutex;
int32_t* static_plan_address[MAX_GPUS] = {};

int32_t* static_plan_buffer() {
  int gpu = -1;
  if (hipGetDevice(&gpu) != hipSuccess || gpu < 0 || gpu >= MAX_GPUS) return nullptr;
  std::lock_guard<std::mutex> lock(static_plan_mutex);
  if (!static_plan_address[gpu]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    static_plan_address[gpu] = static_cast<int32_t*>(p);
  }
  return static_plan_address[gpu];
}

// W counts, each cut to `capacity_rows` on the device, must add up inside an int.
bool counts_fit(long long capacity_rows, int world_size) {
  return capacity_rows * world_size <= INT_MAX;
}

// Workgroups of a ranked row move over `rows` rows.
long long group_items(long long rows, const Geometry& g) {
  return (rows + ROWS - 1) / ROWS * g.wchunks;
}

}  // namespace

extern "C" {

const char* moe_a2a_version(void) { return "moe_a2a 0.6 gfx950"; }

#ifndef MOE_A2A_BUILD_ID
#define MOE_A2A_BUILD_ID "unknown"
#endif
const char* moe_a2a_build_id(void) { return MOE_A2A_BUILD_ID; }

const char* moe_a2a_strerror(int status) {
  switch (status) {
    case MOE_A2A_OK: return "ok";
    case MOE_A2A_EINVAL: return "invalid argument (null pointer, bad shape or unsupported size)";
    case MOE_A2A_EALIGN: return "row buffer is not aligned to its 2-byte elements";
    case MOE_A2A_ELAUNCH: return "kernel launch failed";
    case MOE_A2A_ESCRATCH:
      return "shape beyond the library's static buffer (world_size <= 64 and num_local_experts <= 64), "
             "or the buffer's address is unavailable";
    default: return "unknown status";
  }
}

int moe_a2a_dispatch_send(const moe_a2a_shape* s, const void* x, const int32_t* indices,
                          int32_t num_tokens, void* send_buf, int32_t* send_meta,
                          int32_t* send_counts, int32_t* send_slot, void* stream) {
  if (!shape_ok(s) || num_tokens < 0 || num_tokens > s->max_num_tokens || !send_counts)
    return MOE_A2A_EINVAL;
  const long long S = (long long)num_tokens * s->experts_per_token;
  if (S > 0 && (!x || !indices || !send_buf || !send_meta)) return MOE_A2A_EINVAL;
  if (!all_aligned(2, x, send_buf)) return MOE_A2A_EALIGN;
  const Geometry g = geometry(s, x, send_buf);
  if (!items_fit(S, g.wchunks)) return MOE_A2A_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  // Tokens with several entries: one workgroup per (token, 256-vector chunk) stores the chunk to
  // all of the token's slots (measured at K = 8, H = 7168: 8.4 us against 8.8 us with a wave per
  // entry; one chunk per workgroup beats two or four). With one or two entries per token the
  // wave-per-entry kernel scans fewer keys per byte moved.
#ifndef MOE_A2A_FANOUT_MIN_K
#define MOE_A2A_FANOUT_MIN_K 4
#endif
  Geometry f = g;
  f.nv = 1;
  f.chunks = (f.row_vecs + BLOCK - 1) / BLOCK;
  if (s->experts_per_token >= MOE_A2A_FANOUT_MIN_K && (s->world_size + 2ll) * S <= INT_MAX &&
      items_fit(num_tokens, f.chunks)) {
    const int fan = fan_of(S);
#ifndef MOE_A2A_FANOUT_WIDE
#define MOE_A2A_FANOUT_WIDE 1
#endif
    constexpr int WIDE = 2 * BLOCK;  // rows of more than one 256-lane chunk: 512-lane workgroups
    if (MOE_A2A_FANOUT_WIDE && f.row_vecs > BLOCK && S < 65536 && s->world_size < 16384) {
      // Rows of more than 512 vectors: two vectors per lane, so that a row of up to 1024 vectors
      // is one workgroup's and its entries are ranked once, not once per chunk (measured at
      // H = 7168: the whole step 0.4 us shorter; 256 lanes x 4 and 1024 lanes x 1 were slower).
      const int fnv = f.row_vecs > WIDE ? 2 : 1;
      const int wchunks = (f.row_vecs + WIDE * fnv - 1) / (WIDE * fnv);
      const int wgrid = s->world_size + mover_blocks((long long)num_tokens * wchunks);
      int order_bits = 1;  // S <= 1 << order_bits <= 65536, so (W + 1) << order_bits fits an int
      while ((1ll << order_bits) < S) ++order_bits;
      const bool pow2 = (g.nle & (g.nle - 1)) == 0;
      int nle_shift = 0;
      while ((1 << nle_shift) < g.nle) ++nle_shift;
#define LAUNCH_W(V, NV, POW2, FAN)                                                             \
  dispatch_fanout_wide_kernel<V, WIDE, NV, POW2, FAN><<<wgrid, WIDE, 0, st>>>(                 \
      (const V*)x, indices, num_tokens, s->experts_per_token, g.nle, s->num_experts,           \
      s->world_size, g.magic, nle_shift, order_bits, s->rank, f.row_vecs, wchunks,             \
      (V*)send_buf, send_meta, send_counts, send_slot)
#define LAUNCH_WF(V, NV, POW2)                       \
  do {                                               \
    if (fan == 2) LAUNCH_W(V, NV, POW2, 2);          \
    else LAUNCH_W(V, NV, POW2, 8);                   \
  } while (0)
#define LAUNCH_WV(V)                                                  \
  do {                                                                \
    if (fnv == 2) { if (pow2) LAUNCH_WF(V, 2, true); else LAUNCH_WF(V, 2, false); } \
    else { if (pow2) LAUNCH_WF(V, 1, true); else LAUNCH_WF(V, 1, false); }          \
  } while (0)
      if (f.vec16) LAUNCH_WV(b128);
      else LAUNCH_WV(uint16_t);
#undef LAUNCH_WV
#undef LAUNCH_WF
#undef LAUNCH_W
      return launch_status();
    }
    const int fgrid = s->world_size + mover_blocks((long long)num_tokens * f.chunks);
#define LAUNCH_F(V, FAN)                                                                       \
  dispatch_fanout_kernel<V, 1, FAN><<<fgrid, BLOCK, 0, st>>>(                                  \
      (const V*)x, indices, num_tokens, s->experts_per_token, g.nle, s->num_experts,           \
      s->world_size, g.magic, s->rank, f.row_vecs, f.chunks, (V*)send_buf, send_meta,          \
      send_counts, send_slot)
#define LAUNCH(V)                         \
  do {                                    \
    if (fan == 2) LAUNCH_F(V, 2);         \
    else LAUNCH_F(V, 8);                  \
  } while (0)
    if (f.vec16) LAUNCH(b128);  // one vector per lane is the only shape this kernel is launched with
    else LAUNCH(uint16_t);
#undef LAUNCH
#undef LAUNCH_F
    return launch_status();
  }
  const int grid = s->world_size + mover_blocks(group_items(S, g));
#define LAUNCH(V, NVW)                                                                         \
  dispatch_send_kernel<V, NVW><<<grid, 64 * ROWS, 0, st>>>(                                    \
      (const V*)x, indices, (int)S, s->experts_per_token, g.nle, s->num_experts, s->world_size, \
      g.magic, s->rank, g.row_vecs, g.wchunks, (V*)send_buf, send_meta, send_counts, send_slot)
  MOE_A2A_FOR_WAVE_KERNEL(g, LAUNCH);
#undef LAUNCH
  return launch_status();
}

int moe_a2a_plan_send(const moe_a2a_shape* s, const int32_t* indices, int32_t num_tokens,
                      int32_t* rank_counts, int32_t* rank_offsets, int32_t* expert_counts,
                      int32_t* dst_slot, int32_t* src_entry, void* stream) {
  if (!shape_ok(s) || num_tokens < 0 || num_tokens > s->max_num_tokens || !rank_counts ||
      !rank_offsets || !expert_counts)
    return MOE_A2A_EINVAL;
  if (s->world_size > PLAN_MAX_RANKS || s->num_experts > PLAN_MAX_EXPERTS) return MOE_A2A_EINVAL;
  const long long S = (long long)num_tokens * s->experts_per_token;
  if (S > INT_MAX / 2) return MOE_A2A_EINVAL;
  if (S > 0 && (!indices || !dst_slot || !src_entry)) return MOE_A2A_EINVAL;
  const Geometry g = geometry(s);
  plan_send_kernel<<<1, PLAN_BLOCK, 0, (hipStream_t)stream>>>(
      indices, (int)S, g.nle, s->num_experts, s->world_size, g.magic, rank_counts, rank_offsets,
      expert_counts, dst_slot, src_entry);
  return launch_status();
}

}  // extern "C"

namespace {

// Stage 2; with `row_position` (capacity_rows ints of workspace) the positions come from a
// planning launch and the movers scan nothing.
int launch_dispatch_recv(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                         const int32_t* recv_counts, int32_t rows_hint, int32_t capacity_rows,
                         int32_t* expert_num_tokens, void* expert_x, int32_t* expert_meta,
                         int32_t* send_back_plan, int32_t* row_position, void* stream,
                         int32_t compact_rows = 0, int32_t* expert_offsets = nullptr) {
  if (!shape_ok(s) || rows_hint < 0 || capacity_rows < 0 || !recv_counts || !expert_num_tokens ||
      !expert_x || !expert_meta)
    return MOE_A2A_EINVAL;
  if (compact_rows > 0 && (!expert_offsets || row_position)) return MOE_A2A_EINVAL;
  if (!counts_fit(capacity_rows, s->world_size)) return MOE_A2A_EINVAL;
  if (rows_hint > capacity_rows) rows_hint = capacity_rows;
  if (capacity_rows > 0 && (!recv_buf || !recv_meta)) return MOE_A2A_EINVAL;
  if (!all_aligned(2, recv_buf, expert_x)) return MOE_A2A_EALIGN;
  Geometry g = geometry(s, recv_buf, expert_x);
  hipStream_t st = (hipStream_t)stream;
  const bool planned = send_back_plan && plan_supported(s);
  if (row_position && g.nle <= RPLAN_MAX_EXPERTS && capacity_rows > 0) {
    // no scan to repeat per chunk: a row is split among more waves, as in the planned stage 3
    if (g.vec16 && g.nvw > MOE_A2A_PLANNED_NVW) {
      g.nvw = MOE_A2A_PLANNED_NVW;
      g.wchunks = (g.row_vecs + 64 * g.nvw - 1) / (64 * g.nvw);
    }
    if (!items_fit((long long)g.nle * g.max_recv, g.wchunks)) return MOE_A2A_EINVAL;
    const int tiles = (int)std::min<long long>(((long long)rows_hint + RPLAN_BLOCK - 1) / RPLAN_BLOCK + 1, 1 << 16);
    int expert_bits = 0;  // nle <= 1 << expert_bits
    while ((1 << expert_bits) < g.nle) ++expert_bits;
    plan_recv_kernel<<<tiles, RPLAN_BLOCK, 0, st>>>(recv_meta, recv_counts, s->world_size, rows_hint,
                                                    capacity_rows, g.nle, g.magic, expert_bits, row_position);
    const int grid = g.nle + mover_blocks(group_items(rows_hint, g));
#define LAUNCH_P(V, NVW, PLAN)                                                              \
  dispatch_recv_kernel<V, NVW, PLAN, RECV_POS><<<grid, 64 * ROWS, 0, st>>>(                 \
      (const V*)recv_buf, recv_meta, recv_counts, s->world_size, rows_hint, capacity_rows,   \
      g.nle, g.magic, g.max_recv, g.row_vecs, g.wchunks, expert_num_tokens, (V*)expert_x,    \
      expert_meta, send_back_plan, row_position, nullptr)
#define LAUNCH(V, NVW)                     \
  do {                                     \
    if (planned) LAUNCH_P(V, NVW, true);   \
    else LAUNCH_P(V, NVW, false);          \
  } while (0)
    if (!g.vec16) LAUNCH(uint16_t, 16);
    else if (g.nvw == 1) LAUNCH(b128, 1);
    else if (g.nvw == 2) LAUNCH(b128, 2);
    else LAUNCH(b128, 4);
#undef LAUNCH
#undef LAUNCH_P
    return launch_status();
  }
  // the stream can hold at most nle * max_recv rows that fit the expert buffers
  if (!items_fit((long long)g.nle * g.max_recv, g.wchunks)) return MOE_A2A_EINVAL;
  const int grid = g.nle + mover_blocks(group_items(rows_hint, g));
#define LAUNCH_P(V, NVW, PLAN, MODE)                                                        \
  dispatch_recv_kernel<V, NVW, PLAN, MODE><<<grid, 64 * ROWS, 0, st>>>(                     \
      (const V*)recv_buf, recv_meta, recv_counts, s->world_size, rows_hint, capacity_rows,   \
      g.nle, g.magic, compact_rows > 0 ? compact_rows : g.max_recv, g.row_vecs, g.wchunks,   \
      expert_num_tokens, (V*)expert_x, expert_meta, send_back_plan, nullptr, expert_offsets)
#define LAUNCH(V, NVW)                                         \
  do {                                                         \
    if (compact_rows > 0) {                                    \
      if (planned) LAUNCH_P(V, NVW, true, RECV_COMPACT);       \
      else LAUNCH_P(V, NVW, false, RECV_COMPACT);              \
    } else {                                                   \
      if (planned) LAUNCH_P(V, NVW, true, RECV_SCAN);          \
      else LAUNCH_P(V, NVW, false, RECV_SCAN);                 \
    }                                                          \
  } while (0)
  MOE_A2A_FOR_WAVE_KERNEL(g, LAUNCH);
#undef LAUNCH
#undef LAUNCH_P
  return launch_status();
}

}  // namespace

extern "C" {

int moe_a2a_dispatch_recv(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                          const int32_t* recv_counts, int32_t rows_hint, int32_t capacity_rows,
                          int32_t* expert_num_tokens, void* expert_x, int32_t* expert_meta,
                          int32_t* send_back_plan, void* stream) {
  return launch_dispatch_recv(s, recv_buf, recv_meta, recv_counts, rows_hint, capacity_rows,
                              expert_num_tokens, expert_x, expert_meta, send_back_plan, nullptr, stream);
}

int moe_a2a_dispatch_recv_long(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                               const int32_t* recv_counts, int32_t rows_hint, int32_t capacity_rows,
                               int32_t* expert_num_tokens, void* expert_x, int32_t* expert_meta,
                               int32_t* send_back_plan, int32_t* row_position, void* stream) {
  if (!row_position) return MOE_A2A_EINVAL;
  return launch_dispatch_recv(s, recv_buf, recv_meta, recv_counts, rows_hint, capacity_rows,
                              expert_num_tokens, expert_x, expert_meta, send_back_plan, row_position, stream);
}

int moe_a2a_dispatch_recv_static(const moe_a2a_shape* s, const void* recv_buf,
                                 const int32_t* recv_meta, const int32_t* recv_counts,
                                 int32_t rows_hint, int32_t capacity_rows, int32_t* expert_num_tokens,
                                 void* expert_x, int32_t* expert_meta,
                                 const int32_t** send_back_plan, void* stream) {
  if (!shape_ok(s) || !send_back_plan) return MOE_A2A_EINVAL;
  *send_back_plan = nullptr;
  // the plan needs a lane per source rank and per local expert, and 2 * num_experts ints
  if (!plan_supported(s) || s->num_experts > MOE_A2A_STATIC_PLAN_EXPERTS) return MOE_A2A_ESCRATCH;
  int32_t* plan = static_plan_buffer();
  if (!plan) return MOE_A2A_ESCRATCH;
  // every int of the plan that this shape uses is written by the call: nothing to clear
  const int rc = moe_a2a_dispatch_recv(s, recv_buf, recv_meta, recv_counts, rows_hint, capacity_rows,
                                       expert_num_tokens, expert_x, expert_meta, plan, stream);
  if (rc == MOE_A2A_OK) *send_back_plan = plan;
  return rc;
}

}  // extern "C"

namespace {

// Stage 3; compact_rows > 0: the expert buffers hold the experts' rows back to back.
int launch_combine_send(const moe_a2a_shape* s, const void* expert_y, const int32_t* expert_meta,
                        const int32_t* expert_num_tokens, int32_t rows_hint, int32_t capacity_rows,
                        void* send_buf, int32_t* send_meta, int32_t* send_counts,
                        const int32_t* send_back_plan, int32_t compact_rows, void* stream) {
  if (!shape_ok(s) || rows_hint < 0 || capacity_rows < 0 || compact_rows < 0 || !expert_y || !expert_meta ||
      !expert_num_tokens || !send_counts)
    return MOE_A2A_EINVAL;
  if (capacity_rows > 0 && (!send_buf || !send_meta)) return MOE_A2A_EINVAL;
  if (!all_aligned(2, expert_y, send_buf)) return MOE_A2A_EALIGN;
  Geometry g = geometry(s, expert_y, send_buf);
  if (g.nle > MAX_LOCAL_EXPERTS) return MOE_A2A_EINVAL;
  if (compact_rows > 0) {
    if (!counts_fit(compact_rows, g.nle)) return MOE_A2A_EINVAL;  // counts cut to the capacity add up in an int
    g.max_recv = compact_rows;  // no expert has more rows than the buffers hold
  }
  const bool planned = send_back_plan && plan_supported(s);
  // The planned path has no scan to repeat per chunk, so a row can be split among more waves:
  // 4 vectors per lane (a 256-vector chunk per wave) made the whole step 0.5 us shorter at
  // H = 7168 than the 14 the scan path uses; 2, 6 and 8 were no better than 14.
  if (planned && g.vec16 && g.nvw > MOE_A2A_PLANNED_NVW) {
    g.nvw = MOE_A2A_PLANNED_NVW;
    g.wchunks = (g.row_vecs + 64 * g.nvw - 1) / (64 * g.nvw);
  }
  if (!items_fit(compact_rows > 0 ? (long long)compact_rows : (long long)g.nle * g.max_recv, g.wchunks))
    return MOE_A2A_EINVAL;
  const int grid = s->world_size + mover_blocks(group_items(rows_hint, g));
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH_S(V, NVW, SMALL, PLAN)                                                          \
  combine_send_kernel<V, NVW, SMALL, PLAN><<<grid, 64 * ROWS, 0, st>>>(                       \
      (const V*)expert_y, expert_meta, expert_num_tokens, g.nle, g.max_recv, s->world_size,    \
      g.row_vecs, g.wchunks, capacity_rows, (V*)send_buf, send_meta, send_counts,              \
      send_back_plan, compact_rows)
#define LAUNCH(V, NVW)                                   \
  do {                                                   \
    if (planned) LAUNCH_S(V, NVW, true, true);           \
    else if (g.nle <= 64) LAUNCH_S(V, NVW, true, false); \
    else LAUNCH_S(V, NVW, false, false);                 \
  } while (0)
  MOE_A2A_FOR_WAVE_KERNEL(g, LAUNCH);
#undef LAUNCH
#undef LAUNCH_S
  return launch_status();
}

// Stage 4; with `entry_row` (num_tokens * K ints of workspace) a launch of its own first maps
// every (token, k) to its arriving row and the workgroups look their rows up instead of scanning.
int launch_combine_recv(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                        const int32_t* recv_counts, int32_t rows_hint, int32_t capacity_rows,
                        const float* weights, int32_t num_tokens, void* out_tokens,
                        int32_t accumulate, int32_t dtype, int32_t* entry_row, void* stream) {
  if (!shape_ok(s) || num_tokens < 0 || num_tokens > s->max_num_tokens || !recv_counts ||
      rows_hint < 0 || capacity_rows < 0)
    return MOE_A2A_EINVAL;
  if (!counts_fit(capacity_rows, s->world_size)) return MOE_A2A_EINVAL;
  if (rows_hint > capacity_rows) rows_hint = capacity_rows;
  if (dtype != MOE_A2A_F16 && dtype != MOE_A2A_BF16) return MOE_A2A_EINVAL;
  if (num_tokens == 0) return MOE_A2A_OK;
  if (!recv_buf || !recv_meta || !weights || !out_tokens) return MOE_A2A_EINVAL;
  if (!all_aligned(2, recv_buf, out_tokens)) return MOE_A2A_EALIGN;
  const Geometry g = geometry(s, recv_buf, out_tokens);
  // 256 lanes per (token, chunk), one vector column each; rows of at most 512
  // vectors are not split, their lanes take two columns
  // 256 lanes per (token, chunk) with one vector column each for rows up to 256 vectors and two
  // columns beyond. Every workgroup of a token repeats the scan of the arrivals, so fewer, fatter
  // chunks win until the registers of a lane (8 addends x columns in flight) run out.
#ifndef MOE_A2A_COMBINE_NV_WIDE
#define MOE_A2A_COMBINE_NV_WIDE 1
#endif
  const int nv = g.row_vecs > 2 * BLOCK ? MOE_A2A_COMBINE_NV_WIDE : g.row_vecs > BLOCK ? 2 : 1;
  const int chunks = (g.row_vecs + BLOCK * nv - 1) / (BLOCK * nv);
  if (!items_fit(num_tokens, chunks)) return MOE_A2A_EINVAL;
  const int grid = mover_blocks((long long)num_tokens * chunks);
  hipStream_t st = (hipStream_t)stream;
  const int K = s->experts_per_token, W = s->world_size;
  const bool mapped = entry_row != nullptr && capacity_rows > 0;
  if (mapped) {
    const int mgrid = (int)std::min<long long>(((long long)rows_hint + BLOCK - 1) / BLOCK + 1, 1 << 16);
    return_map_kernel<<<mgrid, BLOCK, 0, st>>>(recv_meta, recv_counts, W, rows_hint, capacity_rows,
                                               num_tokens, K, entry_row);
  }
#define LAUNCH(V, DT, BLK, NV)                                                               \
  do {                                                                                       \
    if (mapped)                                                                              \
      combine_recv_kernel<V, DT, BLK, NV, true><<<grid, BLK, 0, st>>>(                       \
          (const V*)recv_buf, recv_meta, recv_counts, W, rows_hint, capacity_rows, weights,  \
          num_tokens, K, g.row_vecs, chunks, (V*)out_tokens, accumulate, entry_row);         \
    else                                                                                     \
      combine_recv_kernel<V, DT, BLK, NV, false><<<grid, BLK, 0, st>>>(                      \
          (const V*)recv_buf, recv_meta, recv_counts, W, rows_hint, capacity_rows, weights,  \
          num_tokens, K, g.row_vecs, chunks, (V*)out_tokens, accumulate, nullptr);           \
  } while (0)
#define PICK_SHAPE(V, DT)                       \
  do {                                          \
    if (nv == 1) { LAUNCH(V, DT, BLOCK, 1); }   \
    else { LAUNCH(V, DT, BLOCK, 2); }           \
  } while (0)
  if (g.vec16) {
    if (dtype == MOE_A2A_BF16) PICK_SHAPE(b128, MOE_A2A_BF16);
    else PICK_SHAPE(b128, MOE_A2A_F16);
  } else {
    if (dtype == MOE_A2A_BF16) PICK_SHAPE(uint16_t, MOE_A2A_BF16);
    else PICK_SHAPE(uint16_t, MOE_A2A_F16);
  }
#undef PICK_SHAPE
#undef LAUNCH
  return launch_status();
}

}  // namespace

extern "C" {

int moe_a2a_dispatch_recv_compact(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                                  const int32_t* recv_counts, int32_t rows_hint, int32_t capacity_rows,
                                  int32_t* expert_num_tokens, int32_t* expert_offsets, void* expert_x,
                                  int32_t* expert_meta, int32_t compact_capacity_rows,
                                  int32_t* send_back_plan, void* stream) {
  if (compact_capacity_rows < 1 || !expert_offsets) return MOE_A2A_EINVAL;
  return launch_dispatch_recv(s, recv_buf, recv_meta, recv_counts, rows_hint, capacity_rows, expert_num_tokens,
                              expert_x, expert_meta, send_back_plan, nullptr, stream, compact_capacity_rows,
                              expert_offsets);
}

int moe_a2a_combine_send(const moe_a2a_shape* s, const void* expert_y, const int32_t* expert_meta,
                         const int32_t* expert_num_tokens, int32_t rows_hint,
                         int32_t capacity_rows, void* send_buf, int32_t* send_meta, int32_t* send_counts,
                         const int32_t* send_back_plan, void* stream) {
  return launch_combine_send(s, expert_y, expert_meta, expert_num_tokens, rows_hint, capacity_rows, send_buf,
                             send_meta, send_counts, send_back_plan, 0, stream);
}

int moe_a2a_combine_send_compact(const moe_a2a_shape* s, const void* expert_y, const int32_t* expert_meta,
                                 const int32_t* expert_num_tokens, int32_t rows_hint,
                                 int32_t compact_capacity_rows, int32_t capacity_rows, void* send_buf,
                                 int32_t* send_meta, int32_t* send_counts, const int32_t* send_back_plan,
                                 void* stream) {
  if (compact_capacity_rows < 1) return MOE_A2A_EINVAL;
  return launch_combine_send(s, expert_y, expert_meta, expert_num_tokens, rows_hint, capacity_rows, send_buf,
                             send_meta, send_counts, send_back_plan, compact_capacity_rows, stream);
}

int moe_a2a_combine_recv(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                         const int32_t* recv_counts, int32_t rows_hint, int32_t capacity_rows,
                         const float* weights, int32_t num_tokens, void* out_tokens,
                         int32_t accumulate, int32_t dtype, void* stream) {
  return launch_combine_recv(s, recv_buf, recv_meta, recv_counts, rows_hint, capacity_rows, weights,
                             num_tokens, out_tokens, accumulate, dtype, nullptr, stream);
}

int moe_a2a_combine_recv_long(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                              const int32_t* recv_counts, int32_t rows_hint, int32_t capacity_rows,
                              const float* weights, int32_t num_tokens, void* out_tokens,
                              int32_t accumulate, int32_t dtype, int32_t* entry_row, void* stream) {
  if (!entry_row) return MOE_A2A_EINVAL;
  return launch_combine_recv(s, recv_buf, recv_meta, recv_counts, rows_hint, capacity_rows, weights,
                             num_tokens, out_tokens, accumulate, dtype, entry_row, stream);
}

}  // extern "C"

namespace {

// The stand-in expert; compact_rows > 0: the expert buffers hold the experts' rows back to back.
int launch_expert_scale(const moe_a2a_shape* s, const void* expert_x, const int32_t* expert_num_tokens,
                        int32_t rows_hint, int32_t in_dtype, int32_t out_dtype, void* expert_y,
                        int32_t compact_rows, void* stream) {
  if (!shape_ok(s) || rows_hint < 0 || compact_rows < 0 || !expert_x || !expert_num_tokens || !expert_y)
    return MOE_A2A_EINVAL;
  if ((in_dtype != MOE_A2A_F16 && in_dtype != MOE_A2A_BF16) ||
      (out_dtype != MOE_A2A_F16 && out_dtype != MOE_A2A_BF16))
    return MOE_A2A_EINVAL;
  if (!all_aligned(2, expert_x, expert_y)) return MOE_A2A_EALIGN;
  Geometry g = geometry(s, expert_x, expert_y);
  if (g.nle > MAX_LOCAL_EXPERTS) return MOE_A2A_EINVAL;
  if (compact_rows > 0) {
    if (!counts_fit(compact_rows, g.nle)) return MOE_A2A_EINVAL;
    g.max_recv = compact_rows;
  }
  const long long most_rows = compact_rows > 0 ? (long long)compact_rows : (long long)g.nle * g.max_recv;
  if (!items_fit(most_rows, g.chunks)) return MOE_A2A_EINVAL;
  hipStream_t st = (hipStream_t)stream;
  const float scale = (float)(1 + s->rank);
#ifndef MOE_A2A_SCALE_WAVES
#define MOE_A2A_SCALE_WAVES 1
#endif
  if (MOE_A2A_SCALE_WAVES && g.vec16 && g.nle <= 64) {
    const int nvw = g.nvw < 4 ? g.nvw : 4;  // 1, 2 or 4 vectors per lane
    const int wchunks = (g.row_vecs + 64 * nvw - 1) / (64 * nvw);
    if (!items_fit(most_rows, wchunks)) return MOE_A2A_EINVAL;
    const int wgrid = mover_blocks(((long long)rows_hint * wchunks + ROWS - 1) / ROWS);
#define LAUNCH_WT(NVW, DI, DO)                                                                 \
  expert_scale_wave_kernel<NVW, DI, DO><<<wgrid, 64 * ROWS, 0, st>>>(                          \
      (const b128*)expert_x, expert_num_tokens, g.nle, g.max_recv, scale, g.row_vecs, wchunks,  \
      (b128*)expert_y, compact_rows)
#define LAUNCH_W(NVW)                                                                          \
  do {                                                                                         \
    if (in_dtype == MOE_A2A_BF16 && out_dtype == MOE_A2A_BF16)                                 \
      LAUNCH_WT(NVW, MOE_A2A_BF16, MOE_A2A_BF16);                                              \
    else if (in_dtype == MOE_A2A_F16 && out_dtype == MOE_A2A_F16)                              \
      LAUNCH_WT(NVW, MOE_A2A_F16, MOE_A2A_F16);                                                \
    else if (in_dtype == MOE_A2A_F16)                                                          \
      LAUNCH_WT(NVW, MOE_A2A_F16, MOE_A2A_BF16);                                               \
    else                                                                                       \
      LAUNCH_WT(NVW, MOE_A2A_BF16, MOE_A2A_F16);                                               \
  } while (0)
    if (nvw == 1) LAUNCH_W(1);
    else if (nvw == 2) LAUNCH_W(2);
    else LAUNCH_W(4);
#undef LAUNCH_W
#undef LAUNCH_WT
    return launch_status();
  }
  const int grid = mover_blocks((long long)rows_hint * g.chunks);
#define LAUNCH_T(V, NV, DI, DO)                                                              \
  expert_scale_kernel<V, NV, DI, DO><<<grid, BLOCK, 0, st>>>(                                \
      (const V*)expert_x, expert_num_tokens, g.nle, g.max_recv, scale, g.row_vecs, g.chunks, \
      (V*)expert_y, compact_rows)
#define LAUNCH(V, NV)                                                                         \
  do {                                                                                        \
    if (in_dtype == MOE_A2A_BF16 && out_dtype == MOE_A2A_BF16)                                \
      LAUNCH_T(V, NV, MOE_A2A_BF16, MOE_A2A_BF16);                                            \
    else if (in_dtype == MOE_A2A_F16 && out_dtype == MOE_A2A_F16)                             \
      LAUNCH_T(V, NV, MOE_A2A_F16, MOE_A2A_F16);                                              \
    else if (in_dtype == MOE_A2A_F16)                                                         \
      LAUNCH_T(V, NV, MOE_A2A_F16, MOE_A2A_BF16);                                             \
    else                                                                                      \
      LAUNCH_T(V, NV, MOE_A2A_BF16, MOE_A2A_F16);                                             \
  } while (0)
  MOE_A2A_FOR_ROW_KERNEL(g, LAUNCH);
#undef LAUNCH
#undef LAUNCH_T
  return launch_status();
}

}  // namespace

extern "C" {

int moe_a2a_expert_scale(const moe_a2a_shape* s, const void* expert_x,
                         const int32_t* expert_num_tokens, int32_t rows_hint, int32_t in_dtype,
                         int32_t out_dtype, void* expert_y, void* stream) {
  return launch_expert_scale(s, expert_x, expert_num_tokens, rows_hint, in_dtype, out_dtype, expert_y, 0, stream);
}

int moe_a2a_expert_scale_compact(const moe_a2a_shape* s, const void* expert_x,
                                 const int32_t* expert_num_tokens, int32_t rows_hint,
                                 int32_t compact_capacity_rows, int32_t in_dtype, int32_t out_dtype,
                                 void* expert_y, void* stream) {
  if (compact_capacity_rows < 1) return MOE_A2A_EINVAL;
  return launch_expert_scale(s, expert_x, expert_num_tokens, rows_hint, in_dtype, out_dtype, expert_y,
                             compact_capacity_rows, stream);
}

#ifndef MOE_A2A_GEMM_ROWS_FOR_128
#define MOE_A2A_GEMM_ROWS_FOR_128 48  // rows per group (mean, from the hint) above which blocks hold 128 tokens
#endif

}  // extern "C"

namespace {

// y[g, :rows(g), :] = x[g, :rows(g), :] @ w[g]^T (+ bias[g]) for `groups` groups of at most max_rows
// rows; rows_of_group null means max_rows rows in every group.
int launch_grouped_gemm(const void* x, const int32_t* rows_of_group, const void* w, const void* bias,
                        void* y, int groups, long long max_rows, long long rows_hint, int N, int K,
                        int dtype, hipStream_t st, int compact = 0) {
  if (dtype != MOE_A2A_F16 && dtype != MOE_A2A_BF16) return MOE_A2A_EINVAL;
  if (N % 32 != 0 || K % 8 != 0) return MOE_A2A_EINVAL;  // whole wave tiles of columns, whole 16-byte vectors
  if (!all_aligned(16, x, w, y) || !all_aligned(8, bias)) return MOE_A2A_EALIGN;
  // per-lane byte offsets inside a block of tokens and inside a wave's 32 weight rows are 32-bit
  if ((long long)K * 2 * 128 >= (1 << 30) || max_rows > INT_MAX / 2) return MOE_A2A_EINVAL;
  const int tj = rows_hint > (long long)MOE_A2A_GEMM_ROWS_FOR_128 * groups ? 4 : 2;
  // every group can end in a partly filled block of tokens; the kernel strides over what the hint misses
  const long long row_blocks = rows_hint / (tj * 32) + groups;
  // Workgroups of up to 256 columns (8 waves, one workgroup per compute unit) pull an expert's
  // token rows through half as many L1s as workgroups of 128; taken when blocks hold 128 tokens and
  // there are tiles for every unit. One workgroup per unit makes the launch a number of rounds over
  // the units, and half a round at the end leaves half the chip idle (measured: 0.66 of HBM peak at
  // 3.5 rounds, 0.71 at 7.0), so the width is the widest of 8..5 waves whose last round is nearly
  // full, judged from the blocks the row count promises (every group at least one).
#ifndef MOE_A2A_GEMM_WIDE_MIN_TILES
#define MOE_A2A_GEMM_WIDE_MIN_TILES 512
#endif
  constexpr int UNITS = 256;  // compute units of an MI355X
  int gw = 4;
  if (tj == 4 && row_blocks * ((N + 255) / 256) >= MOE_A2A_GEMM_WIDE_MIN_TILES) {
    const long long blocks = std::max<long long>(groups, (rows_hint + 127) / 128);
    double best = -1.0;
    for (int w = 8; w >= 5; --w) {
      const long long tiles = blocks * ((N + 32 * w - 1) / (32 * w));
      const double rounds = (double)tiles / UNITS, fill = rounds / std::ceil(rounds);
      if (fill >= 0.95) { gw = w; break; }
      if (fill > best) { best = fill; gw = w; }
    }
  }
  const int cols = 32 * gw;
  const int col_tiles = (N + cols - 1) / cols;
  if ((max_rows / 64 + 1) * groups * col_tiles > INT_MAX / 2) return MOE_A2A_EINVAL;
  const int grid = mover_blocks(row_blocks * col_tiles);
#define LAUNCH_G(DT, TJ, GW)                                                                          \
  expert_gemm_kernel<DT, TJ, GW><<<grid, 64 * GW, 0, st>>>((const b128*)x, rows_of_group, (const b128*)w, \
                                                           (const uint16_t*)bias, (uint16_t*)y, groups,  \
                                                           (int)max_rows, N, K, col_tiles, compact)
#define LAUNCH_GW(DT)                                 \
  do {                                                \
    if (tj == 2) LAUNCH_G(DT, 2, 4);                  \
    else if (gw == 8) LAUNCH_G(DT, 4, 8);             \
    else if (gw == 7) LAUNCH_G(DT, 4, 7);             \
    else if (gw == 6) LAUNCH_G(DT, 4, 6);             \
    else if (gw == 5) LAUNCH_G(DT, 4, 5);             \
    else LAUNCH_G(DT, 4, 4);                          \
  } while (0)
  if (dtype == MOE_A2A_BF16) LAUNCH_GW(MOE_A2A_BF16);
  else LAUNCH_GW(MOE_A2A_F16);
#undef LAUNCH_GW
#undef LAUNCH_G
  return launch_status();
}

#ifndef MOE_A2A_DENSE_TILE
#define MOE_A2A_DENSE_TILE 0  // (measurements) 256, 128 or 64: that tile height for every shape
#endif
constexpr int MOE_A2A_NOT_DENSE = 1;  // (internal) the shape is left to the next kernel

// Which tile the dense kernel uses for an M x N x K product: 256 x 256 (one workgroup per compute
// unit, the highest rate per unit once every unit has work for several tiles), 128 x 128 (two
// workgroups per unit, about 0.8 of that rate, but four times the tiles: fuller last round, and
// one workgroup's prologue and epilogue overlap the other's MFMAs, which decides short K) or
// 64 x 128 (for outputs that even 128 x 128 tiles cannot spread over the 256 units).
// The costs are in units of a 128 x 128 tile's work at the big tile's rate; the constants are
// fits to measurements on an MI355X (rows 64 .. 8192, K 256 .. 4608).
int dense_tile_rows(long long M, long long N, int K) {
  if (MOE_A2A_DENSE_TILE) return MOE_A2A_DENSE_TILE;
  constexpr double UNITS = 256.0;
  const double steps = (K + GEMM_KSTEP - 1) / GEMM_KSTEP;
  const double big = (double)((M + 255) / 256) * (double)((N + 255) / 256);
  const double mid = (double)((M + 127) / 128) * (double)((N + 127) / 128);
  const double low = (double)((M + 63) / 64) * (double)((N + 127) / 128);
  if (low <= UNITS) return 64;
  // a last round that is partly empty costs about half of what it leaves idle (the busy units
  // run faster meanwhile); per tile, fixed work worth 3 steps (big) and 1 step (mid)
  const double big_cost = 4.0 * 0.5 * (big / UNITS + ceil(big / UNITS)) * (steps + 3.0) / steps;
  const double mid_cost = 1.25 * fmax(mid / UNITS, 1.0) * (steps + 1.0) / steps;
  return big_cost <= mid_cost ? 256 : 128;
}

constexpr size_t dense_lds_bytes(int BM, int BN) { return 2 * (size_t)(BM + BN) * 8 * sizeof(b128); }
constexpr size_t skinny_lds_bytes(int tj, int waves) { return (size_t)waves * (32 + 32 * tj) * 8 * sizeof(b128); }

// The tile buffers can be more LDS than a kernel gets by default: allowed once per GPU, for every
// tile and type at once, so that only the first dense call on a GPU touches kernel attributes.
int allow_large_lds() {
  static bool allowed[MAX_GPUS] = {};
  int gpu = -1;
  if (hipGetDevice(&gpu) != hipSuccess || gpu < 0 || gpu >= MAX_GPUS) return MOE_A2A_ELAUNCH;
  std::lock_guard<std::mutex> lock(static_plan_mutex);
  if (allowed[gpu]) return MOE_A2A_OK;
  bool ok = true;
  auto allow = [&](const void* kernel, size_t bytes) {
    ok = ok && hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) == hipSuccess;
  };
  allow((const void*)dense_gemm_kernel<MOE_A2A_BF16, 2, 2, 4, 4, false>, dense_lds_bytes(256, 256));
  allow((const void*)dense_gemm_kernel<MOE_A2A_F16, 2, 2, 4, 4, false>, dense_lds_bytes(256, 256));
  allow((const void*)dense_gemm_kernel<MOE_A2A_BF16, 2, 2, 2, 2, false>, dense_lds_bytes(128, 128));
  allow((const void*)dense_gemm_kernel<MOE_A2A_F16, 2, 2, 2, 2, false>, dense_lds_bytes(128, 128));
  allow((const void*)dense_gemm_kernel<MOE_A2A_BF16, 2, 2, 1, 2, false>, dense_lds_bytes(64, 128));
  allow((const void*)dense_gemm_kernel<MOE_A2A_F16, 2, 2, 1, 2, false>, dense_lds_bytes(64, 128));
  allow((const void*)dense_gemm_kernel<MOE_A2A_BF16, 2, 2, 4, 4, true>, dense_lds_bytes(256, 256));
  allow((const void*)dense_gemm_kernel<MOE_A2A_F16, 2, 2, 4, 4, true>, dense_lds_bytes(256, 256));
  allow((const void*)dense_gemm_kernel<MOE_A2A_BF16, 2, 2, 2, 2, true>, dense_lds_bytes(128, 128));
  allow((const void*)dense_gemm_kernel<MOE_A2A_F16, 2, 2, 2, 2, true>, dense_lds_bytes(128, 128));
  allow((const void*)dense_gemm_kernel<MOE_A2A_BF16, 2, 2, 1, 2, true>, dense_lds_bytes(64, 128));
  allow((const void*)dense_gemm_kernel<MOE_A2A_F16, 2, 2, 1, 2, true>, dense_lds_bytes(64, 128));
  allow((const void*)skinny_gemm_kernel<MOE_A2A_BF16, 2, 8>, skinny_lds_bytes(2, 8));
  allow((const void*)skinny_gemm_kernel<MOE_A2A_F16, 2, 8>, skinny_lds_bytes(2, 8));
  if (!ok) return MOE_A2A_ELAUNCH;
  allowed[gpu] = true;
  return MOE_A2A_OK;
}

// The dense kernel for products of more than a few rows; MOE_A2A_NOT_DENSE otherwise (the kernels
// that split K over the waves of a workgroup or stream the weights once).
int launch_dense_gemm(const void* a, const void* b, const void* bias, void* c, int M, int N, int K,
                      int dtype, hipStream_t st) {
  if (dtype != MOE_A2A_F16 && dtype != MOE_A2A_BF16) return MOE_A2A_EINVAL;
  if (N % 32 != 0 || K % 8 != 0) return MOE_A2A_EINVAL;
  if (!all_aligned(16, a, b, c) || !all_aligned(8, bias)) return MOE_A2A_EALIGN;
  if ((long long)K * 2 * 256 >= (1 << 30)) return MOE_A2A_NOT_DENSE;  // 32-bit byte offsets inside a tile's rows
  const int tile = dense_tile_rows(M, N, K);
  const int BM = tile, BN = tile == 64 ? 128 : tile;
  const long long tiles_m = ((long long)M + BM - 1) / BM, tiles_n = ((long long)N + BN - 1) / BN;
  if (tiles_m * tiles_n > INT_MAX / 2) return MOE_A2A_NOT_DENSE;
  const size_t lds_bytes = dense_lds_bytes(BM, BN);
  const int grid = (int)(tiles_m * tiles_n);
  if (const int rc = allow_large_lds()) return rc;
#define LAUNCH_D(DT, TM, TN)                                                             \
  dense_gemm_kernel<DT, 2, 2, TM, TN, false><<<grid, 256, lds_bytes, st>>>(              \
      (const b128*)a, (const b128*)b, (const uint16_t*)bias, (uint16_t*)c, M, N, K, (int)tiles_m, (int)tiles_n, \
      nullptr, 0, 0, 0)
#define LAUNCH_DT(DT)                         \
  do {                                        \
    if (tile == 256) LAUNCH_D(DT, 4, 4);      \
    else if (tile == 128) LAUNCH_D(DT, 2, 2); \
    else LAUNCH_D(DT, 1, 2);                  \
  } while (0)
  if (dtype == MOE_A2A_BF16) LAUNCH_DT(MOE_A2A_BF16);
  else LAUNCH_DT(MOE_A2A_F16);
#undef LAUNCH_DT
#undef LAUNCH_D
  return launch_status();
}

#ifndef MOE_A2A_GROUPED_DENSE_MIN_ROWS
#define MOE_A2A_GROUPED_DENSE_MIN_ROWS 56  // rows per group (from the caller's row count) from which tiles are used
#endif
#ifndef MOE_A2A_GROUPED_DENSE_BIG_ROWS
#define MOE_A2A_GROUPED_DENSE_BIG_ROWS 768  // ... and from which they are 256 x 256 instead of 128 x 128
#endif

// The grouped product when groups have hundreds of rows: the weights are then read for enough
// rows that the matrix cores, not the stream of weights, bound the work, and the dense kernel's
// tiles (each weight row read once per 128 or 256 rows, operands shared by four waves through
// LDS) do better than the kernel that is built around streaming. MOE_A2A_NOT_DENSE otherwise.
int launch_grouped_dense(const void* x, const int32_t* rows_of_group, const void* w, const void* bias, void* y,
                         int groups, long long max_rows, long long rows_hint, int N, int K, int dtype,
                         hipStream_t st, int compact = 0) {
  if (dtype != MOE_A2A_F16 && dtype != MOE_A2A_BF16) return MOE_A2A_EINVAL;
  if (N % 32 != 0 || K % 8 != 0) return MOE_A2A_EINVAL;
  if (!all_aligned(16, x, w, y) || !all_aligned(8, bias)) return MOE_A2A_EALIGN;
  if (!rows_of_group || rows_hint < (long long)MOE_A2A_GROUPED_DENSE_MIN_ROWS * groups) return MOE_A2A_NOT_DENSE;
  if ((long long)K * 2 * 256 >= (1 << 30) || max_rows > INT_MAX / 2) return MOE_A2A_NOT_DENSE;
#ifndef MOE_A2A_GROUPED_DENSE_TILE
#define MOE_A2A_GROUPED_DENSE_TILE 0  // (measurements) 256, 128 or 64: that tile height for every launch
#endif
  // 256 x 256 when groups have rows for several bands of them; 64 x 128 when tiles of 128 x 128
  // would not give every compute unit one
  const int tile = MOE_A2A_GROUPED_DENSE_TILE ? MOE_A2A_GROUPED_DENSE_TILE
                   : rows_hint >= (long long)MOE_A2A_GROUPED_DENSE_BIG_ROWS * groups ? 256
                   : (rows_hint / 128 + groups) * ((N + 127) / 128) <= 256 ? 64 : 128;
  const int BM = tile, BN = tile == 64 ? 128 : tile;
  const long long tiles_n = (N + BN - 1) / BN;
  // every group can end in a partly filled row tile; the kernel strides over what the hint misses
  const long long pairs = (rows_hint / BM + groups) * tiles_n;
  if ((max_rows / BM + 1) * groups * tiles_n > INT_MAX / 2) return MOE_A2A_NOT_DENSE;
  const int grid = mover_blocks(pairs);
  const size_t lds_bytes = dense_lds_bytes(BM, BN);
  if (const int rc = allow_large_lds()) return rc;
#define LAUNCH_GD(DT, TM, TN)                                                                 \
  dense_gemm_kernel<DT, 2, 2, TM, TN, true><<<grid, 256, lds_bytes, st>>>(                    \
      (const b128*)x, (const b128*)w, (const uint16_t*)bias, (uint16_t*)y, 0, N, K, 0, (int)tiles_n,        \
      rows_of_group, groups, (int)max_rows, compact)
  if (dtype == MOE_A2A_BF16) {
    if (tile == 256) LAUNCH_GD(MOE_A2A_BF16, 4, 4);
    else if (tile == 128) LAUNCH_GD(MOE_A2A_BF16, 2, 2);
    else LAUNCH_GD(MOE_A2A_BF16, 1, 2);
  } else {
    if (tile == 256) LAUNCH_GD(MOE_A2A_F16, 4, 4);
    else if (tile == 128) LAUNCH_GD(MOE_A2A_F16, 2, 2);
    else LAUNCH_GD(MOE_A2A_F16, 1, 2);
  }
#undef LAUNCH_GD
  return launch_status();
}

#ifndef MOE_A2A_SKINNY_WAVES
#define MOE_A2A_SKINNY_WAVES 0  // (measurements) 4 or 8: that many waves for every shape
#endif
#ifndef MOE_A2A_SKINNY_MAX_TILES
#define MOE_A2A_SKINNY_MAX_TILES 192  // tiles of 128 columns below which K is split inside the workgroup
#endif

// Products of at most 64 rows whose tiles of 128 columns would leave compute units idle: 32
// columns per workgroup, K split over its waves. MOE_A2A_NOT_DENSE when the grouped kernel is
// the better fit.
int launch_skinny_gemm(const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                       int dtype, hipStream_t st) {
  if (dtype != MOE_A2A_F16 && dtype != MOE_A2A_BF16) return MOE_A2A_EINVAL;
  if (N % 32 != 0 || K % 8 != 0) return MOE_A2A_EINVAL;
  if (!all_aligned(16, x, w, y) || !all_aligned(8, bias)) return MOE_A2A_EALIGN;
  if (M > 64 || (long long)K * 2 * 128 >= (1 << 30)) return MOE_A2A_NOT_DENSE;
  const int wide_tiles = (N + GEMM_COLS - 1) / GEMM_COLS;
  const int steps = (K + GEMM_KSTEP - 1) / GEMM_KSTEP;
  if (wide_tiles >= MOE_A2A_SKINNY_MAX_TILES || steps < 2 * NWAVES) return MOE_A2A_NOT_DENSE;
  const int grid = N / 32;
  // eight waves keep more of the stream in flight (measured 10 to 13 % less time from 28 steps
  // on); with few steps the four extra partial sums cost more than that
  const int waves = MOE_A2A_SKINNY_WAVES ? MOE_A2A_SKINNY_WAVES : steps >= 24 ? 8 : 4;
  const int tj = M <= 32 ? 1 : 2;
  if (const int rc = allow_large_lds()) return rc;
#define LAUNCH_K(DT, TJ, KW)                                                              \
  skinny_gemm_kernel<DT, TJ, KW><<<grid, 64 * KW, skinny_lds_bytes(TJ, KW), st>>>(        \
      (const b128*)x, (const b128*)w, (const uint16_t*)bias, (uint16_t*)y, M, N, K, N / 32)
#define LAUNCH_KW(DT)                                      \
  do {                                                     \
    if (waves == 8 && tj == 2) LAUNCH_K(DT, 2, 8);         \
    else if (waves == 8) LAUNCH_K(DT, 1, 8);               \
    else if (tj == 2) LAUNCH_K(DT, 2, 4);                  \
    else LAUNCH_K(DT, 1, 4);                               \
  } while (0)
  if (dtype == MOE_A2A_BF16) LAUNCH_KW(MOE_A2A_BF16);
  else LAUNCH_KW(MOE_A2A_F16);
#undef LAUNCH_KW
#undef LAUNCH_K
  return launch_status();
}

}  // namespace

extern "C" {

int moe_a2a_expert_gemm(const moe_a2a_shape* s, const void* expert_x,
                        const int32_t* expert_num_tokens, int32_t rows_hint, const void* weights,
                        const void* bias, int32_t in_dim, int32_t out_dim, int32_t dtype,
                        void* expert_y, void* stream) {
  if (!shape_ok(s) || rows_hint < 0 || in_dim < 1 || out_dim < 1 || !expert_x || !expert_num_tokens ||
      !weights || !expert_y)
    return MOE_A2A_EINVAL;
  const int nle = s->num_experts / s->world_size;
  const long long max_recv = (long long)s->max_num_tokens * s->world_size;
  const int dense = launch_grouped_dense(expert_x, expert_num_tokens, weights, bias, expert_y, nle, max_recv,
                                         rows_hint, out_dim, in_dim, dtype, (hipStream_t)stream);
  if (dense != MOE_A2A_NOT_DENSE) return dense;
  return launch_grouped_gemm(expert_x, expert_num_tokens, weights, bias, expert_y, nle, max_recv, rows_hint,
                             out_dim, in_dim, dtype, (hipStream_t)stream);
}

int moe_a2a_expert_gemm_compact(const moe_a2a_shape* s, const void* expert_x,
                                const int32_t* expert_num_tokens, int32_t rows_hint,
                                int32_t compact_capacity_rows, const void* weights, const void* bias,
                                int32_t in_dim, int32_t out_dim, int32_t dtype, void* expert_y,
                                void* stream) {
  if (!shape_ok(s) || rows_hint < 0 || compact_capacity_rows < 1 || in_dim < 1 || out_dim < 1 || !expert_x ||
      !expert_num_tokens || !weights || !expert_y)
    return MOE_A2A_EINVAL;
  const int nle = s->num_experts / s->world_size;
  if (!counts_fit(compact_capacity_rows, nle)) return MOE_A2A_EINVAL;
  // (every count is cut to the rows the buffers hold; counts that dispatch_recv_compact wrote add up to at most that)
  const int dense = launch_grouped_dense(expert_x, expert_num_tokens, weights, bias, expert_y, nle,
                                         compact_capacity_rows, rows_hint, out_dim, in_dim, dtype,
                                         (hipStream_t)stream, 1);
  if (dense != MOE_A2A_NOT_DENSE) return dense;
  return launch_grouped_gemm(expert_x, expert_num_tokens, weights, bias, expert_y, nle, compact_capacity_rows,
                             rows_hint, out_dim, in_dim, dtype, (hipStream_t)stream, 1);
}

int moe_a2a_linear(const void* input, const void* weight, const void* bias, int32_t m, int32_t n,
                   int32_t k, int32_t dtype, void* output, void* stream) {
  if (m < 0 || n < 1 || k < 1 || !weight || (m > 0 && (!input || !output))) return MOE_A2A_EINVAL;
  if (m == 0) return MOE_A2A_OK;
  const int skinny = launch_skinny_gemm(input, weight, bias, output, m, n, k, dtype, (hipStream_t)stream);
  if (skinny != MOE_A2A_NOT_DENSE) return skinny;
  const int dense = launch_dense_gemm(input, weight, bias, output, m, n, k, dtype, (hipStream_t)stream);
  if (dense != MOE_A2A_NOT_DENSE) return dense;
  return launch_grouped_gemm(input, nullptr, weight, bias, output, 1, m, m, n, k, dtype,
                             (hipStream_t)stream);
}

int moe_a2a_exchange_local(int32_t world_size, int32_t hidden_dim, const void* send_buf,
                           const int32_t* send_meta, const int32_t* send_counts, int32_t dst_rank,
                           void* recv_buf, int32_t* recv_meta, const int32_t* recv_counts,
                           int32_t src_rank, int32_t rows_hint, int32_t send_capacity_rows,
                           int32_t recv_capacity_rows, void* stream) {
  if (world_size < 1 || hidden_dim < 1 || dst_rank < 0 || dst_rank >= world_size ||
      src_rank < 0 || src_rank >= world_size || rows_hint < 0 || send_capacity_rows < 0 ||
      recv_capacity_rows < 0 || !send_counts || !recv_counts ||
      !counts_fit(send_capacity_rows, world_size) || !counts_fit(recv_capacity_rows, world_size))
    return MOE_A2A_EINVAL;
  if (send_capacity_rows == 0 || recv_capacity_rows == 0) return MOE_A2A_OK;  // nothing can move
  if (!send_buf || !send_meta || !recv_buf || !recv_meta) return MOE_A2A_EINVAL;
  if (!all_aligned(2, send_buf, recv_buf)) return MOE_A2A_EALIGN;
  Geometry g{};
  row_geometry(g, hidden_dim, all_aligned(16, send_buf, recv_buf));
  if (!items_fit(rows_hint, g.chunks)) return MOE_A2A_EINVAL;
  const int grid = mover_blocks((long long)rows_hint * g.chunks);
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(V, NV)                                                                         \
  exchange_local_kernel<V, NV><<<grid, BLOCK, 0, st>>>(                                       \
      (const V*)send_buf, send_meta, send_counts, dst_rank, (V*)recv_buf, recv_meta,          \
      recv_counts, src_rank, g.row_vecs, g.chunks, send_capacity_rows, recv_capacity_rows)
  MOE_A2A_FOR_ROW_KERNEL(g, LAUNCH);
#undef LAUNCH
  return launch_status();
}

int moe_a2a_exchange_gather_local(int32_t world_size, int32_t hidden_dim, const void* const* send_bufs,
                                  const int32_t* const* send_metas, const int32_t* const* send_counts,
                                  int32_t dst_rank, void* recv_buf, int32_t* recv_meta,
                                  int32_t* recv_counts, int32_t rows_hint, int32_t send_capacity_rows,
                                  int32_t recv_capacity_rows, void* stream) {
  if (world_size < 1 || world_size > GATHER_MAX_RANKS || hidden_dim < 1 || dst_rank < 0 ||
      dst_rank >= world_size || rows_hint < 0 || send_capacity_rows < 0 || recv_capacity_rows < 0 ||
      !send_bufs || !send_metas || !send_counts || !recv_counts ||
      !counts_fit(send_capacity_rows, world_size) || !counts_fit(recv_capacity_rows, world_size))
    return MOE_A2A_EINVAL;
  GatherSources src{};
  bool all16 = aligned(recv_buf, 16);
  for (int r = 0; r < world_size; ++r) {
    if (!send_counts[r]) return MOE_A2A_EINVAL;
    if (send_capacity_rows > 0 && (!send_bufs[r] || !send_metas[r])) return MOE_A2A_EINVAL;
    if (!aligned(send_bufs[r], 2)) return MOE_A2A_EALIGN;
    all16 = all16 && aligned(send_bufs[r], 16);
    src.buf[r] = send_bufs[r];
    src.meta[r] = send_metas[r];
    src.counts[r] = send_counts[r];
  }
  if (send_capacity_rows > 0 && recv_capacity_rows > 0 && (!recv_buf || !recv_meta)) return MOE_A2A_EINVAL;
  if (!aligned(recv_buf, 2)) return MOE_A2A_EALIGN;
  Geometry g{};
  row_geometry(g, hidden_dim, all16);
  if (!items_fit(rows_hint, g.chunks)) return MOE_A2A_EINVAL;
  // (the launch also delivers the counts, so it is made even when no row can move)
  const dim3 grid(std::min(mover_blocks((long long)rows_hint * g.chunks), 1 << 16), world_size);
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(V, NV)                                                                          \
  exchange_gather_kernel<V, NV><<<grid, BLOCK, 0, st>>>(src, world_size, dst_rank, (V*)recv_buf, \
                                                        recv_meta, recv_counts, g.row_vecs, g.chunks, \
                                                        send_capacity_rows, recv_capacity_rows)
  MOE_A2A_FOR_ROW_KERNEL(g, LAUNCH);
#undef LAUNCH
  return launch_status();
}


}  // extern "C"
