// MoE dispatch/combine for one rank on MI355X (gfx950, wave64).
//
// Every stage is a "ranked row move": a workgroup owns one (row, chunk) item,
// issues the 16-byte loads of its payload first, then finds the row's
// destination slot by COUNTING the keys that precede it in the stage's stable
// order (a few KB of keys, L2-resident, scanned by all 256 lanes and reduced
// with a wave64 butterfly + LDS), then stores. There are no atomics on global
// memory, no counters to clear and no cross-workgroup dependencies, so the
// result is the same on every run and nothing has to be zeroed between calls.
//
// Reference behaviour reproduced here: all2all/reference.py:68-148 (dispatch),
// :151-234 (combine), :262 (simulated expert).

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <limits.h>

#include "moe_a2a.h"

namespace {

constexpr int META = MOE_A2A_META_DIM;
constexpr int BLOCK = 256;            // 4 wave64 per workgroup
constexpr int NWAVES = BLOCK / 64;
constexpr int COMBINE_CAP = 64;       // addends per token handled by the fast path
constexpr int COMBINE_WEIGHTS = 128;  // weights of one token staged in LDS
constexpr int COMBINE_BATCH = 8;      // addend rows loaded before accumulating
constexpr int MAX_LOCAL_EXPERTS = 4096;  // LDS prefix table of the expert-major walkers
constexpr int NUM_XCD = 8;

// 16 bytes as a native clang vector: loads and stores of it are single
// global_load/store_dwordx4 and the value lives in registers. (HIP's uint4 is a
// struct whose copies become memcpy calls that can pin a local in memory.)
typedef unsigned int b128 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------- wave / block primitives

__device__ __forceinline__ int wave_sum(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Sum over the workgroup; every lane gets the total. `red` is NWAVES ints of
// LDS and may be reused right after the call returns.
__device__ __forceinline__ int block_sum(int v, int* red) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  int s = 0;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) s += red[w];
  __syncthreads();
  return s;
}

// Inclusive prefix sum across the 64 lanes of a wave.
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int n = __shfl_up(v, o, 64);
    if (lane >= o) v += n;
  }
  return v;
}

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
// Ids below 0 and ids >= E form two extra classes before / after all ranks, so
// the classes always partition the integers and slots stay a permutation.
__device__ __forceinline__ void dest_class(int e, int nle, int E, uint32_t magic, int& lo, int& hi,
                                           int& d) {
  if (e < 0) {
    lo = INT_MIN; hi = -1; d = -1;
  } else if (e >= E) {
    lo = E; hi = INT_MAX; d = INT_MAX;
  } else {
    d = (nle == 1) ? e : (int)__umulhi((uint32_t)e, magic);
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
    for (int j = 0; j < NV; ++j) v[j] = row[min(base + j * BLOCK + (int)threadIdx.x, row_vecs - 1)];
  }
  __device__ __forceinline__ void store(V* __restrict__ row, int base, int row_vecs) const {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int idx = base + j * BLOCK + threadIdx.x;
      if (idx < row_vecs) row[idx] = v[j];
    }
  }
  template <typename F>
  __device__ __forceinline__ void map(F f) {
#pragma unroll
    for (int j = 0; j < NV; ++j) v[j] = f(v[j]);
  }
};

__device__ __forceinline__ int sum_counts(const int* __restrict__ counts, int n) {
  int s = 0;
  for (int i = 0; i < n; ++i) s += max(counts[i], 0);
  return s;
}

// Number of keys i in [0, n) that pass `test(key_i, i)`, summed over the lanes
// of this thread only (reduce with block_sum). `load(i)` fetches key i; loads
// are issued SCAN_UNROLL at a time with clamped indices so that all of them are
// in flight before the first compare, and lanes past n are masked out.
constexpr int SCAN_UNROLL = 8;
template <int BLK, typename Load, typename Test>
__device__ __forceinline__ int count_keys(int n, Load load, Test test) {
  int cnt = 0;
  for (int i = threadIdx.x; i < n; i += SCAN_UNROLL * BLK) {
    int key[SCAN_UNROLL];
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u) key[u] = load(min(i + u * BLK, n - 1));
#pragma unroll
    for (int u = 0; u < SCAN_UNROLL; ++u)
      cnt += (i + u * BLK < n) ? (int)test(key[u], i + u * BLK) : 0;
  }
  return cnt;
}

// ---------------------------------------------------------------- stage 1: dispatch, send side
//
// grid = W counting workgroups (rows per destination rank) followed by one
// workgroup per (entry, chunk). Entry i = t*K + k goes to slot
//   #{entries of a lower destination} + #{earlier entries of the same destination}.

template <typename V, int NV>
__global__ __launch_bounds__(BLOCK, 8) void dispatch_send_kernel(
    const V* __restrict__ x, const int* __restrict__ indices, int S, int K, int nle, int E, int W,
    uint32_t magic, int rank, int row_vecs, int chunks, V* __restrict__ send_buf,
    int* __restrict__ send_meta, int* __restrict__ send_counts, int* __restrict__ send_slot) {
  __shared__ int red[NWAVES];
  const int tid = threadIdx.x;
  auto key = [indices](int i) { return indices[i]; };

  if ((int)blockIdx.x < W) {
    const int lo = blockIdx.x * nle, hi = lo + nle - 1;
    int c = count_keys<BLOCK>(S, key, [lo, hi](int e, int) { return (e >= lo) & (e <= hi); });
    c = block_sum(c, red);
    if (tid == 0) send_counts[blockIdx.x] = c;
    return;
  }

  const int items = S * chunks, movers = gridDim.x - W;
  for (int q = xcd_contiguous(blockIdx.x - W, movers); q < items; q += movers) {
    const int i = chunks == 1 ? q : q / chunks, c = q - i * chunks;
    const int e = indices[i];
    const int t = i / K, k = i - t * K;
    const int base = c * (BLOCK * NV);

    Payload<V, NV> p;
    p.load(x + (size_t)t * row_vecs, base, row_vecs);

    int lo, hi, d;
    dest_class(e, nle, E, magic, lo, hi, d);
    const int cnt = count_keys<BLOCK>(S, key, [lo, hi, i](int e2, int i2) {
      return (e2 < lo) | ((e2 <= hi) & (e2 >= lo) & (i2 < i));
    });
    const int slot = block_sum(cnt, red);

    p.store(send_buf + (size_t)slot * row_vecs, base, row_vecs);
    if (c == 0) {
      if (tid < META) {
        int m = tid == 0 ? e : tid == 1 ? rank : tid == 2 ? t : tid == 3 ? k : 0;
        send_meta[(size_t)slot * META + tid] = m;
      }
      if (tid == 0 && send_slot) send_slot[i] = slot;
    }
  }
}

// ---------------------------------------------------------------- stage 2: dispatch, receive side
//
// grid = nle counting workgroups (rows per local expert) followed by one
// workgroup per (received row, chunk). Row i goes to expert le = e % nle at
// position #{earlier rows of the same expert}.

template <typename V, int NV>
__global__ __launch_bounds__(BLOCK, 8) void dispatch_recv_kernel(
    const V* __restrict__ recv_buf, const int* __restrict__ recv_meta,
    const int* __restrict__ recv_counts, int W, int nle, uint32_t magic, int max_recv,
    int row_vecs, int chunks, int* __restrict__ expert_num_tokens, V* __restrict__ expert_x,
    int* __restrict__ expert_meta) {
  __shared__ int red[NWAVES];
  const int tid = threadIdx.x;
  const int R = sum_counts(recv_counts, W);
  auto key = [recv_meta](int i) { return recv_meta[(size_t)i * META]; };

  if ((int)blockIdx.x < nle) {
    const int me = blockIdx.x;
    int c = count_keys<BLOCK>(R, key, [=](int e, int) { return floormod(e, nle, magic) == me; });
    c = block_sum(c, red);
    if (tid == 0) expert_num_tokens[me] = c;
    return;
  }

  const int items = R * chunks, movers = gridDim.x - nle;
  for (int q = blockIdx.x - nle; q < items; q += movers) {
    const int i = chunks == 1 ? q : q / chunks, c = q - i * chunks;
    const int base = c * (BLOCK * NV);

    Payload<V, NV> p;
    p.load(recv_buf + (size_t)i * row_vecs, base, row_vecs);

    int m = 0;
    if (c == 0 && tid < META) m = recv_meta[(size_t)i * META + tid];
    const int le = floormod(recv_meta[(size_t)i * META], nle, magic);
    const int cnt =
        count_keys<BLOCK>(i, key, [=](int e2, int) { return floormod(e2, nle, magic) == le; });
    const int pos = block_sum(cnt, red);

    if (pos < max_recv) {
      const size_t row = (size_t)le * max_recv + pos;
      p.store(expert_x + row * row_vecs, base, row_vecs);
      if (c == 0 && tid < META) expert_meta[row * META + tid] = m;
    }
  }
}

// ---------------------------------------------------------------- expert-major stream helpers

// pre[0..nle] = exclusive prefix of min(cnt[le], max_recv); returns the total.
// Each lane owns a contiguous run of experts; runs are combined by a wave64
// scan and a scan over the wave totals.
__device__ __forceinline__ int expert_prefix(const int* __restrict__ cnt, int nle, int max_recv,
                                             int* pre, int* red) {
  const int tid = threadIdx.x;
  const int per = (nle + BLOCK - 1) / BLOCK;
  const int b = min(tid * per, nle), e = min(b + per, nle);
  int s = 0;
  for (int i = b; i < e; ++i) s += min(max(cnt[i], 0), max_recv);
  const int inc = wave_inclusive_scan(s);
  if ((tid & 63) == 63) red[tid >> 6] = inc;
  __syncthreads();
  int off = 0, total = 0;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) {
    if (w < (tid >> 6)) off += red[w];
    total += red[w];
  }
  int run = off + inc - s;
  for (int i = b; i < e; ++i) {
    pre[i] = run;
    run += min(max(cnt[i], 0), max_recv);
  }
  if (tid == 0) pre[nle] = total;
  __syncthreads();
  return total;
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

// Key (one int of the meta row) of SCAN_UNROLL rows of the expert-major stream
// at once: the searches advance in lock step so their LDS reads overlap.
template <int FIELD>
struct ExpertStreamKeys {
  const int* pre;
  const int* __restrict__ meta;
  int nle, top, max_recv;
  __device__ __forceinline__ int operator()(int g) const {
    const int le = expert_of(pre, nle, top, g);
    const size_t row = (size_t)le * max_recv + (g - pre[le]);
    return meta[row * META + FIELD];
  }
};

// ---------------------------------------------------------------- stage 3: combine, send side
//
// grid = W counting workgroups (rows per origin rank) followed by one workgroup
// per (valid expert row, chunk), rows numbered g in (le, j) order. Row g with
// origin d goes to slot #{rows of a lower origin} + #{earlier rows of origin d}.

template <typename V, int NV>
__global__ __launch_bounds__(BLOCK, 8) void combine_send_kernel(
    const V* __restrict__ expert_y, const int* __restrict__ expert_meta,
    const int* __restrict__ expert_num_tokens, int nle, int max_recv, int W, int row_vecs,
    int chunks, V* __restrict__ send_buf, int* __restrict__ send_meta,
    int* __restrict__ send_counts) {
  __shared__ int red[NWAVES];
  __shared__ int pre[MAX_LOCAL_EXPERTS + 1];
  const int tid = threadIdx.x;
  const int R = expert_prefix(expert_num_tokens, nle, max_recv, pre, red);
  const ExpertStreamKeys<1> key{pre, expert_meta, nle, top_step(nle), max_recv};

  if ((int)blockIdx.x < W) {
    const int me = blockIdx.x;
    int c = count_keys<BLOCK>(R, key, [me](int d, int) { return d == me; });
    c = block_sum(c, red);
    if (tid == 0) send_counts[me] = c;
    return;
  }

  const int items = R * chunks, movers = gridDim.x - W;
  for (int q = blockIdx.x - W; q < items; q += movers) {
    const int g = chunks == 1 ? q : q / chunks, c = q - g * chunks;
    const int base = c * (BLOCK * NV);
    const int le = expert_of(pre, nle, key.top, g);
    const size_t row = (size_t)le * max_recv + (g - pre[le]);

    Payload<V, NV> p;
    p.load(expert_y + row * row_vecs, base, row_vecs);

    int m = 0;
    if (c == 0 && tid < META) m = expert_meta[row * META + tid];
    const int d = expert_meta[row * META + 1];
    const int cnt = count_keys<BLOCK>(
        R, key, [d, g](int d2, int g2) { return (d2 < d) | ((d2 == d) & (g2 < g)); });
    const int slot = block_sum(cnt, red);

    p.store(send_buf + (size_t)slot * row_vecs, base, row_vecs);
    if (c == 0 && tid < META) send_meta[(size_t)slot * META + tid] = m;
  }
}

// ---------------------------------------------------------------- 16-bit float helpers

template <int DT> __device__ __forceinline__ float to_f32(uint16_t b);
template <> __device__ __forceinline__ float to_f32<MOE_A2A_BF16>(uint16_t b) {
  return __uint_as_float((uint32_t)b << 16);
}
template <> __device__ __forceinline__ float to_f32<MOE_A2A_F16>(uint16_t b) {
  return __half2float(__ushort_as_half(b));
}

// Round to nearest even, the conversion torch applies when it stores a float
// into a 16-bit tensor.
template <int DT> __device__ __forceinline__ uint16_t to_b16(float f);
template <> __device__ __forceinline__ uint16_t to_b16<MOE_A2A_BF16>(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
template <> __device__ __forceinline__ uint16_t to_b16<MOE_A2A_F16>(float f) {
  return __half_as_ushort(__float2half_rn(f));
}

template <typename V> struct Lanes;  // 16-bit elements held by one vector
template <> struct Lanes<b128> { static constexpr int N = 8; };
template <> struct Lanes<uint16_t> { static constexpr int N = 1; };

template <typename V>
__device__ __forceinline__ uint16_t get16(const V& v, int e) {
  if constexpr (Lanes<V>::N == 1) {
    return v;
  } else {
    const uint32_t w = e < 2 ? v.x : e < 4 ? v.y : e < 6 ? v.z : v.w;
    return (uint16_t)((e & 1) ? (w >> 16) : (w & 0xffffu));
  }
}

template <typename V>
__device__ __forceinline__ V pack16(const uint16_t* h) {
  if constexpr (Lanes<V>::N == 1) {
    return h[0];
  } else {
    b128 v;
    v.x = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
    v.y = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
    v.z = (uint32_t)h[4] | ((uint32_t)h[5] << 16);
    v.w = (uint32_t)h[6] | ((uint32_t)h[7] << 16);
    return v;
  }
}

// ---------------------------------------------------------------- stage 4: combine, receive side

// One step of `out[t] += row.float() * w` on a 16-bit accumulator.
template <int DT>
__device__ __forceinline__ float combine_step(float acc, uint16_t v, float w) {
  const float p = __fmul_rn(to_f32<DT>(v), w);
  const float a = __fadd_rn(acc, p);
  return to_f32<DT>(to_b16<DT>(a));
}

// Workgroup of BLK lanes per (token, chunk); each lane owns NV vector columns.
// The workgroup finds the rows addressed to its token by scanning the src_token
// column of the arriving meta rows, orders them by arrival index, then walks
// them in that order with all rows of a batch loaded up front.
template <typename V, int DT, int BLK, int NV>
__global__ __launch_bounds__(BLK) void combine_recv_kernel(
    const V* __restrict__ recv_buf, const int* __restrict__ recv_meta,
    const int* __restrict__ recv_counts, int W, const float* __restrict__ weights, int T, int K,
    int row_vecs, int chunks, V* __restrict__ out, int accumulate) {
  constexpr int N = Lanes<V>::N;
  __shared__ int hit_row[COMBINE_CAP], hit_k[COMBINE_CAP];
  __shared__ int ord_row[COMBINE_CAP];
  __shared__ float ord_w[COMBINE_CAP];
  __shared__ float wts[COMBINE_WEIGHTS];
  __shared__ int nhit;
  const int tid = threadIdx.x;
  const int R = sum_counts(recv_counts, W);
  const int kw = min(K, COMBINE_WEIGHTS);

  const int items = T * chunks;
  for (int q = blockIdx.x; q < items; q += gridDim.x) {
    const int t = chunks == 1 ? q : q / chunks, c = q - t * chunks;
    const int base = c * (BLK * NV);
    V* __restrict__ orow = out + (size_t)t * row_vecs;

    // the token's weights travel to LDS while the scan's loads are in flight
    float wreg = 0.0f;
    if (tid < kw) wreg = weights[(size_t)t * K + tid];

    float acc[NV][N];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      V o{};
      if (accumulate) o = orow[min(base + j * BLK + tid, row_vecs - 1)];
#pragma unroll
      for (int e = 0; e < N; ++e) acc[j][e] = accumulate ? to_f32<DT>(get16(o, e)) : 0.0f;
    }

    if (tid == 0) nhit = 0;
    __syncthreads();
    for (int i = tid; i < R; i += SCAN_UNROLL * BLK) {
      int key[SCAN_UNROLL];
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u)
        key[u] = recv_meta[(size_t)min(i + u * BLK, R - 1) * META + 2];
#pragma unroll
      for (int u = 0; u < SCAN_UNROLL; ++u) {
        const int row = i + u * BLK;
        if (row < R && key[u] == t) {
          const int p = atomicAdd(&nhit, 1);
          if (p < COMBINE_CAP) {
            hit_row[p] = row;
            hit_k[p] = recv_meta[(size_t)row * META + 3];
          }
        }
      }
    }
    if (tid < kw) wts[tid] = wreg;
    __syncthreads();
    const int n = nhit;

    if (n <= COMBINE_CAP) {
      if (tid < n) {  // order the hits by arrival index
        const int me = hit_row[tid];
        int r = 0;
        for (int b = 0; b < n; ++b) r += hit_row[b] < me;
        const int k = hit_k[tid];
        const bool ok = (k >= 0) & (k < K);
        ord_row[r] = ok ? me : -1;
        ord_w[r] = !ok ? 0.0f : k < kw ? wts[k] : weights[(size_t)t * K + k];
      }
      __syncthreads();
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
              for (int e = 0; e < N; ++e)
                acc[j][e] = combine_step<DT>(acc[j][e], get16(v[u][j], e), w);
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
            for (int e = 0; e < N; ++e) acc[j][e] = combine_step<DT>(acc[j][e], get16(v, e), w);
          }
        }
      }
    }

#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int idx = base + j * BLK + tid;
      if (idx < row_vecs) {
        uint16_t h[N];
#pragma unroll
        for (int e = 0; e < N; ++e) h[e] = to_b16<DT>(acc[j][e]);
        orow[idx] = pack16<V>(h);
      }
    }
    __syncthreads();  // the LDS lists are reused by the next item
  }
}

// ---------------------------------------------------------------- simulated expert

template <typename V, int NV, int DIN, int DOUT>
__global__ __launch_bounds__(BLOCK) void expert_scale_kernel(
    const V* __restrict__ expert_x, const int* __restrict__ expert_num_tokens, int nle,
    int max_recv, float scale, int row_vecs, int chunks, V* __restrict__ expert_y) {
  __shared__ int red[NWAVES];
  __shared__ int pre[MAX_LOCAL_EXPERTS + 1];
  const int R = expert_prefix(expert_num_tokens, nle, max_recv, pre, red);
  const int top = top_step(nle);
  const int items = R * chunks;
  for (int q = blockIdx.x; q < items; q += gridDim.x) {
    const int g = chunks == 1 ? q : q / chunks, c = q - g * chunks;
    const int base = c * (BLOCK * NV);
    const int le = expert_of(pre, nle, top, g);
    const size_t row = (size_t)le * max_recv + (g - pre[le]);
    Payload<V, NV> p;
    p.load(expert_x + row * row_vecs, base, row_vecs);
    p.map([scale](V v) {
      constexpr int N = Lanes<V>::N;
      uint16_t h[N];
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const float f = to_f32<DOUT>(to_b16<DOUT>(to_f32<DIN>(get16(v, e))));
        h[e] = to_b16<DOUT>(__fmul_rn(f, scale));
      }
      return pack16<V>(h);
    });
    p.store(expert_y + row * row_vecs, base, row_vecs);
  }
}

// ---------------------------------------------------------------- exchange stand-in

template <typename V, int NV>
__global__ __launch_bounds__(BLOCK) void exchange_local_kernel(
    const V* __restrict__ send_buf, const int* __restrict__ send_meta,
    const int* __restrict__ send_counts, int dst_rank, V* __restrict__ recv_buf,
    int* __restrict__ recv_meta, const int* __restrict__ recv_counts, int src_rank, int row_vecs,
    int chunks) {
  const int tid = threadIdx.x;
  const int src_off = sum_counts(send_counts, dst_rank);
  const int dst_off = sum_counts(recv_counts, src_rank);
  const int n = min(max(send_counts[dst_rank], 0), max(recv_counts[src_rank], 0));
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
  int nv;         // vectors per lane of a row-move workgroup: 1, 2 or 4
  int chunks;     // workgroups per row = ceil(row_vecs / (BLOCK * nv))
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

}  // namespace

extern "C" {

const char* moe_a2a_version(void) { return "moe_a2a 0.2 gfx950"; }

const char* moe_a2a_strerror(int status) {
  switch (status) {
    case MOE_A2A_OK: return "ok";
    case MOE_A2A_EINVAL: return "invalid argument (null pointer, bad shape or unsupported size)";
    case MOE_A2A_EALIGN: return "row buffer is not aligned to its 2-byte elements";
    case MOE_A2A_ELAUNCH: return "kernel launch failed";
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
  if (!items_fit(S, g.chunks)) return MOE_A2A_EINVAL;
  const int grid = s->world_size + mover_blocks(S * g.chunks);
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(V, NV)                                                                          \
  dispatch_send_kernel<V, NV><<<grid, BLOCK, 0, st>>>(                                         \
      (const V*)x, indices, (int)S, s->experts_per_token, g.nle, s->num_experts, s->world_size, \
      g.magic, s->rank, g.row_vecs, g.chunks, (V*)send_buf, send_meta, send_counts, send_slot)
  MOE_A2A_FOR_ROW_KERNEL(g, LAUNCH);
#undef LAUNCH
  return launch_status();
}

int moe_a2a_dispatch_recv(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                          const int32_t* recv_counts, int32_t rows_hint,
                          int32_t* expert_num_tokens, void* expert_x, int32_t* expert_meta,
                          void* stream) {
  if (!shape_ok(s) || rows_hint < 0 || !recv_counts || !expert_num_tokens || !expert_x ||
      !expert_meta)
    return MOE_A2A_EINVAL;
  if (rows_hint > 0 && (!recv_buf || !recv_meta)) return MOE_A2A_EINVAL;
  if (!all_aligned(2, recv_buf, expert_x)) return MOE_A2A_EALIGN;
  const Geometry g = geometry(s, recv_buf, expert_x);
  // the stream can hold at most nle * max_recv rows that fit the expert buffers
  if (!items_fit((long long)g.nle * g.max_recv, g.chunks)) return MOE_A2A_EINVAL;
  const int grid = g.nle + mover_blocks((long long)rows_hint * g.chunks);
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(V, NV)                                                                       \
  dispatch_recv_kernel<V, NV><<<grid, BLOCK, 0, st>>>(                                      \
      (const V*)recv_buf, recv_meta, recv_counts, s->world_size, g.nle, g.magic, g.max_recv, \
      g.row_vecs, g.chunks, expert_num_tokens, (V*)expert_x, expert_meta)
  MOE_A2A_FOR_ROW_KERNEL(g, LAUNCH);
#undef LAUNCH
  return launch_status();
}

int moe_a2a_combine_send(const moe_a2a_shape* s, const void* expert_y, const int32_t* expert_meta,
                         const int32_t* expert_num_tokens, int32_t rows_hint, void* send_buf,
                         int32_t* send_meta, int32_t* send_counts, void* stream) {
  if (!shape_ok(s) || rows_hint < 0 || !expert_y || !expert_meta || !expert_num_tokens ||
      !send_counts)
    return MOE_A2A_EINVAL;
  if (rows_hint > 0 && (!send_buf || !send_meta)) return MOE_A2A_EINVAL;
  if (!all_aligned(2, expert_y, send_buf)) return MOE_A2A_EALIGN;
  const Geometry g = geometry(s, expert_y, send_buf);
  if (g.nle > MAX_LOCAL_EXPERTS) return MOE_A2A_EINVAL;
  if (!items_fit((long long)g.nle * g.max_recv, g.chunks)) return MOE_A2A_EINVAL;
  const int grid = s->world_size + mover_blocks((long long)rows_hint * g.chunks);
  hipStream_t st = (hipStream_t)stream;
#define LAUNCH(V, NV)                                                                         \
  combine_send_kernel<V, NV><<<grid, BLOCK, 0, st>>>(                                         \
      (const V*)expert_y, expert_meta, expert_num_tokens, g.nle, g.max_recv, s->world_size,    \
      g.row_vecs, g.chunks, (V*)send_buf, send_meta, send_counts)
  MOE_A2A_FOR_ROW_KERNEL(g, LAUNCH);
#undef LAUNCH
  return launch_status();
}

int moe_a2a_combine_recv(const moe_a2a_shape* s, const void* recv_buf, const int32_t* recv_meta,
                         const int32_t* recv_counts, const float* weights, int32_t num_tokens,
                         void* out_tokens, int32_t accumulate, int32_t dtype, void* stream) {
  if (!shape_ok(s) || num_tokens < 0 || num_tokens > s->max_num_tokens || !recv_counts)
    return MOE_A2A_EINVAL;
  if (dtype != MOE_A2A_F16 && dtype != MOE_A2A_BF16) return MOE_A2A_EINVAL;
  if (num_tokens == 0) return MOE_A2A_OK;
  if (!recv_buf || !recv_meta || !weights || !out_tokens) return MOE_A2A_EINVAL;
  if (!all_aligned(2, recv_buf, out_tokens)) return MOE_A2A_EALIGN;
  const Geometry g = geometry(s, recv_buf, out_tokens);
  // wide rows: one 1024-lane workgroup per token scans the arrivals once; narrower rows use
  // 256 lanes with one or two vector columns each
  const int blk = g.row_vecs >= 768 ? 1024 : BLOCK;
  const int nv = blk == 1024 ? 1 : g.row_vecs <= BLOCK ? 1 : 2;
  const int chunks = (g.row_vecs + blk * nv - 1) / (blk * nv);
  if (!items_fit(num_tokens, chunks)) return MOE_A2A_EINVAL;
  const int grid = mover_blocks((long long)num_tokens * chunks);
  hipStream_t st = (hipStream_t)stream;
  const int K = s->experts_per_token, W = s->world_size;
#define LAUNCH(V, DT, BLK, NV)                                                               \
  combine_recv_kernel<V, DT, BLK, NV><<<grid, BLK, 0, st>>>(                                 \
      (const V*)recv_buf, recv_meta, recv_counts, W, weights, num_tokens, K, g.row_vecs,     \
      chunks, (V*)out_tokens, accumulate)
#define PICK_SHAPE(V, DT)                                  \
  do {                                                     \
    if (blk == 1024) { LAUNCH(V, DT, 1024, 1); }           \
    else if (nv == 1) { LAUNCH(V, DT, BLOCK, 1); }         \
    else { LAUNCH(V, DT, BLOCK, 2); }                      \
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

int moe_a2a_expert_scale(const moe_a2a_shape* s, const void* expert_x,
                         const int32_t* expert_num_tokens, int32_t rows_hint, int32_t in_dtype,
                         int32_t out_dtype, void* expert_y, void* stream) {
  if (!shape_ok(s) || rows_hint < 0 || !expert_x || !expert_num_tokens || !expert_y)
    return MOE_A2A_EINVAL;
  if ((in_dtype != MOE_A2A_F16 && in_dtype != MOE_A2A_BF16) ||
      (out_dtype != MOE_A2A_F16 && out_dtype != MOE_A2A_BF16))
    return MOE_A2A_EINVAL;
  if (!all_aligned(2, expert_x, expert_y)) return MOE_A2A_EALIGN;
  const Geometry g = geometry(s, expert_x, expert_y);
  if (g.nle > MAX_LOCAL_EXPERTS) return MOE_A2A_EINVAL;
  if (!items_fit((long long)g.nle * g.max_recv, g.chunks)) return MOE_A2A_EINVAL;
  const int grid = mover_blocks((long long)rows_hint * g.chunks);
  hipStream_t st = (hipStream_t)stream;
  const float scale = (float)(1 + s->rank);
#define LAUNCH_T(V, NV, DI, DO)                                                              \
  expert_scale_kernel<V, NV, DI, DO><<<grid, BLOCK, 0, st>>>(                                \
      (const V*)expert_x, expert_num_tokens, g.nle, g.max_recv, scale, g.row_vecs, g.chunks, \
      (V*)expert_y)
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

int moe_a2a_exchange_local(int32_t world_size, int32_t hidden_dim, const void* send_buf,
                           const int32_t* send_meta, const int32_t* send_counts, int32_t dst_rank,
                           void* recv_buf, int32_t* recv_meta, const int32_t* recv_counts,
                           int32_t src_rank, int32_t rows_hint, void* stream) {
  if (world_size < 1 || hidden_dim < 1 || dst_rank < 0 || dst_rank >= world_size ||
      src_rank < 0 || src_rank >= world_size || rows_hint < 0 || !send_counts || !recv_counts)
    return MOE_A2A_EINVAL;
  if (rows_hint == 0) return MOE_A2A_OK;
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
      recv_counts, src_rank, g.row_vecs, g.chunks)
  MOE_A2A_FOR_ROW_KERNEL(g, LAUNCH);
#undef LAUNCH
  return launch_status();
}

}  // extern "C"
