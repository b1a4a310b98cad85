// K3: per-row top-k select with the "equal scores -> lower index first" rule,
// fused with the [sink | window | heavy] index-list assembly of
// GPT-FAST/kernels/sparse.py:57-95.
//
// Scores are mapped to order-preserving 32-bit keys and paired with the
// complemented index into 64-bit composites (key << 32 | ~index), so "larger
// composite" is exactly "higher score, then lower index" and all composites of a
// row are distinct.
//
// select_list_kernel, workgroups of 1024 lanes, selects in two ways:
//  * pooled: a superset of the row's m winners, at most kPoolCap composites, is
//    formed and the m-th largest located in it by range refinement -- a 2048-bin
//    LDS histogram over [lo, hi] (initially the pool's min / max, so the bins
//    spread over the values that occur and LDS atomics rarely collide), then the
//    bin holding the m-th becomes the new range, until it holds at most kCandCap
//    entries.  Because the composites are distinct, ties need no special case.
//    The pool is the whole row when that fits; otherwise everything at or above a
//    threshold estimated from a fixed sample of the row and aimed at about 2m
//    entries, found in one streaming pass over the row (compacted in LDS, then
//    held in registers).  Where CUs are to spare several workgroups share a row:
//    each streams its share against the same threshold and appends what passes
//    to the row's list in memory, and the last to arrive selects from that list,
//    in the same launch.  A pool that comes out shorter than m or longer than
//    kPoolCap (the sample misjudged the row, or one key value is massively
//    repeated) is dropped and the row redone from scratch: the result is always
//    exact, only the time differs.
//  * from scratch: the same refinement over the row itself, one pass per level
//    (the row stays in L2), until the m-th key's bin holds at most kCandCap keys;
//    one more pass collects the keys above the bin and the bin's own.  A single
//    key value with more than kCandCap copies (mass ties) is resolved by a
//    histogram over index ranges (lowest indices win).  The scorer can hand over
//    the row's key range, which saves the first pass.
// Either way the winners are put in order without a full sort: their level-0
// histogram bins already order them coarsely and a bin seldom holds more than a
// few, so each winner goes to (#winners in higher bins) + (#bin-mates beating
// it); crowded bins fall back to an in-LDS bitonic sort whose short exchange
// distances stay in registers and wave shuffles.  In the pooled path the first
// refinement pass is that level-0 histogram: every entry keeps the slot its
// bin's counter handed it, the scan that finds the m-th bin turns the counters
// into offsets, and when that one pass isolates the bin (the usual case) the
// winners are grouped by bin with no second count.
#include "socket_common.h"


namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / SOCKET_WAVE;
constexpr int kBins = 2048;
constexpr int kCandCap = 2048;           // entries of the k-th bin kept in LDS
constexpr int kMaxBinForCounting = 128;  // larger bins are sorted, not rank-counted

constexpr int kBatch = kThreads * 16;  // scores a workgroup filters per batch (16 per lane)
constexpr int kPoolCap = 8192;         // composites pooled per row
constexpr int kMaxParts = 16;          // workgroups that share one row at most

typedef unsigned long long u64;

template <bool B>
struct BoolTag {
  static constexpr bool value = B;
};

struct SelectShared {
  u64 lo, hi;           // current key / composite range (inclusive)
  int need;             // winners still to take from inside [lo, hi]
  int bin_count;        // entries in the bin holding the k-th
  int done;
  int fill_above, fill_cand, fill_pool;
  int idx_star;         // mass ties: largest index taken among the ties
  int found_bin, found_before, found_count;
  u64 wmin[kWaves], wmax[kWaves];
  int wsum[kWaves];
  int wflag[kWaves];
  uint32_t kmin, kmax;  // key range of the pool
  int base;             // where this workgroup's entries go in the row's shared list
  int last;             // this workgroup is the last of its row to arrive
  int crowded;          // a bin above the k-th holds more than kMaxBinForCounting entries
};

__device__ __forceinline__ u64 composite(uint32_t key, int idx) {
  return ((u64)key << 32) | (u64)(0xffffffffu - (uint32_t)idx);
}
__device__ __forceinline__ int32_t composite_index(u64 c) {
  return (int32_t)(0xffffffffu - (uint32_t)(c & 0xffffffffull));
}

// Minimum and maximum over the 64 lanes, left in lane 63 (the same six steps as
// the prefix sum; lanes a step does not reach take the identity).
__device__ __forceinline__ void wave_minmax_to_last(uint32_t& kmin, uint32_t& kmax) {
#define SOCKET_MINMAX_STEP(ctrl, rows)                                                                        \
  kmin = min(kmin, (uint32_t)__builtin_amdgcn_update_dpp((int)0xffffffffu, (int)kmin, ctrl, rows, 0xf, false)); \
  kmax = max(kmax, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)kmax, ctrl, rows, 0xf, false));
  SOCKET_MINMAX_STEP(0x111, 0xf)   // row_shr:1
  SOCKET_MINMAX_STEP(0x112, 0xf)   // row_shr:2
  SOCKET_MINMAX_STEP(0x114, 0xf)   // row_shr:4
  SOCKET_MINMAX_STEP(0x118, 0xf)   // row_shr:8
  SOCKET_MINMAX_STEP(0x142, 0xa)   // row_bcast:15 into rows 1 and 3
  SOCKET_MINMAX_STEP(0x143, 0xc)   // row_bcast:31 into rows 2 and 3
#undef SOCKET_MINMAX_STEP
}

__device__ __forceinline__ u64 shfl_xor_u64(u64 v, int mask) {
  const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, mask, SOCKET_WAVE);
  const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), mask, SOCKET_WAVE);
  return ((u64)hi << 32) | lo;
}

// All THREADS lanes.  Ranks the bins from the top (descending != 0) or from the
// bottom, kBins / THREADS per lane, and publishes in `sh` the bin where the
// running count first reaches `need`, the count ranked before it and its own.
// With OFFSETS every bin's counter is replaced by `entries ranked before the bin |
// its own count << 16` (each lane rewrites the bins it read, nobody else's), and
// sh.crowded is raised (never cleared here) when a bin ranked wholly before the
// found one holds more than kMaxBinForCounting entries.
// `on_found(bin, ranked before it, its count)` runs in the one lane that finds the
// bin, before the closing barrier: what it writes to `sh` every lane sees afterwards.
struct NoFoundAction {
  __device__ void operator()(int, int, int) const {}
};
template <int THREADS, bool OFFSETS = false, class F = NoFoundAction>
__device__ __forceinline__ void find_bin(uint32_t* hist, int need, int descending, SelectShared& sh,
                                         int tid, F&& on_found = F()) {
  constexpr int PER = kBins / THREADS;
  const int lane = tid & 63, wave = tid >> 6;
  int c[PER], mine = 0;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int r = tid * PER + i;
    c[i] = (int)hist[descending ? (kBins - 1 - r) : r];
    mine += c[i];
  }
  const int incl_w = wave_incl_scan(mine, lane);
  if (lane == 63) sh.wsum[wave] = incl_w;
  __syncthreads();
  int run = incl_w - mine;
#pragma unroll
  for (int w = 0; w < THREADS / SOCKET_WAVE; ++w) {   // (all entries read at once, the later waves' discarded)
    const int v = sh.wsum[w];
    run += (w < wave) ? v : 0;
  }
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    if (run < need && need <= run + c[i]) {
      const int r = tid * PER + i;
      sh.found_bin = descending ? (kBins - 1 - r) : r;
      sh.found_before = run;
      sh.found_count = c[i];
      on_found(descending ? (kBins - 1 - r) : r, run, c[i]);
    }
    if constexpr (OFFSETS) {
      const int r = tid * PER + i;
      hist[descending ? (kBins - 1 - r) : r] = (uint32_t)run | ((uint32_t)c[i] << 16);
      if (c[i] > kMaxBinForCounting && run + c[i] < need) sh.crowded = 1;
    }
    run += c[i];
  }
  __syncthreads();
}

// Visit row[begin:n) once, 16 bytes per lane per load and eight loads in flight
// per lane (a lone workgroup per row has to cover the memory latency itself).
template <bool VEC, int THREADS, class F>
__device__ __forceinline__ void for_each_in(const float* row, int begin, int n, int tid, F&& f) {
  constexpr int U = 8;
  if (VEC) {  // begin is a multiple of 4
    const int n4 = n & ~3;
    constexpr int kStride = THREADS * 4;
    int i = begin + tid * 4;
    for (; i + (U - 1) * kStride < n4; i += U * kStride) {
      float4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = *reinterpret_cast<const float4*>(row + i + u * kStride);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        f(i + u * kStride, x[u].x);
        f(i + u * kStride + 1, x[u].y);
        f(i + u * kStride + 2, x[u].z);
        f(i + u * kStride + 3, x[u].w);
      }
    }
    for (; i < n4; i += kStride) {
      const float4 x = *reinterpret_cast<const float4*>(row + i);
      f(i, x.x);
      f(i + 1, x.y);
      f(i + 2, x.z);
      f(i + 3, x.w);
    }
    for (int t = max(n4, begin) + tid; t < n; t += THREADS) f(t, row[t]);
  } else {
    int i = begin + tid;
    for (; i + (U - 1) * THREADS < n; i += U * THREADS) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = row[i + u * THREADS];
#pragma unroll
      for (int u = 0; u < U; ++u) f(i + u * THREADS, x[u]);
    }
    for (; i < n; i += THREADS) f(i, row[i]);
  }
}

// Append `value` to a list if `take`: one LDS atomic per wave, positions handed
// out by a ballot prefix count.  Safe under divergence (only active lanes vote).
__device__ __forceinline__ void wave_append(bool take, u64 value, int* cursor, u64* list, int cap) {
  const u64 mask = __ballot(take);
  if (mask == 0) return;
  const int lane = threadIdx.x & 63;
  const int leader = __ffsll((long long)mask) - 1;
  int base = 0;
  if (lane == leader) base = atomicAdd(cursor, __popcll(mask));
  base = __builtin_amdgcn_readlane(base, leader);   // (leader is wave-uniform: a scalar read, no LDS crossbar)
  if (take) {
    const int p = base + __popcll(mask & ((1ull << lane) - 1ull));
    if (p < cap) list[p] = value;
  }
}

// Bitonic sort of buf[0:np] (np a power of two) into descending order by the
// whole 1024-lane workgroup.  Lane t owns elements [t*E, (t+1)*E): exchange
// distances below E stay in registers, below 64*E go through wave shuffles, and
// only the longer ones through LDS with a barrier.  Callers sync before and get
// a synced buffer back.
template <int E>
__device__ __forceinline__ void sort_desc_impl(u64* buf, int np, int tid) {
  const bool active = tid * E < np;
  u64 r[E];
  auto load = [&]() {
#pragma unroll
    for (int e = 0; e < E; ++e) r[e] = active ? buf[tid * E + e] : 0ull;
  };
  auto store = [&]() {
    if (active) {
#pragma unroll
      for (int e = 0; e < E; ++e) buf[tid * E + e] = r[e];
    }
  };
  auto reg_stages = [&](int k, int jstart) {
    for (int j = jstart; j >= E; j >>= 1) {  // partner in another lane of the wave
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const int i = tid * E + e;
        const u64 other = shfl_xor_u64(r[e], j / E);
        const bool lower = (i & j) == 0, desc = (i & k) == 0;
        const u64 mx = r[e] > other ? r[e] : other;
        const u64 mn = r[e] > other ? other : r[e];
        r[e] = (lower == desc) ? mx : mn;
      }
    }
#pragma unroll
    for (int j = E / 2; j >= 1; j >>= 1) {  // partner in this lane
      if (j > jstart) continue;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        if (e & j) continue;
        const int p = e | j;
        const bool desc = ((tid * E + e) & k) == 0;
        const u64 a = r[e], c = r[p];
        const u64 mx = a > c ? a : c, mn = a > c ? c : a;
        r[e] = desc ? mx : mn;
        r[p] = desc ? mn : mx;
      }
    }
  };
  const int span = 64 * E;  // distances below this never leave the wave
  load();
  for (int k = 2; k <= np && k <= span; k <<= 1) reg_stages(k, k >> 1);
  store();
  __syncthreads();
  for (int k = 2 * span; k <= np; k <<= 1) {
    for (int j = k >> 1; j >= span; j >>= 1) {
      for (int i = tid; i < np; i += kThreads) {
        const int p = i ^ j;
        if (p > i) {
          const u64 a = buf[i], c = buf[p];
          const bool desc = (i & k) == 0;
          if (desc ? (a < c) : (a > c)) {
            buf[i] = c;
            buf[p] = a;
          }
        }
      }
      __syncthreads();
    }
    load();
    reg_stages(k, span >> 1);
    store();
    __syncthreads();
  }
}

__device__ __forceinline__ void sort_desc(u64* buf, int np, int tid) {
  if (np <= kThreads) sort_desc_impl<1>(buf, np, tid);
  else if (np == 2 * kThreads) sort_desc_impl<2>(buf, np, tid);
  else if (np == 4 * kThreads) sort_desc_impl<4>(buf, np, tid);
  else if (np == 8 * kThreads) sort_desc_impl<8>(buf, np, tid);
  else sort_desc_impl<16>(buf, np, tid);
}

__device__ __forceinline__ int next_pow2_dev(int x) {
  return x <= 1 ? 1 : 1 << (32 - __clz(x - 1));
}

// Row length n and heavy budget m of a row of sequence b (m clipped to the room
// the list row leaves after the sink / window part), and that part's length.
__device__ __forceinline__ void row_shape(const int32_t* lens, const int32_t* budgets, int b, int T,
                                          int M, int sink, int window, int write_base, int list_width,
                                          int& n, int& m, int& nbase) {
  n = lens ? max(0, min(lens[b], T)) : T;
  m = budgets ? budgets[b] : M;
  m = max(0, min(min(m, M), n));
  nbase = 0;
  if (write_base) {
    const int s_e = max(0, min(sink, n));
    const int w_e = max(0, min(window, n));
    const int win_start = max(n - w_e, s_e);
    nbase = s_e + ((w_e > 0 && win_start < n) ? n - win_start : 0);
    if (nbase == 0) nbase = 1;
  }
  m = max(0, min(nbase + m, list_width) - nbase);
}

// Sink / window part of a list row, its length and the -1 padding.
__device__ __forceinline__ void write_list_base(int32_t* out, int n, int m, int nbase, int sink,
                                                int window, int write_base, int list_width,
                                                int32_t* len_out, int tid, int nthreads) {
  if (write_base) {
    const int s_e = max(0, min(sink, n));
    const int w_e = max(0, min(window, n));
    const int win_start = max(n - w_e, s_e);
    if (s_e + ((w_e > 0 && win_start < n) ? n - win_start : 0) == 0) {
      if (tid == 0 && list_width > 0) out[0] = n - 1;
    } else {
      for (int i = tid; i < nbase && i < list_width; i += nthreads)
        out[i] = i < s_e ? i : win_start + (i - s_e);
    }
  }
  const int total = min(nbase + m, list_width);
  for (int i = total + tid; i < list_width; i += nthreads) out[i] = -1;
  if (len_out && tid == 0) *len_out = total;
}

// Smallest shift for which [lo, hi] maps onto at most kBins bins.
// (In closed form: span >> shift < kBins = 2^11 as soon as shift >= bits(span) - 11.
// Counting the shift up in a loop cost 40-odd trips of 64-bit shifts per call for
// composites, on every wave: 1.5-2 us a call with four waves to a SIMD.)
__device__ __forceinline__ int range_shift(u64 lo, u64 hi) {
  static_assert(kBins == 2048, "range_shift assumes 2^11 bins");
  const u64 span = hi - lo;
  const int bits = span ? 64 - __clzll((long long)span) : 0;
  return bits > 11 ? bits - 11 : 0;
}

// Final step of both paths.  buf[0:n_above) holds the winners above the k-th
// bin, cand[0:ncand) the k-th bin's entries of which the best `need` win; the
// n_above + need winners are written in descending order at out[0:...).
// Winners are placed by their level-0 bin (c - lo0) >> shift0 with counting ranks
// when `counting_ok` (tmp then has 2 * cap_above slots) and no bin is crowded,
// else by the bitonic sort.  All 1024 lanes; callers sync before; no barrier at
// the end.
__device__ __forceinline__ void order_and_write(u64* buf, int n_above, u64* cand, int ncand, int need,
                                                u64 lo0, int shift0, u64* tmp, uint32_t* hist,
                                                SelectShared& sh, bool counting_ok, int32_t* out,
                                                int tid, bool placed = false) {
  const int lane = tid & 63, wave = tid >> 6;
  // ---- the k-th bin: rank its entries, the best `need` follow the winners ----------
  if (ncand <= kMaxBinForCounting || need == ncand) {
    for (int i = tid; i < ncand; i += kThreads) {
      const u64 v = cand[i];
      int r = 0;
      for (int j = 0; j < ncand; ++j) r += cand[j] > v;
      if (r < need) out[n_above + r] = composite_index(v);
    }
  } else {
    const int npc = next_pow2_dev(ncand);
    for (int i = ncand + tid; i < npc; i += kThreads) cand[i] = 0ull;
    __syncthreads();
    sort_desc(cand, npc, tid);
    for (int i = tid; i < need; i += kThreads) out[n_above + i] = composite_index(cand[i]);
  }
  if (n_above == 0) return;

  // ---- winners above the bin ----------------------------------------------------------
  if (placed) {
    // `buf` holds them grouped by level-0 bin already, hist[bin] = offset | population << 16
    for (int p = tid; p < n_above; p += kThreads) {
      const u64 v = buf[p];
      const uint32_t h = hist[(int)((v - lo0) >> shift0)];
      const int s0 = (int)(h & 0xffffu), c = (int)(h >> 16);
      int r = 0;
      for (int q = s0; q < s0 + c; ++q) r += buf[q] > v;
      out[s0 + r] = composite_index(v);
    }
    return;
  }
  if (counting_ok) {
    for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
    __syncthreads();
    for (int i = tid; i < n_above; i += kThreads) {
      const int bin = (int)((buf[i] - lo0) >> shift0);
      const uint32_t slot = atomicAdd(&hist[bin], 1u);
      tmp[i] = ((u64)bin << 32) | slot;  // parked until the offsets are known
    }
    __syncthreads();
    // descending exclusive scan over the bins, two per lane; crowded-bin check
    const int b0 = kBins - 1 - 2 * tid, b1 = b0 - 1;
    const int c0 = (int)hist[b0], c1 = (int)hist[b1];
    const int incl_w = wave_incl_scan(c0 + c1, lane);
    const int crowded = __any((c0 > kMaxBinForCounting || c1 > kMaxBinForCounting) ? 1 : 0);
    if (lane == 63) sh.wsum[wave] = incl_w;
    if (lane == 0) sh.wflag[wave] = crowded;
    __syncthreads();
    int base = 0, any_crowded = 0;
    for (int w = 0; w < kWaves; ++w) {
      if (w < wave) base += sh.wsum[w];
      any_crowded |= sh.wflag[w];
    }
    const int excl = base + incl_w - (c0 + c1);
    __syncthreads();
    if (!any_crowded) {
      hist[b0] = (uint32_t)excl | ((uint32_t)c0 << 16);  // offset | population << 16
      hist[b1] = (uint32_t)(excl + c0) | ((uint32_t)c1 << 16);
      __syncthreads();
      u64* grouped = tmp + n_above;
      for (int i = tid; i < n_above; i += kThreads) {
        const int bin = (int)(tmp[i] >> 32);
        const int slot = (int)(tmp[i] & 0xffffffffull);
        grouped[(hist[bin] & 0xffffu) + slot] = buf[i];
      }
      __syncthreads();
      for (int p = tid; p < n_above; p += kThreads) {
        const u64 v = grouped[p];
        const uint32_t h = hist[(int)((v - lo0) >> shift0)];
        const int s0 = (int)(h & 0xffffu), c = (int)(h >> 16);
        int r = 0;
        for (int q = s0; q < s0 + c; ++q) r += grouped[q] > v;
        out[s0 + r] = composite_index(v);
      }
      return;
    }
  }
  const int np = next_pow2_dev(n_above);
  for (int i = n_above + tid; i < np; i += kThreads) buf[i] = 0ull;
  __syncthreads();
  sort_desc(buf, np, tid);
  for (int j = tid; j < n_above; j += kThreads) out[j] = composite_index(buf[j]);
}

// ---------------------------------------------------------------------------
// threshold from a sample
// ---------------------------------------------------------------------------
// A pool of kPoolCap composites can be relied on to hold a row's m winners when
// it is filled with everything above a threshold aimed at max(2m, 1024) entries.
__host__ __device__ __forceinline__ bool sampling_ok(int m) {
  const int target = 2 * m > 1024 ? 2 * m : 1024;
  return target + target / 2 <= kPoolCap;
}

// All THREADS lanes; returns (to every lane) a key tau such that about
// max(2m, 1024) of the row's n scores have keys >= tau.  The estimate comes from
// a fixed sample of the row -- runs of 64 consecutive scores at evenly spaced
// places, 4096 scores in all (16384 for rows beyond 262144) -- whose r-th largest
// key is located with the same histogram refinement as everywhere else; tau is
// the lower edge of its bin.  Every workgroup that calls this for a row gets the
// same tau.  Needs n > kPoolCap; clears hist itself (nobody may be using it).  When
// it returns every lane has passed the barrier that follows the last read of hist.
template <int THREADS, bool VEC>
__device__ __forceinline__ uint32_t sample_threshold(const float* row, int n, int m, uint32_t* hist,
                                                     SelectShared& sh, int tid) {
  constexpr int kMaxQ = 16384 / 4 / THREADS;  // float4 groups per lane at most
  const int lane = tid & 63, wave = tid >> 6;
  const int nsample = n <= 262144 ? 4096 : 16384;
  const int nchunk = nsample / 64;
  const int nq = nsample / 4 / THREADS;  // 1 or 4 (1024 lanes), 4 or 16 (256 lanes)
  uint32_t key[kMaxQ * 4];
  for (int i = tid; i < kBins; i += THREADS) hist[i] = 0;   // (no one uses hist before this call)
#pragma unroll
  for (int j = 0; j < kMaxQ; ++j) {
    if (j < nq) {
      const int q = j * THREADS + tid;
      const int chunk = q >> 4;
      const int at = (int)(((int64_t)chunk * n / nchunk) & ~3ll) + (q & 15) * 4;
      float x[4];
      if (VEC) {
        const float4 v = *reinterpret_cast<const float4*>(row + at);
        x[0] = v.x;
        x[1] = v.y;
        x[2] = v.z;
        x[3] = v.w;
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) x[c] = row[at + c];
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) key[j * 4 + c] = score_to_key(x[c]);
    }
  }
  uint32_t kmin = 0xffffffffu, kmax = 0u;
#pragma unroll
  for (int j = 0; j < kMaxQ; ++j) {
    if (j < nq) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        kmin = min(kmin, key[j * 4 + c]);
        kmax = max(kmax, key[j * 4 + c]);
      }
    }
  }
  wave_minmax_to_last(kmin, kmax);
  if (lane == 63) {
    sh.wmin[wave] = kmin;
    sh.wmax[wave] = kmax;
  }
  __syncthreads();   // (also: hist is zero everywhere)
  // every wave reduces the waves' extremes for itself
  kmin = (uint32_t)sh.wmin[lane & (THREADS / SOCKET_WAVE - 1)];
  kmax = (uint32_t)sh.wmax[lane & (THREADS / SOCKET_WAVE - 1)];
  wave_minmax_to_last(kmin, kmax);
  const uint32_t smin = (uint32_t)__builtin_amdgcn_readlane((int)kmin, 63);
  const uint32_t smax = max(smin, (uint32_t)__builtin_amdgcn_readlane((int)kmax, 63));
  const int target = max(2 * m, 1024);
  const int r = (int)min((int64_t)nsample, ((int64_t)target * nsample + n - 1) / n);
  const int fine = max(4, r / 8);  // a bin this small pins tau well enough
  for (int iter = 0; iter < 4; ++iter) {
    // the first pass takes its range from the sample's extremes, the later ones from
    // what the pass before published
    const uint32_t lo = iter ? (uint32_t)sh.lo : smin, hi = iter ? (uint32_t)sh.hi : smax;
    const int need_in = iter ? sh.need : r;
    const int shift = range_shift(lo, hi);
    if (iter) {
      for (int i = tid; i < kBins; i += THREADS) hist[i] = 0;
      __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < kMaxQ; ++j) {
      if (j < nq) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint32_t k = key[j * 4 + c];
          if (k >= lo && k <= hi) atomicAdd(&hist[(k - lo) >> shift], 1u);
        }
      }
    }
    __syncthreads();
    find_bin<THREADS>(hist, need_in, 1, sh, tid, [&](int bin, int before, int count) {
      const uint32_t blo = lo + ((uint32_t)bin << shift);
      const uint32_t bspan = (shift == 0) ? 0u : ((1u << shift) - 1u);
      sh.lo = blo;
      sh.hi = (hi - blo < bspan) ? hi : blo + bspan;
      sh.need = need_in - before;
      sh.done = (count <= fine || shift == 0) ? 1 : 0;
    });
    if (sh.done) break;
  }
  return (uint32_t)sh.lo;
}

// ---------------------------------------------------------------------------
// rows
// ---------------------------------------------------------------------------
// Agent-wide coherent accesses without a fence (written through / read past this
// die's caches): what workgroups of one row on different dies exchange.
__device__ __forceinline__ void store_coherent(u64* p, u64 v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 load_coherent(const u64* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// `parts` workgroups per row (blockIdx.x = row * parts + part).  With parts > 1
// each filters its share of the row against the same sampled threshold (every
// part works it out for itself from the same sample), appends what passes to the
// row's list in `loc` (a stretch reserved with one atomic add on row_count), and
// the last part to arrive (row_done) selects from that list; the others leave.
// row_count and row_done are zero on entry and zero again on exit.
// The pooled composites are held in registers, eight per lane, from the moment
// the pool is complete; LDS holds them only while they are being compacted.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void select_list_kernel(
    const float* __restrict__ scores, int64_t score_stride, const int32_t* __restrict__ lens,
    const int32_t* __restrict__ budgets, const uint32_t* __restrict__ row_range, int range_parts,
    int Hq, int T, int M, int sink, int window, int write_base, int32_t* __restrict__ sparse_list,
    int64_t list_stride, int list_width, int32_t* __restrict__ sparse_len, int cap_above,
    int counting_ok, int use_pool, int pool_slots, int parts, u64* __restrict__ loc,
    int32_t* __restrict__ row_count, unsigned int* __restrict__ row_done) {
  __shared__ uint32_t hist[kBins];
  __shared__ SelectShared sh;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  u64* buf = reinterpret_cast<u64*>(lds_raw);  // winners                  [cap_above]
  u64* cand = buf + cap_above;                 // entries of the k-th bin  [kCandCap]
  u64* pool = cand + kCandCap;                 // what passes the filter   [pool_slots]: kPoolCap for rows beyond that
  u64* tmp = pool + pool_slots;                // counting placement       [2*cap_above] if counting_ok

  const int rowi = blockIdx.x / parts, part = blockIdx.x % parts;
  const int b = rowi / Hq;
  const int tid = threadIdx.x;
  const int lane = tid & (SOCKET_WAVE - 1);
  const int wave = tid / SOCKET_WAVE;
  int n, m, nbase;
  row_shape(lens, budgets, b, T, M, sink, window, write_base, list_width, n, m, nbase);
  const float* row = scores + (int64_t)rowi * score_stride;
  int32_t* out = sparse_list + (int64_t)rowi * list_stride;
  if (part == 0)
    write_list_base(out, n, m, nbase, sink, window, write_base, list_width,
                    sparse_len ? sparse_len + rowi : nullptr, tid, kThreads);
  if (m == 0) return;
  int32_t* heavy = out + nbase;

  // ================================ pooled select ======================================
  if (use_pool) {
    if (tid == 0) {
      sh.fill_above = 0;
      sh.fill_cand = 0;
      sh.fill_pool = 0;
      sh.kmin = 0xffffffffu;
      sh.kmax = 0u;
      sh.crowded = 0;
    }
    int total = -1;  // uniform; stays -1 when no pool could be formed
    uint32_t kmin = 0xffffffffu, kmax = 0u;  // key range of what this lane holds
    constexpr int U = kPoolCap / kThreads;
    u64 pv[U];                               // entry tid + u * kThreads of the pool
    if (n <= kPoolCap) {  // the whole row, by one workgroup
      if (part != 0) return;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = tid + u * kThreads;
        const uint32_t k = score_to_key(i < n ? row[i] : 0.f);
        if (i < n) {
          kmin = min(kmin, k);
          kmax = max(kmax, k);
        }
        pv[u] = composite(k, i);
      }
      total = n;
      for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;   // for the first refinement pass
      __syncthreads();
    } else if (sampling_ok(m)) {
      // This part's share of the row; the last part also takes the one to three
      // scores past the last multiple of four.
      const int n4 = n & ~3;
      const int chunk = (((n + parts - 1) / parts) + 3) & ~3;
      const int begin = min(part * chunk, n4), e4 = min(begin + chunk, n4);
      const int tail_end = (part == parts - 1) ? n : e4;
      if (VEC) {
        // In batches of 16 scores per lane (four 16-byte loads, all in flight
        // together); the first two batches are requested before the threshold is
        // worked out, each further one two batches ahead of the one being filtered.  A
        // wave counts what passes in its batch, reserves a stretch of the pool with
        // one LDS atomic and writes its entries there: no barrier in the loop.
        constexpr int kLoads = 4, kStep = kThreads * 4 * kLoads;
        static_assert(kStep == kBatch, "batch size");
        auto fetch = [&](int base, float4 (&x)[kLoads]) {
#pragma unroll
          for (int u = 0; u < kLoads; ++u) {
            // (past the end: the share's last four, fetched and ignored -- a load under
            // a condition would make every wait in the loop a wait for all loads)
            const int i0 = max(min(base + (u * kThreads + tid) * 4, e4 - 4), 0);
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(row + i0));
            x[u] = make_float4(v.x, v.y, v.z, v.w);
          }
        };
        // One batch of one wave.  Each of a lane's 16 scores is tested on the float (one
        // compare per score; keys only for the pool): x passes when it is not below the
        // float whose key is tau.  A tau above +inf's key or below -inf's is no float's
        // key and is widened to that infinity (the pool only has to hold everything at
        // or above tau; more is allowed).  A compare leaves a wave-wide mask in scalar
        // registers; the 16 masks' population is the stretch of the pool that one LDS
        // atomic reserves for the wave, and an entry's place in it is the count of its
        // mask's bits below its lane, on top of a scalar running base -- no per-lane
        // bookkeeping, no cross-lane traffic.  A batch that would run past the pool is
        // counted but not written (the row is then redone from scratch anyway).
        auto filter_batch = [&](auto full, int base, const float4 (&x)[kLoads], float tau_f) {
          constexpr bool FULL = decltype(full)::value;   // every lane's 16 scores are inside the share
          int total = 0;
          u64 mask[kLoads * 4];   // (scalar registers)
#pragma unroll
          for (int u = 0; u < kLoads; ++u) {
            const float xs[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
            const bool in = FULL || base + (u * kThreads + tid) * 4 < e4;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              mask[u * 4 + c] = __builtin_amdgcn_ballot_w64(in && !(xs[c] < tau_f));
              total += __popcll(mask[u * 4 + c]);
            }
          }
          if (total == 0) return;  // uniform
          int at = 0;
          if (lane == 0) at = atomicAdd(&sh.fill_pool, total);
          at = __builtin_amdgcn_readfirstlane(at);
          if (at + total > kPoolCap) return;  // uniform
          const uint32_t cidx = 0xffffffffu - (uint32_t)(base + tid * 4);
#pragma unroll
          for (int u = 0; u < kLoads; ++u) {
            const float xs[4] = {x[u].x, x[u].y, x[u].z, x[u].w};
            const bool in = FULL || base + (u * kThreads + tid) * 4 < e4;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              const bool pass = in && !(xs[c] < tau_f);
              const u64 mk = mask[u * 4 + c];
              const int slot = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mk >> 32),
                                                               __builtin_amdgcn_mbcnt_lo((uint32_t)mk, (uint32_t)at));
              if (pass) {
                // the two halves of the entry from wherever they are, in one write
                // (a 64-bit store would first copy them into a register pair)
                const uint32_t addr = (uint32_t)(uintptr_t)(pool + slot);
                asm volatile("ds_write2_b32 %0, %1, %2 offset1:1"
                             :: "v"(addr), "v"(cidx - (uint32_t)(u * kThreads * 4 + c)), "v"(__float_as_uint(xs[c]))
                             : "memory");
              }
              at += __popcll(mk);
            }
          }
        };
        auto filter = [&](int base, const float4 (&x)[kLoads], float tau_f) {
          if (base >= e4) return;  // uniform
          if (base + kStep <= e4) filter_batch(BoolTag<true>{}, base, x, tau_f);
          else filter_batch(BoolTag<false>{}, base, x, tau_f);
        };
        float4 b0[kLoads], b1[kLoads], b2[kLoads];
        fetch(begin, b0);
        fetch(begin + kStep, b1);
        const uint32_t tau = sample_threshold<kThreads, VEC>(row, n, m, hist, sh, tid);
        for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;   // for the first refinement pass
        const float tau_f = tau >= 0xff800000u ? INFINITY : tau <= 0x007fffffu ? -INFINITY
                            : __uint_as_float((tau & 0x80000000u) ? (tau & 0x7fffffffu) : ~tau);
        for (int base = begin; base < e4; base += 3 * kStep) {
          fetch(base + 2 * kStep, b2);
          filter(base, b0, tau_f);
          fetch(base + 3 * kStep, b0);
          filter(base + kStep, b1, tau_f);
          fetch(base + 4 * kStep, b1);
          filter(base + 2 * kStep, b2, tau_f);
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the pool writes above are not the compiler's to wait for
        if (wave == 0) {
          const int i = e4 + lane;
          const float x = i < tail_end ? row[i] : 0.f;
          wave_append(i < tail_end && !(x < tau_f), composite(__float_as_uint(x), i), &sh.fill_pool, pool, kPoolCap);
        }
      } else {
        const uint32_t tau = sample_threshold<kThreads, VEC>(row, n, m, hist, sh, tid);
        for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;   // for the first refinement pass
        for_each_in<VEC, kThreads>(row, begin, tail_end, tid, [&](int i, float x) {
          wave_append(score_to_key(x) >= tau, composite(__float_as_uint(x), i), &sh.fill_pool, pool, kPoolCap);
        });
      }
      __syncthreads();
      // (an entry of the pool: the score's bits over the complemented index)
      auto keyed = [](u64 e) {
        return ((u64)score_to_key(__uint_as_float((uint32_t)(e >> 32))) << 32) | (e & 0xffffffffull);
      };
      const int got = sh.fill_pool;   // what passed here, also when it is more than the pool holds
      if (parts == 1) {
        if (got >= m && got <= kPoolCap) {
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (tid + u * kThreads < got) pv[u] = keyed(pool[tid + u * kThreads]);
          total = got;
        }
      } else {
        if (tid == 0) sh.base = atomicAdd(&row_count[rowi], got);
        __syncthreads();
        const int at = sh.base;
        u64* mine = loc + (int64_t)rowi * kPoolCap;
        if (at + got <= kPoolCap) {   // (a row whose parts pass more than the list holds is redone from scratch)
          for (int i = tid; i < got; i += kThreads) store_coherent(mine + at + i, keyed(pool[i]));
        }
        // Every lane waits until its written-through stores have been acknowledged,
        // the barrier collects the lanes, and only then is the ticket drawn: whoever
        // draws the last one can read every part's entries.
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid == 0) sh.last = draw_ticket(&row_done[rowi], (unsigned int)(parts - 1)) == (unsigned int)(parts - 1);
        __syncthreads();
        if (!sh.last) return;
        const int sum = __hip_atomic_load(&row_count[rowi], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (tid == 0) __hip_atomic_store(&row_count[rowi], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (sum >= m && sum <= kPoolCap) {
#pragma unroll
          for (int u = 0; u < U; ++u)
            if (tid + u * kThreads < sum) pv[u] = load_coherent(mine + tid + u * kThreads);
          total = sum;
        }
      }
      if (total >= 0) {
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (tid + u * kThreads < total) {
            const uint32_t k = (uint32_t)(pv[u] >> 32);
            kmin = min(kmin, k);
            kmax = max(kmax, k);
          }
      }
    } else if (part != 0) {
      return;   // no threshold can be relied on: one workgroup selects from scratch
    }
    if (total >= 0) {
      // range of the pooled composites, from their keys (the high halves): any range
      // that holds them all serves the refinement
      wave_minmax_to_last(kmin, kmax);
      if (lane == 63) {
        atomicMin(&sh.kmin, kmin);
        atomicMax(&sh.kmax, kmax);
      }
      __syncthreads();
      const u64 lo0 = (u64)sh.kmin << 32, hi0 = ((u64)sh.kmax << 32) | 0xffffffffull;
      const int shift0 = range_shift(lo0, hi0);
      // refinement on the composites; they are distinct, so it ends with a bin of
      // at most kCandCap entries (ties need no special case here).
      // The first pass covers every entry, and every entry keeps the slot that its
      // bin's counter hands out.  When that pass already isolates the k-th bin (the
      // usual case) the bins' counters, turned into offsets by the same scan that
      // finds the bin, and those slots place every winner next to the others of its
      // bin and the k-th bin's entries in their list with no further counting.
      {
        uint32_t slot2[U / 2];   // 16 bits per entry
#pragma unroll
        for (int u = 0; u < U / 2; ++u) slot2[u] = 0;   // (hist is zero: cleared ahead of the pool)
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (tid + u * kThreads < total) {
            const uint32_t sl = atomicAdd(&hist[(int)((pv[u] - lo0) >> shift0)], 1u);
            slot2[u >> 1] |= sl << (16 * (u & 1));
          }
        }
        __syncthreads();
        find_bin<kThreads, true>(hist, m, 1, sh, tid, [&](int bin, int before, int count) {
          const u64 blo = lo0 + ((u64)bin << shift0);
          const u64 bspan = (shift0 == 0) ? 0ull : ((1ull << shift0) - 1ull);
          sh.lo = blo;
          sh.hi = (hi0 - blo < bspan) ? hi0 : blo + bspan;
          sh.need = m - before;
          sh.done = (count <= kCandCap || shift0 == 0) ? 1 : 0;
        });
        if (sh.done && !sh.crowded) {
          const int fb = sh.found_bin, need = sh.need, ncand = min(sh.found_count, kCandCap);
#pragma unroll
          for (int u = 0; u < U; ++u) {
            if (tid + u * kThreads < total) {
              const u64 v = pv[u];
              const int bin = (int)((v - lo0) >> shift0);
              const int sl = (int)((slot2[u >> 1] >> (16 * (u & 1))) & 0xffffu);
              if (bin > fb) buf[(int)(hist[bin] & 0xffffu) + sl] = v;
              else if (bin == fb && sl < kCandCap) cand[sl] = v;
            }
          }
          __syncthreads();
          order_and_write(buf, m - need, cand, ncand, need, lo0, shift0, tmp, hist, sh, counting_ok != 0, heavy,
                          tid, true);
          return;
        }
      }
      for (int iter = 1; iter < 8 && !sh.done; ++iter) {
        const u64 lo = sh.lo, hi = sh.hi;
        const int need_in = sh.need;
        const int shift = range_shift(lo, hi);
        for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
        __syncthreads();
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const u64 v = pv[u];
          if (tid + u * kThreads < total && v >= lo && v <= hi) atomicAdd(&hist[(int)((v - lo) >> shift)], 1u);
        }
        __syncthreads();
        find_bin<kThreads>(hist, need_in, 1, sh, tid);
        if (tid == 0) {
          const u64 blo = lo + ((u64)sh.found_bin << shift);
          const u64 bspan = (shift == 0) ? 0ull : ((1ull << shift) - 1ull);
          sh.lo = blo;
          sh.hi = (hi - blo < bspan) ? hi : blo + bspan;
          sh.need = need_in - sh.found_before;
          sh.done = (sh.found_count <= kCandCap || shift == 0) ? 1 : 0;
        }
        __syncthreads();
        if (sh.done) break;
      }
      const u64 blo = sh.lo, bhi = sh.hi;
      const int need = sh.need;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const u64 v = pv[u];
        const bool have = tid + u * kThreads < total;
        wave_append(have && v > bhi, v, &sh.fill_above, buf, cap_above);
        wave_append(have && v >= blo && v <= bhi, v, &sh.fill_cand, cand, kCandCap);
      }
      __syncthreads();
      order_and_write(buf, m - need, cand, min(sh.fill_cand, kCandCap), need, lo0, shift0, tmp, hist, sh,
                      counting_ok != 0, heavy, tid);
      return;
    }
  } else if (part != 0) {
    return;
  }

  // ================================ from scratch ======================================
  // ---- key range of the row -----------------------------------------------------
  {
    uint32_t kmin = 0xffffffffu, kmax = 0u;
    if (row_range) {
      const uint32_t* rr = row_range + (int64_t)rowi * range_parts * 2;
      for (int i = tid; i < range_parts; i += kThreads) {
        kmin = min(kmin, rr[2 * i]);
        kmax = max(kmax, rr[2 * i + 1]);
      }
    } else {
      for_each_in<VEC, kThreads>(row, 0, n, tid, [&](int, float x) {
        const uint32_t k = score_to_key(x);
        kmin = min(kmin, k);
        kmax = max(kmax, k);
      });
    }
    wave_minmax_to_last(kmin, kmax);
    if (lane == 63) {
      sh.wmin[wave] = kmin;
      sh.wmax[wave] = kmax;
    }
    __syncthreads();
    if (tid == 0) {
      kmin = 0xffffffffu;
      kmax = 0u;
      for (int w = 0; w < kWaves; ++w) {
        kmin = min(kmin, (uint32_t)sh.wmin[w]);
        kmax = max(kmax, (uint32_t)sh.wmax[w]);
      }
      sh.lo = kmin;
      sh.hi = max(kmin, kmax);
      sh.need = m;
      sh.done = 0;
      sh.fill_above = 0;
      sh.fill_cand = 0;
      sh.idx_star = 0x7fffffff;
    }
    __syncthreads();
  }
  const uint32_t lo0 = (uint32_t)sh.lo;
  const int shift0 = range_shift(sh.lo, sh.hi);

  // ---- range refinement -------------------------------------------------------
  for (int iter = 0; iter < 4; ++iter) {
    const uint32_t lo = (uint32_t)sh.lo, hi = (uint32_t)sh.hi;
    const int need_in = sh.need;
    const int shift = range_shift(lo, hi);
    for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
    __syncthreads();
    for_each_in<VEC, kThreads>(row, 0, n, tid, [&](int, float x) {
      const uint32_t k = score_to_key(x);
      if (k >= lo && k <= hi) atomicAdd(&hist[(k - lo) >> shift], 1u);
    });
    __syncthreads();
    find_bin<kThreads>(hist, need_in, 1, sh, tid);
    if (tid == 0) {
      const uint32_t blo = lo + ((uint32_t)sh.found_bin << shift);
      const uint32_t bspan = (shift == 0) ? 0u : ((1u << shift) - 1u);
      sh.lo = blo;
      sh.hi = (hi - blo < bspan) ? hi : blo + bspan;
      sh.need = need_in - sh.found_before;
      sh.bin_count = sh.found_count;
      sh.done = (sh.found_count <= kCandCap || shift == 0) ? 1 : 0;
    }
    __syncthreads();
    if (sh.done) break;
  }

  const uint32_t blo = (uint32_t)sh.lo, bhi = (uint32_t)sh.hi;
  const int need = sh.need;  // keys to take from [blo, bhi]
  const int bin_count = sh.bin_count;
  const bool mass_ties = bin_count > kCandCap;  // then blo == bhi

  if (mass_ties) {
    // Take the `need` lowest indices among the keys equal to blo: histogram over
    // index ranges, then an in-order walk of the one range that straddles.
    const int binw = (n + kBins - 1) / kBins;
    for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
    __syncthreads();
    for_each_in<VEC, kThreads>(row, 0, n, tid, [&](int i, float x) {
      if (score_to_key(x) == blo) atomicAdd(&hist[i / binw], 1u);
    });
    __syncthreads();
    find_bin<kThreads>(hist, need, 0, sh, tid);
    if (wave == 0) {
      int rest = need - sh.found_before;  // >= 1 ties to take inside this index range
      const int i0 = sh.found_bin * binw, i1 = min(n, i0 + binw);
      int star = i0;
      for (int base = i0; base < i1 && rest > 0; base += SOCKET_WAVE) {
        const int i = base + lane;
        const bool eq = (i < i1) && (score_to_key(row[min(i, i1 - 1)]) == blo);
        const u64 mask = __ballot(eq);
        const int c = __popcll(mask);
        if (c >= rest) {
          u64 mm = mask;  // its rest-th set bit is the last tie taken
          for (int r = 1; r < rest; ++r) mm &= mm - 1;
          star = base + (__ffsll((long long)mm) - 1);
          rest = 0;
        } else {
          rest -= c;
        }
      }
      if (lane == 0) sh.idx_star = star;
    }
    __syncthreads();
  }

  // ---- collect ------------------------------------------------------------------
  const int idx_star = sh.idx_star;
  for_each_in<VEC, kThreads>(row, 0, n, tid, [&](int i, float x) {
    const uint32_t k = score_to_key(x);
    const u64 v = composite(k, i);
    const bool in_bin = k >= blo && k <= bhi;
    // mass ties: the ties with the lowest indices are winners outright (there can
    // be more of them than the candidate list holds)
    wave_append(k > bhi || (mass_ties && in_bin && i <= idx_star), v, &sh.fill_above, buf, cap_above);
    wave_append(!mass_ties && in_bin, v, &sh.fill_cand, cand, kCandCap);
  });
  __syncthreads();
  // mass ties: all m winners are in buf and there are no candidates
  const int ncand = mass_ties ? 0 : min(sh.fill_cand, kCandCap);
  const int n_above = mass_ties ? m : m - need;
  order_and_write(buf, n_above, cand, ncand, mass_ties ? 0 : need, (u64)lo0 << 32, shift0 + 32, tmp, hist,
                  sh, counting_ok != 0, heavy, tid);
}

int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

// Workgroups per row.  One workgroup streams its row at what one CU can pull
// (about 35 GB/s: 3.7 us per 32768 scores); sharing a row between several costs
// about 3 us for the exchange through memory, more when the launch then fills
// every CU (each part works out the threshold from the same sample, and each
// needs a CU to itself for its LDS).  Measured on 256 CUs with top-k 2048: two
// parts never pay; 8 or 32 rows gain from 49152 / 65536 scores up (9.5 and 7.6 us
// at 131072), 64 rows from 98304 up, 128 rows never.
int row_parts(int rows, int T, int m_max) {
  if (!(T > kPoolCap && m_max > 0 && sampling_ok(m_max))) return 1;
  const int cus = socket_device_limits().cu_count;
  int p = cus / rows;
  p = p < kMaxParts ? p : kMaxParts;
  p = p < T / kBatch ? p : T / kBatch;
  if (p < 3) return 1;
  const double saved = (double)T * (p - 1) / p;                 // scores a workgroup no longer streams
  return saved >= 24576.0 + 49152.0 * rows * p / cus ? p : 1;
}

struct SplitLayout {
  size_t off_loc, off_count, off_done, total;
};

// per row: a list of kPoolCap composites, its length, the arrivals
SplitLayout split_layout(int rows) {
  SplitLayout l;
  size_t o = 0;
  auto take = [&](size_t bytes) {
    const size_t at = o;
    o += (bytes + 255) / 256 * 256;
    return at;
  };
  l.off_count = take((size_t)rows * sizeof(int32_t));     // the two counter arrays first: they are
  l.off_done = take((size_t)rows * sizeof(uint32_t));     // what has to be zero on entry
  l.off_loc = take((size_t)rows * kPoolCap * sizeof(u64));
  l.total = o;
  return l;
}

}  // namespace

extern "C" size_t socket_select_workspace_bytes(int B, int Hq, int T, int M) {
  if (B <= 0 || Hq <= 0 || T <= 0 || M < 0) return 0;
  if (row_parts(B * Hq, T, M < T ? M : T) < 2) return 0;
  return split_layout(B * Hq).total;
}

extern "C" size_t socket_select_workspace_zero_bytes(int B, int Hq, int T, int M) {
  if (socket_select_workspace_bytes(B, Hq, T, M) == 0) return 0;
  return split_layout(B * Hq).off_loc;
}

extern "C" int socket_select_list(const float* scores, int64_t score_stride, const int32_t* lens,
                                  const int32_t* budgets, const uint32_t* row_range, int range_parts,
                                  int B, int Hq, int T, int M, int sink, int window, int write_base,
                                  int32_t* sparse_list, int64_t list_stride, int list_width,
                                  int32_t* sparse_len, void* workspace, size_t workspace_bytes,
                                  void* stream) {
  SOCKET_REQUIRE(scores && sparse_list, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && T > 0 && M >= 0 && sink >= 0 && window >= 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(score_stride >= T && list_width >= 0 && list_stride >= list_width, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(row_range == nullptr || range_parts > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(M <= SOCKET_TOPK_MAX_M, SOCKET_ERR_UNSUPPORTED);
  const int rows = B * Hq;
  SOCKET_REQUIRE(rows <= 65535, SOCKET_ERR_SHAPE);
  const int m_max = M < T ? M : T;
  const int cap_above = next_pow2(m_max > 0 ? m_max : 1);
  const SocketDeviceLimits& lim = socket_device_limits();
  const size_t lds_max = (size_t)lim.max_lds_per_block;
  const size_t lds_static = kBins * 4 + sizeof(SelectShared) + 256;
  size_t lds = (size_t)(cap_above + kCandCap) * sizeof(u64);
  SOCKET_REQUIRE(lds + lds_static <= lds_max, SOCKET_ERR_UNSUPPORTED);
  const bool vec = socket_aligned16(scores) && (score_stride % 4 == 0);
  hipStream_t s = (hipStream_t)stream;

  // extras as LDS allows: the pool (where a pooled select can apply at all), then
  // counting placement (2 * cap_above more slots)
  // (rows of at most kPoolCap scores are pooled whole, straight into registers)
  int use_pool = 0, counting_ok = 0, pool_slots = 0;
  if (T <= kPoolCap) {
    use_pool = 1;
  } else if (sampling_ok(m_max) && lds + (size_t)kPoolCap * sizeof(u64) + lds_static <= lds_max) {
    use_pool = 1;
    pool_slots = kPoolCap;
    lds += (size_t)kPoolCap * sizeof(u64);
  }
  if (lds + (size_t)2 * cap_above * sizeof(u64) + lds_static <= lds_max) {
    counting_ok = 1;
    lds += (size_t)2 * cap_above * sizeof(u64);
  }

  // rows shared between workgroups exchange their entries through the workspace
  int parts = (workspace && use_pool) ? row_parts(rows, T, m_max) : 1;
  u64* loc = nullptr;
  int32_t* row_count = nullptr;
  unsigned int* row_done = nullptr;
  if (parts > 1) {
    const SplitLayout l = split_layout(rows);
    SOCKET_REQUIRE(workspace_bytes >= l.total, SOCKET_ERR_WORKSPACE);
    SOCKET_REQUIRE(socket_aligned16(workspace), SOCKET_ERR_ALIGN);
    char* ws = (char*)workspace;
    loc = (u64*)(ws + l.off_loc);
    row_count = (int32_t*)(ws + l.off_count);
    row_done = (unsigned int*)(ws + l.off_done);
  }
  SOCKET_REQUIRE((int64_t)rows * parts <= 0x7fffffff, SOCKET_ERR_SHAPE);

  auto kern = vec ? select_list_kernel<true> : select_list_kernel<false>;
  if (lds > 32 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return SOCKET_ERR_LAUNCH;
  hipLaunchKernelGGL(kern, dim3(rows * parts), dim3(kThreads), lds, s, scores, score_stride, lens, budgets,
                     row_range, range_parts, Hq, T, M, sink, window, write_base, sparse_list,
                     list_stride, list_width, sparse_len, cap_above, counting_ok, use_pool, pool_slots, parts,
                     loc, row_count, row_done);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}
