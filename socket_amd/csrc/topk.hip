// K3: per-row top-k select with the "equal scores -> lower index first" rule,
// fused with the [sink | window | heavy] index-list assembly of
// GPT-FAST/kernels/sparse.py:57-95.
//
// One workgroup (1024 lanes) per score row.  Scores are mapped to
// order-preserving 32-bit keys.  The k-th largest key is located by range
// refinement: a 2048-bin LDS histogram over [lo, hi] (initially the row's
// min/max key, so bins are spread over the values that actually occur and the
// LDS atomics rarely collide), then the bin holding the k-th key becomes the
// new range.  As soon as that bin holds at most kCandCap keys the row is read
// one last time: keys above the bin go straight to an LDS buffer, the bin's
// keys are sorted on the side and the best of them appended, and one bitonic
// sort of (key, ~index) composites puts the k winners in descending order.  A
// bin that is a single key value with more than kCandCap copies (mass ties) is
// resolved by a histogram over index ranges instead, taking the lowest indices.
// Only the first read of a row comes from HBM; the row stays in L2 for the later
// passes.  The scorer can hand over each row's key range (per-tile partial
// minima / maxima), which saves the first pass.
//
// A single workgroup is bound by one CU's VALU rate (about ten operations per
// score per pass), so long rows are processed by the split path instead when
// the caller provides a workspace: the row is cut into slices of kSliceLen
// scores and four kernels run over (slice, row) or (row) grids --
//   select_hist_kernel       per-slice histograms over the row's key range
//   select_threshold_kernel  sums them, finds the bin of the k-th key
//   select_collect_kernel    appends winners / bin candidates to per-row lists
// -- after which the one-workgroup kernel only has to rank the gathered keys of
// each row (or, for a row whose k-th bin turned out too crowded for the
// candidate list -- mass ties -- does the whole job as before).
#include "socket_common.h"

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / SOCKET_WAVE;
constexpr int kBins = 2048;
constexpr int kCandCap = 2048;

struct SelectShared {
  uint32_t lo, hi;      // current key range (inclusive)
  int need;             // keys still to take from inside [lo, hi]
  int bin_count;        // keys in the bin holding the k-th key
  int done;             // refinement finished
  int fill_above;       // append cursor: keys above the bin
  int fill_cand;        // append cursor: keys inside the bin
  int idx_star;         // mass-tie case: largest index taken among the ties
  int found_bin, found_before, found_count;
  uint32_t wmin[kWaves], wmax[kWaves];
  int wsum[kWaves];
};

__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
  for (int d = 1; d < SOCKET_WAVE; d <<= 1) {
    int o = __shfl_up(v, d, SOCKET_WAVE);
    if (lane >= d) v += o;
  }
  return v;
}

// All lanes of the workgroup.  Ranks the bins from the top (descending != 0) or
// from the bottom, two per lane, and publishes in `sh` the bin where the running
// count first reaches `need`, the count ranked before it and its own count.
__device__ __forceinline__ void find_bin(const uint32_t* hist, int need, int descending,
                                         SelectShared& sh, int tid) {
  const int lane = tid & 63, wave = tid >> 6;
  const int r0 = 2 * tid, r1 = 2 * tid + 1;
  const int b0 = descending ? (kBins - 1 - r0) : r0;
  const int b1 = descending ? (kBins - 1 - r1) : r1;
  const int c0 = (int)hist[b0], c1 = (int)hist[b1];
  const int incl_w = wave_incl_scan(c0 + c1, lane);
  if (lane == 63) sh.wsum[wave] = incl_w;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; ++w) base += sh.wsum[w];
  const int excl = base + incl_w - (c0 + c1);
  if (excl < need && need <= excl + c0) {
    sh.found_bin = b0;
    sh.found_before = excl;
    sh.found_count = c0;
  } else if (excl + c0 < need && need <= excl + c0 + c1) {
    sh.found_bin = b1;
    sh.found_before = excl + c0;
    sh.found_count = c1;
  }
  __syncthreads();
}

// Visit scores[0:n] once, 16 bytes per lane per load and eight loads in flight
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

template <bool VEC, class F>
__device__ __forceinline__ void for_each_score(const float* row, int n, int tid, F&& f) {
  for_each_in<VEC, kThreads>(row, 0, n, tid, f);
}

// Append `value` to an LDS list if `take`: one atomic per wave, positions handed
// out by a ballot prefix count.  Safe under divergence (only active lanes vote).
__device__ __forceinline__ void wave_append(bool take, unsigned long long value, int* cursor,
                                            unsigned long long* list, int cap) {
  const unsigned long long mask = __ballot(take);
  if (mask == 0) return;
  const int lane = threadIdx.x & 63;
  const int leader = __ffsll((long long)mask) - 1;
  int base = 0;
  if (lane == leader) base = atomicAdd(cursor, __popcll(mask));
  base = __shfl(base, leader, SOCKET_WAVE);
  if (take) {
    const int p = base + __popcll(mask & ((1ull << lane) - 1ull));
    if (p < cap) list[p] = value;
  }
}

__device__ __forceinline__ unsigned long long shfl_xor_u64(unsigned long long v, int mask) {
  const uint32_t lo = (uint32_t)__shfl_xor((int)(uint32_t)v, mask, SOCKET_WAVE);
  const uint32_t hi = (uint32_t)__shfl_xor((int)(uint32_t)(v >> 32), mask, SOCKET_WAVE);
  return ((unsigned long long)hi << 32) | lo;
}

// Bitonic sort of buf[0:np] (np a power of two) into descending order by the
// whole workgroup.  Lane t owns elements [t*E, (t+1)*E): exchange distances
// below E stay in registers, below 64*E go through wave shuffles, and only the
// longer ones through LDS with a barrier.  Callers sync before and get a synced
// buffer back.
template <int E>
__device__ __forceinline__ void sort_desc_impl(unsigned long long* buf, int np, int tid) {
  const bool active = tid * E < np;
  unsigned long long r[E];
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
        const unsigned long long other = shfl_xor_u64(r[e], j / E);
        const bool lower = (i & j) == 0, desc = (i & k) == 0;
        const unsigned long long mx = r[e] > other ? r[e] : other;
        const unsigned long long mn = r[e] > other ? other : r[e];
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
        const unsigned long long a = r[e], c = r[p];
        const unsigned long long mx = a > c ? a : c, mn = a > c ? c : a;
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
          const unsigned long long a = buf[i], c = buf[p];
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

__device__ __forceinline__ void sort_desc(unsigned long long* buf, int np, int tid) {
  if (np <= kThreads) sort_desc_impl<1>(buf, np, tid);
  else if (np == 2 * kThreads) sort_desc_impl<2>(buf, np, tid);
  else if (np == 4 * kThreads) sort_desc_impl<4>(buf, np, tid);
  else if (np == 8 * kThreads) sort_desc_impl<8>(buf, np, tid);
  else sort_desc_impl<16>(buf, np, tid);
}

__device__ __forceinline__ int next_pow2_dev(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

// Sink / window part of a list row, its length and the -1 padding; clips the
// heavy budget m to the room left in the row.  Returns the base length.
__device__ __forceinline__ int write_list_base(int32_t* out, int n, int& m, int sink, int window,
                                               int write_base, int list_width, int32_t* len_out,
                                               int tid, int nthreads) {
  int nbase = 0;
  if (write_base) {
    const int s_e = max(0, min(sink, n));
    const int w_e = max(0, min(window, n));
    const int win_start = max(n - w_e, s_e);
    const int nwin = (w_e > 0 && win_start < n) ? n - win_start : 0;
    nbase = s_e + nwin;
    if (nbase == 0) {
      nbase = 1;
      if (tid == 0 && list_width > 0) out[0] = n - 1;
    } else {
      for (int i = tid; i < nbase && i < list_width; i += nthreads)
        out[i] = i < s_e ? i : win_start + (i - s_e);
    }
  }
  const int total = min(nbase + m, list_width);
  m = max(0, total - nbase);
  for (int i = total + tid; i < list_width; i += nthreads) out[i] = -1;
  if (len_out && tid == 0) *len_out = total;
  return nbase;
}

struct RowRecord {   // per row, written by select_threshold_kernel
  uint32_t range_lo;  // lowest key of the row (origin of the histogram bins)
  uint32_t blo, bhi;  // key range of the bin holding the k-th key
  int need;           // keys to take from that bin
  int bin_count;      // keys in that bin
  int shift;
  int flag;           // 1: left to the one-workgroup kernel
  int cur_above;      // append cursors of the row's global lists
  int cur_cand;
  int pad;
};

// Split path, last step, run by select_list_kernel for the rows the split
// kernels prepared: the winners sit in `win` in no order.  Their bins (the
// histogram bins above the k-th key's bin) already sort them coarsely, and a bin
// rarely holds more than a few, so each winner is placed at
//   (#winners in higher bins) + (#winners of its own bin that beat it)
// and the `need` best candidates of the k-th bin follow, ranked the same way.
// Crowded bins fall back to the bitonic sort.
constexpr int kMaxBinForCounting = 128;

__device__ __forceinline__ void finish_row(
    const RowRecord& rec, uint32_t range_lo, const unsigned long long* __restrict__ win_g,
    const unsigned long long* __restrict__ cand_g, unsigned long long* buf, unsigned long long* tmp,
    unsigned long long* cand, uint32_t* hist, SelectShared& sh, bool counting_ok, int32_t* out,
    int nbase, int m, int tid) {
  const int need = rec.need, n_above = m - need, ncand = min(rec.bin_count, kCandCap);
  const int lane = tid & 63, wave = tid >> 6;
  for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
  for (int i = tid; i < n_above; i += kThreads) buf[i] = win_g[i];
  for (int i = tid; i < ncand; i += kThreads) cand[i] = cand_g[i];
  __syncthreads();

  // ---- candidates of the k-th bin -------------------------------------------------
  if (ncand <= kMaxBinForCounting) {
    for (int i = tid; i < ncand; i += kThreads) {
      const unsigned long long v = cand[i];
      int r = 0;
      for (int j = 0; j < ncand; ++j) r += cand[j] > v;
      if (r < need) out[nbase + n_above + r] = (int32_t)(0xffffffffu - (uint32_t)(v & 0xffffffffull));
    }
  } else {
    const int npc = next_pow2_dev(ncand);
    for (int i = ncand + tid; i < npc; i += kThreads) cand[i] = 0ull;
    __syncthreads();
    sort_desc(cand, npc, tid);
    for (int i = tid; i < need; i += kThreads)
      out[nbase + n_above + i] = (int32_t)(0xffffffffu - (uint32_t)(cand[i] & 0xffffffffull));
  }

  // ---- winners ----------------------------------------------------------------------
  if (counting_ok) {
    // slot of each winner inside its bin, bin populations
    for (int i = tid; i < n_above; i += kThreads) {
      const uint32_t k = (uint32_t)(buf[i] >> 32);
      const int bin = (int)((k - range_lo) >> rec.shift);
      const uint32_t slot = atomicAdd(&hist[bin], 1u);
      tmp[i] = ((unsigned long long)bin << 32) | slot;  // parked until the offsets are known
    }
    __syncthreads();
    // descending exclusive scan: off[bin] = winners in higher bins; crowded-bin check
    const int b0 = kBins - 1 - 2 * tid, b1 = b0 - 1;
    const int c0 = (int)hist[b0], c1 = (int)hist[b1];
    const int incl_w = wave_incl_scan(c0 + c1, lane);
    int crowded = (c0 > kMaxBinForCounting || c1 > kMaxBinForCounting) ? 1 : 0;
    crowded = __any(crowded);
    if (lane == 63) sh.wsum[wave] = incl_w;
    if (lane == 0) sh.wmin[wave] = (uint32_t)crowded;
    __syncthreads();
    int base = 0, any_crowded = 0;
    for (int w = 0; w < kWaves; ++w) {
      if (w < wave) base += sh.wsum[w];
      any_crowded |= (int)sh.wmin[w];
    }
    const int excl = base + incl_w - (c0 + c1);
    __syncthreads();
    if (!any_crowded) {
      hist[b0] = (uint32_t)excl | ((uint32_t)c0 << 16);        // offset | population << 16
      hist[b1] = (uint32_t)(excl + c0) | ((uint32_t)c1 << 16);
      __syncthreads();
      // group by bin: cand[] is free again and doubles as the grouped copy when it is
      // large enough, else tmp's upper half (tmp has 2*cap_above slots)
      unsigned long long* grouped = tmp + n_above;
      for (int i = tid; i < n_above; i += kThreads) {
        const int bin = (int)(tmp[i] >> 32);
        const int slot = (int)(tmp[i] & 0xffffffffull);
        grouped[(hist[bin] & 0xffffu) + slot] = buf[i];
      }
      __syncthreads();
      for (int p = tid; p < n_above; p += kThreads) {
        const unsigned long long v = grouped[p];
        const uint32_t k = (uint32_t)(v >> 32);
        const uint32_t h = hist[(k - range_lo) >> rec.shift];
        const int s0 = (int)(h & 0xffffu), c = (int)(h >> 16);
        int r = 0;
        for (int q = s0; q < s0 + c; ++q) r += grouped[q] > v;
        out[nbase + s0 + r] = (int32_t)(0xffffffffu - (uint32_t)(v & 0xffffffffull));
      }
      return;
    }
  }
  const int np = next_pow2_dev(n_above);
  for (int i = n_above + tid; i < np; i += kThreads) buf[i] = 0ull;
  __syncthreads();
  sort_desc(buf, np, tid);
  for (int j = tid; j < n_above; j += kThreads)
    out[nbase + j] = (int32_t)(0xffffffffu - (uint32_t)(buf[j] & 0xffffffffull));
}

template <bool VEC>
__global__ __launch_bounds__(kThreads) void select_list_kernel(
    const float* __restrict__ scores, int64_t score_stride, const int32_t* __restrict__ lens,
    const int32_t* __restrict__ budgets, const uint32_t* __restrict__ row_range, int range_parts,
    int Hq, int T, int M, int sink, int window, int write_base, int32_t* __restrict__ sparse_list,
    int64_t list_stride, int list_width, int32_t* __restrict__ sparse_len, int cap_above,
    const RowRecord* __restrict__ records, const unsigned long long* __restrict__ win_g,
    const unsigned long long* __restrict__ cand_g, int counting_ok) {
  __shared__ uint32_t hist[kBins];
  __shared__ SelectShared sh;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  unsigned long long* buf = reinterpret_cast<unsigned long long*>(lds_raw);  // winners
  unsigned long long* cand = buf + cap_above;                                // keys of the k-th bin
  unsigned long long* tmp = cand + kCandCap;  // 2*cap_above more slots when counting_ok

  const int rowi = blockIdx.x;
  const int b = rowi / Hq;
  const int tid = threadIdx.x;
  const int lane = tid & (SOCKET_WAVE - 1);
  const int wave = tid / SOCKET_WAVE;
  const int n = lens ? max(0, min(lens[b], T)) : T;
  int m = budgets ? budgets[b] : M;
  m = max(0, min(min(m, M), n));
  const float* row = scores + (int64_t)rowi * score_stride;
  int32_t* out = sparse_list + (int64_t)rowi * list_stride;

  // ---- sink / window part, length, padding ---------------------------------
  const int nbase = write_list_base(out, n, m, sink, window, write_base, list_width,
                                    sparse_len ? sparse_len + rowi : nullptr, tid, kThreads);
  if (m == 0) return;

  // split path: the slice kernels have located the k-th key and gathered the
  // winners unless the row is flagged (then it is done here from scratch)
  if (records) {
    const RowRecord rec = records[rowi];
    if (!rec.flag) {
      finish_row(rec, rec.range_lo, win_g + (int64_t)rowi * cap_above, cand_g + (int64_t)rowi * kCandCap,
                 buf, tmp, cand, hist, sh, counting_ok != 0, out, nbase, m, tid);
      return;
    }
  }

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
      for_each_score<VEC>(row, n, tid, [&](int, float x) {
        const uint32_t k = score_to_key(x);
        kmin = min(kmin, k);
        kmax = max(kmax, k);
      });
    }
#pragma unroll
    for (int d = SOCKET_WAVE / 2; d > 0; d >>= 1) {
      kmin = min(kmin, (uint32_t)__shfl_xor((int)kmin, d, SOCKET_WAVE));
      kmax = max(kmax, (uint32_t)__shfl_xor((int)kmax, d, SOCKET_WAVE));
    }
    if (lane == 0) {
      sh.wmin[wave] = kmin;
      sh.wmax[wave] = kmax;
    }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < kWaves; ++w) {
        kmin = min(kmin, sh.wmin[w]);
        kmax = max(kmax, sh.wmax[w]);
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

  // ---- range refinement -------------------------------------------------------
  for (int iter = 0; iter < 4; ++iter) {
    const uint32_t lo = sh.lo, hi = sh.hi;
    const int need_in = sh.need;
    const uint32_t span = hi - lo;  // width - 1
    int shift = 0;
    while ((span >> shift) >= (uint32_t)kBins) ++shift;
    for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
    __syncthreads();
    for_each_score<VEC>(row, n, tid, [&](int, float x) {
      const uint32_t k = score_to_key(x);
      if (k >= lo && k <= hi) atomicAdd(&hist[(k - lo) >> shift], 1u);
    });
    __syncthreads();
    find_bin(hist, need_in, 1, sh, tid);
    if (tid == 0) {
      const uint32_t blo = lo + ((uint32_t)sh.found_bin << shift);
      const uint32_t bspan = (shift == 0) ? 0u : ((1u << shift) - 1u);
      const uint32_t bhi = (hi - blo < bspan) ? hi : blo + bspan;
      sh.lo = blo;
      sh.hi = bhi;
      sh.need = need_in - sh.found_before;
      sh.bin_count = sh.found_count;
      sh.done = (sh.found_count <= kCandCap || shift == 0) ? 1 : 0;
    }
    __syncthreads();
    if (sh.done) break;
  }

  const uint32_t blo = sh.lo, bhi = sh.hi;
  const int need = sh.need;         // keys to take from [blo, bhi]
  const int bin_count = sh.bin_count;
  const int n_above = m - need;     // keys > bhi, all taken
  const bool mass_ties = bin_count > kCandCap;  // then blo == bhi

  if (mass_ties) {
    // Take the `need` lowest indices among the keys equal to blo: histogram over
    // index ranges, then an in-order walk of the one range that straddles.
    const int binw = (n + kBins - 1) / kBins;
    for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
    __syncthreads();
    for_each_score<VEC>(row, n, tid, [&](int i, float x) {
      if (score_to_key(x) == blo) atomicAdd(&hist[i / binw], 1u);
    });
    __syncthreads();
    find_bin(hist, need, 0, sh, tid);
    if (wave == 0) {
      int rest = need - sh.found_before;  // >= 1 ties to take inside this index range
      const int i0 = sh.found_bin * binw, i1 = min(n, i0 + binw);
      int star = i0;
      for (int base = i0; base < i1 && rest > 0; base += SOCKET_WAVE) {
        const int i = base + lane;
        const bool eq = (i < i1) && (score_to_key(row[i]) == blo);
        const unsigned long long mask = __ballot(eq);
        const int c = __popcll(mask);
        if (c >= rest) {
          unsigned long long mm = mask;  // its rest-th set bit is the last tie taken
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
  for_each_score<VEC>(row, n, tid, [&](int i, float x) {
    const uint32_t k = score_to_key(x);
    const unsigned long long v = ((unsigned long long)k << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
    const bool in_bin = k >= blo && k <= bhi;
    // mass ties: the ties with the lowest indices are winners outright (there can
    // be more of them than the candidate list holds)
    wave_append(k > bhi || (mass_ties && in_bin && i <= idx_star), v, &sh.fill_above, buf, cap_above);
    wave_append(!mass_ties && in_bin, v, &sh.fill_cand, cand, kCandCap);
  });
  __syncthreads();
  // mass ties: sh.fill_above == m, no candidates; else fill_above == n_above, fill_cand == bin_count
  const int ncand = min(sh.fill_cand, kCandCap);
  if (ncand > need) {  // uniform: rank the bin's keys, the best `need` of them win
    const int npc = next_pow2_dev(ncand);
    for (int i = ncand + tid; i < npc; i += kThreads) cand[i] = 0ull;
    __syncthreads();
    sort_desc(cand, npc, tid);
  }
  if (!mass_ties)
    for (int i = tid; i < need; i += kThreads) buf[n_above + i] = cand[i];
  const int np = next_pow2_dev(m);
  for (int i = m + tid; i < np; i += kThreads) buf[i] = 0ull;
  __syncthreads();
  sort_desc(buf, np, tid);

  for (int j = tid; j < m; j += kThreads)
    out[nbase + j] = (int32_t)(0xffffffffu - (uint32_t)(buf[j] & 0xffffffffull));
}

// ---------------------------------------------------------------------------
// split path
// ---------------------------------------------------------------------------
constexpr int kSliceLen = 16384;   // scores per (slice, row) workgroup
constexpr int kSliceThreads = 256;
constexpr int kSliceWaves = kSliceThreads / SOCKET_WAVE;

__device__ __forceinline__ void row_shape(const int32_t* lens, const int32_t* budgets, int b, int T,
                                          int M, int sink, int window, int write_base, int list_width,
                                          int& n, int& m) {
  n = lens ? max(0, min(lens[b], T)) : T;
  m = budgets ? budgets[b] : M;
  m = max(0, min(min(m, M), n));
  int nbase = 0;
  if (write_base) {
    const int s_e = max(0, min(sink, n));
    const int w_e = max(0, min(window, n));
    const int win_start = max(n - w_e, s_e);
    nbase = s_e + ((w_e > 0 && win_start < n) ? n - win_start : 0);
    if (nbase == 0) nbase = 1;
  }
  m = max(0, min(nbase + m, list_width) - nbase);
}

// Key range of the row from `parts` (min, max) pairs; every lane gets it.
template <int THREADS>
__device__ __forceinline__ void reduce_range(const uint32_t* rr, int parts, int tid, uint32_t* red,
                                             uint32_t& lo, uint32_t& hi) {
  uint32_t kmin = 0xffffffffu, kmax = 0u;
  for (int i = tid; i < parts; i += THREADS) {
    kmin = min(kmin, rr[2 * i]);
    kmax = max(kmax, rr[2 * i + 1]);
  }
#pragma unroll
  for (int d = SOCKET_WAVE / 2; d > 0; d >>= 1) {
    kmin = min(kmin, (uint32_t)__shfl_xor((int)kmin, d, SOCKET_WAVE));
    kmax = max(kmax, (uint32_t)__shfl_xor((int)kmax, d, SOCKET_WAVE));
  }
  constexpr int W = THREADS / SOCKET_WAVE;
  if ((tid & 63) == 0) {
    red[2 * (tid >> 6)] = kmin;
    red[2 * (tid >> 6) + 1] = kmax;
  }
  __syncthreads();
  lo = 0xffffffffu;
  hi = 0u;
  for (int w = 0; w < W; ++w) {
    lo = min(lo, red[2 * w]);
    hi = max(hi, red[2 * w + 1]);
  }
  hi = max(lo, hi);
  __syncthreads();
}

__device__ __forceinline__ int range_shift(uint32_t lo, uint32_t hi) {
  const uint32_t span = hi - lo;
  int shift = 0;
  while ((span >> shift) >= (uint32_t)kBins) ++shift;
  return shift;
}

// Per-slice (min, max) keys, for callers that have no ranges from the scorer.
template <bool VEC>
__global__ __launch_bounds__(kSliceThreads) void select_range_kernel(
    const float* __restrict__ scores, int64_t score_stride, const int32_t* __restrict__ lens, int Hq,
    int T, uint32_t* __restrict__ parts, int S) {
  __shared__ uint32_t red[2 * kSliceWaves];
  const int s = blockIdx.x, rowi = blockIdx.y, tid = threadIdx.x;
  const int n = lens ? max(0, min(lens[rowi / Hq], T)) : T;
  const int begin = s * kSliceLen, end = min(n, begin + kSliceLen);
  uint32_t kmin = 0xffffffffu, kmax = 0u;
  if (begin < end) {
    for_each_in<VEC, kSliceThreads>(scores + (int64_t)rowi * score_stride, begin, end, tid, [&](int, float x) {
      const uint32_t k = score_to_key(x);
      kmin = min(kmin, k);
      kmax = max(kmax, k);
    });
  }
#pragma unroll
  for (int d = SOCKET_WAVE / 2; d > 0; d >>= 1) {
    kmin = min(kmin, (uint32_t)__shfl_xor((int)kmin, d, SOCKET_WAVE));
    kmax = max(kmax, (uint32_t)__shfl_xor((int)kmax, d, SOCKET_WAVE));
  }
  if ((tid & 63) == 0) {
    red[2 * (tid >> 6)] = kmin;
    red[2 * (tid >> 6) + 1] = kmax;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < kSliceWaves; ++w) {
      kmin = min(kmin, red[2 * w]);
      kmax = max(kmax, red[2 * w + 1]);
    }
    parts[((int64_t)rowi * S + s) * 2] = kmin;
    parts[((int64_t)rowi * S + s) * 2 + 1] = kmax;
  }
}

template <bool VEC>
__global__ __launch_bounds__(kSliceThreads) void select_hist_kernel(
    const float* __restrict__ scores, int64_t score_stride, const int32_t* __restrict__ lens,
    const uint32_t* __restrict__ row_range, int range_parts, int Hq, int T,
    uint32_t* __restrict__ hist_parts, int S) {
  __shared__ uint32_t hist[kBins];
  __shared__ uint32_t red[2 * kSliceWaves];
  const int s = blockIdx.x, rowi = blockIdx.y, tid = threadIdx.x;
  const int n = lens ? max(0, min(lens[rowi / Hq], T)) : T;
  const int begin = s * kSliceLen, end = min(n, begin + kSliceLen);
  uint32_t* dst = hist_parts + ((int64_t)rowi * S + s) * kBins;
  for (int i = tid; i < kBins; i += kSliceThreads) hist[i] = 0;
  uint32_t lo, hi;
  reduce_range<kSliceThreads>(row_range + (int64_t)rowi * range_parts * 2, range_parts, tid, red, lo, hi);
  if (begin < end) {
    const int shift = range_shift(lo, hi);
    for_each_in<VEC, kSliceThreads>(scores + (int64_t)rowi * score_stride, begin, end, tid, [&](int, float x) {
      const uint32_t k = score_to_key(x);
      if (k >= lo && k <= hi) atomicAdd(&hist[(k - lo) >> shift], 1u);
    });
  }
  __syncthreads();
  for (int i = tid; i < kBins; i += kSliceThreads) dst[i] = hist[i];
}

__global__ __launch_bounds__(kThreads) void select_threshold_kernel(
    const int32_t* __restrict__ lens, const int32_t* __restrict__ budgets,
    const uint32_t* __restrict__ row_range, int range_parts, int Hq, int T, int M, int sink, int window,
    int write_base, int list_width, const uint32_t* __restrict__ hist_parts, int S,
    RowRecord* __restrict__ records) {
  __shared__ uint32_t hist[kBins];
  __shared__ uint32_t red[2 * kWaves];
  __shared__ SelectShared sh;
  const int rowi = blockIdx.x, tid = threadIdx.x;
  int n, m;
  row_shape(lens, budgets, rowi / Hq, T, M, sink, window, write_base, list_width, n, m);
  uint32_t lo, hi;
  reduce_range<kThreads>(row_range + (int64_t)rowi * range_parts * 2, range_parts, tid, red, lo, hi);
  RowRecord rec{lo, 0u, 0u, 0, 0, 0, 0, 0, 0, 0};
  if (m > 0) {
    const uint32_t* src = hist_parts + (int64_t)rowi * S * kBins;
    uint32_t c0 = 0, c1 = 0;
    for (int s = 0; s < S; ++s) {
      c0 += src[(int64_t)s * kBins + 2 * tid];
      c1 += src[(int64_t)s * kBins + 2 * tid + 1];
    }
    hist[2 * tid] = c0;
    hist[2 * tid + 1] = c1;
    __syncthreads();
    find_bin(hist, m, 1, sh, tid);
    const int shift = range_shift(lo, hi);
    const uint32_t blo = lo + ((uint32_t)sh.found_bin << shift);
    const uint32_t bspan = (shift == 0) ? 0u : ((1u << shift) - 1u);
    rec.blo = blo;
    rec.bhi = (hi - blo < bspan) ? hi : blo + bspan;
    rec.need = m - sh.found_before;
    rec.bin_count = sh.found_count;
    rec.shift = shift;
    rec.flag = sh.found_count > kCandCap ? 1 : 0;
  }
  if (tid == 0) records[rowi] = rec;
}

// Winners and bin candidates of the slice are gathered in LDS first, so each
// workgroup makes two global atomics (to reserve its runs in the row's lists),
// not one per wave and load.
template <bool VEC>
__global__ __launch_bounds__(kSliceThreads) void select_collect_kernel(
    const float* __restrict__ scores, int64_t score_stride, const int32_t* __restrict__ lens, int Hq,
    int T, RowRecord* __restrict__ records, unsigned long long* __restrict__ win, int cap_above,
    unsigned long long* __restrict__ cand) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  unsigned long long* lw = reinterpret_cast<unsigned long long*>(lds_raw);  // [cap_above]
  unsigned long long* lc = lw + cap_above;                                  // [kCandCap]
  __shared__ int cur[4];  // local counts, then global bases
  const int s = blockIdx.x, rowi = blockIdx.y, tid = threadIdx.x;
  const int n = lens ? max(0, min(lens[rowi / Hq], T)) : T;
  const int begin = s * kSliceLen, end = min(n, begin + kSliceLen);
  RowRecord* rec = records + rowi;
  if (begin >= end || rec->flag || rec->need <= 0) return;
  const uint32_t blo = rec->blo, bhi = rec->bhi;
  if (tid < 2) cur[tid] = 0;
  __syncthreads();
  for_each_in<VEC, kSliceThreads>(scores + (int64_t)rowi * score_stride, begin, end, tid, [&](int i, float x) {
    const uint32_t k = score_to_key(x);
    const unsigned long long v = ((unsigned long long)k << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
    wave_append(k > bhi, v, &cur[0], lw, cap_above);
    wave_append(k >= blo && k <= bhi, v, &cur[1], lc, kCandCap);
  });
  __syncthreads();
  const int nw = min(cur[0], cap_above), nc = min(cur[1], kCandCap);
  if (tid == 0) cur[2] = nw ? atomicAdd(&rec->cur_above, nw) : 0;
  if (tid == 1) cur[3] = nc ? atomicAdd(&rec->cur_cand, nc) : 0;
  __syncthreads();
  unsigned long long* w = win + (int64_t)rowi * cap_above + cur[2];
  unsigned long long* c = cand + (int64_t)rowi * kCandCap + cur[3];
  for (int i = tid; i < nw; i += kSliceThreads)
    if (cur[2] + i < cap_above) w[i] = lw[i];
  for (int i = tid; i < nc; i += kSliceThreads)
    if (cur[3] + i < kCandCap) c[i] = lc[i];
}

int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

struct SplitLayout {
  int S;
  size_t off_records, off_parts, off_hist, off_win, off_cand, total;
};

SplitLayout split_layout(int rows, int T, int cap_above) {
  SplitLayout l;
  l.S = (T + kSliceLen - 1) / kSliceLen;
  size_t o = 0;
  auto take = [&](size_t bytes) {
    const size_t at = o;
    o += (bytes + 255) / 256 * 256;
    return at;
  };
  l.off_records = take((size_t)rows * sizeof(RowRecord));
  l.off_parts = take((size_t)rows * l.S * 2 * sizeof(uint32_t));
  l.off_hist = take((size_t)rows * l.S * kBins * sizeof(uint32_t));
  l.off_win = take((size_t)rows * cap_above * sizeof(unsigned long long));
  l.off_cand = take((size_t)rows * kCandCap * sizeof(unsigned long long));
  l.total = o;
  return l;
}

// The split path pays off once a row is several slices long.
bool use_split(int T) { return T >= 4 * kSliceLen; }

}  // namespace

extern "C" size_t socket_select_workspace_bytes(int B, int Hq, int T, int M) {
  if (B <= 0 || Hq <= 0 || T <= 0 || M < 0 || !use_split(T)) return 0;
  const int m_max = M < T ? M : T;
  return split_layout(B * Hq, T, next_pow2(m_max > 0 ? m_max : 1)).total;
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
  const int m_max = M < T ? M : T;
  const int cap_above = next_pow2(m_max > 0 ? m_max : 1);
  const size_t lds_base = (size_t)(cap_above + kCandCap) * sizeof(unsigned long long);
  const SocketDeviceLimits& lim = socket_device_limits();
  const size_t lds_static = kBins * 4 + sizeof(SelectShared) + 256;
  SOCKET_REQUIRE(lds_base + lds_static <= (size_t)lim.max_lds_per_block, SOCKET_ERR_UNSUPPORTED);
  // ranking by bins needs two more arrays of cap_above slots
  const size_t lds_counting = lds_base + (size_t)2 * cap_above * sizeof(unsigned long long);
  const int counting_ok = lds_counting + lds_static <= (size_t)lim.max_lds_per_block ? 1 : 0;
  const bool vec = socket_aligned16(scores) && (score_stride % 4 == 0);
  hipStream_t s = (hipStream_t)stream;
  const int rows = B * Hq;
  SOCKET_REQUIRE(rows <= 65535, SOCKET_ERR_SHAPE);

  const RowRecord* records_arg = nullptr;
  const unsigned long long *win_arg = nullptr, *cand_arg = nullptr;
  if (workspace != nullptr && use_split(T) && M > 0) {
    const SplitLayout l = split_layout(rows, T, cap_above);
    SOCKET_REQUIRE(workspace_bytes >= l.total, SOCKET_ERR_WORKSPACE);
    SOCKET_REQUIRE(socket_aligned16(workspace), SOCKET_ERR_ALIGN);
    char* ws = (char*)workspace;
    RowRecord* records = (RowRecord*)(ws + l.off_records);
    uint32_t* parts = (uint32_t*)(ws + l.off_parts);
    uint32_t* hist_parts = (uint32_t*)(ws + l.off_hist);
    unsigned long long* win = (unsigned long long*)(ws + l.off_win);
    unsigned long long* cand = (unsigned long long*)(ws + l.off_cand);
    const dim3 sgrid(l.S, rows);
    if (row_range == nullptr) {
      if (vec) hipLaunchKernelGGL(select_range_kernel<true>, sgrid, dim3(kSliceThreads), 0, s, scores, score_stride, lens, Hq, T, parts, l.S);
      else hipLaunchKernelGGL(select_range_kernel<false>, sgrid, dim3(kSliceThreads), 0, s, scores, score_stride, lens, Hq, T, parts, l.S);
      row_range = parts;
      range_parts = l.S;
    }
    if (vec) hipLaunchKernelGGL(select_hist_kernel<true>, sgrid, dim3(kSliceThreads), 0, s, scores, score_stride, lens, row_range, range_parts, Hq, T, hist_parts, l.S);
    else hipLaunchKernelGGL(select_hist_kernel<false>, sgrid, dim3(kSliceThreads), 0, s, scores, score_stride, lens, row_range, range_parts, Hq, T, hist_parts, l.S);
    hipLaunchKernelGGL(select_threshold_kernel, dim3(rows), dim3(kThreads), 0, s, lens, budgets, row_range,
                       range_parts, Hq, T, M, sink, window, write_base, list_width, hist_parts, l.S, records);
    {
      auto ck = vec ? select_collect_kernel<true> : select_collect_kernel<false>;
      if (lds_base > 32 * 1024 &&
          hipFuncSetAttribute(reinterpret_cast<const void*>(ck),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_base) != hipSuccess)
        return SOCKET_ERR_LAUNCH;
      hipLaunchKernelGGL(ck, sgrid, dim3(kSliceThreads), lds_base, s, scores, score_stride, lens, Hq, T,
                         records, win, cap_above, cand);
    }
    SOCKET_LAUNCH_CHECK();
    records_arg = records;
    win_arg = win;
    cand_arg = cand;
  }

  auto kern = vec ? select_list_kernel<true> : select_list_kernel<false>;
  const size_t lds = (records_arg && counting_ok) ? lds_counting : lds_base;
  if (lds > 32 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return SOCKET_ERR_LAUNCH;
  hipLaunchKernelGGL(kern, dim3(rows), dim3(kThreads), lds, s, scores, score_stride, lens, budgets,
                     row_range, range_parts, Hq, T, M, sink, window, write_base, sparse_list,
                     list_stride, list_width, sparse_len, cap_above, records_arg, win_arg, cand_arg,
                     counting_ok);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}
