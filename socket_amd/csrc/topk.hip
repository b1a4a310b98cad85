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
template <bool VEC, class F>
__device__ __forceinline__ void for_each_score(const float* row, int n, int tid, F&& f) {
  constexpr int U = 8;
  if (VEC) {
    const int n4 = n & ~3;
    constexpr int kStride = kThreads * 4;
    int i = tid * 4;
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
    for (int t = n4 + tid; t < n; t += kThreads) f(t, row[t]);
  } else {
    int i = tid;
    for (; i + (U - 1) * kThreads < n; i += U * kThreads) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = row[i + u * kThreads];
#pragma unroll
      for (int u = 0; u < U; ++u) f(i + u * kThreads, x[u]);
    }
    for (; i < n; i += kThreads) f(i, row[i]);
  }
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

template <bool VEC>
__global__ __launch_bounds__(kThreads) void select_list_kernel(
    const float* __restrict__ scores, int64_t score_stride, const int32_t* __restrict__ lens,
    const int32_t* __restrict__ budgets, const uint32_t* __restrict__ row_range, int range_parts,
    int Hq, int T, int M, int sink, int window, int write_base, int32_t* __restrict__ sparse_list,
    int64_t list_stride, int list_width, int32_t* __restrict__ sparse_len, int cap_above) {
  __shared__ uint32_t hist[kBins];
  __shared__ SelectShared sh;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  unsigned long long* buf = reinterpret_cast<unsigned long long*>(lds_raw);  // winners
  unsigned long long* cand = buf + cap_above;                                // keys of the k-th bin

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
      for (int i = tid; i < nbase && i < list_width; i += kThreads)
        out[i] = i < s_e ? i : win_start + (i - s_e);
    }
  }
  const int total = min(nbase + m, list_width);
  m = max(0, total - nbase);
  for (int i = total + tid; i < list_width; i += kThreads) out[i] = -1;
  if (sparse_len && tid == 0) sparse_len[rowi] = total;
  if (m == 0) return;

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

int next_pow2(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

}  // namespace

extern "C" int socket_select_list(const float* scores, int64_t score_stride, const int32_t* lens,
                                  const int32_t* budgets, const uint32_t* row_range, int range_parts,
                                  int B, int Hq, int T, int M, int sink, int window, int write_base,
                                  int32_t* sparse_list, int64_t list_stride, int list_width,
                                  int32_t* sparse_len, void* stream) {
  SOCKET_REQUIRE(scores && sparse_list, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && T > 0 && M >= 0 && sink >= 0 && window >= 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(score_stride >= T && list_width >= 0 && list_stride >= list_width, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(row_range == nullptr || range_parts > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(M <= SOCKET_TOPK_MAX_M, SOCKET_ERR_UNSUPPORTED);
  const int m_max = M < T ? M : T;
  const int cap_above = next_pow2(m_max > 0 ? m_max : 1);
  const size_t lds = (size_t)(cap_above + kCandCap) * sizeof(unsigned long long);
  const SocketDeviceLimits& lim = socket_device_limits();
  SOCKET_REQUIRE(lds + kBins * 4 + sizeof(SelectShared) + 256 <= (size_t)lim.max_lds_per_block,
                 SOCKET_ERR_UNSUPPORTED);
  const bool vec = socket_aligned16(scores) && (score_stride % 4 == 0);
  hipStream_t s = (hipStream_t)stream;
  const int rows = B * Hq;
  auto kern = vec ? select_list_kernel<true> : select_list_kernel<false>;
  if (lds > 32 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
    return SOCKET_ERR_LAUNCH;
  hipLaunchKernelGGL(kern, dim3(rows), dim3(kThreads), lds, s, scores, score_stride, lens, budgets,
                     row_range, range_parts, Hq, T, M, sink, window, write_base, sparse_list,
                     list_stride, list_width, sparse_len, cap_above);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}
