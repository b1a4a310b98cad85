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
// keys follow as candidates, and one bitonic sort of (key, ~index) composites
// leaves the answer in order in the first k slots.  A bin that is a single key
// value with more than kCandCap copies (mass ties) is resolved by a histogram
// over index ranges instead, taking the lowest indices.  Only the first read of
// a row comes from HBM; the row stays in L2 for the later passes.
#include "socket_common.h"

namespace {

constexpr int kThreads = 1024;
constexpr int kBins = 2048;
constexpr int kCandCap = 2048;

struct SelectShared {
  uint32_t lo, hi;      // current key range (inclusive)
  int need;             // keys still to take from inside [lo, hi]
  int shift;            // bin = (key - lo) >> shift
  int bin;              // bin holding the k-th key
  int bin_count;        // keys in that bin
  int before;           // keys in the bins ranked before it
  int done;             // refinement finished
  int fill;             // append cursor of the sort buffer
  int idx_star;         // mass-tie case: largest index taken among the ties
  uint32_t wmin[kThreads / SOCKET_WAVE], wmax[kThreads / SOCKET_WAVE];
};

__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
  for (int d = 1; d < SOCKET_WAVE; d <<= 1) {
    int o = __shfl_up(v, d, SOCKET_WAVE);
    if (lane >= d) v += o;
  }
  return v;
}

// Executed by wave 0.  Ranks bins from the top (descending != 0) or from the
// bottom and finds the bin where the running count first reaches `need`.
__device__ __forceinline__ void find_bin(const uint32_t* hist, int need, int descending, int lane,
                                         int* bin_out, int* before_out, int* count_out) {
  constexpr int per = kBins / SOCKET_WAVE;  // 32 bins per lane
  int mine = 0;
  for (int i = 0; i < per; ++i) {
    const int r = lane * per + i;  // rank position
    mine += (int)hist[descending ? (kBins - 1 - r) : r];
  }
  const int incl = wave_incl_scan(mine, lane);
  const int excl = incl - mine;
  if (excl < need && need <= incl) {
    int run = excl;
    for (int i = 0; i < per; ++i) {
      const int r = lane * per + i;
      const int bin = descending ? (kBins - 1 - r) : r;
      const int c = (int)hist[bin];
      if (run < need && need <= run + c) {
        *bin_out = bin;
        *before_out = run;
        *count_out = c;
        break;
      }
      run += c;
    }
  }
}

// Visit scores[0:n] once, 16 bytes per lane per load and four loads in flight
// per lane (a lone workgroup per row has to cover the memory latency itself).
template <bool VEC, class F>
__device__ __forceinline__ void for_each_score(const float* row, int n, int tid, F&& f) {
  if (VEC) {
    const int n4 = n & ~3;
    constexpr int kStride = kThreads * 4;
    int i = tid * 4;
    for (; i + 3 * kStride < n4; i += 4 * kStride) {
      float4 x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) x[u] = *reinterpret_cast<const float4*>(row + i + u * kStride);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
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
    for (; i + 3 * kThreads < n; i += 4 * kThreads) {
      float x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) x[u] = row[i + u * kThreads];
#pragma unroll
      for (int u = 0; u < 4; ++u) f(i + u * kThreads, x[u]);
    }
    for (; i < n; i += kThreads) f(i, row[i]);
  }
}

template <bool VEC>
__global__ __launch_bounds__(kThreads) void select_list_kernel(
    const float* __restrict__ scores, int64_t score_stride, const int32_t* __restrict__ lens,
    const int32_t* __restrict__ budgets, int Hq, int T, int M, int sink, int window,
    int write_base, int32_t* __restrict__ sparse_list, int64_t list_stride, int list_width,
    int32_t* __restrict__ sparse_len, int cap) {
  __shared__ uint32_t hist[kBins];
  __shared__ SelectShared sh;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  unsigned long long* buf = reinterpret_cast<unsigned long long*>(lds_raw);

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

  // ---- pass 0: key range of the row -----------------------------------------
  {
    uint32_t kmin = 0xffffffffu, kmax = 0u;
    for_each_score<VEC>(row, n, tid, [&](int, float x) {
      const uint32_t k = score_to_key(x);
      kmin = min(kmin, k);
      kmax = max(kmax, k);
    });
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
      for (int w = 1; w < kThreads / SOCKET_WAVE; ++w) {
        kmin = min(kmin, sh.wmin[w]);
        kmax = max(kmax, sh.wmax[w]);
      }
      sh.lo = kmin;
      sh.hi = kmax;
      sh.need = m;
      sh.done = 0;
      sh.fill = 0;
      sh.idx_star = 0x7fffffff;
    }
    __syncthreads();
  }

  // ---- range refinement -------------------------------------------------------
  for (int iter = 0; iter < 4; ++iter) {
    const uint32_t lo = sh.lo, hi = sh.hi;
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
    if (wave == 0) {
      int bin = 0, before = 0, count = 0;
      find_bin(hist, sh.need, 1, lane, &bin, &before, &count);
      // exactly one lane found it; publish
      const unsigned long long found = __ballot(count > 0);
      const int src = __ffsll((long long)found) - 1;
      bin = __shfl(bin, src, SOCKET_WAVE);
      before = __shfl(before, src, SOCKET_WAVE);
      count = __shfl(count, src, SOCKET_WAVE);
      if (lane == 0) {
        const uint32_t blo = lo + ((uint32_t)bin << shift);
        const uint32_t bspan = (shift == 0) ? 0u : ((1u << shift) - 1u);
        const uint32_t bhi = (hi - blo < bspan) ? hi : blo + bspan;
        sh.lo = blo;
        sh.hi = bhi;
        sh.need = sh.need - before;
        sh.bin_count = count;
        sh.shift = shift;
        sh.done = (count <= kCandCap || shift == 0) ? 1 : 0;
      }
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
    if (wave == 0) {
      int bin = 0, before = 0, count = 0;
      find_bin(hist, need, 0, lane, &bin, &before, &count);
      const unsigned long long found = __ballot(count > 0);
      const int src = __ffsll((long long)found) - 1;
      bin = __shfl(bin, src, SOCKET_WAVE);
      before = __shfl(before, src, SOCKET_WAVE);
      int rest = need - before;  // >= 1 ties to take inside this index range
      const int i0 = bin * binw, i1 = min(n, i0 + binw);
      int star = i0;
      for (int base = i0; base < i1 && rest > 0; base += SOCKET_WAVE) {
        const int i = base + lane;
        const bool eq = (i < i1) && (score_to_key(row[i]) == blo);
        const unsigned long long mask = __ballot(eq);
        const int c = __popcll(mask);
        if (c >= rest) {
          // the rest-th set bit of mask
          unsigned long long mm = mask;
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
    const bool take = (k > bhi) || (k >= blo && (!mass_ties || i <= idx_star));
    if (take) {
      const int p = atomicAdd(&sh.fill, 1);
      if (p < cap) buf[p] = ((unsigned long long)k << 32) | (unsigned long long)(0xffffffffu - (uint32_t)i);
    }
  });
  __syncthreads();
  const int filled = min(sh.fill, cap);  // n_above + (mass_ties ? need : bin_count)
  (void)n_above;
  int np = 1;
  while (np < filled) np <<= 1;
  for (int i = filled + tid; i < np; i += kThreads) buf[i] = 0ull;
  __syncthreads();

  // ---- bitonic sort, descending --------------------------------------------------
  for (int k = 2; k <= np; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = tid; i < np; i += kThreads) {
        const int p = i ^ j;
        if (p > i) {
          const unsigned long long a = buf[i], c = buf[p];
          const bool desc_block = (i & k) == 0;
          if (desc_block ? (a < c) : (a > c)) {
            buf[i] = c;
            buf[p] = a;
          }
        }
      }
      __syncthreads();
    }
  }

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
                                  const int32_t* budgets, int B, int Hq, int T, int M, int sink,
                                  int window, int write_base, int32_t* sparse_list,
                                  int64_t list_stride, int list_width, int32_t* sparse_len,
                                  void* stream) {
  SOCKET_REQUIRE(scores && sparse_list, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && T > 0 && M >= 0 && sink >= 0 && window >= 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(score_stride >= T && list_width >= 0 && list_stride >= list_width, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(M <= SOCKET_TOPK_MAX_M, SOCKET_ERR_UNSUPPORTED);
  const int m_max = M < T ? M : T;
  const int cap = next_pow2(m_max + kCandCap);
  const size_t lds = (size_t)cap * sizeof(unsigned long long);
  const SocketDeviceLimits& lim = socket_device_limits();
  SOCKET_REQUIRE(lds + kBins * 4 + sizeof(SelectShared) + 256 <= (size_t)lim.max_lds_per_block,
                 SOCKET_ERR_UNSUPPORTED);
  const bool vec = socket_aligned16(scores) && (score_stride % 4 == 0);
  hipStream_t s = (hipStream_t)stream;
  const int rows = B * Hq;
  if (vec) {
    auto kern = select_list_kernel<true>;
    if (lds > 32 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return SOCKET_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(rows), dim3(kThreads), lds, s, scores, score_stride, lens, budgets,
                       Hq, T, M, sink, window, write_base, sparse_list, list_stride, list_width,
                       sparse_len, cap);
  } else {
    auto kern = select_list_kernel<false>;
    if (lds > 32 * 1024 &&
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
      return SOCKET_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3(rows), dim3(kThreads), lds, s, scores, score_stride, lens, budgets,
                       Hq, T, M, sink, window, write_base, sparse_list, list_stride, list_width,
                       sparse_len, cap);
  }
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}
