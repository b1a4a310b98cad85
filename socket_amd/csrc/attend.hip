// K4: split-K sparse flash-decode over an index list, the cross-split merge, and
// the dense flash-decode comparator.
//
// Arithmetic follows kernels/socket_triton_kernels.py:31-164: logits
// (q . k) / sqrt(D), running-max softmax, each split emits acc / sum_exp and
// max + log(sum_exp), stage 2 re-weights the splits by exp(lse - max).  Products
// and sums are fp32.
//
// Work layout (wave64): one K or V row of D elements is D / (16 B worth of
// elements) lanes wide, so a wave fetches 64 / lanes_per_row rows with one
// 16-byte load per lane (4 rows for bf16 D=128).  Each row slot keeps its own
// running (max, sum, acc) so the only cross-lane traffic in the loop is the
// dot-product reduction inside a row's lanes; slots and waves are merged once at
// the end through shuffles and LDS.  Loads for kUnroll row groups are issued
// before any is consumed to keep enough gathers in flight.
#include <math.h>

#include <atomic>

#include "socket_common.h"

namespace {

constexpr int kAttThreads = 256;
constexpr int kAttWaves = kAttThreads / SOCKET_WAVE;
constexpr int kUnroll = 4;

__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }

// Stores and loads that are coherent across the whole GPU without a fence: the
// store is written through to where every compute die sees it, the load does not
// take a copy from this die's caches.  (A device-scope fence instead writes back
// everything dirty in the die's L2 -- the scores the scorer has just written
// among it -- and made the one-launch attention slower than two launches.)
__device__ __forceinline__ void store_coherent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_coherent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Merge (m, l, acc) pairs of an online softmax.
template <int E>
__device__ __forceinline__ void merge_state(float& m, float& l, float* acc, float m2, float l2,
                                            const float* acc2) {
  const float nm = fmaxf(m, m2);
  const float s1 = (m == nm) ? 1.f : fast_exp(m - nm);
  const float s2 = (m2 == nm) ? 1.f : fast_exp(m2 - nm);
  l = l * s1 + l2 * s2;
#pragma unroll
  for (int i = 0; i < E; ++i) acc[i] = acc[i] * s1 + acc2[i] * s2;
  m = nm;
}

// The split's output from the waves' states in LDS, records [wave][head] of D
// accumulators (not yet divided by the sum), the running maximum and the sum:
// acc / sum and max + log(sum) per head, as kernels/socket_triton_kernels.py:82-95.
template <int D, int GH, bool COHERENT>
__device__ __forceinline__ void combine_waves(const float* lds, int G, float* mid_o_base, float* mid_lse_base,
                                              int64_t head_stride_o, int64_t head_stride_lse) {
  constexpr int REC = D + 2;
  for (int o = threadIdx.x; o < GH * D; o += kAttThreads) {
    const int g = o / D, d = o % D;
    if (g >= G) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < kAttWaves; ++w) M = fmaxf(M, lds[(w * GH + g) * REC + D]);
    float Lsum = 0.f, val = 0.f;
#pragma unroll
    for (int w = 0; w < kAttWaves; ++w) {
      const float* rec = lds + (w * GH + g) * REC;
      const float sc = (rec[D] == M) ? 1.f : fast_exp(rec[D] - M);
      Lsum += rec[D + 1] * sc;
      val += rec[d] * sc;
    }
    const bool any = Lsum > 0.f;
    if (COHERENT) {
      store_coherent(mid_o_base + g * head_stride_o + d, any ? val / Lsum : 0.f);
      if (d == 0) store_coherent(mid_lse_base + g * head_stride_lse, any ? M + logf(Lsum) : -INFINITY);
    } else {
      mid_o_base[g * head_stride_o + d] = any ? val / Lsum : 0.f;
      if (d == 0) mid_lse_base[g * head_stride_lse] = any ? M + logf(Lsum) : -INFINITY;
    }
  }
}

// Final merge of the workgroup's states and the split's output.  Every lane
// holds the state of (row slot, column chunk); GH heads per lane.
template <int E, int LPR, int GH, bool COHERENT = false>
__device__ __forceinline__ void finish_split(float (&m)[GH], float (&l)[GH], float (&acc)[GH][E],
                                             int G, float* mid_o_base, float* mid_lse_base,
                                             int64_t head_stride_o, int64_t head_stride_lse,
                                             float* lds) {
  constexpr int D = E * LPR;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int chunk = lane % LPR;
  // row slots inside the wave
#pragma unroll
  for (int d = LPR; d < SOCKET_WAVE; d <<= 1) {
#pragma unroll
    for (int g = 0; g < GH; ++g) {
      auto partner = [&](float x) {
        return d == 16 ? lane_xor16(x) : d == 32 ? lane_xor32(x) : __shfl_xor(x, d, SOCKET_WAVE);
      };
      const float m2 = partner(m[g]);
      const float l2 = partner(l[g]);
      float a2[E];
#pragma unroll
      for (int i = 0; i < E; ++i) a2[i] = partner(acc[g][i]);
      merge_state<E>(m[g], l[g], acc[g], m2, l2, a2);
    }
  }
  // waves through LDS: [wave][g][D + 2]
  constexpr int REC = D + 2;
  if (lane < LPR) {
#pragma unroll
    for (int g = 0; g < GH; ++g) {
      float* rec = lds + (wave * GH + g) * REC;
#pragma unroll
      for (int i = 0; i < E; ++i) rec[chunk * E + i] = acc[g][i];
      if (chunk == 0) {
        rec[D] = m[g];
        rec[D + 1] = l[g];
      }
    }
  }
  __syncthreads();
  combine_waves<D, GH, COHERENT>(lds, G, mid_o_base, mid_lse_base, head_stride_o, head_stride_lse);
}

constexpr int kMergeThreads = 256;

// Merge of the per-split partials of one (b, h) by a workgroup of 256 lanes: the
// largest log-sum-exp first, then the lanes, four output coordinates each and
// 256 / (D/4) splits side by side, add up weight * partial with independent
// loads, and LDS folds the side-by-side groups.
constexpr int kMergeEarly = 4;   // rounds of splits a lane of stage2_kernel requests before it knows the row's length

// EARLY (stage2_kernel): the lane's first log-sum-exp of the maximum sweep and its first
// kMergeEarly rounds of (log-sum-exp, partial) were requested by the caller for every split
// that exists, before the row's length was known -- one memory round trip instead of three
// dependent ones; what lies past `nblk` is ignored here.  Same arithmetic in the same order.
struct MergeEarly {
  float m0;
  float lse[kMergeEarly];
  float4 o[kMergeEarly];
};

template <int D, bool COHERENT = false, bool EARLY = false>
__device__ __forceinline__ void merge_splits(const float* mo, const float* ml, int nblk, void* __restrict__ out,
                                             int out_dtype, int64_t out_off, const MergeEarly* early = nullptr) {
  constexpr int LPD = D / 4;                    // lanes across the head dimension
  constexpr int NG = kMergeThreads / LPD;       // splits handled side by side
  constexpr int kW = kMergeThreads / SOCKET_WAVE;
  __shared__ float red[kW];
  __shared__ float part[NG][D + 4];
  __shared__ float psum[NG];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;

  float m = -INFINITY;
  if (EARLY) {
    if (tid < nblk) m = fmaxf(m, early->m0);
    for (int s = tid + kMergeThreads; s < nblk; s += kMergeThreads) m = fmaxf(m, ml[s]);
  } else {
    for (int s = tid; s < nblk; s += kMergeThreads) m = fmaxf(m, COHERENT ? load_coherent(ml + s) : ml[s]);
  }
  m = wave_reduce_to_last<true>(m);
  if (lane == 63) red[wave] = m;
  __syncthreads();
  m = red[0];
#pragma unroll
  for (int w = 1; w < kW; ++w) m = fmaxf(m, red[w]);

  const int grp = tid / LPD, d4 = (tid % LPD) * 4;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  float sum = 0.f;
  // (a split without a live row has lse = -inf and weight 0; so has every split
  // when nothing at all was attended (m = -inf), which leaves 0/0 below)
  auto add = [&](float lse, const float4& o) __attribute__((always_inline)) {
    const float w = (lse == -INFINITY) ? 0.f : fast_exp(lse - m);
    acc.x += w * o.x;
    acc.y += w * o.y;
    acc.z += w * o.z;
    acc.w += w * o.w;
    sum += w;
  };
  int s = grp;
  if (EARLY) {
#pragma unroll
    for (int it = 0; it < kMergeEarly; ++it, s += NG)
      if (s < nblk) add(early->lse[it], early->o[it]);
  }
  for (; s < nblk; s += NG) {
    const float lse = COHERENT ? load_coherent(ml + s) : ml[s];
    float4 o;
    if (COHERENT) {
      const float* src = mo + (int64_t)s * D + d4;
      o = make_float4(load_coherent(src), load_coherent(src + 1), load_coherent(src + 2), load_coherent(src + 3));
    } else {
      o = *reinterpret_cast<const float4*>(mo + (int64_t)s * D + d4);
    }
    add(lse, o);
  }
  part[grp][d4] = acc.x;
  part[grp][d4 + 1] = acc.y;
  part[grp][d4 + 2] = acc.z;
  part[grp][d4 + 3] = acc.w;
  if (d4 == 0) psum[grp] = sum;
  __syncthreads();
  if (tid < D) {
    float a = 0.f, t = 0.f;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      a += part[g][tid];
      t += psum[g];
    }
    const float r = a / t;  // 0/0 -> NaN when nothing was attended, as the reference
    const int64_t o = out_off + tid;
    if (out_dtype == SOCKET_F32) store_elem<DType_f32>(out, o, r);
    else if (out_dtype == SOCKET_BF16) store_elem<DType_bf16>(out, o, r);
    else store_elem<DType_f16>(out, o, r);
  }
}

// One workgroup per (b, h): the merge as a launch of its own.
template <int D>
__global__ __launch_bounds__(kMergeThreads) void stage2_kernel(
    const float* __restrict__ mid_o, const float* __restrict__ mid_lse,
    const int32_t* __restrict__ sparse_len, int64_t len_sb, int64_t len_sh, void* __restrict__ out,
    int out_dtype, int64_t out_sb, int64_t out_sh, int Hq, int nsplit, int block_seq) {
  const int h = blockIdx.x, b = blockIdx.y;
  const float* mo = mid_o + ((int64_t)b * Hq + h) * nsplit * D;
  const float* ml = mid_lse + ((int64_t)b * Hq + h) * nsplit;
  // the partials of every split that exists are requested together with the length (those past the
  // row's length hold whatever the workspace held and are ignored)
  constexpr int LPD = D / 4, NG = kMergeThreads / LPD;
  const int tid = threadIdx.x, grp = tid / LPD, d4 = (tid % LPD) * 4;
  const int len = sparse_len[b * len_sb + h * len_sh];   // (a scalar load: on its way while the rest is requested)
  MergeEarly early;
  early.m0 = ml[min(tid, nsplit - 1)];   // (unconditional: a load under a condition is waited for on the spot)
#pragma unroll
  for (int it = 0; it < kMergeEarly; ++it) {
    const int s = min(grp + it * NG, nsplit - 1);
    early.lse[it] = ml[s];
    early.o[it] = *reinterpret_cast<const float4*>(mo + (int64_t)s * D + d4);
  }
  // (a length beyond nsplit * block_seq is cut to the splits that exist)
  int nblk = len <= 0 ? 0 : (len + block_seq - 1) / block_seq;
  nblk = min(nblk, nsplit);
  merge_splits<D, false, true>(mo, ml, nblk, out, out_dtype, b * out_sb + h * out_sh, &early);
}

// FINISH: the workgroup that completes a row's last outstanding split also merges
// the splits (what stage2_kernel does), so the whole attention is one launch.
// `arrive` holds one counter per row that is zero between launches: every split
// with work takes a ticket with a wrapping increment after publishing its partial
// result, the one that draws the last ticket finds the counter back at zero and
// every other split's result visible.
struct Stage1Finish {
  unsigned int* arrive;
  void* out;
  int out_dtype;
  int64_t out_sb, out_sh;
};

template <class DT, int D, bool FINISH>
__global__ __launch_bounds__(kAttThreads) void sparse_stage1_kernel(
    const void* __restrict__ q_, const void* __restrict__ k_, const void* __restrict__ v_,
    int64_t q_sb, int64_t q_sh, int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb,
    int64_t v_sh, int64_t v_ss, const int32_t* __restrict__ sparse_list, int64_t list_sb,
    int64_t list_sh, const int32_t* __restrict__ sparse_len, int64_t len_sb, int64_t len_sh,
    float* __restrict__ mid_o, float* __restrict__ mid_lse, int Hq, int G, int kv_rows, int list_width,
    int nsplit, int block_seq, float sm_scale, Stage1Finish fin) {
  typedef typename DT::storage ST;
  constexpr int E = DT::kPer16B;
  constexpr int LPR = D / E;
  constexpr int RPW = SOCKET_WAVE / LPR;
  __shared__ float lds[kAttWaves * (D + 2)];

  const int s = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  // a length beyond the list row's width would read the next row's entries
  const int len = min(sparse_len[b * len_sb + h * len_sh], list_width);
  const int lo = s * block_seq;
  const int hi = min(len, lo + block_seq);
  if (FINISH && s == 0 && len <= 0) {
    // nothing listed: no split runs for this row; the reference's 0/0
    if (threadIdx.x < D) {
      const int64_t o = b * fin.out_sb + h * fin.out_sh + threadIdx.x;
      const float nan = __uint_as_float(0x7fc00000u);
      if (fin.out_dtype == SOCKET_F32) store_elem<DType_f32>(fin.out, o, nan);
      else if (fin.out_dtype == SOCKET_BF16) store_elem<DType_bf16>(fin.out, o, nan);
      else store_elem<DType_f16>(fin.out, o, nan);
    }
    return;
  }
  if (hi <= lo) return;
  const int kvh = h / G;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slot = lane / LPR, chunk = lane % LPR;

  const ST* q = (const ST*)q_ + b * q_sb + h * q_sh;
  const ST* kbase = (const ST*)k_ + b * k_sb + kvh * k_sh;
  const ST* vbase = (const ST*)v_ + b * v_sb + kvh * v_sh;
  const int32_t* list = sparse_list + b * list_sb + h * list_sh;

  float qf[E];
  unpack16<DT>(*reinterpret_cast<const uint4*>(q + chunk * E), qf);

  float m[1] = {-INFINITY}, l[1] = {0.f}, acc[1][E];
#pragma unroll
  for (int i = 0; i < E; ++i) acc[0][i] = 0.f;

  constexpr int STEP = kAttWaves * RPW * kUnroll;  // list entries per workgroup iteration
  for (int e0 = lo; e0 < hi; e0 += STEP) {
    int idx[kUnroll];
    bool live[kUnroll];
    uint4 kr[kUnroll], vr[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int e = e0 + (u * kAttWaves + wave) * RPW + slot;
      idx[u] = (e < hi) ? list[e] : -1;
      live[u] = idx[u] >= 0 && idx[u] < kv_rows;
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (live[u]) {
        kr[u] = *reinterpret_cast<const uint4*>(kbase + (int64_t)idx[u] * k_ss + chunk * E);
        vr[u] = *reinterpret_cast<const uint4*>(vbase + (int64_t)idx[u] * v_ss + chunk * E);
      } else {
        kr[u] = make_uint4(0, 0, 0, 0);
        vr[u] = make_uint4(0, 0, 0, 0);
      }
    }
    float sc[kUnroll];
    float nm = m[0];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float kf[E];
      unpack16<DT>(kr[u], kf);
      float d = 0.f;
#pragma unroll
      for (int i = 0; i < E; ++i) d += qf[i] * kf[i];
      d = group_sum<LPR>(d);
      sc[u] = live[u] ? d * sm_scale : -INFINITY;
      nm = fmaxf(nm, sc[u]);
    }
    const float rescale = (m[0] == nm) ? 1.f : fast_exp(m[0] - nm);
    l[0] *= rescale;
#pragma unroll
    for (int i = 0; i < E; ++i) acc[0][i] *= rescale;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const float p = live[u] ? fast_exp(sc[u] - nm) : 0.f;
      float vf[E];
      unpack16<DT>(vr[u], vf);
      l[0] += p;
#pragma unroll
      for (int i = 0; i < E; ++i) acc[0][i] += p * vf[i];
    }
    m[0] = nm;
  }

  float* mo = mid_o + (((int64_t)b * Hq + h) * nsplit + s) * D;
  float* ml = mid_lse + ((int64_t)b * Hq + h) * nsplit + s;
  finish_split<E, LPR, 1, FINISH>(m, l, acc, 1, mo, ml, 0, 0, lds);
  if (FINISH) {
    __shared__ int last;
    const int nblk = min((len + block_seq - 1) / block_seq, nsplit);   // splits of this row that run
    // Every lane waits until its written-through stores of the partial result have been
    // acknowledged, the barrier collects the lanes, and only then is the ticket drawn
    // (an atomic at the same, device-wide, level): whoever draws a later ticket can read
    // this split's result.  No fence: see store_coherent.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (tid == 0) last = draw_ticket(&fin.arrive[b * Hq + h], (unsigned int)(nblk - 1)) == (unsigned int)(nblk - 1);
    __syncthreads();
    if (!last) return;
    merge_splits<D, true>(mid_o + ((int64_t)b * Hq + h) * nsplit * D, mid_lse + ((int64_t)b * Hq + h) * nsplit,
                          nblk, fin.out, fin.out_dtype, b * fin.out_sb + h * fin.out_sh);
  }
}

// Dense flash-decode: rows [s*rows_per_split, ...) of one kv head, all G heads
// of the group computed from a single read of each K and V row.
template <class DT, int D, int GP>
__global__ __launch_bounds__(kAttThreads) void dense_stage1_kernel(
    const void* __restrict__ q_, const void* __restrict__ k_, const void* __restrict__ v_,
    int64_t q_sb, int64_t q_sh, int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb,
    int64_t v_sh, int64_t v_ss, const int32_t* __restrict__ lens, float* __restrict__ mid_o,
    float* __restrict__ mid_lse, int Hq, int Hkv, int G, int T, int nsplit, int rows_per_split,
    float sm_scale) {
  typedef typename DT::storage ST;
  constexpr int E = DT::kPer16B;
  constexpr int LPR = D / E;
  constexpr int RPW = SOCKET_WAVE / LPR;
  __shared__ float lds[kAttWaves * GP * (D + 2)];

  const int s = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int len = lens ? min(lens[b], T) : T;
  const int lo = s * rows_per_split;
  const int hi = min(len, lo + rows_per_split);
  if (hi <= lo) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slot = lane / LPR, chunk = lane % LPR;
  const ST* kbase = (const ST*)k_ + b * k_sb + kvh * k_sh;
  const ST* vbase = (const ST*)v_ + b * v_sb + kvh * v_sh;

  float qf[GP][E];
#pragma unroll
  for (int g = 0; g < GP; ++g) {
    if (g < G) {
      const ST* q = (const ST*)q_ + b * q_sb + (kvh * G + g) * q_sh;
      unpack16<DT>(*reinterpret_cast<const uint4*>(q + chunk * E), qf[g]);
    } else {
#pragma unroll
      for (int i = 0; i < E; ++i) qf[g][i] = 0.f;
    }
  }
  float m[GP], l[GP], acc[GP][E];
#pragma unroll
  for (int g = 0; g < GP; ++g) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int i = 0; i < E; ++i) acc[g][i] = 0.f;
  }

  constexpr int STEP = kAttWaves * RPW * kUnroll;
  for (int e0 = lo; e0 < hi; e0 += STEP) {
    bool live[kUnroll];
    uint4 kr[kUnroll], vr[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int e = e0 + (u * kAttWaves + wave) * RPW + slot;
      live[u] = e < hi;
      if (live[u]) {
        kr[u] = *reinterpret_cast<const uint4*>(kbase + (int64_t)e * k_ss + chunk * E);
        vr[u] = *reinterpret_cast<const uint4*>(vbase + (int64_t)e * v_ss + chunk * E);
      } else {
        kr[u] = make_uint4(0, 0, 0, 0);
        vr[u] = make_uint4(0, 0, 0, 0);
      }
    }
    float sc[kUnroll][GP];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float kf[E];
      unpack16<DT>(kr[u], kf);
#pragma unroll
      for (int g = 0; g < GP; ++g) {
        float d = 0.f;
#pragma unroll
        for (int i = 0; i < E; ++i) d += qf[g][i] * kf[i];
        d = group_sum<LPR>(d);
        sc[u][g] = live[u] ? d * sm_scale : -INFINITY;
      }
    }
#pragma unroll
    for (int g = 0; g < GP; ++g) {
      float nm = m[g];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) nm = fmaxf(nm, sc[u][g]);
      const float rescale = (m[g] == nm) ? 1.f : fast_exp(m[g] - nm);
      l[g] *= rescale;
#pragma unroll
      for (int i = 0; i < E; ++i) acc[g][i] *= rescale;
      m[g] = nm;
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float vf[E];
      unpack16<DT>(vr[u], vf);
#pragma unroll
      for (int g = 0; g < GP; ++g) {
        const float p = live[u] ? fast_exp(sc[u][g] - m[g]) : 0.f;
        l[g] += p;
#pragma unroll
        for (int i = 0; i < E; ++i) acc[g][i] += p * vf[i];
      }
    }
  }

  const int h0 = kvh * G;
  float* mo = mid_o + (((int64_t)b * Hq + h0) * nsplit + s) * D;
  float* ml = mid_lse + ((int64_t)b * Hq + h0) * nsplit + s;
  finish_split<E, LPR, GP>(m, l, acc, G, mo, ml, (int64_t)nsplit * D, (int64_t)nsplit, lds);
}

// ---------------------------------------------------------------------------
// Dense flash-decode on the matrix cores: 16-bit K/V, D = 128, up to 16 query
// heads per kv head.
//
// The lane-per-row kernel above spends, per K/V row, G dot products of 128 terms,
// their cross-lane sums and G x 128 multiply-adds on the vector ALU; from four
// heads per kv head on, that -- not the K/V stream -- is what bounds it (0.63 of
// the HBM peak at G = 4, 0.25 at G = 7).  Here both products are MFMAs in the transposed orientation, with the query head as
// the N index (lane x holds head x % 16 in every accumulator, heads past G are
// zero columns):
//   S^T[key, head] = K . Q^T      v_mfma_f32_16x16x32   A = 16 keys x 32 dims
//   O^T[dim, head] = V^T . P^T    v_mfma_f32_16x16x16   A = 16 dims x 16 keys
// so a head's running maximum and sum are over a lane's own registers and the
// three other lane quarters, the rescale factor is per lane, and the
// probabilities a lane computed (keys 4q..4q+3 of the block, q = lane / 16) are
// the B operand it has to supply for those keys.
//
// A wave walks its own 16-key blocks (blocks wave, wave + 4, ... of the split);
// K and V rows go global -> LDS directly, 1 KB (four whole rows) per
// instruction, into the wave's private ring of STAGES blocks, so no barrier sits
// in the loop and STAGES - 1 blocks per wave are in flight while one is
// consumed.  The lane that copies 16-byte piece c of row r writes it to position
// c ^ r of the row's 16 places: the K fragment reads (16 rows, same piece) and
// the V reads (dwords of 4 rows x 16 neighbouring pieces) then hit 64 different
// banks.  V^T is never materialised: a dword of V holds dims 2x and 2x + 1 of one
// key, four such dwords (keys 4q..4q+3) split into their low and high halves are
// the A operands of the two 16-dim blocks {2x + 32p} and {2x + 1 + 32p}, x < 16.
// ---------------------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 att_bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 att_f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 att_f16x4;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short att_s16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float att_f32x4;

template <class DT>
struct MmaType;
template <>
struct MmaType<DType_bf16> {
  static __device__ __forceinline__ att_f32x4 qk(const uint4& a, const uint4& b, att_f32x4 c) {
    union {
      uint4 u;
      att_bf16x8 v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x.v, y.v, c, 0, 0, 0);
  }
  static __device__ __forceinline__ att_f32x4 pv(const uint2& a, const uint2& b, att_f32x4 c) {
    union {
      uint2 u;
      att_s16x4 v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(x.v, y.v, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    union {
      bf2 v;
      uint32_t u;
    } r;
    r.v = __builtin_convertvector(f2{lo, hi}, bf2);
    return r.u;
  }
};
template <>
struct MmaType<DType_f16> {
  static __device__ __forceinline__ att_f32x4 qk(const uint4& a, const uint4& b, att_f32x4 c) {
    union {
      uint4 u;
      att_f16x8 v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(x.v, y.v, c, 0, 0, 0);
  }
  static __device__ __forceinline__ att_f32x4 pv(const uint2& a, const uint2& b, att_f32x4 c) {
    union {
      uint2 u;
      att_f16x4 v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_16x16x16f16(x.v, y.v, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    union {
      h2 v;
      uint32_t u;
    } r;
    r.v = __builtin_convertvector(f2{lo, hi}, h2);
    return r.u;
  }
};

constexpr int kMmaKeys = 16;                            // keys per block of a wave
constexpr int kMmaTileBytes = kMmaKeys * 128 * 2;       // one K or V tile
constexpr int kMmaStageBytes = 2 * kMmaTileBytes;
constexpr int kMmaHeads = 16;
constexpr int kMmaMaxFlatBatch = SOCKET_WAVE;           // sequences one wave can scan

// s_waitcnt vmcnt(N), also a compiler barrier for the LDS reads that follow
template <int N>
__device__ __forceinline__ void wait_copies() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Grid: one workgroup per (kv head, sequence, split), flattened.  With `flat`
// (B <= 64) the splits that exist -- ceil(len_b / rows_per_split) per sequence --
// are numbered consecutively from the lengths, so a ragged batch occupies the
// first sum-of-splits workgroups and the rest of the grid (sized for the longest
// possible sequence, the lengths live on the device) exits at once; otherwise the
// grid is the rectangle B x nsplit.
template <class DT, int STAGES>
__global__ __launch_bounds__(kAttThreads) void dense_mma_kernel(
    const uint16_t* __restrict__ q_, const uint16_t* __restrict__ k_, const uint16_t* __restrict__ v_,
    int64_t q_sb, int64_t q_sh, int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh,
    int64_t v_ss, const int32_t* __restrict__ lens, float* __restrict__ mid_o, float* __restrict__ mid_lse,
    int B, int Hq, int Hkv, int G, int T, int nsplit, int rows_per_split, float scale_log2, int flat) {
  constexpr int D = 128;
  extern __shared__ __attribute__((aligned(16))) unsigned char att_lds[];
  __shared__ int item[3];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int prow = lane & 15, quarter = lane >> 4;

  const int kvh = blockIdx.x % Hkv;
  const int t = blockIdx.x / Hkv;
  int b, s;
  if (flat) {
    if (wave == 0) {
      const int n = lane < B ? (max(0, min(lens[lane], T)) + rows_per_split - 1) / rows_per_split : 0;
      const int incl = wave_incl_scan(n);
      if (t >= incl - n && t < incl) {
        item[0] = lane;
        item[1] = t - (incl - n);
      }
      if (lane == SOCKET_WAVE - 1) item[2] = incl;
    }
    __syncthreads();
    if (t >= item[2]) return;
    b = item[0];
    s = item[1];
  } else {
    b = t / nsplit;
    s = t % nsplit;
  }
  const int len = min(lens[b], T);
  const int lo = s * rows_per_split;
  const int hi = min(len, lo + rows_per_split);
  if (hi <= lo) return;

  const uint16_t* kbase = k_ + b * k_sb + kvh * k_sh;
  const uint16_t* vbase = v_ + b * v_sb + kvh * v_sh;
  // Q^T fragments (B operand): head prow, dims 32 ks + 8 quarter .. + 7
  uint4 qf[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) qf[ks] = make_uint4(0, 0, 0, 0);
  if (prow < G) {
    const uint16_t* q = q_ + b * q_sb + (int64_t)(kvh * G + prow) * q_sh;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) qf[ks] = *reinterpret_cast<const uint4*>(q + (4 * ks + quarter) * 8);
  }

  // The fragments must have arrived before the first copy is issued: the compiler
  // counts the loads it knows of, not the LDS copies below, and would otherwise
  // wait for "its" loads inside the loop with a count that drains every copy in
  // flight, on every trip.
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) asm volatile("" ::"v"(qf[ks].x), "v"(qf[ks].y), "v"(qf[ks].z), "v"(qf[ks].w));

  unsigned char* ring = att_lds + wave * STAGES * kMmaStageBytes;
  const int nblk = (hi - lo + kMmaKeys - 1) / kMmaKeys;
  const int mine = nblk > wave ? (nblk - wave + kAttWaves - 1) / kAttWaves : 0;
  // Block j of this wave into a ring stage.  Rows past the split's end are fetched
  // from its last row (a live row, so the copy count per block is constant and
  // nothing outside the split is touched); their scores are masked below.
  // The walk starts at a block that differs from workgroup to workgroup and wraps
  // (the softmax does not care about order): splits are a power-of-two number of
  // bytes apart in a cache whose length is a power of two, and workgroups that
  // start together would otherwise sweep the same few memory channels in step.
  const int rot = (int)((blockIdx.x * 2654435761u) >> 8) % nblk;
  auto block_of = [&](int j) {
    const int i = wave + kAttWaves * j + rot;
    return i >= nblk ? i - nblk : i;
  };
  auto fetch = [&](int j, int stage) {
    const int key0 = lo + (j < mine ? block_of(j) : nblk) * kMmaKeys;
    unsigned char* dst = ring + stage * kMmaStageBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = 4 * i + quarter;
      const int key = min(key0 + r, hi - 1);
      const int piece = prow ^ r;
      lds_dma16_stream(kbase + (int64_t)key * k_ss + piece * 8, dst + i * 1024);
      lds_dma16_stream(vbase + (int64_t)key * v_ss + piece * 8, dst + kMmaTileBytes + i * 1024);
    }
  };

  float m_i = -INFINITY, l_part = 0.f;
  att_f32x4 o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = att_f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int j = 0; j < STAGES - 1; ++j) fetch(j, j);
  for (int j = 0; j < mine; ++j) {
    fetch(j + STAGES - 1, (j + STAGES - 1) % STAGES);
    wait_copies<(STAGES - 1) * 8>();
    const unsigned char* st = ring + (j % STAGES) * kMmaStageBytes;
    const uint4* kt = reinterpret_cast<const uint4*>(st);
    const uint32_t* vt = reinterpret_cast<const uint32_t*>(st + kMmaTileBytes);

    // ---- S^T: register i = key 4 quarter + i of the block against head prow
    att_f32x4 sc = att_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) sc = MmaType<DT>::qk(kt[prow * 16 + ((4 * ks + quarter) ^ prow)], qf[ks], sc);
    const int key0 = lo + block_of(j) * kMmaKeys + 4 * quarter;
    float m_blk = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sc[i] = (key0 + i < hi) ? sc[i] : -INFINITY;
      m_blk = fmaxf(m_blk, sc[i]);
    }
    m_blk = fmaxf(m_blk, lane_xor16(m_blk));   // (lane swaps on the vector ALU, not the LDS crossbar)
    m_blk = fmaxf(m_blk, lane_xor32(m_blk));
    // The maximum is kept on the raw dot products and the (positive) scale applied
    // to the difference, in base 2: the largest score of a block then gives exactly
    // exp2(0) whatever its magnitude, which scaling first and subtracting the rounded
    // maximum afterwards does not guarantee.
    const float m_new = fmaxf(m_i, m_blk);
    const bool blind = m_new == -INFINITY;
    const float alpha = blind ? 1.f : __builtin_amdgcn_exp2f((m_i - m_new) * scale_log2);
    const float ref = blind ? 0.f : m_new;
    float p[4], psum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = __builtin_amdgcn_exp2f((sc[i] - ref) * scale_log2);
      psum += p[i];
    }
    l_part = l_part * alpha + psum;
    m_i = m_new;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        o[i][0] *= alpha;
        o[i][1] *= alpha;
        o[i][2] *= alpha;
        o[i][3] *= alpha;
      }
    }
    // ---- O^T += V^T . P^T
    const uint2 pf = make_uint2(MmaType<DT>::pack2(p[0], p[1]), MmaType<DT>::pack2(p[2], p[3]));
#pragma unroll
    for (int pp = 0; pp < 4; ++pp) {
      uint32_t w[4];
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        const int r = 4 * quarter + jj;
        w[jj] = vt[r * 64 + (((4 * pp + (prow >> 2)) ^ r) << 2) + (prow & 3)];
      }
      const uint2 lo2 = make_uint2(__builtin_amdgcn_perm(w[1], w[0], 0x05040100u),
                                   __builtin_amdgcn_perm(w[3], w[2], 0x05040100u));
      const uint2 hi2 = make_uint2(__builtin_amdgcn_perm(w[1], w[0], 0x07060302u),
                                   __builtin_amdgcn_perm(w[3], w[2], 0x07060302u));
      o[2 * pp] = MmaType<DT>::pv(lo2, pf, o[2 * pp]);
      o[2 * pp + 1] = MmaType<DT>::pv(hi2, pf, o[2 * pp + 1]);
    }
  }

  // the copies still under way (fetched past the wave's last block) must land
  // before the ring is reused for the waves' records
  wait_copies<0>();
  float l = l_part;
  l += lane_xor16(l);
  l += lane_xor32(l);
  __syncthreads();
  constexpr int REC = D + 2;
  float* lds = reinterpret_cast<float*>(att_lds);
  if (prow < G) {
    float* rec = lds + (wave * kMmaHeads + prow) * REC;
    // register i of accumulator 2 pp + e: dim 8 quarter + 2 i + 32 pp + e
#pragma unroll
    for (int pp = 0; pp < 4; ++pp)
#pragma unroll
      for (int e = 0; e < 2; ++e)
#pragma unroll
        for (int i = 0; i < 4; ++i) rec[8 * quarter + 2 * i + 32 * pp + e] = o[2 * pp + e][i];
    if (quarter == 0) {
      rec[D] = m_i * (scale_log2 * 0.6931471805599453f);   // the records hold scaled scores, natural base
      rec[D + 1] = l;
    }
  }
  __syncthreads();
  const int h0 = kvh * G;
  combine_waves<D, kMmaHeads, false>(lds, G, mid_o + (((int64_t)b * Hq + h0) * nsplit + s) * D,
                                     mid_lse + ((int64_t)b * Hq + h0) * nsplit + s, (int64_t)nsplit * D,
                                     (int64_t)nsplit);
}

struct AttArgs {
  const void *q, *k, *v;
  int dtype;
  int64_t q_sb, q_sh, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss;
};

int check_common(const AttArgs& a, int B, int Hq, int Hkv, int D) {
  SOCKET_REQUIRE(a.q && a.k && a.v, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(B <= 65535 && Hq <= 65535, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(D == 16 || D == 32 || D == 64 || D == 128, SOCKET_ERR_UNSUPPORTED);
  const int eb = socket_dtype_bytes(a.dtype);
  SOCKET_REQUIRE(eb != 0, SOCKET_ERR_UNSUPPORTED);
  // every row start must be 16-byte aligned
  const int per16 = 16 / eb;
  SOCKET_REQUIRE(socket_aligned16(a.q) && socket_aligned16(a.k) && socket_aligned16(a.v),
                 SOCKET_ERR_ALIGN);
  SOCKET_REQUIRE(a.q_sb % per16 == 0 && a.q_sh % per16 == 0 && a.k_sb % per16 == 0 &&
                     a.k_sh % per16 == 0 && a.k_ss % per16 == 0 && a.v_sb % per16 == 0 &&
                     a.v_sh % per16 == 0 && a.v_ss % per16 == 0,
                 SOCKET_ERR_ALIGN);
  return SOCKET_OK;
}

template <class DT, int D>
void launch_sparse_stage1(const AttArgs& a, const int32_t* list, int64_t list_sb, int64_t list_sh,
                          const int32_t* len, int64_t len_sb, int64_t len_sh, float* mid_o,
                          float* mid_lse, int B, int Hq, int Hkv, int kv_rows, int list_width,
                          int nsplit, int block_seq, const Stage1Finish* fin, hipStream_t s) {
#define SOCKET_S1_ARGS                                                                               \
  a.q, a.k, a.v, a.q_sb, a.q_sh, a.k_sb, a.k_sh, a.k_ss, a.v_sb, a.v_sh, a.v_ss, list, list_sb, list_sh, \
      len, len_sb, len_sh, mid_o, mid_lse, Hq, Hq / Hkv, kv_rows, list_width, nsplit, block_seq,      \
      1.0f / sqrtf((float)D)
  if (fin)
    hipLaunchKernelGGL((sparse_stage1_kernel<DT, D, true>), dim3(nsplit, Hq, B), dim3(kAttThreads), 0, s,
                       SOCKET_S1_ARGS, *fin);
  else
    hipLaunchKernelGGL((sparse_stage1_kernel<DT, D, false>), dim3(nsplit, Hq, B), dim3(kAttThreads), 0, s,
                       SOCKET_S1_ARGS, Stage1Finish{});
#undef SOCKET_S1_ARGS
}

template <class DT, int D>
int launch_dense_stage1(const AttArgs& a, const int32_t* lens, float* mid_o, float* mid_lse, int B,
                        int Hq, int Hkv, int T, int nsplit, int rows_per_split, hipStream_t s) {
  const int G = Hq / Hkv;
  const float sc = 1.0f / sqrtf((float)D);
  dim3 grid(nsplit, Hkv, B), block(kAttThreads);
#define SOCKET_DENSE_ARGS                                                                        \
  a.q, a.k, a.v, a.q_sb, a.q_sh, a.k_sb, a.k_sh, a.k_ss, a.v_sb, a.v_sh, a.v_ss, lens, mid_o,    \
      mid_lse, Hq, Hkv, G, T, nsplit, rows_per_split, sc
  if (G == 1) hipLaunchKernelGGL((dense_stage1_kernel<DT, D, 1>), grid, block, 0, s, SOCKET_DENSE_ARGS);
  else if (G == 2) hipLaunchKernelGGL((dense_stage1_kernel<DT, D, 2>), grid, block, 0, s, SOCKET_DENSE_ARGS);
  else if (G <= 4) hipLaunchKernelGGL((dense_stage1_kernel<DT, D, 4>), grid, block, 0, s, SOCKET_DENSE_ARGS);
  else if (G <= 8) hipLaunchKernelGGL((dense_stage1_kernel<DT, D, 8>), grid, block, 0, s, SOCKET_DENSE_ARGS);
  else return SOCKET_ERR_UNSUPPORTED;
#undef SOCKET_DENSE_ARGS
  return SOCKET_OK;
}

// Two ring stages per wave (64 KB per workgroup, two workgroups per CU) and splits
// of at least 1024 rows measured best from one sequence of 32k rows to 16 ragged
// ones; deeper rings (one workgroup per CU) lose at batch 1 and gain nothing at
// the large shapes.  Measured at 5.4-5.9 TB/s for 1 to 8 heads per kv head, which
// is above the lane-per-row kernel at every group size, so every 16-bit D = 128
// cache takes this path.
constexpr int kMmaStages = 2;
constexpr int kMmaMinRows = 1024;

bool dense_uses_mma(int dtype, int D, int G) {
  return (dtype == SOCKET_BF16 || dtype == SOCKET_F16) && D == 128 && G <= kMmaHeads;
}

template <class DT>
int launch_dense_mma(const AttArgs& a, const int32_t* lens, float* mid_o, float* mid_lse, int B, int Hq,
                     int Hkv, int T, int nsplit, int rows_per_split, hipStream_t s) {
  auto kern = dense_mma_kernel<DT, kMmaStages>;
  constexpr size_t ring = (size_t)kAttWaves * kMmaStages * kMmaStageBytes;
  constexpr size_t records = (size_t)kAttWaves * kMmaHeads * (128 + 2) * sizeof(float);
  constexpr size_t lds = ring > records ? ring : records;
  static std::atomic<bool> ready{false};
  if (!ready.load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds) != hipSuccess)
      return SOCKET_ERR_LAUNCH;
    ready.store(true, std::memory_order_release);
  }
  SOCKET_REQUIRE((int64_t)B * nsplit * Hkv < (int64_t)1 << 31, SOCKET_ERR_SHAPE);
  const float scale_log2 = 1.4426950408889634f / sqrtf(128.f);
  hipLaunchKernelGGL(kern, dim3((unsigned)(B * nsplit * Hkv)), dim3(kAttThreads), lds, s, (const uint16_t*)a.q,
                     (const uint16_t*)a.k, (const uint16_t*)a.v, a.q_sb, a.q_sh, a.k_sb, a.k_sh, a.k_ss, a.v_sb,
                     a.v_sh, a.v_ss, lens, mid_o, mid_lse, B, Hq, Hkv, Hq / Hkv, T, nsplit, rows_per_split,
                     scale_log2, B <= kMmaMaxFlatBatch ? 1 : 0);
  return SOCKET_OK;
}

int launch_stage2(const float* mid_o, const float* mid_lse, const int32_t* len, int64_t len_sb,
                  int64_t len_sh, void* out, int out_dtype, int64_t out_sb, int64_t out_sh, int B,
                  int Hq, int D, int nsplit, int block_seq, hipStream_t s) {
  SOCKET_REQUIRE(socket_aligned16(mid_o), SOCKET_ERR_ALIGN);
#define SOCKET_S2(DD)                                                                              \
  hipLaunchKernelGGL((stage2_kernel<DD>), dim3(Hq, B), dim3(kMergeThreads), 0, s, mid_o, mid_lse, len, len_sb, \
                     len_sh, out, out_dtype, out_sb, out_sh, Hq, nsplit, block_seq)
  if (D == 128) SOCKET_S2(128);
  else if (D == 64) SOCKET_S2(64);
  else if (D == 32) SOCKET_S2(32);
  else SOCKET_S2(16);
#undef SOCKET_S2
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

int dense_rows_per_split(int B, int Hkv, int T, int min_rows = 256) {
  // Aim at >= 8 workgroups per CU over the whole grid, splits of >= min_rows rows.
  const SocketDeviceLimits& lim = socket_device_limits();
  const int want = 8 * lim.cu_count;
  int nsplit = (want + B * Hkv - 1) / (B * Hkv);
  if (nsplit < 1) nsplit = 1;
  int rows = (T + nsplit - 1) / nsplit;
  rows = (rows + 63) / 64 * 64;
  if (rows < min_rows) rows = min_rows;
  return rows;
}

}  // namespace

namespace {

int attend_stage1(const void* q, const void* k, const void* v, int dtype, int64_t q_stride_b,
                  int64_t q_stride_h, int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                  int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s, const int32_t* sparse_list,
                  int64_t list_stride_b, int64_t list_stride_h, const int32_t* sparse_len,
                  int64_t len_stride_b, int64_t len_stride_h, float* mid_o, float* mid_lse, int B, int Hq,
                  int Hkv, int D, int kv_rows, int list_width, int nsplit, int block_seq,
                  const Stage1Finish* fin, void* stream) {
  AttArgs a{q, k, v, dtype, q_stride_b, q_stride_h, k_stride_b, k_stride_h, k_stride_s,
            v_stride_b, v_stride_h, v_stride_s};
  int st = check_common(a, B, Hq, Hkv, D);
  if (st != SOCKET_OK) return st;
  SOCKET_REQUIRE(sparse_list && sparse_len && mid_o && mid_lse, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(nsplit > 0 && nsplit <= 65535 * 32 && block_seq > 0 && kv_rows > 0 && list_width > 0,
                 SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(socket_aligned16(mid_o), SOCKET_ERR_ALIGN);
  hipStream_t s = (hipStream_t)stream;
#define SOCKET_S1(DT, DD)                                                                          \
  launch_sparse_stage1<DT, DD>(a, sparse_list, list_stride_b, list_stride_h, sparse_len,           \
                               len_stride_b, len_stride_h, mid_o, mid_lse, B, Hq, Hkv, kv_rows,    \
                               list_width, nsplit, block_seq, fin, s)
#define SOCKET_S1_D(DD)                                    \
  do {                                                     \
    if (dtype == SOCKET_BF16) SOCKET_S1(DType_bf16, DD);   \
    else if (dtype == SOCKET_F16) SOCKET_S1(DType_f16, DD); \
    else SOCKET_S1(DType_f32, DD);                         \
  } while (0)
  if (D == 128) SOCKET_S1_D(128);
  else if (D == 64) SOCKET_S1_D(64);
  else if (D == 32) SOCKET_S1_D(32);
  else SOCKET_S1_D(16);
#undef SOCKET_S1_D
#undef SOCKET_S1
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

}  // namespace

extern "C" int socket_attend_stage1(const void* q, const void* k, const void* v, int dtype,
                                    int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_b,
                                    int64_t k_stride_h, int64_t k_stride_s, int64_t v_stride_b,
                                    int64_t v_stride_h, int64_t v_stride_s,
                                    const int32_t* sparse_list, int64_t list_stride_b,
                                    int64_t list_stride_h, const int32_t* sparse_len,
                                    int64_t len_stride_b, int64_t len_stride_h, float* mid_o,
                                    float* mid_lse, int B, int Hq, int Hkv, int D, int kv_rows,
                                    int list_width, int nsplit, int block_seq, void* stream) {
  return attend_stage1(q, k, v, dtype, q_stride_b, q_stride_h, k_stride_b, k_stride_h, k_stride_s, v_stride_b,
                       v_stride_h, v_stride_s, sparse_list, list_stride_b, list_stride_h, sparse_len,
                       len_stride_b, len_stride_h, mid_o, mid_lse, B, Hq, Hkv, D, kv_rows, list_width, nsplit,
                       block_seq, nullptr, stream);
}

extern "C" int socket_attend_stage2(const float* mid_o, const float* mid_lse,
                                    const int32_t* sparse_len, int64_t len_stride_b,
                                    int64_t len_stride_h, void* out, int out_dtype,
                                    int64_t out_stride_b, int64_t out_stride_h, int B, int Hq, int D,
                                    int nsplit, int block_seq, void* stream) {
  SOCKET_REQUIRE(mid_o && mid_lse && sparse_len && out, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && nsplit > 0 && block_seq > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(B <= 65535, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(D == 16 || D == 32 || D == 64 || D == 128, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(socket_dtype_bytes(out_dtype) != 0, SOCKET_ERR_UNSUPPORTED);
  return launch_stage2(mid_o, mid_lse, sparse_len, len_stride_b, len_stride_h, out, out_dtype,
                       out_stride_b, out_stride_h, B, Hq, D, nsplit, block_seq, (hipStream_t)stream);
}

extern "C" int socket_sparse_attention_block_seq(int B, int Hq, int max_len) {
  if (B <= 0 || Hq <= 0 || max_len <= 0) return 64;
  // Aim at >= 4 workgroups per CU, in units of the 64 list entries a workgroup
  // consumes per iteration.
  const SocketDeviceLimits& lim = socket_device_limits();
  const int want = 4 * lim.cu_count;
  int nsplit = (want + B * Hq - 1) / (B * Hq);
  if (nsplit < 1) nsplit = 1;
  int bs = (max_len + nsplit - 1) / nsplit;
  bs = (bs + 63) / 64 * 64;
  if (bs < 64) bs = 64;
  // At most five iterations per workgroup: with many rows and lists of unequal length
  // (per-sequence budgets) long splits leave the launch waiting for the longest rows
  // (16 ragged sequences x 28 heads: 54 -> 49 us; batch 4 x 32 heads is at 320 already).
  if (bs > 320) bs = 320;
  return bs;
}

extern "C" size_t socket_sparse_attention_workspace_bytes(int B, int Hq, int D, int max_len) {
  if (B <= 0 || Hq <= 0 || D <= 0 || max_len <= 0) return 0;
  const int bs = socket_sparse_attention_block_seq(B, Hq, max_len);
  const size_t nsplit = (size_t)(max_len + bs - 1) / bs;
  return (size_t)B * Hq * nsplit * (D + 1) * sizeof(float);
}

namespace {

int sparse_attention_on(void* workspace, const void* q, const void* k, const void* v, int dtype,
                        int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_b, int64_t k_stride_h,
                        int64_t k_stride_s, int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s,
                        const int32_t* sparse_list, int64_t list_stride_b, int64_t list_stride_h,
                        const int32_t* sparse_len, int64_t len_stride_b, int64_t len_stride_h, void* out,
                        int64_t out_stride_b, int64_t out_stride_h, int B, int Hq, int Hkv, int D,
                        int kv_rows, int max_len, void* stream) {
  const int bs = socket_sparse_attention_block_seq(B, Hq, max_len);
  const int nsplit = (max_len + bs - 1) / bs;
  float* mid_o = (float*)workspace;
  float* mid_lse = mid_o + (size_t)B * Hq * nsplit * D;
  int st = socket_attend_stage1(q, k, v, dtype, q_stride_b, q_stride_h, k_stride_b, k_stride_h,
                                k_stride_s, v_stride_b, v_stride_h, v_stride_s, sparse_list,
                                list_stride_b, list_stride_h, sparse_len, len_stride_b, len_stride_h,
                                mid_o, mid_lse, B, Hq, Hkv, D, kv_rows, max_len, nsplit, bs, stream);
  if (st != SOCKET_OK) return st;
  return socket_attend_stage2(mid_o, mid_lse, sparse_len, len_stride_b, len_stride_h, out, dtype,
                              out_stride_b, out_stride_h, B, Hq, D, nsplit, bs, stream);
}

}  // namespace

extern "C" int socket_sparse_attention(const void* q, const void* k, const void* v, int dtype,
                                       int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_b,
                                       int64_t k_stride_h, int64_t k_stride_s, int64_t v_stride_b,
                                       int64_t v_stride_h, int64_t v_stride_s,
                                       const int32_t* sparse_list, int64_t list_stride_b,
                                       int64_t list_stride_h, const int32_t* sparse_len,
                                       int64_t len_stride_b, int64_t len_stride_h, void* out,
                                       int64_t out_stride_b, int64_t out_stride_h, void* workspace,
                                       size_t workspace_bytes, int B, int Hq, int Hkv, int D,
                                       int kv_rows, int max_len, void* stream) {
  SOCKET_REQUIRE(out && workspace, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(max_len > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(workspace_bytes >= socket_sparse_attention_workspace_bytes(B, Hq, D, max_len),
                 SOCKET_ERR_WORKSPACE);
  SOCKET_REQUIRE(socket_aligned16(workspace), SOCKET_ERR_ALIGN);
  return sparse_attention_on(workspace, q, k, v, dtype, q_stride_b, q_stride_h, k_stride_b, k_stride_h,
                             k_stride_s, v_stride_b, v_stride_h, v_stride_s, sparse_list, list_stride_b,
                             list_stride_h, sparse_len, len_stride_b, len_stride_h, out, out_stride_b,
                             out_stride_h, B, Hq, Hkv, D, kv_rows, max_len, stream);
}

// ---------------------------------------------------------------------------
// socket_sparse_attention for callers that cannot allocate: the per-split
// partials live in a fixed array in device memory that is part of the library's
// image.  Every GPU the library runs on holds its own copy until the process ends.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[SOCKET_STATIC_SCRATCH_BYTES];
// One arrival counter per (b, h) row for the launch that also merges the splits.
// Zero when the library is loaded and zero again after every call: the tickets are
// drawn with a wrapping increment, so the split that completes a row leaves its
// counter at zero.
constexpr int kArriveRows = 65536;
static __device__ unsigned int arrive_counters[kArriveRows];

namespace {

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];
std::atomic<void*> g_arrive_ptr[kMaxDevices];

// Device addresses of `scratch` and `arrive_counters` on the current device (the
// arrays' names are only host-side handles).  Looked up once per device; no allocation.
int static_scratch(void** out, unsigned int** arrive) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return SOCKET_ERR_LAUNCH;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  void* c = g_arrive_ptr[dev].load(std::memory_order_acquire);
  if (!p || !c) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return SOCKET_ERR_LAUNCH;
    if (hipGetSymbolAddress(&c, HIP_SYMBOL(arrive_counters)) != hipSuccess || !c) return SOCKET_ERR_LAUNCH;
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // every thread finds the same addresses
    g_arrive_ptr[dev].store(c, std::memory_order_release);
  }
  *out = p;
  *arrive = (unsigned int*)c;
  return SOCKET_OK;
}

}  // namespace

extern "C" size_t socket_static_scratch_bytes(void) { return (size_t)SOCKET_STATIC_SCRATCH_BYTES; }

extern "C" int socket_static_scratch_init(void) {
  void* p = nullptr;
  unsigned int* c = nullptr;
  return static_scratch(&p, &c);
}

extern "C" int socket_sparse_attention_static(const void* q, const void* k, const void* v, int dtype,
                                              int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_b,
                                              int64_t k_stride_h, int64_t k_stride_s, int64_t v_stride_b,
                                              int64_t v_stride_h, int64_t v_stride_s,
                                              const int32_t* sparse_list, int64_t list_stride_b,
                                              int64_t list_stride_h, const int32_t* sparse_len,
                                              int64_t len_stride_b, int64_t len_stride_h, void* out,
                                              int64_t out_stride_b, int64_t out_stride_h, int B, int Hq,
                                              int Hkv, int D, int kv_rows, int max_len, void* stream) {
  SOCKET_REQUIRE(out, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(max_len > 0 && B > 0 && Hq > 0 && D > 0, SOCKET_ERR_SHAPE);
  // the partials of this call must fit the fixed array, its rows the counters
  SOCKET_REQUIRE(socket_sparse_attention_workspace_bytes(B, Hq, D, max_len) <= (size_t)SOCKET_STATIC_SCRATCH_BYTES,
                 SOCKET_ERR_WORKSPACE);
  SOCKET_REQUIRE((int64_t)B * Hq <= kArriveRows, SOCKET_ERR_WORKSPACE);
  void* ws = nullptr;
  unsigned int* arrive = nullptr;
  const int st = static_scratch(&ws, &arrive);
  if (st != SOCKET_OK) return st;
  // Nothing in the partials array has to start at zero: a row's merge reads only the
  // splits the same launch wrote (the first ceil(len / split size) of the row).  One
  // launch: the workgroup that finishes a row's last split merges the row.
  const int bs = socket_sparse_attention_block_seq(B, Hq, max_len);
  const int nsplit = (max_len + bs - 1) / bs;
  float* mid_o = (float*)ws;
  float* mid_lse = mid_o + (size_t)B * Hq * nsplit * D;
  const Stage1Finish fin{arrive, out, dtype, out_stride_b, out_stride_h};
  return attend_stage1(q, k, v, dtype, q_stride_b, q_stride_h, k_stride_b, k_stride_h, k_stride_s, v_stride_b,
                       v_stride_h, v_stride_s, sparse_list, list_stride_b, list_stride_h, sparse_len,
                       len_stride_b, len_stride_h, mid_o, mid_lse, B, Hq, Hkv, D, kv_rows, max_len, nsplit, bs,
                       &fin, stream);
}

extern "C" size_t socket_dense_decode_workspace_bytes(int B, int Hq, int D, int T) {
  if (B <= 0 || Hq <= 0 || D <= 0 || T <= 0) return 0;
  // upper bound over every Hkv <= Hq: the split count is largest for Hkv == 1
  const int rows = dense_rows_per_split(B, 1, T);
  const size_t nsplit = (size_t)(T + rows - 1) / rows;
  return (size_t)B * Hq * nsplit * (D + 1) * sizeof(float) + (size_t)B * sizeof(int32_t) + 64;
}

extern "C" int socket_dense_decode(const void* q, const void* k, const void* v, int dtype,
                                   int64_t q_stride_b, int64_t q_stride_h, int64_t k_stride_b,
                                   int64_t k_stride_h, int64_t k_stride_s, int64_t v_stride_b,
                                   int64_t v_stride_h, int64_t v_stride_s, const int32_t* lens,
                                   void* out, int64_t out_stride_b, int64_t out_stride_h,
                                   void* workspace, size_t workspace_bytes, int B, int Hq, int Hkv,
                                   int D, int T, void* stream) {
  AttArgs a{q, k, v, dtype, q_stride_b, q_stride_h, k_stride_b, k_stride_h, k_stride_s,
            v_stride_b, v_stride_h, v_stride_s};
  int st = check_common(a, B, Hq, Hkv, D);
  if (st != SOCKET_OK) return st;
  SOCKET_REQUIRE(out && workspace, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(T > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(lens != nullptr, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(workspace_bytes >= socket_dense_decode_workspace_bytes(B, Hq, D, T),
                 SOCKET_ERR_WORKSPACE);
  SOCKET_REQUIRE(socket_aligned16(workspace), SOCKET_ERR_ALIGN);
  const bool mma = dense_uses_mma(dtype, D, Hq / Hkv);
  const int rows = dense_rows_per_split(B, Hkv, T, mma ? kMmaMinRows : 256);
  const int nsplit = (T + rows - 1) / rows;
  float* mid_o = (float*)workspace;
  float* mid_lse = mid_o + (size_t)B * Hq * nsplit * D;
  hipStream_t s = (hipStream_t)stream;
#define SOCKET_DENSE_D(DD)                                                                             \
  do {                                                                                                 \
    if (dtype == SOCKET_BF16) st = launch_dense_stage1<DType_bf16, DD>(a, lens, mid_o, mid_lse, B, Hq, Hkv, T, nsplit, rows, s); \
    else if (dtype == SOCKET_F16) st = launch_dense_stage1<DType_f16, DD>(a, lens, mid_o, mid_lse, B, Hq, Hkv, T, nsplit, rows, s); \
    else st = launch_dense_stage1<DType_f32, DD>(a, lens, mid_o, mid_lse, B, Hq, Hkv, T, nsplit, rows, s); \
  } while (0)
  if (mma)
    st = dtype == SOCKET_BF16 ? launch_dense_mma<DType_bf16>(a, lens, mid_o, mid_lse, B, Hq, Hkv, T, nsplit, rows, s)
                              : launch_dense_mma<DType_f16>(a, lens, mid_o, mid_lse, B, Hq, Hkv, T, nsplit, rows, s);
  else if (D == 128) SOCKET_DENSE_D(128);
  else if (D == 64) SOCKET_DENSE_D(64);
  else if (D == 32) SOCKET_DENSE_D(32);
  else SOCKET_DENSE_D(16);
#undef SOCKET_DENSE_D
  if (st != SOCKET_OK) return st;
  SOCKET_LAUNCH_CHECK();
  // per-batch lengths drive the merge: len_stride_h = 0
  return launch_stage2(mid_o, mid_lse, lens, 1, 0, out, dtype, out_stride_b, out_stride_h, B, Hq, D,
                       nsplit, rows, s);
}
