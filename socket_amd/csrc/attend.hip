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
      const float m2 = __shfl_xor(m[g], d, SOCKET_WAVE);
      const float l2 = __shfl_xor(l[g], d, SOCKET_WAVE);
      float a2[E];
#pragma unroll
      for (int i = 0; i < E; ++i) a2[i] = __shfl_xor(acc[g][i], d, SOCKET_WAVE);
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
  for (int o = tid; o < GH * D; o += kAttThreads) {
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

constexpr int kMergeThreads = 256;

// Merge of the per-split partials of one (b, h) by a workgroup of 256 lanes: the
// largest log-sum-exp first, then the lanes, four output coordinates each and
// 256 / (D/4) splits side by side, add up weight * partial with independent
// loads, and LDS folds the side-by-side groups.
template <int D, bool COHERENT = false>
__device__ __forceinline__ void merge_splits(const float* mo, const float* ml, int nblk, void* __restrict__ out,
                                             int out_dtype, int64_t out_off) {
  constexpr int LPD = D / 4;                    // lanes across the head dimension
  constexpr int NG = kMergeThreads / LPD;       // splits handled side by side
  constexpr int kW = kMergeThreads / SOCKET_WAVE;
  __shared__ float red[kW];
  __shared__ float part[NG][D + 4];
  __shared__ float psum[NG];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;

  float m = -INFINITY;
  for (int s = tid; s < nblk; s += kMergeThreads) m = fmaxf(m, COHERENT ? load_coherent(ml + s) : ml[s]);
#pragma unroll
  for (int d = SOCKET_WAVE / 2; d > 0; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, SOCKET_WAVE));
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = red[0];
#pragma unroll
  for (int w = 1; w < kW; ++w) m = fmaxf(m, red[w]);

  const int grp = tid / LPD, d4 = (tid % LPD) * 4;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  float sum = 0.f;
  for (int s = grp; s < nblk; s += NG) {
    const float lse = COHERENT ? load_coherent(ml + s) : ml[s];
    // a split without a live row has lse = -inf and weight 0; so has every split
    // when nothing at all was attended (m = -inf), which leaves 0/0 below
    const float w = (lse == -INFINITY) ? 0.f : fast_exp(lse - m);
    float4 o;
    if (COHERENT) {
      const float* src = mo + (int64_t)s * D + d4;
      o = make_float4(load_coherent(src), load_coherent(src + 1), load_coherent(src + 2), load_coherent(src + 3));
    } else {
      o = *reinterpret_cast<const float4*>(mo + (int64_t)s * D + d4);
    }
    acc.x += w * o.x;
    acc.y += w * o.y;
    acc.z += w * o.z;
    acc.w += w * o.w;
    sum += w;
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
  const int len = sparse_len[b * len_sb + h * len_sh];
  // (a length beyond nsplit * block_seq is cut to the splits that exist)
  int nblk = len <= 0 ? 0 : (len + block_seq - 1) / block_seq;
  nblk = min(nblk, nsplit);
  merge_splits<D>(mid_o + ((int64_t)b * Hq + h) * nsplit * D, mid_lse + ((int64_t)b * Hq + h) * nsplit, nblk, out,
                  out_dtype, b * out_sb + h * out_sh);
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
#pragma unroll
      for (int x = 1; x < LPR; x <<= 1) d += __shfl_xor(d, x, SOCKET_WAVE);
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
    if (tid == 0) last = atomicInc(&fin.arrive[b * Hq + h], (unsigned int)(nblk - 1)) == (unsigned int)(nblk - 1);
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
#pragma unroll
        for (int x = 1; x < LPR; x <<= 1) d += __shfl_xor(d, x, SOCKET_WAVE);
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

int dense_rows_per_split(int B, int Hkv, int T) {
  // Aim at >= 8 workgroups per CU over the whole grid, splits of >= 256 rows.
  const SocketDeviceLimits& lim = socket_device_limits();
  const int want = 8 * lim.cu_count;
  int nsplit = (want + B * Hkv - 1) / (B * Hkv);
  if (nsplit < 1) nsplit = 1;
  int rows = (T + nsplit - 1) / nsplit;
  rows = (rows + 63) / 64 * 64;
  if (rows < 256) rows = 256;
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
  const int rows = dense_rows_per_split(B, Hkv, T);
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
  if (D == 128) SOCKET_DENSE_D(128);
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
