// Decode-step helpers around the attention hook: each replaces a chain of small
// elementwise launches of the reference's decode step by one launch, with the
// same arithmetic (fp32 inside, the same roundings to the storage type).
//
//  * rope_append_kernel: rotary embedding of the new token's q and k, and the
//    append of k / v to the cache at the token's position, read from the fused
//    qkv projection (GPT-FAST/model.py:433-444 apply_rotary_emb :626-639, and the
//    K/V part of KVCache.update :215-217); also raises the cache's device-side
//    lengths.  The position comes from device memory, nothing is read back.
//  * add_rmsnorm_kernel: optional residual add + RMSNorm (model.py:603-614 and
//    the `x + ...` of TransformerBlock :340-342).
//  * silu_mul_kernel: silu(a) * b of the feed-forward (model.py:599-600).
#include "socket_common.h"

namespace {

template <class DT>
__device__ __forceinline__ float ld(const void* p, int64_t i);
template <>
__device__ __forceinline__ float ld<DType_f32>(const void* p, int64_t i) { return ((const float*)p)[i]; }
template <>
__device__ __forceinline__ float ld<DType_bf16>(const void* p, int64_t i) {
  return bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
template <>
__device__ __forceinline__ float ld<DType_f16>(const void* p, int64_t i) {
  return f16_bits_to_f32(((const uint16_t*)p)[i]);
}

// round to the storage type and back (what a torch op on that dtype leaves behind)
template <class DT>
__device__ __forceinline__ float rnd(float x);
template <>
__device__ __forceinline__ float rnd<DType_f32>(float x) { return x; }
template <>
__device__ __forceinline__ float rnd<DType_bf16>(float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); }
template <>
__device__ __forceinline__ float rnd<DType_f16>(float x) { return f16_bits_to_f32(f32_to_f16_bits(x)); }

// One 16-byte vector of elements from floats (rounded to the storage type).
template <class DT>
__device__ __forceinline__ void store16(void* base, int64_t idx, const float* v);
template <>
__device__ __forceinline__ void store16<DType_f32>(void* base, int64_t idx, const float* v) {
  *reinterpret_cast<float4*>((float*)base + idx) = make_float4(v[0], v[1], v[2], v[3]);
}
template <>
__device__ __forceinline__ void store16<DType_bf16>(void* base, int64_t idx, const float* v) {
  uint4 w;
  w.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
  w.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
  w.z = (uint32_t)f32_to_bf16_bits(v[4]) | ((uint32_t)f32_to_bf16_bits(v[5]) << 16);
  w.w = (uint32_t)f32_to_bf16_bits(v[6]) | ((uint32_t)f32_to_bf16_bits(v[7]) << 16);
  *reinterpret_cast<uint4*>((uint16_t*)base + idx) = w;
}
template <>
__device__ __forceinline__ void store16<DType_f16>(void* base, int64_t idx, const float* v) {
  uint4 w;
  w.x = (uint32_t)f32_to_f16_bits(v[0]) | ((uint32_t)f32_to_f16_bits(v[1]) << 16);
  w.y = (uint32_t)f32_to_f16_bits(v[2]) | ((uint32_t)f32_to_f16_bits(v[3]) << 16);
  w.z = (uint32_t)f32_to_f16_bits(v[4]) | ((uint32_t)f32_to_f16_bits(v[5]) << 16);
  w.w = (uint32_t)f32_to_f16_bits(v[6]) | ((uint32_t)f32_to_f16_bits(v[7]) << 16);
  *reinterpret_cast<uint4*>((uint16_t*)base + idx) = w;
}

// One workgroup per (head of the fused projection, sequence); lane i owns the
// pair (2i, 2i+1).  Heads [0,Hq) are queries, [Hq,Hq+Hkv) keys, the rest values.
template <class DT, class FT>
__global__ void rope_append_kernel(const void* __restrict__ qkv, int64_t qkv_sb, const void* __restrict__ freqs,
                                   const int64_t* __restrict__ pos, int pos_stride, void* __restrict__ q_out,
                                   void* __restrict__ k_cache, void* __restrict__ v_cache, int64_t c_sb,
                                   int64_t c_sh, int64_t c_ss, int32_t* __restrict__ lens,
                                   void* __restrict__ k_new, void* __restrict__ v_new, int Hq, int Hkv, int D,
                                   int64_t Tcap, int64_t n_pos) {
  const int hh = blockIdx.x, b = blockIdx.y, i = threadIdx.x;
  const int64_t p = pos[(int64_t)b * pos_stride];
  const bool ok = p >= 0 && p < Tcap && p < n_pos;   // a position outside the cache or the table writes nothing
  // the cached length follows the position: rows past it are older contents, not context
  if (hh == 0 && i == 0 && ok && lens) lens[b] = (int32_t)p + 1;
  const int64_t src = (int64_t)b * qkv_sb + (int64_t)hh * D + 2 * i;
  const float x0 = ld<DT>(qkv, src), x1 = ld<DT>(qkv, src + 1);
  if (hh >= Hq + Hkv) {  // value: plain copy
    if (v_new) {
      const int64_t o = ((int64_t)b * Hkv + (hh - Hq - Hkv)) * D + 2 * i;
      store_elem<DT>(v_new, o, x0);
      store_elem<DT>(v_new, o + 1, x1);
    }
    if (ok) {
      const int64_t o = b * c_sb + (int64_t)(hh - Hq - Hkv) * c_sh + p * c_ss + 2 * i;
      store_elem<DT>(v_cache, o, x0);
      store_elem<DT>(v_cache, o + 1, x1);
    }
    return;
  }
  float re = x0, im = x1;
  if (p >= 0 && p < n_pos) {
    const float c = ld<FT>(freqs, (p * (D / 2) + i) * 2), s = ld<FT>(freqs, (p * (D / 2) + i) * 2 + 1);
    rotate_pair(x0, x1, c, s, re, im);
  }
  if (hh < Hq) {
    const int64_t o = ((int64_t)b * Hq + hh) * D + 2 * i;
    store_elem<DT>(q_out, o, re);
    store_elem<DT>(q_out, o + 1, im);
  } else {
    if (k_new) {
      const int64_t o = ((int64_t)b * Hkv + (hh - Hq)) * D + 2 * i;
      store_elem<DT>(k_new, o, re);
      store_elem<DT>(k_new, o + 1, im);
    }
    if (ok) {
      const int64_t o = b * c_sb + (int64_t)(hh - Hq) * c_sh + p * c_ss + 2 * i;
      store_elem<DT>(k_cache, o, re);
      store_elem<DT>(k_cache, o + 1, im);
    }
  }
}

constexpr int kNormThreads = 256;
constexpr int kNormVecs = 4;  // 16-byte vectors a lane keeps between the two sweeps

// One workgroup per row.  h = x + r (rounded to the storage type) when r is
// given, y = round(h * rsqrt(mean(h^2) + eps)) * w, rounded again.  Rows of up to
// 256 * 4 vectors (8192 bf16 / 4096 fp32 elements, 16-byte aligned) are read once,
// 16 bytes per lane, and kept in registers for the second sweep.
template <class DT>
__global__ __launch_bounds__(kNormThreads) void add_rmsnorm_kernel(
    const void* __restrict__ x, const void* __restrict__ r, const void* __restrict__ w,
    void* __restrict__ h_out, void* __restrict__ y_out, int dim, float eps, int vec_ok) {
  constexpr int E = DT::kPer16B;
  __shared__ float red[kNormThreads / SOCKET_WAVE];
  const int64_t row = (int64_t)blockIdx.x * dim;
  const int tid = threadIdx.x;
  float ss = 0.f;
  float hreg[kNormVecs][E];
  const int nvec = dim / E;
  if (vec_ok) {
#pragma unroll
    for (int k = 0; k < kNormVecs; ++k) {
      const int v = tid + k * kNormThreads;
      if (v < nvec) {
        unpack16<DT>(*reinterpret_cast<const uint4*>((const typename DT::storage*)x + row + (int64_t)v * E), hreg[k]);
        if (r) {
          float rr[E];
          unpack16<DT>(*reinterpret_cast<const uint4*>((const typename DT::storage*)r + row + (int64_t)v * E), rr);
#pragma unroll
          for (int e = 0; e < E; ++e) hreg[k][e] = rnd<DT>(hreg[k][e] + rr[e]);
        }
#pragma unroll
        for (int e = 0; e < E; ++e) ss += hreg[k][e] * hreg[k][e];
      }
    }
  } else {
    for (int i = tid; i < dim; i += kNormThreads) {
      float h = ld<DT>(x, row + i);
      if (r) h = rnd<DT>(h + ld<DT>(r, row + i));
      ss += h * h;
    }
  }
  ss = wave_reduce_to_last<false>(ss);
  if ((tid & 63) == 63) red[tid >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int k = 0; k < kNormThreads / SOCKET_WAVE; ++k) tot += red[k];
  const float rs = rsqrtf(tot / (float)dim + eps);
  if (vec_ok) {
#pragma unroll
    for (int k = 0; k < kNormVecs; ++k) {
      const int v = tid + k * kNormThreads;
      if (v < nvec) {
        float ww[E];
        unpack16<DT>(*reinterpret_cast<const uint4*>((const typename DT::storage*)w + (int64_t)v * E), ww);
        float y[E];
#pragma unroll
        for (int e = 0; e < E; ++e) y[e] = rnd<DT>(hreg[k][e] * rs) * ww[e];
        if (h_out) store16<DT>(h_out, row + (int64_t)v * E, hreg[k]);
        store16<DT>(y_out, row + (int64_t)v * E, y);
      }
    }
  } else {
    for (int i = tid; i < dim; i += kNormThreads) {
      float h = ld<DT>(x, row + i);
      if (r) h = rnd<DT>(h + ld<DT>(r, row + i));
      if (h_out) store_elem<DT>(h_out, row + i, h);
      store_elem<DT>(y_out, row + i, rnd<DT>(h * rs) * ld<DT>(w, i));
    }
  }
}

template <class DT>
__global__ void silu_mul_kernel(const void* __restrict__ a, const void* __restrict__ b, void* __restrict__ out,
                                int64_t n, int vec_ok) {
  constexpr int E = DT::kPer16B;
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (vec_ok) {
    const int64_t i = t * E;
    if (i >= n) return;
    float x[E], y[E], o[E];
    unpack16<DT>(*reinterpret_cast<const uint4*>((const typename DT::storage*)a + i), x);
    unpack16<DT>(*reinterpret_cast<const uint4*>((const typename DT::storage*)b + i), y);
#pragma unroll
    for (int e = 0; e < E; ++e) o[e] = rnd<DT>(x[e] / (1.f + expf(-x[e]))) * y[e];
    store16<DT>(out, i, o);
    return;
  }
  for (int64_t i = t * E; i < min(n, (t + 1) * E); ++i) {
    const float x = ld<DT>(a, i);
    store_elem<DT>(out, i, rnd<DT>(x / (1.f + expf(-x))) * ld<DT>(b, i));
  }
}


// y[m,n] = sum_k x[m,k] * w[n,k] for a handful of rows m (a decode step's linear
// layers are matrix-vector products: the weight matrix is streamed once, HBM bound).
// One wave per output feature n: 16 bytes of the weight row per lane and step,
// four steps in flight, fp32 accumulation, a butterfly over the lanes at the end.
// GATE: two weight matrices, y = round(silu(round(x.w[n]))) * round(x.wg[n]) -- the
// roundings of the three torch ops this replaces.
constexpr int kGemvThreads = 256;
constexpr int kGemvUnroll = 4;
constexpr int kGemvStep = 64 * 8;  // elements of a row per wave and step
constexpr int kGemvWgPerCu = 4;    // workgroups per CU of the persistent launch

template <int M, bool GATE>
__global__ __launch_bounds__(kGemvThreads) void gemv_bf16_kernel(
    const uint16_t* __restrict__ x, int64_t x_stride, const uint16_t* __restrict__ w,
    const uint16_t* __restrict__ wg, uint16_t* __restrict__ y, int64_t y_stride, int N, int K) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * (kGemvThreads / 64) + wave;
  if (n >= N) return;
  const uint16_t* wr = w + (int64_t)n * K;
  const uint16_t* gr = GATE ? wg + (int64_t)n * K : nullptr;
  float acc[M], accg[M];
#pragma unroll
  for (int m = 0; m < M; ++m) acc[m] = accg[m] = 0.f;
  for (int k0 = lane * 8; k0 < K; k0 += kGemvStep * kGemvUnroll) {  // K is a multiple of the unrolled step
    u32x4 wv[kGemvUnroll], gv[kGemvUnroll];
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      wv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wr + k0 + u * kGemvStep));
      if (GATE) gv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(gr + k0 + u * kGemvStep));
    }
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const uint4 xv = *reinterpret_cast<const uint4*>(x + (int64_t)m * x_stride + k0 + u * kGemvStep);
        const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float x0 = __uint_as_float(xw[i] << 16), x1 = __uint_as_float(xw[i] & 0xffff0000u);
          acc[m] = fmaf(__uint_as_float(wv[u][i] << 16), x0, acc[m]);
          acc[m] = fmaf(__uint_as_float(wv[u][i] & 0xffff0000u), x1, acc[m]);
          if (GATE) {
            accg[m] = fmaf(__uint_as_float(gv[u][i] << 16), x0, accg[m]);
            accg[m] = fmaf(__uint_as_float(gv[u][i] & 0xffff0000u), x1, accg[m]);
          }
        }
      }
    }
  }
  // (sums over the wave on the data-parallel-primitive path, left in the last lane)
#pragma unroll
  for (int m = 0; m < M; ++m) {
    acc[m] = wave_reduce_to_last<false>(acc[m]);
    if (GATE) accg[m] = wave_reduce_to_last<false>(accg[m]);
  }
  if (lane == 63) {
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float r = acc[m];
      if (GATE) {
        const float a = rnd<DType_bf16>(acc[m]);
        r = rnd<DType_bf16>(a / (1.f + expf(-a))) * rnd<DType_bf16>(accg[m]);
      }
      y[(int64_t)m * y_stride + n] = f32_to_bf16_bits(r);
    }
  }
}

// The product with the RMSNorm that feeds it (and the residual add before that) in the same
// launch.  The vector is RMSNorm(x + r) * nw, worked out by every workgroup for itself while
// its first weight vectors are on their way -- h = x + r, xn = round(h * rsqrt(mean(h^2) + eps))
// * nw, rounded: lane for lane and sum for sum what add_rmsnorm_kernel computes -- and kept in
// LDS (M rows of K).  So that few workgroups pay for it the launch is persistent: a few
// workgroups per CU, wave g of the launch takes output features g, g + waves, g + 2 waves, ...;
// its weight vectors run through two register buffers, the next 2048 elements of its row -- or
// the first of its next row -- requested before the current ones are multiplied, so a wave
// streams without a gap from its first row to its last.  A lane adds its products in the
// order of gemv_bf16_kernel: the result equals the two launches bit for bit.  Workgroup 0
// writes h.  (On 256 CUs, one row of 4096: 6144 outputs 11.6 against 13.7 us for the two
// launches, 2 x 14336 gated 39.8 against 41.9; one workgroup per four outputs, as
// gemv_bf16_kernel has them, pays for the norm 1536 and 3584 times and is no faster than
// two launches; without a norm to share, the short-lived workgroups of gemv_bf16_kernel are
// the faster form by 0.5-1 us.)
template <int M, bool GATE>
__global__ __launch_bounds__(kGemvThreads) void norm_gemv_rows_kernel(
    const uint16_t* __restrict__ x, int64_t x_stride, const uint16_t* __restrict__ r,
    const uint16_t* __restrict__ nw, float eps, uint16_t* __restrict__ h_out, const uint16_t* __restrict__ w,
    const uint16_t* __restrict__ wg, uint16_t* __restrict__ y, int64_t y_stride, int N, int K) {
  static_assert(kGemvThreads == kNormThreads, "the norm's lane map");
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  typedef DType_bf16 DT;
  constexpr int E = DT::kPer16B;
  constexpr int kChunk = kGemvStep * kGemvUnroll;
  extern __shared__ __attribute__((aligned(16))) uint16_t xs[];   // [M][K]
  __shared__ float red[M][kNormThreads / SOCKET_WAVE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int waves = gridDim.x * (kGemvThreads / 64);
  int n = blockIdx.x * (kGemvThreads / 64) + wave;   // (wave-uniform)
  const int nk = K / kChunk;
  u32x4 wa[kGemvUnroll], ga[kGemvUnroll], wb[kGemvUnroll], gb[kGemvUnroll];
  auto fetch = [&](u32x4 (&wv)[kGemvUnroll], u32x4 (&gv)[kGemvUnroll], int row, int kc) __attribute__((always_inline)) {
    const int64_t at = (int64_t)row * K + kc * kChunk + lane * 8;
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
      wv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(w + at + u * kGemvStep));
      if (GATE) gv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wg + at + u * kGemvStep));
    }
  };
  if (n < N) fetch(wa, ga, n, 0);
  // ---- the vector into LDS ----
  const int nvec = K / E;
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const int64_t row = (int64_t)m * x_stride;
    float hreg[kNormVecs][E];
    uint4 wraw[kNormVecs];   // (the norm's weights, requested with the row instead of after the barrier)
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < kNormVecs; ++k) {
      const int v = tid + k * kNormThreads;
      if (v < nvec) wraw[k] = *reinterpret_cast<const uint4*>(nw + (int64_t)v * E);
    }
#pragma unroll
    for (int k = 0; k < kNormVecs; ++k) {
      const int v = tid + k * kNormThreads;
      if (v < nvec) {
        unpack16<DT>(*reinterpret_cast<const uint4*>(x + row + (int64_t)v * E), hreg[k]);
        if (r) {
          float rr[E];
          unpack16<DT>(*reinterpret_cast<const uint4*>(r + row + (int64_t)v * E), rr);
#pragma unroll
          for (int e = 0; e < E; ++e) hreg[k][e] = rnd<DT>(hreg[k][e] + rr[e]);
        }
#pragma unroll
        for (int e = 0; e < E; ++e) ss += hreg[k][e] * hreg[k][e];
      }
    }
    ss = wave_reduce_to_last<false>(ss);
    if (lane == 63) red[m][wave] = ss;
    __syncthreads();
    float tot = 0.f;
#pragma unroll
    for (int k = 0; k < kNormThreads / SOCKET_WAVE; ++k) tot += red[m][k];
    const float rs = rsqrtf(tot / (float)K + eps);
#pragma unroll
    for (int k = 0; k < kNormVecs; ++k) {
      const int v = tid + k * kNormThreads;
      if (v < nvec) {
        float ww[E], yn[E];
        unpack16<DT>(wraw[k], ww);
#pragma unroll
        for (int e = 0; e < E; ++e) yn[e] = rnd<DT>(hreg[k][e] * rs) * ww[e];
        if (h_out && blockIdx.x == 0) store16<DT>(h_out, row + (int64_t)v * E, hreg[k]);
        store16<DT>(xs, (int64_t)m * K + (int64_t)v * E, yn);
      }
    }
  }
  __syncthreads();
  // ---- the rows of this wave ----
  float acc[M], accg[M];
#pragma unroll
  for (int m = 0; m < M; ++m) acc[m] = accg[m] = 0.f;
  int kc = 0;
  // one chunk: request the one after it into the other buffers, multiply this one, and at a
  // row's end reduce over the lanes and store
  auto step = [&](u32x4 (&cw)[kGemvUnroll], u32x4 (&cg)[kGemvUnroll], u32x4 (&nwv)[kGemvUnroll],
                  u32x4 (&ngv)[kGemvUnroll]) __attribute__((always_inline)) {
    const bool row_ends = kc + 1 == nk;
    const int n2 = row_ends ? n + waves : n, kc2 = row_ends ? 0 : kc + 1;
    if (n2 < N) fetch(nwv, ngv, n2, kc2);
#pragma unroll
    for (int u = 0; u < kGemvUnroll; ++u) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const uint4 xv = *reinterpret_cast<const uint4*>(xs + (int64_t)m * K + kc * kChunk + lane * 8 + u * kGemvStep);
        const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float x0 = __uint_as_float(xw[i] << 16), x1 = __uint_as_float(xw[i] & 0xffff0000u);
          acc[m] = fmaf(__uint_as_float(cw[u][i] << 16), x0, acc[m]);
          acc[m] = fmaf(__uint_as_float(cw[u][i] & 0xffff0000u), x1, acc[m]);
          if (GATE) {
            accg[m] = fmaf(__uint_as_float(cg[u][i] << 16), x0, accg[m]);
            accg[m] = fmaf(__uint_as_float(cg[u][i] & 0xffff0000u), x1, accg[m]);
          }
        }
      }
    }
    if (row_ends) {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float o = wave_reduce_to_last<false>(acc[m]);
        if (GATE) {
          const float gsum = wave_reduce_to_last<false>(accg[m]);
          const float a = rnd<DType_bf16>(o);
          o = rnd<DType_bf16>(a / (1.f + expf(-a))) * rnd<DType_bf16>(gsum);
        }
        if (lane == 63) y[(int64_t)m * y_stride + n] = f32_to_bf16_bits(o);
        acc[m] = accg[m] = 0.f;
      }
    }
    n = n2;
    kc = kc2;
  };
  while (n < N) {
    step(wa, ga, wb, gb);
    if (n >= N) break;
    step(wb, gb, wa, ga);
  }
}

template <int M>
int launch_norm_gemv_rows(const uint16_t* x, int64_t xs, const uint16_t* r, const uint16_t* nw, float eps,
                          uint16_t* h_out, const uint16_t* w, const uint16_t* wg, uint16_t* y, int64_t ys, int N,
                          int K, hipStream_t s) {
  const SocketDeviceLimits& lim = socket_device_limits();
  const size_t lds = (size_t)M * K * 2;
  if (lds + 256 > (size_t)lim.max_lds_per_block) return SOCKET_ERR_UNSUPPORTED;
  // kGemvWgPerCu workgroups per CU (2: 12.1 / 41.4 us for the two shapes above, 3: 12.0 / 41.0,
  // 4: 11.6 / 39.8), each wave with two chunks of its rows in flight; never more waves than rows
  int n_wg = lim.cu_count * kGemvWgPerCu;
  const int by_rows = (N + kGemvThreads / 64 - 1) / (kGemvThreads / 64);
  if (n_wg > by_rows) n_wg = by_rows;
  const dim3 grid((unsigned)n_wg), block(kGemvThreads);
#define SOCKET_GR(GATE)                                                                                          \
  do {                                                                                                           \
    auto kern = norm_gemv_rows_kernel<M, GATE>;                                                                 \
    if (lds > 48 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                              \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
      return SOCKET_ERR_LAUNCH;                                                                                  \
    hipLaunchKernelGGL(kern, grid, block, lds, s, x, xs, r, nw, eps, h_out, w, wg, y, ys, N, K);                 \
  } while (0)
  if (wg) SOCKET_GR(true);
  else SOCKET_GR(false);
#undef SOCKET_GR
  return SOCKET_OK;
}

template <int M>
void launch_gemv(const uint16_t* x, int64_t xs, const uint16_t* w, const uint16_t* wg, uint16_t* y, int64_t ys, int N,
                 int K, hipStream_t s) {
  const dim3 grid((unsigned)((N + kGemvThreads / 64 - 1) / (kGemvThreads / 64))), block(kGemvThreads);
  if (wg) hipLaunchKernelGGL((gemv_bf16_kernel<M, true>), grid, block, 0, s, x, xs, w, wg, y, ys, N, K);
  else hipLaunchKernelGGL((gemv_bf16_kernel<M, false>), grid, block, 0, s, x, xs, w, wg, y, ys, N, K);
}

}  // namespace

extern "C" int socket_rope_append(const void* qkv, int dtype, int64_t qkv_stride_b, const void* freqs_cis,
                                  int freqs_dtype, int64_t n_pos, const int64_t* pos, int pos_stride, void* q_out,
                                  void* k_cache, void* v_cache, int64_t cache_stride_b, int64_t cache_stride_h,
                                  int64_t cache_stride_s, int32_t* lens, void* k_new, void* v_new, int B, int Hq,
                                  int Hkv, int D, int64_t Tcap, void* stream) {
  SOCKET_REQUIRE(qkv && freqs_cis && pos && q_out && k_cache && v_cache, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(socket_dtype_bytes(dtype) != 0, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(freqs_dtype == SOCKET_F32 || freqs_dtype == SOCKET_BF16, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(B > 0 && B <= 65535 && Hq > 0 && Hkv > 0 && Tcap > 0 && n_pos > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(D >= 2 && D % 2 == 0 && D <= 2048, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(pos_stride == 0 || pos_stride == 1, SOCKET_ERR_SHAPE);
  const dim3 grid(Hq + 2 * Hkv, B), block(D / 2);
  hipStream_t s = (hipStream_t)stream;
#define SOCKET_RA(DT, FT)                                                                                  \
  hipLaunchKernelGGL((rope_append_kernel<DT, FT>), grid, block, 0, s, qkv, qkv_stride_b, freqs_cis, pos,   \
                     pos_stride, q_out, k_cache, v_cache, cache_stride_b, cache_stride_h, cache_stride_s,  \
                     lens, k_new, v_new, Hq, Hkv, D, Tcap, n_pos)
#define SOCKET_RA_F(DT)                                      \
  do {                                                       \
    if (freqs_dtype == SOCKET_F32) SOCKET_RA(DT, DType_f32); \
    else SOCKET_RA(DT, DType_bf16);                          \
  } while (0)
  if (dtype == SOCKET_F32) SOCKET_RA_F(DType_f32);
  else if (dtype == SOCKET_BF16) SOCKET_RA_F(DType_bf16);
  else SOCKET_RA_F(DType_f16);
#undef SOCKET_RA_F
#undef SOCKET_RA
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

extern "C" int socket_add_rmsnorm(const void* x, const void* residual, const void* weight, void* h_out,
                                  void* y_out, int dtype, int64_t rows, int dim, float eps, void* stream) {
  SOCKET_REQUIRE(x && weight && y_out, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(socket_dtype_bytes(dtype) != 0, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(rows > 0 && rows < (1LL << 31) && dim > 0, SOCKET_ERR_SHAPE);
  hipStream_t s = (hipStream_t)stream;
  const int per16 = 16 / socket_dtype_bytes(dtype);
  const int vec_ok = dim % per16 == 0 && dim / per16 <= kNormThreads * kNormVecs && socket_aligned16(x) &&
                     socket_aligned16(weight) && socket_aligned16(y_out) &&
                     (residual == nullptr || socket_aligned16(residual)) &&
                     (h_out == nullptr || socket_aligned16(h_out));
#define SOCKET_RN(DT)                                                                                     \
  hipLaunchKernelGGL((add_rmsnorm_kernel<DT>), dim3((unsigned)rows), dim3(kNormThreads), 0, s, x, residual, \
                     weight, h_out, y_out, dim, eps, vec_ok)
  if (dtype == SOCKET_F32) SOCKET_RN(DType_f32);
  else if (dtype == SOCKET_BF16) SOCKET_RN(DType_bf16);
  else SOCKET_RN(DType_f16);
#undef SOCKET_RN
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

extern "C" int socket_silu_mul(const void* a, const void* b, void* out, int dtype, int64_t n, void* stream) {
  SOCKET_REQUIRE(a && b && out, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(socket_dtype_bytes(dtype) != 0, SOCKET_ERR_UNSUPPORTED);
  const int per16 = 16 / socket_dtype_bytes(dtype);
  const int64_t nthreads = (n + per16 - 1) / per16;
  SOCKET_REQUIRE(n > 0 && (nthreads + 255) / 256 < (1LL << 31), SOCKET_ERR_SHAPE);
  const int vec_ok = n % per16 == 0 && socket_aligned16(a) && socket_aligned16(b) && socket_aligned16(out);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((nthreads + 255) / 256)), block(256);
  if (dtype == SOCKET_F32) hipLaunchKernelGGL((silu_mul_kernel<DType_f32>), grid, block, 0, s, a, b, out, n, vec_ok);
  else if (dtype == SOCKET_BF16) hipLaunchKernelGGL((silu_mul_kernel<DType_bf16>), grid, block, 0, s, a, b, out, n, vec_ok);
  else hipLaunchKernelGGL((silu_mul_kernel<DType_f16>), grid, block, 0, s, a, b, out, n, vec_ok);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

extern "C" int socket_gemv_bf16(const void* x, int64_t x_stride, const void* w, const void* w_gate, void* y,
                                int64_t y_stride, int M, int N, int K, void* stream) {
  SOCKET_REQUIRE(x && w && y, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(M >= 1 && N >= 1 && K >= 1 && x_stride >= K && y_stride >= N, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(M <= 4 && K % (kGemvStep * kGemvUnroll) == 0, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(socket_aligned16(x) && socket_aligned16(w) && (!w_gate || socket_aligned16(w_gate)) && x_stride % 8 == 0,
                 SOCKET_ERR_ALIGN);
  hipStream_t s = (hipStream_t)stream;
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)w;
  const uint16_t* gp = (const uint16_t*)w_gate;
  uint16_t* yp = (uint16_t*)y;
  switch (M) {
    case 1: launch_gemv<1>(xp, x_stride, wp, gp, yp, y_stride, N, K, s); break;
    case 2: launch_gemv<2>(xp, x_stride, wp, gp, yp, y_stride, N, K, s); break;
    case 3: launch_gemv<3>(xp, x_stride, wp, gp, yp, y_stride, N, K, s); break;
    default: launch_gemv<4>(xp, x_stride, wp, gp, yp, y_stride, N, K, s); break;
  }
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

extern "C" int socket_norm_gemv_bf16(const void* x, const void* residual, const void* norm_weight, float eps,
                                     void* h_out, const void* w, const void* w_gate, void* y, int M, int N, int K,
                                     void* stream) {
  SOCKET_REQUIRE(x && norm_weight && w && y, SOCKET_ERR_NULL);
  SOCKET_REQUIRE((residual == nullptr) == (h_out == nullptr), SOCKET_ERR_NULL);
  SOCKET_REQUIRE(M >= 1 && N >= 1 && K >= 1, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(M <= 4 && K % (kGemvStep * kGemvUnroll) == 0 && K <= kNormThreads * kNormVecs * 8,
                 SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(socket_aligned16(x) && socket_aligned16(norm_weight) && socket_aligned16(w) &&
                     (!w_gate || socket_aligned16(w_gate)) && (!residual || socket_aligned16(residual)) &&
                     (!h_out || socket_aligned16(h_out)),
                 SOCKET_ERR_ALIGN);
  hipStream_t s = (hipStream_t)stream;
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* rp = (const uint16_t*)residual;
  const uint16_t* np = (const uint16_t*)norm_weight;
  const uint16_t* wp = (const uint16_t*)w;
  const uint16_t* gp = (const uint16_t*)w_gate;
  uint16_t* hp = (uint16_t*)h_out;
  uint16_t* yp = (uint16_t*)y;
  int rc;
  switch (M) {
    case 1: rc = launch_norm_gemv_rows<1>(xp, K, rp, np, eps, hp, wp, gp, yp, N, N, K, s); break;
    case 2: rc = launch_norm_gemv_rows<2>(xp, K, rp, np, eps, hp, wp, gp, yp, N, N, K, s); break;
    case 3: rc = launch_norm_gemv_rows<3>(xp, K, rp, np, eps, hp, wp, gp, yp, N, N, K, s); break;
    default: rc = launch_norm_gemv_rows<4>(xp, K, rp, np, eps, hp, wp, gp, yp, N, N, K, s); break;
  }
  if (rc != SOCKET_OK) return rc;
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}
