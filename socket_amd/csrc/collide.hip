// Soft-collision scores on the reference's own operand layout: one int16 bucket
// code per (query head, table, token), [B,H,L,T], a table of probabilities
// [B,H,L,R], a mask byte and a value norm per (head, token).
//
// Replaces soft_hash_collision of the reference's extension (the call is
// GPT-FAST/kernels/sparse.py:40-49, the kernel GPT-FAST/kernels/soft_hash_collision.cu:25-54)
// and its fp16 variant (GPT-FAST/kernels/soft_hash_score/soft_hash_score.cu:7-42):
//   out[b,h,t] = allowed ? (sum_l table[b,h,l, code[b,h,l,t]]) * v[b,h,t] : -inf
// summed over l in ascending order in fp32; codes outside [0, R) add nothing.
//
// This layout costs 2 L + 9 bytes of HBM per (head, token) -- eight times the
// packed per-kv-head cache of score.hip at G = 4 -- and the launch is bound by
// that stream if the tables stay out of its way.  A workgroup therefore keeps a
// tile of THREADS x 8 tokens of one (b, h) row and walks the tables in LDS-sized
// slices (two slices of 30 fp32 tables at L60 x R1024; one slice for fp16): a
// slice is read once per 8192 tokens instead of once per 256, each thread
// fetches the codes of its eight consecutive tokens with one 16-byte load per
// table, and the eight running sums stay in registers across slices.
#include <atomic>

#include "socket_common.h"

namespace {

constexpr int kTokensPerThread = 8;
constexpr size_t kCollideLdsSlack = 1024;

__device__ __forceinline__ float entry_to_f32(float x) { return x; }
__device__ __forceinline__ float entry_to_f32(uint16_t x) { return f16_bits_to_f32(x); }

// ct: tables per LDS slice; 0 = a single table exceeds LDS, gather from global memory.
// VEC: rows are 16-byte aligned (T % 8 == 0 and aligned bases): 16-byte code loads.
template <typename QT, int THREADS, bool VEC>
__global__ __launch_bounds__(THREADS) void collision_i16_kernel(
    const QT* __restrict__ q_probs, const int16_t* __restrict__ key_buckets,
    const uint8_t* __restrict__ allowed, const QT* __restrict__ v_hist, float* __restrict__ out,
    int L, int R, int T, int ct) {
  extern __shared__ __attribute__((aligned(16))) unsigned char collide_lds[];
  QT* table = reinterpret_cast<QT*>(collide_lds);
  constexpr int TPT = kTokensPerThread;
  const int bh = blockIdx.y;
  const int t0 = (blockIdx.x * THREADS + threadIdx.x) * TPT;
  const QT* qp = q_probs + (int64_t)bh * L * R;
  const int16_t* kb = key_buckets + (int64_t)bh * L * T;
  float sum[TPT];
#pragma unroll
  for (int i = 0; i < TPT; ++i) sum[i] = 0.f;

  auto codes_of = [&](int l, int (&r)[TPT]) {
    const int16_t* row = kb + (int64_t)l * T + t0;
    if (VEC) {
      if (t0 < T) {
        const uint4 w = *reinterpret_cast<const uint4*>(row);
        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          r[2 * i] = (int)(int16_t)(u[i] & 0xffffu);
          r[2 * i + 1] = (int)(int16_t)(u[i] >> 16);
        }
      } else {
#pragma unroll
        for (int i = 0; i < TPT; ++i) r[i] = -1;
      }
    } else {
#pragma unroll
      for (int i = 0; i < TPT; ++i) r[i] = (t0 + i < T) ? (int)row[i] : -1;
    }
  };

  if (ct == 0) {
    for (int l = 0; l < L; ++l) {
      int r[TPT];
      codes_of(l, r);
#pragma unroll
      for (int i = 0; i < TPT; ++i)
        if (r[i] >= 0 && r[i] < R) sum[i] += entry_to_f32(qp[(int64_t)l * R + r[i]]);
    }
  } else {
    for (int l0 = 0; l0 < L; l0 += ct) {
      const int nt = min(ct, L - l0);
      __syncthreads();   // the previous slice has been consumed
      {
        // 16 bytes per lane where the slice starts and ends on 16-byte boundaries
        const int n16 = nt * R * (int)sizeof(QT) / 16;
        const uint4* src = reinterpret_cast<const uint4*>(qp + (int64_t)l0 * R);
        uint4* dst = reinterpret_cast<uint4*>(table);
        if (((uintptr_t)src & 15) == 0 && (nt * R * (int)sizeof(QT)) % 16 == 0) {
          for (int i = threadIdx.x; i < n16; i += THREADS) dst[i] = src[i];
        } else {
          for (int i = threadIdx.x; i < nt * R; i += THREADS) table[i] = qp[(int64_t)l0 * R + i];
        }
      }
      __syncthreads();
      for (int l = 0; l < nt; ++l) {
        int r[TPT];
        codes_of(l0 + l, r);
        const QT* tab = table + l * R;
#pragma unroll
        for (int i = 0; i < TPT; ++i)
          if (r[i] >= 0 && r[i] < R) sum[i] += entry_to_f32(tab[r[i]]);
      }
    }
  }

  if (t0 >= T) return;
  const int64_t o = (int64_t)bh * T + t0;
  if (VEC) {   // all eight tokens exist and every operand row is 16-byte aligned at o
    const uint2 aw = *reinterpret_cast<const uint2*>(allowed + o);
    const uint32_t ab[2] = {aw.x, aw.y};
    float vh[TPT];
    if (sizeof(QT) == 4) {
      const float4 v0 = *reinterpret_cast<const float4*>(v_hist + o);
      const float4 v1 = *reinterpret_cast<const float4*>(v_hist + o + 4);
      vh[0] = v0.x, vh[1] = v0.y, vh[2] = v0.z, vh[3] = v0.w;
      vh[4] = v1.x, vh[5] = v1.y, vh[6] = v1.z, vh[7] = v1.w;
    } else {
      const uint4 w = *reinterpret_cast<const uint4*>(v_hist + o);
      const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        vh[2 * i] = f16_bits_to_f32((uint16_t)(u[i] & 0xffffu));
        vh[2 * i + 1] = f16_bits_to_f32((uint16_t)(u[i] >> 16));
      }
    }
    float res[TPT];
#pragma unroll
    for (int i = 0; i < TPT; ++i)
      res[i] = ((ab[i >> 2] >> (8 * (i & 3))) & 0xffu) ? sum[i] * vh[i] : -INFINITY;
    *reinterpret_cast<float4*>(out + o) = make_float4(res[0], res[1], res[2], res[3]);
    *reinterpret_cast<float4*>(out + o + 4) = make_float4(res[4], res[5], res[6], res[7]);
  } else {
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      if (t0 + i < T) out[o + i] = allowed[o + i] ? sum[i] * entry_to_f32(v_hist[o + i]) : -INFINITY;
    }
  }
}

template <typename QT>
int launch_collision_i16(const QT* q_probs, const int16_t* key_buckets, const uint8_t* allowed,
                         const QT* v_hist, float* out, int B, int H, int L, int R, int T,
                         hipStream_t stream) {
  const SocketDeviceLimits& lim = socket_device_limits();
  const size_t per_table = (size_t)R * sizeof(QT);
  const size_t budget = (size_t)lim.max_lds_per_block - kCollideLdsSlack;
  int ct = (int)(budget / per_table);
  if (ct > L) ct = L;
  if (ct > 0) {   // slices of equal size
    const int slices = (L + ct - 1) / ct;
    ct = (L + slices - 1) / slices;
  }
  const size_t lds = (size_t)ct * per_table;
  const bool vec = T % 8 == 0 && (((uintptr_t)key_buckets | (uintptr_t)allowed | (uintptr_t)v_hist | (uintptr_t)out) & 15) == 0;
  // short rows: a quarter of the threads, so that a tile is not mostly idle lanes
  const bool small = T <= 256 * kTokensPerThread;
  const int threads = small ? 256 : 1024;
  dim3 grid((T + threads * kTokensPerThread - 1) / (threads * kTokensPerThread), B * H);
#define SOCKET_COLLIDE(TH, V)                                                                         \
  do {                                                                                                \
    auto kern = collision_i16_kernel<QT, TH, V>;                                                      \
    if (lds > 64 * 1024) {                                                                            \
      static std::atomic<size_t> granted{0};                                                          \
      if (granted.load(std::memory_order_acquire) < lds) {                                            \
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                  \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)budget) != hipSuccess) \
          return SOCKET_ERR_LAUNCH;                                                                   \
        granted.store(budget, std::memory_order_release);                                             \
      }                                                                                               \
    }                                                                                                 \
    hipLaunchKernelGGL(kern, grid, dim3(TH), lds, stream, q_probs, key_buckets, allowed, v_hist, out, L, R, T, ct); \
  } while (0)
  if (small) {
    if (vec) SOCKET_COLLIDE(256, true);
    else SOCKET_COLLIDE(256, false);
  } else {
    if (vec) SOCKET_COLLIDE(1024, true);
    else SOCKET_COLLIDE(1024, false);
  }
#undef SOCKET_COLLIDE
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

}  // namespace

extern "C" int socket_soft_hash_collision(const float* q_probs, const int16_t* key_buckets,
                                          const uint8_t* allowed, const float* v_hist, float* out,
                                          int B, int H, int L, int R, int T, void* stream) {
  SOCKET_REQUIRE(q_probs && key_buckets && allowed && v_hist && out, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(B > 0 && H > 0 && L > 0 && R > 0 && T > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE((int64_t)B * H <= 65535, SOCKET_ERR_SHAPE);
  return launch_collision_i16<float>(q_probs, key_buckets, allowed, v_hist, out, B, H, L, R, T,
                                     (hipStream_t)stream);
}

extern "C" int socket_soft_hash_score_f16(const uint16_t* q_probs, const int16_t* key_buckets,
                                          const uint16_t* v_norm, const uint8_t* allowed, float* out,
                                          int B, int H, int L, int R, int T, void* stream) {
  SOCKET_REQUIRE(q_probs && key_buckets && allowed && v_norm && out, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(B > 0 && H > 0 && L > 0 && R > 0 && T > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE((int64_t)B * H <= 65535, SOCKET_ERR_SHAPE);
  return launch_collision_i16<uint16_t>(q_probs, key_buckets, allowed, v_norm, out, B, H, L, R, T,
                                        (hipStream_t)stream);
}
