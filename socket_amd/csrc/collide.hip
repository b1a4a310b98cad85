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
// slices (two slices of 30 fp32 tables at L60 x R1024; one slice for fp16), and
// serves several such tiles under each slice; a thread fetches the codes of its
// eight consecutive tokens with one 16-byte load per table, six tables ahead of
// their use, and gathers without branches.
#include <atomic>

#include "socket_common.h"

namespace {

constexpr int kTokensPerThread = 8;
constexpr int kAhead = 6;   // tables whose codes are in flight per lane
constexpr size_t kCollideLdsSlack = 1024;

__device__ __forceinline__ float entry_to_f32(float x) { return x; }
__device__ __forceinline__ float entry_to_f32(uint16_t x) { return f16_bits_to_f32(x); }

// ct: tables per LDS slice.  INLDS false: a single table exceeds LDS, gather from global memory.
// VEC: rows are 16-byte aligned (T % 8 == 0 and aligned bases): 16-byte code loads.
// A workgroup serves `chunks` consecutive tiles of THREADS x 8 tokens under every
// slice it brings into LDS; with more than one slice the running sums of a tile
// wait in `out` between slices (each thread re-reads what it wrote itself), which
// costs 8 bytes per token and slice against the 2 L + 9 of the stream and keeps
// the order of the fp32 adds.
// STREAM: the codes are loaded with the streaming hint (a code array too large to
// stay in the memory-side cache from one call to the next; VEC only).
template <typename QT, int THREADS, bool VEC, bool INLDS, bool STREAM>
__global__ __launch_bounds__(THREADS) void collision_i16_kernel(
    const QT* __restrict__ q_probs, const int16_t* __restrict__ key_buckets,
    const uint8_t* __restrict__ allowed, const QT* __restrict__ v_hist, float* __restrict__ out,
    int L, int R, int T, int ct, int chunks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char collide_lds[];
  QT* table = reinterpret_cast<QT*>(collide_lds);
  constexpr int TPT = kTokensPerThread;
  const int bh = blockIdx.y;
  const QT* qp = q_probs + (int64_t)bh * L * R;
  const int16_t* kb = key_buckets + (int64_t)bh * L * T;

  // the eight codes of a thread's tokens for table l, as loaded (two per word; -1 where no token is)
  auto codes_of = [&](int l, int t0) -> uint4 {
    const int16_t* row = kb + (int64_t)l * T + t0;
    if (VEC && !STREAM) return *reinterpret_cast<const uint4*>(row);
    if (VEC) {
      typedef uint32_t u32x4_stream __attribute__((ext_vector_type(4)));
      const u32x4_stream v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_stream*>(row));
      return make_uint4(v.x, v.y, v.z, v.w);
    }
    uint32_t u[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t lo = (t0 + 2 * i < T) ? (uint16_t)row[2 * i] : 0xffffu;
      const uint32_t hi = (t0 + 2 * i + 1 < T) ? (uint16_t)row[2 * i + 1] : 0xffffu;
      u[i] = lo | (hi << 16);
    }
    return make_uint4(u[0], u[1], u[2], u[3]);
  };
  auto load_partial = [&](int64_t o, int t0, float (&sum)[TPT]) {
    if (VEC) {
      const float4 a = *reinterpret_cast<const float4*>(out + o);
      const float4 b = *reinterpret_cast<const float4*>(out + o + 4);
      sum[0] = a.x, sum[1] = a.y, sum[2] = a.z, sum[3] = a.w;
      sum[4] = b.x, sum[5] = b.y, sum[6] = b.z, sum[7] = b.w;
    } else {
#pragma unroll
      for (int i = 0; i < TPT; ++i) sum[i] = (t0 + i < T) ? out[o + i] : 0.f;
    }
  };
  auto store_partial = [&](int64_t o, int t0, const float (&sum)[TPT]) {
    if (VEC) {
      *reinterpret_cast<float4*>(out + o) = make_float4(sum[0], sum[1], sum[2], sum[3]);
      *reinterpret_cast<float4*>(out + o + 4) = make_float4(sum[4], sum[5], sum[6], sum[7]);
    } else {
#pragma unroll
      for (int i = 0; i < TPT; ++i)
        if (t0 + i < T) out[o + i] = sum[i];
    }
  };
  auto finish = [&](int64_t o, int t0, const float (&sum)[TPT]) {
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
  };

  const int step = INLDS ? ct : L;   // (without LDS: one pass over all tables)
  for (int l0 = 0; l0 < L; l0 += step) {
    const int nt = min(step, L - l0);
    if (INLDS) {
      __syncthreads();   // the previous slice has been consumed
      // 16 bytes per lane where the slice starts and ends on 16-byte boundaries
      const int n16 = nt * R * (int)sizeof(QT) / 16;
      const uint4* src = reinterpret_cast<const uint4*>(qp + (int64_t)l0 * R);
      uint4* dst = reinterpret_cast<uint4*>(table);
      if (((uintptr_t)src & 15) == 0 && (nt * R * (int)sizeof(QT)) % 16 == 0) {
        for (int i = threadIdx.x; i < n16; i += THREADS) dst[i] = src[i];
      } else {
        for (int i = threadIdx.x; i < nt * R; i += THREADS) table[i] = qp[(int64_t)l0 * R + i];
      }
      __syncthreads();
    }
    for (int c = 0; c < chunks; ++c) {
      const int t0 = ((blockIdx.x * chunks + c) * THREADS + threadIdx.x) * TPT;
      if (t0 >= T) continue;
      const int64_t o = (int64_t)bh * T + t0;
      float sum[TPT];
      if (l0 == 0) {
#pragma unroll
        for (int i = 0; i < TPT; ++i) sum[i] = 0.f;
      } else {
        load_partial(o, t0, sum);
      }
      // A ring of kAhead code words per lane stays in flight (one 16-byte load per lane
      // would leave the stream waiting on latency): slot a always holds table lb + a;
      // the loop is unrolled by the ring's depth, so a slot is a fixed set of registers
      // and the wait before its use counts exactly the loads behind it.
      uint4 ring[kAhead];
#pragma unroll
      for (int a = 0; a < kAhead; ++a) ring[a] = codes_of(l0 + min(a, nt - 1), t0);
      for (int lb = 0; lb < nt; lb += kAhead) {
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
          const int l = lb + a;
          if (l >= nt) break;
          const uint4 cur = ring[a];
          ring[a] = codes_of(l0 + min(l + kAhead, nt - 1), t0);   // (past the slice: its last table again, unused)
          const uint32_t u[4] = {cur.x, cur.y, cur.z, cur.w};
          // branch-free: a stray code reads entry 0 and adds +0.0 instead (x + 0.0 == x;
          // the sums start at +0.0, so no -0.0 can be lost), and the LDS variant has no
          // global load in here for the compiler to wait on with the ring in flight
#pragma unroll
          for (int i = 0; i < TPT; ++i) {
            const int r = (int)(int16_t)((i & 1) ? (u[i >> 1] >> 16) : (u[i >> 1] & 0xffffu));
            const bool hit = r >= 0 && r < R;
            const int rr = hit ? r : 0;
            const float e = entry_to_f32(INLDS ? table[l * R + rr] : qp[(int64_t)(l0 + l) * R + rr]);
            sum[i] += hit ? e : 0.f;
          }
        }
      }
      if (l0 + nt >= L) finish(o, t0, sum);
      else store_partial(o, t0, sum);
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
  const int tiles = (T + threads * kTokensPerThread - 1) / (threads * kTokensPerThread);
  // tiles per workgroup: as many as leave two workgroups per CU (they amortise the
  // slices a workgroup pulls through LDS), at most 8
  int chunks = (int)((int64_t)tiles * B * H / (2 * (int64_t)lim.cu_count));
  chunks = chunks < 1 ? 1 : chunks > 8 ? 8 : chunks;
  if (chunks > tiles) chunks = tiles;
  dim3 grid((tiles + chunks - 1) / chunks, B * H);
  // (measured: 2 GB of codes gain 10 % from the hint, 135 MB that the cache still holds from the last call lose 7 %)
  const bool stream_codes = (int64_t)B * H * L * T * (int64_t)sizeof(int16_t) > (192ll << 20);
#define SOCKET_COLLIDE(TH, V, LD, ST)                                                                     \
  do {                                                                                                \
    auto kern = collision_i16_kernel<QT, TH, V, LD, ST>;                                                 \
    if (lds > 64 * 1024) {                                                                            \
      static std::atomic<size_t> granted{0};                                                          \
      if (granted.load(std::memory_order_acquire) < lds) {                                            \
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                  \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)budget) != hipSuccess) \
          return SOCKET_ERR_LAUNCH;                                                                   \
        granted.store(budget, std::memory_order_release);                                             \
      }                                                                                               \
    }                                                                                                 \
    hipLaunchKernelGGL(kern, grid, dim3(TH), lds, stream, q_probs, key_buckets, allowed, v_hist, out, L, R, T, ct, chunks); \
  } while (0)
#define SOCKET_COLLIDE_V(TH, LD)         \
  do {                                   \
    if (vec && stream_codes) SOCKET_COLLIDE(TH, true, LD, true); \
    else if (vec) SOCKET_COLLIDE(TH, true, LD, false); \
    else SOCKET_COLLIDE(TH, false, LD, false);  \
  } while (0)
  if (ct > 0) {
    if (small) SOCKET_COLLIDE_V(256, true);
    else SOCKET_COLLIDE_V(1024, true);
  } else {
    if (small) SOCKET_COLLIDE_V(256, false);
    else SOCKET_COLLIDE_V(1024, false);
  }
#undef SOCKET_COLLIDE_V
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
