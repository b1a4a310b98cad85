// K2: soft-collision scorer.
//
// score[b,h,t] = (sum_{l<L} q_probs[b,h,l,code_l(t)]) * v_norm[t], masked to -inf.
// The arithmetic is the loop of GPT-FAST/kernels/soft_hash_collision.cu:45-53:
// one fp32 add per table in ascending table order, then one multiply.
//
// Two kernels:
//  * score_packed_kernel: this library's packed, per-KV-head, table-major code
//    cache.  A workgroup owns a tile of tokens of one (b, kv head); it walks the
//    packed words in order, staging the soft-hash table slice of the tables in
//    the current word(s) in LDS with the G query heads of the kv head
//    interleaved ([table][bucket][g]), so one LDS gather returns the terms of
//    all G heads.  Partial sums stay in registers across slices, which keeps the
//    reference's summation order.  Codes are read once per kv head, 16 bytes per
//    lane, fully coalesced.
//  * collision_i16_kernel: the reference's own operand layout (int16 codes per
//    query head), for drop-in callers.
#include "socket_common.h"

namespace {

// ---------------------------------------------------------------------------
// native packed scorer
// ---------------------------------------------------------------------------
template <int GP>
struct LdsEntry;  // GP floats, stored with the widest LDS access available
template <>
struct LdsEntry<1> { float v[1]; };
template <>
struct __attribute__((aligned(8))) LdsEntry<2> { float v[2]; };
template <>
struct __attribute__((aligned(16))) LdsEntry<4> { float v[4]; };
template <>
struct __attribute__((aligned(16))) LdsEntry<8> { float v[8]; };

// PT: P known at compile time (0 = use the runtime value).
template <int GP, int KT4, int THREADS, int PT>
__global__ __launch_bounds__(THREADS) void score_packed_kernel(
    const float* __restrict__ q_probs, const uint32_t* __restrict__ codes,
    const uint16_t* __restrict__ v_norm, const int32_t* __restrict__ lens,
    float* __restrict__ scores, int Hq, int Hkv, int G, int L, int P_rt, int R, int T,
    int64_t Tcap, int64_t score_stride, int NW, int chunk_words, int n_pairs, int n_tiles,
    int xcd_remap) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  LdsEntry<GP>* table = reinterpret_cast<LdsEntry<GP>*>(lds_raw);

  const int P = PT ? PT : P_rt;
  const int cpw = 32 / P;
  const uint32_t code_mask = (1u << P) - 1u;
  constexpr int TW = THREADS * 4 * KT4;

  // Workgroup -> (pair, tile).  Workgroups are dealt to the 8 XCDs round-robin
  // by linear id; with the remap all tiles of one (b, kv head) land on one XCD,
  // so its L2 serves that pair's table slices to every tile.
  int pair, tile;
  {
    const int n = blockIdx.x;
    if (xcd_remap) {
      const int xcd = n & 7, slot = n >> 3;
      pair = (slot / n_tiles) * 8 + xcd;
      tile = slot % n_tiles;
    } else {
      pair = n / n_tiles;
      tile = n % n_tiles;
    }
  }
  if (pair >= n_pairs) return;
  const int b = pair / Hkv, kvh = pair % Hkv;
  const int tid = threadIdx.x;
  const int len = lens ? min(lens[b], T) : T;

  const uint32_t* codes_pair = codes + (int64_t)pair * NW * Tcap;
  const float* qp_pair = q_probs + ((int64_t)(b * Hq + kvh * G)) * L * R;

  int tbase[KT4];
  bool live[KT4];
#pragma unroll
  for (int j = 0; j < KT4; ++j) {
    tbase[j] = tile * TW + j * (THREADS * 4) + tid * 4;
    live[j] = tbase[j] < T;
  }

  float acc[KT4][4][GP];
#pragma unroll
  for (int j = 0; j < KT4; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int g = 0; g < GP; ++g) acc[j][i][g] = 0.f;

  uint4 nxt[KT4];
#pragma unroll
  for (int j = 0; j < KT4; ++j)
    nxt[j] = live[j] ? *reinterpret_cast<const uint4*>(codes_pair + tbase[j]) : make_uint4(0, 0, 0, 0);

  for (int w0 = 0; w0 < NW; w0 += chunk_words) {
    const int l0 = w0 * cpw;
    const int nt = min(chunk_words * cpw, L - l0);
    __syncthreads();  // gathers of the previous slice are done
    {
      // Slice fill: for each head g the nt*R floats are contiguous in q_probs.
      const int n4 = (nt * R) >> 2;
      const float* src = qp_pair + (int64_t)l0 * R;
      for (int i4 = tid; i4 < n4; i4 += THREADS) {
        float4 x[GP];
#pragma unroll
        for (int g = 0; g < GP; ++g)
          x[g] = (g < G) ? *reinterpret_cast<const float4*>(src + (int64_t)g * L * R + 4 * i4)
                         : make_float4(0.f, 0.f, 0.f, 0.f);
        LdsEntry<GP> e[4];
#pragma unroll
        for (int g = 0; g < GP; ++g) {
          e[0].v[g] = x[g].x;
          e[1].v[g] = x[g].y;
          e[2].v[g] = x[g].z;
          e[3].v[g] = x[g].w;
        }
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) table[4 * i4 + rr] = e[rr];
      }
    }
    __syncthreads();

    const int wend = min(w0 + chunk_words, NW);
    for (int w = w0; w < wend; ++w) {
      uint4 cur[KT4];
#pragma unroll
      for (int j = 0; j < KT4; ++j) cur[j] = nxt[j];
      if (w + 1 < NW) {
        const uint32_t* row = codes_pair + (int64_t)(w + 1) * Tcap;
#pragma unroll
        for (int j = 0; j < KT4; ++j)
          if (live[j]) nxt[j] = *reinterpret_cast<const uint4*>(row + tbase[j]);
      }
      const int ntw = min(cpw, L - w * cpw);
      const int ent0 = (w - w0) * cpw * R;
#pragma unroll
      for (int jj = 0; jj < (PT ? 32 / PT : 32); ++jj) {
        if (jj >= ntw) break;
        const LdsEntry<GP>* tb = table + ent0 + jj * R;
        const int sh = jj * P;
#pragma unroll
        for (int j = 0; j < KT4; ++j) {
          const uint32_t wv[4] = {cur[j].x, cur[j].y, cur[j].z, cur[j].w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t code = (wv[i] >> sh) & code_mask;
            const LdsEntry<GP> e = tb[code];
#pragma unroll
            for (int g = 0; g < GP; ++g) acc[j][i][g] += e.v[g];
          }
        }
      }
    }
  }

  // epilogue: multiply by the value norm, mask, store one float4 per head
  const uint16_t* vn_pair = v_norm + (int64_t)pair * Tcap;
#pragma unroll
  for (int j = 0; j < KT4; ++j) {
    if (!live[j]) continue;
    const uint2 vraw = *reinterpret_cast<const uint2*>(vn_pair + tbase[j]);
    float vn[4];
    vn[0] = f16_bits_to_f32((uint16_t)(vraw.x & 0xffffu));
    vn[1] = f16_bits_to_f32((uint16_t)(vraw.x >> 16));
    vn[2] = f16_bits_to_f32((uint16_t)(vraw.y & 0xffffu));
    vn[3] = f16_bits_to_f32((uint16_t)(vraw.y >> 16));
#pragma unroll
    for (int g = 0; g < GP; ++g) {
      if (g >= G) break;
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o[i] = (tbase[j] + i < len) ? acc[j][i][g] * vn[i] : -INFINITY;
      float* dst = scores + ((int64_t)(b * Hq + kvh * G + g)) * score_stride + tbase[j];
      if (tbase[j] + 4 <= T) {
        *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
      } else {
        for (int i = 0; i < 4 && tbase[j] + i < T; ++i) dst[i] = o[i];
      }
    }
  }
}

template <int GP, int KT4, int THREADS, int PT>
int launch_score_packed(const float* q_probs, const uint32_t* codes, const uint16_t* v_norm,
                        const int32_t* lens, float* scores, int B, int Hq, int Hkv, int L, int P,
                        int R, int T, int64_t Tcap, int64_t score_stride, hipStream_t stream) {
  const SocketDeviceLimits& lim = socket_device_limits();
  const int G = Hq / Hkv;
  const int cpw = 32 / P;
  const int NW = (L + cpw - 1) / cpw;
  const size_t bytes_per_word = (size_t)cpw * R * GP * sizeof(float);
  // Slice size: as many words as fit a third of the CU's LDS (three resident
  // workgroups overlap one another's slice fills), at least one word.
  size_t budget = (size_t)lim.max_lds_per_block / 3;
  int chunk_words = (int)(budget / bytes_per_word);
  if (chunk_words < 1) chunk_words = 1;
  if (chunk_words > NW) chunk_words = NW;
  const size_t lds_bytes = bytes_per_word * chunk_words;
  if (lds_bytes > (size_t)lim.max_lds_per_block) return SOCKET_ERR_UNSUPPORTED;

  auto kern = score_packed_kernel<GP, KT4, THREADS, PT>;
  if (lds_bytes > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
      return SOCKET_ERR_LAUNCH;
  }
  constexpr int TW = THREADS * 4 * KT4;
  const int n_tiles = (T + TW - 1) / TW;
  const int n_pairs = B * Hkv;
  const int xcd_remap = (n_pairs % 8 == 0) ? 1 : 0;
  const int n_wg = n_pairs * n_tiles;
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(THREADS), lds_bytes, stream, q_probs, codes, v_norm,
                     lens, scores, Hq, Hkv, G, L, P, R, T, Tcap, score_stride, NW, chunk_words,
                     n_pairs, n_tiles, xcd_remap);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

template <int GP, int KT4>
int dispatch_p(const float* q_probs, const uint32_t* codes, const uint16_t* v_norm,
               const int32_t* lens, float* scores, int B, int Hq, int Hkv, int L, int P, int R,
               int T, int64_t Tcap, int64_t score_stride, hipStream_t stream) {
#define SOCKET_SCORE_ARGS q_probs, codes, v_norm, lens, scores, B, Hq, Hkv, L, P, R, T, Tcap, score_stride, stream
  if (P == 10) return launch_score_packed<GP, KT4, 512, 10>(SOCKET_SCORE_ARGS);
  if (P == 8) return launch_score_packed<GP, KT4, 512, 8>(SOCKET_SCORE_ARGS);
  return launch_score_packed<GP, KT4, 512, 0>(SOCKET_SCORE_ARGS);
#undef SOCKET_SCORE_ARGS
}

// ---------------------------------------------------------------------------
// reference-layout scorer (int16 codes per query head)
// ---------------------------------------------------------------------------
__device__ __forceinline__ float table_to_f32(float x) { return x; }
__device__ __forceinline__ float table_to_f32(uint16_t x) { return f16_bits_to_f32(x); }

// One thread per token; tables staged in LDS in slices of `ct` tables
// (ct == 0: R too large for LDS, gather from global memory instead).
template <typename QT, int THREADS>
__global__ __launch_bounds__(THREADS) void collision_i16_kernel(
    const QT* __restrict__ q_probs, const int16_t* __restrict__ key_buckets,
    const uint8_t* __restrict__ allowed, const QT* __restrict__ v_hist, float* __restrict__ out,
    int L, int R, int T, int ct) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  QT* table = reinterpret_cast<QT*>(lds_raw);
  const int bh = blockIdx.y;
  const int t = blockIdx.x * THREADS + threadIdx.x;
  const bool in = t < T;
  const QT* qp = q_probs + (int64_t)bh * L * R;
  const int16_t* kb = key_buckets + (int64_t)bh * L * T;
  float sum = 0.f;
  if (ct == 0) {
    if (in) {
      for (int l = 0; l < L; ++l) {
        const int r = (int)kb[(int64_t)l * T + t];
        if (r >= 0 && r < R) sum += table_to_f32(qp[(int64_t)l * R + r]);
      }
    }
  } else {
    for (int l0 = 0; l0 < L; l0 += ct) {
      const int nt = min(ct, L - l0);
      __syncthreads();
      for (int i = threadIdx.x; i < nt * R; i += THREADS) table[i] = qp[(int64_t)l0 * R + i];
      __syncthreads();
      if (in) {
        for (int l = 0; l < nt; ++l) {
          const int r = (int)kb[(int64_t)(l0 + l) * T + t];
          if (r >= 0 && r < R) sum += table_to_f32(table[l * R + r]);
        }
      }
    }
  }
  if (in) {
    const int64_t o = (int64_t)bh * T + t;
    out[o] = allowed[o] ? sum * table_to_f32(v_hist[o]) : -INFINITY;
  }
}

template <typename QT>
int launch_collision_i16(const QT* q_probs, const int16_t* key_buckets, const uint8_t* allowed,
                         const QT* v_hist, float* out, int B, int H, int L, int R, int T,
                         hipStream_t stream) {
  constexpr int THREADS = 256;
  const size_t per_table = (size_t)R * sizeof(QT);
  int ct = (int)((48 * 1024) / per_table);
  if (ct > L) ct = L;
  const size_t lds = (size_t)ct * per_table;
  dim3 grid((T + THREADS - 1) / THREADS, B * H);
  hipLaunchKernelGGL((collision_i16_kernel<QT, THREADS>), grid, dim3(THREADS), lds, stream, q_probs,
                     key_buckets, allowed, v_hist, out, L, R, T, ct);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

}  // namespace

extern "C" int socket_score_packed(const void* q_probs, int q_dtype, const uint32_t* codes,
                                   const uint16_t* v_norm, const int32_t* lens, float* scores,
                                   int B, int Hq, int Hkv, int L, int P, int R, int T,
                                   int64_t Tcap, int64_t score_stride, void* stream) {
  SOCKET_REQUIRE(q_probs && codes && v_norm && scores, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(q_dtype == SOCKET_F32, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && L > 0 && T > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(Hq % Hkv == 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(P >= 1 && P <= 16, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(R >= (1 << P) && (R & (R - 1)) == 0 && R >= 4, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(T <= Tcap && score_stride >= T, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE((int64_t)B * Hkv * ((T + 2047) / 2048) < (1LL << 31), SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(Tcap % 4 == 0 && score_stride % 4 == 0, SOCKET_ERR_ALIGN);
  SOCKET_REQUIRE(socket_aligned16(q_probs) && socket_aligned16(codes) && socket_aligned16(v_norm) &&
                     socket_aligned16(scores),
                 SOCKET_ERR_ALIGN);
  const int G = Hq / Hkv;
  SOCKET_REQUIRE(G <= 8, SOCKET_ERR_UNSUPPORTED);
  hipStream_t s = (hipStream_t)stream;
  const float* qp = (const float*)q_probs;
#define SOCKET_SCORE_ARGS qp, codes, v_norm, lens, scores, B, Hq, Hkv, L, P, R, T, Tcap, score_stride, s
  // 8 tokens per thread once the context is long enough to fill the chip with
  // 4096-token tiles, 4 per thread below that.
  const bool big = (int64_t)B * Hkv * ((T + 4095) / 4096) >= 512;
  if (G == 1) return big ? dispatch_p<1, 2>(SOCKET_SCORE_ARGS) : dispatch_p<1, 1>(SOCKET_SCORE_ARGS);
  if (G == 2) return big ? dispatch_p<2, 2>(SOCKET_SCORE_ARGS) : dispatch_p<2, 1>(SOCKET_SCORE_ARGS);
  if (G <= 4) return big ? dispatch_p<4, 2>(SOCKET_SCORE_ARGS) : dispatch_p<4, 1>(SOCKET_SCORE_ARGS);
  return big ? dispatch_p<8, 2>(SOCKET_SCORE_ARGS) : dispatch_p<8, 1>(SOCKET_SCORE_ARGS);
#undef SOCKET_SCORE_ARGS
}

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
