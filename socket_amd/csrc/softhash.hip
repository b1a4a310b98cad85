// K5: query soft hash -- the producer of the scorer's bucket-probability table.
//
//   proj[l,k]  = q . planes[l,k,:]
//   t[k]       = tanh(proj[l,k]) * tanh_scale            (tanh_scale = 1 / sqrt(D))
//   logit[l,r] = inv_temperature * sum_k t[k] * protos_T[k,r]
//   probs[l,:] = softmax_r(logit[l,:])
//
// GPT-FAST/model.py:392-401 (inv_temperature 1) and the HuggingFace twin
// pipeline/train_quest/modeling/modeling_llama.py:618-638 (logits / 0.3), which
// run this as two einsums, a tanh, a division and a softmax, five launches with
// [B,H,L,K] and [B,H,L,R] intermediates rounded to the model dtype.  Here it is
// one launch computing in fp32 from the inputs as stored and rounding once, to
// the output dtype.
//
// One workgroup per (table l, batch b, KV head): the K planes of the table and
// the G query heads of the group sit in LDS, G*K lanes take the projections,
// then every lane owns runs of four buckets and makes three sweeps over them
// (maximum, sum of exponentials, normalised write), recomputing the K-term
// logits each time rather than holding R/64 of them per head in registers.
#include <type_traits>

#include "socket_common.h"

namespace {

constexpr int kSHThreads = 256;
constexpr int kSHWaves = kSHThreads / SOCKET_WAVE;
constexpr int kSHMaxK = 16;
constexpr int kSHMaxG = 8;
constexpr int kSHMaxD = 256;

template <class DT>
__device__ __forceinline__ float sh_load(const void* p, int64_t i);
template <>
__device__ __forceinline__ float sh_load<DType_f32>(const void* p, int64_t i) {
  return ((const float*)p)[i];
}
template <>
__device__ __forceinline__ float sh_load<DType_bf16>(const void* p, int64_t i) {
  return bf16_bits_to_f32(((const uint16_t*)p)[i]);
}
template <>
__device__ __forceinline__ float sh_load<DType_f16>(const void* p, int64_t i) {
  return f16_bits_to_f32(((const uint16_t*)p)[i]);
}

// Four consecutive elements starting at index i (the address must be aligned to
// the size of the four).
template <class DT>
__device__ __forceinline__ void sh_load4(const void* p, int64_t i, float (&o)[4]);
template <>
__device__ __forceinline__ void sh_load4<DType_f32>(const void* p, int64_t i, float (&o)[4]) {
  const float4 v = *reinterpret_cast<const float4*>((const float*)p + i);
  o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
}
template <>
__device__ __forceinline__ void sh_load4<DType_bf16>(const void* p, int64_t i, float (&o)[4]) {
  const uint2 v = *reinterpret_cast<const uint2*>((const uint16_t*)p + i);
  o[0] = bf16_bits_to_f32(v.x & 0xffffu); o[1] = bf16_bits_to_f32(v.x >> 16);
  o[2] = bf16_bits_to_f32(v.y & 0xffffu); o[3] = bf16_bits_to_f32(v.y >> 16);
}
template <>
__device__ __forceinline__ void sh_load4<DType_f16>(const void* p, int64_t i, float (&o)[4]) {
  const uint2 v = *reinterpret_cast<const uint2*>((const uint16_t*)p + i);
  o[0] = f16_bits_to_f32((uint16_t)(v.x & 0xffffu)); o[1] = f16_bits_to_f32((uint16_t)(v.x >> 16));
  o[2] = f16_bits_to_f32((uint16_t)(v.y & 0xffffu)); o[3] = f16_bits_to_f32((uint16_t)(v.y >> 16));
}

// GC: heads per group the registers are sized for (4 or 8).  KC: K when known at
// compile time (then, with a single sweep, a lane's 4 x K prototype entries are
// fetched straight into registers at kernel entry: no LDS copy of the prototypes,
// a small LDS footprint and several workgroups per CU), 0 = runtime K.
// LDS (dynamic): qs [G][D] | ps [K][D+1] | ts [G][K] | red [waves][GC] | protos [K][R] (optional)
template <class DT, int GC, int KC>
__global__ __launch_bounds__(kSHThreads) void soft_hash_kernel(
    const void* __restrict__ q, int64_t q_sb, int64_t q_sh, const void* __restrict__ planes,
    const void* __restrict__ protos_T, void* __restrict__ out, int out_dtype, int Hq, int Hkv, int G,
    int D, int L, int K, int R, float tanh_scale, float inv_temperature, int parts, int width,
    int protos_in_lds, int vec_ok) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;
  float* ps = qs + G * D;
  float* ts = ps + ((K * (D + 1) + 3) / 4) * 4;   // (16-byte aligned when G * D is a multiple of 4: read as float4)
  float* red = ts + ((G * K + 3) / 4) * 4;
  float* protos_lds = lds + ((G * D + ((K * (D + 1) + 3) / 4) * 4 + ((G * K + 3) / 4) * 4 + kSHWaves * GC + 3) / 4) * 4;
  const int DP = D + 1;
  const int l = blockIdx.x, pair = blockIdx.y;
  const int b = pair / Hkv, kvh = pair % Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr bool direct = KC > 0;   // prototypes from global memory into registers, once

  float pk[direct ? KC : 1][4];
  if (direct && tid * 4 < R) {
#pragma unroll
    for (int k = 0; k < KC; ++k) sh_load4<DT>(protos_T, (int64_t)k * R + tid * 4, pk[k]);
  }

  if (vec_ok) {
    // Staging with every global load issued before the first LDS store: the whole
    // set-up costs one memory latency.  (A load-convert-store loop exposes one per
    // iteration.)
    constexpr int QV = kSHMaxG * kSHMaxD / 4 / kSHThreads;   // vectors of four per lane
    constexpr int PV = kSHMaxK * kSHMaxD / 4 / kSHThreads;
    constexpr int RV = direct ? 1 : 10;                       // prototype vectors per batch
    float qv[QV][4], pv[PV][4], rv[RV][4];
    const int nr4 = (!direct && protos_in_lds) ? K * R / 4 : 0;
#pragma unroll
    for (int u = 0; u < QV; ++u) {
      const int i = (tid + u * kSHThreads) * 4;
      if (i < G * D) sh_load4<DT>(q, b * q_sb + (int64_t)(kvh * G + i / D) * q_sh + i % D, qv[u]);
    }
#pragma unroll
    for (int u = 0; u < PV; ++u) {
      const int i = (tid + u * kSHThreads) * 4;
      if (i < K * D) sh_load4<DT>(planes, (int64_t)l * K * D + i, pv[u]);
    }
    if (!direct) {
#pragma unroll
      for (int u = 0; u < RV; ++u) {
        const int i = tid + u * kSHThreads;
        if (i < nr4) sh_load4<DT>(protos_T, (int64_t)i * 4, rv[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < QV; ++u) {
      const int i = (tid + u * kSHThreads) * 4;
      if (i < G * D) {
#pragma unroll
        for (int e = 0; e < 4; ++e) qs[i + e] = qv[u][e];
      }
    }
#pragma unroll
    for (int u = 0; u < PV; ++u) {
      const int i = (tid + u * kSHThreads) * 4;
      if (i < K * D) {
#pragma unroll
        for (int e = 0; e < 4; ++e) ps[(i / D) * DP + i % D + e] = pv[u][e];
      }
    }
    if (!direct) {
#pragma unroll
      for (int u = 0; u < RV; ++u) {
        const int i = tid + u * kSHThreads;
        if (i < nr4) *reinterpret_cast<float4*>(protos_lds + (size_t)i * 4) = make_float4(rv[u][0], rv[u][1], rv[u][2], rv[u][3]);
      }
      // (prototype tables beyond one batch: the rest in further batches)
      for (int i0 = RV * kSHThreads; i0 < nr4; i0 += RV * kSHThreads) {
#pragma unroll
        for (int u = 0; u < RV; ++u) {
          const int i = i0 + tid + u * kSHThreads;
          if (i < nr4) sh_load4<DT>(protos_T, (int64_t)i * 4, rv[u]);
        }
#pragma unroll
        for (int u = 0; u < RV; ++u) {
          const int i = i0 + tid + u * kSHThreads;
          if (i < nr4) *reinterpret_cast<float4*>(protos_lds + (size_t)i * 4) = make_float4(rv[u][0], rv[u][1], rv[u][2], rv[u][3]);
        }
      }
    }
  } else {
    for (int i = tid; i < G * D; i += kSHThreads) {
      const int g = i / D, d = i % D;
      qs[i] = sh_load<DT>(q, b * q_sb + (int64_t)(kvh * G + g) * q_sh + d);
    }
    for (int i = tid; i < K * D; i += kSHThreads) ps[(i / D) * DP + i % D] = sh_load<DT>(planes, (int64_t)l * K * D + i);
    if (protos_in_lds)
      for (int i = tid; i < K * R; i += kSHThreads) protos_lds[i] = sh_load<DT>(protos_T, i);
  }
  __syncthreads();
  // projections: four lanes per (head, plane) pair, a quarter of the dimension each
  for (int p0 = 0; p0 < G * K; p0 += kSHThreads / 4) {
    const int p = p0 + tid / 4, part = tid % 4;
    float s = 0.f;
    if (p < G * K) {
      const float* qrow = qs + (p / K) * D;
      const float* prow = ps + (p % K) * DP;
#pragma unroll 8
      for (int d = part; d < D; d += 4) s += qrow[d] * prow[d];
    }
    s += __shfl_xor(s, 1, SOCKET_WAVE);
    s += __shfl_xor(s, 2, SOCKET_WAVE);
    if (p < G * K && part == 0) ts[p] = tanhf(s) * tanh_scale * inv_temperature;   // ts[g][k], p = g*K + k
  }
  __syncthreads();

  // logits of buckets r0..r0+3 for every head of the group
  auto logits4 = [&](int r0, float (&lg)[GC][4]) {
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) lg[g][i] = 0.f;
    auto add_plane = [&](int k, const float (&pr)[4]) {
#pragma unroll
      for (int g = 0; g < GC; ++g) {
        if (g < G) {
          const float t = ts[g * K + k];
#pragma unroll
          for (int i = 0; i < 4; ++i) lg[g][i] += t * pr[i];
        }
      }
    };
    if constexpr (direct) {
      // the G x K scaled projections as a handful of 16-byte broadcast reads instead
      // of one LDS read per (head, plane) term
      if ((G * D) % 4 == 0) {
        constexpr int NV = (GC * (KC > 0 ? KC : 1) + 3) / 4;
        float tv[NV * 4];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          const float4 t4 = (i * 4 < G * K) ? *reinterpret_cast<const float4*>(ts + i * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
          tv[4 * i] = t4.x, tv[4 * i + 1] = t4.y, tv[4 * i + 2] = t4.z, tv[4 * i + 3] = t4.w;
        }
#pragma unroll
        for (int g = 0; g < GC; ++g) {
          if (g < G) {
#pragma unroll
            for (int k = 0; k < KC; ++k) {
              const float t = tv[g * KC + k];
#pragma unroll
              for (int i = 0; i < 4; ++i) lg[g][i] += t * pk[k][i];
            }
          }
        }
      } else {
#pragma unroll
        for (int k = 0; k < KC; ++k) add_plane(k, pk[k]);
      }
    } else {
      for (int k = 0; k < K; ++k) {
        float pr[4];
        if (protos_in_lds) {
          const float4 v = *reinterpret_cast<const float4*>(protos_lds + (size_t)k * R + r0);
          pr[0] = v.x;
          pr[1] = v.y;
          pr[2] = v.z;
          pr[3] = v.w;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) pr[i] = sh_load<DT>(protos_T, (int64_t)k * R + r0 + i);
        }
        add_plane(k, pr);
      }
    }
  };
  // workgroup-wide reduction of one value per head; every lane gets the result
  auto reduce = [&](float (&v)[GC], bool is_max) {
#pragma unroll
    for (int g = 0; g < GC; ++g) {
#pragma unroll
      for (int d = SOCKET_WAVE / 2; d > 0; d >>= 1) {
        const float o = __shfl_xor(v[g], d, SOCKET_WAVE);
        v[g] = is_max ? fmaxf(v[g], o) : v[g] + o;
      }
    }
    __syncthreads();  // earlier readers of `red` are done
    if (lane == 0) {
#pragma unroll
      for (int g = 0; g < GC; ++g) red[wave * GC + g] = v[g];
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < GC; ++g) {
      float a = red[g];
#pragma unroll
      for (int w = 1; w < kSHWaves; ++w) a = is_max ? fmaxf(a, red[w * GC + g]) : a + red[w * GC + g];
      v[g] = a;
    }
  };

  // With R <= 1024 a lane owns a single run of four buckets: its logits are
  // computed once and kept; otherwise each sweep recomputes them.
  const bool keep = direct || R <= kSHThreads * 4;
  float lg[GC][4];
  float mx[GC], sm[GC];
#pragma unroll
  for (int g = 0; g < GC; ++g) {
    mx[g] = -INFINITY;
    sm[g] = 0.f;
  }
  for (int r0 = tid * 4; r0 < R; r0 += kSHThreads * 4) {
    logits4(r0, lg);
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) mx[g] = fmaxf(mx[g], lg[g][i]);
  }
  reduce(mx, true);
  for (int r0 = tid * 4; r0 < R; r0 += kSHThreads * 4) {
    if (!keep) logits4(r0, lg);
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float e = expf(lg[g][i] - mx[g]);
        sm[g] += e;
        if (keep) lg[g][i] = e;   // kept for the write sweep
      }
  }
  reduce(sm, false);
  for (int r0 = tid * 4; r0 < R; r0 += kSHThreads * 4) {
    if (!keep) logits4(r0, lg);
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i)   // now probabilities
        lg[g][i] = (g < G) ? (keep ? lg[g][i] : expf(lg[g][i] - mx[g])) / sm[g] : 0.f;
    if (parts == 0) {
      // reference layout [B,Hq,L,R]
#pragma unroll
      for (int g = 0; g < GC; ++g) {
        if (g < G) {
          const int64_t o = (((int64_t)b * Hq + kvh * G + g) * L + l) * R + r0;
          if (out_dtype == SOCKET_F32) {
            *reinterpret_cast<float4*>((float*)out + o) = make_float4(lg[g][0], lg[g][1], lg[g][2], lg[g][3]);
          } else {
            uint2 w;
            w.x = (uint32_t)f32_to_bf16_bits(lg[g][0]) | ((uint32_t)f32_to_bf16_bits(lg[g][1]) << 16);
            w.y = (uint32_t)f32_to_bf16_bits(lg[g][2]) | ((uint32_t)f32_to_bf16_bits(lg[g][3]) << 16);
            *reinterpret_cast<uint2*>((uint16_t*)out + o) = w;
          }
        }
      }
    } else {
      // grouped layout [B*Hkv*parts, L, R, width]: the scorer's LDS image.  Width and
      // part are compile-time in each instance below, so v[] is indexed statically
      // (with a runtime width the compiler kept it in scratch memory).
      auto write_part = [&](auto width_c, auto part_c) {
        constexpr int W = decltype(width_c)::value, PART = decltype(part_c)::value;
        if constexpr (PART * W < GC) {
          const int64_t o = ((((int64_t)pair * parts + PART) * L + l) * R + r0) * W;
          float v[4 * W];  // [bucket][head of this part]: 4 * W consecutive elements of the table
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int gg = 0; gg < W; ++gg) v[i * W + gg] = lg[PART * W + gg][i];
          if (out_dtype == SOCKET_F32) {
#pragma unroll
            for (int c = 0; c < W; ++c)
              *reinterpret_cast<float4*>((float*)out + o + 4 * c) =
                  make_float4(v[4 * c], v[4 * c + 1], v[4 * c + 2], v[4 * c + 3]);
          } else {
            uint32_t w[2 * W];
#pragma unroll
            for (int c = 0; c < 2 * W; ++c)
              w[c] = (uint32_t)f32_to_bf16_bits(v[2 * c]) | ((uint32_t)f32_to_bf16_bits(v[2 * c + 1]) << 16);
            uint16_t* dst = (uint16_t*)out + o;
            if constexpr (W == 4) {
              *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
              *reinterpret_cast<uint4*>(dst + 8) = make_uint4(w[4], w[5], w[6], w[7]);
            } else if constexpr (W == 2) {
              *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
            } else {
              *reinterpret_cast<uint2*>(dst) = make_uint2(w[0], w[1]);
            }
          }
        }
      };
      using std::integral_constant;
      if (width == 4) {
        write_part(integral_constant<int, 4>{}, integral_constant<int, 0>{});
        if (parts > 1) write_part(integral_constant<int, 4>{}, integral_constant<int, 1>{});
      } else if (width == 2) {
        write_part(integral_constant<int, 2>{}, integral_constant<int, 0>{});
      } else {
        write_part(integral_constant<int, 1>{}, integral_constant<int, 0>{});
      }
    }
  }
}

}  // namespace

namespace {

int soft_hash_entry(const void* q, int dtype, int64_t q_stride_b, int64_t q_stride_h, const void* planes,
                    const void* protos_T, void* out, int out_dtype, int B, int Hq, int Hkv, int D, int L, int K,
                    int R, float tanh_scale, float inv_temperature, void* stream, int grouped) {
  SOCKET_REQUIRE(q && planes && protos_T && out, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(socket_dtype_bytes(dtype) != 0, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(out_dtype == SOCKET_F32 || out_dtype == SOCKET_BF16, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && L > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(D >= 1 && D <= kSHMaxD && K >= 1 && K <= kSHMaxK, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(Hq / Hkv <= kSHMaxG, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(R >= 4 && R % 4 == 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE((int64_t)B * Hkv <= 65535, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(socket_aligned16(out), SOCKET_ERR_ALIGN);
  int parts = 0, width = 0;
  if (grouped) {
    const int st = socket_group_shape(Hq, Hkv, &parts, &width);
    if (st != SOCKET_OK) return st;
  }
  const dim3 grid(L, B * Hkv);
  hipStream_t s = (hipStream_t)stream;
  // vector loads of four elements: everything a lane fetches starts at a multiple of four
  const int vec_ok = (D % 4 == 0 && q_stride_b % 4 == 0 && q_stride_h % 4 == 0 && socket_aligned16(q) &&
                      socket_aligned16(planes) && socket_aligned16(protos_T))
                         ? 1
                         : 0;
  const int G = Hq / Hkv;
  // K = 10 with a single sweep (R <= 4 buckets per lane) and vector loads: the
  // prototypes go from global memory straight into registers.  Otherwise they go
  // to LDS as fp32 when they fit in 64 KB, else they are read from global memory
  // in every sweep.
  const bool direct = K == 10 && R <= kSHThreads * 4 && vec_ok;
  const size_t protos_bytes = (size_t)K * R * sizeof(float);
  const int protos_in_lds = (!direct && protos_bytes <= 64 * 1024) ? 1 : 0;
  const int GC = G <= 4 ? 4 : 8;
  const size_t head_floats = (((size_t)G * D + (((size_t)K * (D + 1) + 3) / 4) * 4 + (((size_t)G * K + 3) / 4) * 4 +
                               kSHWaves * GC + 3) / 4) * 4;
  const size_t dyn_lds = head_floats * sizeof(float) + (protos_in_lds ? protos_bytes : 0);
#define SOCKET_SH_LAUNCH(DT, GCV, KCV)                                                                     \
  do {                                                                                                     \
    auto kern = soft_hash_kernel<DT, GCV, KCV>;                                                            \
    if (dyn_lds > 16 * 1024 &&                                                                             \
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                            (int)dyn_lds) != hipSuccess)                                                   \
      return SOCKET_ERR_LAUNCH;                                                                            \
    hipLaunchKernelGGL(kern, grid, dim3(kSHThreads), dyn_lds, s, q, q_stride_b, q_stride_h, planes,        \
                       protos_T, out, out_dtype, Hq, Hkv, G, D, L, K, R, tanh_scale, inv_temperature,       \
                       parts, width, protos_in_lds, vec_ok);                                               \
  } while (0)
#define SOCKET_SH(DT)                                          \
  do {                                                         \
    if (direct) {                                              \
      if (GC == 4) SOCKET_SH_LAUNCH(DT, 4, 10);                \
      else SOCKET_SH_LAUNCH(DT, 8, 10);                        \
    } else {                                                   \
      if (GC == 4) SOCKET_SH_LAUNCH(DT, 4, 0);                 \
      else SOCKET_SH_LAUNCH(DT, 8, 0);                         \
    }                                                          \
  } while (0)
  if (dtype == SOCKET_F32) SOCKET_SH(DType_f32);
  else if (dtype == SOCKET_BF16) SOCKET_SH(DType_bf16);
  else SOCKET_SH(DType_f16);
#undef SOCKET_SH
#undef SOCKET_SH_LAUNCH
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

}  // namespace

extern "C" int socket_soft_hash(const void* q, int dtype, int64_t q_stride_b, int64_t q_stride_h,
                                const void* planes, const void* protos_T, void* out, int out_dtype,
                                int B, int Hq, int Hkv, int D, int L, int K, int R,
                                float tanh_scale, float inv_temperature, void* stream) {
  return soft_hash_entry(q, dtype, q_stride_b, q_stride_h, planes, protos_T, out, out_dtype, B, Hq, Hkv, D, L,
                         K, R, tanh_scale, inv_temperature, stream, 0);
}

extern "C" int socket_soft_hash_grouped(const void* q, int dtype, int64_t q_stride_b, int64_t q_stride_h,
                                        const void* planes, const void* protos_T, void* q_table,
                                        int out_dtype, int B, int Hq, int Hkv, int D, int L, int K, int R,
                                        float tanh_scale, float inv_temperature, void* stream) {
  return soft_hash_entry(q, dtype, q_stride_b, q_stride_h, planes, protos_T, q_table, out_dtype, B, Hq, Hkv, D,
                         L, K, R, tanh_scale, inv_temperature, stream, 1);
}
