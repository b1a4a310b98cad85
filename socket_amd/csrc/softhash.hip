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

// x rounded to the storage type and widened again (what a stored value reads back as)
template <class DT>
__device__ __forceinline__ float sh_round(float x);
template <>
__device__ __forceinline__ float sh_round<DType_f32>(float x) { return x; }
template <>
__device__ __forceinline__ float sh_round<DType_bf16>(float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); }
template <>
__device__ __forceinline__ float sh_round<DType_f16>(float x) { return f16_bits_to_f32(f32_to_f16_bits(x)); }

// Four consecutive elements (already representable in the storage type) to index i.
template <class DT>
__device__ __forceinline__ void sh_store4(void* p, int64_t i, const float (&v)[4]);
template <>
__device__ __forceinline__ void sh_store4<DType_f32>(void* p, int64_t i, const float (&v)[4]) {
  *reinterpret_cast<float4*>((float*)p + i) = make_float4(v[0], v[1], v[2], v[3]);
}
template <>
__device__ __forceinline__ void sh_store4<DType_bf16>(void* p, int64_t i, const float (&v)[4]) {
  *reinterpret_cast<uint2*>((uint16_t*)p + i) =
      make_uint2((uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16),
                 (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16));
}
template <>
__device__ __forceinline__ void sh_store4<DType_f16>(void* p, int64_t i, const float (&v)[4]) {
  *reinterpret_cast<uint2*>((uint16_t*)p + i) =
      make_uint2((uint32_t)f32_to_f16_bits(v[0]) | ((uint32_t)f32_to_f16_bits(v[1]) << 16),
                 (uint32_t)f32_to_f16_bits(v[2]) | ((uint32_t)f32_to_f16_bits(v[3]) << 16));
}

// GC: heads per group the registers are sized for (4 or 8).  KC: K when known at
// compile time (then, with a single sweep, a lane's 4 x K prototype entries are
// fetched straight into registers at kernel entry: no LDS copy of the prototypes,
// a small LDS footprint and several workgroups per CU), 0 = runtime K.
// LDS (dynamic): qs [G][D] | ps [K][D+1] | ts [G][K] | red [waves][GC] | protos [K][R] (optional)
//
// FT: void, or the element type of a rotary table: then the queries arrive
// unrotated (the q part of a fused qkv projection), are rotated by the angles of
// position `rope_pos` (when `rope_on`) and rounded to DT as they are staged, and
// the workgroups of table 0 also write them to `q_out` [B,Hq,D] (vector path only).
template <class DT, int GC, int KC, class FT>
__device__ __forceinline__ void soft_hash_block(
    const int l, const int pair, const void* __restrict__ q, int64_t q_sb, int64_t q_sh,
    const void* __restrict__ planes, const void* __restrict__ protos_T, void* __restrict__ out, int out_dtype,
    int Hq, int Hkv, int G, int D, int L, int K, int R, float tanh_scale, float inv_temperature, int parts,
    int width, int protos_in_lds, int vec_ok, const void* __restrict__ freqs, int64_t rope_pos, bool rope_on,
    void* __restrict__ q_out) {
  constexpr bool kRope = !std::is_void<FT>::value;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;
  float* ps = qs + G * D;
  float* ts = ps + ((K * (D + 1) + 3) / 4) * 4;   // (16-byte aligned when G * D is a multiple of 4: read as float4)
  float* red = ts + ((G * K + 3) / 4) * 4;
  float* protos_lds = lds + ((G * D + ((K * (D + 1) + 3) / 4) * 4 + ((G * K + 3) / 4) * 4 + kSHWaves * GC + 3) / 4) * 4;
  const int DP = D + 1;
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
    float fv[kRope ? QV : 1][4];   // (cos, sin) of the two pairs a vector holds
#pragma unroll
    for (int u = 0; u < QV; ++u) {
      const int i = (tid + u * kSHThreads) * 4;
      if (i < G * D) {
        sh_load4<DT>(q, b * q_sb + (int64_t)(kvh * G + i / D) * q_sh + i % D, qv[u]);
        if constexpr (kRope) {
          // (always fetched, from row 0 when the position is outside the table: a load under a
          // condition would make the compiler wait for every load issued so far, one by one)
          sh_load4<FT>(freqs, ((rope_on ? rope_pos : 0) * (D / 2) + (i % D) / 2) * 2, fv[u]);
        }
      }
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
        if constexpr (kRope) {
          if (rope_on) {
            float re, im;
            rotate_pair(qv[u][0], qv[u][1], fv[u][0], fv[u][1], re, im);
            qv[u][0] = sh_round<DT>(re), qv[u][1] = sh_round<DT>(im);
            rotate_pair(qv[u][2], qv[u][3], fv[u][2], fv[u][3], re, im);
            qv[u][2] = sh_round<DT>(re), qv[u][3] = sh_round<DT>(im);
          }
          if (l == 0) sh_store4<DT>(q_out, ((int64_t)b * Hq + kvh * G + i / D) * D + i % D, qv[u]);
        }
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
    s = group_sum<4>(s);
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
    for (int g = 0; g < GC; ++g) v[g] = is_max ? wave_reduce_to_last<true>(v[g]) : wave_reduce_to_last<false>(v[g]);
    __syncthreads();  // earlier readers of `red` are done
    if (lane == 63) {   // (the reduction leaves a wave's result in its last lane)
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
  // (one reciprocal per head and a product per bucket where there were sixteen divisions a lane:
  // the last write sweep was the longest phase of the workgroup)
  float inv[GC];
#pragma unroll
  for (int g = 0; g < GC; ++g) inv[g] = 1.f / sm[g];
  for (int r0 = tid * 4; r0 < R; r0 += kSHThreads * 4) {
    if (!keep) logits4(r0, lg);
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i)   // now probabilities
        lg[g][i] = (g < G) ? (keep ? lg[g][i] : expf(lg[g][i] - mx[g])) * inv[g] : 0.f;
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

template <class DT, int GC, int KC>
__global__ __launch_bounds__(kSHThreads) void soft_hash_kernel(
    const void* __restrict__ q, int64_t q_sb, int64_t q_sh, const void* __restrict__ planes,
    const void* __restrict__ protos_T, void* __restrict__ out, int out_dtype, int Hq, int Hkv, int G,
    int D, int L, int K, int R, float tanh_scale, float inv_temperature, int parts, int width,
    int protos_in_lds, int vec_ok) {
  soft_hash_block<DT, GC, KC, void>(blockIdx.x, blockIdx.y, q, q_sb, q_sh, planes, protos_T, out, out_dtype, Hq,
                                    Hkv, G, D, L, K, R, tanh_scale, inv_temperature, parts, width, protos_in_lds,
                                    vec_ok, nullptr, 0, false, nullptr);
}

// ---------------------------------------------------------------------------
// The head of a single-token decode step in one launch (bf16, head dimension
// 128): rotary embedding of the new token's query and key, append of the key and
// value to the cache, hash of the new key with the value norm, and the soft hash
// of the rotated query (GPT-FAST/model.py:433-451 and :392-401).  Each of these
// is a few microseconds of dependent latency on its own, so as three launches
// they cost three launch floors; here they are workgroups of one grid:
//
//   blocks [0, n_key_blocks): block (pair, part) has wave w hash packed word
//     4 * part + w of the new key of (sequence, kv head) `pair`; part 0's first
//     wave also writes the K/V rows, the value norm and the cached length;
//   the rest: the soft hash's workgroups (table l, pair), which rotate the
//     queries as they stage them; those of table 0 write the rotated queries.
//
// The key's sign bits come from the same matrix-core contraction as the cache
// hashing kernel's (planes the M operand, the key column 0 of the N operand, the
// k-steps in the same order), so both give the same bits for the same key.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 sh_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float sh_f32x4;
union ShFrag {
  uint4 u;
  sh_bf16x8 v;
};

// eight consecutive table entries (cos, sin of four pairs) as floats
template <class FT>
__device__ __forceinline__ void sh_load8(const void* p, int64_t i, float (&o)[8]);
template <>
__device__ __forceinline__ void sh_load8<DType_bf16>(const void* p, int64_t i, float (&o)[8]) {
  unpack16<DType_bf16>(*reinterpret_cast<const uint4*>((const uint16_t*)p + i), o);
}
template <>
__device__ __forceinline__ void sh_load8<DType_f32>(const void* p, int64_t i, float (&o)[8]) {
  const float4 a = *reinterpret_cast<const float4*>((const float*)p + i);
  const float4 c = *reinterpret_cast<const float4*>((const float*)p + i + 4);
  o[0] = a.x, o[1] = a.y, o[2] = a.z, o[3] = a.w, o[4] = c.x, o[5] = c.y, o[6] = c.z, o[7] = c.w;
}

constexpr int kPrologueD = 128;

template <int GC, class FT>
__global__ __launch_bounds__(kSHThreads) void decode_prologue_kernel(
    const uint16_t* __restrict__ qkv, int64_t qkv_sb, const void* __restrict__ freqs,
    const int64_t* __restrict__ pos, int pos_stride, int64_t n_pos, uint16_t* __restrict__ q_out,
    uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache, int64_t c_sb, int64_t c_sh, int64_t c_ss,
    int32_t* __restrict__ lens, const uint16_t* __restrict__ planes_words, uint32_t* __restrict__ codes,
    uint16_t* __restrict__ v_norm, int NW, int64_t Tcap, const void* __restrict__ planes,
    const void* __restrict__ protos_T, void* __restrict__ q_table, int out_dtype, int Hq, int Hkv, int G, int L,
    int K, int R, float tanh_scale, float inv_temperature, int parts, int width, int word_blocks,
    int n_key_blocks) {
  constexpr int D = kPrologueD;
  const int bx = blockIdx.x;
  if (bx >= n_key_blocks) {
    const int i = bx - n_key_blocks;
    const int l = i % L, pair = i / L;
    const int64_t p = pos[(int64_t)(pair / Hkv) * pos_stride];
    soft_hash_block<DType_bf16, GC, 10, FT>(l, pair, qkv, qkv_sb, D, planes, protos_T, q_table, out_dtype, Hq, Hkv,
                                            G, D, L, K, R, tanh_scale, inv_temperature, parts, width, 0, 1, freqs, p,
                                            p >= 0 && p < n_pos, q_out);
    return;
  }
  const int pair = bx / word_blocks, part = bx % word_blocks;
  const int b = pair / Hkv, kvh = pair % Hkv;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int prow = lane & 15, quarter = lane >> 4;
  const int64_t p = pos[(int64_t)b * pos_stride];
  const bool rope_on = p >= 0 && p < n_pos;               // a position outside the table is not rotated,
  const bool rows_ok = rope_on && p < Tcap;               // one outside the cache or the table writes no K/V row,
  const bool cached = (uint64_t)p < (uint64_t)Tcap;       // one outside the cache no code and no norm
  const int w = part * kSHWaves + wave;
  const bool first = part == 0 && wave == 0;
  if (w >= NW && !first) return;

  // plane fragments of this wave's word (they do not depend on the key: requested first)
  const int pbit0 = 8 * (prow >> 2) + 7 - (prow & 3);
  ShFrag pf[4][2];
  if (w < NW) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) {
        const int col = w * 32 + pbit0 - 4 * mb;
        pf[ks][mb].u = reinterpret_cast<const uint4*>(planes_words)[(int64_t)col * 16 + ks * 4 + quarter];
      }
  }
  // the new key as column 0 of the N operand: lane 16 * quarter holds elements
  // 32 * ks + 8 * quarter .. + 7 of k-step ks, every other column is zero
  const uint16_t* krow = qkv + b * qkv_sb + (int64_t)(Hq + kvh) * D;
  const uint16_t* vrow = qkv + b * qkv_sb + (int64_t)(Hq + Hkv + kvh) * D;
  ShFrag kf[4], vf[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    kf[ks].u = make_uint4(0, 0, 0, 0);
    vf[ks].u = make_uint4(0, 0, 0, 0);
  }
  if (prow == 0) {
    uint4 raw[4];
    float f[4][8];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int e0 = ks * 32 + quarter * 8;
      // (all three fetched whether needed or not -- the angles from row 0 for a position outside
      // the table, the value row by every wave: loads under a condition are waited for one by one)
      raw[ks] = *reinterpret_cast<const uint4*>(krow + e0);
      sh_load8<FT>(freqs, (rope_on ? p : 0) * D + e0, f[ks]);   // ((p * D/2) + e0/2) * 2
      vf[ks].u = *reinterpret_cast<const uint4*>(vrow + e0);
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (rope_on) {
        float x[8];
        unpack16<DType_bf16>(raw[ks], x);
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float re, im;
          rotate_pair(x[2 * j], x[2 * j + 1], f[ks][2 * j], f[ks][2 * j + 1], re, im);
          o[j] = (uint32_t)f32_to_bf16_bits(re) | ((uint32_t)f32_to_bf16_bits(im) << 16);
        }
        kf[ks].u = make_uint4(o[0], o[1], o[2], o[3]);
      } else {
        kf[ks].u = raw[ks];
      }
    }
    if (first && rows_ok) {
      uint16_t* kdst = k_cache + b * c_sb + kvh * c_sh + p * c_ss;
      uint16_t* vdst = v_cache + b * c_sb + kvh * c_sh + p * c_ss;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int e0 = ks * 32 + quarter * 8;
        *reinterpret_cast<uint4*>(kdst + e0) = kf[ks].u;
        *reinterpret_cast<uint4*>(vdst + e0) = vf[ks].u;
      }
    }
  }
  if (first) {
    // the cached length follows the position
    if (kvh == 0 && lane == 0 && rows_ok && lens) lens[b] = (int32_t)p + 1;
    // ||v||^2 = element (0, 0) of the value column against itself: register 0 of lane 0
    sh_f32x4 g = sh_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) g = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[ks].v, vf[ks].v, g, 0, 0, 0);
    if (lane == 0 && cached) v_norm[(int64_t)pair * Tcap + p] = f32_to_f16_bits(sqrtf(g[0]));
  }
  if (w < NW) {
    sh_f32x4 acc[2] = {sh_f32x4{0.f, 0.f, 0.f, 0.f}, sh_f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[ks][mb].v, kf[ks].v, acc[mb], 0, 0, 0);
    // register r of block mb in lane quarter q is the plane at bit 8q + 7 - 4mb - r
    uint32_t neg = 0;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 4; ++r) neg = __builtin_amdgcn_alignbit(neg, __float_as_uint(acc[mb][r]), 31);
    const uint32_t word = (__builtin_amdgcn_readlane(neg, 0) & 0xffu) | ((__builtin_amdgcn_readlane(neg, 16) & 0xffu) << 8) |
                          ((__builtin_amdgcn_readlane(neg, 32) & 0xffu) << 16) |
                          ((__builtin_amdgcn_readlane(neg, 48) & 0xffu) << 24);
    const int cpw = 32 / K;
    const int nbits = min(cpw, L - w * cpw) * K;
    const uint32_t valid = nbits >= 32 ? 0xffffffffu : ((1u << nbits) - 1u);
    if (lane == 0 && cached) codes[((int64_t)pair * NW + w) * Tcap + p] = ~word & valid;
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

extern "C" int socket_decode_prologue(const void* qkv, int dtype, int64_t qkv_stride_b, const void* freqs_cis,
                                      int freqs_dtype, int64_t n_pos, const int64_t* pos, int pos_stride,
                                      void* q_out, void* k_cache, void* v_cache, int64_t cache_stride_b,
                                      int64_t cache_stride_h, int64_t cache_stride_s, int32_t* lens,
                                      const void* planes_words, void* codes, void* v_norm, const void* planes,
                                      const void* protos_T, void* q_table, int out_dtype, int grouped, int B,
                                      int Hq, int Hkv, int D, int L, int K, int R, int64_t Tcap,
                                      float tanh_scale, float inv_temperature, void* stream) {
  SOCKET_REQUIRE(qkv && freqs_cis && pos && q_out && k_cache && v_cache && planes_words && codes && v_norm &&
                     planes && protos_T && q_table,
                 SOCKET_ERR_NULL);
  // the shapes the fused launch is written for; anything else takes the separate entry points
  SOCKET_REQUIRE(dtype == SOCKET_BF16 && D == kPrologueD && K == 10, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(freqs_dtype == SOCKET_F32 || freqs_dtype == SOCKET_BF16, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(out_dtype == SOCKET_F32 || out_dtype == SOCKET_BF16, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && L > 0 && Tcap > 0 && n_pos > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(Hq / Hkv <= kSHMaxG, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(R >= 4 && R % 4 == 0 && R <= kSHThreads * 4, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(pos_stride == 0 || pos_stride == 1, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(qkv_stride_b % 8 == 0 && cache_stride_b % 8 == 0 && cache_stride_h % 8 == 0 &&
                     cache_stride_s % 8 == 0,
                 SOCKET_ERR_ALIGN);
  SOCKET_REQUIRE(socket_aligned16(qkv) && socket_aligned16(freqs_cis) && socket_aligned16(q_out) &&
                     socket_aligned16(k_cache) && socket_aligned16(v_cache) && socket_aligned16(planes_words) &&
                     socket_aligned16(planes) && socket_aligned16(protos_T) && socket_aligned16(q_table),
                 SOCKET_ERR_ALIGN);
  int parts = 0, width = 0;
  if (grouped) {
    const int st = socket_group_shape(Hq, Hkv, &parts, &width);
    if (st != SOCKET_OK) return st;
  }
  const int G = Hq / Hkv, GC = G <= 4 ? 4 : 8;
  const int cpw = 32 / K, NW = (L + cpw - 1) / cpw;
  const int word_blocks = (NW + kSHWaves - 1) / kSHWaves;
  const int64_t n_key_blocks = (int64_t)B * Hkv * word_blocks;
  const int64_t n_blocks = n_key_blocks + (int64_t)B * Hkv * L;
  SOCKET_REQUIRE(n_blocks < (1LL << 31), SOCKET_ERR_SHAPE);
  const size_t head_floats = (((size_t)G * D + (((size_t)K * (D + 1) + 3) / 4) * 4 + (((size_t)G * K + 3) / 4) * 4 +
                               kSHWaves * GC + 3) / 4) * 4;
  const size_t dyn_lds = head_floats * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
#define SOCKET_DP(GCV, FT)                                                                                      \
  hipLaunchKernelGGL((decode_prologue_kernel<GCV, FT>), dim3((unsigned)n_blocks), dim3(kSHThreads), dyn_lds, s, \
                     (const uint16_t*)qkv, qkv_stride_b, freqs_cis, pos, pos_stride, n_pos, (uint16_t*)q_out,   \
                     (uint16_t*)k_cache, (uint16_t*)v_cache, cache_stride_b, cache_stride_h, cache_stride_s,    \
                     lens, (const uint16_t*)planes_words, (uint32_t*)codes, (uint16_t*)v_norm, NW, Tcap,        \
                     planes, protos_T, q_table, out_dtype, Hq, Hkv, G, L, K, R, tanh_scale, inv_temperature,    \
                     parts, width, word_blocks, (int)n_key_blocks)
  if (GC == 4) {
    if (freqs_dtype == SOCKET_F32) SOCKET_DP(4, DType_f32);
    else SOCKET_DP(4, DType_bf16);
  } else {
    if (freqs_dtype == SOCKET_F32) SOCKET_DP(8, DType_f32);
    else SOCKET_DP(8, DType_bf16);
  }
#undef SOCKET_DP
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}
