// K1: key hashing.  codes = pack(sign(keys . planes^T)) with the value norm fused.
//
// Replaces hard_hash_keys + pack_bits (GPT-FAST/model.py:403-413): the einsum
// that materialises [B,S,Hkv,L,P] projections, the bool compare and the int16
// weighted sum become one MFMA contraction whose epilogue is a wave ballot.
//
// The hyperplanes are pre-ordered (socket_permute_planes) so that column
// w*32 + p of the contraction is the plane whose sign is bit p of packed word w.
// With keys as the M operand and planes as the N operand of
// v_mfma_f32_32x32x16_bf16, accumulator register r of lane x holds
//   key row 8*(r/4) + 4*(x/32) + r%4,  column x%32,
// so ballot(acc[r] >= 0) is, in its low and high halves, the complete packed
// word w of two keys: no bit shuffling, no LDS round trip.  The words of 32
// consecutive keys are gathered into lanes 0..31 and stored as one 128-byte
// run of the table-major code cache.
//
// A wave owns 64 consecutive keys of one (b, kv head) (two 32-row M tiles) at a
// time and keeps their A fragments in registers for the whole column sweep; the
// planes sit in LDS (all NW words when NW*8 KB fits, which L=60 x P=10 exactly
// does at 160 KB) and workgroups are persistent, so the planes are fetched once
// per CU, not once per tile.
#include "socket_common.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;

constexpr int kHashThreads = 512;
constexpr int kHashWaves = kHashThreads / SOCKET_WAVE;
constexpr int kKeysPerWave = 64;
constexpr int kD = 128;
constexpr int kKSteps = kD / 16;  // MFMA k-steps

union Frag {
  uint4 u;
  bf16x8 v;
};

// 8 consecutive elements starting at `p` as a bf16x8 fragment.
template <class DT>
__device__ __forceinline__ uint4 load_frag8(const typename DT::storage* p);
template <>
__device__ __forceinline__ uint4 load_frag8<DType_bf16>(const uint16_t* p) {
  return *reinterpret_cast<const uint4*>(p);
}
template <>
__device__ __forceinline__ uint4 load_frag8<DType_f32>(const float* p) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 c = *reinterpret_cast<const float4*>(p + 4);
  uint4 r;
  r.x = (uint32_t)f32_to_bf16_bits(a.x) | ((uint32_t)f32_to_bf16_bits(a.y) << 16);
  r.y = (uint32_t)f32_to_bf16_bits(a.z) | ((uint32_t)f32_to_bf16_bits(a.w) << 16);
  r.z = (uint32_t)f32_to_bf16_bits(c.x) | ((uint32_t)f32_to_bf16_bits(c.y) << 16);
  r.w = (uint32_t)f32_to_bf16_bits(c.z) | ((uint32_t)f32_to_bf16_bits(c.w) << 16);
  return r;
}
template <>
__device__ __forceinline__ uint4 load_frag8<DType_f16>(const uint16_t* p) {
  const uint4 raw = *reinterpret_cast<const uint4*>(p);
  float f[8];
  unpack16<DType_f16>(raw, f);
  uint4 r;
  r.x = (uint32_t)f32_to_bf16_bits(f[0]) | ((uint32_t)f32_to_bf16_bits(f[1]) << 16);
  r.y = (uint32_t)f32_to_bf16_bits(f[2]) | ((uint32_t)f32_to_bf16_bits(f[3]) << 16);
  r.z = (uint32_t)f32_to_bf16_bits(f[4]) | ((uint32_t)f32_to_bf16_bits(f[5]) << 16);
  r.w = (uint32_t)f32_to_bf16_bits(f[6]) | ((uint32_t)f32_to_bf16_bits(f[7]) << 16);
  return r;
}

// Sum of squares of 8 consecutive elements starting at p (fp32).
template <class DT>
__device__ __forceinline__ float sumsq8(const typename DT::storage* p) {
  float s = 0.f;
  if (DT::kPer16B == 8) {
    float f[8];
    unpack16<DT>(*reinterpret_cast<const uint4*>(p), f);
#pragma unroll
    for (int i = 0; i < 8; ++i) s += f[i] * f[i];
  } else {
    float f[4];
    unpack16<DT>(*reinterpret_cast<const uint4*>(p), f);
#pragma unroll
    for (int i = 0; i < 4; ++i) s += f[i] * f[i];
    unpack16<DT>(*reinterpret_cast<const uint4*>((const char*)p + 16), f);
#pragma unroll
    for (int i = 0; i < 4; ++i) s += f[i] * f[i];
  }
  return s;
}

// Persistent: the grid is sized to the CU count and every wave walks the 64-key
// tiles tile = first, first + stride, ...; the plane slice is loaded into LDS once
// per workgroup (all of it when NW*8 KB fits) and amortised over all of them.
template <class DT>
__global__ __launch_bounds__(kHashThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void hash_keys_kernel(
    const void* __restrict__ k_, const void* __restrict__ v_, int64_t k_sb, int64_t k_sh,
    int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss,
    const uint16_t* __restrict__ planes_words,  // bf16 [NW*32, 128]
    uint32_t* __restrict__ codes, uint16_t* __restrict__ v_norm,
    const int32_t* __restrict__ pos_b, int t0, int Hkv, int S, int L, int P, int NW, int64_t Tcap,
    int tiles_per_row, int n_tiles, int wc, int words_per_wg) {
  typedef typename DT::storage ST;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  // planes slice in LDS: [wc*32 columns][128] bf16, 16-byte groups XOR-swizzled
  // by column so the per-lane fragment reads (stride 256 B) spread over banks.
  uint4* plds = reinterpret_cast<uint4*>(lds_raw);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int first_tile = blockIdx.x * kHashWaves + wave;
  const int tile_stride = gridDim.x * kHashWaves;
  const int cpw = 32 / P;

  // gridDim.y splits the packed words between workgroups when there are too
  // few key tiles to occupy the chip (the per-step append of a handful of keys)
  const int word_begin = blockIdx.y * words_per_wg;
  const int word_end = min(NW, word_begin + words_per_wg);

  for (int w0 = word_begin; w0 < word_end; w0 += wc) {
    const int nw = min(wc, word_end - w0);
    __syncthreads();
    {
      // fill: nw*32 columns x 16 groups of 16 bytes, eight loads in flight per lane
      const uint4* src = reinterpret_cast<const uint4*>(planes_words) + (int64_t)w0 * 32 * 16;
      const int total = nw * 32 * 16;
      constexpr int U = 8;
      int i0 = tid;
      for (; i0 + (U - 1) * kHashThreads < total; i0 += U * kHashThreads) {
        uint4 x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) x[u] = src[i0 + u * kHashThreads];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = i0 + u * kHashThreads;
          const int col = i >> 4, grp = i & 15;
          plds[col * 16 + (grp ^ (col & 15))] = x[u];
        }
      }
      for (; i0 < total; i0 += kHashThreads) {
        const int col = i0 >> 4, grp = i0 & 15;
        plds[col * 16 + (grp ^ (col & 15))] = src[i0];
      }
    }
    __syncthreads();

    for (int tile = first_tile; tile < n_tiles; tile += tile_stride) {
      const int pair = tile / tiles_per_row;
      const int s0 = (tile % tiles_per_row) * kKeysPerWave;
      const int b = pair / Hkv, h = pair % Hkv;
      const int pos0 = pos_b ? pos_b[b] : t0;

      // A fragments: lane x holds row x%32, elements 64*(x/32) + 8*kk .. +7, so a
      // lane reads one contiguous half row over the 8 k-steps.  (The contraction
      // only needs A and B to agree on which k each slot holds.)
      Frag afrag[2][kKSteps];
      const ST* kbase = (const ST*)k_ + b * k_sb + h * k_sh;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
        const int srow = s0 + mt * 32 + (lane & 31);
        const bool ok = srow < S;
#pragma unroll
        for (int kk = 0; kk < kKSteps; ++kk) {
          afrag[mt][kk].u = ok ? load_frag8<DT>(kbase + (int64_t)srow * k_ss + (lane >> 5) * 64 + kk * 8)
                               : make_uint4(0, 0, 0, 0);
        }
      }
      const bool second = s0 + 32 < S;  // the tile's second 32 rows hold keys at all

      uint32_t* codes_pair = codes + (int64_t)pair * NW * Tcap;
      for (int ww = 0; ww < nw; ++ww) {
        f32x16 acc0 = {0}, acc1 = {0};
        const int col = ww * 32 + (lane & 31);
#pragma unroll
        for (int kk = 0; kk < kKSteps; ++kk) {
          Frag bf;
          const int grp = (lane >> 5) * 8 + kk;
          bf.u = plds[col * 16 + (grp ^ (col & 15))];
          acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afrag[0][kk].v, bf.v, acc0, 0, 0, 0);
          if (second) acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afrag[1][kk].v, bf.v, acc1, 0, 0, 0);
        }
        const int w = w0 + ww;
        const int nbits = min(cpw, L - w * cpw) * P;
        const uint32_t valid = nbits >= 32 ? 0xffffffffu : ((1u << nbits) - 1u);
        uint32_t word0 = 0, word1 = 0;  // lane x < 32: packed word of key row x in M tile 0 / 1
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row_lo = 8 * (r / 4) + (r % 4);  // lanes 0..31 of the ballot
          const unsigned long long b0 = __ballot(acc0[r] >= 0.f);
          const unsigned long long b1 = __ballot(acc1[r] >= 0.f);
          if (lane == row_lo) {
            word0 = (uint32_t)b0;
            word1 = (uint32_t)b1;
          } else if (lane == row_lo + 4) {
            word0 = (uint32_t)(b0 >> 32);
            word1 = (uint32_t)(b1 >> 32);
          }
        }
        if (lane < 32) {
          uint32_t* dst = codes_pair + (int64_t)w * Tcap + pos0 + s0;
          if (s0 + lane < S) dst[lane] = word0 & valid;
          if (s0 + 32 + lane < S) dst[32 + lane] = word1 & valid;
        }
      }

      // fused value norm: 16 lanes per row, 4 rows per pass (once per tile)
      if (v_ != nullptr && w0 == 0) {  // only the workgroups that own word 0
        const ST* vbase = (const ST*)v_ + b * v_sb + h * v_sh;
        uint16_t* vn = v_norm + (int64_t)pair * Tcap + pos0;
        const int sub = lane >> 4, part = lane & 15;
        const int rows_here = min(kKeysPerWave, S - s0);
        for (int r0 = 0; r0 < rows_here; r0 += 4) {
          const int srow = s0 + r0 + sub;
          float ss = (srow < S) ? sumsq8<DT>(vbase + (int64_t)srow * v_ss + part * 8) : 0.f;
#pragma unroll
          for (int x = 1; x < 16; x <<= 1) ss += __shfl_xor(ss, x, SOCKET_WAVE);
          if (part == 0 && srow < S) vn[srow] = f32_to_f16_bits(sqrtf(ss));
        }
      }
    }
  }
}

template <class PT>
__global__ void permute_planes_kernel(const void* __restrict__ planes_, uint16_t* __restrict__ out,
                                      int L, int P, int D, int NW) {
  typedef typename PT::storage ST;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (int64_t)NW * 32 * D) return;
  const int d = (int)(i % D);
  const int colw = (int)(i / D);
  const int w = colw / 32, p = colw % 32;
  const int cpw = 32 / P;
  const int l = w * cpw + p / P;
  uint16_t r = 0;
  if (p < cpw * P && l < L) {
    const int k = P - 1 - (p % P);
    const ST* planes = (const ST*)planes_;
    const int64_t src = ((int64_t)l * P + k) * D + d;
    float f;
    if (PT::kEnum == SOCKET_F32) f = ((const float*)planes)[src];
    else if (PT::kEnum == SOCKET_BF16) f = bf16_bits_to_f32(((const uint16_t*)planes)[src]);
    else f = f16_bits_to_f32(((const uint16_t*)planes)[src]);
    r = f32_to_bf16_bits(f);
  }
  out[i] = r;
}

__global__ void unpack_codes_kernel(const uint32_t* __restrict__ codes, int16_t* __restrict__ out,
                                    int Hkv, int L, int P, int t0, int T, int64_t Tcap, int NW,
                                    int64_t osb, int64_t osh, int64_t osl, int64_t ost) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  const int pair = blockIdx.y;
  if (t >= T) return;
  const int b = pair / Hkv, h = pair % Hkv;
  const int cpw = 32 / P;
  const uint32_t mask = (1u << P) - 1u;
  const uint32_t* src = codes + (int64_t)pair * NW * Tcap + t0 + t;
  int16_t* dst = out + b * osb + h * osh + (int64_t)t * ost;
  for (int w = 0; w < NW; ++w) {
    const uint32_t word = src[(int64_t)w * Tcap];
    for (int j = 0; j < cpw && w * cpw + j < L; ++j)
      dst[(int64_t)(w * cpw + j) * osl] = (int16_t)((word >> (j * P)) & mask);
  }
}

__global__ void pack_codes_kernel(const int16_t* __restrict__ in, int64_t isb, int64_t ish,
                                  int64_t isl, int64_t ist, uint32_t* __restrict__ codes, int Hkv,
                                  int L, int P, int t0, int T, int64_t Tcap, int NW) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  const int pair = blockIdx.y;
  if (t >= T) return;
  const int b = pair / Hkv, h = pair % Hkv;
  const int cpw = 32 / P;
  const uint32_t mask = (1u << P) - 1u;
  const int16_t* src = in + b * isb + h * ish + (int64_t)t * ist;
  uint32_t* dst = codes + (int64_t)pair * NW * Tcap + t0 + t;
  for (int w = 0; w < NW; ++w) {
    uint32_t word = 0;
    for (int j = 0; j < cpw && w * cpw + j < L; ++j)
      word |= ((uint32_t)(uint16_t)src[(int64_t)(w * cpw + j) * isl] & mask) << (j * P);
    dst[(int64_t)w * Tcap] = word;
  }
}

int words_per_key(int L, int P) {
  if (P < 1 || P > 16 || L < 1) return 0;
  const int cpw = 32 / P;
  return (L + cpw - 1) / cpw;
}

}  // namespace

extern "C" int socket_words_per_key(int L, int P) { return words_per_key(L, P); }

extern "C" int socket_permute_planes(const void* planes, int planes_dtype, int L, int P, int D,
                                     void* planes_words, void* stream) {
  SOCKET_REQUIRE(planes && planes_words, SOCKET_ERR_NULL);
  const int NW = words_per_key(L, P);
  SOCKET_REQUIRE(NW > 0 && D > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(socket_dtype_bytes(planes_dtype) != 0, SOCKET_ERR_UNSUPPORTED);
  const int64_t n = (int64_t)NW * 32 * D;
  const int threads = 256;
  const dim3 grid((unsigned)((n + threads - 1) / threads));
  hipStream_t s = (hipStream_t)stream;
  uint16_t* out = (uint16_t*)planes_words;
  if (planes_dtype == SOCKET_F32)
    hipLaunchKernelGGL((permute_planes_kernel<DType_f32>), grid, dim3(threads), 0, s, planes, out, L, P, D, NW);
  else if (planes_dtype == SOCKET_BF16)
    hipLaunchKernelGGL((permute_planes_kernel<DType_bf16>), grid, dim3(threads), 0, s, planes, out, L, P, D, NW);
  else
    hipLaunchKernelGGL((permute_planes_kernel<DType_f16>), grid, dim3(threads), 0, s, planes, out, L, P, D, NW);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

extern "C" int socket_hash_keys(const void* k, const void* v, int dtype, int64_t k_stride_b,
                                int64_t k_stride_h, int64_t k_stride_s, int64_t v_stride_b,
                                int64_t v_stride_h, int64_t v_stride_s, const void* planes_words,
                                uint32_t* codes, uint16_t* v_norm, const int32_t* pos_b, int t0,
                                int B, int Hkv, int S, int D, int L, int P, int64_t Tcap,
                                void* stream) {
  SOCKET_REQUIRE(k && planes_words && codes, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(v == nullptr || v_norm != nullptr, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(D == kD, SOCKET_ERR_UNSUPPORTED);
  const int NW = words_per_key(L, P);
  SOCKET_REQUIRE(NW > 0 && B > 0 && Hkv > 0 && S > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(t0 >= 0 && (pos_b != nullptr || (int64_t)t0 + S <= Tcap), SOCKET_ERR_SHAPE);
  const int eb = socket_dtype_bytes(dtype);
  SOCKET_REQUIRE(eb != 0, SOCKET_ERR_UNSUPPORTED);
  const int per16 = 16 / eb;
  SOCKET_REQUIRE(socket_aligned16(k) && socket_aligned16(planes_words) &&
                     k_stride_b % per16 == 0 && k_stride_h % per16 == 0 && k_stride_s % per16 == 0,
                 SOCKET_ERR_ALIGN);
  if (v) {
    SOCKET_REQUIRE(socket_aligned16(v) && v_stride_b % per16 == 0 && v_stride_h % per16 == 0 &&
                       v_stride_s % per16 == 0,
                   SOCKET_ERR_ALIGN);
  }
  const int tiles_per_row = (S + kKeysPerWave - 1) / kKeysPerWave;
  const int64_t n_tiles64 = (int64_t)B * Hkv * tiles_per_row;
  SOCKET_REQUIRE(n_tiles64 < (1LL << 31), SOCKET_ERR_SHAPE);
  const int n_tiles = (int)n_tiles64;
  const SocketDeviceLimits& lim = socket_device_limits();
  // plane slice: every word when they all fit in LDS (one slice, loaded once per
  // workgroup), else as many as fit; one persistent workgroup per CU
  int wc = lim.max_lds_per_block / (32 * kD * 2);
  if (wc < 1) wc = 1;
  if (wc > NW) wc = NW;
  int n_wg = (n_tiles + kHashWaves - 1) / kHashWaves;
  if (n_wg > lim.cu_count) n_wg = lim.cu_count;
  int wsplit = lim.cu_count / n_wg;  // > 1 only when the tiles leave CUs idle
  if (wsplit > NW) wsplit = NW;
  if (wsplit < 1) wsplit = 1;
  const int words_per_wg = (NW + wsplit - 1) / wsplit;
  wsplit = (NW + words_per_wg - 1) / words_per_wg;
  if (wc > words_per_wg) wc = words_per_wg;
  const size_t lds = (size_t)wc * 32 * kD * 2;
  const dim3 grid(n_wg, wsplit);
  hipStream_t s = (hipStream_t)stream;
#define SOCKET_HASH_LAUNCH(DT)                                                                     \
  do {                                                                                             \
    auto kern = hash_keys_kernel<DT>;                                                              \
    if (lds > 48 * 1024 &&                                                                         \
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                   \
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)   \
      return SOCKET_ERR_LAUNCH;                                                                    \
    hipLaunchKernelGGL(kern, grid, dim3(kHashThreads), lds, s, k, v, k_stride_b, k_stride_h,       \
                       k_stride_s, v_stride_b, v_stride_h, v_stride_s,                             \
                       (const uint16_t*)planes_words, codes, v_norm, pos_b, t0, Hkv, S, L, P, NW,  \
                       Tcap, tiles_per_row, n_tiles, wc, words_per_wg);                            \
  } while (0)
  if (dtype == SOCKET_BF16) SOCKET_HASH_LAUNCH(DType_bf16);
  else if (dtype == SOCKET_F16) SOCKET_HASH_LAUNCH(DType_f16);
  else SOCKET_HASH_LAUNCH(DType_f32);
#undef SOCKET_HASH_LAUNCH
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

extern "C" int socket_unpack_codes(const uint32_t* codes, int16_t* out, int B, int Hkv, int L, int P,
                                   int t0, int T, int64_t Tcap, int64_t out_stride_b,
                                   int64_t out_stride_h, int64_t out_stride_l, int64_t out_stride_t,
                                   void* stream) {
  SOCKET_REQUIRE(codes && out, SOCKET_ERR_NULL);
  const int NW = words_per_key(L, P);
  SOCKET_REQUIRE(NW > 0 && B > 0 && Hkv > 0 && T > 0 && t0 >= 0 && (int64_t)t0 + T <= Tcap,
                 SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE((int64_t)B * Hkv <= 65535, SOCKET_ERR_SHAPE);
  dim3 grid((T + 255) / 256, B * Hkv);
  hipLaunchKernelGGL(unpack_codes_kernel, grid, dim3(256), 0, (hipStream_t)stream, codes, out, Hkv, L,
                     P, t0, T, Tcap, NW, out_stride_b, out_stride_h, out_stride_l, out_stride_t);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

extern "C" int socket_pack_codes(const int16_t* in, int64_t in_stride_b, int64_t in_stride_h,
                                 int64_t in_stride_l, int64_t in_stride_t, uint32_t* codes, int B,
                                 int Hkv, int L, int P, int t0, int T, int64_t Tcap, void* stream) {
  SOCKET_REQUIRE(codes && in, SOCKET_ERR_NULL);
  const int NW = words_per_key(L, P);
  SOCKET_REQUIRE(NW > 0 && B > 0 && Hkv > 0 && T > 0 && t0 >= 0 && (int64_t)t0 + T <= Tcap,
                 SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE((int64_t)B * Hkv <= 65535, SOCKET_ERR_SHAPE);
  dim3 grid((T + 255) / 256, B * Hkv);
  hipLaunchKernelGGL(pack_codes_kernel, grid, dim3(256), 0, (hipStream_t)stream, in, in_stride_b,
                     in_stride_h, in_stride_l, in_stride_t, codes, Hkv, L, P, t0, T, Tcap, NW);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}
