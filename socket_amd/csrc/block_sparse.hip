// Block-sparse prefill attention: every 64-row block of queries attends to a
// listed set of 64-key blocks, causally, with an online softmax.
//
// Replaces random_walk_fwd + random_walk_sparse_attention,
// kernels/block_sparse_flash_attention.py:280-437 (grid (row blocks, B*H), one
// list of KLIST always-valid block ids per (b, h, row block), walked in order;
// a block listed twice is attended twice, as there).
//
// One workgroup of four waves per row block; wave w owns query rows 16w .. 16w+15.
// Both products run on v_mfma_f32_16x16x32 in the TRANSPOSED orientation, which
// makes the query row the N index of every accumulator -- lane x holds row x % 16
// in all its registers:
//   S^T[key, row] = K . Q^T     A = K fragment (LDS), B = Q fragment (registers)
//   O^T[dim, row] = V^T . P^T   A = V^T fragment (LDS), B = P^T (the lane's own
//                                exponentials, rounded to the input type)
// so the softmax needs no data movement at all: a row's maximum and sum are over a
// lane's own registers plus the three other lane quarters (two lane-swap steps),
// the rescale factor is uniform per lane, and the probabilities a lane computed
// are exactly the B operand it has to supply.  The k index of the second product
// is the key; its order inside an MFMA is free as long as both operands agree, so
// slot i of lane quarter q stands for key 32c + 4q + i (i < 4) or 32c + 16 + 4q +
// i - 4 -- the keys whose scores that quarter already holds.  V is stored
// transposed in LDS ([dim][key]) so that those two runs of four keys are two
// 8-byte reads: rows of 72 elements, the sixteen 4-key groups of a row placed at
// group ^ (dim / 8 % 16), which keeps both the transposing stores and the
// fragment reads at the two LDS passes their 512 bytes need.
#include "socket_common.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bs_bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 bs_f16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float bs_f32x4;

constexpr int kBsBlock = 64;     // rows per query block, keys per key block
constexpr int kBsThreads = 256;
constexpr int kBsVtStride = kBsBlock + 8;  // elements per row of the transposed V tile

template <class DT>
struct BsType;
template <>
struct BsType<DType_bf16> {
  static __device__ __forceinline__ bs_f32x4 mfma(const uint4& a, const uint4& b, bs_f32x4 c) {
    union {
      uint4 u;
      bs_bf16x8 v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x.v, y.v, c, 0, 0, 0);
  }
  // (the conversion instruction of the target, round to nearest even)
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
struct BsType<DType_f16> {
  static __device__ __forceinline__ bs_f32x4 mfma(const uint4& a, const uint4& b, bs_f32x4 c) {
    union {
      uint4 u;
      bs_f16x8 v;
    } x, y;
    x.u = a;
    y.u = b;
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(x.v, y.v, c, 0, 0, 0);
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

// value of lane x ^ 16 / x ^ 32 (see hash.hip: v_permlane16_swap / v_permlane32_swap)
__device__ __forceinline__ float bs_xor16(float v, bool odd_row) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(odd_row ? r[0] : r[1]);
}
__device__ __forceinline__ float bs_xor32(float v, bool upper_half) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(upper_half ? r[0] : r[1]);
}

template <class DT, int D>
__global__ __launch_bounds__(kBsThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void block_sparse_fwd_kernel(
    const uint16_t* __restrict__ q_, const uint16_t* __restrict__ k_, const uint16_t* __restrict__ v_,
    int64_t q_sb, int64_t q_sh, int64_t q_sm, int64_t k_sb, int64_t k_sh, int64_t k_sn, int64_t v_sb,
    int64_t v_sh, int64_t v_sn, const int32_t* __restrict__ seqlens, const int32_t* __restrict__ block_index,
    uint16_t* __restrict__ out, int64_t o_sb, int64_t o_sh, int64_t o_sm, int H, int T, int num_rows, int klist,
    int num_cols, float scale_log2) {
  constexpr int CH = D / 8;                 // 16-byte chunks per row
  constexpr int KS = (D + 31) / 32;         // k-steps of the first product
  constexpr int DB = D / 16;                // 16-dim blocks of the output
  __shared__ __attribute__((aligned(16))) uint4 k_lds[kBsBlock * CH];
  __shared__ __attribute__((aligned(16))) uint16_t vt_lds[D * kBsVtStride];

  // Workgroups are dealt to the 8 XCDs round-robin by linear id.  Renumbered so
  // that each XCD walks one contiguous eighth of the (head, row block) space in
  // order: neighbouring row blocks share their window tiles, which then come from
  // that XCD's L2 instead of being fetched once per XCD.
  int start_m = blockIdx.x, bh = blockIdx.y;
  {
    const int64_t total = (int64_t)gridDim.x * gridDim.y;
    if (total % 8 == 0) {
      const int64_t n = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
      const int64_t id = (n % 8) * (total / 8) + n / 8;
      start_m = (int)(id % num_rows);
      bh = (int)(id / num_rows);
    }
  }
  const int b = bh / H, h = bh % H;
  const int seqlen = min(seqlens[b], T);
  if (start_m * kBsBlock >= seqlen) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int prow = lane & 15, quarter = lane >> 4;
  const int row = start_m * kBsBlock + wave * 16 + prow;   // this lane's query row (N index of every product)
  const bool row_ok = row < seqlen;

  const uint16_t* qb = q_ + b * q_sb + h * q_sh;
  const uint16_t* kb = k_ + b * k_sb + h * k_sh;
  const uint16_t* vb = v_ + b * v_sb + h * v_sh;

  // Q fragments (B operand of S^T): row `row`, dims 32*ks + 8*quarter .. +7
  uint4 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int chunk = 4 * ks + quarter;
    qf[ks] = (chunk < CH && row_ok) ? *reinterpret_cast<const uint4*>(qb + (int64_t)row * q_sm + chunk * 8)
                                    : make_uint4(0, 0, 0, 0);
  }

  bs_f32x4 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = bs_f32x4{0.f, 0.f, 0.f, 0.f};
  float m_i = -INFINITY, l_part = 0.f;

  const int32_t* blocks = block_index + ((int64_t)bh * num_rows + start_m) * klist;
  // Staging: thread t < 16*CH takes chunk t % CH of the four keys 4*(t / CH) .. +3 of
  // a tile.  The K chunks go to LDS as they are; the V chunks are transposed in
  // registers (two byte-selects per output word) so that the four keys of one dim
  // leave as a single 8-byte store.
  const bool stager = tid < 16 * CH;
  const int st_chunk = tid % CH, st_key0 = 4 * (tid / CH);
  uint4 kr[4], vr[4];
  auto fetch_tile = [&](int j) {
    const int blk = min(max(blocks[j], 0), num_cols - 1);   // (the lists hold valid ids; a stray one must not fault)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int col = blk * kBsBlock + st_key0 + i;
      kr[i] = vr[i] = make_uint4(0, 0, 0, 0);
      if (stager && col < seqlen) {  // keys past the sequence read as zero (and are masked below)
        kr[i] = *reinterpret_cast<const uint4*>(kb + (int64_t)col * k_sn + st_chunk * 8);
        vr[i] = *reinterpret_cast<const uint4*>(vb + (int64_t)col * v_sn + st_chunk * 8);
      }
    }
  };
  auto store_tile = [&]() {
    if (!stager) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = st_key0 + i;
      k_lds[key * CH + (st_chunk ^ (key & (CH - 1)))] = kr[i];
    }
    const uint32_t w[4][4] = {{vr[0].x, vr[0].y, vr[0].z, vr[0].w},
                              {vr[1].x, vr[1].y, vr[1].z, vr[1].w},
                              {vr[2].x, vr[2].y, vr[2].z, vr[2].w},
                              {vr[3].x, vr[3].y, vr[3].z, vr[3].w}};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;   // high / low halves of the two words
      uint2 t;
      t.x = __builtin_amdgcn_perm(w[1][e >> 1], w[0][e >> 1], sel);   // keys 0, 1
      t.y = __builtin_amdgcn_perm(w[3][e >> 1], w[2][e >> 1], sel);   // keys 2, 3
      *reinterpret_cast<uint2*>(vt_lds + (st_chunk * 8 + e) * kBsVtStride + (((st_key0 >> 2) ^ st_chunk) << 2)) = t;
    }
  };

  // what of the fragment addresses does not change from tile to tile
  const uint4* k_frag[KS];   // key row `prow`, this lane's chunk of k-step ks; key block nb adds nb*16 rows
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    k_frag[ks] = k_lds + prow * CH + (((4 * ks + quarter) & (CH - 1)) ^ (prow & (CH - 1)));
  // transposed V tile: row of dim db*16 + prow is v_row0 + db*16 rows; 4-key group g of it sits at
  // element ((g ^ (dim / 8 % 16)) * 4, and dim / 8 = 2*db + prow / 8
  const uint16_t* v_row0 = vt_lds + prow * kBsVtStride;
  const int v_swz0 = prow >> 3;

  for (int j = 0; j < klist; ++j) {
    const int start_n = min(max(blocks[j], 0), num_cols - 1) * kBsBlock;
    // (requested here rather than a tile ahead: holding the next tile in registers
    // during the contraction costs a wave of occupancy per SIMD and is slower)
    fetch_tile(j);
    __syncthreads();  // the previous tiles have been consumed
    store_tile();
    __syncthreads();

    // ---- S^T = K . Q^T: register r of block nb is key nb*16 + 4*quarter + r against row `row`
    bs_f32x4 s[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) s[nb] = bs_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        const uint4 a = (4 * ks + quarter < CH) ? k_frag[ks][nb * 16 * CH] : make_uint4(0, 0, 0, 0);
        s[nb] = BsType<DT>::mfma(a, qf[ks], s[nb]);
      }
    }
    // ---- causal mask, running maximum (of the raw dot products: the scale is
    // positive and is applied inside the exponent).  A tile wholly at or left of
    // this wave's first row needs no mask.
    const bool tile_open = start_n + kBsBlock - 1 <= start_m * kBsBlock + wave * 16 &&
                           start_m * kBsBlock + wave * 16 + 15 < seqlen;   // (wave-uniform)
    float m_blk = -INFINITY;
    if (tile_open) {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int r = 0; r < 4; ++r) m_blk = fmaxf(m_blk, s[nb][r]);
    } else {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int col = start_n + nb * 16 + 4 * quarter + r;
          const float x = (row_ok && col <= row) ? s[nb][r] : -INFINITY;
          s[nb][r] = x;
          m_blk = fmaxf(m_blk, x);
        }
    }
    m_blk = fmaxf(m_blk, bs_xor16(m_blk, quarter & 1));
    m_blk = fmaxf(m_blk, bs_xor32(m_blk, quarter & 2));
    const float m_new = fmaxf(m_i, m_blk * scale_log2);
    // (a row with nothing visible so far keeps alpha = 1 and p = 0 instead of the
    // NaN of exp2(-inf - -inf); v_exp_f32 directly: its arguments are <= 0 and a
    // result that underflows may as well be zero)
    const bool blind = m_new == -INFINITY;
    const float alpha = blind ? 1.f : __builtin_amdgcn_exp2f(m_i - m_new);
    const float shift = blind ? 0.f : -m_new;
    float psum = 0.f;
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[nb][r], scale_log2, shift));
        s[nb][r] = p;
        psum += p;
      }
    l_part = l_part * alpha + psum;
    m_i = m_new;
    // The output accumulators are rescaled only when some row of the wave has a new
    // maximum (alpha == 1 is the identity, so skipping it changes nothing): after the
    // first few tiles that is rare, and the accumulators need not leave the matrix
    // core's registers.
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        o[db][0] *= alpha;
        o[db][1] *= alpha;
        o[db][2] *= alpha;
        o[db][3] *= alpha;
      }
    }
    // ---- O^T += V^T . P^T
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      uint4 pf;  // slots 0..3: keys 32c + 4q + r, slots 4..7: keys 32c + 16 + 4q + r
      pf.x = BsType<DT>::pack2(s[2 * c][0], s[2 * c][1]);
      pf.y = BsType<DT>::pack2(s[2 * c][2], s[2 * c][3]);
      pf.z = BsType<DT>::pack2(s[2 * c + 1][0], s[2 * c + 1][1]);
      pf.w = BsType<DT>::pack2(s[2 * c + 1][2], s[2 * c + 1][3]);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        // group (8c + quarter [+ 4]) ^ swizzle = (quarter ^ swizzle) ^ (8c [+ 4]): one xor on the lane's constant
        const uint16_t* vrow = v_row0 + db * 16 * kBsVtStride;
        const int grp = (quarter ^ (2 * db + v_swz0)) << 2;
        const uint2 lo = *reinterpret_cast<const uint2*>(vrow + (grp ^ (32 * c)));
        const uint2 hi = *reinterpret_cast<const uint2*>(vrow + (grp ^ (32 * c + 16)));
        o[db] = BsType<DT>::mfma(make_uint4(lo.x, lo.y, hi.x, hi.y), pf, o[db]);
      }
    }
  }

  float l = l_part;
  l += bs_xor16(l, quarter & 1);
  l += bs_xor32(l, quarter & 2);
  if (!row_ok) return;
  const float inv = 1.f / (l + 1e-9f);
  uint16_t* orow = out + b * o_sb + h * o_sh + (int64_t)row * o_sm;
#pragma unroll
  for (int db = 0; db < DB; ++db) {
    uint2 w;
    w.x = BsType<DT>::pack2(o[db][0] * inv, o[db][1] * inv);
    w.y = BsType<DT>::pack2(o[db][2] * inv, o[db][3] * inv);
    *reinterpret_cast<uint2*>(orow + db * 16 + 4 * quarter) = w;
  }
}

template <class DT>
int launch_block_sparse(const void* q, const void* k, const void* v, int64_t q_sb, int64_t q_sh, int64_t q_sm,
                        int64_t k_sb, int64_t k_sh, int64_t k_sn, int64_t v_sb, int64_t v_sh, int64_t v_sn,
                        const int32_t* seqlens, const int32_t* block_index, void* out, int64_t o_sb, int64_t o_sh,
                        int64_t o_sm, int B, int H, int T, int D, int num_rows, int klist, hipStream_t s) {
  const int num_cols = (T + kBsBlock - 1) / kBsBlock;
  const float scale_log2 = 1.44269504f / sqrtf((float)D);
  const dim3 grid(num_rows, B * H);
#define SOCKET_BS(DD)                                                                                        \
  hipLaunchKernelGGL((block_sparse_fwd_kernel<DT, DD>), grid, dim3(kBsThreads), 0, s, (const uint16_t*)q,    \
                     (const uint16_t*)k, (const uint16_t*)v, q_sb, q_sh, q_sm, k_sb, k_sh, k_sn, v_sb, v_sh, \
                     v_sn, seqlens, block_index, (uint16_t*)out, o_sb, o_sh, o_sm, H, T, num_rows, klist,    \
                     num_cols, scale_log2)
  if (D == 128) SOCKET_BS(128);
  else if (D == 64) SOCKET_BS(64);
  else if (D == 32) SOCKET_BS(32);
  else SOCKET_BS(16);
#undef SOCKET_BS
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

}  // namespace

extern "C" int socket_block_sparse_attention(const void* q, const void* k, const void* v, int dtype,
                                             int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_m,
                                             int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                             int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                                             const int32_t* seqlens, const int32_t* block_index, void* out,
                                             int64_t o_stride_b, int64_t o_stride_h, int64_t o_stride_m, int B,
                                             int H, int T, int D, int num_rows, int klist, int block_m,
                                             int block_n, void* stream) {
  SOCKET_REQUIRE(q && k && v && seqlens && block_index && out, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(dtype == SOCKET_BF16 || dtype == SOCKET_F16, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(D == 16 || D == 32 || D == 64 || D == 128, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(block_m == kBsBlock && block_n == kBsBlock, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(B > 0 && H > 0 && T > 0 && klist > 0 && (int64_t)B * H <= 65535, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(num_rows == (T + kBsBlock - 1) / kBsBlock, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(socket_aligned16(q) && socket_aligned16(k) && socket_aligned16(v) && socket_aligned16(out),
                 SOCKET_ERR_ALIGN);
  SOCKET_REQUIRE(q_stride_b % 8 == 0 && q_stride_h % 8 == 0 && q_stride_m % 8 == 0 && k_stride_b % 8 == 0 &&
                     k_stride_h % 8 == 0 && k_stride_n % 8 == 0 && v_stride_b % 8 == 0 && v_stride_h % 8 == 0 &&
                     v_stride_n % 8 == 0 && o_stride_b % 4 == 0 && o_stride_h % 4 == 0 && o_stride_m % 4 == 0,
                 SOCKET_ERR_ALIGN);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == SOCKET_BF16)
    return launch_block_sparse<DType_bf16>(q, k, v, q_stride_b, q_stride_h, q_stride_m, k_stride_b, k_stride_h,
                                           k_stride_n, v_stride_b, v_stride_h, v_stride_n, seqlens, block_index,
                                           out, o_stride_b, o_stride_h, o_stride_m, B, H, T, D, num_rows, klist, s);
  return launch_block_sparse<DType_f16>(q, k, v, q_stride_b, q_stride_h, q_stride_m, k_stride_b, k_stride_h,
                                        k_stride_n, v_stride_b, v_stride_h, v_stride_n, seqlens, block_index, out,
                                        o_stride_b, o_stride_h, o_stride_m, B, H, T, D, num_rows, klist, s);
}
