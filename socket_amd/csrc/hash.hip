// K1: key hashing.  codes = pack(sign(keys . planes^T)) with the value norm fused.
//
// Replaces hard_hash_keys + pack_bits (GPT-FAST/model.py:403-413): the einsum
// that materialises [B,S,Hkv,L,P] projections, the bool compare and the int16
// weighted sum become one MFMA contraction with a sign-bit epilogue.
//
// The hyperplanes are pre-ordered (socket_permute_planes) so that column
// w*32 + p of the contraction is the plane whose sign is bit p of packed word w.
// With planes as the M operand and keys as the N operand of
// v_mfma_f32_16x16x32_bf16, accumulator register r of lane x holds
//   plane row 4*(x/16) + r of a 16-plane block,  key x%16,
// so each lane has sign bits of ITS key in its own registers: they are shifted
// into a byte one v_alignbit per register, the four lane quarters are OR-ed into
// the 32-bit word, and lane x ends up with the packed word of key x of the
// 64-key tile, stored as one 256-byte run of the table-major code cache.  No
// compares, no ballots, no LDS round trip.  The 16x16x32 shape is chosen for the
// key loads: its N operand wants 64 consecutive bytes of a row from four lanes,
// so a load instruction touches 16 rows x one 64-byte sector (the 32x32x16 shape
// touches 64 lines for 16 bytes each, eight times over).
//
// A wave owns 64 consecutive keys of one (b, kv head) (four 16-key blocks) at a
// time and keeps their fragments in registers for the whole column sweep; the
// planes sit in LDS (all NW words when NW*8 KB fits, which L=60 x P=10 exactly
// does at 160 KB) and workgroups are persistent, so the planes are fetched once
// per CU, not once per tile.
#include "socket_common.h"

#include <type_traits>

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

constexpr int kHashThreads = 512;
constexpr int kHashWaves = kHashThreads / SOCKET_WAVE;
constexpr int kKeysPerWave = 64;
constexpr int kD = 128;
constexpr int kKSteps = kD / 32;      // MFMA k-steps (16x16x32)
constexpr int kKeyBlocks = kKeysPerWave / 16;

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

// A cache position handed over on the device (per-sequence positions) is not
// checked by the host: rows that would land outside [0, Tcap) are dropped.
__device__ __forceinline__ bool in_cache(int pos, int64_t Tcap) { return (uint64_t)(int64_t)pos < (uint64_t)Tcap; }

// LDS placement of the planes: row `col` is 16 groups of 16 bytes, group g stored
// at slot g ^ plane_swizzle(col).  A fragment read has sixteen lanes on sixteen
// columns {4..7} + 8j (or {0..3} + 8j) at one group; the swizzle sends those to
// sixteen different slots, i.e. all 64 banks once.
__device__ __forceinline__ int plane_swizzle(int col) { return (col & 3) | (((col >> 3) & 3) << 2); }

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
          plds[col * 16 + (grp ^ plane_swizzle(col))] = x[u];
        }
      }
      for (; i0 < total; i0 += kHashThreads) {
        const int col = i0 >> 4, grp = i0 & 15;
        plds[col * 16 + (grp ^ plane_swizzle(col))] = src[i0];
      }
    }
    __syncthreads();

    // Key fragments (the N operand of v_mfma_f32_16x16x32_bf16): for key block nb
    // and k-step ks, lane x holds key nb*16 + x%16, elements 32*ks + 8*(x/16) .. +7,
    // so the four lanes x, x+16, x+32, x+48 read 64 consecutive bytes of one row:
    // a load instruction touches 16 rows x one 64-byte sector each.
    auto load_rows = [&](const void* base_, int64_t sb, int64_t sh, int64_t ss, int tile,
                         Frag (&dst)[kKeyBlocks][kKSteps]) {
      const int pair = tile / tiles_per_row;
      const int s0 = (tile % tiles_per_row) * kKeysPerWave;
      const ST* base = (const ST*)base_ + (pair / Hkv) * sb + (pair % Hkv) * sh;
#pragma unroll
      for (int nb = 0; nb < kKeyBlocks; ++nb) {
        const int srow = s0 + nb * 16 + (lane & 15);
        const bool ok = srow < S;
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks) {
          dst[nb][ks].u = ok ? load_frag8<DT>(base + (int64_t)srow * ss + ks * 32 + (lane >> 4) * 8)
                             : make_uint4(0, 0, 0, 0);
        }
      }
    };
    // bf16 values: their norms come from the matrix core too (see below), from
    // fragments requested together with the keys'
    constexpr bool kNormByMfma = DT::kEnum == SOCKET_BF16;
    const bool want_norm = v_ != nullptr && w0 == 0;  // only the workgroups that own word 0
    Frag kfrag[kKeyBlocks][kKSteps];

    for (int tile = first_tile; tile < n_tiles; tile += tile_stride) {
      const int pair = tile / tiles_per_row;
      const int s0 = (tile % tiles_per_row) * kKeysPerWave;
      const int b = pair / Hkv, h = pair % Hkv;
      const int pos0 = pos_b ? pos_b[b] : t0;
      load_rows(k_, k_sb, k_sh, k_ss, tile, kfrag);
      Frag vfrag[kKeyBlocks][kKSteps];
      if (kNormByMfma && want_norm) load_rows(v_, v_sb, v_sh, v_ss, tile, vfrag);

      const int prow = lane & 15, quarter = lane >> 4;
      // fused value norm, bf16 values (once per tile; done first so that the value
      // fragments are not live across the contraction)
      if (kNormByMfma) {
        // ||v||^2 is the diagonal of V V^T: the value fragments against themselves.
        // Element (i, i) of a 16 x 16 block sits in register i % 4 of lane
        // 16 * (i / 4) + i, so sixteen lanes of the wave hold the sixteen norms and
        // store them; no cross-lane reduction.  (bf16 products are exact in fp32.)
        if (want_norm) {
          uint16_t* vn = v_norm + (int64_t)pair * Tcap + pos0;
          const int r = prow - 4 * quarter;
#pragma unroll
          for (int nb = 0; nb < kKeyBlocks; ++nb) {
            f32x4 g = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < kKSteps; ++ks)
              g = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vfrag[nb][ks].v, vfrag[nb][ks].v, g, 0, 0, 0);
            const float d = r == 0 ? g[0] : r == 1 ? g[1] : r == 2 ? g[2] : g[3];
            const int srow = s0 + nb * 16 + prow;
            if (r >= 0 && r < 4 && srow < S && in_cache(pos0 + srow, Tcap)) vn[srow] = f32_to_f16_bits(sqrtf(d));
          }
        }
      }

      uint32_t* codes_pair = codes + (int64_t)pair * NW * Tcap;
      // Planes are the M operand: accumulator register r of lane x is plane row
      // 4*(x/16) + r of its 16-plane block against key x%16.  A lane shifts the sign
      // bits of its eight accumulators (two plane blocks x four registers) into a
      // byte, one v_alignbit each; byte q of the word comes from lane quarter q.
      // Block mb, register r, quarter q therefore lands at bit 8q + 7 - 4mb - r, and
      // the lane fetches for plane row i of block mb the plane column that belongs
      // at that bit, so the word comes out in the packed order.
      const int pbit0 = 8 * (prow >> 2) + 7 - (prow & 3);  // block 0; block 1 is 4 lower
      // Byte q of a key's word is made in lane quarter q, and a lane makes one byte
      // for each of the four key blocks: a 4 x 4 byte transpose between the quarters,
      // done on whole words in two exchanges (lanes x ^ 16, then x ^ 32) with a
      // byte-select each.  Afterwards lane x holds the word of key s0 + x.
      const uint32_t sel1 = (quarter & 1) ? 0x03070105u : 0x06020400u;
      const uint32_t sel2 = (quarter & 2) ? 0x03020706u : 0x05040100u;
      // plane fragments of one packed word: [k-step][plane block], straight from LDS
      auto load_planes = [&](int ww, Frag (&pf)[kKSteps][2]) {
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks) {
          const int grp = ks * 4 + quarter;
#pragma unroll
          for (int mb = 0; mb < 2; ++mb) {
            const int col = ww * 32 + pbit0 - 4 * mb;
            pf[ks][mb].u = plds[col * 16 + (grp ^ plane_swizzle(col))];
          }
        }
      };
      auto do_word = [&](int ww, const Frag (&pf)[kKSteps][2]) {
        f32x4 acc[2][kKeyBlocks];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int nb = 0; nb < kKeyBlocks; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks)
#pragma unroll
          for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int nb = 0; nb < kKeyBlocks; ++nb)  // (blocks past the last key hold zeros: no branch here)
              acc[mb][nb] =
                  __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[ks][mb].v, kfrag[nb][ks].v, acc[mb][nb], 0, 0, 0);
        const int w = w0 + ww;
        const int nbits = min(cpw, L - w * cpw) * P;
        const uint32_t valid = nbits >= 32 ? 0xffffffffu : ((1u << nbits) - 1u);
        // sign bits (set = negative projection; an accumulator that starts at +0 never
        // becomes -0, so "sign clear" is exactly "projection >= 0"); byte nb of `neg`
        // is this quarter's byte for key block nb
        uint32_t neg = 0;
#pragma unroll
        for (int nb = kKeyBlocks - 1; nb >= 0; --nb)
#pragma unroll
          for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) neg = __builtin_amdgcn_alignbit(neg, __float_as_uint(acc[mb][nb][r]), 31);
        const uint32_t t = lane_xor16(neg, quarter & 1);
        const uint32_t x = __builtin_amdgcn_perm(t, neg, sel1);   // two blocks x this pair of quarters
        const uint32_t u = lane_xor32(x, quarter & 2);
        const uint32_t word = __builtin_amdgcn_perm(u, x, sel2);  // block `quarter` x all four quarters
        if (s0 + lane < S && in_cache(pos0 + s0 + lane, Tcap)) codes_pair[(int64_t)w * Tcap + pos0 + s0 + lane] = ~word & valid;
      };
      // two fragment sets: the next word's LDS reads are in flight during the
      // current word's contraction
      Frag pfa[kKSteps][2], pfb[kKSteps][2];
      load_planes(0, pfa);
      for (int ww = 0; ww < nw; ww += 2) {
        if (ww + 1 < nw) load_planes(ww + 1, pfb);
        do_word(ww, pfa);
        if (ww + 1 < nw) {
          if (ww + 2 < nw) load_planes(ww + 2, pfa);
          do_word(ww + 1, pfb);
        }
      }

      // fused value norm for the other element types (once per tile)
      if (!kNormByMfma && want_norm) {
        // they keep their precision: 16 lanes per row, 4 rows per pass
        const ST* vbase = (const ST*)v_ + b * v_sb + h * v_sh;
        uint16_t* vn = v_norm + (int64_t)pair * Tcap + pos0;
        const int sub = lane >> 4, part = lane & 15;
        // all sixteen row groups' loads are issued before the first is reduced
        float ss[kKeysPerWave / 4];
#pragma unroll
        for (int g = 0; g < kKeysPerWave / 4; ++g) {
          const int srow = s0 + g * 4 + sub;
          ss[g] = (srow < S) ? sumsq8<DT>(vbase + (int64_t)srow * v_ss + part * 8) : 0.f;
        }
#pragma unroll
        for (int g = 0; g < kKeysPerWave / 4; ++g) {
          const int srow = s0 + g * 4 + sub;
          float t = ss[g];
#pragma unroll
          for (int x = 1; x < 16; x <<= 1) t += __shfl_xor(t, x, SOCKET_WAVE);
          if (part == 0 && srow < S && in_cache(pos0 + srow, Tcap)) vn[srow] = f32_to_f16_bits(sqrtf(t));
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Streamed variant for large bf16 launches (prefill).
//
// The roles are turned round: the PLANES are stationary in registers and the
// keys stream through LDS.  Wave i of the eight owns packed words i, i + 8 and
// i + 16 (96 plane rows = 96 registers per lane, loaded once per kernel), and all
// eight waves read the same 128-key tile, which arrives by direct global -> LDS
// loads (no registers, no LDS store instructions) one tile ahead of the
// contraction: the memory latency that the register-staged kernel above exposes
// once per tile is hidden behind a whole tile of MFMA work.  Values come the same
// way; wave i takes the norms of key block i of the tile from the Gram diagonal.
//
// LDS image of a tile: row r (256 bytes) holds its sixteen 16-byte chunks at slot
// chunk ^ (r & 15); the lane that fetches slot s of row r asks global memory for
// chunk s ^ (r & 15), so the image needs no pass of its own, and the sixteen
// lanes of a fragment read (sixteen consecutive rows, one chunk) hit sixteen
// different slots.
constexpr int kStreamTile = 128;                       // keys per tile
constexpr int kStreamTileBytes = kStreamTile * kD * 2;  // 32 KB
constexpr int kStreamStageBytes = 2 * kStreamTileBytes; // keys | values
constexpr int kStreamWordsPerWave = 3;
constexpr int kStreamMaxWords = kStreamWordsPerWave * kHashWaves;

__global__ __launch_bounds__(kHashThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void hash_keys_stream_kernel(
    const uint16_t* __restrict__ k_, const uint16_t* __restrict__ v_, int64_t k_sb, int64_t k_sh,
    int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss,
    const uint16_t* __restrict__ planes_words,  // bf16 [NW*32, 128]
    uint32_t* __restrict__ codes, uint16_t* __restrict__ v_norm,
    const int32_t* __restrict__ pos_b, int t0, int Hkv, int S, int L, int P, int NW, int64_t Tcap,
    int tiles_per_row, int n_tiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  // (the wave index as a scalar: every address that depends on it -- this wave's
  // words of the code cache above all -- then stays out of the vector registers;
  // with it in a VGPR the kernel spilled three registers, and each reload in the
  // middle of a tile came with a vmcnt(0) that also waited for the NEXT tile's
  // copies, so the copies never overlapped the contraction)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int prow = lane & 15, quarter = lane >> 4;
  const int cpw = 32 / P;
  const bool with_values = v_ != nullptr;

  // this wave's plane rows, in the operand order of the sign-bit epilogue (see
  // hash_keys_kernel): register set [j][k-step][plane block]
  const int pbit0 = 8 * (prow >> 2) + 7 - (prow & 3);
  Frag preg[kStreamWordsPerWave][kKSteps][2];
  {
    const uint4* planes16 = reinterpret_cast<const uint4*>(planes_words);
#pragma unroll
    for (int j = 0; j < kStreamWordsPerWave; ++j) {
      const int w = wave + kHashWaves * j;
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          const int col = w * 32 + pbit0 - 4 * mb;
          preg[j][ks][mb].u = w < NW ? planes16[(int64_t)col * 16 + ks * 4 + quarter] : make_uint4(0, 0, 0, 0);
        }
    }
  }
  const uint32_t sel1 = (quarter & 1) ? 0x03070105u : 0x06020400u;
  const uint32_t sel2 = (quarter & 2) ? 0x03020706u : 0x05040100u;

  // this wave's four 1 KB pieces of a tile (rows 4p .. 4p+3 of piece p), keys and values
  auto issue_tile = [&](int tile, int stage) {
    const int pair = tile / tiles_per_row;
    const int s0 = (tile % tiles_per_row) * kStreamTile;
    const int b = pair / Hkv, h = pair % Hkv;
    const uint16_t* kbase = k_ + b * k_sb + h * k_sh;
    const uint16_t* vbase = with_values ? v_ + b * v_sb + h * v_sh : nullptr;
    unsigned char* dst = lds_raw + (size_t)stage * kStreamStageBytes;
#pragma unroll
    for (int q = 0; q < kStreamTile / 4 / kHashWaves; ++q) {
      const int p = wave + kHashWaves * q;
      const int row = 4 * p + quarter;
      const int srow = min(s0 + row, S - 1);  // rows past the end re-read the last one; never stored
      const int chunk = prow ^ (row & 15);
      lds_dma16_stream(kbase + (int64_t)srow * k_ss + chunk * 8, dst + p * 1024);
      if (with_values) lds_dma16_stream(vbase + (int64_t)srow * v_ss + chunk * 8, dst + kStreamTileBytes + p * 1024);
    }
  };

  int tile = blockIdx.x;
  if (tile < n_tiles) issue_tile(tile, 0);
  for (int it = 0; tile < n_tiles; tile += gridDim.x, ++it) {
    const int stage = it & 1;
    const int next = tile + gridDim.x;
    // One barrier per tile: behind it every wave's pieces of this tile are in place
    // AND every wave is done with the previous tile, whose stage the next tile's
    // loads may therefore overwrite while this one is contracted.
    wait_vmcnt(0);
    __syncthreads();
    if (next < n_tiles) issue_tile(next, stage ^ 1);

    const int pair = tile / tiles_per_row;
    const int s0 = (tile % tiles_per_row) * kStreamTile;
    const int pos0 = pos_b ? pos_b[pair / Hkv] : t0;
    const uint4* ktile = reinterpret_cast<const uint4*>(lds_raw + (size_t)stage * kStreamStageBytes);
    const uint4* vtile = ktile + kStreamTileBytes / 16;
    // chunk c of row r of a tile (r & 15 == prow for every row this lane reads)
    auto frag_at = [&](const uint4* t, int r, int c) { return t[r * 16 + (c ^ prow)]; };

    if (with_values) {
      // ||v||^2 = diagonal of V V^T (see hash_keys_kernel), key block `wave` of the tile
      Frag vf[kKSteps];
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) vf[ks].u = frag_at(vtile, wave * 16 + prow, ks * 4 + quarter);
      f32x4 g = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) g = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[ks].v, vf[ks].v, g, 0, 0, 0);
      const int r = prow - 4 * quarter;
      const float d = r == 0 ? g[0] : r == 1 ? g[1] : r == 2 ? g[2] : g[3];
      const int srow = s0 + wave * 16 + prow;
      if (r >= 0 && r < 4 && srow < S && in_cache(pos0 + srow, Tcap))
        v_norm[(int64_t)pair * Tcap + pos0 + srow] = f32_to_f16_bits(sqrtf(d));
    }

    uint32_t* codes_pair = codes + (int64_t)pair * NW * Tcap;
    // The tile's eight 16-key blocks go through in pairs, the next pair's
    // fragments on their way from LDS while the current pair is contracted.  A
    // 64-key group is taken high blocks first, (3,2) then (1,0), so that the sign
    // bits shift into `neg` in the byte order the transpose expects.
    auto pair_block = [](int pp) { return (pp >> 1) * 4 + ((pp & 1) ? 0 : 2); };  // lower block of pair pp
    auto load_pair = [&](int pp, Frag (&kf)[2][kKSteps]) {
      const int nb0 = pair_block(pp);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks)
          kf[i][ks].u = frag_at(ktile, (nb0 + i) * 16 + prow, ks * 4 + quarter);
    };
    auto tile_body = [&](auto nwords_c) {
      constexpr int NWD = decltype(nwords_c)::value;
      uint32_t neg[NWD];
#pragma unroll
      for (int j = 0; j < NWD; ++j) neg[j] = 0;
      auto do_pair = [&](int pp, const Frag (&kf)[2][kKSteps]) {
#pragma unroll
        for (int j = 0; j < NWD; ++j) {
          f32x4 acc[2][2];
#pragma unroll
          for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int i = 0; i < 2; ++i) acc[mb][i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < kKSteps; ++ks)
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
              for (int i = 0; i < 2; ++i)
                acc[mb][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(preg[j][ks][mb].v, kf[i][ks].v, acc[mb][i], 0, 0, 0);
          // sign bits -> this quarter's byte per key block (higher block first)
#pragma unroll
          for (int i = 1; i >= 0; --i)
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
              for (int r = 0; r < 4; ++r) neg[j] = __builtin_amdgcn_alignbit(neg[j], __float_as_uint(acc[mb][i][r]), 31);
          if (pp & 1) {
            // all four blocks of the 64-key group are in: 4 x 4 byte transpose between
            // the quarters (as in hash_keys_kernel), lane x gets key x's word
            const int w = wave + kHashWaves * j;
            const int nbits = min(cpw, L - w * cpw) * P;
            const uint32_t valid = nbits >= 32 ? 0xffffffffu : ((1u << nbits) - 1u);
            const uint32_t t = lane_xor16(neg[j], quarter & 1);
            const uint32_t x = __builtin_amdgcn_perm(t, neg[j], sel1);
            const uint32_t u = lane_xor32(x, quarter & 2);
            const uint32_t word = __builtin_amdgcn_perm(u, x, sel2);
            const int key = s0 + (pp >> 1) * kKeysPerWave + lane;
            if (key < S && in_cache(pos0 + key, Tcap)) codes_pair[(int64_t)w * Tcap + pos0 + key] = ~word & valid;
          }
        }
      };
      Frag kfa[2][kKSteps], kfb[2][kKSteps];
      load_pair(0, kfa);
#pragma unroll
      for (int pp = 0; pp < kStreamTile / 32; pp += 2) {
        load_pair(pp + 1, kfb);
        do_pair(pp, kfa);
        if (pp + 2 < kStreamTile / 32) load_pair(pp + 2, kfa);
        do_pair(pp + 1, kfb);
      }
    };
    // (uniform per wave: waves 0 .. NW % 8 - 1 own one word more than the others)
    const int my_words = wave < NW ? (NW - wave + kHashWaves - 1) / kHashWaves : 0;
    if (my_words == 3) tile_body(std::integral_constant<int, 3>{});
    else if (my_words == 2) tile_body(std::integral_constant<int, 2>{});
    else if (my_words == 1) tile_body(std::integral_constant<int, 1>{});
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
  const SocketDeviceLimits& lim = socket_device_limits();
  hipStream_t s = (hipStream_t)stream;
  {
    // enough 128-key tiles to keep every CU streaming: the variant with the planes in registers
    const int tiles_per_row = (S + kStreamTile - 1) / kStreamTile;
    const int64_t n_tiles64 = (int64_t)B * Hkv * tiles_per_row;
    SOCKET_REQUIRE(n_tiles64 < (1LL << 30), SOCKET_ERR_SHAPE);  // tile + grid size stays an int
    if (dtype == SOCKET_BF16 && NW <= kStreamMaxWords && n_tiles64 >= lim.cu_count &&
        2 * kStreamStageBytes <= lim.max_lds_per_block) {
      const size_t lds = 2 * (size_t)kStreamStageBytes;
      auto kern = hash_keys_stream_kernel;
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)lds) != hipSuccess)
        return SOCKET_ERR_LAUNCH;
      const int n_wg = (int)(n_tiles64 < lim.cu_count ? n_tiles64 : lim.cu_count);
      hipLaunchKernelGGL(kern, dim3(n_wg), dim3(kHashThreads), lds, s, (const uint16_t*)k, (const uint16_t*)v,
                         k_stride_b, k_stride_h, k_stride_s, v_stride_b, v_stride_h, v_stride_s,
                         (const uint16_t*)planes_words, codes, v_norm, pos_b, t0, Hkv, S, L, P, NW, Tcap,
                         tiles_per_row, (int)n_tiles64);
      SOCKET_LAUNCH_CHECK();
      return SOCKET_OK;
    }
  }
  const int tiles_per_row = (S + kKeysPerWave - 1) / kKeysPerWave;
  const int64_t n_tiles64 = (int64_t)B * Hkv * tiles_per_row;
  SOCKET_REQUIRE(n_tiles64 < (1LL << 31), SOCKET_ERR_SHAPE);
  const int n_tiles = (int)n_tiles64;
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
