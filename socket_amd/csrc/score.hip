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
//    lane, fully coalesced, three words ahead of their use.  The table may be
//    fp32 or bf16 (a bf16 soft-hash producer loses nothing, halves the LDS bytes
//    per gather and lets the matrix core do the four head adds of a lookup).
//    A table given in the grouped layout (the LDS image itself, written by the
//    soft-hash kernel) is copied rather than interleaved, and for large launches
//    the copy is global_load_lds: global memory straight into LDS.
// (The reference's own operand layout, int16 codes per query head, is served by
// collide.hip.)
#include <type_traits>

#include "socket_common.h"

namespace {

// ---------------------------------------------------------------------------
// native packed scorer
// ---------------------------------------------------------------------------
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;

struct TabF32 {
  typedef float elem;
  static constexpr int kEnum = SOCKET_F32;
};
struct TabBF16 {
  typedef uint16_t elem;
  static constexpr int kEnum = SOCKET_BF16;
};

// One LDS entry (the GP heads' values for one bucket of one table) as raw words,
// so that the gather (load) and the accumulation can be scheduled apart.
template <int BYTES>
struct RawEntry;
template <>
struct RawEntry<2> { uint16_t w; };
template <>
struct RawEntry<4> { uint32_t w; };
template <>
struct RawEntry<8> { uint2 w; };
template <>
struct RawEntry<16> { uint4 w; };
template <>
struct RawEntry<32> { uint4 w[2]; };

template <int BYTES>
__device__ __forceinline__ RawEntry<BYTES> load_entry(const void* lds) {
  return *reinterpret_cast<const RawEntry<BYTES>*>(lds);
}

// bf16 entries are widened and added by the matrix core used as a four-wide
// adder: v_mfma_f32_4x4x4_16B_bf16 computes, in each of its 16 independent 4x4
// blocks (4 lanes each), D[i][j] = C[i][j] + sum_k A[i][k] * B[k][j], where lane
// j of a block supplies column B[:,j] (4 bf16 = one 8-byte LDS entry: the four
// heads' values) and holds column D[:,j] (4 fp32 = that lane's four head sums),
// and lane i supplies row A[i,:].  With A the identity (lane i holds e_i) this is
// acc[h] += entry[h] for h = 0..3 in one instruction, on a pipe that is
// otherwise idle, instead of four VALU operations.  The products are exact; the
// matrix core's accumulate may round differently from the fp32 adder in the last
// place (and flushes denormals), hence the 2e-6 relative bound stated for bf16
// tables; the fp32-table path uses plain adds and reproduces the reference sum
// exactly.
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// Streamed once: loads and stores that should not displace the table slices,
// which every tile of a (b, kv head) pair re-reads, from the L2.
__device__ __forceinline__ uint4 load_stream16(const uint32_t* p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void store_stream16(float* p, float a, float b, float c, float d) {
  float4_t v = {a, b, c, d};
  __builtin_nontemporal_store(v, reinterpret_cast<float4_t*>(p));
}

struct Bf16Select {
  short4_t identity_row;  // e_{lane % 4} as four bf16
};

__device__ __forceinline__ Bf16Select make_bf16_select(uint32_t bf16_one) {
  const int r = threadIdx.x & 3;
  uint2 w = make_uint2(0u, 0u);
  if (r == 0) w.x = bf16_one;
  else if (r == 1) w.x = bf16_one << 16;
  else if (r == 2) w.y = bf16_one;
  else w.y = bf16_one << 16;
  Bf16Select s;
  __builtin_memcpy(&s.identity_row, &w, 8);
  return s;
}

__device__ __forceinline__ void add4_bf16(float* acc, uint2 four, const Bf16Select& sel) {
  short4_t b;
  __builtin_memcpy(&b, &four, 8);
  float4_t c = {acc[0], acc[1], acc[2], acc[3]};
  c = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(sel.identity_row, b, c, 0, 0, 0);
  acc[0] = c[0];
  acc[1] = c[1];
  acc[2] = c[2];
  acc[3] = c[3];
}

// acc[g] += entry[g], fp32 table
template <int GP>
__device__ __forceinline__ void accumulate(float* acc, const RawEntry<GP * 4>& e, const TabF32*,
                                           const Bf16Select&) {
  if constexpr (GP == 1) {
    acc[0] += __uint_as_float(e.w);
  } else if constexpr (GP == 2) {
    acc[0] += __uint_as_float(e.w.x);
    acc[1] += __uint_as_float(e.w.y);
  } else if constexpr (GP == 4) {
    acc[0] += __uint_as_float(e.w.x);
    acc[1] += __uint_as_float(e.w.y);
    acc[2] += __uint_as_float(e.w.z);
    acc[3] += __uint_as_float(e.w.w);
  } else {
#pragma unroll
    for (int v = 0; v < 2; ++v) {
      acc[4 * v + 0] += __uint_as_float(e.w[v].x);
      acc[4 * v + 1] += __uint_as_float(e.w[v].y);
      acc[4 * v + 2] += __uint_as_float(e.w[v].z);
      acc[4 * v + 3] += __uint_as_float(e.w[v].w);
    }
  }
}

// acc[g] += entry[g], bf16 table
template <int GP>
__device__ __forceinline__ void accumulate(float* acc, const RawEntry<GP * 2>& e, const TabBF16*,
                                           const Bf16Select& sel) {
  if constexpr (GP == 1) {
    acc[0] += bf16_bits_to_f32(e.w);
  } else if constexpr (GP == 2) {
    float a4[4] = {acc[0], acc[1], 0.f, 0.f};
    add4_bf16(a4, make_uint2(e.w, 0u), sel);
    acc[0] = a4[0];
    acc[1] = a4[1];
  } else if constexpr (GP == 4) {
    add4_bf16(acc, e.w, sel);
  } else {
    add4_bf16(acc, make_uint2(e.w.x, e.w.y), sel);
    add4_bf16(acc + 4, make_uint2(e.w.z, e.w.w), sel);
  }
}

// One 16-byte vector of table elements per head (GP heads) -> the same elements
// regrouped entry-major: out word stream holds entry e = {head 0..GP-1}.
template <int GP, class TT>
__device__ __forceinline__ void interleave_heads(const uint4 (&x)[GP], uint4 (&out)[GP]) {
  constexpr int EPV = 16 / (int)sizeof(typename TT::elem);
  uint32_t xw[GP][4], ow[4 * GP];
#pragma unroll
  for (int g = 0; g < GP; ++g) {
    xw[g][0] = x[g].x;
    xw[g][1] = x[g].y;
    xw[g][2] = x[g].z;
    xw[g][3] = x[g].w;
  }
  if (sizeof(typename TT::elem) == 4) {
#pragma unroll
    for (int e = 0; e < EPV; ++e)
#pragma unroll
      for (int g = 0; g < GP; ++g) ow[e * GP + g] = xw[g][e];
  } else if (GP == 1) {
#pragma unroll
    for (int k = 0; k < 4; ++k) ow[k] = xw[0][k];
  } else {
#pragma unroll
    for (int e = 0; e < EPV; ++e)
#pragma unroll
      for (int g = 0; g < GP; g += 2) {
        const uint32_t lo = (xw[g][e >> 1] >> (16 * (e & 1))) & 0xffffu;
        const uint32_t hi = (xw[g + 1][e >> 1] >> (16 * (e & 1))) & 0xffffu;
        ow[(e * GP + g) >> 1] = lo | (hi << 16);
      }
  }
#pragma unroll
  for (int v = 0; v < GP; ++v) out[v] = make_uint4(ow[4 * v], ow[4 * v + 1], ow[4 * v + 2], ow[4 * v + 3]);
}

// PT: P known at compile time (0 = use the runtime value).
// The table slice of the tables held by `chunk_words` packed words sits in LDS;
// with two LDS buffers the next slice is fetched into registers while the
// current one is being gathered from, and there is one barrier per slice.
// One tile of one workgroup's (b, kv head, head part).  `table_resident`: the whole
// table is already in LDS from the tile this workgroup did before (single-buffer
// launches only), so nothing is copied.  `red_off`: byte offset in LDS, past the
// table buffers, of the small scratch area of the key-range reduction.
// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
template <int N, int I = 0, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

template <int GP, class TT, int KT4, int THREADS, int PT, int MODE>
__device__ __forceinline__ void score_tile(
    const typename TT::elem* __restrict__ q_probs, const uint32_t* __restrict__ codes,
    const uint16_t* __restrict__ v_norm, const int32_t* __restrict__ lens,
    float* __restrict__ scores, int Hq, int Hkv, int G, int L, int P_rt, int R, int T,
    int64_t Tcap, int64_t score_stride, int NW, int chunk_words, int nbuf,
    int n_tiles, uint32_t bf16_one, uint32_t* __restrict__ row_range, int hsplit, int pair, int tile,
    bool table_resident, int red_off, int tile_tokens) {
  // tile_tokens: tokens between the starts of two tiles, a multiple of 4 and at most the
  // 4 * KT4 * THREADS a workgroup can hold (less: the lanes past it stay idle, so that a
  // context which overhangs a whole number of tiles by a little is cut into one more, equal,
  // tile per row rather than scored by half as many workgroups of the next size up)
  // MODE: 0 = table in the reference layout [B,Hq,L,R], interleaved while staged;
  // 1 = grouped table, copied through registers; 2 = grouped table, copied from
  // global memory straight into LDS
  constexpr bool grouped = MODE != 0;
  constexpr bool DMA = MODE == 2;
  typedef typename TT::elem TE;
  const Bf16Select sel = make_bf16_select(bf16_one);
  constexpr int EPV = 16 / (int)sizeof(TE);   // table elements per 16-byte vector
  constexpr int SL = 1024 / THREADS;           // staging slots (one 16-byte vector per head) per lane
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

  const int P = PT ? PT : P_rt;
  const int cpw = 32 / P;
  const uint32_t code_mask = (1u << P) - 1u;
  // DMA: table slices (grouped layout only) go from global memory straight into
  // LDS, 1 KB per instruction, shared out over the waves; no staging registers,
  // no interleave, no LDS store instructions.
  constexpr int CT = THREADS;  // lanes that own tokens
  constexpr int TW = CT * 4 * KT4;

  // A group of more than GP query heads is shared out over `hsplit` workgroups
  // (each streams the pair's codes): this one takes heads [h0, h0 + G) of it.
  const int vpair = pair;  // (b, kv head, part of the head group)
  const int h0 = (pair % hsplit) * GP;
  pair /= hsplit;
  const int b = pair / Hkv, kvh = pair % Hkv;
  const int head0 = b * Hq + kvh * G + h0;   // first of this workgroup's query heads (rows of q_probs, scores)
  G = min(GP, G - h0);
  const int tid = threadIdx.x;
  const int len = lens ? min(lens[b], T) : T;

  const int tile0 = tile * tile_tokens;               // first token of the tile
  const int tile_end = min(T, tile0 + tile_tokens);   // one past its last
  if (tile0 >= len) {
    // nothing cached this far out for this sequence: the tile is all masked
    for (int g = 0; g < G; ++g) {
      float* dst = scores + ((int64_t)(head0 + g)) * score_stride + tile0;
      const int n = tile_end - tile0;
      for (int t = tid * 4; t < n; t += THREADS * 4) {
        if (t + 4 <= n) {
          store_stream16(dst + t, -INFINITY, -INFINITY, -INFINITY, -INFINITY);
        } else {
          for (int i = t; i < n; ++i) dst[i] = -INFINITY;
        }
      }
    }
    if (row_range && tid < G) {
      uint32_t* dst = row_range + (((int64_t)(head0 + tid)) * n_tiles + tile) * 2;
      dst[0] = 0xffffffffu;
      dst[1] = 0u;
    }
    return;
  }

  const uint32_t* codes_pair = codes + (int64_t)pair * NW * Tcap;
  // reference layout: row `head0` of [B*Hq, L, R]; grouped layout: block `vpair` of
  // [B*Hkv*hsplit, L, R, GP], which is the LDS layout itself
  const TE* qp_pair = grouped ? q_probs + (int64_t)vpair * L * R * GP : q_probs + ((int64_t)head0) * L * R;
  const int chunk_tables = chunk_words * cpw;
  const int chunk_elems = chunk_tables * R * GP;  // table elements per LDS buffer

  // tsafe: where a lane group without tokens (tile tail) reads instead, so that
  // code loads need no predicate; its results are never stored
  int tbase[KT4], tsafe[KT4];
  bool live[KT4];
#pragma unroll
  for (int j = 0; j < KT4; ++j) {
    tbase[j] = tile0 + j * (CT * 4) + tid * 4;
    live[j] = tid < CT && tbase[j] < tile_end;
    tsafe[j] = live[j] ? tbase[j] : tile0;
  }

  // The value norms of the lane's tokens are requested now and used in the epilogue:
  // asked for there, every tile would end on one exposed memory latency with nothing
  // else on the CU to cover it.
  const uint16_t* vn_pair = v_norm + (int64_t)pair * Tcap;
  uint2 vn_raw[KT4];
#pragma unroll
  for (int j = 0; j < KT4; ++j) vn_raw[j] = *reinterpret_cast<const uint2*>(vn_pair + tsafe[j]);

  float acc[KT4][4][GP];
#pragma unroll
  for (int j = 0; j < KT4; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int g = 0; g < GP; ++g) acc[j][i][g] = 0.f;

  // DMA: this wave's share of the slice that starts at table l0 -> buffer `buf`
  // (every 16th 1 KB piece); returns nothing, completion is awaited with vmcnt
  auto dma_slice = [&](int l0, int buf) {
    const int nt = min(chunk_tables, L - l0);
    const int bytes = nt * R * GP * (int)sizeof(TE);
    const char* src = reinterpret_cast<const char*>(qp_pair + (int64_t)l0 * R * GP);
    unsigned char* dst = lds_raw + (size_t)buf * chunk_elems * sizeof(TE);
    const int lane = tid & 63, wave = tid >> 6;
    for (int o = wave * 1024; o < bytes; o += (THREADS / SOCKET_WAVE) * 1024) {
      if (o + lane * 16 < bytes) lds_dma16(src + o + lane * 16, dst + o);
    }
  };
  // A wave whose first token lies at or past the cached length has nothing to
  // gather (a ragged batch; a context that overhangs the last full tile by a
  // little): it only takes its share of the table copies and meets the barriers.
  // The test is wave-uniform and made once, outside the gather loop.
  const bool wave_active = !DMA || tile0 + (tid >> 6) * 256 < min(len, tile_end);
  if (!wave_active) {
    const int chunk_tables_ = chunk_words * cpw;
    if (!table_resident) {
      dma_slice(0, 0);
      wait_vmcnt(0);
      __syncthreads();
    }
    int chunk_ = 0;
    for (int w0 = 0; w0 < NW; w0 += chunk_words, ++chunk_) {
      const int buf = nbuf == 2 ? (chunk_ & 1) : 0;
      if (w0 + chunk_words < NW) dma_slice(w0 * cpw + chunk_tables_, buf ^ 1);
      wait_vmcnt(0);
      __syncthreads();
    }
  } else {
    // Packed words of the lane's token groups, kPrefetch words deep: ring[0] is the
    // word being consumed, ring[d] the word d steps ahead.  The code stream is the
    // HBM traffic of this kernel and a CU needs tens of KB of it in flight to cover
    // the memory latency; one word ahead (16 B x tokens/4 per lane) is not enough.
    // In the direct-to-LDS variant word w lives in slot w % kPrefetch for as long as
    // it is needed and the word loop is unrolled by kPrefetch, so that every slot is
    // a fixed set of registers: a ring that is shifted at the loop's back edge has
    // its newest, still outstanding load copied there, and the copy waits for it --
    // every word would then cost a full memory latency.
    // (Only where the adds run on the matrix core: with plain adds the compiler
    // lets the unrolled loop's register use run far past what a 1024-thread
    // workgroup has.  There it serves the direct copies and the double-buffered
    // register staging alike.)
    constexpr bool kFlat = GP > 1 && std::is_same<TT, TabBF16>::value;
    constexpr int kPrefetch = kFlat ? (DMA ? (KT4 == 1 ? 8 : 4) : (KT4 == 2 && THREADS == 1024 ? 2 : 3)) : DMA ? 4 : 3;
    uint4 ring[kPrefetch][KT4];
    // (the first slice's copies go out ahead of the code words, so that the wait below
    // can leave all but the first word in flight)
    if (DMA && !table_resident) {
      dma_slice(0, 0);
      // the copies are issued before the code words below: the start-up wait counts on that
      // order, and nothing else in the source ties the two together
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int d = 0; d < kPrefetch; ++d)
#pragma unroll
      for (int j = 0; j < KT4; ++j)
        ring[d][j] = load_stream16(codes_pair + (int64_t)min(d, NW - 1) * Tcap + tsafe[j]);
    // group j has consumed its current word: shift the ring and fetch the word
    // kPrefetch steps ahead (past the end it refetches the last word, unused)
    auto advance = [&](int j, int w) {
#pragma unroll
      for (int d = 0; d + 1 < kPrefetch; ++d) ring[d][j] = ring[d + 1][j];
      ring[kPrefetch - 1][j] = load_stream16(codes_pair + (int64_t)min(w + kPrefetch, NW - 1) * Tcap + tsafe[j]);
    };

    // slice staging: slot s covers table elements [s*EPV, (s+1)*EPV) of every head
    uint4 stage[SL][GP];
    auto stage_load = [&](int l0) {
      const int nt = min(chunk_tables, L - l0);
      const int nslots = (nt * R) / EPV;
      if (grouped) {  // straight copy: 16-byte vector i of the slice goes to vector i of the buffer
        const uint4* src = reinterpret_cast<const uint4*>(qp_pair + (int64_t)l0 * R * GP);
#pragma unroll
        for (int k = 0; k < SL; ++k)
#pragma unroll
          for (int g = 0; g < GP; ++g) {
            const int i = tid + (k * GP + g) * THREADS;
            // (unconditional assignment: an element left unwritten on one path made
            // the compiler keep the whole array in scratch memory)
            stage[k][g] = (i < nslots * GP) ? src[i] : make_uint4(0, 0, 0, 0);
          }
        return;
      }
      const TE* src = qp_pair + (int64_t)l0 * R;
#pragma unroll
      for (int k = 0; k < SL; ++k) {
        const int s = tid + k * THREADS;
        if (s < nslots) {
#pragma unroll
          for (int g = 0; g < GP; ++g)
            stage[k][g] = (g < G) ? *reinterpret_cast<const uint4*>(src + (int64_t)g * L * R + (int64_t)s * EPV)
                                  : make_uint4(0, 0, 0, 0);
        }
      }
    };
    auto stage_store = [&](int l0, int buf) {
      const int nt = min(chunk_tables, L - l0);
      const int nslots = (nt * R) / EPV;
      uint4* dst = reinterpret_cast<uint4*>(lds_raw + (size_t)buf * chunk_elems * sizeof(TE));
      if (grouped) {
#pragma unroll
        for (int k = 0; k < SL; ++k)
#pragma unroll
          for (int g = 0; g < GP; ++g) {
            const int i = tid + (k * GP + g) * THREADS;
            if (i < nslots * GP) dst[i] = stage[k][g];
          }
        return;
      }
#pragma unroll
      for (int k = 0; k < SL; ++k) {
        const int s = tid + k * THREADS;
        if (s < nslots) {
          uint4 o[GP];
          interleave_heads<GP, TT>(stage[k], o);
#pragma unroll
          for (int v = 0; v < GP; ++v) dst[(size_t)s * GP + v] = o[v];
        }
      }
    };

    const bool staged = nbuf == 2;
    if (DMA) {
      if (!table_resident) {
        // loads retire in order: with the words 1 .. kPrefetch-1 still outstanding, slice
        // 0 and word 0 have landed
        wait_vmcnt((kPrefetch - 1) * KT4);
        __syncthreads();  // slice 0 is in place
      }
    } else if (staged) {
      stage_load(0);
      stage_store(0, 0);
      __syncthreads();
    }

    bool flat_done = false;
    if constexpr (kFlat) if (DMA || staged) {
      flat_done = true;
      constexpr int EB = GP * (int)sizeof(TE);
      constexpr int CPW = PT ? 32 / PT : 1;
      // one word of one token group: all its tables, `d` = the word's ring slot
      auto word_full = [&](const TE* tw, int w, auto slot) {
        constexpr int d = decltype(slot)::value;
        // The lookups are cut into batches of four (one table, one group of four
        // tokens) and the LDS reads of batch k+1 are issued before batch k is
        // accumulated, so the gather latency overlaps the adds.
        constexpr int NB = KT4 * CPW;
        RawEntry<EB> ent[2][4];
        auto issue = [&](int bi, RawEntry<EB>(&dst)[4]) {
          const int j = bi / CPW, jj = bi % CPW;
          const uint32_t wv[4] = {ring[d][j].x, ring[d][j].y, ring[d][j].z, ring[d][j].w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t code = __builtin_amdgcn_ubfe(wv[i], jj * (PT ? PT : 1), PT ? PT : 1);
            dst[i] = load_entry<EB>(tw + (size_t)jj * R * GP + (size_t)code * GP);
          }
          if (jj == CPW - 1)  // last use of this group's word: its slot takes the word kPrefetch ahead
            ring[d][j] = load_stream16(codes_pair + (int64_t)min(w + kPrefetch, NW - 1) * Tcap + tsafe[j]);
        };
        issue(0, ent[0]);
#pragma unroll
        for (int bi = 0; bi < NB; ++bi) {
          if (bi + 1 < NB) issue(bi + 1, ent[(bi + 1) & 1]);
          const int j = bi / CPW;
#pragma unroll
          for (int i = 0; i < 4; ++i) accumulate<GP>(acc[j][i], ent[bi & 1][i], (const TT*)nullptr, sel);
        }
      };
      // a word with fewer real tables than it has room for (the last one), or a
      // code width that is not a template constant
      auto word_any = [&](const TE* tw, int w, int ntw, auto slot) {
        constexpr int d = decltype(slot)::value;
#pragma unroll
        for (int j = 0; j < KT4; ++j) {
          const uint32_t wv[4] = {ring[d][j].x, ring[d][j].y, ring[d][j].z, ring[d][j].w};
          for (int jj = 0; jj < ntw; ++jj) {
            const TE* tb = tw + (size_t)jj * R * GP;
            const int sh = jj * P;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const uint32_t code = (wv[i] >> sh) & code_mask;
              accumulate<GP>(acc[j][i], load_entry<EB>(tb + (size_t)code * GP), (const TT*)nullptr, sel);
            }
          }
          ring[d][j] = load_stream16(codes_pair + (int64_t)min(w + kPrefetch, NW - 1) * Tcap + tsafe[j]);
        }
      };

      int w0 = 0, wend = min(chunk_words, NW), buf = 0;
      if (wend < NW) {
        if (DMA) dma_slice(wend * cpw, 1);
        else stage_load(wend * cpw);
      }
      // One word: the slice switch if the word opens a slice, then its lookups.
      // `full`: the word holds CPW real tables (straight-line body).
      auto word = [&](int w, auto slot, auto full) {
        if (w == wend) {
          // The copies of the slice that starts here were issued at the top of the
          // one that ends; since then this wave has issued one code load per word
          // and token group.  Loads retire in order, so allowing that many to be
          // outstanding, less one word's worth as a margin, means the copies have
          // landed (a slice of one word: no margin, its loads are pinned by the
          // scheduling barrier that closes the word).
          if (DMA) wait_vmcnt(max(wend - w0 - 1, 1) * KT4);
          else stage_store(w * cpw, buf ^ 1);  // the slice fetched into registers while the last one was read
          __syncthreads();
          if (nbuf == 2) buf ^= 1;
          w0 = w;
          wend = min(w + chunk_words, NW);
          if (wend < NW) {
            if (DMA) dma_slice(wend * cpw, buf ^ 1);
            else stage_load(wend * cpw);
          }
        }
        const TE* tw =
            reinterpret_cast<const TE*>(lds_raw) + (size_t)buf * chunk_elems + (size_t)(w - w0) * cpw * R * GP;
        if constexpr (decltype(full)::value) word_full(tw, w, slot);
        else word_any(tw, w, min(cpw, L - w * cpw), slot);
        // keep the words apart: left alone, the scheduler hoists the gathers of later
        // words over the adds of earlier ones until the registers run out
        __builtin_amdgcn_sched_barrier(0);
      };
      // Words [0, wlimit).  Whole rounds of the ring run without a test per word: a
      // path on which some slots are skipped would make the compiler assume, where a
      // slot is consumed, that its load may be the newest one outstanding, and wait
      // for everything.  The two bodies are never mixed in one loop either: the two
      // definitions of a slot's next word would end up in different registers and be
      // copied at the join, and the copy of an outstanding load waits for it.
      auto run = [&](int wlimit, auto full) {
        int wb = 0;
        for (; wb + kPrefetch <= wlimit; wb += kPrefetch)
          static_for<kPrefetch>([&](auto slot) { word(wb + decltype(slot)::value, slot, full); });
        static_for<kPrefetch>([&](auto slot) {
          const int w = wb + decltype(slot)::value;
          if (w < wlimit) word(w, slot, full);
        });
      };
      if constexpr (PT != 0) {
        const int nfull = min(NW, L / CPW);  // all but possibly the last word
        run(nfull, std::true_type{});
        if (nfull < NW)
          static_for<kPrefetch>([&](auto slot) {
            if (nfull % kPrefetch == decltype(slot)::value) word(nfull, slot, std::false_type{});
          });
      } else {
        run(NW, std::false_type{});
      }
      if (DMA) wait_vmcnt(0);
      __syncthreads();
    }
    if (!flat_done) {
    int chunk = 0;
    for (int w0 = 0; w0 < NW; w0 += chunk_words, ++chunk) {
      const int l0 = w0 * cpw;
      const int buf = staged ? (chunk & 1) : 0;
      const bool more = w0 + chunk_words < NW;
      if (DMA) {
        if (more) dma_slice(l0 + chunk_tables, buf ^ 1);
      } else if (staged) {
        if (more) stage_load(l0 + chunk_tables);
      } else {
        __syncthreads();  // gathers of the previous slice are done
        const int nt = min(chunk_tables, L - l0);
        const int nslots = (nt * R) / EPV;
        const TE* src = qp_pair + (int64_t)l0 * R;
        uint4* dst = reinterpret_cast<uint4*>(lds_raw);
        if (grouped) {
          const uint4* src16 = reinterpret_cast<const uint4*>(qp_pair + (int64_t)l0 * R * GP);
          for (int i = tid; i < nslots * GP; i += THREADS) dst[i] = src16[i];
        }
        for (int s = tid; s < (grouped ? 0 : nslots); s += THREADS) {
          uint4 x[GP], o[GP];
#pragma unroll
          for (int g = 0; g < GP; ++g)
            x[g] = (g < G) ? *reinterpret_cast<const uint4*>(src + (int64_t)g * L * R + (int64_t)s * EPV)
                           : make_uint4(0, 0, 0, 0);
          interleave_heads<GP, TT>(x, o);
#pragma unroll
          for (int v = 0; v < GP; ++v) dst[(size_t)s * GP + v] = o[v];
        }
        __syncthreads();
      }

      const TE* table = reinterpret_cast<const TE*>(lds_raw) + (size_t)buf * chunk_elems;
      const int wend = min(w0 + chunk_words, NW);
      for (int w = w0; w < wend; ++w) {
        const int ntw = min(cpw, L - w * cpw);
        const TE* tw = table + (size_t)(w - w0) * cpw * R * GP;
        constexpr int EB = GP * (int)sizeof(TE);
        if (PT != 0 && ntw == 32 / (PT ? PT : 1)) {
          // Every table of the word is real: straight-line code.  The lookups are
          // cut into batches of four (one table, one group of four tokens) and the
          // LDS reads of batch k+1 are issued before batch k is accumulated, so the
          // gather latency overlaps the adds instead of preceding them.
          constexpr int CPW = PT ? 32 / PT : 1;
          constexpr int NB = KT4 * CPW;
          RawEntry<EB> ent[2][4];
          auto issue = [&](int bi, RawEntry<EB>(&dst)[4]) {
            const int j = bi / CPW, jj = bi % CPW;
            const uint32_t wv[4] = {ring[0][j].x, ring[0][j].y, ring[0][j].z, ring[0][j].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const uint32_t code = __builtin_amdgcn_ubfe(wv[i], jj * (PT ? PT : 1), PT ? PT : 1);
              dst[i] = load_entry<EB>(tw + (size_t)jj * R * GP + (size_t)code * GP);
            }
            if (jj == CPW - 1) advance(j, w);  // last use of this group's word
          };
          issue(0, ent[0]);
#pragma unroll
          for (int bi = 0; bi < NB; ++bi) {
            if (bi + 1 < NB) issue(bi + 1, ent[(bi + 1) & 1]);
            const int j = bi / CPW;
#pragma unroll
            for (int i = 0; i < 4; ++i) accumulate<GP>(acc[j][i], ent[bi & 1][i], (const TT*)nullptr, sel);
          }
        } else {
#pragma unroll
          for (int j = 0; j < KT4; ++j) {
            const uint32_t wv[4] = {ring[0][j].x, ring[0][j].y, ring[0][j].z, ring[0][j].w};
            for (int jj = 0; jj < ntw; ++jj) {
              const TE* tb = tw + (size_t)jj * R * GP;
              const int sh = jj * P;
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const uint32_t code = (wv[i] >> sh) & code_mask;
                accumulate<GP>(acc[j][i], load_entry<EB>(tb + (size_t)code * GP), (const TT*)nullptr, sel);
              }
            }
            advance(j, w);
          }
        }
      }

      if (DMA) {
        // The direct loads were issued at the top of the slice; since then this wave
        // has issued one code prefetch per word and token group.  Loads retire in
        // order, so allowing that many to be outstanding, less one word's worth as a
        // margin, means the direct loads have landed.
        wait_vmcnt(max(0, (min(w0 + chunk_words, NW) - w0 - 1) * KT4));
        __syncthreads();
      } else if (staged) {
        if (more) stage_store(l0 + chunk_tables, buf ^ 1);
        __syncthreads();
      }
    }
    }  // staged / in-place variants

  }

  // epilogue: multiply by the value norm, mask, store one float4 per head; on
  // request also the tile's range of score keys per head, for the select kernel
  uint32_t kmin[GP], kmax[GP];
#pragma unroll
  for (int g = 0; g < GP; ++g) {
    kmin[g] = 0xffffffffu;
    kmax[g] = 0u;
  }
#pragma unroll
  for (int j = 0; j < KT4; ++j) {
    if (!live[j]) continue;
    const uint2 vraw = vn_raw[j];
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
      for (int i = 0; i < 4; ++i) {
        const bool valid = tbase[j] + i < len;
        o[i] = valid ? acc[j][i][g] * vn[i] : -INFINITY;
        if (valid) {
          const uint32_t key = score_to_key(o[i]);
          kmin[g] = min(kmin[g], key);
          kmax[g] = max(kmax[g], key);
        }
      }
      float* dst = scores + ((int64_t)(head0 + g)) * score_stride + tbase[j];
      if (tbase[j] + 4 <= T) {
        store_stream16(dst, o[0], o[1], o[2], o[3]);
      } else {
        for (int i = 0; i < 4 && tbase[j] + i < T; ++i) dst[i] = o[i];
      }
    }
  }
  if (row_range) {
    const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int g = 0; g < GP; ++g) {
#pragma unroll
      for (int d = 32; d > 0; d >>= 1) {
        kmin[g] = min(kmin[g], (uint32_t)__shfl_xor((int)kmin[g], d, SOCKET_WAVE));
        kmax[g] = max(kmax[g], (uint32_t)__shfl_xor((int)kmax[g], d, SOCKET_WAVE));
      }
    }
    __syncthreads();  // an earlier tile's readers of the scratch area are done
    uint32_t* red = reinterpret_cast<uint32_t*>(lds_raw + red_off);
    if (lane == 0) {
#pragma unroll
      for (int g = 0; g < GP; ++g) {
        red[(wave * GP + g) * 2] = kmin[g];
        red[(wave * GP + g) * 2 + 1] = kmax[g];
      }
    }
    __syncthreads();
    if (tid < G) {
      uint32_t lo = 0xffffffffu, hi = 0u;
      for (int w = 0; w < THREADS / 64; ++w) {
        lo = min(lo, red[(w * GP + tid) * 2]);
        hi = max(hi, red[(w * GP + tid) * 2 + 1]);
      }
      uint32_t* dst = row_range + (((int64_t)(head0 + tid)) * n_tiles + tile) * 2;
      dst[0] = lo;
      dst[1] = hi;
    }
  }
}

template <int GP, class TT, int KT4, int THREADS, int PT, int MODE>
__global__ __launch_bounds__(THREADS) void score_packed_kernel(
    const typename TT::elem* __restrict__ q_probs, const uint32_t* __restrict__ codes,
    const uint16_t* __restrict__ v_norm, const int32_t* __restrict__ lens,
    float* __restrict__ scores, int Hq, int Hkv, int G, int L, int P_rt, int R, int T,
    int64_t Tcap, int64_t score_stride, int NW, int chunk_words, int nbuf, int n_pairs,
    int n_tiles, int n_launch_tiles, int xcd_remap, uint32_t bf16_one, uint32_t* __restrict__ row_range,
    int hsplit, int red_off, int tile_tokens) {
  // Workgroup -> (pair, tile).  Workgroups are dealt to the 8 XCDs round-robin
  // by linear id; with the remap all tiles of one (b, kv head), and all the
  // workgroups that share its query heads out between them, land on one XCD: its
  // L2 serves that pair's table slices to every tile, and the pair's code stream
  // comes from HBM once however many workgroups read it.
  int pair, tile;
  {
    const int n = blockIdx.x;
    if (xcd_remap) {
      const int xcd = n & 7, slot = n >> 3;
      const int per_kv = n_launch_tiles * hsplit;
      const int rem = slot % per_kv;
      pair = ((slot / per_kv) * 8 + xcd) * hsplit + rem % hsplit;
      tile = rem / hsplit;
    } else {
      pair = n / n_launch_tiles;
      tile = n % n_launch_tiles;
    }
  }
  if (pair >= n_pairs) return;
  score_tile<GP, TT, KT4, THREADS, PT, MODE>(q_probs, codes, v_norm, lens, scores, Hq, Hkv, G, L, P_rt, R, T, Tcap,
                                             score_stride, NW, chunk_words, nbuf, n_tiles, bf16_one, row_range,
                                             hsplit, pair, tile, false, red_off, tile_tokens);
  // A short last tile is not given a workgroup of its own (a whole extra round of
  // them on a full chip): the workgroup of the tile before it, with the table
  // still in LDS, does it as well.  Only where one workgroup holds a whole table.
  if constexpr (GP == 1 && MODE == 2) {
    if (n_launch_tiles < n_tiles && tile == n_launch_tiles - 1)
      score_tile<GP, TT, KT4, THREADS, PT, MODE>(q_probs, codes, v_norm, lens, scores, Hq, Hkv, G, L, P_rt, R, T,
                                                 Tcap, score_stride, NW, chunk_words, nbuf, n_tiles, bf16_one,
                                                 row_range, hsplit, pair, tile + 1, true, red_off, tile_tokens);
  }
}

// ---------------------------------------------------------------------------
// The same scoring as one persistent launch dealt from the cached lengths.
//
// Tokens are counted in units of 512 (what one wave scores in a tile: two groups of
// 256, four tokens per lane each).  The units of all (sequence, kv head) rows, each
// row as long as its sequence's cached length, are laid end to end and cut into equal
// stretches, whose tiles -- up to 16 units of one row for one part of the head group;
// the waves past a short tile's end skip the lookups and only join the copies and
// barriers -- are dealt to the workgroups (how: at `spread` below).  Across a tile
// boundary nothing drains: the last LDS slice of a tile is gathered from while
// the first slice of the next tile's table is being copied, the code ring fetches
// the next tile's first words where it would run past the current tile's last, and
// the sums of the finished tile are stored after the next tile's first slice has
// been waited for -- so the stores are the oldest memory operations by the time
// the following slice is waited on, and never hold a wait up.  Every wave runs the
// same instruction stream whether it has tokens in a tile or not (the ring's loads
// are unconditional, clamped to the tile's first token), which keeps the exact
// s_waitcnt counts of the slice copies valid for all of them.
// Needs: grouped table, entries of 2 or 4 heads x bf16 or fp32, every packed word
// full (L a multiple of 32/P), a word count that is a multiple of the ring depth,
// at most 64 sequences (one wave ranks their lengths).
// ---------------------------------------------------------------------------
constexpr int kFlatTileUnits = 16;   // waves of a workgroup: units of a full tile
constexpr int kFlatPrefetch = 4;

// KT4: token groups (of 256) per wave and tile: 2 (units of 512, tiles of 8192) where every CU
// has a tile or more, 1 (units of 256, tiles of 4096) below that, so that the waves of a
// workgroup stay in work when there are fewer tokens per CU.
template <int GP, class TT, int PT, int KT4>
__global__ __launch_bounds__(1024) void score_flat_kernel(
    const typename TT::elem* __restrict__ q_table, const uint32_t* __restrict__ codes,
    const uint16_t* __restrict__ v_norm, const int32_t* __restrict__ lens, float* __restrict__ scores,
    int B, int Hq, int Hkv, int G, int L, int R, int T, int64_t Tcap, int64_t score_stride, int NW,
    int chunk_words, int hsplit, uint32_t bf16_one, int fill_masked, int spread) {
  typedef typename TT::elem TE;
  constexpr int THREADS = 1024, kPrefetch = kFlatPrefetch;
  constexpr int kFlatUnit = 256 * KT4;               // tokens one wave scores in a tile
  constexpr int CPW = 32 / PT, EB = GP * (int)sizeof(TE);
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const Bf16Select sel = make_bf16_select(bf16_one);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int VS = Hkv * hsplit;                      // rows of the flattened space per sequence
  const int chunk_elems = chunk_words * CPW * R * GP;
  const int offl = wave * kFlatUnit + lane * 4;      // the lane's first token in a tile (group j: + 256 j)

  // ---- this workgroup's stretch of the flattened unit space -----------------------------
  int len_l = 0;                                     // lane l: cached length of sequence l
  if (lane < B) len_l = lens ? max(0, min(lens[lane], T)) : T;
  const int u_l = (len_l + kFlatUnit - 1) / kFlatUnit;
  const int incl = wave_incl_scan(u_l);
  // Rows are (sequence, kv head) pairs, each as long as its sequence, laid end to end in
  // units.  The row space is cut into equal stretches, and the tiles of a stretch -- every
  // row segment in ceil(n / 16) tiles of equal size, the head parts of a tile next to each
  // other -- are dealt in turn to the workgroups that share the stretch:
  //   spread == 0: a stretch per workgroup (it walks consecutive tiles of one row); workgroup
  //     n of N takes stretch (n % 8) * N / 8 + n / 8, so that neighbouring stretches, the
  //     tiles of one row, sit on one XCD (workgroup n runs on XCD n % 8) and share its L2;
  //   spread == 1: a stretch per XCD, its tiles dealt round to its workgroups.  They then work
  //     on neighbouring tiles at any moment: few tables are live in the XCD's L2 however many
  //     rows its stretch holds, and the parts of a wide head group, which read the same
  //     codes, read them at the same time -- the second read is served by the L2.
  const int nwg = gridDim.x;
  const bool by_xcd = (nwg & 7) == 0;
  const int ngroups = spread ? (by_xcd ? 8 : 1) : nwg, gsize = nwg / ngroups;
  const int xcd = by_xcd ? (int)(blockIdx.x & 7) : 0, slot = by_xcd ? (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  const int group = spread ? xcd : (by_xcd ? xcd * (nwg >> 3) + slot : slot);
  const int64_t total = (int64_t)__builtin_amdgcn_readlane(incl, 63) * Hkv;
  const int64_t x0 = total * group / ngroups, x1 = total * (group + 1) / ngroups;
  int wk_b = 0, wk_kvh = 0, wk_a = 0, wk_left = (int)(x1 - x0);
  int wk_skip = spread ? slot : 0;   // tiles of the stretch before this workgroup's next
  if (wk_left > 0) {
    wk_b = __popcll(__builtin_amdgcn_ballot_w64((int64_t)incl * Hkv <= x0));
    const int ub = __builtin_amdgcn_readlane(u_l, wk_b);
    const int rem = (int)(x0 - (int64_t)(__builtin_amdgcn_readlane(incl, wk_b) - ub) * Hkv);
    wk_kvh = rem / ub;
    wk_a = rem % ub;
  }
  struct Tile {   // tokens [start, end) of row (b, vp); end <= the sequence's length; start == end: none
    int b, vp, start, end;
  };
  auto next_tile = [&]() __attribute__((always_inline)) {
    Tile t{0, 0, 0, 0};
    while (wk_left > 0) {
      const int ub = __builtin_amdgcn_readlane(u_l, wk_b);
      const int n = min(ub - wk_a, wk_left);               // units of this row inside the stretch
      const int k = (n + kFlatTileUnits - 1) / kFlatTileUnits;
      const int sz = (n + k - 1) / k;
      const int cnt = k * hsplit;
      if (wk_skip < cnt) {
        const int j = wk_skip / hsplit;
        t.b = wk_b;
        t.vp = wk_kvh * hsplit + wk_skip % hsplit;
        t.start = (wk_a + j * sz) * kFlatUnit;
        t.end = min((wk_a + min((j + 1) * sz, n)) * kFlatUnit, __builtin_amdgcn_readlane(len_l, wk_b));
        wk_skip += gsize;
        return t;
      }
      wk_skip -= cnt;
      wk_left -= n;
      wk_a = 0;
      if (++wk_kvh == Hkv) {
        wk_kvh = 0;
        do ++wk_b;
        while (wk_b < B && __builtin_amdgcn_readlane(u_l, wk_b) == 0);
      }
    }
    return t;
  };
  auto codes_of = [&](const Tile& t) __attribute__((always_inline)) { return codes + (int64_t)(t.b * Hkv + t.vp / hsplit) * NW * Tcap; };
  auto table_of = [&](const Tile& t) __attribute__((always_inline)) { return q_table + (int64_t)(t.b * VS + t.vp) * L * R * GP; };

  float acc[KT4][4][GP];
  uint4 ring[kPrefetch][KT4];
  uint2 vn_raw[KT4];
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < KT4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < GP; ++g) acc[j][i][g] = 0.f;
  };
  // a wave's share of the table slice that starts at table l0 -> LDS buffer `b`
  auto dma_slice = [&](const TE* table, int l0, int b) __attribute__((always_inline)) {
    const int nt = min(chunk_words * CPW, L - l0);
    const int bytes = nt * R * GP * (int)sizeof(TE);
    const char* src = reinterpret_cast<const char*>(table + (int64_t)l0 * R * GP);
    unsigned char* dst = lds_raw + (size_t)b * chunk_elems * sizeof(TE);
    for (int o = wave * 1024; o < bytes; o += (THREADS / SOCKET_WAVE) * 1024)
      if (o + lane * 16 < bytes) lds_dma16(src + o + lane * 16, dst + o);
  };
  // the lane's token of group j in a tile, or the tile's first token where it has none
  auto token_of = [&](int start, int end, int j) __attribute__((always_inline)) {
    const int t = start + offl + j * 256;
    return t < end ? t : start;
  };
  auto load_norms = [&](const Tile& t) __attribute__((always_inline)) {
    const uint16_t* vn = v_norm + (int64_t)(t.b * Hkv + t.vp / hsplit) * Tcap;
#pragma unroll
    for (int j = 0; j < KT4; ++j) vn_raw[j] = *reinterpret_cast<const uint2*>(vn + token_of(t.start, t.end, j));
  };
  // sums of a finished tile -> scores
  auto flush = [&](const Tile& t) __attribute__((always_inline)) {
    const int part = t.vp % hsplit, kvh = t.vp / hsplit;
    const int geff = min(GP, G - part * GP);
    const int len = __builtin_amdgcn_readlane(len_l, t.b);
    float* row0 = scores + (int64_t)(t.b * Hq + kvh * G + part * GP) * score_stride;
#pragma unroll
    for (int j = 0; j < KT4; ++j) {
      const int tok = t.start + offl + j * 256;
      if (tok >= t.end) continue;
      const uint2 vraw = vn_raw[j];
      float vn[4];
      vn[0] = f16_bits_to_f32((uint16_t)(vraw.x & 0xffffu));
      vn[1] = f16_bits_to_f32((uint16_t)(vraw.x >> 16));
      vn[2] = f16_bits_to_f32((uint16_t)(vraw.y & 0xffffu));
      vn[3] = f16_bits_to_f32((uint16_t)(vraw.y >> 16));
#pragma unroll
      for (int g = 0; g < GP; ++g) {
        if (g >= geff) break;
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = tok + i < len ? acc[j][i][g] * vn[i] : -INFINITY;
        float* dst = row0 + (int64_t)g * score_stride + tok;
        if (tok + 4 <= T) {
          store_stream16(dst, o[0], o[1], o[2], o[3]);
        } else {
          for (int i = 0; i < 4 && tok + i < T; ++i) dst[i] = o[i];
        }
      }
    }
  };

  Tile cur = next_tile();
  if (cur.end > cur.start) {
    Tile nxt = next_tile();
    bool more = nxt.end > nxt.start;
    Tile prev = cur;
    // what the ring fetches: the tile being scored and the one after it (itself when it is the last)
    const uint32_t* cur_codes = codes_of(cur);
    const uint32_t* nxt_codes = more ? codes_of(nxt) : cur_codes;
    const TE* cur_table = table_of(cur);
    int buf = 0, w0 = 0, wend = min(chunk_words, NW);
    bool act = cur.start + wave * kFlatUnit < cur.end;

    // the slice after the one that has just become current
    auto issue_next_slice = [&]() __attribute__((always_inline)) {
      if (wend < NW) dma_slice(cur_table, wend * CPW, buf ^ 1);
      else if (more) dma_slice(table_of(nxt), 0, buf ^ 1);
    };
    // One word of the tile: the lookups of the wave's two token groups from the slice in
    // LDS (batches of four, the reads of batch k+1 issued before batch k is added up), then
    // the ring slot takes the word kPrefetch ahead -- of this tile or of the next.
    auto lookups = [&](const TE* tw, auto slot) __attribute__((always_inline)) {
      constexpr int d = decltype(slot)::value;
      constexpr int NB = KT4 * CPW;
      RawEntry<EB> ent[2][4];
      auto issue = [&](int bi, RawEntry<EB>(&dst)[4]) {
        const int j = bi / CPW, jj = bi % CPW;
        const uint32_t wv[4] = {ring[d][j].x, ring[d][j].y, ring[d][j].z, ring[d][j].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t code = __builtin_amdgcn_ubfe(wv[i], jj * PT, PT);
          dst[i] = load_entry<EB>(tw + (size_t)jj * R * GP + (size_t)code * GP);
        }
      };
      issue(0, ent[0]);
#pragma unroll
      for (int bi = 0; bi < NB; ++bi) {
        if (bi + 1 < NB) issue(bi + 1, ent[(bi + 1) & 1]);
        const int j = bi / CPW;
#pragma unroll
        for (int i = 0; i < 4; ++i) accumulate<GP>(acc[j][i], ent[bi & 1][i], (const TT*)nullptr, sel);
      }
    };
    auto refill = [&](int w, auto slot) __attribute__((always_inline)) {
      constexpr int d = decltype(slot)::value;
      const int wn = w + kPrefetch;
      const bool over = wn >= NW;
      const uint32_t* base = over ? nxt_codes + (int64_t)(wn - NW) * Tcap : cur_codes + (int64_t)wn * Tcap;
      const int st = over ? nxt.start : cur.start, en = over ? nxt.end : cur.end;
#pragma unroll
      for (int j = 0; j < KT4; ++j) ring[d][j] = load_stream16(base + token_of(st, en, j));
    };
    // `first`: word 0 of a tile that follows another one of this workgroup
    auto word = [&](int w, auto slot, auto first) __attribute__((always_inline)) {
      if (decltype(first)::value || w == wend) {
        // The copies of the slice that starts here were issued at the top of the one
        // that ends; since then this wave has issued one code load per word and token
        // group (each word's, pinned before the scheduling barrier that closes it).
        // Memory operations retire in order, so allowing that many to be outstanding --
        // less one word's worth as a margin where the slice had more than one word --
        // means the copies have landed.
        wait_vmcnt(max(wend - w0 - 1, 1) * KT4);
        __syncthreads();
        buf ^= 1;
        w0 = w;
        wend = min(w + chunk_words, NW);
        issue_next_slice();
        if constexpr (decltype(first)::value) {
          flush(prev);
          zero_acc();
          load_norms(cur);
        }
      }
      const TE* tw = reinterpret_cast<const TE*>(lds_raw) + (size_t)buf * chunk_elems + (size_t)(w - w0) * CPW * R * GP;
      if (act) lookups(tw, slot);
      refill(w, slot);
      // keep the words apart: left alone, the scheduler hoists the gathers of later
      // words over the adds of earlier ones until the registers run out
      __builtin_amdgcn_sched_barrier(0);
    };
    auto rounds_from = [&](int wb) __attribute__((always_inline)) {
      for (; wb < NW; wb += kPrefetch)
        static_for<kPrefetch>([&](auto s) __attribute__((always_inline)) { word(wb + decltype(s)::value, s, std::false_type{}); });
    };

    // ---- first tile: nothing is in flight yet ------------------------------------------------
    zero_acc();
    load_norms(cur);
    dma_slice(cur_table, 0, 0);
    __builtin_amdgcn_sched_barrier(0);   // the copies are issued before the code words: the wait below counts on it
#pragma unroll
    for (int d = 0; d < kPrefetch; ++d)
#pragma unroll
      for (int j = 0; j < KT4; ++j)
        ring[d][j] = load_stream16(cur_codes + (int64_t)d * Tcap + token_of(cur.start, cur.end, j));
    __builtin_amdgcn_sched_barrier(0);
    wait_vmcnt((kPrefetch - 1) * KT4);   // all but the first word may still be in flight
    __syncthreads();                     // slice 0 is in place
    issue_next_slice();
    rounds_from(0);
    // ---- the tiles after it --------------------------------------------------------------------
    while (more) {
      prev = cur;
      cur = nxt;
      nxt = next_tile();
      more = nxt.end > nxt.start;
      cur_codes = nxt_codes;
      nxt_codes = more ? codes_of(nxt) : cur_codes;
      cur_table = table_of(cur);
      act = cur.start + wave * kFlatUnit < cur.end;
      static_for<kPrefetch>([&](auto s) __attribute__((always_inline)) {
        if constexpr (decltype(s)::value == 0) word(0, s, std::true_type{});
        else word(decltype(s)::value, s, std::false_type{});
      });
      rounds_from(kPrefetch);
    }
    flush(cur);
  }

  // ---- positions past a sequence's cached length ------------------------------------------------
  if (fill_masked) {
    for (int row = blockIdx.x; row < B * Hq; row += gridDim.x) {
      const int len = __builtin_amdgcn_readlane(len_l, row / Hq);
      float* dst = scores + (int64_t)row * score_stride;
      // the scored tiles wrote -inf up to the next multiple of four past the length
      const int from = (len + 3) & ~3;
      for (int t = from + tid * 4; t < T; t += THREADS * 4) {
        if (t + 4 <= T) {
          store_stream16(dst + t, -INFINITY, -INFINITY, -INFINITY, -INFINITY);
        } else {
          for (int i = t; i < T; ++i) dst[i] = -INFINITY;
        }
      }
    }
  }
}

// LDS past the table buffers in every launch: scratch of the key-range reduction
constexpr size_t kScoreScratchBytes = 1024;

struct ScoreArgs {
  const void* q_probs;
  const uint32_t* codes;
  const uint16_t* v_norm;
  const int32_t* lens;
  float* scores;
  int B, Hq, Hkv, L, P, R, T;
  int64_t Tcap, score_stride;
  uint32_t* row_range;
  int range_parts;
  hipStream_t stream;
  int grouped;  // table layout: 0 = [B,Hq,L,R], 1 = [B*Hkv*parts, L, R, group width]
  int flags;    // SOCKET_SCORE_*
};

// How a workgroup's table passes through LDS: buffers, packed words per slice.
// Shared by the launch and by the cost model, so that both see the same slices.
struct SliceLayout {
  int nbuf, chunk_words;
  bool ok;
};

SliceLayout slice_layout(bool dma, size_t bytes_per_word, size_t slots_per_word, int NW, size_t lds_budget) {
  SliceLayout s{2, 1, true};
  if (dma) {
    if (bytes_per_word * NW <= lds_budget) {
      // the whole table at once: one copy, no slices
      s.nbuf = 1;
      s.chunk_words = NW;
    } else {
      // two buffers, as many words per slice as LDS holds (no register staging to fit)
      if (2 * bytes_per_word > lds_budget) s.ok = false;
      while (s.ok && s.chunk_words < NW && 2 * bytes_per_word * (s.chunk_words + 1) <= lds_budget) ++s.chunk_words;
    }
  } else if (2 * bytes_per_word <= lds_budget && slots_per_word <= 1024) {
    // Double-buffered when one word's tables fit twice in LDS and in the staging
    // registers (1024 vector slots per workgroup); as many words per slice as that
    // allows.  Otherwise a single buffer filled in place.
    while (s.chunk_words < NW && 2 * bytes_per_word * (s.chunk_words + 1) <= lds_budget / 2 &&
           slots_per_word * (s.chunk_words + 1) <= 1024)
      ++s.chunk_words;
  } else {
    s.nbuf = 1;
    if (bytes_per_word > lds_budget) s.ok = false;
  }
  return s;
}

template <int GP, class TT, int KT4, int THREADS, int PT, int MODE>
int launch_score_packed(const ScoreArgs& a) {
  typedef typename TT::elem TE;
  const SocketDeviceLimits& lim = socket_device_limits();
  const int G = a.Hq / a.Hkv;
  const int cpw = 32 / a.P;
  const int NW = (a.L + cpw - 1) / cpw;
  constexpr int EPV = 16 / (int)sizeof(TE);
  const size_t bytes_per_word = (size_t)cpw * a.R * GP * sizeof(TE);
  const size_t slots_per_word = (size_t)cpw * a.R / EPV;
  constexpr bool DMA = MODE == 2;
  const size_t lds_budget = (size_t)lim.max_lds_per_block - kScoreScratchBytes;
  // The slice copy needs the table block of a workgroup contiguous: the grouped
  // layout, or any layout when a workgroup serves one head.
  if (DMA && (!(a.grouped || GP == 1) || (a.grouped && GP == 1 && G != 1))) return SOCKET_ERR_UNSUPPORTED;
  const SliceLayout sl = slice_layout(DMA, bytes_per_word, slots_per_word, NW, lds_budget);
  if (!sl.ok) return SOCKET_ERR_UNSUPPORTED;
  const int nbuf = sl.nbuf, chunk_words = sl.chunk_words;
  const size_t table_bytes = bytes_per_word * chunk_words * nbuf;
  const size_t lds_bytes = table_bytes + kScoreScratchBytes;

  auto kern = score_packed_kernel<GP, TT, KT4, THREADS, PT, MODE>;
  if (lds_bytes > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
      return SOCKET_ERR_LAUNCH;
  }
  constexpr int TW = THREADS * 4 * KT4;
  // Tokens per tile: what a workgroup holds -- unless that leaves CUs without a workgroup
  // and cutting every row into as many equal tiles as there are CUs for it keeps more than
  // half of each workgroup's waves in work (a 65536-token context grown by a few hundred
  // tokens: 17 tiles of 4096 per row on 136 of 256 CUs, or 29 of 2304 on 232).  Only where
  // idle lanes cost nothing else: one token group per lane, slices copied global -> LDS.
  int tile_tokens = TW;
  if (KT4 == 1 && DMA && GP > 1 && !a.row_range) {
    const int64_t rows = (int64_t)a.B * a.Hkv * ((G + GP - 1) / GP);
    const int per_row = (int)(lim.cu_count / rows);
    if (rows * ((a.T + TW - 1) / TW) < lim.cu_count && per_row > (a.T + TW - 1) / TW) {
      const int even = (((a.T + per_row - 1) / per_row) + 255) / 256 * 256;
      if (even < TW && 2 * even > TW) tile_tokens = even;
    }
  }
  const int n_tiles = (a.T + tile_tokens - 1) / tile_tokens;
  if (a.row_range && a.range_parts != n_tiles) return SOCKET_ERR_SHAPE;
  const int hsplit = (G + GP - 1) / GP;
  const int n_pairs = a.B * a.Hkv * hsplit;
  const int xcd_remap = ((a.B * a.Hkv) % 8 == 0) ? 1 : 0;
  // whole table resident (one buffer, one slice) and a last tile of at most a
  // quarter of a tile's tokens: folded into the workgroup of the tile before it
  int n_launch_tiles = n_tiles;
  if (GP == 1 && DMA && nbuf == 1 && n_tiles >= 2 && a.T - (n_tiles - 1) * TW <= TW / 4) n_launch_tiles = n_tiles - 1;
  const int n_wg = n_pairs * n_launch_tiles;
  hipLaunchKernelGGL(kern, dim3(n_wg), dim3(THREADS), lds_bytes, a.stream, (const TE*)a.q_probs,
                     a.codes, a.v_norm, a.lens, a.scores, a.Hq, a.Hkv, G, a.L, a.P, a.R, a.T, a.Tcap,
                     a.score_stride, NW, chunk_words, nbuf, n_pairs, n_tiles, n_launch_tiles, xcd_remap,
                     0x3f80u, a.row_range, hsplit, (int)table_bytes, tile_tokens);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

template <int GP, class TT, int KT4, int THREADS, int MODE>
int dispatch_p(const ScoreArgs& a) {
  if (a.P == 10) return launch_score_packed<GP, TT, KT4, THREADS, 10, MODE>(a);
  if (a.P == 8) return launch_score_packed<GP, TT, KT4, THREADS, 8, MODE>(a);
  return launch_score_packed<GP, TT, KT4, THREADS, 0, MODE>(a);
}

template <int GP, class TT, int KT4, int THREADS>
int dispatch_layout(const ScoreArgs& a) {
  return a.grouped ? dispatch_p<GP, TT, KT4, THREADS, 1>(a) : dispatch_p<GP, TT, KT4, THREADS, 0>(a);
}

constexpr int kDmaKT4 = 2;  // token groups of four per lane in the direct-to-LDS variant

// How a scorer launch is shaped.
struct ScorePlan {
  int tile;    // tokens per workgroup
  bool dma;    // table slices copied global -> LDS directly
  bool solo;   // one query head per workgroup, its whole table resident in LDS
  float cost;  // rough time estimate, for comparing plans only
};

// Cost model of a launch shape.  A workgroup's time on its CU is priced from what it
// does, and a round of workgroups from that and from the HBM stream they share:
//
//   t_cu   = a + s * slices + r * (table KB per wave) + c[entry bytes] * lookups
//   t_mem  = workgroups in the round * tokens per tile * HBM bytes per token / kStreamGBs
//   round  = (t_cu^3 + t_mem^3)^(1/3)        (the two overlap, imperfectly)
//   launch = rounds * round
//
//   slices         LDS slices a tile walks (slice_layout: the launch's own arithmetic)
//   table KB/wave  the table block every tile pulls through LDS, shared out over its waves
//   lookups        tokens per tile * tables: the LDS gathers of a workgroup
//   entry bytes    heads per lookup * element size: what one gather returns
//
// with one set of coefficients per kernel variant (they are different kernels:
// direct global -> LDS copies, slices staged through registers from either table
// layout, one head per workgroup with its table resident).  The coefficients are
// a non-negative least-squares fit to 1008 timed launches on one MI355X: every
// variant and tile size forced in turn on 8 table geometries (L60xP10 with 1, 2
// and 4 heads per kv head in bf16 and with 4 in fp32; L48xP10 with 4 and 7; L32xP8
// in bf16 and fp32) times 7 batch / context shapes from B1 x 32768 to B16 x 65536.
// Choosing by the model costs 1% on average and at most 31% over the best
// measured shape of a layout (the hand-written table it replaces: 14% / 125%).
// Its error between variants is larger than within one, so the layout preference
// asks for a margin (kLayoutMargin).
struct VariantCost {
  float a, s, r;      // us; us per slice; us per table KB per wave
  float c[4];         // picoseconds per lookup for entries of 2, 4, 8, 16 bytes
};
constexpr VariantCost kCostDirect = {3.331f, 0.535f, 0.068f, {64.2f, 63.2f, 64.6f, 112.1f}};
constexpr VariantCost kCostStagedRef = {0.536f, 0.0f, 0.102f, {63.4f, 68.8f, 91.1f, 145.1f}};
constexpr VariantCost kCostStagedGrouped = {0.670f, 0.668f, 0.284f, {49.9f, 70.2f, 95.7f, 143.7f}};
constexpr VariantCost kCostSolo = {0.0f, 0.0f, 0.222f, {63.6f, 53.3f, 53.3f, 53.3f}};
constexpr float kStreamGBs = 6000.f;   // what the code stream and the score stores get when every CU pulls
constexpr float kLayoutMargin = 1.3f;  // the grouped layout is preferred unless the other is this much cheaper

int threads_of(int tile, bool dma) {
  if (dma) return tile >= 4096 ? 1024 : tile == 2048 ? 512 : 256;
  return tile == 8192 ? 1024 : tile >= 2048 ? 512 : 256;
}

// Estimated microseconds of a launch of the given shape; < 0 if the shape cannot be launched.
float shape_cost(int B, int Hkv, int G, int T, int grouped, size_t eb, int L, int P, int R, int tile, bool dma,
                 bool solo, int* slices_out = nullptr, int* waves_out = nullptr) {
  const SocketDeviceLimits& lim = socket_device_limits();
  if (P < 1 || P > 16 || L < 1) return -1.f;
  const int cpw = 32 / P, NW = (L + cpw - 1) / cpw;
  const int width = (G == 1 || solo) ? 1 : G == 2 ? 2 : 4;
  const int hsplit = solo ? G : (G + width - 1) / width;
  if (solo && (grouped || G == 1 || !dma)) return -1.f;
  if (dma && !solo && !(grouped || G == 1)) return -1.f;
  const size_t bytes_per_word = (size_t)cpw * R * width * eb;
  const size_t slots_per_word = (size_t)cpw * R / (16 / eb);
  const size_t budget = (size_t)lim.max_lds_per_block - kScoreScratchBytes;
  const SliceLayout sl = slice_layout(dma, bytes_per_word, slots_per_word, NW, budget);
  if (!sl.ok) return -1.f;
  if (solo && sl.nbuf != 1) return -1.f;   // one head per workgroup only with its whole table resident
  const int waves = threads_of(tile, dma) / SOCKET_WAVE;
  const int slices = (NW + sl.chunk_words - 1) / sl.chunk_words;
  if (slices_out) *slices_out = slices;
  if (waves_out) *waves_out = waves;
  const int64_t wgs = (int64_t)B * Hkv * hsplit * ((T + tile - 1) / tile);
  const int64_t rounds = (wgs + lim.cu_count - 1) / lim.cu_count;
  const int64_t active = wgs < lim.cu_count ? wgs : lim.cu_count;
  const VariantCost& v = solo ? kCostSolo : dma ? kCostDirect : grouped ? kCostStagedGrouped : kCostStagedRef;
  const size_t entry = (size_t)width * eb;
  const float c = v.c[entry <= 2 ? 0 : entry <= 4 ? 1 : entry <= 8 ? 2 : 3];
  const float table_kb = (float)((size_t)L * R * width * eb) / 1e3f;
  const float t_cu = v.a + v.s * slices + v.r * table_kb / waves + c * 1e-6f * (float)tile * L;
  // HBM bytes per token of a workgroup: codes + norm (shared through the L2 by the G
  // workgroups of a kv head when each serves one head) + the scores it stores
  const float bpt = (NW * 4.f + 2.f) / (solo ? G : 1) + 4.f * width;
  const float t_mem = (float)active * tile * bpt / (kStreamGBs * 1e3f);
  return (float)rounds * cbrtf(t_cu * t_cu * t_cu + t_mem * t_mem * t_mem);
}

// The cheapest launchable shape for a table in the given layout.
ScorePlan score_plan(int B, int Hkv, int G, int T, int grouped, size_t table_elem_bytes, int L, int P, int R) {
  ScorePlan best{1024, false, false, -1.f};
  for (int tile = 8192; tile >= 1024; tile >>= 1)
    for (int variant = 0; variant < 3; ++variant) {
      const bool dma = variant != 1, solo = variant == 2;
      const float cost = shape_cost(B, Hkv, G, T, grouped, table_elem_bytes, L, P, R, tile, dma, solo);
      if (cost >= 0.f && (best.cost < 0.f || cost < best.cost)) best = {tile, dma, solo, cost};
    }
  return best;
}

// Packed words per LDS slice of the persistent kernel (two buffers, no register staging).
int flat_chunk_words(size_t bytes_per_word, int NW, size_t lds_budget) {
  int cw = 0;
  while (cw < NW && 2 * bytes_per_word * (cw + 1) <= lds_budget) ++cw;
  return cw;
}

// Whether the persistent kernel serves this call: the operands it is written for, and at
// least a sixteenth of an 8192-token tile for every CU, i.e. two waves' worth of tokens per
// workgroup (measured against the tiled launches on 256 CUs, bf16 table of 4 heads x 60
// tables, rows x tokens: 8 x 131072 24.6 against 26.4 us, 16 x 65536 24.5 against 27.5,
// 8 x 65536 17.3 against 20.3, 8 x 32768 16.6 against 18.6, 8 x 16384 15.9 against 18.0;
// 8 x 8192 the same 17.6: there every launch is the ~17 us it takes to pass the table
// through LDS in seven slices, one copy latency and one barrier each).
constexpr int kFlatMinTilesNum = 16;
// (groups_out: token groups per wave the launch should use)
bool flat_serves(const ScoreArgs& a, size_t elem_bytes, int* groups_out = nullptr) {
  const SocketDeviceLimits& lim = socket_device_limits();
  const int G = a.Hq / a.Hkv;
  if (!a.grouped || a.row_range || G < 2 || a.B > 64 || (a.P != 8 && a.P != 10)) return false;
  const int cpw = 32 / a.P, NW = (a.L + cpw - 1) / cpw;
  if (a.L % cpw != 0 || NW % kFlatPrefetch != 0) return false;
  const int width = G == 2 ? 2 : 4, hsplit = (G + width - 1) / width;
  const size_t bytes_per_word = (size_t)cpw * a.R * width * elem_bytes;
  if (flat_chunk_words(bytes_per_word, NW, (size_t)lim.max_lds_per_block - kScoreScratchBytes) < 1) return false;
  const int64_t tiles = (int64_t)a.B * a.Hkv * hsplit * ((a.T + 8191) / 8192);
  if (groups_out) *groups_out = tiles >= lim.cu_count ? 2 : 1;
  return kFlatMinTilesNum * tiles >= lim.cu_count;
}

template <int GP, class TT, int PT, int KT4>
int launch_score_flat(const ScoreArgs& a) {
  typedef typename TT::elem TE;
  const SocketDeviceLimits& lim = socket_device_limits();
  const int G = a.Hq / a.Hkv;
  constexpr int cpw = 32 / PT;
  const int NW = a.L / cpw;
  const size_t bytes_per_word = (size_t)cpw * a.R * GP * sizeof(TE);
  const int chunk_words = flat_chunk_words(bytes_per_word, NW, (size_t)lim.max_lds_per_block - kScoreScratchBytes);
  const size_t lds_bytes = 2 * bytes_per_word * chunk_words;
  auto kern = score_flat_kernel<GP, TT, PT, KT4>;
  if (lds_bytes > 48 * 1024 &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)lds_bytes) != hipSuccess)
    return SOCKET_ERR_LAUNCH;
  const int hsplit = (G + GP - 1) / GP;
  // How the tiles are dealt.  A stretch per workgroup keeps a workgroup on consecutive tiles of
  // one row (measured 3 % faster where it applies: B4 x 8 kv heads x 131072 tokens, 79 against
  // 81.5 us), but every XCD then has all the rows of its eighth of the batch in work at once;
  // when their tables outgrow its L2 (4 MB, which the code stream passes through as well), or
  // the head group is split in parts that should walk the codes together, the tiles are
  // dealt round within each XCD instead (B16 x 4 kv heads x 7 query heads, ragged: 109 against
  // 130 us).
  const int64_t rows_per_xcd = ((int64_t)a.B * a.Hkv + 7) / 8;
  const size_t table_bytes = (size_t)a.L * a.R * GP * sizeof(TE);
  const int spread = (hsplit > 1 || rows_per_xcd * hsplit * table_bytes > (size_t)3 << 20) ? 1 : 0;
  // one workgroup per CU (each needs the CU's LDS to itself)
  hipLaunchKernelGGL(kern, dim3(lim.cu_count), dim3(1024), lds_bytes, a.stream, (const TE*)a.q_probs, a.codes,
                     a.v_norm, a.lens, a.scores, a.B, a.Hq, a.Hkv, G, a.L, a.R, a.T, a.Tcap, a.score_stride, NW,
                     chunk_words, hsplit, 0x3f80u, (a.flags & SOCKET_SCORE_SKIP_MASKED) ? 0 : 1, spread);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

template <int GP, class TT>
int dispatch_flat(const ScoreArgs& a) {
  if constexpr (GP == 1) {
    return SOCKET_ERR_UNSUPPORTED;
  } else {
    int groups = 2;
    flat_serves(a, sizeof(typename TT::elem), &groups);
    if (groups == 2) return a.P == 10 ? launch_score_flat<GP, TT, 10, 2>(a) : launch_score_flat<GP, TT, 8, 2>(a);
    return a.P == 10 ? launch_score_flat<GP, TT, 10, 1>(a) : launch_score_flat<GP, TT, 8, 1>(a);
  }
}

template <int GP, class TT>
int dispatch_tile(const ScoreArgs& a, const ScorePlan& plan) {
  if (plan.dma) {
    if (plan.tile == 8192) return dispatch_p<GP, TT, 2, 1024, 2>(a);
    if (plan.tile == 4096) return dispatch_p<GP, TT, 1, 1024, 2>(a);
    if (plan.tile == 2048) return dispatch_p<GP, TT, 1, 512, 2>(a);
    return dispatch_p<GP, TT, 1, 256, 2>(a);
  }
  if (plan.tile == 8192) return dispatch_layout<GP, TT, 2, 1024>(a);
  if (plan.tile == 4096) return dispatch_layout<GP, TT, 2, 512>(a);
  if (plan.tile == 2048) return dispatch_layout<GP, TT, 1, 512>(a);
  return dispatch_layout<GP, TT, 1, 256>(a);
}

template <class TT>
int dispatch_g(const ScoreArgs& a) {
  const int G = a.Hq / a.Hkv;
  ScorePlan plan = score_plan(a.B, a.Hkv, G, a.T, a.grouped, sizeof(typename TT::elem), a.L, a.P, a.R);
  if (flat_serves(a, sizeof(typename TT::elem))) return G == 2 ? dispatch_flat<2, TT>(a) : dispatch_flat<4, TT>(a);
  if (G == 1 || plan.solo) return dispatch_tile<1, TT>(a, plan);
  if (G == 2) return dispatch_tile<2, TT>(a, plan);
  return dispatch_tile<4, TT>(a, plan);
}

}  // namespace

namespace {
int range_parts_of(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R, int grouped) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || T <= 0 || Hq % Hkv != 0 || L <= 0 || P < 1 || P > 16 || R <= 0) return 0;
  if (q_dtype != SOCKET_F32 && q_dtype != SOCKET_BF16) return 0;
  const ScorePlan plan = score_plan(B, Hkv, Hq / Hkv, T, grouped, q_dtype == SOCKET_F32 ? 4 : 2, L, P, R);
  return (T + plan.tile - 1) / plan.tile;
}
}  // namespace

extern "C" int socket_score_range_parts(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R) {
  return range_parts_of(B, Hq, Hkv, T, q_dtype, L, P, R, 0);
}

extern "C" int socket_score_prefers_grouped(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R) {
  if (range_parts_of(B, Hq, Hkv, T, q_dtype, L, P, R, 0) == 0) return -1;
  const size_t eb = q_dtype == SOCKET_F32 ? 4 : 2;
  const ScorePlan ref = score_plan(B, Hkv, Hq / Hkv, T, 0, eb, L, P, R);
  const ScorePlan grp = score_plan(B, Hkv, Hq / Hkv, T, 1, eb, L, P, R);
  if (grp.cost < 0.f) return 0;
  if (ref.cost < 0.f) return 1;
  return grp.cost <= ref.cost * kLayoutMargin ? 1 : 0;
}

extern "C" int socket_score_plan_query(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R, int grouped,
                                       int* tile, int* direct_copy, int* one_head, float* cost_us) {
  if (range_parts_of(B, Hq, Hkv, T, q_dtype, L, P, R, grouped) == 0) return SOCKET_ERR_SHAPE;
  if (Hq / Hkv > 8) return SOCKET_ERR_UNSUPPORTED;
  const ScorePlan plan = score_plan(B, Hkv, Hq / Hkv, T, grouped, q_dtype == SOCKET_F32 ? 4 : 2, L, P, R);
  if (plan.cost < 0.f) return SOCKET_ERR_UNSUPPORTED;
  if (tile) *tile = plan.tile;
  if (direct_copy) *direct_copy = plan.dma ? 1 : 0;
  if (one_head) *one_head = plan.solo ? 1 : 0;
  if (cost_us) *cost_us = plan.cost;
  return SOCKET_OK;
}

extern "C" int socket_score_shape_cost(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R, int grouped,
                                       int tile, int direct_copy, int one_head, int* slices, int* waves,
                                       float* cost_us) {
  if (range_parts_of(B, Hq, Hkv, T, q_dtype, L, P, R, grouped) == 0) return SOCKET_ERR_SHAPE;
  if (Hq / Hkv > 8 || (tile != 8192 && tile != 4096 && tile != 2048 && tile != 1024)) return SOCKET_ERR_UNSUPPORTED;
  const float cost = shape_cost(B, Hkv, Hq / Hkv, T, grouped, q_dtype == SOCKET_F32 ? 4 : 2, L, P, R, tile,
                                direct_copy != 0, one_head != 0, slices, waves);
  if (cost < 0.f) return SOCKET_ERR_UNSUPPORTED;
  if (cost_us) *cost_us = cost;
  return SOCKET_OK;
}

extern "C" int socket_score_persistent_serves(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R) {
  if (range_parts_of(B, Hq, Hkv, T, q_dtype, L, P, R, 1) == 0) return -1;
  ScoreArgs a{};
  a.B = B; a.Hq = Hq; a.Hkv = Hkv; a.L = L; a.P = P; a.R = R; a.T = T;
  a.grouped = 1;
  return flat_serves(a, q_dtype == SOCKET_F32 ? 4 : 2) ? 1 : 0;
}

extern "C" int socket_score_range_parts_grouped(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R) {
  return range_parts_of(B, Hq, Hkv, T, q_dtype, L, P, R, 1);
}

namespace {

int score_entry(const void* q_probs, int q_dtype, const uint32_t* codes, const uint16_t* v_norm,
                const int32_t* lens, float* scores, uint32_t* row_range, int range_parts, int B, int Hq,
                int Hkv, int L, int P, int R, int T, int64_t Tcap, int64_t score_stride, void* stream,
                int grouped, int flags) {
  SOCKET_REQUIRE(q_probs && codes && v_norm && scores, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(q_dtype == SOCKET_F32 || q_dtype == SOCKET_BF16, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && L > 0 && T > 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(Hq % Hkv == 0, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(P >= 1 && P <= 16, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(R >= (1 << P) && (R & (R - 1)) == 0 && R >= 8, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(T <= Tcap && score_stride >= T, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE((int64_t)B * Hkv * 2 * ((T + 1023) / 1024) < (1LL << 31), SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(Tcap % 4 == 0 && score_stride % 4 == 0, SOCKET_ERR_ALIGN);
  SOCKET_REQUIRE(socket_aligned16(q_probs) && socket_aligned16(codes) && socket_aligned16(v_norm) &&
                     socket_aligned16(scores),
                 SOCKET_ERR_ALIGN);
  SOCKET_REQUIRE(Hq / Hkv <= 8, SOCKET_ERR_UNSUPPORTED);
  const ScoreArgs a{q_probs, codes, v_norm, lens, scores, B, Hq, Hkv, L, P, R, T, Tcap, score_stride,
                    row_range, range_parts, (hipStream_t)stream, grouped, flags};
  return q_dtype == SOCKET_F32 ? dispatch_g<TabF32>(a) : dispatch_g<TabBF16>(a);
}

// [B,Hq,L,R] -> [B*Hkv*parts, L, R, width]: element (pair, part, l, r, g) is head
// kvh*G + part*width + g of the pair, zero where that is past the group.  A thread
// makes one entry (the `width` heads of one bucket): reads coalesced along the
// bucket axis of each head's row, one 4- to 16-byte store.
template <typename TE, int WIDTH>
__global__ __launch_bounds__(256) void group_q_probs_kernel(const TE* __restrict__ in, TE* __restrict__ out,
                                                            int Hq, int Hkv, int G, int parts, int64_t LR) {
  const int blk = blockIdx.y;                 // (pair, part)
  const int part = blk % parts, pair = blk / parts;
  const int b = pair / Hkv, kvh = pair % Hkv;
  const TE* src = in + ((int64_t)b * Hq + kvh * G + part * WIDTH) * LR;
  TE* dst = out + (int64_t)blk * LR * WIDTH;
  const int live = min(WIDTH, G - part * WIDTH);
  for (int64_t lr = (int64_t)blockIdx.x * 256 + threadIdx.x; lr < LR; lr += (int64_t)gridDim.x * 256) {
    TE e[WIDTH];
#pragma unroll
    for (int g = 0; g < WIDTH; ++g) e[g] = g < live ? src[(int64_t)g * LR + lr] : (TE)0;
    typedef TE Entry __attribute__((ext_vector_type(WIDTH)));
    Entry v;
#pragma unroll
    for (int g = 0; g < WIDTH; ++g) v[g] = e[g];
    *reinterpret_cast<Entry*>(dst + lr * WIDTH) = v;
  }
}

template <typename TE>
void launch_group_q_probs(const void* in, void* out, int B, int Hq, int Hkv, int parts, int width, int64_t LR,
                          hipStream_t s) {
  const int bx = (int)((LR + 255) / 256 < 64 ? (LR + 255) / 256 : 64);
  const dim3 grid(bx, B * Hkv * parts);
  const int G = Hq / Hkv;
  if (width == 1)
    hipLaunchKernelGGL((group_q_probs_kernel<TE, 1>), grid, dim3(256), 0, s, (const TE*)in, (TE*)out, Hq, Hkv, G, parts, LR);
  else if (width == 2)
    hipLaunchKernelGGL((group_q_probs_kernel<TE, 2>), grid, dim3(256), 0, s, (const TE*)in, (TE*)out, Hq, Hkv, G, parts, LR);
  else
    hipLaunchKernelGGL((group_q_probs_kernel<TE, 4>), grid, dim3(256), 0, s, (const TE*)in, (TE*)out, Hq, Hkv, G, parts, LR);
}

}  // namespace

extern "C" int socket_score_packed(const void* q_probs, int q_dtype, const uint32_t* codes,
                                   const uint16_t* v_norm, const int32_t* lens, float* scores,
                                   uint32_t* row_range, int range_parts,
                                   int B, int Hq, int Hkv, int L, int P, int R, int T,
                                   int64_t Tcap, int64_t score_stride, int flags, void* stream) {
  return score_entry(q_probs, q_dtype, codes, v_norm, lens, scores, row_range, range_parts, B, Hq, Hkv, L, P,
                     R, T, Tcap, score_stride, stream, 0, flags);
}

extern "C" int socket_score_packed_grouped(const void* q_table, int q_dtype, const uint32_t* codes,
                                           const uint16_t* v_norm, const int32_t* lens, float* scores,
                                           uint32_t* row_range, int range_parts,
                                           int B, int Hq, int Hkv, int L, int P, int R, int T,
                                           int64_t Tcap, int64_t score_stride, int flags, void* stream) {
  return score_entry(q_table, q_dtype, codes, v_norm, lens, scores, row_range, range_parts, B, Hq, Hkv, L, P,
                     R, T, Tcap, score_stride, stream, 1, flags);
}

extern "C" int socket_group_shape(int Hq, int Hkv, int* parts, int* width) {
  SOCKET_REQUIRE(parts && width, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(Hq > 0 && Hkv > 0 && Hq % Hkv == 0, SOCKET_ERR_SHAPE);
  const int G = Hq / Hkv;
  SOCKET_REQUIRE(G <= 8, SOCKET_ERR_UNSUPPORTED);
  *width = G == 1 ? 1 : G == 2 ? 2 : 4;
  *parts = (G + *width - 1) / *width;
  return SOCKET_OK;
}

extern "C" int socket_group_q_probs(const void* q_probs, int q_dtype, void* q_table, int B, int Hq, int Hkv,
                                    int L, int R, void* stream) {
  SOCKET_REQUIRE(q_probs && q_table, SOCKET_ERR_NULL);
  SOCKET_REQUIRE(q_dtype == SOCKET_F32 || q_dtype == SOCKET_BF16, SOCKET_ERR_UNSUPPORTED);
  SOCKET_REQUIRE(B > 0 && L > 0 && R > 0, SOCKET_ERR_SHAPE);
  int parts = 0, width = 0;
  const int st = socket_group_shape(Hq, Hkv, &parts, &width);
  if (st != SOCKET_OK) return st;
  const int64_t LR = (int64_t)L * R;
  SOCKET_REQUIRE((int64_t)B * Hkv * parts <= 65535, SOCKET_ERR_SHAPE);
  SOCKET_REQUIRE(socket_aligned16(q_table), SOCKET_ERR_ALIGN);
  hipStream_t s = (hipStream_t)stream;
  if (q_dtype == SOCKET_F32) launch_group_q_probs<float>(q_probs, q_table, B, Hq, Hkv, parts, width, LR, s);
  else launch_group_q_probs<uint16_t>(q_probs, q_table, B, Hq, Hkv, parts, width, LR, s);
  SOCKET_LAUNCH_CHECK();
  return SOCKET_OK;
}

