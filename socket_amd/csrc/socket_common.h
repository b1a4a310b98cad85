// Shared device/host helpers for the SOCKET sparse-decode kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/socket_hip.h"

#define SOCKET_WAVE 64

// Validate a condition on the host before any launch; the entry point returns
// the given status instead of launching a kernel on operands it cannot handle.
#define SOCKET_REQUIRE(cond, status) \
  do {                               \
    if (!(cond)) return (status);    \
  } while (0)

#define SOCKET_LAUNCH_CHECK()                                    \
  do {                                                           \
    hipError_t e__ = hipGetLastError();                          \
    if (e__ != hipSuccess) return SOCKET_ERR_LAUNCH;             \
  } while (0)

static inline int socket_dtype_bytes(int dt) {
  return dt == SOCKET_F32 ? 4 : (dt == SOCKET_BF16 || dt == SOCKET_F16) ? 2 : 0;
}

static inline bool socket_aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }

// ---- element conversions -------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {  // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  _Float16 x;
  __builtin_memcpy(&x, &h, 2);
  return (float)x;
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 x = (_Float16)f;  // v_cvt_f16_f32: round to nearest even
  uint16_t h;
  __builtin_memcpy(&h, &x, 2);
  return h;
}

// Order-preserving map float -> uint32 used by the top-k select: larger float
// <=> larger key.  -0.0 is folded onto +0.0 and every NaN onto the largest key,
// which is how a stable descending sort of floats ranks them.
__device__ __forceinline__ uint32_t score_to_key(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;
  if (u == 0x80000000u) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct DType_f32 {
  typedef float storage;
  static constexpr int kEnum = SOCKET_F32;
  static constexpr int kPer16B = 4;
};
struct DType_bf16 {
  typedef uint16_t storage;
  static constexpr int kEnum = SOCKET_BF16;
  static constexpr int kPer16B = 8;
};
struct DType_f16 {
  typedef uint16_t storage;
  static constexpr int kEnum = SOCKET_F16;
  static constexpr int kPer16B = 8;
};

// Unpack one 16-byte vector of elements into floats.
template <class DT>
__device__ __forceinline__ void unpack16(const uint4& raw, float* out);

template <>
__device__ __forceinline__ void unpack16<DType_f32>(const uint4& raw, float* out) {
  out[0] = __uint_as_float(raw.x);
  out[1] = __uint_as_float(raw.y);
  out[2] = __uint_as_float(raw.z);
  out[3] = __uint_as_float(raw.w);
}
template <>
__device__ __forceinline__ void unpack16<DType_bf16>(const uint4& raw, float* out) {
  out[0] = __uint_as_float(raw.x << 16);
  out[1] = __uint_as_float(raw.x & 0xffff0000u);
  out[2] = __uint_as_float(raw.y << 16);
  out[3] = __uint_as_float(raw.y & 0xffff0000u);
  out[4] = __uint_as_float(raw.z << 16);
  out[5] = __uint_as_float(raw.z & 0xffff0000u);
  out[6] = __uint_as_float(raw.w << 16);
  out[7] = __uint_as_float(raw.w & 0xffff0000u);
}
template <>
__device__ __forceinline__ void unpack16<DType_f16>(const uint4& raw, float* out) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[2 * i] = f16_bits_to_f32((uint16_t)(w[i] & 0xffffu));
    out[2 * i + 1] = f16_bits_to_f32((uint16_t)(w[i] >> 16));
  }
}

template <class DT>
__device__ __forceinline__ void store_elem(void* base, int64_t idx, float v);
template <>
__device__ __forceinline__ void store_elem<DType_f32>(void* base, int64_t idx, float v) {
  ((float*)base)[idx] = v;
}
template <>
__device__ __forceinline__ void store_elem<DType_bf16>(void* base, int64_t idx, float v) {
  ((uint16_t*)base)[idx] = f32_to_bf16_bits(v);
}
template <>
__device__ __forceinline__ void store_elem<DType_f16>(void* base, int64_t idx, float v) {
  ((uint16_t*)base)[idx] = f32_to_f16_bits(v);
}

// (x0 + i x1) * (c + i s) with separately rounded products, as the reference's
// elementwise multiplies, subtraction and addition round (apply_rotary_emb,
// GPT-FAST/model.py:626-639): no contraction into fused multiply-adds here.
__device__ __forceinline__ void rotate_pair(float x0, float x1, float c, float s, float& re, float& im) {
#pragma clang fp contract(off)
  const float a = x0 * c, b = x1 * s, cc = x1 * c, d = x0 * s;
  re = a - b;
  im = cc + d;
}

// v of lane x ^ 16 / x ^ 32, without the LDS crossbar: v_permlane16_swap exchanges
// the odd 16-lane rows of its first operand with the even rows of its second,
// v_permlane32_swap the upper half of the first with the lower half of the second.
__device__ __forceinline__ uint32_t lane_xor16(uint32_t v, bool odd_row) {
  const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  return odd_row ? r[0] : r[1];
}
__device__ __forceinline__ uint32_t lane_xor32(uint32_t v, bool upper_half) {
  const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return upper_half ? r[0] : r[1];
}
__device__ __forceinline__ float lane_xor16(float v) {
  return __uint_as_float(lane_xor16(__float_as_uint(v), (threadIdx.x >> 4) & 1));
}
__device__ __forceinline__ float lane_xor32(float v) {
  return __uint_as_float(lane_xor32(__float_as_uint(v), (threadIdx.x >> 5) & 1));
}

// Step MASK (1, 2, 4 or 8) of a butterfly sum over lanes: the value a lane adds to
// its own.  After the steps below MASK every lane of an aligned group of MASK
// lanes holds the same value, so any lane of the partner group serves, and the
// quad permutes and the half-row and row mirrors of the vector ALU's data-parallel
// primitives deliver one -- without a trip through the LDS crossbar.
template <int MASK>
__device__ __forceinline__ float butterfly_partner(float x) {
  static_assert(MASK == 1 || MASK == 2 || MASK == 4 || MASK == 8, "inside a row of 16 lanes");
  constexpr int ctrl = MASK == 1 ? 0xB1     // quad_perm [1,0,3,2]
                     : MASK == 2 ? 0x4E     // quad_perm [2,3,0,1]
                     : MASK == 4 ? 0x141    // row_half_mirror: lane i <- lane 7 - i of its half row
                                 : 0x140;   // row_mirror: lane i <- lane 15 - i of its row
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), ctrl, 0xf, 0xf, false));
}

// Sum of x over each aligned group of N lanes (N a power of two up to 64), left in
// every lane of the group; the same pairs in the same order as the butterfly
// x += shfl_xor(x, 1), 2, 4, ... so the result is the same bit for bit.
template <int N>
__device__ __forceinline__ float group_sum(float x) {
  if constexpr (N >= 2) x += butterfly_partner<1>(x);
  if constexpr (N >= 4) x += butterfly_partner<2>(x);
  if constexpr (N >= 8) x += butterfly_partner<4>(x);
  if constexpr (N >= 16) x += butterfly_partner<8>(x);
  if constexpr (N >= 32) x += lane_xor16(x);
  if constexpr (N >= 64) x += lane_xor32(x);
  return x;
}

// Inclusive prefix sum over the 64 lanes on the data-parallel-primitive path of the
// vector ALU: four shifts inside each row of 16 lanes, then the last lane of row 0
// (and 2) is added to the row after it and the last lane of the lower half to the
// upper half.  (Six dependent LDS-crossbar shuffles took ~0.25 us per scan.)
__device__ __forceinline__ int wave_incl_scan(int v, int /*lane*/ = 0) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);   // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);   // row_bcast:31 into rows 2 and 3
  return v;
}

// Sum (or maximum) of x over the 64 lanes, left in lane 63: four shifts inside
// each row of 16 lanes, then the last lane of a row is folded into the row after
// it and the lower half's last lane into the upper half; lanes a step does not
// reach take the identity.
template <bool MAX>
__device__ __forceinline__ float wave_reduce_to_last(float x) {
  const int ident = __float_as_int(MAX ? -INFINITY : 0.f);
#define SOCKET_REDUCE_STEP(ctrl, rows)                                                                       \
  {                                                                                                          \
    const float o = __int_as_float(__builtin_amdgcn_update_dpp(ident, __float_as_int(x), ctrl, rows, 0xf, false)); \
    x = MAX ? fmaxf(x, o) : x + o;                                                                           \
  }
  SOCKET_REDUCE_STEP(0x111, 0xf)   // row_shr:1
  SOCKET_REDUCE_STEP(0x112, 0xf)   // row_shr:2
  SOCKET_REDUCE_STEP(0x114, 0xf)   // row_shr:4
  SOCKET_REDUCE_STEP(0x118, 0xf)   // row_shr:8
  SOCKET_REDUCE_STEP(0x142, 0xa)   // row_bcast:15 into rows 1 and 3
  SOCKET_REDUCE_STEP(0x143, 0xc)   // row_bcast:31 into rows 2 and 3
#undef SOCKET_REDUCE_STEP
  return x;
}

// The ticket of a last-arriver hand-over between workgroups of one launch (the splits
// of an attention row, the parts of a selection row): a wrapping increment of the row's
// counter; whoever draws ticket `wrap` is last and finds the counter back at zero.
// The data it hands over is published without a fence, on what gfx950 guarantees for
// the instructions used, not on the HIP memory model (under which relaxed stores, a
// relaxed RMW and relaxed loads are a data race):
//   * the partial results are written with agent-scope atomic stores, which the
//     compiler emits as write-through stores (sc1): they bypass nothing but are
//     forwarded to the memory side of the die-local L2, and vmcnt counts them down only
//     when that write has been acknowledged;
//   * every lane executes s_waitcnt vmcnt(0) and the workgroup barrier before lane 0
//     draws the ticket, so all of the workgroup's stores are acknowledged before its
//     increment is issued; the increment is an agent-scope atomic, performed at the
//     same memory-side point, so increments are ordered after the stores of the
//     workgroups that issued them;
//   * the last arriver reads with agent-scope atomic loads (sc1: they miss the local L2
//     and are served from the memory side), after its own increment has returned.
// A device-scope release fence in that place is correct by the model and costs a
// write-back of the whole L2 (the scorer's 67 MB of scores at 4 x 131072 tokens: the
// step took 315 us with it against 150).  -DSOCKET_STRICT_ATOMICS builds the ticket as an
// acquire-release agent-scope RMW instead, for comparing results and timings; the
// product build does not define it.
__device__ __forceinline__ unsigned int draw_ticket(unsigned int* counter, unsigned int wrap) {
#ifdef SOCKET_STRICT_ATOMICS
  return __builtin_amdgcn_atomic_inc32(counter, wrap, __ATOMIC_ACQ_REL, "agent");
#else
  return atomicInc(counter, wrap);
#endif
}

// 16 bytes per lane from global memory straight into LDS: lane i's bytes land at
// lds_dst + 16 * i (lds_dst is the same for the whole wave).  Written as assembly
// so that the compiler does not serialise later LDS reads behind it; M0, which
// carries the LDS address, is saved and restored.  Completion: vmcnt.
__device__ __forceinline__ void lds_dma16(const void* src_lane, void* lds_dst) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds_dst);
  uint32_t saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(src_lane), "s"(base)
      : "memory");
}
// The same copy with the streaming hint: data that is read once and should not
// displace what the caches hold.
__device__ __forceinline__ void lds_dma16_stream(const void* src_lane, void* lds_dst) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds_dst);
  uint32_t saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off nt\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved)
      : "v"(src_lane), "s"(base)
      : "memory");
}

// s_waitcnt vmcnt(n) only (n <= 15 here; larger requests wait for 15)
__device__ __forceinline__ void wait_vmcnt(int n) {
#define SOCKET_VM(k) \
  case k: __builtin_amdgcn_s_waitcnt((k) | (7 << 4) | (15 << 8)); break;
  switch (n) {
    SOCKET_VM(0) SOCKET_VM(1) SOCKET_VM(2) SOCKET_VM(3) SOCKET_VM(4) SOCKET_VM(5) SOCKET_VM(6) SOCKET_VM(7)
    SOCKET_VM(8) SOCKET_VM(9) SOCKET_VM(10) SOCKET_VM(11) SOCKET_VM(12) SOCKET_VM(13) SOCKET_VM(14)
    default: __builtin_amdgcn_s_waitcnt(15 | (7 << 4) | (15 << 8)); break;
  }
#undef SOCKET_VM
}

// Cached device limits (read once per process; the library keeps no other state).
struct SocketDeviceLimits {
  int cu_count;
  int max_lds_per_block;
};
const SocketDeviceLimits& socket_device_limits();
