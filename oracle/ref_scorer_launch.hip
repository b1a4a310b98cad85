// Builds the REFERENCE's own scorer kernel for gfx950, unmodified, from the file
// where it lies in the reference checkout, plus the launch its doc-comment
// prescribes (GPT-FAST/kernels/soft_hash_collision.cu:7-23: 256 threads,
// grid (ceil(T/256), H, B)).  TEST INFRASTRUCTURE ONLY: the resulting
// oracle/_ref/libref_scorer.so is loaded by tests/ as a checker for the HIP
// scorer at sizes the CPU oracle is too slow for.  The kernel source is
// included by path at build time and never copied into this repository.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#ifndef REF_KERNEL_PATH
#error "define REF_KERNEL_PATH to <reference>/GPT-FAST/kernels/soft_hash_collision.cu"
#endif
#include REF_KERNEL_PATH

extern "C" int ref_soft_hash_collision(const float* q_probs, const int16_t* key_buckets,
                                       const bool* allowed_ext, const float* v_hist, float* out, int B,
                                       int H, int L, int R, int T_k, void* stream) {
  int threads = 256;
  dim3 block(threads, 1, 1);
  dim3 grid((T_k + threads - 1) / threads, H, B);
  hipLaunchKernelGGL(soft_hash_collision_kernel_3, grid, block, 0, (hipStream_t)stream, q_probs,
                     key_buckets, allowed_ext, v_hist, out, B, H, L, R, T_k);
  return (int)hipGetLastError();
}
