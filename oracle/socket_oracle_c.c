/* Plain-C restatement of SOCKET's decode-step arithmetic.  TEST INFRASTRUCTURE
 * ONLY: built into oracle/libsocket_oracle_c.so and called from tests/ as a
 * second, independently written checker next to oracle/socket_oracle.py (the
 * two are compared with each other on the CPU, and the HIP kernels with both).
 * Nothing in the shipped package links or loads it.
 *
 * Scalar loops in the order the reference's device code runs them; citations
 * are paths inside the reference checkout.
 *
 * No function here is pinned by a vector of the reference's own (it ships no
 * tests); each is pinned by tests/test_oracle_pins.py through closed forms and
 * by agreement with the torch restatement.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* GPT-FAST/kernels/soft_hash_collision.cu:25-54: one (b,h,t) per iteration,
 * fp32 sum over l ascending, times v_hist, -inf where not allowed.
 * q_probs [BH,L,R] f32, key_buckets [BH,L,T] i16, allowed [BH,T] u8, v_hist [BH,T] f32. */
void oracle_c_collision_score(const float* q_probs, const int16_t* key_buckets, const uint8_t* allowed,
                              const float* v_hist, float* out, int BH, int L, int R, int T) {
  for (int bh = 0; bh < BH; ++bh) {
    for (int t = 0; t < T; ++t) {
      const long o = (long)bh * T + t;
      if (!allowed[o]) {
        out[o] = -INFINITY;
        continue;
      }
      volatile float sum = 0.0f; /* volatile: keep every add in fp32, no reassociation */
      for (int l = 0; l < L; ++l) {
        const int r = (int)key_buckets[((long)bh * L + l) * T + t];
        sum = sum + q_probs[((long)bh * L + l) * R + r];
      }
      out[o] = sum * v_hist[o];
    }
  }
}

/* Big-endian bit pack (GPT-FAST/model.py:403-407) of sign(k . plane >= 0)
 * (model.py:409-413) with the projection accumulated in double.
 * keys [N,D] f32, planes [L,P,D] f32 -> codes [N,L] i16. */
void oracle_c_hard_hash(const float* keys, const float* planes, int16_t* codes, int N, int D, int L, int P) {
  for (int n = 0; n < N; ++n)
    for (int l = 0; l < L; ++l) {
      int code = 0;
      for (int k = 0; k < P; ++k) {
        double proj = 0.0;
        for (int d = 0; d < D; ++d) proj += (double)keys[(long)n * D + d] * (double)planes[((long)l * P + k) * D + d];
        if (proj >= 0.0) code |= 1 << (P - 1 - k);
      }
      codes[(long)n * L + l] = (int16_t)code;
    }
}

/* Top-m of one row by (score descending, index ascending): selection by
 * repeated scan, O(T*m) -- for small cases only.  NaN ranks above everything,
 * -0.0 == +0.0, as a stable descending sort of floats gives. */
static int beats(float a, int ia, float b, int ib) {
  const int na = isnan(a), nb = isnan(b);
  if (na != nb) return na;
  if (!na && a != b) return a > b;
  return ia < ib;
}
void oracle_c_topk(const float* row, int T, int m, int32_t* out) {
  uint8_t* taken = (uint8_t*)calloc((size_t)T, 1);
  for (int j = 0; j < m; ++j) {
    int best = -1;
    for (int t = 0; t < T; ++t) {
      if (taken[t]) continue;
      if (best < 0 || beats(row[t], t, row[best], best)) best = t;
    }
    taken[best] = 1;
    out[j] = best;
  }
  free(taken);
}

/* Sink + window part of the list (GPT-FAST/kernels/sparse.py:70-84); returns its length. */
int oracle_c_base_indices(int T, int sink, int window, int32_t* out) {
  if (sink > T) sink = T;
  if (sink < 0) sink = 0;
  if (window > T) window = T;
  if (window < 0) window = 0;
  int n = 0;
  for (int i = 0; i < sink; ++i) out[n++] = i;
  if (window > 0) {
    int win_start = T - window > sink ? T - window : sink;
    for (int i = win_start; i < T; ++i) out[n++] = i;
  }
  if (n == 0) out[n++] = T - 1;
  return n;
}

/* One (b,h): softmax(q.K_sel/sqrt(D)).V_sel over list entries >= 0, double
 * accumulation (textbook form of kernels/socket_triton_kernels.py:31-164).
 * k, v are the kv head's rows [S,D] f32. */
void oracle_c_sparse_attend(const float* q, const float* k, const float* v, const int32_t* list, int len,
                            int D, double* out) {
  double mx = -INFINITY;
  double* logit = (double*)malloc(sizeof(double) * (size_t)(len > 0 ? len : 1));
  for (int e = 0; e < len; ++e) {
    if (list[e] < 0) {
      logit[e] = -INFINITY;
      continue;
    }
    double s = 0.0;
    for (int d = 0; d < D; ++d) s += (double)q[d] * (double)k[(long)list[e] * D + d];
    logit[e] = s / sqrt((double)D);
    if (logit[e] > mx) mx = logit[e];
  }
  double den = 0.0;
  for (int d = 0; d < D; ++d) out[d] = 0.0;
  for (int e = 0; e < len; ++e) {
    if (list[e] < 0) continue;
    const double w = exp(logit[e] - mx);
    den += w;
    for (int d = 0; d < D; ++d) out[d] += w * (double)v[(long)list[e] * D + d];
  }
  for (int d = 0; d < D; ++d) out[d] /= den; /* 0/0 = NaN for an empty list, as the reference */
  free(logit);
}
