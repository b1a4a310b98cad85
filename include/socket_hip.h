/* C ABI of libsocket_hip.so: SOCKET's sparse-decode hot path on MI355X (gfx950).
 *
 * Every entry point takes raw device pointers, explicit sizes and element
 * strides, and a HIP stream handle passed as void* (hipStream_t; NULL = the
 * default stream).  Outputs and workspaces are allocated by the caller; the
 * library allocates nothing, keeps no state besides cached device limits, and
 * is re-entrant.  Kernels are enqueued on `stream` and the call returns without
 * synchronising.  The return value is a status: 0 on success, a negative
 * SOCKET_ERR_* otherwise; on error nothing was launched.
 *
 * Citations name the reference interface each entry point replaces, as
 * path:line inside the SOCKET checkout.
 *
 * Shapes use B batch, Hq query heads, Hkv key/value heads, G = Hq / Hkv,
 * D head dim, T context length, Tcap cache capacity (row pitch of the hash
 * cache), L hash tables, P hyperplanes per table (code < 2^P), R entries per
 * soft-hash table (R >= 2^P), M top-k budget.
 *
 * Packed code format (this library's own; the reference keeps int16 codes
 * [B,Hkv,T,L]): c = 32 / P codes per 32-bit word, NW = ceil(L / c) words per
 * key; table l lives in word l / c at bit offset (l % c) * P; unused high bits
 * are zero.  Words are stored table-major per KV head: uint32 [B,Hkv,NW,Tcap],
 * so consecutive tokens of one word index are consecutive in memory.
 */
#ifndef SOCKET_HIP_H_
#define SOCKET_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SOCKET_ABI_VERSION 4   /* 4: the packed scorers take a flags word */

/* status codes */
#define SOCKET_OK 0
#define SOCKET_ERR_NULL (-1)        /* a required pointer is NULL */
#define SOCKET_ERR_SHAPE (-2)       /* sizes inconsistent or out of range */
#define SOCKET_ERR_UNSUPPORTED (-3) /* dtype / head dim / table size not built */
#define SOCKET_ERR_ALIGN (-4)       /* pointer or pitch not aligned as required */
#define SOCKET_ERR_WORKSPACE (-5)   /* workspace smaller than *_workspace_bytes */
#define SOCKET_ERR_LAUNCH (-6)      /* hipGetLastError() after the launch */

/* element types of q / k / v / out */
#define SOCKET_F32 0
#define SOCKET_BF16 1
#define SOCKET_F16 2

int socket_abi_version(void);
const char* socket_status_string(int status);
/* Compute-unit count and LDS bytes per workgroup of the current device. */
int socket_device_query(int* cu_count, int* max_lds_bytes);

/* ------------------------------------------------------------------------
 * K1  key hashing (+ fused value norm)
 * ---------------------------------------------------------------------- */

/* NW for (L, P); 0 if P is outside [1,16] or L < 1. */
int socket_words_per_key(int L, int P);

/* planes [L,P,D] (SOCKET_F32/BF16/F16) -> bf16 [NW*32, D]: row w*32+p is the
 * hyperplane whose sign becomes bit p of packed word w, zero rows for unused
 * bits.  Done once per layer.  Replaces the weights tensor of pack_bits,
 * GPT-FAST/model.py:403-407, by ordering the contraction's columns. */
int socket_permute_planes(const void* planes, int planes_dtype, int L, int P, int D,
                          void* planes_words, void* stream);

/* Hash S new keys per (b, kv head) and store their packed codes and value
 * norms at cache positions pos0(b)+s, s in [0,S): pos0(b) = pos_b ? pos_b[b] : t0.
 * t0 + S > Tcap is an error; with pos_b (int32 on the device, not visible to the
 * host) rows whose position falls outside [0, Tcap) are dropped.
 * k, v address element [0,0,0,0] of the new rows with the given element strides
 * (last dim contiguous); v may be NULL (then v_norm is not written).
 * bit = (k . plane >= 0) from an MFMA bf16 contraction with fp32 accumulation.
 * Replaces Attention.hard_hash_keys + pack_bits, GPT-FAST/model.py:403-413, the
 * value norm at GPT-FAST/model.py:450 and the k_hard / v_norm writes of
 * KVCache.update, GPT-FAST/model.py:222-226.
 * Requires D == 128, 16-byte aligned rows. */
int socket_hash_keys(const void* k, const void* v, int dtype,
                     int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                     int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s,
                     const void* planes_words, uint32_t* codes, uint16_t* v_norm,
                     const int32_t* pos_b, int t0,
                     int B, int Hkv, int S, int D, int L, int P, int64_t Tcap,
                     void* stream);

/* Packed words -> int16 codes with arbitrary output strides (elements) over
 * (b, h, l, t) for tokens [t0, t0+T).  out[b,h,l,t-t0].  Gives the reference's
 * k_hard layouts: [B,S,Hkv,L] (GPT-FAST/model.py:413) or [B,H,L,T]
 * (pipeline/train_quest/modeling/modeling_llama.py:615). */
int socket_unpack_codes(const uint32_t* codes, int16_t* out, int B, int Hkv, int L, int P,
                        int t0, int T, int64_t Tcap,
                        int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_l,
                        int64_t out_stride_t, void* stream);

/* int16 codes with arbitrary strides over (b, h, l, t) -> packed words at
 * positions [t0, t0+T) of the cache. */
int socket_pack_codes(const int16_t* in, int64_t in_stride_b, int64_t in_stride_h,
                      int64_t in_stride_l, int64_t in_stride_t,
                      uint32_t* codes, int B, int Hkv, int L, int P, int t0, int T,
                      int64_t Tcap, void* stream);

/* ------------------------------------------------------------------------
 * K2  soft-collision scorer
 * ---------------------------------------------------------------------- */

#define SOCKET_SCORE_SKIP_MASKED 1   /* flags bit of the packed scorers, see below */

/* Native scorer on the packed cache.  For every b, kv head, token t < T and
 * each of the G query heads h of that kv head:
 *   scores[b,h,t] = t < len(b) ? (sum_{l<L} q_probs[b,h,l,code_l(b,kv,t)]) * v_norm[b,kv,t] : -inf
 * with the sum taken over l ascending in fp32 (the order of the loop at
 * GPT-FAST/kernels/soft_hash_collision.cu:45-53), len(b) = lens ? lens[b] : T.
 * q_probs: [B,Hq,L,R] contiguous, q_dtype SOCKET_F32 or SOCKET_BF16 (bf16 values are
 * widened exactly, as the reference's q_probs.float() does).
 * scores: fp32, row (b,h) at scores + (b*Hq+h)*score_stride.
 * Codes are read once per kv head, not once per query head.
 * Replaces the relayout at GPT-FAST/model.py:490-509 and the scorer call at
 * GPT-FAST/kernels/sparse.py:42-55.
 * Requires Tcap % 4 == 0, score_stride % 4 == 0, 16-byte aligned pointers,
 * R a power of two >= 8, 2^P <= R, G <= 8, and the tables of one packed word
 * (32/P tables x R entries x G values) must fit in LDS.
 * flags: 0, or SOCKET_SCORE_SKIP_MASKED -- scores[b,h,t] for t >= len(b) may be left
 * unwritten (a caller that reads rows only up to len(b), as socket_select_list does
 * with the same lens, saves the write: 73 MB of -inf on a ragged batch of 16 x 28
 * rows of 98304).  Positions below len(b) are not affected.
 *
 * row_range (optional, may be NULL): uint32 [B*Hq, range_parts, 2]; for every row
 * and token tile the minimum and maximum order-preserving key of the tile's
 * scores at t < len(b) (0xffffffff / 0 for a tile without such a token).
 * range_parts must equal socket_score_range_parts(...) of the same call (the
 * tile size follows from the shape; 0 = invalid shape).  Passing the array on to
 * socket_select_list saves that kernel a pass over the scores for the rows it has
 * to select without its sampled threshold.
 *
 * With few (b, kv head) pairs and a context too short to give every CU a tile,
 * and a table of one head (L*R elements) that fits LDS, a workgroup serves one
 * query head with its whole table resident instead of a head group with table
 * slices; results are the same. */
int socket_score_range_parts(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R);
int socket_score_packed(const void* q_probs, int q_dtype, const uint32_t* codes,
                        const uint16_t* v_norm, const int32_t* lens, float* scores,
                        uint32_t* row_range, int range_parts,
                        int B, int Hq, int Hkv, int L, int P, int R, int T, int64_t Tcap,
                        int64_t score_stride, int flags, void* stream);

/* Grouped table layout.  The scorer gathers from an LDS image of the table in which
 * the query heads that share a KV head are interleaved: [table][bucket][head].
 * A table already stored that way is copied into LDS as it is:
 *   q_table [B*Hkv*parts, L, R, width]  (same element type as q_probs)
 *   element (b*Hkv + kvh, part, l, r, g) = q_probs[b, kvh*G + part*width + g, l, r],
 *   zero where part*width + g >= G;  socket_group_shape gives width (1, 2 or 4)
 *   and parts (2 for G = 5..8, else 1).
 * socket_group_q_probs converts a [B,Hq,L,R] table; socket_soft_hash_grouped
 * produces the layout directly.  socket_score_packed_grouped is socket_score_packed
 * on such a table: same arguments, same results, except that its row_range has
 * socket_score_range_parts_grouped(...) parts (its tiles can be of another size),
 * and bf16 scores may differ in the last place (within the bound above).
 * socket_score_prefers_grouped: which layout a producer should write for this
 * shape (T = the context length the scorer will be called with): 1 = grouped,
 * 0 = [B,Hq,L,R] (the shapes the scorer serves one head per workgroup, see
 * socket_score_packed), -1 = invalid shape.  Either layout is always accepted.
 * socket_score_plan_query: the launch shape the scorer would use for a table in the
 * given layout (tokens per workgroup; whether table slices are copied global ->
 * LDS directly; whether a workgroup serves one head with its table resident) and
 * the cost model's estimate of the launch in microseconds.  The model prices a
 * shape from table bytes per workgroup, LDS slices, lookups per tile, entry width
 * and workgroups against compute units; it ranks shapes, it is not a timing promise. */
int socket_score_plan_query(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R, int grouped,
                            int* tile, int* direct_copy, int* one_head, float* cost_us);
/* The same estimate for one given shape (tile 8192, 4096, 2048 or 1024), with the
 * LDS slices per workgroup and the waves per workgroup it was priced on;
 * SOCKET_ERR_UNSUPPORTED if that shape cannot be launched for this table.
 * socket_score_plan_query returns the cheapest of these. */
int socket_score_shape_cost(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R, int grouped,
                            int tile, int direct_copy, int one_head, int* slices, int* waves, float* cost_us);
int socket_group_shape(int Hq, int Hkv, int* parts, int* width);
int socket_score_prefers_grouped(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R);
int socket_score_range_parts_grouped(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R);
/* socket_score_persistent_serves: 1 if socket_score_packed_grouped would serve a call
 * of this shape (without row_range) with its persistent launch -- one workgroup per
 * CU, the token range of every (sequence, kv head, head part) dealt out by the cached
 * lengths, no drain between tiles -- 0 if with the tiled launches, -1 for an invalid
 * shape.  A caller that holds the table as [B,Hq,L,R] can use it to decide whether
 * converting it with socket_group_q_probs first pays (socket_score_packed itself
 * never takes the persistent launch: its table slices need an interleaving pass). */
int socket_score_persistent_serves(int B, int Hq, int Hkv, int T, int q_dtype, int L, int P, int R);
int socket_group_q_probs(const void* q_probs, int q_dtype, void* q_table, int B, int Hq, int Hkv,
                         int L, int R, void* stream);
int socket_score_packed_grouped(const void* q_table, int q_dtype, const uint32_t* codes,
                                const uint16_t* v_norm, const int32_t* lens, float* scores,
                                uint32_t* row_range, int range_parts,
                                int B, int Hq, int Hkv, int L, int P, int R, int T, int64_t Tcap,
                                int64_t score_stride, int flags, void* stream);

/* The reference extension's entry point on its own layout:
 * q_probs f32 [B,H,1,L,R], key_buckets i16 [B,H,L,T], allowed bool [B,H,1,T],
 * v_hist f32 [B,H,1,T] -> out f32 [B,H,1,T], all contiguous.
 * Replaces ext.soft_hash_collision, GPT-FAST/kernels/soft_hash_collision_loader.py:14-74
 * (kernel GPT-FAST/kernels/soft_hash_collision.cu:25-54). */
int socket_soft_hash_collision(const float* q_probs, const int16_t* key_buckets,
                               const uint8_t* allowed, const float* v_hist, float* out,
                               int B, int H, int L, int R, int T, void* stream);

/* fp16 variant: q_probs f16 [B,H,L,R], v_norm f16 [B,H,T], any L.
 * Replaces soft_hash_score, GPT-FAST/kernels/soft_hash_score/soft_hash_score_bindings.cpp:10-36
 * (kernel GPT-FAST/kernels/soft_hash_score/soft_hash_score.cu:7-42). */
int socket_soft_hash_score_f16(const uint16_t* q_probs, const int16_t* key_buckets,
                               const uint16_t* v_norm, const uint8_t* allowed, float* out,
                               int B, int H, int L, int R, int T, void* stream);

/* Query soft hash: bucket probabilities of every query head for every table,
 *   probs[b,h,l,:] = softmax_r( inv_temperature * sum_k tanh(q[b,h,:] . planes[l,k,:]) * tanh_scale
 *                                                 * protos_T[k,r] )
 * with tanh_scale = 1 / max(sqrt(D), 1e-6) in both callers and inv_temperature = 1
 * (GPT-FAST/model.py:392-401) or 1 / 0.3
 * (pipeline/train_quest/modeling/modeling_llama.py:618-638).
 * q [B,Hq,D] (element strides, unit-stride last dim), planes [L,K,D] and protos_T
 * [K,R] contiguous, all of `dtype`; out [B,Hq,L,R] contiguous, out_dtype
 * SOCKET_F32 or SOCKET_BF16, 16-byte aligned.  Computed in fp32 and rounded once.
 * Requires D <= 256, K <= 16, Hq / Hkv <= 8, R % 4 == 0, B * Hkv <= 65535.
 * Hkv only groups the heads that share a workgroup; any divisor of Hq with
 * Hq / Hkv <= 8 gives the same result. */
int socket_soft_hash(const void* q, int dtype, int64_t q_stride_b, int64_t q_stride_h,
                     const void* planes, const void* protos_T, void* out, int out_dtype,
                     int B, int Hq, int Hkv, int D, int L, int K, int R,
                     float tanh_scale, float inv_temperature, void* stream);
/* The same, written in the grouped table layout described at
 * socket_score_packed_grouped (Hkv must then be the real number of KV heads). */
int socket_soft_hash_grouped(const void* q, int dtype, int64_t q_stride_b, int64_t q_stride_h,
                             const void* planes, const void* protos_T, void* q_table, int out_dtype,
                             int B, int Hq, int Hkv, int D, int L, int K, int R,
                             float tanh_scale, float inv_temperature, void* stream);

/* ------------------------------------------------------------------------
 * K3  top-k select and index list
 * ---------------------------------------------------------------------- */

/* Per row (b,h) of fp32 scores: the m = min(budget(b), len(b)) largest entries
 * of scores[0:len(b)] in descending score order, equal scores by ascending
 * index, written as int32 after the sink/window part so that the row of
 * sparse_list is [sink | window | heavy | -1 padding up to list_width]:
 *   sink   = 0 .. min(sink,len)-1
 *   window = max(len - min(window,len), min(sink,len)) .. len-1
 *   (both empty -> the single index len-1)
 * and sparse_len[b,h] = entries before the padding.  len(b) = lens ? lens[b] : T,
 * budget(b) = budgets ? budgets[b] : M.  With write_base == 0 only the heavy
 * part is written, starting at column 0.
 * Replaces torch.topk + the list assembly of build_sparse_list_decode,
 * GPT-FAST/kernels/sparse.py:57-95.  NaN scores rank above +inf, -0.0 equals +0.0.
 * row_range / range_parts: the key ranges written by socket_score_packed for
 * these scores, or NULL / 0 (then the kernel finds a row's range itself when it
 * needs it).
 * workspace: optional scratch of socket_select_workspace_bytes(B, Hq, T, M) bytes
 * (0 where it would not help: short rows, or as many rows as the GPU has CUs).
 * With it, a few long rows are each shared between several workgroups that
 * exchange their candidates through it, in the same launch; without it (NULL) one
 * workgroup handles a whole row.  Same result.  Its first
 * socket_select_workspace_zero_bytes(B, Hq, T, M) bytes are arrival counters that
 * must be zero when the call starts and are zero again when it has finished: zero
 * them once, then the workspace can serve every later call of the same shape
 * issued in order on one stream (calls that overlap on one workspace race).
 * Requires M <= SOCKET_TOPK_MAX_M, B*Hq <= 65535. */
#define SOCKET_TOPK_MAX_M 16384
size_t socket_select_workspace_bytes(int B, int Hq, int T, int M);
size_t socket_select_workspace_zero_bytes(int B, int Hq, int T, int M);
int socket_select_list(const float* scores, int64_t score_stride, const int32_t* lens,
                       const int32_t* budgets, const uint32_t* row_range, int range_parts,
                       int B, int Hq, int T, int M, int sink, int window, int write_base,
                       int32_t* sparse_list, int64_t list_stride, int list_width,
                       int32_t* sparse_len, void* workspace, size_t workspace_bytes,
                       void* stream);

/* ------------------------------------------------------------------------
 * K4  sparse flash-decode
 * ---------------------------------------------------------------------- */

/* Stage 1: for split s of query head (b,h), attend over list entries
 * [s*block_seq, min(len, (s+1)*block_seq)) of the kv head h / G; entries < 0
 * are skipped.  Writes mid_o[b,h,s,:] = acc / sum_exp (fp32 [B,Hq,nsplit,D]) and
 * mid_lse[b,h,s] = max + log(sum_exp) (fp32 [B,Hq,nsplit]); a split with no
 * live row gets mid_lse = -inf, mid_o = 0; splits at or beyond len are left
 * untouched.  Strides are in elements; the last dim of q, k, v is contiguous.
 * list_width: entries in a row of sparse_list; a length beyond it is cut to it.
 * Replaces sparse_decode_stage1, kernels/socket_triton_kernels.py:167-205
 * (kernel :31-118).  D in {16,32,64,128}; q,k,v of one dtype. */
int socket_attend_stage1(const void* q, const void* k, const void* v, int dtype,
                         int64_t q_stride_b, int64_t q_stride_h,
                         int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                         int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s,
                         const int32_t* sparse_list, int64_t list_stride_b, int64_t list_stride_h,
                         const int32_t* sparse_len, int64_t len_stride_b, int64_t len_stride_h,
                         float* mid_o, float* mid_lse,
                         int B, int Hq, int Hkv, int D, int kv_rows, int list_width, int nsplit,
                         int block_seq, void* stream);

/* Stage 2: merge the ceil(len / block_seq) splits of every (b,h) into
 * out[b,h,:] (out_dtype); len == 0 gives NaN like the reference's 0/0.
 * mid_o must be 16-byte aligned.
 * Replaces sparse_decode_stage2, kernels/socket_triton_kernels.py:208-235
 * (kernel :121-164). */
int socket_attend_stage2(const float* mid_o, const float* mid_lse,
                         const int32_t* sparse_len, int64_t len_stride_b, int64_t len_stride_h,
                         void* out, int out_dtype, int64_t out_stride_b, int64_t out_stride_h,
                         int B, int Hq, int D, int nsplit, int block_seq, void* stream);

/* Split size (list entries per workgroup) socket_sparse_attention uses for a
 * list of width max_len, and its workspace need. */
int socket_sparse_attention_block_seq(int B, int Hq, int max_len);
size_t socket_sparse_attention_workspace_bytes(int B, int Hq, int D, int max_len);

/* Stage 1 + stage 2 with the split size chosen by the library; max_len is the
 * width of sparse_list (an upper bound of every sparse_len, so no device->host
 * read of the lengths is needed).
 * Replaces sparse_attention_fwd, kernels/socket_triton_kernels.py:238-258. */
int socket_sparse_attention(const void* q, const void* k, const void* v, int dtype,
                            int64_t q_stride_b, int64_t q_stride_h,
                            int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                            int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s,
                            const int32_t* sparse_list, int64_t list_stride_b, int64_t list_stride_h,
                            const int32_t* sparse_len, int64_t len_stride_b, int64_t len_stride_h,
                            void* out, int64_t out_stride_b, int64_t out_stride_h,
                            void* workspace, size_t workspace_bytes,
                            int B, int Hq, int Hkv, int D, int kv_rows, int max_len, void* stream);

/* socket_sparse_attention without a workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The per-split partials go to a fixed array of SOCKET_STATIC_SCRATCH_BYTES in
 * device memory that belongs to the library's image, next to 65536 row counters
 * (each GPU the library runs on holds one copy until the process ends); a call
 * whose socket_sparse_attention_workspace_bytes(B, Hq, D, max_len) exceeds that
 * size, or with more than 65536 (b, h) rows, returns SOCKET_ERR_WORKSPACE and
 * launches nothing.  The call allocates and frees nothing, and it is ONE launch:
 * the workgroup that completes a row's last split merges the row's splits (the
 * counters are zero between calls: tickets are drawn with a wrapping increment).
 * All calls on one GPU share the arrays: calls that overlap in time on the same
 * GPU (different streams or threads) race; serialise them.
 * Same results as socket_sparse_attention, bit for bit.
 * socket_static_scratch_init looks the arrays' device addresses up for the current
 * device ahead of the first call (optional; the first call does it otherwise). */
#define SOCKET_STATIC_SCRATCH_BYTES (4u << 20)
size_t socket_static_scratch_bytes(void);
int socket_static_scratch_init(void);
int socket_sparse_attention_static(const void* q, const void* k, const void* v, int dtype,
                                   int64_t q_stride_b, int64_t q_stride_h,
                                   int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                                   int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s,
                                   const int32_t* sparse_list, int64_t list_stride_b, int64_t list_stride_h,
                                   const int32_t* sparse_len, int64_t len_stride_b, int64_t len_stride_h,
                                   void* out, int64_t out_stride_b, int64_t out_stride_h,
                                   int B, int Hq, int Hkv, int D, int kv_rows, int max_len, void* stream);

/* Dense split-K flash-decode over rows [0, len(b)) of the cache (the
 * comparator the sparse path is timed against; the reference's dense decode is
 * Attention.forward, GPT-FAST/model.py:562-589).  K/V rows are read once per kv
 * head and shared by its G = Hq / Hkv query heads.  bf16 / fp16 caches with D = 128
 * run on the matrix cores (G <= 16; probabilities are rounded to the cache's type
 * before the value product, as flash attention kernels do); other head dims and
 * fp32 caches on the vector ALU (G <= 8).  SOCKET_ERR_UNSUPPORTED beyond that. */
size_t socket_dense_decode_workspace_bytes(int B, int Hq, int D, int T);
int socket_dense_decode(const void* q, const void* k, const void* v, int dtype,
                        int64_t q_stride_b, int64_t q_stride_h,
                        int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_s,
                        int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_s,
                        const int32_t* lens, void* out, int64_t out_stride_b, int64_t out_stride_h,
                        void* workspace, size_t workspace_bytes,
                        int B, int Hq, int Hkv, int D, int T, void* stream);

/* ------------------------------------------------------------------------
 * Decode-step helpers around the attention hook
 * ---------------------------------------------------------------------- */

/* Rotary embedding of the new token's q and k and the append of k / v to the
 * cache, from the fused projection qkv [B, (Hq + 2*Hkv) * D] (row stride
 * qkv_stride_b): q_out [B,Hq,D] contiguous; rotated k and v are written at
 * row pos of k_cache / v_cache (element strides b, h, s; unit-stride last dim),
 * and lens[b] (may be NULL) is set to pos + 1 (the cached length follows the
 * position, as the reference's mask arange(T) <= pos does, GPT-FAST/model.py:486-487).  pos: int64 on the device,
 * one for all sequences (pos_stride 0) or one each (pos_stride 1); a position
 * outside [0, min(Tcap, n_pos)) writes nothing.  freqs_cis [n_pos, D/2, 2] holds
 * (cos, sin) in bf16 or f32.  k_new / v_new (may be NULL): [B,Hkv,D] contiguous
 * copies of the rotated key and the value, for the hashing kernel.  Pairs (2i, 2i+1) are rotated in fp32 with separately
 * rounded products, then rounded to `dtype`.
 * Replaces apply_rotary_emb on q and k (GPT-FAST/model.py:443-444, :626-639) and the
 * K/V writes and length update of KVCache.update (:215-217, :228) for one token. */
int socket_rope_append(const void* qkv, int dtype, int64_t qkv_stride_b, const void* freqs_cis,
                       int freqs_dtype, int64_t n_pos, const int64_t* pos, int pos_stride, void* q_out,
                       void* k_cache, void* v_cache, int64_t cache_stride_b, int64_t cache_stride_h,
                       int64_t cache_stride_s, int32_t* lens, void* k_new, void* v_new, int B, int Hq, int Hkv,
                       int D, int64_t Tcap, void* stream);

/* The head of a single-token decode step in ONE launch: what socket_rope_append,
 * socket_hash_keys on the new key and socket_soft_hash (out_dtype / grouped as
 * socket_soft_hash_grouped when grouped != 0) do in three, with the same results bit
 * for bit -- rotary embedding of the new token's q and k from the fused projection
 * qkv [B, (Hq + 2*Hkv) * D], K/V rows written at pos, lens[b] = pos + 1, packed
 * codes and value norm of the new key written at pos (planes_words as for
 * socket_hash_keys, P = K), q_out [B,Hq,D], and the rotated queries' bucket
 * probabilities in q_table ([B,Hq,L,R], or the grouped layout).  Arguments as in
 * those three entry points.  Written for dtype = SOCKET_BF16, D = 128, K = 10,
 * R <= 1024, Hq / Hkv <= 8, 16-byte aligned operands and strides that are
 * multiples of 8 elements: anything else returns SOCKET_ERR_UNSUPPORTED /
 * SOCKET_ERR_ALIGN and the caller uses the three entry points.
 * Replaces GPT-FAST/model.py:433-451 (rotary, KVCache.update, hard_hash_keys of
 * the new key, value norm) and :392-401 (soft_hash) for one new token. */
int socket_decode_prologue(const void* qkv, int dtype, int64_t qkv_stride_b, const void* freqs_cis,
                           int freqs_dtype, int64_t n_pos, const int64_t* pos, int pos_stride, void* q_out,
                           void* k_cache, void* v_cache, int64_t cache_stride_b, int64_t cache_stride_h,
                           int64_t cache_stride_s, int32_t* lens, const void* planes_words, void* codes,
                           void* v_norm, const void* planes, const void* protos_T, void* q_table, int out_dtype,
                           int grouped, int B, int Hq, int Hkv, int D, int L, int K, int R, int64_t Tcap,
                           float tanh_scale, float inv_temperature, void* stream);

/* h = x + residual (residual may be NULL: h = x), rounded to `dtype`;
 * y = round(h * rsqrt(mean(h^2) + eps)) * weight.  x, residual, h_out (may be
 * NULL), y_out: [rows, dim] contiguous; weight [dim].
 * Replaces RMSNorm.forward (GPT-FAST/model.py:603-614) and the residual add in front
 * of it (TransformerBlock, :340-342). */
int socket_add_rmsnorm(const void* x, const void* residual, const void* weight, void* h_out, void* y_out,
                       int dtype, int64_t rows, int dim, float eps, void* stream);

/* out = round(silu(a)) * b elementwise over n elements (FeedForward, GPT-FAST/model.py:599-600). */
int socket_silu_mul(const void* a, const void* b, void* out, int dtype, int64_t n, void* stream);

/* y[m,n] = sum_k x[m,k] * w[n,k]: the linear layers of a single-token step as matrix-vector
 * products (M <= 4 rows, bf16, fp32 accumulation; K a multiple of 2048; x rows `x_stride`
 * elements apart, y rows `y_stride`; w [N,K] contiguous).  With w_gate (another [N,K]):
 * y = round(silu(round(x.w[n]))) * round(x.w_gate[n]), i.e. w1, w3 and the product of
 * FeedForward in one pass.  Replaces the nn.Linear calls of a decode step
 * (GPT-FAST/model.py:436, :476, :599-600); SOCKET_ERR_UNSUPPORTED tells the caller to use its
 * own matrix product. */
int socket_gemv_bf16(const void* x, int64_t x_stride, const void* w, const void* w_gate, void* y,
                     int64_t y_stride, int M, int N, int K, void* stream);

/* socket_add_rmsnorm followed by socket_gemv_bf16 on its output, as one launch: every
 * workgroup works out h = x + residual and RMSNorm(h) * norm_weight for itself (the same
 * arithmetic in the same order: results equal the two launches bit for bit) and multiplies
 * from there.  x, residual, h_out [M,K] and y [M,N] contiguous bf16, K <= 8192; residual and
 * h_out are given together or not at all (without them h is x), and h_out must not overlap
 * x or residual (other workgroups are still reading them when it is written).  Replaces
 * RMSNorm + nn.Linear of a decode step (GPT-FAST/model.py:603-614 with :436 and :599-600). */
int socket_norm_gemv_bf16(const void* x, const void* residual, const void* norm_weight, float eps,
                          void* h_out, const void* w, const void* w_gate, void* y, int M, int N, int K,
                          void* stream);

/* Block-sparse prefill attention: out[b,h,row,:] = softmax over the listed key
 * blocks (causal inside them) of q.k^T / sqrt(D), times v.  q, k, v, out are
 * [B,H,T,D] views (element strides for dims 0-2, last dim contiguous), bf16 or
 * fp16; seqlens int32 [B] (rows and keys at or past seqlens[b] do not take part,
 * such rows of `out` are left untouched); block_index int32 [B,H,num_rows,klist],
 * contiguous, every entry a key-block id in [0, ceil(T/64)) (entries outside are
 * clamped into it); a block listed twice is attended twice.  num_rows must equal
 * ceil(T/64); block_m and block_n must both be 64 (the reference's defaults).
 * Replaces random_walk_fwd and its launcher random_walk_sparse_attention,
 * kernels/block_sparse_flash_attention.py:280-437 (which pads T to whole blocks
 * with zero rows instead of bounding the loads).  A row with no visible key in any
 * listed block gives zeros here (the reference's exp2(-inf - -inf) gives NaN). */
int socket_block_sparse_attention(const void* q, const void* k, const void* v, int dtype,
                                  int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_m,
                                  int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_n,
                                  int64_t v_stride_b, int64_t v_stride_h, int64_t v_stride_n,
                                  const int32_t* seqlens, const int32_t* block_index, void* out,
                                  int64_t o_stride_b, int64_t o_stride_h, int64_t o_stride_m,
                                  int B, int H, int T, int D, int num_rows, int klist,
                                  int block_m, int block_n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SOCKET_HIP_H_ */
