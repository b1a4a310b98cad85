"""CPU restatement of SOCKET's sparse-decode path.  TEST INFRASTRUCTURE ONLY.

This module is the checker that the HIP kernels are compared against.  It is
imported by the test-suite, by the smoke check and by the CPU-baseline leg of
the benchmark, and by nothing in the shipped package: the product path has no
CPU route and raises when the HIP library is missing.

Everything here is plain torch-on-CPU / numpy arithmetic written to follow the
reference's algorithm statement by statement (citations are paths relative to
the reference checkout):

  pack_bits                 GPT-FAST/model.py:403-407
  hard_hash_keys            GPT-FAST/model.py:409-413
  hard_hash_bhln            pipeline/train_quest/modeling/modeling_llama.py:605-615
  hypercube_protos_T        pipeline/train_quest/modeling/modeling_llama.py:569-590
  soft_hash                 GPT-FAST/model.py:392-401 (temperature 1) and
                            pipeline/train_quest/modeling/modeling_llama.py:618-638 (logits / 0.3)
  value_norm                GPT-FAST/model.py:450
  collision_score           GPT-FAST/kernels/soft_hash_collision.cu:25-54
  collision_score_vnorm16   GPT-FAST/kernels/soft_hash_score/soft_hash_score.cu:7-42
  topk_lower_index_first    torch.topk call at GPT-FAST/kernels/sparse.py:57 with
                            the tie rule "equal scores -> lower index first"
  build_sparse_list_decode  GPT-FAST/kernels/sparse.py:16-95
  sparse_decode_stage1      kernels/socket_triton_kernels.py:31-118,167-205
  sparse_decode_stage2      kernels/socket_triton_kernels.py:121-164,208-235
  sparse_attention_fwd      kernels/socket_triton_kernels.py:238-258
  sparse_attend_textbook    gather -> softmax(q.K^T / sqrt(D)) -> .V in float64
  dense_attend              GPT-FAST/model.py:562-589 (decode, S=1)
  kv_cache_update           GPT-FAST/model.py:187-229

The reference ships no tests, golden vectors or fixtures for this path, so no
function here can be pinned on the reference's own vectors.  Each function is
instead pinned in tests/test_oracle_pins.py by closed forms, invariants,
library routines and brute force (listed per function in that file).  The one
behaviour nothing can pin is the order torch.topk gives equal scores on a GPU,
which the reference leaves unspecified: this build fixes it as "lower index
first" and topk_lower_index_first is the statement of that rule.

Packed-code helpers at the end (codes_per_word / pack_code_words /
unpack_code_words / permute_planes_for_words) describe this build's own HBM
format, not anything in the reference; they are checked by round trip.
"""
from __future__ import annotations

import itertools
import math
from typing import Optional, Tuple

import numpy as np
import torch

NEG_INF = float("-inf")


# ----------------------------------------------------------------------------
# hashing
# ----------------------------------------------------------------------------
def pack_bits(bits: torch.Tensor) -> torch.Tensor:
    """Big-endian pack of the last axis: code = sum_k bit_k << (P-1-k)  -> int16.

    GPT-FAST/model.py:403-407 (same in modeling_llama.py:593-602).
    """
    P = bits.shape[-1]
    code = torch.zeros(bits.shape[:-1], dtype=torch.int32)
    for k in range(P):
        code |= bits[..., k].to(torch.int32) << (P - 1 - k)
    return code.to(torch.int16)


def hard_hash_keys(keys_bshd: torch.Tensor, planes_lpd: torch.Tensor) -> torch.Tensor:
    """keys [B,S,Hkv,D], planes [L,P,D] -> int16 codes [B,S,Hkv,L]; bit = (k.p >= 0).

    GPT-FAST/model.py:409-413.  The projection runs in the dtype of the inputs
    (bf16 in GPT-FAST), exactly as the reference einsum does.
    """
    proj = torch.einsum("bshd,lkd->bshlk", keys_bshd, planes_lpd.to(keys_bshd.dtype))
    return pack_bits(proj >= 0)


def hard_hash_bhln(x_bhnd: torch.Tensor, planes_lpd: torch.Tensor) -> torch.Tensor:
    """[B,H,N,D] -> table-major codes [B,H,L,N] (modeling_llama.py:605-615)."""
    proj = torch.einsum("bhnd,lkd->bhnlk", x_bhnd, planes_lpd.to(x_bhnd.dtype))
    return pack_bits(proj >= 0).permute(0, 1, 3, 2).contiguous()


def projections_f64(keys_bshd: torch.Tensor, planes_lpd: torch.Tensor) -> torch.Tensor:
    """float64 projections [B,S,Hkv,L,P]; used to decide which sign bits are
    far enough from zero to be compared exactly."""
    return torch.einsum("bshd,lkd->bshlk", keys_bshd.double(), planes_lpd.double())


def hypercube_protos_T(P: int, dtype=torch.float32) -> torch.Tensor:
    """Corners of {-1,+1}^P as columns, [P, 2^P]; corner r has +1 at coordinate
    k exactly when bit (P-1-k) of r is set, i.e. the same order as pack_bits.

    modeling_llama.py:569-590 (itertools.product, first coordinate slowest).
    """
    corners = torch.tensor(list(itertools.product([-1.0, 1.0], repeat=P)), dtype=torch.float32)
    return corners.t().contiguous().to(dtype)


def soft_hash(
    queries_bhd: torch.Tensor,
    planes_lpd: torch.Tensor,
    protos_T: torch.Tensor,
    temperature: float = 1.0,
) -> torch.Tensor:
    """Query soft bucket probabilities [B,H,L,R].

    logits = (tanh(q.planes) / sqrt(D)) @ protos_T ; softmax(logits / temperature).
    GPT-FAST/model.py:392-401 has no temperature (1.0); the HuggingFace twin
    divides the logits by 0.3 (modeling_llama.py:638).
    Runs in the dtype of `queries_bhd`, as the reference does.
    """
    dt = queries_bhd.dtype
    q_proj = torch.einsum("bhd,lkd->bhlk", queries_bhd, planes_lpd.to(dt))
    temp = max(math.sqrt(queries_bhd.shape[-1]), 1e-6)
    logits = torch.einsum("bhlk,kr->bhlr", torch.tanh(q_proj) / temp, protos_T.to(dt))
    if temperature != 1.0:
        logits = logits / temperature
    return torch.softmax(logits, dim=-1)


def sigmoid_product_probs(proj_bhlp: torch.Tensor, tau: float) -> torch.Tensor:
    """q_probs[l, r] = prod_k sigmoid(tau * c_{r,k} * proj[l,k]) with c the
    hypercube corner of bucket r (big-endian, as pack_bits).  This is the closed
    form of softmax over hypercube prototypes: softmax_r(sum_k c_rk s_k) =
    prod_k sigmoid(2 c_rk s_k)."""
    P = proj_bhlp.shape[-1]
    corners = hypercube_protos_T(P, torch.float64).t()  # [R,P]
    x = proj_bhlp.double().unsqueeze(-2) * corners  # [...,R,P]
    return torch.sigmoid(tau * x).prod(dim=-1)


def value_norm(v: torch.Tensor) -> torch.Tensor:
    """||v||_2 over the last axis in fp32, stored as fp16 (GPT-FAST/model.py:450)."""
    return torch.linalg.vector_norm(v.float(), ord=2, dim=-1).to(torch.float16)


# ----------------------------------------------------------------------------
# soft-collision scorer
# ----------------------------------------------------------------------------
def collision_score(
    q_probs: torch.Tensor,      # [B,H,L,R] float32
    key_buckets: torch.Tensor,  # [B,H,L,T] int16
    allowed: torch.Tensor,      # [B,H,T] bool
    v_hist: torch.Tensor,       # [B,H,T] float32
) -> torch.Tensor:
    """score[b,h,t] = allowed ? (sum_l q_probs[b,h,l,code[b,h,l,t]]) * v_hist : -inf.

    The sum runs over l = 0..L-1 in that order in fp32, one add per table, as in
    the device loop at GPT-FAST/kernels/soft_hash_collision.cu:45-53.
    """
    assert q_probs.dtype == torch.float32 and v_hist.dtype == torch.float32
    B, H, L, R = q_probs.shape
    T = key_buckets.shape[-1]
    acc = torch.zeros((B, H, T), dtype=torch.float32)
    idx = key_buckets.long()
    for l in range(L):
        acc = acc + torch.gather(q_probs[:, :, l, :], -1, idx[:, :, l, :])
    out = acc * v_hist
    return torch.where(allowed, out, torch.full_like(out, NEG_INF))


def collision_score_vnorm16(q_probs_f16, key_buckets, v_norm_f16, allowed):
    """fp16-table variant: same sum with fp16 inputs widened to fp32
    (GPT-FAST/kernels/soft_hash_score/soft_hash_score.cu:7-42)."""
    return collision_score(q_probs_f16.float(), key_buckets, allowed, v_norm_f16.float())


# ----------------------------------------------------------------------------
# top-k with the lower-index tie rule
# ----------------------------------------------------------------------------
def topk_lower_index_first(scores: torch.Tensor, M: int) -> torch.Tensor:
    """Indices of the M largest entries of the last axis, descending by score,
    equal scores ordered by ascending index (a stable descending sort)."""
    order = torch.sort(scores, dim=-1, descending=True, stable=True).indices
    return order[..., :M]


# ----------------------------------------------------------------------------
# index list: [sink | window | heavy]
# ----------------------------------------------------------------------------
def base_indices(T: int, sink: int, window: int) -> np.ndarray:
    """Sink and local-window part of the list (GPT-FAST/kernels/sparse.py:70-84)."""
    sink = max(0, min(sink, T))
    window = max(0, min(window, T))
    parts = []
    if sink > 0:
        parts.append(np.arange(sink, dtype=np.int32))
    if window > 0:
        win_start = max(T - window, sink)
        if win_start < T:
            parts.append(np.arange(win_start, T, dtype=np.int32))
    if not parts:
        return np.array([T - 1], dtype=np.int32)
    return np.concatenate(parts)


def build_sparse_list_decode(
    q_probs: torch.Tensor,      # [B,H,L,R]
    k_hard_bhlt: torch.Tensor,  # [B,H,L,T] int16/int32
    v_norm_bht: torch.Tensor,   # [B,H,T]
    allowed_bht: torch.Tensor,  # [B,H,T] bool
    sink: int,
    window: int,
    M: int,
    return_scores: bool = False,
):
    """GPT-FAST/kernels/sparse.py:16-95: scorer -> top-M -> [sink, window, heavy]
    int32 list with -1 for disallowed positions; sparse_len is the list width for
    every (b,h)."""
    B, H, L, R = q_probs.shape
    T = k_hard_bhlt.shape[-1]
    M_eff = min(M, T)
    scores = None
    if M_eff > 0:
        scores = collision_score(
            q_probs.float().contiguous(),
            k_hard_bhlt.to(torch.int16),
            allowed_bht,
            v_norm_bht.float(),
        )
        heavy = topk_lower_index_first(scores, M_eff).to(torch.int32)
    else:
        heavy = torch.empty((B, H, 0), dtype=torch.int32)
    in_range = (heavy >= 0) & (heavy < T)
    ok = torch.gather(allowed_bht, -1, heavy.clamp(0, max(T - 1, 0)).long()) if heavy.numel() else in_range
    heavy = heavy.masked_fill(~(in_range & ok), -1)

    base = torch.from_numpy(base_indices(T, sink, window)).view(1, 1, -1).expand(B, H, -1)
    base_ok = torch.gather(allowed_bht, -1, base.long())
    base = base.masked_fill(~base_ok, -1)

    sparse_list = torch.cat([base, heavy], dim=-1).contiguous()
    sparse_len = torch.full((B, H), sparse_list.shape[-1], dtype=torch.int32)
    if return_scores:
        return sparse_list, sparse_len, scores
    return sparse_list, sparse_len


# ----------------------------------------------------------------------------
# sparse flash-decode
# ----------------------------------------------------------------------------
def sparse_decode_stage1(
    q: torch.Tensor,            # [B,H,D]
    k: torch.Tensor,            # [B,Hkv,S,D]
    v: torch.Tensor,            # [B,Hkv,S,D]
    sparse_list: torch.Tensor,  # [B,H,Ktotal] int32
    sparse_len: torch.Tensor,   # [B,H] int32
    max_len_in_batch: int,
    block_seq: int = 256,
    block_n: int = 16,
    round_products: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per (b,h,split) partial attention over list[split*block_seq : ...] in
    chunks of `block_n` rows with the running-max recurrence of
    kernels/socket_triton_kernels.py:73-104; returns (acc/sum_exp, max+log(sum_exp))
    as the kernel stores them (:117-118).  Splits with no rows are left as NaN
    (the kernel does not write them).  A list entry < 0 is a skipped row: it gets
    weight zero (the reference would read row -1, which never happens on its
    call path because every position up to the newest token is allowed).

    round_products=True additionally rounds q*k and the row sums to the input
    dtype, which is what the reference's bf16 tile arithmetic does; the default
    keeps fp32 throughout.
    """
    B, H, D = q.shape
    G = H // k.shape[1]
    nsplit = (max_len_in_batch + block_seq - 1) // block_seq
    mid_o = torch.full((B, H, nsplit, D), float("nan"), dtype=torch.float32)
    mid_lse = torch.full((B, H, nsplit), float("nan"), dtype=torch.float32)
    sm_scale = 1.0 / math.sqrt(D)
    for b in range(B):
        for h in range(H):
            n = int(sparse_len[b, h])
            kv = h // G
            qv = q[b, h]
            for s in range(nsplit):
                lo, hi = s * block_seq, min(n, (s + 1) * block_seq)
                if hi <= lo:
                    continue
                m_run = torch.tensor(NEG_INF)
                sum_exp = torch.tensor(0.0)
                acc = torch.zeros(D, dtype=torch.float32)
                for c0 in range(lo, hi, block_n):
                    ids = sparse_list[b, h, c0:min(c0 + block_n, hi)].long()
                    live = ids >= 0
                    rows = ids.clamp(min=0)
                    kk = k[b, kv, rows]
                    vv = v[b, kv, rows].float()
                    if round_products:
                        att = (qv[None, :] * kk).float().sum(1).to(q.dtype) * sm_scale
                        att = att.to(q.dtype).float()
                    else:
                        att = (qv.float()[None, :] * kk.float()).sum(1) * sm_scale
                    att = torch.where(live, att, torch.full_like(att, NEG_INF))
                    new_m = torch.maximum(att.max(), m_run)
                    if new_m == NEG_INF:
                        continue
                    p = torch.exp(att - new_m)
                    scale = torch.exp(m_run - new_m)
                    acc = acc * scale + (p[:, None] * vv).sum(0)
                    sum_exp = sum_exp * scale + p.sum()
                    m_run = new_m
                mid_o[b, h, s] = acc / sum_exp
                mid_lse[b, h, s] = m_run + torch.log(sum_exp)
    return mid_o, mid_lse


def sparse_decode_stage2(
    mid_o: torch.Tensor, mid_lse: torch.Tensor, sparse_len: torch.Tensor,
    out_dtype: torch.dtype, block_seq: int = 256,
) -> torch.Tensor:
    """Merge of the per-split partials (kernels/socket_triton_kernels.py:121-164)."""
    B, H, _, D = mid_o.shape
    out = torch.empty((B, H, D), dtype=out_dtype)
    for b in range(B):
        for h in range(H):
            n = int(sparse_len[b, h])
            nblk = 0 if n <= 0 else (n + block_seq - 1) // block_seq
            m_run = torch.tensor(NEG_INF)
            sum_exp = torch.tensor(0.0)
            acc = torch.zeros(D, dtype=torch.float32)
            for s in range(nblk):
                lse = mid_lse[b, h, s]
                new_m = torch.maximum(lse, m_run)
                old = torch.exp(m_run - new_m)
                w = torch.exp(lse - new_m)
                acc = acc * old + w * mid_o[b, h, s]
                sum_exp = sum_exp * old + w
                m_run = new_m
            out[b, h] = (acc / sum_exp).to(out_dtype)
    return out


def sparse_attention_fwd(q, k, v, sparse_list, sparse_len, block_seq: int = 256,
                         round_products: bool = False) -> torch.Tensor:
    """kernels/socket_triton_kernels.py:238-258."""
    max_len = int(sparse_len.max())
    mid_o, mid_lse = sparse_decode_stage1(q, k, v, sparse_list, sparse_len, max_len,
                                          block_seq, round_products=round_products)
    return sparse_decode_stage2(mid_o, mid_lse, sparse_len, q.dtype, block_seq)


def sparse_attend_textbook(q, k, v, sparse_list, sparse_len) -> torch.Tensor:
    """softmax(q.K_sel^T / sqrt(D)) . V_sel over the listed rows (duplicates are
    counted as many times as they appear, negative entries not at all) in
    float64; returns float64 [B,H,D].  Vectorised: usable at full config sizes."""
    B, H, D = q.shape
    G = H // k.shape[1]
    Kt = sparse_list.shape[-1]
    out = torch.empty((B, H, D), dtype=torch.float64)
    pos = torch.arange(Kt)
    for b in range(B):
        for h in range(H):
            ids = sparse_list[b, h].long()
            live = (pos < int(sparse_len[b, h])) & (ids >= 0)
            rows = ids.clamp(min=0)
            kk = k[b, h // G, rows].double()
            vv = v[b, h // G, rows].double()
            att = (kk @ q[b, h].double()) / math.sqrt(D)
            att = torch.where(live, att, torch.full_like(att, NEG_INF))
            w = torch.softmax(att, dim=0)
            out[b, h] = w @ vv
    return out


def dense_attend(q, k, v, lengths=None) -> torch.Tensor:
    """Full attention of one query per head over rows [0, len_b) of a [B,Hkv,T,D]
    cache with the GQA map kv = h // G (GPT-FAST/model.py:583-587 for S=1), float64."""
    B, H, D = q.shape
    Hkv, T = k.shape[1], k.shape[2]
    G = H // Hkv
    out = torch.empty((B, H, D), dtype=torch.float64)
    for b in range(B):
        n = T if lengths is None else int(lengths[b])
        for h in range(H):
            kk = k[b, h // G, :n].double()
            vv = v[b, h // G, :n].double()
            w = torch.softmax((kk @ q[b, h].double()) / math.sqrt(D), dim=0)
            out[b, h] = w @ vv
    return out


# ----------------------------------------------------------------------------
# cache
# ----------------------------------------------------------------------------
def kv_cache_update(cache: dict, input_pos: torch.Tensor, k_val, v_val, v_norm=None, k_hard=None):
    """GPT-FAST/model.py:187-229 on a dict of tensors
    {k_cache,v_cache [B,H,T,D], k_hard [B,H,T,L], v_norm [B,H,T], prefill_len int}."""
    pos = input_pos.long()
    Tcap = cache["k_cache"].shape[2]
    if pos.numel() and (int(pos.max()) >= Tcap or int(pos.min()) < 0):
        raise RuntimeError("KVCache.update out-of-bounds")
    cache["k_cache"][:, :, pos, :] = k_val.permute(0, 2, 1, 3)
    cache["v_cache"][:, :, pos, :] = v_val.permute(0, 2, 1, 3)
    if v_norm is not None:
        cache["v_norm"][:, :, pos] = v_norm.permute(0, 2, 1)
    if k_hard is not None:
        cache["k_hard"][:, :, pos, :] = k_hard.permute(0, 2, 1, 3)
    cache["prefill_len"] = max(int(cache["prefill_len"]), int(pos.max()) + 1 if pos.numel() else 0)
    return cache["k_cache"], cache["v_cache"]


# ----------------------------------------------------------------------------
# this build's packed-code format (not in the reference)
# ----------------------------------------------------------------------------
def codes_per_word(P: int) -> int:
    return 32 // P


def words_per_key(L: int, P: int) -> int:
    c = codes_per_word(P)
    return (L + c - 1) // c


def pack_code_words(codes_blt: np.ndarray, P: int) -> np.ndarray:
    """int codes [..., L, T] -> uint32 words [..., NW, T]; table l sits in word
    l // c at bit offset (l % c) * P, c = 32 // P; unused high bits are zero."""
    L, T = codes_blt.shape[-2:]
    c, nw = codes_per_word(P), words_per_key(L, P)
    words = np.zeros(codes_blt.shape[:-2] + (nw, T), dtype=np.uint32)
    for l in range(L):
        words[..., l // c, :] |= (codes_blt[..., l, :].astype(np.uint32) & ((1 << P) - 1)) << np.uint32((l % c) * P)
    return words


def unpack_code_words(words: np.ndarray, L: int, P: int) -> np.ndarray:
    c = codes_per_word(P)
    out = np.empty(words.shape[:-2] + (L, words.shape[-1]), dtype=np.int16)
    for l in range(L):
        out[..., l, :] = ((words[..., l // c, :] >> np.uint32((l % c) * P)) & np.uint32((1 << P) - 1)).astype(np.int16)
    return out


def permute_planes_for_words(planes_lpd: torch.Tensor) -> torch.Tensor:
    """[L,P,D] -> [NW*32, D]: row w*32 + p holds the plane whose sign becomes bit
    p of packed word w (table w*c + p // P, hyperplane P-1 - p % P); rows for
    unused bit positions are zero."""
    L, P, D = planes_lpd.shape
    c, nw = codes_per_word(P), words_per_key(L, P)
    out = torch.zeros((nw * 32, D), dtype=planes_lpd.dtype)
    for w in range(nw):
        for p in range(c * P):
            l = w * c + p // P
            if l < L:
                out[w * 32 + p] = planes_lpd[l, P - 1 - (p % P)]
    return out
