"""The HIP-native decode path: packed per-KV-head hash cache and the
score -> select -> attend step on it.

This is what the attention hook calls instead of the reference's per-step
relayout (GPT-FAST/model.py:490-509), scorer + torch.topk + list assembly
(GPT-FAST/kernels/sparse.py:16-95) and K/V prefix copies
(GPT-FAST/model.py:541-542).  HBM layout per layer:

  k_cache, v_cache  [B, Hkv, Tcap, D]   model dtype      (as KVCache, model.py:175-176)
  codes             [B, Hkv, NW, Tcap]  uint32 (int32 tensor), packed bucket codes,
                                        table-major; replaces k_hard [B,Hkv,T,L] int16
  v_norm            [B, Hkv, Tcap]      float16          (as KVCache, model.py:182)
  lens              [B]                 int32, device    (replaces the 0-d prefill_len)

Nothing on the step path reads a length back to the host.
"""
from __future__ import annotations

import functools
import math
from typing import Optional, Tuple

import torch

from ._lib import check, dtype_enum, lib, ptr, stream_ptr
from .socket_kernels import prefers_one_launch, sparse_attention_fwd, sparse_attention_fwd_static
from .sparse import select_list


HASH_DIM = 128     # coordinates the hashing kernel contracts over


def words_per_key(L: int, P: int) -> int:
    nw = lib().socket_words_per_key(int(L), int(P))
    if nw <= 0:
        raise RuntimeError(f"unsupported hash shape L={L}, P={P} (need L >= 1, 1 <= P <= 16)")
    return nw


@torch.no_grad()
def permute_planes(planes_lpd: torch.Tensor) -> torch.Tensor:
    """[L,P,D] hyperplanes -> bf16 [NW*32, D] in packed-bit column order.  The
    hashing kernel contracts over 128 coordinates: planes of a narrower head are
    padded with zeros up to 128 (`hash_keys_into` pads the rows to match; a zero
    coordinate changes no projection)."""
    assert planes_lpd.is_cuda and planes_lpd.dim() == 3
    L, P, D = planes_lpd.shape
    if D < HASH_DIM:
        planes_lpd = torch.nn.functional.pad(planes_lpd, (0, HASH_DIM - D))
        D = HASH_DIM
    planes_lpd = planes_lpd.contiguous()
    out = torch.empty((words_per_key(L, P) * 32, D), dtype=torch.bfloat16, device=planes_lpd.device)
    check("socket_permute_planes", lib().socket_permute_planes(
        ptr(planes_lpd), dtype_enum(planes_lpd.dtype), L, P, D, ptr(out), stream_ptr(planes_lpd.device)))
    return out


@torch.no_grad()
def hash_keys_into(k: torch.Tensor, v: Optional[torch.Tensor], planes_words: torch.Tensor,
                   codes: torch.Tensor, v_norm: Optional[torch.Tensor], L: int, P: int,
                   t0: int = 0, pos_b: Optional[torch.Tensor] = None, layout: str = "bhsd") -> None:
    """Hash new keys (and take value norms) into the packed cache at positions
    t0 + s (or pos_b[b] + s).  `k`/`v` are [B,Hkv,S,D] (layout "bhsd") or
    [B,S,Hkv,D] ("bshd"), any strides with a contiguous last dim."""
    assert k.is_cuda and codes.is_cuda and codes.dtype == torch.int32 and codes.is_contiguous()
    if layout == "bhsd":
        B, Hkv, S, D = k.shape
        ks = (k.stride(0), k.stride(1), k.stride(2))
        vs = (v.stride(0), v.stride(1), v.stride(2)) if v is not None else (0, 0, 0)
    elif layout == "bshd":
        B, S, Hkv, D = k.shape
        ks = (k.stride(0), k.stride(2), k.stride(1))
        vs = (v.stride(0), v.stride(2), v.stride(1)) if v is not None else (0, 0, 0)
    else:
        raise ValueError(layout)
    assert k.stride(-1) == 1 and (v is None or (v.stride(-1) == 1 and v.shape == k.shape and v.dtype == k.dtype))
    if D < HASH_DIM and planes_words.shape[1] == HASH_DIM and S > 0:
        # a narrower head: the new rows are padded with zeros to the kernel's 128 coordinates
        # (same sign bits, same value norms); strides are then those of the padded copies
        k = torch.nn.functional.pad(k, (0, HASH_DIM - D))
        v = None if v is None else torch.nn.functional.pad(v, (0, HASH_DIM - D))
        D = HASH_DIM
        if layout == "bhsd":
            ks = (k.stride(0), k.stride(1), k.stride(2))
            vs = (v.stride(0), v.stride(1), v.stride(2)) if v is not None else (0, 0, 0)
        else:
            ks = (k.stride(0), k.stride(2), k.stride(1))
            vs = (v.stride(0), v.stride(2), v.stride(1)) if v is not None else (0, 0, 0)
    NW, Tcap = codes.shape[2], codes.shape[3]
    assert codes.shape[0] == B and codes.shape[1] == Hkv and NW == words_per_key(L, P)
    if v is not None:
        assert v_norm is not None and v_norm.dtype == torch.float16 and v_norm.is_contiguous()
        assert tuple(v_norm.shape) == (B, Hkv, Tcap)
    if pos_b is not None:
        assert pos_b.dtype == torch.int32 and pos_b.is_cuda and pos_b.numel() == B
    if S == 0:
        return
    check("socket_hash_keys", lib().socket_hash_keys(
        ptr(k), ptr(v), dtype_enum(k.dtype), *ks, *vs, ptr(planes_words), ptr(codes), ptr(v_norm),
        ptr(pos_b), int(t0), B, Hkv, S, D, int(L), int(P), Tcap, stream_ptr(k.device)))


@torch.no_grad()
def unpack_codes(codes: torch.Tensor, L: int, P: int, t0: int, T: int, layout: str = "bhlt") -> torch.Tensor:
    """Packed words -> int16 codes in one of the reference's layouts:
    "bhlt" [B,Hkv,L,T] (modeling_llama.py:615) or "bthl" [B,T,Hkv,L] (model.py:413)."""
    B, Hkv, NW, Tcap = codes.shape
    if layout == "bhlt":
        out = torch.empty((B, Hkv, L, T), dtype=torch.int16, device=codes.device)
        st = (out.stride(0), out.stride(1), out.stride(2), out.stride(3))
    elif layout == "bthl":
        out = torch.empty((B, T, Hkv, L), dtype=torch.int16, device=codes.device)
        st = (out.stride(0), out.stride(2), out.stride(3), out.stride(1))
    else:
        raise ValueError(layout)
    if T > 0:
        check("socket_unpack_codes", lib().socket_unpack_codes(
            ptr(codes), ptr(out), B, Hkv, int(L), int(P), int(t0), int(T), Tcap, *st,
            stream_ptr(codes.device)))
    return out


@torch.no_grad()
def pack_codes_into(codes_i16_bhlt: torch.Tensor, codes: torch.Tensor, P: int, t0: int = 0) -> None:
    """int16 [B,Hkv,L,T] (any strides) -> packed words at cache positions [t0, t0+T)."""
    B, Hkv, L, T = codes_i16_bhlt.shape
    assert codes_i16_bhlt.dtype == torch.int16 and codes.dtype == torch.int32 and codes.is_contiguous()
    c = codes_i16_bhlt
    if T > 0:
        check("socket_pack_codes", lib().socket_pack_codes(
            ptr(c), c.stride(0), c.stride(1), c.stride(2), c.stride(3), ptr(codes), B, Hkv, L, int(P),
            int(t0), T, codes.shape[3], stream_ptr(codes.device)))


def group_shape(n_heads: int, n_kv_heads: int) -> Tuple[int, int]:
    """(parts, width) of the grouped table layout for this head geometry."""
    import ctypes
    parts, width = ctypes.c_int(0), ctypes.c_int(0)
    check("socket_group_shape", lib().socket_group_shape(int(n_heads), int(n_kv_heads), ctypes.byref(parts),
                                                         ctypes.byref(width)))
    return parts.value, width.value


@functools.lru_cache(maxsize=4096)
def _prefers_grouped(B: int, Hq: int, Hkv: int, T: int, dtype_code: int, L: int, P: int, R: int) -> bool:
    r = lib().socket_score_prefers_grouped(B, Hq, Hkv, T, dtype_code, L, P, R)
    if r < 0:
        raise ValueError(f"socket_score_prefers_grouped: invalid shape B={B} Hq={Hq} Hkv={Hkv} T={T} L={L} P={P} R={R}")
    return bool(r)


@functools.lru_cache(maxsize=4096)
def _persistent_serves(B: int, Hq: int, Hkv: int, T: int, dtype_code: int, L: int, P: int, R: int) -> bool:
    return lib().socket_score_persistent_serves(B, Hq, Hkv, T, dtype_code, L, P, R) == 1


def prefers_grouped(q_bhd: torch.Tensor, planes: torch.Tensor, protos_T: torch.Tensor, n_kv_heads: int,
                    context_len: int, out_dtype: Optional[torch.dtype] = None) -> bool:
    """Which table layout `soft_hash` should write for a scorer call over
    `context_len` cached tokens: True = grouped, False = [B,Hq,L,R] (short
    contexts with few kv heads, which the scorer serves one head per workgroup)."""
    B, Hq = int(q_bhd.shape[0]), int(q_bhd.shape[1])
    L, P = int(planes.shape[0]), int(planes.shape[1])
    if out_dtype is None:
        out_dtype = torch.bfloat16 if q_bhd.dtype == torch.bfloat16 else torch.float32
    return _prefers_grouped(B, Hq, int(n_kv_heads), int(context_len), dtype_enum(out_dtype), L, P,
                            int(protos_T.shape[1]))


@torch.no_grad()
def group_q_probs(q_probs: torch.Tensor, n_kv_heads: int) -> torch.Tensor:
    """[B,Hq,L,R] (float32 / bfloat16) -> grouped table [B, Hkv*parts, L, R, width]:
    the query heads of a KV head interleaved per bucket, which is how the scorer
    keeps the table in LDS."""
    assert q_probs.is_cuda and q_probs.dim() == 4
    if q_probs.dtype not in (torch.float32, torch.bfloat16):
        q_probs = q_probs.float()
    q_probs = q_probs.contiguous()
    B, Hq, L, R = q_probs.shape
    parts, width = group_shape(Hq, n_kv_heads)
    out = torch.empty((B, n_kv_heads * parts, L, R, width), dtype=q_probs.dtype, device=q_probs.device)
    check("socket_group_q_probs", lib().socket_group_q_probs(
        ptr(q_probs), dtype_enum(q_probs.dtype), ptr(out), B, Hq, int(n_kv_heads), L, R,
        stream_ptr(q_probs.device)))
    return out


@torch.no_grad()
def soft_hash(queries_bhd: torch.Tensor, planes_lkd: torch.Tensor, protos_T: torch.Tensor,
              temperature: float = 1.0, n_kv_heads: Optional[int] = None,
              out_dtype: Optional[torch.dtype] = None, grouped: bool = False) -> torch.Tensor:
    """Query soft bucket probabilities [B,Hq,L,R] in one launch:
    softmax_r((tanh(q . planes) / sqrt(D)) @ protos_T / temperature)
    (GPT-FAST/model.py:392-401 with temperature 1; modeling_llama.py:618-638 with
    0.3).  fp32 arithmetic on the stored inputs, one rounding to `out_dtype`
    (bfloat16 for bfloat16 queries, else float32).  `grouped=True` writes the
    scorer's grouped table layout [B, Hkv*parts, L, R, width] instead (same values;
    `n_kv_heads` is then required)."""
    assert queries_bhd.is_cuda and queries_bhd.dim() == 3 and queries_bhd.stride(-1) == 1
    B, Hq, D = queries_bhd.shape
    L, K, D2 = planes_lkd.shape
    K2, R = protos_T.shape
    assert D2 == D and K2 == K
    dt = queries_bhd.dtype
    planes_lkd = planes_lkd.to(dt).contiguous()
    protos_T = protos_T.to(dt).contiguous()
    if out_dtype is None:
        out_dtype = torch.bfloat16 if dt == torch.bfloat16 else torch.float32
    args = lambda out, Hkv: (
        ptr(queries_bhd), dtype_enum(dt), queries_bhd.stride(0), queries_bhd.stride(1), ptr(planes_lkd),
        ptr(protos_T), ptr(out), dtype_enum(out_dtype), B, Hq, Hkv, D, L, K, R,
        1.0 / max(math.sqrt(D), 1e-6), 1.0 / float(temperature), stream_ptr(queries_bhd.device))
    if grouped:
        assert n_kv_heads, "the grouped layout is defined by the number of KV heads"
        parts, width = group_shape(Hq, n_kv_heads)
        out = torch.empty((B, n_kv_heads * parts, L, R, width), dtype=out_dtype, device=queries_bhd.device)
        check("socket_soft_hash_grouped", lib().socket_soft_hash_grouped(*args(out, int(n_kv_heads))))
        return out
    Hkv = n_kv_heads if n_kv_heads else Hq
    if Hq % Hkv != 0 or Hq // Hkv > 8:
        Hkv = Hq
    out = torch.empty((B, Hq, L, R), dtype=out_dtype, device=queries_bhd.device)
    check("socket_soft_hash", lib().socket_soft_hash(*args(out, Hkv)))
    return out


def decode_prologue_fits(qkv: torch.Tensor, head_dim: int, K: int, R: int, n_heads: int, n_kv_heads: int) -> bool:
    """Whether `decode_prologue` takes these operands (else: rope_append, hash_keys_into
    and soft_hash, three launches with the same results)."""
    return (qkv.is_cuda and qkv.dtype == torch.bfloat16 and head_dim == HASH_DIM and K == 10 and R % 4 == 0 and
            4 <= R <= 1024 and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads <= 8)


@torch.no_grad()
def decode_prologue(qkv: torch.Tensor, freqs_cis: torch.Tensor, input_pos: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, lens: Optional[torch.Tensor], planes_words: torch.Tensor,
                    codes: torch.Tensor, v_norm: torch.Tensor, planes_lkd: torch.Tensor, protos_T: torch.Tensor,
                    n_heads: int, n_kv_heads: int, temperature: float = 1.0, grouped: bool = False):
    """The head of a single-token decode step in one launch: rotary embedding of the
    new q and k (from the fused projection qkv [B,(Hq+2Hkv)*D]), K/V append at
    input_pos, `lens` raised, hash + value norm of the new key into `codes` /
    `v_norm`, and the soft hash of the rotated queries (GPT-FAST/model.py:433-451 and
    :392-401).  Returns (q [B,Hq,D], q_probs in the reference's or the grouped
    layout).  Same results as decode_ops.rope_append + hash_keys_into + soft_hash."""
    B = qkv.shape[0]
    q2 = qkv.reshape(B, -1)
    D = k_cache.shape[-1]
    L, K, D2 = planes_lkd.shape
    K2, R = protos_T.shape
    assert decode_prologue_fits(q2, D, K, R, n_heads, n_kv_heads) and D2 == D and K2 == K
    assert q2.stride(-1) == 1 and q2.shape[1] == (n_heads + 2 * n_kv_heads) * D
    assert k_cache.shape == v_cache.shape and k_cache.stride() == v_cache.stride() and k_cache.stride(-1) == 1
    assert k_cache.dtype == q2.dtype and k_cache.shape[0] == B and k_cache.shape[1] == n_kv_heads
    assert input_pos.dtype == torch.int64 and input_pos.is_cuda and input_pos.numel() in (1, B)
    assert freqs_cis.is_contiguous() and freqs_cis.shape[1:] == (D // 2, 2)
    Tcap = k_cache.shape[2]
    NW = words_per_key(L, K)
    assert codes.dtype == torch.int32 and codes.is_contiguous() and tuple(codes.shape) == (B, n_kv_heads, NW, Tcap)
    assert v_norm.dtype == torch.float16 and v_norm.is_contiguous() and tuple(v_norm.shape) == (B, n_kv_heads, Tcap)
    assert planes_words.dtype == torch.bfloat16 and planes_words.is_contiguous()
    assert tuple(planes_words.shape) == (NW * 32, HASH_DIM)
    if lens is not None:
        assert lens.dtype == torch.int32 and lens.numel() == B
    planes_lkd = planes_lkd.to(q2.dtype).contiguous()
    protos_T = protos_T.to(q2.dtype).contiguous()
    q_out = torch.empty((B, n_heads, D), dtype=q2.dtype, device=q2.device)
    if grouped:
        parts, width = group_shape(n_heads, n_kv_heads)
        table = torch.empty((B, n_kv_heads * parts, L, R, width), dtype=q2.dtype, device=q2.device)
    else:
        table = torch.empty((B, n_heads, L, R), dtype=q2.dtype, device=q2.device)
    check("socket_decode_prologue", lib().socket_decode_prologue(
        ptr(q2), dtype_enum(q2.dtype), q2.stride(0), ptr(freqs_cis), dtype_enum(freqs_cis.dtype), freqs_cis.shape[0],
        ptr(input_pos), 0 if input_pos.numel() == 1 else 1, ptr(q_out), ptr(k_cache), ptr(v_cache),
        k_cache.stride(0), k_cache.stride(1), k_cache.stride(2), ptr(lens), ptr(planes_words), ptr(codes),
        ptr(v_norm), ptr(planes_lkd), ptr(protos_T), ptr(table), dtype_enum(q2.dtype), int(bool(grouped)), B,
        n_heads, n_kv_heads, D, L, K, R, Tcap, 1.0 / max(math.sqrt(D), 1e-6), 1.0 / float(temperature),
        stream_ptr(q2.device)))
    return q_out, table


@torch.no_grad()
def score_packed(q_probs: torch.Tensor, codes: torch.Tensor, v_norm: torch.Tensor, T: int, P: int,
                 lens: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                 with_range: bool = False, n_heads: Optional[int] = None, skip_masked: bool = False):
    """Soft-collision scores [B,Hq,T] fp32 (row pitch padded to a multiple of 4)
    from q_probs [B,Hq,L,R] and the packed cache.  q_probs may be float32 or
    bfloat16; a bfloat16 table is read as is (the reference widens it with
    `.float()`, GPT-FAST/kernels/sparse.py:42, which changes no value) and halves
    the LDS bytes per gather.  float16 is widened to float32 first.
    with_range=True also returns the per-tile key ranges of every row (int32
    [B,Hq,parts,2]) for `select_list(..., row_range=...)`.
    skip_masked=True: positions at or past `lens[b]` may be left unwritten instead of
    set to -inf (for a consumer that reads rows only up to `lens[b]`)."""
    assert q_probs.is_cuda and q_probs.dim() in (4, 5)
    if q_probs.dtype not in (torch.float32, torch.bfloat16):
        q_probs = q_probs.float()
    q_probs = q_probs.contiguous()
    _, Hkv, NW, Tcap = codes.shape
    grouped = q_probs.dim() == 5
    if grouped:       # [B, Hkv*parts, L, R, width] as written by soft_hash(grouped=True) / group_q_probs
        assert n_heads is not None, "a grouped table does not carry the number of query heads: pass n_heads"
        Hq = int(n_heads)
        B = codes.shape[0]
        parts, width = group_shape(Hq, Hkv)
        assert q_probs.shape[0] == B and q_probs.shape[1] == Hkv * parts and q_probs.shape[4] == width
        L, R = q_probs.shape[2], q_probs.shape[3]
    else:
        B, Hq, L, R = q_probs.shape
        if not with_range and Hq % Hkv == 0 and _persistent_serves(B, Hq, Hkv, int(T), dtype_enum(q_probs.dtype),
                                                                   L, int(P), R):
            # a call large enough for the persistent launch, which wants the grouped table:
            # one pass over the table (a few percent of the scorer's bytes) buys it
            q_probs = group_q_probs(q_probs, Hkv)
            grouped = True
    assert codes.dtype == torch.int32 and codes.is_contiguous() and codes.shape[0] == B
    assert v_norm.dtype == torch.float16 and v_norm.is_contiguous() and tuple(v_norm.shape) == (B, Hkv, Tcap)
    assert NW == words_per_key(L, P), "codes were packed for a different (L, P)"
    pitch = (T + 3) // 4 * 4
    if out is None:
        out = torch.empty((B, Hq, pitch), dtype=torch.float32, device=q_probs.device)
    else:
        assert out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (B, Hq, pitch)
    if lens is not None:
        assert lens.dtype == torch.int32 and lens.is_cuda and lens.numel() == B
    rng, parts = None, 0
    if with_range:
        count = lib().socket_score_range_parts_grouped if grouped else lib().socket_score_range_parts
        parts = count(B, Hq, Hkv, int(T), dtype_enum(q_probs.dtype), L, int(P), R)
        rng = torch.empty((B, Hq, parts, 2), dtype=torch.int32, device=q_probs.device)
    entry = lib().socket_score_packed_grouped if grouped else lib().socket_score_packed
    check("socket_score_packed", entry(
        ptr(q_probs), dtype_enum(q_probs.dtype), ptr(codes), ptr(v_norm), ptr(lens), ptr(out),
        ptr(rng), parts, B, Hq, Hkv, L, int(P), R, int(T), Tcap, pitch, 1 if skip_masked else 0,
        stream_ptr(q_probs.device)))
    if with_range:
        return out[:, :, :T], rng
    return out[:, :, :T]


# Devices whose copy of the library's fixed scratch array has had its address looked up
# (socket_static_scratch_init), which has to happen outside any stream capture.
_STATIC_READY = set()


def prepare_one_launch_attention(device=None) -> None:
    """Look up the library's fixed scratch array on `device` (default: the current
    one).  Call it outside stream capture -- `generate.warmup_sparse_decode` and any
    eager `sparse_decode_step` do -- before a step is recorded into a graph."""
    idx = torch.cuda.current_device() if device is None or torch.device(device).index is None \
        else torch.device(device).index
    if idx in _STATIC_READY or torch.cuda.is_current_stream_capturing():
        return
    with torch.cuda.device(idx):
        check("socket_static_scratch_init", lib().socket_static_scratch_init())
    _STATIC_READY.add(idx)


def _use_one_launch(q: torch.Tensor, width: int, one_launch: Optional[bool]) -> bool:
    B, Hq, D = q.shape
    if one_launch is False or not prefers_one_launch(B, Hq, D, width):
        return False
    idx = q.device.index if q.device.index is not None else torch.cuda.current_device()
    capturing = torch.cuda.is_current_stream_capturing()
    if not capturing:
        prepare_one_launch_attention(q.device)
    if one_launch is True:
        return idx in _STATIC_READY
    # default: only inside a graph capture, whose replays the caller issues one after another
    return capturing and idx in _STATIC_READY


@torch.no_grad()
def sparse_decode_step(q: torch.Tensor, q_probs: torch.Tensor, k_cache: torch.Tensor,
                       v_cache: torch.Tensor, codes: torch.Tensor, v_norm: torch.Tensor, T: int, P: int,
                       sink: int, window: int, M: int, lens: Optional[torch.Tensor] = None,
                       budgets: Optional[torch.Tensor] = None,
                       return_details: bool = False, one_launch: Optional[bool] = None,
                       scores_buf: Optional[torch.Tensor] = None):
    """One decode step of sparse attention for one layer: score every cached key,
    select top-M + sink + window, attend over the selected rows.

    q [B,Hq,D]; q_probs [B,Hq,L,R]; T = number of cached tokens to consider (an
    upper bound when `lens` gives per-sequence lengths).  Returns out [B,Hq,D].

    `one_launch`: the attention has a one-launch form whose split partials and
    arrival counters live in ONE array per GPU inside the library
    (`socket_sparse_attention_static`): two such calls that overlap on a GPU -- two
    streams, two threads, an eager step beside a graph replay -- corrupt each other
    silently.  The default (None) therefore takes it only while the step is being
    recorded into a HIP graph, where it also saves the allocation, and the eager
    step takes the re-entrant two-launch form with a workspace per call (same
    output, bit for bit).  Replays of graphs that hold this step must not overlap
    on one GPU.  True forces the one-launch form (the caller answers for the
    serialisation), False forbids it.

    `scores_buf`: an fp32 [B, Hq, T rounded up to 4] tensor to score into (67 MB at
    4 x 32 heads x 131072 tokens); without it the step allocates one per call, which an
    eager serving loop may want to avoid (under graph capture the allocation is the
    graph pool's and costs nothing per replay).
    """
    # (no per-tile key ranges from the scorer: the selection draws its threshold from a
    # sample of the row and only a row whose sample misleads it falls back to a pass
    # that would use them; tracking them costs the scorer more than that pass saves)
    # (positions past a sequence's length are written only when the caller gets the scores back:
    # the selection reads a row up to the same `lens`)
    scores = score_packed(q_probs, codes, v_norm, T, P, lens=lens, n_heads=q.shape[1], out=scores_buf,
                          skip_masked=not return_details)
    sparse_list, sparse_len = select_list(scores, sink, window, M, lens=lens, budgets=budgets)
    B, Hq, D = q.shape
    if _use_one_launch(q, sparse_list.shape[-1], one_launch):
        out = sparse_attention_fwd_static(q, k_cache, v_cache, sparse_list, sparse_len,
                                          torch.empty((B, Hq, D), dtype=q.dtype, device=q.device))
    else:
        out = sparse_attention_fwd(q, k_cache, v_cache, sparse_list, sparse_len)
    if return_details:
        return out, scores, sparse_list, sparse_len
    return out


@functools.lru_cache(maxsize=1024)
def step_cost_estimate(B: int, Hq: int, Hkv: int, D: int, T: int, L: int, P: int, R: int, M: int,
                       sink: int, window: int, table_bf16: bool = True, cache_bytes: int = 2) -> Tuple[float, float]:
    """(sparse_us, dense_us): rough device time of one layer's decode attention
    over T cached tokens, for choosing between the two.  The scorer's figure is the
    library's own launch-shape estimate (`socket_score_plan_query`); the selection,
    the two attentions and the launches are priced from what they read at the rates
    measured for them on a 256-CU MI355X (a row's selection: ~11 us of threshold
    and placement plus 3.7 us per 32768 scores a workgroup streams, 3 us more when
    a row is shared; gathers at 5.2 TB/s; the dense stream at 6.4 TB/s; ~4 us a
    launch).  Good to some 20 %: it places the crossover, it is not a timing."""
    import ctypes
    cus = ctypes.c_int(0)
    lib().socket_device_query(ctypes.byref(cus), None)
    cu = max(1, cus.value)
    cost = ctypes.c_float(0.0)
    check("socket_score_plan_query", lib().socket_score_plan_query(
        B, Hq, Hkv, T, dtype_enum(torch.bfloat16 if table_bf16 else torch.float32), L, P, R, 1,
        None, None, None, ctypes.byref(cost)))
    rows = B * Hq
    parts = 1
    ws = lib().socket_select_workspace_bytes(B, Hq, T, M)
    if ws:
        parts = max(1, min(16, cu // rows, T // 16384))
    rounds = -(-rows * parts // cu)
    select = rounds * (11.0 + 3.7 * (T / parts) / 32768.0 + (3.0 if parts > 1 else 0.0))
    listed = min(T, sink + window + M)
    esize = int(cache_bytes)             # bytes per K/V element
    attend = rows * listed * (2 * D * esize + 4) / 5.2e6 + (0.0 if 2 * rows >= cu else 5.0)
    dense = B * Hkv * T * 2 * D * esize / 6.4e6 + 5.0
    launch = 4.0
    return float(cost.value + select + attend + 3 * launch), float(dense + launch)


class SocketHashCache:
    """Per-layer K/V + hash cache in the layout above, with in-place append."""

    def __init__(self, max_batch_size: int, max_seq_length: int, n_kv_heads: int, head_dim: int,
                 L: int, P: int, dtype=torch.bfloat16, device="cuda"):
        B, H, D = max_batch_size, n_kv_heads, head_dim
        Tcap = (max_seq_length + 7) // 8 * 8
        self.L, self.P, self.NW, self.Tcap = L, P, words_per_key(L, P), Tcap
        self.k_cache = torch.zeros((B, H, Tcap, D), dtype=dtype, device=device)
        self.v_cache = torch.zeros((B, H, Tcap, D), dtype=dtype, device=device)
        self.codes = torch.zeros((B, H, self.NW, Tcap), dtype=torch.int32, device=device)
        self.v_norm = torch.zeros((B, H, Tcap), dtype=torch.float16, device=device)
        self.lens = torch.zeros((B,), dtype=torch.int32, device=device)
        self.planes_words: Optional[torch.Tensor] = None

    def set_planes(self, planes_lpd: torch.Tensor) -> None:
        assert tuple(planes_lpd.shape[:2]) == (self.L, self.P)
        self.planes_words = permute_planes(planes_lpd.to(self.k_cache.device))

    @torch.no_grad()
    def append(self, pos0: int, k_bshd: torch.Tensor, v_bshd: torch.Tensor) -> None:
        """Write S new tokens at positions [pos0, pos0+S) for every sequence:
        K/V rows, packed codes and value norms (KVCache.update,
        GPT-FAST/model.py:187-229, with the hashing of :449-450 folded in)."""
        assert self.planes_words is not None, "call set_planes() first"
        B, S, H, D = k_bshd.shape
        assert B == self.k_cache.shape[0], "append expects the cache's full batch"
        if pos0 < 0 or pos0 + S > self.Tcap:
            raise RuntimeError(
                f"KVCache.update out-of-bounds: positions [{pos0},{pos0 + S - 1}] but cache T={self.Tcap}")
        self.k_cache[:, :, pos0:pos0 + S].copy_(k_bshd.permute(0, 2, 1, 3))
        self.v_cache[:, :, pos0:pos0 + S].copy_(v_bshd.permute(0, 2, 1, 3))
        hash_keys_into(self.k_cache[:, :, pos0:pos0 + S], self.v_cache[:, :, pos0:pos0 + S],
                       self.planes_words, self.codes, self.v_norm, self.L, self.P, t0=pos0)
        self.lens.fill_(pos0 + S)      # the cached length follows the position
