"""Index-list builder with the reference's signature, plus the sparse
flash-decode entry points re-exported as the reference's module does
(GPT-FAST/kernels/sparse.py holds both: `build_sparse_list_decode` at :16-95 and
a copy of the decode kernels at :98-329).

`build_sparse_list_decode` takes the reference's operand layout (int16 codes per
query head, [B,H,L,T]) and returns the same `(sparse_list, sparse_len)`.  The
scorer and the top-k + list assembly are HIP kernels; heavy entries are in
descending score order with equal scores ordered by ascending index.  For the
layout the HIP path is designed around (packed codes per KV head, no relayout),
use `socket_amd.hash_cache`.
"""
from __future__ import annotations

import collections

import torch

from ._lib import SOCKET_TOPK_MAX_M, check, lib, ptr, stream_ptr
from .socket_kernels import (  # noqa: F401  (re-exported, as in the reference module)
    attention_mask_to_allowed_prob,
    sparse_attention_fwd,
    sparse_decode_stage1,
    sparse_decode_stage2,
)

_SOFT_HASH_EXT = None


def _get_soft_hash_ext():
    global _SOFT_HASH_EXT
    if _SOFT_HASH_EXT is None:
        from .soft_hash_collision_loader import load_soft_hash_collision
        _SOFT_HASH_EXT = load_soft_hash_collision(3)
    return _SOFT_HASH_EXT


# Workspaces of the selection.  The kernel wants the arrival counters at a workspace's
# head zero on entry and leaves them zero, so a workspace is zeroed once, when it is made,
# and serves every later call that cannot overlap with another user of it:
#   * eager calls: one per (device, stream, size) -- calls on one stream are ordered;
#   * calls recorded into a HIP graph: one per (device, size), made and zeroed OUTSIDE the
#     capture by the eager call of the same shape that precedes any capture (a buffer made
#     during a capture would live in that graph's private pool, be zeroed only by a
#     recorded node, and outlive the graph in this table).  Replays of graphs that hold a
#     decode step must not overlap on one GPU (hash_cache.sparse_decode_step), which is
#     what lets them share it.
# The table is bounded: the least recently used entries are dropped beyond _SELECT_WS_MAX.
_SELECT_WS = collections.OrderedDict()
_SELECT_WS_MAX = 32


def _new_workspace(device: torch.device, nbytes: int, zero_bytes: int) -> torch.Tensor:
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    ws[:zero_bytes].zero_()
    return ws


def _select_workspace(device: torch.device, nbytes: int, zero_bytes: int) -> torch.Tensor:
    capturing = torch.cuda.is_current_stream_capturing()
    graph_key = (device.index, None, nbytes)
    if capturing:
        ws = _SELECT_WS.get(graph_key)
        if ws is None:
            # no eager call of this shape came first: a buffer of this capture's own, zeroed by a
            # recorded node on every replay, and not kept here
            return _new_workspace(device, nbytes, zero_bytes)
        _SELECT_WS.move_to_end(graph_key)
        return ws[0]
    key = (device.index, torch.cuda.current_stream(device).cuda_stream, nbytes)
    for k in (key, graph_key):
        if k not in _SELECT_WS:
            _SELECT_WS[k] = (_new_workspace(device, nbytes, zero_bytes), zero_bytes)
        _SELECT_WS.move_to_end(k)
    while len(_SELECT_WS) > _SELECT_WS_MAX:
        _SELECT_WS.popitem(last=False)
    return _SELECT_WS[key][0]


def reset_select_workspaces() -> None:
    """Zero the arrival counters of every cached workspace again.  A selection that
    was aborted mid-launch (a device error) can leave them counting; `select_list`
    calls this when the library reports a failure, and a caller who tore down a
    stream with work in flight should too."""
    if torch.cuda.is_current_stream_capturing():
        return
    for ws, zero_bytes in _SELECT_WS.values():
        ws[:zero_bytes].zero_()


def select_list(scores: torch.Tensor, sink: int, window: int, M: int, *, lens=None, budgets=None,
                write_base: bool = True, list_width=None, row_range=None, split: bool = True):
    """Top-M + [sink | window | heavy] assembly on fp32 score rows [B,H,T]
    (row pitch = scores.stride(1)).  Returns (sparse_list int32 [B,H,width],
    sparse_len int32 [B,H]).  `lens`/`budgets`: optional int32 [B] device tensors
    (per-sequence context length and top-k budget).  `row_range`: the int32
    [B,H,parts,2] key ranges `hash_cache.score_packed(..., with_range=True)`
    returns for these scores (saves the kernel's first pass).  `split=False`
    keeps every row to one workgroup (the result is the same)."""
    assert scores.is_cuda and scores.dtype == torch.float32 and scores.dim() == 3
    assert scores.stride(2) == 1 and scores.stride(0) == scores.shape[1] * scores.stride(1)
    B, H, T = scores.shape
    M = int(M)
    if M > SOCKET_TOPK_MAX_M:
        raise RuntimeError(f"top-k budget {M} exceeds the supported maximum {SOCKET_TOPK_MAX_M}")
    if list_width is None:
        s_e, w_e = max(0, min(sink, T)), max(0, min(window, T))
        nbase = 0
        if write_base:
            nbase = s_e + (T - max(T - w_e, s_e) if w_e > 0 else 0)
            nbase = max(nbase, 1)
        list_width = nbase + min(M, T)
    sparse_list = torch.empty((B, H, list_width), dtype=torch.int32, device=scores.device)
    sparse_len = torch.empty((B, H), dtype=torch.int32, device=scores.device)
    if list_width == 0:
        return sparse_list, sparse_len.zero_()
    L = lib()
    ws, ws_bytes = None, L.socket_select_workspace_bytes(B, H, T, M) if split else 0
    if ws_bytes:
        ws = _select_workspace(scores.device, ws_bytes, L.socket_select_workspace_zero_bytes(B, H, T, M))
    try:
        check("socket_select_list", L.socket_select_list(
            ptr(scores), scores.stride(1), ptr(lens), ptr(budgets), ptr(row_range),
            0 if row_range is None else row_range.shape[2], B, H, T, M, int(sink), int(window),
            1 if write_base else 0, ptr(sparse_list), list_width, list_width, ptr(sparse_len),
            ptr(ws), ws_bytes, stream_ptr(scores.device)))
    except RuntimeError:
        if ws is not None:
            reset_select_workspaces()
        raise
    return sparse_list, sparse_len


@torch.no_grad()
def build_sparse_list_decode(
    q_probs: torch.Tensor,       # [B,H,L,R] fp16/bf16/fp32
    k_hard_bhlt: torch.Tensor,   # [B,H,L,T] int16/int32
    v_norm_bht: torch.Tensor,    # [B,H,T] fp16/bf16/fp32
    allowed_bht: torch.Tensor,   # [B,H,T] bool
    sink: int,
    window: int,
    M: int,
    KC: int = 8,
    BLOCK_N: int = 512,
    num_warps: int = 8,
    num_stages: int = 2,
):
    """GPT-FAST/kernels/sparse.py:16-95.  KC, BLOCK_N, num_warps, num_stages are
    accepted and ignored, as in the reference (:38)."""
    assert q_probs.is_cuda and k_hard_bhlt.is_cuda and v_norm_bht.is_cuda and allowed_bht.is_cuda
    assert q_probs.dtype in (torch.float16, torch.bfloat16, torch.float32)
    assert allowed_bht.dtype == torch.bool
    B, H, L, R = q_probs.shape
    _, _, L2, T = k_hard_bhlt.shape
    assert L2 == L
    device = q_probs.device
    M_eff = min(M, T)
    if M_eff > 0:
        ext = _get_soft_hash_ext()
        q_probs_f32 = q_probs.float().unsqueeze(2).contiguous()
        key_buckets = k_hard_bhlt if k_hard_bhlt.dtype == torch.int16 else k_hard_bhlt.to(torch.int16)
        key_buckets = key_buckets.contiguous()
        allowed_ext = allowed_bht.unsqueeze(2).contiguous()
        v_hist = v_norm_bht.float().unsqueeze(2).contiguous()
        scores = ext.soft_hash_collision(q_probs_f32, key_buckets, allowed_ext, v_hist).squeeze(2)
        heavy_idx, _ = select_list(scores, 0, 0, M_eff, write_base=False)
        # disallowed positions carry -inf and may still be selected when fewer
        # than M_eff positions are allowed: they become -1 (:62-68)
        ok = torch.gather(allowed_bht, -1, heavy_idx.clamp(0, T - 1).long())
        heavy_idx = heavy_idx.masked_fill(~ok, -1)
    else:
        heavy_idx = torch.empty((B, H, 0), device=device, dtype=torch.int32)

    sink = max(0, min(sink, T))
    window = max(0, min(window, T))
    parts = []
    if sink > 0:
        parts.append(torch.arange(sink, device=device, dtype=torch.int32))
    if window > 0:
        win_start = max(T - window, sink)
        if win_start < T:
            parts.append(torch.arange(win_start, T, device=device, dtype=torch.int32))
    base = torch.cat(parts, dim=0) if parts else torch.tensor([T - 1], device=device, dtype=torch.int32)
    base = base.view(1, 1, -1).expand(B, H, -1)
    base_ok = torch.gather(allowed_bht, -1, base.long())
    base = base.masked_fill(~base_ok, -1)

    sparse_list = torch.cat([base, heavy_idx], dim=-1).contiguous()
    sparse_len = torch.full((B, H), sparse_list.shape[-1], device=device, dtype=torch.int32)
    return sparse_list, sparse_len
