"""Block-sparse prefill attention with "random walk" block selection.

Counterpart of kernels/block_sparse_flash_attention.py (index builders :11-274,
Triton kernel `random_walk_fwd` :280-367, launcher :370-437, convenience wrapper
:440-453) with the same function names, arguments and results.  The index
builders are host-side tensor logic and stay in torch; the attention itself is
one HIP kernel of libsocket_hip (`socket_block_sparse_attention`) -- there is no
other route, a missing library raises.

How a block list comes about (both builders): every row block has a set of
*forced* key blocks (block 0, the diagonal, an optional window behind the
diagonal; all causal) and fills up with the best-scoring other causal blocks.
The reference then de-duplicates by sorting, overwriting repeats with 0, sorting
again, cutting to K entries, putting the diagonal into the first slot and sorting
once more.  Because block 0 is always forced, that pipeline has a closed form,
which is what is computed here: with U the distinct chosen blocks of a row and
n = (largest forced count of any row) + K, the list is

    diagonal,  min(K, n - |U| + 1) - 1 zeros,  the K - min(K, n - |U| + 1) smallest non-zero members of U

sorted ascending (tests check it against a literal restatement of the pipeline).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from ._lib import check, dtype_enum, lib, ptr, stream_ptr

__all__ = [
    "random_walk_indices", "random_walk_indices_from_block_probs", "expand_block_index_to_heads",
    "block_mask_to_indices", "random_walk_sparse_attention", "build_and_run_rw_sparse_attn",
]


def _assemble(scores: torch.Tensor, valid: torch.Tensor, forced: torch.Tensor, K: int,
              diag: Optional[torch.Tensor]) -> torch.Tensor:
    """scores [B,R,C] float, valid/forced [R,C] bool (forced within valid, column 0 forced) -> int32 [B,R,min(K,C)]."""
    B, R, C = scores.shape
    device = scores.device
    k_eff = min(K, C)
    cols = torch.arange(C, device=device)
    # flat scores: prefer recent blocks (kernels/block_sparse_flash_attention.py:77-79)
    s = scores + 1e-6 * (cols.to(scores.dtype) / max(1, C))[None, None, :]
    pool = s.masked_fill((~valid | forced).unsqueeze(0), float("-inf"))
    top = torch.topk(pool, k_eff, dim=-1)
    fill = torch.where(top.values.isneginf(), torch.zeros_like(top.indices), top.indices)    # too few candidates: block 0
    member = forced.unsqueeze(0).expand(B, R, C).clone()
    member.scatter_(-1, fill, True)
    n_slots = int(forced.sum(-1).max()) + k_eff if R > 0 else k_eff
    distinct = member.sum(-1)                                                                 # |U|, >= 1 (block 0)
    zeros = torch.clamp(n_slots - distinct + 1, max=k_eff)                                    # zeros among the first K slots
    nonzero = member.clone()
    nonzero[..., 0] = False
    keep = nonzero & (nonzero.cumsum(-1) <= (k_eff - zeros).unsqueeze(-1))
    ids = torch.where(keep, cols.expand(B, R, C), torch.full((), C, device=device, dtype=cols.dtype))
    out = torch.sort(ids, dim=-1).values[..., :k_eff]
    out = torch.where(out >= C, torch.zeros_like(out), out)                                   # the zeros come last here
    if diag is not None:
        out[..., -1] = diag.view(1, R).expand(B, R)                                           # one zero makes way for the diagonal
    out = out.clamp_(0, C - 1)
    return torch.sort(out, dim=-1).values.to(torch.int32)


@torch.no_grad()
def random_walk_indices(random_walk_probs: torch.Tensor, block_m: int, block_n: int, K: int,
                        q_quantile: float = 0.8, enforce_causal_blocks: bool = True,
                        force_include_diagonal: bool = True,
                        window_blocks: Optional[int] = None) -> torch.Tensor:
    """Token-level probabilities [B,T_q,T_k] -> block lists int32 [B, ceil(T_q/block_m), min(K, ceil(T_k/block_n))]:
    always valid ids, causal, diagonal included, sorted
    (kernels/block_sparse_flash_attention.py:11-136; `q_quantile` is unused there too)."""
    assert random_walk_probs.dim() == 3
    B, T_q, T_k = random_walk_probs.shape
    assert block_m > 0 and block_n > 0
    assert K > 0
    device = random_walk_probs.device
    R, C = -(-T_q // block_m), -(-T_k // block_n)
    x = F.pad(random_walk_probs, (0, C * block_n - T_k, 0, R * block_m - T_q))
    scores = x.view(B, R, block_m, C, block_n).sum(dim=(2, 4))
    rows = torch.arange(R, device=device)
    cols = torch.arange(C, device=device)
    if enforce_causal_blocks:
        q_last = torch.clamp((rows + 1) * block_m - 1, max=T_q - 1)      # last query token of the row block
        valid = cols[None, :] <= (q_last // block_n)[:, None]
    else:
        valid = torch.ones((R, C), dtype=torch.bool, device=device)
    diag = ((rows * block_m) // block_n).clamp(0, C - 1)
    forced = torch.zeros((R, C), dtype=torch.bool, device=device)
    if force_include_diagonal:
        forced |= cols[None, :] == diag[:, None]
    if window_blocks is not None and window_blocks > 0:
        d = ((rows * block_m) // block_n)[:, None]
        forced |= (cols[None, :] <= d) & (cols[None, :] >= d - (window_blocks - 1))
    forced &= valid
    forced[:, 0] = True
    forced &= valid
    return _assemble(scores, valid, forced, K, diag if force_include_diagonal else None)


@torch.no_grad()
def random_walk_indices_from_block_probs(random_walk_probs_blk: torch.Tensor, K: int, q_quantile: float = 0.8,
                                         enforce_causal_blocks: bool = True,
                                         force_include_diagonal: bool = True,
                                         window_blocks: Optional[int] = None) -> torch.Tensor:
    """The same from block-level scores [B,Tb_q,Tb_k] (kernels/block_sparse_flash_attention.py:139-222)."""
    assert random_walk_probs_blk.dim() == 3
    B, R, C = random_walk_probs_blk.shape
    assert K > 0
    device = random_walk_probs_blk.device
    rows = torch.arange(R, device=device)
    cols = torch.arange(C, device=device)
    if enforce_causal_blocks:
        valid = cols[None, :] <= torch.clamp(rows, max=C - 1)[:, None]
    else:
        valid = torch.ones((R, C), dtype=torch.bool, device=device)
    diag = rows.clamp(0, C - 1)
    forced = torch.zeros((R, C), dtype=torch.bool, device=device)
    if force_include_diagonal:
        forced |= cols[None, :] == diag[:, None]
    if window_blocks is not None and window_blocks > 0:
        d = rows[:, None]
        forced |= (cols[None, :] <= d) & (cols[None, :] >= d - (window_blocks - 1))
    forced &= valid
    forced[:, 0] = True
    forced &= valid
    return _assemble(random_walk_probs_blk, valid, forced, K, diag if force_include_diagonal else None)


@torch.no_grad()
def expand_block_index_to_heads(block_index_brk: torch.Tensor, H: int) -> torch.Tensor:
    """[B,R,K] -> int32 [B,H,R,K], contiguous (kernels/block_sparse_flash_attention.py:225-229)."""
    assert block_index_brk.dtype in (torch.int32, torch.int64)
    B, R, K = block_index_brk.shape
    return block_index_brk[:, None].expand(B, H, R, K).contiguous().to(torch.int32)


@torch.no_grad()
def block_mask_to_indices(allow_blocks: torch.Tensor, block_m: int, block_n: int, K: Optional[int] = None,
                          force_include_diagonal: bool = True, enforce_causal_blocks: bool = True) -> torch.Tensor:
    """Block mask bool [B,R,C] -> ascending lists of the allowed blocks, cut or
    padded (with block 0) to K entries; K None / <= 0: the longest row
    (kernels/block_sparse_flash_attention.py:232-274)."""
    assert allow_blocks.dim() == 3
    assert allow_blocks.dtype == torch.bool
    assert block_m > 0 and block_n > 0
    B, R, C = allow_blocks.shape
    device = allow_blocks.device
    rows = torch.arange(R, device=device)
    cols = torch.arange(C, device=device)
    mask = allow_blocks
    if enforce_causal_blocks:
        q_last = torch.clamp((rows + 1) * block_m - 1, max=R * block_m - 1)
        mask = mask & (cols[None, :] <= (q_last // block_n)[:, None]).unsqueeze(0)
    if force_include_diagonal:
        diag = ((rows * block_m) // block_n).clamp(0, C - 1)
        mask = mask | (cols[None, :] == diag[:, None]).unsqueeze(0)
    if K is None or K <= 0:
        k_eff = int(mask.sum(dim=-1).max().item()) if C > 0 else 0
    else:
        k_eff = K
    k_eff = max(1, min(k_eff, C))
    ids = torch.where(mask, cols.expand(B, R, C), torch.full((), C, device=device, dtype=cols.dtype))
    out = torch.sort(ids, dim=-1).values[..., :k_eff]
    return torch.where(out >= C, torch.zeros_like(out), out).to(torch.int32)


@torch.no_grad()
def random_walk_sparse_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seqlens: torch.Tensor,
                                 block_index: torch.Tensor, block_m: int = 64, block_n: int = 64) -> torch.Tensor:
    """q, k, v [B,H,T,D] fp16/bf16, seqlens int32 [B], block_index int32
    [B,H,ceil(T/64),K] without -1 entries -> out [B,H,T,D]
    (kernels/block_sparse_flash_attention.py:370-437).  Rows at or past
    seqlens[b] come back as zeros (the reference leaves them uninitialised)."""
    assert q.is_cuda and k.is_cuda and v.is_cuda
    assert q.dtype in (torch.float16, torch.bfloat16)
    assert q.shape == k.shape == v.shape
    B, H, T, D = q.shape
    assert D in (16, 32, 64, 128)
    assert block_index.dtype == torch.int32
    if block_m != 64 or block_n != 64:
        raise RuntimeError("socket_block_sparse_attention supports 64 x 64 blocks only")
    num_rows = -(-T // block_m)
    assert tuple(block_index.shape[:3]) == (B, H, num_rows), "block_index must be [B,H,ceil(T/block_m),K]"
    assert seqlens.is_cuda and seqlens.dtype == torch.int32 and seqlens.numel() == B
    q, k, v = (t if t.stride(-1) == 1 else t.contiguous() for t in (q, k, v))
    block_index = block_index.contiguous()
    seqlens = seqlens.contiguous()
    out = torch.zeros((B, H, T, D), dtype=q.dtype, device=q.device)
    check("socket_block_sparse_attention", lib().socket_block_sparse_attention(
        ptr(q), ptr(k), ptr(v), dtype_enum(q.dtype),
        q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
        v.stride(0), v.stride(1), v.stride(2), ptr(seqlens), ptr(block_index), ptr(out),
        out.stride(0), out.stride(1), out.stride(2), B, H, T, D, num_rows, block_index.shape[3],
        int(block_m), int(block_n), stream_ptr(q.device)))
    return out


def build_and_run_rw_sparse_attn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, random_walk_probs: torch.Tensor,
                                 block_size: int = 64, Kblocks: int = 8, q_quantile: float = 0.8,
                                 window_blocks: Optional[int] = 4) -> torch.Tensor:
    """Index building + attention in one call (kernels/block_sparse_flash_attention.py:440-453)."""
    B, H, T, D = q.shape
    seqlens = torch.full((B,), T, device=q.device, dtype=torch.int32)
    blocks = random_walk_indices(random_walk_probs, block_size, block_size, Kblocks, q_quantile=q_quantile,
                                 enforce_causal_blocks=True, force_include_diagonal=True,
                                 window_blocks=window_blocks)
    return random_walk_sparse_attention(q, k, v, seqlens, expand_block_index_to_heads(blocks, H),
                                        block_m=block_size, block_n=block_size)
