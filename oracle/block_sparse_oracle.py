"""CPU restatement of the reference's block-sparse prefill attention.  TEST INFRASTRUCTURE ONLY.

Imported by the test-suite only; nothing in the shipped package uses it.  Plain
Python loops over lists (index builders) and float64 torch arithmetic
(attention), written to follow the reference statement by statement (citations
are paths relative to the reference checkout):

  random_walk_indices                   kernels/block_sparse_flash_attention.py:11-136
  random_walk_indices_from_block_probs  kernels/block_sparse_flash_attention.py:139-222
  block_mask_to_indices                 kernels/block_sparse_flash_attention.py:232-274
  block_sparse_attention                kernels/block_sparse_flash_attention.py:280-367 (random_walk_fwd)
                                        and :370-437 (zero padding to whole blocks)

Pinning (tests/test_block_sparse.py): the builders' outputs are checked against
the properties their docstring promises (valid ids, causal, diagonal present,
sorted, fixed length) and against hand-worked cases; the attention against a
dense masked softmax wherever the listed blocks have no repeats, and against the
doubling of a block's weight where one is listed twice.  The one library call
whose behaviour is not pinned by the reference is torch.topk on tied scores; the
tests use scores without ties.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch


def _finish(forced_rows: List[List[int]], fill_rows: List[List[int]], k_eff: int, diag: Optional[List[int]],
            num_cols: int) -> List[List[int]]:
    """Lines :103-136 / :197-222 for one batch entry: pad the forced lists to a common
    length with 0, append the fill, sort, overwrite repeats with 0, sort, cut, put the
    diagonal first, clamp, sort."""
    max_f = max((len(f) for f in forced_rows), default=0)
    out = []
    for r, (forced, fill) in enumerate(zip(forced_rows, fill_rows)):
        cat = sorted(list(forced) + [0] * (max_f - len(forced)) + list(fill))
        dedup = [cat[0]] + [0 if cat[i] == cat[i - 1] else cat[i] for i in range(1, len(cat))] if cat else []
        cut = sorted(dedup)[:k_eff]
        if diag is not None and cut:
            cut[0] = diag[r]
        cut = [min(max(c, 0), num_cols - 1) for c in cut]
        out.append(sorted(cut))
    return out


def _select(scores, valid, forced, K: int, diag):
    """scores [B][R][C] floats; valid/forced [R][C] bools."""
    B, R, C = len(scores), len(valid), len(valid[0]) if valid else 0
    k_eff = min(K, C)
    result = []
    for b in range(B):
        fill_rows, forced_rows = [], []
        for r in range(R):
            s = [scores[b][r][c] + 1e-6 * (c / max(1, C)) for c in range(C)]
            pool = [s[c] if (valid[r][c] and not forced[r][c]) else -math.inf for c in range(C)]
            order = sorted(range(C), key=lambda c: -pool[c])[:k_eff]          # top-k (no ties in the tests)
            fill_rows.append([0 if pool[c] == -math.inf else c for c in order])
            forced_rows.append([c for c in range(C) if forced[r][c]])
        result.append(_finish(forced_rows, fill_rows, k_eff, diag, C))
    return torch.tensor(result, dtype=torch.int32).reshape(B, R, k_eff)


def random_walk_indices(probs: torch.Tensor, block_m: int, block_n: int, K: int, enforce_causal_blocks: bool = True,
                        force_include_diagonal: bool = True, window_blocks: Optional[int] = None) -> torch.Tensor:
    B, T_q, T_k = probs.shape
    R, C = -(-T_q // block_m), -(-T_k // block_n)
    p = probs.double()
    scores = [[[float(p[b, r * block_m:(r + 1) * block_m, c * block_n:(c + 1) * block_n].sum()) for c in range(C)]
               for r in range(R)] for b in range(B)]
    valid, forced, diag = [], [], []
    for r in range(R):
        q_last = min((r + 1) * block_m - 1, T_q - 1)
        max_kblk = q_last // block_n
        valid.append([(c <= max_kblk) if enforce_causal_blocks else True for c in range(C)])
        d = (r * block_m) // block_n
        diag.append(min(max(d, 0), C - 1))
        f = [False] * C
        if force_include_diagonal:
            f[diag[r]] = True
        if window_blocks is not None and window_blocks > 0:
            for c in range(C):
                if d - (window_blocks - 1) <= c <= d:
                    f[c] = True
        f = [f[c] and valid[r][c] for c in range(C)]
        f[0] = valid[r][0]
        forced.append(f)
    return _select(scores, valid, forced, K, diag if force_include_diagonal else None)


def random_walk_indices_from_block_probs(block_probs: torch.Tensor, K: int, enforce_causal_blocks: bool = True,
                                         force_include_diagonal: bool = True,
                                         window_blocks: Optional[int] = None) -> torch.Tensor:
    B, R, C = block_probs.shape
    scores = block_probs.double().tolist()
    valid, forced, diag = [], [], []
    for r in range(R):
        valid.append([(c <= min(r, C - 1)) if enforce_causal_blocks else True for c in range(C)])
        diag.append(min(max(r, 0), C - 1))
        f = [False] * C
        if force_include_diagonal:
            f[diag[r]] = True
        if window_blocks is not None and window_blocks > 0:
            for c in range(C):
                if r - (window_blocks - 1) <= c <= r:
                    f[c] = True
        f = [f[c] and valid[r][c] for c in range(C)]
        f[0] = valid[r][0]
        forced.append(f)
    return _select(scores, valid, forced, K, diag if force_include_diagonal else None)


def block_mask_to_indices(allow: torch.Tensor, block_m: int, block_n: int, K: Optional[int] = None,
                          force_include_diagonal: bool = True, enforce_causal_blocks: bool = True) -> torch.Tensor:
    B, R, C = allow.shape
    rows = []
    for b in range(B):
        per_row = []
        for r in range(R):
            q_last = min((r + 1) * block_m - 1, R * block_m - 1)
            m = [bool(allow[b, r, c]) and ((c <= q_last // block_n) or not enforce_causal_blocks) for c in range(C)]
            if force_include_diagonal:
                m[min(max((r * block_m) // block_n, 0), C - 1)] = True
            per_row.append([c for c in range(C) if m[c]])
        rows.append(per_row)
    longest = max((len(x) for per_row in rows for x in per_row), default=0)
    k_eff = max(1, min(longest if (K is None or K <= 0) else K, C))
    out = [[(x + [0] * k_eff)[:k_eff] for x in per_row] for per_row in rows]
    return torch.tensor(out, dtype=torch.int32).reshape(B, R, k_eff)


def block_sparse_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, seqlens: torch.Tensor,
                           block_index: torch.Tensor, block: int = 64) -> torch.Tensor:
    """float64 [B,H,T,D]; rows at or past seqlens[b] are NaN (the kernel does not write them).
    The listed blocks are walked in order with the reference's running maximum; a
    block listed twice enters the sums twice."""
    B, H, T, D = q.shape
    qd, kd, vd = q.double(), k.double(), v.double()
    scale = (D ** -0.5) * 1.44269504
    out = torch.full((B, H, T, D), float("nan"), dtype=torch.float64)
    for b in range(B):
        n = int(seqlens[b])
        for h in range(H):
            for rb in range(-(-T // block)):
                r0 = rb * block
                if r0 >= n:
                    continue
                rows = torch.arange(r0, min(r0 + block, T))
                qr = qd[b, h, rows] * scale                                         # [m,D]
                m_i = torch.full((len(rows),), -math.inf, dtype=torch.float64)
                l_i = torch.zeros(len(rows), dtype=torch.float64)
                acc = torch.zeros(len(rows), D, dtype=torch.float64)
                for blk in block_index[b, h, rb].tolist():
                    cols = torch.arange(blk * block, (blk + 1) * block)
                    inside = cols < min(n, T)
                    kk = torch.zeros(block, D, dtype=torch.float64)
                    vv = torch.zeros(block, D, dtype=torch.float64)
                    kk[inside] = kd[b, h, cols[inside]]
                    vv[inside] = vd[b, h, cols[inside]]
                    s = qr @ kk.T
                    ok = (rows[:, None] < n) & (cols[None, :] <= rows[:, None])
                    s = torch.where(ok, s, torch.full_like(s, -math.inf))
                    m_new = torch.maximum(m_i, s.max(dim=1).values)
                    safe = torch.where(torch.isinf(m_new), torch.zeros_like(m_new), m_new)   # rows with nothing visible yet
                    alpha = torch.where(torch.isinf(m_new), torch.ones_like(m_new), torch.exp2(m_i - safe))
                    p = torch.where(torch.isinf(m_new)[:, None], torch.zeros_like(s), torch.exp2(s - safe[:, None]))
                    acc = acc * alpha[:, None] + p @ vv
                    l_i = l_i * alpha + p.sum(dim=1)
                    m_i = m_new
                res = acc / (l_i[:, None] + 1e-9)
                live = rows < n
                out[b, h, rows[live]] = res[live]
    return out
