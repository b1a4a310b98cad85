"""Host wrappers of the decode-step helper kernels (rotary + cache append,
residual + RMSNorm, SiLU-multiply): each stands for a chain of elementwise torch
launches in GPT-FAST/model.py's decode step and rounds exactly where that chain
rounds."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ._lib import check, dtype_enum, lib, ptr, stream_ptr


@torch.no_grad()
def rope_append(qkv: torch.Tensor, freqs_cis: torch.Tensor, input_pos: torch.Tensor, k_cache: torch.Tensor,
                v_cache: torch.Tensor, lens: Optional[torch.Tensor], n_heads: int, n_kv_heads: int,
                return_new: bool = False):
    """qkv [B,1,(Hq+2Hkv)*D] or [B,(Hq+2Hkv)*D] -> rotated queries [B,Hq,D]; the
    rotated key and the value are written into the caches [B,Hkv,Tcap,D] at
    input_pos (int64 on the device, one element or one per sequence) and `lens`
    is raised (GPT-FAST/model.py:433-451 for one new token, without the hash).
    return_new=True also returns the rotated key and the value as [B,1,Hkv,D]."""
    assert qkv.is_cuda and qkv.stride(-1) == 1
    B = qkv.shape[0]
    q2 = qkv.reshape(B, -1)
    D = k_cache.shape[-1]
    assert q2.shape[1] == (n_heads + 2 * n_kv_heads) * D and k_cache.shape == v_cache.shape
    assert k_cache.stride(-1) == 1 and v_cache.stride() == k_cache.stride() and k_cache.dtype == qkv.dtype
    assert input_pos.dtype == torch.int64 and input_pos.is_cuda and input_pos.numel() in (1, B)
    assert freqs_cis.is_contiguous() and freqs_cis.shape[1:] == (D // 2, 2)
    if lens is not None:
        assert lens.dtype == torch.int32 and lens.numel() == B
    q_out = torch.empty((B, n_heads, D), dtype=qkv.dtype, device=qkv.device)
    k_new = v_new = None
    if return_new:
        k_new = torch.empty((B, 1, n_kv_heads, D), dtype=qkv.dtype, device=qkv.device)
        v_new = torch.empty_like(k_new)
    check("socket_rope_append", lib().socket_rope_append(
        ptr(q2), dtype_enum(qkv.dtype), q2.stride(0), ptr(freqs_cis), dtype_enum(freqs_cis.dtype),
        freqs_cis.shape[0], ptr(input_pos), 0 if input_pos.numel() == 1 else 1, ptr(q_out), ptr(k_cache),
        ptr(v_cache), k_cache.stride(0), k_cache.stride(1), k_cache.stride(2), ptr(lens), ptr(k_new), ptr(v_new),
        B, n_heads, n_kv_heads, D, k_cache.shape[2], stream_ptr(qkv.device)))
    if return_new:
        return q_out, k_new, v_new
    return q_out


@torch.no_grad()
def add_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float,
                residual: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(h, y): h = x + residual (x itself without a residual), y = RMSNorm(h) * weight
    (GPT-FAST/model.py:603-614)."""
    assert x.is_cuda and x.is_contiguous() and weight.dtype == x.dtype and weight.is_contiguous()
    dim = x.shape[-1]
    rows = x.numel() // dim
    y = torch.empty_like(x)
    h = x
    if residual is not None:
        assert residual.shape == x.shape and residual.dtype == x.dtype and residual.is_contiguous()
        h = torch.empty_like(x)
    check("socket_add_rmsnorm", lib().socket_add_rmsnorm(
        ptr(x), ptr(residual), ptr(weight), ptr(h) if residual is not None else None, ptr(y), dtype_enum(x.dtype),
        rows, dim, float(eps), stream_ptr(x.device)))
    return h, y


@torch.no_grad()
def silu_mul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """silu(a) * b (GPT-FAST/model.py:599-600)."""
    assert a.is_cuda and a.is_contiguous() and b.is_contiguous() and a.shape == b.shape and a.dtype == b.dtype
    out = torch.empty_like(a)
    check("socket_silu_mul", lib().socket_silu_mul(ptr(a), ptr(b), ptr(out), dtype_enum(a.dtype), a.numel(),
                                                   stream_ptr(a.device)))
    return out


@torch.no_grad()
def linear_rows(x: torch.Tensor, weight: torch.Tensor, gate_weight: torch.Tensor = None) -> torch.Tensor:
    """x @ weight.T for the few rows of a decode step (nn.Linear without bias,
    GPT-FAST/model.py:436, :476), or with `gate_weight` silu(x @ weight.T) * (x @ gate_weight.T)
    (FeedForward, :599-600) in one pass over both matrices.  Shapes the
    matrix-vector kernel does not take go to torch's own product."""
    rows = x.numel() // x.shape[-1]
    K, N = x.shape[-1], weight.shape[0]
    # measured against torch's product: ahead for one row (and, gated, up to four); behind for more
    fits = (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
            and rows <= (1 if gate_weight is None else 4)
            and K % 2048 == 0 and weight.is_contiguous() and x.is_contiguous()
            and (gate_weight is None or (gate_weight.is_contiguous() and gate_weight.shape == weight.shape
                                         and gate_weight.dtype == torch.bfloat16)))
    if not fits:
        y = torch.nn.functional.linear(x, weight)
        return y if gate_weight is None else silu_mul(y, torch.nn.functional.linear(x, gate_weight))
    y = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
    check("socket_gemv_bf16", lib().socket_gemv_bf16(ptr(x), K, ptr(weight), ptr(gate_weight),
                                                     ptr(y), N, rows, N, K, stream_ptr(x.device)))
    return y


@torch.no_grad()
def norm_linear_rows(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor],
                     weight: torch.Tensor, gate_weight: torch.Tensor = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(h, y) with h, xn = add_rmsnorm(x, norm_weight, eps, residual) and y = linear_rows(xn,
    weight, gate_weight): one launch where the matrix-vector kernel takes the shape (every
    workgroup normalises the row for itself; same values bit for bit), the two calls otherwise."""
    rows = x.numel() // x.shape[-1]
    K, N = x.shape[-1], weight.shape[0]
    fits = (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
            and norm_weight.dtype == torch.bfloat16 and norm_weight.is_contiguous()
            and rows <= (1 if gate_weight is None else 4)
            and K % 2048 == 0 and K <= 8192 and weight.is_contiguous() and x.is_contiguous()
            and (residual is None or (residual.shape == x.shape and residual.dtype == x.dtype
                                      and residual.is_contiguous()))
            and (gate_weight is None or (gate_weight.is_contiguous() and gate_weight.shape == weight.shape
                                         and gate_weight.dtype == torch.bfloat16)))
    if not fits:
        h, xn = add_rmsnorm(x, norm_weight, eps, residual=residual)
        return h, linear_rows(xn, weight, gate_weight)
    h = x if residual is None else torch.empty_like(x)
    y = torch.empty(*x.shape[:-1], N, dtype=x.dtype, device=x.device)
    check("socket_norm_gemv_bf16", lib().socket_norm_gemv_bf16(
        ptr(x), ptr(residual), ptr(norm_weight), float(eps), ptr(h) if residual is not None else None,
        ptr(weight), ptr(gate_weight), ptr(y), rows, N, K, stream_ptr(x.device)))
    return h, y

