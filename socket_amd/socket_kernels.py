"""Sparse flash-decode: the Python API of the reference's
kernels/socket_triton_kernels.py (and of the copy in GPT-FAST/kernels/sparse.py),
served by the HIP kernels in csrc/attend.hip through the C ABI.

Same names, argument order and meaning as the reference:
  attention_mask_to_allowed_prob   kernels/socket_triton_kernels.py:9-25
  sparse_decode_stage1             kernels/socket_triton_kernels.py:167-205
  sparse_decode_stage2             kernels/socket_triton_kernels.py:208-235
  sparse_attention_fwd             kernels/socket_triton_kernels.py:238-258
Shape/device violations raise AssertionError as the reference's asserts do;
anything the library rejects raises RuntimeError (SocketHipError).
"""
from __future__ import annotations

import ctypes
import functools

import torch

from . import _lib
from ._lib import check, dtype_enum, lib, ptr, stream_ptr


def attention_mask_to_allowed_prob(attention_mask: torch.Tensor, K: int) -> torch.Tensor:
    """bool mask (True = forbidden) or additive mask (>= 0 = allowed) -> float32
    {0,1} of shape [B,1,*,K] (kernels/socket_triton_kernels.py:9-25)."""
    am = attention_mask[..., :K]
    if am.dtype == torch.bool:
        allowed = (am == 0).to(torch.float32)
    else:
        allowed = (am >= 0).to(torch.float32)
    if allowed.dim() == 3:
        allowed = allowed.unsqueeze(1)
    return allowed


def _check_qkv(q, k, v):
    assert q.is_cuda and k.is_cuda and v.is_cuda
    assert q.dim() == 3 and k.dim() == 4 and v.dim() == 4
    D = q.shape[-1]
    assert D in {16, 32, 64, 128}
    assert q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1, "last dim must be contiguous"
    assert k.shape[-1] == D and v.shape[-1] == D
    assert q.dtype == k.dtype == v.dtype
    assert q.shape[1] % k.shape[1] == 0
    return D


def _int32(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.int32 else t.to(torch.int32)


@torch.no_grad()
def sparse_decode_stage1(
    q: torch.Tensor,              # [B,H,D]
    k: torch.Tensor,              # [B,Kv,S,D]
    v: torch.Tensor,              # [B,Kv,S,D]
    sparse_list: torch.Tensor,    # [B,H,Ktotal] int32
    sparse_len: torch.Tensor,     # [B,H] int32
    max_len_in_batch: int,
    mid_out: torch.Tensor,            # [B,H,block_seq_num,D] fp32
    mid_out_logsumexp: torch.Tensor,  # [B,H,block_seq_num] fp32
    block_seq: int,
):
    D = _check_qkv(q, k, v)
    B, H = q.shape[0], q.shape[1]
    assert sparse_list.is_cuda and sparse_len.is_cuda and mid_out.is_cuda and mid_out_logsumexp.is_cuda
    assert mid_out.dtype == torch.float32 and mid_out_logsumexp.dtype == torch.float32
    assert mid_out.is_contiguous() and mid_out_logsumexp.is_contiguous()
    sparse_list, sparse_len = _int32(sparse_list), _int32(sparse_len)
    assert sparse_list.stride(-1) == 1
    nsplit = (int(max_len_in_batch) + block_seq - 1) // block_seq
    assert mid_out.shape[2] >= nsplit and mid_out.shape[2] == mid_out_logsumexp.shape[2]
    if nsplit == 0:
        return
    check("socket_attend_stage1", lib().socket_attend_stage1(
        ptr(q), ptr(k), ptr(v), dtype_enum(q.dtype),
        q.stride(0), q.stride(1),
        k.stride(0), k.stride(1), k.stride(2),
        v.stride(0), v.stride(1), v.stride(2),
        ptr(sparse_list), sparse_list.stride(0), sparse_list.stride(1),
        ptr(sparse_len), sparse_len.stride(0), sparse_len.stride(1),
        ptr(mid_out), ptr(mid_out_logsumexp),
        B, H, k.shape[1], D, k.shape[2], sparse_list.shape[-1], mid_out.shape[2], int(block_seq),
        stream_ptr(q.device)))


@torch.no_grad()
def sparse_decode_stage2(
    mid_out: torch.Tensor,
    mid_out_logsumexp: torch.Tensor,
    sparse_len: torch.Tensor,
    out: torch.Tensor,            # [B,H,D]
    block_seq: int,
):
    D = out.shape[-1]
    assert D in {16, 32, 64, 128}
    assert mid_out.is_cuda and out.is_cuda and out.stride(-1) == 1
    assert mid_out.is_contiguous() and mid_out_logsumexp.is_contiguous()
    B, H = out.shape[0], out.shape[1]
    sparse_len = _int32(sparse_len)
    check("socket_attend_stage2", lib().socket_attend_stage2(
        ptr(mid_out), ptr(mid_out_logsumexp),
        ptr(sparse_len), sparse_len.stride(0), sparse_len.stride(1),
        ptr(out), dtype_enum(out.dtype), out.stride(0), out.stride(1),
        B, H, D, mid_out.shape[2], int(block_seq), stream_ptr(out.device)))


@torch.no_grad()
def sparse_attention_fwd(
    query: torch.Tensor,        # [B,H,D]
    key: torch.Tensor,          # [B,Kv,S,D]
    value: torch.Tensor,        # [B,Kv,S,D]
    sparse_list: torch.Tensor,  # [B,H,Ktotal]
    sparse_len: torch.Tensor,   # [B,H]
    block_seq: int = 256,
) -> torch.Tensor:
    """Attention of one query per head over the listed K/V rows.

    Differences from the reference launcher, none visible in the result: the
    split size is chosen by the library from the list width and the CU count
    (`block_seq` is kept for signature compatibility; the output does not depend
    on the split beyond fp32 rounding), and the list width bounds the lengths,
    so there is no `sparse_len.max().item()` device-to-host read.
    """
    assert query.is_cuda and key.is_cuda and value.is_cuda and sparse_list.is_cuda and sparse_len.is_cuda
    D = _check_qkv(query, key, value)
    B, H, _ = query.shape
    sparse_list, sparse_len = _int32(sparse_list), _int32(sparse_len)
    assert sparse_list.stride(-1) == 1
    width = sparse_list.shape[-1]
    out = torch.empty((B, H, D), dtype=query.dtype, device=query.device)
    if width == 0:
        return out.fill_(float("nan"))
    L = lib()
    nbytes = L.socket_sparse_attention_workspace_bytes(B, H, D, width)
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=query.device)
    check("socket_sparse_attention", L.socket_sparse_attention(
        ptr(query), ptr(key), ptr(value), dtype_enum(query.dtype),
        query.stride(0), query.stride(1),
        key.stride(0), key.stride(1), key.stride(2),
        value.stride(0), value.stride(1), value.stride(2),
        ptr(sparse_list), sparse_list.stride(0), sparse_list.stride(1),
        ptr(sparse_len), sparse_len.stride(0), sparse_len.stride(1),
        ptr(out), out.stride(0), out.stride(1),
        ptr(ws), nbytes,
        B, H, key.shape[1], D, key.shape[2], width, stream_ptr(query.device)))
    return out


@torch.no_grad()
def sparse_attention_fwd_static(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                sparse_list: torch.Tensor, sparse_len: torch.Tensor,
                                out: torch.Tensor) -> torch.Tensor:
    """`sparse_attention_fwd` into a caller-provided `out` [B,H,D] without allocating
    anything, as one launch: the per-split partials live in a fixed array inside the
    library and the workgroup that finishes a row's last split merges the row
    (one array per GPU, shared by every call on it: calls that overlap on one GPU race).
    `sparse_list` / `sparse_len` must already be int32.  Raises RuntimeError when
    the call needs more than the array holds."""
    assert query.is_cuda and key.is_cuda and value.is_cuda and sparse_list.is_cuda and sparse_len.is_cuda
    D = _check_qkv(query, key, value)
    B, H, _ = query.shape
    assert sparse_list.dtype == torch.int32 and sparse_len.dtype == torch.int32 and sparse_list.stride(-1) == 1
    assert out.is_cuda and tuple(out.shape) == (B, H, D) and out.dtype == query.dtype and out.stride(-1) == 1
    width = sparse_list.shape[-1]
    assert width > 0
    check("socket_sparse_attention_static", lib().socket_sparse_attention_static(
        ptr(query), ptr(key), ptr(value), dtype_enum(query.dtype),
        query.stride(0), query.stride(1),
        key.stride(0), key.stride(1), key.stride(2),
        value.stride(0), value.stride(1), value.stride(2),
        ptr(sparse_list), sparse_list.stride(0), sparse_list.stride(1),
        ptr(sparse_len), sparse_len.stride(0), sparse_len.stride(1),
        ptr(out), out.stride(0), out.stride(1),
        B, H, key.shape[1], D, key.shape[2], width, stream_ptr(query.device)))
    return out


def fits_static_scratch(B: int, H: int, D: int, width: int) -> bool:
    """True if `sparse_attention_fwd_static` takes a call of this shape."""
    L = lib()
    return (width > 0 and B * H <= 65536 and
            L.socket_sparse_attention_workspace_bytes(B, H, D, width) <= L.socket_static_scratch_bytes())


@functools.lru_cache(maxsize=1024)
def prefers_one_launch(B: int, H: int, D: int, width: int) -> bool:
    """Which of the two attention entry points a decode step should take: the
    one-launch variant (the last split of a row merges it) wherever it fits and
    there is a row for every other CU or more.  With few rows the merge is a
    serial tail that every row reaches at about the same time, and a second, tiny
    launch does as well or better (on 256 CUs, steps of 32 rows: 55.6 against
    57.5 us with lists of 1156 entries, equal with 2308; 128 rows: 162.6 against
    165.7 us the other way)."""
    if not fits_static_scratch(B, H, D, width):
        return False
    cus = ctypes.c_int(0)
    lib().socket_device_query(ctypes.byref(cus), None)
    return 2 * B * H >= cus.value


@torch.no_grad()
def dense_decode_fwd(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                     lengths: torch.Tensor) -> torch.Tensor:
    """Dense flash-decode over rows [0, lengths[b]) of the cache: the comparator
    the sparse path is timed against (reference dense decode:
    Attention.forward, GPT-FAST/model.py:562-589)."""
    D = _check_qkv(query, key, value)
    B, H, _ = query.shape
    lengths = _int32(lengths).contiguous()
    assert lengths.is_cuda and lengths.numel() == B
    T = key.shape[2]
    out = torch.empty((B, H, D), dtype=query.dtype, device=query.device)
    L = lib()
    nbytes = L.socket_dense_decode_workspace_bytes(B, H, D, T)
    ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=query.device)
    check("socket_dense_decode", L.socket_dense_decode(
        ptr(query), ptr(key), ptr(value), dtype_enum(query.dtype),
        query.stride(0), query.stride(1),
        key.stride(0), key.stride(1), key.stride(2),
        value.stride(0), value.stride(1), value.stride(2),
        ptr(lengths), ptr(out), out.stride(0), out.stride(1),
        ptr(ws), nbytes, B, H, key.shape[1], D, T, stream_ptr(query.device)))
    return out
