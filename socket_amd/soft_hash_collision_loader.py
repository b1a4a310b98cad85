"""The scorer extension object of the reference, backed by libsocket_hip.so.

`load_soft_hash_collision(version)` mirrors
GPT-FAST/kernels/soft_hash_collision_loader.py:142-161: it returns an object
whose `soft_hash_collision(q_probs, key_buckets, allowed_ext, v_hist)` takes and
returns exactly what the reference's JIT-compiled wrapper does (:14-74), with
the wrapper's checks raising RuntimeError.  Nothing is compiled at call time:
the kernel is prebuilt in the shared library.
"""
from __future__ import annotations

import torch

from ._lib import check, lib, ptr, stream_ptr


def _torch_check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


class _SoftHashCollisionExt:
    """Stand-in for the module object `load_inline` returns in the reference."""

    @staticmethod
    @torch.no_grad()
    def soft_hash_collision(q_probs: torch.Tensor, key_buckets: torch.Tensor,
                            allowed_ext: torch.Tensor, v_hist_in: torch.Tensor) -> torch.Tensor:
        _torch_check(q_probs.is_cuda, "q_probs must be CUDA")
        _torch_check(key_buckets.is_cuda, "key_buckets must be CUDA")
        _torch_check(allowed_ext.is_cuda, "allowed_ext must be CUDA")
        _torch_check(v_hist_in.is_cuda, "v_hist must be CUDA")
        _torch_check(q_probs.is_contiguous(), "q_probs must be contiguous")
        _torch_check(key_buckets.is_contiguous(), "key_buckets must be contiguous")
        _torch_check(allowed_ext.is_contiguous(), "allowed_ext must be contiguous")
        _torch_check(v_hist_in.is_contiguous(), "v_hist must be contiguous")
        _torch_check(q_probs.dtype == torch.float32, "q_probs must be float32")
        _torch_check(key_buckets.dtype == torch.int16, "key_buckets must be int16")
        _torch_check(allowed_ext.dtype == torch.bool, "allowed_ext must be bool")
        _torch_check(v_hist_in.dtype == torch.float32, "v_hist must be float32")
        _torch_check(q_probs.dim() == 5, "q_probs must be [B,H,1,L,R]")
        _torch_check(key_buckets.dim() == 4, "key_buckets must be [B,H,L,T_k]")
        _torch_check(allowed_ext.dim() == 4, "allowed_ext must be [B,H,1,T_k]")
        _torch_check(v_hist_in.dim() == 4, "v_hist must be [B,H,1,T_k]")
        B, H, _, L, R = q_probs.shape
        T = key_buckets.shape[3]
        _torch_check(tuple(key_buckets.shape[:3]) == (B, H, L), "key_buckets shape mismatch")
        _torch_check(tuple(allowed_ext.shape) == (B, H, 1, T), "allowed_ext shape mismatch")
        _torch_check(tuple(v_hist_in.shape) == (B, H, 1, T), "v_hist shape mismatch")
        out = torch.empty((B, H, 1, T), dtype=torch.float32, device=q_probs.device)
        if T == 0:
            return out
        check("socket_soft_hash_collision", lib().socket_soft_hash_collision(
            ptr(q_probs), ptr(key_buckets), ptr(allowed_ext), ptr(v_hist_in), ptr(out),
            B, H, L, R, T, stream_ptr(q_probs.device)))
        return out


def load_soft_hash_collision(version: int = 3, *, verbose: bool = False):
    """Only kernel version 3 exists in the reference source
    (GPT-FAST/kernels/soft_hash_collision.cu:1); any other version raises
    ValueError as the reference's marker search would."""
    if version != 3:
        raise ValueError(f"Start marker for soft_hash_collision_kernel_{version} not found")
    lib()  # fail now, not at first call, if the library is missing
    return _SoftHashCollisionExt()


@torch.no_grad()
def soft_hash_score(q_probs: torch.Tensor, key_buckets: torch.Tensor, v_norm: torch.Tensor,
                    allowed: torch.Tensor) -> torch.Tensor:
    """fp16 scorer: q_probs f16 [B,H,L,R], key_buckets i16 [B,H,L,T], v_norm f16
    [B,H,T], allowed bool [B,H,T] -> f32 [B,H,T]
    (GPT-FAST/kernels/soft_hash_score/soft_hash_score_bindings.cpp:10-36).
    Unlike the reference it is not limited to L in {32,50,64}."""
    _torch_check(q_probs.is_cuda, "q_probs must be CUDA")
    _torch_check(key_buckets.is_cuda, "key_buckets must be CUDA")
    _torch_check(v_norm.is_cuda, "v_norm must be CUDA")
    _torch_check(allowed.is_cuda, "allowed must be CUDA")
    _torch_check(q_probs.dtype == torch.float16, "q_probs must be fp16 (half)")
    _torch_check(key_buckets.dtype == torch.int16, "key_buckets must be int16")
    _torch_check(v_norm.dtype == torch.float16, "v_norm must be fp16 (half)")
    _torch_check(allowed.dtype == torch.bool, "allowed must be bool")
    _torch_check(q_probs.is_contiguous(), "q_probs must be contiguous")
    _torch_check(key_buckets.is_contiguous(), "key_buckets must be contiguous")
    _torch_check(v_norm.is_contiguous(), "v_norm must be contiguous")
    _torch_check(allowed.is_contiguous(), "allowed must be contiguous")
    B, H, L, R = q_probs.shape
    T = key_buckets.shape[3]
    out = torch.empty((B, H, T), dtype=torch.float32, device=q_probs.device)
    if T == 0:
        return out
    check("socket_soft_hash_score_f16", lib().socket_soft_hash_score_f16(
        ptr(q_probs), ptr(key_buckets), ptr(v_norm), ptr(allowed), ptr(out),
        B, H, L, R, T, stream_ptr(q_probs.device)))
    return out
