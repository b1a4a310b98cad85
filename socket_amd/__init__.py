"""MI355X-native implementation of SOCKET's sparse-decode hot path.

Public surface (same names as the reference):
  socket_amd.socket_kernels   sparse_attention_fwd, sparse_decode_stage1/2,
                              attention_mask_to_allowed_prob
  socket_amd.sparse           build_sparse_list_decode (+ re-exports)
  socket_amd.soft_hash_collision_loader   load_soft_hash_collision, soft_hash_score
  socket_amd.hash_cache       the packed-code cache and the fused decode step
All compute runs in libsocket_hip.so (HIP, gfx950); there is no CPU fallback.
"""
from .socket_kernels import (  # noqa: F401
    attention_mask_to_allowed_prob,
    dense_decode_fwd,
    sparse_attention_fwd,
    sparse_decode_stage1,
    sparse_decode_stage2,
)
from .sparse import build_sparse_list_decode, select_list  # noqa: F401

__all__ = [
    "attention_mask_to_allowed_prob", "dense_decode_fwd", "sparse_attention_fwd",
    "sparse_decode_stage1", "sparse_decode_stage2", "build_sparse_list_decode", "select_list",
]
