"""SOCKET attention for HuggingFace-style Llama decoders on the HIP decode path.

Host-side mirror of the `LlamaAttention` of
pipeline/train_quest/modeling/modeling_llama.py (constructor :415-455, planes /
prototypes / hashes :544-638, budgets :644-648, state container :651-678,
forward :680-864): same constructor arguments, method names, forward signature
and return triple, so a decoder layer can hold this module instead.  It has no
dependency on the `transformers` package: `config` is any object with the
usual Llama attributes, `past_key_values` any object with
`get_seq_length()` and `update(k, v, layer_idx, cache_kwargs)` (a
`transformers` cache, or `SimpleKVCache` below).

What differs from the reference is how the per-layer bucket state is kept
(under `past_key_values.bucket_states[layer_idx]`, as there):

  * `codes`  int32 [B,Hkv,NW,cap]: packed table-major bucket codes per KV head.
    The reference hashes the GQA-repeated keys and grows an int16 [B,Hq,L,T]
    tensor with `torch.cat` every step (:785); repeated heads share planes, so
    their codes are equal and one copy per KV head loses nothing.
  * `v_norm` fp16 [B,Hkv,cap]: only the new rows' norms are taken per step (the
    reference recomputes all T of them, :790).
  * `cached`: host count of hashed positions.  The key length of a step is a
    tensor shape, so nothing is read back from the device.

A decode step is: hash-append (1 launch), soft hash (1), score (1), select (2),
attend (2).  Every cached position is allowed (monotonic decode; the reference
builds `arange(T_k) <= cache_position.max()`, :797-799, which is all-true then).
With `attention_mask=None` a multi-token block attends causally (the reference
passes `is_causal=False` and would attend to the future there).
"""
from __future__ import annotations

import itertools
import math
from typing import Optional

import torch
import torch.nn as nn
from torch.nn import functional as F

from . import hash_cache
from .socket_kernels import dense_decode_fwd


def rotate_half(x):
    x1 = x[..., : x.shape[-1] // 2]
    x2 = x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, position_ids=None, unsqueeze_dim=1):
    """HF rotary convention (modeling_llama.py:228-252): halves, not pairs."""
    cos = cos.unsqueeze(unsqueeze_dim)
    sin = sin.unsqueeze(unsqueeze_dim)
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


class SimpleKVCache:
    """Minimal stand-in for a `transformers` cache: preallocated K/V per layer,
    `update` appends and returns views of the filled prefix."""

    def __init__(self, n_layers: int, batch: int, n_kv_heads: int, head_dim: int, max_seq: int, dtype, device):
        self.k = [torch.zeros((batch, n_kv_heads, max_seq, head_dim), dtype=dtype, device=device)
                  for _ in range(n_layers)]
        self.v = [torch.zeros_like(t) for t in self.k]
        self.seen = [0] * n_layers

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return self.seen[layer_idx]

    def update(self, k, v, layer_idx: int, cache_kwargs=None):
        n0, n1 = self.seen[layer_idx], self.seen[layer_idx] + k.shape[2]
        self.k[layer_idx][:, :, n0:n1].copy_(k)
        self.v[layer_idx][:, :, n0:n1].copy_(v)
        self.seen[layer_idx] = n1
        return self.k[layer_idx][:, :, :n1], self.v[layer_idx][:, :, :n1]


class SocketLlamaAttention(nn.Module):
    def __init__(self, config, layer_idx: int):
        super().__init__()
        self.config = config
        self.layer_idx = layer_idx
        self.head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
        self.num_key_value_groups = config.num_attention_heads // config.num_key_value_heads
        self.scaling = self.head_dim ** -0.5
        self.attention_dropout = getattr(config, "attention_dropout", 0.0)
        self.is_causal = True
        bias = getattr(config, "attention_bias", False)
        self.q_proj = nn.Linear(config.hidden_size, config.num_attention_heads * self.head_dim, bias=bias)
        self.k_proj = nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=bias)
        self.v_proj = nn.Linear(config.hidden_size, config.num_key_value_heads * self.head_dim, bias=bias)
        self.o_proj = nn.Linear(config.num_attention_heads * self.head_dim, config.hidden_size, bias=bias)
        self.bucket_K = getattr(config, "bucket_K", 8)    # P, bits per table
        self.bucket_L = getattr(config, "bucket_L", 60)   # L, tables
        self._planes_cache = {}
        self._protos_cache = {}
        self._seed = 123456789
        self._rng_cache = {}

    # ---- planes, prototypes, hashes (modeling_llama.py:458-638) --------------------------
    PLANE_SEED_OFFSET = 7777      # modeling_llama.py:463 seeds its plane generator with seed + 7777

    def _rng(self, device) -> Optional[torch.Generator]:
        """One seeded generator per device for drawing the hyperplanes (none when the
        seed is unset: planes then come from torch's default generator)."""
        if self._seed is None:
            return None
        try:
            return self._rng_cache[device]
        except KeyError:
            gen = torch.Generator(device=device).manual_seed(int(self._seed) + self.PLANE_SEED_OFFSET)
            self._rng_cache[device] = gen
            return gen

    def get_hyper_planes(self, cache, D: int, L: int, P: int, device, dtype, rng=None) -> torch.Tensor:
        key = (D, device, dtype, L, P)
        planes = cache.get(key)
        if planes is None:
            planes = torch.randn((L, P, D), device=device, dtype=torch.float32, generator=rng).to(dtype)
            cache[key] = planes
        return planes

    def get_protos_T(self, cache, P: int, device, dtype) -> torch.Tensor:
        """Hypercube corners [P, 2^P]; column r is the corner whose big-endian sign
        pattern is r, the order `pack_bits` uses."""
        key = (P, device, dtype)
        protos_T = cache.get(key)
        if protos_T is None:
            corners = torch.tensor(list(itertools.product([-1.0, +1.0], repeat=P)), device=device,
                                   dtype=torch.float32)
            protos_T = corners.t().contiguous().to(dtype)
            cache[key] = protos_T
        return protos_T

    def pack_bits(self, bits: torch.Tensor) -> torch.Tensor:
        P = bits.shape[-1]
        weights = 1 << torch.arange(P - 1, -1, -1, device=bits.device, dtype=torch.int16)
        return torch.sum(bits.to(torch.int16) * weights, dim=-1)

    def hard_hash(self, tensor: torch.Tensor, planes: torch.Tensor) -> torch.Tensor:
        """[B,H,N,D] x planes [L,P,D] -> int16 codes [B,H,L,N] (modeling_llama.py:605-615)."""
        if tensor.is_cuda and tensor.shape[-1] == 128:
            B, H, N, _ = tensor.shape
            L, P, _ = planes.shape
            words = torch.empty((B, H, hash_cache.words_per_key(L, P), (N + 3) // 4 * 4), dtype=torch.int32,
                                device=tensor.device)
            hash_cache.hash_keys_into(tensor, None, hash_cache.permute_planes(planes), words, None, L, P, t0=0)
            return hash_cache.unpack_codes(words, L, P, 0, N, layout="bhlt")
        proj = torch.einsum("bhnd,lkd->bhnlk", tensor, planes)
        return self.pack_bits(proj >= 0).permute(0, 1, 3, 2).contiguous()

    def soft_hash(self, queries: torch.Tensor, planes: torch.Tensor, protos_T: torch.Tensor) -> torch.Tensor:
        """[B,H,Q,D] -> [B,H,Q,L,R], softmax of the logits / 0.3 (modeling_llama.py:618-638)."""
        if queries.is_cuda and queries.shape[2] == 1:
            return hash_cache.soft_hash(queries[:, :, 0], planes, protos_T, 0.3,
                                        self.config.num_key_value_heads).unsqueeze(2)
        q_proj = torch.einsum("bhqd,lkd->bhqlk", queries, planes)
        qh = torch.tanh(q_proj) / max(math.sqrt(queries.size(-1)), 1e-6)
        return F.softmax(torch.einsum("bhqlk,kr->bhqlr", qh, protos_T) / 0.3, dim=-1)

    def _effective_size(self, size, N: int) -> int:
        return int(size * N) if isinstance(size, float) else int(size)

    def _get_states_container(self, past_key_values, runtime_states):
        """Where the per-layer hash state lives between decode steps: on the HF cache
        object (attribute `bucket_states`, created on first use) when there is one,
        else in the dict the caller passes (modeling_llama.py:651-678)."""
        if past_key_values is None:
            return runtime_states if runtime_states is not None else {}
        if not hasattr(past_key_values, "bucket_states") or past_key_values.bucket_states is None:
            past_key_values.bucket_states = {}
        return past_key_values.bucket_states

    # ---- bucket state ----------------------------------------------------------------------------
    def _hash_append(self, st: dict, k: torch.Tensor, v: torch.Tensor, T_k: int) -> None:
        """Hash rows [cached, T_k) of k / take their value norms into the state."""
        t0 = st["cached"]
        if t0 >= T_k:
            return
        if T_k > st["codes"].shape[-1]:          # cache outgrew the state: double it
            cap = max(T_k, 2 * st["codes"].shape[-1])
            cap = (cap + 7) // 8 * 8
            codes = torch.zeros(st["codes"].shape[:3] + (cap,), dtype=torch.int32, device=k.device)
            v_norm = torch.zeros(st["v_norm"].shape[:2] + (cap,), dtype=torch.float16, device=k.device)
            codes[..., :t0] = st["codes"][..., :t0]
            v_norm[..., :t0] = st["v_norm"][..., :t0]
            st["codes"], st["v_norm"] = codes, v_norm
        _hash_rows(st, k[:, :, t0:T_k], v[:, :, t0:T_k], t0)
        st["cached"] = T_k

    def forward(self, hidden_states: torch.Tensor, position_embeddings, attention_mask=None,
                past_key_values=None, cache_position=None, cra_states: Optional[dict] = None, **kwargs):
        input_shape = hidden_states.shape[:-1]
        B, T_q, _ = hidden_states.shape
        hidden_shape = (*input_shape, -1, self.head_dim)
        q = self.q_proj(hidden_states).view(hidden_shape).transpose(1, 2)   # [B,H,T_q,D]
        k = self.k_proj(hidden_states).view(hidden_shape).transpose(1, 2)   # [B,Hkv,T_q,D]
        v = self.v_proj(hidden_states).view(hidden_shape).transpose(1, 2)
        cos, sin = position_embeddings
        q, k = apply_rotary_pos_emb(q, k, cos, sin)

        past_len = 0
        if past_key_values is not None:
            past_len = past_key_values.get_seq_length()
            k, v = past_key_values.update(k, v, self.layer_idx, {"sin": sin, "cos": cos,
                                                                  "cache_position": cache_position})
        Hkv, T_k, D = k.shape[1], k.shape[2], k.shape[3]
        H = Hkv * self.num_key_value_groups
        device = q.device
        states = self._get_states_container(past_key_values, cra_states)
        P, L = int(self.bucket_K), int(self.bucket_L)

        if not (T_q == 1 and past_len > 0):
            # prefill / multi-token block: dense attention, (re)build the bucket state
            if attention_mask is not None:
                y = F.scaled_dot_product_attention(q, k, v, attn_mask=attention_mask, scale=self.scaling,
                                                   enable_gqa=H != Hkv)
            else:
                y = F.scaled_dot_product_attention(q, k, v, is_causal=T_q > 1 and T_q == T_k, scale=self.scaling,
                                                   enable_gqa=H != Hkv)
            out = self.o_proj(y.transpose(1, 2).contiguous().reshape(*input_shape, -1))
            planes = self.get_hyper_planes(self._planes_cache, D, L, P, device, k.dtype, self._rng(device))
            max_seq = int(getattr(self.config, "max_position_embeddings", max(2048, T_k)))
            cap = (max(max_seq, T_k) + 7) // 8 * 8
            st = {
                "P": P, "L": L, "R": 1 << P, "planes": planes, "planes_words": _planes_to_words(planes),
                "codes": torch.zeros((B, Hkv, hash_cache.words_per_key(L, P), cap), dtype=torch.int32, device=device),
                "v_norm": torch.zeros((B, Hkv, cap), dtype=torch.float16, device=device),
                "cached": 0, "max_seq": max_seq, "device": device, "B": B, "H": H,
            }
            self._hash_append(st, k, v, T_k)
            states[self.layer_idx] = st
            return out, None, {"bucket_sparse": False}

        # single-token decode: expected-collision top-M + sink + local window
        st = states[self.layer_idx]
        P, L, R = int(st["P"]), int(st["L"]), int(st["R"])
        self._hash_append(st, k, v, T_k)
        sink = int(getattr(self.config, "sink_size", 20))
        window = int(getattr(self.config, "window_size", 20))
        M_cfg = getattr(self.config, "heavy_const", getattr(self.config, "heavy_size", 0.1))
        M = max(0, min(self._effective_size(M_cfg, T_k), T_k))
        protos_T = self.get_protos_T(self._protos_cache, P, device, k.dtype)
        q_bhd = q[:, :, 0]
        if _dense_is_cheaper(self.config, q_bhd, k, L, P, R, T_k, sink, window, M):
            # config.dense_below_crossover (not in the reference): exact attention over a context
            # short enough for the dense kernel to be priced below score + select + attend
            out_bhd = _dense_step(q_bhd, k, v, T_k)
            out = self.o_proj(out_bhd.reshape(B, 1, -1))
            return out, None, {"bucket_sparse": False, "mode": "dense_below_crossover", "T_k": int(T_k)}
        q_probs = _soft_hash(q_bhd, st["planes"], protos_T, Hkv, T_k)
        out_bhd = _sparse_step(q_bhd, q_probs, k, v, st, T_k, sink, window, M)
        out = self.o_proj(out_bhd.reshape(B, 1, -1))
        return out, None, {"bucket_sparse": True, "mode": "cra_sparse", "T_k": int(T_k), "P": P, "R": R,
                           "L": L, "M": int(M)}


# Where this module enters the HIP library (module-level so that a test can put
# a checker in one's place; the product has no other route).
def _planes_to_words(planes):
    return hash_cache.permute_planes(planes)


def _hash_rows(st: dict, k_new, v_new, t0: int) -> None:
    hash_cache.hash_keys_into(k_new, v_new, st["planes_words"], st["codes"], st["v_norm"], st["L"], st["P"], t0=t0)


def _soft_hash(q_bhd, planes, protos_T, n_kv_heads: int, context_len: int):
    grouped = hash_cache.prefers_grouped(q_bhd, planes, protos_T, n_kv_heads, context_len)
    return hash_cache.soft_hash(q_bhd, planes, protos_T, 0.3, n_kv_heads, grouped=grouped)


def _dense_is_cheaper(config, q_bhd, k, L: int, P: int, R: int, T_k: int, sink: int, window: int, M: int) -> bool:
    if not getattr(config, "dense_below_crossover", False) or not q_bhd.is_cuda:
        return False
    B, Hq, D = q_bhd.shape
    sparse_us, dense_us = hash_cache.step_cost_estimate(B, Hq, k.shape[1], D, int(T_k), L, P, R, int(M), int(sink),
                                                        int(window), q_bhd.dtype == torch.bfloat16, k.element_size())
    return dense_us < sparse_us


def _dense_step(q_bhd, k, v, T_k: int):
    lengths = torch.full((q_bhd.shape[0],), int(T_k), dtype=torch.int32, device=q_bhd.device)
    return dense_decode_fwd(q_bhd, k, v, lengths)


def _sparse_step(q_bhd, q_probs, k, v, st: dict, T_k: int, sink: int, window: int, M: int):
    return hash_cache.sparse_decode_step(q_bhd, q_probs, k, v, st["codes"], st["v_norm"], T_k, st["P"],
                                         min(sink, T_k), min(window, T_k), M)
