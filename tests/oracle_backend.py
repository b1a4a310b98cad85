"""Checker stand-ins for the three places where socket_amd.model enters the HIP
library, built on the CPU oracle.  Test infrastructure only: installed with
monkeypatch by the model tests, never imported by the package."""
from __future__ import annotations

import numpy as np
import torch

from oracle import socket_oracle as orc


def planes_to_words(planes):
    """The oracle hashes with the [L,P,D] planes themselves."""
    return planes.detach().float().cpu()


def hash_rows(cache, k_bshd, v_bshd, t0=0, pos_b=None):
    planes = cache.planes_words
    k = k_bshd.detach().float().cpu()
    v = v_bshd.detach().float().cpu()
    B, S, H, _ = k.shape
    codes = orc.hard_hash_keys(k, planes)                                         # [B,S,H,L]
    words = orc.pack_code_words(codes.permute(0, 2, 3, 1).numpy(), cache.K)       # [B,H,NW,S]
    words = torch.from_numpy(words.view(np.int32)).to(cache.codes.device)
    vn = orc.value_norm(v).permute(0, 2, 1).to(cache.v_norm.device)               # [B,H,S]
    for b in range(B):
        p0 = int(pos_b[b]) if pos_b is not None else t0
        cache.codes[b, :, :, p0:p0 + S] = words[b]
        cache.v_norm[b, :, p0:p0 + S] = vn[b]


def ungroup(q_table, H, Hkv):
    """Grouped table [B, Hkv*parts, L, R, width] -> [B,H,L,R]."""
    if q_table.dim() == 4:
        return q_table
    B, _, L, R, width = q_table.shape
    G = H // Hkv
    parts = q_table.shape[1] // Hkv
    t = q_table.view(B, Hkv, parts, L, R, width).permute(0, 1, 2, 5, 3, 4).reshape(B, Hkv, parts * width, L, R)
    return t[:, :, :G].reshape(B, H, L, R)


def sparse_step(q_bhd, q_probs, cache, T, sink, window, M):
    dev, dt = q_bhd.device, q_bhd.dtype
    B, H, D = q_bhd.shape
    Hkv = cache.k_cache.shape[1]
    G = H // Hkv
    q_probs = ungroup(q_probs, H, Hkv)
    out = torch.empty((B, H, D), dtype=dt)
    for b in range(B):
        n = min(int(cache.lens[b]), T)
        words = cache.codes[b, :, :, :n].cpu().numpy().view(np.uint32)             # [Hkv,NW,n]
        codes = torch.from_numpy(orc.unpack_code_words(words, cache.L, cache.K))   # [Hkv,L,n]
        codes = codes.repeat_interleave(G, dim=0)[None]                             # [1,H,L,n]
        vn = cache.v_norm[b, :, :n].cpu().repeat_interleave(G, dim=0)[None]
        allowed = torch.ones((1, H, n), dtype=torch.bool)
        sl, ln = orc.build_sparse_list_decode(q_probs[b:b + 1].detach().cpu(), codes, vn, allowed,
                                              min(sink, n), min(window, n), min(M, n))
        k = cache.k_cache[b:b + 1, :, :n].cpu()
        v = cache.v_cache[b:b + 1, :, :n].cpu()
        out[b] = orc.sparse_attend_textbook(q_bhd[b:b + 1].detach().cpu(), k, v, sl, ln)[0].to(dt)
    return out.to(dev)


def dense_step(q_bhd, cache):
    out = orc.dense_attend(q_bhd.detach().cpu(), cache.k_cache.cpu(), cache.v_cache.cpu(), cache.lens.cpu())
    return out.to(q_bhd.dtype).to(q_bhd.device)


def install(monkeypatch, model_module, *, hashing=True, sparse=True, dense=True):
    """Route the chosen entries of socket_amd.model through the oracle."""
    if hashing:
        monkeypatch.setattr(model_module, "_planes_to_words", planes_to_words)
        monkeypatch.setattr(model_module, "_hash_rows", hash_rows)
    if sparse:
        monkeypatch.setattr(model_module, "_sparse_step", sparse_step)
    if dense:
        monkeypatch.setattr(model_module, "_dense_step", dense_step)
