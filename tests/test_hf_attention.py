"""The HuggingFace-style attention hook (socket_amd/hf_attention.py): host glue on
the CPU with oracle stand-ins for its entries into the HIP library, and the real
path on the MI355X against the oracle's restatement of the reference's decode
branch (modeling_llama.py:764-864)."""
import types

import numpy as np
import pytest
import torch

from oracle import socket_oracle as orc
from socket_amd import hf_attention as hf


def make_config(**kw):
    base = dict(hidden_size=512, num_attention_heads=4, num_key_value_heads=2, head_dim=128, attention_bias=False,
                attention_dropout=0.0, max_position_embeddings=256, bucket_K=8, bucket_L=12, sink_size=3,
                window_size=5, heavy_size=0.1)
    base.update(kw)
    return types.SimpleNamespace(**base)


def rope_tables(positions, D, base=10000.0):
    inv = 1.0 / (base ** (torch.arange(0, D, 2).float() / D))
    ang = torch.outer(positions.float(), inv)
    emb = torch.cat([ang, ang], dim=-1)[None]          # [1,S,D], HF convention
    return emb.cos(), emb.sin()


def make_module(cfg, seed=0, dtype=torch.float32, device="cpu"):
    torch.manual_seed(seed)
    m = hf.SocketLlamaAttention(cfg, layer_idx=0)
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(0, 0.05)
    return m.to(device=device, dtype=dtype).eval()


# ---- oracle stand-ins (CPU tests) -----------------------------------------------------------------
def _o_planes_to_words(planes):
    return planes.detach().float().cpu()


def _o_hash_rows(st, k_new, v_new, t0):
    k = k_new.detach().float().cpu()
    codes = orc.hard_hash_bhln(k, st["planes_words"])                                      # [B,H,L,S]
    words = orc.pack_code_words(codes.numpy(), st["P"])
    S = k.shape[2]
    st["codes"][:, :, :, t0:t0 + S] = torch.from_numpy(words.view(np.int32))
    st["v_norm"][:, :, t0:t0 + S] = orc.value_norm(v_new.detach().float().cpu())


def _o_soft_hash(q_bhd, planes, protos_T, n_kv_heads, context_len):
    return orc.soft_hash(q_bhd.detach().float().cpu(), planes.float().cpu(), protos_T.float().cpu(), 0.3)


def _o_sparse_step(q_bhd, q_probs, k, v, st, T_k, sink, window, M):
    return _oracle_decode(q_bhd, q_probs, k, v, st, T_k, sink, window, M).to(q_bhd.dtype)


def _oracle_decode(q_bhd, q_probs, k, v, st, T_k, sink, window, M):
    """scorer -> stable top-M -> [sink | window | heavy] -> textbook softmax, on the CPU."""
    G = q_bhd.shape[1] // k.shape[1]
    words = st["codes"][:, :, :, :T_k].cpu().numpy().view(np.uint32)
    codes = torch.from_numpy(orc.unpack_code_words(words, st["L"], st["P"])).repeat_interleave(G, dim=1)
    vn = st["v_norm"][:, :, :T_k].cpu().repeat_interleave(G, dim=1)
    allowed = torch.ones(vn.shape, dtype=torch.bool)
    sl, ln = orc.build_sparse_list_decode(q_probs.detach().float().cpu(), codes, vn, allowed, sink, window, M)
    return orc.sparse_attend_textbook(q_bhd.detach().float().cpu(), k.detach().float().cpu(),
                                      v.detach().float().cpu(), sl, ln).float()


def _install_oracle(monkeypatch):
    monkeypatch.setattr(hf, "_planes_to_words", _o_planes_to_words)
    monkeypatch.setattr(hf, "_hash_rows", _o_hash_rows)
    monkeypatch.setattr(hf, "_soft_hash", _o_soft_hash)
    monkeypatch.setattr(hf, "_sparse_step", _o_sparse_step)


@torch.no_grad()
def _drive(m, x, n_prompt, cache):
    """Prefill n_prompt tokens, then one token at a time; returns outputs [B,S,hidden] and infos."""
    S, D = x.shape[1], m.head_dim
    dev = x.device
    cos, sin = rope_tables(torch.arange(n_prompt), D)
    outs = [m(x[:, :n_prompt], (cos.to(dev, x.dtype), sin.to(dev, x.dtype)), None, cache,
              torch.arange(n_prompt, device=dev))[0]]
    infos = []
    for t in range(n_prompt, S):
        cos, sin = rope_tables(torch.tensor([t]), D)
        o, _, info = m(x[:, t:t + 1], (cos.to(dev, x.dtype), sin.to(dev, x.dtype)), None, cache,
                       torch.tensor([t], device=dev))
        outs.append(o)
        infos.append(info)
    return torch.cat(outs, 1), infos


def test_helpers_match_oracle_definitions():
    m = make_module(make_config())
    planes = m.get_hyper_planes({}, 128, 12, 8, torch.device("cpu"), torch.float32, m._rng(torch.device("cpu")))
    again = hf.SocketLlamaAttention(make_config(), 0)
    planes2 = again.get_hyper_planes({}, 128, 12, 8, torch.device("cpu"), torch.float32,
                                     again._rng(torch.device("cpu")))
    assert torch.equal(planes, planes2)                                                   # seeded, reproducible
    protos = m.get_protos_T({}, 8, torch.device("cpu"), torch.float32)
    assert torch.equal(protos, orc.hypercube_protos_T(8))
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 4, 9, 128, generator=g)
    assert torch.equal(m.hard_hash(x, planes), orc.hard_hash_bhln(x, planes))
    q = torch.randn(2, 4, 1, 128, generator=g)
    torch.testing.assert_close(m.soft_hash(q, planes, protos)[:, :, 0], orc.soft_hash(q[:, :, 0], planes, protos, 0.3),
                               rtol=1e-5, atol=1e-8)
    assert m._effective_size(0.1, 250) == 25 and m._effective_size(40, 250) == 40
    # HF rotary: halves rotated, norm preserved
    cos, sin = rope_tables(torch.tensor([7]), 128)
    qr, kr = hf.apply_rotary_pos_emb(q, q, cos, sin)
    torch.testing.assert_close(qr.norm(dim=-1), q.norm(dim=-1), rtol=1e-5, atol=1e-5)
    assert torch.equal(qr, kr)


def test_all_covering_window_equals_causal_attention(monkeypatch):
    """No sink, no heavy budget, window longer than the context: every cached
    position is listed once, so token-by-token decode through the sparse branch
    equals one dense causal pass."""
    _install_oracle(monkeypatch)
    cfg = make_config(sink_size=0, window_size=1000, heavy_size=0.0)
    m = make_module(cfg, seed=1)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 24, 512, generator=g)
    cache = hf.SimpleKVCache(1, 2, 2, 128, 64, torch.float32, "cpu")
    step, infos = _drive(m, x, 15, cache)
    cos, sin = rope_tables(torch.arange(24), 128)
    full = m(x, (cos, sin), None, None, torch.arange(24))[0]
    torch.testing.assert_close(step, full, rtol=2e-4, atol=2e-5)
    assert all(i["bucket_sparse"] and i["M"] == 0 for i in infos)
    st = cache.bucket_states[0]
    assert st["cached"] == 24 and st["codes"].shape == (2, 2, 3, 256)


def test_budget_bookkeeping_and_state_growth(monkeypatch):
    _install_oracle(monkeypatch)
    cfg = make_config(max_position_embeddings=16, heavy_size=0.25)
    m = make_module(cfg, seed=2)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, 30, 512, generator=g)
    cache = hf.SimpleKVCache(1, 1, 2, 128, 64, torch.float32, "cpu")
    _, infos = _drive(m, x, 12, cache)
    assert [i["M"] for i in infos] == [int(0.25 * t) for t in range(13, 31)]
    assert [i["T_k"] for i in infos] == list(range(13, 31))
    st = cache.bucket_states[0]
    assert st["cached"] == 30 and st["codes"].shape[-1] >= 30                             # grew past the 16 it started with
    want = orc.hard_hash_bhln(cache.k[0][:, :, :30], st["planes"])
    have = orc.unpack_code_words(st["codes"][..., :30].numpy().view(np.uint32), 12, 8)
    assert torch.equal(torch.from_numpy(have), want)


@pytest.mark.gpu
@torch.no_grad()
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-3), (torch.bfloat16, 5e-2)])
def test_decode_branch_on_device_matches_oracle(dev, dtype, tol):
    cfg = make_config(heavy_size=0.2, bucket_L=20)
    m = make_module(cfg, seed=3, dtype=dtype, device=dev)
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(2, 130, 512, generator=g)).to(dtype).to(dev)
    cache = hf.SimpleKVCache(1, 2, 2, 128, 160, dtype, dev)
    have, infos = _drive(m, x, 120, cache)
    st = cache.bucket_states[0]
    assert st["cached"] == 130 and infos[-1] == {"bucket_sparse": True, "mode": "cra_sparse", "T_k": 130, "P": 8,
                                                  "R": 256, "L": 20, "M": 26}
    # hash state: decided bits equal the oracle's hash of the cached keys; norms of the cached values
    # (the kernel multiplies bf16-rounded keys and planes on the matrix cores)
    keys = cache.k[0][:, :, :130].cpu().to(torch.bfloat16).float()
    proj = orc.projections_f64(keys.permute(0, 2, 1, 3), st["planes"].cpu().to(torch.bfloat16).float())   # [B,T,H,L,P]
    clear = (proj.abs() > 1e-3 * proj.abs().mean()).all(-1)
    codes = torch.from_numpy(orc.unpack_code_words(st["codes"][..., :130].cpu().numpy().view(np.uint32), 20, 8))
    assert clear.float().mean() > 0.9
    assert torch.equal(codes.permute(0, 3, 1, 2)[clear], orc.pack_bits(proj >= 0)[clear])
    torch.testing.assert_close(st["v_norm"][..., :130].float().cpu(),
                               cache.v[0][:, :, :130].float().norm(dim=-1).cpu(), rtol=2e-3, atol=1e-3)
    # every decode step's output against the oracle run on the same state
    planes, protos = st["planes"].float().cpu(), orc.hypercube_protos_T(8)
    for i, t in enumerate(range(120, 130)):
        T_k = t + 1
        cos, sin = rope_tables(torch.tensor([t]), 128)
        xs = x[:, t:t + 1]
        q = m.q_proj(xs).view(2, 1, 4, 128).transpose(1, 2)
        q, _ = hf.apply_rotary_pos_emb(q, q, cos.to(dev, dtype), sin.to(dev, dtype))
        q_bhd = q[:, :, 0].float().cpu()
        q_probs = orc.soft_hash(q_bhd, planes.to(dtype).float(), protos, 0.3)
        if dtype == torch.bfloat16:
            q_probs = q_probs.to(torch.bfloat16).float()
        att = _oracle_decode(q_bhd, q_probs, cache.k[0][:, :, :T_k], cache.v[0][:, :, :T_k], st, T_k, 3, 5,
                             int(0.2 * T_k))
        want = m.o_proj(att.to(dtype).to(dev).reshape(2, 1, -1)).float().cpu()
        got = have[:, 120 + i:121 + i].float().cpu()
        assert float((got - want).abs().max()) <= tol * max(1.0, float(want.abs().max())), t


@pytest.mark.gpu
@torch.no_grad()
def test_dense_below_crossover_in_the_hf_hook(dev):
    """config.dense_below_crossover on a short context: the decode branch reports the
    dense mode, its output is causal attention over the cache (the prefill branch's own
    arithmetic on the same tokens), and the bucket state still receives every key."""
    cfg = make_config(heavy_size=0.2, bucket_L=20)
    cfg.dense_below_crossover = True
    m = make_module(cfg, seed=3, dtype=torch.float32, device=dev)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, 130, 512, generator=g).to(dev)
    cache = hf.SimpleKVCache(1, 2, 2, 128, 160, torch.float32, dev)
    have, infos = _drive(m, x, 120, cache)
    assert infos[-1] == {"bucket_sparse": False, "mode": "dense_below_crossover", "T_k": 130}
    assert cache.bucket_states[0]["cached"] == 130
    full = hf.SimpleKVCache(1, 2, 2, 128, 160, torch.float32, dev)
    want, _ = _drive(m, x, 130, full)                      # one causal pass over all 130 tokens
    assert float((have[:, 120:] - want[:, 120:]).abs().max()) <= 2e-3 * max(1.0, float(want.abs().max()))


@pytest.mark.gpu
def test_device_helpers_use_reference_layouts(dev):
    m = make_module(make_config(), device=dev)
    planes = m.get_hyper_planes(m._planes_cache, 128, 12, 8, dev, torch.float32, m._rng(dev))
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 2, 33, 128, generator=g)
    have = m.hard_hash(x.to(dev), planes).cpu()
    assert have.dtype == torch.int16 and tuple(have.shape) == (2, 2, 12, 33)
    proj = orc.projections_f64(x.to(torch.bfloat16).float().permute(0, 2, 1, 3), planes.cpu().to(torch.bfloat16).float())
    clear = (proj.abs() > 1e-3 * proj.abs().mean()).all(-1)                               # [B,N,H,L]
    assert torch.equal(have.permute(0, 3, 1, 2)[clear], orc.pack_bits(proj >= 0)[clear])
    q = torch.randn(2, 4, 1, 128, generator=g).to(dev)
    protos = m.get_protos_T(m._protos_cache, 8, dev, torch.float32)
    p = m.soft_hash(q, planes, protos)
    assert tuple(p.shape) == (2, 4, 1, 12, 256)
    torch.testing.assert_close(p[:, :, 0].cpu(), orc.soft_hash(q[:, :, 0].cpu(), planes.cpu(), protos.cpu(), 0.3),
                               rtol=2e-5, atol=1e-9)
