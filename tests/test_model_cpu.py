"""Host-side model and harness on the CPU.  The attention hook's three entries
into the HIP library are replaced by oracle stand-ins (tests/oracle_backend.py),
so these tests pin the glue: projections, rotary embedding, cache bookkeeping,
greedy decoding -- not the kernels."""
import math

import pytest
import torch

from oracle import socket_oracle as orc
from socket_amd import generate as gen
from socket_amd import model as M
from tests import oracle_backend


def toy_args(**kw):
    base = dict(block_size=256, vocab_size=211, n_layer=2, n_head=2, n_local_heads=1, dim=256, L=6, K=4, R=16,
                heavy_const=4096, sink_size=2, window_size=4, rope_base=10000)
    base.update(kw)
    return M.ModelArgs(**base)


def toy_model(seed=0, **kw):
    torch.manual_seed(seed)
    model = M.Transformer(toy_args(**kw)).float().eval()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if not name.endswith("norm.weight"):
                p.normal_(0, 0.08)
        for blk in model.layers:
            blk.attention.planes.normal_(0, 1.0)
            blk.attention.protos_T.copy_(orc.hypercube_protos_T(4) * 2.0)
    return model


def test_model_args_match_reference_defaults():
    a = M.ModelArgs()
    assert (a.block_size, a.vocab_size, a.n_layer, a.n_head, a.dim) == (300000, 32000, 1, 32, 4096)
    assert (a.L, a.R, a.K, a.heavy_const) == (60, 1024, 10, 3600)
    assert a.n_local_heads == 32 and a.head_dim == 128 and a.intermediate_size == 11008
    b = M.ModelArgs.from_name("Llama-3.1-8B")
    assert (b.n_layer, b.n_head, b.n_local_heads, b.dim, b.intermediate_size, b.vocab_size) == \
        (32, 32, 8, 4096, 14336, 128256)
    assert M.ModelArgs.from_name("70B").n_local_heads == 8
    with pytest.raises(AssertionError):
        M.ModelArgs.from_name("no-such-model")


def test_pack_bits_and_hard_hash_match_oracle_and_closed_form():
    attn = M.Attention(toy_args())
    g = torch.Generator().manual_seed(1)
    bits = torch.rand(3, 5, 4, generator=g) > 0.5
    assert torch.equal(attn.pack_bits(bits), orc.pack_bits(bits))
    assert int(attn.pack_bits(torch.tensor([True, False, True, True]))) == 0b1011      # first bit is the MSB
    keys = torch.randn(2, 7, 1, 128, generator=g)
    attn.planes.normal_(0, 1.0, generator=g)
    codes = attn.hard_hash_keys(keys)
    assert codes.dtype == torch.int16 and tuple(codes.shape) == (2, 7, 1, 6)
    assert torch.equal(codes, orc.hard_hash_keys(keys, attn.planes))
    assert torch.equal(attn.hard_hash_keys(keys * 3.5), codes)                          # scale invariance
    assert torch.equal(attn.hard_hash_keys(-keys), (~codes) & 0xF)                      # sign flip = complement


def test_soft_hash_matches_oracle_and_its_argmax_is_the_hard_hash():
    attn = M.Attention(toy_args())
    g = torch.Generator().manual_seed(2)
    attn.planes.normal_(0, 1.0, generator=g)
    attn.protos_T.copy_(orc.hypercube_protos_T(4))
    q = torch.randn(2, 2, 128, generator=g)
    p = attn.soft_hash(q)
    assert tuple(p.shape) == (2, 2, 6, 16)
    torch.testing.assert_close(p, orc.soft_hash(q, attn.planes, attn.protos_T), rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(p.sum(-1), torch.ones(2, 2, 6), rtol=1e-5, atol=1e-6)
    hard = attn.hard_hash_keys(q.unsqueeze(2).permute(0, 2, 1, 3).reshape(2, 1, 2, 128))   # [B,1,H,L]
    assert torch.equal(p.argmax(-1), hard[:, 0].long())


def test_rotary_is_a_rotation_that_depends_on_relative_position():
    fc = M.precompute_freqs_cis(64, 128, 10000).float()
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, 1, 1, 128, generator=g)
    y = torch.randn(1, 1, 1, 128, generator=g)
    def rot(t, pos):
        return M.apply_rotary_emb(t, fc[pos:pos + 1])
    torch.testing.assert_close(rot(x, 9).norm(), x.norm(), rtol=2e-3, atol=0)
    torch.testing.assert_close(rot(x, 0), x)                                            # angle 0
    a = (rot(x, 5) * rot(y, 3)).sum()
    b = (rot(x, 22) * rot(y, 20)).sum()
    torch.testing.assert_close(a, b, rtol=2e-2, atol=2e-2)                              # bf16 angle table
    # pair (2i, 2i+1) is rotated by pos * base^(-2i/D)
    ang = 7 * 10000.0 ** (-2 * 3 / 128)
    e = torch.zeros(1, 1, 1, 128); e[..., 6] = 1.0
    r = rot(e, 7)
    assert abs(float(r[..., 6]) - math.cos(ang)) < 1e-2 and abs(float(r[..., 7]) - math.sin(ang)) < 1e-2


def test_rmsnorm_closed_form():
    n = M.RMSNorm(8, eps=0.0)
    x = torch.arange(1.0, 9.0).view(1, 8)
    torch.testing.assert_close(n(x), x / math.sqrt(float((x * x).mean())))


def test_kv_cache_update_bookkeeping(monkeypatch):
    oracle_backend.install(monkeypatch, M)
    c = M.KVCache(2, 30, 1, 128, L=6, R=16, dtype=torch.float32, K=4)
    assert c.k_cache.shape == (2, 1, 32, 128) and c.codes.shape == (2, 1, 1, 32) and c.codes.dtype == torch.int32
    c.planes_words = oracle_backend.planes_to_words(torch.randn(6, 4, 128))
    g = torch.Generator().manual_seed(4)
    k = torch.randn(2, 5, 1, 128, generator=g); v = torch.randn(2, 5, 1, 128, generator=g)
    c.update(torch.arange(3, 8), k, v, hash_keys=True)
    assert c.lens.tolist() == [8, 8] and int(c.prefill_len) == 8
    assert torch.equal(c.k_cache[:, 0, 3:8], k[:, :, 0]) and torch.equal(c.v_cache[:, 0, 3:8], v[:, :, 0])
    torch.testing.assert_close(c.v_norm[:, 0, 3:8].float(), v[:, :, 0].norm(dim=-1), rtol=2e-3, atol=1e-3)
    k1 = torch.randn(2, 1, 1, 128, generator=g); v1 = torch.randn(2, 1, 1, 128, generator=g)
    c.update(torch.tensor([8]), k1, v1, hash_keys=True)                                 # decode step: device positions
    assert c.lens.tolist() == [9, 9] and torch.equal(c.k_cache[:, 0, 8], k1[:, 0, 0])
    c.update(torch.tensor([2]), k1, v1)                                                 # earlier position: the length follows it
    assert c.lens.tolist() == [3, 3]
    before = c.k_cache.clone()
    c.update(torch.tensor([32]), k1, v1)                                                # outside the cache: nothing written
    assert c.lens.tolist() == [3, 3] and torch.equal(c.k_cache, before)
    with pytest.raises(RuntimeError, match="out-of-bounds"):
        c.update(torch.arange(30, 35), k, v)
    with pytest.raises(AssertionError):
        c.update(torch.arange(4), k, v)


def test_kv_cache_update_takes_any_position_tensor(monkeypatch):
    """GPT-FAST/model.py:208-226 writes with an advanced index, so any position
    tensor is legal there: scattered positions, a descending order, two runs.  Every
    buffer must end up as that indexed write leaves it (codes and norms as a cache
    that received the same rows in one ascending piece holds them)."""
    oracle_backend.install(monkeypatch, M)
    planes = oracle_backend.planes_to_words(torch.randn(6, 4, 128, generator=torch.Generator().manual_seed(40)))
    g = torch.Generator().manual_seed(41)
    pos = torch.tensor([9, 10, 11, 3, 20, 19, 2])
    k = torch.randn(2, 7, 1, 128, generator=g); v = torch.randn(2, 7, 1, 128, generator=g)
    c = M.KVCache(2, 30, 1, 128, L=6, R=16, dtype=torch.float32, K=4)
    c.planes_words = planes
    c.update(pos, k, v, hash_keys=True)
    want_k = torch.zeros_like(c.k_cache); want_v = torch.zeros_like(c.v_cache)
    want_k[:, :, pos] = k.permute(0, 2, 1, 3); want_v[:, :, pos] = v.permute(0, 2, 1, 3)
    assert torch.equal(c.k_cache, want_k) and torch.equal(c.v_cache, want_v)
    assert c.lens.tolist() == [21, 21]
    # the same rows given to a second cache in ascending order, one piece per position
    d = M.KVCache(2, 30, 1, 128, L=6, R=16, dtype=torch.float32, K=4)
    d.planes_words = planes
    for i in torch.argsort(pos).tolist():
        d.update(pos[i:i + 1], k[:, i:i + 1], v[:, i:i + 1], hash_keys=True, pos0=int(pos[i]))
    assert torch.equal(c.codes, d.codes) and torch.equal(c.v_norm, d.v_norm)
    e = M.KVCache(2, 30, 1, 128, L=6, R=16, dtype=torch.float32, K=4)
    with pytest.raises(RuntimeError, match="out-of-bounds"):
        e.update(torch.tensor([4, 32, 5]), k[:, :3], v[:, :3])
    with pytest.raises(RuntimeError, match="out-of-bounds"):
        e.update(torch.tensor([4, -1]), k[:, :2], v[:, :2])


def test_sparse_decode_with_an_all_covering_window_reproduces_dense_tokens(monkeypatch):
    """With no sink, no heavy budget and a window longer than the context the
    list is every cached row exactly once (sparse.py:70-84), so greedy decoding
    through the sparse hook must give the dense run's tokens.  (A heavy budget
    would list sink / window rows twice, as the reference does.)"""
    oracle_backend.install(monkeypatch, M)
    model = toy_model(sink_size=0, window_size=4096, heavy_const=0)
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(0, 211, (2, 19), generator=g)
    seq_d, st_d = gen.generate(model, prompt, 9, decode_type="dense")
    seq_s, st_s = gen.generate(model, prompt, 9, decode_type="sparse")
    assert seq_d.shape == (2, 28) and torch.equal(seq_d[:, :19], prompt)
    assert torch.equal(seq_s, seq_d)
    assert st_s["decode_only_tokens"] == 16 and st_s["graph"] is False


def test_decode_steps_equal_one_long_prefill(monkeypatch):
    """Logits of position t from step-by-step dense decoding equal those of a
    single causal pass over the whole sequence (cache + rotary bookkeeping)."""
    oracle_backend.install(monkeypatch, M)
    model = toy_model(seed=1)
    g = torch.Generator().manual_seed(6)
    ids = torch.randint(0, 211, (1, 14), generator=g)
    model.setup_caches(1, 16)
    full = model(ids, torch.arange(14), pos0=0)
    for layer in model.layers:
        layer.attention.kv_cache.lens.zero_()
    step = [model(ids[:, :6], torch.arange(6), pos0=0)[:, -1]]
    for t in range(6, 14):
        step.append(model(ids[:, t:t + 1], torch.tensor([t]))[:, -1])
    torch.testing.assert_close(torch.stack(step, 1), full[:, 5:], rtol=2e-4, atol=2e-4)
    # a second block prefilled on top of the cache (explicit mask path)
    for layer in model.layers:
        layer.attention.kv_cache.lens.zero_()
    model(ids[:, :6], torch.arange(6), pos0=0)
    tail = model(ids[:, 6:], torch.arange(6, 14), pos0=6)
    torch.testing.assert_close(tail, full[:, 6:], rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("sparse", [True, False])
def test_a_cache_reused_for_a_shorter_prompt_forgets_the_longer_one(monkeypatch, sparse):
    """A long prompt, then a shorter one on the same caches through the public
    forward calls (no generate(), nothing reset by hand): rows the longer sequence
    left behind are past the current position and must be neither scored nor
    attended (GPT-FAST/model.py:486-487 masks by the position every step)."""
    oracle_backend.install(monkeypatch, M)
    g = torch.Generator().manual_seed(8)
    long_ids = torch.randint(0, 211, (1, 40), generator=g)
    short_ids = torch.randint(0, 211, (1, 12), generator=g)

    def run(model, ids, n_prompt):
        fwd = model.sparse_forward if sparse else model.forward
        out = [fwd(ids[:, :n_prompt], torch.arange(n_prompt), pos0=0)[:, -1]]
        for t in range(n_prompt, ids.shape[1]):
            out.append(fwd(ids[:, t:t + 1], torch.tensor([t]))[:, -1])
        return torch.stack(out, 1)

    used = toy_model(seed=3, heavy_const=5)
    used.setup_caches(1, 48)
    run(used, long_ids, 30)
    assert used.layers[0].attention.kv_cache.lens.tolist() == [40]
    have = run(used, short_ids, 7)
    assert used.layers[0].attention.kv_cache.lens.tolist() == [12]
    fresh = toy_model(seed=3, heavy_const=5)
    fresh.setup_caches(1, 48)
    want = run(fresh, short_ids, 7)
    torch.testing.assert_close(have, want, rtol=0, atol=0)


def test_sparse_hook_with_small_budget_keeps_cache_codes_consistent(monkeypatch):
    oracle_backend.install(monkeypatch, M)
    model = toy_model(seed=2, heavy_const=3)
    g = torch.Generator().manual_seed(7)
    prompt = torch.randint(0, 211, (1, 25), generator=g)
    seq, _ = gen.generate(model, prompt, 5, decode_type="sparse")
    assert seq.shape == (1, 30)
    attn = model.layers[1].attention
    cache = attn.kv_cache
    n = int(cache.lens[0])
    assert n == 29                                                                       # prompt + 4 decoded positions
    # every cached code equals the hash of the cached key
    want = orc.hard_hash_keys(cache.k_cache[:, :, :n].permute(0, 2, 1, 3), attn.planes)  # [B,n,H,L]
    import numpy as np
    have = orc.unpack_code_words(cache.codes[:, :, :, :n].numpy().view(np.uint32), 6, 4)  # [B,H,L,n]
    assert torch.equal(torch.from_numpy(have).permute(0, 3, 1, 2), want)


def test_generate_refuses_a_request_longer_than_the_model_allows():
    """Prompt + new tokens beyond block_size would decode past the end of the
    cache; the harness says so before launching anything."""
    model = toy_model()
    prompt = torch.randint(0, 211, (1, 250))
    with pytest.raises(ValueError, match="block_size"):
        gen.generate(model, prompt, 7, decode_type="sparse")          # 257 > 256


def test_sample_is_greedy():
    logits = torch.tensor([[[0.1, 2.0, -1.0], [3.0, 0.0, 0.5]]])
    tok, probs = gen.sample(logits)
    assert tok.tolist() == [[0]] and tok.dtype == torch.int and abs(float(probs.sum()) - 1) < 1e-6
