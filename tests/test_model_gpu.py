"""The model hook and the generation harness on the MI355X: every attention
step goes through libsocket_hip; the oracle stand-ins of tests/oracle_backend.py
are swapped in only to produce the expected values."""
import copy

import numpy as np
import pytest
import torch

from oracle import socket_oracle as orc
from socket_amd import generate as gen
from socket_amd import hash_cache
from socket_amd import model as M
from tests import oracle_backend

pytestmark = pytest.mark.gpu


def toy_args(**kw):
    base = dict(block_size=1024, vocab_size=331, n_layer=2, n_head=4, n_local_heads=2, dim=512, L=20, K=10, R=1024,
                heavy_const=48, sink_size=4, window_size=16, rope_base=10000)
    base.update(kw)
    return M.ModelArgs(**base)


def toy_model(dev, dtype=torch.float32, seed=0, **kw):
    torch.manual_seed(seed)
    model = M.Transformer(toy_args(**kw)).eval()
    with torch.no_grad():
        for name, p in model.named_parameters():
            if not name.endswith("norm.weight"):
                p.normal_(0, 0.06)
        for blk in model.layers:
            blk.attention.planes.normal_(0, 1.0)
            blk.attention.protos_T.copy_(orc.hypercube_protos_T(model.config.K) * 3.0)
    return model.to(device=dev, dtype=dtype)


def _reset(model):
    for layer in model.layers:
        layer.attention.kv_cache.lens.zero_()


@torch.no_grad()
def _run_steps(model, ids, n_prompt, sparse=True):
    fwd = model.sparse_forward if sparse else model.forward
    dev = ids.device
    logits = [fwd(ids[:, :n_prompt], torch.arange(n_prompt, device=dev), pos0=0, last_only=True)[:, -1]]
    for t in range(n_prompt, ids.shape[1]):
        logits.append(fwd(ids[:, t:t + 1], torch.tensor([t], device=dev))[:, -1])
    return torch.stack(logits, 1).float().cpu()


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-3), (torch.bfloat16, 6e-2)])
def test_sparse_hook_matches_oracle_attention(dev, monkeypatch, dtype, tol):
    """Same model, same cache contents; the decode attention once through the
    HIP kernels and once through the oracle (scorer -> stable top-k -> list ->
    textbook softmax).  The selected lists coincide (scores are bit-exact), so
    the logits agree to the attention tolerance."""
    model = toy_model(dev, dtype)
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 331, (2, 150), generator=g).to(dev)
    model.setup_caches(2, 160)
    have = _run_steps(model, ids, 140)
    _reset(model)
    oracle_backend.install(monkeypatch, M, hashing=False, sparse=True, dense=False)
    want = _run_steps(model, ids, 140)
    assert torch.isfinite(have).all()
    scale = float(want.abs().max())
    assert float((have - want).abs().max()) <= tol * max(scale, 1.0)
    if dtype == torch.float32:
        assert torch.equal(have.argmax(-1), want.argmax(-1))


@pytest.mark.parametrize("sparse", [True, False])
def test_a_cache_reused_for_a_shorter_prompt_forgets_the_longer_one(dev, sparse):
    """A long prompt and some decode steps, then a shorter prompt on the same caches
    through the public forward calls: identical logits to a model whose caches
    never held the longer sequence."""
    g = torch.Generator().manual_seed(21)
    long_ids = torch.randint(0, 331, (2, 300), generator=g).to(dev)
    short_ids = torch.randint(0, 331, (2, 90), generator=g).to(dev)
    used = toy_model(dev, torch.bfloat16, seed=9)
    used.setup_caches(2, 320)
    _run_steps(used, long_ids, 290, sparse=sparse)
    assert used.layers[0].attention.kv_cache.lens.tolist() == [300, 300]
    have = _run_steps(used, short_ids, 80, sparse=sparse)
    assert used.layers[0].attention.kv_cache.lens.tolist() == [90, 90]
    fresh = toy_model(dev, torch.bfloat16, seed=9)
    fresh.setup_caches(2, 320)
    want = _run_steps(fresh, short_ids, 80, sparse=sparse)
    assert torch.equal(have, want)


def test_dense_below_crossover_takes_the_dense_kernel_and_keeps_the_hash_state(dev):
    """ModelArgs.dense_below_crossover on a short cache (where dense attention is priced
    below score + select + attend): the sparse hook's logits are the dense hook's, plain
    and fused step alike, and the cache's codes are those a sparse run writes."""
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, 331, (2, 150), generator=g).to(dev)
    plain = toy_model(dev, torch.bfloat16)
    plain.setup_caches(2, 160)
    _run_steps(plain, ids, 140)
    # (layer 0: its keys do not depend on any attention output, so both runs cache the same ones)
    want_sparse_codes = plain.layers[0].attention.kv_cache.codes.clone()
    _reset(plain)
    want = _run_steps(plain, ids, 140, sparse=False)
    model = toy_model(dev, torch.bfloat16, dense_below_crossover=True)
    model.setup_caches(2, 160)
    c = model.layers[0].attention.kv_cache
    s_us, d_us = hash_cache.step_cost_estimate(2, 4, 2, 128, c.k_cache.shape[2], 20, 10, 1024, 48, 4, 16)
    assert d_us < s_us
    have = _run_steps(model, ids, 140)
    assert torch.equal(have, want)
    assert torch.equal(model.layers[0].attention.kv_cache.codes, want_sparse_codes)
    assert model.layers[1].attention.kv_cache.codes.any()
    # the fused single-token step (what the decode graph records)
    step = gen.DecodeGraph(model, 2, "sparse", dev)
    ref = gen.DecodeGraph(plain, 2, "dense", dev)
    for dg in (step, ref):
        dg.tok.copy_(ids[:, 149:150].to(torch.int))
        dg.pos.fill_(149)
    a, _ = step._step()
    b, _ = ref._step()
    assert torch.equal(a, b)


def test_eager_decode_step_at_a_position_outside_the_cache_writes_nothing(dev):
    """The unfused single-token path with a device-side position past the cache:
    no row is written and the length stays (the fused path and the hashing kernel
    behave the same way)."""
    c = M.KVCache(2, 64, 2, 128, L=20, R=1024, dtype=torch.bfloat16, K=10, device=dev)
    g = torch.Generator().manual_seed(22)
    k = torch.randn(2, 1, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    c.planes_words = hash_cache_planes(dev)
    c.update(torch.tensor([5], device=dev), k, k, hash_keys=True)
    assert c.lens.tolist() == [6, 6] and torch.equal(c.k_cache[:, :, 5], k[:, 0])
    snap = (c.k_cache.clone(), c.codes.clone(), c.v_norm.clone())
    c.update(torch.tensor([64], device=dev), k, k, hash_keys=True)
    assert c.lens.tolist() == [6, 6]
    assert torch.equal(c.k_cache, snap[0]) and torch.equal(c.codes, snap[1]) and torch.equal(c.v_norm, snap[2])


def test_kv_cache_update_scatters_rows_codes_and_norms(dev):
    """Positions in any order with the reference's calling convention (precomputed
    v_norm and k_hard, GPT-FAST/model.py:222-226) and with the fused hashing: every
    buffer as the reference's advanced-index write leaves it."""
    g = torch.Generator().manual_seed(24)
    pos = torch.tensor([9, 10, 11, 3, 40, 39, 2], device=dev)
    k = torch.randn(2, 7, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(2, 7, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    kh = torch.randint(0, 1024, (2, 7, 2, 20), generator=g).to(torch.int16).to(dev)
    vn = torch.rand(2, 7, 2, generator=g).to(torch.float16).to(dev)
    c = M.KVCache(2, 64, 2, 128, L=20, R=1024, dtype=torch.bfloat16, K=10, device=dev)
    c.update(pos, k, v, v_norm=vn, k_hard=kh)
    want_k = torch.zeros_like(c.k_cache)
    want_k[:, :, pos] = k.permute(0, 2, 1, 3)
    assert torch.equal(c.k_cache, want_k) and c.lens.tolist() == [41, 41]
    assert torch.equal(c.k_hard(64)[:, :, pos], kh.permute(0, 2, 1, 3))
    assert torch.equal(c.v_norm[:, :, pos], vn.permute(0, 2, 1))
    untouched = torch.ones(64, dtype=torch.bool, device=dev)
    untouched[pos] = False
    assert not c.k_hard(64)[:, :, untouched].any() and not c.v_norm[:, :, untouched].any()
    # fused hashing: the same as one position at a time
    a = M.KVCache(2, 64, 2, 128, L=20, R=1024, dtype=torch.bfloat16, K=10, device=dev)
    b = M.KVCache(2, 64, 2, 128, L=20, R=1024, dtype=torch.bfloat16, K=10, device=dev)
    a.planes_words = b.planes_words = hash_cache_planes(dev)
    a.update(pos, k, v, hash_keys=True)
    for i in range(7):
        b.update(pos[i:i + 1], k[:, i:i + 1], v[:, i:i + 1], hash_keys=True)
    assert torch.equal(a.codes, b.codes) and torch.equal(a.v_norm, b.v_norm) and torch.equal(a.v_cache, b.v_cache)


def hash_cache_planes(dev):
    from socket_amd import hash_cache
    g = torch.Generator().manual_seed(23)
    return hash_cache.permute_planes(torch.randn(20, 10, 128, generator=g).to(dev))


def test_sparse_hook_with_64_dim_heads(dev, monkeypatch):
    """A model whose heads are 64 wide (the hashing kernel contracts over 128
    coordinates: rows and planes are zero-padded on the way in): cached codes
    equal the oracle's hash of the cached keys, logits equal the oracle hook's."""
    model = toy_model(dev, torch.float32, n_head=8, n_local_heads=4)
    assert model.config.head_dim == 64
    g = torch.Generator().manual_seed(31)
    ids = torch.randint(0, 331, (2, 120), generator=g).to(dev)
    model.setup_caches(2, 128)
    have = _run_steps(model, ids, 110)
    attn, cache = model.layers[1].attention, model.layers[1].attention.kv_cache
    # (the kernel contracts keys and planes rounded to bf16, with fp32 accumulation)
    keys = cache.k_cache[:, :, :120].permute(0, 2, 1, 3).cpu().to(torch.bfloat16).float()
    proj = orc.projections_f64(keys, attn.planes.float().cpu().to(torch.bfloat16).float())
    clear = (proj.abs() > 1e-3 * proj.abs().mean()).all(-1)
    assert clear.float().mean() > 0.9
    assert torch.equal(cache.k_hard(120).cpu().permute(0, 2, 1, 3)[clear], orc.pack_bits(proj >= 0)[clear])
    _reset(model)
    oracle_backend.install(monkeypatch, M, hashing=False, sparse=True, dense=False)
    want = _run_steps(model, ids, 110)
    assert float((have - want).abs().max()) <= 2e-3 * max(float(want.abs().max()), 1.0)


def test_cache_hash_state_after_prefill_and_decode(dev):
    """Codes and value norms written by the fused append equal the oracle's hash
    of the cached rows wherever the fp64 projection is clear of zero."""
    model = toy_model(dev, torch.bfloat16, seed=3)
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 331, (2, 70), generator=g).to(dev)
    model.setup_caches(2, 80)
    _run_steps(model, ids, 61)
    for layer in model.layers:
        attn, cache = layer.attention, layer.attention.kv_cache
        assert cache.lens.tolist() == [70, 70]
        keys = cache.k_cache[:, :, :70].permute(0, 2, 1, 3).float().cpu()           # [B,T,H,D]
        planes = attn.planes.float().cpu()
        proj = orc.projections_f64(keys, planes.to(torch.bfloat16).float())          # the kernel hashes with bf16 planes
        want = orc.pack_bits(proj >= 0)                                              # [B,T,H,L]
        have = cache.k_hard(70).cpu()                                                # [B,H,T,L]
        assert have.dtype == torch.int16 and tuple(have.shape) == (2, 2, 70, 20)
        clear = (proj.abs() > 1e-3 * proj.abs().mean()).all(-1)                      # every bit of the code is safe
        assert clear.float().mean() > 0.9
        assert torch.equal(have.permute(0, 2, 1, 3)[clear], want[clear])
        vn = cache.v_cache[:, :, :70].float().norm(dim=-1).cpu()
        torch.testing.assert_close(cache.v_norm[:, :, :70].float().cpu(), vn, rtol=2e-3, atol=1e-3)


def test_hard_hash_keys_on_device_uses_reference_layout(dev):
    attn = M.Attention(toy_args()).to(dev)
    g = torch.Generator().manual_seed(4)
    attn.planes.copy_(torch.randn(20, 10, 128, generator=g))
    keys = torch.randn(2, 37, 2, 128, generator=g).to(torch.bfloat16)
    have = attn.hard_hash_keys(keys.to(dev)).cpu()
    assert have.dtype == torch.int16 and tuple(have.shape) == (2, 37, 2, 20)
    proj = orc.projections_f64(keys.float(), attn.planes.cpu().to(torch.bfloat16).float())
    clear = (proj.abs() > 1e-3 * proj.abs().mean()).all(-1)
    assert torch.equal(have[clear], orc.pack_bits(proj >= 0)[clear])


def test_kv_cache_takes_precomputed_codes_in_the_reference_convention(dev):
    c = M.KVCache(2, 64, 2, 128, L=20, R=1024, dtype=torch.bfloat16, K=10, device=dev)
    g = torch.Generator().manual_seed(5)
    k = torch.randn(2, 9, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(2, 9, 2, 128, generator=g).to(torch.bfloat16).to(dev)
    k_hard = torch.randint(0, 1024, (2, 9, 2, 20), generator=g).to(torch.int16).to(dev)
    v_norm = torch.rand(2, 9, 2, generator=g).to(torch.float16).to(dev)
    c.update(torch.arange(5, 14, device=dev), k, v, v_norm=v_norm, k_hard=k_hard)
    assert c.lens.tolist() == [14, 14]
    assert torch.equal(c.k_hard(14)[:, :, 5:14], k_hard.permute(0, 2, 1, 3))
    assert torch.equal(c.v_norm[:, :, 5:14], v_norm.permute(0, 2, 1))
    assert torch.equal(c.k_cache[:, :, 5:14], k.permute(0, 2, 1, 3))


@pytest.mark.parametrize("decode_type", ["sparse", "dense"])
def test_decode_graph_replays_equal_the_eager_step(dev, decode_type):
    model = toy_model(dev, torch.bfloat16, seed=6)
    g = torch.Generator().manual_seed(6)
    prompt = torch.randint(0, 331, (2, 200), generator=g).to(dev)
    seq_g, st = gen.generate(model, prompt, 12, decode_type=decode_type, use_graph=True, check_graph=True)
    assert st["graph"] and st["graph_check"]["same_token"]
    assert st["graph_check"]["max_abs_logit_diff"] <= 1e-2
    seq_e, st_e = gen.generate(model, prompt, 12, decode_type=decode_type, use_graph=False)
    assert not st_e["graph"]
    assert torch.equal(seq_g, seq_e)


def test_generate_up_to_the_last_row_of_the_cache_and_no_further(dev):
    """prompt + new tokens == block_size: the last decoded position is the cache's
    last row; graph and eager runs agree.  One token more is refused on the host."""
    model = toy_model(dev, torch.bfloat16, seed=8)
    g = torch.Generator().manual_seed(8)
    prompt = torch.randint(0, 331, (1, 1000), generator=g).to(dev)
    seq_g, st = gen.generate(model, prompt, 24, decode_type="sparse", use_graph=True)
    assert seq_g.shape[1] == 1024 and model.max_seq_length == 1024
    assert int(model.layers[0].attention.kv_cache.lens[0]) == 1023      # the last token is sampled, not appended
    seq_e, _ = gen.generate(model, prompt, 24, decode_type="sparse", use_graph=False)
    assert torch.equal(seq_g, seq_e)
    with pytest.raises(ValueError, match="block_size"):
        gen.generate(model, prompt, 25, decode_type="sparse")


def test_all_covering_window_reproduces_dense_tokens_on_device(dev):
    model = toy_model(dev, torch.float32, seed=7, sink_size=0, window_size=4096, heavy_const=0)
    g = torch.Generator().manual_seed(7)
    prompt = torch.randint(0, 331, (2, 90), generator=g).to(dev)
    seq_d, _ = gen.generate(model, prompt, 10, decode_type="dense")
    seq_s, _ = gen.generate(model, prompt, 10, decode_type="sparse")
    assert torch.equal(seq_s, seq_d)


def test_load_random_model_and_warmup(dev):
    model = gen.load_random_model(toy_args(n_layer=1), dev, torch.bfloat16, seed=1)
    assert model.layers[0].attention.planes.dtype == torch.bfloat16 and model.norm.weight.eq(1).all()
    assert 0.015 < float(model.output.weight.float().std()) < 0.025
    model.setup_caches(1, 512)
    gen.warmup_sparse_decode(model, dev, T=300)


# ---------------------------------------------------------------- fused single-token helpers
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_rope_append_equals_the_torch_chain(dev, dtype):
    g = torch.Generator().manual_seed(11)
    B, Hq, Hkv, D, Tcap = 3, 4, 2, 128, 64
    from socket_amd import decode_ops
    qkv = torch.randn(B, 1, (Hq + 2 * Hkv) * D, generator=g).to(dtype).to(dev)
    table = M.precompute_freqs_cis(80, D, 10000).to(dev)
    for pos in (0, 5, 63):
        kc = torch.zeros(B, Hkv, Tcap, D, dtype=dtype, device=dev)
        vc = torch.zeros_like(kc)
        lens = torch.tensor([3, 10, 70], dtype=torch.int32, device=dev)
        ip = torch.tensor([pos], device=dev)
        q, kn, vn = decode_ops.rope_append(qkv, table, ip, kc, vc, lens, Hq, Hkv, return_new=True)
        qs, ks, vs = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        want_q = M.apply_rotary_emb(qs.view(B, 1, Hq, D), table[ip])
        want_k = M.apply_rotary_emb(ks.view(B, 1, Hkv, D), table[ip])
        assert torch.equal(q, want_q[:, 0]) and torch.equal(kn, want_k) and torch.equal(vn, vs.view(B, 1, Hkv, D))
        assert torch.equal(kc[:, :, pos], want_k[:, 0]) and torch.equal(vc[:, :, pos], vs.view(B, Hkv, D))
        kc[:, :, pos] = 0
        vc[:, :, pos] = 0
        assert not kc.any() and not vc.any()                                   # nothing else was touched
        assert lens.tolist() == [pos + 1] * 3                                  # the length follows the position
    # per-sequence positions; one of them outside the cache writes nothing
    kc = torch.zeros(B, Hkv, Tcap, D, dtype=dtype, device=dev)
    vc = torch.zeros_like(kc)
    lens = torch.zeros(B, dtype=torch.int32, device=dev)
    ip = torch.tensor([2, 64, 9], device=dev)
    decode_ops.rope_append(qkv, table, ip, kc, vc, lens, Hq, Hkv)
    assert lens.tolist() == [3, 0, 10] and not kc[1].any() and kc[0, :, 2].any() and kc[2, :, 9].any()


@pytest.mark.parametrize("Hq,Hkv,L,grouped,ftype", [(32, 8, 60, True, torch.bfloat16), (32, 8, 60, False, torch.float32),
                                                    (28, 4, 48, True, torch.bfloat16), (8, 8, 7, False, torch.bfloat16),
                                                    (16, 8, 33, True, torch.float32)])
def test_decode_prologue_equals_the_three_launches(dev, Hq, Hkv, L, grouped, ftype):
    """rope_append + hash of the new key + soft hash in one launch: every output
    bit for bit what the three launches leave (queries, K/V rows, lengths, packed
    codes, value norms, the probability table in either layout), rows elsewhere in
    the cache untouched, and positions outside the cache or the rotary table
    handled as the three launches handle them."""
    from socket_amd import decode_ops, hash_cache
    g = torch.Generator().manual_seed(100 + Hq + L)
    B, D, K, R, Tcap, n_pos = 4, 128, 10, 1024, 72, 70
    dt = torch.bfloat16
    qkv = (torch.randn(B, 1, (Hq + 2 * Hkv) * D, generator=g) * 2).to(dt).to(dev)
    table = M.precompute_freqs_cis(n_pos, D, 10000).to(ftype).to(dev)
    planes = (torch.randn(L, K, D, generator=g) * 0.3).to(dt).to(dev)
    protos_T = torch.randn(K, R, generator=g).to(dt).to(dev)
    words = hash_cache.permute_planes(planes)
    NW = hash_cache.words_per_key(L, K)

    def fresh():
        gg = torch.Generator().manual_seed(5)
        kc = torch.randn(B, Hkv, Tcap, D, generator=gg).to(dt).to(dev)
        vc = torch.randn(B, Hkv, Tcap, D, generator=gg).to(dt).to(dev)
        codes = torch.randint(0, 2 ** 31 - 1, (B, Hkv, NW, Tcap), generator=gg, dtype=torch.int32).to(dev)
        vn = torch.rand(B, Hkv, Tcap, generator=gg).to(torch.float16).to(dev)
        lens = torch.tensor([3, 10, 70, 1], dtype=torch.int32, device=dev)
        return kc, vc, codes, vn, lens

    # one position for all; one each, with one beyond the cache (72) and one inside the
    # cache but beyond the rotary table (70, 71)
    for ip in (torch.tensor([17], device=dev), torch.tensor([0, 69, 72, 71], device=dev),
               torch.tensor([5, -1, 33, 70], device=dev)):
        a, b = fresh(), fresh()
        q_a, kn, vn_new = decode_ops.rope_append(qkv, table, ip, a[0], a[1], a[4], Hq, Hkv, return_new=True)
        hash_cache.hash_keys_into(kn, vn_new, words, a[2], a[3], L, K, pos_b=ip.to(torch.int32).expand(B).contiguous(),
                                  layout="bshd")
        t_a = hash_cache.soft_hash(q_a, planes, protos_T, 1.0, Hkv, grouped=grouped)
        q_b, t_b = hash_cache.decode_prologue(qkv, table, ip, b[0], b[1], b[4], words, b[2], b[3], planes, protos_T,
                                              Hq, Hkv, grouped=grouped)
        assert torch.equal(q_a, q_b), ip.tolist()
        assert t_a.shape == t_b.shape and torch.equal(t_a, t_b), ip.tolist()
        for x, y, name in zip(a, b, ("k_cache", "v_cache", "codes", "v_norm", "lens")):
            assert torch.equal(x, y), (name, ip.tolist())
    # and the new key's codes are the hard hash of the rotated key (GPT-FAST/model.py:403-413)
    ip = torch.tensor([9], device=dev)
    kc, vc, codes, vn, lens = fresh()
    hash_cache.decode_prologue(qkv, table, ip, kc, vc, lens, words, codes, vn, planes, protos_T, Hq, Hkv)
    got = hash_cache.unpack_codes(codes, L, K, 9, 1, layout="bhlt")[..., 0].cpu()          # [B,Hkv,L]
    proj = torch.einsum("bhd,lkd->bhlk", kc[:, :, 9].double().cpu(), planes.double().cpu())
    want = ((proj >= 0).long() * (1 << torch.arange(K - 1, -1, -1))).sum(-1)
    decided = proj.abs().min(-1).values > 1e-3
    assert torch.equal(got.long()[decided], want[decided]) and float(decided.float().mean()) > 0.9
    assert torch.allclose(vn[:, :, 9].float().cpu(), vc[:, :, 9].float().norm(dim=-1).cpu(), rtol=1e-3)


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 1e-2), (torch.float32, 1e-6)])
def test_add_rmsnorm_and_silu_mul_equal_the_torch_chain(dev, dtype, tol):
    from socket_amd import decode_ops
    g = torch.Generator().manual_seed(12)
    x = torch.randn(5, 1, 4096, generator=g).to(dtype).to(dev)
    r = torch.randn(5, 1, 4096, generator=g).to(dtype).to(dev)
    norm = M.RMSNorm(4096, 1e-5).to(dev).to(dtype)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(4096, generator=g).to(dtype))
        h, y = decode_ops.add_rmsnorm(x, norm.weight, norm.eps, residual=r)
        assert torch.equal(h, x + r)
        want = norm(x + r)
        # the mean is summed in another order, so the scale can differ in its last bit:
        # in bf16 that shows in a few outputs, in fp32 in whole rows, by one ulp
        few = 0.02 if dtype == torch.bfloat16 else 1.0
        assert float((y.float() - want.float()).abs().max()) <= tol * float(want.float().abs().max())
        assert float((y != want).float().mean()) <= few
        h2, y2 = decode_ops.add_rmsnorm(x, norm.weight, norm.eps)
        assert h2 is x and float((y2 != norm(x)).float().mean()) <= few
        assert float((y2.float() - norm(x).float()).abs().max()) <= tol * float(want.float().abs().max())
        a = torch.randn(3, 1, 14336, generator=g).to(dtype).to(dev) * 3
        b = torch.randn(3, 1, 14336, generator=g).to(dtype).to(dev)
        got, want = decode_ops.silu_mul(a, b), torch.nn.functional.silu(a) * b
        assert float((got.float() - want.float()).abs().max()) <= tol * float(want.float().abs().max())
        assert float((got != want).float().mean()) <= few


@pytest.mark.parametrize("rows,N,K", [(1, 6144, 4096), (1, 4096, 14336), (4, 1000, 2048), (3, 4099, 4096), (2, 128256, 4096)])
def test_linear_rows_equals_the_fp32_product_rounded_once(dev, rows, N, K):
    """The matrix-vector kernel against the float64 product: within one bf16
    rounding of it (torch's own bf16 linear is held to the same bar here), and the
    gated form against the chain of three torch ops."""
    from socket_amd import decode_ops
    g = torch.Generator().manual_seed(N + K + rows)
    x = torch.randn(rows, 1, K, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    got = decode_ops.linear_rows(x, w)
    assert got.shape == (rows, 1, N) and got.dtype == torch.bfloat16
    exact = x.double() @ w.double().T
    scale = float(exact.abs().max())
    ulp = 2.0 ** -8                                                     # half a bf16 ulp relative, plus summation noise
    assert float((got.double() - exact).abs().max()) <= 1.5 * ulp * scale
    theirs = torch.nn.functional.linear(x, w)
    assert float((theirs.double() - exact).abs().max()) <= 1.5 * ulp * scale
    assert float((got != theirs).float().mean()) <= 0.1                 # last-bit differences only, and few
    if N <= 8192:
        wg = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16).to(dev)
        gated = decode_ops.linear_rows(x, w, wg)
        want = torch.nn.functional.silu(torch.nn.functional.linear(x, w)) * torch.nn.functional.linear(x, wg)
        assert float((gated.float() - want.float()).abs().max()) <= 3e-2 * float(want.float().abs().max())
    # shapes outside the kernel's range take torch's product
    x5 = torch.randn(5, 1, K, generator=g).to(torch.bfloat16).to(dev)
    assert torch.equal(decode_ops.linear_rows(x5, w), torch.nn.functional.linear(x5, w))


@pytest.mark.parametrize("rows,N,K,gate,res", [
    (1, 6144, 4096, False, True), (1, 6144, 4096, False, False), (1, 14336, 4096, True, True),
    (4, 1001, 2048, True, True), (3, 515, 8192, True, False), (2, 4099, 4096, True, True),
])
def test_norm_linear_rows_equals_the_two_launches(dev, rows, N, K, gate, res):
    """RMSNorm (with the residual add before it) inside the matrix-vector launch: h and
    the product equal add_rmsnorm followed by linear_rows bit for bit, also twice in a
    row and for an output count that does not fill the last workgroup; shapes the
    kernel does not take go through the two calls."""
    from socket_amd import decode_ops
    g = torch.Generator().manual_seed(N * 3 + K + rows)
    x = torch.randn(rows, 1, K, generator=g).to(torch.bfloat16).to(dev)
    r = torch.randn(rows, 1, K, generator=g).to(torch.bfloat16).to(dev) if res else None
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16).to(dev)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    wg = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16).to(dev) if gate else None
    x0, r0 = x.clone(), None if r is None else r.clone()
    h_want, xn = decode_ops.add_rmsnorm(x, nw, 1e-5, residual=r)
    y_want = decode_ops.linear_rows(xn, w, wg)
    for _ in range(2):
        h, y = decode_ops.norm_linear_rows(x, nw, 1e-5, r, w, wg)
        assert torch.equal(h, h_want) and torch.equal(y, y_want)
        assert (h is x) == (r is None)
    assert torch.equal(x, x0) and (r is None or torch.equal(r, r0))     # inputs untouched
    if not gate:
        x2 = torch.randn(2, 1, K, generator=g).to(torch.bfloat16).to(dev)
        h2, y2 = decode_ops.norm_linear_rows(x2, nw, 1e-5, None, w)
        assert torch.equal(y2, decode_ops.linear_rows(decode_ops.add_rmsnorm(x2, nw, 1e-5)[1], w))


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.bfloat16, 3e-2)])
@pytest.mark.parametrize("sparse", [True, False])
def test_fused_decode_step_equals_the_plain_one(dev, dtype, tol, sparse):
    model = toy_model(dev, dtype, seed=8)
    g = torch.Generator().manual_seed(13)
    ids = torch.randint(0, 331, (2, 60), generator=g).to(dev)
    model.setup_caches(2, 64)
    model.fused_decode = True
    fused = _run_steps(model, ids, 50, sparse=sparse)
    codes_fused = model.layers[1].attention.kv_cache.codes.clone()
    _reset(model)
    model.fused_decode = False
    plain = _run_steps(model, ids, 50, sparse=sparse)
    scale = float(plain.abs().max())
    assert float((fused - plain).abs().max()) <= tol * max(scale, 1.0)
    if sparse and dtype == torch.float32:
        assert torch.equal(codes_fused, model.layers[1].attention.kv_cache.codes)
