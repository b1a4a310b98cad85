"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).
CPU: the oracle still reproduces them.  GPU: the HIP kernels reproduce them."""
import os

import numpy as np
import pytest
import torch

from oracle import socket_oracle as orc

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(GOLD, name + ".npz"), allow_pickle=False))


def bf16(a):
    return torch.from_numpy(a.copy()).view(torch.bfloat16)


def f16(a):
    return torch.from_numpy(a.copy()).view(torch.float16)


# ------------------------------------------------------------------------------- CPU: oracle drift
def test_oracle_reproduces_hash_fixture():
    f = load("hash")
    keys, planes = bf16(f["keys_bf16"]).float(), bf16(f["planes_bf16"]).float()
    codes = orc.hard_hash_keys(keys, planes)
    dec = torch.from_numpy(f["decided"])
    assert torch.equal(codes[dec], torch.from_numpy(f["codes"])[dec])
    words = orc.pack_code_words(f["codes"].transpose(0, 2, 3, 1), int(f["P"]))
    assert np.array_equal(words, f["words"])
    assert torch.equal(orc.value_norm(bf16(f["vals_bf16"])), f16(f["v_norm_f16"]))


def test_oracle_reproduces_score_select_attend_soft_hash_fixtures():
    f = load("score")
    q, codes, vn = torch.from_numpy(f["q_probs"]), torch.from_numpy(f["codes"]), f16(f["v_norm_f16"]).float()
    B, Hq, L, R = q.shape
    G, T = Hq // codes.shape[1], codes.shape[-1]
    allowed = (torch.arange(T)[None, None] < torch.from_numpy(f["lens"])[:, None, None]).expand(B, Hq, T)
    got = orc.collision_score(q, codes.repeat_interleave(G, 1), allowed, vn.repeat_interleave(G, 1))
    assert torch.equal(got, torch.from_numpy(f["scores"]))

    f = load("select")
    s, lens = torch.from_numpy(f["scores"]), f["lens"]
    for b in range(s.shape[0]):
        n = int(lens[b])
        for h in range(s.shape[1]):
            heavy = orc.topk_lower_index_first(s[b, h, :n], int(f["M"])).to(torch.int32)
            row = torch.cat([torch.from_numpy(orc.base_indices(n, int(f["sink"]), int(f["window"]))), heavy])
            assert torch.equal(row, torch.from_numpy(f["sparse_list"])[b, h, :row.numel()])

    f = load("attend")
    out = orc.sparse_attend_textbook(bf16(f["q_bf16"]), bf16(f["k_bf16"]), bf16(f["v_bf16"]),
                                     torch.from_numpy(f["sparse_list"]), torch.from_numpy(f["sparse_len"]))
    np.testing.assert_allclose(out.numpy(), f["out_f64"], rtol=1e-12, atol=1e-14)

    f = load("soft_hash")
    q, planes = torch.from_numpy(f["q"]), torch.from_numpy(f["planes"])
    torch.testing.assert_close(orc.soft_hash(q, planes, torch.from_numpy(f["protos"]), 1.0),
                               torch.from_numpy(f["probs"]), rtol=1e-5, atol=1e-9)
    torch.testing.assert_close(orc.soft_hash(q, planes, orc.hypercube_protos_T(planes.shape[1]), 0.3),
                               torch.from_numpy(f["probs_cube_t03"]), rtol=1e-5, atol=1e-9)


# ------------------------------------------------------------------------------- GPU: HIP vs fixtures
@pytest.mark.gpu
def test_hip_hash_reproduces_fixture(dev):
    from socket_amd import hash_cache
    f = load("hash")
    L, P = int(f["L"]), int(f["P"])
    keys, vals, planes = bf16(f["keys_bf16"]).to(dev), bf16(f["vals_bf16"]).to(dev), bf16(f["planes_bf16"]).to(dev)
    B, S, Hkv, _ = keys.shape
    codes = torch.zeros((B, Hkv, hash_cache.words_per_key(L, P), 16), dtype=torch.int32, device=dev)
    v_norm = torch.zeros((B, Hkv, 16), dtype=torch.float16, device=dev)
    hash_cache.hash_keys_into(keys, vals, hash_cache.permute_planes(planes), codes, v_norm, L, P, t0=0, layout="bshd")
    have = hash_cache.unpack_codes(codes, L, P, 0, S, layout="bthl").cpu()
    dec = torch.from_numpy(f["decided"])
    assert torch.equal(have[dec], torch.from_numpy(f["codes"])[dec])
    want_vn = f16(f["v_norm_f16"]).permute(0, 2, 1).float()
    torch.testing.assert_close(v_norm[..., :S].float().cpu(), want_vn, rtol=1e-3, atol=1e-3)


@pytest.mark.gpu
def test_hip_score_select_attend_soft_hash_reproduce_fixtures(dev):
    from socket_amd import hash_cache, socket_kernels, sparse
    f = load("score")
    P = int(f["P"])
    codes = torch.from_numpy(f["codes"])
    B, Hkv, L, T = codes.shape
    Tcap = (T + 7) // 8 * 8
    words = np.zeros((B, Hkv, orc.words_per_key(L, P), Tcap), dtype=np.uint32)
    words[..., :T] = orc.pack_code_words(f["codes"], P)
    vn = torch.zeros((B, Hkv, Tcap), dtype=torch.float16)
    vn[..., :T] = f16(f["v_norm_f16"])
    packed = torch.from_numpy(words.view(np.int32)).to(dev)
    lens = torch.from_numpy(f["lens"]).to(dev)
    got = hash_cache.score_packed(torch.from_numpy(f["q_probs"]).to(dev), packed, vn.to(dev), T, P, lens=lens).cpu()
    assert torch.equal(got, torch.from_numpy(f["scores"]))                      # fp32 table: bit-exact
    got16 = hash_cache.score_packed(bf16(f["q_probs_bf16"]).to(dev), packed, vn.to(dev), T, P, lens=lens).cpu()
    want16 = torch.from_numpy(f["scores_bf16_table"])
    rel = ((got16 - want16).abs() / want16.abs().clamp_min(1e-30)).nan_to_num(0).max()
    assert rel <= 1e-5

    f = load("select")
    sl, ln = sparse.select_list(torch.from_numpy(f["scores"]).to(dev), int(f["sink"]), int(f["window"]), int(f["M"]),
                                lens=torch.from_numpy(f["lens"]).to(dev))
    assert torch.equal(sl.cpu(), torch.from_numpy(f["sparse_list"]))
    assert torch.equal(ln.cpu(), torch.from_numpy(f["sparse_len"]))

    f = load("attend")
    out = socket_kernels.sparse_attention_fwd(bf16(f["q_bf16"]).to(dev), bf16(f["k_bf16"]).to(dev),
                                              bf16(f["v_bf16"]).to(dev), torch.from_numpy(f["sparse_list"]).to(dev),
                                              torch.from_numpy(f["sparse_len"]).to(dev))
    assert float((out.float().cpu() - torch.from_numpy(f["out_f64"]).float()).abs().max()) <= 2e-2

    f = load("soft_hash")
    q, planes = torch.from_numpy(f["q"]).to(dev), torch.from_numpy(f["planes"]).to(dev)
    p = hash_cache.soft_hash(q, planes, torch.from_numpy(f["protos"]).to(dev), 1.0, 2)
    torch.testing.assert_close(p.cpu(), torch.from_numpy(f["probs"]), rtol=2e-5, atol=1e-9)
    cube = orc.hypercube_protos_T(planes.shape[1]).to(dev)
    p = hash_cache.soft_hash(q, planes, cube, 0.3, 4)
    torch.testing.assert_close(p.cpu(), torch.from_numpy(f["probs_cube_t03"]), rtol=2e-5, atol=1e-9)
