"""Pins for the CPU oracle (oracle/socket_oracle.py and its C twin).

The reference ships no tests or golden vectors for this path, so each oracle
function is pinned here by something it did not compute itself: a closed form,
an invariant of the mathematics, a library routine of a different kind, brute
force on tiny inputs, or the independently written C restatement.  Each check
is chosen so that a plausible slip (dropped term, wrong sign or index,
transposed operand, reversed bit order) fails it.
"""
import ctypes
import itertools
import math
import os

import numpy as np
import pytest
import torch

from oracle import socket_oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
C_LIB = os.path.join(os.path.dirname(HERE), "oracle", "libsocket_oracle_c.so")


@pytest.fixture(scope="module")
def clib():
    if not os.path.exists(C_LIB):
        import subprocess
        subprocess.run(["make", "-C", os.path.dirname(C_LIB), "all"], check=True)
    return ctypes.CDLL(C_LIB)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


# ------------------------------------------------------------------ pack / hash
def test_pack_bits_is_big_endian_brute_force():
    P = 5
    for r, bits in enumerate(itertools.product([0, 1], repeat=P)):       # first bit slowest = MSB
        got = int(orc.pack_bits(torch.tensor(bits, dtype=torch.bool)))
        assert got == r == int("".join(map(str, bits)), 2)
    # P = 10: all codes stay inside [0, 2^P)
    b = torch.rand(1000, 10) > 0.5
    c = orc.pack_bits(b)
    assert c.dtype == torch.int16 and int(c.min()) >= 0 and int(c.max()) < 1024


def test_hard_hash_closed_forms():
    g = torch.Generator().manual_seed(0)
    L, P, D = 6, 8, 32
    # planes = +-unit vectors -> the bits are sign bits of key coordinates
    coord = torch.randperm(D, generator=g)[:L * P].view(L, P) if L * P <= D else torch.randint(0, D, (L, P), generator=g)
    sign = torch.where(torch.rand(L, P, generator=g) > 0.5, 1.0, -1.0)
    planes = torch.zeros(L, P, D)
    planes.view(-1, D)[torch.arange(L * P), coord.view(-1)] = sign.view(-1)
    k = torch.randn(2, 7, 3, D, generator=g)
    codes = orc.hard_hash_keys(k, planes)
    bits = (k[..., coord] * sign) >= 0                                           # [2,7,3,L,P]
    assert torch.equal(codes, orc.pack_bits(bits))
    # scale invariance and complement under negation
    planes = torch.randn(L, P, D, generator=g)
    c1 = orc.hard_hash_keys(k, planes)
    assert torch.equal(orc.hard_hash_keys(3.7 * k, planes), c1)
    assert torch.equal(orc.hard_hash_keys(-k, planes).int(), (~c1.int()) & ((1 << P) - 1))
    # table-major twin agrees after the layout change
    c2 = orc.hard_hash_bhln(k.permute(0, 2, 1, 3), planes)                        # [B,H,L,N]
    assert torch.equal(c2, c1.permute(0, 2, 3, 1))
    # a projection of exactly zero hashes to bit 1 (>= 0)
    z = torch.zeros(1, 1, 1, D)
    assert int(orc.hard_hash_keys(z, planes)[0, 0, 0, 0]) == (1 << P) - 1


def test_hard_hash_against_c_double_loops(clib):
    g = torch.Generator().manual_seed(1)
    N, D, L, P = 50, 16, 5, 7
    keys = torch.randn(N, D, generator=g)
    planes = torch.randn(L, P, D, generator=g)
    out = np.zeros((N, L), dtype=np.int16)
    clib.oracle_c_hard_hash(_p(keys.numpy()), _p(planes.numpy()), _p(out), N, D, L, P)
    got = orc.hard_hash_keys(keys.view(1, N, 1, D), planes)[0, :, 0]
    proj = orc.projections_f64(keys.view(1, N, 1, D), planes)[0, :, 0]
    assert (proj.abs() > 1e-5).all()
    assert np.array_equal(got.numpy(), out)


# ------------------------------------------------------------------ soft hash
def test_hypercube_protos_match_pack_order():
    P = 6
    pt = orc.hypercube_protos_T(P)                        # [P,R]
    assert pt.shape == (P, 64) and set(pt.unique().tolist()) == {-1.0, 1.0}
    for r in (0, 1, 37, 63):
        bits = pt[:, r] > 0
        assert int(orc.pack_bits(bits)) == r              # corner r <-> code r


def test_soft_hash_invariants_and_sigmoid_product():
    g = torch.Generator().manual_seed(2)
    B, H, D, L, P = 2, 3, 16, 5, 6
    q = torch.randn(B, H, D, generator=g)
    planes = torch.randn(L, P, D, generator=g)
    protos = orc.hypercube_protos_T(P)
    for temp in (1.0, 0.3):
        pr = orc.soft_hash(q, planes, protos, temperature=temp)
        assert pr.shape == (B, H, L, 1 << P)
        assert torch.allclose(pr.sum(-1), torch.ones(B, H, L), atol=1e-6)
        # softmax over hypercube corners factorises: p(r) = prod_k sigmoid(2 c_rk s_k / temp)
        s = torch.tanh(torch.einsum("bhd,lkd->bhlk", q, planes)) / math.sqrt(D)
        closed = orc.sigmoid_product_probs(s, 2.0 / temp)
        assert torch.allclose(pr.double(), closed, rtol=1e-5, atol=1e-9)
        # the most probable bucket is the query's own hard code
        hard = orc.hard_hash_keys(q.view(B, 1, H, D), planes)[:, 0]       # [B,H,L]
        assert torch.equal(pr.argmax(-1), hard.long())
    # random (non-hypercube) prototypes: plain library softmax of the same logits
    protos_r = torch.randn(P, 50, generator=g)
    pr = orc.soft_hash(q, planes, protos_r)
    logits = (torch.tanh(q @ planes.view(L * P, D).t()).view(B, H, L, P) / math.sqrt(D)) @ protos_r
    assert torch.allclose(pr, torch.softmax(logits, -1), atol=1e-7)


def test_value_norm():
    v = torch.tensor([[3.0, 4.0], [0.0, 0.0], [1e3, 1e3]])
    n = orc.value_norm(v)
    assert n.dtype == torch.float16
    assert n.tolist() == [5.0, 0.0, float(torch.tensor(math.sqrt(2e6)).half())]


# ------------------------------------------------------------------ scorer
def test_collision_score_counts_and_mask():
    """One-hot q_probs at the query's codes -> score = #colliding tables * v_norm."""
    g = torch.Generator().manual_seed(3)
    B, H, L, R, T = 1, 2, 9, 16, 40
    qcode = torch.randint(0, R, (B, H, L), generator=g)
    q_probs = torch.zeros(B, H, L, R).scatter_(-1, qcode.unsqueeze(-1), 1.0)
    codes = torch.randint(0, R, (B, H, L, T), generator=g).to(torch.int16)
    codes[0, 1, :, 5] = qcode[0, 1].to(torch.int16)
    allowed = torch.ones(B, H, T, dtype=torch.bool)
    allowed[0, 0, 7] = False
    v = torch.full((B, H, T), 0.5)
    s = orc.collision_score(q_probs, codes, allowed, v)
    count = (codes.long() == qcode.unsqueeze(-1)).sum(2).float()
    want = torch.where(allowed, count * 0.5, torch.tensor(float("-inf")))
    assert torch.equal(s, want) and s[0, 1, 5] == L * 0.5 and s[0, 0, 7] == float("-inf")


def test_collision_score_against_c_loops_and_order(clib):
    g = torch.Generator().manual_seed(4)
    B, H, L, R, T = 2, 3, 60, 64, 333
    q_probs = torch.rand(B, H, L, R, generator=g) * torch.exp(-20 * torch.rand(B, H, L, R, generator=g))
    codes = torch.randint(0, R, (B, H, L, T), generator=g).to(torch.int16)
    allowed = torch.rand(B, H, T, generator=g) > 0.1
    v = torch.rand(B, H, T, generator=g) * 3
    got = orc.collision_score(q_probs, codes, allowed, v)
    out = np.zeros((B * H, T), dtype=np.float32)
    clib.oracle_c_collision_score(_p(q_probs.numpy()), _p(codes.numpy()), _p(allowed.numpy().astype(np.uint8)),
                                  _p(v.numpy()), _p(out), B * H, L, R, T)
    assert np.array_equal(got.numpy().reshape(B * H, T), out)             # same adds, same order: identical
    # and it is the plain gather-sum up to fp32 rounding of a different order
    ref = torch.stack([q_probs[..., l, :].double().gather(-1, codes[:, :, l].long())
                       for l in range(L)]).sum(0) * v.double()
    ok = allowed
    assert torch.allclose(got[ok].double(), ref[ok], rtol=1e-5)
    # fp16 variant widens and does the same
    got16 = orc.collision_score_vnorm16(q_probs.half(), codes, v.half(), allowed)
    assert torch.equal(got16, orc.collision_score(q_probs.half().float(), codes, allowed, v.half().float()))


# ------------------------------------------------------------------ top-k
def test_topk_rule(clib):
    g = torch.Generator().manual_seed(5)
    s = torch.randn(4, 500, generator=g)
    M = 37
    idx = orc.topk_lower_index_first(s, M)
    # distinct values: same set (and order) as torch.topk
    tk = torch.topk(s, M, dim=-1).indices
    assert torch.equal(idx, tk)
    # selected >= unselected
    for r in range(4):
        sel = set(idx[r].tolist())
        rest = [s[r, t].item() for t in range(500) if t not in sel]
        assert min(s[r, list(sel)]).item() >= max(rest)
    # all equal -> 0..M-1 ; two-valued with ties straddling the cut -> lowest indices of the tie class
    assert orc.topk_lower_index_first(torch.ones(1, 50), 7)[0].tolist() == list(range(7))
    t = torch.tensor([[1.0, 2.0, 1.0, 2.0, 1.0, 1.0]])
    assert orc.topk_lower_index_first(t, 4)[0].tolist() == [1, 3, 0, 2]
    # -inf rows, NaN first, signed zeros equal
    t = torch.tensor([[float("-inf"), 0.0, -0.0, float("nan"), float("inf"), -1.0]])
    assert orc.topk_lower_index_first(t, 6)[0].tolist() == [3, 4, 1, 2, 5, 0]
    # against the C selection-by-scan on a row with many ties
    row = torch.randint(0, 5, (300,), generator=g).float().numpy()
    out = np.zeros(40, dtype=np.int32)
    clib.oracle_c_topk(_p(row), 300, 40, _p(out))
    assert orc.topk_lower_index_first(torch.from_numpy(row), 40).tolist() == out.tolist()


# ------------------------------------------------------------------ list
def test_base_indices_enumeration(clib):
    for T in range(1, 14):
        for sink, window in itertools.product((0, 1, 3, 20), (0, 2, 5, 20)):
            got = orc.base_indices(T, sink, window)
            s_e, w_e = min(sink, T), min(window, T)
            want = list(range(s_e)) + [t for t in range(T) if t >= max(T - w_e, s_e) and w_e > 0]
            if not want:
                want = [T - 1]
            assert got.tolist() == want
            buf = np.zeros(64, dtype=np.int32)
            n = clib.oracle_c_base_indices(T, sink, window, _p(buf))
            assert buf[:n].tolist() == want
            assert len(set(want)) == len(want)          # sink and window never overlap


def test_build_sparse_list_layout_and_masking():
    g = torch.Generator().manual_seed(6)
    B, H, L, R, T = 1, 2, 4, 8, 30
    q_probs = torch.rand(B, H, L, R, generator=g)
    codes = torch.randint(0, R, (B, H, L, T), generator=g).to(torch.int16)
    v = torch.rand(B, H, T, generator=g).half()
    allowed = torch.ones(B, H, T, dtype=torch.bool)
    allowed[0, 1, 10:] = False                  # only 10 allowed keys on row 1
    sl, ln, sc = orc.build_sparse_list_decode(q_probs, codes, v, allowed, sink=2, window=3, M=12, return_scores=True)
    assert sl.dtype == torch.int32 and ln.dtype == torch.int32
    assert sl.shape == (B, H, 2 + 3 + 12) and (ln == 17).all()
    assert sl[0, 0, :5].tolist() == [0, 1, 27, 28, 29]
    assert sl[0, 1, :5].tolist() == [0, 1, -1, -1, -1]               # window masked out
    heavy1 = sl[0, 1, 5:]
    assert (heavy1[:10] >= 0).all() and (heavy1[:10] < 10).all() and (heavy1[10:] == -1).all()
    assert torch.equal(sl[0, 0, 5:], orc.topk_lower_index_first(sc[0, 0], 12).int())
    # M > T is clipped; M = 0 leaves only the base
    sl2, ln2 = orc.build_sparse_list_decode(q_probs, codes, v, allowed, 2, 3, 1000)
    assert sl2.shape[-1] == 5 + T
    sl3, _ = orc.build_sparse_list_decode(q_probs, codes, v, allowed, 2, 3, 0)
    assert sl3.shape[-1] == 5


# ------------------------------------------------------------------ attend
def _attend_inputs(seed, dtype=torch.float32, B=2, Hq=4, Hkv=2, D=16, S=200, Kt=70):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    k = torch.randn(B, Hkv, S, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, S, D, generator=g).to(dtype)
    sl = torch.randint(0, S, (B, Hq, Kt), generator=g, dtype=torch.int32)
    ln = torch.randint(1, Kt + 1, (B, Hq), generator=g, dtype=torch.int32)
    return q, k, v, sl, ln


def test_attend_textbook_special_cases(clib):
    q, k, v, sl, ln = _attend_inputs(7)
    B, Hq, D = q.shape
    G = Hq // k.shape[1]
    S = k.shape[2]
    # full list == library SDPA (GQA map kv = h // G)
    full = torch.arange(S, dtype=torch.int32).view(1, 1, S).expand(B, Hq, S).contiguous()
    lfull = torch.full((B, Hq), S, dtype=torch.int32)
    got = orc.sparse_attend_textbook(q, k, v, full, lfull)
    sdpa = torch.nn.functional.scaled_dot_product_attention(
        q.unsqueeze(2).double(), k.repeat_interleave(G, 1).double(), v.repeat_interleave(G, 1).double()).squeeze(2)
    assert torch.allclose(got, sdpa, atol=1e-12)
    assert torch.allclose(orc.dense_attend(q, k, v), sdpa, atol=1e-12)
    # single index -> that V row; duplicate index -> doubled weight; -1 -> ignored
    one = torch.full((B, Hq, 1), 17, dtype=torch.int32)
    got = orc.sparse_attend_textbook(q, k, v, one, torch.ones(B, Hq, dtype=torch.int32))
    assert torch.allclose(got, v[:, :, 17].repeat_interleave(G, 1).double())
    a = orc.sparse_attend_textbook(q, k, v, torch.tensor([5, 9, 9], dtype=torch.int32).expand(B, Hq, 3).contiguous(),
                                   torch.full((B, Hq), 3, dtype=torch.int32))
    kk, vv = k.repeat_interleave(G, 1).double(), v.repeat_interleave(G, 1).double()
    lg = torch.stack([(q.double() * kk[:, :, 5]).sum(-1), (q.double() * kk[:, :, 9]).sum(-1)], -1) / math.sqrt(D)
    w = torch.softmax(lg + torch.tensor([0.0, math.log(2.0)], dtype=torch.float64), -1)
    assert torch.allclose(a, w[..., :1] * vv[:, :, 5] + w[..., 1:] * vv[:, :, 9], atol=1e-12)
    b = orc.sparse_attend_textbook(q, k, v, torch.tensor([5, -1, 9, 9], dtype=torch.int32).expand(B, Hq, 4).contiguous(),
                                   torch.full((B, Hq), 4, dtype=torch.int32))
    assert torch.allclose(a, b, atol=1e-12)
    # the C loops, one head
    out = np.zeros(D, dtype=np.float64)
    lst = sl[1, 3, :int(ln[1, 3])].contiguous().numpy()
    clib.oracle_c_sparse_attend(_p(q[1, 3].numpy()), _p(k[1, 1].contiguous().numpy()), _p(v[1, 1].contiguous().numpy()),
                                _p(lst), len(lst), D, _p(out))
    want = orc.sparse_attend_textbook(q, k, v, sl, ln)[1, 3]
    assert np.allclose(out, want.numpy(), atol=1e-12)


def test_staged_attend_is_split_invariant_and_matches_textbook():
    q, k, v, sl, ln = _attend_inputs(8, Kt=90)
    want = orc.sparse_attend_textbook(q, k, v, sl, ln)
    for block_seq in (16, 32, 256):
        got = orc.sparse_attention_fwd(q, k, v, sl, ln, block_seq=block_seq)
        assert got.dtype == q.dtype
        assert torch.allclose(got.double(), want, atol=2e-6)
    # stage 1 leaves splits past the list untouched and reports max + log(sum_exp)
    mo, ml = orc.sparse_decode_stage1(q, k, v, sl, ln, int(ln.max()), block_seq=32)
    b, h = 0, 1
    n = int(ln[b, h])
    nblk = (n + 31) // 32
    assert torch.isnan(ml[b, h, nblk:]).all() and not torch.isnan(ml[b, h, :nblk]).any()
    rows = sl[b, h, :32].long()
    logits = (k[b, h // 2, rows[:min(n, 32)]] @ q[b, h]) / math.sqrt(q.shape[-1])
    assert torch.allclose(ml[b, h, 0], torch.logsumexp(logits, 0), atol=1e-5)
    # rounding the products to bf16 as the reference's tile arithmetic does stays inside the 2e-2 bar
    qb, kb, vb = q.bfloat16(), k.bfloat16(), v.bfloat16()
    a = orc.sparse_attention_fwd(qb, kb, vb, sl, ln, round_products=True).double()
    t = orc.sparse_attend_textbook(qb, kb, vb, sl, ln)
    assert (a - t).abs().max() <= 2e-2
    # empty list -> NaN like the reference's 0/0
    z = orc.sparse_attention_fwd(q, k, v, sl, torch.zeros_like(ln))
    assert torch.isnan(z).all()


# ------------------------------------------------------------------ cache
def test_kv_cache_update_semantics():
    B, H, T, D, L = 1, 2, 8, 4, 3
    cache = {"k_cache": torch.zeros(B, H, T, D), "v_cache": torch.zeros(B, H, T, D),
             "k_hard": torch.zeros(B, H, T, L, dtype=torch.int16), "v_norm": torch.zeros(B, H, T, dtype=torch.float16),
             "prefill_len": 0}
    k = torch.arange(B * 3 * H * D, dtype=torch.float32).view(B, 3, H, D)
    orc.kv_cache_update(cache, torch.tensor([2, 3, 4]), k, -k, v_norm=torch.ones(B, 3, H).half(),
                        k_hard=torch.full((B, 3, H, L), 7, dtype=torch.int16))
    assert cache["prefill_len"] == 5
    assert torch.equal(cache["k_cache"][0, 1, 3], k[0, 1, 1]) and torch.equal(cache["v_cache"][0, 0, 4], -k[0, 2, 0])
    assert cache["k_hard"][0, :, 2:5].eq(7).all() and cache["k_hard"][0, :, :2].eq(0).all()
    orc.kv_cache_update(cache, torch.tensor([0]), k[:, :1], k[:, :1])
    assert cache["prefill_len"] == 5            # never shrinks
    with pytest.raises(RuntimeError):
        orc.kv_cache_update(cache, torch.tensor([8]), k[:, :1], k[:, :1])


# ------------------------------------------------------------------ packed format (this build's own)
def test_packed_words_round_trip_and_plane_order():
    g = torch.Generator().manual_seed(9)
    for L, P in ((60, 10), (32, 8), (5, 16), (33, 1), (7, 11)):
        codes = torch.randint(0, 1 << min(P, 15), (2, L, 50), generator=g).numpy().astype(np.int16)
        w = orc.pack_code_words(codes, P)
        assert w.shape == (2, orc.words_per_key(L, P), 50) and w.dtype == np.uint32
        assert np.array_equal(orc.unpack_code_words(w, L, P), codes)
        c = 32 // P
        assert (w >> np.uint32(min(c * P, 31)) == 0).all() or c * P == 32
    # plane order: bit p of word w is the sign of plane (w*c + p//P, P-1 - p%P)
    L, P, D = 7, 10, 8
    planes = torch.randn(L, P, D, generator=g)
    pw = orc.permute_planes_for_words(planes)
    key = torch.randn(D, generator=g)
    bits = (pw @ key) >= 0
    words = [(int(sum(int(bits[w * 32 + p]) << p for p in range(30)))) for w in range(orc.words_per_key(L, P))]
    code = orc.hard_hash_keys(key.view(1, 1, 1, D), planes)[0, 0, 0]
    valid = np.array(words, dtype=np.uint32).reshape(1, -1, 1)
    # rows for unused bits are zero planes (projection 0 -> bit 1): masked off by the packer
    got = orc.unpack_code_words(valid, L, P)[0, :, 0]
    assert got.tolist() == code.tolist()
