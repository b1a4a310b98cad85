"""HIP kernels vs the CPU oracle, through the C ABI (socket_amd -> ctypes -> libsocket_hip.so).

Bars: top-k / lists bit-exact on identical fp32 scores (ties -> lower index);
scores within 1e-5 relative (the packed scorer sums in the reference's order,
so it is in fact compared for equality as well where stated); attention within
2e-2 absolute for bf16/fp16 inputs and 2e-5 for fp32 inputs.
"""
import math
import os

import numpy as np
import pytest
import torch

from oracle import socket_oracle as orc
from socket_amd import hash_cache, socket_kernels, sparse
from socket_amd.soft_hash_collision_loader import load_soft_hash_collision, soft_hash_score
from socket_amd.workloads import WORKLOADS, make_inputs, scaled

pytestmark = pytest.mark.gpu

ATOL = {torch.float32: 2e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}


def _score_keys(scores: torch.Tensor) -> np.ndarray:
    """The select kernel's order-preserving float -> uint32 map (finite inputs)."""
    u = scores.contiguous().numpy().view(np.uint32).copy()
    u[u == 0x80000000] = 0
    neg = (u & 0x80000000) != 0
    return np.where(neg, ~u, u | np.uint32(0x80000000))


def _rand_codes(g, B, H, L, T, P):
    return torch.randint(0, 1 << P, (B, H, L, T), generator=g, dtype=torch.int32).to(torch.int16)


def _packed_cache(codes_i16_bhlt, P, Tcap, dev):
    """oracle-packed words -> device int32 [B,Hkv,NW,Tcap]"""
    words = orc.pack_code_words(codes_i16_bhlt.numpy(), P)  # uint32 [B,H,NW,T]
    B, H, NW, T = words.shape
    full = np.zeros((B, H, NW, Tcap), dtype=np.uint32)
    full[..., :T] = words
    return torch.from_numpy(full.view(np.int32)).to(dev)


# ---------------------------------------------------------------- K2 scorer
@pytest.mark.parametrize("B,Hq,Hkv,L,P,T", [
    (1, 8, 2, 32, 8, 1000),      # G=4, P=8 (4 codes / word)
    (2, 8, 2, 60, 10, 4099),     # G=4, P=10, ragged tail
    (1, 4, 4, 7, 10, 513),       # G=1, L not a multiple of codes/word
    (1, 4, 2, 5, 6, 300),        # G=2, runtime-P kernel
    (1, 14, 2, 48, 10, 2500),    # G=7 (padded to 8)
    (4, 32, 8, 60, 10, 20000),   # enough work for the 8-tokens-per-lane variant
])
@pytest.mark.parametrize("table_dtype", [torch.float32, torch.bfloat16])
def test_score_packed_matches_oracle(dev, B, Hq, Hkv, L, P, T, table_dtype):
    g = torch.Generator().manual_seed(B * 1000 + L * 10 + P)
    R = 1 << P
    G = Hq // Hkv
    # a wide dynamic range, including bf16 subnormals, as a softmax output has
    q_probs = (torch.rand(B, Hq, L, R, generator=g) * torch.exp(-30 * torch.rand(B, Hq, L, R, generator=g)))
    q_probs[..., :3] = torch.tensor([0.0, 1e-39, 1.0])
    q_probs = q_probs.to(table_dtype)
    codes = _rand_codes(g, B, Hkv, L, T, P)
    v_norm = (torch.rand(B, Hkv, T, generator=g) * 10).to(torch.float16)
    lens = torch.randint(T // 2, T + 1, (B,), generator=g, dtype=torch.int32)
    Tcap = (T + 64 + 7) // 8 * 8
    vn_full = torch.zeros(B, Hkv, Tcap, dtype=torch.float16)
    vn_full[..., :T] = v_norm
    got, rng = hash_cache.score_packed(q_probs.to(dev), _packed_cache(codes, P, Tcap, dev), vn_full.to(dev),
                                       T, P, lens=lens.to(dev), with_range=True)
    got, rng = got.cpu(), rng.cpu()
    allowed = (torch.arange(T)[None, None, :] < lens[:, None, None]).expand(B, Hq, T)
    # per-tile key ranges handed to the select kernel: their union is the row's range
    keys = _score_keys(got)
    for b in range(B):
        kk = keys[b, :, :int(lens[b])]
        r = rng[b].numpy().view(np.uint32)
        assert np.array_equal(r[..., 0].min(-1), kk.min(-1)) and np.array_equal(r[..., 1].max(-1), kk.max(-1))
    want = orc.collision_score(q_probs.float(), codes.repeat_interleave(G, dim=1), allowed,
                               v_norm.float().repeat_interleave(G, dim=1))
    rel = ((got - want).abs() / want.abs().clamp_min(1e-30)).nan_to_num(0).max()
    assert rel <= 1e-5, f"max rel diff {rel}"
    if table_dtype == torch.float32:
        # same adds in the same order as the reference loop: identical results
        assert torch.equal(got, want), f"max abs diff {(got - want).abs().nan_to_num(0).max()}"
    else:
        # bf16 entries are widened and added by v_dot2_f32_bf16, whose final
        # rounding is not always the fp32 adder's: a few ulp over L adds
        assert rel <= 2e-6, f"max rel diff {rel}"


def test_score_packed_collision_counts(dev):
    """Known answer: one-hot q_probs at the query's own codes -> score = (#tables
    whose code equals the query's) * v_norm, an exact small integer multiple."""
    g = torch.Generator().manual_seed(7)
    B, Hq, Hkv, L, P, T = 1, 4, 1, 60, 10, 3000
    R = 1 << P
    qcode = torch.randint(0, R, (B, Hq, L), generator=g)
    q_probs = torch.zeros(B, Hq, L, R).scatter_(-1, qcode.unsqueeze(-1), 1.0)
    codes = _rand_codes(g, B, Hkv, L, T, P)
    codes[0, 0, :, 17] = qcode[0, 2].to(torch.int16)          # key 17 collides with head 2 in every table
    codes[0, 0, :30, 99] = qcode[0, 0, :30].to(torch.int16)   # key 99: >= 30 tables of head 0
    v_norm = torch.full((B, Hkv, T), 2.0, dtype=torch.float16)
    Tcap = 3008
    vn = torch.zeros(B, Hkv, Tcap, dtype=torch.float16); vn[..., :T] = v_norm
    got = hash_cache.score_packed(q_probs.to(dev), _packed_cache(codes, P, Tcap, dev), vn.to(dev), T, P).cpu()
    count = (codes[:, 0].long().unsqueeze(1) == qcode.unsqueeze(-1)).sum(2)   # [B,Hq,T]
    assert torch.equal(got, count.float() * 2.0)
    assert got[0, 2, 17] == 120.0 and got[0, 0, 99] >= 60.0


@pytest.mark.parametrize("L,R,T", [(32, 256, 777), (60, 1024, 4096), (3, 32768, 100), (60, 1024, 9000),
                                   (17, 1024, 10001), (5, 8192, 2056), (40, 2048, 16384),
                                   # rows long enough for several tiles per workgroup under each table slice,
                                   # one table per slice: the sums wait in the output between slices
                                   (3, 32768, 1400000), (3, 32768, 1400001)])
def test_reference_layout_scorer(dev, L, R, T):
    """Rows on and off the 16-byte grid, one to several table slices in LDS, more
    than one tile of tokens per row, codes outside [0, R) (they add nothing)."""
    g = torch.Generator().manual_seed(L + T)
    B, H = 2, 3
    q_probs = torch.rand(B, H, L, R, generator=g)
    codes = torch.randint(0, R, (B, H, L, T), generator=g, dtype=torch.int32).to(torch.int16)
    if R < 32768:
        stray = torch.rand(B, H, L, T, generator=g)
        codes[stray < 0.01] = -1
        codes[stray > 0.99] = R
    allowed = torch.rand(B, H, T, generator=g) > 0.2
    v_hist = torch.rand(B, H, T, generator=g) * 5
    ext = load_soft_hash_collision(3)
    got = ext.soft_hash_collision(q_probs.unsqueeze(2).contiguous().to(dev), codes.to(dev),
                                  allowed.unsqueeze(2).contiguous().to(dev),
                                  v_hist.unsqueeze(2).contiguous().to(dev)).squeeze(2).cpu()
    # the oracle sees the strays as hits of an extra all-zero bucket (x + 0.0 == x)
    padded = torch.cat([q_probs, torch.zeros(B, H, L, 1)], -1)
    mapped = torch.where((codes < 0) | (codes.int() >= R), torch.full_like(codes.int(), R), codes.int())
    assert torch.equal(got, orc.collision_score(padded, mapped, allowed, v_hist))
    got16 = soft_hash_score(q_probs.half().to(dev), codes.to(dev), v_hist.half().to(dev), allowed.to(dev)).cpu()
    assert torch.equal(got16, orc.collision_score_vnorm16(padded.half(), mapped, v_hist.half(), allowed))


REF_SO = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "libref_scorer.so")


@pytest.mark.skipif(not os.path.exists(REF_SO), reason="oracle/_ref not built (needs the reference checkout at build time)")
def test_scorers_vs_the_reference_kernel_at_config2_size(dev):
    """The reference's own soft_hash_collision_kernel_3, compiled unmodified for
    gfx950 (oracle/Makefile `ref`), as the checker at the full configuration-2
    shape: B1, 32/8 heads, T=32768, L=60, P=10."""
    import ctypes
    ref = ctypes.CDLL(REF_SO)
    g = torch.Generator().manual_seed(2000)
    B, Hq, Hkv, L, P, T = 1, 32, 8, 60, 10, 32768
    R, G = 1 << P, Hq // Hkv
    q_probs = torch.softmax(torch.randn(B, Hq, L, R, generator=g) * 3, -1).to(dev)
    codes = _rand_codes(g, B, Hkv, L, T, P).to(dev)
    v_norm = (torch.rand(B, Hkv, T, generator=g) * 12).to(torch.float16).to(dev)
    lens = torch.tensor([T - 77], dtype=torch.int32, device=dev)
    # reference operands: codes and norms repeated per query head, bool mask
    kb = codes.repeat_interleave(G, 1).contiguous()
    allowed = (torch.arange(T, device=dev) < lens[0]).view(1, 1, T).expand(B, Hq, T).contiguous()
    v_hist = v_norm.float().repeat_interleave(G, 1).contiguous()
    want = torch.empty(B, Hq, T, dtype=torch.float32, device=dev)
    rc = ref.ref_soft_hash_collision(
        ctypes.c_void_p(q_probs.data_ptr()), ctypes.c_void_p(kb.data_ptr()), ctypes.c_void_p(allowed.data_ptr()),
        ctypes.c_void_p(v_hist.data_ptr()), ctypes.c_void_p(want.data_ptr()), B, Hq, L, R, T,
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    torch.cuda.synchronize()
    # packed scorer, fp32 table: bit-identical
    words = torch.zeros((B, Hkv, orc.words_per_key(L, P), T), dtype=torch.int32, device=dev)
    hash_cache.pack_codes_into(codes, words, P)
    got = hash_cache.score_packed(q_probs, words, v_norm, T, P, lens=lens)
    assert torch.equal(got, want)
    # packed scorer, bf16 table against the reference fed the same bf16 values widened
    qb = q_probs.to(torch.bfloat16)
    rc = ref.ref_soft_hash_collision(
        ctypes.c_void_p(qb.float().contiguous().data_ptr()), ctypes.c_void_p(kb.data_ptr()),
        ctypes.c_void_p(allowed.data_ptr()), ctypes.c_void_p(v_hist.data_ptr()), ctypes.c_void_p(want.data_ptr()),
        B, Hq, L, R, T, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    gotb = hash_cache.score_packed(qb, words, v_norm, T, P, lens=lens)
    ok = allowed
    rel = ((gotb[ok] - want[ok]).abs() / want[ok].abs().clamp_min(1e-30)).max()
    assert rel <= 1e-5 and torch.equal(gotb[~ok], want[~ok])
    # the drop-in scorer on the reference's own operand layout: bit-identical
    ext = load_soft_hash_collision(3)
    qf = q_probs
    rc = ref.ref_soft_hash_collision(
        ctypes.c_void_p(qf.data_ptr()), ctypes.c_void_p(kb.data_ptr()), ctypes.c_void_p(allowed.data_ptr()),
        ctypes.c_void_p(v_hist.data_ptr()), ctypes.c_void_p(want.data_ptr()), B, Hq, L, R, T,
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    got2 = ext.soft_hash_collision(qf.unsqueeze(2).contiguous(), kb, allowed.unsqueeze(2).contiguous(),
                                   v_hist.unsqueeze(2).contiguous()).squeeze(2)
    assert torch.equal(got2, want)


def test_loader_errors(dev):
    ext = load_soft_hash_collision()
    with pytest.raises(ValueError):
        load_soft_hash_collision(2)
    q = torch.rand(1, 1, 1, 2, 16, device=dev)
    kb = torch.zeros(1, 1, 2, 8, dtype=torch.int16, device=dev)
    al = torch.ones(1, 1, 1, 8, dtype=torch.bool, device=dev)
    vh = torch.ones(1, 1, 1, 8, device=dev)
    with pytest.raises(RuntimeError, match="float32"):
        ext.soft_hash_collision(q.half(), kb, al, vh)
    with pytest.raises(RuntimeError, match="int16"):
        ext.soft_hash_collision(q, kb.int(), al, vh)
    with pytest.raises(RuntimeError, match="shape mismatch"):
        ext.soft_hash_collision(q, kb, al[..., :4].contiguous(), vh)
    with pytest.raises(RuntimeError, match="CUDA"):
        ext.soft_hash_collision(q.cpu(), kb, al, vh)


# ---------------------------------------------------------------- K3 select
def _check_select(scores, sink, window, M, dev, lens=None, budgets=None):
    """Both kernels paths (rows split over many workgroups / one workgroup per
    row; they coincide for short rows) against the stable-sort oracle."""
    for split in (True, False):
        _check_select_path(scores, sink, window, M, dev, lens, budgets, split)


def _check_select_path(scores, sink, window, M, dev, lens, budgets, split):
    B, H, T = scores.shape
    pitch = (T + 3) // 4 * 4
    buf = torch.full((B, H, pitch), float("nan"))
    buf[..., :T] = scores
    sl, ln = sparse.select_list(buf.to(dev)[..., :T], sink, window, M,
                                lens=None if lens is None else lens.to(dev),
                                budgets=None if budgets is None else budgets.to(dev), split=split)
    sl, ln = sl.cpu(), ln.cpu()
    for b in range(B):
        n = T if lens is None else int(lens[b])
        m = min(M if budgets is None else min(int(budgets[b]), M), n)
        base = torch.from_numpy(orc.base_indices(n, sink, window))
        for h in range(H):
            heavy = orc.topk_lower_index_first(scores[b, h, :n], m).to(torch.int32)
            want = torch.cat([base, heavy])
            assert int(ln[b, h]) == want.numel()
            assert torch.equal(sl[b, h, :want.numel()], want), (b, h)
            assert (sl[b, h, want.numel():] == -1).all()


@pytest.mark.parametrize("T,M", [(5000, 128), (131072, 2048), (300, 300), (64, 1), (4097, 4000)])
def test_select_random_scores(dev, T, M):
    g = torch.Generator().manual_seed(T + M)
    scores = torch.randn(2, 3, T, generator=g).abs() * 7
    _check_select(scores, 4, 64, M, dev)


@pytest.mark.parametrize("T", [20000, 70001, 140001])
def test_select_ties_and_special_values(dev, T):
    g = torch.Generator().manual_seed(3)
    s = torch.randint(0, 50, (1, 6, T), generator=g).float()     # heavy ties, few distinct values
    s[0, 1] = 1.0                                                 # all equal -> indices 0..M-1
    s[0, 2, ::3] = float("-inf")                                  # masked keys
    s[0, 3, 5] = float("nan"); s[0, 3, 77] = float("inf")         # NaN ranks first, then +inf
    s[0, 4] = torch.randn(T, generator=g)                         # negative values
    s[0, 4, 10] = 0.0; s[0, 4, 11] = -0.0                         # signed zeros compare equal
    s[0, 5] = torch.where(torch.arange(T) % 2 == 0, 3.0, 2.0)     # one huge tie class straddling M
    for M in (1, 700, 5000):
        _check_select(s, 4, 16, M, dev)


@pytest.mark.parametrize("T,M", [(131072, 2048), (40000, 700), (300000, 1024)])
def test_select_rows_that_mislead_the_sampled_threshold(dev, T, M):
    """Long rows are selected from a pool of everything above a threshold that
    is estimated from runs of 64 scores at evenly spaced places.  These rows make
    that estimate wrong in every direction (pool too small, too large, one slice
    holding all winners); the result must still be the exact top-M."""
    g = torch.Generator().manual_seed(T)
    base = torch.rand(6, T, generator=g)
    s = base.clone()
    nchunk = (4096 if T <= 262144 else 16384) // 64
    starts = (torch.arange(nchunk) * T // nchunk) // 4 * 4
    sampled = (starts[:, None] + torch.arange(64)[None, :]).flatten()
    s[0, sampled] += 100.0                                   # only the sampled places are hot: pool < M
    s[1] = base[1] * 0.001
    s[1, sampled] = -5.0                                     # sampled places are cold: threshold too low
    s[2] = base[2] + torch.arange(T) * (50.0 / T)            # trend: winners all in the last slice
    s[3, 12345] = 1e30                                       # one outlier stretches the key range
    s[4, T // 3: T // 3 + 3 * M] += 10.0                     # a contiguous hot block larger than M
    s[5] = (base[5] * 4).floor()                             # four values: the threshold sits in a huge tie
    _check_select(s.view(1, 6, T), 4, 32, M, dev)


@pytest.mark.parametrize("T", [9000, 66000])
def test_select_ragged_lengths_and_budgets(dev, T):
    g = torch.Generator().manual_seed(11)
    B, H = 4, 2
    scores = torch.rand(B, H, T, generator=g)
    lens = torch.tensor([T, 130, T // 2 + 1, 1], dtype=torch.int32)
    budgets = torch.tensor([180, 500, 81, 3], dtype=torch.int32)
    _check_select(scores, 4, 128, 500, dev, lens=lens, budgets=budgets)


def test_select_long_rows_with_an_odd_pitch(dev):
    """Rows long and few enough to be shared between workgroups, at a row pitch
    that rules out 16-byte loads (the scalar-load variant of the same kernel),
    with ragged lengths and budgets."""
    g = torch.Generator().manual_seed(23)
    B, H, T, M = 2, 2, 100003, 700
    scores = (torch.randn(B, H, T, generator=g) * 2).to(dev)          # pitch T: odd
    assert scores.stride(1) % 4 != 0
    lens = torch.tensor([T, 60001], dtype=torch.int32)
    budgets = torch.tensor([700, 333], dtype=torch.int32)
    sl, ln = sparse.select_list(scores, 4, 64, M, lens=lens.to(dev), budgets=budgets.to(dev))
    sl, ln, sc = sl.cpu(), ln.cpu(), scores.cpu()
    for b in range(B):
        n, m = int(lens[b]), int(budgets[b])
        base = torch.from_numpy(orc.base_indices(n, 4, 64))
        for h in range(H):
            want = torch.cat([base, orc.topk_lower_index_first(sc[b, h, :n], m).to(torch.int32)])
            assert int(ln[b, h]) == want.numel() and torch.equal(sl[b, h, :want.numel()], want), (b, h)


def test_select_base_enumeration(dev):
    """List arithmetic for every small T (sparse.py:70-95), including the
    'empty base -> [T-1]' rule."""
    for T in range(1, 12):
        for sink, window in ((0, 0), (2, 3), (4, 0), (0, 5), (20, 20)):
            scores = torch.arange(T, dtype=torch.float32).flip(0).view(1, 1, T).contiguous()
            _check_select(scores, sink, window, 3, dev)


@pytest.mark.parametrize("T,M,sink,window", [(700, 64, 4, 32), (50, 80, 4, 64), (9, 0, 2, 2)])
def test_build_sparse_list_decode_reference_layout(dev, T, M, sink, window):
    g = torch.Generator().manual_seed(T)
    B, H, L, P = 2, 4, 12, 8
    R = 1 << P
    q_probs = torch.rand(B, H, L, R, generator=g).to(torch.bfloat16)
    codes = _rand_codes(g, B, H, L, T, P)
    v_norm = torch.rand(B, H, T, generator=g).to(torch.float16)
    allowed = torch.rand(B, H, T, generator=g) > 0.1
    allowed[1, 2, T // 4:] = False          # fewer allowed keys than M on one row
    sl, ln = sparse.build_sparse_list_decode(q_probs.to(dev), codes.to(dev), v_norm.to(dev), allowed.to(dev),
                                             sink=sink, window=window, M=M)
    wl, wn = orc.build_sparse_list_decode(q_probs, codes, v_norm, allowed, sink, window, M)
    assert sl.dtype == torch.int32 and ln.dtype == torch.int32
    assert torch.equal(sl.cpu(), wl) and torch.equal(ln.cpu(), wn)


# ---------------------------------------------------------------- K4 attend
def _attend_case(dev, dtype, B, Hq, Hkv, D, S, Kt, seed, neg_frac=0.0, ragged=False):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    k = torch.randn(B, Hkv, S, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, S, D, generator=g).to(dtype)
    sl = torch.randint(0, S, (B, Hq, Kt), generator=g, dtype=torch.int32)   # duplicates on purpose
    if neg_frac:
        sl[torch.rand(B, Hq, Kt, generator=g) < neg_frac] = -1
    ln = torch.full((B, Hq), Kt, dtype=torch.int32)
    if ragged:
        ln = torch.randint(1, Kt + 1, (B, Hq), generator=g, dtype=torch.int32)
    return q, k, v, sl, ln


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("D", [128, 64])
def test_sparse_attention_vs_textbook(dev, dtype, D):
    q, k, v, sl, ln = _attend_case(dev, dtype, 2, 8, 2, D, 3000, 777, seed=D, neg_frac=0.05, ragged=True)
    got = socket_kernels.sparse_attention_fwd(q.to(dev), k.to(dev), v.to(dev), sl.to(dev), ln.to(dev))
    assert got.dtype == dtype
    want = orc.sparse_attend_textbook(q, k, v, sl, ln)
    assert (got.cpu().double() - want).abs().max() <= ATOL[dtype]


def test_sparse_attention_small_head_dims(dev):
    for D in (16, 32):
        q, k, v, sl, ln = _attend_case(dev, torch.bfloat16, 1, 4, 2, D, 500, 100, seed=D)
        got = socket_kernels.sparse_attention_fwd(q.to(dev), k.to(dev), v.to(dev), sl.to(dev), ln.to(dev))
        want = orc.sparse_attend_textbook(q, k, v, sl, ln)
        assert (got.cpu().double() - want).abs().max() <= 2e-2


def test_stage1_stage2_match_reference_blocking(dev):
    """Stage outputs in the reference's own split geometry (block_seq = 256)."""
    q, k, v, sl, ln = _attend_case(dev, torch.float32, 1, 4, 2, 128, 2000, 600, seed=5, ragged=True)
    block_seq = 256
    max_len = int(ln.max())
    ns = (max_len + block_seq - 1) // block_seq
    mid_o = torch.full((1, 4, ns, 128), float("nan"), device=dev)
    mid_l = torch.full((1, 4, ns), float("nan"), device=dev)
    socket_kernels.sparse_decode_stage1(q.to(dev), k.to(dev), v.to(dev), sl.to(dev), ln.to(dev), max_len,
                                        mid_o, mid_l, block_seq)
    wo, wl = orc.sparse_decode_stage1(q, k, v, sl, ln, max_len, block_seq)
    written = ~torch.isnan(wl)
    assert torch.equal(~torch.isnan(mid_l.cpu()), written)        # untouched splits stay untouched
    assert torch.allclose(mid_l.cpu()[written], wl[written], rtol=1e-5, atol=1e-5)
    assert torch.allclose(mid_o.cpu()[written], wo[written], rtol=1e-4, atol=1e-5)
    out = torch.empty(1, 4, 128, device=dev)
    socket_kernels.sparse_decode_stage2(mid_o, mid_l, ln.to(dev), out, block_seq)
    want = orc.sparse_decode_stage2(wo, wl, ln, torch.float32, block_seq)
    assert torch.allclose(out.cpu(), want, rtol=1e-4, atol=1e-5)


def test_attention_special_cases(dev):
    g = torch.Generator().manual_seed(9)
    B, Hq, Hkv, D, S = 1, 8, 2, 128, 1500
    q = torch.randn(B, Hq, D, generator=g)
    k = torch.randn(B, Hkv, S, D, generator=g)
    v = torch.randn(B, Hkv, S, D, generator=g)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    # list = arange(S)  ==  dense attention (library routine)
    full = torch.arange(S, dtype=torch.int32).view(1, 1, S).expand(B, Hq, S).contiguous()
    ln = torch.full((B, Hq), S, dtype=torch.int32)
    got = socket_kernels.sparse_attention_fwd(qd, kd, vd, full.to(dev), ln.to(dev)).cpu()
    sdpa = torch.nn.functional.scaled_dot_product_attention(
        q.unsqueeze(2), k.repeat_interleave(4, 1), v.repeat_interleave(4, 1)).squeeze(2)
    assert torch.allclose(got, sdpa, atol=2e-5)
    dense = socket_kernels.dense_decode_fwd(qd, kd, vd, torch.tensor([S], dtype=torch.int32, device=dev)).cpu()
    assert torch.allclose(dense, sdpa, atol=2e-5)
    # single index -> that V row (GQA map kv = h // G)
    one = torch.full((B, Hq, 1), 123, dtype=torch.int32)
    got = socket_kernels.sparse_attention_fwd(qd, kd, vd, one.to(dev), torch.ones(B, Hq, dtype=torch.int32, device=dev)).cpu()
    assert torch.allclose(got, v[:, :, 123].repeat_interleave(4, 1), atol=1e-6)
    # a duplicated index doubles its weight
    dup = torch.tensor([5, 9, 9], dtype=torch.int32).view(1, 1, 3).expand(B, Hq, 3).contiguous()
    got = socket_kernels.sparse_attention_fwd(qd, kd, vd, dup.to(dev), torch.full((B, Hq), 3, dtype=torch.int32, device=dev)).cpu()
    kk = k.repeat_interleave(4, 1); vv = v.repeat_interleave(4, 1)
    lg = torch.stack([(q * kk[:, :, 5]).sum(-1), (q * kk[:, :, 9]).sum(-1)], -1) / math.sqrt(D)
    w = torch.softmax(lg + torch.tensor([0.0, math.log(2.0)]), -1)
    want = w[..., :1] * vv[:, :, 5] + w[..., 1:] * vv[:, :, 9]
    assert torch.allclose(got, want, atol=1e-5)
    # empty list -> NaN (0/0), as the reference
    got = socket_kernels.sparse_attention_fwd(qd, kd, vd, dup.to(dev), torch.zeros(B, Hq, dtype=torch.int32, device=dev))
    assert torch.isnan(got).all()


def test_strided_kv_views(dev):
    """K/V as views of a larger cache (non-contiguous in dims 0-2)."""
    g = torch.Generator().manual_seed(21)
    q = torch.randn(2, 4, 128, generator=g).to(torch.bfloat16)
    cache_k = torch.randn(2, 2, 900, 128, generator=g).to(torch.bfloat16)
    cache_v = torch.randn(2, 2, 900, 128, generator=g).to(torch.bfloat16)
    sl = torch.randint(0, 500, (2, 4, 64), generator=g, dtype=torch.int32)
    ln = torch.full((2, 4), 64, dtype=torch.int32)
    kd, vd = cache_k.to(dev)[:, :, :500], cache_v.to(dev)[:, :, :500]
    assert not kd.is_contiguous()
    got = socket_kernels.sparse_attention_fwd(q.to(dev), kd, vd, sl.to(dev), ln.to(dev))
    want = orc.sparse_attend_textbook(q, cache_k[:, :, :500], cache_v[:, :, :500], sl, ln)
    assert (got.cpu().double() - want).abs().max() <= 2e-2


def test_dense_decode_ragged(dev):
    g = torch.Generator().manual_seed(33)
    B, Hq, Hkv, D, T = 3, 14, 2, 128, 5000     # G = 7
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, T, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, T, D, generator=g).to(torch.bfloat16)
    lens = torch.tensor([5000, 17, 2049], dtype=torch.int32)
    got = socket_kernels.dense_decode_fwd(q.to(dev), k.to(dev), v.to(dev), lens.to(dev))
    want = orc.dense_attend(q, k, v, lens)
    assert (got.cpu().double() - want).abs().max() <= 2e-2


@pytest.mark.parametrize("dtype,B,Hq,Hkv,T,strided", [
    (torch.bfloat16, 2, 8, 2, 3000, False),     # G = 4
    (torch.bfloat16, 3, 10, 2, 2500, True),     # G = 5, K/V as [B,T,Hkv,D] views
    (torch.float16, 2, 14, 2, 1111, False),     # G = 7, half precision
    (torch.bfloat16, 1, 16, 1, 4097, False),    # G = 16: every column of the tile is a head
    (torch.bfloat16, 1, 12, 1, 600, False),     # G = 12
    (torch.bfloat16, 70, 8, 1, 300, False),     # more sequences than one wave can scan: rectangular grid
])
def test_dense_decode_matrix_core_path(dev, dtype, B, Hq, Hkv, T, strided):
    """16-bit caches with four or more heads per kv head run the MFMA dense
    kernel: ragged lengths down to one row, lengths off the 16-key block and off
    the split, scores that must be masked, and rows after a sequence's end holding
    huge values that must never be read into a result."""
    g = torch.Generator().manual_seed(B * 1000 + Hq)
    D = 128
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    k = torch.randn(B, Hkv, T, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, T, D, generator=g).to(dtype)
    lens = torch.randint(1, T + 1, (B,), generator=g, dtype=torch.int32)
    lens[0] = T
    if B > 1:
        lens[1] = 1
    if B > 2:
        lens[2] = 17
    big = 3e4 if dtype == torch.bfloat16 else 100.0       # (4 * big must stay finite in the cache's type)
    for b in range(B):                      # poison what lies beyond each sequence
        k[b, :, int(lens[b]):] = big
        v[b, :, int(lens[b]):] = -big
    if strided:
        kd = k.to(dev).transpose(1, 2).contiguous().transpose(1, 2)      # [B,Hkv,T,D] view of [B,T,Hkv,D]
        vd = v.to(dev).transpose(1, 2).contiguous().transpose(1, 2)
        assert not kd.is_contiguous()
    else:
        kd, vd = k.to(dev), v.to(dev)
    got = socket_kernels.dense_decode_fwd(q.to(dev), kd, vd, lens.to(dev))
    want = orc.dense_attend(q, k, v, lens)
    assert torch.isfinite(got.float()).all()
    assert (got.cpu().double() - want).abs().max() <= 2e-2
    # sharply peaked rows: one key dominates (scores of the order of 1e11 where the
    # query was taken from a poisoned row), the result is that key's value row
    q2 = (k[:, :, 5].repeat_interleave(Hq // Hkv, 1).float() * 4).to(dtype)
    lens2 = torch.full((B,), min(T, 64), dtype=torch.int32)
    got2 = socket_kernels.dense_decode_fwd(q2.to(dev), kd, vd, lens2.to(dev))
    want2 = orc.dense_attend(q2, k, v, lens2)
    assert (got2.cpu().double() - want2).abs().max() <= 2e-2


def test_dense_decode_with_empty_sequences(dev):
    """A sequence of length zero (or a negative length) takes no split; its
    neighbours' splits are still numbered and attended correctly."""
    g = torch.Generator().manual_seed(77)
    B, Hq, Hkv, T = 5, 8, 2, 3000
    q = torch.randn(B, Hq, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, T, 128, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, T, 128, generator=g).to(torch.bfloat16)
    lens = torch.tensor([0, 2500, -7, 1, 3000], dtype=torch.int32)
    got = socket_kernels.dense_decode_fwd(q.to(dev), k.to(dev), v.to(dev), lens.to(dev)).cpu()
    live = [1, 3, 4]
    want = orc.dense_attend(q[live], k[live], v[live], lens[live])
    assert (got[live].double() - want).abs().max() <= 2e-2
    assert torch.isnan(got[[0, 2]].float()).all()        # nothing attended: 0 / 0, as the sparse path's empty list


@pytest.mark.parametrize("draw", range(12))
def test_dense_decode_random_shapes(dev, draw):
    """Drawn geometries for the MFMA dense kernel: 1 to 16 heads per kv head, 1 to 5
    sequences of 1 to 6000 rows (one to several splits, blocks and waves with
    nothing to do), both 16-bit types, contiguous caches and `[B,T,Hkv,D]` views."""
    import random
    rnd = random.Random(7000 + draw)
    G = rnd.choice([1, 2, 3, 4, 6, 7, 8, 11, 16])
    Hkv = rnd.choice([1, 2, 3])
    B = rnd.randint(1, 5)
    T = rnd.choice([1, 15, 16, 17, 63, 64, 65, 500, 1023, 1025, 2500, 6000])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    g = torch.Generator().manual_seed(7000 + draw)
    q = torch.randn(B, Hkv * G, 128, generator=g).to(dtype)
    k = torch.randn(B, Hkv, T, 128, generator=g).to(dtype)
    v = torch.randn(B, Hkv, T, 128, generator=g).to(dtype)
    lens = torch.randint(1, T + 1, (B,), generator=g, dtype=torch.int32)
    lens[rnd.randrange(B)] = T
    print(f"G{G} Hkv{Hkv} B{B} T{T} {dtype} lens {lens.tolist()}", flush=True)
    kd, vd = k.to(dev), v.to(dev)
    if rnd.random() < 0.5:
        kd = kd.transpose(1, 2).contiguous().transpose(1, 2)
        vd = vd.transpose(1, 2).contiguous().transpose(1, 2)
    got = socket_kernels.dense_decode_fwd(q.to(dev), kd, vd, lens.to(dev))
    want = orc.dense_attend(q, k, v, lens)
    assert (got.cpu().double() - want).abs().max() <= 2e-2


# ---------------------------------------------------------------- K1 hash
@pytest.mark.parametrize("dtype,L,P,S,D", [(torch.bfloat16, 60, 10, 1000, 128), (torch.float32, 32, 8, 333, 128),
                                           (torch.float16, 7, 5, 65, 128), (torch.bfloat16, 48, 10, 1, 128),
                                           (torch.bfloat16, 60, 10, 500, 64), (torch.float32, 20, 8, 3, 32)])
def test_hash_keys_vs_oracle(dev, dtype, L, P, S, D):
    """(Head dims below 128 are padded with zeros by the wrapper: same bits, same norms.)"""
    g = torch.Generator().manual_seed(L * P + S)
    B, Hkv, t0 = 2, 3, 24
    Tcap = (t0 + S + 15) // 8 * 8
    k = torch.randn(B, S, Hkv, D, generator=g).to(dtype)          # [B,S,Hkv,D] as the reference hashes them
    v = torch.randn(B, S, Hkv, D, generator=g).to(dtype)
    planes = torch.randn(L, P, D, generator=g)
    NW = orc.words_per_key(L, P)
    codes = torch.full((B, Hkv, NW, Tcap), -1, dtype=torch.int32, device=dev)
    vn = torch.full((B, Hkv, Tcap), -1.0, dtype=torch.float16, device=dev)
    pw = hash_cache.permute_planes(planes.to(dev))
    assert torch.equal(pw.cpu()[:, :D], orc.permute_planes_for_words(planes.to(torch.bfloat16)))
    assert pw.shape[1] == 128 and not pw[:, D:].any()
    hash_cache.hash_keys_into(k.to(dev), v.to(dev), pw, codes, vn, L, P, t0=t0, layout="bshd")
    got = hash_cache.unpack_codes(codes, L, P, t0, S, layout="bthl").cpu()      # [B,S,Hkv,L]
    # untouched cache positions stay untouched
    assert (codes[..., :t0] == -1).all() and (codes[..., t0 + S:] == -1).all()
    assert (vn[..., :t0] == -1).all() and (vn[..., t0 + S:] == -1).all()
    # the kernel contracts bf16 operands with fp32 accumulation
    kb, pb = k.to(torch.bfloat16), planes.to(torch.bfloat16)
    proj = orc.projections_f64(kb, pb)                                            # [B,S,Hkv,L,P]
    want_bits = proj >= 0
    got_bits = ((got.long().unsqueeze(-1) >> torch.arange(P - 1, -1, -1)) & 1).bool()
    margin = 1e-3 * kb.double().norm(dim=-1)[..., None, None] * pb.double().norm(dim=-1)
    decided = proj.abs() > margin
    assert decided.float().mean() > 0.98
    assert torch.equal(got_bits[decided], want_bits[decided])
    # and against the reference's own formulation run in the input dtype, on the same decided bits
    ref_codes = orc.hard_hash_keys(k, planes)                                      # int16 [B,S,Hkv,L]
    ref_bits = ((ref_codes.long().unsqueeze(-1) >> torch.arange(P - 1, -1, -1)) & 1).bool()
    assert torch.equal(got_bits[decided], ref_bits[decided])
    # value norm: fp32 reduce, fp16 store (1 ulp of fp16 for the different summation order)
    want_vn = orc.value_norm(v).permute(0, 2, 1)                                   # [B,Hkv,S]
    got_vn = vn[..., t0:t0 + S].cpu()
    assert torch.allclose(got_vn.float(), want_vn.float(), rtol=1e-3, atol=0)


def test_hash_keys_streamed_variant_equals_the_staged_one(dev):
    """A launch with a 128-key tile for every CU takes the variant that keeps the
    planes in registers and streams the keys through LDS.  Same contraction order,
    so codes and norms must equal, bit for bit, those of the same rows hashed in
    pieces small enough for the register-staged kernel; plus the oracle check."""
    g = torch.Generator().manual_seed(60)
    B, Hkv, D, L, P, S, t0 = 2, 8, 128, 60, 10, 2100, 40          # 17 tiles x 16 pairs, ragged last tile
    Tcap = 2160
    k = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
    v = (torch.randn(B, S, Hkv, D, generator=g) * 2).to(torch.bfloat16)
    planes = torch.randn(L, P, D, generator=g)
    NW = orc.words_per_key(L, P)
    pw = hash_cache.permute_planes(planes.to(dev))
    kd, vd = k.to(dev), v.to(dev)

    def fresh():
        return (torch.full((B, Hkv, NW, Tcap), -1, dtype=torch.int32, device=dev),
                torch.full((B, Hkv, Tcap), -1.0, dtype=torch.float16, device=dev))

    codes, vn = fresh()
    hash_cache.hash_keys_into(kd, vd, pw, codes, vn, L, P, t0=t0, layout="bshd")
    codes_p, vn_p = fresh()
    for a in range(0, S, 700):
        hash_cache.hash_keys_into(kd[:, a:a + 700], vd[:, a:a + 700], pw, codes_p, vn_p, L, P, t0=t0 + a, layout="bshd")
    assert torch.equal(codes, codes_p) and torch.equal(vn, vn_p)
    assert (codes[..., :t0] == -1).all() and (codes[..., t0 + S:] == -1).all()
    assert (vn[..., :t0] == -1).all() and (vn[..., t0 + S:] == -1).all()
    # per-sequence positions, no values
    pos = torch.tensor([3, 57], dtype=torch.int32, device=dev)
    codes_q, vn_q = fresh()
    hash_cache.hash_keys_into(kd, None, pw, codes_q, None, L, P, pos_b=pos, layout="bshd")
    for b in range(B):
        p0 = int(pos[b])
        assert torch.equal(codes_q[b, :, :, p0:p0 + S], codes[b, :, :, t0:t0 + S])
        assert (codes_q[b, :, :, :p0] == -1).all() and (codes_q[b, :, :, p0 + S:] == -1).all()
    assert (vn_q == -1).all()
    # against fp64 projections on the decided bits, and the norms
    got = hash_cache.unpack_codes(codes, L, P, t0, S, layout="bthl").cpu()
    pb = planes.to(torch.bfloat16)
    proj = orc.projections_f64(k, pb)
    got_bits = ((got.long().unsqueeze(-1) >> torch.arange(P - 1, -1, -1)) & 1).bool()
    decided = proj.abs() > 1e-3 * k.double().norm(dim=-1)[..., None, None] * pb.double().norm(dim=-1)
    assert decided.float().mean() > 0.98
    assert torch.equal(got_bits[decided], (proj >= 0)[decided])
    want_vn = orc.value_norm(v).permute(0, 2, 1)
    assert torch.allclose(vn[..., t0:t0 + S].cpu().float(), want_vn.float(), rtol=1e-3, atol=0)


def test_hash_keys_drops_rows_whose_device_position_is_outside_the_cache(dev):
    """Per-sequence positions live on the device; a row that would land at or past
    the cache's capacity (or before its start) must be dropped, not written: the
    word after the last row of `codes` is outside the buffer."""
    g = torch.Generator().manual_seed(3)
    B, Hkv, D, L, P, Tcap = 3, 2, 128, 60, 10, 64
    NW = orc.words_per_key(L, P)
    pw = hash_cache.permute_planes(torch.randn(L, P, D, generator=g).to(dev))
    k = torch.randn(B, 1, Hkv, D, generator=g).to(torch.bfloat16).to(dev)
    v = torch.randn(B, 1, Hkv, D, generator=g).to(torch.bfloat16).to(dev)
    # one buffer with guard words around the cache proper
    pad = 16
    raw_c = torch.full((B * Hkv * NW * Tcap + 2 * pad,), -1, dtype=torch.int32, device=dev)
    raw_n = torch.full((B * Hkv * Tcap + 2 * pad,), -1.0, dtype=torch.float16, device=dev)
    codes = raw_c[pad:-pad].view(B, Hkv, NW, Tcap)
    vn = raw_n[pad:-pad].view(B, Hkv, Tcap)
    pos = torch.tensor([Tcap, 5, -1], dtype=torch.int32, device=dev)      # past the end, inside, before the start
    hash_cache.hash_keys_into(k, v, pw, codes, vn, L, P, pos_b=pos, layout="bshd")
    torch.cuda.synchronize()
    assert (raw_c[:pad] == -1).all() and (raw_c[-pad:] == -1).all()
    assert (raw_n[:pad] == -1).all() and (raw_n[-pad:] == -1).all()
    assert (codes[0] == -1).all() and (codes[2] == -1).all() and (vn[0] == -1).all() and (vn[2] == -1).all()
    assert (codes[1, :, :, 5] != -1).all() and (vn[1, :, 5] != -1).all()
    touched = codes[1].clone(); touched[:, :, 5] = -1
    assert (touched == -1).all()


def test_hash_identity_planes_and_sign_flip(dev):
    """planes = +-unit vectors -> bits are the sign bits of key coordinates;
    hash(a*k) = hash(k) for a > 0; hash(-k) = ~hash(k) when no projection is 0."""
    L, P, D, S = 8, 10, 128, 200
    g = torch.Generator().manual_seed(1)
    planes = torch.zeros(L, P, D)
    coord = torch.randperm(D, generator=g)[:L * P].view(L, P)
    sign = torch.where(torch.rand(L, P, generator=g) > 0.5, 1.0, -1.0)
    planes.view(-1, D).scatter_(1, coord.view(-1, 1), sign.view(-1, 1))
    k = torch.randn(1, S, 1, D, generator=g).to(torch.bfloat16)
    NW = orc.words_per_key(L, P)
    pw = hash_cache.permute_planes(planes.to(dev))

    def run(x):
        codes = torch.zeros((1, 1, NW, 208), dtype=torch.int32, device=dev)
        hash_cache.hash_keys_into(x.to(dev), None, pw, codes, None, L, P, layout="bshd")
        return hash_cache.unpack_codes(codes, L, P, 0, S, layout="bthl").cpu()

    got = run(k)
    bits = (k.float()[0, :, 0][:, coord] * sign) >= 0                      # [S,L,P]
    assert torch.equal(got[0, :, 0], orc.pack_bits(bits))
    assert torch.equal(run(k * 3), got)
    assert torch.equal(run(-k)[0, :, 0].int(), (~got[0, :, 0].int()) & ((1 << P) - 1))


def test_pack_unpack_round_trip(dev):
    g = torch.Generator().manual_seed(2)
    for L, P in ((60, 10), (32, 8), (5, 16), (33, 1), (7, 11)):
        T = 301
        codes = _rand_codes(g, 2, 3, L, T, min(P, 15))
        NW = orc.words_per_key(L, P)
        words = torch.zeros((2, 3, NW, 304), dtype=torch.int32, device=dev)
        hash_cache.pack_codes_into(codes.to(dev), words, P, t0=2)
        want = orc.pack_code_words(codes.numpy(), P)
        assert np.array_equal(words[..., 2:2 + T].cpu().numpy().view(np.uint32), want)
        back = hash_cache.unpack_codes(words, L, P, 2, T).cpu()
        assert torch.equal(back, codes)


# ---------------------------------------------------------------- K5 query soft hash
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Hq,Hkv,D,L,K,R,temp,cube", [
    (2, 8, 2, 128, 20, 10, 1024, 1.0, False),      # GPT-FAST: random prototypes, no temperature
    (1, 28, 4, 128, 12, 10, 1024, 0.3, True),      # HF twin: hypercube corners, logits / 0.3, G = 7
    (3, 4, 4, 64, 5, 4, 16, 1.0, True),            # small R, one head per group
    (1, 6, 3, 32, 3, 3, 8, 0.3, False),
])
def test_soft_hash_matches_oracle(dev, dtype, B, Hq, Hkv, D, L, K, R, temp, cube):
    g = torch.Generator().manual_seed(B * 1000 + Hq + L)
    q = torch.randn(B, Hq, D, generator=g).to(dtype)
    planes = (torch.randn(L, K, D, generator=g) * (1.0 if cube else 0.3)).to(dtype)
    protos = (orc.hypercube_protos_T(K) if cube else torch.randn(K, R, generator=g) * 3.0).to(dtype)
    want = orc.soft_hash(q.float(), planes.float(), protos.float(), temperature=temp)       # fp32 on the stored values
    have32 = hash_cache.soft_hash(q.to(dev), planes.to(dev), protos.to(dev), temp, Hkv, out_dtype=torch.float32).cpu()
    assert have32.dtype == torch.float32 and tuple(have32.shape) == (B, Hq, L, R)
    torch.testing.assert_close(have32, want, rtol=2e-5, atol=1e-9)
    torch.testing.assert_close(have32.sum(-1), torch.ones(B, Hq, L), rtol=1e-5, atol=1e-5)
    # grouping of heads into workgroups does not change the values
    alone = hash_cache.soft_hash(q.to(dev), planes.to(dev), protos.to(dev), temp, Hq, out_dtype=torch.float32).cpu()
    assert torch.equal(alone, have32)
    # bf16 output: the fp32 value rounded once
    have16 = hash_cache.soft_hash(q.to(dev), planes.to(dev), protos.to(dev), temp, Hkv, out_dtype=torch.bfloat16).cpu()
    assert have16.dtype == torch.bfloat16 and torch.equal(have16, have32.to(torch.bfloat16))
    if cube and R == 1 << K:
        # hypercube prototypes: the most probable bucket is the query's hard hash
        proj = orc.projections_f64(q.float().unsqueeze(1).permute(0, 1, 2, 3).reshape(B, 1, Hq, D), planes.float())
        clear = (proj.abs() > 1e-4).all(-1)[:, 0]                                            # [B,Hq,L]
        hard = orc.pack_bits(proj >= 0)[:, 0].long()
        assert torch.equal(have32.argmax(-1)[clear], hard[clear])


def _bf16_ulps(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in bf16 units in the last place between two non-negative bf16 tensors."""
    return (a.view(torch.int16).int() - b.view(torch.int16).int()).abs()


@pytest.mark.parametrize("name,Hq,Hkv,L,temp,cube,plane_scale,proto_scale", [
    ("gpt-fast", 32, 8, 60, 1.0, False, 0.3, 3.0),    # GPT-FAST/model.py:392-401: random prototypes, no temperature
    ("hf", 28, 4, 48, 0.3, True, 1.0, 1.0),           # modeling_llama.py:618-638: hypercube corners, logits / 0.3
])
def test_bf16_soft_hash_against_the_reference_dtype_chain(dev, name, Hq, Hkv, L, temp, cube, plane_scale, proto_scale):
    """The reference runs its two einsums, the tanh, the division and the softmax in the
    model dtype, rounding to bf16 after each (the oracle's soft_hash does the same when
    it is handed bf16 tensors); the kernel computes in fp32 and rounds once.  Stated
    bound: every entry within 8 bf16 units in the last place of the reference-dtype
    chain (measured: at most 4, 0.04-31 % of the entries differ at all, depending on how
    peaked the tables are), every row still summing to 1 within bf16 rounding -- and the
    difference does not move the selection: at a 32768-token context with top-1024 the
    lists built from the two tables share at least 98 % of their entries in every row."""
    g = torch.Generator().manual_seed(77 + L)
    B, D, K, T, M = 1, 128, 10, 32768, 1024
    R, G = 1 << K, Hq // Hkv
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16)
    planes = (torch.randn(L, K, D, generator=g) * plane_scale).to(torch.bfloat16)
    protos = (orc.hypercube_protos_T(K) if cube else torch.randn(K, R, generator=g) * proto_scale).to(torch.bfloat16)
    chain = orc.soft_hash(q, planes, protos, temperature=temp)                        # bf16 at every step
    assert chain.dtype == torch.bfloat16
    have = hash_cache.soft_hash(q.to(dev), planes.to(dev), protos.to(dev), temp, Hkv, out_dtype=torch.bfloat16)
    ulps = _bf16_ulps(have.cpu(), chain)
    frac = float((ulps > 0).float().mean())
    print(f"soft hash {name}: {100 * frac:.2f} % of entries differ from the bf16 chain, max {int(ulps.max())} ulps")
    assert int(ulps.max()) <= 8
    assert float((have.float().sum(-1) - 1).abs().max()) <= 4e-3
    # the selection from either table
    keys = torch.randn(B, T, Hkv, D, generator=g).to(torch.bfloat16)
    vals = torch.randn(B, T, Hkv, D, generator=g).to(torch.bfloat16)
    cache = hash_cache.SocketHashCache(B, T, Hkv, D, L, K, dtype=torch.bfloat16, device=dev)
    cache.set_planes(planes.float())
    cache.append(0, keys.to(dev), vals.to(dev))
    lists = []
    for table in (have, chain.to(dev)):
        scores = hash_cache.score_packed(table, cache.codes, cache.v_norm, T, K)
        sl, _ = sparse.select_list(scores, 0, 0, M, write_base=False)
        lists.append(sl.cpu())
    worst = 1.0
    for h in range(Hq):
        a, b = set(lists[0][0, h].tolist()), set(lists[1][0, h].tolist())
        assert len(a) == M and len(b) == M
        worst = min(worst, len(a & b) / M)
    print(f"soft hash {name}: smallest top-{M} overlap over {Hq} rows {worst:.4f}")
    assert worst >= 0.98


@pytest.mark.parametrize("B,Hq,Hkv,L,P,T,dtype", [
    (2, 8, 2, 20, 10, 5000, torch.bfloat16),     # G=4
    (1, 14, 2, 12, 10, 3000, torch.bfloat16),    # G=7: two parts of width 4
    (2, 6, 2, 9, 8, 2000, torch.float32),        # G=3 padded to 4
    (1, 4, 4, 7, 10, 1500, torch.float32),       # G=1
    (1, 4, 2, 6, 10, 1500, torch.bfloat16),      # G=2
    (4, 32, 8, 60, 10, 20000, torch.bfloat16),   # large tile
    (8, 32, 8, 60, 10, 70000, torch.bfloat16),   # a tile for every CU: slices go straight from global memory to LDS
    (8, 56, 8, 20, 10, 33000, torch.float32),    # the same with fp32 entries and split head groups
    (16, 16, 16, 7, 8, 9000, torch.bfloat16),    # ... and one head per group, P = 8
    (1, 32, 8, 60, 10, 65792, torch.bfloat16),   # a context that overhangs 16 tiles of 4096 by a little: 29 even tiles per row
    (1, 32, 8, 60, 10, 100000, torch.float32),   # ... 25 tiles of 4096 on 200 CUs, or 31 of 3328
    (2, 14, 2, 48, 10, 50000, torch.bfloat16),   # ... with two head parts per kv head
])
def test_grouped_table_layout_gives_identical_scores(dev, B, Hq, Hkv, L, P, T, dtype):
    """The grouped table (converter and fused producer) is a relayout only: the
    scorer returns bit-identical scores from it."""
    g = torch.Generator().manual_seed(Hq * 100 + L)
    R, G = 1 << P, Hq // Hkv
    q_probs = torch.softmax(torch.randn(B, Hq, L, R, generator=g) * 3, -1).to(dtype).to(dev)
    parts, width = hash_cache.group_shape(Hq, Hkv)
    assert width == (1 if G == 1 else 2 if G == 2 else 4) and parts == (G + width - 1) // width
    table = hash_cache.group_q_probs(q_probs, Hkv)
    assert tuple(table.shape) == (B, Hkv * parts, L, R, width) and table.dtype == dtype
    # the layout itself
    want = torch.zeros(B, Hkv, parts * width, L, R, dtype=dtype)
    want[:, :, :G] = q_probs.cpu().view(B, Hkv, G, L, R)
    want = want.view(B, Hkv, parts, width, L, R).permute(0, 1, 2, 4, 5, 3).reshape(B, Hkv * parts, L, R, width)
    assert torch.equal(table.cpu(), want)
    codes = _rand_codes(g, B, Hkv, L, T, P)
    Tcap = (T + 7) // 8 * 8
    vn = torch.zeros(B, Hkv, Tcap, dtype=torch.float16)
    vn[..., :T] = (torch.rand(B, Hkv, T, generator=g) * 5).to(torch.float16)
    lens = torch.randint(T // 2, T + 1, (B,), generator=g, dtype=torch.int32).to(dev)
    packed = _packed_cache(codes, P, Tcap, dev)
    a, ra = hash_cache.score_packed(q_probs, packed, vn.to(dev), T, P, lens=lens, with_range=True)
    b, rb = hash_cache.score_packed(table, packed, vn.to(dev), T, P, lens=lens, with_range=True, n_heads=Hq)
    # without the key ranges the launch is free to cut the rows otherwise (even tiles for a
    # context that overhangs a whole number of them, the persistent launch): same scores
    c = hash_cache.score_packed(table, packed, vn.to(dev), T, P, lens=lens, n_heads=Hq)
    assert torch.equal(torch.isinf(c), torch.isinf(b))
    assert ((c - b).abs() / b.abs().clamp_min(1e-30)).nan_to_num(0).max() <= (0.0 if dtype == torch.float32 else 2e-6)
    # A short context with few kv heads is scored from the [B,Hq,L,R] table one
    # head per workgroup, with plain fp32 adds; the grouped table always goes
    # through the several-heads-at-once accumulate, whose last-place rounding can
    # differ for bf16 entries.  fp32 entries: identical either way.
    if dtype == torch.float32:
        assert torch.equal(a, b)
    else:
        rel = ((a - b).abs() / b.abs().clamp_min(1e-30)).nan_to_num(0).max()
        assert rel <= 2e-6, f"max rel diff {rel}"
    if True:
        for r, sc in ((ra, a), (rb, b)):   # each range array against its own scores
            u, keys = r.cpu().numpy().view(np.uint32), _score_keys(sc.cpu())
            for bb in range(B):
                kk = keys[bb, :, :int(lens[bb])]
                assert np.array_equal(u[bb, ..., 0].min(-1), kk.min(-1))
                assert np.array_equal(u[bb, ..., 1].max(-1), kk.max(-1))


def test_soft_hash_grouped_output_is_the_grouped_relayout(dev):
    g = torch.Generator().manual_seed(77)
    for Hq, Hkv in ((8, 2), (14, 2), (6, 2), (4, 4)):
        q = torch.randn(2, Hq, 128, generator=g).to(torch.bfloat16).to(dev)
        planes = (torch.randn(7, 10, 128, generator=g) * 0.3).to(torch.bfloat16).to(dev)
        protos = (torch.randn(10, 1024, generator=g) * 3).to(torch.bfloat16).to(dev)
        for out_dtype in (torch.bfloat16, torch.float32):
            std = hash_cache.soft_hash(q, planes, protos, 1.0, Hkv, out_dtype=out_dtype)
            grp = hash_cache.soft_hash(q, planes, protos, 1.0, Hkv, out_dtype=out_dtype, grouped=True)
            assert torch.equal(grp, hash_cache.group_q_probs(std, Hkv))


def test_soft_hash_strided_queries_and_argument_checks(dev):
    g = torch.Generator().manual_seed(9)
    qkv = torch.randn(2, 1, 12, 128, generator=g).to(torch.bfloat16).to(dev)      # queries are heads 0..7 of a wider row
    q = qkv[:, 0, :8]
    planes = torch.randn(6, 10, 128, generator=g).to(torch.bfloat16).to(dev)
    protos = torch.randn(10, 1024, generator=g).to(torch.bfloat16).to(dev)
    a = hash_cache.soft_hash(q, planes, protos, 1.0, 2)
    b = hash_cache.soft_hash(q.contiguous(), planes, protos, 1.0, 2)
    assert a.dtype == torch.bfloat16 and torch.equal(a, b)
    from socket_amd._lib import SocketHipError
    with pytest.raises(SocketHipError):
        hash_cache.soft_hash(q, planes, protos[:, :6].contiguous(), 1.0, 2)       # R not a multiple of 4
    with pytest.raises(AssertionError):
        hash_cache.soft_hash(q, planes[:, :4], protos, 1.0, 2)


# ---------------------------------------------------------------- whole step
@pytest.mark.parametrize("name,T", [("c1", 4096), ("c2", 8192)])
def test_decode_step_end_to_end(dev, name, T):
    """hash -> score -> select -> attend on a benchmark configuration (C2 with a
    shorter context so the oracle finishes in seconds)."""
    w = scaled(WORKLOADS[name], T=T, M=min(WORKLOADS[name].M, T // 8))
    inp = make_inputs(w, device="cpu")
    cache = hash_cache.SocketHashCache(w.B, T, w.Hkv, w.D, w.L, w.P, dtype=w.dtype, device=dev)
    cache.set_planes(inp.planes)
    cache.append(0, inp.k.permute(0, 2, 1, 3).to(dev), inp.v.permute(0, 2, 1, 3).to(dev))
    out, scores, sl, ln = hash_cache.sparse_decode_step(
        inp.q.to(dev), inp.q_probs.to(dev), cache.k_cache, cache.v_cache, cache.codes, cache.v_norm,
        T, w.P, w.sink, w.window, w.M, return_details=True)
    # oracle on the device's own codes / norms (hash parity is covered separately)
    codes = hash_cache.unpack_codes(cache.codes, w.L, w.P, 0, T).cpu()
    vnorm = cache.v_norm[..., :T].cpu()
    allowed = torch.ones(w.B, w.Hq, T, dtype=torch.bool)
    wl, wn, wscores = orc.build_sparse_list_decode(
        inp.q_probs, codes.repeat_interleave(w.G, 1), vnorm.repeat_interleave(w.G, 1), allowed,
        w.sink, w.window, w.M, return_scores=True)
    rel = ((scores.cpu() - wscores).abs() / wscores.abs().clamp_min(1e-30)).max()
    assert rel <= 1e-5
    # top-k exact on the device's own scores, and (scores being equal) on the oracle's
    wl2 = torch.cat([wl[..., :wl.shape[-1] - w.M], orc.topk_lower_index_first(scores.cpu(), w.M).int()], -1)
    assert torch.equal(sl.cpu(), wl2) and torch.equal(ln.cpu(), wn)
    assert torch.equal(sl.cpu(), wl)
    want = orc.sparse_attend_textbook(inp.q, inp.k, inp.v, wl, wn)
    assert (out.cpu().double() - want).abs().max() <= ATOL[w.dtype]
    # planted heavy keys are found: most of them are inside the selected set
    # (a sanity check of the whole chain, not a parity bar)
    assert out.dtype == w.dtype

# ---------------------------------------------------------------- persistent scorer
def _definition_scores(qp, codes, vn, lens, T, G):
    """Sequential fp32 sum over tables of gathered entries, times the value norm, -inf
    past the length (soft_hash_collision.cu:45-53), with torch on the device."""
    B, Hq, L, _ = qp.shape
    want = torch.zeros(B, Hq, T, dtype=torch.float32, device=qp.device)
    ce, qf = codes.long().repeat_interleave(G, dim=1), qp.float()
    for l in range(L):
        want += torch.gather(qf[:, :, l], 2, ce[:, :, l])
    want *= vn[..., :T].float().repeat_interleave(G, dim=1)
    if lens is not None:
        want = want.masked_fill(torch.arange(T, device=qp.device)[None, None, :] >= lens[:, None, None], float("-inf"))
    return want


@pytest.mark.parametrize("B,Hkv,G,L,P,T,dt,lens_kind", [
    (16, 4, 7, 48, 10, 16400, torch.bfloat16, "ragged"),   # two head parts per kv head, odd context
    (16, 4, 7, 48, 10, 16400, torch.float32, "ragged"),
    (4, 8, 4, 60, 10, 66000, torch.bfloat16, "ragged"),
    (4, 8, 4, 60, 10, 66000, torch.float32, "edges"),
    (8, 8, 2, 32, 8, 33000, torch.bfloat16, "edges"),      # P = 8, two heads per entry
    (64, 2, 3, 12, 10, 17000, torch.bfloat16, "ragged"),   # the most sequences one wave ranks, a padded head group
    (4, 8, 4, 60, 10, 65536, torch.bfloat16, "none"),      # no lengths: every row full
    (2, 16, 4, 60, 10, 70001, torch.float32, "full"),
    (1, 8, 4, 60, 10, 131072, torch.bfloat16, "ragged"),   # half a tile per CU: one token group per wave
    (2, 8, 4, 60, 10, 40000, torch.float32, "edges"),      # ... a third
    (1, 8, 4, 60, 10, 65792, torch.bfloat16, "full"),      # ... a quarter, and a context that overhangs the tiles
    (3, 4, 7, 48, 10, 50000, torch.bfloat16, "ragged"),    # ... with two head parts
])
def test_persistent_scorer_on_ragged_batches(dev, B, Hkv, G, L, P, T, dt, lens_kind):
    """Calls large enough for the one-workgroup-per-CU launch that is dealt from the
    cached lengths (a quarter of a tile for every CU and more, grouped table, full packed words):
    sequences of length 0, 1, around the 512-token unit and the 8192-token tile, equal
    to the context, or absent; with and without the -inf fill past the lengths.
    Scores equal the definition (bit for bit with an fp32 table)."""
    R, Hq = 1 << P, Hkv * G
    g = torch.Generator(device=dev).manual_seed(B * 131 + T)
    qp = (torch.rand(B, Hq, L, R, generator=g, device=dev) *
          torch.exp(-8 * torch.rand(B, Hq, L, R, generator=g, device=dev))).to(dt)
    codes = torch.randint(0, R, (B, Hkv, L, T), generator=g, device=dev, dtype=torch.int32).to(torch.int16)
    Tcap = (T + 64 + 7) // 8 * 8
    packed = torch.zeros(B, Hkv, orc.words_per_key(L, P), Tcap, dtype=torch.int32, device=dev)
    hash_cache.pack_codes_into(codes, packed, P, t0=0)
    vn = torch.zeros(B, Hkv, Tcap, dtype=torch.float16, device=dev)
    vn[..., :T] = (torch.rand(B, Hkv, T, generator=g, device=dev) * 6).to(torch.float16)
    if lens_kind == "none":
        lens = None
    elif lens_kind == "full":
        lens = torch.full((B,), T, dtype=torch.int32, device=dev)
    elif lens_kind == "edges":
        pool = [0, 1, 3, 4, 511, 512, 513, 8191, 8192, 8193, 8704, T - 1, T, T // 2 + 2, 12345, 1025]
        lens = torch.tensor([pool[i % len(pool)] for i in range(B)], dtype=torch.int32, device=dev).clamp_(max=T)
    else:
        lens = torch.randint(0, T + 1, (B,), generator=g, device=dev, dtype=torch.int32)
        lens[0] = T
        if B > 2:
            lens[1] = 0
    table = hash_cache.group_q_probs(qp, Hkv)
    want = _definition_scores(qp, codes, vn, lens, T, G)
    tol = 0.0 if dt == torch.float32 else 2e-6
    got = hash_cache.score_packed(table, packed, vn, T, P, lens=lens, n_heads=Hq)
    assert torch.equal(torch.isinf(got), torch.isinf(want))
    rel = ((got - want).abs() / want.abs().clamp_min(1e-30)).nan_to_num(0).max().item()
    assert rel <= tol, f"max rel diff {rel}"
    # the tiled launches (asking for the key ranges keeps a call on them): same values
    ref_layout, _ = hash_cache.score_packed(qp, packed, vn, T, P, lens=lens, with_range=True)
    # a [B,Hq,L,R] table of this size is regrouped on the way in and served the same way
    assert torch.equal(hash_cache.score_packed(qp, packed, vn, T, P, lens=lens), got)
    rel = ((got - ref_layout).abs() / ref_layout.abs().clamp_min(1e-30)).nan_to_num(0).max().item()
    assert rel <= tol
    # without the fill: rows equal up to their lengths, nothing written past the length's float4
    pitch = (T + 3) // 4 * 4
    out = torch.full((B, Hq, pitch), 123.0, dtype=torch.float32, device=dev)
    got2 = hash_cache.score_packed(table, packed, vn, T, P, lens=lens, n_heads=Hq, out=out, skip_masked=True)
    for b in range(B):
        n = T if lens is None else int(lens[b])
        assert torch.equal(got2[b, :, :n], got[b, :, :n])
        assert (out[b, :, (n + 3) // 4 * 4:T] == 123.0).all()
    # twice in a row into the same buffer: no state is carried between launches
    again = hash_cache.score_packed(table, packed, vn, T, P, lens=lens, n_heads=Hq)
    assert torch.equal(again, got)


# ---------------------------------------------------------------- randomized shapes
@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_score_and_select(dev, seed):
    """Scorer and selector on randomly drawn geometries (head groups, table sizes,
    context lengths around the tile and slice boundaries, ragged lengths, padding
    in the cache rows), checked on the device against the definitions: the score
    as a sequential fp32 sum over tables of gathered entries
    (soft_hash_collision.cu:45-53), the heavy part of the list as a stable
    descending sort of the row (ties: lower index first)."""
    import random
    rnd = random.Random(seed)
    for _ in range(8):
        G = rnd.choice([1, 2, 3, 4, 4, 7, 8])
        Hkv = rnd.choice([1, 2, 4, 8])
        B = rnd.choice([1, 1, 2, 4])
        P = rnd.choice([10, 10, 8, 6])
        L = rnd.choice([60, 48, 20, 7, 33])
        T = rnd.choice([300, 1000, 4099, 8192, 8200, 16384, 20000, 40000, 65536, 65792, 70000, 98304, 131072])
        if B * Hkv * G * T > 30e6:
            T = 20000
        dt = rnd.choice([torch.bfloat16, torch.float32])
        R, Hq = 1 << P, Hkv * G
        g = torch.Generator(device=dev).manual_seed(rnd.randrange(1 << 30))
        case = f"B{B} Hq{Hq} Hkv{Hkv} L{L} P{P} T{T} {dt}"
        qp = (torch.rand(B, Hq, L, R, generator=g, device=dev) *
              torch.exp(-8 * torch.rand(B, Hq, L, R, generator=g, device=dev))).to(dt)
        codes = torch.randint(0, R, (B, Hkv, L, T), generator=g, device=dev, dtype=torch.int32).to(torch.int16)
        Tcap = (T + rnd.choice([0, 8, 64]) + 7) // 8 * 8
        packed = torch.zeros(B, Hkv, orc.words_per_key(L, P), Tcap, dtype=torch.int32, device=dev)
        hash_cache.pack_codes_into(codes, packed, P, t0=0)
        vn = torch.zeros(B, Hkv, Tcap, dtype=torch.float16, device=dev)
        vn[..., :T] = (torch.rand(B, Hkv, T, generator=g, device=dev) * 6).to(torch.float16)
        lens = torch.randint(max(1, T // 3), T + 1, (B,), generator=g, device=dev, dtype=torch.int32)
        a, ra = hash_cache.score_packed(qp, packed, vn, T, P, lens=lens, with_range=True)
        b_ = hash_cache.score_packed(hash_cache.group_q_probs(qp, Hkv), packed, vn, T, P, lens=lens, n_heads=Hq)
        want = torch.zeros(B, Hq, T, dtype=torch.float32, device=dev)
        ce, qf = codes.long().repeat_interleave(G, dim=1), qp.float()
        for l in range(L):
            want += torch.gather(qf[:, :, l], 2, ce[:, :, l])
        want *= vn[..., :T].float().repeat_interleave(G, dim=1)
        want = want.masked_fill(torch.arange(T, device=dev)[None, None, :] >= lens[:, None, None], float("-inf"))
        for name, got in (("[B,Hq,L,R] table", a[..., :T]), ("grouped table", b_[..., :T])):
            assert torch.equal(torch.isinf(got), torch.isinf(want)), f"{case}: {name}"
            rel = ((got - want).abs() / want.abs().clamp_min(1e-30)).nan_to_num(0).max().item()
            assert rel <= (0.0 if dt == torch.float32 else 2e-6), f"{case}: {name} max rel diff {rel}"
        M = rnd.choice([0, 1, 64, 1024, 2048, 3600])
        sink, window = rnd.choice([(4, 256), (0, 0), (120, 120), (4, 16)])
        sl, ln = sparse.select_list(a, sink, window, M, lens=lens, row_range=ra if rnd.random() < 0.5 else None)
        for bb in range(B):
            n = int(lens[bb])
            m, s_e, w_e = min(M, n), min(sink, n), min(window, n)
            ws = max(n - w_e, s_e)
            nbase = s_e + (n - ws if w_e > 0 else 0)
            nbase = max(nbase, 1)      # no sink, no window: the reference lists the newest token
            order = torch.sort(a[bb, :, :n], dim=-1, descending=True, stable=True).indices[:, :m]
            assert torch.equal(sl[bb, :, nbase:nbase + m].long(), order), f"{case}: sequence {bb}, M={M}"
            assert (sl[bb, :, nbase + m:] == -1).all() and (ln[bb] == nbase + m).all(), f"{case}: sequence {bb}"
