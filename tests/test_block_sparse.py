"""Block-sparse prefill attention (kernels/block_sparse_flash_attention.py): the
index builders against a literal restatement of the reference's pipeline and the
properties it promises, the oracle attention against dense causal attention, and
the HIP kernel against the oracle (2e-2 absolute in bf16 / fp16, the bar stated
for attention outputs)."""
import math
import random

import pytest
import torch
import torch.nn.functional as F

from oracle import block_sparse_oracle as bso
from socket_amd import block_sparse_flash_attention as bsa


def _rand_cases(seed, n):
    rnd = random.Random(seed)
    for _ in range(n):
        yield dict(B=rnd.choice([1, 2]), R=rnd.choice([1, 2, 5, 9, 16]), C=rnd.choice([1, 3, 9, 16, 20]),
                   K=rnd.choice([1, 2, 4, 8, 30]), window=rnd.choice([None, 0, 1, 2, 4]),
                   causal=rnd.choice([True, True, False]), diag=rnd.choice([True, True, False]),
                   seed=rnd.randrange(1 << 30))


# ---------------------------------------------------------------- index builders (CPU)
def test_block_level_builder_matches_the_literal_pipeline():
    for c in _rand_cases(1, 60):
        g = torch.Generator().manual_seed(c["seed"])
        probs = torch.rand(c["B"], c["R"], c["C"], generator=g)
        got = bsa.random_walk_indices_from_block_probs(probs, c["K"], enforce_causal_blocks=c["causal"],
                                                       force_include_diagonal=c["diag"], window_blocks=c["window"])
        want = bso.random_walk_indices_from_block_probs(probs, c["K"], c["causal"], c["diag"], c["window"])
        assert got.dtype == torch.int32 and torch.equal(got, want), c


def test_token_level_builder_matches_the_literal_pipeline():
    rnd = random.Random(2)
    for _ in range(25):
        bm, bn = rnd.choice([(4, 4), (8, 4), (4, 8), (3, 5)])
        B, Tq, Tk = rnd.choice([1, 2]), rnd.randrange(1, 40), rnd.randrange(1, 40)
        K, window = rnd.choice([1, 3, 8]), rnd.choice([None, 2, 4])
        g = torch.Generator().manual_seed(rnd.randrange(1 << 30))
        # integer-valued entries: block sums are exact in fp32 and in the float64 restatement alike
        probs = torch.randint(0, 1000, (B, Tq, Tk), generator=g).float()
        got = bsa.random_walk_indices(probs, bm, bn, K, window_blocks=window)
        want = bso.random_walk_indices(probs, bm, bn, K, window_blocks=window)
        assert torch.equal(got, want), (bm, bn, B, Tq, Tk, K, window)


def test_builders_keep_their_promises():
    """Valid ids, causal, diagonal present, sorted, min(K, C) entries
    (kernels/block_sparse_flash_attention.py:21-27)."""
    g = torch.Generator().manual_seed(3)
    B, T, blk, K = 2, 1000, 64, 6
    probs = torch.rand(B, T, T, generator=g)
    idx = bsa.random_walk_indices(probs, blk, blk, K, window_blocks=3)
    R = C = -(-T // blk)
    assert tuple(idx.shape) == (B, R, min(K, C)) and idx.dtype == torch.int32
    assert (idx >= 0).all() and (idx < C).all()
    assert (idx[..., 1:] >= idx[..., :-1]).all()
    rows = torch.arange(R)
    assert (idx <= rows[None, :, None]).all()                       # square blocks: causal = at or left of the diagonal
    assert (idx == rows[None, :, None]).any(-1).all()               # the diagonal block is always listed
    # (not promised, and not the case: block 0 and the window survive the cut only where the
    # list has room -- the cut keeps the SMALLEST ids and the diagonal)


def test_hand_worked_block_list():
    """5 row blocks, K = 3, window of 2: forced = {0, r-1, r}; the pipeline pads the
    forced lists to three entries, appends three fills, and after the repeats are
    zeroed the first three slots are zeros for every row; slot 0 becomes the diagonal."""
    probs = torch.tensor([[[0.0, 0, 0, 0, 0], [5, 0, 0, 0, 0], [1, 9, 0, 0, 0], [7, 1, 2, 0, 0], [1, 8, 3, 2, 0]]])
    got = bsa.random_walk_indices_from_block_probs(probs, 3, window_blocks=2)
    # row 4: forced {0,3,4}; fill = top-3 of {1:8, 2:3} -> [1, 2, (-inf -> 0)]; cat sorted [0,0,1,2,3,4] -> repeats
    # zeroed [0,0,1,2,3,4] -> first three [0,0,1] -> slot 0 := 4 -> sorted [0,1,4]
    assert got[0, 4].tolist() == [0, 1, 4]
    # row 0: only block 0 is causal: [0,0,0] -> diagonal 0
    assert got[0, 0].tolist() == [0, 0, 0]
    assert torch.equal(got, bso.random_walk_indices_from_block_probs(probs, 3, window_blocks=2))


def test_block_mask_builder():
    g = torch.Generator().manual_seed(4)
    for K in (None, 0, 2, 5, 40):
        allow = torch.rand(2, 7, 7, generator=g) > 0.5
        got = bsa.block_mask_to_indices(allow, 64, 64, K)
        assert torch.equal(got, bso.block_mask_to_indices(allow, 64, 64, K)), K
    full = bsa.block_mask_to_indices(torch.ones(1, 4, 4, dtype=torch.bool), 64, 64)
    assert full[0].tolist() == [[0, 0, 0, 0], [0, 1, 0, 0], [0, 1, 2, 0], [0, 1, 2, 3]]   # padding with block 0 at the end
    heads = bsa.expand_block_index_to_heads(full, 3)
    assert tuple(heads.shape) == (1, 3, 4, 4) and heads.is_contiguous() and heads.dtype == torch.int32
    assert torch.equal(heads[0, 2], full[0])


# ---------------------------------------------------------------- oracle attention pins (CPU)
def _all_causal_lists(B, H, T):
    """Every causal block exactly once per row block, padded with FUTURE blocks
    (fully masked, so they add nothing) instead of repeats of block 0."""
    R = -(-T // 64)
    idx = torch.zeros(B, H, R, R, dtype=torch.int32)
    for r in range(R):
        idx[:, :, r] = torch.tensor(list(range(r + 1)) + [R - 1] * (R - r - 1) if r < R - 1 else list(range(R)))
    return idx


def test_oracle_equals_dense_causal_attention_when_every_block_is_listed_once():
    g = torch.Generator().manual_seed(5)
    B, H, T, D = 1, 2, 150, 32
    q, k, v = (torch.randn(B, H, T, D, generator=g) for _ in range(3))
    idx = _all_causal_lists(B, H, T)
    # the last row block's padding would repeat a visible block: there is none (R-1 entries + itself)
    got = bso.block_sparse_attention(q, k, v, torch.tensor([T]), idx)
    want = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=True)
    assert torch.allclose(got, want, atol=1e-7, rtol=1e-7)


def test_oracle_counts_a_block_listed_twice_twice():
    """One row block, block 0 listed k times: softmax weights are unchanged (every
    term is multiplied by k), so the output equals plain causal attention up to the
    1e-9 in the denominator -- and listing a second block once next to a doubled
    first one shifts weight towards the first by exactly the factor 2."""
    g = torch.Generator().manual_seed(6)
    q, k, v = (torch.randn(1, 1, 128, 16, generator=g) for _ in range(3))
    once = bso.block_sparse_attention(q, k, v, torch.tensor([128]), torch.tensor([[[[0], [0]]]], dtype=torch.int32))
    thrice = bso.block_sparse_attention(q, k, v, torch.tensor([128]), torch.tensor([[[[0, 0, 0], [0, 0, 0]]]], dtype=torch.int32))
    assert torch.allclose(once, thrice, atol=1e-8)
    # row 100 sees keys 0..63 (block 0) and 64..100 (block 1); with block 0 doubled:
    got = bso.block_sparse_attention(q, k, v, torch.tensor([128]), torch.tensor([[[[0, 0, 0], [0, 0, 1]]]], dtype=torch.int32))
    s = (q[0, 0, 100].double() @ k[0, 0, :101].double().T) / math.sqrt(16)
    w = torch.exp(s - s.max())
    w[:64] *= 2
    want = (w[:, None] * v[0, 0, :101].double()).sum(0) / w.sum()
    assert torch.allclose(got[0, 0, 100], want, atol=1e-7)


# ---------------------------------------------------------------- the HIP kernel
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,H,T,D,K", [(2, 3, 300, 128, 4), (1, 2, 64, 64, 1), (2, 2, 257, 32, 3), (1, 4, 200, 16, 5),
                                       (1, 1, 1000, 128, 8)])
def test_kernel_matches_oracle(dev, dtype, B, H, T, D, K):
    g = torch.Generator().manual_seed(T + D)
    q, k, v = (torch.randn(B, H, T, D, generator=g).to(dtype) for _ in range(3))
    seqlens = torch.tensor([T] + [max(1, T - 70)] * (B - 1), dtype=torch.int32)
    probs = torch.rand(B, T, T, generator=g)
    blocks = bsa.expand_block_index_to_heads(bsa.random_walk_indices(probs, 64, 64, K, window_blocks=2), H)
    got = bsa.random_walk_sparse_attention(q.to(dev), k.to(dev), v.to(dev), seqlens.to(dev), blocks.to(dev)).cpu()
    want = bso.block_sparse_attention(q.float(), k.float(), v.float(), seqlens, blocks)
    live = ~torch.isnan(want[..., 0])
    assert live.any() and (got[~live] == 0).all()                       # rows past the sequence come back as zeros
    err = (got.double()[live] - want[live]).abs().max().item()
    assert err <= 2e-2, f"max abs err {err}"


@pytest.mark.gpu
def test_kernel_is_dense_causal_attention_when_every_block_is_listed(dev):
    g = torch.Generator().manual_seed(9)
    B, H, T, D = 1, 4, 1500, 128
    q, k, v = (torch.randn(B, H, T, D, generator=g).to(torch.bfloat16).to(dev) for _ in range(3))
    blocks = _all_causal_lists(B, H, T).to(dev)
    seqlens = torch.full((B,), T, dtype=torch.int32, device=dev)
    got = bsa.random_walk_sparse_attention(q, k, v, seqlens, blocks)
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert (got.float() - want).abs().max().item() <= 2e-2


@pytest.mark.gpu
def test_kernel_takes_strided_views_and_the_wrapper(dev):
    g = torch.Generator().manual_seed(10)
    B, H, T, D = 2, 2, 130, 64
    qkv = torch.randn(B, T, 3, H, D, generator=g).to(torch.bfloat16).to(dev)
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))           # [B,H,T,D] views, last dim contiguous
    probs = torch.rand(B, T, T, generator=g).to(dev)
    got = bsa.build_and_run_rw_sparse_attn(q, k, v, probs, block_size=64, Kblocks=2, window_blocks=1)
    blocks = bsa.expand_block_index_to_heads(bsa.random_walk_indices(probs.cpu(), 64, 64, 2, window_blocks=1), H)
    want = bso.block_sparse_attention(q.float().cpu(), k.float().cpu(), v.float().cpu(), torch.tensor([T, T]), blocks)
    assert (got.double().cpu() - want).abs().max().item() <= 2e-2
    with pytest.raises(RuntimeError):
        bsa.random_walk_sparse_attention(q, k, v, torch.full((B,), T, dtype=torch.int32, device=dev),
                                         blocks.to(dev), block_m=32, block_n=32)
