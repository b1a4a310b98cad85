"""socket_sparse_attention_static (the entry point that allocates nothing: its
per-split partials and row counters live in fixed arrays inside the library, and
the last split of a row merges the row in the same launch) against
socket_sparse_attention on the same inputs, through the C ABI.  Both use the same
split and the same merge arithmetic, so the outputs must be identical bit for bit.
Calls in a row share the arrays; later ones are smaller than the first."""
import pytest
import torch

from socket_amd import _lib, socket_kernels

pytestmark = pytest.mark.gpu


def _case(dev, seed, B, Hq, Hkv, T, width, dtype):
    g = torch.Generator().manual_seed(seed)
    D = 128
    q = torch.randn(B, Hq, D, generator=g).to(dtype).to(dev)
    k = torch.randn(B, Hkv, T, D, generator=g).to(dtype).to(dev)
    v = torch.randn(B, Hkv, T, D, generator=g).to(dtype).to(dev)
    sl = torch.randint(0, T, (B, Hq, width), generator=g, dtype=torch.int32)
    ln = torch.randint(1, width + 1, (B, Hq), generator=g, dtype=torch.int32)
    ln[0, 0] = width
    sl[0, 1, :3] = -1            # skipped entries
    ln[-1, -1] = 0               # nothing listed: the reference's 0/0
    ln[-1, 0] = 1
    return q, k, v, sl.to(dev), ln.to(dev)


def test_static_scratch_variant_equals_the_workspace_variant(dev):
    lib = _lib.lib()
    assert lib.socket_static_scratch_init() == 0
    # first a large call, then a smaller one that reuses the front of the same array
    for seed, (B, Hq, Hkv, T, width, dtype) in enumerate([
            (4, 32, 8, 6000, 2308, torch.bfloat16),
            (1, 8, 2, 900, 196, torch.float32),
            (2, 28, 4, 3000, 1100, torch.float16)]):
        q, k, v, sl, ln = _case(dev, 100 + seed, B, Hq, Hkv, T, width, dtype)
        want = socket_kernels.sparse_attention_fwd(q, k, v, sl, ln)
        out = torch.full_like(want, float("nan"))
        torch.cuda.synchronize()
        allocs = torch.cuda.memory_stats()["allocation.all.allocated"]
        got = socket_kernels.sparse_attention_fwd_static(q, k, v, sl, ln, out)
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == allocs   # no allocation through torch either
        torch.cuda.synchronize()
        assert torch.isnan(want[-1, -1]).all() and torch.isnan(got[-1, -1]).all()
        want[-1, -1] = 0
        got[-1, -1] = 0
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got, want), f"case {seed}: max diff {(got.float() - want.float()).abs().max()}"
    # the row counters are back at zero: the same call again gives the same result
    again = socket_kernels.sparse_attention_fwd_static(q, k, v, sl, ln, torch.empty_like(got))
    again[-1, -1] = 0
    assert torch.equal(again, got)


def test_one_launch_merge_over_many_rows_and_split_counts(dev):
    """The hand-over between the splits of a row (written-through partials, a ticket per
    row, the last arriver merges) under load: hundreds of rows whose lengths give every
    number of running splits from 1 to the launch's maximum, calls of different shapes
    issued back to back on one stream with no synchronisation in between, three rounds.
    Every output must equal the two-launch result bit for bit; the first mismatch stops
    the test and names its call."""
    lib = _lib.lib()
    shapes = [(8, 32, 8, 5000, 4096), (2, 32, 8, 3000, 1156), (16, 28, 4, 4000, 2100), (32, 32, 8, 900, 600),
              (1, 32, 8, 7000, 2308)]
    cases = []
    for i, (B, Hq, Hkv, T, width) in enumerate(shapes):
        g = torch.Generator().manual_seed(500 + i)
        q = torch.randn(B, Hq, 128, generator=g).to(torch.bfloat16).to(dev)
        k = torch.randn(B, Hkv, T, 128, generator=g).to(torch.bfloat16).to(dev)
        v = torch.randn(B, Hkv, T, 128, generator=g).to(torch.bfloat16).to(dev)
        sl = torch.randint(0, T, (B, Hq, width), generator=g, dtype=torch.int32).to(dev)
        bs = lib.socket_sparse_attention_block_seq(B, Hq, width)
        nsplit = (width + bs - 1) // bs
        # row r runs 1 + r % nsplit splits: every count occurs, neighbours differ
        rows = torch.arange(B * Hq)
        ln = ((rows % nsplit) * bs + 1 + (rows * 7) % bs).clamp(max=width).to(torch.int32).view(B, Hq).to(dev)
        want = socket_kernels.sparse_attention_fwd(q, k, v, sl, ln)
        cases.append((q, k, v, sl, ln, want, torch.empty_like(want), nsplit))
    assert max(c[-1] for c in cases) >= 8
    torch.cuda.synchronize()
    for rnd in range(3):
        for c in cases:
            socket_kernels.sparse_attention_fwd_static(c[0], c[1], c[2], c[3], c[4], c[6])
        torch.cuda.synchronize()
        for i, c in enumerate(cases):
            assert torch.equal(c[6], c[5]), f"round {rnd}, call {i} {shapes[i]}: " \
                                            f"{int((c[6] != c[5]).any(-1).sum())} rows differ"
            c[6].fill_(float("nan"))


def test_static_scratch_variant_refuses_what_does_not_fit(dev):
    lib = _lib.lib()
    B, Hq, Hkv, T, width = 64, 512, 8, 64, 4096
    assert lib.socket_sparse_attention_workspace_bytes(B, Hq, 128, width) > lib.socket_static_scratch_bytes()
    q = torch.zeros(B, Hq, 128, dtype=torch.bfloat16, device=dev)
    k = torch.zeros(B, Hkv, T, 128, dtype=torch.bfloat16, device=dev)
    sl = torch.zeros(B, Hq, width, dtype=torch.int32, device=dev)
    ln = torch.ones(B, Hq, dtype=torch.int32, device=dev)
    with pytest.raises(_lib.SocketHipError, match="workspace"):
        socket_kernels.sparse_attention_fwd_static(q, k, k, sl, ln, torch.empty_like(q))
