"""Host-side checks that need no GPU: the C-ABI library loads and exports every
symbol include/socket_hip.h declares, entry points reject bad arguments before
touching a device, the Python shims keep the reference's signatures, and the
synthetic workloads are deterministic."""
import ctypes
import inspect
import os
import re

import pytest
import torch

from socket_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "socket_hip.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        from socket_amd import build
        build.build()
    return _lib.lib()


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(socket_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    names = _declared()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in socket_hip.h but not exported"
    # and the binding table covers exactly the header
    assert sorted(_lib.SIGNATURES) == names


def test_status_strings_and_version(lib):
    assert lib.socket_abi_version() == 4
    seen = set()
    for st in range(0, -7, -1):
        s = lib.socket_status_string(st).decode()
        assert s and s != "unknown status"
        seen.add(s)
    assert len(seen) == 7
    assert lib.socket_status_string(-99).decode() == "unknown status"


def test_words_per_key(lib):
    assert lib.socket_words_per_key(60, 10) == 20      # 80 B per key
    assert lib.socket_words_per_key(48, 10) == 16      # 64 B
    assert lib.socket_words_per_key(32, 8) == 8        # 32 B
    assert lib.socket_words_per_key(5, 16) == 3
    assert lib.socket_words_per_key(0, 10) == 0 and lib.socket_words_per_key(4, 17) == 0 and lib.socket_words_per_key(4, 0) == 0


def test_entry_points_reject_bad_arguments_without_a_device(lib):
    nul = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)          # non-NULL, 16-byte aligned, never dereferenced: validation fails first
    # NULL pointers
    assert lib.socket_score_packed(nul, 0, one, one, nul, one, nul, 0, 1, 4, 1, 8, 10, 1024, 64, 64, 64, 0, nul) == _lib.SOCKET_ERR_NULL
    assert lib.socket_select_list(nul, 64, nul, nul, nul, 0, 1, 1, 64, 4, 0, 0, 1, one, 8, 8, nul, nul, 0, nul) == _lib.SOCKET_ERR_NULL
    assert lib.socket_hash_keys(nul, nul, 1, 0, 0, 128, 0, 0, 128, one, one, nul, nul, 0, 1, 1, 1, 128, 60, 10, 8, nul) == _lib.SOCKET_ERR_NULL
    # shapes
    assert lib.socket_score_packed(one, 0, one, one, nul, one, nul, 0, 1, 5, 2, 8, 10, 1024, 64, 64, 64, 0, nul) == _lib.SOCKET_ERR_SHAPE    # Hq % Hkv
    assert lib.socket_score_packed(one, 0, one, one, nul, one, nul, 0, 1, 4, 1, 8, 10, 512, 64, 64, 64, 0, nul) == _lib.SOCKET_ERR_SHAPE     # R < 2^P
    assert lib.socket_score_packed(one, 0, one, one, nul, one, nul, 0, 1, 4, 1, 8, 10, 1024, 65, 64, 68, 0, nul) == _lib.SOCKET_ERR_SHAPE    # T > Tcap
    assert lib.socket_score_packed(one, 0, one, one, nul, one, nul, 0, 1, 4, 1, 8, 10, 1024, 64, 66, 64, 0, nul) == _lib.SOCKET_ERR_ALIGN    # Tcap % 4
    assert lib.socket_score_packed(one, 2, one, one, nul, one, nul, 0, 1, 4, 1, 8, 10, 1024, 64, 64, 64, 0, nul) == _lib.SOCKET_ERR_UNSUPPORTED  # fp16 table
    assert lib.socket_score_packed(one, 0, one, one, nul, one, nul, 0, 1, 16, 1, 8, 10, 1024, 64, 64, 64, 0, nul) == _lib.SOCKET_ERR_UNSUPPORTED  # G = 16
    assert lib.socket_hash_keys(one, nul, 1, 0, 0, 64, 0, 0, 64, one, one, nul, nul, 0, 1, 1, 1, 64, 60, 10, 8, nul) == _lib.SOCKET_ERR_UNSUPPORTED  # D != 128
    assert lib.socket_hash_keys(one, nul, 1, 0, 0, 128, 0, 0, 128, one, one, nul, nul, 4, 1, 1, 8, 128, 60, 10, 8, nul) == _lib.SOCKET_ERR_SHAPE  # t0 + S > Tcap
    assert lib.socket_select_list(one, 64, nul, nul, nul, 0, 1, 1, 64, 20000, 0, 0, 1, one, 8, 8, nul, nul, 0, nul) == _lib.SOCKET_ERR_UNSUPPORTED  # M too large
    assert lib.socket_select_list(one, 32, nul, nul, nul, 0, 1, 1, 64, 4, 0, 0, 1, one, 8, 8, nul, nul, 0, nul) == _lib.SOCKET_ERR_SHAPE  # pitch < T
    need = lib.socket_select_workspace_bytes(1, 8, 131072, 2048)       # few long rows: a workspace is asked for
    assert need > lib.socket_select_workspace_zero_bytes(1, 8, 131072, 2048) > 0
    assert lib.socket_select_list(one, 131072, nul, nul, nul, 0, 1, 8, 131072, 2048, 4, 64, 1, one, 2400, 2400, nul, one, need - 1,
                                  nul) == _lib.SOCKET_ERR_WORKSPACE
    a = [one, one, one, 1, 128, 128, 0, 0, 128, 0, 0, 128, one, 8, 8, one, 1, 1, one, one]
    assert lib.socket_attend_stage1(*a, 1, 4, 1, 48, 16, 8, 1, 256, nul) == _lib.SOCKET_ERR_UNSUPPORTED       # D = 48
    assert lib.socket_attend_stage1(*a, 1, 5, 2, 128, 16, 8, 1, 256, nul) == _lib.SOCKET_ERR_SHAPE             # Hq % Hkv
    a[5] = 100                                                                                            # q head stride not 16-byte aligned for bf16
    assert lib.socket_attend_stage1(*a, 1, 4, 1, 128, 16, 8, 1, 256, nul) == _lib.SOCKET_ERR_ALIGN
    # the fused head of a decode step: bf16, D = 128, K = 10 only; strides in steps of 16 bytes
    def prologue(dtype=1, D=128, K=10, qkv=one, qkv_sb=6144, Hq=32, Hkv=8, R=1024, css=128):
        return lib.socket_decode_prologue(qkv, dtype, qkv_sb, one, 1, 64, one, 0, one, one, one, 8 * 64 * 128, 64 * 128, css, nul,
                                          one, one, one, one, one, one, 1, 1, 1, Hq, Hkv, D, 60, K, R, 64, 0.088, 1.0, nul)
    assert prologue(qkv=nul) == _lib.SOCKET_ERR_NULL
    assert prologue(dtype=0) == _lib.SOCKET_ERR_UNSUPPORTED          # fp32 activations: the three separate entry points
    assert prologue(D=64) == _lib.SOCKET_ERR_UNSUPPORTED
    assert prologue(K=8) == _lib.SOCKET_ERR_UNSUPPORTED
    assert prologue(R=2048) == _lib.SOCKET_ERR_UNSUPPORTED
    assert prologue(Hq=36, Hkv=8) == _lib.SOCKET_ERR_SHAPE            # Hq % Hkv
    assert prologue(Hq=72, Hkv=8) == _lib.SOCKET_ERR_UNSUPPORTED      # nine heads per KV head
    assert prologue(qkv_sb=6148) == _lib.SOCKET_ERR_ALIGN
    assert prologue(css=132) == _lib.SOCKET_ERR_ALIGN
    # workspace too small
    need = lib.socket_sparse_attention_workspace_bytes(1, 4, 128, 300)
    assert need > 0
    r = lib.socket_sparse_attention(one, one, one, 1, 128, 128, 0, 0, 128, 0, 0, 128, one, 300, 300, one, 4, 1, one, 512, 128,
                                    one, need - 1, 1, 4, 1, 128, 16, 300, nul)
    assert r == _lib.SOCKET_ERR_WORKSPACE
    with pytest.raises(_lib.SocketHipError, match="workspace"):
        _lib.check("socket_sparse_attention", r)
    # the variant on the library's own fixed array refuses what does not fit it (checked before any device call)
    assert lib.socket_static_scratch_bytes() == 4 << 20
    big = lib.socket_sparse_attention_workspace_bytes(64, 512, 128, 4096)
    assert big > lib.socket_static_scratch_bytes()
    r = lib.socket_sparse_attention_static(one, one, one, 1, 128, 128, 0, 0, 128, 0, 0, 128, one, 4096, 4096, one, 512, 1,
                                           one, 65536, 128, 64, 512, 8, 128, 16, 4096, nul)
    assert r == _lib.SOCKET_ERR_WORKSPACE


def test_sizes_helpers(lib):
    bs = lib.socket_sparse_attention_block_seq(4, 32, 2308)
    assert bs % 64 == 0 and bs >= 64
    ns = (2308 + bs - 1) // bs
    assert lib.socket_sparse_attention_workspace_bytes(4, 32, 128, 2308) == 4 * 32 * ns * 129 * 4
    assert lib.socket_select_workspace_bytes(4, 32, 4096, 128) == 0        # short rows: one workgroup per row
    assert lib.socket_select_workspace_bytes(1, 32, 131072, 2048) > 0      # few long rows: shared between workgroups
    assert lib.socket_select_workspace_bytes(4, 32, 131072, 2048) == 0     # a row per CU and more: one workgroup each
    assert lib.socket_score_range_parts(4, 32, 8, 131072, 1, 60, 10, 1024) * 8192 >= 131072
    assert lib.socket_score_range_parts_grouped(4, 32, 8, 131072, 1, 60, 10, 1024) == 16
    assert lib.socket_score_range_parts(1, 5, 2, 100, 1, 60, 10, 1024) == 0
    # which table layout a producer should write (bf16 entries, L60 x P10): the grouped
    # one wherever its tiles are at least as cheap as one head per workgroup
    assert lib.socket_score_prefers_grouped(4, 32, 8, 131072, 1, 60, 10, 1024) == 1    # full chip, two rounds
    assert lib.socket_score_prefers_grouped(1, 32, 8, 131072, 1, 60, 10, 1024) == 1    # half the chip, still cheaper
    assert lib.socket_score_prefers_grouped(1, 32, 8, 65536, 1, 60, 10, 1024) == 1     # one round of 2048-token tiles
    assert lib.socket_score_prefers_grouped(1, 32, 8, 32768, 1, 60, 10, 1024) == 1
    assert lib.socket_score_range_parts_grouped(1, 32, 8, 131072, 1, 60, 10, 1024) == 32   # 4096-token tiles fill the chip
    assert lib.socket_score_range_parts_grouped(1, 32, 8, 65536, 1, 60, 10, 1024) == 32    # 2048-token tiles
    assert lib.socket_score_range_parts_grouped(1, 32, 8, 65536, 0, 60, 10, 1024) == 32    # fp32 entries too
    assert lib.socket_score_prefers_grouped(1, 32, 8, 65536, 0, 60, 10, 1024) == 1     # fp32: a head's table exceeds LDS
    assert lib.socket_score_prefers_grouped(1, 5, 2, 100, 1, 60, 10, 1024) == -1


def test_attention_entry_point_by_launch_size(lib):
    """The decode step takes the one-launch attention where there is a row for
    every other CU or more (256 CUs assumed without a device) and the call fits
    the library's fixed scratch array, else the two-launch one."""
    from socket_amd import socket_kernels as sk
    sk.prefers_one_launch.cache_clear()
    assert sk.prefers_one_launch(4, 32, 128, 2308)            # 128 rows
    assert sk.prefers_one_launch(16, 28, 128, 2100)           # 448 rows
    assert not sk.prefers_one_launch(1, 32, 128, 1156)        # 32 rows
    assert not sk.prefers_one_launch(64, 512, 128, 4096)      # beyond the scratch array
    sk.prefers_one_launch.cache_clear()


def _plan(lib, B, Hq, Hkv, T, dt, L, P, grouped):
    from ctypes import byref, c_float, c_int
    tile, direct, one_head, cost = c_int(), c_int(), c_int(), c_float()
    rc = lib.socket_score_plan_query(B, Hq, Hkv, T, dt, L, P, 1 << P, grouped, byref(tile), byref(direct),
                                     byref(one_head), byref(cost))
    return rc, tile.value, direct.value, one_head.value, cost.value


def _shape_cost(lib, B, Hq, Hkv, T, dt, L, P, grouped, tile, direct, one_head):
    from ctypes import byref, c_float, c_int
    slices, waves, cost = c_int(), c_int(), c_float()
    rc = lib.socket_score_shape_cost(B, Hq, Hkv, T, dt, L, P, 1 << P, grouped, tile, direct, one_head, byref(slices),
                                     byref(waves), byref(cost))
    return rc, slices.value, waves.value, cost.value


SCORE_GEOMETRIES = [(32, 8, 60, 10), (28, 4, 48, 10), (32, 8, 32, 8), (16, 8, 60, 10), (16, 16, 60, 10), (32, 8, 16, 12)]


@pytest.mark.parametrize("Hq,Hkv,L,P", SCORE_GEOMETRIES)
@pytest.mark.parametrize("dt", [0, 1])
def test_score_plan_is_the_cheapest_launchable_shape(Hq, Hkv, L, P, dt):
    from socket_amd._lib import lib as load
    lib = load()
    for grouped in (0, 1):
        for B, T in ((1, 8192), (1, 65536), (4, 131072), (16, 57344)):
            rc, tile, direct, one_head, cost = _plan(lib, B, Hq, Hkv, T, dt, L, P, grouped)
            assert rc == 0 and tile in (1024, 2048, 4096, 8192) and cost > 0
            costs = {}
            for t in (8192, 4096, 2048, 1024):
                for d, o in ((1, 0), (0, 0), (1, 1)):
                    rc, slices, waves, c = _shape_cost(lib, B, Hq, Hkv, T, dt, L, P, grouped, t, d, o)
                    if rc == 0:
                        assert slices >= 1 and waves in (4, 8, 16) and c > 0
                        costs[(t, d, o)] = c
            assert (tile, direct, one_head) in costs
            assert cost == min(costs.values()) == costs[(tile, direct, one_head)]
            # one head per workgroup only on the [B,Hq,L,R] layout of a grouped-query model
            assert not (one_head and (grouped or Hq == Hkv))
            # the row ranges the scorer writes are per tile of the planned shape
            parts = (lib.socket_score_range_parts_grouped if grouped else lib.socket_score_range_parts)(
                B, Hq, Hkv, T, dt, L, P, 1 << P)
            assert parts == -(-T // tile)


@pytest.mark.parametrize("Hq,Hkv,L,P", SCORE_GEOMETRIES)
def test_score_plan_cost_never_falls_with_more_work(Hq, Hkv, L, P):
    """More tokens, more sequences, more tables or wider entries never make the
    estimate cheaper: each shape's price is monotone in them, so their minimum is."""
    from socket_amd._lib import lib as load
    lib = load()
    for grouped in (0, 1):
        for dt in (0, 1):
            prev = 0.0
            for T in (1000, 4096, 8192, 20000, 32768, 65536, 100000, 131072, 262144, 1 << 20):
                cost = _plan(lib, 2, Hq, Hkv, T, dt, L, P, grouped)[4]
                assert cost >= prev, (grouped, dt, T)
                prev = cost
            prev = 0.0
            for B in (1, 2, 3, 4, 8, 16, 64):
                cost = _plan(lib, B, Hq, Hkv, 65536, dt, L, P, grouped)[4]
                assert cost >= prev, (grouped, dt, B)
                prev = cost
            prev = 0.0
            for tables in (L // 4, L // 2, L, 2 * L):
                cost = _plan(lib, 4, Hq, Hkv, 65536, dt, tables, P, grouped)[4]
                assert cost >= prev, (grouped, dt, tables)
                prev = cost
        # fp32 entries are never priced below bf16 entries of the same table
        assert _plan(lib, 4, Hq, Hkv, 131072, 0, L, P, grouped)[4] >= _plan(lib, 4, Hq, Hkv, 131072, 1, L, P, grouped)[4]


def test_score_plan_on_the_benchmark_shapes():
    from socket_amd._lib import lib as load
    lib = load()
    # B4 x 128k, L60 x P10, bf16 grouped table: two rounds of 8192-token tiles, slices copied straight into LDS
    rc, tile, direct, one_head, cost = _plan(lib, 4, 32, 8, 131072, 1, 60, 10, 1)
    assert (rc, tile, direct, one_head) == (0, 8192, 1, 0) and 60 < cost < 140
    # batch 1 at 32k: a quarter of the tile so that the chip is filled
    assert _plan(lib, 1, 32, 8, 32768, 1, 60, 10, 1)[1:4] == (2048, 1, 0)
    # short context on the [B,Hq,L,R] layout: one head per workgroup, table resident
    assert _plan(lib, 1, 32, 8, 8192, 1, 60, 10, 0)[3] == 1
    # fp32 entries: a head's table (60 x 1024 x 4 B) no longer fits LDS, so never one head per workgroup
    assert _plan(lib, 1, 32, 8, 8192, 0, 60, 10, 0)[3] == 0
    # the layout a producer is told to write is the cheaper one, with a margin in favour of the grouped one
    for B, Hq, Hkv, T, dt, L, P in ((1, 32, 8, 8192, 1, 60, 10), (4, 32, 8, 131072, 1, 60, 10), (16, 28, 4, 57344, 1, 48, 10),
                                    (1, 32, 8, 65536, 0, 60, 10), (2, 16, 8, 30000, 1, 32, 8)):
        grp, ref = _plan(lib, B, Hq, Hkv, T, dt, L, P, 1)[4], _plan(lib, B, Hq, Hkv, T, dt, L, P, 0)[4]
        assert lib.socket_score_prefers_grouped(B, Hq, Hkv, T, dt, L, P, 1 << P) == int(grp <= 1.3 * ref)
    # bad shapes are refused, not priced
    assert _plan(lib, 1, 5, 2, 100, 1, 60, 10, 1)[0] != 0
    assert _shape_cost(lib, 1, 32, 8, 8192, 1, 60, 10, 1, 3000, 1, 0)[0] != 0       # not a tile the kernels have
    assert _shape_cost(lib, 1, 32, 8, 8192, 1, 60, 10, 1, 2048, 1, 1)[0] != 0       # one head per workgroup on a grouped table


def test_step_cost_estimate_places_the_crossover():
    """The estimate behind ModelArgs.dense_below_crossover: sparse is priced below dense
    at 4 x 131072 and at 1 x 131072 tokens, above it at 1 x 32768 (as measured on the
    device), and neither price falls as the context grows."""
    from socket_amd import hash_cache as hc
    geo = dict(Hq=32, Hkv=8, D=128, L=60, P=10, R=1024, sink=4, window=256)
    at = lambda B, T, M: hc.step_cost_estimate(B, geo["Hq"], geo["Hkv"], geo["D"], T, geo["L"], geo["P"], geo["R"],
                                               M, geo["sink"], geo["window"])
    s, d = at(4, 131072, 2048)
    assert s < d and 1.6 < d / s < 3.0
    s, d = at(1, 131072, 2048)
    assert s < d
    s, d = at(1, 32768, 1024)
    assert d < s
    prev = (0.0, 0.0)
    for T in (8192, 16384, 32768, 65536, 131072, 262144):
        cur = at(1, T, 1024)
        assert cur[1] >= prev[1] and cur[0] > 0
        prev = cur


def test_python_api_keeps_reference_signatures():
    from socket_amd import socket_kernels, sparse
    from socket_amd.soft_hash_collision_loader import load_soft_hash_collision

    def params(f):
        return list(inspect.signature(f).parameters)

    # kernels/socket_triton_kernels.py:167-258
    assert params(socket_kernels.sparse_attention_fwd) == ["query", "key", "value", "sparse_list", "sparse_len", "block_seq"]
    assert inspect.signature(socket_kernels.sparse_attention_fwd).parameters["block_seq"].default == 256
    assert params(socket_kernels.sparse_decode_stage1) == ["q", "k", "v", "sparse_list", "sparse_len", "max_len_in_batch",
                                                           "mid_out", "mid_out_logsumexp", "block_seq"]
    assert params(socket_kernels.sparse_decode_stage2) == ["mid_out", "mid_out_logsumexp", "sparse_len", "out", "block_seq"]
    assert params(socket_kernels.attention_mask_to_allowed_prob) == ["attention_mask", "K"]
    # GPT-FAST/kernels/sparse.py:16-28
    sig = inspect.signature(sparse.build_sparse_list_decode)
    assert list(sig.parameters) == ["q_probs", "k_hard_bhlt", "v_norm_bht", "allowed_bht", "sink", "window", "M",
                                    "KC", "BLOCK_N", "num_warps", "num_stages"]
    assert [sig.parameters[k].default for k in ("KC", "BLOCK_N", "num_warps", "num_stages")] == [8, 512, 8, 2]
    assert inspect.signature(load_soft_hash_collision).parameters["version"].default == 3


def test_attention_mask_to_allowed_prob():
    from socket_amd.socket_kernels import attention_mask_to_allowed_prob as f

    m = torch.tensor([[[False, True, False, True]]])                # bool: True = forbidden
    out = f(m, 3)
    assert out.shape == (1, 1, 1, 3) and out.dtype == torch.float32 and out.flatten().tolist() == [1.0, 0.0, 1.0]
    add = torch.tensor([[[[0.0, -1e9, 0.0, 0.0]]]])                  # additive: < 0 = forbidden
    assert f(add, 4).flatten().tolist() == [1.0, 0.0, 1.0, 1.0]


def test_asserts_fire_on_cpu_tensors():
    from socket_amd import socket_kernels, sparse

    q = torch.zeros(1, 4, 128)
    kv = torch.zeros(1, 1, 8, 128)
    sl = torch.zeros(1, 4, 3, dtype=torch.int32)
    ln = torch.zeros(1, 4, dtype=torch.int32)
    with pytest.raises(AssertionError):
        socket_kernels.sparse_attention_fwd(q, kv, kv, sl, ln)
    with pytest.raises(AssertionError):
        sparse.build_sparse_list_decode(torch.zeros(1, 4, 2, 16), torch.zeros(1, 4, 2, 8, dtype=torch.int16),
                                        torch.zeros(1, 4, 8), torch.ones(1, 4, 8, dtype=torch.bool), 1, 1, 2)


def test_workloads_are_deterministic_and_shaped():
    from socket_amd.workloads import WORKLOADS, make_inputs, scaled

    w = scaled(WORKLOADS["c1"], T=256)
    a, b = make_inputs(w), make_inputs(w)
    assert torch.equal(a.k, b.k) and torch.equal(a.q_probs, b.q_probs) and torch.equal(a.planes, b.planes)
    assert a.q.shape == (1, 32, 128) and a.k.shape == (1, 8, 256, 128) and a.q_probs.shape == (1, 32, 32, 256)
    assert torch.allclose(a.q_probs.sum(-1), torch.ones(1, 32, 32), atol=1e-5)
    c = make_inputs(w, layer=1)
    assert not torch.equal(a.k, c.k)
    r = make_inputs(scaled(WORKLOADS["c5"], T=2048, t_min=512, B=3))
    assert r.lens.dtype == torch.int32 and int(r.lens.max()) == 2048 and int(r.lens.min()) >= 512
    assert torch.equal(r.budgets, (r.lens.double() * 0.02).floor().int())
    # planted keys point along the group's mean query direction: they outscore a typical key
    w2 = scaled(WORKLOADS["c1"], T=1024)
    i2 = make_inputs(w2)
    qdir = i2.q.view(1, 8, 4, 128).mean(2)
    proj = torch.einsum("bhtd,bhd->bht", i2.k, qdir / qdir.norm(dim=-1, keepdim=True))
    top16 = proj.topk(16, dim=-1).values.min()
    assert top16 > 2.0 and proj.median() < 1.0
