"""The benchmark configurations at their full size on the MI355X: hash ->
append -> score -> select -> attend through the C ABI, checked against the CPU
oracle where the oracle finishes in seconds (one (sequence, kv head) of scores at
full context, the attention of every row on the gathered K/V rows) and against
the definitions evaluated on the device for the rest (stable descending sort for
every row's top-k; float64 projections for sampled hash rows).

  c2  B1  32/8 heads, T 32768, L60 x P10, top-k 1024 + 4 + 128
  c3  B4  32/8 heads, T 131072, L60 x P10, top-k 2048 + 4 + 256, one key appended per step
  c5  B16 28/4 heads (G = 7), ragged T_b in [16384, 98304], L48 x P10, top-k 2% of T_b + 4 + 128
  c4  Llama-3.1-8B geometry (two of its 32 layers), 65536-token prompt, sparse decode
"""
import numpy as np
import pytest
import torch

from oracle import socket_oracle as orc
from socket_amd import generate as gen
from socket_amd import hash_cache
from socket_amd import model as M
from socket_amd.workloads import WORKLOADS, make_inputs
from tests import oracle_backend

pytestmark = pytest.mark.gpu


def _attend_oracle_on_gathered_rows(q, k, v, sl, ln, G):
    """orc.sparse_attend_textbook for every row, fed with the listed K/V rows only
    (gathered on the device, so the full cache never travels to the host)."""
    B, Hq, Kt = sl.shape
    rows = sl.clamp(min=0).long()
    kvh = (torch.arange(Hq, device=sl.device) // G)[:, None]
    kk = torch.stack([k[b][kvh, rows[b]] for b in range(B)]).cpu()                               # [B,Hq,Kt,D]
    vv = torch.stack([v[b][kvh, rows[b]] for b in range(B)]).cpu()
    compact = torch.arange(Kt, dtype=torch.int32).expand(B, Hq, Kt).clone()
    compact[sl.cpu() < 0] = -1
    return orc.sparse_attend_textbook(q.cpu(), kk, vv, compact, ln.cpu())


@pytest.mark.parametrize("name", ["c2", "c3", "c5"])
def test_full_size_decode_step(dev, name):
    w = WORKLOADS[name]
    B, Hq, Hkv, D, T, L, P, G = w.B, w.Hq, w.Hkv, w.D, w.T, w.L, w.P, w.G
    print(f"config {name}: B{B} Hq{Hq}/Hkv{Hkv} T{T} L{L} P{P} M{w.M}", flush=True)
    inp = make_inputs(w, device=dev, device_rng=True)
    lens, budgets = inp.lens, inp.budgets
    lens_cpu = [T] * B if lens is None else lens.cpu().tolist()
    m_cpu = [w.M] * B if budgets is None else budgets.cpu().tolist()
    NW = hash_cache.words_per_key(L, P)
    Tcap = (T + 7) // 8 * 8
    codes = torch.zeros((B, Hkv, NW, Tcap), dtype=torch.int32, device=dev)
    v_norm = torch.zeros((B, Hkv, Tcap), dtype=torch.float16, device=dev)
    planes_words = hash_cache.permute_planes(inp.planes)

    # ---- prefill hash of the whole cache, then the newest key of every sequence once
    # more through the append path (device-side positions): same words, same norms
    hash_cache.hash_keys_into(inp.k, inp.v, planes_words, codes, v_norm, L, P, t0=0, layout="bhsd")
    last = torch.tensor([n - 1 for n in lens_cpu], dtype=torch.int32, device=dev)
    bi = torch.arange(B, device=dev)
    want_words = codes[bi, :, :, last.long()].clone()                      # [B,Hkv,NW]
    want_norm = v_norm[bi, :, last.long()].clone()
    codes[bi, :, :, last.long()] = 0
    v_norm[bi, :, last.long()] = 0
    k_last = inp.k[bi, :, last.long()].unsqueeze(1).contiguous()           # [B,1,Hkv,D]
    v_last = inp.v[bi, :, last.long()].unsqueeze(1).contiguous()
    hash_cache.hash_keys_into(k_last, v_last, planes_words, codes, v_norm, L, P, pos_b=last, layout="bshd")
    assert torch.equal(codes[bi, :, :, last.long()], want_words)
    assert torch.equal(v_norm[bi, :, last.long()], want_norm)

    # ---- hash bits of sampled rows against float64 projections, where the sign is decided
    g = torch.Generator(device=dev).manual_seed(5)
    ns = 4096
    sb = torch.randint(0, B, (ns,), generator=g, device=dev)
    sh = torch.randint(0, Hkv, (ns,), generator=g, device=dev)
    st = (torch.rand(ns, generator=g, device=dev) * torch.tensor(lens_cpu, device=dev)[sb]).long()
    keys = inp.k[sb, sh, st].double()                                                        # [ns,D]
    proj = keys @ inp.planes.to(torch.bfloat16).double().view(L * P, D).T                    # [ns,L*P]
    proj = proj.view(ns, L, P)
    wantc = orc.pack_bits((proj >= 0).cpu()).to(dev)                                          # [ns,L]
    words = codes[sb, sh, :, st].cpu().numpy().view(np.uint32)                                # [ns,NW]
    have = torch.from_numpy(orc.unpack_code_words(words.T.copy()[None], L, P)[0].T.copy()).to(dev)   # [ns,L]
    clear = (proj.abs() > 1e-3 * proj.abs().mean()).all(-1)
    assert clear.float().mean() > 0.9
    assert torch.equal(have[clear].to(torch.int16), wantc[clear].to(torch.int16))
    vn_want = inp.v[sb, sh, st].float().norm(dim=-1)
    torch.testing.assert_close(v_norm[sb, sh, st].float(), vn_want, rtol=2e-3, atol=1e-3)

    # ---- the step, on the table the model produces: bf16, in the layout the scorer asks for
    q_table = inp.q_probs.to(torch.bfloat16)
    if hash_cache._prefers_grouped(B, Hq, Hkv, T, 1, L, P, q_table.shape[-1]):
        table = hash_cache.group_q_probs(q_table, Hkv)
    else:
        table = q_table
    out, scores, sl, ln = hash_cache.sparse_decode_step(
        inp.q, table, inp.k, inp.v, codes, v_norm, T, P, w.sink, w.window, w.M, lens=lens, budgets=budgets,
        return_details=True)
    torch.cuda.synchronize()

    # scores: the longest sequence's first kv head at full context against the oracle
    # (bf16 table: 2e-6 relative; the same table widened to fp32: identical)
    n0 = lens_cpu[0]
    c16 = hash_cache.unpack_codes(codes[:1, :1].contiguous(), L, P, 0, n0).cpu()              # [1,1,L,n0]
    vn0 = v_norm[:1, :1, :n0].cpu().float()
    allowed = torch.ones(1, G, n0, dtype=torch.bool)
    want_s = orc.collision_score(q_table[:1, :G].float().cpu(), c16.repeat_interleave(G, 1), allowed,
                                 vn0.repeat_interleave(G, 1))
    got_s = scores[:1, :G, :n0].cpu()
    rel = ((got_s - want_s).abs() / want_s.abs().clamp_min(1e-30)).max()
    assert rel <= 2e-6, f"scores: max rel diff {rel}"
    s32 = hash_cache.score_packed(q_table.float(), codes, v_norm, T, P, lens=lens)
    assert torch.equal(s32[:1, :G, :n0].cpu(), want_s)
    if lens is not None:                                                                    # masked beyond each length
        for b in range(B):
            assert torch.isinf(scores[b, :, lens_cpu[b]:]).all() and torch.isfinite(scores[b, :, :lens_cpu[b]]).all()

    # every row's list: [sink | window | heavy | -1 ...], heavy = stable descending sort of the row
    for b in range(B):
        n, m = lens_cpu[b], min(m_cpu[b], lens_cpu[b])
        base = torch.from_numpy(orc.base_indices(n, w.sink, w.window)).to(dev)
        nbase = base.numel()
        order = torch.sort(scores[b, :, :n], dim=-1, descending=True, stable=True).indices[:, :m]
        assert torch.equal(sl[b, :, :nbase], base.to(torch.int32).expand(Hq, -1)), f"sequence {b}: sink / window part"
        assert torch.equal(sl[b, :, nbase:nbase + m].long(), order), f"sequence {b}: heavy part"
        assert (sl[b, :, nbase + m:] == -1).all() and (ln[b] == nbase + m).all()
    # the oracle's selection rule on the checked rows' scores
    m0 = min(m_cpu[0], n0)
    nb0 = orc.base_indices(n0, w.sink, w.window).size
    assert torch.equal(sl[0, :G, nb0:nb0 + m0].cpu().long(), orc.topk_lower_index_first(got_s, m0)[0])

    # attention of every row against the float64 textbook on the listed rows
    want_o = _attend_oracle_on_gathered_rows(inp.q, inp.k, inp.v, sl, ln, G)
    err = (out.cpu().double() - want_o).abs().max().item()
    assert err <= 2e-2, f"attention: max abs err {err}"
    assert out.dtype == w.dtype and torch.isfinite(out.float()).all()


def test_c4_model_decode_at_65536_tokens(dev, monkeypatch):
    """Two layers of the Llama-3.1-8B geometry, a 65536-token random prompt, a few
    sparse decode steps; the last step once more with the attention hook routed
    through the CPU oracle on the same caches; graph replays equal the eager step."""
    cfg = M.ModelArgs.from_name("Llama-3.1-8B")
    cfg.n_layer = 2
    cfg.block_size = 65536 + 64
    model = gen.load_random_model(cfg, dev, torch.bfloat16, seed=4000)
    g = torch.Generator().manual_seed(4000)
    T0, steps = 65536, 4
    prompt = torch.randint(0, cfg.vocab_size, (1, T0), generator=g).to(dev)
    print("c4: prefill", flush=True)
    seq, st = gen.generate(model, prompt, steps + 1, decode_type="sparse", use_graph=True, check_graph=True)
    assert st["graph"] and st["graph_check"]["same_token"] and st["graph_check"]["max_abs_logit_diff"] <= 1e-2
    cache = model.layers[0].attention.kv_cache
    assert int(cache.lens[0]) == T0 + steps
    # the last decoded position again, eagerly: through the kernels, then through the oracle
    tok = seq[:, T0 + steps - 1:T0 + steps].to(torch.int)
    pos = torch.tensor([T0 + steps - 1], device=dev)
    print("c4: last step on the device", flush=True)
    have = model.sparse_forward(tok, pos)[:, -1].float().cpu()
    oracle_backend.install(monkeypatch, M, hashing=False, sparse=True, dense=False)
    print("c4: last step through the oracle", flush=True)
    want = model.sparse_forward(tok, pos)[:, -1].float().cpu()
    assert torch.isfinite(have).all()
    scale = max(float(want.abs().max()), 1.0)
    assert float((have - want).abs().max()) <= 6e-2 * scale
    assert int(have.argmax(-1)) == int(seq[0, T0 + steps])          # what the graph-driven run produced
