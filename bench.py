#!/usr/bin/env python3
"""Benchmark of the sparse-decode hot path on one MI355X.

A step is one decode step of one attention layer on synthetic inputs of the
configured shape, resident in HBM before timing starts: hash the newly appended
key of every (sequence, kv head), score every cached key, select the top-k +
sink + window list, and attend over the listed rows.  The default workload is
configuration 3 (batch 4, 32/8 heads, head dim 128, 131072-token bf16 cache,
L=60 x P=10, top-k 2048 + 4 sink + 256 window).

Prints one JSON line.  `value` is microseconds per layer per step of the sparse
path on configuration 3: exactly --steps steps after --warmup, recorded back to
back into one HIP graph as the layers of a decode step are in the model's graph
(`power_state.steps_per_graph`; the figure with one graph launch per step is
beside it as `us_per_step_one_graph_launch_each`), taken in the sustained power
state of a decode loop (a settle phase of untimed replays comes first; the
figure of a burst that starts on an idle GPU is reported as
`power_state.us_per_step_from_idle`); `roofline`
prices the scorer (the kernel moving the most bytes) against HBM peak; `kernels`
does the same for every kernel of the step and for the dense flash-decode
comparator on the same GPU (each timed as a HIP-graph replay of ten launches, so
small kernels are not priced at the cost of an eager Python call); `c2` and `c5`
are the same records for configurations 2 and 5; `drop_in_operator` times
`build_sparse_list_decode` on the reference's own operand layout; `decode_tok_s` is the end-to-end
greedy decode of the 32-layer Llama-3.1-8B-shaped model, sparse and dense, at
128k context and at configuration 4's 65536-token prompt; `cpu_baseline` is the
CPU oracle timed on the host's cores on a slice of configuration 3.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3|c4|c5] [--no-extra]
                  [--only score|score_grouped|select|attend|hash|dense|step|decode|...] [--no-cpu] [--no-parity]
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published

# HBM bytes per launch of the scorer from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# `bench.py --workload W --only score_grouped` (profiles/score_flat_c3_hbm_counters.txt and
# profiles/score_flat_c5_hbm_counters.txt hold the commands, the raw counters and the
# calibration), keyed by workload; None until a counter run for that workload has been
# recorded there.  The profiler cannot run inside this process, so the figure is a
# recorded one and says so.
MEASURED_TRAFFIC_BYTES = {"c3": int(175940.4 * 1024 * 2.000 + 65569.8 * 1024 * 1.000),
                          "c5": int(150077.5 * 1024 * 2.000 + 94275.5 * 1024 * 1.000)}
MEASURED_TRAFFIC_SOURCE = ("recorded, not measured in this run: rocprofv3 --pmc FETCH_SIZE (x2.000, calibrated on a 1 GiB "
                           "read stream of the same request width) + WRITE_SIZE (x1.000, device copy) of "
                           "score_flat_kernel; profiles/score_flat_{w}_hbm_counters.txt")


def algorithmic_bytes(w, lens=None, budgets=None):
    """Per-launch algorithmic bytes of each kernel on the packed format."""
    cpw = 32 // w.P
    wc = 4 * ((w.L + cpw - 1) // cpw)
    G = w.Hq // w.Hkv
    if lens is None:
        tok = w.B * w.T
        sel = w.B * w.Hq * (4 * w.T + 4 * w.M)
        kt = w.B * (w.sink + w.window + w.M)
    else:
        tok = int(lens.sum())
        sel = int((w.Hq * (4 * lens.long() + 4 * budgets.long())).sum())
        kt = int((w.sink + w.window + budgets.long()).sum())
    return {
        "hash": w.B * w.Hkv * w.new_keys * (2 * 2 * w.D + wc + 2),
        "score": w.Hkv * tok * (wc + 2 + 4 * G),
        "score_f32": w.Hkv * tok * (wc + 2 + 4 * G),
        "score_f32_table": w.Hkv * tok * (wc + 2 + 4 * G),
        "score_f32_table_grouped": w.Hkv * tok * (wc + 2 + 4 * G),
        "score_reference_layout": w.Hkv * tok * (wc + 2 + 4 * G),
        "select": sel,
        "attend": w.Hq * kt * (4 * w.D + 4) + w.B * w.Hq * 4 * w.D,
        "dense": w.Hkv * tok * 4 * w.D,
    }


SETTLE_MS = 60.0


def settle(run, ms=None):
    """Keeps the GPU busy with `run` for about `ms` milliseconds, untimed, and returns
    how many times it ran.  A burst that starts on an idle GPU runs in a transient
    power state: the scorer of the 128k workload takes 95-114 us per launch in the
    first milliseconds after an idle gap and 88-89 us once the card has been busy
    for some tens of milliseconds, which is the state of a decode loop (32 layers
    back to back, token after token).  Timed regions therefore follow a settle
    phase; the figure without one is reported beside the step's."""
    ms = SETTLE_MS if ms is None else ms
    if ms <= 0:
        return 0
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    run()
    e1.record()
    e1.synchronize()
    n = int(min(20000, max(1, ms / max(e0.elapsed_time(e1), 1e-3))))
    for _ in range(n):
        run()
    return n + 1


def time_graph(fn, iters, warmup=2, per_graph=10):
    """Average device time in microseconds of one call of `fn`: `per_graph` calls are
    recorded into one HIP graph and the graph is replayed between two HIP events, so
    the figure is kernel time plus the in-graph launch gap, without the Python and
    ctypes cost of an eager call (which is several microseconds, more than some of
    these kernels take).  The timed replays (at least 100 calls) follow a settle
    phase.  Falls back to eager launches if capture fails."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(warmup, 2)):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(per_graph):
                fn()
        g.replay()
        torch.cuda.synchronize()
        reps = max(1, (max(iters, 100) + per_graph - 1) // per_graph)
        settle(g.replay)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) * 1000.0 / (reps * per_graph)
    except Exception as e:  # noqa: BLE001
        print(f"bench: graph timing unavailable ({e}); timing eager launches", file=sys.stderr)
        return time_launches(fn, iters, warmup)


def time_launches(fn, iters, warmup=3):
    """Average duration in microseconds of `fn` (which enqueues on torch's current
    stream) measured with HIP events recorded on that same stream."""
    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) * 1000.0 / iters


def block_sparse_bench(dev, iters, warmup):
    """Block-sparse prefill attention (kernels/block_sparse_flash_attention.py) at the
    C4 prompt: B1, 32 heads, T 65536, D128, bf16, 8 key blocks of 64 per 64-row block
    (window of 4 + best-scoring others, from random block scores)."""
    from socket_amd import block_sparse_flash_attention as bsa
    B, H, T, D, K = 1, 32, 65536, 128, 8
    g = torch.Generator(device=dev).manual_seed(4000)
    q, k, v = (torch.randn(B, H, T, D, generator=g, device=dev, dtype=torch.bfloat16) for _ in range(3))
    R = T // 64
    blocks = bsa.random_walk_indices_from_block_probs(torch.rand(B, R, R, generator=g, device=dev), K, window_blocks=4)
    blocks = bsa.expand_block_index_to_heads(blocks, H)
    seqlens = torch.full((B,), T, dtype=torch.int32, device=dev)
    us = time_launches(lambda: bsa.random_walk_sparse_attention(q, k, v, seqlens, blocks), iters, warmup=warmup)
    flops = 2.0 * 2 * 64 * 64 * D * K * R * B * H              # both products over every listed block
    tile_bytes = (2 * K * 64 * D * 2 + 2 * 64 * D * 2) * R * B * H   # K/V tiles fetched + q read + out written
    print(json.dumps({"only": "block_sparse", "shape": f"B{B} H{H} T{T} D{D} bf16, {K} key blocks per row block",
                      "us": round(us, 1), "mfma_tflops": round(flops / us / 1e6, 1),
                      "mfma_frac": round(flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                      "tile_traffic_gbs": round(tile_bytes / us / 1e3, 1),
                      "unique_MB": round(4 * B * H * T * D * 2 / 1e6, 1)}))


def copy_ceiling_gbs(dev):
    """Measured device-to-device copy rate (read + write bytes) of a 1 GiB buffer."""
    n = 1 << 28
    a = torch.empty(n, dtype=torch.float32, device=dev).normal_()
    b = torch.empty_like(a)
    us = time_launches(lambda: b.copy_(a), 10)
    del a, b
    return 2 * n * 4 / us / 1e3


def read_ceiling_gbs(dev):
    """Measured rate of a pure read stream: the matrix-vector kernel over a 1 GiB
    bf16 matrix (non-temporal 16-byte loads, 8 KB per output feature, 262 KB written)."""
    from socket_amd import decode_ops
    n_out, k = 131072, 4096
    w_ = torch.empty(n_out, k, dtype=torch.bfloat16, device=dev).normal_(0, 0.02)
    x = torch.empty(1, 1, k, dtype=torch.bfloat16, device=dev).normal_()
    us = time_launches(lambda: decode_ops.linear_rows(x, w_), 10)
    del w_, x
    return n_out * k * 2 / us / 1e3


def cpu_baseline(w, inp_cpu, codes_cpu, vnorm_cpu, seconds_budget=20.0):
    """The CPU oracle on a slice of the workload: sequence 0, the first two kv
    heads (2*G query heads), full context; scaled to the whole layer."""
    from oracle import socket_oracle as orc

    # every core this job may use: the cores the process is allowed on, capped by the
    # thread budget the environment sets for it (OMP_NUM_THREADS; a shared host reports all
    # its cores to every job); the threads actually used and the host's count are both recorded
    host_cores = os.cpu_count() or 1
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else host_cores
    try:
        cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    except ValueError:
        pass
    torch.set_num_threads(cores)
    cores = torch.get_num_threads()
    G = w.Hq // w.Hkv
    nkv = min(2, w.Hkv)
    T = int(inp_cpu["len0"])
    M = int(inp_cpu["m0"])
    q = inp_cpu["q"][:1, :nkv * G]
    qp = inp_cpu["q_probs"][:1, :nkv * G].float().contiguous()
    k = inp_cpu["k"][:1, :nkv, :T]
    v = inp_cpu["v"][:1, :nkv, :T]
    codes = codes_cpu[:1, :nkv, :, :T].repeat_interleave(G, 1)
    vn = vnorm_cpu[:1, :nkv, :T].repeat_interleave(G, 1)
    allowed = torch.ones(1, nkv * G, T, dtype=torch.bool)

    def once():
        t0 = time.perf_counter()
        scores = orc.collision_score(qp, codes, allowed, vn.float())
        t1 = time.perf_counter()
        heavy = orc.topk_lower_index_first(scores, M).to(torch.int32)
        base = torch.from_numpy(orc.base_indices(T, w.sink, w.window)).view(1, 1, -1).expand(1, nkv * G, -1)
        sl = torch.cat([base, heavy], -1).contiguous()
        ln = torch.full((1, nkv * G), sl.shape[-1], dtype=torch.int32)
        t2 = time.perf_counter()
        orc.sparse_attend_textbook(q, k, v, sl, ln)
        t3 = time.perf_counter()
        return t1 - t0, t2 - t1, t3 - t2

    once()
    reps = []
    t_start = time.perf_counter()
    while len(reps) < 5 or (time.perf_counter() - t_start < seconds_budget and len(reps) < 15):
        reps.append(once())
    med = [statistics.median(r[i] for r in reps) for i in range(3)]
    # keys scored by the whole layer / keys scored by the sample
    scale = (w.Hkv * float(inp_cpu["tok_total"])) / (nkv * T)
    total_us = sum(med) * 1e6 * scale
    return {
        "value": round(total_us, 1),
        "unit": "us/layer/step",
        "cores": cores,
        "host_cpu_count": host_cores,
        "kind": "port",
        "sample": f"sequence 0, {nkv} of {w.Hkv} kv heads ({nkv * G} query heads), context {T}, "
                  f"median of {len(reps)} reps, scaled x{scale:.2f} to the whole layer",
        "stage_us_scaled": {"score": round(med[0] * 1e6 * scale, 1), "select": round(med[1] * 1e6 * scale, 1),
                            "attend": round(med[2] * 1e6 * scale, 1)},
        "cpu_model": _cpu_model(),
    }


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


class Step:
    """One workload's tensors on the device and the closures that run each kernel of the
    step on them (the same calls the attention hook makes)."""

    def __init__(self, w, dev, reference_table_layout=False):
        from socket_amd import hash_cache, socket_kernels, sparse
        from socket_amd.workloads import make_inputs
        self.w, self.dev = w, dev
        self.hc, self.sk, self.sp = hash_cache, socket_kernels, sparse
        t0 = time.perf_counter()
        self.inp = inp = make_inputs(w, device=dev, device_rng=True)
        torch.cuda.synchronize()
        self.input_generation_s = time.perf_counter() - t0
        B, Hq, Hkv, T = w.B, w.Hq, w.Hkv, w.T
        self.NW = hash_cache.words_per_key(w.L, w.P)
        Tcap = (T + 7) // 8 * 8
        self.codes = torch.zeros((B, Hkv, self.NW, Tcap), dtype=torch.int32, device=dev)
        self.v_norm = torch.zeros((B, Hkv, Tcap), dtype=torch.float16, device=dev)
        self.planes_words = hash_cache.permute_planes(inp.planes)
        self.lens, self.budgets = inp.lens, inp.budgets
        self.abytes = algorithmic_bytes(w, None if self.lens is None else self.lens.cpu(),
                                        None if self.budgets is None else self.budgets.cpu())
        pitch = (T + 3) // 4 * 4
        self.scores_buf = torch.full((B, Hq, pitch), float("-inf"), dtype=torch.float32, device=dev)
        self.new_pos = None if self.lens is None else (self.lens - w.new_keys).to(torch.int32)
        # the soft-hash table in the dtype the model produces it in: the reference's
        # soft_hash runs in the model dtype (GPT-FAST/model.py:392-401), bf16 here
        self.q_table = inp.q_probs.to(torch.bfloat16) if w.dtype == torch.bfloat16 else inp.q_probs
        self.q_table_f32 = self.q_table.float()
        self.q_table_f32_grouped = None
        # ... and in the layout the fused soft-hash kernel writes it in (heads of a KV head
        # interleaved per bucket: the scorer's LDS image); same values
        self.q_table_grouped = hash_cache.group_q_probs(self.q_table, Hkv)
        # the step uses the layout the library asks its producers for at this shape
        self.use_grouped = (not reference_table_layout and
                            hash_cache._prefers_grouped(B, Hq, Hkv, T, 1 if self.q_table.dtype == torch.bfloat16 else 0,
                                                        w.L, w.P, self.q_table.shape[-1]))
        self.dense_lens = self.lens if self.lens is not None else torch.full((B,), T, dtype=torch.int32, device=dev)

    # ---- K1 at scale: hash of the whole cache
    def prefill_hash(self):
        w = self.w
        self.hc.hash_keys_into(self.inp.k, self.inp.v, self.planes_words, self.codes, self.v_norm, w.L, w.P, t0=0,
                               layout="bhsd")

    # ---- the kernels of one step
    def k_hash(self):
        # the newly appended key(s) of every (sequence, kv head) land on the last
        # position(s), so the context length is the same every step
        w = self.w
        self.hc.hash_keys_into(self.inp.k_new, self.inp.v_new, self.planes_words, self.codes, self.v_norm, w.L, w.P,
                               t0=w.T - w.new_keys, pos_b=self.new_pos, layout="bshd")

    def k_score_ref(self):
        return self.hc.score_packed(self.q_table, self.codes, self.v_norm, self.w.T, self.w.P, lens=self.lens,
                                    out=self.scores_buf)

    def k_score_grouped(self):
        # (as the step calls it: positions past a sequence's length are not written)
        return self.hc.score_packed(self.q_table_grouped, self.codes, self.v_norm, self.w.T, self.w.P, lens=self.lens,
                                    out=self.scores_buf, n_heads=self.w.Hq, skip_masked=True)

    def k_score_f32_grouped(self):
        if self.q_table_f32_grouped is None:
            self.q_table_f32_grouped = self.hc.group_q_probs(self.q_table_f32, self.w.Hkv)
        return self.hc.score_packed(self.q_table_f32_grouped, self.codes, self.v_norm, self.w.T, self.w.P,
                                    lens=self.lens, out=self.scores_buf, n_heads=self.w.Hq, skip_masked=True)

    def k_score_f32(self):
        return self.hc.score_packed(self.q_table_f32, self.codes, self.v_norm, self.w.T, self.w.P, lens=self.lens,
                                    out=self.scores_buf)

    def k_score(self):
        return self.k_score_grouped() if self.use_grouped else self.k_score_ref()

    def k_select(self, scores):
        w = self.w
        return self.sp.select_list(scores, w.sink, w.window, w.M, lens=self.lens, budgets=self.budgets)

    def k_attend(self, sl, ln):
        return self.sk.sparse_attention_fwd(self.inp.q, self.inp.k, self.inp.v, sl, ln)

    def k_dense(self):
        return self.sk.dense_decode_fwd(self.inp.q, self.inp.k, self.inp.v, self.dense_lens)

    def step(self):
        """hash-append + score + select + attend, as `hash_cache.sparse_decode_step` after the append."""
        w = self.w
        self.k_hash()
        return self.hc.sparse_decode_step(self.inp.q, self.q_table_grouped if self.use_grouped else self.q_table,
                                          self.inp.k, self.inp.v, self.codes, self.v_norm, w.T, w.P, w.sink, w.window,
                                          w.M, lens=self.lens, budgets=self.budgets)

    # ---- parity gates on the full-size tensors (device-side checks, not timed)
    def parity(self, scores, sl, ln, out):
        w, inp, dev = self.w, self.inp, self.dev
        T, D, Hq, Hkv = w.T, w.D, w.Hq, w.Hkv
        res = {}
        s0 = scores[0, :8]
        n0 = T if self.lens is None else int(self.lens[0])
        m0 = w.M if self.budgets is None else int(self.budgets[0])
        order = torch.sort(s0[:, :n0], dim=-1, descending=True, stable=True).indices[:, :m0].to(torch.int32)
        nbase = int(ln[0, 0]) - m0
        res["topk_exact_rows_checked"] = 8
        res["topk_exact"] = bool(torch.equal(sl[0, :8, nbase:nbase + m0], order))
        # attention vs an fp32 gather-softmax over the same list, one sequence
        idx = sl[0, :, :int(ln[0, 0])].long()
        kvh = (torch.arange(Hq, device=dev) // (Hq // Hkv))[:, None]
        kk = inp.k[0][kvh, idx].float()
        vv = inp.v[0][kvh, idx].float()
        att = torch.softmax((kk @ inp.q[0].float().unsqueeze(-1)).squeeze(-1) / D ** 0.5, -1)
        ref = (att.unsqueeze(1) @ vv).squeeze(1)
        res["attend_max_abs_err"] = float((out[0].float() - ref).abs().max())
        # scores vs an fp32 gather-sum in table order on the unpacked codes, one kv head
        c16 = self.hc.unpack_codes(self.codes[:1, :1].contiguous(), w.L, w.P, 0, n0).long()[0, 0]   # [L,T]
        acc = torch.zeros(n0, dtype=torch.float32, device=dev)
        for l in range(w.L):
            acc = acc + self.q_table_f32[0, 0, l].gather(0, c16[l])
        ref_s = acc * self.v_norm[0, 0, :n0].float()
        res["score_max_rel_err"] = float(((scores[0, 0, :n0] - ref_s).abs() / ref_s.abs().clamp_min(1e-30)).max())
        return res


def timed_graph_steps(step_fn, steps, warmup, eager=False):
    """Records one step into a HIP graph, checks three replays against the eager
    result, then times exactly `steps` replays after `warmup` untimed ones.  Returns
    (ms per step, wall ms of the timed region, "hip graph replay" | "eager", replay == eager)."""
    graph, ok = None, None
    if not eager:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(2):
                    step_fn()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            out_eager = step_fn().clone()   # the state is stationary from here on (same key re-appended)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out_graph = step_fn()
            for _ in range(3):
                graph.replay()
                torch.cuda.synchronize()
                if not torch.equal(out_graph, out_eager):
                    raise RuntimeError("graph replay differs from the eager step")
                _ = float(out_eager.float().sum())        # unrelated eager work between the replays
            ok = True
        except Exception as e:  # noqa: BLE001  fall back to eager launches, and say so in the result
            print(f"bench: HIP graph capture unavailable ({e}); timing eager launches", file=sys.stderr)
            graph, ok = None, None
    run = graph.replay if graph is not None else step_fn

    # The timed replays: `per` steps recorded back to back into one graph, as the
    # layers of a decode step are (32 of them per token in the model's graph), so
    # the figure carries the in-graph gap between steps and not the larger one
    # between two graph launches.  `per` divides `steps`: exactly `steps` steps run.
    per, graph_k = 1, None
    if graph is not None:
        per = max(d for d in range(1, min(steps, 64) + 1) if steps % d == 0)
        if per > 1:
            try:
                graph_k = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph_k):
                    for _ in range(per):
                        out_k = step_fn()
                graph_k.replay()
                torch.cuda.synchronize()
                if not torch.equal(out_k, out_eager):
                    raise RuntimeError("replay of the multi-step graph differs from the eager step")
            except Exception as e:  # noqa: BLE001
                print(f"bench: multi-step graph unavailable ({e}); one graph launch per step", file=sys.stderr)
                per, graph_k = 1, None
        if graph_k is None:
            per = 1
    run_k = graph_k.replay if graph_k is not None else run

    def timed(fn, calls, steps_per_call):
        for _ in range(warmup):
            run()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(calls):
            fn()
        e1.record()
        # host clock between seeing the first event done and the second: the region is
        # queued behind the settle phase's replays, which this must not count (and a
        # synchronize before the region would idle the GPU the settle phase warmed)
        e0.synchronize()
        t0 = time.perf_counter()
        e1.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (calls * steps_per_call), wall_ms

    # once from an idle GPU (reported beside the result), then after the settle phase
    torch.cuda.synchronize()
    time.sleep(0.05)
    after_idle_ms, _ = timed(run_k, steps // per, per)
    settled = settle(run)
    ms_per_step, wall_ms = timed(run_k, steps // per, per)
    state = {"settle_steps_untimed": settled, "settle_ms": SETTLE_MS,
             "us_per_step_from_idle": round(after_idle_ms * 1e3, 2), "steps_per_graph": per}
    if graph_k is not None:
        single_ms, _ = timed(run, steps, 1)
        state["us_per_step_one_graph_launch_each"] = round(single_ms * 1e3, 2)
    return (ms_per_step, wall_ms, ("hip graph replay" if graph is not None else "eager"), ok, state)


def measure_workload(w, dev, steps, warmup, args, full):
    """Per-kernel times, the graph-replayed step and the dense comparator for one
    workload.  `full`: also the scorer's other table layouts, the prefill hash and
    the parity gates (the headline workload)."""
    st = Step(w, dev, reference_table_layout=args.reference_table_layout)
    settle(st.prefill_hash)
    prefill_us = time_launches(st.prefill_hash, 10, warmup=2)
    scores = st.k_score()
    sl, ln = st.k_select(scores)
    out = st.k_attend(sl, ln)
    torch.cuda.synchronize()
    iters = max(steps, 1)
    parity = None if (args.no_parity or not full) else st.parity(scores, sl, ln, out)
    per = {
        "hash": time_graph(st.k_hash, iters),
        "score": time_graph(st.k_score, iters),
        "select": time_graph(lambda: st.k_select(scores), iters),
        "attend": time_graph(lambda: st.k_attend(sl, ln), iters),
        "dense": time_graph(st.k_dense, max(iters // 2, 5), per_graph=5),
    }
    if full:
        per["score_reference_layout"] = time_graph(st.k_score_ref, iters)
        per["score_f32_table"] = time_graph(st.k_score_f32, iters)
        per["score_f32_table_grouped"] = time_graph(st.k_score_f32_grouped, iters)
    ab = st.abytes
    kernels = {k: {"us": round(v, 2), "algorithmic_MB": round(ab[k] / 1e6, 2), "gbs": round(ab[k] / v / 1e3, 1),
                   "hbm_frac": round(ab[k] / v / 1e3 / HBM_PEAK_GBS, 4)} for k, v in per.items()}
    ms_per_step, wall_ms, launch, replay_ok, power_state = timed_graph_steps(st.step, steps, warmup, eager=args.eager)
    sparse_us = ms_per_step * 1e3
    sparse_bytes = ab["score"] + ab["select"] + ab["attend"]
    kernel_sum_us = per["score"] + per["select"] + per["attend"]
    from socket_amd._lib import lib
    rows = w.B * w.Hkv * w.T
    rec = {
        "workload": f"{w.name}: B{w.B} Hq{w.Hq}/Hkv{w.Hkv} D{w.D} T{w.T} bf16 KV cache, L{w.L}xP{w.P} packed codes, "
                    f"{str(st.q_table.dtype).split('.')[-1]} soft-hash table "
                    f"({'grouped' if st.use_grouped else '[B,Hq,L,R]'} layout), "
                    f"top-k {w.M} + sink {w.sink} + window {w.window}" + (", ragged lengths" if w.ragged else ""),
        "step_us": round(sparse_us, 2),
        "ms_per_step": ms_per_step,
        "launch": launch,
        "power_state": power_state,
        "kernel_timing": "HIP-graph replay of 10 launches between two HIP events (kernel time + in-graph launch gap), "
                         f">= 100 launches timed after {SETTLE_MS:.0f} ms of untimed replays",
        "kernels": kernels,
        "sparse_total": {"algorithmic_MB": round(sparse_bytes / 1e6, 2), "kernel_sum_us": round(kernel_sum_us, 2),
                         "hbm_frac_of_kernel_sum": round(sparse_bytes / kernel_sum_us / 1e3 / HBM_PEAK_GBS, 4),
                         "hbm_frac_of_step": round(sparse_bytes / sparse_us / 1e3 / HBM_PEAK_GBS, 4),
                         "speedup_vs_dense": round(per["dense"] / sparse_us, 3),
                         "attend_block_seq": lib().socket_sparse_attention_block_seq(w.B, w.Hq, sl.shape[-1])},
        "hash_prefill": {
            "prefill_ms": round(prefill_us / 1e3, 3), "rows": rows,
            # flops of the contraction the reference performs: 2 * D * L * P per key row
            "mfma_tflops": round(2.0 * rows * w.D * w.L * w.P / prefill_us / 1e6, 1),
            "mfma_frac": round(2.0 * rows * w.D * w.L * w.P / prefill_us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
            "hbm_gbs": round(rows * (2 * 2 * w.D + 4 * st.NW + 2) / prefill_us / 1e3, 1),
            "hbm_frac": round(rows * (2 * 2 * w.D + 4 * st.NW + 2) / prefill_us / 1e3 / HBM_PEAK_GBS, 4)},
        "parity": parity,
        "graph_replay_equals_eager": replay_ok,
        "wall_ms_timed_region": round(wall_ms, 2),
        "input_generation_s": round(st.input_generation_s, 1),
        "new_keys_hashed_per_step": w.B * w.Hkv * w.new_keys,
    }
    return rec, st, per


def drop_in_operator(st):
    """`sparse.build_sparse_list_decode` on the reference's own operands
    (GPT-FAST/kernels/sparse.py:16-95: q_probs [B,H,L,R] in the model's type,
    int16 codes per QUERY head [B,H,L,T], fp16 value norms and a boolean mask per
    query head) at this workload's size: what a caller that keeps the reference's
    cache layout pays.  Eager launches, torch's relayouts included, as the
    reference's call site runs it; the collision kernel alone beside it."""
    from socket_amd import sparse
    w = st.w
    G = w.Hq // w.Hkv
    T = w.T
    k_hard = st.hc.unpack_codes(st.codes, w.L, w.P, 0, T).repeat_interleave(G, dim=1).contiguous()      # [B,H,L,T] int16
    v_norm = st.v_norm[:, :, :T].repeat_interleave(G, dim=1).contiguous()
    pos = torch.arange(T, device=st.dev)
    lens = st.lens if st.lens is not None else torch.full((w.B,), T, dtype=torch.int32, device=st.dev)
    allowed = (pos[None, None, :] < lens[:, None, None]).expand(w.B, w.Hq, T).contiguous()
    q_probs = st.q_table                                                                                 # [B,H,L,R] bf16

    def op():
        return sparse.build_sparse_list_decode(q_probs, k_hard, v_norm, allowed, w.sink, w.window, w.M)

    ext = sparse._get_soft_hash_ext()
    q32 = q_probs.float().unsqueeze(2).contiguous()
    a_ext, v_ext = allowed.unsqueeze(2).contiguous(), v_norm.float().unsqueeze(2).contiguous()
    sl, ln = op()
    # the packed path's selection for the same step (its bf16-table sums may differ from
    # this fp32-table kernel's in the last place, so near-ties at the cut may swap)
    want_sl, want_ln = st.k_select(st.k_score())
    overlap = 1.0
    for b in (0, w.B - 1):
        for h in (0, w.Hq - 1):
            a = set(sl[b, h, :int(ln[b, h])].tolist())
            c = set(want_sl[b, h, :int(want_ln[b, h])].tolist())
            overlap = min(overlap, len(a & c) / max(len(c), 1))
    settle(op, 20.0)
    total = time_launches(op, 10, warmup=2)
    kern = time_graph(lambda: ext.soft_hash_collision(q32, k_hard, a_ext, v_ext), 20)
    nbytes = w.B * w.Hq * T * (2 * w.L + 1 + 4 + 4)         # int16 codes, mask byte, fp32 norm, fp32 score per (head, token)
    return {"operator_us": round(total, 1), "collision_kernel_us": round(kern, 1),
            "collision_kernel_algorithmic_MB": round(nbytes / 1e6, 1),
            "collision_kernel_gbs": round(nbytes / kern / 1e3, 1),
            "list_overlap_with_packed_path_min": round(overlap, 4),
            "operands": "q_probs bf16 [B,H,L,R], int16 codes [B,H,L,T] per query head, fp16 norms, bool mask"}


def decode_tok_s(dev, prompt_len, new_tokens, n_layer=None, kinds=("sparse", "dense")):
    """End-to-end greedy decode of the Llama-3.1-8B-shaped random-weight model through
    socket_amd.generate: decode-only tokens per second (the prefill's token excluded, as
    GPT-FAST/generate.py:361-369 counts), whole step replayed as one HIP graph."""
    from socket_amd import generate as gen
    from socket_amd.model import ModelArgs
    cfg = ModelArgs.from_name("Llama-3.1-8B")
    if n_layer is not None:
        cfg.n_layer = n_layer
    model = gen.load_random_model(cfg, dev, torch.bfloat16, 1234)
    g = torch.Generator().manual_seed(1234)
    prompt = torch.randint(0, cfg.vocab_size, (1, prompt_len), generator=g).to(dev)
    rec = {"model": f"Llama-3.1-8B geometry, {cfg.n_layer} layers, random bf16 weights N(0, 0.02)",
           "prompt_len": prompt_len, "new_tokens": new_tokens, "batch": 1,
           "budget": f"top-k {cfg.heavy_const} + sink {cfg.sink_size} + window {cfg.window_size}"}
    for kind in kinds:
        # "sparse_or_dense": decode_type "sparse" with ModelArgs.dense_below_crossover, i.e. the hook takes
        # the dense kernel while the library's estimate prices it below score + select + attend
        model.config.dense_below_crossover = kind == "sparse_or_dense"
        # check_graph: before the timed tokens the recorded step is replayed three times from one
        # state and compared with the eager step (logits and chosen token); the figures travel
        # with the tok/s so that a fast run whose graph went wrong cannot pass unnoticed
        _, st = gen.generate(model, prompt, new_tokens, decode_type="dense" if kind == "dense" else "sparse",
                             use_graph=True, check_graph=True)
        chk = st.get("graph_check") or {}
        rec[kind] = {"decode_tok_s": round(st["decode_only_tokens"] / st["decode_time_s"], 2),
                     "ms_per_token": round(1e3 * st["decode_time_s"] / st["decode_only_tokens"], 3),
                     "prefill_s": round(st["prefill_time_s"], 2), "graph": st["graph"],
                     "same_token": chk.get("same_token"), "max_abs_logit_diff": chk.get("max_abs_logit_diff")}
    model.config.dense_below_crossover = False
    if "sparse" in rec and "dense" in rec:
        rec["sparse_vs_dense"] = round(rec["sparse"]["decode_tok_s"] / rec["dense"]["decode_tok_s"], 3)
    if "sparse_or_dense" in rec and "dense" in rec:
        rec["sparse_or_dense_vs_dense"] = round(rec["sparse_or_dense"]["decode_tok_s"] / rec["dense"]["decode_tok_s"], 3)
    del model
    torch.cuda.empty_cache()
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=["c2", "c3", "c4", "c5"])
    ap.add_argument("--only", default=None,
                    choices=["score", "score_f32", "score_grouped", "select", "attend", "hash", "prefill_hash", "dense", "copy",
                             "block_sparse", "step", "decode", "read_probe"])
    ap.add_argument("--reference-table-layout", action="store_true",
                    help="feed the scorer q_probs as [B,Hq,L,R] instead of the grouped layout the soft-hash kernel writes")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="untimed GPU-busy time before each timed region (0: time from whatever state the GPU is in)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the other workloads' sub-records and the end-to-end decode runs")
    ap.add_argument("--eager", action="store_true", help="time plain launches instead of a recorded HIP graph")
    args = ap.parse_args()
    globals()["SETTLE_MS"] = args.settle_ms
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every (sequence, kv head) "
              "pair is independent, so the path shards over sequences or kv heads without exchange). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(2)

    from socket_amd import hash_cache
    from socket_amd.workloads import WORKLOADS

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.only == "block_sparse":
        block_sparse_bench(dev, max(args.steps, 1), args.warmup)
        return
    if args.only == "read_probe":
        # a pure read stream of known size (1 GiB of bf16 weights through the matrix-vector
        # kernel, 16-byte non-temporal loads): the calibration kernel for FETCH_SIZE when the
        # kernel under study issues full-width read requests, as the scorer's code stream does
        print(json.dumps({"only": "read_probe", "bytes_read": 131072 * 4096 * 2,
                          "gbs": round(read_ceiling_gbs(dev), 1)}))
        return
    if args.only == "decode":
        if args.workload == "c4":
            print(json.dumps({"only": "decode", "c4_prompt_65536": decode_tok_s(
                dev, 65536, 256, kinds=("sparse", "dense", "sparse_or_dense"))}))
        else:
            print(json.dumps({"only": "decode", "ctx_128k": decode_tok_s(dev, 131072 - 128, 128)}))
        return
    w = WORKLOADS[args.workload]
    iters = max(args.steps, 1)

    if args.only == "copy":
        # a plain device copy of known size (256 MiB read + 256 MiB written per launch):
        # the calibration kernel for the FETCH_SIZE / WRITE_SIZE counters
        a = torch.empty(1 << 26, dtype=torch.float32, device=dev).normal_()
        b = torch.empty_like(a)
        us = time_launches(lambda: b.copy_(a), iters, warmup=args.warmup)
        print(json.dumps({"only": "copy", "bytes_read": a.numel() * 4, "bytes_written": a.numel() * 4,
                          "us": round(us, 2), "gbs": round(2 * a.numel() * 4 / us / 1e3, 1), "iters": iters}))
        return
    if args.only:
        st = Step(w, dev, reference_table_layout=args.reference_table_layout)
        if args.only == "prefill_hash":
            settle(st.prefill_hash)
            us = time_launches(st.prefill_hash, iters, warmup=args.warmup)
            rows = w.B * w.Hkv * w.T
            print(json.dumps({"only": "prefill_hash", "workload": w.name, "us": round(us, 1), "rows": rows,
                              "mfma_tflops": round(2.0 * rows * w.D * w.L * w.P / us / 1e6, 1)}))
            return
        st.prefill_hash()
        scores = st.k_score()
        sl, ln = st.k_select(scores)
        torch.cuda.synchronize()
        fn = {"score": st.k_score_ref, "score_f32": st.k_score_f32, "score_grouped": st.k_score_grouped,
              "select": lambda: st.k_select(scores), "attend": lambda: st.k_attend(sl, ln), "hash": st.k_hash,
              "dense": st.k_dense, "step": st.step}[args.only]
        settle(fn)
        us = time_launches(fn, iters, warmup=args.warmup)
        key = args.only.replace("_grouped", "")
        nbytes = st.abytes[key] if key in st.abytes else st.abytes["score"] + st.abytes["select"] + st.abytes["attend"]
        print(json.dumps({"only": args.only, "workload": w.name, "us": round(us, 2),
                          "gbs": round(nbytes / us / 1e3, 1), "iters": iters}))
        return

    # ---- the headline workload: exactly --steps timed steps after --warmup -------------------
    rec, st, per = measure_workload(w, dev, args.steps, args.warmup, args, full=True)
    ceiling = copy_ceiling_gbs(dev)
    read_ceiling = read_ceiling_gbs(dev)
    ab = st.abytes
    result = {
        "metric": "sparse-attn us/layer/step at 128k ctx (score+select+attend+hash-append), % of HBM peak"
                  if w.name == "c3" else "sparse-attn us/layer/step (score+select+attend+hash-append), % of HBM peak",
        "value": rec["step_us"],
        "unit": "us/layer/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(rec["ms_per_step"], 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": rec["workload"], "layers_timed": 1,
                   "new_keys_hashed_per_step": rec["new_keys_hashed_per_step"], "launch": rec["launch"]},
        "roofline": {"kernel": "score_flat_kernel" if st.use_grouped else "score_packed_kernel", "bound": "hbm",
                     "achieved": round(ab["score"] / per["score"] / 1e3, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(ab["score"] / per["score"] / 1e3 / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(w.name) if st.use_grouped else None,
                     "traffic_source": (MEASURED_TRAFFIC_SOURCE.format(w=w.name)
                                        if MEASURED_TRAFFIC_BYTES.get(w.name) and st.use_grouped else None)},
        "kernels": rec["kernels"],
        "kernel_timing": rec["kernel_timing"],
        "power_state": rec["power_state"],
        "sparse_total": rec["sparse_total"],
        "hash_prefill": rec["hash_prefill"],
        "copy_ceiling_gbs": round(ceiling, 1),
        "read_ceiling_gbs": round(read_ceiling, 1),
        "parity": rec["parity"],
        "graph_replay_equals_eager": rec["graph_replay_equals_eager"],
        "wall_ms_timed_region": rec["wall_ms_timed_region"],
        "input_generation_s": rec["input_generation_s"],
    }

    if not args.no_extra and w.name == "c3":
        result["drop_in_operator"] = drop_in_operator(st)
    if not args.no_cpu:
        T, Hkv, Hq = w.T, w.Hkv, w.Hq
        lens, budgets = st.lens, st.budgets
        n0 = T if lens is None else int(lens[0])
        m0 = w.M if budgets is None else int(budgets[0])
        nkv = min(2, Hkv)
        G = Hq // Hkv
        inp_cpu = {"q": st.inp.q.cpu(), "q_probs": st.inp.q_probs[:1, :nkv * G].cpu(), "k": st.inp.k[:1, :nkv].cpu(),
                   "v": st.inp.v[:1, :nkv].cpu(), "len0": n0, "m0": m0,
                   "tok_total": w.B * T if lens is None else int(lens.sum())}
        codes_cpu = hash_cache.unpack_codes(st.codes[:1, :nkv].contiguous(), w.L, w.P, 0, n0).cpu()
        vn_cpu = st.v_norm[:1, :nkv].cpu()
    del st
    torch.cuda.empty_cache()

    # ---- the other single-layer workloads and the end-to-end decode runs ---------------------
    if not args.no_extra and args.workload == "c3":
        sub_steps = max(10, args.steps // 2)
        for name in ("c2", "c5"):
            r, s2, _ = measure_workload(WORKLOADS[name], dev, sub_steps, 3, args, full=False)
            for k in ("ms_per_step", "parity", "input_generation_s", "kernel_timing"):
                r.pop(k, None)
            r["steps"] = sub_steps
            if name == "c2":
                r["drop_in_operator"] = drop_in_operator(s2)
            result[name] = r
            del s2
            torch.cuda.empty_cache()
        # the metric's second half: decode tokens per second at 128k context (prompt
        # 130944 + 128 new tokens = the model's block_size), and configuration 4 as its definition
        # states it (65536-token prompt, 256 greedy tokens)
        result["decode_tok_s"] = {"ctx_128k": decode_tok_s(dev, 131072 - 128, 128),
                                  "c4_prompt_65536": decode_tok_s(dev, 65536, 256,
                                                                  kinds=("sparse", "dense", "sparse_or_dense"))}

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(w, inp_cpu, codes_cpu, vn_cpu)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
