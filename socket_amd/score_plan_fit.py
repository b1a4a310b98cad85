"""Where the constants of the scorer's launch-shape cost model come from.

The scorer (csrc/score.hip) picks the tokens per workgroup, the way table slices
reach LDS and whether a workgroup serves one query head by pricing every
launchable shape:

    t_cu   = a + s * slices + r * table_KB / waves + c[entry] * 1e-6 * tile * L      (us)
    t_mem  = active_workgroups * tile * bytes_per_token / (stream_GB/s * 1e3)        (us)
    cost   = rounds * cbrt(t_cu^3 + t_mem^3)

with one (a, s, r, c[]) set per kernel variant.  This module measures forced
shapes on the device and refits those sets:

    python -m socket_amd.build --measurement-lib /tmp/libsocket_forced.so
    python -m socket_amd.score_plan_fit sweep --lib /tmp/libsocket_forced.so --out sweep.jsonl
    python -m socket_amd.score_plan_fit fit sweep.jsonl

`sweep` needs a GPU and a measurement build of the library (the shape is forced
through the SOCKET_SCORE_FORCE environment variable, which product builds do not
read); `fit` runs anywhere and prints the constants in the form score.hip holds
them, with the regret of the model's choices against the best measured shape.
"""
import argparse
import itertools
import json
import math
import os
from collections import defaultdict
from ctypes import byref, c_float, c_int

import numpy as np

TILES = (8192, 4096, 2048, 1024)
VARIANTS = ((1, 0), (0, 0), (1, 1))                     # (direct copy, one head per workgroup)
GEOMETRIES = [(60, 10, 4, "bfloat16"), (48, 10, 4, "bfloat16"), (32, 8, 4, "bfloat16"), (60, 10, 2, "bfloat16"),
              (60, 10, 1, "bfloat16"), (60, 10, 4, "float32"), (48, 10, 7, "bfloat16"), (32, 8, 4, "float32")]
BATCHES = [(1, 8, 32768), (1, 8, 65536), (1, 8, 131072), (4, 8, 131072), (2, 8, 65536), (16, 4, 65536), (4, 8, 16384)]
STREAM_GBS = (4400, 4800, 5200, 5600, 6000, 6500)
ENTRY_BYTES = (2, 4, 8, 16)
VARIANT_NAMES = ("kCostDirect", "kCostStagedRef", "kCostStagedGrouped", "kCostSolo")


def sweep(lib_path, out_path, iters=10):
    import torch
    from socket_amd import _lib
    _lib.LIB_PATH = os.path.abspath(lib_path)
    from socket_amd import hash_cache
    dev = torch.device("cuda:0")

    def time_us(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) * 1000 / iters

    with open(out_path, "w") as out:
        for (L, P, G, dt), (B, Hkv, T) in itertools.product(GEOMETRIES, BATCHES):
            Hq, R = Hkv * G, 1 << P
            if B * Hq * T * 4 > 3e9:
                continue
            g = torch.Generator(device=dev).manual_seed(1)
            ref = torch.rand(B, Hq, L, R, generator=g, device=dev).to(getattr(torch, dt))
            grouped = hash_cache.group_q_probs(ref, Hkv)
            NW = hash_cache.words_per_key(L, P)
            codes = torch.randint(0, 2 ** 31 - 1, (B, Hkv, NW, T), generator=g, device=dev, dtype=torch.int32)
            vn = torch.rand(B, Hkv, T, generator=g, device=dev).to(torch.float16)
            sc = torch.empty(B, Hq, T, dtype=torch.float32, device=dev)
            for tile, (dma, solo) in itertools.product(TILES, VARIANTS):
                tables = (("grouped", grouped),) if (dma and not solo) else (("ref", ref),) if solo else \
                    (("grouped", grouped), ("ref", ref))
                for layout, tab in tables:
                    os.environ["SOCKET_SCORE_FORCE"] = f"{tile},{dma},{solo}"
                    kw = {"n_heads": Hq} if tab.dim() == 5 else {}
                    try:
                        us = time_us(lambda: hash_cache.score_packed(tab, codes, vn, T, P, out=sc, **kw))
                    except RuntimeError:
                        us = None                                  # the shape cannot be launched for this table
                    out.write(json.dumps(dict(L=L, P=P, G=G, dt=dt, B=B, Hkv=Hkv, T=T, tile=tile, dma=dma, solo=solo,
                                              layout=layout, us=us)) + "\n")
                    out.flush()
            os.environ.pop("SOCKET_SCORE_FORCE", None)
            print("measured", L, P, G, dt, B, Hkv, T, flush=True)


def _features(lib, r, cu_count):
    """What the model prices a shape on; slices and waves come from the library's own layout code."""
    L, P, G, B, Hkv, T, tile = r["L"], r["P"], r["G"], r["B"], r["Hkv"], r["T"], r["tile"]
    eb = 2 if r["dt"] == "bfloat16" else 4
    solo, dma, grouped = bool(r["solo"]), bool(r["dma"]), r["layout"] == "grouped"
    if G == 1 and solo:                                  # runs as the direct-copy shape
        solo = False
    slices, waves, cost = c_int(), c_int(), c_float()
    rc = lib.socket_score_shape_cost(B, Hkv * G, Hkv, T, 0 if eb == 4 else 1, L, P, 1 << P, int(grouped), tile,
                                     int(dma), int(solo), byref(slices), byref(waves), byref(cost))
    if rc != 0:
        return None
    cpw = 32 // P
    NW = (L + cpw - 1) // cpw
    width = 1 if (G == 1 or solo) else 2 if G == 2 else 4
    hsplit = G if solo else (G + width - 1) // width
    wgs = B * Hkv * hsplit * math.ceil(T / tile)
    return dict(variant=3 if solo else 0 if dma else 2 if grouped else 1, slices=slices.value, waves=waves.value,
                table_kb=L * (1 << P) * width * eb / 1e3, lookups=tile * L, entry=width * eb,
                rounds=math.ceil(wgs / cu_count), active=min(wgs, cu_count), tile=tile,
                bpt=(NW * 4 + 2) / (G if solo else 1) + 4 * width, model_cost=cost.value)


def _row(f):
    return [1.0, f["slices"], f["table_kb"] / f["waves"]] + [f["lookups"] * 1e-6 if f["entry"] == e else 0.0
                                                            for e in ENTRY_BYTES]


def _t_mem(f, gbs):
    return f["active"] * f["tile"] * f["bpt"] / (gbs * 1e3)


def _fit_variants(F, y, gbs):
    from scipy.optimize import nnls
    coef = {}
    for v in range(4):
        A = []
        for f, us in zip(F, y):
            if f["variant"] != v:
                continue
            t_round, t_mem = us / f["rounds"], _t_mem(f, gbs)
            if t_round <= t_mem * 1.02:                  # stream-bound sample: says nothing about t_cu
                continue
            t_cu = (t_round ** 3 - t_mem ** 3) ** (1 / 3)
            A.append([x / t_cu for x in _row(f)])        # relative error
        coef[v] = nnls(np.array(A), np.ones(len(A)))[0]
    return coef


def _predict(coef, gbs, f):
    t_cu = float(np.dot(coef[f["variant"]], _row(f)))
    return f["rounds"] * (t_cu ** 3 + _t_mem(f, gbs) ** 3) ** (1 / 3)


def fit(path, cu_count=256, margin=1.3):
    from socket_amd import _lib
    lib = _lib.lib()
    rows = [json.loads(line) for line in open(path)]
    meas, F = [], []
    for r in rows:
        if r.get("us") is None or not r.get("tile"):
            continue
        f = _features(lib, r, cu_count)
        if f is not None:
            meas.append(r)
            F.append(f)
    y = np.array([r["us"] for r in meas])
    by_case = defaultdict(lambda: defaultdict(list))
    for r, f in zip(meas, F):
        by_case[(r["L"], r["P"], r["G"], r["dt"], r["B"], r["Hkv"], r["T"])][r["layout"]].append((r, f))

    def regrets(cost_of):
        shape, layout = [], []
        for d in by_case.values():
            for lst in d.values():
                shape.append(min(lst, key=lambda t: cost_of(t[1]))[0]["us"] / min(r["us"] for r, _ in lst))
            if len(d) == 2:
                best = min(r["us"] for lst in d.values() for r, _ in lst)
                pg = min(cost_of(f) for _, f in d["grouped"])
                pr = min(cost_of(f) for _, f in d["ref"])
                lay = "grouped" if pg <= pr * margin else "ref"
                layout.append(min(d[lay], key=lambda t: cost_of(t[1]))[0]["us"] / best)
        return np.mean(shape), max(shape), np.mean(layout), max(layout)

    best = None
    for gbs in STREAM_GBS:
        coef = _fit_variants(F, y, gbs)
        reg = regrets(lambda f: _predict(coef, gbs, f))
        err = np.array([math.log(_predict(coef, gbs, f) / us) for f, us in zip(F, y)])
        print(f"stream {gbs} GB/s: rms log error {np.sqrt((err ** 2).mean()):.3f}; shape regret mean {reg[0]:.3f} "
              f"max {reg[1]:.3f}; layout regret (margin {margin}) mean {reg[2]:.3f} max {reg[3]:.3f}")
        if best is None or reg[2] < best[0]:
            best = (reg[2], gbs, coef)
    _, gbs, coef = best
    print(f"\nconstexpr float kStreamGBs = {gbs}.f;")
    for v, name in enumerate(VARIANT_NAMES):
        a, s, r, *c = (float(x) for x in coef[v])
        print(f"constexpr VariantCost {name} = {{{a:.3f}f, {s:.3f}f, {r:.3f}f, "
              f"{{{', '.join(f'{x:.1f}f' for x in c)}}}}};")
    reg = regrets(lambda f: f["model_cost"])
    print(f"\nthe library as built: shape regret mean {reg[0]:.3f} max {reg[1]:.3f}; "
          f"layout regret mean {reg[2]:.3f} max {reg[3]:.3f}  ({len(meas)} measurements, {len(by_case)} cases)")
    return reg


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    s = sub.add_parser("sweep")
    s.add_argument("--lib", required=True)
    s.add_argument("--out", required=True)
    f = sub.add_parser("fit")
    f.add_argument("jsonl")
    a = ap.parse_args()
    if a.cmd == "sweep":
        sweep(a.lib, a.out)
    else:
        fit(a.jsonl)


if __name__ == "__main__":
    main()
