"""Writes tests/golden/*.npz: small seeded input/output vectors for every kernel
of the path, computed by the CPU oracle (oracle/socket_oracle.py).

The reference ships no golden vectors for this path, so these pin the oracle
against drift and give the HIP tests fixed cases; the oracle itself is pinned by
closed forms and invariants in tests/test_oracle_pins.py.

    python tests/golden/make_fixtures.py        # rewrites the fixtures in place
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import socket_oracle as orc  # noqa: E402


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().copy()


def hash_case(seed=101, B=2, S=13, Hkv=2, D=128, L=20, P=10):
    g = torch.Generator().manual_seed(seed)
    keys = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
    vals = torch.randn(B, S, Hkv, D, generator=g).to(torch.bfloat16)
    planes = torch.randn(L, P, D, generator=g).to(torch.bfloat16)
    proj = orc.projections_f64(keys.float(), planes.float())
    codes = orc.pack_bits(proj >= 0)                                            # [B,S,Hkv,L]
    decided = (proj.abs() > 1e-3 * proj.abs().mean()).all(-1)
    words = orc.pack_code_words(codes.permute(0, 2, 3, 1).numpy(), P)           # [B,Hkv,NW,S]
    return dict(keys_bf16=bf16_bits(keys), vals_bf16=bf16_bits(vals), planes_bf16=bf16_bits(planes),
                codes=codes.numpy(), decided=decided.numpy(), words=words,
                v_norm_f16=orc.value_norm(vals).view(torch.int16).numpy(), L=L, P=P)


def score_case(seed=202, B=2, Hq=4, Hkv=1, L=13, P=8, T=500):
    g = torch.Generator().manual_seed(seed)
    R, G = 1 << P, Hq // Hkv
    q_probs = torch.softmax(torch.randn(B, Hq, L, R, generator=g) * 3, -1)
    codes = torch.randint(0, R, (B, Hkv, L, T), generator=g, dtype=torch.int32).to(torch.int16)
    v_norm = (torch.rand(B, Hkv, T, generator=g) * 9).to(torch.float16)
    lens = torch.tensor([T, T - 123], dtype=torch.int32)
    allowed = (torch.arange(T)[None, None] < lens[:, None, None]).expand(B, Hq, T)
    scores = orc.collision_score(q_probs, codes.repeat_interleave(G, 1), allowed, v_norm.float().repeat_interleave(G, 1))
    q16 = q_probs.to(torch.bfloat16)
    scores16 = orc.collision_score(q16.float(), codes.repeat_interleave(G, 1), allowed,
                                   v_norm.float().repeat_interleave(G, 1))
    return dict(q_probs=q_probs.numpy(), q_probs_bf16=bf16_bits(q16), codes=codes.numpy(),
                v_norm_f16=v_norm.view(torch.int16).numpy(), lens=lens.numpy(), scores=scores.numpy(),
                scores_bf16_table=scores16.numpy(), P=P)


def select_case(seed=303, B=2, H=3, T=3000, M=200, sink=4, window=32):
    g = torch.Generator().manual_seed(seed)
    s = torch.randn(B, H, T, generator=g)
    s[0, 1] = torch.randint(0, 6, (T,), generator=g).float()                    # heavy ties
    s[1, 0, ::5] = float("-inf")
    s[1, 2, 17] = float("nan")
    lens = torch.tensor([T, T - 701], dtype=torch.int32)
    lists, counts = [], []
    for b in range(B):
        n = int(lens[b])
        base = torch.from_numpy(orc.base_indices(n, sink, window))
        for h in range(H):
            heavy = orc.topk_lower_index_first(s[b, h, :n], min(M, n)).to(torch.int32)
            row = torch.cat([base, heavy])
            counts.append(row.numel())
            lists.append(torch.cat([row, torch.full((sink + window + M - row.numel(),), -1, dtype=torch.int32)]))
    return dict(scores=s.numpy(), lens=lens.numpy(), sparse_list=torch.stack(lists).view(B, H, -1).numpy(),
                sparse_len=np.array(counts, dtype=np.int32).reshape(B, H), M=M, sink=sink, window=window)


def attend_case(seed=404, B=1, Hq=4, Hkv=2, D=64, S=200, Kt=90):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, S, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, S, D, generator=g).to(torch.bfloat16)
    sl = torch.randint(0, S, (B, Hq, Kt), generator=g, dtype=torch.int32)
    sl[torch.rand(B, Hq, Kt, generator=g) < 0.05] = -1
    ln = torch.randint(Kt // 2, Kt + 1, (B, Hq), generator=g, dtype=torch.int32)
    out = orc.sparse_attend_textbook(q, k, v, sl, ln)
    return dict(q_bf16=bf16_bits(q), k_bf16=bf16_bits(k), v_bf16=bf16_bits(v), sparse_list=sl.numpy(),
                sparse_len=ln.numpy(), out_f64=out.numpy())


def soft_hash_case(seed=505, B=1, Hq=4, D=128, L=5, K=8):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, D, generator=g)
    planes = torch.randn(L, K, D, generator=g) * 0.3
    protos = torch.randn(K, 1 << K, generator=g) * 3
    cube = orc.hypercube_protos_T(K)
    return dict(q=q.numpy(), planes=planes.numpy(), protos=protos.numpy(),
                probs=orc.soft_hash(q, planes, protos, 1.0).numpy(),
                probs_cube_t03=orc.soft_hash(q, planes, cube, 0.3).numpy())


CASES = {"hash": hash_case, "score": score_case, "select": select_case, "attend": attend_case,
         "soft_hash": soft_hash_case}


def main():
    torch.set_num_threads(1)        # one summation order, whatever the machine
    for name, fn in CASES.items():
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **fn())
        print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
