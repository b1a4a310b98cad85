"""Seeded synthetic inputs for the five benchmark configurations.

Every tensor is drawn from `torch.Generator().manual_seed(1000 * config + layer)`.
Small configurations (and every test) draw on the CPU and move to the device;
`device_rng=True` draws the bulk K/V tensors with a seeded device generator
instead, which is what the benchmark uses at 128k context where a CPU draw of
2 x 0.5 G normals would dominate the run.

The query-side soft-hash is the hypercube form used by the reference's
HuggingFace path (pipeline/train_quest/modeling/modeling_llama.py:569-590,
618-638), written in its closed form: q_probs[l, r] = prod_k sigmoid(tau *
c_{r,k} * proj_{l,k}) with proj = planes . q / ||q|| and c the +-1 corner of
bucket r in pack_bits order.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch


@dataclass
class Workload:
    name: str
    config: int
    B: int
    Hq: int
    Hkv: int
    D: int
    T: int                      # context length (max over the batch when ragged)
    L: int
    P: int
    M: int                      # top-k budget (max over the batch when ragged)
    sink: int
    window: int
    dtype: torch.dtype
    tau: float = 4.0
    planted_frac: float = 0.0   # fraction of keys planted along the query direction
    planted_count: int = 0      # or an absolute count per KV head
    channel_scale: bool = False
    ragged: bool = False
    t_min: int = 0
    budget_frac: float = 0.0
    new_keys: int = 1           # keys appended per (b, kv head) per step

    @property
    def R(self) -> int:
        return 1 << self.P

    @property
    def G(self) -> int:
        return self.Hq // self.Hkv


WORKLOADS = {
    "c1": Workload("c1", 1, 1, 32, 8, 128, 4096, 32, 8, 128, 4, 64, torch.float32, planted_count=16),
    "c2": Workload("c2", 2, 1, 32, 8, 128, 32768, 60, 10, 1024, 4, 128, torch.bfloat16,
                   planted_frac=0.005, channel_scale=True),
    "c3": Workload("c3", 3, 4, 32, 8, 128, 131072, 60, 10, 2048, 4, 256, torch.bfloat16,
                   planted_frac=0.005, channel_scale=True),
    # one attention layer of the 32-layer model run: one sequence, 65536 cached tokens
    "c4": Workload("c4", 4, 1, 32, 8, 128, 65536, 60, 10, 2048, 4, 256, torch.bfloat16,
                   planted_frac=0.005, channel_scale=True),
    "c5": Workload("c5", 5, 16, 28, 4, 128, 98304, 48, 10, 1966, 4, 128, torch.bfloat16,
                   planted_frac=0.005, channel_scale=True, ragged=True, t_min=16384, budget_frac=0.02),
}


def scaled(w: Workload, **kw) -> Workload:
    """A copy of `w` with some fields replaced (tests shrink T, B, M)."""
    d = dict(w.__dict__)
    d.update(kw)
    return Workload(**d)


@dataclass
class Inputs:
    q: torch.Tensor            # [B,Hq,D]
    k: torch.Tensor            # [B,Hkv,T,D]
    v: torch.Tensor            # [B,Hkv,T,D]
    planes: torch.Tensor       # [L,P,D] float32
    q_probs: torch.Tensor      # [B,Hq,L,R] float32
    lens: Optional[torch.Tensor] = None      # [B] int32 (ragged only)
    budgets: Optional[torch.Tensor] = None   # [B] int32 (ragged only)
    k_new: Optional[torch.Tensor] = None     # [B,new,Hkv,D]
    v_new: Optional[torch.Tensor] = None


def hypercube_corners(P: int, device=None) -> torch.Tensor:
    """[R,P] of +-1; corner r has +1 at coordinate k iff bit (P-1-k) of r is set."""
    r = torch.arange(1 << P, device=device).unsqueeze(1)
    k = torch.arange(P, device=device).unsqueeze(0)
    return (((r >> (P - 1 - k)) & 1) * 2 - 1).to(torch.float32)


def soft_probs_sigmoid_product(q: torch.Tensor, planes: torch.Tensor, tau: float) -> torch.Tensor:
    """q [B,Hq,D], planes [L,P,D] -> q_probs [B,Hq,L,R] float32."""
    qn = q.float() / q.float().norm(dim=-1, keepdim=True).clamp_min(1e-20)
    proj = torch.einsum("bhd,lkd->bhlk", qn, planes.float().to(q.device))
    corners = hypercube_corners(planes.shape[1], q.device)            # [R,P]
    x = proj.unsqueeze(-2) * corners                                   # [B,H,L,R,P]
    return torch.sigmoid(tau * x).prod(dim=-1).contiguous()


def make_inputs(w: Workload, device="cpu", layer: int = 0, device_rng: bool = False) -> Inputs:
    seed = 1000 * w.config + layer
    g = torch.Generator().manual_seed(seed)
    B, Hq, Hkv, D, T = w.B, w.Hq, w.Hkv, w.D, w.T
    q = torch.randn(B, Hq, D, generator=g)
    planes = torch.randn(w.L, w.P, D, generator=g)
    scale_k = torch.ones(D)
    scale_v = torch.ones(D)
    if w.channel_scale:
        scale_k = torch.rand(D, generator=g) * 1.5 + 0.5
        scale_v = torch.rand(D, generator=g) * 1.5 + 0.5
    n_plant = w.planted_count if w.planted_count else int(round(w.planted_frac * T))
    plant_pos = torch.stack([torch.randperm(T, generator=g)[:n_plant] for _ in range(B * Hkv)]).view(B, Hkv, n_plant)
    plant_noise = torch.randn(B, Hkv, n_plant, D, generator=g)
    lens = budgets = None
    if w.ragged:
        lens = torch.randint(w.t_min, T + 1, (B,), generator=g, dtype=torch.int64)
        lens[0] = T  # the longest sequence defines the cache extent
        budgets = (lens.double() * w.budget_frac).floor().to(torch.int32)
        lens = lens.to(torch.int32)
    k_new = torch.randn(B, w.new_keys, Hkv, D, generator=g)
    v_new = torch.randn(B, w.new_keys, Hkv, D, generator=g)

    dev = torch.device(device)
    if device_rng and dev.type == "cuda":
        gd = torch.Generator(device=dev).manual_seed(seed)
        k = torch.empty(B, Hkv, T, D, dtype=w.dtype, device=dev)
        v = torch.empty(B, Hkv, T, D, dtype=w.dtype, device=dev)
        for b in range(B):  # per batch element: bounds the fp32 temporaries
            k[b] = (torch.randn(Hkv, T, D, generator=gd, device=dev) * scale_k.to(dev)).to(w.dtype)
            v[b] = (torch.randn(Hkv, T, D, generator=gd, device=dev) * scale_v.to(dev)).to(w.dtype)
    else:
        k = (torch.randn(B, Hkv, T, D, generator=g) * scale_k).to(w.dtype).to(dev)
        v = (torch.randn(B, Hkv, T, D, generator=g) * scale_v).to(w.dtype).to(dev)

    # planted heavy keys: 4 * unit mean query direction of the kv head's group + noise
    qdir = q.view(B, Hkv, w.G, D).mean(dim=2)
    qdir = qdir / qdir.norm(dim=-1, keepdim=True)
    planted = (4.0 * qdir.unsqueeze(2) + plant_noise).to(w.dtype).to(dev)
    idx = plant_pos.to(dev).unsqueeze(-1).expand(-1, -1, -1, D)
    k.scatter_(2, idx, planted)

    q = q.to(w.dtype).to(dev)
    q_probs = soft_probs_sigmoid_product(q, planes.to(dev), w.tau)
    return Inputs(q=q, k=k, v=v, planes=planes.to(dev), q_probs=q_probs,
                  lens=None if lens is None else lens.to(dev),
                  budgets=None if budgets is None else budgets.to(dev),
                  k_new=(k_new * scale_k).to(w.dtype).to(dev), v_new=(v_new * scale_v).to(w.dtype).to(dev))
