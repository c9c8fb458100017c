"""Synthetic inputs of the five benchmark configurations.

Activations N(0,1), weights N(0,0.02), routing uniform without replacement
(Zipf s=1.2 for the decode case), gates = softmax over the k chosen N(0,1)
logits.  Activations and routing come from a seeded CPU generator (same bits on
any machine); weights are generated expert by expert, on the target device when
it is a GPU (seeded there) so that the multi-GB tensors never exist in fp32.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    E: int
    d: int
    I: int
    T: int
    k: int
    routing: str = "uniform"   # "uniform" | "zipf"
    fp8: bool = False
    seed: int = 20250

    @property
    def R(self) -> int:
        return self.T * self.k

    @property
    def gemm_flops(self) -> float:
        return 6.0 * self.R * self.d * self.I

    @property
    def permute_bytes(self) -> float:
        return 2.0 * self.R * self.d * 2 + 8.0 * self.R

    @property
    def combine_bytes(self) -> float:
        return self.R * self.d * 2 + self.T * self.d * 2 + 8.0 * self.R + 4.0 * self.R

    @property
    def route_bytes(self) -> float:
        return 4.0 * self.R + 8.0 * self.R + 16.0 * self.E


WORKLOADS = {
    "C1": Workload("C1-tiny", E=8, d=1024, I=2816, T=512, k=2, seed=20250),
    "C2": Workload("C2-mixtral-8x7b", E=8, d=4096, I=14336, T=4096, k=2, seed=20251),
    "C3": Workload("C3-decode-zipf", E=8, d=4096, I=14336, T=256, k=2, routing="zipf", seed=20252),
    "C4": Workload("C4-fine-grained", E=64, d=2048, I=1408, T=8192, k=6, seed=20253),
    "C5": Workload("C5-mixtral-8x22b-fp8", E=8, d=6144, I=16384, T=16384, k=2, fp8=True, seed=20254),
}


def make_routing(w: Workload, T: int | None = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(topk_ids [T, k] int32, topk_weights [T, k] fp32)`` on the CPU."""
    T = w.T if T is None else T
    g = torch.Generator().manual_seed(w.seed)
    if w.routing == "zipf":
        p = (torch.arange(1, w.E + 1, dtype=torch.float64) ** -1.2)
        p = (p / p.sum()).float()
        ids = torch.multinomial(p.expand(T, w.E), w.k, replacement=False, generator=g)
    else:
        ids = torch.argsort(torch.rand(T, w.E, generator=g), dim=1)[:, :w.k]
    logits = torch.randn(T, w.k, generator=g)
    return ids.to(torch.int32).contiguous(), torch.softmax(logits, dim=1).contiguous()


def make_activations(w: Workload, T: int | None = None) -> torch.Tensor:
    T = w.T if T is None else T
    g = torch.Generator().manual_seed(w.seed + 1000)
    return torch.randn(T, w.d, generator=g).to(torch.bfloat16)


def make_weights(w: Workload, device: torch.device | str = "cpu", std: float = 0.02,
                 E: int | None = None, d: int | None = None, I: int | None = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(w13 [E, d, 2I], w2 [E, I, d])`` bf16 on ``device``."""
    E = w.E if E is None else E
    d = w.d if d is None else d
    I = w.I if I is None else I
    device = torch.device(device)
    g = torch.Generator(device=device).manual_seed(w.seed + 2000)
    w13 = torch.empty((E, d, 2 * I), dtype=torch.bfloat16, device=device)
    w2 = torch.empty((E, I, d), dtype=torch.bfloat16, device=device)
    for e in range(E):
        w13[e] = (torch.randn((d, 2 * I), generator=g, device=device) * std).to(torch.bfloat16)
        w2[e] = (torch.randn((I, d), generator=g, device=device) * std).to(torch.bfloat16)
    return w13, w2
