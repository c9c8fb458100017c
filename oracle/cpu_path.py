"""The reference's CPU-expressible expert layer, timed by ``bench.py`` as the
``cpu_baseline`` (kind "port").  Test infrastructure only.

Steps: host counting-sort mapping (disagmoe/ops/memory.py:34-54 semantics),
``torch.index_select`` gather-permute (tests/dp/test_split.py:33), the
per-expert matmul loop ``silu(x_e @ w1[e]) * (x_e @ w3[e]) @ w2[e]``
(disagmoe/models/experts.py:105-120 with w1/w3 the halves of w13), then the
gate-weighted gather-sum back to token order (disagmoe/frontend/engine.py:
726-734, 624-628).  Storage dtype is the input dtype (bf16); torch's CPU matmul
accumulates in fp32.
"""
from __future__ import annotations

import time
from typing import Dict

import numpy as np
import torch

from . import routing


def expert_layer(x: torch.Tensor, topk_ids: torch.Tensor, topk_weights: torch.Tensor,
                 w13: torch.Tensor, w2: torch.Tensor, timings: Dict[str, float] | None = None) -> torch.Tensor:
    """One pass over ``x [T, d]`` with ``topk_ids/topk_weights [T, k]``; returns
    ``[T, d]``.  ``timings`` (if given) receives seconds per stage."""
    E, _, I2 = w13.shape
    I = I2 // 2
    T, k = topk_ids.shape
    t0 = time.perf_counter()
    mappings, cnt = routing.get_mappings_from_exp_ids(topk_ids, E)
    m = torch.tensor(mappings, dtype=torch.int64)
    inv = torch.empty_like(m)
    inv[m] = torch.arange(m.numel(), dtype=torch.int64)
    t1 = time.perf_counter()
    xp = torch.index_select(x, 0, inv // k)
    t2 = time.perf_counter()
    outs = []
    o = 0
    for e in range(E):
        n = cnt[e]
        if n == 0:
            continue
        xe = xp[o:o + n]
        h = torch.nn.functional.silu(xe @ w13[e, :, :I]) * (xe @ w13[e, :, I:])
        outs.append(h @ w2[e])
        o += n
    y = torch.cat(outs) if outs else xp.new_zeros((0, w2.shape[2]))
    t3 = time.perf_counter()
    w = topk_weights.to(y.dtype)
    out = (y[m.view(T, k)] * w[:, :, None]).sum(dim=1)
    t4 = time.perf_counter()
    if timings is not None:
        timings.update(route=t1 - t0, permute=t2 - t1, ffn=t3 - t2, combine=t4 - t3, total=t4 - t0)
    return out
