"""Row movement oracle (torch, CPU).  Test infrastructure only."""
from __future__ import annotations

from typing import Sequence

import torch


def _as_long(mappings) -> torch.Tensor:
    if not torch.is_tensor(mappings):
        mappings = torch.tensor(list(mappings), dtype=torch.int64)
    return mappings.detach().cpu().to(torch.int64).reshape(-1)


def permute_tokens(tokens: torch.Tensor, mappings) -> torch.Tensor:
    """``out[mappings[t], :] = tokens[t // k, :]`` with ``k = R // T``.

    csrc/cuda_ops/permute.cu:53-58 (kernel), :86-112 (entry: ``R % T == 0``,
    output ``[R, d]`` with the options of ``tokens``); the Python wrapper is
    disagmoe/ops/memory.py:94-102.  With ``R == T`` it is the plain scatter the
    reference's test spells out (tests/ops/test_memory.py:27-31)."""
    tokens = tokens.detach().cpu()
    m = _as_long(mappings)
    T, d = tokens.shape
    R = m.numel()
    out = torch.empty((R, d), dtype=tokens.dtype)
    if R == 0:
        return out
    assert T > 0 and R % T == 0
    k = R // T
    src = torch.arange(R, dtype=torch.int64) // k
    out[m] = tokens[src]
    return out


def gather_rows(tokens: torch.Tensor, index) -> torch.Tensor:
    """``out[t, :] = tokens[index[t], :]`` -- the index form of the expert-side
    merge gather (csrc/cuda_ops/permute.cu:114-119, where the sources are raw row
    pointers prepared at csrc/include/datatypes.hpp:529-543) and the
    ``torch.index_select`` permute of tests/dp/test_split.py:33."""
    return torch.index_select(tokens.detach().cpu(), 0, _as_long(index))


def gather_row_slabs(slabs: Sequence[torch.Tensor], mappings) -> torch.Tensor:
    """``TensorBatch::merge`` (csrc/include/datatypes.hpp:508-549): rows of the
    slabs, taken in arrival order as one stream ``s``, land at
    ``out[mappings[s]]``."""
    stream = torch.cat([s.detach().cpu() for s in slabs], dim=0)
    return permute_tokens(stream, mappings)
