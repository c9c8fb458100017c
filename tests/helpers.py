"""Shared helpers of the GPU parity tests."""
import sys

import torch

#: stated tolerances: max|out - ref| / max|ref|
TOL_BF16 = 1e-2   # bf16 GEMM / FFN / combine against the fp32-accumulated oracle
TOL_FP8 = 3e-2    # fp8 path against the bf16 oracle on de-quantised weights


def dev() -> torch.device:
    return torch.device("cuda", 0)


def announce(**case) -> None:
    """Name the case before anything is launched, so that a fault can be traced."""
    print("[case] " + " ".join(f"{k}={v}" for k, v in case.items()), flush=True)
    sys.stdout.flush()


def max_rel_err(out: torch.Tensor, ref: torch.Tensor) -> float:
    ref64 = ref.detach().cpu().double()
    den = ref64.abs().max().item()
    num = (out.detach().cpu().double() - ref64).abs().max().item()
    return num / den if den > 0 else num


def ragged_sizes(E: int, R: int, seed: int, empty_every: int = 3):
    """Random split of R rows over E experts with some empty experts."""
    g = torch.Generator().manual_seed(seed)
    w = torch.rand(E, generator=g)
    for e in range(E):
        if empty_every and e % empty_every == 1:
            w[e] = 0
    if w.sum() == 0:
        w[0] = 1
    sizes = torch.floor(w / w.sum() * R).long()
    sizes[int(torch.argmax(w))] += R - int(sizes.sum())
    assert int(sizes.sum()) == R and (sizes >= 0).all()
    return sizes
