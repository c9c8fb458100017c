"""Floating-point oracle: grouped GEMM, SwiGLU expert FFN, gate-weighted combine.

Test infrastructure only.  All contractions accumulate in fp32 (or fp64 when
asked) on bf16/fp16 inputs and round ONCE at the end, which is the result the
tolerance of the HIP kernels is stated against.
"""
from __future__ import annotations

from typing import Optional

import torch


def _sizes(batch_sizes) -> list:
    if torch.is_tensor(batch_sizes):
        return [int(v) for v in batch_sizes.detach().cpu().reshape(-1).tolist()]
    return [int(v) for v in batch_sizes]


def gmm(a: torch.Tensor, b: torch.Tensor, batch_sizes, trans_b: bool = False,
        c: Optional[torch.Tensor] = None, acc_dtype: torch.dtype = torch.float32,
        out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Grouped GEMM: ``C[o_e:o_e+n_e] = A[o_e:o_e+n_e] @ B[e]`` (``B[e].T`` with
    ``trans_b``), ``o_e`` the running sum of ``batch_sizes``; experts with zero
    rows contribute nothing; rows past ``sum(batch_sizes)`` are left untouched.

    The implementation (third-party ``grouped_gemm.backend.gmm``) is absent from
    the reference tree; this follows its call sites
    (disagmoe/models/experts.py:84,89,92,94; tests/ops/test_gemm.py:15)."""
    a = a.detach().cpu()
    b = b.detach().cpu()
    sizes = _sizes(batch_sizes)
    E = b.shape[0]
    assert len(sizes) == E
    N = b.shape[1] if trans_b else b.shape[2]
    out_dtype = out_dtype or a.dtype
    if c is None:
        c = torch.zeros((a.shape[0], N), dtype=out_dtype)
    o = 0
    for e, n in enumerate(sizes):
        if n == 0:
            continue
        be = b[e].to(acc_dtype)
        if trans_b:
            be = be.t()
        c[o:o + n] = (a[o:o + n].to(acc_dtype) @ be).to(c.dtype)
        o += n
    return c


def moe_experts_forward(hiddens: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, batch_sizes,
                        acc_dtype: torch.dtype = torch.float32,
                        out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Per-expert SwiGLU FFN with a single final rounding.

    Math of disagmoe/models/experts.py:92-96 (grouped form) and :115-116 (serial
    form): ``silu(x_e @ w1[e]) * (x_e @ w3[e]) @ w2[e]`` with
    ``w1 = w13[..., :I]`` (gate) and ``w3 = w13[..., I:]`` (up) (:42-47)."""
    hiddens = hiddens.detach().cpu()
    w13 = w13.detach().cpu()
    w2 = w2.detach().cpu()
    sizes = _sizes(batch_sizes)
    I = w2.shape[1]
    out_dtype = out_dtype or hiddens.dtype
    out = torch.zeros((hiddens.shape[0], w2.shape[2]), dtype=out_dtype)
    o = 0
    for e, n in enumerate(sizes):
        if n == 0:
            continue
        x = hiddens[o:o + n].to(acc_dtype)
        up = x @ w13[e].to(acc_dtype)
        h = torch.nn.functional.silu(up[:, :I]) * up[:, I:]
        out[o:o + n] = (h @ w2[e].to(acc_dtype)).to(out_dtype)
        o += n
    return out


def moe_experts_forward_reference_rounding(hiddens, w13, w2, batch_sizes) -> torch.Tensor:
    """Same FFN with the reference's intermediate roundings: the gate-up result,
    SiLU, the product and the down result are each stored in the input dtype
    (disagmoe/models/experts.py:92-94).  Used to show that the difference
    between the two rounding schedules sits inside the stated tolerance."""
    dt = hiddens.dtype
    I = w2.shape[1]
    up = gmm(hiddens, w13, batch_sizes)
    act = torch.nn.functional.silu(up[:, :I].float()).to(dt)
    h = (act.float() * up[:, I:].float()).to(dt)
    return gmm(h, w2, batch_sizes)


def combine(y: torch.Tensor, mappings, weights: torch.Tensor, acc_dtype=torch.float32) -> torch.Tensor:
    """Gate-weighted unpermute back to token order with one rounding:
    ``out[i] = sum_j w[i, j] * y[mappings[i*k + j]]``.

    Single-GPU statement of disagmoe/frontend/engine.py:726-734 (scale by the
    top-k weights, permute back) followed by :624-628 (sum of the k copies)."""
    y = y.detach().cpu()
    w = weights.detach().cpu().to(acc_dtype)
    T, k = w.shape
    m = torch.as_tensor(mappings, dtype=torch.int64).reshape(T, k)
    acc = torch.zeros((T, y.shape[1]), dtype=acc_dtype)
    for j in range(k):
        acc += w[:, j:j + 1] * y[m[:, j]].to(acc_dtype)
    return acc.to(y.dtype)


def combine_reference_chain(y: torch.Tensor, mappings, weights: torch.Tensor) -> torch.Tensor:
    """The reference's own rounding chain, bit for bit: weights cast to the row
    dtype (engine.py:726), ``y * w`` rounded to the row dtype (:732), then the
    copies added left to right, each sum rounded (:627 for k = 2; extended to
    k > 2 in the same order)."""
    y = y.detach().cpu()
    dt = y.dtype
    T, k = weights.shape
    m = torch.as_tensor(mappings, dtype=torch.int64).reshape(T, k)
    w = weights.detach().cpu().to(dt)
    acc = y[m[:, 0]] * w[:, 0:1]
    for j in range(1, k):
        acc = acc + y[m[:, j]] * w[:, j:j + 1]
    return acc


def max_rel_err(out: torch.Tensor, ref: torch.Tensor) -> float:
    """``max|out - ref| / max|ref|`` in fp64: the error measure every floating
    point tolerance in the tests is stated in."""
    ref64 = ref.detach().cpu().double()
    den = ref64.abs().max().item()
    num = (out.detach().cpu().double() - ref64).abs().max().item()
    return num / den if den > 0 else num
