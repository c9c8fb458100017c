"""fp8 (OCP e4m3fn, max 448) quantisation oracle.  Test infrastructure only.

The reference holds no fp8 code; the rules are the ones the benchmark
configuration states: weights per output channel ``scale = absmax / 448``,
activations per token ``scale = absmax / 448``, values cast with torch's
``float8_e4m3fn`` (round to nearest even, saturating at the scaled range).
"""
from __future__ import annotations

import torch

E4M3_MAX = 448.0


def _scale(absmax: torch.Tensor) -> torch.Tensor:
    s = absmax.float() / E4M3_MAX
    return torch.where(s > 0, s, torch.ones_like(s))


def quantize_rows(x: torch.Tensor):
    """Per-token: ``q[r, :] = fp8(x[r, :] / s[r])``, ``s[r] = absmax(x[r, :]) / 448``
    (1 for an all-zero row).  Returns ``(q [R, d] float8_e4m3fn, s [R] fp32)``."""
    xf = x.detach().cpu().float()
    s = _scale(xf.abs().amax(dim=1))
    q = (xf / s[:, None]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return q, s


def quantize_weight_channels(w: torch.Tensor):
    """Per output channel of ``w [E, K, N]``: ``s[e, n] = absmax_k |w[e, k, n]| / 448``.
    Returns ``(q [E, N, K] float8_e4m3fn -- K contiguous --, s [E, N] fp32)``."""
    wf = w.detach().cpu().float()
    s = _scale(wf.abs().amax(dim=1))
    q = (wf / s[:, None, :]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return q.transpose(1, 2).contiguous(), s


def dequantize_weight(q_nk: torch.Tensor, s: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """``[E, N, K]`` fp8 + ``[E, N]`` scales -> ``[E, K, N]`` in ``dtype``."""
    w = q_nk.detach().cpu().float() * s.detach().cpu().float()[:, :, None]
    return w.transpose(1, 2).contiguous().to(dtype)


def dequantize_rows(q: torch.Tensor, s: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    return (q.detach().cpu().float() * s.detach().cpu().float()[:, None]).to(dtype)


def moe_experts_forward_fp8(x: torch.Tensor, q13: torch.Tensor, s13: torch.Tensor, q2: torch.Tensor,
                            s2: torch.Tensor, batch_sizes) -> torch.Tensor:
    """The fp8 expert FFN with its quantisation points stated: rows of ``x`` and of
    the intermediate ``h`` are quantised per token, both GEMMs contract the
    de-quantised fp8 values in fp32, ``h`` and the result are rounded to bf16."""
    from . import ffn
    xq, xs = quantize_rows(x)
    w13 = dequantize_weight(q13, s13, torch.float32)
    inter = w13.shape[2] // 2
    up = ffn.gmm(dequantize_rows(xq, xs, torch.float32), w13, batch_sizes, out_dtype=torch.float32)
    h = (torch.nn.functional.silu(up[:, :inter]) * up[:, inter:]).to(torch.bfloat16)
    hq, hs = quantize_rows(h)
    out = ffn.gmm(dequantize_rows(hq, hs, torch.float32), dequantize_weight(q2, s2, torch.float32), batch_sizes,
                  out_dtype=torch.float32)
    return out.to(torch.bfloat16)
