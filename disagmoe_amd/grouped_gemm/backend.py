"""Grouped GEMM with the call signatures of ``grouped_gemm.backend`` as the
reference uses them (disagmoe/models/experts.py:3,69-77,84-94 and
tests/ops/test_gemm.py:15,24-31): ``gmm``, ``get_arguments``,
``gmm_with_arguments``; plus the fused gate-up form and the fp8 forms of the HIP
library.  Everything runs on the current stream of ``a``'s device.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import _lib


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _sizes_on_device(batch_sizes: torch.Tensor, device: torch.device) -> torch.Tensor:
    """``batch_sizes`` may live on the host or the device (the reference passes
    either, engine.py:377-380,690-701); the kernels read it on the device."""
    assert torch.is_tensor(batch_sizes) and batch_sizes.dim() == 1
    return batch_sizes.to(device=device, dtype=torch.int64, non_blocking=True).contiguous()


def _check_operands(a: torch.Tensor, b: torch.Tensor, dtype: torch.dtype) -> torch.device:
    if not a.is_cuda:
        raise RuntimeError("gmm needs device tensors; disagmoe_amd has no CPU fallback")
    assert a.dim() == 2 and b.dim() == 3, "a is [rows, K], b is [E, K, N] (or [E, N, K] with trans_b)"
    assert a.dtype == dtype and b.dtype == dtype, f"expected {dtype} operands, got {a.dtype} / {b.dtype}"
    assert a.is_contiguous() and b.is_contiguous()
    assert b.device == a.device
    return a.device


def gmm(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, trans_b: bool = False,
        c: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``c[o_e:o_e+n_e] = a[o_e:o_e+n_e] @ b[e]`` (``b[e].T`` with ``trans_b``),
    bf16 operands, fp32 accumulation, bf16 result.  ``c`` (optional) is a
    preallocated ``[>= rows, N]`` buffer written in place and returned
    (experts.py:84,89); rows past ``sum(batch_sizes)`` are left untouched."""
    device = _check_operands(a, b, torch.bfloat16)
    rows, K = a.shape
    E = b.shape[0]
    N = b.shape[1] if trans_b else b.shape[2]
    assert (b.shape[2] if trans_b else b.shape[1]) == K, "contraction length mismatch"
    assert batch_sizes.numel() == E
    if c is None:
        c = torch.empty((rows, N), dtype=a.dtype, device=device)
    else:
        assert c.is_contiguous() and c.dtype == a.dtype and c.device == device
        assert c.dim() == 2 and c.shape[1] == N and c.shape[0] >= rows
    bs = _sizes_on_device(batch_sizes, device)
    with torch.cuda.device(device):
        _lib.call("dmoe_gmm", a.data_ptr(), b.data_ptr(), c.data_ptr(), bs.data_ptr(), rows, E, K, N,
                  1 if trans_b else 0, _lib.BF16, _stream(device))
    return c


def gmm_swiglu(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, trans_b: bool = False,
               c: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Gate-up projection with the activation fused: ``silu(u[:, :I]) * u[:, I:]``
    for ``u = gmm(a, b)``, ``b [E, K, 2I]`` (``[E, 2I, K]`` with ``trans_b``);
    returns ``[rows, I]``.  The two steps of experts.py:92-93 in one kernel, taken
    on the fp32 accumulators with one rounding."""
    device = _check_operands(a, b, torch.bfloat16)
    rows, K = a.shape
    E = b.shape[0]
    N2 = b.shape[1] if trans_b else b.shape[2]
    assert (b.shape[2] if trans_b else b.shape[1]) == K, "contraction length mismatch"
    assert N2 % 2 == 0 and batch_sizes.numel() == E
    inter = N2 // 2
    if c is None:
        c = torch.empty((rows, inter), dtype=a.dtype, device=device)
    else:
        assert c.is_contiguous() and c.dtype == a.dtype and c.shape[1] == inter and c.shape[0] >= rows
    bs = _sizes_on_device(batch_sizes, device)
    with torch.cuda.device(device):
        _lib.call("dmoe_gmm_swiglu", a.data_ptr(), b.data_ptr(), c.data_ptr(), bs.data_ptr(), rows, E, K, inter,
                  1 if trans_b else 0, _lib.BF16, _stream(device))
    return c


def get_arguments(num_experts: int, device: torch.device) -> Tuple[int, int]:
    """``(workspace_size, arguments_ptr)`` as in experts.py:69-72.  The HIP
    scheduler builds its work list on the device inside the kernel, so the
    workspace is a token allocation and the handle is 0."""
    need = _lib.c_size_t(0)
    _lib.call("dmoe_gmm_workspace_bytes", int(num_experts), _lib.ctypes.byref(need))
    return int(need.value), 0


def gmm_with_arguments(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, workspace: torch.Tensor,
                       arguments_ptr: int, **kwargs) -> torch.Tensor:
    """Same result as :func:`gmm`, bit for bit, with a caller-owned workspace
    (experts.py:74-77; tests/ops/test_gemm.py:30-36 call it repeatedly with one
    workspace).  Neither form allocates scheduler state on the host."""
    size, _ = get_arguments(b.shape[0], a.device)
    assert workspace.dtype == torch.uint8 and workspace.numel() >= size
    return gmm(a, b, batch_sizes, **kwargs)


# ---- fp8 (e4m3fn) forms: no counterpart in the reference --------------------

def quantize_rows(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row fp8 quantisation on the device: ``(q [rows, d] float8_e4m3fn,
    scale [rows] fp32)`` with ``scale = absmax / 448``."""
    assert x.is_cuda and x.dim() == 2 and x.is_contiguous() and x.dtype in (torch.bfloat16, torch.float16)
    rows, d = x.shape
    q = torch.empty((rows, d), dtype=torch.float8_e4m3fn, device=x.device)
    s = torch.empty(rows, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.call("dmoe_quant_rows", x.data_ptr(), q.data_ptr(), s.data_ptr(), rows, d,
                  _lib.BF16 if x.dtype == torch.bfloat16 else _lib.FP16, _stream(x.device))
    return q, s


def quantize_weight(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Offline weight quantisation: ``w [E, K, N]`` -> ``(q [E, N, K]
    float8_e4m3fn, scale [E, N] fp32)``, per output channel ``scale = absmax_k /
    448``.  An output channel is a row of ``w[e].T``, so the row quantiser does
    the arithmetic."""
    assert w.is_cuda and w.dim() == 3
    E, K, N = w.shape
    q = torch.empty((E, N, K), dtype=torch.float8_e4m3fn, device=w.device)
    s = torch.empty((E, N), dtype=torch.float32, device=w.device)
    for e in range(E):
        qe, se = quantize_rows(w[e].t().contiguous())
        q[e] = qe
        s[e] = se
    return q, s


def _fp8_common(a, a_scale, b, b_scale):
    assert a.is_cuda and a.dtype == torch.float8_e4m3fn and b.dtype == torch.float8_e4m3fn
    assert a.dim() == 2 and b.dim() == 3 and a.is_contiguous() and b.is_contiguous()
    rows, K = a.shape
    E, N, Kb = b.shape
    assert Kb == K
    assert a_scale.dtype == torch.float32 and a_scale.numel() == rows and a_scale.is_contiguous()
    assert b_scale.dtype == torch.float32 and b_scale.shape == (E, N) and b_scale.is_contiguous()
    return rows, K, E, N


def gmm_fp8(a: torch.Tensor, a_scale: torch.Tensor, b: torch.Tensor, b_scale: torch.Tensor,
            batch_sizes: torch.Tensor, c: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``c = (a @ b[e].T) * a_scale[:, None] * b_scale[e][None, :]`` in bf16; ``a``
    fp8 ``[rows, K]``, ``b`` fp8 ``[E, N, K]``."""
    rows, K, E, N = _fp8_common(a, a_scale, b, b_scale)
    if c is None:
        c = torch.empty((rows, N), dtype=torch.bfloat16, device=a.device)
    bs = _sizes_on_device(batch_sizes, a.device)
    with torch.cuda.device(a.device):
        _lib.call("dmoe_gmm_fp8", a.data_ptr(), a_scale.data_ptr(), b.data_ptr(), b_scale.data_ptr(), c.data_ptr(),
                  bs.data_ptr(), rows, E, K, N, _stream(a.device))
    return c


def gmm_fp8_swiglu(a: torch.Tensor, a_scale: torch.Tensor, b: torch.Tensor, b_scale: torch.Tensor,
                   batch_sizes: torch.Tensor, c: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp8 gate-up projection with fused ``silu(gate) * up``; ``b`` fp8 ``[E, 2I,
    K]``; returns bf16 ``[rows, I]``."""
    rows, K, E, N2 = _fp8_common(a, a_scale, b, b_scale)
    assert N2 % 2 == 0
    if c is None:
        c = torch.empty((rows, N2 // 2), dtype=torch.bfloat16, device=a.device)
    bs = _sizes_on_device(batch_sizes, a.device)
    with torch.cuda.device(a.device):
        _lib.call("dmoe_gmm_fp8_swiglu", a.data_ptr(), a_scale.data_ptr(), b.data_ptr(), b_scale.data_ptr(),
                  c.data_ptr(), bs.data_ptr(), rows, E, K, N2 // 2, _stream(a.device))
    return c


def set_tile_variant(variant: int) -> None:
    """Tuning hook: 0 picks the tile by rows per expert (default); 1..3 force a
    tile shape.  For benchmarks only."""
    _lib.call("dmoe_gmm_tune", int(variant))
