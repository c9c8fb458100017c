"""Routing and row-movement operators, same names and argument meaning as the
reference's ``disagmoe/ops/memory.py`` (get_mappings_from_exp_ids :34,
get_mappings_from_exp_ids_cuda :57, permute_tokens_triton :72,
permute_tokens_cuda :94), computed by the HIP kernels of libdmoe_hip.so on the
current stream of the tensors' device.  Additional device-resident entry points
(``route_tokens``, ``gather_rows``, ``gather_row_ptrs``, ``combine_tokens``)
expose the rest of the C ABI.
"""
from __future__ import annotations

from typing import List, Optional, Tuple, Union

import torch

from .. import _lib

_ROW_DTYPES = {torch.bfloat16: _lib.BF16, torch.float16: _lib.FP16}
if hasattr(torch, "float8_e4m3fn"):
    _ROW_DTYPES[torch.float8_e4m3fn] = _lib.FP8_E4M3
_INT_TYPES = {torch.int32: _lib.I32, torch.int64: _lib.I64}


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _device_of(t) -> torch.device:
    if torch.is_tensor(t) and t.is_cuda:
        return t.device
    if not torch.cuda.is_available():
        raise RuntimeError("disagmoe_amd operators need a HIP device; there is no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


def _row_dtype(t: torch.Tensor) -> int:
    try:
        return _ROW_DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported row dtype {t.dtype}; expected bf16, fp16 or float8_e4m3fn") from None


def _index_tensor(values, device: torch.device, default_dtype: torch.dtype) -> torch.Tensor:
    """Mappings given as a list are uploaded as the reference does
    (memory.py:96-99); tensors keep their integer type."""
    if not torch.is_tensor(values):
        values = torch.tensor(values, dtype=default_dtype, device=device)
    values = values.to(device)
    if values.dtype not in _INT_TYPES:
        raise TypeError(f"index tensor must be int32 or int64, got {values.dtype}")
    return values.contiguous().view(-1)


def route_tokens(exp_ids: torch.Tensor, num_experts: int, order: int = _lib.ORDER_REFERENCE,
                 map_dtype: torch.dtype = torch.int64) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Device-resident routing: ``(mappings [R], batch_sizes [E] int64, offsets
    [E+1] int64)`` from the flat expert ids (token-major ``t = i*k + j``).  No
    host synchronisation.  ``order`` selects the reference's host order
    (descending ``t`` inside an expert, memory.py:50-52) or the stable ascending
    order of its device variant (:57-69)."""
    device = _device_of(exp_ids)
    ids = exp_ids.to(device).contiguous().view(-1)
    if ids.dtype not in _INT_TYPES:
        raise TypeError(f"expert ids must be int32 or int64, got {ids.dtype}")
    R = ids.numel()
    with torch.cuda.device(device):
        need = _lib.c_size_t(0)
        _lib.call("dmoe_route_scratch_bytes", R, num_experts, _lib.ctypes.byref(need))
        mappings = torch.empty(R, dtype=map_dtype, device=device)
        batch_sizes = torch.empty(num_experts, dtype=torch.int64, device=device)
        offsets = torch.empty(num_experts + 1, dtype=torch.int64, device=device)
        scratch = torch.empty(max(need.value, 1), dtype=torch.uint8, device=device)
        _lib.call("dmoe_route", ids.data_ptr(), _INT_TYPES[ids.dtype], R, num_experts, order, mappings.data_ptr(),
                  _INT_TYPES[map_dtype], batch_sizes.data_ptr(), offsets.data_ptr(), scratch.data_ptr(),
                  scratch.numel(), _stream(device))
    return mappings, batch_sizes, offsets


def route_tokens_with_sources(topk_ids: torch.Tensor, num_experts: int, order: int = _lib.ORDER_REFERENCE,
                              map_dtype: torch.dtype = torch.int64):
    """:func:`route_tokens` of ``topk_ids [T, k]`` that also returns ``row_token [R]`` int32, the token
    whose row stands at each place of the expert-sorted order (``row_token[mappings[i*k + j]] = i``):
    what ``grouped_gemm.backend.gmm_swiglu_rows`` fetches its rows by."""
    device = _device_of(topk_ids)
    assert topk_ids.dim() == 2
    k = topk_ids.shape[1]
    ids = topk_ids.to(device).contiguous().view(-1)
    if ids.dtype not in _INT_TYPES:
        raise TypeError(f"expert ids must be int32 or int64, got {ids.dtype}")
    R = ids.numel()
    with torch.cuda.device(device):
        need = _lib.c_size_t(0)
        _lib.call("dmoe_route_scratch_bytes", R, num_experts, _lib.ctypes.byref(need))
        mappings = torch.empty(R, dtype=map_dtype, device=device)
        batch_sizes = torch.empty(num_experts, dtype=torch.int64, device=device)
        offsets = torch.empty(num_experts + 1, dtype=torch.int64, device=device)
        row_token = torch.empty(R, dtype=torch.int32, device=device)
        scratch = torch.empty(max(need.value, 1), dtype=torch.uint8, device=device)
        _lib.call("dmoe_route_sources", ids.data_ptr(), _INT_TYPES[ids.dtype], R, num_experts, order, mappings.data_ptr(),
                  _INT_TYPES[map_dtype], batch_sizes.data_ptr(), offsets.data_ptr(), k, row_token.data_ptr(),
                  scratch.data_ptr(), scratch.numel(), _stream(device))
    return mappings, batch_sizes, offsets, row_token


def get_mappings_from_exp_ids(exp_ids: Union[torch.Tensor, List[int]], num_experts: int) -> Tuple[List[int], List[int]]:
    """Reference signature and return types (memory.py:34-54): Python lists
    ``(mappings, exp_cnt)``.  Ids that live on the host (a list, as the reference's
    engine passes at engine.py:675, or a CPU tensor) are sorted on the host by the
    library's ``dmoe_host_mappings``: no upload, no kernel, no read-back.  Ids on the
    device are sorted there and the lists read back (the reference's ``.tolist()``
    is the same sync point)."""
    if torch.is_tensor(exp_ids) and exp_ids.is_cuda:
        ids = exp_ids.reshape(-1)
        if ids.numel() and (int(ids.min()) < 0 or int(ids.max()) >= num_experts):
            raise IndexError("list index out of range")  # what the reference's host loop raises
        mappings, batch_sizes, _ = route_tokens(ids, num_experts, _lib.ORDER_REFERENCE)
        return mappings.tolist(), batch_sizes.tolist()
    from .metadata import host_mappings
    ids = exp_ids.reshape(-1).tolist() if torch.is_tensor(exp_ids) else list(exp_ids)
    try:
        return host_mappings(ids, num_experts)
    except _lib.DmoeError as err:
        if err.code == _lib.ERR_ARG:
            raise IndexError("list index out of range") from None
        raise


def get_mappings_from_exp_ids_cuda(exp_ids: torch.Tensor, num_experts: int):
    """Reference signature (memory.py:57-69): ``(int32 mappings on the ids'
    device, [])``, rows of an expert in ascending order of ``t``."""
    assert isinstance(exp_ids, torch.Tensor)
    mappings, _, _ = route_tokens(exp_ids, num_experts, _lib.ORDER_STABLE, map_dtype=torch.int32)
    return mappings, []


def permute_tokens_cuda(tokens: torch.Tensor, mappings: Union[torch.Tensor, List[int]],
                        row_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[mappings[t], :] = tokens[t // k, :]`` with ``k = len(mappings) //
    tokens.shape[0]`` (memory.py:94-102, csrc/cuda_ops/permute.cu:86-112).
    ``row_scale`` (optional ``[R]`` or ``[R, 1]``, row dtype) multiplies routed row
    ``t`` on the way: the ``output * topk_weights`` of engine.py:731-732."""
    assert tokens.dim() == 2
    assert tokens.is_contiguous()
    device = _device_of(tokens)
    tokens = tokens.to(device)
    m = _index_tensor(mappings, device, torch.int64)
    T, d = tokens.shape
    R = m.numel()
    assert T == 0 or R % T == 0, f"{R} mappings for {T} tokens"
    out = torch.empty((R, d), dtype=tokens.dtype, device=device)
    scale_ptr = None
    if row_scale is not None:
        row_scale = row_scale.to(device=device, dtype=tokens.dtype).contiguous().view(-1)
        assert row_scale.numel() == R
        scale_ptr = row_scale.data_ptr()
    with torch.cuda.device(device):
        _lib.call("dmoe_permute", tokens.data_ptr(), out.data_ptr(), m.data_ptr(), _INT_TYPES[m.dtype], T, R, d,
                  _row_dtype(tokens), scale_ptr, _stream(device))
    return out


def permute_quantize(tokens: torch.Tensor, mappings: Union[torch.Tensor, List[int]]):
    """``permute_tokens_cuda`` and the per-row fp8 quantisation in one kernel (no counterpart in the
    reference, which has no fp8 path): ``(q [R, d] float8_e4m3fn, scale [R] fp32)`` with
    ``q[mappings[t]] = fp8(tokens[t // k] / scale)``, ``scale = absmax / 448``.  Same bits as
    ``quantize_rows(permute_tokens_cuda(tokens, mappings))``; the bf16 copy of the routed rows is never written."""
    assert tokens.dim() == 2 and tokens.is_contiguous() and tokens.dtype in (torch.bfloat16, torch.float16)
    device = _device_of(tokens)
    tokens = tokens.to(device)
    m = _index_tensor(mappings, device, torch.int64)
    T, d = tokens.shape
    R = m.numel()
    assert T == 0 or R % T == 0, f"{R} mappings for {T} tokens"
    q = torch.empty((R, d), dtype=torch.float8_e4m3fn, device=device)
    scale = torch.empty(R, dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        _lib.call("dmoe_permute_quant", tokens.data_ptr(), q.data_ptr(), scale.data_ptr(), m.data_ptr(),
                  _INT_TYPES[m.dtype], T, R, d, _row_dtype(tokens), _stream(device))
    return q, scale


def permute_tokens_triton(tokens: torch.Tensor, mappings: Union[torch.Tensor, List[int]]) -> torch.Tensor:
    """Reference name kept (memory.py:72-91): the top-1 permute with int32 or
    int64 mappings.  Served by the same HIP kernel; there is no Triton here."""
    assert len(tokens.shape) == 2
    assert tokens.is_contiguous()
    device = _device_of(tokens)
    m = _index_tensor(mappings, device, torch.int32)
    assert m.numel() == tokens.shape[0]
    return permute_tokens_cuda(tokens, m)


def gather_rows(tokens: torch.Tensor, index: Union[torch.Tensor, List[int]]) -> torch.Tensor:
    """``out[t, :] = tokens[index[t], :]`` (index form of gather_tokens_cuda,
    csrc/cuda_ops/permute.cu:144-152; ``torch.index_select`` semantics)."""
    assert tokens.dim() == 2 and tokens.is_contiguous()
    device = _device_of(tokens)
    idx = _index_tensor(index, device, torch.int64)
    out = torch.empty((idx.numel(), tokens.shape[1]), dtype=tokens.dtype, device=device)
    with torch.cuda.device(device):
        _lib.call("dmoe_gather_rows", tokens.data_ptr(), out.data_ptr(), idx.data_ptr(), _INT_TYPES[idx.dtype],
                  idx.numel(), tokens.shape[0], tokens.shape[1], _row_dtype(tokens), _stream(device))
    return out


def gather_row_ptrs(row_ptrs: torch.Tensor, hidden_size: int, dtype: torch.dtype,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[t, :] = *row_ptrs[t]``: the expert-side merge of several received
    slabs (TensorBatch::merge, csrc/include/datatypes.hpp:508-549) with the
    pointer table already on the device (int64/uint64 ``[N]``)."""
    assert row_ptrs.is_cuda and row_ptrs.dtype in (torch.int64, torch.uint64)
    device = row_ptrs.device
    n = row_ptrs.numel()
    if out is None:
        out = torch.empty((n, hidden_size), dtype=dtype, device=device)
    assert out.is_contiguous() and out.shape == (n, hidden_size) and out.dtype == dtype
    with torch.cuda.device(device):
        _lib.call("dmoe_gather_ptrs", row_ptrs.data_ptr(), out.data_ptr(), n, hidden_size, _row_dtype(out),
                  _stream(device))
    return out


def combine_tokens(expert_out: torch.Tensor, mappings: Union[torch.Tensor, List[int]], topk_weights: torch.Tensor,
                   reference_rounding: bool = False) -> torch.Tensor:
    """Gate-weighted unpermute back to token order:
    ``out[i] = sum_j topk_weights[i, j] * expert_out[mappings[i*k + j]]``.

    One kernel for the reference's three steps (scale engine.py:731-732, return
    permute :734, top-k sum :624-628).  fp32 accumulation with one rounding, or
    the reference's own rounding chain with ``reference_rounding=True``."""
    assert expert_out.dim() == 2 and expert_out.is_contiguous()
    device = _device_of(expert_out)
    T, k = topk_weights.shape
    m = _index_tensor(mappings, device, torch.int64)
    assert m.numel() == T * k == expert_out.shape[0]
    w = topk_weights.to(device=device, dtype=torch.float32).contiguous()
    out = torch.empty((T, expert_out.shape[1]), dtype=expert_out.dtype, device=device)
    mode = _lib.COMBINE_REFERENCE if reference_rounding else _lib.COMBINE_FP32
    with torch.cuda.device(device):
        _lib.call("dmoe_combine", expert_out.data_ptr(), m.data_ptr(), _INT_TYPES[m.dtype], w.data_ptr(),
                  out.data_ptr(), T, k, expert_out.shape[1], _row_dtype(expert_out), mode, _stream(device))
    return out
