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


# ---- state blocks and workspaces ---------------------------------------------
# A launch keeps its work counters in a zeroed state block and the partial sums of
# the tiles it cuts along K in a workspace (include/dmoe.h).  ``get_arguments``
# hands out a state block (its address is the ``arguments_ptr`` of the reference's
# API) and the caller allocates the workspace, as experts.py:69-77 does; calls
# without them use a pair that this module keeps per device and stream.
#
# Footprint: a state block is 33 KB; a workspace of the size ``get_arguments``
# states is 2 x (compute units) x 256 KiB = 128 MiB on a 256-CU device.  Launches
# that follow each other on one stream can share one workspace (it carries nothing
# from one launch to the next), so layers should take ``shared_workspace`` rather
# than allocate one each; only launches that may overlap in time (graphs replayed
# on different streams) need workspaces of their own.

_STATE_BLOCKS = {}     # address -> the zeroed uint8 tensor behind an arguments_ptr
_DEFAULTS = {}         # (device index, stream handle) -> (state block, workspace)


def workspace_bytes(num_experts: int = 1) -> int:
    """Size of the workspace at which no launch is short of room (dmoe_gmm_workspace_bytes)."""
    need = _lib.c_size_t(0)
    _lib.call("dmoe_gmm_workspace_bytes", int(num_experts), _lib.ctypes.byref(need))
    return int(need.value)


def _new_state_block(device: torch.device) -> torch.Tensor:
    return torch.zeros(_lib.GMM_STATE_BYTES, dtype=torch.uint8, device=device)


def _default_pair(device: torch.device, stream: int):
    key = (device.index, stream)
    pair = _DEFAULTS.get(key)
    if pair is None:
        if torch.cuda.is_current_stream_capturing():
            # memory allocated and zero-filled inside a capture belongs to that graph's replays, and the state block
            # would be shared by every graph recorded on this capture stream
            raise RuntimeError("a grouped GEMM recorded into a graph needs its own state: pass the arguments_ptr of "
                               "get_arguments() (and a workspace), as MoEExperts does")
        with torch.cuda.device(device):
            state, ws = _new_state_block(device), torch.empty(workspace_bytes(), dtype=torch.uint8, device=device)
        pair = (state, ws)
        _DEFAULTS[key] = pair
    return pair


def shared_workspace(device: torch.device, stream: Optional[int] = None) -> torch.Tensor:
    """The workspace this module keeps for ``stream`` (default: the current stream) of
    ``device``: launches on one stream never overlap, so every layer that runs there can
    use it.  Created on first use, outside any graph capture."""
    device = torch.device(device)
    return _default_pair(device, _stream(device) if stream is None else stream)[1]


def _state_args(device: torch.device, workspace: Optional[torch.Tensor], arguments_ptr: Optional[int], stream: int,
                host_sizes: Optional[torch.Tensor] = None):
    """The trailing arguments of a dmoe_gmm* call: state block, workspace and its size, the host copy of the sizes
    (or NULL), the stream."""
    return (*_state_triple(device, workspace, arguments_ptr, stream),
            None if host_sizes is None else host_sizes.data_ptr(), stream)


def _host_sizes(batch_sizes: torch.Tensor, host_batch_sizes: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """The sizes in host memory, if the caller has them there: ``batch_sizes`` itself when it is a host tensor (what the
    reference passes off its CUTLASS path, engine.py:377-380,690-701), or the copy given beside a device tensor.
    The library then counts the tiles of a launch instead of estimating them (include/dmoe.h)."""
    h = host_batch_sizes if host_batch_sizes is not None else (batch_sizes if batch_sizes.device.type == "cpu" else None)
    if h is None or torch.cuda.is_current_stream_capturing():
        return None     # (a recorded launch is replayed on other batches: it keeps the plan that fits any of them)
    assert h.device.type == "cpu" and h.dim() == 1 and h.numel() == batch_sizes.numel()
    return h.to(dtype=torch.int64).contiguous()


def _state_triple(device, workspace, arguments_ptr, stream):
    if arguments_ptr is None and workspace is None:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("a grouped GEMM recorded into a graph needs its own state: pass the arguments_ptr of "
                               "get_arguments() (and a workspace), as MoEExperts does")
        state, ws = _default_pair(device, stream)
        return state.data_ptr(), ws.data_ptr(), ws.numel()
    if not arguments_ptr:
        raise ValueError("a caller-owned workspace needs the arguments_ptr that get_arguments returned with its size")
    if arguments_ptr not in _STATE_BLOCKS:
        raise ValueError(f"arguments_ptr {arguments_ptr:#x} does not come from get_arguments")
    if workspace is None:
        return arguments_ptr, None, 0
    assert workspace.dtype == torch.uint8 and workspace.is_contiguous() and workspace.device == device
    return arguments_ptr, workspace.data_ptr(), workspace.numel()


def release_arguments(arguments_ptr: int) -> None:
    """Gives back the state block behind an ``arguments_ptr`` of :func:`get_arguments`
    (no launch that uses it may be pending or recorded in a live graph)."""
    _STATE_BLOCKS.pop(arguments_ptr, None)


KERNEL_NAMES = {0: "dmoe::gmm_kernel", 1: "dmoe::gmm_direct_kernel", 2: "dmoe::gmm_tile256_kernel",
                3: "dmoe::gmm_tile256_fp8_kernel", 4: "dmoe::gmm_wave128_kernel", 5: "dmoe::gmm_wave128_fp8_kernel"}


def launch_plan(rows: int, num_experts: int, K: int, N: int, swiglu: bool = False, fp8: bool = False,
                workspace_bytes: int = 0, batch_sizes=None, trans_b: bool = False, sizes_passed: bool = False) -> dict:
    """What the library would launch for these shapes (its own answer, dmoe_gmm_plan):
    kernel, tile rows, wavefronts, workgroups; with ``batch_sizes`` (host values) also the
    tiles, how many of them are cut along K into how many pieces, and the work items.
    ``N`` is the number of result columns (``I`` for the swiglu form).  ``sizes_passed``: the
    launch is given the sizes in host memory too (``host_batch_sizes`` or a host ``batch_sizes``
    tensor) and decides tile rows and workgroups from them instead of from ``rows / E``."""
    out = (_lib.ctypes.c_int64 * 9)()
    sizes = None
    if batch_sizes is not None:
        vals = [int(v) for v in (batch_sizes.tolist() if torch.is_tensor(batch_sizes) else batch_sizes)]
        assert len(vals) == num_experts
        sizes = (_lib.ctypes.c_int64 * num_experts)(*vals)
    _lib.call("dmoe_gmm_plan", sizes, 1 if (sizes_passed and sizes is not None) else 0, int(rows), int(num_experts),
              int(K), int(N), 1 if trans_b else 0, 1 if swiglu else 0, _lib.FP8_E4M3 if fp8 else _lib.BF16,
              int(workspace_bytes), out)
    keys = ("kernel_id", "tile_rows", "wavefronts", "workgroups", "stage_k", "tiles", "cut_tiles", "pieces_per_cut_tile", "items")
    plan = dict(zip(keys, (int(v) for v in out)))
    plan["kernel"] = KERNEL_NAMES[plan["kernel_id"]]
    return plan


def _check_operands(a: torch.Tensor, b: torch.Tensor, dtype: torch.dtype) -> torch.device:
    if not a.is_cuda:
        raise RuntimeError("gmm needs device tensors; disagmoe_amd has no CPU fallback")
    assert a.dim() == 2 and b.dim() == 3, "a is [rows, K], b is [E, K, N] (or [E, N, K] with trans_b)"
    assert a.dtype == dtype and b.dtype == dtype, f"expected {dtype} operands, got {a.dtype} / {b.dtype}"
    assert a.is_contiguous() and b.is_contiguous()
    assert b.device == a.device
    return a.device


def gmm(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, trans_b: bool = False,
        c: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
        arguments_ptr: Optional[int] = None, host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``c[o_e:o_e+n_e] = a[o_e:o_e+n_e] @ b[e]`` (``b[e].T`` with ``trans_b``),
    bf16 operands, fp32 accumulation, bf16 result.  ``c`` (optional) is a
    preallocated ``[>= rows, N]`` buffer written in place and returned
    (experts.py:84,89); rows past ``sum(batch_sizes)`` are left untouched.
    ``workspace``/``arguments_ptr`` as :func:`gmm_with_arguments` takes them;
    without them the call uses the pair this module keeps for the current stream."""
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
                  1 if trans_b else 0, _lib.BF16, *_state_args(device, workspace, arguments_ptr, _stream(device),
                               _host_sizes(batch_sizes, host_batch_sizes)))
    return c


def gmm_swiglu(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, trans_b: bool = False,
               c: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
               arguments_ptr: Optional[int] = None, host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
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
                  1 if trans_b else 0, _lib.BF16, *_state_args(device, workspace, arguments_ptr, _stream(device),
                               _host_sizes(batch_sizes, host_batch_sizes)))
    return c


def gmm_swiglu_rows(x: torch.Tensor, row_token: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor,
                    c: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
                    arguments_ptr: Optional[int] = None, host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """:func:`gmm_swiglu` on rows fetched where they lie: row ``r`` of the product is row
    ``row_token[r]`` of ``x [T, K]`` (``ops.memory.route_tokens_with_sources``), so the permute
    in front of the FFN (engine.py:671-680) needs no launch.  ``b [E, K, 2I]``; returns
    ``[R, I]``.  Runs on tiles of 256 rows whatever the batch: see :func:`takes_rows`."""
    device = _check_operands(x, b, torch.bfloat16)
    T, K = x.shape
    E, Kb, N2 = b.shape
    assert Kb == K and N2 % 2 == 0 and batch_sizes.numel() == E
    assert row_token.dtype == torch.int32 and row_token.is_contiguous() and row_token.device == device
    rows, inter = row_token.numel(), N2 // 2
    if c is None:
        c = torch.empty((rows, inter), dtype=x.dtype, device=device)
    else:
        assert c.is_contiguous() and c.dtype == x.dtype and c.shape[1] == inter and c.shape[0] >= rows
    bs = _sizes_on_device(batch_sizes, device)
    with torch.cuda.device(device):
        _lib.call("dmoe_gmm_swiglu_rows", x.data_ptr(), row_token.data_ptr(), T, b.data_ptr(), c.data_ptr(), bs.data_ptr(),
                  rows, E, K, inter, _lib.BF16, *_state_args(device, workspace, arguments_ptr, _stream(device),
                               _host_sizes(batch_sizes, host_batch_sizes)))
    return c


def takes_rows(T: int, rows: int, num_experts: int, K: int, inter: int) -> bool:
    """Whether :func:`gmm_swiglu_rows` is the form to use for a gate-up projection of these
    shapes.  It always runs the 256-row tile kernel, so it needs the library to choose that
    kernel anyway (and the 32-bit row offsets to reach); and it has to beat the permute it
    saves: a tile that fetches 256 scattered rows pays for them on every stage (measured on
    MI355X: about 12 us per GB that the launch moves from the tokens to LDS, i.e. rows x K x 2
    bytes x column tiles; 92 us on 8192 x 4096 x 14336, 19 us on 49152 x 2048 x 1408, 3 us on
    512 x 4096 x 14336), against a permute kernel that moves (T + rows) x K x 2 bytes at about
    5.5 TB/s behind a launch of 7 us."""
    if K % 32 or T * K * 2 >= 1 << 32 or K * 2 * inter * 2 >= 1 << 32:
        return False
    if launch_plan(rows, num_experts, K, inter, swiglu=True, workspace_bytes=1 << 30)["kernel_id"] != 2:
        return False
    column_tiles = -(-inter // 128)
    fetch_us = 2.0 + 12.0 * (rows * K * 2.0 * column_tiles) / 1e9
    permute_us = 7.0 + (T + rows) * K * 2.0 / 5.5e6
    return fetch_us < permute_us


def get_arguments(num_experts: int, device: torch.device) -> Tuple[int, int]:
    """``(workspace_size, arguments_ptr)`` as in experts.py:69-72 and
    tests/ops/test_gemm.py:24.  ``arguments_ptr`` is the address of a zeroed state
    block on ``device`` that this module keeps alive (the launch's work counters
    live there); ``workspace_size`` is the size of the buffer the caller allocates
    (``torch.empty``, any contents) for the partial sums of tiles cut along K."""
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("get_arguments needs a HIP device; disagmoe_amd has no CPU fallback")
    with torch.cuda.device(device):
        block = _new_state_block(device)
    _STATE_BLOCKS[block.data_ptr()] = block
    return workspace_bytes(num_experts), block.data_ptr()


def gmm_with_arguments(a: torch.Tensor, b: torch.Tensor, batch_sizes: torch.Tensor, workspace: torch.Tensor,
                       arguments_ptr: int, **kwargs) -> torch.Tensor:
    """:func:`gmm` with the caller's workspace and the state block behind
    ``arguments_ptr`` (experts.py:74-77; tests/ops/test_gemm.py:30-36 call it
    repeatedly with one pair).  Same result as :func:`gmm`, bit for bit, for a
    workspace of the size ``get_arguments`` stated; nothing is allocated."""
    assert workspace.dtype == torch.uint8
    return gmm(a, b, batch_sizes, workspace=workspace, arguments_ptr=arguments_ptr, **kwargs)


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
            batch_sizes: torch.Tensor, c: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
            arguments_ptr: Optional[int] = None, host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``c = (a @ b[e].T) * a_scale[:, None] * b_scale[e][None, :]`` in bf16; ``a``
    fp8 ``[rows, K]``, ``b`` fp8 ``[E, N, K]``."""
    rows, K, E, N = _fp8_common(a, a_scale, b, b_scale)
    if c is None:
        c = torch.empty((rows, N), dtype=torch.bfloat16, device=a.device)
    bs = _sizes_on_device(batch_sizes, a.device)
    with torch.cuda.device(a.device):
        _lib.call("dmoe_gmm_fp8", a.data_ptr(), a_scale.data_ptr(), b.data_ptr(), b_scale.data_ptr(), c.data_ptr(),
                  bs.data_ptr(), rows, E, K, N,
                  *_state_args(a.device, workspace, arguments_ptr, _stream(a.device),
                               _host_sizes(batch_sizes, host_batch_sizes)))
    return c


def gmm_fp8_swiglu(a: torch.Tensor, a_scale: torch.Tensor, b: torch.Tensor, b_scale: torch.Tensor,
                   batch_sizes: torch.Tensor, c: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
                   arguments_ptr: Optional[int] = None, host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp8 gate-up projection with fused ``silu(gate) * up``; ``b`` fp8 ``[E, 2I,
    K]``; returns bf16 ``[rows, I]``."""
    rows, K, E, N2 = _fp8_common(a, a_scale, b, b_scale)
    assert N2 % 2 == 0
    if c is None:
        c = torch.empty((rows, N2 // 2), dtype=torch.bfloat16, device=a.device)
    bs = _sizes_on_device(batch_sizes, a.device)
    with torch.cuda.device(a.device):
        _lib.call("dmoe_gmm_fp8_swiglu", a.data_ptr(), a_scale.data_ptr(), b.data_ptr(), b_scale.data_ptr(),
                  c.data_ptr(), bs.data_ptr(), rows, E, K, N2 // 2,
                  *_state_args(a.device, workspace, arguments_ptr, _stream(a.device),
                               _host_sizes(batch_sizes, host_batch_sizes)))
    return c


def set_tile_variant(variant: int) -> None:
    """Tuning hook: 0 picks the tile by rows per expert (default); 1..3 force a
    tile shape.  For benchmarks only."""
    _lib.call("dmoe_gmm_tune", int(variant))
