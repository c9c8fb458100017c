"""Expert layer modules with the constructor, parameters and ``forward`` of the
reference's ``disagmoe/models/experts.py`` (MoEExperts :9-96, MoEExpertsSerial
:98-120), running on the HIP grouped GEMM.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..grouped_gemm import backend as gg

MAX_BATCH_SIZE = 256  # disagmoe/utils/constants.py:20-22


class _GemmState:
    """State of a layer's grouped-GEMM launches (experts.py:69-77: ``get_arguments`` and the workspace).

    The 33 KB state block (work counters) is the layer's own: a recorded graph of the layer then shares
    its scheduler state with no other launch.  The workspace (fp32 partial sums of tiles cut along K,
    128 MiB on a 256-CU device) carries nothing from one launch to the next, so eager launches use the
    one the backend keeps for the stream they run on, shared by every layer that runs there.  A layer
    gets a workspace of its own when one is passed in (``workspace=``; the caller may hand the same
    tensor to layers whose launches never overlap in time), with ``own_workspace=True``, or when it
    is recorded into a graph without one (replays may run beside anything; the tensor then comes from
    the graph's memory pool and stays with the layer)."""

    def _init_gemm_state(self, device, workspace: Optional[torch.Tensor] = None, own_workspace: bool = False):
        self.workspace_size, self.arguments_ptr = gg.get_arguments(self.num_experts, device)
        self._gemm_device = torch.device(device)
        self.workspace = workspace
        if workspace is None and own_workspace:
            self.workspace = torch.empty([self.workspace_size], dtype=torch.uint8, device=device)

    def _gemm_state(self) -> dict:
        ws = self.workspace
        if ws is None:
            if torch.cuda.is_current_stream_capturing():
                ws = self.workspace = torch.empty([self.workspace_size], dtype=torch.uint8, device=self._gemm_device)
            else:
                ws = gg.shared_workspace(self._gemm_device)
        return dict(workspace=ws, arguments_ptr=self.arguments_ptr)

    def __del__(self):
        ptr = getattr(self, "arguments_ptr", None)
        if ptr is not None:
            gg.release_arguments(ptr)


class MoEExperts(_GemmState, torch.nn.Module):
    """Fused-w13 SwiGLU experts.

    Parameters (experts.py:42-55): ``w13_weight [E, d, 2I]`` (gate = columns
    ``[0, I)``, up = ``[I, 2I)``) and ``w2_weight [E, I, d]``, bf16, no grad.
    ``forward(bs, hiddens, batch_sizes)`` (:81-96) maps expert-sorted rows
    ``[R, d]`` to ``[R, d]``.
    """

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, tp_size: int = 1,
                 enable_cutlass_cache: bool = True, max_batch_size: int = MAX_BATCH_SIZE,
                 device: Optional[torch.device] = None, init_std: float = 1.0,
                 workspace: Optional[torch.Tensor] = None, own_workspace: bool = False):
        super().__init__()
        self._workspace_arg, self._own_workspace_arg = workspace, own_workspace
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.num_experts = num_experts
        self.tp_size = tp_size
        assert tp_size == 1, "Not implemented TP for experts yet"  # experts.py:24
        self._device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        self._init_std = init_std
        self.create_weights(enable_cutlass_cache=enable_cutlass_cache, max_batch_size=max_batch_size)
        self.gmm = gg.gmm
        self.gmm_cache_max_batch_size = max_batch_size

    def create_weights(self, params_dtype: Optional[torch.dtype] = None, enable_cutlass_cache: bool = False,
                       max_batch_size: int = MAX_BATCH_SIZE):
        params_dtype = params_dtype or torch.bfloat16
        dev = self._device

        def randn(*shape):
            # generated on the device expert by expert: the full fp32 tensor never exists
            w = torch.empty(shape, dtype=params_dtype, device=dev)
            for e in range(shape[0]):
                w[e] = (torch.randn(shape[1:], dtype=torch.float32, device=dev) * self._init_std).to(params_dtype)
            return w

        self.w13_weight = torch.nn.Parameter(randn(self.num_experts, self.hidden_size, self.intermediate_size * 2),
                                             requires_grad=False)
        self.w2_weight = torch.nn.Parameter(randn(self.num_experts, self.intermediate_size, self.hidden_size),
                                            requires_grad=False)
        self.act_fn = torch.nn.SiLU(inplace=True)
        # static buffers for batches below max_batch_size (experts.py:66-67): forward does not allocate
        self.cache_up = torch.empty((max_batch_size, self.intermediate_size), dtype=params_dtype, device=dev)
        self.cache_down = torch.empty((max_batch_size, self.hidden_size), dtype=params_dtype, device=dev)
        self.enable_cache = enable_cutlass_cache
        # state block of this layer's launches and where their workspace comes from (experts.py:69-77)
        self._init_gemm_state(dev, getattr(self, "_workspace_arg", None), getattr(self, "_own_workspace_arg", False))

    def forward(self, bs: int, hiddens: torch.Tensor, batch_sizes: torch.Tensor,
                host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``gmm(silu(u[:, :I]) * u[:, I:], w2)`` with ``u = gmm(hiddens, w13)``
        (experts.py:92-96); gate-up, SiLU and the product are one kernel.  Below
        ``max_batch_size`` rows the static buffers are used (the reference's
        cached branch, :83-90).  ``batch_sizes`` on the host (what the reference passes
        off its CUTLASS path) or ``host_batch_sizes`` beside a device tensor let the
        library count the launch's tiles instead of estimating them."""
        ws = dict(self._gemm_state(), host_batch_sizes=host_batch_sizes)
        if self.enable_cache and bs <= self.gmm_cache_max_batch_size and hiddens.shape[0] <= self.cache_up.shape[0]:
            h = gg.gmm_swiglu(hiddens, self.w13_weight, batch_sizes, c=self.cache_up, **ws)[:hiddens.shape[0]]
            return gg.gmm(h, self.w2_weight, batch_sizes, c=self.cache_down, **ws)[:hiddens.shape[0]]
        h = gg.gmm_swiglu(hiddens, self.w13_weight, batch_sizes, **ws)
        return gg.gmm(h, self.w2_weight, batch_sizes, **ws)

    def forward_rows(self, x: torch.Tensor, row_token: torch.Tensor, batch_sizes: torch.Tensor,
                     host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
        """:meth:`forward` on rows that are fetched where they lie: ``x [T, d]`` in token order
        and ``row_token [R]`` (``ops.memory.route_tokens_with_sources``) instead of the
        expert-sorted copy ``hiddens [R, d]``: the gate-up kernel reads row ``row_token[r]`` of
        ``x``, and the permute in front of the FFN (engine.py:671-680) is never launched."""
        ws = dict(self._gemm_state(), host_batch_sizes=host_batch_sizes)
        h = gg.gmm_swiglu_rows(x, row_token, self.w13_weight, batch_sizes, **ws)
        return gg.gmm(h, self.w2_weight, batch_sizes, **ws)

    def takes_rows(self, T: int, rows: int) -> bool:
        """Whether :meth:`forward_rows` is the faster form for a batch of these sizes."""
        return gg.takes_rows(T, rows, self.num_experts, self.hidden_size, self.intermediate_size)

    def forward_unfused(self, bs: int, hiddens: torch.Tensor, batch_sizes: torch.Tensor) -> torch.Tensor:
        """The reference's own schedule, statement by statement (experts.py:92-94):
        the gate-up result, SiLU and the product are each rounded to bf16."""
        ws = self._gemm_state()
        up = self.gmm(hiddens, self.w13_weight, batch_sizes, **ws)
        up = self.act_fn(up[:, :self.intermediate_size]) * up[:, self.intermediate_size:]
        return self.gmm(up, self.w2_weight, batch_sizes, **ws)


class MoEExpertsSerial(MoEExperts):
    """Per-expert loop of plain library matmuls (experts.py:98-120; selected by
    ``enable_grouped_gemm=False``, executor.py:353).  The reference reads
    ``w1_weight``/``w3_weight`` that it never creates; here they are the two
    halves of ``w13_weight`` as the layout comment (:42-47) defines them.  Reads
    ``batch_sizes`` on the host (one synchronisation), like the reference's loop."""

    def __init__(self, hidden_size, intermediate_size, num_experts, tp_size=1, max_batch_size: int = MAX_BATCH_SIZE,
                 **kwargs):
        super().__init__(hidden_size, intermediate_size, num_experts, tp_size, enable_cutlass_cache=False,
                         max_batch_size=max_batch_size, **kwargs)

    def forward(self, num_tokens: int, hiddens: torch.Tensor, batch_sizes: torch.Tensor,
                host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
        inter = self.intermediate_size
        results = []
        s = 0
        single = batch_sizes.shape[0] == 1
        # (the sizes on the host, if the caller has them there: no synchronisation then)
        for i, n in enumerate((batch_sizes if host_batch_sizes is None else host_batch_sizes).tolist()):
            cur = hiddens if single else hiddens[s:s + n]
            gate = torch.matmul(cur, self.w13_weight[i, :, :inter])
            up = torch.matmul(cur, self.w13_weight[i, :, inter:])
            results.append(torch.matmul(self.act_fn(gate) * up, self.w2_weight[i]))
            s += n
        return torch.cat(results)


class MoEExpertsFP8(_GemmState, torch.nn.Module):
    """fp8-e4m3 experts (no counterpart in the reference): weights quantised per
    output channel and stored K-contiguous (``w13_q [E, 2I, d]``, ``w2_q [E, d,
    I]``), activations quantised per row on the fly, bf16 in and out."""

    def __init__(self, w13: torch.Tensor, w2: torch.Tensor, workspace: Optional[torch.Tensor] = None,
                 own_workspace: bool = False):
        super().__init__()
        self.num_experts, self.hidden_size, two_i = w13.shape
        self.intermediate_size = two_i // 2
        q13, s13 = gg.quantize_weight(w13)
        q2, s2 = gg.quantize_weight(w2)
        self.w13_q = torch.nn.Parameter(q13, requires_grad=False)
        self.w13_scale = torch.nn.Parameter(s13, requires_grad=False)
        self.w2_q = torch.nn.Parameter(q2, requires_grad=False)
        self.w2_scale = torch.nn.Parameter(s2, requires_grad=False)
        self._init_gemm_state(w13.device, workspace, own_workspace)

    def forward(self, bs: int, hiddens: torch.Tensor, batch_sizes: torch.Tensor,
                host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
        xq, xs = gg.quantize_rows(hiddens)
        return self.forward_quantized(bs, xq, xs, batch_sizes, host_batch_sizes)

    def forward_quantized(self, bs: int, xq: torch.Tensor, xs: torch.Tensor, batch_sizes: torch.Tensor,
                          host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The same on rows that arrive quantised (``ops.memory.permute_quantize``)."""
        ws = dict(self._gemm_state(), host_batch_sizes=host_batch_sizes)
        h = gg.gmm_fp8_swiglu(xq, xs, self.w13_q, self.w13_scale, batch_sizes, **ws)
        hq, hs = gg.quantize_rows(h)
        return gg.gmm_fp8(hq, hs, self.w2_q, self.w2_scale, batch_sizes, **ws)
