"""MI355X-native expert-worker hot path: routing, token permute, ragged grouped
GEMM SwiGLU FFN and gate-weighted combine, as hand-written gfx950 HIP kernels
behind the operator API of DisagMoE (``ops.memory``, ``grouped_gemm.backend``,
``models.experts``, ``executor.executor``).

The compute lives in ``libdmoe_hip.so`` (C ABI in ``include/dmoe.h``); there is
no CPU or eager fallback: every operator raises if the library is missing.
"""
from . import _lib  # noqa: F401

__all__ = ["_lib"]
__version__ = "0.1.0"
