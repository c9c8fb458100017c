"""The reference's package name for the expert-worker hot path.

A caller written against DisagMoE imports ``disagmoe.ops.memory``
(disagmoe/frontend/engine.py:13), ``disagmoe.models.experts`` and
``disagmoe.executor.executor`` (disagmoe/executor/executor.py:14,
disagmoe/frontend/engine.py:6), ``disagmoe.config`` (:7) and
``grouped_gemm.backend`` (disagmoe/models/experts.py:3).  Each of those module
paths resolves to the module of ``disagmoe_amd`` that implements it on the HIP
library: the same module object under a second name, not a copy.  Only the
expert-worker path exists under this name; the controller, transport,
schedulers and attention of DisagMoE are not part of this package.
"""
import disagmoe_amd as _impl

__version__ = _impl.__version__
