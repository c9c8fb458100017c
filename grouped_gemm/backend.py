"""grouped_gemm.backend as the reference imports it (disagmoe/models/experts.py:3, tests/ops/test_gemm.py:1): gmm, get_arguments, gmm_with_arguments (same module object as disagmoe_amd.grouped_gemm.backend)."""
import sys

import disagmoe_amd.grouped_gemm.backend as _impl

sys.modules[__name__] = _impl
