"""``grouped_gemm`` as the reference imports it: the ``backend`` module (``gmm``, ``get_arguments``,
``gmm_with_arguments``) on the HIP grouped GEMM.  ``ops`` of the upstream package (autograd wrapper) is not part of the
expert-worker path."""
from . import backend  # noqa: F401
