"""disagmoe/executor/executor.py of the reference, its expert half: ExpertsExecutor (same module object as disagmoe_amd.executor.executor)."""
import sys

import disagmoe_amd.executor.executor as _impl

sys.modules[__name__] = _impl
