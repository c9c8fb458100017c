"""disagmoe/frontend/datatypes.py of the reference, the per-row bookkeeping the expert step uses: Metadata, TensorBatch (same module object as disagmoe_amd.ops.metadata)."""
import sys

import disagmoe_amd.ops.metadata as _impl

sys.modules[__name__] = _impl
