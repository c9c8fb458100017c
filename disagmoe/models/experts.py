"""disagmoe/models/experts.py of the reference: MoEExperts, MoEExpertsSerial (same module object as disagmoe_amd.models.experts)."""
import sys

import disagmoe_amd.models.experts as _impl

sys.modules[__name__] = _impl
