"""disagmoe/config.py of the reference, the fields the expert path reads: ModelConfig (same module object as disagmoe_amd.config)."""
import sys

import disagmoe_amd.config as _impl

sys.modules[__name__] = _impl
