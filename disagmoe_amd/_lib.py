"""ctypes binding of libdmoe_hip.so (the C ABI declared in include/dmoe.h)."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_int64, c_size_t, c_void_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdmoe_hip.so")

# dmoe.h constants
OK = 0
ERR_ARG, ERR_SHAPE, ERR_DTYPE, ERR_WORKSPACE, ERR_HIP = -1, -2, -3, -4, -5
BF16, FP16, FP8_E4M3, FP32 = 0, 1, 2, 3
I32, I64 = 4, 8
ORDER_REFERENCE, ORDER_STABLE = 0, 1
COMBINE_FP32, COMBINE_REFERENCE = 0, 1

#: every symbol include/dmoe.h declares: name -> (restype, argtypes)
SIGNATURES = {
    "dmoe_version": (c_char_p, []),
    "dmoe_last_error": (c_char_p, []),
    "dmoe_device_cus": (c_int, [POINTER(c_int)]),
    "dmoe_route_scratch_bytes": (c_int, [c_int64, c_int, POINTER(c_size_t)]),
    "dmoe_route": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p,
                           c_void_p, c_size_t, c_void_p]),
    "dmoe_route_sources": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                                   c_void_p, c_void_p, c_size_t, c_void_p]),
    "dmoe_route_noalloc_max_bytes": (c_int, [POINTER(c_size_t)]),
    "dmoe_route_noalloc": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p,
                                   c_void_p]),
    "dmoe_topk_softmax": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "dmoe_sort_by_prefill_order": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "dmoe_move_row_infos": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p]),
    "dmoe_expert_batch_sizes": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_int, c_void_p]),
    "dmoe_host_mappings": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p]),
    "dmoe_metadata_wire_bytes": (c_int, [c_void_p, POINTER(c_size_t)]),
    "dmoe_metadata_serialize": (c_int, [c_void_p, c_void_p, c_size_t]),
    "dmoe_metadata_parse": (c_int, [c_void_p, c_size_t, c_void_p]),
    "dmoe_permute": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_void_p,
                             c_void_p]),
    "dmoe_gather_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "dmoe_gather_ptrs": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "dmoe_combine": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int, c_int,
                             c_void_p]),
    "dmoe_gmm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int, c_int,
                         c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
    "dmoe_gmm_swiglu": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_int,
                                c_int, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
    "dmoe_gmm_swiglu_rows": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64,
                                     c_int64, c_int, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
    "dmoe_gmm_workspace_bytes": (c_int, [c_int, POINTER(c_size_t)]),
    "dmoe_quant_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p]),
    "dmoe_permute_quant": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int,
                                   c_void_p]),
    "dmoe_gmm_fp8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64,
                             c_int64, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
    "dmoe_gmm_fp8_swiglu": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                    c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]),
}

#: exported for the library's own tests and benchmarks, not declared in include/dmoe.h (csrc/tuning.h)
TEST_HOOKS = {
    "dmoe_gmm_tune": (c_int, [c_int]),
    "dmoe_gmm_plan": (c_int, [c_void_p, c_int, c_int64, c_int, c_int64, c_int64, c_int, c_int, c_int, c_size_t, c_void_p]),
}
GMM_STATE_BYTES = 33024



class MetadataView(ctypes.Structure):
    """dmoe_metadata_view of include/dmoe.h."""
    _fields_ = [("shape", c_void_p), ("n_shape", ctypes.c_uint64), ("dtype", c_void_p), ("n_dtype", ctypes.c_uint64),
                ("layer_id", ctypes.c_int32),
                ("req_ids", c_void_p), ("n_req_ids", ctypes.c_uint64), ("exp_ids", c_void_p), ("n_exp_ids", ctypes.c_uint64),
                ("attn_dp_ranks", c_void_p), ("n_attn_dp_ranks", ctypes.c_uint64),
                ("init_prefill_lens", c_void_p), ("n_init_prefill_lens", ctypes.c_uint64),
                ("topk_weights", c_void_p), ("n_topk_weights", ctypes.c_uint64)]


class MetadataLayout(ctypes.Structure):
    """dmoe_metadata_layout of include/dmoe.h."""
    _fields_ = [("off_shape", ctypes.c_uint64), ("n_shape", ctypes.c_uint64), ("off_dtype", ctypes.c_uint64),
                ("n_dtype", ctypes.c_uint64), ("layer_id", ctypes.c_int32),
                ("off_req_ids", ctypes.c_uint64), ("n_req_ids", ctypes.c_uint64),
                ("off_exp_ids", ctypes.c_uint64), ("n_exp_ids", ctypes.c_uint64),
                ("off_attn_dp_ranks", ctypes.c_uint64), ("n_attn_dp_ranks", ctypes.c_uint64),
                ("off_init_prefill_lens", ctypes.c_uint64), ("n_init_prefill_lens", ctypes.c_uint64),
                ("off_topk_weights", ctypes.c_uint64), ("n_topk_weights", ctypes.c_uint64)]


_lib = None


class DmoeError(RuntimeError):
    """A libdmoe_hip entry point returned a DMOE_ERR_* code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libdmoe_hip error {code}: {message}")
        self.code = code


def load() -> ctypes.CDLL:
    """Load the HIP library (once).  Raises if it has not been built: there is no
    fallback implementation."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m disagmoe_amd.build` "
            "(hipcc, gfx950). disagmoe_amd has no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in {**SIGNATURES, **TEST_HOOKS}.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != OK:
        raise DmoeError(rc, load().dmoe_last_error().decode("utf-8", "replace"))


def call(name: str, *args) -> None:
    check(getattr(load(), name)(*args))


def version() -> str:
    return load().dmoe_version().decode()
