"""ctypes binding of libstk_amd.so (declared in include/stk_amd.h).

The library is built in-tree by `make -C stk_amd/csrc` (or __graft_entry__.build()).
There is no other implementation behind these symbols: when the shared object
is missing, every device entry point raises.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libstk_amd.so")

ABI_VERSION = 16
STK_OK, STK_ERR_DIMS, STK_ERR_UNSUPPORTED, STK_ERR_HIP, STK_ERR_WORKSPACE = 0, 1, 2, 3, 4
STK_F16, STK_BF16, STK_F32 = 0, 1, 2
STK_I16, STK_I32 = 0, 1

_p, _i64, _int, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/stk_amd.h one to one
SIGNATURES = {
    "stk_last_error": (ctypes.c_char_p, []),
    "stk_abi_version": (_int, []),
    "stk_stream_capture_id": (_int, [_p, _p]),
    "stk_plan_bytes": (_sz, [_i64, _i64, _i64]),
    "stk_build_plan": (_int, [_p, _p, _i64, _p, _p, _i64, _i64, _int, _int, _p, _sz, _p]),
    "stk_sdd": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p, _i64, _int, _int, _int, _p, _p]),
    "stk_sdd_fused": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p, _i64, _int, _int, _int, _p, _int, _p, _p]),
    "stk_sdd_fused_sums": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _p, _i64, _int, _int, _int, _p, _int, _p, _p, _p]),
    "stk_activation_product": (_int, [_p, _p, _p, _i64, _int, _int, _p]),
    "stk_dsd_workspace_bytes": (_i64, [_i64, _i64, _int]),
    "stk_dsd_workspace_counter_bytes": (_i64, []),
    "stk_dsd_workspace_slot_bytes": (_i64, []),
    "stk_dsd_tail_slices": (_int, [_i64, _i64, _i64, ctypes.c_double, _int]),
    "stk_dsd": (_int, [_i64, _i64, _i64, _p, _p, _p, _p, _p, _p, _int, _p, _i64, _i64, _p, _i64, _i64, _int, _int, _int, _p, _p, _i64, _p]),
    "stk_dds": (_int, [_i64, _i64, _i64, _p, _i64, _i64, _p, _p, _p, _p, _p, _p, _int, _p, _i64, _i64, _int, _int, _int, _p, _p]),
    "stk_dsd_dds": (_int, [_i64, _i64, _p, _p, _p, _p, _p, _p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64,
                           _i64, _int, _int, _int, _p, _p]),
    "stk_dsd_dsd": (_int, [_i64, _i64, _p, _p, _p, _p, _p, _p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64,
                           _i64, _int, _int, _int, _p, _p]),
    "stk_sdd_dsd": (_int, [_i64, _i64, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _p, _i64, _i64, _i64, _p,
                           _p, _int, _i64, _p, _i64, _i64, _p, _i64, _i64, _int, _int, _int, _p, _p]),
    "stk_row_indices": (_int, [_p, _i64, _i64, _p, _int, _p]),
    "stk_transpose_meta_workspace_bytes": (_sz, [_i64]),
    "stk_transpose_meta": (_int, [_p, _p, _i64, _i64, _int, _p, _p, _p, _p, _sz, _p]),
    "stk_to_dense": (_int, [_p, _p, _p, _i64, _int, _i64, _i64, _int, _int, _p, _p]),
    "stk_to_sparse_count": (_int, [_p, _i64, _i64, _i64, _int, _int, _p, _p, _p]),
    "stk_to_sparse_count_nnz": (_int, [_p, _i64, _i64, _i64, _int, _int, _p, _p, _p, _p]),
    "stk_to_sparse_fill": (_int, [_p, _i64, _i64, _i64, _int, _int, _p, _p, _i64, _p, _p, _p, _int, _p]),
    "stk_to_sparse_coordinates": (_int, [_i64, _i64, _int, _p, _p, _p, _p, _int, _p]),
    "stk_to_sparse_gather": (_int, [_p, _i64, _i64, _i64, _int, _int, _p, _p, _i64, _int, _p, _p]),
    "stk_dmoe_topology": (_int, [_p, _i64, _int, _i64, _i64, _int, _p, _p, _p, _p, _p, _p, _p]),
    "stk_route_workspace_bytes": (_sz, [_i64, _i64]),
    "stk_route": (_int, [_p, _i64, _i64, _int, _i64, _p, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "stk_route_static": (_int, [_p, _i64, _i64, _int, _i64, _p, _p, _p, _p, _p, _p, _p]),
    "stk_padded_gather": (_int, [_p, _i64, _i64, _i64, _p, _p, _int, _i64, _p, _i64, _int, _p]),
    "stk_padded_scatter": (_int, [_p, _i64, _i64, _i64, _p, _p, _int, _i64, _p, _i64, _int, _p]),
    "stk_padded_scatter_weight_gradient": (_int, [_p, _i64, _i64, _i64, _p, _i64, _p, _int, _i64, _p, _int, _p]),
    "stk_sdd_gather": (_int, [_p, _i64, _i64, _p, _int, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _i64, _int, _int, _int, _p, _int, _p]),
    "stk_dsd_scatter": (_int, [_i64, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _p, _p, _i64, _p, _i64, _i64, _int, _int, _int, _p, _p, _i64, _p]),
}

_lock = threading.Lock()
_lib = None


def load():
    """Returns the loaded library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"stk_amd: {LIB_PATH} is missing. Build it with `make -C stk_amd/csrc` "
                    "(hipcc, gfx950); there is no fallback implementation.")
            lib = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
            if lib.stk_abi_version() != ABI_VERSION:
                raise RuntimeError("stk_amd: libstk_amd.so has an unexpected ABI version; rebuild it")
            _lib = lib
    return _lib


def check(status):
    """Maps a status code to the exception the reference raises in the same situation."""
    if status == STK_OK:
        return
    msg = load().stk_last_error().decode("utf-8", "replace")
    if status == STK_ERR_DIMS:
        raise AssertionError(msg)
    if status == STK_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
