"""ctypes binding of libjgamd.so (declarations in include/jgamd.h)."""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libjgamd.so")

_c = ctypes
_P, _I32, _I64, _F32, _SZP = _c.c_void_p, _c.c_int32, _c.c_int64, _c.c_float, _c.POINTER(_c.c_size_t)

# name -> argument types; every function returns int32 unless noted
SIGNATURES = {
    "jgamd_coo_to_csx_workspace": [_I64, _I32, _I32, _SZP],
    "jgamd_coo_to_csx": [_P, _P, _I64, _I32, _I32, _P, _P, _P, _P, _P, _c.c_size_t, _P],
    "jgamd_csx_transpose_workspace": [_I64, _I32, _I32, _SZP],
    "jgamd_csx_transpose": [_P, _P, _P, _I32, _I32, _I64, _P, _P, _P, _P, _P, _c.c_size_t, _P],
    "jgamd_invert_permutation": [_P, _I64, _P, _P],
    "jgamd_scale_csx_weights_workspace": [_I64, _SZP],
    "jgamd_scale_csx_weights": [_P, _P, _P, _P, _P, _I32, _I64, _I32, _P, _P, _c.c_size_t, _P],
    "jgamd_add_remaining_self_loops_workspace": [_I64, _I32, _SZP],
    "jgamd_add_remaining_self_loops": [_P, _P, _I64, _I32, _c.c_float, _P, _P, _P, _P, _c.c_size_t, _P],
    "jgamd_degree_power": [_P, _I32, _c.c_float, _P, _P],
    "jgamd_scale_edge_weights": [_P, _P, _P, _P, _I64, _I32, _P, _P],
    "jgamd_sample_neighbors": [_P, _P, _P, _P, _I32, _I32, _I32, _I64, _c.c_uint64, _P, _P],
    "jgamd_layer_column_counts": [_P, _P, _I32, _I32, _I32, _P, _P],
    "jgamd_layer_column_offsets_workspace": [_I32, _SZP],
    "jgamd_layer_column_offsets": [_P, _P, _I32, _I32, _I32, _P, _P, _c.c_size_t, _P],
    "jgamd_getweight_workspace": [_I32, _SZP],
    "jgamd_getweight": [_P, _P, _P, _I32, _I32, _I64, _P, _P, _c.c_size_t, _P],
    "jgamd_spmm_csx_workspace": [_I32, _I64, _I32, _SZP],
    "jgamd_spmm_csx": [_P, _P, _P, _P, _P, _I32, _I32, _I64, _I32, _P, _c.c_size_t, _P],
    "jgamd_spmm_csx_noalloc": [_P, _P, _P, _P, _P, _I32, _I32, _I64, _I32, _P],
    "jgamd_spmm_csx_axpby": [_P, _P, _P, _P, _P, _c.c_float, _c.c_float, _P, _I32, _I32, _I32, _I64, _I32, _P,
                             _c.c_size_t, _P],
    "jgamd_csx_plan_bytes": [_I32, _I64, _I32, _SZP],
    "jgamd_csx_plan": [_P, _I32, _I64, _I32, _P, _c.c_size_t, _P],
    "jgamd_csx_plan_counts": [_P, _c.POINTER(_I32), _c.POINTER(_I32), _P],
    "jgamd_spmm_csx_planned_workspace": [_I32, _I64, _I32, _SZP],
    "jgamd_spmm_csx_planned": [_P, _P, _I32, _I32, _P, _P, _P, _P, _P, _F32, _F32, _P, _I32, _I32, _I32, _I32, _I64,
                               _I32, _P, _c.c_size_t, _P],
    "jgamd_spmm_block_plan": [_I32, _I32, _I64, _I32, _c.POINTER(_I32), _c.POINTER(_I32)],
    "jgamd_csx_block_columns_workspace": [_I32, _I32, _SZP],
    "jgamd_csx_block_columns": [_P, _P, _P, _I32, _I64, _I32, _I32, _P, _P, _P, _P, _c.c_size_t, _P],
    "jgamd_spmm_csx_blocked_workspace": [_I32, _I32, _I64, _I32, _I32, _SZP],
    "jgamd_spmm_csx_blocked": [_P, _P, _P, _P, _P, _F32, _F32, _P, _I32, _I32, _I32, _I64, _I32, _I32, _P,
                               _c.c_size_t, _P],
    "jgamd_spmm_csx_blocked_timed": [_P, _P, _P, _P, _P, _I32, _I32, _I64, _I32, _I32, _P, _c.c_size_t, _P, _I32,
                                     _c.POINTER(_c.c_float), _c.POINTER(_c.c_float)],
    "jgamd_spmm_csx_timed": [_P, _I32, _I32, _P, _P, _P, _P, _P, _I32, _I32, _I64, _I32, _P, _c.c_size_t, _P, _I32,
                             _c.POINTER(_c.c_float), _c.POINTER(_c.c_float)],
    "jgamd_edge_softmax_workspace": [_I32, _I64, _SZP],
    "jgamd_edge_softmax_fwd": [_P, _P, _P, _I32, _I64, _I32, _P, _c.c_size_t, _P],
    "jgamd_edge_softmax_bwd": [_P, _P, _P, _P, _I32, _I64, _I32, _P, _c.c_size_t, _P],
    "jgamd_edge_softmax_fwd_planned": [_P, _P, _P, _P, _I32, _I64, _I32, _P, _c.c_size_t, _P],
    "jgamd_edge_softmax_bwd_planned": [_P, _P, _P, _P, _P, _I32, _I64, _I32, _P, _c.c_size_t, _P],
    "jgamd_scatter_to_edge": [_P, _P, _P, _P, _I32, _I64, _I32, _I32, _P],
    "jgamd_dense_rows_supported": [_I32, _I32, _I32],
    "jgamd_dense_rows": [_P, _P, _I32, _P, _P, _I32, _P, _P, _I32, _I32, _I32, _P],
    "jgamd_column_sum_workspace": [_I64, _I32, _SZP],
    "jgamd_column_sum": [_P, _P, _I64, _I32, _P, _c.c_size_t, _P],
    "jgamd_relu_backward_column_sum": [_P, _P, _P, _P, _I64, _I32, _P, _c.c_size_t, _P],
    "jgamd_cross_entropy_workspace": [_I64, _I32, _SZP],
    "jgamd_cross_entropy_fwd": [_P, _P, _I32, _I32, _I64, _I32, _P, _P, _P, _P, _c.c_size_t, _P],
    "jgamd_cross_entropy_bwd": [_P, _P, _I32, _P, _P, _P, _I64, _I32, _P, _P],
    "jgamd_gat_fwd_workspace": [_I32, _I64, _I32, _I32, _SZP],
    "jgamd_gat_fwd": [_P, _I32, _I32, _P, _P, _P, _P, _P, _F32, _P, _P, _P, _P, _P, _P, _P, _P, _I32, _I64, _I32,
                      _I32, _P, _c.c_size_t, _P],
    "jgamd_gat_bwd_workspace": [_I32, _I64, _I32, _I32, _SZP],
    "jgamd_gat_bwd": [_P, _I32, _I32, _P, _P, _P, _P, _P, _F32, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I32,
                      _I64, _I32, _I32, _P, _c.c_size_t, _P],
}

_lib = None


class JgamdError(RuntimeError):
    pass


def load():
    """Loads the library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise JgamdError(
            "libjgamd.so is not built (%s). Build it with "
            "`python -m jittorgeometric_amd.build`; there is no fallback path." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)   # AttributeError here means a stale build
        fn.argtypes = argtypes
        fn.restype = _I32
    lib.jgamd_version.restype = _I32
    lib.jgamd_last_error.restype = _c.c_char_p
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        msg = load().jgamd_last_error().decode("utf-8", "replace")
        raise JgamdError("jgamd status %d: %s" % (rc, msg))


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


def stream_ptr(device):
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu(*tensors):
    """The operators run on the GPU only; anything else is an error."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise JgamdError("jittorgeometric_amd operators need GPU tensors (got a %s tensor); "
                             "there is no CPU path" % t.device)
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise JgamdError("tensors on different devices: %s and %s" % (dev, t.device))
    if dev is None:
        raise JgamdError("no tensor given")
    return dev


def workspace(nbytes, device):
    """Scratch for one call, from torch's caching allocator (stream-ordered)."""
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def query(fn, *args):
    n = ctypes.c_size_t(0)
    check(fn(*args, ctypes.byref(n)))
    return n.value
