"""Helpers shared by the operator wrappers."""
import torch

from .. import _lib


def as_i32(t, name):
    if t.dtype != torch.int32:
        # the reference's Data casts edge_index to int32 (data/data.py:103-106);
        # int64 inputs (tests/test_spmmcsr.py:14-15) are narrowed the same way
        t = t.to(torch.int32)
    return t.contiguous()


def as_f32(t, name):
    if t.dtype != torch.float32:
        t = t.to(torch.float32)
    return t.contiguous()


def transposed(holder, off, idx, w, R, C):
    """(off_t, idx_t, w_t, perm) of a compressed structure, built on first use
    and kept on the CSR/CSC object it belongs to."""
    cached = getattr(holder, "_jgamd_transposed", None)
    if cached is not None and cached[4] is off and cached[5] is idx and cached[6] is w:
        return cached[:4]
    lib = _lib.load()
    dev = _lib.require_gpu(off, idx, w)
    E = idx.shape[0]
    off_t = torch.empty(C + 1, dtype=torch.int32, device=dev)
    idx_t = torch.empty(E, dtype=torch.int32, device=dev)
    w_t = torch.empty(E, dtype=torch.float32, device=dev) if w is not None else None
    perm = torch.empty(E, dtype=torch.int32, device=dev)
    nbytes = _lib.query(lib.jgamd_csx_transpose_workspace, E, R, C)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_csx_transpose(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(w), R, C, E, _lib.ptr(off_t),
                                       _lib.ptr(idx_t), _lib.ptr(w_t), _lib.ptr(perm), _lib.ptr(ws), nbytes,
                                       _lib.stream_ptr(dev)))
    holder._jgamd_transposed = (off_t, idx_t, w_t, perm, off, idx, w)
    return off_t, idx_t, w_t, perm


def transposed_inverse(holder, perm):
    """inv with inv[perm[j]] = j (original slot -> transposed slot) for the perm
    that `transposed` returned for `holder`; built once and kept beside it."""
    cached = getattr(holder, "_jgamd_transposed_inv", None)
    if cached is not None and cached[1] is perm:
        return cached[0]
    lib = _lib.load()
    dev = _lib.require_gpu(perm)
    inv = torch.empty_like(perm)
    _lib.check(lib.jgamd_invert_permutation(_lib.ptr(perm), perm.shape[0], _lib.ptr(inv), _lib.stream_ptr(dev)))
    holder._jgamd_transposed_inv = (inv, perm)
    return inv


def spmm(off, idx, w, x, R):
    """out[r,:] = sum_j w[j] * x[idx[j],:]; idx/w may be None (identity / ones)."""
    lib = _lib.load()
    dev = _lib.require_gpu(off, x, idx, w)
    x = as_f32(x, "x")
    C, F = x.shape
    E = int(idx.shape[0]) if idx is not None else C
    out = torch.empty((R, F), dtype=torch.float32, device=dev)
    nbytes = _lib.query(lib.jgamd_spmm_csx_workspace, R, E, F)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_spmm_csx(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(w), _lib.ptr(x), _lib.ptr(out), R, C, E, F,
                                  _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
    return out


def spmm_axpby(off, idx, w, x, R, beta, alpha, h):
    """out[r,:] = beta * sum_j w[j] * x[idx[j],:] + alpha * h[r,:]; h is [R,F], or [F] / [1,F]
    for one row added to every output row, or None."""
    lib = _lib.load()
    dev = _lib.require_gpu(off, x, idx, w, h)
    x = as_f32(x, "x")
    h = as_f32(h, "h") if h is not None else None
    C, F = x.shape
    h_rows = R
    if h is not None:
        if h.dim() == 1 or (h.dim() == 2 and h.shape[0] == 1 and R != 1):
            h_rows = 1
        if h.numel() != h_rows * F:
            raise ValueError("h must be [%d, %d] or [%d], got %s" % (R, F, F, tuple(h.shape)))
    E = int(idx.shape[0]) if idx is not None else C
    out = torch.empty((R, F), dtype=torch.float32, device=dev)
    nbytes = _lib.query(lib.jgamd_spmm_csx_workspace, R, E, F)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_spmm_csx_axpby(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(w), _lib.ptr(x), _lib.ptr(out),
                                        float(beta), float(alpha), _lib.ptr(h), h_rows, R, C, E, F, _lib.ptr(ws), nbytes,
                                        _lib.stream_ptr(dev)))
    return out


def both_orders(csc, csr):
    """((off, idx, w) gathering into destinations, (off, idx, w) gathering into
    sources) from whichever of the CSC / CSR objects is given; the missing one is
    the cached transpose of the other."""
    if csc is None and csr is None:
        raise ValueError("need a CSC or a CSR")
    if csc is not None:
        fwd = (as_i32(csc.column_offset, "column_offset"), as_i32(csc.row_indices, "row_indices"),
               as_f32(csc.edge_weight, "edge_weight"))
    if csr is not None:
        bwd = (as_i32(csr.row_offset, "row_offset"), as_i32(csr.column_indices, "column_indices"),
               as_f32(csr.edge_weight, "edge_weight"))
    if csc is None:
        V = bwd[0].shape[0] - 1
        fwd = transposed(csr, bwd[0], bwd[1], bwd[2], V, V)[:3]
    if csr is None:
        V = fwd[0].shape[0] - 1
        bwd = transposed(csc, fwd[0], fwd[1], fwd[2], V, V)[:3]
    return fwd, bwd
