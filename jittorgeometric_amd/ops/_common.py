"""Helpers shared by the operator wrappers."""
import ctypes as _c
import os

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


def _stamp(t):
    """Identity and in-place version of a tensor: changes whenever the holder's
    attribute is rebound or written in place."""
    return None if t is None else (id(t), t._version)


def _same_storage(a, b):
    """a and b are the same array: one object, or two views of the same memory with the same
    shape and strides (x.reshape(-1) of a flat tensor makes a new object every call)."""
    if a is b:
        return True
    if a is None or b is None:
        return False
    return (a.data_ptr() == b.data_ptr() and a.shape == b.shape and a.stride() == b.stride()
            and a.dtype == b.dtype and a._version == b._version)


def _holder_arrays(holder, names, what):
    """(off, idx, w) of a CSC / CSR object as contiguous int32 / int32 / float32
    device arrays.  Holders built by hand carry whatever torch.tensor([...]) gave
    them (int64 indices, float64 weights, as in the reference's own test scripts,
    tests/test_aggregate.py:43-54); the kernels read int32 / float32 only, so
    anything else is converted here, once, and kept on the holder until one of
    its arrays is rebound or written in place."""
    src = tuple(getattr(holder, n, None) for n in names)
    off, idx, w = src
    if off is None or idx is None:
        raise _lib.JgamdError("%s: %s and %s must be set" % (what, names[0], names[1]))
    stamp = tuple(_stamp(t) for t in src)
    cached = getattr(holder, "_jgamd_arrays", None)
    if cached is not None and cached[0] == stamp and all(a is b for a, b in zip(cached[1], src)):
        return cached[2]
    for n, t in zip(names, src):
        if t is not None and not isinstance(t, torch.Tensor):
            raise _lib.JgamdError("%s.%s must be a torch tensor, got %s" % (what, n, type(t).__name__))
    _lib.require_gpu(off, idx, w)
    out = (as_i32(off, names[0]).reshape(-1), as_i32(idx, names[1]).reshape(-1),
           as_f32(w, names[2]).reshape(-1) if w is not None else None)
    if out[0].shape[0] < 1:
        raise _lib.JgamdError("%s.%s is empty (needs V+1 entries)" % (what, names[0]))
    if out[2] is not None and out[2].shape[0] != out[1].shape[0]:
        raise _lib.JgamdError("%s: %d weights for %d indices" % (what, out[2].shape[0], out[1].shape[0]))
    holder._jgamd_arrays = (stamp, src, out)
    return out


def csc_arrays(csc):
    """(column_offset, row_indices, edge_weight) ready for the C ABI."""
    return _holder_arrays(csc, ("column_offset", "row_indices", "edge_weight"), "CSC")


def csr_arrays(csr):
    """(row_offset, column_indices, edge_weight) ready for the C ABI."""
    return _holder_arrays(csr, ("row_offset", "column_indices", "edge_weight"), "CSR")


def transposed(holder, off, idx, w, R, C):
    """(off_t, idx_t, w_t, perm) of a compressed structure, built on first use
    and kept on the CSR/CSC object it belongs to; rebuilt when any of the three
    arrays is another tensor or has been written in place since."""
    stamp = (_stamp(off), _stamp(idx), _stamp(w))
    cached = getattr(holder, "_jgamd_transposed", None)
    if cached is not None and cached[7] == stamp and cached[4] is off and cached[5] is idx and cached[6] is w:
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
    holder._jgamd_transposed = (off_t, idx_t, w_t, perm, off, idx, w, stamp)
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


PLAN_SPMM, PLAN_GAT, PLAN_TILES = 0, 1, 2


def csx_plan(off, R, E, kind, now=False):
    """(plan, n_fix, n_grp) for the offsets `off` of R rows and E entries: the partition the
    merge-path kernels (PLAN_SPMM, PLAN_GAT) or the tile kernels (PLAN_TILES) work from, kept on
    the offsets tensor until it is written in place (a rebound attribute is another tensor and
    gets its own).  The two counts are the lengths of the plan's lists of cut rows, read back
    once when the plan is built; 0 lets a call skip the kernels that add up row pieces.

    A chunk plan costs two launches and that read-back, a synchronisation with the device, so it
    is built on the second use of the same offsets (or at once with now=True): the graph of a
    training run is used thousands of times, the sampled subgraph of a mini-batch once, and its
    one call takes the entry point that partitions on the fly.  A tile plan costs the one launch
    an unplanned call makes anyway and is built on first use.  Returns (None, -1, -1) when there
    is no plan (yet), also while a HIP graph is being captured: building one would allocate from
    the graph's pool and read back.  Planned and unplanned calls give the same bits."""
    cache = getattr(off, "_jgamd_plans", None)
    if cache is None:
        cache = {}
        off._jgamd_plans = cache
    stamp = (off._version, R, E)
    hit = cache.get(kind)
    if hit is not None and hit[0] == stamp:
        return hit[1], hit[2], hit[3]
    if torch.cuda.is_current_stream_capturing():
        return None, -1, -1
    if kind != PLAN_TILES and not now and cache.get(("seen", kind)) != stamp:
        cache[("seen", kind)] = stamp
        return None, -1, -1
    lib = _lib.load()
    dev = off.device
    nbytes = _lib.query(lib.jgamd_csx_plan_bytes, R, E, kind)
    plan = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
    stream = _lib.stream_ptr(dev)
    _lib.check(lib.jgamd_csx_plan(_lib.ptr(off), R, E, kind, _lib.ptr(plan), nbytes, stream))
    n_fix, n_grp = _c.c_int32(-1), _c.c_int32(-1)
    if kind != PLAN_TILES and R > 0:
        _lib.check(lib.jgamd_csx_plan_counts(_lib.ptr(plan), _c.byref(n_fix), _c.byref(n_grp), stream))
    cache[kind] = (stamp, plan, n_fix.value, n_grp.value)
    return plan, n_fix.value, n_grp.value


def _raw_arrays(off, idx, w, R):
    """Last line of defence in front of the pointer hand-over: dtype, layout and the
    length of the offsets (no copy when the arrays already are what the kernels read)."""
    off = as_i32(off, "off")
    idx = as_i32(idx, "idx") if idx is not None else None
    w = as_f32(w, "w") if w is not None else None
    if off.numel() != R + 1:
        raise _lib.JgamdError("offsets have %d entries for %d rows" % (off.numel(), R))
    if idx is not None and w is not None and idx.numel() != w.numel():
        raise _lib.JgamdError("%d weights for %d indices" % (w.numel(), idx.numel()))
    return off, idx, w


def _blocked_arrays(off, idx, w, R, E, nb, cols):
    """The matrix regrouped by column block (csrc/spmm_blocked.hip), built on first use and
    kept on the offsets tensor it was built from until one of the three arrays is another
    tensor or has been written in place."""
    # the weights are matched by memory and version, not by object: an explicit edge_weight
    # arrives as a fresh view (reshape(-1)) on every call
    stamp = (_stamp(off), _stamp(idx), None if w is None else w._version, nb, cols)
    cached = getattr(off, "_jgamd_blocked", None)
    if cached is not None and cached[0] == stamp and cached[1] is idx and _same_storage(cached[2], w):
        return cached[3]
    lib = _lib.load()
    dev = off.device
    b_off = torch.empty(nb * R + 1, dtype=torch.int32, device=dev)
    b_idx = torch.empty(E, dtype=torch.int32, device=dev)
    b_w = torch.empty(E, dtype=torch.float32, device=dev) if w is not None else None
    nbytes = _lib.query(lib.jgamd_csx_block_columns_workspace, R, nb)
    ws = _lib.workspace(nbytes, dev)
    _lib.check(lib.jgamd_csx_block_columns(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(w), R, E, cols, nb, _lib.ptr(b_off),
                                           _lib.ptr(b_idx), _lib.ptr(b_w), _lib.ptr(ws), nbytes, _lib.stream_ptr(dev)))
    off._jgamd_blocked = (stamp, idx, w, (b_off, b_idx, b_w))
    return b_off, b_idx, b_w


def _product(off, idx, w, x, R, beta, alpha, h, relu=False):
    """beta * (A x) + alpha * h through the plain or the column-blocked kernels; with relu the
    result is clamped at zero, in the product's row store where the kernels offer it."""
    lib = _lib.load()
    dev = _lib.require_gpu(off, x, idx, w, h)
    # rows padded apart (a [V,F] view of a wider buffer, as rows_times(..., pad_rows=True) returns):
    # gathered in place by the planned chunk kernels
    x_stride = 0
    if (x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1 and x.stride(0) > x.shape[1]
            and x.stride(0) % 4 == 0 and x.stride(0) < 1 << 22 and x.data_ptr() % 16 == 0):
        x_stride = x.stride(0)
    else:
        x = as_f32(x, "x")
    off, idx, w = _raw_arrays(off, idx, w, R)
    if x.dim() != 2:
        raise _lib.JgamdError("x must be [rows, F], got %s" % (tuple(x.shape),))
    C, F = x.shape
    h_rows = R
    if h is not None:
        h = as_f32(h, "h")
        if h.dim() == 1 or (h.dim() == 2 and h.shape[0] == 1 and R != 1):
            h_rows = 1
        if h.numel() != h_rows * F:
            raise ValueError("h must be [%d, %d] or [%d], got %s" % (R, F, F, tuple(h.shape)))
    E = int(idx.shape[0]) if idx is not None else C
    out = torch.empty((R, F), dtype=torch.float32, device=dev)
    stream = _lib.stream_ptr(dev)
    nb, cols = _c.c_int32(0), _c.c_int32(0)
    if idx is not None:
        _lib.check(lib.jgamd_spmm_block_plan(R, C, E, F, _c.byref(nb), _c.byref(cols)))
    if nb.value > 0:
        x = x.contiguous()
        x_stride = 0
        b_off, b_idx, b_w = _blocked_arrays(off, idx, w, R, E, nb.value, cols.value)
        nbytes = _lib.query(lib.jgamd_spmm_csx_blocked_workspace, R, C, E, F, nb.value)
        ws = _lib.workspace(nbytes, dev)
        _lib.check(lib.jgamd_spmm_csx_blocked(_lib.ptr(b_off), _lib.ptr(b_idx), _lib.ptr(b_w), _lib.ptr(x), _lib.ptr(out),
                                              float(beta), float(alpha), _lib.ptr(h), h_rows, R, C, E, F, nb.value,
                                              _lib.ptr(ws), nbytes, stream))
        return out.relu_() if relu else out
    # the partition of the rows is kept with the offsets: the chunk plan, or the tile plan for
    # plain products with rows of 1, 2, 4 or 8 floats (the tile kernels have no row finish and
    # read whole aligned rows)
    plain = h is None and beta == 1.0 and not relu
    narrow = (F in (1, 2, 4, 8) and E > 0 and plain and x.data_ptr() % min(16, 4 * F) == 0 and not x_stride
              and not os.environ.get("JGAMD_SPMM_NARROW", "").startswith("m"))
    plan, n_fix, n_grp = csx_plan(off, R, E, PLAN_TILES if narrow else PLAN_SPMM) if R > 0 else (None, -1, -1)
    if plan is None and x_stride:
        x = x.contiguous()          # only the planned entry point takes padded rows
        x_stride = 0
    if plan is not None:
        nbytes = _lib.query(lib.jgamd_spmm_csx_planned_workspace, R, E, F)
        ws = _lib.workspace(nbytes, dev)
        _lib.check(lib.jgamd_spmm_csx_planned(None if narrow else _lib.ptr(plan), _lib.ptr(plan) if narrow else None,
                                              n_fix, n_grp, _lib.ptr(off), _lib.ptr(idx), _lib.ptr(w), _lib.ptr(x),
                                              _lib.ptr(out), float(beta), float(alpha), _lib.ptr(h), h_rows,
                                              (1 if relu else 0) | (x_stride << 8), R, C, E, F, _lib.ptr(ws), nbytes,
                                              stream))
        return out
    nbytes = _lib.query(lib.jgamd_spmm_csx_workspace, R, E, F)
    ws = _lib.workspace(nbytes, dev)
    if h is None and beta == 1.0:
        _lib.check(lib.jgamd_spmm_csx(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(w), _lib.ptr(x), _lib.ptr(out), R, C, E, F,
                                      _lib.ptr(ws), nbytes, stream))
    else:
        _lib.check(lib.jgamd_spmm_csx_axpby(_lib.ptr(off), _lib.ptr(idx), _lib.ptr(w), _lib.ptr(x), _lib.ptr(out),
                                            float(beta), float(alpha), _lib.ptr(h), h_rows, R, C, E, F, _lib.ptr(ws),
                                            nbytes, stream))
    return out.relu_() if relu else out


def spmm(off, idx, w, x, R):
    """out[r,:] = sum_j w[j] * x[idx[j],:]; idx/w may be None (identity / ones)."""
    return _product(off, idx, w, x, R, 1.0, 0.0, None)


def spmm_axpby(off, idx, w, x, R, beta, alpha, h, relu=False):
    """out[r,:] = beta * sum_j w[j] * x[idx[j],:] + alpha * h[r,:]; h is [R,F], or [F] / [1,F]
    for one row added to every output row, or None.  relu clamps the result at zero."""
    return _product(off, idx, w, x, R, beta, alpha, h, relu)


def both_orders(csc, csr):
    """((off, idx, w) gathering into destinations, (off, idx, w) gathering into
    sources) from whichever of the CSC / CSR objects is given; the missing one is
    the cached transpose of the other."""
    if csc is None and csr is None:
        raise ValueError("need a CSC or a CSR")
    if csc is not None:
        fwd = csc_arrays(csc)
    if csr is not None:
        bwd = csr_arrays(csr)
    if csc is None:
        V = bwd[0].shape[0] - 1
        fwd = transposed(csr, bwd[0], bwd[1], bwd[2], V, V)[:3]
    if csr is None:
        V = fwd[0].shape[0] - 1
        bwd = transposed(csc, fwd[0], fwd[1], fwd[2], V, V)[:3]
    return fwd, bwd
