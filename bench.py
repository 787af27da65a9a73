#!/usr/bin/env python3
"""Benchmark of the sparse message-passing hot path on one MI355X.

Default workload (--config 2): weighted CSR/CSC SpMM at F=128 on the 1M-node
power-law graph (Chung-Lu, exponent 2.1, 16M directed edges, degree cap 20,000,
self-loops appended, gcn_norm weights, edges in random order), plus the
COO->CSR/CSC conversion of the same graph, a GCN layer forward+backward, edge
softmax and one fused propagation hop on it.  One "step" is one SpMM pass
(out[dst] = sum w * x[src]) over the whole graph.  --config 1, 3, 4, 5 run the
other benchmark configurations with the same one-line JSON shape.  Inputs are
synthetic and resident in HBM before the timed region.

The line's `value` is algorithmic bytes per step / time per step
(SpMM: 4(R+1) + 8E + 4EF + 4RF: offsets, (idx,w) per entry, one F-row gather per
entry, the output) or the step time for the time-like configurations.

`roofline` describes the dominant kernel of the step:
  traffic           bytes one launch moves between L2 and the memory fabric, from the rocprofv3
                    counter summary under profiles/ (FETCH_SIZE and WRITE_SIZE, each scaled by
                    what it reads for a plain copy of known size); the summary must describe this
                    very workload (V, E, F are compared) or the run stops
  achieved, frac    traffic / the kernel's mean launch time measured in this run with HIP events
                    on the launch stream, and that rate over the 8 TB/s HBM peak.  A gathered row
                    that L2 serves is not memory traffic, so this -- not the algorithmic figure --
                    is what is held against the memory roofline.  Hits in the memory-side Infinity
                    Cache cannot be told from HBM reads by any counter the GPU exposes, so `frac`
                    is an upper bound of the HBM share; `compulsory_frac` (every array once) is
                    the lower bound
  effective         algorithmic bytes / kernel time (can exceed the peak: it counts rows L2 serves)
  copy_gbps         what a plain 1 GiB device-to-device copy moves per second on this GPU in this
                    run (bytes read + bytes written, HIP events); frac_of_copy = achieved / copy_gbps
  hbm_frac_range    [compulsory_frac, frac]: the share of the HBM peak lies between every array
                    moved once and everything that missed L2

Times: `ms_per_step` and `value` are the wall-clock mean over exactly --steps steps between two
device synchronisations; `ms_per_step_event_median` is the median of per-step HIP-event times of a
second loop of the same length.
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def spmm_bytes(R, E, feat):
    return 4 * (R + 1) + 8 * E + 4 * E * feat + 4 * R * feat


def spmm_compulsory_bytes(R, C, E, feat):
    return 4 * (R + 1) + 8 * E + 4 * C * feat + 4 * R * feat


def read_profile(name, expect):
    """Key figures of a rocprofv3 summary under profiles/ ('@key value' lines), or None when there
    is no summary or it was taken on another workload than this run's (then the line carries no
    counted traffic, and says why)."""
    path = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(path):
        return None
    vals = {}
    for line in open(path):
        m = re.match(r"@(\w+)\s+(\S+)", line)
        if m:
            vals[m.group(1)] = m.group(2)
    for key, want in expect.items():
        have = int(float(vals[key])) if key in vals else None
        # The generators call the host's math library; a last-bit difference between two hosts can
        # move an edge or two.  Up to 0.1 % of the edge count the counted bytes are scaled with it.
        if key == "E" and have and have != int(want) and abs(have - int(want)) <= 1e-3 * have:
            if "traffic_bytes" in vals:
                vals["traffic_bytes"] = str(float(vals["traffic_bytes"]) * int(want) / have)
            continue
        if have != int(want):
            print("bench.py: %s describes %s=%s, this run has %s=%s: its counters are not used; take them "
                  "again (the command is in the file's header)" % (path, key, vals.get(key), key, want),
                  file=sys.stderr)
            return None
    return vals


def roofline(profile_name, expect, kernel, kernel_ms, algorithmic, compulsory, timing, copy_gbps=None,
             bound="hbm"):
    prof = read_profile(profile_name, expect)
    traffic = float(prof["traffic_bytes"]) if prof and "traffic_bytes" in prof else None
    rate = lambda b: round(b / (kernel_ms * 1e-3) / 1e9, 1)
    out = {"bound": bound, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "kernel": kernel, "kernel_ms": round(kernel_ms, 4),
           "kernel_ms_source": timing, "traffic": traffic,
           "traffic_source": ("profiles/" + profile_name) if traffic else None,
           "algorithmic_bytes": algorithmic, "compulsory_bytes": compulsory,
           "effective": rate(algorithmic), "compulsory_frac": round(rate(compulsory) / HBM_PEAK_GBPS, 4)}
    if traffic:
        out["achieved"], out["achieved_basis"] = rate(traffic), "counted L2<->fabric bytes / kernel time"
    else:
        out["achieved"], out["achieved_basis"] = rate(algorithmic), "algorithmic bytes / kernel time (no counter summary)"
    out["frac"] = round(out["achieved"] / HBM_PEAK_GBPS, 4)
    out["hbm_frac_range"] = [out["compulsory_frac"], out["frac"]]
    if copy_gbps:
        out["copy_gbps"] = round(copy_gbps, 1)
        out["frac_of_copy"] = round(out["achieved"] / copy_gbps, 4)
    if prof:
        for k in ("l2_hit_rate", "profile_kernel_us"):
            if k in prof:
                out[k] = float(prof[k])
    return out


class Ms(float):
    """A mean time in ms that also carries the event-timed median of the same call."""
    median = None


class Bench:
    def __init__(self, args):
        import torch
        from jittorgeometric_amd import _lib
        self.args = args
        self.torch = torch
        self._lib = _lib
        self.lib = _lib.load()
        self.dev = torch.device("cuda:0")
        torch.manual_seed(0)

    def timed(self, fn, iters, warm):
        """Wall-clock mean per call over `iters` calls between two synchronisations (the returned
        number) and, as its .median, the median of per-call HIP-event times of a second loop."""
        torch = self.torch
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        mean = Ms((time.perf_counter() - t0) / iters * 1e3)
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
        for a, b in ev:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        times = sorted(a.elapsed_time(b) for a, b in ev)
        mean.median = times[len(times) // 2] if len(times) % 2 else 0.5 * (times[len(times) // 2 - 1] + times[len(times) // 2])
        return mean

    def copy_rate_gbps(self):
        """Bytes read + written per second by a plain 1 GiB device copy, median of 7 (HIP events)."""
        torch = self.torch
        a = torch.empty(1 << 28, dtype=torch.float32, device=self.dev).fill_(1.0)
        b = torch.empty_like(a)
        ms = self.timed(lambda: b.copy_(a), 7, 2).median
        del a, b
        return 2 * (1 << 30) / (ms * 1e-3) / 1e9

    def graph(self, name, norm="gcn", time_conversions=True):
        """(edge_index, weights, V, CSC, CSR, conversion times) of a configuration after the
        normalisation with self-loops, converted on the device."""
        from jittorgeometric_amd import synthetic
        from jittorgeometric_amd.nn import gcn_norm, sage_norm
        from jittorgeometric_amd.ops import cootocsc, cootocsr
        ei_np, V = synthetic.make(name)
        ei = self.torch.from_numpy(ei_np).to(self.dev)
        ei, w = (gcn_norm if norm == "gcn" else sage_norm)(ei, None, V)
        ei = ei.contiguous()
        csr_ms = self.timed(lambda: cootocsr(ei, w, V), 10, 2) if time_conversions else 0.0
        csc_ms = self.timed(lambda: cootocsc(ei, w, V), 10, 2) if time_conversions else 0.0
        return ei, w, V, cootocsc(ei, w, V), cootocsr(ei, w, V), csr_ms, csc_ms

    def spmm_kernel_ms(self, off, idx, w, x, R, iters):
        """Mean duration of the gather kernel (spmm_merge) and of the whole call, from HIP events
        recorded on the launch stream inside the library; through the column-blocked kernels when
        the library's plan picks them for this shape, as the operators do."""
        torch, _lib, lib = self.torch, self._lib, self.lib
        from jittorgeometric_amd.ops._common import _blocked_arrays
        C, F = x.shape
        E = idx.shape[0]
        out = torch.empty(R, F, device=self.dev)
        k_ms, c_ms = ctypes.c_float(), ctypes.c_float()
        nb, cols = ctypes.c_int32(0), ctypes.c_int32(0)
        _lib.check(lib.jgamd_spmm_block_plan(R, C, E, F, ctypes.byref(nb), ctypes.byref(cols)))
        self.blocked = nb.value
        if nb.value > 0:
            b_off, b_idx, b_w = _blocked_arrays(off, idx, w, R, E, nb.value, cols.value)
            nbytes = _lib.query(lib.jgamd_spmm_csx_blocked_workspace, R, C, E, F, nb.value)
            ws = _lib.workspace(nbytes, self.dev)
            torch.cuda.synchronize()
            _lib.check(lib.jgamd_spmm_csx_blocked_timed(b_off.data_ptr(), b_idx.data_ptr(), b_w.data_ptr(), x.data_ptr(),
                                                        out.data_ptr(), R, C, E, F, nb.value, ws.data_ptr(), nbytes,
                                                        _lib.stream_ptr(self.dev), iters, ctypes.byref(k_ms),
                                                        ctypes.byref(c_ms)))
            return k_ms.value, c_ms.value
        from jittorgeometric_amd.ops._common import PLAN_SPMM, csx_plan
        plan, n_fix, n_grp = csx_plan(off, R, E, PLAN_SPMM, now=True)       # the partition the operators keep with the offsets
        nbytes = _lib.query(lib.jgamd_spmm_csx_planned_workspace, R, E, F)
        ws = _lib.workspace(nbytes, self.dev)
        torch.cuda.synchronize()
        _lib.check(lib.jgamd_spmm_csx_timed(plan.data_ptr(), n_fix, n_grp, off.data_ptr(), idx.data_ptr(), w.data_ptr(),
                                            x.data_ptr(), out.data_ptr(), R, C, E, F, ws.data_ptr(), nbytes,
                                            _lib.stream_ptr(self.dev), iters, ctypes.byref(k_ms), ctypes.byref(c_ms)))
        return k_ms.value, c_ms.value

    def calibrate_copy(self):
        torch = self.torch
        a = torch.empty(1 << 28, dtype=torch.float32, device=self.dev).fill_(1.0)
        b = torch.empty_like(a)
        torch.cuda.synchronize()
        b.copy_(a)                      # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()

    def cpu_spmm_baseline(self, csc, x, step, bytes_step, conv_inputs, what):
        """The reference's single-threaded loops (oracle port) on this host, bounded to about
        10-30 s, and the GPU result of the same step held against them."""
        import numpy as np
        import oracle
        col, off, wv = (t.cpu().numpy() for t in (csc.row_indices, csc.column_offset, csc.edge_weight))
        xh = x.cpu().numpy()
        V, F = xh.shape
        passes, t0 = 0, time.perf_counter()
        while passes < 1 or (time.perf_counter() - t0 < 10.0 and passes < 64):
            ref = oracle.aggregate(xh, col, off, wv)
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        # Tolerance of the path: 1e-5 of the sum of absolute terms + 1e-6, held against the exact
        # (float64) row sums.  The reference's loop adds a row in fp32 one term after the other and
        # is itself only good to (entries - 1) * 2^-24 of that sum, which the comparison with it allows.
        exact, terms = oracle.aggregate_f64(xh, col, off, wv)
        deg = np.diff(off).astype(np.float64)[:, None]
        got = step().cpu().numpy().astype(np.float64)
        err_exact = float(np.max(np.abs(got - exact) / (1e-6 + 1e-5 * terms)))
        err_loop = float(np.max(np.abs(got - ref) / (1e-6 + (1e-5 + deg * 2.0 ** -24) * terms)))
        err = max(err_exact, err_loop)
        ei, w = conv_inputs
        t0 = time.perf_counter()
        oracle.cootocsr(ei.cpu().numpy(), w.cpu().numpy(), V)
        cpu_conv_s = time.perf_counter() - t0
        return {"value": round(bytes_step / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "%d full passes of %s, %.2f s each" % (passes, what, cpu_s),
                "cpu_model": cpu_model(), "host_cores_available": os.cpu_count(),
                "coo_to_csr_edges_per_s": round(ei.shape[1] / cpu_conv_s),
                "gpu_vs_exact_max_scaled_err": round(err_exact, 4),
                "gpu_vs_cpu_max_scaled_err": round(err_loop, 4)}, err


def cpu_spmm_rows_baseline(csc, x, step, what, seconds=12.0):
    """The reference's loop (oracle port, one thread) on a random sample of the rows of a product
    too large for a full pass within the time the benchmark may take: a 0.5 % sample is timed
    first, then a sample sized for about `seconds` of work.  The rate is the sample's own
    algorithmic bytes over its time; the GPU's rows of the same sample are held against the
    exact (float64) sums and against the loop."""
    import numpy as np
    import oracle
    col, off, wv = (t.cpu().numpy() for t in (csc.row_indices, csc.column_offset, csc.edge_weight))
    xh = x.cpu().numpy()
    V, F = xh.shape
    rng = np.random.default_rng(0)

    def run(nrows):
        rows = np.sort(rng.choice(V, size=nrows, replace=False))
        t0 = time.perf_counter()
        ref = oracle.aggregate_rows(xh, col, off, wv, rows)
        return rows, ref, time.perf_counter() - t0
    rows, ref, dt = run(max(V // 200, 1))
    entries = int((off[rows + 1] - off[rows]).sum())
    want = int(min(V, max(len(rows), len(rows) * seconds / max(dt, 1e-3))))
    if want > 2 * len(rows):
        rows, ref, dt = run(want)
        entries = int((off[rows + 1] - off[rows]).sum())
    nbytes = 4 * (len(rows) + 1) + 8 * entries + 4 * entries * F + 4 * len(rows) * F
    exact, terms = oracle.aggregate_rows_f64(xh, col, off, wv, rows)
    deg = (off[rows + 1] - off[rows]).astype(np.float64)[:, None]
    got = step().cpu().numpy()[rows].astype(np.float64)
    err_exact = float(np.max(np.abs(got - exact) / (1e-6 + 1e-5 * terms)))
    err_loop = float(np.max(np.abs(got - ref) / (1e-6 + (1e-5 + deg * 2.0 ** -24) * terms)))
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d of %d rows (%d of %d entries) of %s, chosen at random, one pass of %.1f s; a full pass "
                      "would take about %.0f s" % (len(rows), V, entries, int(off[-1]), what, dt, dt * int(off[-1]) / max(entries, 1)),
            "cpu_model": cpu_model(), "host_cores_available": os.cpu_count(),
            "gpu_vs_exact_max_scaled_err": round(err_exact, 4),
            "gpu_vs_cpu_max_scaled_err": round(err_loop, 4)}, max(err_exact, err_loop)


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def base_line(args, metric, value, unit, ms, higher, workload, extra_config):
    cfg = {"workload": workload}
    cfg.update(extra_config)
    line = {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms, 4), "higher_is_better": higher, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32", "data": "synthetic", "config": cfg}
    if getattr(ms, "median", None) is not None:
        line["ms_per_step_event_median"] = round(ms.median, 4)
    return line


# --------------------------------------------------------------------------------- config 2
def config2(b):
    from jittorgeometric_amd import synthetic
    from jittorgeometric_amd.nn import GCNConv, SAGEConv
    from jittorgeometric_amd.ops import EdgeSoftmax, cootocsc, gat_aggregate
    from jittorgeometric_amd.ops._common import spmm, spmm_axpby
    from jittorgeometric_amd.ops.gat import gat_forward_raw
    from jittorgeometric_amd.utils import add_remaining_self_loops
    torch, args, dev = b.torch, b.args, b.dev
    F = 128
    ei, w, V, csc, csr, conv_csr_ms, conv_csc_ms = b.graph("powerlaw_1m")
    E = ei.shape[1]
    x = torch.randn(V, F, device=dev)
    if args.calibrate_copy:
        b.calibrate_copy()

    if args.part == "softmax":
        return config2_softmax(b, csc, V, E), 0.0
    if args.part == "propagate":
        return config2_propagate(b, csc, csr, V, E), 0.0
    if args.part == "convert":
        # only the two conversions of the normalised edge list (what profiles/coo_to_csx_powerlaw_1m.txt
        # is taken from)
        from jittorgeometric_amd.ops import cootocsr
        iters, warm = max(args.steps, 10), args.warmup
        csr_ms = b.timed(lambda: cootocsr(ei, w, V), iters, warm)
        csc_ms = b.timed(lambda: cootocsc(ei, w, V), iters, warm)
        conv_bytes = 24 * E + 8 * (V + 1)
        line = base_line(args, "coo_to_csr_edges_per_s", round(E / (csr_ms * 1e-3)), "edges/s", csr_ms, True,
                         "config 2: cootocsr / cootocsc of the gcn_norm edge list, V=1,000,000, E=%d" % E,
                         {"V": V, "E": E})
        line.update({"coo_to_csr_ms": round(csr_ms, 4), "coo_to_csc_ms": round(csc_ms, 4),
                     "coo_to_csr_ms_event_median": round(csr_ms.median, 4),
                     "coo_to_csc_edges_per_s": round(E / (csc_ms * 1e-3)),
                     "roofline": {"bound": "hbm", "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                  "kernel": "csx_partition_pack + csx_sub_scatter (+ 7 short kernels)",
                                  "algorithmic_bytes": conv_bytes,
                                  "achieved": round(conv_bytes / (csr_ms * 1e-3) / 1e9, 1),
                                  "frac": round(conv_bytes / (csr_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                  "traffic": None, "achieved_basis": "algorithmic bytes / operator time"},
                     "cpu_baseline": None})
        return line, 0.0
    step = lambda: spmm(csc.column_offset, csc.row_indices, csc.edge_weight, x, V)
    bytes_step = spmm_bytes(V, E, F)
    setup_ms = None
    if args.part == "all":
        # the graph set-up of examples/gcn_example.py:48-59 as one sequence: normalisation with
        # self-loops, then both conversions of the normalised edge list
        from jittorgeometric_amd.nn import gcn_norm
        from jittorgeometric_amd.ops import cootocsr
        raw = torch.from_numpy(synthetic.make("powerlaw_1m")[0]).to(dev)

        def setup():
            e2, w2 = gcn_norm(raw, None, V)
            return cootocsc(e2, w2, V), cootocsr(e2, w2, V)
        setup_ms = b.timed(setup, 10, 2)
        del raw
    line = base_line(args, "spmm_f128_algorithmic_bandwidth", 0.0, "GB/s", 0.0, True,
                     "config 2: weighted CSC SpMM, V=1,000,000 Chung-Lu power-law (exp 2.1, cap 20000) "
                     "+ self-loops, gcn_norm weights, F=128", {"V": V, "E": E, "F": F, "bytes_per_step": bytes_step})
    if args.part != "layers":
        ms_per_step = b.timed(step, args.steps, args.warmup)
        value = bytes_step / (ms_per_step * 1e-3) / 1e9
        k_ms, c_ms = b.spmm_kernel_ms(csc.column_offset, csc.row_indices, csc.edge_weight, x, V, max(args.steps, 10))
        line.update({
            "value": round(value, 1), "ms_per_step": round(ms_per_step, 4),
            "ms_per_step_event_median": round(ms_per_step.median, 4),
            "pct_hbm_peak_algorithmic": round(100 * value / HBM_PEAK_GBPS, 2),
            "coo_to_csr_edges_per_s": round(E / (conv_csr_ms * 1e-3)),
            "coo_to_csc_edges_per_s": round(E / (conv_csc_ms * 1e-3)),
            "coo_to_csr_ms": round(conv_csr_ms, 4),
            "coo_to_csr_algorithmic_gbps": round((24 * E + 8 * (V + 1)) / (conv_csr_ms * 1e-3) / 1e9, 1),
            "roofline": roofline("spmm_merge_powerlaw_1m_f128.txt", {"V": V, "E": E, "F": F}, "spmm_merge", k_ms,
                                 bytes_step, spmm_compulsory_bytes(V, V, E, F), "hipEvents in this run",
                                 b.copy_rate_gbps()),
            "spmm_call_ms": round(c_ms, 4),
        })
        if setup_ms is not None:
            line["graph_setup_gcn_norm_csc_csr_ms"] = round(setup_ms, 4)

    if args.part in ("all", "layers"):
        # one GCN layer and one GraphSAGE (mean) layer, forward + backward, on the same graph
        xg = x.clone().requires_grad_(True)
        g_up = torch.randn(V, F, device=dev)

        def layer_ms(layer, call):
            def one():
                layer.zero_grad(set_to_none=True)
                xg.grad = None
                call(layer).backward(g_up)
            return b.timed(one, max(args.steps, 10) if args.part == "layers" else 10, 2)
        gcn_ms = layer_ms(GCNConv(F, F, spmm=False).to(dev), lambda l: l(xg, csc, csr))
        ei_s, w_s, _, csc_s, csr_s, _, _ = b.graph("powerlaw_1m", "sage", time_conversions=False)
        sage_ms = layer_ms(SAGEConv(F, F, spmm=False).to(dev), lambda l: l(xg, None, None, csc_s, csr_s))
        del ei_s, w_s, csc_s, csr_s
        line.update({
            "gcn_layer_fwd_bwd_ms": round(gcn_ms, 4),
            "gcn_layer_shape": "GCNConv(128->128) on the same graph, aggregateWithWeight path: x@W, SpMM + bias; "
                               "backward: bias column sum, transposed SpMM, W.grad, x.grad",
            "sage_layer_fwd_bwd_ms": round(sage_ms, 4),
            "sage_layer_shape": "SAGEConv(128->128, root weight, bias) on the same graph with mean weights: SpMM, "
                                "both dense products + bias in one pass; backward: column sum, two W.grad, two "
                                "input-gradient products, transposed SpMM with the root term added in its row store",
        })
        if args.part == "layers":
            line.update({"metric": "gcn_layer_fwd_bwd_ms", "value": round(gcn_ms, 4), "unit": "ms",
                         "ms_per_step": round(gcn_ms, 4), "higher_is_better": False})

    if args.part == "all":
        bwd_ms = b.timed(lambda: spmm(csr.row_offset, csr.column_indices, csr.edge_weight, x, V), 20, 3)
        # fused GAT layer core on the 169k-node configuration
        gei_np, gV = synthetic.make("gat_169k")
        gei, _ = add_remaining_self_loops(torch.from_numpy(gei_np).to(dev), None, 1.0, gV)
        gei = gei.contiguous()
        gE = gei.shape[1]
        gcsc = cootocsc(gei, torch.ones(gE, device=dev), gV)
        H, D = 8, 16
        gh = torch.randn(gV, H, D, device=dev, requires_grad=True)
        ga_s = (torch.randn(H, D, device=dev) / 4).requires_grad_(True)
        ga_d = (torch.randn(H, D, device=dev) / 4).requires_grad_(True)
        gg = torch.randn(gV, H, D, device=dev)
        gat_fwd_ms = b.timed(lambda: gat_forward_raw(gh.detach(), gcsc, ga_s.detach(), ga_d.detach(), 0.2), 20, 3)

        def gat_step():
            gh.grad = ga_s.grad = ga_d.grad = None
            gat_aggregate(gh, gcsc, ga_s, ga_d, 0.2).backward(gg)
        gat_fb_ms = b.timed(gat_step, 20, 3)
        gat_bytes = gE * (4 + 4 * H * D) + gV * (4 + 8 * H + 4 * H * D) + gV * H * D * 4 + 2 * gV * H * 4

        # edge softmax (the reference's [E,1] shape, and 8 heads) and one propagation hop
        logits = torch.randn(E, 1, device=dev, requires_grad=True)
        esm_fwd_ms = b.timed(lambda: EdgeSoftmax(logits.detach(), csc), 20, 3)
        y1 = EdgeSoftmax(logits, csc)
        g1 = torch.randn(E, 1, device=dev)
        esm_bwd_ms = b.timed(lambda: torch.autograd.grad(y1, logits, g1, retain_graph=True), 20, 3)
        del y1, g1, logits
        logits8 = torch.randn(E, 8, device=dev)
        esm8_fwd_ms = b.timed(lambda: EdgeSoftmax(logits8, csc), 10, 2)
        del logits8
        hop_ms = b.timed(lambda: spmm_axpby(csc.column_offset, csc.row_indices, csc.edge_weight, x, V, 0.9, 0.1, x), 10, 2)
        esm_b = lambda h, per: (per * E * h + 4 * (V + 1))
        line.update({
            "spmm_csr_backward_ms": round(bwd_ms, 4),
            "gat_fused_fwd_ms": round(gat_fwd_ms, 4),
            "gat_fused_fwd_bwd_ms": round(gat_fb_ms, 4),
            "gat_fused_fwd_algorithmic_gbps": round(gat_bytes / (gat_fwd_ms * 1e-3) / 1e9, 1),
            "gat_shape": "V=%d, E=%d (power-law exp 2.3 + self-loops), 8 heads x 16" % (gV, gE),
            "edge_softmax_fwd_ms": round(esm_fwd_ms, 4),
            "edge_softmax_fwd_algorithmic_gbps": round(esm_b(1, 8) / (esm_fwd_ms * 1e-3) / 1e9, 1),
            "edge_softmax_bwd_ms": round(esm_bwd_ms, 4),
            "edge_softmax_bwd_algorithmic_gbps": round(esm_b(1, 12) / (esm_bwd_ms * 1e-3) / 1e9, 1),
            "edge_softmax_h8_fwd_ms": round(esm8_fwd_ms, 4),
            "edge_softmax_h8_fwd_algorithmic_gbps": round(esm_b(8, 8) / (esm8_fwd_ms * 1e-3) / 1e9, 1),
            "appnp_hop_f128_ms": round(hop_ms, 4),
        })

    cpu, err = (None, 0.0)
    if not args.no_cpu_baseline and args.part == "all":
        cpu, err = b.cpu_spmm_baseline(csc, x, step, bytes_step, (ei, w),
                                       "the same SpMM workload (V=%d, E=%d, F=%d)" % (V, E, F))
    line["cpu_baseline"] = cpu
    return line, err


def config2_softmax(b, csc, V, E):
    """Only the standalone edge softmax on config 2's graph, forward and backward at 1 and 8 heads
    (what profiles/edge_softmax_powerlaw_1m.txt is taken from).  Times are of the operator's
    C entry points through the wrappers, without autograd's dispatch."""
    from jittorgeometric_amd.ops import EdgeSoftmax
    from jittorgeometric_amd.ops.edgesoftmax import EdgeSoftmaxFunc
    torch, args, dev = b.torch, b.args, b.dev
    iters, warm = max(args.steps, 5), args.warmup
    out = {}

    class Ctx:      # what EdgeSoftmaxFunc.backward reads from its context
        pass
    for H in (1, 8):
        x = torch.randn(E, H, device=dev)
        g = torch.randn(E, H, device=dev)
        y = EdgeSoftmax(x, csc)
        fwd = b.timed(lambda: EdgeSoftmax(x, csc), iters, warm)
        ctx = Ctx()
        ctx.saved_tensors, ctx.csc = (y,), csc
        bwd = b.timed(lambda: EdgeSoftmaxFunc.backward(ctx, g), iters, warm)
        fb, bb = 8 * E * H + 4 * (V + 1), 12 * E * H + 4 * (V + 1)
        out["edge_softmax_h%d_fwd_ms" % H] = round(fwd, 4)
        out["edge_softmax_h%d_fwd_frac_hbm_peak" % H] = round(fb / (fwd * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)
        out["edge_softmax_h%d_bwd_ms" % H] = round(bwd, 4)
        out["edge_softmax_h%d_bwd_frac_hbm_peak" % H] = round(bb / (bwd * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)
        del x, g, y
    ms = out["edge_softmax_h1_fwd_ms"]
    line = base_line(args, "edge_softmax_fwd_ms", ms, "ms", ms, False,
                     "config 2 graph, standalone edge softmax over the CSC columns, [E,1] and [E,8] logits",
                     {"V": V, "E": E})
    line.update(out)
    line["roofline"] = {"bound": "hbm", "peak": HBM_PEAK_GBPS, "unit": "GB/s", "kernel": "esm_fwd_tile + esm_merge + esm_finish",
                        "algorithmic_bytes": 8 * E + 4 * (V + 1),
                        "achieved": round((8 * E + 4 * (V + 1)) / (ms * 1e-3) / 1e9, 1),
                        "frac": out["edge_softmax_h1_fwd_frac_hbm_peak"], "traffic": None,
                        "achieved_basis": "algorithmic bytes / operator time"}
    line["cpu_baseline"] = None
    return line


def config2_propagate(b, csc, csr, V, E):
    """Forward passes of the propagation layers on config 2's graph at 64 features: each layer
    as this build runs it (the element-wise tail of every hop in the product's row store; BernNet
    by Horner's rule) and as the reference's chain of operators (fused=False)."""
    from jittorgeometric_amd.nn import APPNP, BernNet, ChebNetII, EvenNet, GCN2Conv
    torch, args, dev = b.torch, b.args, b.dev
    F, K = 64, 10
    iters, warm = max(args.steps // 5, 5), 2
    x = torch.randn(V, F, device=dev)
    x0 = torch.randn(V, F, device=dev)
    out = {}
    with torch.no_grad():
        for name, make, call in (
                ("appnp_k10", lambda f: APPNP(K, 0.1, spmm=False, fused=f), lambda l: l(x, csc, csr)),
                ("chebnet2_k10", lambda f: ChebNetII(K, spmm=False, fused=f).to(dev), lambda l: l(x, csc, csr)),
                ("evennet_k10", lambda f: EvenNet(K, 0.1, spmm=False, fused=f), lambda l: l(x, csc, csr)),
                ("gcn2conv", lambda f: GCN2Conv(F, F, spmm=False, fused=f).to(dev), lambda l: l(x, x0, csc, csr, 0.1, 0.4)),
                ("bernnet_k10", lambda f: BernNet(K, spmm=False, fused=f).to(dev), lambda l: l(x, csc, csr, csc, csr))):
            for fused in (True, False):
                layer = make(fused)
                out["%s_f64_fwd_%s_ms" % (name, "fused" if fused else "chain")] = round(
                    b.timed(lambda: call(layer), iters if fused or name != "bernnet_k10" else 3, warm), 4)
    ms = out["chebnet2_k10_f64_fwd_fused_ms"]
    line = base_line(args, "chebnet2_k10_f64_fwd_ms", ms, "ms", ms, False,
                     "config 2 graph, forward of the propagation layers at 64 features (K = 10 hops where the layer has K)",
                     {"V": V, "E": E, "F": F, "K": K})
    line.update(out)
    hop_bytes = 4 * (V + 1) + 8 * E + 4 * E * F + 4 * V * F
    line["roofline"] = {"bound": "hbm", "peak": HBM_PEAK_GBPS, "unit": "GB/s", "kernel": "spmm_merge (one per hop)",
                        "algorithmic_bytes": hop_bytes + 4 * V * F, "traffic": None,
                        "achieved": round(K * (hop_bytes + 4 * V * F) / (ms * 1e-3) / 1e9, 1),
                        "frac": round(K * (hop_bytes + 4 * V * F) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                        "achieved_basis": "K hops x (product bytes + the added row) / layer time"}
    line["cpu_baseline"] = None
    return line


# --------------------------------------------------------------------------------- config 1
def config1(b):
    """2-layer GCN forward + backward on the 2,708-node graph (1433 -> 256 -> 7)."""
    import numpy as np
    from jittorgeometric_amd.nn import GCNConv, cross_entropy_loss
    from jittorgeometric_amd.ops._common import spmm
    torch, args, dev = b.torch, b.args, b.dev
    ei, w, V, csc, csr, conv_csr_ms, conv_csc_ms = b.graph("cora_like")
    E = ei.shape[1]
    rng = np.random.default_rng(1)
    xh = (rng.random((V, 1433)) < 0.013).astype(np.float32)
    xh /= np.maximum(xh.sum(1, keepdims=True), 1)
    x = torch.from_numpy(xh).to(dev)
    y = torch.from_numpy(rng.integers(0, 7, V)).to(dev)
    l1, l2 = GCNConv(1433, 256, spmm=False).to(dev), GCNConv(256, 7, spmm=False).to(dev)

    def step():
        l1.zero_grad(set_to_none=True)
        l2.zero_grad(set_to_none=True)
        out = l2(torch.relu(l1(x, csc, csr)), csc, csr)
        cross_entropy_loss(out, y).backward()
    ms = b.timed(step, args.steps, args.warmup)
    # the same step recorded into a HIP graph once and replayed: at this size the eager step is
    # a few dozen launches of a few microseconds each
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    graph_ms = b.timed(graph.replay, args.steps, args.warmup)
    h = torch.randn(V, 256, device=dev)
    k_ms, _ = b.spmm_kernel_ms(csc.column_offset, csc.row_indices, csc.edge_weight, h, V, 50)
    cpu = None
    if not args.no_cpu_baseline:
        import oracle
        W1, W2 = l1.weight.detach().cpu().numpy(), l2.weight.detach().cpu().numpy()
        oc = tuple(t.cpu().numpy() for t in (csc.row_indices, csc.column_offset, csc.edge_weight))
        orr = tuple(t.cpu().numpy() for t in (csr.column_indices, csr.row_offset, csr.edge_weight))
        n, t0 = 0, time.perf_counter()
        while n < 3 or time.perf_counter() - t0 < 3.0:
            a1 = oracle.aggregate(xh @ W1, *oc)
            a2 = oracle.aggregate(np.maximum(a1, 0) @ W2, *oc)
            g2 = oracle.aggregate(a2, *orr)                       # stand-in upstream gradient of the same shape
            g1 = oracle.aggregate((g2 @ W2.T) * (a1 > 0), *orr)
            _ = xh.T @ g1
            n += 1
        cpu = {"value": round((time.perf_counter() - t0) / n * 1e3, 3), "unit": "ms", "cores": 1, "kind": "port",
               "sample": "%d passes of the four aggregations and the dense products of the step (numpy + oracle loops)" % n,
               "cpu_model": cpu_model()}
    line = base_line(args, "gcn2_fwd_bwd_ms", round(ms, 4), "ms", ms, False,
                     "config 1: 2-layer GCN forward+backward, V=2708, 10556 directed edges + self-loops, 1433->256->7",
                     {"V": V, "E": E})
    line.update({"coo_to_csr_ms": round(conv_csr_ms, 4), "gcn2_fwd_bwd_graph_replay_ms": round(graph_ms, 4),
                 "gcn2_fwd_bwd_graph_replay_event_median_ms": round(graph_ms.median, 4),
                 "roofline": roofline("spmm_merge_cora_like_f256.txt", {"V": V, "E": E, "F": 256}, "spmm_merge", k_ms,
                                      spmm_bytes(V, E, 256), spmm_compulsory_bytes(V, V, E, 256), "hipEvents in this run",
                                      b.copy_rate_gbps(), bound="launch latency (13k entries; every array fits L2)"),
                 "note": "launch-bound at this size: 13k entries are one launch of a few microseconds",
                 "cpu_baseline": cpu})
    return line, 0.0


# --------------------------------------------------------------------------------- config 3
def config3(b):
    """Fused GAT core (edge softmax + weighted aggregation), 8 heads x 16, forward and backward."""
    from jittorgeometric_amd import synthetic
    from jittorgeometric_amd.ops import cootocsc, gat_aggregate
    from jittorgeometric_amd.ops.gat import gat_forward_raw
    from jittorgeometric_amd.utils import add_remaining_self_loops
    torch, args, dev = b.torch, b.args, b.dev
    ei_np, V = synthetic.make("gat_169k")
    ei, _ = add_remaining_self_loops(torch.from_numpy(ei_np).to(dev), None, 1.0, V)
    ei = ei.contiguous()
    E = ei.shape[1]
    csc = cootocsc(ei, torch.ones(E, device=dev), V)
    H, D = 8, 16
    h = torch.randn(V, H, D, device=dev, requires_grad=True)
    a_s = (torch.randn(H, D, device=dev) / 4).requires_grad_(True)
    a_d = (torch.randn(H, D, device=dev) / 4).requires_grad_(True)
    g = torch.randn(V, H, D, device=dev)
    fwd_ms = b.timed(lambda: gat_forward_raw(h.detach(), csc, a_s.detach(), a_d.detach(), 0.2), 20, 3)

    def step():
        h.grad = a_s.grad = a_d.grad = None
        gat_aggregate(h, csc, a_s, a_d, 0.2).backward(g)
    ms = b.timed(step, args.steps, args.warmup)
    fwd_bytes = E * (4 + 4 * H * D) + V * (4 + 8 * H + 4 * H * D) + V * H * D * 4 + 2 * V * H * 4
    compulsory = 8 * E + 4 * (V + 1) + 2 * V * H * D * 4 + 4 * V * H * 4
    cpu = None
    if not args.no_cpu_baseline:
        import oracle
        row, off = csc.row_indices.cpu().numpy(), csc.column_offset.cpu().numpy()
        hh, s, d = h.detach().cpu().numpy(), a_s.detach().cpu().numpy(), a_d.detach().cpu().numpy()
        gh = g.cpu().numpy()
        n, t0, fwd_s = 0, time.perf_counter(), 0.0
        while n < 1 or time.perf_counter() - t0 < 10.0:
            t1 = time.perf_counter()
            oracle.gat_forward_heads(hh, (row, off, None), s, d, 0.2)
            fwd_s += time.perf_counter() - t1
            oracle.gat_backward_heads(hh, (row, off, None), s, d, gh, 0.2)
            n += 1
        cpu = {"value": round((time.perf_counter() - t0) / n * 1e3, 2), "unit": "ms", "cores": 1, "kind": "port",
               "forward_only_ms": round(fwd_s / n * 1e3, 2),
               "sample": "%d passes of the same step, forward + backward, all heads: the reference's operator chain and "
                         "the chain of its operators' grad functions (oracle loops; the backward recomputes the "
                         "forward's per-edge tensors as autograd would have kept them)" % n,
               "cpu_model": cpu_model()}
    prof = read_profile("gat_merge_gat_169k_h8x16.txt", {"V": V, "E": E, "F": H * D})
    k_ms = float(prof["profile_kernel_us"]) / 1e3 if prof and "profile_kernel_us" in prof else fwd_ms
    line = base_line(args, "gat_fused_fwd_bwd_ms", round(ms, 4), "ms", ms, False,
                     "config 3: fused GAT core fwd+bwd, V=169,343, power-law exp 2.3 + self-loops, 8 heads x 16",
                     {"V": V, "E": E, "H": H, "D": D})
    line.update({"gat_fused_fwd_ms": round(fwd_ms, 4),
                 "gat_fused_fwd_algorithmic_gbps": round(fwd_bytes / (fwd_ms * 1e-3) / 1e9, 1),
                 "gat_fused_fwd_event_median_ms": round(fwd_ms.median, 4),
                 "roofline": roofline("gat_merge_gat_169k_h8x16.txt", {"V": V, "E": E, "F": H * D}, "gat_fwd_merge", k_ms,
                                      fwd_bytes, compulsory,
                                      "rocprofv3 summary" if prof else "whole forward call in this run (4 launches)",
                                      b.copy_rate_gbps(),
                                      bound="fabric (L2-miss traffic; the 87 MB feature table fits the 256 MB "
                                            "Infinity Cache, so most of it is not HBM traffic)"),
                 "cpu_baseline": cpu})
    return line, 0.0


# --------------------------------------------------------------------------------- config 4
def config4(b):
    """Dense-degree aggregation at F = 602, 256, 41 and the conversion of the 114.6M-edge list."""
    from jittorgeometric_amd.ops._common import spmm
    torch, args, dev = b.torch, b.args, b.dev
    ei, w, V, csc, csr, conv_csr_ms, conv_csc_ms = b.graph("dense_233k")
    E = ei.shape[1]
    res = {}
    for F in ((602,) if args.part == "main" else (602, 256, 41)):
        x = torch.randn(V, F, device=dev)
        step = lambda x=x: spmm(csc.column_offset, csc.row_indices, csc.edge_weight, x, V)
        ms = b.timed(step, args.steps if F == 602 else 10, args.warmup if F == 602 else 2)
        k_ms, _ = b.spmm_kernel_ms(csc.column_offset, csc.row_indices, csc.edge_weight, x, V, 10)
        res[F] = (ms, k_ms, x, step, b.blocked)
    ms, k_ms, x, step, blocks = res[602]

    def regroup():
        # the once-per-matrix regrouping by column block, which the timed steps above reuse
        from jittorgeometric_amd.ops._common import _blocked_arrays
        nb, cols = ctypes.c_int32(0), ctypes.c_int32(0)
        b._lib.check(b.lib.jgamd_spmm_block_plan(V, V, E, 602, ctypes.byref(nb), ctypes.byref(cols)))
        if nb.value:
            csc.column_offset._jgamd_blocked = None
            _blocked_arrays(csc.column_offset, csc.row_indices, csc.edge_weight, V, E, nb.value, cols.value)
    regroup_ms = b.timed(regroup, 3, 1) if blocks else 0.0
    bytes_step = spmm_bytes(V, E, 602)
    cpu, err = (None, 0.0)
    if not args.no_cpu_baseline and args.part == "all":
        cpu, err = cpu_spmm_rows_baseline(csc, x, step, "the F=602 product of this graph (V=%d, E=%d)" % (V, E))
    line = base_line(args, "spmm_f602_algorithmic_bandwidth", round(bytes_step / (ms * 1e-3) / 1e9, 1), "GB/s", ms, True,
                     "config 4: weighted CSC SpMM, V=232,965, lognormal degrees (mean 492) + self-loops, F=602",
                     {"V": V, "E": E, "F": 602, "bytes_per_step": bytes_step})
    if args.part == "all":
        line.update({"spmm_f256_ms": round(res[256][0], 4),
                     "spmm_f256_algorithmic_gbps": round(spmm_bytes(V, E, 256) / (res[256][0] * 1e-3) / 1e9, 1),
                     "spmm_f41_ms": round(res[41][0], 4),
                     "spmm_f41_algorithmic_gbps": round(spmm_bytes(V, E, 41) / (res[41][0] * 1e-3) / 1e9, 1)})
    if blocks:
        line["note"] = ("column-blocked product: most gathers are served by L2 (l2_hit_rate), so roofline.frac, the "
                        "share of the HBM peak that the counted L2-miss traffic amounts to, is low by design; the kernel "
                        "is bound by L2 delivery")
    line.update({"column_blocks": blocks,
                 "regroup_by_column_block_ms_once_per_matrix": round(regroup_ms, 4),
                 "coo_to_csr_ms": round(conv_csr_ms, 4), "coo_to_csr_edges_per_s": round(E / (conv_csr_ms * 1e-3)),
                 "coo_to_csc_edges_per_s": round(E / (conv_csc_ms * 1e-3)),
                 "roofline": roofline("spmm_merge_dense_233k_f602.txt", {"V": V, "E": E, "F": 602}, "spmm_merge", k_ms,
                                      bytes_step, spmm_compulsory_bytes(V, V, E, 602), "hipEvents in this run",
                                      b.copy_rate_gbps(),
                                      bound="L2 delivery (column-blocked gathers; hbm_frac_range is what reaches the fabric)"
                                      if blocks else "hbm"),
                 "cpu_baseline": cpu})
    return line, err


# --------------------------------------------------------------------------------- config 5
def config5(b):
    """Full-graph 3-layer GCN and GraphSAGE-mean forward + backward (100 -> 256 -> 256 -> 47)."""
    from jittorgeometric_amd.nn import GCNConv, SAGEConv, cross_entropy_loss
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from jittorgeometric_amd.ops._common import spmm
    torch, args, dev = b.torch, b.args, b.dev
    ei, w, V, csc, csr, conv_csr_ms, conv_csc_ms = b.graph("powerlaw_2m4")
    E = ei.shape[1]
    dims = [100, 256, 256, 47]
    x = torch.randn(V, 100, device=dev)
    y = torch.randint(0, 47, (V,), device=dev)

    def model_step(layers, call, loss_fn=cross_entropy_loss, relu_inside=False):
        for layer in layers:
            layer.zero_grad(set_to_none=True)
        hcur = x
        for i, layer in enumerate(layers):
            hcur = call(layer, hcur)
            if i < 2 and not relu_inside:
                hcur = torch.relu(hcur)
        loss_fn(hcur, y).backward()

    main_only = args.part == "main"
    gcn_ms = sage_ms = gcn_af_ms = sage_tf_ms = gcn_torch_loss_ms = gcn_act_ms = sage_act_ms = 0.0
    if not main_only:
        gcn = [GCNConv(dims[i], dims[i + 1], spmm=False).to(dev) for i in range(3)]
        gcn_ms = b.timed(lambda: model_step(gcn, lambda l, t: l(t, csc, csr)), args.steps, args.warmup)
        # the same step with the framework's generic loss instead of the library's kernel
        gcn_torch_loss_ms = b.timed(lambda: model_step(gcn, lambda l, t: l(t, csc, csr), torch.nn.functional.cross_entropy),
                                    args.steps, args.warmup)
        # the same model with each layer's two products in the cheaper order (an option of this build's GCNConv)
        gcn_af = [GCNConv(dims[i], dims[i + 1], spmm=False, aggregate_first=dims[i] < dims[i + 1]).to(dev) for i in range(3)]
        gcn_af_ms = b.timed(lambda: model_step(gcn_af, lambda l, t: l(t, csc, csr)), args.steps, args.warmup)
        del gcn_af
        # the same model with the activation applied in the product's row store (an option of this build's GCNConv)
        gcn_act = [GCNConv(dims[i], dims[i + 1], spmm=False, activation="relu" if i < 2 else None).to(dev) for i in range(3)]
        gcn_act_ms = b.timed(lambda: model_step(gcn_act, lambda l, t: l(t, csc, csr), relu_inside=True), args.steps, args.warmup)
        del gcn_act
        from jittorgeometric_amd.nn import sage_norm
        sei, sw = sage_norm(ei[:, :E - V].contiguous(), None, V)       # same edges, mean weights
        sei = sei.contiguous()
        scsc, scsr = cootocsc(sei, sw, V), cootocsr(sei, sw, V)
        sage = [SAGEConv(dims[i], dims[i + 1], root_weight=False, spmm=False).to(dev) for i in range(3)]
        sage_ms = b.timed(lambda: model_step(sage, lambda l, t: l(t, None, None, scsc, scsr)), args.steps, args.warmup)
        sage_tf = [SAGEConv(dims[i], dims[i + 1], root_weight=False, spmm=False,
                            transform_first=dims[i + 1] < dims[i]).to(dev) for i in range(3)]
        sage_tf_ms = b.timed(lambda: model_step(sage_tf, lambda l, t: l(t, None, None, scsc, scsr)), args.steps, args.warmup)
        sage_act = [SAGEConv(dims[i], dims[i + 1], root_weight=False, spmm=False,
                             activation="relu" if i < 2 else None).to(dev) for i in range(3)]
        sage_act_ms = b.timed(lambda: model_step(sage_act, lambda l, t: l(t, None, None, scsc, scsr), relu_inside=True),
                              args.steps, args.warmup)
        del sei, sw, scsc, scsr, sage, gcn, sage_tf, sage_act
    widths = (256,) if main_only else (100, 256, 47)
    prod = {}
    for F in widths:
        xf = torch.randn(V, F, device=dev)
        prod[F] = (b.timed(lambda xf=xf: spmm(csc.column_offset, csc.row_indices, csc.edge_weight, xf, V), 10, 2),
                   b.spmm_kernel_ms(csc.column_offset, csc.row_indices, csc.edge_weight, xf, V, 10)[0], xf)
    f47_padded_ms = None
    if not main_only:
        # the same product with the rows of x 64 floats apart, as the 256 -> 47 layer's x @ W is written
        x47 = torch.randn(V, 64, device=dev)[:, :47]
        f47_padded_ms = b.timed(lambda: spmm(csc.column_offset, csc.row_indices, csc.edge_weight, x47, V), 10, 2)
        del x47
    cpu, err = (None, 0.0)
    if not args.no_cpu_baseline and not main_only:
        xf = prod[256][2]
        cpu, err = cpu_spmm_rows_baseline(csc, xf, lambda: spmm(csc.column_offset, csc.row_indices, csc.edge_weight, xf, V),
                                          "the F=256 product of this graph (V=%d, E=%d)" % (V, E))
    line = base_line(args, "gcn3_fullgraph_fwd_bwd_ms", round(gcn_ms, 3), "ms", gcn_ms, False,
                     "config 5: 3-layer GCN full-graph forward+backward, V=2,449,029 power-law (exp 2.1, mean 50) "
                     "+ self-loops, 100->256->256->47", {"V": V, "E": E})
    line.update({"loss": "mean cross-entropy over all nodes, library kernel (jgamd_cross_entropy_fwd / _bwd)",
                 "gcn3_with_torch_cross_entropy_ms": round(gcn_torch_loss_ms, 3),
                 "sage3_fullgraph_fwd_bwd_ms": round(sage_ms, 3),
                 "gcn3_aggregate_first_where_narrower_ms": round(gcn_af_ms, 3),
                 "gcn3_relu_in_row_store_ms": round(gcn_act_ms, 3),
                 "sage3_relu_in_dense_store_ms": round(sage_act_ms, 3),
                 "sage3_transform_first_where_narrower_ms": round(sage_tf_ms, 3),
                 "coo_to_csr_ms": round(conv_csr_ms, 4), "coo_to_csr_edges_per_s": round(E / (conv_csr_ms * 1e-3)),
                 "coo_to_csc_edges_per_s": round(E / (conv_csc_ms * 1e-3))})
    for F in widths:
        line["spmm_f%d_ms" % F] = round(prod[F][0], 4)
        line["spmm_f%d_algorithmic_gbps" % F] = round(spmm_bytes(V, E, F) / (prod[F][0] * 1e-3) / 1e9, 1)
    if f47_padded_ms is not None:
        line["spmm_f47_rows_64_apart_ms"] = round(f47_padded_ms, 4)
        line["spmm_f47_rows_64_apart_algorithmic_gbps"] = round(spmm_bytes(V, E, 47) / (f47_padded_ms * 1e-3) / 1e9, 1)
    line["roofline"] = roofline("spmm_merge_powerlaw_2m4_f256.txt", {"V": V, "E": E, "F": 256}, "spmm_merge", prod[256][1],
                                spmm_bytes(V, E, 256), spmm_compulsory_bytes(V, V, E, 256), "hipEvents in this run",
                                b.copy_rate_gbps())
    line["cpu_baseline"] = cpu
    if main_only:
        # only the F=256 product ran (the part the counter summaries are taken from): that is the line's metric
        ms = prod[256][0]
        line.update({"metric": "spmm_f256_algorithmic_bandwidth", "value": round(spmm_bytes(V, E, 256) / (ms * 1e-3) / 1e9, 1),
                     "unit": "GB/s", "ms_per_step": round(ms, 4), "higher_is_better": True})
        for k in ("loss", "gcn3_with_torch_cross_entropy_ms", "sage3_fullgraph_fwd_bwd_ms", "gcn3_relu_in_row_store_ms", "sage3_relu_in_dense_store_ms",
                  "gcn3_aggregate_first_where_narrower_ms", "sage3_transform_first_where_narrower_ms"):
            line.pop(k, None)
    return line, err


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4, 5],
                    help="benchmark configuration; 2 (the headline SpMM workload) is the default")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the single-thread CPU timing")
    ap.add_argument("--part", default="all", choices=["all", "main", "layers", "softmax", "convert", "propagate"],
                    help="main: only the timed workload of the metric (what the counter profiles under profiles/ "
                         "are taken from); layers: only the GCN and GraphSAGE layer steps of config 2")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (known traffic, for scaling rocprof counters)")
    args = ap.parse_args()
    if args.part in ("layers", "softmax", "convert", "propagate") and args.config != 2:
        sys.exit("bench.py: --part %s belongs to --config 2" % args.part)
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only; --gpus %d is not supported "
                 "(no collectives or sharding are part of it)" % args.gpus)
    defaults = {1: (200, 20), 2: (50, 5), 3: (50, 5), 4: (10, 2), 5: (5, 1)}
    if args.steps is None:
        args.steps = defaults[args.config][0]
    if args.warmup is None:
        args.warmup = defaults[args.config][1]

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    b = Bench(args)
    if args.calibrate_copy and args.config != 2:
        b.calibrate_copy()
    line, err = {1: config1, 2: config2, 3: config3, 4: config4, 5: config5}[args.config](b)
    print(json.dumps(line))
    if err > 1.0:
        sys.exit("bench.py: the GPU result is %.2f times the tolerance away from the CPU result "
                 "(1e-5 of the sum of absolute terms + 1e-6 against the exact row sums; against the "
                 "reference's fp32 loop its own sequential rounding is allowed on top)" % err)


if __name__ == "__main__":
    main()
