#!/usr/bin/env python3
"""Benchmark of the sparse message-passing hot path on one MI355X.

Workload: weighted CSR/CSC SpMM at F=128 on the 1M-node power-law graph
(Chung-Lu, exponent 2.1, 16M directed edges, degree cap 20,000, self-loops
appended, gcn_norm weights, edges in random order), plus the COO->CSR/CSC
conversion of the same graph and a GCN layer forward+backward on it.  One
"step" is one SpMM pass (out[dst] = sum w * x[src]) over the whole graph.
Inputs are synthetic and resident in HBM before the timed region.

Prints ONE JSON line.  `value` is algorithmic bytes per step / time per step
(bytes = 4(R+1) + 8E + 4EF + 4RF: offsets, (idx,w) per entry, one F-row
gather per entry, the output).  Gathered rows that hit the L2 / Infinity
Cache never reach HBM, so this figure can exceed what the HBM moved; the
`roofline.traffic` field holds the measured HBM bytes when a counter run has
supplied them.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
F = 128
# FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 per spmm_merge launch on this exact (seeded) workload;
# factors from a plain 1 GiB copy in the same counter runs.
PROFILED_TRAFFIC_BYTES = 7.074e9


def spmm_bytes(R, E, feat):
    return 4 * (R + 1) + 8 * E + 4 * E * feat + 4 * R * feat


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the single-thread CPU timing")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (known traffic, for scaling rocprof counters)")
    ap.add_argument("--traffic-bytes", type=float, default=PROFILED_TRAFFIC_BYTES,
                    help="bytes moved between L2 and the fabric per spmm_merge launch, from the separate "
                         "rocprofv3 --pmc runs summarised under profiles/ (counters cannot be read in-process)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only; --gpus %d is not supported "
                 "(no collectives or sharding are part of it)" % args.gpus)

    import numpy as np
    import torch
    from jittorgeometric_amd import _lib, synthetic
    from jittorgeometric_amd.nn import GCNConv, gcn_norm
    from jittorgeometric_amd.ops import cootocsc, cootocsr
    from jittorgeometric_amd.ops._common import spmm

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.manual_seed(0)

    # ---- inputs (host generation, then resident on the device) -------------
    ei_np, V = synthetic.make("powerlaw_1m")
    ei = torch.from_numpy(ei_np).to(dev)
    ei, w = gcn_norm(ei, None, V)
    ei = ei.contiguous()
    E = ei.shape[1]
    x = torch.randn(V, F, device=dev)

    def timed(fn, iters, warm):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / iters * 1e3

    if args.calibrate_copy:
        a = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
        b = torch.empty_like(a)
        torch.cuda.synchronize()
        b.copy_(a)                      # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del a, b

    # ---- conversion ---------------------------------------------------------
    conv_csr_ms = timed(lambda: cootocsr(ei, w, V), 10, 2)
    conv_csc_ms = timed(lambda: cootocsc(ei, w, V), 10, 2)
    csr = cootocsr(ei, w, V)
    csc = cootocsc(ei, w, V)

    # ---- the timed steps: SpMM over the CSC arrays at F=128 ------------------
    step = lambda: spmm(csc.column_offset, csc.row_indices, csc.edge_weight, x, V)
    ms_per_step = timed(step, args.steps, args.warmup)
    bytes_step = spmm_bytes(V, E, F)
    value = bytes_step / (ms_per_step * 1e-3) / 1e9

    # backward direction (CSR arrays), same kernel
    bwd_ms = timed(lambda: spmm(csr.row_offset, csr.column_indices, csr.edge_weight, x, V), 20, 3)

    # ---- dominant kernel alone: hipEvents around each spmm_merge launch ------
    out = torch.empty(V, F, device=dev)
    nbytes = _lib.query(lib.jgamd_spmm_csx_workspace, V, E, F)
    ws = _lib.workspace(nbytes, dev)
    k_ms, c_ms = ctypes.c_float(), ctypes.c_float()
    torch.cuda.synchronize()
    _lib.check(lib.jgamd_spmm_csx_timed(csc.column_offset.data_ptr(), csc.row_indices.data_ptr(),
                                        csc.edge_weight.data_ptr(), x.data_ptr(), out.data_ptr(), V, V, E, F,
                                        ws.data_ptr(), nbytes, _lib.stream_ptr(dev), max(args.steps, 10),
                                        ctypes.byref(k_ms), ctypes.byref(c_ms)))
    achieved = bytes_step / (k_ms.value * 1e-3) / 1e9

    # ---- one GCN layer forward + backward on the same graph ------------------
    layer = GCNConv(F, F, spmm=False).to(dev)
    xg = x.clone().requires_grad_(True)

    g_up = torch.randn(V, F, device=dev)

    def layer_step():
        layer.zero_grad(set_to_none=True)
        xg.grad = None
        layer(xg, csc, csr).backward(g_up)
    gcn_ms = timed(layer_step, 10, 2)

    # ---- fused GAT layer core on the 169k-node configuration ----------------------
    from jittorgeometric_amd.ops import gat_aggregate
    from jittorgeometric_amd.ops.gat import gat_forward_raw
    from jittorgeometric_amd.utils import add_remaining_self_loops
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
    gat_fwd_ms = timed(lambda: gat_forward_raw(gh.detach(), gcsc, ga_s.detach(), ga_d.detach(), 0.2), 20, 3)

    def gat_step():
        gh.grad = ga_s.grad = ga_d.grad = None
        gat_aggregate(gh, gcsc, ga_s, ga_d, 0.2).backward(gg)
    gat_fb_ms = timed(gat_step, 20, 3)
    gat_bytes = gE * (4 + 4 * H * D) + gV * (4 + 8 * H + 4 * H * D) + gV * H * D * 4 + 2 * gV * H * 4

    # ---- edge softmax (the reference's [E,1] shape) and one APPNP hop on the main graph ----
    from jittorgeometric_amd.ops import EdgeSoftmax
    from jittorgeometric_amd.ops._common import spmm_axpby
    logits = torch.randn(E, 1, device=dev)
    esm_fwd_ms = timed(lambda: EdgeSoftmax(logits, csc), 20, 3)
    hop_ms = timed(lambda: spmm_axpby(csc.column_offset, csc.row_indices, csc.edge_weight, x, V, 0.9, 0.1, x), 10, 2)
    del logits

    # ---- CPU baseline: the reference's single-threaded loop (oracle port) ----
    cpu = None
    if not args.no_cpu_baseline:
        import oracle
        col = csc.row_indices.cpu().numpy()
        off = csc.column_offset.cpu().numpy()
        wv = csc.edge_weight.cpu().numpy()
        xh = x.cpu().numpy()
        passes, t0 = 0, time.perf_counter()
        while passes < 3 or (time.perf_counter() - t0 < 10.0 and passes < 64):
            ref = oracle.aggregate(xh, col, off, wv)
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        got = step().cpu().numpy()
        err = float(np.max(np.abs(got - ref) / (1e-6 + 1e-5 * np.abs(ref) + 1e-5)))
        t0 = time.perf_counter()
        oracle.cootocsr(ei.cpu().numpy(), w.cpu().numpy(), V)
        cpu_conv_s = time.perf_counter() - t0
        cpu = {"value": round(bytes_step / cpu_s / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
               "sample": "%d full SpMM passes of the same workload (V=%d, E=%d, F=%d), %.2f s each"
                         % (passes, V, E, F, cpu_s),
               "host_cores_available": os.cpu_count(),
               "coo_to_csr_edges_per_s": round(E / cpu_conv_s),
               "gpu_vs_cpu_max_scaled_err": round(err, 4)}

    line = {
        "metric": "spmm_f128_algorithmic_bandwidth",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "weighted CSC SpMM, V=1,000,000 Chung-Lu power-law (exp 2.1, cap 20000) "
                               "+ self-loops, gcn_norm weights, F=128", "V": V, "E": E, "F": F,
                   "bytes_per_step": bytes_step},
        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "spmm_csr_backward_ms": round(bwd_ms, 4),
        "coo_to_csr_edges_per_s": round(E / (conv_csr_ms * 1e-3)),
        "coo_to_csc_edges_per_s": round(E / (conv_csc_ms * 1e-3)),
        "coo_to_csr_ms": round(conv_csr_ms, 4),
        "gcn_layer_fwd_bwd_ms": round(gcn_ms, 4),
        "gcn_layer_shape": "GCNConv(128->128) on the same graph, aggregateWithWeight path: x@W, SpMM, bias; "
                           "backward SpMM, W.grad, x.grad",
        "gat_fused_fwd_ms": round(gat_fwd_ms, 4),
        "gat_fused_fwd_bwd_ms": round(gat_fb_ms, 4),
        "gat_fused_fwd_algorithmic_gbps": round(gat_bytes / (gat_fwd_ms * 1e-3) / 1e9, 1),
        "gat_shape": "V=%d, E=%d (power-law exp 2.3 + self-loops), 8 heads x 16" % (gV, gE),
        "edge_softmax_fwd_ms": round(esm_fwd_ms, 4),
        "edge_softmax_fwd_algorithmic_gbps": round((8 * E + 4 * (V + 1)) / (esm_fwd_ms * 1e-3) / 1e9, 1),
        "appnp_hop_f128_ms": round(hop_ms, 4),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": args.traffic_bytes,
                     "traffic_source": "profiles/bench_workload_mi355x.txt",
                     "traffic_rate_gbps": round(args.traffic_bytes / (k_ms.value * 1e-3) / 1e9, 1) if args.traffic_bytes else None,
                     "kernel": "spmm_merge<2,1,16,false,true,false>", "kernel_ms": round(k_ms.value, 4),
                     "call_ms": round(c_ms.value, 4), "algorithmic_bytes": bytes_step},
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
