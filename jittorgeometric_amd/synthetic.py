"""Seeded synthetic graphs of the benchmark configurations (numpy, host side).

Every generator returns `edge_index` as an int32 [2, E] array in the order a
user would hand it to gcn_norm / cootocsr: no sorting by source or
destination, duplicates kept (the reference conversion does not deduplicate),
self-loops removed (gcn_norm appends one per node afterwards).
"""
import numpy as np


def _sample_endpoints(rng, weights, n_edges, chunk=1 << 22, threads=8):
    """n_edges draws with P(i) proportional to weights[i].  The uniforms come from
    `rng` in one sequence; the table look-ups (the slow part, and independent of
    one another) are spread over a few threads."""
    from concurrent.futures import ThreadPoolExecutor
    cdf = np.cumsum(weights, dtype=np.float64)
    cdf /= cdf[-1]
    out = np.empty(n_edges, np.int32)
    top = len(weights) - 1

    def look_up(args):
        s, u = args
        out[s:s + len(u)] = np.minimum(np.searchsorted(cdf, u, side="right"), top)

    def chunks():
        for s in range(0, n_edges, chunk):
            yield s, rng.random(min(n_edges, s + chunk) - s)

    if n_edges <= chunk:
        for c in chunks():
            look_up(c)
        return out
    with ThreadPoolExecutor(max_workers=threads) as pool:
        pending = []
        for c in chunks():
            pending.append(pool.submit(look_up, c))
            if len(pending) >= 2 * threads:          # bounds the uniforms held at once
                pending.pop(0).result()
        for f in pending:
            f.result()
    return out


def powerlaw_weights(num_nodes, exponent, mean_degree, max_degree=None):
    """Expected degrees d_i ~ (i + i0)^(-1/(exponent-1)), scaled to the mean
    and capped (the scale is re-fitted after capping)."""
    alpha = 1.0 / (exponent - 1.0)
    base = (np.arange(num_nodes, dtype=np.float64) + 1.0) ** (-alpha)
    w = base * (mean_degree * num_nodes / base.sum())
    if max_degree is not None:
        for _ in range(50):
            w = np.minimum(w, max_degree)
            free = w < max_degree
            deficit = mean_degree * num_nodes - w.sum()
            if deficit <= 1e-6 * mean_degree * num_nodes or not free.any():
                break
            w[free] *= 1.0 + deficit / w[free].sum()
        w = np.minimum(w, max_degree)
    return w


def chung_lu(num_nodes, num_edges, exponent, max_degree=None, seed=0):
    """Directed Chung-Lu graph: both endpoints drawn proportional to a
    power-law expected-degree sequence; node ids are shuffled so hubs are
    spread over the id range; self-loops dropped."""
    rng = np.random.default_rng(seed)
    w = powerlaw_weights(num_nodes, exponent, num_edges / num_nodes, max_degree)
    relabel = rng.permutation(num_nodes).astype(np.int32)
    src = relabel[_sample_endpoints(rng, w, num_edges)]
    dst = relabel[_sample_endpoints(rng, w, num_edges)]
    keep = src != dst
    return np.stack([src[keep], dst[keep]])


def uniform_undirected(num_nodes, num_pairs, seed=0):
    """num_pairs distinct unordered pairs u != v, both directions emitted
    back to back in generated order (the Cora-like small configuration)."""
    rng = np.random.default_rng(seed)
    seen = set()
    src, dst = [], []
    while len(seen) < num_pairs:
        u, v = (int(t) for t in rng.integers(0, num_nodes, 2))
        if u == v:
            continue
        key = (min(u, v), max(u, v))
        if key in seen:
            continue
        seen.add(key)
        src += [u, v]
        dst += [v, u]
    return np.array([src, dst], np.int32)


def lognormal_degree(num_nodes, mean_degree, sigma=1.0, seed=0):
    """Out-degrees round(lognormal) with the requested mean, destinations
    uniform, edges of one source contiguous (as an adjacency-list dump is),
    self-loops dropped."""
    rng = np.random.default_rng(seed)
    mu = np.log(mean_degree) - 0.5 * sigma * sigma
    # Normal variates from two uniforms each (Box-Muller), not from the generator's own normal
    # sampler: that one rejects and redraws on a comparison of library logarithms, so a last-bit
    # difference between two hosts' math libraries shifts every later draw and the graph comes
    # out with another edge count.  Here such a difference can only move one degree by one.
    u1, u2 = rng.random(num_nodes), rng.random(num_nodes)
    z = np.sqrt(-2.0 * np.log1p(-u1)) * np.cos(2.0 * np.pi * u2)
    deg = np.maximum(np.rint(np.exp(mu + sigma * z)), 0).astype(np.int64)
    src = np.repeat(np.arange(num_nodes, dtype=np.int32), deg)
    dst = rng.integers(0, num_nodes, src.shape[0], dtype=np.int32)
    keep = src != dst
    return np.stack([src[keep], dst[keep]])


CONFIGS = {
    # name: (generator, kwargs) -- sizes of the benchmark configurations
    "cora_like": (uniform_undirected, dict(num_nodes=2708, num_pairs=5278, seed=1)),
    "powerlaw_1m": (chung_lu, dict(num_nodes=1_000_000, num_edges=16_000_000, exponent=2.1,
                                   max_degree=20_000, seed=2)),
    "gat_169k": (chung_lu, dict(num_nodes=169_343, num_edges=1_166_243, exponent=2.3, seed=3)),
    "dense_233k": (lognormal_degree, dict(num_nodes=232_965, mean_degree=492.0, sigma=1.0, seed=4)),
    "powerlaw_2m4": (chung_lu, dict(num_nodes=2_449_029, num_edges=123_700_000, exponent=2.1, seed=5)),
}


def make(name):
    gen, kw = CONFIGS[name]
    return gen(**kw), kw["num_nodes"]
