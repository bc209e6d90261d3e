"""Deterministic synthetic CSR graphs for the tests (numpy, host side)."""
import numpy as np


def csr_from_edges(V, src, dst, sort_lists=True):
    """Deduplicated, self-loop-free CSR from directed edge arrays."""
    src = np.asarray(src, dtype=np.int64)
    dst = np.asarray(dst, dtype=np.int64)
    keep = src != dst
    key = np.unique(src[keep] * V + dst[keep])
    s = (key // V).astype(np.int64)
    d = (key % V).astype(np.int32)
    xadj = np.zeros(V + 1, dtype=np.uint32)
    np.cumsum(np.bincount(s, minlength=V), out=xadj[1:])
    return xadj, d


def uniform_graph(V=7115, E=103689, seed=1, w_lo=1.0, w_hi=5.0, n_labels=5):
    """Directed uniform-random graph with exactly E distinct (src != dst) edges, seeded."""
    rng = np.random.RandomState(seed)
    keys = np.empty(0, dtype=np.int64)
    while len(keys) < E:
        need = int((E - len(keys)) * 1.2) + 16
        s = rng.randint(0, V, size=need).astype(np.int64)
        d = rng.randint(0, V, size=need).astype(np.int64)
        k = (s * V + d)[s != d]
        keys = np.unique(np.concatenate([keys, k]))
    if len(keys) > E:
        keys = np.sort(rng.choice(keys, size=E, replace=False))
    s = keys // V
    d = (keys % V).astype(np.int32)
    xadj = np.zeros(V + 1, dtype=np.uint32)
    np.cumsum(np.bincount(s, minlength=V), out=xadj[1:])
    weight = (w_lo + (w_hi - w_lo) * rng.random_sample(E)).astype(np.float32)
    label = rng.randint(0, n_labels, size=E).astype(np.int32)
    return xadj, d, weight, label


def hub_graph(V=3000, hub_degrees=(5000,), base_degree=6, seed=7, w_lo=1.0, w_hi=100.0, n_labels=5, symmetric=True,
              zero_weight_fraction=0.0):
    """Small-world style graph with a few planted hubs (degree may exceed V-1 only if V allows it).

    Neighbour lists are ascending and duplicate free; with symmetric=True the graph is undirected and both
    directions of an edge carry the same weight and label.
    """
    rng = np.random.RandomState(seed)
    src = [np.repeat(np.arange(V), base_degree)]
    dst = [rng.randint(0, V, size=V * base_degree)]
    for h, deg in enumerate(hub_degrees):
        nbrs = rng.choice(V, size=min(deg, V - 1), replace=False)
        src.append(np.full(len(nbrs), h))
        dst.append(nbrs)
    src = np.concatenate(src).astype(np.int64)
    dst = np.concatenate(dst).astype(np.int64)
    if symmetric:
        src, dst = np.concatenate([src, dst]), np.concatenate([dst, src])
    xadj, adj = csr_from_edges(V, src, dst)
    E = len(adj)
    s = np.repeat(np.arange(V, dtype=np.int64), np.diff(xadj.astype(np.int64)))
    lo = np.minimum(s, adj)
    hi = np.maximum(s, adj)
    pair = lo * V + hi
    # weight / label are functions of the unordered pair, so both directions agree
    uniq, inv = np.unique(pair, return_inverse=True)
    wu = (w_lo + (w_hi - w_lo) * rng.random_sample(len(uniq))).astype(np.float32)
    if zero_weight_fraction > 0:
        wu[rng.random_sample(len(uniq)) < zero_weight_fraction] = 0.0
    lu = rng.randint(0, n_labels, size=len(uniq)).astype(np.int32)
    return xadj, adj, wu[inv], lu[inv]


# ---- host mirror of the device R-MAT generator (integer arithmetic on Philox4x32-10 draws) ----

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10_np(c0, c1, c2, c3, k0, k1):
    """Vectorised Philox4x32-10 over uint64-held 32-bit words."""
    c0, c1, c2, c3 = [np.asarray(x, dtype=np.uint64) & _MASK for x in (c0, c1, c2, c3)]
    k0 = np.uint64(k0) & _MASK
    k1 = np.uint64(k1) & _MASK
    for _ in range(10):
        p0 = _M0 * c0
        p1 = _M1 * c2
        n0 = (p1 >> np.uint64(32)) ^ c1 ^ k0
        n1 = p1 & _MASK
        n2 = (p0 >> np.uint64(32)) ^ c3 ^ k1
        n3 = p0 & _MASK
        c0, c1, c2, c3 = n0, n1, n2, n3
        k0 = (k0 + np.uint64(0x9E3779B9)) & _MASK
        k1 = (k1 + np.uint64(0xBB67AE85)) & _MASK
    return c0, c1, c2, c3


def rmat_graph(scale, edge_factor=16, a=0.57, b=0.19, c=0.19, symmetrise=False, w_lo=1.0, w_hi=100.0, n_labels=0,
               make_weights=True, seed=1):
    """Host restatement of the device generator's published definition; returns (xadj, adjncy, weight, label)."""
    V = 1 << scale
    n_gen = edge_factor << scale
    a, b, c = float(np.float32(a)), float(np.float32(b)), float(np.float32(c))
    thr = lambda x: min(int(x * 4294967296.0), 0xFFFFFFFF)
    ta, tab, tabc = thr(a), thr(a + b), thr(a + b + c)
    k0, k1 = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
    e = np.arange(n_gen, dtype=np.uint64)
    src = np.zeros(n_gen, dtype=np.uint64)
    dst = np.zeros(n_gen, dtype=np.uint64)
    r = None
    for i in range(scale):
        if i % 4 == 0:
            r = philox4x32_10_np(e & _MASK, e >> np.uint64(32), np.full(n_gen, i >> 2, dtype=np.uint64),
                                 np.full(n_gen, 0x524D4154, dtype=np.uint64), k0, k1)
        x = r[i % 4]
        row = (x >= tab).astype(np.uint64)
        col = (((x >= ta) & (x < tab)) | (x >= tabc)).astype(np.uint64)
        src = (src << np.uint64(1)) | row
        dst = (dst << np.uint64(1)) | col
    keep = src != dst
    s, d = src[keep], dst[keep]
    if symmetrise:
        s, d = np.concatenate([s, d]), np.concatenate([d, s])
    key = np.unique((s << np.uint64(32)) | d)
    s = (key >> np.uint64(32)).astype(np.int64)
    d = (key & _MASK).astype(np.int64)
    xadj = np.zeros(V + 1, dtype=np.uint32)
    np.cumsum(np.bincount(s, minlength=V), out=xadj[1:])
    weight = label = None
    if make_weights or n_labels > 0:
        lo, hi = np.minimum(s, d), np.maximum(s, d)
        z = np.zeros(len(lo), dtype=np.uint64)
        r = philox4x32_10_np(lo, hi, z, np.full(len(lo), 0x45444745, dtype=np.uint64), k0, k1)
        if make_weights:
            u = (r[0] >> np.uint64(8)).astype(np.float32) * np.float32(2.0 ** -24)
            scaled = np.float32(np.float32(w_hi) - np.float32(w_lo)) * u
            weight = (np.float32(w_lo) + scaled).astype(np.float32)
        if n_labels > 0:
            label = ((r[1] * np.uint64(n_labels)) >> np.uint64(32)).astype(np.int32)
    return xadj, d.astype(np.int32), weight, label
