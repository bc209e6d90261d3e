"""The benchmark configurations at their real sizes, checked through size-independent properties
(the oracle would need minutes to hours at these sizes): start column, -1 suffix, every hop a CSR edge, workload
counters recomputed from the paths, and byte-identical output under a different launch shape."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _check_paths(xadj, adj, paths, starts, st, max_depth, sample=200000, label=None, schema=None):
    n = len(starts)
    assert (paths[:, 0] == starts).all()
    live = paths >= 0
    L = live.sum(axis=1)
    assert (live == (np.arange(max_depth)[None, :] < L[:, None])).all()       # -1 only as a suffix
    assert st.steps == int((L - 1).sum())
    deg = np.diff(xadj.astype(np.int64))
    src = paths[:, :-1]
    hop = live[:, 1:]
    assert st.sampled_edges == int(deg[src[hop]].sum())                         # src/main.cu:101-103
    # every hop of a sample of walks is a CSR edge (binary search in the ascending lists)
    rows = np.random.RandomState(0).choice(n, size=min(sample, n), replace=False)
    a = paths[rows, :-1][live[rows, 1:]].astype(np.int64)
    b = paths[rows, 1:][live[rows, 1:]].astype(np.int64)
    lo, hi = xadj[a].astype(np.int64), xadj[a + 1].astype(np.int64)
    while (lo < hi).any():
        mid = (lo + hi) // 2
        go = adj[np.minimum(mid, len(adj) - 1)] < b
        act = lo < hi
        lo = np.where(act & go, mid + 1, lo)
        hi = np.where(act & ~go, mid, hi)
    assert (lo < xadj[a + 1]).all() and (adj[np.minimum(lo, len(adj) - 1)] == b).all()
    if label is not None:
        step = np.broadcast_to(np.arange(max_depth - 1)[None, :], (len(rows), max_depth - 1))[live[rows, 1:]]
        assert (label[lo] == np.asarray(schema)[step % len(schema)]).all()
    return L


def test_config2_deepwalk_rmat22(gpu):
    g = gpu.Graph.rmat(22, 16, symmetrise=False, seed=1)
    try:
        xadj, adj, w, _ = g.download()
        starts = np.arange(g.V, dtype=np.int32)
        p = gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=81, seed=1)
        paths, st = g.walk_batch(p, starts, batch_size=0)                       # --all: autobatch
        L = _check_paths(xadj, adj, paths, starts, st, 81)
        deg = np.diff(xadj.astype(np.int64))
        assert (L[deg == 0] == 1).all()                                         # sinks: the walk is its start
        p2 = gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=81, seed=1, grid=97)
        again, _ = g.walk_batch(p2, starts, batch_size=1_000_003)               # other grid, uneven batches
        assert (again == paths).all()
    finally:
        g.destroy()


def test_config3_ppr_rmat22(gpu):
    g = gpu.Graph.rmat(22, 16, symmetrise=False, seed=1)
    try:
        xadj, adj, w, _ = g.download()
        starts = np.arange(g.V, dtype=np.int32)
        p = gpu.default_params(app=gpu.APP_PPR, max_depth=81, tp=0.2, seed=1)
        paths, st = g.walk(p, starts)
        L = _check_paths(xadj, adj, paths, starts, st, 81)
        assert L.max() <= 81
    finally:
        g.destroy()


def test_config4_rmat24_symmetrised(gpu):
    """Headline graph: DeepWalk from every vertex and node2vec (p = 2, q = 0.5) on a 2M-query prefix."""
    g = gpu.Graph.rmat(24, 16, symmetrise=True, seed=1)
    try:
        assert g.is_sorted()
        xadj, adj, _, _ = g.download(weights=False)
        starts = np.arange(g.V, dtype=np.int32)
        p = gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=81, seed=1)
        paths, st = g.walk(p, starts)
        L = _check_paths(xadj, adj, paths, starts, st, 81, sample=50000)
        deg = np.diff(xadj.astype(np.int64))
        assert (L[deg > 0] == 81).all()                                         # undirected: no dead ends
        del paths
        sub = starts[:2_000_000]
        p = gpu.default_params(app=gpu.APP_NODE2VEC, max_depth=81, p=2.0, q=0.5, seed=1)
        paths, st = g.walk(p, sub)
        _check_paths(xadj, adj, paths, sub, st, 81, sample=50000)
    finally:
        g.destroy()


def test_config5_metapath_rmat26(gpu):
    g = gpu.Graph.rmat(26, 16, symmetrise=False, n_labels=5, make_weights=False, seed=1)
    try:
        md, _ = g.max_degree()
        assert md > 100000                                                       # hubs beyond 1e5
        xadj, adj, _, lab = g.download(weights=False, labels=True)
        starts = np.random.RandomState(12345).randint(0, g.V, size=10_000_000).astype(np.int32)
        schema = [0, 1, 2, 3, 4]
        p = gpu.default_params(app=gpu.APP_METAPATH, max_depth=6, schema=schema, seed=1)
        paths, st = g.walk(p, starts)
        _check_paths(xadj, adj, paths, starts, st, 6, sample=500000, label=lab, schema=schema)
    finally:
        g.destroy()
