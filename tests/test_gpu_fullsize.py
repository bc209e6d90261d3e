"""The benchmark configurations at their real sizes and with the library's default parameters.  The whole output is
checked through size-independent properties (the oracle would need minutes to hours for all of it): start column, -1
suffix, every hop a CSR edge, workload counters recomputed from the paths, byte-identical output under a different
launch shape.  Draws are addressed by walker id, so any row of the full job equals the oracle's walk of that walker:
the first rows, the last rows and the rows that start on the highest-degree vertices are compared bit for bit."""
import numpy as np
import pytest

import fw_oracle_binding as orc

pytestmark = pytest.mark.gpu


def _check_rows_against_oracle(xadj, adj, w, lab, p, starts, paths, k=2000, walker_base=0):
    """Rows [0, k), [n - k, n) and the (at most k) rows that start on the k highest-degree vertices."""
    og = orc.Graph(xadj, adj, w, lab)
    n = len(starts)
    deg = np.diff(xadj.astype(np.int64))
    top = np.argpartition(deg, len(deg) - k)[len(deg) - k:]
    is_top = np.zeros(len(deg), dtype=bool)
    is_top[top] = True
    hub_rows = np.nonzero(is_top[starts])[0][:k]
    rows = np.unique(np.concatenate([np.arange(min(k, n)), np.arange(max(n - k, 0), n), hub_rows]))
    op = orc.from_walk_params(p)
    ref = orc.walk_ids(og, op, starts[rows], (rows + walker_base).astype(np.uint32))
    bad = np.nonzero((paths[rows] != ref).any(axis=1))[0]
    assert len(bad) == 0, "row %d differs:\n gpu %s\n ref %s" % (rows[bad[0]], paths[rows[bad[0]]], ref[bad[0]])
    print("oracle rows compared: %d (of which start on a top-%d vertex: %d, max degree %d)" % (
        len(rows), k, len(hub_rows), deg.max()), flush=True)


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
        _check_rows_against_oracle(xadj, adj, w, None, p, starts, paths)
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
        _check_rows_against_oracle(xadj, adj, w, None, p, starts, paths)
        assert L.max() <= 81
    finally:
        g.destroy()


def test_config4_rmat24_symmetrised(gpu):
    """Headline graph: DeepWalk and node2vec (p = 2, q = 0.5, then two points where the acceptance step rejects more
    often), one query per vertex each, library defaults."""
    g = gpu.Graph.rmat(24, 16, symmetrise=True, seed=1)
    try:
        assert g.is_sorted()
        xadj, adj, w, _ = g.download()
        starts = np.arange(g.V, dtype=np.int32)
        p = gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=81, seed=1)
        print("deepwalk, %d queries" % g.V, flush=True)
        paths, st = g.walk(p, starts)
        assert st.launches > 3 and st.hub_steps > 0                             # the default rule parks at this size
        L = _check_paths(xadj, adj, paths, starts, st, 81, sample=50000)
        deg = np.diff(xadj.astype(np.int64))
        assert (L[deg > 0] == 81).all()                                         # undirected: no dead ends
        _check_rows_against_oracle(xadj, adj, w, None, p, starts, paths)
        del paths
        p = gpu.default_params(app=gpu.APP_NODE2VEC, max_depth=81, p=2.0, q=0.5, seed=1)
        print("node2vec, %d queries" % g.V, flush=True)
        paths, st = g.walk(p, starts)
        print("node2vec done: %.0f ms" % st.kernel_ms, flush=True)
        L = _check_paths(xadj, adj, paths, starts, st, 81, sample=50000)
        assert (L[deg > 0] == 81).all()
        _check_rows_against_oracle(xadj, adj, w, None, p, starts, paths, k=700)
        # away from the benchmark's parameters: q > 1 takes about q trials per step where most proposals are not
        # adjacent to the previous vertex (more pipeline rounds), and 1/p > max(1, 1/q) makes the return edge's excess a
        # component of its own of every trial; the same law
        for pp, qq in ((4.0, 0.25), (0.25, 4.0)):
            del paths
            p = gpu.default_params(app=gpu.APP_NODE2VEC, max_depth=81, p=pp, q=qq, seed=1)
            print("node2vec p = %g, q = %g, %d queries" % (pp, qq, g.V), flush=True)
            paths, st = g.walk(p, starts)
            print("node2vec done: %.0f ms, %d launches" % (st.kernel_ms, st.launches), flush=True)
            L = _check_paths(xadj, adj, paths, starts, st, 81, sample=50000)
            assert (L[deg > 0] == 81).all()
            _check_rows_against_oracle(xadj, adj, w, None, p, starts, paths, k=200)
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
        _check_rows_against_oracle(xadj, adj, None, lab, p, starts, paths, k=20000)
    finally:
        g.destroy()


def test_csr_offsets_above_two_to_the_31(gpu):
    """A CSR with more than 2^31 entries (the format's offsets are uint32, include/graph.cuh:93-136): the walkers
    live on the vertices whose lists start above 2^31, among them eight lists of 200,000 neighbours (workgroup
    sampler, crowded buckets) and 32,760 of 520 (wave sampler, parked or not).  Bit-exact against the oracle."""
    V, d, n_hubs, d_hub, C = 1 << 22, 520, 8, 200_000, 1 << 15
    deg = np.full(V, d, dtype=np.int64)
    deg[-n_hubs:] = d_hub
    xadj64 = np.concatenate(([0], np.cumsum(deg)))
    E = int(xadj64[-1])
    assert (1 << 31) < E < (1 << 32) - 16
    xadj = xadj64.astype(np.uint32)
    first = V - C                                  # the community the walkers stay in; its lists start above 2^31
    assert xadj64[first] > (1 << 31)
    rng = np.random.default_rng(5)
    # below the community: any valid graph will do, nobody walks there (every edge leads to vertex 0, weight 1)
    adj = np.zeros(E, dtype=np.int32)
    w = np.ones(E, dtype=np.float32)
    lo = int(xadj64[first])
    m = E - lo
    inside = rng.integers(first, V, size=m, dtype=np.int32)
    to_hub = rng.random(m) < 0.2                   # a fifth of the steps lands on one of the eight long lists
    inside[to_hub] = (V - n_hubs + rng.integers(0, n_hubs, size=int(to_hub.sum()))).astype(np.int32)
    adj[lo:] = inside
    w[lo:] = (1.0 + 99.0 * rng.random(m, dtype=np.float32)).astype(np.float32)
    w[lo:][rng.random(m) < 0.05] = 0.0
    print("graph made: E = %d" % E, flush=True)

    g = gpu.Graph.from_csr(xadj, adj, w, None)
    og = orc.Graph(xadj, adj, w, None)
    starts = rng.integers(first, V, size=20_000).astype(np.int32)
    starts[:1000] = V - 1
    try:
        for kw in (dict(app=gpu.APP_DEEPWALK, max_depth=11, park_threshold=100, seed=71),
                   dict(app=gpu.APP_DEEPWALK, max_depth=11, park_threshold=-1, seed=72),
                   dict(app=gpu.APP_PPR, max_depth=21, tp=0.15, park_threshold=100, hub_threshold=1000, seed=73)):
            p = gpu.default_params(**kw)
            print("walk", kw, flush=True)
            paths, st = g.walk(p, starts)
            ref, steps, edges = orc.walk(og, orc.from_walk_params(p), starts)
            assert (paths == ref).all(), kw
            assert (st.steps, st.sampled_edges) == (steps, edges)
            assert (paths[:, 1] >= first).all()
    finally:
        g.destroy()


def test_path_matrix_of_more_than_two_to_the_32_entries(gpu):
    """54 million walks of length 80: the path matrix has 4.4e9 entries, so a walker's row starts beyond what 32 bits
    index for every query past 53 million.  The first and the last rows equal the oracle's walks with the same
    walker ids (draws are addressed by walker id), with parking (crowded buckets of millions) and without."""
    import _graphs

    xadj, adj, w, lab = _graphs.hub_graph(V=12000, hub_degrees=(9000, 2500, 700), base_degree=5, seed=11)
    n, depth, k = 54_000_000, 81, 4000
    assert n * depth > (1 << 32)
    starts = (np.arange(n, dtype=np.int64) * 7919 % 12000).astype(np.int32)
    g = gpu.Graph.from_csr(xadj, adj, w, lab)
    og = orc.Graph(xadj, adj, w, lab)
    try:
        for park in (0, -1):
            p = gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=depth, hub_threshold=1000, park_threshold=park, seed=91)
            print("walk park", park, flush=True)
            paths, st = g.walk(p, starts)
            assert (paths[:, 0] == starts).all()
            assert st.steps == int((paths[:, 1:] >= 0).sum(dtype=np.int64))
            head, _, _ = orc.walk(og, orc.from_walk_params(p), starts[:k])
            assert (paths[:k] == head).all()
            p.walker_base = n - k
            tail, _, _ = orc.walk(og, orc.from_walk_params(p), starts[n - k:])
            assert (paths[n - k:] == tail).all()
            del paths
    finally:
        g.destroy()
