"""GPU parity: walks from the HIP kernels (through the C ABI) must equal the CPU oracle bit for bit.

Integer / index work, so the bar is exact equality of the whole path matrix and of the workload
counters (steps, sum of source degrees).
"""
import numpy as np
import pytest

import _graphs
import fw_oracle_binding as _oracle

pytestmark = pytest.mark.gpu


def _check(fw, csr, starts, placement=0, **kw):
    xadj, adj, w, lab = csr
    og = _oracle.Graph(xadj, adj, w, lab)
    g = fw.Graph.from_csr(xadj, adj, w, lab, placement=placement)
    try:
        p = fw.default_params(**kw)
        paths, st = g.walk(p, starts)
    finally:
        g.destroy()
    ref, steps, edges = _oracle.walk(og, _oracle.from_walk_params(p), starts)
    bad = np.nonzero((paths != ref).any(axis=1))[0]
    assert len(bad) == 0, "first differing walk %d:\n gpu %s\n ref %s" % (bad[0], paths[bad[0]], ref[bad[0]])
    assert (st.steps, st.sampled_edges) == (steps, edges)
    return paths, st


@pytest.fixture(scope="module")
def c1_graph():
    return _graphs.uniform_graph(7115, 103689, seed=1)


@pytest.fixture(scope="module")
def hub():
    # hubs of degree ~9000 and ~2500 plus a low-degree bulk; some zero weights
    return _graphs.hub_graph(V=12000, hub_degrees=(9000, 2500, 700), base_degree=5, seed=11, zero_weight_fraction=0.05)


def test_config1_deepwalk(gpu, c1_graph):
    """Benchmark configuration 1: 7,115 vertices, 103,689 edges, 100 seeded starts, length 80."""
    starts = np.random.RandomState(1).randint(0, 7115, size=100).astype(np.int32)
    paths, st = _check(gpu, c1_graph, starts, app=gpu.APP_DEEPWALK, max_depth=81, seed=1)
    assert (paths[:, 0] == starts).all()
    assert st.steps > 0


@pytest.mark.parametrize("wg", [256, 512, 1024])
@pytest.mark.parametrize("thr", [64, 1000, 16384])
def test_deepwalk_wave_and_workgroup(gpu, hub, wg, thr):
    """Both sampler granularities: the hub threshold moves lists between the wave and workgroup samplers."""
    starts = np.random.RandomState(2).randint(0, 12000, size=3000).astype(np.int32)
    starts[:64] = 0  # the 9000-degree hub
    _check(gpu, hub, starts, app=gpu.APP_DEEPWALK, max_depth=21, wg_threads=wg, hub_threshold=thr, seed=99)


def test_ppr(gpu, hub):
    starts = np.arange(4000, dtype=np.int32)
    paths, _ = _check(gpu, hub, starts, app=gpu.APP_PPR, max_depth=81, tp=0.2, hub_threshold=1000, seed=5)
    lens = (paths >= 0).sum(axis=1) - 1
    assert 3.5 < lens.mean() < 6.5  # geometric with mean 1/tp = 5


def test_node2vec(gpu, hub):
    starts = np.arange(0, 12000, 3, dtype=np.int32)
    _check(gpu, hub, starts, app=gpu.APP_NODE2VEC, max_depth=16, p=2.0, q=0.5, hub_threshold=1000, seed=6)


def test_node2vec_on_a_multigraph(gpu):
    """Duplicate edges: neighbour lists that ascend with equal entries are accepted (fw_graph_is_sorted, the adjacency
    test is a binary search), every copy of an edge is a candidate of its own, and the walks equal the oracle's; a
    list that descends somewhere is still refused."""
    rng = np.random.RandomState(77)
    V = 3000
    deg = rng.randint(1, 40, size=V)
    deg[:3] = (2500, 900, 200)
    xadj = np.zeros(V + 1, dtype=np.uint32)
    np.cumsum(deg, out=xadj[1:])
    adj = np.concatenate([np.sort(rng.randint(0, V // 4 if d > 100 else V, size=d)) for d in deg]).astype(np.int32)
    assert any((np.diff(adj[xadj[v]:xadj[v + 1]]) == 0).any() for v in range(3))   # the hubs hold duplicates
    w = (1.0 + 9.0 * rng.random_sample(len(adj))).astype(np.float32)
    lab = rng.randint(0, 5, size=len(adj)).astype(np.int32)
    starts = rng.randint(0, V, size=4000).astype(np.int32)
    starts[:200] = 0
    for park in (-1, 16):
        for p, q in ((2.0, 0.5), (0.25, 4.0)):
            _check(gpu, (xadj, adj, w, lab), starts, app=gpu.APP_NODE2VEC, max_depth=12, p=p, q=q, hub_threshold=1000,
                   park_threshold=park, seed=31)
    bad = adj.copy()
    bad[[0, 1]] = bad[[1, 0]] if bad[0] != bad[1] else (bad[1] + 1, bad[1])
    g = gpu.Graph.from_csr(xadj, bad, w, lab)
    try:
        with pytest.raises(gpu.FlowWalkerError) as e:
            g.walk(gpu.default_params(app=gpu.APP_NODE2VEC, max_depth=3), starts[:10])
        assert "ascending neighbour lists" in str(e.value)
    finally:
        g.destroy()


def test_node2vec_on_lists_of_every_length(gpu):
    """node2vec proposes by weight and accepts with one search in N(prev): hubs of 30,000 / 20,000 / 5,000 / 600 / 70
    neighbours as cur and as prev, p < 1 < q and p > 1 > q (rejections on every kind of neighbour), wave and
    workgroup granularity, with and without parking (rejected walkers wait on their vertex for another round)."""
    csr = _graphs.hub_graph(V=40000, hub_degrees=(30000, 20000, 5000, 600, 70), base_degree=4, seed=23)
    starts = np.random.RandomState(6).randint(0, 40000, size=4000).astype(np.int32)
    starts[:300] = 0
    starts[300:500] = 1
    starts[500:600] = 2
    for thr in (64, 4096, 1 << 30):
        _check(gpu, csr, starts, app=gpu.APP_NODE2VEC, max_depth=9, p=0.5, q=2.0, hub_threshold=thr, seed=31)
    _check(gpu, csr, starts, app=gpu.APP_NODE2VEC, max_depth=9, p=4.0, q=0.25, hub_threshold=1000, wg_threads=256, seed=32)
    for park, thr in ((3, 1000), (500, 64), (2000, 100000)):
        _, st = _check(gpu, csr, starts, app=gpu.APP_NODE2VEC, max_depth=13, p=0.25, q=4.0, hub_threshold=thr,
                       park_threshold=park, seed=33)
        assert st.launches >= 3 and st.hub_steps > 0
    # 15,000 walkers on one hub: crowded buckets (rows made once per round), rejected walkers stay in them
    many = np.zeros(15000, dtype=np.int32)
    _, st = _check(gpu, csr, many, app=gpu.APP_NODE2VEC, max_depth=6, p=0.5, q=3.0, hub_threshold=4096, park_threshold=100,
                   seed=34)
    assert st.hub_steps > 0


def test_metapath(gpu, hub):
    starts = np.arange(0, 12000, 2, dtype=np.int32)
    _check(gpu, hub, starts, app=gpu.APP_METAPATH, max_depth=6, schema=[0, 1, 2, 3, 4], hub_threshold=1000, seed=7)
    _check(gpu, hub, starts, app=gpu.APP_METAPATH, max_depth=9, schema=[3, 1], hub_threshold=64, seed=8)


@pytest.mark.parametrize("wg", [256, 512, 1024])
@pytest.mark.parametrize("app", ["deepwalk", "ppr", "metapath"])
def test_hub_parking_does_not_change_results(gpu, hub, app, wg):
    """Hub parking (walkers waiting on a hub are served 64 at a time by one shared scan) is an execution
    strategy: with it forced on, every path must still equal the oracle's, which knows nothing about it."""
    starts = np.random.RandomState(4).randint(0, 12000, size=6000).astype(np.int32)
    starts[:700] = 0       # many walkers meet on the 9000-degree hub at once (several batches of 64)
    starts[700:800] = 1    # and on the 2500-degree one
    kw = dict(deepwalk=dict(app=gpu.APP_DEEPWALK, max_depth=41),
              ppr=dict(app=gpu.APP_PPR, max_depth=81, tp=0.15),
              metapath=dict(app=gpu.APP_METAPATH, max_depth=11, schema=[1, 3, 0]))[app]
    # park threshold at / above the hub threshold: workgroup batches only; below it: vertices in between are served
    # by single waves (wave-granularity sampling); 3: nearly every vertex of the graph is parked on
    for hub_thr, park in ((1000, 1000), (64, 2000), (500, 8000), (4096, 3), (100000, 600), (1000, 12)):
        _, st = _check(gpu, hub, starts, wg_threads=wg, hub_threshold=hub_thr, park_threshold=park, seed=77, **kw)
        assert st.launches >= 3                      # walk, hub batch, walk ...
        assert 0 < st.hub_steps <= st.steps


@pytest.mark.parametrize("app", ["deepwalk", "ppr", "metapath"])
def test_crowded_hub_is_scanned_once(gpu, hub, app):
    """Every query starts on the same hub (the reference's --ppr start rule, src/main.cu:277-281, with many queries):
    a bucket with hundreds of walkers on a long list is served in two passes (the list's rows once, then every
    walker from the rows), its counters are updated once per wave, and the paths still equal the oracle's.  Both
    sampler granularities: hub threshold below and above the hub's degree."""
    starts = np.zeros(20000, dtype=np.int32)            # vertex 0: the 9000-degree hub
    starts[15000:] = 1                                   # and 5000 on the 2500-degree one
    kw = dict(deepwalk=dict(app=gpu.APP_DEEPWALK, max_depth=9),
              ppr=dict(app=gpu.APP_PPR, max_depth=41, tp=0.2),
              metapath=dict(app=gpu.APP_METAPATH, max_depth=6, schema=[2, 0, 4, 1, 3]))[app]
    for hub_thr, park, wg in ((1000, 600, 512), (100000, 600, 256), (4000, 2000, 1024)):
        _, st = _check(gpu, hub, starts, wg_threads=wg, hub_threshold=hub_thr, park_threshold=park, seed=5, **kw)
        assert st.launches >= 3 and st.hub_steps >= 20000


def test_walkers_that_move_together(gpu):
    """Two centres joined to every other vertex, which are joined to the centres only: from a leaf every walker
    moves to one of two vertices, so most lanes of a wave ask for a position in the same bucket at the same time
    (one counter update per wave and bucket instead of one per walker).  Parked on everything (threshold 1)."""
    leaves = 60
    src = np.concatenate([np.zeros(leaves), np.ones(leaves), np.arange(2, leaves + 2), np.arange(2, leaves + 2)])
    dst = np.concatenate([np.arange(2, leaves + 2), np.arange(2, leaves + 2), np.zeros(leaves), np.ones(leaves)])
    xadj, adj = _graphs.csr_from_edges(leaves + 2, src.astype(np.int64), dst.astype(np.int64))
    rs = np.random.RandomState(9)
    w = rs.uniform(1.0, 9.0, size=len(adj)).astype(np.float32)
    lab = rs.randint(0, 2, size=len(adj)).astype(np.int32)
    starts = rs.randint(0, leaves + 2, size=30000).astype(np.int32)
    for kw in (dict(app=gpu.APP_DEEPWALK, max_depth=12), dict(app=gpu.APP_PPR, max_depth=30, tp=0.1),
               dict(app=gpu.APP_METAPATH, max_depth=7, schema=[0, 1, 1])):
        _, st = _check(gpu, (xadj, adj, w, lab), starts, park_threshold=1, seed=13, **kw)
        assert st.launches >= 3 and st.hub_steps > 0


def test_default_parking_rule_and_its_tail(gpu, hub):
    """park_threshold = 0: the library decides (batches of at least 65,536 queries park where about four walkers
    meet), and once few walkers are left they finish in one launch without parking.  Same paths either way."""
    xadj, adj, w, lab = hub
    starts = np.random.RandomState(8).randint(0, 12000, size=600000).astype(np.int32)  # ~50,000 of them park per round
    og = _oracle.Graph(xadj, adj, w, lab)
    g = gpu.Graph.from_csr(xadj, adj, w, lab)
    try:
        for kw in (dict(app=gpu.APP_PPR, max_depth=61, tp=0.3), dict(app=gpu.APP_DEEPWALK, max_depth=9)):
            p = gpu.default_params(seed=21, **kw)
            assert p.park_threshold == 0
            ref, steps, edges = _oracle.walk(og, _oracle.from_walk_params(p), starts)
            paths, st = g.walk(p, starts)
            assert (paths == ref).all()
            assert (st.steps, st.sampled_edges) == (steps, edges)
            assert st.launches >= 3 and 0 < st.hub_steps < st.steps
    finally:
        g.destroy()


def test_hub_parking_through_the_batch_driver(gpu, hub):
    xadj, adj, w, lab = hub
    starts = np.random.RandomState(5).randint(0, 12000, size=9000).astype(np.int32)
    starts[::7] = 0
    og = _oracle.Graph(xadj, adj, w, lab)
    g = gpu.Graph.from_csr(xadj, adj, w, lab)
    try:
        p = gpu.default_params(max_depth=31, hub_threshold=1000, park_threshold=1500, seed=3)
        ref, steps, edges = _oracle.walk(og, _oracle.from_walk_params(p), starts)
        for bs, sync in ((9000, False), (2048, False), (2500, True)):
            paths, st = g.walk_batch(p, starts, batch_size=bs, sync=sync)
            assert (paths == ref).all()
            assert (st.steps, st.sampled_edges) == (steps, edges)
        p_off = gpu.default_params(max_depth=31, hub_threshold=1000, park_threshold=-1, seed=3)
        paths, st = g.walk(p_off, starts)
        assert (paths == ref).all() and st.launches == 1
        # the other applications through the same driver, parked from a low degree on (short lists four to a wave,
        # path entries stored in pairs, node2vec's rejected walkers waiting in their buckets)
        for kw in (dict(app=gpu.APP_PPR, tp=0.1), dict(app=gpu.APP_NODE2VEC, p=2.0, q=0.5),
                   dict(app=gpu.APP_METAPATH, schema=[1, 0, 2])):
            p = gpu.default_params(max_depth=24, hub_threshold=1000, park_threshold=20, seed=11, **kw)
            ref, steps, edges = _oracle.walk(og, _oracle.from_walk_params(p), starts)
            for bs in (9000, 3001):
                paths, st = g.walk_batch(p, starts, batch_size=bs, sync=False)
                assert (paths == ref).all(), (kw, bs)
                assert (st.steps, st.sampled_edges) == (steps, edges)
    finally:
        g.destroy()


def test_result_independent_of_launch_shape(gpu, hub):
    """Row q depends only on (seed, walker id, graph, parameters): grid size, workgroup scheduling and
    batching must not change a byte (the reference is not reproducible here: include/walker.cuh:1324,1339)."""
    xadj, adj, w, lab = hub
    starts = np.random.RandomState(3).randint(0, 12000, size=5000).astype(np.int32)
    g = gpu.Graph.from_csr(xadj, adj, w, lab)
    try:
        base = None
        for grid in (0, 1, 3, 64):
            p = gpu.default_params(max_depth=31, hub_threshold=1000, seed=42, grid=grid)
            paths, st = g.walk(p, starts)
            if base is None:
                base = paths
            assert (paths == base).all(), "grid=%d changed the walks" % grid
        p = gpu.default_params(max_depth=31, hub_threshold=1000, seed=42)
        for bs, sync in ((5000, False), (777, False), (1024, True), (0, False)):
            paths, st = g.walk_batch(p, starts, batch_size=bs, sync=sync)
            assert (paths == base).all(), "batch_size=%d sync=%s changed the walks" % (bs, sync)
            assert st.launches == (1 if bs in (0, 5000) else -(-5000 // bs))
    finally:
        g.destroy()


def test_edge_cases(gpu):
    """Sinks (degree 0), all-zero weights, out-of-range start, max_depth 1, a single query."""
    # 0 -> 1 -> 2 (sink); 3 has only zero-weight edges; 4 isolated
    xadj = np.array([0, 1, 2, 2, 4, 4], dtype=np.uint32)
    adj = np.array([1, 2, 0, 1], dtype=np.int32)
    w = np.array([1.0, 2.0, 0.0, 0.0], dtype=np.float32)
    lab = np.array([0, 1, 0, 0], dtype=np.int32)
    csr = (xadj, adj, w, lab)
    starts = np.array([0, 1, 2, 3, 4, 7, -1], dtype=np.int32)
    paths, st = _check(gpu, csr, starts, max_depth=5, seed=1)
    assert paths[0].tolist() == [0, 1, 2, -1, -1]
    assert paths[2].tolist() == [2, -1, -1, -1, -1]
    assert paths[3].tolist() == [3, -1, -1, -1, -1]
    assert paths[5].tolist() == [7, -1, -1, -1, -1]
    assert st.steps == 3
    _check(gpu, csr, starts, max_depth=1, seed=1)
    _check(gpu, csr, np.array([0], dtype=np.int32), max_depth=3, seed=1)
    paths, _ = _check(gpu, csr, starts, app=gpu.APP_METAPATH, max_depth=4, schema=[0, 1], seed=1)
    assert paths[0].tolist() == [0, 1, 2, -1]


def test_rmat_generator_matches_host_definition(gpu):
    """The device generator against the numpy restatement of its definition, all arrays equal."""
    for sym in (False, True):
        g = gpu.Graph.rmat(11, edge_factor=8, symmetrise=sym, n_labels=5, seed=3)
        try:
            xadj, adj, w, lab = g.download(weights=True, labels=True)
            assert g.is_sorted()
        finally:
            g.destroy()
        rx, ra, rw, rl = _graphs.rmat_graph(11, edge_factor=8, symmetrise=sym, n_labels=5, seed=3)
        assert (xadj == rx).all() and (adj == ra).all()
        assert (w.view(np.uint32) == rw.view(np.uint32)).all()
        assert (lab == rl).all()


def test_walk_on_generated_rmat(gpu):
    """R-MAT scale 14 (directed and symmetrised), every vertex a query, against the oracle."""
    for sym, app in ((False, 0), (True, 0), (True, 2)):
        g = gpu.Graph.rmat(14, edge_factor=16, symmetrise=sym, seed=5)
        try:
            xadj, adj, w, _ = g.download()
            p = gpu.default_params(app=app, max_depth=41 if app == 0 else 11, hub_threshold=512, seed=17)
            starts = np.arange(g.V, dtype=np.int32)
            paths, st = g.walk(p, starts)
        finally:
            g.destroy()
        og = _oracle.Graph(xadj, adj, w)
        ref, steps, edges = _oracle.walk(og, _oracle.from_walk_params(p), starts)
        assert (paths == ref).all()
        assert (st.steps, st.sampled_edges) == (steps, edges)


def test_edges_in_pinned_host_memory(gpu, hub):
    """FW_GRAPH_HOST_PINNED (the reference's --umgraph, include/gpu_graph.cuh:46-54): the edge arrays stay in host
    memory and the kernels read them over the bus.  Where the arrays live changes no draw and no path: all four
    applications, the walk kernel alone and the parking pipeline, equal the oracle; downloading the graph returns
    the arrays that went in."""
    xadj, adj, w, lab = hub
    g = gpu.Graph.from_csr(xadj, adj, w, lab, placement=gpu.GRAPH_HOST_PINNED)
    try:
        back = g.download(weights=True, labels=True)
        assert g.is_sorted()
    finally:
        g.destroy()
    for a, b in zip(back, hub):
        assert (a == b).all()
    starts = np.random.RandomState(8).randint(0, 12000, size=6000).astype(np.int32)
    starts[:500] = 0
    for park in (-1, 50):
        _check(gpu, hub, starts, placement=gpu.GRAPH_HOST_PINNED, app=gpu.APP_DEEPWALK, max_depth=21,
               hub_threshold=1000, park_threshold=park, seed=41)
        _check(gpu, hub, starts, placement=gpu.GRAPH_HOST_PINNED, app=gpu.APP_PPR, max_depth=81, tp=0.2,
               hub_threshold=1000, park_threshold=park, seed=42)
        _check(gpu, hub, starts, placement=gpu.GRAPH_HOST_PINNED, app=gpu.APP_METAPATH, max_depth=6,
               schema=[0, 1, 2, 3, 4], hub_threshold=1000, park_threshold=park, seed=43)
    _check(gpu, hub, starts[:2000], placement=gpu.GRAPH_HOST_PINNED, app=gpu.APP_NODE2VEC, max_depth=11, p=2.0, q=0.5,
           hub_threshold=1000, seed=44)


def test_randomized_configurations(gpu):
    """Seeded random graphs (planted hubs up to degree 33,000, directed or undirected, zero weights), applications,
    depths, workgroup sizes, granularity and parking thresholds, start sets (spread, all on one vertex, a handful of
    vertices): every case bit-exact against the oracle."""
    rng = np.random.RandomState(20240)
    apps = [gpu.APP_DEEPWALK, gpu.APP_PPR, gpu.APP_NODE2VEC, gpu.APP_METAPATH]
    for _ in range(24):
        V = int(rng.choice([300, 2000, 9000, 40000]))
        nh = int(rng.randint(0, 5))
        hubs = tuple(int(min(V - 1, rng.choice([70, 130, 300, 1100, 2500, 5000, 17000, 33000]))) for _ in range(nh))
        csr = _graphs.hub_graph(V=V, hub_degrees=hubs, base_degree=int(rng.choice([1, 3, 8, 20])),
                                seed=int(rng.randint(1, 1 << 30)), symmetric=bool(rng.randint(0, 2)),
                                zero_weight_fraction=float(rng.choice([0.0, 0.0, 0.05, 0.5])))
        xadj, adj, w, lab = csr
        og = _oracle.Graph(xadj, adj, w, lab)
        g = gpu.Graph.from_csr(xadj, adj, w, lab)
        try:
            for _ in range(6):
                app = int(rng.choice(apps))
                depth = int(rng.choice([2, 4, 6])) if app == gpu.APP_METAPATH else int(rng.choice([2, 3, 11, 41, 81]))
                n = int(rng.choice([1, 63, 1000, 20000]))
                mode = rng.randint(0, 3)
                if mode == 0:
                    starts = rng.randint(0, V, size=n)
                elif mode == 1:
                    starts = np.full(n, rng.randint(0, nh if nh else V))
                else:
                    starts = rng.randint(0, min(V, 8), size=n)
                kw = dict(app=app, max_depth=depth, wg_threads=int(rng.choice([256, 512, 1024])),
                          hub_threshold=int(rng.choice([0, 64, 500, 1024, 16384, 1 << 30])),
                          park_threshold=int(rng.choice([-1, 0, 1, 4, 16, 64, 200, 3000])),
                          seed=int(rng.randint(0, 1 << 31)))
                if app == gpu.APP_NODE2VEC:
                    kw["p"], kw["q"] = float(rng.choice([0.25, 1.0, 2.0])), float(rng.choice([0.5, 1.0, 4.0]))
                if app == gpu.APP_PPR:
                    kw["tp"] = float(rng.choice([0.05, 0.2, 0.9]))
                if app == gpu.APP_METAPATH:
                    kw["schema"] = [int(x) for x in rng.randint(0, 5, size=depth - 1)]
                p = gpu.default_params(**kw)
                paths, st = g.walk(p, starts.astype(np.int32))
                ref, steps, edges = _oracle.walk(og, _oracle.from_walk_params(p), starts.astype(np.int32))
                bad = np.nonzero((paths != ref).any(axis=1))[0]
                assert len(bad) == 0, "hubs %s, %s: first differing walk %d:\n gpu %s\n ref %s" % (
                    hubs, kw, bad[0], paths[bad[0]], ref[bad[0]])
                assert (st.steps, st.sampled_edges) == (steps, edges), (hubs, kw)
        finally:
            g.destroy()


@pytest.mark.parametrize("static", [0, 1])
@pytest.mark.parametrize("sampler", ["ref_zprs", "ref_dprs"])
def test_reference_engine_on_wave64(gpu, hub, sampler, static):
    """FW_SAMPLER_REF_ZPRS / _DPRS: the reference's own samplers and round structure restated for 64-lane waves
    (include/sampler.cuh:46-200, include/walker.cuh:1357-1438), with the global dispenser or static assignment.  The
    oracle runs the CPU restatement of the same definition: bit-exact paths and counters, all four applications, wave
    and workgroup granularity."""
    sid = (gpu.SAMPLER_REF_ZPRS if sampler == "ref_zprs" else gpu.SAMPLER_REF_DPRS) | (gpu.SAMPLER_REF_STATIC if static else 0)
    starts = np.random.RandomState(8).randint(0, 12000, size=1500).astype(np.int32)
    starts[:40] = 0
    starts[40:60] = 1
    for kw in (dict(app=gpu.APP_DEEPWALK, max_depth=21, hub_threshold=1024, wg_threads=512),
               dict(app=gpu.APP_DEEPWALK, max_depth=11, hub_threshold=1 << 30, wg_threads=256),
               dict(app=gpu.APP_DEEPWALK, max_depth=11, hub_threshold=100, wg_threads=1024),
               dict(app=gpu.APP_PPR, max_depth=41, tp=0.15, hub_threshold=1024),
               dict(app=gpu.APP_NODE2VEC, max_depth=9, p=2.0, q=0.5, hub_threshold=2000, wg_threads=256),
               dict(app=gpu.APP_METAPATH, max_depth=7, schema=[1, 3, 0], hub_threshold=1024)):
        paths, st = _check(gpu, hub, starts, sampler=sid, seed=55, **kw)
        assert st.launches == 1 and st.hub_steps == 0  # the reference's engine never parks


@pytest.mark.parametrize("sampler", ["ref_zprs", "ref_dprs"])
def test_reference_engine_with_thread_owned_generators(gpu, hub, sampler):
    """FW_SAMPLER_REF_RNG_GLOBAL / _LDS with static assignment: the "FW" and "+ RNG" levels of the reference's ablation
    (README.md:152-163), generators that belong to the threads with their state in device memory (cuRAND's place,
    include/walker.cuh:1584-1696) or in LDS (include/myrand.cuh:83-86).  The walks are a function of the launch, which
    the oracle replays thread by thread: bit-exact paths and counters for both placements, all four applications,
    wave and workgroup granularity, several launch shapes; without static assignment the flags are refused."""
    base = (gpu.SAMPLER_REF_ZPRS if sampler == "ref_zprs" else gpu.SAMPLER_REF_DPRS) | gpu.SAMPLER_REF_STATIC
    starts = np.random.RandomState(8).randint(0, 12000, size=1500).astype(np.int32)
    starts[:40] = 0
    starts[40:60] = 1
    xadj, adj, w, lab = hub
    og = _oracle.Graph(xadj, adj, w, lab)
    g = gpu.Graph.from_csr(xadj, adj, w, lab)
    try:
        for kw in (dict(app=gpu.APP_DEEPWALK, max_depth=21, hub_threshold=1024, wg_threads=512, grid=7),
                   dict(app=gpu.APP_DEEPWALK, max_depth=11, hub_threshold=1 << 30, wg_threads=256, grid=24),
                   dict(app=gpu.APP_DEEPWALK, max_depth=11, hub_threshold=100, wg_threads=1024, grid=3),
                   dict(app=gpu.APP_PPR, max_depth=41, tp=0.15, hub_threshold=1024, grid=11),
                   dict(app=gpu.APP_NODE2VEC, max_depth=9, p=2.0, q=0.5, hub_threshold=2000, wg_threads=256, grid=5),
                   dict(app=gpu.APP_METAPATH, max_depth=7, schema=[1, 3, 0], hub_threshold=1024, grid=1000)):
            got = []
            for place in (gpu.SAMPLER_REF_RNG_LDS, gpu.SAMPLER_REF_RNG_GLOBAL):
                p = gpu.default_params(sampler=base | place, seed=55, **kw)
                paths, st = g.walk(p, starts)
                assert st.launches == 1 and st.hub_steps == 0
                ref, steps, edges = _oracle.walk_ref_threads(og, _oracle.from_walk_params(p), starts, st.grid)
                bad = np.nonzero((paths != ref).any(axis=1))[0]
                assert len(bad) == 0, "%s: first differing walk %d:\n gpu %s\n ref %s" % (kw, bad[0], paths[bad[0]], ref[bad[0]])
                assert (st.steps, st.sampled_edges) == (steps, edges)
                got.append(paths)
            assert (got[0] == got[1]).all()  # where the state lives changes what a draw costs, not its value
        p = gpu.default_params(sampler=(base & 0xFF) | gpu.SAMPLER_REF_RNG_LDS, max_depth=5, seed=1)
        with pytest.raises(gpu.FlowWalkerError) as e:
            g.walk(p, starts)
        assert e.value.status == 1 and "FW_SAMPLER_REF_STATIC" in str(e.value)
    finally:
        g.destroy()


def test_kernel_times_on_request(gpu):
    """fw_walk_params.time_kernels: the split of kernel_ms over the walk and the hub launches is measured on request
    only (an event pair per launch costs the stream time); the walks and the counters are the same either way."""
    csr = _graphs.hub_graph(V=30000, hub_degrees=(20000, 8000), base_degree=8, seed=5)
    g = gpu.Graph.from_csr(*csr)
    try:
        starts = np.random.RandomState(2).randint(0, 30000, size=200000).astype(np.int32)
        p = gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=21, seed=9)
        plain, st0 = g.walk(p, starts)
        assert st0.launches > 1 and st0.hub_steps > 0                      # the parking pipeline ran
        assert st0.kernel_ms > 0.0 and st0.walk_kernel_ms == 0.0 and st0.hub_kernel_ms == 0.0
        assert st0.requested_bytes > 0 and st0.scattered_writes > 0
        p.time_kernels = 1
        timed, st1 = g.walk(p, starts)
        assert (timed == plain).all()
        assert (st1.steps, st1.sampled_edges, st1.hub_steps, st1.launches) == \
               (st0.steps, st0.sampled_edges, st0.hub_steps, st0.launches)
        assert st1.requested_bytes == st0.requested_bytes
        assert st1.walk_kernel_ms > 0.0 and st1.hub_kernel_ms > 0.0
        assert st1.walk_kernel_ms + st1.hub_kernel_ms <= st1.kernel_ms
        paths_b, stb = g.walk_batch(p, starts, batch_size=0)
        assert (paths_b == plain).all() and stb.hub_kernel_ms > 0.0
    finally:
        g.destroy()


def test_batch_calls_reuse_their_buffers(gpu):
    """fw_walk_batch keeps its device buffers with the graph: calls of growing and shrinking size, other batch sizes,
    another application (other parking lists) and a fw_walk_device call in between all give the walks of one plain call."""
    csr = _graphs.hub_graph(V=30000, hub_degrees=(20000, 8000), base_degree=8, seed=5)
    g = gpu.Graph.from_csr(*csr)
    try:
        rng = np.random.RandomState(4)
        for app, n, bs, sync, extra in ((gpu.APP_DEEPWALK, 90000, 0, False, {}), (gpu.APP_DEEPWALK, 200000, 70001, False, {}),
                                        (gpu.APP_METAPATH, 150000, 0, False, {"schema": [0, 1, 2]}),
                                        (gpu.APP_DEEPWALK, 1000, 0, True, {}), (gpu.APP_PPR, 200000, 50000, True, {}),
                                        (gpu.APP_NODE2VEC, 120000, 60000, False, {"p": 0.5, "q": 2.0})):
            starts = rng.randint(0, 30000, size=n).astype(np.int32)
            p = gpu.default_params(app=app, max_depth=13, seed=n, **extra)
            want, st0 = g.walk(p, starts)
            got, st = g.walk_batch(p, starts, batch_size=bs, sync=sync)
            assert (got == want).all(), (app, n, bs)
            assert (st.steps, st.sampled_edges) == (st0.steps, st0.sampled_edges)
    finally:
        g.destroy()


def test_graph_destroy_returns_the_cached_buffers(gpu):
    """What the walk calls keep with a graph (parking lists, annotated adjacency, the batch call's buffers) goes with
    fw_graph_destroy: a dozen create / walk / destroy cycles leave the free device memory where it was."""
    import ctypes as C
    csr = _graphs.hub_graph(V=30000, hub_degrees=(20000, 8000), base_degree=8, seed=5)
    starts = np.random.RandomState(1).randint(0, 30000, size=300000).astype(np.int32)
    p = gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=41, seed=3)

    def free_bytes():
        f, t = C.c_size_t(0), C.c_size_t(0)
        gpu.check(gpu.lib().fw_device_mem_info(C.byref(f), C.byref(t)))
        return f.value

    def cycle():
        g = gpu.Graph.from_csr(*csr)
        try:
            a, st = g.walk_batch(p, starts, batch_size=100000)
            assert st.hub_steps > 0
            b, _ = g.walk(p, starts)
            assert (a == b).all()
        finally:
            g.destroy()

    cycle()  # what the runtime itself keeps after first use is allocated now
    before = free_bytes()
    for _ in range(12):
        cycle()
    assert abs(free_bytes() - before) <= 64 << 20  # a leak of the buffers would be 12 x 120 MB


def test_one_walk_call_at_a_time_per_graph(gpu):
    """The parking index, the parking lists and the launch record are cached in the fw_graph, so a second call on
    the same graph while one is running is refused with a status code (it used to race); afterwards the graph works
    as before, and a second graph walks while the first one is busy."""
    import threading
    import time

    csr = _graphs.hub_graph(V=30000, hub_degrees=(20000, 8000), base_degree=8, seed=5)
    g = gpu.Graph.from_csr(*csr)
    g2 = gpu.Graph.from_csr(*csr)
    n = 400000
    starts = np.random.RandomState(1).randint(0, 30000, size=n).astype(np.int32)
    long_p = gpu.default_params(app=gpu.APP_NODE2VEC, max_depth=81, seed=3)
    short_p = gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=5, seed=3)
    d_starts = gpu.DeviceBuffer.from_numpy(starts)
    d_long = gpu.DeviceBuffer(n * 81 * 4)
    d_short = gpu.DeviceBuffer(100 * 5 * 4)
    state = {"stop": False, "calls": 0, "error": None}

    def keep_busy():  # one long call after the other, for at most ten seconds
        t_end = time.time() + 10.0
        try:
            while not state["stop"] and time.time() < t_end:
                try:
                    g.walk_device(long_p, d_starts, n, d_long)
                    state["calls"] += 1
                except gpu.FlowWalkerError as e:  # the other thread's short call held the graph: that is the rule too
                    if "another walk call" not in str(e):
                        raise
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            state["error"] = e

    try:
        th = threading.Thread(target=keep_busy)
        th.start()
        refused = False
        t_end = time.time() + 9.0
        while time.time() < t_end and th.is_alive() and not refused:
            try:
                g.walk_device(short_p, d_starts, 100, d_short)  # may slip in between two long calls: try again
            except gpu.FlowWalkerError as e:
                assert e.status == 1 and "another walk call" in str(e)
                refused = True
                g2.walk_device(short_p, d_starts, 100, d_short)  # a second graph is independent
        state["stop"] = True
        th.join()
        assert state["error"] is None, state["error"]
        assert refused, "no call was refused while %d long calls ran" % state["calls"]
        paths, _ = g.walk(long_p, starts[:2000])  # the graph is free again and walks as before
        ref, _ = g2.walk(long_p, starts[:2000])
        assert (paths == ref).all()
    finally:
        for b in (d_starts, d_long, d_short):
            b.free()
        g.destroy()
        g2.destroy()


def test_random_access_calibration(gpu):
    """fw_dev_random_access_rate: refuses buffers it could index out of, and reports a rate for reads and stores."""
    import ctypes as C
    buf = gpu.DeviceBuffer(64 << 20)
    rate = C.c_double(0.0)
    L = gpu.lib()
    try:
        assert L.fw_dev_random_access_rate(buf.ptr, 0, 0, C.byref(rate)) == 1          # empty
        assert L.fw_dev_random_access_rate(buf.ptr, (64 << 20) + 4, 0, C.byref(rate)) == 1  # not a multiple of a line
        assert L.fw_dev_random_access_rate(buf.ptr, 64 << 20, 7, C.byref(rate)) == 1    # unknown mode
        assert L.fw_dev_random_access_rate(None, 64 << 20, 0, C.byref(rate)) == 1
        for mode in (0, 1, 3, 4, 5):
            gpu.check(L.fw_dev_random_access_rate(buf.ptr, 64 << 20, mode, C.byref(rate)))
            assert 1e9 < rate.value < 1e13
    finally:
        buf.free()
