"""Per-vertex transition frequencies from the HIP kernels must follow the bias-proportional law:
chi-square p > 0.01 over 1e7 samples on hub vertices, for every application and both sampler granularities."""
import numpy as np
import pytest
from scipy.stats import chisquare

import _graphs

pytestmark = pytest.mark.gpu
N = 10_000_000


@pytest.fixture(scope="module")
def hub_graph(gpu):
    csr = _graphs.hub_graph(V=40000, hub_degrees=(30000, 6000, 1500), base_degree=6, seed=21, zero_weight_fraction=0.03)
    g = gpu.Graph.from_csr(*csr)
    yield g, csr
    g.destroy()


def _first_steps(fw, g, vertex, **kw):
    p = fw.default_params(max_depth=2, **kw)
    paths, st = g.walk(p, np.full(N, vertex, dtype=np.int32))
    assert st.steps == N
    return paths[:, 1]


@pytest.mark.parametrize("hub,thr", [(0, 1 << 30), (0, 4096), (1, 1 << 30), (1, 1024), (2, 1 << 30)])
def test_deepwalk_hub_frequencies(gpu, hub_graph, hub, thr):
    g, (xadj, adj, w, lab) = hub_graph
    lo, hi = int(xadj[hub]), int(xadj[hub + 1])
    nxt = _first_steps(gpu, g, hub, app=gpu.APP_DEEPWALK, hub_threshold=thr, seed=100 + hub)
    cnt = np.bincount(nxt, minlength=g.V).astype(np.float64)
    exp = np.zeros(g.V)
    exp[adj[lo:hi]] = w[lo:hi].astype(np.float64)
    m = exp > 0
    assert cnt[~m].sum() == 0                                   # zero-weight neighbours are never taken
    assert chisquare(cnt[m], exp[m] * N / exp.sum()).pvalue > 0.01


def test_metapath_hub_frequencies(gpu, hub_graph):
    g, (xadj, adj, w, lab) = hub_graph
    nxt = _first_steps(gpu, g, 0, app=gpu.APP_METAPATH, schema=[3], hub_threshold=4096, seed=7)
    match = adj[xadj[0]:xadj[1]][lab[xadj[0]:xadj[1]] == 3]
    cnt = np.bincount(nxt, minlength=g.V)
    assert cnt[match].sum() == N                                 # only edges with the wanted label
    assert chisquare(cnt[match]).pvalue > 0.01                   # weights ignored: uniform among them


def test_ppr_lengths(gpu, hub_graph):
    g, (xadj, adj, w, lab) = hub_graph
    tp, d, n = 0.2, 30, 2_000_000
    starts = np.random.RandomState(5).randint(0, g.V, size=n).astype(np.int32)
    paths, st = g.walk(gpu.default_params(app=gpu.APP_PPR, max_depth=d + 1, tp=tp, seed=9), starts)
    L = (paths >= 0).sum(axis=1) - 1
    dead = L < d                                                   # walks that ended before the cap ...
    last = paths[np.arange(n), L]
    lo, hi = xadj[last].astype(np.int64), xadj[last + 1].astype(np.int64)
    csum = np.concatenate([[0.0], np.cumsum(w.astype(np.float64))])
    deadend = (csum[hi] - csum[lo]) == 0                           # ... at a vertex with no positive weight
    ok = ~(dead & deadend)
    exp = np.array([(1 - tp) ** (k - 1) * tp for k in range(1, d)] + [(1 - tp) ** (d - 1)])
    obs = np.bincount(L[ok], minlength=d + 1)[1:]
    # dead ends are rare here; compare the remaining walks with the geometric law
    assert deadend.mean() < 0.2
    assert chisquare(obs, exp * obs.sum()).pvalue > 0.01
    assert abs(L[ok].mean() - 1 / tp) < 0.2


@pytest.mark.parametrize("pp,qq", [(2.0, 0.5), (0.25, 4.0), (0.02, 1.0), (0.4, 0.5)])
def test_node2vec_second_step_frequencies(gpu, pp, qq):
    """Vertex P hangs on hub H with a heavy edge and shares 60 neighbours with it.  From P the first step goes to H
    almost surely; the second step must follow w/p (back to P), w (common neighbours), w/q (others).  With 1/p above
    max(1, 1/q) the return edge's excess is a component of its own of the trial (the last three points; at p = 0.02 a
    good part of the steps goes back)."""
    rng = np.random.RandomState(3)
    V, H, P = 20000, 0, 1
    hub_nb = rng.choice(np.arange(2, V), size=6000, replace=False)
    common = hub_nb[:60]
    src = np.concatenate([np.full(len(hub_nb), H), np.full(len(common), P), [P]])
    dst = np.concatenate([hub_nb, common, [H]])
    xadj, adj = _graphs.csr_from_edges(V, np.concatenate([src, dst]), np.concatenate([dst, src]))
    s = np.repeat(np.arange(V), np.diff(xadj.astype(np.int64)))
    pair = np.minimum(s, adj).astype(np.int64) * V + np.maximum(s, adj)
    uniq, inv = np.unique(pair, return_inverse=True)
    wu = (1.0 + 99.0 * rng.random_sample(len(uniq))).astype(np.float32)
    w = wu[inv]
    w[(pair == min(H, P) * V + max(H, P))] = 1.0e6
    g = gpu.Graph.from_csr(xadj, adj, w)
    try:
        for thr in (1 << 30, 1024):
            prm = gpu.default_params(app=gpu.APP_NODE2VEC, max_depth=3, p=pp, q=qq, hub_threshold=thr, seed=thr % 97)
            paths, _ = g.walk(prm, np.full(N, P, dtype=np.int32))
            sel = paths[paths[:, 1] == H, 2]
            assert len(sel) > 0.99 * N
            lo, hi = int(xadj[H]), int(xadj[H + 1])
            pset = set(adj[xadj[P]:xadj[P + 1]].tolist())
            exp = np.zeros(V)
            for i in range(lo, hi):
                t = int(adj[i])
                exp[t] = w[i] / pp if t == P else (w[i] if t in pset else w[i] / qq)
            cnt = np.bincount(sel, minlength=V).astype(np.float64)
            m = exp > 0
            assert cnt[~m].sum() == 0
            assert chisquare(cnt[m], exp[m] * len(sel) / exp.sum()).pvalue > 0.01
    finally:
        g.destroy()


@pytest.mark.parametrize("kind", ["its", "rjs", "als"])
@pytest.mark.parametrize("workgroup,list_len", [(False, 40), (False, 700), (True, 700), (True, 5000)])
def test_baseline_sampler_frequencies(gpu, kind, workgroup, list_len):
    """fw_sampler_baseline_run: the three textbook samplers draw index i with probability w_i / sum(w); zero weights
    are never drawn, an all-zero slice and a slice beyond the array answer -1."""
    rng = np.random.RandomState(list_len)
    w = np.stack([rng.uniform(0.5, 20.0, list_len), np.zeros(list_len), rng.uniform(1.0, 2.0, list_len)]).astype(np.float32)
    w[0, rng.rand(list_len) < 0.1] = 0.0
    w[0, list_len // 3] = 60.0                                   # one heavy element: rejection needs several rounds
    n = 2_000_000
    tasks = np.zeros(n, dtype=np.uint32)
    tasks[-3:] = (1, 2, 3)                                       # slice 1 is all zero, slice 3 does not exist
    k = {"its": gpu.BASELINE_ITS, "rjs": gpu.BASELINE_RJS, "als": gpu.BASELINE_ALS}[kind]
    out, ms = gpu.sampler_baseline(k, w.reshape(-1), list_len, tasks=tasks, workgroup=workgroup, seed=77)
    assert ms > 0 and out[-3] == -1 and out[-1] == -1 and 0 <= out[-2] < list_len
    draws = out[:-3]
    assert draws.min() >= 0 and draws.max() < list_len
    cnt = np.bincount(draws, minlength=list_len).astype(np.float64)
    exp = w[0].astype(np.float64)
    m = exp > 0
    assert cnt[~m].sum() == 0
    assert chisquare(cnt[m], exp[m] * len(draws) / exp.sum()).pvalue > 0.01
    again, _ = gpu.sampler_baseline(k, w.reshape(-1), list_len, tasks=tasks, workgroup=workgroup, seed=77)
    assert np.array_equal(again, out)                            # deterministic in the seed
