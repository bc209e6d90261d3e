"""CPU tests that pin the oracle: known-answer vectors, an independent model, closed forms, invariants."""
import json
import os

import numpy as np
import pytest
from scipy.stats import chisquare

import _graphs
import _model
import fw_oracle_binding as orc

HERE = os.path.dirname(os.path.abspath(__file__))


# ---- RNG ------------------------------------------------------------------------------------------

def test_philox_known_answers():
    kat = json.load(open(os.path.join(HERE, "golden", "philox4x32_10_kat.json")))
    assert len(kat["vectors"]) >= 3
    for v in kat["vectors"]:
        assert orc.philox(v["ctr"], v["key"]) == v["out"]
        assert _model.philox(v["ctr"], v["key"]) == v["out"]


def test_uniform_is_24_bit_and_matches_philox_words():
    seed = 0x1234567890ABCDEF
    for n in range(9):
        bits = orc.philox([77, 3, 5, n >> 2], [seed & 0xFFFFFFFF, seed >> 32])[n & 3]
        u = orc.uniform(seed, 77, 3, 5, n)
        assert u == (bits >> 8) / 2.0 ** 24
        assert 0.0 <= u < 1.0


def test_uniform_equidistribution():
    us = np.array([orc.uniform(9, w, 0, 0, 0) for w in range(20000)])
    hist = np.bincount((us * 50).astype(int), minlength=50)
    assert chisquare(hist).pvalue > 1e-3
    # neighbouring words of one block and neighbouring walkers are uncorrelated
    a = np.array([orc.uniform(9, w, 1, 0, 1) for w in range(20000)])
    assert abs(np.corrcoef(us, a)[0, 1]) < 0.03
    assert abs(np.corrcoef(us[:-1], us[1:])[0, 1]) < 0.03


# ---- scan tree ------------------------------------------------------------------------------------

def test_wave_scan_tree():
    assert (orc.wave_scan(np.ones(64)) == np.arange(1, 65)).all()
    rng = np.random.RandomState(0)
    for _ in range(20):
        x = (rng.random_sample(64) * 100).astype(np.float32)
        got = orc.wave_scan(x)
        assert [float(v) for v in got] == [float(v) for v in _model.wave_scan(x)]
        assert np.allclose(got, np.cumsum(x.astype(np.float64)), rtol=1e-5)
    # zeros are exact no-ops: a scan of a one-hot vector is a step function
    x = np.zeros(64, dtype=np.float32)
    x[37] = 3.25
    assert (orc.wave_scan(x) == np.where(np.arange(64) >= 37, 3.25, 0)).all()


# ---- sampler mechanics: C oracle against the independent model ------------------------------------

def _one_list_graph(bias, pad_before):
    """A graph whose vertex 1 owns `bias` as its neighbour list, starting at CSR offset pad_before."""
    deg = len(bias)
    V = max(deg, 1) + 2
    xadj = np.zeros(V + 1, dtype=np.uint32)
    xadj[1] = pad_before
    xadj[2:] = pad_before + deg
    adj = np.concatenate([np.arange(pad_before) % V, np.arange(deg) % V]).astype(np.int32)
    w = np.concatenate([np.full(pad_before, 7.0), np.asarray(bias, dtype=np.float32)]).astype(np.float32)
    if len(adj) == 0:
        adj = np.zeros(1, dtype=np.int32)
        w = np.zeros(1, dtype=np.float32)
    return orc.Graph(xadj, adj, w)


@pytest.mark.parametrize("deg,pad", [(1, 0), (2, 3), (5, 1), (63, 2), (255, 1), (256, 0), (257, 3), (1023, 1),
                                     (1024, 0), (1025, 2), (3000, 5), (5000, 7)])
def test_sampler_matches_independent_model(deg, pad):
    rng = np.random.RandomState(deg * 31 + pad)
    bias = (rng.random_sample(deg) * 10).astype(np.float32)
    bias[rng.random_sample(deg) < 0.2] = 0.0
    g = _one_list_graph(bias, pad)
    for wg, thr in ((256, 1 << 30), (256, 0), (1024, 0)):
        p = orc.make_params(wg_threads=wg, hub_threshold=thr, seed=42)
        nw = wg // 64 if deg > thr else 1
        for walker in range(6):
            for step in (0, 5):
                got = orc.sample(g, p, 1, -1, walker, step)
                want = _model.sample(bias, pad, nw, 42, walker, step)
                assert got == want, (deg, pad, wg, thr, walker, step)
                if got >= 0:
                    assert bias[got] > 0


def test_sampler_special_cases():
    # degree 1 -> that neighbour; one positive weight -> that one; all zero / degree 0 -> -1
    p = orc.make_params(seed=3)
    assert orc.sample(_one_list_graph([2.5], 1), p, 1, -1, 0, 0) == 0
    b = np.zeros(700, dtype=np.float32)
    b[333] = 1e-3
    for thr in (1 << 30, 0):
        p = orc.make_params(hub_threshold=thr, seed=3)
        assert all(orc.sample(_one_list_graph(b, 2), p, 1, -1, w, 0) == 333 for w in range(50))
        assert orc.sample(_one_list_graph(np.zeros(700), 2), p, 1, -1, 0, 0) == -1
    assert orc.sample(_one_list_graph([], 0), p, 1, -1, 0, 0) == -1


def _first_step_counts(g, p, vertex, n):
    paths, _, _ = orc.walk(g, p, np.full(n, vertex, dtype=np.int32))
    return np.bincount(paths[:, 1], minlength=g.V)


@pytest.mark.parametrize("thr", [1 << 30, 1000])
def test_transition_frequencies_follow_the_weights(thr):
    """P(select i) = w_i / sum w on hub vertices, wave and workgroup granularity, chi-square p > 0.01."""
    xadj, adj, w, lab = _graphs.hub_graph(V=12000, hub_degrees=(9000, 2500, 700), base_degree=5, seed=11,
                                          zero_weight_fraction=0.05)
    g = orc.Graph(xadj, adj, w, lab)
    for hub in (0, 1):
        lo, hi = int(xadj[hub]), int(xadj[hub + 1])
        exp = np.zeros(g.V)
        exp[adj[lo:hi]] = w[lo:hi].astype(np.float64)
        n = 400000
        p = orc.make_params(max_depth=2, hub_threshold=thr, wg_threads=512, seed=2024 + hub)
        cnt = _first_step_counts(g, p, hub, n)
        m = exp > 0
        assert cnt[~m].sum() == 0  # zero-weight neighbours are never taken
        assert chisquare(cnt[m], exp[m] * n / exp.sum()).pvalue > 0.01


def test_equal_weights_are_uniform():
    deg = 777
    g = _one_list_graph(np.full(deg, 3.0, dtype=np.float32), 3)
    p = orc.make_params(max_depth=2, seed=5)
    n = 200000
    paths, _, _ = orc.walk(g, p, np.full(n, 1, dtype=np.int32))
    # adjacency of vertex 1 is arange(deg) % V, a bijection here
    cnt = np.bincount(paths[:, 1], minlength=g.V)[:deg]
    assert cnt.sum() == n
    assert chisquare(cnt).pvalue > 0.01


# ---- walks ----------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def hub_csr():
    return _graphs.hub_graph(V=6000, hub_degrees=(4000, 900), base_degree=5, seed=3, zero_weight_fraction=0.03)


def _edge_set(xadj, adj):
    src = np.repeat(np.arange(len(xadj) - 1, dtype=np.int64), np.diff(xadj.astype(np.int64)))
    return set((src * (len(xadj) - 1) + adj).tolist())


def test_walk_invariants_and_counters(hub_csr):
    xadj, adj, w, lab = hub_csr
    g = orc.Graph(xadj, adj, w, lab)
    V = g.V
    starts = np.random.RandomState(0).randint(0, V, size=2000).astype(np.int32)
    p = orc.make_params(max_depth=31, hub_threshold=1024, seed=8)
    paths, steps, edges = orc.walk(g, p, starts)
    es = _edge_set(xadj, adj)
    deg = np.diff(xadj.astype(np.int64))
    n_steps = n_edges = 0
    for row, s in zip(paths, starts):
        assert row[0] == s
        live = row >= 0
        k = int(live.sum())
        assert live[:k].all() and not live[k:].any()      # -1 only as a suffix
        for a, b in zip(row[:k - 1], row[1:k]):
            assert int(a) * V + int(b) in es               # every hop is a CSR edge
            n_edges += deg[a]
        n_steps += k - 1
        if k < 31:                                         # stopped early only at a dead end
            lo, hi = int(xadj[row[k - 1]]), int(xadj[row[k - 1] + 1])
            assert hi == lo or (w[lo:hi] == 0).all()
    assert (steps, edges) == (n_steps, n_edges)            # src/main.cu:93-104
    # row q depends on (seed, walker id) only: a permuted batch with matching walker ids gives the same rows
    p2 = orc.make_params(max_depth=31, hub_threshold=1024, seed=8, walker_base=1000)
    again, _, _ = orc.walk(g, p2, starts[1000:])
    assert (again == paths[1000:]).all()
    other, _, _ = orc.walk(g, orc.make_params(max_depth=31, hub_threshold=1024, seed=9), starts)
    assert (other != paths).any()


def test_ppr_length_distribution(hub_csr):
    """Steps L: P(L = k) = (1 - tp)^(k-1) tp for k < d, the rest at k = d (no dead ends from these starts)."""
    xadj, adj, w, lab = hub_csr
    w = np.maximum(w, 0.5).astype(np.float32)  # no zero weights, so no dead ends
    g = orc.Graph(xadj, adj, w, lab)
    tp, d, n = 0.2, 20, 200000
    p = orc.make_params(app=1, max_depth=d + 1, tp=tp, seed=77)
    paths, steps, _ = orc.walk(g, p, np.random.RandomState(1).randint(0, g.V, size=n).astype(np.int32))
    L = (paths >= 0).sum(axis=1) - 1
    assert L.min() >= 1 and L.max() <= d
    exp = np.array([(1 - tp) ** (k - 1) * tp for k in range(1, d)] + [(1 - tp) ** (d - 1)]) * n
    assert chisquare(np.bincount(L, minlength=d + 1)[1:], exp).pvalue > 0.01
    assert steps == L.sum()


def test_node2vec_reduces_to_deepwalk_for_p_q_one(hub_csr):
    xadj, adj, w, lab = hub_csr
    g = orc.Graph(xadj, adj, w, lab)
    starts = np.arange(0, g.V, 7, dtype=np.int32)
    a, _, _ = orc.walk(g, orc.make_params(app=0, max_depth=12, seed=4), starts)
    b, _, _ = orc.walk(g, orc.make_params(app=2, max_depth=12, p=1.0, q=1.0, seed=4), starts)
    assert (a == b).all()


@pytest.mark.parametrize("pp,qq", [(2.0, 0.5), (0.25, 4.0), (0.25, 1.0), (0.4, 0.5), (0.05, 0.5)])
def test_node2vec_second_step_distribution(hub_csr, pp, qq):
    """From a fixed (prev, cur): weights w/p for the return edge, w for common neighbours, w/q otherwise.  With 1/p
    above max(1, 1/q) the return edge's excess is a component of its own (the last four points; at p = 0.05 it takes
    most of the steps)."""
    xadj, adj, w, lab = hub_csr
    g = orc.Graph(xadj, adj, w, lab)
    prev = 1                                    # the 900-degree hub
    nb = adj[xadj[prev]:xadj[prev + 1]]
    cur = int(nb[np.argmax(np.diff(xadj.astype(np.int64))[nb])])
    p = orc.make_params(app=2, max_depth=3, p=pp, q=qq, seed=31)
    lo, hi = int(xadj[cur]), int(xadj[cur + 1])
    prev_set = set(nb.tolist())
    exp = np.zeros(g.V)
    for i in range(lo, hi):
        t = int(adj[i])
        exp[t] = w[i] / pp if t == prev else (w[i] if t in prev_set else w[i] / qq)
    n = 300000
    cnt = np.zeros(g.V)
    for walker in range(n):
        s = orc.sample(g, p, cur, prev, walker, 1)
        cnt[adj[lo + s]] += 1
    m = exp > 0
    assert cnt[~m].sum() == 0
    assert chisquare(cnt[m], exp[m] * n / exp.sum()).pvalue > 0.01


@pytest.mark.parametrize("pp,qq", [(0.25, 4.0), (0.3, 0.7), (3.0, 2.0)])
def test_node2vec_return_edges_of_a_multigraph(pp, qq):
    """Several entries of N(cur) lead back to prev, with weights of their own: every one of them carries w / p, so the
    vertex prev is taken in proportion to their sum (brute force over the entries)."""
    # vertex 0 = cur: three edges to 1 (prev), one each to 2 (common neighbour of prev), 3, 4, 5; vertex 1: 0, 2, 6
    lists = {0: [1, 1, 1, 2, 3, 4, 5], 1: [0, 2, 6], 2: [0, 1], 3: [0], 4: [0], 5: [0], 6: [1]}
    V = 7
    xadj = np.zeros(V + 1, dtype=np.uint32)
    np.cumsum([len(lists[v]) for v in range(V)], out=xadj[1:])
    adj = np.concatenate([lists[v] for v in range(V)]).astype(np.int32)
    w = (1.0 + 9.0 * np.random.RandomState(8).random_sample(len(adj))).astype(np.float32)
    g = orc.Graph(xadj, adj, w, None)
    p = orc.make_params(app=2, max_depth=3, p=pp, q=qq, seed=77)
    exp = np.zeros(V)
    for i in range(int(xadj[0]), int(xadj[1])):
        t = int(adj[i])
        exp[t] += w[i] / pp if t == 1 else (w[i] if t in (0, 2, 6) else w[i] / qq)
    n = 200000
    cnt = np.zeros(V)
    for walker in range(n):
        cnt[adj[orc.sample(g, p, 0, 1, walker, 1)]] += 1
    m = exp > 0
    assert cnt[~m].sum() == 0
    assert chisquare(cnt[m], exp[m] * n / exp.sum()).pvalue > 0.01


def test_metapath_follows_schema_and_is_uniform_among_matches(hub_csr):
    xadj, adj, w, lab = hub_csr
    g = orc.Graph(xadj, adj, None, lab)
    schema = [2, 0, 4]
    p = orc.make_params(app=3, max_depth=7, schema=schema, seed=12)
    starts = np.arange(g.V, dtype=np.int32)
    paths, _, _ = orc.walk(g, p, starts)
    for row in paths[::13]:
        k = int((row >= 0).sum())
        for j in range(1, k):                    # label of the j-th traversed edge == schema[(j-1) % len]
            a, b = int(row[j - 1]), int(row[j])
            lo, hi = int(xadj[a]), int(xadj[a + 1])
            idx = lo + int(np.nonzero(adj[lo:hi] == b)[0][0])
            assert lab[idx] == schema[(j - 1) % len(schema)]
        if k < 7:                                # ended because no edge carries the wanted label
            a = int(row[k - 1])
            assert not (lab[xadj[a]:xadj[a + 1]] == schema[(k - 1) % len(schema)]).any()
    # weights are ignored: among the matching edges of the hub the choice is uniform (include/app.cuh:141-146)
    n = 200000
    cnt = _first_step_counts(g, orc.make_params(app=3, max_depth=2, schema=[1], seed=5), 0, n)
    match = adj[xadj[0]:xadj[1]][lab[xadj[0]:xadj[1]] == 1]
    assert cnt.sum() == n and cnt[match].sum() == n
    assert chisquare(cnt[match]).pvalue > 0.01


def test_config1_plumbing_on_the_cpu_path():
    """Benchmark configuration 1 on the CPU reference path: 7,115 vertices, 103,689 edges, 100 seeded starts, length 80."""
    xadj, adj, w, lab = _graphs.uniform_graph(7115, 103689, seed=1)
    assert len(xadj) == 7116 and len(adj) == 103689 and w.min() >= 1.0 and w.max() < 5.0
    g = orc.Graph(xadj, adj, w, lab)
    starts = np.random.RandomState(1).randint(0, 7115, size=100).astype(np.int32)
    paths, steps, edges = orc.walk(g, orc.make_params(max_depth=81, seed=1), starts)
    assert paths.shape == (100, 81) and (paths[:, 0] == starts).all()
    assert steps == ((paths >= 0).sum(axis=1) - 1).sum()
    one, _, _ = orc.walk(g, orc.make_params(max_depth=81, seed=1), starts, nthreads=1)
    assert (one == paths).all()                  # thread count does not change a byte
