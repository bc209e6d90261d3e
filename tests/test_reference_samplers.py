"""The reference's own samplers (include/sampler.cuh), restated thread by thread in oracle/fw_ref_samplers.c, against
their sequential ground truth and against this build's sampler.

The walk engine here samples with a different algorithm than the reference, so what the two must share is the law of
one sampling step, P(i) = w_i / sum w, and the special cases.  These tests pin that on the reference's algorithm
itself: (1) its parallel samplers are the sequential weighted reservoir over a permutation of the list (exact
equality on integer-valued biases, where f32 sums do not depend on the order of the additions), and (2) all of them
and this build's sampler follow the same distribution on the same list (chi-square).
"""
import numpy as np
import pytest
from scipy.stats import chisquare

import fw_oracle_binding as orc


def _uniforms(rng, shape):
    """(0, 1] like cuRAND's (include/myrand.cuh:213-215): x * 2^-32 + 2^-33 on 32 random bits."""
    bits = rng.randint(0, 2 ** 32, size=shape, dtype=np.uint64)
    return (bits.astype(np.float64) * 2.0 ** -32 + 2.0 ** -33).astype(np.float32)


def _int_biases(rng, n, zero_fraction):
    w = rng.randint(1, 50, size=n).astype(np.float32)
    w[rng.random_sample(n) < zero_fraction] = 0.0
    return w


@pytest.mark.parametrize("width", [32, 512])
@pytest.mark.parametrize("n", [1, 2, 31, 32, 33, 100, 511, 512, 513, 2000])
def test_zprs_is_the_sequential_reservoir_over_the_lane_major_order(n, width):
    """include/sampler.cuh:46-127: lane l owns elements l, l + W, ...; the key i + size * lane makes the highest lane's
    latest acceptance win, which is sequential reservoir sampling over (lane 0's elements, lane 1's, ...)."""
    rng = np.random.RandomState(1000 * width + n)
    for zero_fraction in (0.0, 0.3, 1.0):
        w = _int_biases(rng, n, zero_fraction)
        u = _uniforms(rng, (200, n))
        order = np.concatenate([np.arange(l, n, width) for l in range(min(width, n))])
        assert sorted(order) == list(range(n))
        got = orc.ref_sample_many(orc.REF_ZPRS, w, u, width)
        seq = orc.ref_sample_many(orc.REF_THREAD, w[order], u[:, order], width)
        # positions in the permuted list map back through the order; the fallback "index 0" of :37 / :75 is
        # position 0 there and element 0 here, and order[0] == 0
        want = np.where(seq < 0, -1, order[np.maximum(seq, 0)])
        assert (got == want).all()
        if zero_fraction == 1.0:
            assert (got == -1).all()


@pytest.mark.parametrize("width", [32, 512])
@pytest.mark.parametrize("n", [1, 2, 31, 32, 33, 64, 100, 512, 513, 2000])
def test_dprs_is_the_sequential_reservoir_in_list_order(n, width):
    """include/sampler.cuh:129-200: chunks of W in list order with a carried prefix; the running maximum of the accepted
    indices is the last acceptance of sequential reservoir sampling."""
    rng = np.random.RandomState(7000 * width + n)
    for zero_fraction in (0.0, 0.3, 1.0):
        w = _int_biases(rng, n, zero_fraction)
        u = _uniforms(rng, (200, n))
        got = orc.ref_sample_many(orc.REF_DPRS, w, u, width)
        seq = orc.ref_sample_many(orc.REF_THREAD, w, u, width)
        assert (got == seq).all()


def test_sequential_reservoir_matches_this_builds_ground_truth():
    """fw_oracle_sequential_reservoir (accept iff u * S < w) and the reference's form (u < w / S) agree."""
    rng = np.random.RandomState(5)
    w = _int_biases(rng, 300, 0.2)
    u = _uniforms(rng, (2000, 300))
    ref = orc.ref_sample_many(orc.REF_THREAD, w, u)
    ours = np.array([orc.lib().fw_oracle_sequential_reservoir(w.ctypes.data, u[r].ctypes.data, len(w))
                     for r in range(len(u))])
    assert (ref == ours).mean() > 0.999  # the two forms can round differently when u is within an ulp of w / S
    assert ((ref >= 0) == (ours >= 0)).all()


def test_all_samplers_follow_the_same_law():
    """Reference thread / ZPRS / DPRS samplers and this build's group-reservoir sampler on one list of 1500 biases
    (f32 U[1, 100), a tenth of them zero): chi-square against w / sum w, p > 0.01 each; zero biases never taken."""
    rng = np.random.RandomState(99)
    n, m = 1500, 90000
    w = (1.0 + 99.0 * rng.random_sample(n)).astype(np.float32)
    w[rng.random_sample(n) < 0.1] = 0.0
    pos = w > 0
    expect = w[pos].astype(np.float64) / w.astype(np.float64).sum() * m
    for kind, width in ((orc.REF_THREAD, 32), (orc.REF_ZPRS, 32), (orc.REF_ZPRS, 512), (orc.REF_DPRS, 32),
                        (orc.REF_DPRS, 512)):
        cnt = np.zeros(n)
        for _ in range(3):  # three slabs of uniforms keep the memory small
            u = _uniforms(rng, (m // 3, n))
            cnt += np.bincount(orc.ref_sample_many(kind, w, u, width), minlength=n)
        assert cnt[~pos].sum() == 0
        assert chisquare(cnt[pos], expect).pvalue > 0.01, (kind, width)
    # this build's sampler: vertex 1 of a small graph owns the same list (neighbour i is vertex i % V)
    V = n + 2
    xadj = np.zeros(V + 1, dtype=np.uint32)
    xadj[2:] = n
    g = orc.Graph(xadj, (np.arange(n) % V).astype(np.int32), w)
    for thr in (1 << 30, 1000):
        p = orc.make_params(max_depth=2, hub_threshold=thr, seed=77)
        paths, _, _ = orc.walk(g, p, np.full(m, 1, dtype=np.int32))
        cnt = np.bincount(paths[:, 1], minlength=V)[:n].astype(np.float64)
        assert cnt.sum() == m and cnt[~pos].sum() == 0
        assert chisquare(cnt[pos], expect).pvalue > 0.01, thr


@pytest.mark.parametrize("width", [64, 256, 512])
@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 200, 511, 512, 513, 3000])
def test_wave64_restatements_are_the_same_sequential_reservoirs(n, width):
    """The two samplers for groups of 64-lane waves (what FW_SAMPLER_REF_ZPRS / _DPRS run on the GPU): ZPRS is the
    sequential reservoir over the lane-major order, DPRS the one in list order, exactly, for integer-valued biases
    (their sums are exact in any association, so the scan tree cannot matter)."""
    rng = np.random.RandomState(31 * width + n)
    for zero_fraction in (0.0, 0.3, 1.0):
        w = _int_biases(rng, n, zero_fraction)
        u = _uniforms(rng, (150, n))
        order = np.concatenate([np.arange(l, n, width) for l in range(min(width, n))])
        got = orc.ref_sample_many(orc.REF64_ZPRS, w, u, width)
        seq = orc.ref_sample_many(orc.REF_THREAD, w[order], u[:, order], width)
        assert (got == np.where(seq < 0, -1, order[np.maximum(seq, 0)])).all()
        got = orc.ref_sample_many(orc.REF64_DPRS, w, u, width)
        assert (got == orc.ref_sample_many(orc.REF_THREAD, w, u, width)).all()
        # and they agree with the reference's own 32- / 512-lane forms wherever both are defined on the same width
        if width == 512:
            assert (orc.ref_sample_many(orc.REF64_ZPRS, w, u, 512) == orc.ref_sample_many(orc.REF_ZPRS, w, u, 512)).all()
            assert (orc.ref_sample_many(orc.REF64_DPRS, w, u, 512) == orc.ref_sample_many(orc.REF_DPRS, w, u, 512)).all()


def test_wave64_restatements_follow_the_law_in_whole_walks():
    """First steps of the oracle's walks with sampler = reference ZPRS / DPRS on 64-lane waves (keyed Philox uniforms in
    (0, 1]) from one vertex: chi-square against w / sum w at wave and at workgroup granularity."""
    rng = np.random.RandomState(98)
    n, m = 1500, 120000
    w = (1.0 + 99.0 * rng.random_sample(n)).astype(np.float32)
    w[rng.random_sample(n) < 0.1] = 0.0
    pos = w > 0
    expect = w[pos].astype(np.float64) / w.astype(np.float64).sum() * m
    V = n + 2
    xadj = np.zeros(V + 1, dtype=np.uint32)
    xadj[2:] = n
    g = orc.Graph(xadj, (np.arange(n) % V).astype(np.int32), w)
    for sampler in (2, 3):
        for thr in (1 << 30, 1000):
            p = orc.make_params(sampler=sampler, max_depth=2, hub_threshold=thr, wg_threads=256, seed=78)
            paths, _, _ = orc.walk(g, p, np.full(m, 1, dtype=np.int32))
            cnt = np.bincount(paths[:, 1], minlength=V)[:n].astype(np.float64)
            assert cnt.sum() == m and cnt[~pos].sum() == 0
            assert chisquare(cnt[pos], expect).pvalue > 0.01, (sampler, thr)


def _thread_uniform(seed, gid, k):
    """k-th uniform of the generator that thread `gid` owns: word k & 3 of Philox block (gid, k >> 2, 0x08000000, 0),
    mapped to (0, 1]."""
    out = orc.philox([gid, k >> 2, 0x08000000, 0], [seed & 0xFFFFFFFF, seed >> 32])
    return np.float32(((int(out[k & 3]) >> 8) + 1) * 2.0 ** -24)


def _replay_model(xadj, adj, w, starts, grid, W, thr, depth, seed, dprs):
    """The launch of the reference's engine with thread-owned generators, written down independently of the C replay:
    who owns which query, which slot is stepped when and by which threads, and which of its draws a thread spends on
    which element.  The samplers themselves are the pinned fw_ref64_* (orc.ref_sample_many)."""
    n = len(starts)
    grid = min(grid, (n + 63) // 64)
    per = (n + grid - 1) // grid
    nw = W // 64
    paths = np.full((n, depth), -1, dtype=np.int32)
    for b in range(grid):
        lo, hi = min(b * per, n), min(b * per + per, n)
        count = [0] * W
        nxt = lo
        slots = [None] * 64

        def take(s):
            nonlocal nxt
            if nxt < hi:
                q = nxt
                nxt += 1
                paths[q, 0] = starts[q]
                slots[s] = dict(q=q, cur=int(starts[q]), len=1)
            else:
                slots[s] = None

        def step(sl, threads):
            off, deg = int(xadj[sl["cur"]]), int(xadj[sl["cur"] + 1] - xadj[sl["cur"]])
            if deg == 0:
                return -1
            Wg = len(threads)
            u = np.zeros(deg, dtype=np.float32)
            if dprs:
                for base in range(0, deg + Wg - deg % Wg, Wg):
                    for l, t in enumerate(threads):
                        d = _thread_uniform(seed, b * W + t, count[t])
                        count[t] += 1
                        if base + l < deg:
                            u[base + l] = d
            else:
                for l, t in enumerate(threads):
                    for i in range(l, deg, Wg):
                        u[i] = _thread_uniform(seed, b * W + t, count[t])
                        count[t] += 1
            kind = orc.REF64_DPRS if dprs else orc.REF64_ZPRS
            return int(orc.ref_sample_many(kind, w[off:off + deg], u[None, :], Wg)[0])

        for s in range(64):
            take(s)
        while any(sl is not None for sl in slots):
            large = []
            for v in range(nw):
                for s in range(v, 64, nw):
                    sl = slots[s]
                    if sl is None or sl["len"] >= depth:
                        continue
                    if int(xadj[sl["cur"] + 1] - xadj[sl["cur"]]) > thr:
                        large.append(s)
                        continue
                    sel = step(sl, list(range(64 * v, 64 * v + 64)))
                    if sel < 0:
                        sl["len"] = depth
                    else:
                        nv = int(adj[int(xadj[sl["cur"]]) + sel])
                        paths[sl["q"], sl["len"]] = nv
                        sl["cur"], sl["len"] = nv, sl["len"] + 1
            for s in sorted(large):
                sl = slots[s]
                sel = step(sl, list(range(W)))
                if sel < 0:
                    sl["len"] = depth
                else:
                    nv = int(adj[int(xadj[sl["cur"]]) + sel])
                    paths[sl["q"], sl["len"]] = nv
                    sl["cur"], sl["len"] = nv, sl["len"] + 1
            for s in range(64):
                sl = slots[s]
                if sl is not None and (sl["len"] >= depth or xadj[sl["cur"] + 1] == xadj[sl["cur"]]):
                    take(s)
    return paths


@pytest.mark.parametrize("dprs", [False, True])
def test_thread_owned_generators_replay_against_an_independent_model(dprs):
    """fw_oracle_walk_ref_threads (the reference's engine with generators that belong to the threads, static assignment)
    against a Python model of the same launch: a small graph with a list above the workgroup threshold, dead ends,
    three workgroups with uneven shares, two waves per workgroup."""
    import _graphs
    xadj, adj, w, lab = _graphs.hub_graph(V=300, hub_degrees=(200,), base_degree=3, seed=4, symmetric=False)
    rng = np.random.RandomState(5)
    starts = rng.randint(0, 300, size=170).astype(np.int32)
    starts[:6] = 0
    for grid, W, thr in ((3, 128, 100), (2, 64, 1 << 30), (1, 256, 2)):
        p = orc.make_params(sampler=3 if dprs else 2, max_depth=6, wg_threads=W, hub_threshold=thr, seed=91)
        got, steps, edges = orc.walk_ref_threads(orc.Graph(xadj, adj, w, lab), p, starts, grid)
        want = _replay_model(xadj, adj, w, starts, grid, W, thr, 6, 91, dprs)
        assert (got == want).all(), (grid, W, thr)
        deg = np.diff(xadj.astype(np.int64))
        assert steps == int((got[:, 1:] >= 0).sum())
        assert edges == int(sum(deg[row[j - 1]] for row in got for j in range(1, 6) if row[j] >= 0))


def test_thread_owned_generators_follow_the_law():
    """First steps from one vertex with thread-owned generators: chi-square against w / sum w for both samplers, wave and
    workgroup granularity, and launches of different shape (the walks depend on the launch, the law does not)."""
    rng = np.random.RandomState(99)
    n, m = 900, 100000
    w = (1.0 + 99.0 * rng.random_sample(n)).astype(np.float32)
    w[rng.random_sample(n) < 0.1] = 0.0
    pos = w > 0
    expect = w[pos].astype(np.float64) / w.astype(np.float64).sum() * m
    V = n + 2
    xadj = np.zeros(V + 1, dtype=np.uint32)
    xadj[2:] = n
    g = orc.Graph(xadj, (np.arange(n) % V).astype(np.int32), w)
    seen = []
    for sampler in (2, 3):
        for thr, grid, W in ((1 << 30, 40, 256), (500, 7, 128)):
            p = orc.make_params(sampler=sampler, max_depth=2, hub_threshold=thr, wg_threads=W, seed=78)
            paths, steps, _ = orc.walk_ref_threads(g, p, np.full(m, 1, dtype=np.int32), grid)
            cnt = np.bincount(paths[:, 1], minlength=V)[:n].astype(np.float64)
            assert steps == m and cnt.sum() == m and cnt[~pos].sum() == 0
            assert chisquare(cnt[pos], expect).pvalue > 0.01, (sampler, thr)
            seen.append(paths[:, 1].copy())
    assert (seen[0] != seen[1]).any()  # another launch shape, other walks
