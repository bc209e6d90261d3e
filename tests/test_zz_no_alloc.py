"""fw_walk_device_noalloc (scratch in the library's static device array, no allocation per call) against
fw_walk_device: same path matrix and same workload counters, bit for bit, on two calls in a row, the second with a
smaller input -- the array keeps the first call's dispenser word and counters, which the second call must clear.
Collected last: a failure here must not hide the other GPU tests."""
import numpy as np
import pytest

import _graphs

pytestmark = pytest.mark.gpu


def _both(fw, g, p, starts):
    n = len(starts)
    d_starts = fw.DeviceBuffer.from_numpy(starts)
    d_paths = fw.DeviceBuffer(n * p.max_depth * 4)
    try:
        # poison the output so that entries the call does not write show up
        fw.check(fw.lib().fw_dev_fill_i32(d_paths.ptr, 0x5A5A5A5A, n * p.max_depth))
        st = g.walk_device_noalloc(p, d_starts, n, d_paths)
        got = d_paths.to_numpy(np.int32, (n, p.max_depth))
    finally:
        d_starts.free()
        d_paths.free()
    ref, st_ref = g.walk(p, starts)
    return got, st, ref, st_ref


@pytest.mark.parametrize("app", ["deepwalk", "ppr", "node2vec", "metapath"])
def test_noalloc_equals_walk_device_twice(gpu, app):
    fw = gpu
    xadj, adj, w, lab = _graphs.hub_graph(V=12000, hub_degrees=(9000, 2500, 700), base_degree=5, seed=11,
                                          zero_weight_fraction=0.05)
    g = fw.Graph.from_csr(xadj, adj, w, lab)
    kw = dict(deepwalk=dict(app=fw.APP_DEEPWALK, max_depth=41),
              ppr=dict(app=fw.APP_PPR, max_depth=81, tp=0.15),
              node2vec=dict(app=fw.APP_NODE2VEC, max_depth=12, p=2.0, q=0.5),
              metapath=dict(app=fw.APP_METAPATH, max_depth=11, schema=[1, 3, 0]))[app]
    try:
        rng = np.random.RandomState(5)
        for n, park in ((40000, 600), (3000, -1)):  # the second call is the smaller one
            starts = rng.randint(0, 12000, size=n).astype(np.int32)
            starts[:200] = 0
            # the reference call parks (first round) or not (second): the no-alloc call must equal both
            p = fw.default_params(hub_threshold=1000, park_threshold=park, seed=4242, walker_base=17, **kw)
            got, st, ref, st_ref = _both(fw, g, p, starts)
            bad = np.nonzero((got != ref).any(axis=1))[0]
            assert len(bad) == 0, "first differing walk %d:\n noalloc %s\n device  %s" % (bad[0], got[bad[0]], ref[bad[0]])
            assert (st.steps, st.sampled_edges) == (st_ref.steps, st_ref.sampled_edges)
            assert st.launches == 1 and st.steps > 0
    finally:
        g.destroy()


def test_noalloc_rejects_oversized_batches(gpu):
    fw = gpu
    xadj, adj, w, lab = _graphs.uniform_graph(2000, 16000, seed=3)
    g = fw.Graph.from_csr(xadj, adj, w, lab)
    n = 65536  # FW_WALK_NOALLOC_MAX_QUERIES + 1
    d_starts = fw.DeviceBuffer.from_numpy(np.zeros(n, dtype=np.int32))
    d_paths = fw.DeviceBuffer(n * 4 * 4)
    try:
        p = fw.default_params(app=fw.APP_DEEPWALK, max_depth=4)
        with pytest.raises(fw.FlowWalkerError) as e:
            g.walk_device_noalloc(p, d_starts, n, d_paths)
        assert e.value.status == 1 and "FW_WALK_NOALLOC_MAX_QUERIES" in str(e.value)
        st = g.walk_device_noalloc(p, d_starts, n - 1, d_paths)  # the limit itself is served
        assert st.launches == 1
    finally:
        d_starts.free()
        d_paths.free()
        g.destroy()
