"""CPU tests of the host side: the C-ABI library loads and exports every declared symbol, the autobatch rule,
the on-disk CSR format, input validation and the command-line front end.  No GPU compute is called."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

import _graphs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_DATA = "/root/reference/data/wiki-Vote"
BIN = os.path.join(ROOT, "flowwalker-artifact_amd", "bin")


def test_library_exports_every_declared_symbol(fw):
    header = open(os.path.join(ROOT, "include", "flowwalker.h")).read()
    declared = set(re.findall(r"^(?:const char\*|int|void|uint32_t)\s+(fw_[a-z0-9_]+)\s*\(", header, flags=re.M))
    assert len(declared) >= 25
    L = fw.lib()
    missing = [s for s in sorted(declared) if not hasattr(L, s)]
    assert not missing, "not exported: %s" % missing
    assert set(fw.EXPORTED) == declared


def test_struct_layouts_match_the_header(fw):
    # fw_walk_params: 6 int32 + 64 int32 + 3 float + uint32 + uint64 + 2 int32
    assert C.sizeof(fw.WalkParams) == 6 * 4 + 64 * 4 + 3 * 4 + 4 + 8 + 8 + 8
    assert C.sizeof(fw.WalkStats) == 8 + 8 + 8 + 8 + 4 + 4 + 8 + 8 + 8 + 8 + 8 + 4 * 8
    assert C.sizeof(fw.RmatParams) == 48


def test_default_params_follow_the_reference_flags(fw):
    p = fw.default_params()
    assert (p.app, p.max_depth) == (fw.APP_DEEPWALK, 81)           # --d 80 (src/main.cu:47, :342)
    assert abs(p.tp - 0.2) < 1e-7 and p.p == 2.0 and p.q == 0.5    # src/main.cu:58-60
    assert [p.schema[i] for i in range(p.schema_len)] == [0, 1, 2, 3, 4]
    assert p.wg_threads in (256, 512, 1024) and p.hub_threshold > 0


def test_default_params_per_application(fw):
    """Per-application defaults are the plain ones with the application set: no application needs other choices."""
    base = fw.default_params()
    for app in (fw.APP_DEEPWALK, fw.APP_PPR, fw.APP_NODE2VEC, fw.APP_METAPATH):
        p = fw.default_params(app=app)
        assert p.app == app and p.hub_threshold == base.hub_threshold
        assert (p.max_depth, p.wg_threads, p.seed) == (base.max_depth, base.wg_threads, base.seed)
    assert fw.default_params(app=fw.APP_NODE2VEC, hub_threshold=4096).hub_threshold == 4096


def test_autobatch_rule(fw):
    """bs = min((free - headroom MB) / (4 (d + 2)), INT_MAX); halved unless sync; capped at the query count
    (src/main.cu:259-271)."""
    f = fw.lib().fw_autobatch_size
    free = 40 * 2 ** 30
    assert f(free, 512, 81, 1, 2 ** 31) == (free - 512 * 2 ** 20) // (4 * 82)
    assert f(free, 512, 81, 0, 2 ** 31) == (free - 512 * 2 ** 20) // (4 * 82) // 2
    assert f(free, 512, 81, 0, 1000) == 1000
    assert f(300 * 2 ** 30, 0, 2, 1, 2 ** 32 - 1) == 2 ** 31 - 1     # INT_MAX cap
    assert f(100, 512, 81, 0, 1000) == 0                              # headroom exceeds free memory


def test_csr_files_round_trip(fw, tmp_path):
    xadj, adj, w, lab = _graphs.uniform_graph(500, 4000, seed=3)
    prefix = str(tmp_path / "g")
    fw.csr_write(prefix, xadj, adj, w, lab)
    assert os.path.getsize(prefix + "_xadj.bin") == 4 * (500 + 3)    # int32 V, uint32 E, uint32 xadj[V+1]
    assert os.path.getsize(prefix + "_edge.bin") == 4 * 4000
    hdr = np.fromfile(prefix + "_xadj.bin", dtype=np.uint32, count=2)
    assert hdr.tolist() == [500, 4000]
    x2, a2, w2, l2 = fw.csr_read(prefix, weights=True, labels=True)
    assert (x2 == xadj).all() and (a2 == adj).all() and (w2 == w).all() and (l2 == lab).all()
    x3, a3, w3, l3 = fw.csr_read(prefix, weights=False, labels=False)
    assert w3 is None and l3 is None


def test_csr_loader_rejects_inconsistent_files(fw, tmp_path):
    xadj, adj, w, lab = _graphs.uniform_graph(200, 1000, seed=4)
    prefix = str(tmp_path / "g")
    fw.csr_write(prefix, xadj, adj, w, lab)
    with pytest.raises(fw.FlowWalkerError, match="cannot open"):
        fw.csr_read(str(tmp_path / "missing"))
    with open(prefix + "_edge.bin", "ab") as f:                      # edge file longer than the header says
        f.write(b"\0\0\0\0")
    with pytest.raises(fw.FlowWalkerError, match="edges"):
        fw.csr_read(prefix)
    fw.csr_write(prefix, xadj, adj, w, lab)
    os.truncate(prefix + "_weight.bin", 100)
    with pytest.raises(fw.FlowWalkerError, match="weight"):
        fw.csr_read(prefix, weights=True)
    fw.csr_read(prefix, weights=False)                                # still fine without weights


@pytest.mark.skipif(not os.path.exists(REF_DATA + "_xadj.bin"), reason="reference data not mounted")
def test_loader_on_the_shipped_wiki_vote_graph(fw):
    """Known answers of the one graph the reference ships: V, E, file sizes, max degree and its vertex, and the
    edge list text equals the CSR (src, dst) order."""
    xadj, adj, w, lab = fw.csr_read(REF_DATA, weights=True, labels=True)
    assert len(xadj) - 1 == 7115 and len(adj) == 201524 and int(xadj[-1]) == 201524
    assert os.path.getsize(REF_DATA + "_xadj.bin") == 28472 and os.path.getsize(REF_DATA + "_edge.bin") == 806096
    deg = np.diff(xadj.astype(np.int64))
    assert deg.max() == 1065 and deg.argmax() == 742 and deg.min() == 1
    assert np.bincount(lab).tolist() == [40650, 39908, 40092, 40640, 40234]
    assert 0 < w.min() < 1e-4 and w.max() < 5.0
    el = np.loadtxt(REF_DATA + ".edgelist", dtype=np.int64, usecols=(0, 1), max_rows=5000)
    src = np.repeat(np.arange(7115), deg)
    assert (el[:, 0] == src[:5000]).all() and (el[:, 1] == adj[:5000]).all()


def test_graph_create_validates_before_touching_the_device(fw):
    x = np.array([0, 2, 3], dtype=np.uint32)
    a = np.array([1, 0, 0], dtype=np.int32)
    w = np.array([1.0, 2.0, 3.0], dtype=np.float32)
    for bad_x, bad_a, bad_w, msg in (
            (np.array([1, 2, 3], dtype=np.uint32), a, w, r"xadj\[0\]"),
            (np.array([0, 2, 4], dtype=np.uint32), a, w, "does not match"),
            (np.array([0, 3, 3], dtype=np.uint32), np.array([1, 0, 5], dtype=np.int32), w, "outside"),
            (x, a, np.array([1.0, -2.0, 3.0], dtype=np.float32), "non-negative"),
            (x, a, np.array([1.0, np.nan, 3.0], dtype=np.float32), "non-negative"),
            (x, a, np.array([1.0, np.inf, 3.0], dtype=np.float32), "finite")):
        with pytest.raises(fw.FlowWalkerError, match=msg) as e:
            fw.Graph.from_csr(bad_x, bad_a, bad_w)
        assert e.value.status == 1
        with pytest.raises(fw.FlowWalkerError, match=msg):  # the same checks whichever memory the edges go to
            fw.Graph.from_csr(bad_x, bad_a, bad_w, placement=fw.GRAPH_HOST_PINNED)
    with pytest.raises(fw.FlowWalkerError, match="unknown placement 7") as e:
        fw.Graph.from_csr(x, a, w, placement=7)
    assert e.value.status == 1


def test_no_cpu_fallback(fw):
    """Without a device the compute entry points fail loudly; nothing routes to a CPU implementation."""
    if fw.device_count() > 0:
        pytest.skip("a GPU is visible here")
    x = np.array([0, 1, 2], dtype=np.uint32)
    a = np.array([1, 0], dtype=np.int32)
    w = np.ones(2, dtype=np.float32)
    with pytest.raises(fw.FlowWalkerError, match="no HIP device") as e:
        fw.Graph.from_csr(x, a, w)
    assert e.value.status == 3
    with pytest.raises(fw.FlowWalkerError, match="no HIP device"):
        fw.Graph.from_csr(x, a, w, placement=fw.GRAPH_HOST_PINNED)
    with pytest.raises(fw.FlowWalkerError, match="no HIP device"):
        fw.Graph.rmat(8)
    with pytest.raises(fw.FlowWalkerError):
        fw.DeviceBuffer(16)


def test_host_mirror_of_the_rmat_generator():
    xadj, adj, w, lab = _graphs.rmat_graph(10, edge_factor=8, symmetrise=True, n_labels=5, seed=2)
    V = 1 << 10
    deg = np.diff(xadj.astype(np.int64))
    src = np.repeat(np.arange(V), deg)
    assert (src != adj).all()                                          # no self loops
    key = src * V + adj
    assert (np.diff(key) > 0).all()                                    # ascending lists, no duplicates
    rev = set((adj.astype(np.int64) * V + src).tolist())
    assert rev == set(key.tolist())                                    # symmetric
    assert w.min() >= 1.0 and w.max() < 100.0 and lab.min() >= 0 and lab.max() <= 4
    order = np.argsort(adj.astype(np.int64) * V + src, kind="stable")  # weight / label equal on both directions
    assert (w[order] == w).all() and (lab[order] == lab).all()
    assert deg.max() > 20 * deg.mean()                                 # skewed, as R-MAT should be


def _run(tool, *args):
    return subprocess.run([os.path.join(BIN, tool)] + list(args), stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          text=True, timeout=120)


@pytest.mark.skipif(not os.path.exists(os.path.join(BIN, "flowwalker")), reason="tools not built")
def test_cli_flag_surface(fw, tmp_path):
    r = _run("flowwalker")
    assert r.returncode == 0 and "Please choose a walk mode" in r.stdout          # src/walk.cu:565-568
    r = _run("flowwalker", "--bogus")
    assert r.returncode == 2 and "unknown command line flag 'bogus'" in r.stderr
    r = _run("flowwalker", "--deepwalk", "--n")
    assert r.returncode == 2 and "missing its argument" in r.stderr
    r = _run("flowwalker", "--deepwalk", "--n=abc")
    assert r.returncode == 2 and "illegal value" in r.stderr
    if fw.device_count() == 0:
        r = _run("flowwalker", "--deepwalk", "--noseq", "--input", str(tmp_path / "nope"))
        assert r.returncode == 3 and "no CPU fallback" in r.stderr
    r = _run("fw_gen", "--out", str(tmp_path / "u"), "--kind", "uniform", "--vertices", "7115", "--edges", "103689",
             "--whi", "5")
    assert r.returncode == 0
    xadj, adj, w, lab = fw.csr_read(str(tmp_path / "u"), True, True)
    assert len(xadj) - 1 == 7115 and len(adj) == 103689
    src = np.repeat(np.arange(7115), np.diff(xadj.astype(np.int64)))
    assert (src != adj).all() and len(np.unique(src * 7115 + adj)) == 103689
    assert w.min() >= 1.0 and w.max() < 5.0


def test_sort_neighbours_moves_weights_and_labels_with_their_edges(fw):
    """fw_csr_sort_neighbours: every list ascending afterwards, the (neighbour, weight, label) triples of a vertex
    unchanged as a set, lists that already ascend untouched."""
    import _graphs
    xadj, adj, w, lab = _graphs.uniform_graph(500, 6000, seed=2)
    rng = np.random.RandomState(0)
    a2, w2, l2 = adj.copy(), w.copy(), lab.copy()
    shuffled = 0
    for v in range(0, 500, 2):                                   # every other list in random order
        b, e = int(xadj[v]), int(xadj[v + 1])
        perm = rng.permutation(e - b)
        if (perm != np.arange(e - b)).any():
            shuffled += 1
        a2[b:e], w2[b:e], l2[b:e] = a2[b:e][perm], w2[b:e][perm], l2[b:e][perm]
    assert fw.csr_sort_neighbours(xadj, a2, w2, l2) == shuffled
    assert (a2 == adj).all() and (w2 == w).all() and (l2 == lab).all()   # uniform_graph's lists ascend, no duplicates
    assert fw.csr_sort_neighbours(xadj, a2, w2, l2) == 0


def test_sort_neighbours_keeps_duplicate_edges_in_order(fw):
    """A multigraph: a list with equal neighbours counts as ascending (the adjacency test is a binary search, which only
    needs a non-decreasing list, include/gpu_graph.cuh:97-112), the sort keeps every copy of an edge with its own weight,
    and a sorted list with duplicates is left alone."""
    xadj = np.array([0, 6, 6, 9], dtype=np.uint32)
    adj = np.array([2, 1, 2, 0, 1, 2, 0, 0, 1], dtype=np.int32)
    w = np.arange(9, dtype=np.float32) + 1.0
    lab = np.arange(9, dtype=np.int32)
    assert fw.csr_sort_neighbours(xadj, adj, w, lab) == 1                 # the second list (0, 0, 1) already ascends
    assert adj.tolist() == [0, 1, 1, 2, 2, 2, 0, 0, 1]
    assert w.tolist() == [4.0, 2.0, 5.0, 1.0, 3.0, 6.0, 7.0, 8.0, 9.0]   # stable: copies keep their order
    assert lab.tolist() == [3, 1, 4, 0, 2, 5, 6, 7, 8]
    assert fw.csr_sort_neighbours(xadj, adj, w, lab) == 0


def test_bench_measures_one_gpu_only():
    """bench.py --gpus N with N above 1 exits with a message that says so (no figure at several GPUs is produced)."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode != 0 and r.stdout.strip() == ""
    assert "one GPU" in r.stderr and "--gpus 1" in r.stderr


def test_bench_byte_formulas():
    """The algorithmic bytes of a pass: 4*D + 16*S + 16*Q, for node2vec 8*D + 24*S + 16*Q (src/main.cu:93-104 counts D and S)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert bench.algorithmic_bytes("deepwalk", 10, 1000, 3) == 4 * 1000 + 16 * 10 + 16 * 3
    assert bench.algorithmic_bytes("metapath", 10, 1000, 3) == bench.algorithmic_bytes("ppr", 10, 1000, 3)
    assert bench.algorithmic_bytes("node2vec", 10, 1000, 3) == 8 * 1000 + 24 * 10 + 16 * 3
    assert bench.HBM_PEAK_GBS == 8000.0
