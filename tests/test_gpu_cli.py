"""The flowwalker command-line front end end to end on the GPU: same flags as the reference, walk paths equal
to the oracle's, printed report in the reference's format."""
import os
import re
import subprocess

import numpy as np
import pytest

import _graphs
import fw_oracle_binding as orc

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "flowwalker-artifact_amd", "bin", "flowwalker")


def _run(*args):
    r = subprocess.run([CLI] + list(args), stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    return r.stdout


@pytest.fixture(scope="module")
def graph_files(gpu, tmp_path_factory):
    d = tmp_path_factory.mktemp("g")
    xadj, adj, w, lab = _graphs.hub_graph(V=7115, hub_degrees=(3000,), base_degree=7, seed=1, w_hi=5.0)
    prefix = str(d / "hub")
    gpu.csr_write(prefix, xadj, adj, w, lab)
    return prefix, (xadj, adj, w, lab)


def test_deepwalk_n100_print(gpu, graph_files, tmp_path):
    prefix, csr = graph_files
    out = str(tmp_path / "paths.bin")
    text = _run("--input", prefix, "--deepwalk", "--n=100", "--seq", "--seed=5", "--printresult", "--printworkload",
                "--savepaths", out)
    paths = np.fromfile(out, dtype=np.int32).reshape(100, 81)
    ref, steps, edges = orc.walk(orc.Graph(*csr), orc.make_params(max_depth=81, seed=5), np.arange(100, dtype=np.int32))
    assert (paths == ref).all()
    assert "Vertex count:7115 Expected edge count: %d" % len(csr[1]) in text
    assert "Read Graph!" in text and re.search(r"Max degree: \d+, idx: 0", text)
    assert "grid:" in text and "sampling time:" in text
    assert text.count("Walker ") == 100                                          # src/main.cu:165
    row0 = re.search(r"Walker 0:\n([^\n]*)\nTotal length=(\d+)", text)
    assert [int(t) for t in row0.group(1).split()] == ref[0][ref[0] >= 0].tolist()
    assert int(row0.group(2)) == int((ref[0] >= 0).sum())
    assert "Total sampled vertex: %d" % steps in text                            # src/main.cu:109-111
    assert "Total sampled edge: %d," % edges in text


def test_all_batch_modes_agree(gpu, graph_files, tmp_path):
    prefix, csr = graph_files
    V = len(csr[0]) - 1
    ref, _, _ = orc.walk(orc.Graph(*csr), orc.make_params(app=2, max_depth=21, seed=1337), np.arange(V, dtype=np.int32))
    for i, extra in enumerate((["--all"], ["--all", "--syn"], ["--n=%d" % V, "--seq", "--batch", "--batchsize=1000"],
                               ["--n=%d" % V, "--seq", "--dprs"])):
        out = str(tmp_path / ("p%d.bin" % i))
        text = _run("--input", prefix, "--node2vec", "--d=20", "--p=2.0", "--q=0.5", "--savepaths", out, *extra)
        assert (np.fromfile(out, dtype=np.int32).reshape(V, 21) == ref).all(), extra
        if "--all" in extra:
            assert "batch size=%d" % V in text                                   # src/main.cu:270


def test_metapath_and_ppr(gpu, graph_files, tmp_path):
    prefix, csr = graph_files
    xadj, adj, w, lab = csr
    out = str(tmp_path / "m.bin")
    text = _run("--input", prefix, "--metapath", "--schema=2,0,1", "--n=50", "--seq", "--printresult", "--savepaths", out)
    assert "schema len=3" in text
    ref, _, _ = orc.walk(orc.Graph(xadj, adj, None, lab), orc.make_params(app=3, max_depth=4, schema=[2, 0, 1], seed=1337),
                         np.arange(50, dtype=np.int32))
    assert (np.fromfile(out, dtype=np.int32).reshape(50, 4) == ref).all()
    assert text.count("Walker ") == 50 and re.search(r"\[2\]\t\d+\t", text)       # labels printed before each hop
    # --ppr starts every query from the max-degree vertex (src/main.cu:277-281); --pprstart=seq from 0..n-1
    out = str(tmp_path / "p.bin")
    _run("--input", prefix, "--ppr", "--n=300", "--tp=0.3", "--savepaths", out)
    got = np.fromfile(out, dtype=np.int32).reshape(300, 81)
    assert (got[:, 0] == 0).all()
    ref, _, _ = orc.walk(orc.Graph(*csr), orc.make_params(app=1, max_depth=81, tp=0.3, seed=1337), np.zeros(300, dtype=np.int32))
    assert (got == ref).all()
    _run("--input", prefix, "--ppr", "--n=300", "--seq", "--pprstart=seq", "--savepaths", out)
    assert (np.fromfile(out, dtype=np.int32).reshape(300, 81)[:, 0] == np.arange(300)).all()


def test_sampler_micro_benchmark_and_converter(gpu, tmp_path):
    """fw_sampler_bench (one sampling step at fixed list lengths, six algorithms, both granularities) runs and reports every sample;
    a graph written by fw_convert loads and walks."""
    tool = os.path.join(ROOT, "flowwalker-artifact_amd", "bin", "fw_sampler_bench")
    r = subprocess.run([tool, "--elements", "1048576", "--samples", "20000", "--lengths", "16,1024", "--reps", "1",
                        "--type", "native,zprs,dprs,its,rjs,als"],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    rows = [ln.split() for ln in r.stdout.splitlines()[1:]]
    # per list length: this engine's sampler, the reference's ZPRS and DPRS on 64-lane waves, then inverse transform sampling,
    # rejection sampling and the alias method, each at both granularities
    want = [(g, t, s) for g in ("16", "1024") for t in ("native", "zprs", "dprs", "its", "rjs", "als") for s in ("wave", "workgroup")]
    assert [(row[0], row[1], row[2]) for row in rows] == want
    assert all(int(row[3]) == 20000 and float(row[4]) > 0 for row in rows)

    conv = os.path.join(ROOT, "flowwalker-artifact_amd", "bin", "fw_convert")
    rng = np.random.RandomState(11)
    src = tmp_path / "edges.txt"
    src.write_text("".join("%d %d\n" % (a, b) for a, b in rng.randint(0, 500, size=(6000, 2))))
    prefix = str(tmp_path / "conv")
    subprocess.run([conv, str(src), prefix, "5", "--sorted", "--seed", "3"], check=True, capture_output=True)
    xadj, adj, w, lab = gpu.csr_read(prefix)
    out = str(tmp_path / "p.bin")
    _run("--input", prefix, "--node2vec", "--n=200", "--seq", "--d=10", "--seed=9", "--savepaths", out)
    paths = np.fromfile(out, dtype=np.int32).reshape(200, 11)
    ref, _, _ = orc.walk(orc.Graph(xadj, adj, w, lab), orc.make_params(app=2, max_depth=11, seed=9, p=2.0, q=0.5),
                         np.arange(200, dtype=np.int32))
    assert (paths == ref).all()


def test_sampler_micro_benchmark_takes_the_reference_command_lines(gpu):
    """The commands of the reference's README for Figure 6a / 6b (README.md:128-149: `--groupsize=$SAMPLING_SIZE --gran=32
    --type=1` ...) and the same measurements spelled as the flags' own descriptions have them (src/sampler_test.cu:33-35:
    --groupsize = threads of a sampler, --gran = elements per sampler) run, sample every list once and end with the
    reference's "Elapsed time" line (src/sampler_test.cu:915).  --elements shrinks the 512 Mi-element array for the test."""
    tool = os.path.join(ROOT, "flowwalker-artifact_amd", "bin", "fw_sampler_bench")
    size = 1 << 20
    readme = [(1, 32), (2, 512), (5, 32), (6, 512), (7, 32), (8, 512), (3, 32), (4, 512)]
    names = {1: "zprs", 2: "zprs", 3: "dprs", 4: "dprs", 5: "its", 6: "its", 7: "als", 8: "als"}
    for sampling_size in (128, 2048):
        for typ, gran in (readme if sampling_size == 128 else readme[:2]):
            for args in (["--groupsize=%d" % sampling_size, "--gran=%d" % gran, "--type=%d" % typ],       # README.md
                         ["--groupsize=%d" % gran, "--gran=%d" % sampling_size, "--type=%d" % typ]):      # the source's flags
                r = subprocess.run([tool, "--elements=%d" % size] + args, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                                   text=True, timeout=300)
                assert r.returncode == 0, (args, r.stderr)
                cfg = re.search(r"Number of Threads in a Sampler: (\d+), Sampler Type: (\d+) \((\w+)\), Number of Elements "
                                r"Processed by a Sampler: (\d+), Number of tasks: (\d+)", r.stdout)
                assert cfg, r.stdout
                assert int(cfg.group(1)) == (64 if typ % 2 else 512) and int(cfg.group(2)) == typ
                assert cfg.group(3) == names[typ]
                assert int(cfg.group(4)) == sampling_size and int(cfg.group(5)) == size // sampling_size
                assert int(re.search(r"Samples: (\d+),", r.stdout).group(1)) == size // sampling_size
                assert float(re.search(r"Elapsed time: ([0-9.]+) ms", r.stdout).group(1)) > 0.0
    # a size flag without a numeric type is refused instead of being read as this tool's own list-length flag
    r = subprocess.run([tool, "--gran=32", "--type", "native"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert r.returncode == 2 and "--lengths" in r.stderr


def test_save_degree_and_lognorm(gpu, graph_files, tmp_path):
    """--save_degree writes how many steps left a vertex of each degree (src/main.cu:115-149); --lognorm replaces
    the file's weights by log-normal(0, 3) draws (include/graph.cuh:79-91), so the walks change but stay walks."""
    prefix, (xadj, adj, w, lab) = graph_files
    out, hist = str(tmp_path / "p.bin"), str(tmp_path / "bucket.csv")
    _run("--input", prefix, "--deepwalk", "--n=300", "--seq", "--d=12", "--seed=4", "--save_degree", "--b_file", hist,
         "--savepaths", out)
    paths = np.fromfile(out, dtype=np.int32).reshape(300, 13)
    deg = np.diff(xadj.astype(np.int64))
    want = {}
    for row in paths:
        for j in range(1, 13):
            if row[j] < 0:
                break
            want[int(deg[row[j - 1]])] = want.get(int(deg[row[j - 1]]), 0) + 1
    got = {int(a): int(b) for a, b in (ln.split(",") for ln in open(hist).read().split())}
    assert got == want and list(got) == sorted(got)

    out2 = str(tmp_path / "p2.bin")
    _run("--input", prefix, "--deepwalk", "--n=300", "--seq", "--d=12", "--seed=4", "--lognorm", "--savepaths", out2)
    p2 = np.fromfile(out2, dtype=np.int32).reshape(300, 13)
    assert (p2[:, 0] == paths[:, 0]).all() and (p2 != paths).any()
    for row in p2[:50]:                                    # every hop is an edge of the graph
        for j in range(1, 13):
            if row[j] < 0:
                break
            assert row[j] in adj[xadj[row[j - 1]]:xadj[row[j - 1] + 1]]


def test_ablation_levels_and_park_threshold(gpu, graph_files, tmp_path):
    """--walkmode 9 / 10 / 1 / 6 are the reference's ablation levels (README.md:152-163), run by its own samplers restated
    for 64-lane waves: DPRS, static assignment, thread-owned generators in device memory; the same with the generators
    in LDS (same walks); ZPRS instead of DPRS; ZPRS with the dispenser (draws addressed by walker, step and element).
    20 / 21 / 22 are this engine's levels (wave sampler alone, + workgroup sampler, + parking).  Every level equals the
    oracle run with its settings -- the statically assigned levels the oracle's thread-by-thread replay of the launch
    the tool reports (grid and block)."""
    prefix, csr = graph_files
    V = len(csr[0]) - 1
    starts = np.arange(V, dtype=np.int32)
    og = orc.Graph(*csr)
    ref_wg, _, _ = orc.walk(og, orc.make_params(max_depth=11, seed=3, hub_threshold=1000), starts)
    ref_wave, _, _ = orc.walk(og, orc.make_params(max_depth=11, seed=3, hub_threshold=0x7FFFFFFF), starts)
    ref_zprs, _, _ = orc.walk(og, orc.make_params(sampler=2, max_depth=11, seed=3, hub_threshold=1000), starts)
    assert (ref_zprs != ref_wg).any()
    seen = {}
    for mode, ref, note in ((9, None, "DPRS samplers on 64-lane waves, static query assignment, thread-owned generators in device memory"),
                            (10, None, "DPRS samplers on 64-lane waves, static query assignment, thread-owned generators in LDS"),
                            (1, None, "ZPRS samplers on 64-lane waves, static query assignment, thread-owned generators in LDS"),
                            (6, ref_zprs, "ZPRS samplers on 64-lane waves, global query dispenser, draws addressed by"),
                            (20, ref_wave, "wave sampler only"), (21, ref_wg, "no parking"), (22, ref_wg, "full engine")):
        out = str(tmp_path / ("m%d.bin" % mode))
        text = _run("--input", prefix, "--deepwalk", "--all", "--d=10", "--seed=3", "--hub_threshold=1000",
                    "--walkmode=%d" % mode, "--savepaths", out)
        assert "ablation level %d" % mode in text and note in text
        got = np.fromfile(out, dtype=np.int32).reshape(V, 11)
        if ref is None:
            launch = re.search(r"grid:(\d+),block:(\d+)", text)
            ref, _, _ = orc.walk_ref_threads(og, orc.make_params(sampler=3 if mode in (9, 10) else 2, max_depth=11, seed=3,
                                                                 hub_threshold=1000, wg_threads=int(launch.group(2))),
                                             starts, int(launch.group(1)))
        assert (got == ref).all(), mode
        seen[mode] = got
    assert (seen[9] == seen[10]).all() and (seen[10] != seen[1]).any() and (seen[1] != seen[6]).any()
    for park in (-1, 50):
        out = str(tmp_path / ("k%d.bin" % park))
        _run("--input", prefix, "--deepwalk", "--all", "--d=10", "--seed=3", "--hub_threshold=1000",
             "--park_threshold=%d" % park, "--savepaths", out)
        assert (np.fromfile(out, dtype=np.int32).reshape(V, 11) == ref_wg).all(), park


def test_umgraph_keeps_edges_on_the_host(gpu, graph_files, tmp_path):
    """--umgraph (src/main.cu:48): the graph's edge arrays are not copied to the device; same walks."""
    prefix, csr = graph_files
    V = len(csr[0]) - 1
    ref, _, _ = orc.walk(orc.Graph(*csr), orc.make_params(max_depth=11, seed=9), np.arange(V, dtype=np.int32))
    out = str(tmp_path / "um.bin")
    text = _run("--input", prefix, "--deepwalk", "--all", "--d=10", "--seed=9", "--umgraph", "--savepaths", out)
    assert "umgraph: edge arrays stay in pinned host memory" in text
    assert (np.fromfile(out, dtype=np.int32).reshape(V, 11) == ref).all()


def _shuffled_lists(csr, seed):
    """The same graph with every neighbour list in random order (weights and labels move with their edges)."""
    xadj, adj, w, lab = (a.copy() for a in csr)
    rng = np.random.RandomState(seed)
    for v in range(len(xadj) - 1):
        b, e = int(xadj[v]), int(xadj[v + 1])
        perm = rng.permutation(e - b)
        adj[b:e], w[b:e], lab[b:e] = adj[b:e][perm], w[b:e][perm], lab[b:e][perm]
    return xadj, adj, w, lab


def test_node2vec_on_unsorted_lists(gpu, graph_files, tmp_path):
    """The reference's converter writes neighbour lists in insertion order (data/EdgeListToCSR.cpp:182-191) and its
    README runs --node2vec on such files.  The command line sorts them at load (weights follow their edges), so the
    walks equal those on the sorted graph; the C ABI refuses node2vec on an unsorted device graph instead of
    computing wrong biases."""
    prefix, csr = graph_files
    V = len(csr[0]) - 1
    shuffled = _shuffled_lists(csr, seed=4)
    assert (shuffled[1] != csr[1]).any()
    sp = str(tmp_path / "shuffled")
    gpu.csr_write(sp, *shuffled)
    out = str(tmp_path / "n2v.bin")
    text = _run("--input", sp, "--node2vec", "--n=500", "--seq", "--d=12", "--seed=21", "--dprs", "--savepaths", out)
    assert re.search(r"node2vec: \d+ neighbour lists were not ascending and have been sorted", text)
    ref, _, _ = orc.walk(orc.Graph(*csr), orc.make_params(app=2, max_depth=13, seed=21, hub_threshold=(1 << 31) - 1),
                         np.arange(500, dtype=np.int32))
    assert (np.fromfile(out, dtype=np.int32).reshape(500, 13) == ref).all()

    g = gpu.Graph.from_csr(*shuffled)
    try:
        assert not g.is_sorted()
        with pytest.raises(gpu.FlowWalkerError) as e:
            g.walk(gpu.default_params(app=gpu.APP_NODE2VEC, max_depth=5), np.arange(10, dtype=np.int32))
        assert e.value.status == 1 and "ascending" in str(e.value)
        g.walk(gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=5), np.arange(10, dtype=np.int32))  # others do not care
    finally:
        g.destroy()


REF_WIKI = "/root/reference/data/wiki-Vote"


@pytest.mark.skipif(not os.path.exists(REF_WIKI + "_xadj.bin"), reason="the reference's data directory is not mounted here")
def test_readme_node2vec_command_on_the_shipped_graph(gpu, tmp_path):
    """`flowwalker --input ../data/wiki-Vote --node2vec --n=100 --dprs` (README.md:99-105) on the reference's own files,
    3,990 of whose 7,115 lists are not ascending."""
    out = str(tmp_path / "wiki.bin")
    text = _run("--input", REF_WIKI, "--node2vec", "--n=100", "--seq", "--dprs", "--seed=3", "--savepaths", out)
    assert "node2vec: 3990 neighbour lists were not ascending and have been sorted" in text
    xadj, adj, w, _ = gpu.csr_read(REF_WIKI)
    assert gpu.csr_sort_neighbours(xadj, adj, w) == 3990
    ref, _, _ = orc.walk(orc.Graph(xadj, adj, w), orc.make_params(app=2, max_depth=81, seed=3, hub_threshold=(1 << 31) - 1),
                         np.arange(100, dtype=np.int32))
    assert (np.fromfile(out, dtype=np.int32).reshape(100, 81) == ref).all()


def test_bench_line_contract(gpu):
    """bench.py prints ONE JSON line with the agreed fields; the roofline fraction is a fraction (small graph, no CPU leg)."""
    import json
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--scale", "16", "--steps", "2", "--warmup", "1",
                        "--no-cpu"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
    assert r.returncode == 0, r.stderr
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 2 and d["warmup"] == 1 and d["unit"] == "steps/s" and d["vs_baseline"] is None
    assert d["higher_is_better"] is True and d["data"] == "synthetic" and "workload" in d["config"]
    rf = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in rf, key
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and 0.0 < rf["frac"] <= 1.0
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    assert d["value"] > 0 and abs(d["value"] - d["config"]["walk_steps_per_pass"] / (d["ms_per_step"] * 1e-3)) < 1e-6 * d["value"]
