"""fw_convert (edge list -> on-disk CSR) against a restatement of the reference converter's rules
(data/EdgeListToCSR.cpp: GetEdgeList :22-65, WriteCSR :132-268) and, when the reference tree is mounted, against the
graph it ships (data/wiki-Vote*).  Host code only."""
import os
import subprocess

import numpy as np
import pytest

import _graphs  # noqa: F401  (keeps the tests' import path set-up in one place)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "flowwalker-artifact_amd", "bin", "fw_convert")
REF_EDGELIST = "/root/reference/data/wiki-Vote.edgelist"

pytestmark = pytest.mark.skipif(not os.path.exists(TOOL), reason="fw_convert is not built")


def expected_csr(lines):
    """The reference's rules, restated: normalise, drop loops and duplicates, sort, renumber by first appearance,
    append both directions in pair order."""
    pairs = set()
    for ln in lines:
        if not ln.strip() or ln.startswith("#"):
            continue
        u, v = (int(t) for t in ln.split()[:2])
        if u != v:
            pairs.add((min(u, v), max(u, v)))
    renum = {}
    nbrs = []
    for u, v in sorted(pairs):
        for x in (u, v):
            if x not in renum:
                renum[x] = len(renum)
                nbrs.append([])
        a, b = renum[u], renum[v]
        nbrs[a].append(b)
        nbrs[b].append(a)
    xadj = np.zeros(len(nbrs) + 1, dtype=np.uint32)
    xadj[1:] = np.cumsum([len(n) for n in nbrs])
    adj = np.array([x for n in nbrs for x in n], dtype=np.int32)
    return xadj, adj


def run_tool(tmp_path, lines, *flags, labels=5):
    src = tmp_path / "in.txt"
    src.write_text("".join(ln + "\n" for ln in lines))
    prefix = str(tmp_path / "out")
    subprocess.run([TOOL, str(src), prefix, str(labels), *flags], check=True, capture_output=True)
    hdr = np.fromfile(prefix + "_xadj.bin", dtype=np.int32, count=2)
    V, E = int(hdr[0]), int(hdr[1])
    xadj = np.fromfile(prefix + "_xadj.bin", dtype=np.uint32, offset=8)
    adj = np.fromfile(prefix + "_edge.bin", dtype=np.int32)
    w = np.fromfile(prefix + "_weight.bin", dtype=np.float32)
    lab = np.fromfile(prefix + "_label.bin", dtype=np.int32)
    assert len(xadj) == V + 1 and len(adj) == len(w) == len(lab) == E == int(xadj[-1])
    text = open(prefix + ".edgelist").read().split("\n")
    return xadj, adj, w, lab, [t for t in text if t]


def edge_attrs(xadj, adj, vals):
    src = np.repeat(np.arange(len(xadj) - 1), np.diff(xadj.astype(np.int64)))
    return {(int(s), int(d)): v for s, d, v in zip(src, adj, vals)}


SMALL = ["# a comment", "10 3", "3 10", "7 7", "10 3", "5 3", "42 10", "8 5", "", "3 99", "99 3", "1000 8"]


def test_rules_on_a_small_list(tmp_path):
    xadj, adj, w, lab, text = run_tool(tmp_path, SMALL)
    ex, ea = expected_csr(SMALL)
    assert (xadj == ex).all() and (adj == ea).all()
    assert len(xadj) - 1 == 7            # 3 5 8 10 42 99 1000: vertex 7 only had a loop and disappears
    wa, la = edge_attrs(xadj, adj, w), edge_attrs(xadj, adj, lab)
    for (s, d), v in wa.items():         # one weight and one label per undirected edge
        assert wa[(d, s)] == v and la[(d, s)] == la[(s, d)]
    assert ((w >= 1.0) & (w < 5.0)).all() and ((lab >= 0) & (lab < 5)).all()
    src = np.repeat(np.arange(len(xadj) - 1), np.diff(xadj.astype(np.int64)))
    assert text == ["%d %d" % (s, d) for s, d in zip(src, adj)]


def test_seed_and_sorted_lists(tmp_path):
    rng = np.random.RandomState(3)
    lines = ["%d %d" % (a, b) for a, b in rng.randint(0, 300, size=(4000, 2))]
    a1 = run_tool(tmp_path, lines, "--seed", "7")
    a2 = run_tool(tmp_path, lines, "--seed", "7")
    a3 = run_tool(tmp_path, lines, "--seed", "8")
    assert all((x == y).all() for x, y in zip(a1[:4], a2[:4]))
    assert (a1[1] == a3[1]).all() and not (a1[2] == a3[2]).all()
    xs, adj_s, ws, labs, _ = run_tool(tmp_path, lines, "--seed", "7", "--sorted", "--wlo", "2", "--whi", "3", labels=2)
    assert (xs == a1[0]).all()
    for v in range(len(xs) - 1):
        assert (np.diff(adj_s[xs[v]:xs[v + 1]]) > 0).all()
    assert edge_attrs(xs, adj_s, labs).keys() == edge_attrs(a1[0], a1[1], a1[3]).keys()
    assert ((ws >= 2.0) & (ws < 3.0)).all() and set(np.unique(labs)) <= {0, 1}
    wa = edge_attrs(xs, adj_s, ws)
    assert all(wa[(d, s)] == v for (s, d), v in wa.items())


@pytest.mark.skipif(not os.path.exists(REF_EDGELIST), reason="the reference's example graph is not mounted")
def test_shipped_example_graph(tmp_path):
    lines = open(REF_EDGELIST).read().split("\n")
    xadj, adj, w, lab, _ = run_tool(tmp_path, lines)
    ex, ea = expected_csr(lines)
    assert (xadj == ex).all() and (adj == ea).all()
    hdr = np.fromfile("/root/reference/data/wiki-Vote_xadj.bin", dtype=np.int32, count=2)
    ref_xadj = np.fromfile("/root/reference/data/wiki-Vote_xadj.bin", dtype=np.uint32, offset=8)
    assert (len(xadj) - 1, len(adj)) == (int(hdr[0]), int(hdr[1])) == (7115, 201524)
    # the shipped list is already renumbered, and renumbering it again permutes the vertices: same degree multiset
    assert (np.sort(np.diff(xadj.astype(np.int64))) == np.sort(np.diff(ref_xadj.astype(np.int64)))).all()
