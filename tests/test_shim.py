"""The drop-in shim for the reference's host entry points (flowwalker-artifact_amd/host/fw_shim.cpp, quoted in the
integration notes) compiles against the reference's own prototypes of walk_test / walk_batch (include/walker.cuh:49-57,
held by tests/shim_stubs/shim_driver.cpp) and links libflowwalker_hip.so; on a GPU the driver's two path matrices
equal the library's walks."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
STUBS = os.path.join(ROOT, "tests", "shim_stubs")
SHIM = os.path.join(ROOT, "flowwalker-artifact_amd", "host", "fw_shim.cpp")
LIBDIR = os.path.join(ROOT, "flowwalker-artifact_amd", "lib")


def _build(out):
    cmd = ["g++", "-O1", "-std=c++17", "-Wall", "-Werror", "-I" + os.path.join(ROOT, "include"), "-I" + STUBS,
           SHIM, os.path.join(STUBS, "shim_driver.cpp"), "-o", out, "-L" + LIBDIR, "-lflowwalker_hip",
           "-Wl,-rpath," + LIBDIR]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout


def test_shim_compiles_against_the_reference_prototypes(tmp_path):
    _build(str(tmp_path / "shim_driver"))
    listing = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    body = open(SHIM).read()
    assert body[:body.index("// for callers that only see gpu_graph")].strip() in listing  # the notes quote the file itself


@pytest.mark.gpu
def test_shim_walks_equal_the_library(gpu, tmp_path):
    exe = str(tmp_path / "shim_driver")
    _build(exe)
    a, b = str(tmp_path / "test.bin"), str(tmp_path / "batch.bin")
    r = subprocess.run([exe, a, b], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0, r.stdout
    V, deg, depth, n = 2000, 12, 21, 500
    xadj = (np.arange(V + 1) * deg).astype(np.uint32)
    v = np.repeat(np.arange(V), deg)
    k = np.tile(np.arange(deg), V)
    adj = ((v + 1 + k * 37) % V).astype(np.int32)
    w = (1.0 + ((v * 31 + k * 17) % 97)).astype(np.float32)
    adj = np.sort(adj.reshape(V, deg), axis=1).reshape(-1)  # the driver sorts the lists and leaves the weights in place
    g = gpu.Graph.from_csr(xadj, adj, w)
    try:
        starts = ((np.arange(n) * 7) % V).astype(np.int32)
        ref, _ = g.walk(gpu.default_params(app=gpu.APP_DEEPWALK, max_depth=depth), starts)
    finally:
        g.destroy()
    assert (np.fromfile(a, dtype=np.int32).reshape(n, depth) == ref).all()
    assert (np.fromfile(b, dtype=np.int32).reshape(n, depth) == ref).all()
