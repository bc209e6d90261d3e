"""ctypes binding of the CPU oracle (oracle/libfw_oracle.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "libfw_oracle.so")

FW_MAX_SCHEMA = 64
STREAM_WAVE = 0x40000000
STREAM_STOP = 0x80000000


class OracleParams(C.Structure):
    _fields_ = [
        ("app", C.c_int32), ("sampler", C.c_int32), ("max_depth", C.c_int32), ("wg_threads", C.c_int32),
        ("hub_threshold", C.c_int32), ("schema_len", C.c_int32), ("schema", C.c_int32 * FW_MAX_SCHEMA),
        ("tp", C.c_float), ("inv_p", C.c_float), ("inv_q", C.c_float), ("walker_base", C.c_uint32),
        ("seed", C.c_uint64),
    ]


class OracleGraph(C.Structure):
    _fields_ = [("V", C.c_int32), ("xadj", C.c_void_p), ("adjncy", C.c_void_p), ("weight", C.c_void_p),
                ("label", C.c_void_p)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_LIB):
            subprocess.check_call(["make", "-C", ORACLE_DIR])
        L = C.CDLL(ORACLE_LIB)
        L.fw_oracle_philox4x32_10.argtypes = [C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
        L.fw_oracle_philox4x32_10.restype = None
        L.fw_oracle_uniform.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32]
        L.fw_oracle_uniform.restype = C.c_float
        L.fw_oracle_wave_scan.argtypes = [C.c_void_p]
        L.fw_oracle_wave_scan.restype = None
        L.fw_oracle_sample.argtypes = [C.POINTER(OracleGraph), C.POINTER(OracleParams), C.c_int32, C.c_int32,
                                       C.c_uint32, C.c_uint32]
        L.fw_oracle_sample.restype = C.c_int32
        L.fw_oracle_walk.argtypes = [C.POINTER(OracleGraph), C.POINTER(OracleParams), C.c_void_p, C.c_int64,
                                     C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.c_int]
        L.fw_oracle_walk.restype = C.c_int
        L.fw_oracle_num_threads.restype = C.c_int
        L.fw_oracle_walk_ref_threads.argtypes = [C.POINTER(OracleGraph), C.POINTER(OracleParams), C.c_void_p, C.c_int64,
                                                 C.c_int32, C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        L.fw_oracle_walk_ref_threads.restype = C.c_int
        L.fw_oracle_enumerate_draw.argtypes = [C.c_void_p, C.c_int32, C.c_uint32, C.c_int32, C.c_uint32, C.c_uint32,
                                               C.c_uint64, C.c_uint32, C.c_uint32, C.c_void_p]
        L.fw_oracle_sample_forced.argtypes = [C.c_void_p, C.c_int32, C.c_uint32, C.c_int32, C.c_uint32, C.c_uint32,
                                              C.c_float, C.c_uint64, C.c_uint32, C.c_uint32]
        L.fw_oracle_sample_forced.restype = C.c_int32
        L.fw_oracle_walk_ids.argtypes = [C.POINTER(OracleGraph), C.POINTER(OracleParams), C.c_void_p, C.c_void_p,
                                         C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        L.fw_oracle_sequential_reservoir.argtypes = [C.c_void_p, C.c_void_p, C.c_int32]
        L.fw_oracle_sequential_reservoir.restype = C.c_int32
        for name in ("fw_ref_sampler_thread", "fw_ref_sampler_zprs", "fw_ref_sampler_dprs"):
            getattr(L, name).restype = C.c_int32
        L.fw_ref_sampler_thread.argtypes = [C.c_void_p, C.c_int32, C.c_void_p]
        L.fw_ref_sampler_zprs.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]
        L.fw_ref_sampler_dprs.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]
        L.fw_ref_sample_many.argtypes = [C.c_int, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_int64, C.c_void_p]
        L.fw_ref_sample_many.restype = C.c_int
        _lib = L
    return _lib


def philox(ctr, key):
    c = (C.c_uint32 * 4)(*ctr)
    k = (C.c_uint32 * 2)(*key)
    o = (C.c_uint32 * 4)()
    lib().fw_oracle_philox4x32_10(c, k, o)
    return [int(x) for x in o]


def uniform(seed, walker, step, stream, n):
    return float(lib().fw_oracle_uniform(seed, walker, step, stream, n))


def wave_scan(x):
    x = np.ascontiguousarray(x, dtype=np.float32).copy()
    assert x.shape == (64,)
    lib().fw_oracle_wave_scan(x.ctypes.data_as(C.c_void_p))
    return x


class Graph:
    """Host CSR handed to the oracle; keeps the numpy arrays alive."""

    def __init__(self, xadj, adjncy, weight=None, label=None):
        self.xadj = np.ascontiguousarray(xadj, dtype=np.uint32)
        self.adjncy = np.ascontiguousarray(adjncy, dtype=np.int32)
        self.weight = None if weight is None else np.ascontiguousarray(weight, dtype=np.float32)
        self.label = None if label is None else np.ascontiguousarray(label, dtype=np.int32)
        self.V = len(self.xadj) - 1
        self.E = len(self.adjncy)
        p = lambda a: None if a is None else a.ctypes.data_as(C.c_void_p)
        self.c = OracleGraph(self.V, p(self.xadj), p(self.adjncy), p(self.weight), p(self.label))

    def degree(self, v):
        return int(self.xadj[v + 1]) - int(self.xadj[v])


def make_params(app=0, sampler=0, max_depth=81, wg_threads=512, hub_threshold=16384, schema=(0, 1, 2, 3, 4), tp=0.2,
                p=2.0, q=0.5, walker_base=0, seed=1337):
    op = OracleParams()
    op.app, op.sampler, op.max_depth = app, sampler, max_depth
    op.wg_threads, op.hub_threshold = wg_threads, hub_threshold
    op.schema_len = len(schema)
    for i, s in enumerate(schema):
        op.schema[i] = int(s)
    op.tp = tp
    op.inv_p = np.float32(1.0) / np.float32(p)
    op.inv_q = np.float32(1.0) / np.float32(q)
    op.walker_base = walker_base
    op.seed = seed
    return op


def from_walk_params(wp):
    """OracleParams mirroring a flowwalker WalkParams structure."""
    return make_params(app=wp.app, sampler=wp.sampler, max_depth=wp.max_depth, wg_threads=wp.wg_threads,
                       hub_threshold=wp.hub_threshold, schema=[wp.schema[i] for i in range(wp.schema_len)],
                       tp=wp.tp, p=wp.p, q=wp.q, walker_base=wp.walker_base, seed=wp.seed)


def sample(graph, params, cur, prev, walker, step):
    return int(lib().fw_oracle_sample(C.byref(graph.c), C.byref(params), cur, prev, walker, step))


def walk(graph, params, starts, nthreads=0):
    starts = np.ascontiguousarray(starts, dtype=np.int32)
    n = len(starts)
    paths = np.empty((n, params.max_depth), dtype=np.int32)
    steps, edges = C.c_uint64(), C.c_uint64()
    rc = lib().fw_oracle_walk(C.byref(graph.c), C.byref(params), starts.ctypes.data_as(C.c_void_p), n,
                              paths.ctypes.data_as(C.c_void_p), C.byref(steps), C.byref(edges), nthreads)
    assert rc == 0, "oracle rejected the parameters"
    return paths, steps.value, edges.value


def walk_ref_threads(graph, params, starts, grid):
    """The reference's engine with thread-owned generators and static assignment (FW_SAMPLER_REF_ZPRS / _DPRS |
    FW_SAMPLER_REF_STATIC | FW_SAMPLER_REF_RNG_LDS or _GLOBAL), replayed thread by thread for a launch of `grid`
    workgroups of params.wg_threads."""
    starts = np.ascontiguousarray(starts, dtype=np.int32)
    n = len(starts)
    paths = np.empty((n, params.max_depth), dtype=np.int32)
    steps, edges = C.c_uint64(), C.c_uint64()
    rc = lib().fw_oracle_walk_ref_threads(C.byref(graph.c), C.byref(params), starts.ctypes.data_as(C.c_void_p), n,
                                          int(grid), paths.ctypes.data_as(C.c_void_p), C.byref(steps), C.byref(edges))
    assert rc == 0, "oracle rejected the parameters"
    return paths, steps.value, edges.value


def walk_ids(graph, params, starts, walker_ids, nthreads=0):
    """Walks of chosen global walker ids (rows of a larger job): returns the path rows."""
    starts = np.ascontiguousarray(starts, dtype=np.int32)
    ids = np.ascontiguousarray(walker_ids, dtype=np.uint32)
    assert len(ids) == len(starts)
    paths = np.empty((len(starts), params.max_depth), dtype=np.int32)
    rc = lib().fw_oracle_walk_ids(C.byref(graph.c), C.byref(params), starts.ctypes.data, ids.ctypes.data, len(starts),
                                  paths.ctypes.data, None, None, nthreads)
    assert rc == 0, "oracle rejected the parameters"
    return paths


def sequential_reservoir(w, u):
    w = np.ascontiguousarray(w, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    return int(lib().fw_oracle_sequential_reservoir(w.ctypes.data_as(C.c_void_p), u.ctypes.data_as(C.c_void_p), len(w)))


REF_THREAD, REF_ZPRS, REF_DPRS, REF64_ZPRS, REF64_DPRS = 0, 1, 2, 3, 4


def ref_sample_many(kind, w, u, width=32):
    """The reference's own samplers restated (fw_ref_samplers.c): row r of `u` (one uniform per bias) drives step r."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    assert u.ndim == 2 and u.shape[1] == len(w)
    out = np.empty(u.shape[0], dtype=np.int32)
    rc = lib().fw_ref_sample_many(kind, w.ctypes.data, len(w), width, u.ctypes.data, u.shape[0], out.ctypes.data)
    if rc != 0:
        raise ValueError("fw_ref_sample_many: bad arguments")
    return out


STREAM_WAVE = 0x40000000


def enumerate_draw(bias, off, nw, stream, index, seed=1, walker=0, step=0):
    """Counts, over all 2^24 values of one uniform of a sampling step, how often each local index is picked.
    Returns int64[deg + 1]: entry 0 counts "no pick" (-1), entry i + 1 counts index i."""
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    counts = np.zeros(len(bias) + 1, dtype=np.uint64)
    rc = lib().fw_oracle_enumerate_draw(bias.ctypes.data, len(bias), off, nw, stream, index, seed, walker, step,
                                        counts.ctypes.data)
    if rc != 0:
        raise ValueError("fw_oracle_enumerate_draw failed")
    return counts.astype(np.int64)


def sample_forced(bias, off, nw, stream, index, value, seed=1, walker=0, step=0):
    """The local index one sampling step returns when one of its uniforms is forced to `value`."""
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    return int(lib().fw_oracle_sample_forced(bias.ctypes.data, len(bias), off, nw, stream, index, float(value), seed,
                                             walker, step))
