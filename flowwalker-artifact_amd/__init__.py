"""ctypes binding of libflowwalker_hip.so (the C ABI declared in include/flowwalker.h).

This is plumbing for tests and benchmarks: every compute call goes through the C ABI into the HIP
kernels.  There is no CPU fallback; loading fails loudly when the library has not been built
(`python flowwalker-artifact_amd/build.py`).

The package directory name contains a hyphen, so import it with
    importlib.import_module("flowwalker-artifact_amd")
"""
import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
# FLOWWALKER_LIB points at an alternative build of the same library (A/B measurements)
LIB_PATH = os.environ.get("FLOWWALKER_LIB") or os.path.join(_PKG, "lib", "libflowwalker_hip.so")

FW_MAX_SCHEMA = 64
APP_DEEPWALK, APP_PPR, APP_NODE2VEC, APP_METAPATH = 0, 1, 2, 3
SAMPLER_ZPRS, SAMPLER_DPRS, SAMPLER_REF_ZPRS, SAMPLER_REF_DPRS, SAMPLER_REF_STATIC = 0, 1, 2, 3, 0x100
SAMPLER_REF_RNG_LDS, SAMPLER_REF_RNG_GLOBAL = 0x200, 0x400
FW_OK = 0
GRAPH_DEVICE, GRAPH_HOST_PINNED = 0, 1

# every symbol include/flowwalker.h declares
EXPORTED = [
    "fw_last_error", "fw_device_count", "fw_device_mem_info", "fw_walk_params_default", "fw_walk_params_default_for", "fw_autobatch_size",
    "fw_dev_alloc", "fw_dev_free", "fw_dev_upload", "fw_dev_download", "fw_dev_fill_i32", "fw_dev_copy", "fw_dev_sync",
    "fw_graph_create", "fw_graph_adopt_device", "fw_graph_destroy", "fw_graph_info", "fw_graph_is_sorted",
    "fw_graph_download", "fw_walk_device", "fw_walk_batch", "fw_host_alloc_pinned", "fw_host_free_pinned",
    "fw_gen_rmat", "fw_csr_read_header", "fw_csr_load", "fw_csr_write", "fw_graph_load",
    "fw_graph_create_placed", "fw_graph_load_placed", "fw_walk_device_noalloc", "fw_csr_sort_neighbours",
    "fw_sampler_baseline_run", "fw_dev_random_access_rate",
]


BASELINE_ITS, BASELINE_RJS, BASELINE_ALS = 0, 1, 2


class WalkParams(C.Structure):
    _fields_ = [
        ("app", C.c_int32), ("sampler", C.c_int32), ("max_depth", C.c_int32), ("wg_threads", C.c_int32),
        ("hub_threshold", C.c_int32), ("schema_len", C.c_int32), ("schema", C.c_int32 * FW_MAX_SCHEMA),
        ("tp", C.c_float), ("p", C.c_float), ("q", C.c_float), ("walker_base", C.c_uint32),
        ("seed", C.c_uint64), ("grid", C.c_int32), ("park_threshold", C.c_int32),
        ("time_kernels", C.c_int32), ("reserved", C.c_int32),
    ]


class WalkStats(C.Structure):
    _fields_ = [
        ("kernel_ms", C.c_double), ("total_ms", C.c_double), ("steps", C.c_uint64),
        ("sampled_edges", C.c_uint64), ("launches", C.c_int32), ("grid", C.c_int32),
        ("walk_kernel_ms", C.c_double), ("hub_kernel_ms", C.c_double), ("hub_steps", C.c_uint64),
        ("hub_sampled_edges", C.c_uint64), ("requested_bytes", C.c_uint64), ("list_bytes", C.c_uint64),
        ("scattered_reads", C.c_uint64), ("scattered_writes", C.c_uint64), ("record_bytes", C.c_uint64),
    ]


class RmatParams(C.Structure):
    _fields_ = [
        ("scale", C.c_int32), ("edge_factor", C.c_int32), ("a", C.c_float), ("b", C.c_float), ("c", C.c_float),
        ("symmetrise", C.c_int32), ("w_lo", C.c_float), ("w_hi", C.c_float), ("n_labels", C.c_int32),
        ("make_weights", C.c_int32), ("seed", C.c_uint64),
    ]


def sources_sha():
    """Short hash of the kernel sources (csrc/*.hip, *.h and the public header): names the build a measurement was
    taken on."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(_PKG, "csrc")
    files = sorted(os.path.join(csrc, f) for f in os.listdir(csrc) if f.endswith((".hip", ".h")))
    files.append(os.path.join(os.path.dirname(_PKG), "include", "flowwalker.h"))
    for f in files:
        h.update(os.path.basename(f).encode())
        h.update(open(f, "rb").read())
    return h.hexdigest()[:12]


class FlowWalkerError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("flowwalker status %d: %s" % (status, message))
        self.status = status


_lib = None


def lib():
    """Loads the shared library once; raises if it is missing (no fallback path exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                "%s is not built; run `python flowwalker-artifact_amd/build.py` (there is no CPU fallback)" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        L.fw_last_error.restype = C.c_char_p
        L.fw_autobatch_size.restype = C.c_uint32
        L.fw_autobatch_size.argtypes = [C.c_size_t, C.c_int32, C.c_int32, C.c_int, C.c_uint32]
        L.fw_device_mem_info.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
        L.fw_walk_params_default.argtypes = [C.POINTER(WalkParams)]
        L.fw_walk_params_default.restype = None
        L.fw_walk_params_default_for.argtypes = [C.POINTER(WalkParams), C.c_int]
        L.fw_walk_params_default_for.restype = None
        L.fw_dev_alloc.argtypes = [C.c_size_t, C.POINTER(C.c_void_p)]
        L.fw_dev_free.argtypes = [C.c_void_p]
        L.fw_dev_upload.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.fw_dev_download.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.fw_dev_fill_i32.argtypes = [C.c_void_p, C.c_int32, C.c_size_t]
        L.fw_dev_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.fw_graph_create.argtypes = [C.c_int32, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.POINTER(C.c_void_p)]
        L.fw_graph_create_placed.argtypes = [C.c_int32, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                             C.c_int, C.POINTER(C.c_void_p)]
        L.fw_graph_adopt_device.argtypes = [C.c_int32, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                            C.c_int, C.POINTER(C.c_void_p)]
        L.fw_graph_destroy.argtypes = [C.c_void_p]
        L.fw_graph_info.argtypes = [C.c_void_p, C.POINTER(C.c_int32), C.POINTER(C.c_uint64), C.POINTER(C.c_int32),
                                    C.POINTER(C.c_int32)]
        L.fw_graph_is_sorted.argtypes = [C.c_void_p, C.POINTER(C.c_int)]
        L.fw_graph_download.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.fw_walk_device.argtypes = [C.c_void_p, C.POINTER(WalkParams), C.c_void_p, C.c_int32, C.c_void_p,
                                     C.c_void_p, C.POINTER(WalkStats)]
        L.fw_walk_device_noalloc.argtypes = L.fw_walk_device.argtypes
        L.fw_walk_batch.argtypes = [C.c_void_p, C.POINTER(WalkParams), C.c_void_p, C.c_int32, C.c_uint32, C.c_int,
                                    C.c_void_p, C.POINTER(WalkStats)]
        L.fw_host_alloc_pinned.argtypes = [C.c_size_t, C.POINTER(C.c_void_p)]
        L.fw_host_free_pinned.argtypes = [C.c_void_p]
        L.fw_gen_rmat.argtypes = [C.POINTER(RmatParams), C.POINTER(C.c_void_p)]
        L.fw_csr_read_header.argtypes = [C.c_char_p, C.POINTER(C.c_int32), C.POINTER(C.c_uint64)]
        L.fw_csr_load.argtypes = [C.c_char_p, C.c_int32, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.fw_csr_write.argtypes = [C.c_char_p, C.c_int32, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.fw_csr_sort_neighbours.argtypes = [C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                             C.POINTER(C.c_int64)]
        L.fw_graph_load.argtypes = [C.c_char_p, C.c_int, C.c_int, C.POINTER(C.c_void_p)]
        L.fw_dev_random_access_rate.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.POINTER(C.c_double)]
        L.fw_sampler_baseline_run.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_uint64, C.c_uint32, C.c_void_p, C.c_uint32,
                                              C.c_int, C.c_uint64, C.c_void_p, C.POINTER(C.c_double)]
        L.fw_graph_load_placed.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_void_p)]
        _lib = L
    return _lib


def check(status):
    if status != FW_OK:
        raise FlowWalkerError(status, lib().fw_last_error().decode("utf-8", "replace"))


def device_count():
    return int(lib().fw_device_count())


def mem_info():
    f, t = C.c_size_t(), C.c_size_t()
    check(lib().fw_device_mem_info(C.byref(f), C.byref(t)))
    return f.value, t.value


def default_params(**overrides):
    p = WalkParams()
    if "app" in overrides:  # the library's choices for that application (node2vec: wave granularity)
        lib().fw_walk_params_default_for(C.byref(p), int(overrides["app"]))
    else:
        lib().fw_walk_params_default(C.byref(p))
    set_params(p, **overrides)
    return p


def set_params(params, /, **kw):
    for k, v in kw.items():
        if k == "schema":
            v = list(v)
            params.schema_len = len(v)
            for i, s in enumerate(v[:FW_MAX_SCHEMA]):
                params.schema[i] = int(s)
        else:
            if not hasattr(params, k):
                raise AttributeError("unknown walk parameter %r" % k)
            setattr(params, k, v)
    return params


def _ptr(arr):
    return None if arr is None else arr.ctypes.data_as(C.c_void_p)


def csr_read(prefix, weights=True, labels=False):
    """Reads <prefix>_xadj/_edge/_weight/_label.bin (host side only).  Returns (xadj, adjncy, weight, label)."""
    V, E = C.c_int32(), C.c_uint64()
    check(lib().fw_csr_read_header(prefix.encode(), C.byref(V), C.byref(E)))
    xadj = np.empty(V.value + 1, dtype=np.uint32)
    adjncy = np.empty(E.value, dtype=np.int32)
    weight = np.empty(E.value, dtype=np.float32) if weights else None
    label = np.empty(E.value, dtype=np.int32) if labels else None
    check(lib().fw_csr_load(prefix.encode(), V.value, E.value, _ptr(xadj), _ptr(adjncy), _ptr(weight), _ptr(label)))
    return xadj, adjncy, weight, label


def csr_write(prefix, xadj, adjncy, weight=None, label=None):
    xadj = np.ascontiguousarray(xadj, dtype=np.uint32)
    adjncy = np.ascontiguousarray(adjncy, dtype=np.int32)
    weight = None if weight is None else np.ascontiguousarray(weight, dtype=np.float32)
    label = None if label is None else np.ascontiguousarray(label, dtype=np.int32)
    check(lib().fw_csr_write(prefix.encode(), len(xadj) - 1, len(adjncy), _ptr(xadj), _ptr(adjncy), _ptr(weight),
                             _ptr(label)))


def csr_sort_neighbours(xadj, adjncy, weight=None, label=None):
    """Sorts the neighbour lists in place (weight / label follow their edges).  Returns the number of lists changed."""
    n = C.c_int64()
    check(lib().fw_csr_sort_neighbours(len(xadj) - 1, _ptr(xadj), _ptr(adjncy), _ptr(weight), _ptr(label), C.byref(n)))
    return n.value


class DeviceBuffer:
    """A device allocation owned by the library (so hosts need no HIP binding of their own)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(lib().fw_dev_alloc(self.nbytes, C.byref(p)))
        self.ptr = p

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        check(lib().fw_dev_upload(buf.ptr, _ptr(arr), arr.nbytes))
        return buf

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        check(lib().fw_dev_download(_ptr(out), self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr is not None and self.ptr.value:
            check(lib().fw_dev_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Graph:
    """Device CSR mirror (fw_graph)."""

    def __init__(self, handle):
        self.handle = handle
        V, E, md, mv = C.c_int32(), C.c_uint64(), C.c_int32(), C.c_int32()
        check(lib().fw_graph_info(self.handle, C.byref(V), C.byref(E), None, None))
        self.V, self.E = V.value, E.value

    @classmethod
    def from_csr(cls, xadj, adjncy, weight=None, label=None, placement=GRAPH_DEVICE):
        xadj = np.ascontiguousarray(xadj, dtype=np.uint32)
        adjncy = np.ascontiguousarray(adjncy, dtype=np.int32)
        weight = None if weight is None else np.ascontiguousarray(weight, dtype=np.float32)
        label = None if label is None else np.ascontiguousarray(label, dtype=np.int32)
        h = C.c_void_p()
        check(lib().fw_graph_create_placed(len(xadj) - 1, len(adjncy), _ptr(xadj), _ptr(adjncy), _ptr(weight),
                                           _ptr(label), placement, C.byref(h)))
        return cls(h)

    @classmethod
    def load(cls, prefix, weights=True, labels=False, placement=GRAPH_DEVICE):
        h = C.c_void_p()
        check(lib().fw_graph_load_placed(prefix.encode(), int(weights), int(labels), placement, C.byref(h)))
        return cls(h)

    @classmethod
    def rmat(cls, scale, edge_factor=16, a=0.57, b=0.19, c=0.19, symmetrise=False, w_lo=1.0, w_hi=100.0,
             n_labels=0, make_weights=True, seed=1):
        rp = RmatParams(scale, edge_factor, a, b, c, int(symmetrise), w_lo, w_hi, n_labels, int(make_weights), seed)
        h = C.c_void_p()
        check(lib().fw_gen_rmat(C.byref(rp), C.byref(h)))
        return cls(h)

    def max_degree(self):
        md, mv = C.c_int32(), C.c_int32()
        check(lib().fw_graph_info(self.handle, None, None, C.byref(md), C.byref(mv)))
        return md.value, mv.value

    def is_sorted(self):
        s = C.c_int()
        check(lib().fw_graph_is_sorted(self.handle, C.byref(s)))
        return bool(s.value)

    def download(self, weights=True, labels=False):
        xadj = np.empty(self.V + 1, dtype=np.uint32)
        adjncy = np.empty(self.E, dtype=np.int32)
        weight = np.empty(self.E, dtype=np.float32) if weights else None
        label = np.empty(self.E, dtype=np.int32) if labels else None
        check(lib().fw_graph_download(self.handle, _ptr(xadj), _ptr(adjncy), _ptr(weight), _ptr(label)))
        return xadj, adjncy, weight, label

    def download_xadj(self):
        xadj = np.empty(self.V + 1, dtype=np.uint32)
        check(lib().fw_graph_download(self.handle, _ptr(xadj), None, None, None))
        return xadj

    def walk_device(self, params, d_starts, n, d_paths):
        """One launch over device-resident starts / paths (DeviceBuffer objects).  Returns WalkStats."""
        st = WalkStats()
        check(lib().fw_walk_device(self.handle, C.byref(params), d_starts.ptr, int(n), d_paths.ptr, None, C.byref(st)))
        return st

    def walk_device_noalloc(self, params, d_starts, n, d_paths):
        """fw_walk_device_noalloc: one launch, scratch in the library's static device array.  Returns WalkStats."""
        st = WalkStats()
        check(lib().fw_walk_device_noalloc(self.handle, C.byref(params), d_starts.ptr, int(n), d_paths.ptr, None,
                                           C.byref(st)))
        return st

    def walk(self, params, starts):
        """Uploads starts, runs one launch, downloads the path matrix.  Returns (paths, WalkStats)."""
        starts = np.ascontiguousarray(starts, dtype=np.int32)
        n = len(starts)
        d_starts = DeviceBuffer.from_numpy(starts)
        d_paths = DeviceBuffer(n * params.max_depth * 4)
        try:
            st = self.walk_device(params, d_starts, n, d_paths)
            paths = d_paths.to_numpy(np.int32, (n, params.max_depth))
        finally:
            d_starts.free()
            d_paths.free()
        return paths, st

    def walk_batch(self, params, starts, batch_size=0, sync=False):
        """Double-buffered batched walk over host arrays (fw_walk_batch).  Returns (paths, WalkStats)."""
        starts = np.ascontiguousarray(starts, dtype=np.int32)
        n = len(starts)
        paths = np.empty((n, params.max_depth), dtype=np.int32)
        st = WalkStats()
        check(lib().fw_walk_batch(self.handle, C.byref(params), _ptr(starts), n, int(batch_size), int(sync),
                                  _ptr(paths), C.byref(st)))
        return paths, st

    def destroy(self):
        if self.handle is not None and self.handle.value:
            check(lib().fw_graph_destroy(self.handle))
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def sampler_baseline(kind, weights, list_len, tasks=None, workgroup=False, wg_threads=512, seed=1):
    """fw_sampler_baseline_run on host arrays: one index per task from its list_len-element slice of `weights`
    by inverse transform (BASELINE_ITS) or rejection sampling (BASELINE_RJS).  Returns (indices, kernel_ms)."""
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    n = len(tasks) if tasks is not None else len(weights) // int(list_len)
    d_w = DeviceBuffer.from_numpy(weights)
    d_t = DeviceBuffer.from_numpy(np.ascontiguousarray(tasks, dtype=np.uint32)) if tasks is not None else None
    d_o = DeviceBuffer(max(n, 1) * 4)
    ms = C.c_double(0.0)
    try:
        check(lib().fw_sampler_baseline_run(int(kind), int(bool(workgroup)), d_w.ptr, len(weights), int(list_len),
                                            d_t.ptr if d_t is not None else None, n, int(wg_threads), int(seed),
                                            d_o.ptr, C.byref(ms)))
        out = d_o.to_numpy(np.int32, (n,))
    finally:
        d_w.free()
        d_o.free()
        if d_t is not None:
            d_t.free()
    return out, ms.value
