"""Python handle on the test oracle (oracle/coral_oracle.c) and, where it was
built, on the reference harness (oracle/_ref/libcoral_ref.so).

TEST INFRASTRUCTURE: imported by tests/, by the smoke check and by the
cpu_baseline leg of bench.py only.  Nothing under coral_amd/ imports this.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libcoral_oracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libcoral_ref.so")

L2, IP = 0, 1
ORDER_GPU_SEQ, ORDER_GPU_WARP32, ORDER_CPU_AVX512, ORDER_WAVE64 = 0, 1, 2, 3


class OracleIndex(C.Structure):
    _fields_ = [("base", C.c_void_p), ("nbrs", C.c_void_p), ("n", C.c_int64), ("dim", C.c_int32),
                ("R", C.c_int32), ("start_ids", C.c_void_p), ("n_start", C.c_int32),
                ("deleted", C.c_void_p)]


_lib = None
_ref = None


def build():
    subprocess.run(["make", "-s", "-C", HERE], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.oracle_dist.restype = C.c_float
        _lib.oracle_dist.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int]
        _lib.oracle_dist_avx512_scalar.restype = C.c_float
        _lib.oracle_dist_avx512_scalar.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        _lib.oracle_recall_hits.restype = C.c_int64
        _lib.oracle_recall_hits.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        _lib.oracle_normalize_l2.restype = None
        _lib.oracle_normalize_l2.argtypes = [C.c_void_p, C.c_int64, C.c_int64]
        _lib.oracle_bruteforce.restype = None
        _lib.oracle_bruteforce.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_int, C.c_int,
                                           C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.oracle_bruteforce_order.restype = None
        _lib.oracle_bruteforce_order.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_void_p, C.c_int, C.c_int,
                                                 C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.oracle_search_A.restype = C.c_int
        _lib.oracle_search_A.argtypes = [C.POINTER(OracleIndex), C.c_void_p, C.c_int, C.c_int, C.c_int,
                                         C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_int, C.POINTER(C.c_double)]
        _lib.oracle_search_B.restype = C.c_int
        _lib.oracle_search_B.argtypes = [C.POINTER(OracleIndex), C.c_void_p, C.c_int, C.c_int, C.c_int,
                                         C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_int, C.POINTER(C.c_double)]
        _lib.oracle_queue_run.restype = C.c_int
        _lib.oracle_queue_run.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                          C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    return _lib


def ref():
    """The reference harness, or None where it was not built."""
    global _ref
    if _ref is None and os.path.exists(REF_PATH):
        try:
            _ref = C.CDLL(REF_PATH)
        except OSError:
            return None
        _ref.ref_distance_l2.restype = C.c_float
        _ref.ref_distance_l2.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        _ref.ref_queue_run.restype = C.c_int
        _ref.ref_queue_run.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        _ref.ref_search_in_cpu.restype = C.c_int
        _ref.ref_search_in_cpu.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_void_p,
                                           C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                           C.c_void_p, C.c_void_p, C.c_int, C.POINTER(C.c_double)]
    return _ref


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def dist(q, b, metric=L2, order=ORDER_GPU_SEQ):
    q, b = _f32(q), _f32(b)
    return float(lib().oracle_dist(_p(q), _p(b), q.size, metric, order))


class Problem:
    """Keeps the arrays an OracleIndex points to alive."""

    def __init__(self, base, nbrs, start_ids, deleted=None):
        self.base, self.nbrs, self.start_ids = _f32(base), _i32(nbrs), _i32(start_ids)
        self.deleted = None if deleted is None else np.ascontiguousarray(deleted, dtype=np.uint32)
        self.c = OracleIndex(_p(self.base), _p(self.nbrs), self.base.shape[0], self.base.shape[1],
                             self.nbrs.shape[1], _p(self.start_ids), self.start_ids.size, _p(self.deleted))


def search_A(prob, queries, k, L, M=None, metric=L2, order=ORDER_CPU_AVX512, nthreads=0):
    q = _f32(queries)
    Q = q.shape[0]
    M = prob.start_ids.size if M is None else M
    ids = np.empty((Q, k), np.int32)
    dists = np.empty((Q, k), np.float32)
    stats = np.zeros((Q, 4), np.int32)
    t = C.c_double()
    rc = lib().oracle_search_A(C.byref(prob.c), _p(q), Q, k, L, M, metric, order, _p(ids), _p(dists),
                               _p(stats), nthreads, C.byref(t))
    if rc != 0:
        raise ValueError("oracle_search_A rejected its arguments (%d)" % rc)
    return ids, dists, stats, t.value


def search_B(prob, queries, k, L, metric=L2, start_order=ORDER_GPU_WARP32, nbr_order=ORDER_GPU_SEQ,
             nthreads=0):
    q = _f32(queries)
    Q = q.shape[0]
    ids = np.empty((Q, k), np.int32)
    dists = np.empty((Q, k), np.float32)
    stats = np.zeros((Q, 4), np.int32)
    t = C.c_double()
    rc = lib().oracle_search_B(C.byref(prob.c), _p(q), Q, k, L, metric, start_order, nbr_order, _p(ids),
                               _p(dists), _p(stats), nthreads, C.byref(t))
    if rc != 0:
        raise ValueError("oracle_search_B rejected its arguments (%d)" % rc)
    return ids, dists, stats, t.value


def ref_search_in_cpu(prob, queries, k, L, M=None, nthreads=0):
    r = ref()
    if r is None:
        raise RuntimeError("oracle/_ref is not built")
    q = _f32(queries)
    Q = q.shape[0]
    M = prob.start_ids.size if M is None else M
    ids = np.empty((Q, k), np.int32)
    dists = np.empty((Q, k), np.float32)
    stats = np.zeros((Q, 4), np.int32)
    t = C.c_double()
    r.ref_search_in_cpu(_p(prob.base), _p(prob.nbrs), prob.base.shape[0], prob.base.shape[1],
                        prob.nbrs.shape[1], _p(prob.start_ids), M, _p(q), Q, k, L, _p(ids), _p(dists),
                        _p(stats), nthreads, C.byref(t))
    return ids, dists, stats, t.value


def bruteforce(base, queries, k, metric=L2, deleted=None, order=-1):
    """Exact kNN under (distance, id); order -1 = fp64 closed form, else an fp32 summation order."""
    base, q = _f32(base), _f32(queries)
    ids = np.empty((q.shape[0], k), np.int32)
    dists = np.empty((q.shape[0], k), np.float32)
    d = None if deleted is None else np.ascontiguousarray(deleted, dtype=np.uint32)
    lib().oracle_bruteforce_order(_p(base), base.shape[0], base.shape[1], _p(q), q.shape[0], k, metric, order,
                                  _p(d), _p(ids), _p(dists))
    return ids, dists


def fps(nbrs, first, M):
    nbrs = _i32(nbrs)
    out = np.empty(M, np.int32)
    fn = lib().oracle_fps
    fn.restype, fn.argtypes = None, [C.c_void_p, C.c_int64, C.c_int, C.c_int32, C.c_int, C.c_void_p]
    fn(_p(nbrs), nbrs.shape[0], nbrs.shape[1], int(first), M, _p(out))
    return out


class GraphState:
    """Rows under construction: nbrs [n][R] (-1 padded), dists [n][R], deg [n]; updated in place."""

    def __init__(self, n, R):
        self.nbrs = np.full((n, R), -1, np.int32)
        self.dists = np.zeros((n, R), np.float32)
        self.deg = np.zeros(n, np.int32)

    def copy(self):
        g = GraphState(0, self.nbrs.shape[1])
        g.nbrs, g.dists, g.deg = self.nbrs.copy(), self.dists.copy(), self.deg.copy()
        return g


def nap_batch(base, state, knn, metric=L2, need_discard=True):
    """One batch of the query-aware construction on `state`; returns [written, occlusion evals, member pairs]."""
    base, knn = _f32(base), _i32(knn)
    stats = np.zeros(3, np.int64)
    fn = lib().oracle_nap_batch
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                   C.c_int, C.c_int, C.c_int, C.c_void_p]
    rc = fn(_p(base), base.shape[0], base.shape[1], metric, state.nbrs.shape[1], _p(state.nbrs), _p(state.dists),
            _p(state.deg), _p(knn), knn.shape[0], knn.shape[1], int(bool(need_discard)), _p(stats))
    if rc:
        raise MemoryError("oracle_nap_batch")
    return stats


def enhance_batch(base, state, iso_ids, knn_ids, knn_dists, metric=L2):
    """One batch of the connectivity enhancement; returns [reverse edges, rejected claims, distance evals]."""
    base, iso_ids, knn_ids, knn_dists = _f32(base), _i32(iso_ids), _i32(knn_ids), _f32(knn_dists)
    stats = np.zeros(3, np.int64)
    fn = lib().oracle_enhance_batch
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                   C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
    rc = fn(_p(base), base.shape[0], base.shape[1], metric, state.nbrs.shape[1], _p(state.nbrs), _p(state.dists),
            _p(state.deg), _p(iso_ids), _p(knn_ids), _p(knn_dists), iso_ids.size, knn_ids.shape[1], _p(stats))
    if rc:
        raise MemoryError("oracle_enhance_batch")
    return stats


def enhance_top_batch(base, state, top_ids, knn_ids, knn_dists, metric=L2):
    """One batch of the second enhancement phase (most-hit nodes): candidates = found list + current row."""
    base, top_ids, knn_ids, knn_dists = _f32(base), _i32(top_ids), _i32(knn_ids), _f32(knn_dists)
    stats = np.zeros(3, np.int64)
    fn = lib().oracle_enhance_top_batch
    fn.restype = C.c_int
    fn.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                   C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
    rc = fn(_p(base), base.shape[0], base.shape[1], metric, state.nbrs.shape[1], _p(state.nbrs), _p(state.dists),
            _p(state.deg), _p(top_ids), _p(knn_ids), _p(knn_dists), top_ids.size, knn_ids.shape[1], _p(stats))
    if rc:
        raise MemoryError("oracle_enhance_top_batch")
    return stats


def top_hit_ids(hits, top_n):
    hits = np.ascontiguousarray(hits, dtype=np.uint32)
    out = np.empty(top_n, np.int32)
    fn = lib().oracle_top_hit_ids
    fn.restype, fn.argtypes = None, [C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
    fn(_p(hits), hits.size, top_n, _p(out))
    return out


def max_threads():
    fn = lib().oracle_max_threads
    fn.restype, fn.argtypes = C.c_int, []
    return int(fn())


def recall_hits(res, gt, k):
    res, gt = _i32(res), _i32(gt)
    return int(lib().oracle_recall_hits(res.shape[0], k, gt.shape[1], _p(res), _p(gt)))


def _queue(fn, capacity, ops, dists):
    ops, dists = _i32(ops), _f32(dists)
    ids = np.empty(capacity + 1, np.int32)
    ds = np.empty(capacity + 1, np.float32)
    fl = np.empty(capacity + 1, np.int32)
    cur, npop = np.zeros(1, np.int32), np.zeros(1, np.int32)
    popped = np.empty(max(1, ops.size), np.int32)
    n = fn(capacity, _p(ops), _p(dists), ops.size, _p(ids), _p(ds), _p(fl), _p(cur), _p(popped), _p(npop))
    return ids[:n].copy(), ds[:n].copy(), fl[:n].copy(), int(cur[0]), popped[:npop[0]].copy()


def queue_run(capacity, ops, dists):
    return _queue(lib().oracle_queue_run, capacity, ops, dists)


def ref_queue_run(capacity, ops, dists):
    return _queue(ref().ref_queue_run, capacity, ops, dists)
