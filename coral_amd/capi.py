"""ctypes binding of libcoral_search.so (include/coral_search.h).

Loading fails loudly when the library has not been built: there is no Python or
CPU fallback for the search path.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
# CORAL_SEARCH_LIB points at another build of the same library (e.g. an instrumented one)
LIB_PATH = os.environ.get("CORAL_SEARCH_LIB") or os.path.join(HERE, "lib", "libcoral_search.so")

L2, IP = 0, 1
POLICY_ROUNDS, POLICY_BEST_FIRST = 0, 1
MAX_LDS_BEAM, MAX_BEAM = 2048, 65536  # CORAL_MAX_LDS_BEAM, CORAL_MAX_BEAM

OK, ERR_ARG, ERR_GRAPH, ERR_DEVICE, ERR_MEMORY, ERR_IO, ERR_STATE = range(7)


class CoralError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("coral status %d: %s" % (code, msg))
        self.code = code


class IndexDesc(C.Structure):
    _fields_ = [("base", C.c_void_p), ("nbrs", C.c_void_p), ("n", C.c_int64), ("dim", C.c_int32),
                ("R", C.c_int32), ("start_ids", C.c_void_p), ("n_start", C.c_int32),
                ("metric", C.c_int32), ("device", C.c_int32)]


class Stats(C.Structure):
    _fields_ = [("time_s", C.c_double), ("kernel_s", C.c_double), ("hops", C.c_int64), ("expansions", C.c_int64),
                ("dist_evals", C.c_int64), ("rounds", C.c_int64), ("spills", C.c_int64),
                ("screened_rows", C.c_int64), ("exact_rows", C.c_int64), ("beam_words", C.c_int64),
                ("visited_requests", C.c_int64), ("visited_dedupes", C.c_int64)]

    def as_dict(self):
        return {f: getattr(self, f) for f, _ in self._fields_}


class PlanInfo(C.Structure):
    _fields_ = [("kernel", C.c_int32), ("threads", C.c_int32), ("workgroups", C.c_int32), ("lds_bytes", C.c_int32),
                ("screening", C.c_int32), ("screen_row_bytes", C.c_int32), ("visited_form", C.c_int32),
                ("visited_slots_log2", C.c_int32), ("beam_in_hbm", C.c_int32), ("todo_cap", C.c_int32),
                ("cand_cap", C.c_int32), ("query_slots", C.c_int32), ("reserved", C.c_int32 * 4)]

    KERNELS = ("beam_search_kernel", "best_first_wave_kernel", "best_first_long_kernel")
    SCREENING = ("none", "fp16", "int8")
    VISITED = ("lds_table16+hbm_bitmap", "lds_bitmap", "hbm_bytes", "hbm_packed_words", "lds_table16+hbm_state",
               "lds_buckets16x3+hbm_bitmap")

    def as_dict(self):
        d = {f: getattr(self, f) for f, _ in self._fields_ if f != "reserved"}
        d["kernel"] = self.KERNELS[self.kernel]
        d["screening"] = self.SCREENING[self.screening]
        d["visited_form"] = self.VISITED[self.visited_form]
        return d


class Tuning(C.Structure):
    _fields_ = [("visited_slots_log2", C.c_int32), ("workgroups", C.c_int32), ("threads", C.c_int32),
                ("policy", C.c_int32), ("best_first_in_lds", C.c_int32), ("best_first_packed", C.c_int32),
                ("best_first_table_log2", C.c_int32), ("beam_in_hbm", C.c_int32), ("prefetch_rows", C.c_int32),
                ("cand_cap", C.c_int32), ("best_first_long", C.c_int32), ("best_first_buffer", C.c_int32),
                ("screening", C.c_int32), ("visited_choices", C.c_int32)]


class BuildParams(C.Structure):
    _fields_ = [("R", C.c_int32), ("k_b", C.c_int32), ("batch", C.c_int32), ("need_discard", C.c_int32),
                ("connect_enhance", C.c_int32), ("enhance_search_batch", C.c_int32), ("enhance_nap_batch", C.c_int32),
                ("enhance_L", C.c_int32), ("n_start", C.c_int32), ("first_start_id", C.c_int32),
                ("top_hit_num", C.c_int32), ("test_search_frequency", C.c_int32), ("monitor", C.c_void_p),
                ("reserved", C.c_int32 * 2)]


MONITOR_BATCHES, MONITOR_ISOLATED, MONITOR_TOP, MONITOR_DONE = 0, 1, 2, 3
BUILD_REPORT_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.POINTER(Stats), C.c_int64)


class BuildMonitor(C.Structure):
    _fields_ = [("h_queries", C.c_void_p), ("h_gt", C.c_void_p), ("Q", C.c_int32), ("k", C.c_int32), ("L", C.c_int32),
                ("reserved", C.c_int32), ("report", BUILD_REPORT_FN), ("user", C.c_void_p)]


class Monitor:
    """GPUFuncs::test_search during a build: `queries` [Q][dim] searched with beam L and compared with their true
    neighbours `gt` [Q][k] at the points where the reference does it.  Attach to build parameters with `attach`;
    `reports` then collects (phase, done, total, hits, hops, kernel seconds) per search.  Keep the object alive
    while the build runs."""

    def __init__(self, queries, gt, L):
        self.queries = np.ascontiguousarray(queries, dtype=np.float32)
        self.gt = np.ascontiguousarray(gt, dtype=np.int32)
        self.reports = []

        def report(_user, phase, done, total, st, hits):
            self.reports.append((phase, done, total, hits, st.contents.hops, st.contents.kernel_s))

        self._fn = BUILD_REPORT_FN(report)
        self.c = BuildMonitor(self.queries.ctypes.data, self.gt.ctypes.data, self.queries.shape[0], self.gt.shape[1], L,
                              0, self._fn, None)

    def attach(self, params, every_batches=None):
        params.monitor = C.addressof(self.c)
        if every_batches is not None:
            params.test_search_frequency = every_batches
        return params


class BuildStats(C.Structure):
    _fields_ = [("knn_s", C.c_double), ("nap_s", C.c_double), ("enhance_s", C.c_double), ("total_s", C.c_double),
                ("batches", C.c_int64), ("isolated", C.c_int64), ("reverse_edges", C.c_int64),
                ("reverse_rejected", C.c_int64), ("edges", C.c_int64), ("top_hit_nodes", C.c_int64),
                ("top_reverse_edges", C.c_int64)]

    def as_dict(self):
        return {f: getattr(self, f) for f, _ in self._fields_}


def build_params(**kw):
    """The reference's defaults (config.json, CLI), overridden by keyword."""
    p = BuildParams()
    _check(lib().coral_build_params_default(C.byref(p)))
    for k, v in kw.items():
        if not hasattr(p, k):
            raise TypeError("no build parameter %r" % k)
        setattr(p, k, v)
    return p


_lib = None

# name -> (restype, argtypes); also the list of symbols the header declares
SIGNATURES = {
    "coral_last_error": (C.c_char_p, []),
    "coral_index_create": (C.c_int, [C.POINTER(IndexDesc), C.POINTER(C.c_void_p)]),
    "coral_index_destroy": (None, [C.c_void_p]),
    "coral_index_set_graph": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32]),
    "coral_index_set_deleted": (C.c_int, [C.c_void_p, C.c_void_p]),
    "coral_index_mark_deleted": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32]),
    "coral_index_get_deleted": (C.c_int, [C.c_void_p, C.c_void_p]),
    "coral_index_info": (C.c_int, [C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int32),
                                   C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "coral_search_prepare": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.POINTER(Tuning)]),
    "coral_search_gpu": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                   C.c_int32, C.c_int32, C.c_void_p, C.POINTER(Stats)]),
    "coral_search_gpu_noalloc": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                           C.c_int32, C.c_int32, C.c_int32, C.c_void_p]),
    "coral_search_query_counters": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32]),
    "coral_search_row_counters": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32]),
    "coral_search_plan_info": (C.c_int, [C.c_void_p, C.POINTER(PlanInfo)]),
    "coral_search": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                               C.c_int32, C.c_void_p, C.c_void_p, C.POINTER(Stats)]),
    "coral_search_verify": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                      C.POINTER(C.c_int64)]),
    "coral_bruteforce_knn_gpu": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                                           C.c_void_p, C.c_void_p, C.POINTER(C.c_double)]),
    "coral_build_params_default": (C.c_int, [C.c_void_p]),
    "coral_build_begin": (C.c_int, [C.c_void_p, C.c_int32]),
    "coral_build_end": (C.c_int, [C.c_void_p]),
    "coral_build_nap_batch": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32]),
    "coral_build_enhance_batch": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                            C.c_void_p, C.c_void_p]),
    "coral_build_enhance_top_batch": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                                C.c_void_p, C.c_void_p]),
    "coral_build_resume": (C.c_int, [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "coral_build_top_hit_ids": (C.c_int, [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "coral_build_test_search": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int64]),
    "coral_build_connect_enhance": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p]),
    "coral_build_graph": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "coral_build_graph_from_clusters": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "coral_index_get_graph": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "coral_start_ids_fps": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "coral_bruteforce_set_exact_only": (C.c_int, [C.c_void_p, C.c_int32]),
    "coral_bruteforce_last_redone": (C.c_int64, [C.c_void_p]),
    "coral_bruteforce_last_fused": (C.c_int32, [C.c_void_p]),
    "coral_membench": (C.c_int, [C.c_int32, C.c_size_t, C.c_int32, C.c_int32, C.POINTER(C.c_double),
                                 C.POINTER(C.c_double)]),
    "coral_bruteforce_knn": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                                       C.c_void_p, C.POINTER(C.c_double)]),
}


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("%s is missing: build it with `python -m coral_amd.build`" % LIB_PATH)
        _lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(_lib, name)
            fn.restype, fn.argtypes = res, args
        from . import formats  # registers the format entry points on the same handle
        formats.register(_lib)
    return _lib


def _check(rc):
    if rc != 0:
        raise CoralError(rc, lib().coral_last_error().decode("utf-8", "replace"))


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def membench(bytes_=8 << 30, row_bytes=800, reps=3, device=0):
    """(streaming read GB/s, random row gather GB/s) of the device's memory: coral_membench."""
    a, b = C.c_double(), C.c_double()
    _check(lib().coral_membench(device, bytes_, row_bytes, reps, C.byref(a), C.byref(b)))
    return a.value, b.value


class Index:
    """An HBM-resident index (vectors + compact graph rows + start ids)."""

    def __init__(self, base, nbrs, start_ids, metric=L2, device=0):
        """nbrs=None makes a vectors-only index (brute force only)."""
        base = np.ascontiguousarray(base, dtype=np.float32)
        if nbrs is None:
            nbrs, start_ids = np.empty((base.shape[0], 0), np.int32), np.empty(0, np.int32)
            d = IndexDesc(_ptr(base), None, base.shape[0], base.shape[1], 0, None, 0, metric, device)
        else:
            nbrs = np.ascontiguousarray(nbrs, dtype=np.int32)
            start_ids = np.ascontiguousarray(start_ids, dtype=np.int32)
            if base.ndim != 2 or nbrs.ndim != 2 or nbrs.shape[0] != base.shape[0]:
                raise ValueError("base must be [n,dim] and nbrs [n,R]")
            d = IndexDesc(_ptr(base), _ptr(nbrs), base.shape[0], base.shape[1], nbrs.shape[1], _ptr(start_ids),
                          start_ids.size, metric, device)
        h = C.c_void_p()
        _check(lib().coral_index_create(C.byref(d), C.byref(h)))
        self._h = h
        self.n, self.dim, self.R, self.metric = base.shape[0], base.shape[1], nbrs.shape[1], metric
        self.n_start = int(start_ids.size)

    def close(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.coral_index_destroy(self._h)
            self._h = None

    __del__ = close

    def set_graph(self, nbrs, start_ids):
        nbrs = np.ascontiguousarray(nbrs, dtype=np.int32)
        start_ids = np.ascontiguousarray(start_ids, dtype=np.int32)
        if nbrs.shape != (self.n, self.R):
            raise ValueError("nbrs must be [n,R]")
        _check(lib().coral_index_set_graph(self._h, _ptr(nbrs), _ptr(start_ids), start_ids.size))
        self.n_start = int(start_ids.size)

    def set_deleted(self, mask_words):
        if mask_words is None:
            _check(lib().coral_index_set_deleted(self._h, None))
            return
        m = np.ascontiguousarray(mask_words, dtype=np.uint32)
        if m.size != (self.n + 31) // 32:
            raise ValueError("mask must hold ceil(n/32) words")
        _check(lib().coral_index_set_deleted(self._h, _ptr(m)))

    def mark_deleted(self, ids):
        """Tombstone the given ids on the device (GPUFuncs::del_node_mark); earlier tombstones stay."""
        ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
        _check(lib().coral_index_mark_deleted(self._h, _ptr(ids) if ids.size else None, ids.size))

    def get_deleted(self):
        m = np.empty((self.n + 31) // 32, np.uint32)
        _check(lib().coral_index_get_deleted(self._h, _ptr(m)))
        return m

    def prepare(self, Q, L, visited_slots_log2=0, workgroups=0, threads=0, policy=POLICY_ROUNDS, best_first_in_lds=False,
                best_first_packed=False, best_first_table_log2=0, beam_in_hbm=False, prefetch_rows=0, cand_cap=0,
                best_first_long=0, best_first_buffer=0, screening=0, visited_choices=0):
        t = Tuning(visited_slots_log2, workgroups, threads, policy, int(bool(best_first_in_lds)),
                   int(bool(best_first_packed)), best_first_table_log2, int(bool(beam_in_hbm)), prefetch_rows,
                   cand_cap, best_first_long, best_first_buffer, screening, visited_choices)
        _check(lib().coral_search_prepare(self._h, Q, L, C.byref(t)))

    def search(self, queries, k, L, policy=POLICY_ROUNDS, have_delete=False, want_dists=True):
        """Host buffers in and out (the IndexGPU::Search shape)."""
        q = np.ascontiguousarray(queries, dtype=np.float32)
        Q = q.shape[0]
        ids = np.empty((Q, k), dtype=np.int32)
        dists = np.empty((Q, k), dtype=np.float32) if want_dists else None
        st = Stats()
        _check(lib().coral_search(self._h, _ptr(q), Q, k, L, policy, int(have_delete), _ptr(ids), _ptr(dists),
                                  C.byref(st)))
        return ids, dists, st

    def search_device(self, d_queries, d_ids, d_dists, Q, k, policy=POLICY_ROUNDS, have_delete=False,
                      stream=None):
        """Device pointers (ints) in and out (the GPUFuncs::search_gpu shape)."""
        st = Stats()
        _check(lib().coral_search_gpu(self._h, d_queries, d_ids, d_dists, Q, k, policy, int(have_delete),
                                      stream, C.byref(st)))
        return st

    def search_device_noalloc(self, d_queries, d_ids, d_dists, Q, k, L, policy=POLICY_ROUNDS, have_delete=False,
                              stream=None):
        """coral_search_gpu_noalloc: device pointers (ints), fixed scratch inside the library, no allocation, no
        wait: synchronise the stream before reading the results."""
        _check(lib().coral_search_gpu_noalloc(self._h, d_queries, d_ids, d_dists, Q, k, L, policy, int(have_delete),
                                              stream))

    def query_counters(self, Q):
        out = np.empty((Q, 4), dtype=np.int32)
        _check(lib().coral_search_query_counters(self._h, _ptr(out), Q))
        return out

    def row_counters(self, Q):
        """int32 [Q][4] of the last search: rows measured on the smaller copy, fp32 rows read, words of beam state
        moved in global memory, visited-state requests to global memory."""
        out = np.empty((Q, 4), dtype=np.int32)
        _check(lib().coral_search_row_counters(self._h, _ptr(out), Q))
        return out

    def plan_info(self):
        p = PlanInfo()
        _check(lib().coral_search_plan_info(self._h, C.byref(p)))
        return p

    def bruteforce(self, queries, k, have_delete=False, want_dists=True):
        """Exact kNN of host queries among the index's vectors: (ids, dists, seconds)."""
        q = np.ascontiguousarray(queries, dtype=np.float32)
        Q = q.shape[0]
        ids = np.empty((Q, k), dtype=np.int32)
        dists = np.empty((Q, k), dtype=np.float32) if want_dists else None
        t = C.c_double()
        _check(lib().coral_bruteforce_knn(self._h, _ptr(q), Q, k, int(have_delete), _ptr(ids), _ptr(dists),
                                          C.byref(t)))
        return ids, dists, t.value

    def bruteforce_exact_only(self, on=True):
        """Skip (True / 1) or restore (False / 0) the matrix-core screening pass of the exact kNN; 2 keeps the
        screening and selects the candidates from the full distance matrix instead of inside the kernel."""
        _check(lib().coral_bruteforce_set_exact_only(self._h, int(on)))

    def bruteforce_last_fused(self):
        return int(lib().coral_bruteforce_last_fused(self._h))

    def bruteforce_last_redone(self):
        return int(lib().coral_bruteforce_last_redone(self._h))

    def bruteforce_device(self, d_queries, d_ids, d_dists, Q, k, have_delete=False, stream=None):
        t = C.c_double()
        _check(lib().coral_bruteforce_knn_gpu(self._h, d_queries, Q, k, int(have_delete), d_ids, d_dists, stream,
                                              C.byref(t)))
        return t.value

    def start_ids_fps(self, first_id, M):
        """M entry points by farthest-point sampling in hop distance, starting from first_id."""
        out = np.empty(M, dtype=np.int32)
        _check(lib().coral_start_ids_fps(self._h, int(first_id), M, _ptr(out)))
        return out

    # ---- graph construction
    def build_begin(self, R):
        _check(lib().coral_build_begin(self._h, R))
        self.R = R

    def build_end(self):
        _check(lib().coral_build_end(self._h))

    def build_resume(self, nbrs, dists, hits=None):
        """construction state from the rows [n][R], distances and hit counts of an earlier build"""
        nbrs = np.ascontiguousarray(nbrs, np.int32)
        dists = np.ascontiguousarray(dists, np.float32)
        if nbrs.ndim != 2 or nbrs.shape[0] != self.n or dists.shape != nbrs.shape:
            raise ValueError("nbrs and dists must both be [n][R]")
        if hits is not None:
            hits = np.ascontiguousarray(hits, np.uint32)
            if hits.shape != (self.n,):
                raise ValueError("hits must be [n]")
        _check(lib().coral_build_resume(self._h, nbrs.shape[1], _ptr(nbrs), _ptr(dists),
                                        _ptr(hits) if hits is not None else None))
        self.R = nbrs.shape[1]

    def build_nap_batch(self, d_knn_ids, batch, k_b, need_discard=True):
        """d_knn_ids: device pointer (int) to int32 [batch][k_b]."""
        _check(lib().coral_build_nap_batch(self._h, d_knn_ids, batch, k_b, int(bool(need_discard))))

    def build_enhance_batch(self, d_iso_ids, d_knn_ids, d_knn_dists, batch, kn):
        ins, rej = C.c_int64(), C.c_int64()
        _check(lib().coral_build_enhance_batch(self._h, d_iso_ids, d_knn_ids, d_knn_dists, batch, kn, C.byref(ins),
                                               C.byref(rej)))
        return ins.value, rej.value

    def build_enhance_top_batch(self, d_top_ids, d_knn_ids, d_knn_dists, batch, k):
        ins, rej = C.c_int64(), C.c_int64()
        _check(lib().coral_build_enhance_top_batch(self._h, d_top_ids, d_knn_ids, d_knn_dists, batch, k, C.byref(ins),
                                                   C.byref(rej)))
        return ins.value, rej.value

    def build_top_hit_ids(self, top_n):
        """(ids [top_n] by hits descending then id, hits [n])"""
        ids = np.empty(top_n, np.int32)
        hits = np.empty(self.n, np.uint32)
        _check(lib().coral_build_top_hit_ids(self._h, top_n, _ptr(ids), _ptr(hits)))
        return ids, hits

    def build_connect_enhance(self, params):
        st = BuildStats()
        _check(lib().coral_build_connect_enhance(self._h, C.byref(params), C.byref(st)))
        self._refresh_n_start()
        return st

    def _refresh_n_start(self):
        m = C.c_int32()
        _check(lib().coral_index_info(self._h, None, None, None, C.byref(m), None))
        self.n_start = m.value

    def build_graph(self, aux, params):
        """IndexGPU::BuildGPU: the whole construction from host auxiliary queries [A][dim]."""
        aux = np.ascontiguousarray(aux, dtype=np.float32)
        st = BuildStats()
        _check(lib().coral_build_graph(self._h, _ptr(aux), aux.shape[0], C.byref(params), C.byref(st)))
        self.R = params.R
        self._refresh_n_start()
        return st

    def build_test_search(self, params, phase=MONITOR_DONE, done=0, total=0):
        """GPUFuncs::test_search on the graph as it stands, reported to the monitor attached to `params`."""
        _check(lib().coral_build_test_search(self._h, C.byref(params), phase, done, total))

    def build_graph_from_clusters(self, clusters, params):
        """The construction from precomputed clusters, int32 [A][k_b] (the reference's --train_gt_file)."""
        c = np.ascontiguousarray(clusters, dtype=np.int32)
        if c.ndim != 2 or c.shape[1] != params.k_b:
            raise ValueError("clusters must be [A][k_b]")
        st = BuildStats()
        _check(lib().coral_build_graph_from_clusters(self._h, _ptr(c), c.shape[0], C.byref(params), C.byref(st)))
        self.R = params.R
        self._refresh_n_start()
        return st

    def get_graph(self, with_build_state=False):
        """(nbrs, start_ids) or, during a build, (nbrs, dists, deg, start_ids)."""
        nbrs = np.empty((self.n, self.R), np.int32)
        starts = np.empty(self.n_start, np.int32)
        if not with_build_state:
            _check(lib().coral_index_get_graph(self._h, _ptr(nbrs), None, None, _ptr(starts) if starts.size else None))
            return nbrs, starts
        dists = np.empty((self.n, self.R), np.float32)
        deg = np.empty(self.n, np.int32)
        _check(lib().coral_index_get_graph(self._h, _ptr(nbrs), _ptr(dists), _ptr(deg),
                                           _ptr(starts) if starts.size else None))
        return nbrs, dists, deg, starts

    def verify(self, d_ids_res, d_ids_gt, Q, k):
        hits = C.c_int64()
        _check(lib().coral_search_verify(self._h, d_ids_res, d_ids_gt, Q, k, C.byref(hits)))
        return hits.value
