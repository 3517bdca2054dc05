"""Readers and writers for the reference's file formats, bound to the C++
implementation in libcoral_search.so (include/coral_formats.h)."""
import ctypes as C
import os

import numpy as np

_lib = None

SIGNATURES = {
    "coral_fbin_read_meta": (C.c_int, [C.c_char_p, C.POINTER(C.c_int64), C.POINTER(C.c_int32)]),
    "coral_fbin_read": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32]),
    "coral_fbin_write": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int64, C.c_int32]),
    "coral_gt_read_meta": (C.c_int, [C.c_char_p, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "coral_gt_read": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int32, C.c_int32]),
    "coral_gt_write": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int32, C.c_int32]),
    "coral_graph_dir_read": (C.c_int, [C.c_char_p, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]),
    "coral_graph_dir_write": (C.c_int, [C.c_char_p, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]),
    "coral_start_ids_read": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int32, C.POINTER(C.c_int32)]),
    "coral_start_ids_write": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int32]),
    "coral_hits_read": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int64]),
    "coral_hits_write": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int64]),
    "coral_roargraph_read": (C.c_int, [C.c_char_p, C.c_int64, C.c_int32, C.c_void_p, C.POINTER(C.c_int32)]),
    "coral_roargraph_write": (C.c_int, [C.c_char_p, C.c_int64, C.c_int32, C.c_void_p, C.c_int32]),
    "coral_lz4_compress_bound": (C.c_int, [C.c_int]),
    "coral_lz4_compress": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_int]),
    "coral_lz4_decompress": (C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_int]),
    "coral_normalize_l2": (None, [C.c_void_p, C.c_int64, C.c_int64]),
    "coral_recall_hits": (C.c_int64, [C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]),
}


def register(lib):
    global _lib
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def _L():
    if _lib is None:
        from . import capi
        capi.lib()
    return _lib


def _check(rc):
    if rc != 0:
        from . import capi
        raise capi.CoralError(rc, _L().coral_last_error().decode("utf-8", "replace"))


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _s(path):
    return os.fspath(path).encode()


def fbin_meta(path):
    n, d = C.c_int64(), C.c_int32()
    _check(_L().coral_fbin_read_meta(_s(path), C.byref(n), C.byref(d)))
    return n.value, d.value


def fbin_read(path, pad_to=4):
    """[n][dim'] float32 with dim' = dim rounded up to a multiple of pad_to, zero filled."""
    n, d = fbin_meta(path)
    stride = (d + pad_to - 1) // pad_to * pad_to
    out = np.empty((n, stride), dtype=np.float32)
    _check(_L().coral_fbin_read(_s(path), _p(out), n, d, stride))
    return out


def fbin_write(path, data):
    data = np.ascontiguousarray(data, dtype=np.float32)
    _check(_L().coral_fbin_write(_s(path), _p(data), data.shape[0], data.shape[1]))


def gt_read(path):
    nq, k = C.c_int32(), C.c_int32()
    _check(_L().coral_gt_read_meta(_s(path), C.byref(nq), C.byref(k)))
    ids = np.empty((nq.value, k.value), dtype=np.int32)
    _check(_L().coral_gt_read(_s(path), _p(ids), nq.value, k.value))
    return ids


def gt_write(path, ids):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    _check(_L().coral_gt_write(_s(path), _p(ids), ids.shape[0], ids.shape[1]))


def graph_dir_read(path, n, R=32, want_dists=False):
    nbrs = np.empty((n, R), dtype=np.int32)
    dists = np.empty((n, R), dtype=np.float32) if want_dists else None
    _check(_L().coral_graph_dir_read(_s(path), n, R, _p(nbrs), _p(dists)))
    return (nbrs, dists) if want_dists else nbrs


def graph_dir_write(path, nbrs, dists=None):
    nbrs = np.ascontiguousarray(nbrs, dtype=np.int32)
    d = None if dists is None else np.ascontiguousarray(dists, dtype=np.float32)
    _check(_L().coral_graph_dir_write(_s(path), nbrs.shape[0], nbrs.shape[1], _p(nbrs), _p(d)))


def start_ids_read(path, capacity=4096):
    ids = np.empty(capacity, dtype=np.int32)
    cnt = C.c_int32()
    _check(_L().coral_start_ids_read(_s(path), _p(ids), capacity, C.byref(cnt)))
    return ids[:cnt.value].copy()


def start_ids_write(path, ids):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    _check(_L().coral_start_ids_write(_s(path), _p(ids), ids.size))


def hits_read(path, n):
    """<path>/hits.bin -> uint32 [n] (include/ivf.cuh:647-656)"""
    hits = np.empty(n, dtype=np.uint32)
    _check(_L().coral_hits_read(_s(path), _p(hits), n))
    return hits


def hits_write(path, hits):
    hits = np.ascontiguousarray(hits, dtype=np.uint32)
    _check(_L().coral_hits_write(_s(path), _p(hits), hits.size))


def roargraph_read(path, n, R=32):
    nbrs = np.empty((n, R), dtype=np.int32)
    ep = C.c_int32()
    _check(_L().coral_roargraph_read(_s(path), n, R, _p(nbrs), C.byref(ep)))
    return nbrs, ep.value


def roargraph_write(path, nbrs, ep):
    nbrs = np.ascontiguousarray(nbrs, dtype=np.int32)
    _check(_L().coral_roargraph_write(_s(path), nbrs.shape[0], nbrs.shape[1], _p(nbrs), ep))


def lz4_compress(data):
    src = np.frombuffer(bytes(data), dtype=np.uint8)
    cap = _L().coral_lz4_compress_bound(src.size)
    dst = np.empty(cap, dtype=np.uint8)
    n = _L().coral_lz4_compress(_p(src) if src.size else None, src.size, _p(dst), cap)
    if n <= 0:
        raise ValueError("lz4 compression failed")
    return dst[:n].tobytes()


def lz4_decompress(data, raw_size):
    src = np.frombuffer(bytes(data), dtype=np.uint8)
    dst = np.empty(max(raw_size, 1), dtype=np.uint8)
    n = _L().coral_lz4_decompress(_p(src), src.size, _p(dst), raw_size)
    if n < 0:
        raise ValueError("malformed LZ4 block")
    return dst[:n].tobytes()


def normalize_l2(x):
    x = np.ascontiguousarray(x, dtype=np.float32).copy()
    _L().coral_normalize_l2(_p(x), x.shape[0], x.shape[1])
    return x


def recall_hits(res, gt, k):
    res = np.ascontiguousarray(res, dtype=np.int32)
    gt = np.ascontiguousarray(gt, dtype=np.int32)
    return int(_L().coral_recall_hits(res.shape[0], k, gt.shape[1], _p(res), _p(gt)))
