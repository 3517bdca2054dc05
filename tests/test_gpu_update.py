"""The update evaluation in its delete-only mode (tests/update_compute_gt.cpp, tests/test_update.cpp with --upd_mode 1):
ground truth after every deletion batch against the oracle's brute force with the same ids tombstoned, and the
driver's recall table against the same loop through the C ABI."""
import os
import subprocess

import numpy as np
import pytest

from coral_amd import capi, formats, synth
from util import make_queries

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "coral_amd", "lib")


def mask_of(n, upto):
    m = np.zeros((n + 31) // 32, np.uint32)
    ids = np.arange(upto, dtype=np.int64)
    np.bitwise_or.at(m, ids >> 5, np.uint32(1) << (ids & 31).astype(np.uint32))
    return m


def test_delete_only_evaluation_loop(orc, tmp_path):
    total, dim, A, Q, k, R, L = 8000, 32, 500, 60, 10, 16, 64
    half, rounds = total // 2, 100
    batch = (half + rounds - 1) // rounds
    base = synth.gaussian_matrix(41, total, dim)
    aux = make_queries(A, dim, 42)
    q = make_queries(Q, dim, 43)
    work = tmp_path / "run"
    os.makedirs(work / "cwd")
    formats.fbin_write(work / "base.fbin", base)
    formats.fbin_write(work / "aux.fbin", aux)
    formats.fbin_write(work / "query.fbin", q)
    (work / "config.json").write_text('{"batch": 128, "search_start_nodes_num": 8, "upd_type": 0, "upd_build": 1}')
    # ---- ground truth of every round
    r = subprocess.run([os.path.join(LIB, "update_compute_gt"), "--dist", "l2", "--dataset", "syn", "--base_data_path",
                        str(work / "base.fbin"), "--query_path", str(work / "query.fbin"), "--update_gt_file",
                        str(work / "upd_gt"), "--k", str(k), "--upd_mode", "1"], cwd=work / "cwd", capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    raw = np.fromfile(work / "upd_gt.del", dtype=np.int32)
    assert raw[0] == rounds and raw.size == 1 + (rounds // 2 + 1) * Q * k
    gts = raw[1:].reshape(rounds // 2 + 1, Q, k)
    for b in (0, 1, 2, 25, 50):
        gone = min(half, b * batch)
        want, _ = orc.bruteforce(base[:half], q, k, deleted=mask_of(half, gone) if gone else None, order=0)
        assert np.array_equal(gts[b], want), b
        assert (gts[b] >= gone).all()
    # ---- the evaluation driver
    r = subprocess.run([os.path.join(LIB, "test_update"), "--dataset", "syn", "--base_data_path", str(work / "base.fbin"),
                        "--update_gt_file", str(work / "upd_gt"), "--sampled_query_data_path", str(work / "aux.fbin"),
                        "--dist", "l2", "--max_degree", str(R), "--k", str(k), "--L", str(L), "--query_path",
                        str(work / "query.fbin"), "--upd_mode", "1", "--config_file", str(work / "config.json")],
                       cwd=work / "cwd", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr + r.stdout
    assert (work / "indexes" / "syn_l2_16_upd" / "graph.part0.idx").exists()
    rows = (work / "evaluation" / "upd" / "1_0.csv").read_text().splitlines()
    assert rows[0] == "round, recall, avg_hops, time, qps" and len(rows) == 2 + rounds // 2
    # ---- the same loop through the C ABI
    idx = capi.Index(base[:half], None, None)
    idx.build_graph(aux, capi.build_params(R=R, k_b=k, batch=128, n_start=8))
    idx.build_end()
    for b in range(rounds // 2 + 1):
        if b:
            lo = min(half, (b - 1) * batch)
            idx.mark_deleted(np.arange(lo, min(half, lo + batch), dtype=np.int32))
        ids, _, st = idx.search(q, k, L, have_delete=b > 0, want_dists=False)
        recall = 100.0 * orc.recall_hits(ids, gts[b], k) / (Q * k)
        f = [float(x) for x in rows[1 + b].split(",")]
        assert int(f[0]) == b
        assert abs(f[1] - recall) < 1e-3, (b, f[1], recall)
        assert abs(f[2] - st.hops / Q) < 1e-2
        if b:
            assert not np.isin(ids, np.arange(min(half, b * batch))).any()
    idx.close()
    # modes that insert are refused
    r = subprocess.run([os.path.join(LIB, "test_update"), "--dataset", "syn", "--base_data_path", str(work / "base.fbin"),
                        "--update_gt_file", str(work / "upd_gt"), "--sampled_query_data_path", str(work / "aux.fbin"),
                        "--query_path", str(work / "query.fbin"), "--upd_mode", "0"], cwd=work / "cwd",
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 255 and "upd_mode 1" in r.stderr
