"""Host-side checks that need no GPU: the shared library loads, exports every
symbol the public headers declare, and rejects bad arguments before touching a
device."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from coral_amd import capi, formats

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = []
    for h in ("coral_search.h", "coral_formats.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        names += re.findall(r"CORAL_API\s+[\w\s\*]+?\b(coral_\w+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib = capi.lib()
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), n
    bound = set(capi.SIGNATURES) | set(formats.SIGNATURES)
    assert set(names) == bound


LAYOUT_PROBE = r"""
#include <stddef.h>
#include <stdio.h>
#include "coral_search.h"
#define S(t) printf(#t " size %zu\n", sizeof(t))
#define F(t, f) printf(#t " " #f " %zu\n", offsetof(t, f))
int main(void) {
    S(coral_stats); F(coral_stats, hops); F(coral_stats, screened_rows); F(coral_stats, visited_dedupes);
    S(coral_tuning); F(coral_tuning, visited_choices);
    S(coral_plan_info); F(coral_plan_info, query_slots);
    S(coral_build_params); F(coral_build_params, top_hit_num); F(coral_build_params, test_search_frequency);
    F(coral_build_params, monitor);
    S(coral_build_monitor); F(coral_build_monitor, L); F(coral_build_monitor, report); F(coral_build_monitor, user);
    S(coral_build_stats); F(coral_build_stats, top_reverse_edges);
    return 0;
}
"""


def test_ctypes_structures_have_the_layout_of_the_header(tmp_path):
    """What a C compiler makes of include/coral_search.h (the header is plain C) against the ctypes mirror that the
    tests and bench.py call through: sizes and the offsets of the fields added last."""
    (tmp_path / "probe.c").write_text(LAYOUT_PROBE)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(tmp_path / "probe.c"),
                    "-o", str(tmp_path / "probe")], check=True)
    out = subprocess.run([str(tmp_path / "probe")], capture_output=True, text=True, check=True).stdout
    mirror = {"coral_stats": capi.Stats, "coral_tuning": capi.Tuning, "coral_plan_info": capi.PlanInfo,
              "coral_build_params": capi.BuildParams, "coral_build_monitor": capi.BuildMonitor,
              "coral_build_stats": capi.BuildStats}
    lines = out.splitlines()
    assert len(lines) >= 17
    for line in lines:
        if not line:
            continue
        name, what, value = line.split()
        cls = mirror[name]
        assert (ctypes.sizeof(cls) if what == "size" else getattr(cls, what).offset) == int(value), line


def test_cxx_class_symbols_are_exported():
    out = subprocess.run(["nm", "-DC", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    for sym in ("efanna2e::IndexGPU::Search(float const*, int, int, int*, int)",
                "efanna2e::IndexGPU::Search_and_Verify(float const*, int const*, int, int)",
                "efanna2e::IndexGPU::RunPrepare(efanna2e::Parameters&, efanna2e::Mode, unsigned long, float*)",
                "efanna2e::IndexGPU::LoadSearchNeededData(char const*, char const*, DIST_METRIC)",
                "efanna2e::IndexGPU::LoadRoarGraph(", "efanna2e::IndexGPU::load_config(",
                "efanna2e::IndexGPU::RunFree()", "efanna2e::GetProConfig()",
                # the reference's class hierarchy (include/efanna2e/index.h:20-40, include/index_gpu.h:42-46)
                "efanna2e::IndexGPU::IndexGPU(unsigned long, unsigned long, efanna2e::Metric, efanna2e::Index*)",
                "efanna2e::Index::Index(unsigned long, unsigned long, efanna2e::Metric)",
                "vtable for efanna2e::Index", "vtable for efanna2e::IndexGPU", "typeinfo for efanna2e::Index",
                "efanna2e::IndexGPU::BuildGPU(unsigned long, float*, unsigned long, float*, efanna2e::Parameters&)",
                "efanna2e::IndexGPU::Delete(std::vector<int, std::allocator<int> >)"):
        assert sym in out, sym


CALLER = r"""
// A caller in the shape of the reference's search driver (tests/test_search_pipeline.cpp:241-292) and of code that
// holds the index through its base class (include/efanna2e/index.h:20-64).
#include <cstring>
#include <iostream>
#include <string>
#include <vector>
#include "efanna2e/index.h"
#include "efanna2e/index_gpu.h"
#include "efanna2e/parameters.h"

using namespace efanna2e;  // as the reference's driver does (tests/test_search_pipeline.cpp:23)

static float run(efanna2e::Index* base_ptr, const std::vector<float>& queries, int q_pts, int k,
                 std::vector<int> L_vec, const std::string& index_type) {
    efanna2e::IndexGPU& index = *static_cast<efanna2e::IndexGPU*>(base_ptr);
    int* res = new int[(size_t)q_pts * k];
    std::memset(res, 0, sizeof(int) * (size_t)q_pts * k);
    float last = 0.f;
    for (size_t i = 0; i < L_vec.size(); ++i) {
        int L = L_vec[i];
        auto tr = index_type == "" ? index.Search(queries.data(), q_pts, L, res)
                                   : index.Search(queries.data(), q_pts, L, res, 1);
        const float qps = (float)q_pts / tr.get_time(), time = tr.get_time();
        const float avg_hops = tr.avg_hops(q_pts);
        std::cout << L << "		" << qps << "		" << time << "		" << avg_hops << std::endl;
        last = qps;
    }
    delete[] res;
    return last;
}

int main(int argc, char** argv) {
    efanna2e::Metric dist_metric = efanna2e::INNER_PRODUCT;
    DIST_METRIC metric = DIST_METRIC::IP_;
    size_t q_dim = 200, base_num = 0, sq_num = 0;
    efanna2e::Parameters parameters;
    parameters.Set<std::string>("config_file", "default");
    parameters.Set<std::string>("graph_file", "../indexes/x_ip_32_1.0_1/");
    parameters.Set<int>("k", 100);
    parameters.Set<int>("max_degree", 32);
    parameters.Set<std::string>("dist", "ip");
    efanna2e::IndexGPU index(q_dim, base_num + sq_num, dist_metric, nullptr);
    efanna2e::Index* as_base = &index;                       // IndexGPU is an Index
    efanna2e::IndexGPU second(q_dim, 0, efanna2e::L2, as_base);  // ... and takes one as its initializer
    if (argc > 100) {  // never run: this file is compiled and linked, not executed
        index.LoadSearchNeededData(argv[1], argv[2], metric);
        index.RunPrepare(parameters, Mode::SEARCH);
        index.LoadRoarGraph(std::string("../data/") + argv[3] + "/indexes/roar.index");
        std::vector<float> q(q_dim);
        run(as_base, q, 1, 100, {256, 512}, "");
        Test_Result tr = index.Search_and_Verify(q.data(), nullptr, 1, 256);
        tr.calc_recall(100);
        as_base->Save("x");
        as_base->Load("x");
        as_base->Build(0, nullptr, parameters);
        as_base->Search(nullptr, nullptr, 0, parameters, nullptr, nullptr);
        index.RunFree();
    }
    return (int)(as_base->GetDimension() - q_dim) + (second.initializer_ == as_base ? 0 : 1) +
           (as_base->HasBuilt() ? 1 : 0) + (int)as_base->GetSizeOfDataset();
}
"""


def test_a_caller_written_against_the_reference_class_compiles_and_links(tmp_path):
    """The fragment of the reference's driver that constructs, loads, prepares and searches the index, and a use of
    the index through its abstract base, compile against include/efanna2e/*.h and link against the library (the
    program constructs two indexes, touches no device and exits 0)."""
    src = tmp_path / "caller.cpp"
    src.write_text(CALLER)
    exe = tmp_path / "caller"
    libdir = os.path.dirname(capi.LIB_PATH)
    r = subprocess.run(["g++", "-std=c++17", "-Wall", "-I" + os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                        "-L" + libdir, "-lcoral_search", "-Wl,-rpath," + libdir], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_index_create_validates_before_any_device_call():
    base = np.zeros((10, 8), np.float32)
    good = np.full((10, 4), -1, np.int32)
    good[:, 0] = (np.arange(10) + 1) % 10

    def create(base, nbrs, starts, metric=0):
        try:
            capi.Index(base, nbrs, starts, metric).close()
        except capi.CoralError as e:
            return e.code, str(e)
        return 0, ""

    bad = good.copy()
    bad[3, 0] = 10
    assert create(base, bad, [0])[0] == capi.ERR_GRAPH
    bad = good.copy()
    bad[3, 0], bad[3, 1] = -1, 2
    code, msg = create(base, bad, [0])
    assert code == capi.ERR_GRAPH and "end-of-row" in msg
    assert create(base, good, [10])[0] == capi.ERR_GRAPH
    code, msg = create(base, good, [2, 2])
    assert code == capi.ERR_GRAPH and "duplicate" in msg
    assert create(base, good, [])[0] == capi.ERR_ARG
    assert create(np.zeros((10, 6), np.float32), good, [0])[0] == capi.ERR_ARG  # dim % 4
    assert create(base, np.full((10, 33), -1, np.int32), [0])[0] == capi.ERR_ARG  # R > 32
    assert create(base, good, [0], metric=7)[0] == capi.ERR_ARG


def test_null_arguments_are_errors_not_crashes():
    lib = capi.lib()
    assert lib.coral_index_create(None, None) == capi.ERR_ARG
    assert lib.coral_search_prepare(None, 1, 1, None) == capi.ERR_ARG
    assert lib.coral_search_gpu(None, None, None, None, 1, 1, 0, 0, None, None) == capi.ERR_ARG
    assert lib.coral_search(None, None, 1, 1, 1, 0, 0, None, None, None) == capi.ERR_ARG
    assert b"null" in lib.coral_last_error()
    lib.coral_index_destroy(None)


CLI = os.path.join(ROOT, "coral_amd", "lib", "test_search_pipeline")


def run_cli(*args):
    return subprocess.run([CLI] + list(args), capture_output=True, text=True)


def test_cli_flag_handling():
    r = run_cli("--help")
    assert r.returncode == 0
    for flag in ("--data_type", "--dist", "--base_data_path", "--dataset", "--query_path", "--gt_path", "--L",
                 "--k", "--max_degree", "--query_thres", "--CE", "--config_file", "--index_type", "--log_file",
                 "--res_file", "--recall_thres", "--max_recall", "--max_hop"):
        assert flag in r.stdout
    r = run_cli("--dist", "l2")
    assert r.returncode == 255 and "required but missing" in r.stderr  # the reference returns -1
    r = run_cli("--bogus", "1")
    assert r.returncode == 255 and "unrecognised option" in r.stderr
    base = ["--data_type", "float", "--base_data_path", "/nonexistent.fbin", "--dataset", "t", "--query_path",
            "/nonexistent_q.fbin", "--gt_path", "/nonexistent_gt", "--k", "10", "--L", "32", "64", "-T", "16"]
    r = run_cli(*base, "--dist", "cosine")
    assert r.returncode == 255 and "Unknown distance type" in r.stdout
    r = run_cli(*base, "--dist", "l2")
    assert r.returncode == 1 and "open file error" in r.stderr
    r = run_cli(*base, "--dist=l2", "--k", "ten")
    assert r.returncode == 255


def test_build_cli_flag_handling():
    cli = os.path.join(ROOT, "coral_amd", "lib", "test_build_pipeline")

    def run(*args):
        return subprocess.run([cli] + list(args), capture_output=True, text=True)

    r = run("--help")
    assert r.returncode == 0
    for flag in ("--data_type", "--dist", "--N", "--dataset", "--base_data_path", "--train_gt_file",
                 "--sampled_query_data_path", "--query_test_file", "--gt_test_file", "--M_sq", "--M_pjbp", "--L_pjpq",
                 "--num_threads", "--CE", "--k", "--iso_thres", "--recall_thres", "--query_thres", "--log_file",
                 "--config_file"):  # tests/test_build_pipeline.cpp:45-121
        assert flag in r.stdout
    r = run("--dist", "l2")
    assert r.returncode == 255 and "required but missing" in r.stderr
    base = ["--data_type", "float", "--dataset", "t", "--base_data_path", "/nonexistent.fbin",
            "--sampled_query_data_path", "/nonexistent_sq.fbin", "--k", "100", "-T", "32", "--index_dir", "/tmp/x"]
    r = run(*base, "--dist", "cosine")
    assert r.returncode == 255 and "Unknown distance type" in r.stdout
    r = run(*base, "--dist", "l2")
    assert r.returncode == 1 and "open file error" in r.stderr
    r = run(*base, "--dist", "l2", "--gt_test_file", "gt.bin")
    assert r.returncode == 255 and "gt_test_file" in r.stderr
    r = run(*base, "--dist", "l2", "--CE", "x")
    assert r.returncode == 255


def test_build_entry_points_reject_bad_arguments_before_any_device_call():
    lib = capi.lib()
    assert lib.coral_build_begin(None, 32) == capi.ERR_ARG
    assert lib.coral_build_nap_batch(None, None, 1, 10, 1) == capi.ERR_ARG
    assert lib.coral_build_enhance_batch(None, None, None, None, 1, 10, None, None) == capi.ERR_ARG
    assert lib.coral_build_connect_enhance(None, None, None) == capi.ERR_ARG
    assert lib.coral_build_graph(None, None, 0, None, None) == capi.ERR_ARG
    assert lib.coral_build_graph_from_clusters(None, None, 0, None, None) == capi.ERR_ARG
    assert lib.coral_index_get_graph(None, None, None, None, None) == capi.ERR_ARG
    assert lib.coral_start_ids_fps(None, 0, 1, None) == capi.ERR_ARG
    assert lib.coral_index_mark_deleted(None, None, 0) == capi.ERR_ARG
    p = capi.build_params()
    assert (p.R, p.k_b, p.batch, p.need_discard, p.connect_enhance) == (32, 100, 1024, 1, 1)  # config.json:3-6,14
    assert (p.enhance_search_batch, p.enhance_nap_batch, p.enhance_L, p.n_start) == (524288, 4096, 256, 16)
    with pytest.raises(TypeError):
        capi.build_params(no_such_field=1)


def test_update_drivers_flag_handling():
    for tool, required in (("update_compute_gt", ("--dist", "--dataset", "--base_data_path", "--query_path",
                                                  "--update_gt_file", "--k", "--upd_mode", "--data_type")),
                           ("test_update", ("--dataset", "--base_data_path", "--update_gt_file",
                                            "--sampled_query_data_path", "--dist", "--data_type", "--recall_thres",
                                            "--query_thres", "--max_degree", "--k", "--L", "--query_path", "--upd_mode",
                                            "--config_file"))):  # tests/update_compute_gt.cpp:40-55, tests/test_update.cpp:42-74
        exe = os.path.join(ROOT, "coral_amd", "lib", tool)
        r = subprocess.run([exe, "--help"], capture_output=True, text=True)
        assert r.returncode == 0
        for flag in required:
            assert flag in r.stdout, (tool, flag)
        r = subprocess.run([exe, "--dataset", "t"], capture_output=True, text=True)
        assert r.returncode == 255 and "required but missing" in r.stderr
    exe = os.path.join(ROOT, "coral_amd", "lib", "update_compute_gt")
    args = ["--dist", "l2", "--dataset", "t", "--base_data_path", "/nonexistent.fbin", "--query_path", "/q.fbin",
            "--update_gt_file", "/tmp/x", "--k", "10"]
    r = subprocess.run([exe] + args + ["--upd_mode", "2"], capture_output=True, text=True)
    assert r.returncode == 255 and "upd_mode 1" in r.stderr
    r = subprocess.run([exe] + args + ["--upd_mode", "1"], capture_output=True, text=True)
    assert r.returncode == 1 and "open file error" in r.stderr
