// index_gpu.cpp -- efanna2e::IndexGPU over the C ABI (see include/efanna2e/index_gpu.h).
#include "efanna2e/index_gpu.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>
#include <stdexcept>

#include "coral_formats.h"

namespace efanna2e {

namespace {

ProConfig g_config;

[[noreturn]] void raise(const char* what) {
    throw std::runtime_error(std::string(what) + ": " + coral_last_error());
}

// config.json is one flat object of numbers (config.json:1-40): a scanner for
// "key": number pairs is all that is needed; unknown keys are ignored like
// nlohmann's j.value(key, default) ignores them.
bool json_number(const std::string& text, const char* key, double* out) {
    const std::string needle = std::string("\"") + key + "\"";
    size_t p = text.find(needle);
    if (p == std::string::npos) return false;
    p = text.find(':', p + needle.size());
    if (p == std::string::npos) return false;
    ++p;
    while (p < text.size() && std::isspace((unsigned char)text[p])) ++p;
    char* end = nullptr;
    const double v = std::strtod(text.c_str() + p, &end);
    if (end == text.c_str() + p) return false;
    *out = v;
    return true;
}

}  // namespace

ProConfig& GetProConfig() { return g_config; }

// src/index.cpp:9-29 without the host-side Distance object and its message
Index::Index(const size_t dimension, const size_t n, Metric metric) : dimension_(dimension), nd_(n), metric_(metric) {}
Index::~Index() {}

IndexGPU::IndexGPU(const size_t dimension, const size_t n, Metric m, Index* initializer)
    : Index(dimension, n, m), initializer_(initializer), row_width_((dimension + 3) / 4 * 4) {
    if (m == COSINE) need_normalize = true;
}

// empty in the reference as well (src/index_gpu.cpp:652-654)
void IndexGPU::Build(size_t, const float*, const Parameters&) {}
void IndexGPU::Search(const float*, const float*, size_t, const Parameters&, unsigned*, float*) {}

IndexGPU::~IndexGPU() { RunFree(); }

void IndexGPU::RunFree() {
    if (index_) coral_index_destroy(index_);
    index_ = nullptr;
    std::free(h_base_);
    h_base_ = nullptr;
    data_bp_ = nullptr;
}

void IndexGPU::load_config(const std::string& config_file) {
    std::ifstream f(config_file == "default" ? "../config.json" : config_file);
    if (!f.is_open()) {
        std::cerr << "Cannot open config file, using defaults" << std::endl;
        return;
    }
    std::stringstream ss;
    ss << f.rdbuf();
    const std::string text = ss.str();
    double v;
    ProConfig& pc = g_config;
    if (json_number(text, "dim", &v)) pc.dim = (int)v;
    if (json_number(text, "k", &v)) pc.k = (int)v;
    if (json_number(text, "max_degree", &v)) pc.max_degree = (int)v;
    if (json_number(text, "beam_capacity", &v)) pc.beam_capacity = (int)v;
    if (json_number(text, "batch", &v)) pc.batch = (int)v;
    if (json_number(text, "test_beam_capacity", &v)) pc.test_beam_capacity = (int)v;
    if (json_number(text, "search_start_nodes_num", &v)) pc.search_start_nodes_num = (int)v;
    if (json_number(text, "search_in_cpu", &v)) pc.search_in_cpu = (int)v;
    if (json_number(text, "need_discard", &v)) pc.need_discard = (int)v;
    if (json_number(text, "enhance_nap_batch", &v)) pc.enhance_nap_batch = (int)v;
    if (json_number(text, "top_hit_num", &v)) pc.top_hit_num = (int)v;
    if (json_number(text, "enhance_search_batch", &v)) pc.enhance_search_batch = (int)v;
    if (json_number(text, "test_search", &v)) pc.test_search = (int)v;
    if (json_number(text, "test_search_frequency", &v)) pc.test_search_frequency = (int)v;
}

void IndexGPU::LoadSearchNeededData(const char* base_file, const char* sampled_query_file, DIST_METRIC m) {
    int64_t n = 0;
    int32_t dim = 0;
    if (coral_fbin_read_meta(base_file, &n, &dim)) raise("load_meta");
    if (sampled_query_file && std::strlen(sampled_query_file) != 0) {
        int64_t nq = 0;
        int32_t qdim = 0;
        if (coral_fbin_read_meta(sampled_query_file, &nq, &qdim)) raise("load_meta");
        if (qdim != dim) throw std::runtime_error("base and query dimension mismatch");
    }
    // rows are padded with zeros to a multiple of 4 floats (include/efanna2e/util.h:194-208);
    // unlike the reference the padded width is then used consistently
    const int32_t stride = (dim + 3) / 4 * 4;
    if ((size_t)stride != row_width_)
        throw std::runtime_error("base dimension does not match the index dimension");
    std::free(h_base_);
    h_base_ = nullptr;
    if (posix_memalign((void**)&h_base_, 32, (size_t)n * stride * sizeof(float)) != 0)
        throw std::runtime_error("out of host memory for the base vectors");
    if (coral_fbin_read(base_file, h_base_, n, dim, stride)) raise("load_data");
    if (m == DIST_METRIC::IP_) coral_normalize_l2(h_base_, n, stride);
    nd_ = (size_t)n;
    data_bp_ = h_base_;
    dist_metric_ = m;
}

void IndexGPU::RunPrepare(Parameters& parameters, Mode mode, size_t n_bp, float* bp_data) {
    // Mode::UPD loads the same state as Mode::SEARCH here: deletions are tombstones, rows are never rewritten
    if (mode != Mode::SEARCH && mode != Mode::UPD)
        throw std::runtime_error("only Mode::SEARCH and Mode::UPD are provided by this library");
    SetParameters(parameters);
    load_config(parameters.Get<std::string>("config_file", std::string("default")));
    graph_dir_ = parameters.Get<std::string>("graph_file");
    k_ = parameters.Get<int>("k");
    max_degree_ = parameters.Get<int>("max_degree");
    dist_metric_ = parameters.Get<std::string>("dist") == "l2" ? DIST_METRIC::L2_ : DIST_METRIC::IP_;
    if (n_bp > 0) {  // caller-owned vectors (src/index_gpu.cpp:246-251); copied, rows GetRowWidth() wide
        std::free(h_base_);
        h_base_ = nullptr;
        if (posix_memalign((void**)&h_base_, 32, n_bp * row_width_ * sizeof(float)) != 0)
            throw std::runtime_error("out of host memory for the base vectors");
        std::memcpy(h_base_, bp_data, n_bp * row_width_ * sizeof(float));
        nd_ = n_bp;
        data_bp_ = h_base_;
    }
    if (!h_base_) throw std::runtime_error("RunPrepare before LoadSearchNeededData");
    nbrs_.assign(nd_ * (size_t)max_degree_, -1);
    if (coral_graph_dir_read(graph_dir_.c_str(), (int64_t)nd_, max_degree_, nbrs_.data(), nullptr))
        raise("load graph");
    start_ids_.assign(4096, 0);
    int32_t m = 0;
    if (coral_start_ids_read(graph_dir_.c_str(), start_ids_.data(), (int32_t)start_ids_.size(), &m))
        raise("load start ids");
    start_ids_.resize((size_t)m);
    if (start_ids_.empty()) throw std::runtime_error("graph.search_start_ids is missing or empty in " + graph_dir_);
    coral_index_desc d;
    std::memset(&d, 0, sizeof d);
    d.base = h_base_, d.nbrs = nbrs_.data(), d.n = (int64_t)nd_, d.dim = (int32_t)row_width_;
    d.R = max_degree_, d.start_ids = start_ids_.data(), d.n_start = (int32_t)start_ids_.size();
    d.metric = dist_metric_ == DIST_METRIC::L2_ ? CORAL_L2 : CORAL_IP, d.device = 0;
    if (index_) coral_index_destroy(index_);
    index_ = nullptr;
    if (coral_index_create(&d, &index_)) raise("create index");
}

void IndexGPU::BuildGPU(size_t n_sq, float* sq_data, size_t n_bp, float* bp_data, Parameters& parameters) {
    SetParameters(parameters);
    load_config(parameters.Get<std::string>("config_file", std::string("default")));
    const int CE = parameters.Get<int>("CE");
    if (CE < 0 || CE > 2) throw std::runtime_error("BuildGPU: CE must be 0 (none), 1 (after the build) or 2 (only)");
    max_degree_ = parameters.Get<int>("max_degree");
    k_ = parameters.Get<int>("k");
    dist_metric_ = parameters.Get<std::string>("dist") == "l2" ? DIST_METRIC::L2_ : DIST_METRIC::IP_;
    graph_dir_ = parameters.Get<std::string>("graph_file");
    if (!bp_data || n_bp == 0) throw std::runtime_error("BuildGPU: empty input");
    if (bp_data != h_base_) {  // keep a copy, like RunPrepare does with caller-owned vectors
        std::free(h_base_);
        h_base_ = nullptr;
        if (posix_memalign((void**)&h_base_, 32, n_bp * row_width_ * sizeof(float)) != 0)
            throw std::runtime_error("out of host memory for the base vectors");
        std::memcpy(h_base_, bp_data, n_bp * row_width_ * sizeof(float));
        data_bp_ = h_base_;
    }
    nd_ = n_bp;
    coral_index_desc d;
    std::memset(&d, 0, sizeof d);
    d.base = h_base_, d.n = (int64_t)nd_, d.dim = (int32_t)row_width_;
    d.metric = dist_metric_ == DIST_METRIC::L2_ ? CORAL_L2 : CORAL_IP, d.device = 0;
    if (index_) coral_index_destroy(index_);
    index_ = nullptr;
    if (coral_index_create(&d, &index_)) raise("create index");
    coral_build_params p;
    coral_build_params_default(&p);
    p.R = max_degree_, p.k_b = k_, p.batch = PC.batch, p.need_discard = PC.need_discard, p.connect_enhance = CE;
    p.enhance_search_batch = PC.enhance_search_batch, p.enhance_nap_batch = PC.enhance_nap_batch;
    p.top_hit_num = PC.top_hit_num;
    p.n_start = PC.search_start_nodes_num;
    p.test_search_frequency = PC.test_search_frequency;
    // the test queries of the searches during the build: the first TEST_SEARCH_QUERY_SIZE = "batch" of query_test_file
    // (include/uni.h:63) with their true neighbours from gt_test_file
    std::vector<float> test_queries;
    std::vector<int32_t> test_gt;
    coral_build_monitor monitor{};
    struct Sink {
        IndexGPU* self;
        int Q, k;
    } sink{this, 0, 0};
    test_reports.clear();
    const std::string qt = parameters.Get<std::string>("query_test_file", std::string("None"));
    const std::string gt = parameters.Get<std::string>("gt_test_file", std::string("None"));
    if (PC.test_search && qt != "None" && !qt.empty() && gt != "None" && !gt.empty()) {
        int64_t nq = 0;
        int32_t qdim = 0, gn = 0, gk = 0;
        if (coral_fbin_read_meta(qt.c_str(), &nq, &qdim)) raise("query_test_file");
        if ((size_t)((qdim + 3) / 4 * 4) != row_width_) throw std::runtime_error("BuildGPU: test queries of another dimension");
        if (coral_gt_read_meta(gt.c_str(), &gn, &gk)) raise("gt_test_file");
        const int Q = (int)std::min<int64_t>({nq, (int64_t)gn, (int64_t)PC.batch});
        const int gtk = std::min(k_, (int)gk);
        if (Q > 0 && gtk > 0) {
            test_queries.resize((size_t)Q * row_width_);
            if (coral_fbin_read(qt.c_str(), test_queries.data(), Q, qdim, (int32_t)row_width_)) raise("query_test_file");
            if (dist_metric_ == DIST_METRIC::IP_) coral_normalize_l2(test_queries.data(), Q, (int32_t)row_width_);
            std::vector<int32_t> rows((size_t)gn * gk);
            if (coral_gt_read(gt.c_str(), rows.data(), gn, gk)) raise("gt_test_file");
            test_gt.resize((size_t)Q * gtk);
            for (int q = 0; q < Q; ++q) std::copy_n(rows.data() + (size_t)q * gk, gtk, test_gt.data() + (size_t)q * gtk);
            sink.Q = Q, sink.k = gtk;
            monitor.h_queries = test_queries.data(), monitor.h_gt = test_gt.data();
            monitor.Q = Q, monitor.k = gtk, monitor.L = std::max(PC.test_beam_capacity, gtk);
            monitor.user = &sink;
            monitor.report = [](void* user, int32_t phase, int64_t done, int64_t total, const coral_stats* st, int64_t h) {
                Sink* s = (Sink*)user;
                Test_Result res((int)h, (size_t)st->hops, (float)st->time_s);
                const float recall = res.calc_recall(s->Q * s->k), avg_hops = res.avg_hops(s->Q);
                static const char* const kWhen[] = {"batches", "isolated nodes attached", "most-hit nodes", "graph complete"};
                std::cout << "[" << kWhen[phase & 3] << " " << done << "/" << total << "] Testing recall-" << recall
                          << "%, avg_hops-" << avg_hops << ", cost_time-" << res.get_time() << "s" << std::endl;
                s->self->test_reports.push_back(TestReport{phase, (long long)done, (long long)total, res});
            };
            p.monitor = &monitor;
        }
    }
    std::vector<uint32_t> hits(nd_);
    if (CE == 2) {
        // enhancement only (src/index_gpu.cpp:332-333, 367-373): the rows, their distances and the hit counts of an
        // earlier BuildGPU with CE 0 come back from graph_file
        nbrs_.assign(nd_ * (size_t)max_degree_, -1);
        std::vector<float> saved(nd_ * (size_t)max_degree_);
        if (coral_graph_dir_read(graph_dir_.c_str(), (int64_t)nd_, max_degree_, nbrs_.data(), saved.data()))
            raise("BuildGPU: load graph");
        if (coral_hits_read(graph_dir_.c_str(), hits.data(), (int64_t)nd_)) raise("BuildGPU: load hits");
        if (coral_build_resume(index_, max_degree_, nbrs_.data(), saved.data(), hits.data())) raise("BuildGPU");
        p.connect_enhance = 1;
        if (coral_build_connect_enhance(index_, &p, &last_build)) raise("BuildGPU");
        if (coral_build_test_search(index_, &p, CORAL_MONITOR_DONE, (int64_t)nd_, (int64_t)nd_)) raise("BuildGPU");
    } else {
        const std::string train_gt = parameters.Get<std::string>("train_gt_file", std::string("None"));
        if (train_gt != "None" && !train_gt.empty()) {
            // clusters from a ground-truth file of the sampled queries (src/index_gpu.cpp:505-515: nq, k, ids)
            int32_t nq = 0, gk = 0;
            if (coral_gt_read_meta(train_gt.c_str(), &nq, &gk)) raise("train_gt_file");
            if (gk != k_) throw std::runtime_error("BuildGPU: train_gt_file holds k=" + std::to_string(gk) + ", expected " +
                                                   std::to_string(k_));
            std::vector<int32_t> clusters((size_t)nq * gk);
            if (coral_gt_read(train_gt.c_str(), clusters.data(), nq, gk)) raise("train_gt_file");
            if (coral_build_graph_from_clusters(index_, clusters.data(), nq, &p, &last_build)) raise("BuildGPU");
        } else if (coral_build_graph(index_, sq_data, (int64_t)n_sq, &p, &last_build)) {
            raise("BuildGPU");
        }
        // gpufuncs->save_hits() (src/index_gpu.cpp:362): the counts are complete once the clusters are through
        if (coral_build_top_hit_ids(index_, 0, nullptr, hits.data())) raise("BuildGPU");
    }
    // Graph::save_build (include/graph.cuh:481-484): start ids, then every row with its distances
    nbrs_.assign(nd_ * (size_t)max_degree_, -1);
    std::vector<float> dists(nd_ * (size_t)max_degree_);
    int32_t n_start = 0;  // can be below p.n_start when fewer nodes are reachable
    if (coral_index_info(index_, nullptr, nullptr, nullptr, &n_start, nullptr)) raise("BuildGPU");
    start_ids_.assign((size_t)n_start, 0);
    if (coral_index_get_graph(index_, nbrs_.data(), dists.data(), nullptr, start_ids_.data())) raise("download graph");
    if (coral_build_end(index_)) raise("BuildGPU");
    if (coral_graph_dir_write(graph_dir_.c_str(), (int64_t)nd_, max_degree_, nbrs_.data(), dists.data()))
        raise("save graph");
    if (coral_start_ids_write(graph_dir_.c_str(), start_ids_.data(), (int32_t)start_ids_.size())) raise("save start ids");
    if (coral_hits_write(graph_dir_.c_str(), hits.data(), (int64_t)nd_)) raise("save hits");
}

void IndexGPU::LoadRoarGraph(std::string filename) {
    if (!index_) throw std::runtime_error("LoadRoarGraph before RunPrepare");
    int32_t ep = 0;
    if (coral_roargraph_read(filename.c_str(), (int64_t)nd_, max_degree_, nbrs_.data(), &ep)) raise("LoadRoarGraph");
    start_ids_.assign(1, ep);
    if (coral_index_set_graph(index_, nbrs_.data(), start_ids_.data(), 1)) raise("LoadRoarGraph");
}

void IndexGPU::Delete(const std::vector<int> del_ids) {
    if (!index_) throw std::runtime_error("Delete before RunPrepare");
    if (coral_index_mark_deleted(index_, del_ids.data(), (int32_t)del_ids.size())) raise("Delete");
    have_delete_ = true;
}

void IndexGPU::SetDeleted(const uint32_t* mask_words) {
    if (!index_) throw std::runtime_error("SetDeleted before RunPrepare");
    if (coral_index_set_deleted(index_, mask_words)) raise("SetDeleted");
    have_delete_ = mask_words != nullptr;
}

Test_Result IndexGPU::run(const float* queries, int num, int L, int* ids_res, float* dists_res) {
    if (!index_) throw std::runtime_error("Search before RunPrepare");
    coral_stats st;
    if (coral_search(index_, queries, num, k_, L, GetPolicy(), have_delete_ ? 1 : 0, ids_res, dists_res, &st))
        raise("Search");
    Test_Result tr(-1, (size_t)st.hops, (float)st.time_s);
    tr.expansions = (size_t)st.expansions, tr.dist_evals = (size_t)st.dist_evals;
    tr.rounds = (size_t)st.rounds, tr.spills = (size_t)st.spills;
    return tr;
}

Test_Result IndexGPU::Search(const float* queries, int num, int beam_capacity, int* ids_res, int M) {
    (void)M;  // the reference fills a default and then ignores it too (src/index_gpu.cpp:119,127)
    return run(queries, num, beam_capacity, ids_res, nullptr);
}

Test_Result IndexGPU::SearchWithDists(const float* queries, int num, int beam_capacity, int* ids_res,
                                      float* dists_res) {
    return run(queries, num, beam_capacity, ids_res, dists_res);
}

Test_Result IndexGPU::Search_and_Verify(const float* queries, const int* gts, int num, int beam_capacity) {
    if (!index_) throw std::runtime_error("Search_and_Verify before RunPrepare");
    const int L = beam_capacity > 0 ? beam_capacity : PC.test_beam_capacity;
    float* d_q = nullptr;
    int32_t *d_ids = nullptr, *d_gt = nullptr;
    const size_t qb = (size_t)num * row_width_ * sizeof(float), ib = (size_t)num * k_ * sizeof(int32_t);
    auto release = [&]() {
        (void)hipFree(d_q);
        (void)hipFree(d_ids);
        (void)hipFree(d_gt);
    };
    if (hipMalloc(&d_q, qb) != hipSuccess || hipMalloc(&d_ids, ib) != hipSuccess ||
        hipMalloc(&d_gt, ib) != hipSuccess || hipMemcpy(d_q, queries, qb, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(d_gt, gts, ib, hipMemcpyHostToDevice) != hipSuccess) {
        release();
        throw std::runtime_error("Search_and_Verify: device allocation or upload failed");
    }
    // the reference prepares once per process (a function-local static, src/index_gpu.cpp:101-108) and breaks if a
    // later call is larger; here every call states its batch, beam and traversal (other calls on this index may
    // have prepared it differently in between, and preparing what is already there costs next to nothing)
    coral_tuning tuning;
    std::memset(&tuning, 0, sizeof tuning);
    tuning.policy = GetPolicy();
    if (coral_search_prepare(index_, num, L, &tuning)) {
        release();
        raise("search_prepare");
    }
    coral_stats st;
    int64_t hits = 0;
    if (coral_search_gpu(index_, d_q, d_ids, nullptr, num, k_, GetPolicy(), have_delete_ ? 1 : 0, nullptr, &st) ||
        coral_search_verify(index_, d_ids, d_gt, num, k_, &hits)) {
        release();
        raise("Search_and_Verify");
    }
    release();
    Test_Result tr((int)hits, (size_t)st.hops, (float)st.time_s);
    tr.expansions = (size_t)st.expansions, tr.dist_evals = (size_t)st.dist_evals;
    tr.rounds = (size_t)st.rounds, tr.spills = (size_t)st.spills;
    return tr;
}

}  // namespace efanna2e
