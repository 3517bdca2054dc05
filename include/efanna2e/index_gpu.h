// efanna2e::IndexGPU -- the search-side surface of the reference's index class
// (include/index_gpu.h:42-76, src/index_gpu.cpp), implemented on the MI355X path
// of libcoral_search.so.  A caller written against the reference's
// test_search_pipeline.cpp:241-292 compiles against this header unchanged:
//
//     efanna2e::IndexGPU index(dim, n, efanna2e::L2, nullptr);
//     index.LoadSearchNeededData(base_file, "", DIST_METRIC::L2_);
//     index.RunPrepare(parameters, Mode::SEARCH);
//     Test_Result tr = index.Search(queries, Q, L, ids);
//
// Differences, all on purpose:
//   * the whole index is HBM resident for every N; the reference switches to a
//     CPU or disk tier above 10.01M / 100M nodes (src/index_gpu.cpp:256-257).
//     SetPolicy() chooses the traversal instead: ROUNDS (the reference's GPU
//     kernel) by default, BEST_FIRST (its CPU path) on request;
//   * BuildGPU (all three --CE modes) and Delete in its tombstone-only mode are provided;
//     Insert and the repair of rows after a deletion are not part of this library;
//   * failures throw std::runtime_error with the library's message where the
//     reference prints and exits (include/utils.cuh:50-58).
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "../coral_search.h"
#include "index.h"
#include "parameters.h"

enum DIST_METRIC { L2_, IP_, COS_ };  // include/uni.h:93

namespace efanna2e {

enum Mode { CONS, SEARCH, UPD, CE };                                          // include/uni.h:147
enum GraphType { GPU, CPU, DISK };                                            // include/uni.h:149

// The keys of config.json that search and construction read (src/index_gpu.cpp:40-87); defaults
// are the reference's (include/uni.h:97-132).
struct ProConfig {
    int dim = 200;
    int k = 100;
    int max_degree = 32;
    int beam_capacity = 1024;
    int batch = 1024;
    int test_beam_capacity = 512;
    int search_start_nodes_num = 16;
    int search_in_cpu = 0;
    // read by the builder
    int need_discard = 1;
    int enhance_nap_batch = 4096;
    int enhance_search_batch = 524288;
    int top_hit_num = 0;  // include/uni.h:124; the shipped config.json sets 5000000
    int test_search = 1;             // include/uni.h:109: search the test queries while the graph grows
    int test_search_frequency = 100; // include/uni.h:122: ... every so many batches
};
CORAL_API ProConfig& GetProConfig();
#define PC (::efanna2e::GetProConfig())

// include/uni.h:411-437
class CORAL_API Test_Result {
   public:
    Test_Result() : recall(0.0f), time(0.0f), hits(0), hops(0) {}
    Test_Result(const int hits, const size_t hops, const float time)
        : recall(0.0f), time(time), hits(hits), hops(hops) {}
    Test_Result(const int hits, const size_t hops) : recall(0.0f), time(0.0f), hits(hits), hops(hops) {}
    float get_recall() const { return recall; }
    size_t get_hops() const { return hops; }
    float get_time() const { return time; }
    float calc_recall(int total_num) { return recall = 100.0 * hits / total_num; }
    float avg_hops(int search_num) { return 1.0 * hops / search_num; }
    void accumulate(const Test_Result& res) {
        hops += res.hops;
        time += res.time;
        hits += res.hits;
    }

    float recall, time;
    int hits;
    size_t hops;
    // beyond the reference: counters behind the roofline figures of the last call
    size_t expansions = 0, dist_evals = 0, rounds = 0, spills = 0;
};

class CORAL_API IndexGPU : public Index {
   public:
    // include/index_gpu.h:46; `initializer` is stored and never used, as in the reference
    // (src/index_gpu.cpp:26-27)
    explicit IndexGPU(const size_t dimension, const size_t n, Metric m, Index* initializer);
    virtual ~IndexGPU();
    IndexGPU(const IndexGPU&) = delete;
    IndexGPU& operator=(const IndexGPU&) = delete;
    // the base class's interface; all four are empty in the reference too (include/index_gpu.h:48-49,
    // src/index_gpu.cpp:652-654)
    virtual void Save(const char*) override {}
    virtual void Load(const char*) override {}
    virtual void Build(size_t n, const float* data, const Parameters& parameters) override;
    virtual void Search(const float* query, const float* x, size_t k, const Parameters& parameters,
                        unsigned* indices, float* res_dists) override;
    Index* initializer_;

    // src/index_gpu.cpp:625-650: reads base_file (.fbin), L2-normalises it for IP_
    void LoadSearchNeededData(const char* base_file, const char* sampled_query_file,
                              DIST_METRIC m = DIST_METRIC::L2_);
    // src/index_gpu.cpp:226-262: reads config_file, graph_file (index directory), k,
    // max_degree, dist from `parameters`; uploads vectors and graph
    void RunPrepare(Parameters& parameters, Mode mode, size_t n_bp = 0, float* bp_data = nullptr);
    void RunFree();
    void SetParameters(Parameters& parameters) { parameters_ = parameters; }
    void load_config(const std::string& config_file);

    // src/index_gpu.cpp:117-136; ids_res holds num*k ints, best first
    Test_Result Search(const float* queries, int num, int beam_capacity, int* ids_res, int M = 0);
    // src/index_gpu.cpp:89-115; gts holds num*k ints; hits are counted on the device
    Test_Result Search_and_Verify(const float* queries, const int* gts, int num, int beam_capacity = 0);
    // src/graph.cu:709-743
    void LoadRoarGraph(std::string filename);
    // src/index_gpu.cpp:308-383: builds the graph over the n_bp base vectors from the n_sq auxiliary ("sampled")
    // queries and writes the index directory parameters["graph_file"] (graph.part*.idx/.data, graph.search_start_ids,
    // graph.batch_id).  Reads config_file, CE (0, 1, or 2 = the enhancement alone on the rows, distances and
    // hits.bin that a CE = 0 build left in graph_file, src/index_gpu.cpp:332-333, 367-373), max_degree, k (the cluster
    // size), dist, graph_file, train_gt_file (optional: the clusters, as a ground-truth file of the sampled queries with k
    // ids per row; sq_data is then unused).  Both arrays hold rows of GetRowWidth() floats.  The built index stays loaded, so
    // Search works right after.  The timings and counts of the run are in last_build.
    // With query_test_file and gt_test_file among the parameters (tests/test_build_pipeline.cpp:215-216) and
    // config.json's "test_search" not 0, the first "batch" test queries are searched with beam test_beam_capacity while
    // the graph grows (GPUFuncs::test_search, include/gpufuncs.cuh:688-702, at the points where the reference calls it)
    // and a line per search goes to stdout in the wording of src/enhance_disk.cu:468-469; test_reports keeps them.
    struct TestReport {
        int phase;  // CORAL_MONITOR_*
        long long done, total;
        Test_Result result;
    };
    std::vector<TestReport> test_reports;
    void BuildGPU(size_t n_sq, float* sq_data, size_t n_bp, float* bp_data, Parameters& parameters);
    coral_build_stats last_build{};
    // src/index_gpu.cpp:138-206 with upd_type 0: the ids are tombstoned on the device (del_node_mark,
    // src/update.cu:660-672) and later searches leave them out of their results; the graph is not repaired
    void Delete(const std::vector<int> del_ids);

    // --- beyond the reference ---
    // CORAL_POLICY_BEST_FIRST is the traversal of GPUFuncs::search_in_cpu; it starts from every start id of the index,
    // where the CPU path takes the first search_start_nodes_num of them (src/search_in_cpu.cpp:26, 74-79): the same
    // set whenever graph.search_start_ids holds that many ids, as the builder writes it
    // Unless named here, the traversal is the one the reference would run for an index of this size: the CUDA kernel's
    // rounds up to GPU_N = 10 010 000 nodes, the CPU path's best-first above (src/index_gpu.cpp:257, include/uni.h:70).
    void SetPolicy(int coral_policy) { policy_ = coral_policy; }
    int GetPolicy() const {
        return policy_ >= 0 ? policy_ : (nd_ > 10010000 ? CORAL_POLICY_BEST_FIRST : CORAL_POLICY_ROUNDS);
    }
    // tombstones (src/update.cu:406-412): ceil(n/32) words, or nullptr to clear
    void SetDeleted(const uint32_t* mask_words);
    // as Search, also returning distances (num*k floats)
    Test_Result SearchWithDists(const float* queries, int num, int beam_capacity, int* ids_res,
                                float* dists_res);

    Metric GetMetric() const { return metric_; }
    // floats per vector row as the library holds them: the dimension padded to a multiple of 4 with zeros, which
    // is what the reference's loaders hand to the constructor in the first place (include/efanna2e/util.h:194-208)
    size_t GetRowWidth() const { return row_width_; }
    const std::vector<int>& GetStartIds() const { return start_ids_; }
    bool need_normalize = false;

   private:
    Test_Result run(const float* queries, int num, int L, int* ids_res, float* dists_res);
    size_t row_width_;
    DIST_METRIC dist_metric_ = DIST_METRIC::L2_;
    Parameters parameters_;
    int k_ = 0, max_degree_ = 32;
    int policy_ = -1;  // -1: by size, see GetPolicy
    bool have_delete_ = false;
    float* h_base_ = nullptr;
    std::vector<int> start_ids_;
    std::vector<int32_t> nbrs_;
    std::string graph_dir_;
    coral_index* index_ = nullptr;
};

}  // namespace efanna2e
