// test_search_pipeline -- the reference's search driver
// (tests/test_search_pipeline.cpp:68-322) over efanna2e::IndexGPU of this
// library: same flags, same index-directory and CSV naming, same stdout table.
//
// Flags of the reference (tests/test_search_pipeline.cpp:88-128), all accepted:
//   --data_type --dist {l2,ip} --base_data_path --dataset --query_path --gt_path
//   --k --max_degree --L <ints...> --config_file --query_thres --CE --index_type
//   --log_file --res_file --recall_thres --max_recall --max_hop
// plus -T / --num_threads, which the reference documents (README.md:117) but
// does not register; it is accepted and ignored.
// Extensions: --policy {auto,rounds,best_first} (auto: rounds up to 10 010 000 nodes, best-first above, the
// reference's choice of GPU or CPU search by size, src/index_gpu.cpp:257), --index_dir <dir> (overrides the
// derived ../indexes/<dataset>_<dist>_<R>_<thres>_<CE> path), --index_prefix
// and --evaluation_prefix (default ../indexes/ and ../evaluation/),
// --device_recall 1 (recall through IndexGPU::Search_and_Verify, the loop of
// the reference's tests/test_update.cpp:196-197, instead of the host count).
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "cli_options.h"
#include "coral_formats.h"
#include "efanna2e/index_gpu.h"

using namespace efanna2e;

namespace {

const cli::Option kOptions[] = {
    {"data_type", true, false, nullptr, "data type <int8/uint8/float>"},
    {"dist", true, false, nullptr, "distance function <l2/ip>"},
    {"base_data_path", true, false, nullptr, "Input data file in bin format"},
    {"dataset", true, false, nullptr, "dataset <t2i>"},
    {"recall_thres", false, false, "100", "The threshold of the recall of index"},
    {"query_path", true, false, nullptr, "Query file in bin format"},
    {"gt_path", true, false, nullptr, "Groundtruth file in bin format"},
    {"L", false, true, nullptr, "Priority queue length for searching"},
    {"max_recall", false, false, "0", "Max recall required to reach, must > 0.5"},
    {"max_hop", false, false, "1000000000", "Max limited hops"},
    {"k", false, false, "1", "k nearest neighbors"},
    {"max_degree", false, false, "32", "max_degree"},
    {"query_thres", false, false, "1.0", "The threshold of the size of query data"},
    {"log_file", false, false, "", "log file path"},
    {"res_file", false, false, "", "result file path"},
    {"config_file", false, false, "default", "config file path"},
    {"CE", false, false, "1", "Use connectivity enhancement or not"},
    {"index_type", false, false, "", ""},
    {"num_threads", false, false, "0", "accepted for compatibility, unused"},
    {"policy", false, false, "auto", "traversal <auto/rounds/best_first>; auto = by index size, as the reference"},
    {"index_dir", false, false, "", "index directory (overrides the derived name)"},
    {"index_prefix", false, false, "../indexes/", "directory holding index directories"},
    {"evaluation_prefix", false, false, "../evaluation/", "directory receiving the CSV"},
    {"device_recall", false, false, "0", "1: count hits on the device (IndexGPU::Search_and_Verify)"},
};

// tests/test_search_pipeline.cpp:25-39
float ComputeRecall(int q_num, int k, int gt_dim, int* res, int* gt) {
    return (float)coral_recall_hits(q_num, k, gt_dim, res, gt) / (float)((size_t)k * q_num);
}

}  // namespace

int main(int argc, char** argv) {
    std::map<std::string, std::vector<std::string>> opt;
    bool help = false;
    const size_t n_options = sizeof kOptions / sizeof kOptions[0];
    if (!cli::parse(kOptions, n_options, argc, argv, opt, &help)) return -1;
    if (help) {
        cli::usage(kOptions, n_options);
        return 0;
    }
    auto str = [&](const char* n) { return opt[n].empty() ? std::string() : opt[n][0]; };
    int k, max_degree, CE;
    float query_thres;
    double max_recall;
    std::vector<int> L_vec;
    try {
        k = std::stoi(str("k"));
        max_degree = std::stoi(str("max_degree"));
        CE = std::stoi(str("CE"));
        query_thres = std::stof(str("query_thres"));
        max_recall = std::stod(str("max_recall"));
        (void)std::stof(str("recall_thres"));
        (void)std::stod(str("max_hop"));
        for (const std::string& s : opt["L"]) L_vec.push_back(std::stoi(s));
    } catch (const std::exception& ex) {
        std::cerr << "the argument for an option is invalid: " << ex.what() << '\n';
        return -1;
    }
    const std::string dist = str("dist"), dataset = str("dataset"), index_type = str("index_type");
    const std::string base_data_file = str("base_data_path"), query_file = str("query_path"),
                      gt_file = str("gt_path"), res_file = str("res_file");

    char thres_buf[32];
    std::snprintf(thres_buf, sizeof thres_buf, "%.1f", query_thres);
    const std::string query_thres_str = thres_buf;
    const std::string dataset_dist = dataset + "_" + dist + "_" + std::to_string(max_degree);
    const std::string eval_dir = str("evaluation_prefix") + (res_file.empty() ? "search" : res_file);
    const std::string evaluation_save_file =
        eval_dir + "/" +
        (index_type.empty() ? dataset_dist + "_" + query_thres_str + "_" + std::to_string(CE) + ".csv"
                            : index_type + "_" + dataset_dist + ".csv");
    std::string graph_file = str("index_dir");
    if (graph_file.empty())
        graph_file = str("index_prefix") + dataset_dist + "_" + query_thres_str + "_" + std::to_string(CE ? 1 : 0);

    Parameters parameters;
    parameters.Set<std::string>("dist", dist);
    parameters.Set<int>("k", k);
    parameters.Set<int>("max_degree", max_degree);
    parameters.Set<int>("CE", CE);
    parameters.Set<std::string>("graph_file", graph_file);
    parameters.Set<std::string>("base_file", base_data_file);
    parameters.Set<std::string>("log_file", str("log_file"));
    parameters.Set<std::string>("config_file", str("config_file"));

    efanna2e::Metric dist_metric;
    DIST_METRIC metric;
    if (dist == "l2") {
        dist_metric = efanna2e::L2, metric = DIST_METRIC::L2_;
        std::cout << "Using l2 as distance metric" << std::endl;
    } else if (dist == "ip") {
        dist_metric = efanna2e::INNER_PRODUCT, metric = DIST_METRIC::IP_;
        std::cout << "Using inner product as distance metric" << std::endl;
    } else {
        std::cout << "Unknown distance type: " << dist << std::endl;
        return -1;
    }

    try {
        int64_t q_pts = 0;
        int32_t q_dim = 0;
        if (coral_fbin_read_meta(query_file.c_str(), &q_pts, &q_dim)) throw std::runtime_error(coral_last_error());
        const int32_t q_stride = (q_dim + 3) / 4 * 4;
        std::vector<float> query_data((size_t)q_pts * q_stride);
        if (coral_fbin_read(query_file.c_str(), query_data.data(), q_pts, q_dim, q_stride))
            throw std::runtime_error(coral_last_error());
        if (dist == "ip") coral_normalize_l2(query_data.data(), q_pts, q_stride);

        int32_t gt_pts = 0, gt_dim = 0;
        if (coral_gt_read_meta(gt_file.c_str(), &gt_pts, &gt_dim)) throw std::runtime_error(coral_last_error());
        std::vector<int> gt_ids((size_t)gt_pts * gt_dim);
        if (coral_gt_read(gt_file.c_str(), gt_ids.data(), gt_pts, gt_dim)) throw std::runtime_error(coral_last_error());
        std::cout << "gt_pts: " << gt_pts << ", gt_dim: " << gt_dim << std::endl;
        if (gt_pts < q_pts || gt_dim < k) throw std::runtime_error("ground truth smaller than queries x k");

        IndexGPU index((size_t)q_dim, 0, dist_metric, nullptr);
        index.LoadSearchNeededData(base_data_file.c_str(), "", metric);
        std::cout << "Load graph index: " << graph_file << std::endl;
        index.RunPrepare(parameters, Mode::SEARCH);
        if (index_type == "roar")
            index.LoadRoarGraph(std::string("../data/") + dataset + "/indexes/roar.index");
        else if (index_type == "para")
            index.LoadRoarGraph(std::string("../data/") + dataset + "/indexes/para-t2i-test-5");
        else if (index_type == "cdmg")
            index.LoadRoarGraph(std::string("../data/") + dataset + "/indexes/cdmg.index");
        const bool device_recall = str("device_recall") == "1";
        const std::string policy = str("policy");
        if (policy == "best_first")
            index.SetPolicy(CORAL_POLICY_BEST_FIRST);
        else if (policy == "rounds")
            index.SetPolicy(CORAL_POLICY_ROUNDS);
        else if (policy != "auto") {
            std::cerr << "unknown policy: " << policy << '\n';
            return -1;
        }
        std::cout << "traversal: " << (index.GetPolicy() == CORAL_POLICY_BEST_FIRST ? "best_first" : "rounds") << std::endl;

        std::cout << "k: " << k << std::endl;
        std::vector<int> res((size_t)q_pts * k, 0);
        cli::make_dirs(eval_dir);
        std::ofstream evaluation_out(evaluation_save_file, std::ios::out);
        if (!evaluation_out.is_open()) {
            std::cout << "Unable to open evaluation file: " << evaluation_save_file << std::endl;
            return 1;
        }
        std::cout << "L" << "\t\tQPS" << "\t\tavg_time" << "\t\trecall@" << k << "\t\tavg_hops" << std::endl;
        evaluation_out << "L, QPS, time, recall@" << k << ", avg_hops" << std::endl;
        if (L_vec.empty() && max_recall > 0.5) L_vec.push_back(128);

        for (size_t i = 0; i < L_vec.size(); ++i) {
            const int L = L_vec[i];
            if (k > L) {
                std::cout << "L must greater or equal than k" << std::endl;
                return 1;
            }
            float recall;
            Test_Result tr;
            if (device_recall) {
                // the device count assumes gt rows k apart (src/index_gpu.cpp:96-98)
                std::vector<int> gt_k((size_t)q_pts * k);
                for (int64_t qi = 0; qi < q_pts; ++qi)
                    std::copy_n(gt_ids.data() + (size_t)qi * gt_dim, k, gt_k.data() + (size_t)qi * k);
                tr = index.Search_and_Verify(query_data.data(), gt_k.data(), (int)q_pts, L);
                recall = tr.calc_recall((int)q_pts * k) / 100.0f;
            } else {
                tr = index_type.empty() ? index.Search(query_data.data(), (int)q_pts, L, res.data())
                                        : index.Search(query_data.data(), (int)q_pts, L, res.data(), 1);
                recall = ComputeRecall((int)q_pts, k, gt_dim, res.data(), gt_ids.data());
            }
            const float time = tr.get_time(), qps = (float)q_pts / time;
            const float avg_hops = tr.avg_hops((int)q_pts);
            std::cout << L << "\t\t" << qps << "\t\t" << time << "\t\t" << recall << "\t\t" << avg_hops << std::endl;
            evaluation_out << L << "," << qps << "," << time << "," << recall << "," << avg_hops << std::endl;
            if (max_recall > 0.5 && recall < max_recall) {
                if (128 + L_vec.back() > CORAL_MAX_BEAM) {
                    std::cout << "Beam capacity limit " << CORAL_MAX_BEAM
                              << " reached, judged as unable to meet the recall requirement, termination" << std::endl;
                    break;
                }
                L_vec.push_back(128 + L_vec.back());
            }
            if (i > 50) {
                std::cout << "Queue is too long, judged as unable to meet the recall requirement, termination"
                          << std::endl;
                break;
            }
        }
    } catch (const std::exception& ex) {
        std::cerr << ex.what() << std::endl;
        return 1;
    }
    return 0;
}
