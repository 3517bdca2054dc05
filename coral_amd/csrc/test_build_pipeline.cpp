// test_build_pipeline -- the reference's construction driver (tests/test_build_pipeline.cpp:27-258) over
// efanna2e::IndexGPU::BuildGPU of this library: same flags, same index-directory naming.
//
// Flags of the reference (tests/test_build_pipeline.cpp:45-121), all accepted:
//   --data_type --dist {l2,ip} --N --dataset --base_data_path --train_gt_file --sampled_query_data_path
//   --query_test_file --gt_test_file --M_sq --M_pjbp --L_pjpq --num_threads/-T --CE --k --iso_thres
//   --recall_thres --query_thres --log_file --config_file
// --M_pjbp is the row width, --k the cluster size (nearest base points per sampled query).  --train_gt_file names
// precomputed clusters (a ground-truth file of the sampled queries with k ids per row).  --query_test_file with
// --gt_test_file: the reference searches these queries with beam test_beam_capacity when the graph is complete and
// logs recall and hops (src/index_gpu.cpp:376-378, include/gpufuncs.cuh:688-702); so does this driver, on stdout.
// The knn cache is not provided.
// Extensions: --index_dir <dir> (overrides the derived <index_prefix><dataset>_<dist>_<R>_<thres>_<CE> path) and
// --index_prefix (default ../indexes/).
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <iostream>
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
    {"N", false, false, "0", "base n"},
    {"dataset", true, false, nullptr, "dataset <t2i>"},
    {"base_data_path", true, false, nullptr, "Input data file in bin format"},
    {"train_gt_file", false, false, "", "train_gt_file in bin format"},
    {"sampled_query_data_path", true, false, nullptr, "Sampled query file in bin format"},
    {"query_test_file", false, false, "None", "query_test_file"},
    {"gt_test_file", false, false, "None", "gt_test_file"},
    {"M_sq", false, false, "32", "Number of neighbors for sampled query points to build the bipartite graph"},
    {"M_pjbp", false, false, "32", "Number of neighbors for projection graph"},
    {"L_pjpq", false, false, "32", "Priority queue length for projection graph searching"},
    {"num_threads", false, false, "0", "accepted for compatibility, unused"},
    {"CE", false, false, "1", "Use connectivity enhancement or not"},
    {"k", false, false, "1", "k nearest neighbors"},
    {"iso_thres", false, false, "0.9", "The threshold of the proportion of isolated nodes"},
    {"recall_thres", false, false, "100", "The threshold of the recall of index"},
    {"query_thres", false, false, "100.0", "The threshold of the size of query data"},
    {"log_file", false, false, "", "log file path"},
    {"config_file", false, false, "default", "config file path"},
    {"index_dir", false, false, "", "index directory (overrides the derived name)"},
    {"index_prefix", false, false, "../indexes/", "directory holding index directories"},
};

std::vector<float> load_padded(const std::string& path, int64_t* n, int32_t* stride) {
    int32_t dim = 0;
    if (coral_fbin_read_meta(path.c_str(), n, &dim)) throw std::runtime_error(coral_last_error());
    *stride = (dim + 3) / 4 * 4;  // include/efanna2e/util.h:194-208
    std::vector<float> data((size_t)*n * *stride);
    if (coral_fbin_read(path.c_str(), data.data(), *n, dim, *stride)) throw std::runtime_error(coral_last_error());
    return data;
}

}  // namespace

int main(int argc, char** argv) {
    cli::Values opt;
    bool help = false;
    const size_t n_options = sizeof kOptions / sizeof kOptions[0];
    if (!cli::parse(kOptions, n_options, argc, argv, opt, &help)) return -1;
    if (help) {
        cli::usage(kOptions, n_options);
        return 0;
    }
    auto str = [&](const char* n) { return opt[n].empty() ? std::string() : opt[n][0]; };
    int max_degree, CE, k;
    long long N;
    float query_thres;
    try {
        max_degree = std::stoi(str("M_pjbp"));
        CE = std::stoi(str("CE"));
        k = std::stoi(str("k"));
        N = std::stoll(str("N"));
        query_thres = std::stof(str("query_thres"));
        (void)std::stoi(str("M_sq")), (void)std::stoi(str("L_pjpq")), (void)std::stoi(str("num_threads"));
        (void)std::stof(str("iso_thres")), (void)std::stof(str("recall_thres"));
    } catch (const std::exception& ex) {
        std::cerr << "the argument for an option is invalid: " << ex.what() << '\n';
        return -1;
    }
    const std::string dist = str("dist"), dataset = str("dataset");
    if (str("data_type") != "float") {
        std::cerr << "only --data_type float is provided\n";
        return -1;
    }
    const bool test_search = str("query_test_file") != "None";
    if (test_search != (str("gt_test_file") != "None")) {
        std::cerr << "--query_test_file and --gt_test_file go together\n";
        return -1;
    }
    std::cout << "sampled query: " << str("sampled_query_data_path") << std::endl;
    Metric dist_metric;
    if (dist == "l2") {
        dist_metric = efanna2e::L2;
        std::cout << "Using l2 as distance metric" << std::endl;
    } else if (dist == "ip") {
        dist_metric = efanna2e::INNER_PRODUCT;
        std::cout << "Using inner product as distance metric" << std::endl;
    } else {
        std::cout << "Unknown distance type: " << dist << std::endl;
        return -1;
    }
    char thres_buf[32];
    std::snprintf(thres_buf, sizeof thres_buf, "%.1f", query_thres);
    const std::string dataset_dist = dataset + "_" + dist + "_" + std::to_string(max_degree);
    std::string graph_file = str("index_dir");
    if (graph_file.empty()) {
        cli::make_dirs(str("index_prefix"));
        graph_file = str("index_prefix") + dataset_dist + "_" + thres_buf + "_" + std::to_string(CE ? 1 : 0);
    }
    std::cout << "Index graph save path: " << graph_file << std::endl;

    try {
        int64_t base_num = 0, sq_num = 0;
        int32_t base_stride = 0, sq_stride = 0;
        std::vector<float> data_bp = load_padded(str("base_data_path"), &base_num, &base_stride);
        std::vector<float> data_sq = load_padded(str("sampled_query_data_path"), &sq_num, &sq_stride);
        if (base_stride != sq_stride) throw std::runtime_error("base and sampled-query dimensions differ");
        if (N > 0 && N < base_num) base_num = N;  // tests/test_build_pipeline.cpp:245
        if (dist_metric == efanna2e::INNER_PRODUCT) {
            // the reference passes (data, dim, dim) for the base here (tests/test_build_pipeline.cpp:170), which
            // normalises only the first dim rows; every row is normalised here, as the search driver's loader does
            coral_normalize_l2(data_bp.data(), base_num, base_stride);
            coral_normalize_l2(data_sq.data(), sq_num, sq_stride);
        }
        Parameters parameters;
        parameters.Set<int>("max_degree", max_degree);
        parameters.Set<int>("CE", CE);
        parameters.Set<int>("k", k);
        parameters.Set<std::string>("base_file", str("base_data_path"));
        parameters.Set<std::string>("graph_file", graph_file);
        parameters.Set<std::string>("log_file", str("log_file"));
        parameters.Set<std::string>("config_file", str("config_file"));
        parameters.Set<std::string>("dist", dist);
        parameters.Set<std::string>("dataset", dataset);
        parameters.Set<std::string>("train_gt_file", str("train_gt_file").empty() ? "None" : str("train_gt_file"));
        // tests/test_build_pipeline.cpp:215-216: BuildGPU searches these while the graph grows (config.json "test_search")
        parameters.Set<std::string>("query_test_file", str("query_test_file"));
        parameters.Set<std::string>("gt_test_file", str("gt_test_file"));

        IndexGPU index((size_t)base_stride, (size_t)(base_num + sq_num), dist_metric, nullptr);
        const auto s = std::chrono::high_resolution_clock::now();
        index.BuildGPU((size_t)sq_num, data_sq.data(), (size_t)base_num, data_bp.data(), parameters);
        const std::chrono::duration<double> diff = std::chrono::high_resolution_clock::now() - s;
        const coral_build_stats& b = index.last_build;
        std::cout << "batches: " << b.batches << ", isolated after the batches: " << b.isolated
                  << ", reverse edges: " << b.reverse_edges << ", most-hit nodes rewired: " << b.top_hit_nodes
                  << ", average degree: " << (double)b.edges / (double)base_num << std::endl;
        std::cout << "knn " << b.knn_s << " s, batch updates " << b.nap_s << " s, enhancement " << b.enhance_s << " s"
                  << std::endl;
        std::cout << "indexing time: " << diff.count() << std::endl;
        std::cout << "Save index to " << graph_file << std::endl;
        if (test_search) {
            int64_t q_num = 0;
            int32_t q_stride = 0, gt_num = 0, gt_dim = 0;
            std::vector<float> queries = load_padded(str("query_test_file"), &q_num, &q_stride);
            if (q_stride != base_stride) throw std::runtime_error("base and test-query dimensions differ");
            if (dist_metric == efanna2e::INNER_PRODUCT) coral_normalize_l2(queries.data(), q_num, q_stride);
            if (coral_gt_read_meta(str("gt_test_file").c_str(), &gt_num, &gt_dim))
                throw std::runtime_error(coral_last_error());
            if (gt_num < q_num || gt_dim < k) throw std::runtime_error("test ground truth smaller than queries x k");
            std::vector<int> gt((size_t)gt_num * gt_dim), gt_k((size_t)q_num * k);
            if (coral_gt_read(str("gt_test_file").c_str(), gt.data(), gt_num, gt_dim))
                throw std::runtime_error(coral_last_error());
            for (int64_t q = 0; q < q_num; ++q)  // the device count takes rows k apart (src/index_gpu.cpp:96-98)
                std::copy_n(gt.data() + (size_t)q * gt_dim, k, gt_k.data() + (size_t)q * k);
            const int L = std::max(PC.test_beam_capacity, k);
            Test_Result tr = index.Search_and_Verify(queries.data(), gt_k.data(), (int)q_num, L);
            std::cout << "test search: L " << L << ", recall@" << k << " " << tr.calc_recall((int)q_num * k)
                      << " %, avg hops " << tr.avg_hops((int)q_num) << ", QPS " << (double)q_num / tr.get_time()
                      << std::endl;
        }
    } catch (const std::exception& ex) {
        std::cerr << ex.what() << std::endl;
        return 1;
    }
    return 0;
}
