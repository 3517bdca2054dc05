// test_update -- the reference's update evaluation driver (tests/test_update.cpp:30-283) in its delete-only mode
// (--upd_mode 1) over efanna2e::IndexGPU of this library.
//
// The first half of the base file is the index (built here when config "upd_build" is 1, tests/test_update.cpp:192-195,
// else read from ../indexes/<dataset>_<dist>_<R>_upd); then round / 2 batches of ids are deleted, and after each one
// the queries are searched and scored on the device against the ground truth of update_compute_gt
// (IndexGPU::Search_and_Verify, :252-268).  Deleting tombstones the ids (GPUFuncs::del_node_mark); the repair of the
// remaining rows that the reference adds for upd_type 1-3 and every mode that inserts (0, 2, 4) are not provided.
// Output: ../evaluation/upd/<upd_mode>_<upd_type>.csv with the header "round, recall, avg_hops, time, qps".
// Flags as in the reference: --dataset --base_data_path --update_gt_file --sampled_query_data_path --dist --data_type
// --recall_thres --query_thres --max_degree --k --L --query_path --upd_mode --config_file; extensions --index_prefix,
// --evaluation_prefix.
#include <cstdio>
#include <fstream>
#include <iostream>
#include <numeric>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "cli_options.h"
#include "coral_formats.h"
#include "efanna2e/index_gpu.h"

using namespace efanna2e;

namespace {
const cli::Option kOptions[] = {
    {"dataset", true, false, nullptr, "dataset <t2i>"},
    {"base_data_path", true, false, nullptr, "Input data file in bin format"},
    {"update_gt_file", true, false, nullptr, "update gt file in bin format"},
    {"sampled_query_data_path", true, false, nullptr, "Sampled query file in bin format"},
    {"dist", false, false, "l2", "distance function <l2/ip>"},
    {"data_type", false, false, "float", "data type <int8/uint8/float>"},
    {"recall_thres", false, false, "80", "The threshold of the recall of index"},
    {"query_thres", false, false, "10.0", "The threshold of the size of query data"},
    {"max_degree", false, false, "2", "Number of neighbors for graph"},
    {"k", false, false, "1", "k nearest neighbors"},
    {"L", false, false, "512", "beam capacity"},
    {"query_path", true, false, nullptr, "Query file in bin format"},
    {"upd_mode", true, false, nullptr, "update mode"},
    {"config_file", false, false, "default", "config file"},
    {"index_prefix", false, false, "../indexes/", "directory holding index directories"},
    {"evaluation_prefix", false, false, "../evaluation/", "directory receiving the CSV"},
};

std::vector<float> load_padded(const std::string& path, int64_t* n, int32_t* stride) {
    int32_t dim = 0;
    if (coral_fbin_read_meta(path.c_str(), n, &dim)) throw std::runtime_error(coral_last_error());
    *stride = (dim + 3) / 4 * 4;
    std::vector<float> data((size_t)*n * *stride);
    if (coral_fbin_read(path.c_str(), data.data(), *n, dim, *stride)) throw std::runtime_error(coral_last_error());
    return data;
}

// "upd_type" of config.json names the repair strategy in the reference; here it only names the CSV
int config_int(const std::string& config_file, const char* key, int fallback) {
    std::ifstream f(config_file == "default" ? "../config.json" : config_file);
    if (!f.is_open()) return fallback;
    std::stringstream ss;
    ss << f.rdbuf();
    const std::string text = ss.str(), needle = std::string("\"") + key + "\"";
    size_t p = text.find(needle);
    if (p == std::string::npos || (p = text.find(':', p)) == std::string::npos) return fallback;
    return std::atoi(text.c_str() + p + 1);
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
    int max_degree, k, L, upd_mode;
    try {
        max_degree = std::stoi(str("max_degree"));
        k = std::stoi(str("k"));
        L = std::stoi(str("L"));
        upd_mode = std::stoi(str("upd_mode"));
        (void)std::stof(str("recall_thres")), (void)std::stof(str("query_thres"));
    } catch (const std::exception& ex) {
        std::cerr << "the argument for an option is invalid: " << ex.what() << '\n';
        return -1;
    }
    const std::string dist = str("dist"), dataset = str("dataset"), config_file = str("config_file");
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
    if (upd_mode != 1) {
        std::cerr << "only --upd_mode 1 (delete only) is provided\n";
        return -1;
    }
    try {
        int64_t total_num = 0, sq_num = 0, query_num = 0;
        int32_t stride = 0, sq_stride = 0, q_stride = 0;
        std::vector<float> data_bp = load_padded(str("base_data_path"), &total_num, &stride);
        std::vector<float> data_sq = load_padded(str("sampled_query_data_path"), &sq_num, &sq_stride);
        std::vector<float> queries = load_padded(str("query_path"), &query_num, &q_stride);
        if (stride != sq_stride || stride != q_stride) throw std::runtime_error("dimensions of the three files differ");
        const int64_t base_num = total_num / 2, upd_num = base_num;  // tests/test_update.cpp:129

        const std::string dataset_dist = dataset + "_" + dist + "_" + std::to_string(max_degree) + "_upd";
        const std::string graph_file = str("index_prefix") + dataset_dist;
        const int upd_type = config_int(config_file, "upd_type", 1), upd_build = config_int(config_file, "upd_build", 1);
        const std::string eval_dir = str("evaluation_prefix") + "upd";
        const std::string evaluation_save_file = eval_dir + "/" + std::to_string(upd_mode) + "_" + std::to_string(upd_type) + ".csv";

        Parameters parameters;
        parameters.Set<int>("max_degree", max_degree);
        parameters.Set<int>("k", k);
        parameters.Set<int>("CE", 1);
        parameters.Set<std::string>("base_file", str("base_data_path"));
        parameters.Set<std::string>("graph_file", graph_file);
        parameters.Set<std::string>("config_file", config_file);
        parameters.Set<std::string>("dist", dist);
        parameters.Set<std::string>("dataset", dataset);

        const std::string gt_path = str("update_gt_file") + ".del";
        std::ifstream gt_file(gt_path, std::ios::binary);
        if (!gt_file.is_open()) {
            std::cout << "Failed to open update_gt_file: " << gt_path << std::endl;
            return 255;
        }
        cli::make_dirs(eval_dir);
        std::ofstream eva_file(evaluation_save_file, std::ios::out);
        if (!eva_file.is_open()) {
            std::cout << "Failed to open evaluation_save_file: " << evaluation_save_file << std::endl;
            return 255;
        }
        int round = 0;
        gt_file.read(reinterpret_cast<char*>(&round), sizeof(int));
        if (round < 2 || round > 1000000) throw std::runtime_error("update_gt_file: implausible round count");
        // delete-only files hold round / 2 + 1 blocks; the reference reads round + 1 and leaves the rest zero
        std::vector<int> gts((size_t)query_num * k * (round + 1), 0);
        gt_file.read(reinterpret_cast<char*>(gts.data()), (std::streamsize)(sizeof(int) * gts.size()));
        if ((size_t)gt_file.gcount() < sizeof(int) * (size_t)query_num * k * (round / 2 + 1))
            throw std::runtime_error("update_gt_file is shorter than round / 2 + 1 blocks of nq * k ids");
        eva_file << "round, recall, avg_hops, time, qps" << std::endl;

        IndexGPU index((size_t)stride, (size_t)(base_num + sq_num), dist_metric, nullptr);
        index.load_config(config_file);
        if (upd_build) {
            std::cout << "Building initial index..." << std::endl;
            cli::make_dirs(str("index_prefix"));
            index.BuildGPU((size_t)sq_num, data_sq.data(), (size_t)base_num, data_bp.data(), parameters);
        }
        index.RunPrepare(parameters, Mode::UPD, (size_t)base_num, data_bp.data());
        auto report = [&](int row, Test_Result tr, bool per_query_time) {
            const float recall = tr.calc_recall((int)query_num * k), hops = tr.avg_hops((int)query_num);
            eva_file << row << ", " << recall << ", " << hops << ", "
                     << (per_query_time ? tr.get_time() / query_num : tr.get_time()) << ", " << query_num / tr.get_time()
                     << std::endl;
            std::cout << "Batch " << row << "/" << round / 2 << " Search result: recall=" << recall << "%, avg_hops=" << hops
                      << ", time=" << tr.get_time() << "s" << std::endl;
        };
        report(0, index.Search_and_Verify(queries.data(), gts.data(), (int)query_num, L), false);
        const int64_t batch = (upd_num + round - 1) / round;
        std::vector<int> del_ids;
        for (int batch_i = 0; batch_i < round / 2; ++batch_i) {
            const int64_t lo = std::min(upd_num, batch_i * batch), upd_n = std::min(batch, upd_num - lo);
            del_ids.resize((size_t)upd_n);
            std::iota(del_ids.begin(), del_ids.end(), (int)lo);
            index.Delete(del_ids);
            report(batch_i + 1,
                   index.Search_and_Verify(queries.data(), gts.data() + (size_t)query_num * k * (batch_i + 1), (int)query_num, L),
                   true);
        }
        std::cout << "Finished\n";
    } catch (const std::exception& ex) {
        std::cerr << ex.what() << std::endl;
        return 1;
    }
    return 0;
}
