// update_compute_gt -- the ground truth of the reference's update evaluation (tests/update_compute_gt.cpp:32-207)
// for its delete-only mode (--upd_mode 1), with this library's brute-force kernels where the reference calls faiss.
//
// The index under test holds the first half of the base file.  The file written is
//   int32 round (= 100), then blocks of int32 ids[nq][k]:
//   block 0      the k nearest of every query among ids [0, n/2)
//   block b >= 1 the same after the ids [0, b * batch) are gone, batch = ceil((n/2) / round); round / 2 blocks
// (tests/update_compute_gt.cpp:120-132, 169-186).  The file name gets ".del" appended (:115-116).
// Flags as in the reference: --dist --dataset --base_data_path --query_path --update_gt_file --k --upd_mode
// [--data_type float].  The modes that insert (0, 2, 4) are not provided.
#include <cstdio>
#include <fstream>
#include <iostream>
#include <numeric>
#include <stdexcept>
#include <string>
#include <vector>

#include "cli_options.h"
#include "coral_formats.h"
#include "coral_search.h"

namespace {
const cli::Option kOptions[] = {
    {"dist", true, false, nullptr, "distance function <l2/ip>"},
    {"dataset", true, false, nullptr, "dataset <t2i>"},
    {"base_data_path", true, false, nullptr, "Input data file in bin format"},
    {"query_path", true, false, nullptr, "Query file in bin format"},
    {"update_gt_file", true, false, nullptr, "update gt file in bin format"},
    {"k", true, false, nullptr, "k nearest neighbors"},
    {"upd_mode", true, false, nullptr, "update mode"},
    {"data_type", false, false, "float", "data type <int8/uint8/float>"},
};
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
    int k, upd_mode;
    try {
        k = std::stoi(str("k"));
        upd_mode = std::stoi(str("upd_mode"));
    } catch (const std::exception& ex) {
        std::cerr << "the argument for an option is invalid: " << ex.what() << '\n';
        return -1;
    }
    const std::string dist = str("dist");
    int metric;
    if (dist == "l2") {
        metric = CORAL_L2;
        std::cout << "Using l2 as distance metric" << std::endl;
    } else if (dist == "ip") {
        metric = CORAL_IP;
        std::cout << "Using inner product as distance metric" << std::endl;
    } else {
        std::cout << "Unknown distance type: " << dist << std::endl;
        return -1;
    }
    if (upd_mode != 1) {
        std::cerr << "only --upd_mode 1 (delete only) is provided\n";
        return -1;
    }
    coral_index* idx = nullptr;
    try {
        auto check = [](int rc) {
            if (rc) throw std::runtime_error(coral_last_error());
        };
        int64_t total = 0, nq = 0;
        int32_t dim = 0, qdim = 0;
        check(coral_fbin_read_meta(str("base_data_path").c_str(), &total, &dim));
        check(coral_fbin_read_meta(str("query_path").c_str(), &nq, &qdim));
        if (dim != qdim) throw std::runtime_error("base and query dimension mismatch");
        const int32_t stride = (dim + 3) / 4 * 4;
        const int64_t base_num = total / 2;  // tests/update_compute_gt.cpp:104-105
        if (base_num < 1) throw std::runtime_error("the base file holds fewer than two vectors");
        std::vector<float> base((size_t)base_num * stride), queries((size_t)nq * stride);
        check(coral_fbin_read(str("base_data_path").c_str(), base.data(), base_num, dim, stride));
        std::cout << "load query\n";
        check(coral_fbin_read(str("query_path").c_str(), queries.data(), nq, dim, stride));
        const std::string path = str("update_gt_file") + ".del";
        std::ofstream gt_file(path, std::ios::binary);
        if (!gt_file.is_open()) {
            std::cout << "Failed to open update_gt_file: " << path << std::endl;
            return 255;
        }
        const int round = 100;
        const int64_t batch = (base_num + round - 1) / round;
        gt_file.write(reinterpret_cast<const char*>(&round), sizeof(int));

        coral_index_desc d{};
        d.base = base.data(), d.n = base_num, d.dim = stride, d.metric = metric;
        check(coral_index_create(&d, &idx));
        std::vector<int32_t> ids((size_t)nq * k);
        check(coral_bruteforce_knn(idx, queries.data(), (int32_t)nq, k, 0, ids.data(), nullptr, nullptr));
        gt_file.write(reinterpret_cast<const char*>(ids.data()), sizeof(int32_t) * ids.size());
        std::vector<int32_t> gone;
        for (int batch_i = 0; batch_i < round / 2; ++batch_i) {
            std::cout << "Update " << batch_i << " round" << std::endl;
            const int64_t lo = std::min(base_num, batch_i * batch), hi = std::min(base_num, lo + batch);
            gone.resize((size_t)(hi - lo));
            std::iota(gone.begin(), gone.end(), (int32_t)lo);
            check(coral_index_mark_deleted(idx, gone.data(), (int32_t)gone.size()));
            check(coral_bruteforce_knn(idx, queries.data(), (int32_t)nq, k, 1, ids.data(), nullptr, nullptr));
            gt_file.write(reinterpret_cast<const char*>(ids.data()), sizeof(int32_t) * ids.size());
        }
        coral_index_destroy(idx);
        std::cout << "Finished\n";
    } catch (const std::exception& ex) {
        if (idx) coral_index_destroy(idx);
        std::cerr << ex.what() << std::endl;
        return 1;
    }
    return 0;
}
