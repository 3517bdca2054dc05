// comp_gt -- ground-truth tool with the flags and output file of the reference's
// tests/comp_gt.cpp:36-176, computing the exact k nearest neighbours with this library's
// brute-force kernels where the reference calls faiss.
//   --base_data_path <fbin> --query_data_path <fbin> --gt_save_file <file>
//   [--k 10] [--nq 0 (= all)] [--dist l2|ip] [--data_type float]
// Output: uint32 nq, uint32 k, int32 ids[nq*k] (tests/comp_gt.cpp:142-175).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <map>
#include <string>
#include <vector>

#include "coral_formats.h"
#include "coral_search.h"

int main(int argc, char** argv) {
    std::map<std::string, std::string> opt = {{"data_type", "float"}, {"dist", "l2"}, {"k", "10"}, {"nq", "0"}};
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "-h" || a == "--help") {
            std::cout << "Arguments:\n  --data_type arg (=float)\n  --dist arg (=l2)\n  --base_data_path arg\n"
                         "  --query_data_path arg\n  --gt_save_file arg\n  --k arg (=10)\n  --nq arg (=0)\n";
            return 0;
        }
        if (a.rfind("--", 0) != 0) {
            std::cerr << "unrecognised option '" << a << "'\n";
            return -1;
        }
        const size_t eq = a.find('=');
        const std::string name = a.substr(2, eq == std::string::npos ? std::string::npos : eq - 2);
        static const char* known[] = {"data_type", "dist", "base_data_path", "query_data_path", "gt_save_file", "k", "nq"};
        bool ok = false;
        for (const char* kname : known) ok |= name == kname;
        if (!ok) {
            std::cerr << "unrecognised option '" << a << "'\n";
            return -1;
        }
        if (eq != std::string::npos)
            opt[name] = a.substr(eq + 1);
        else if (i + 1 < argc)
            opt[name] = argv[++i];
        else {
            std::cerr << "the required argument for option '--" << name << "' is missing\n";
            return -1;
        }
    }
    for (const char* req : {"base_data_path", "query_data_path", "gt_save_file"})
        if (!opt.count(req)) {
            std::cerr << "the option '--" << req << "' is required but missing\n";
            return -1;
        }
    const std::string dist = opt["dist"];
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
    const int k = std::atoi(opt["k"].c_str()), nq_opt = std::atoi(opt["nq"].c_str());
    int64_t nb = 0, nq = 0;
    int32_t dim = 0, qdim = 0;
    auto die = [](const char* what) {
        std::cerr << what << ": " << coral_last_error() << std::endl;
        return 1;
    };
    if (coral_fbin_read_meta(opt["base_data_path"].c_str(), &nb, &dim)) return die("load_meta");
    if (coral_fbin_read_meta(opt["query_data_path"].c_str(), &nq, &qdim)) return die("load_meta");
    if (dim != qdim) {
        std::cerr << "base and query dimension mismatch" << std::endl;
        return 1;
    }
    if (nq_opt > 0 && nq_opt < nq) nq = nq_opt;
    const int32_t stride = (dim + 3) / 4 * 4;
    std::vector<float> base((size_t)nb * stride), query((size_t)nq * stride);
    if (coral_fbin_read(opt["base_data_path"].c_str(), base.data(), nb, dim, stride)) return die("load_data");
    if (coral_fbin_read(opt["query_data_path"].c_str(), query.data(), nq, dim, stride)) return die("load_data");
    if (metric == CORAL_IP) {
        coral_normalize_l2(base.data(), nb, stride);
        coral_normalize_l2(query.data(), nq, stride);
    }
    std::cout << "base_num: " << nb << " sq_num: " << nq << " dim: " << dim << std::endl;
    coral_index_desc d;
    std::memset(&d, 0, sizeof d);
    d.base = base.data(), d.n = nb, d.dim = stride, d.metric = metric;
    coral_index* idx = nullptr;
    if (coral_index_create(&d, &idx)) return die("index");
    std::vector<int32_t> ids((size_t)nq * k);
    double t = 0;
    if (coral_bruteforce_knn(idx, query.data(), (int32_t)nq, k, 0, ids.data(), nullptr, &t)) return die("search");
    coral_index_destroy(idx);
    if (coral_gt_write(opt["gt_save_file"].c_str(), ids.data(), (int32_t)nq, k)) return die("gt_save_file");
    std::cout << nq << " gt comp finished, time: " << t << ", avg_time: " << t / nq << std::endl;
    return 0;
}
