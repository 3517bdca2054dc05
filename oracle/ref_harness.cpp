// ref_harness.cpp -- TEST INFRASTRUCTURE.  Compiles the reference's own
// arithmetic core for the CPU search path in place: the header-only
// NeighborPriorityQueue (include/efanna2e/neighbor.h:148-237) and
// DistanceL2::compare (include/efanna2e/distance.h:39-89) are included from the
// reference tree (-I<reference>/include at build time; nothing is copied).
//
// src/search_in_cpu.cpp itself cannot be a translation unit here (its includes
// pull in CUDA, faiss, thrust and Roaring, src/search_in_cpu.cpp:15-19), so the
// per-query loop of src/search_in_cpu.cpp:63-108 is driven below around those
// two reference classes: same calls in the same order, with the graph row read
// from the compact neighbour table instead of a Slot.
//
// Output goes to oracle/_ref/ only.  Used to (1) pin oracle/coral_oracle.c's
// policy A, queue and AVX-512 distance bit for bit, (2) write the fixtures under
// tests/golden/, (3) optionally serve as the timed CPU baseline.
#include <omp.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

#include "efanna2e/distance.h"
#include "efanna2e/neighbor.h"

using efanna2e::DistanceL2;
using efanna2e::Neighbor;
using efanna2e::NeighborPriorityQueue;

extern "C" {

__attribute__((visibility("default"))) float ref_distance_l2(const float* a, const float* b,
                                                             int dim) {
    DistanceL2 d;
    return d.compare(a, b, (unsigned)dim);
}

// ops[i] >= 0: insert {ops[i], dists[i]}; ops[i] == -1: closest_unexpanded (if any)
__attribute__((visibility("default"))) int ref_queue_run(int capacity, const int32_t* ops,
                                                         const float* dists, int n_ops,
                                                         int32_t* ids_out, float* dists_out,
                                                         int32_t* flags_out, int32_t* cur_out,
                                                         int32_t* popped, int32_t* n_popped) {
    NeighborPriorityQueue q((size_t)capacity);
    int np = 0;
    for (int i = 0; i < n_ops; ++i) {
        if (ops[i] >= 0)
            q.insert(Neighbor(ops[i], dists[i], false));
        else if (q.has_unexpanded_node())
            popped[np++] = q.closest_unexpanded().id;
    }
    for (size_t i = 0; i < q.size(); ++i) {
        ids_out[i] = q[i].id;
        dists_out[i] = q[i].distance;
        flags_out[i] = q[i].flag ? 1 : 0;
    }
    *cur_out = (int32_t)q.cur();
    *n_popped = np;
    return (int)q.size();
}

// The loop of src/search_in_cpu.cpp:41-111.  stats per query: [0] hops (M + expansions),
// [1] expansions, [2] distance evaluations, [3] expansions.
__attribute__((visibility("default"))) int ref_search_in_cpu(
    const float* vectors, const int32_t* nbr_table, int64_t n_nodes, int dim, int R,
    const int32_t* entry_ids, int M, const float* queries, int Q, int k, int L, int32_t* out_ids,
    float* out_dists, int32_t* stats, int nthreads, double* time_s) {
    const size_t total = (size_t)Q * k;
    std::fill(out_ids, out_ids + total, -1);
    if (out_dists) std::fill(out_dists, out_dists + total, std::numeric_limits<float>::infinity());
    const int T = nthreads > 0 ? nthreads : std::max(1, omp_get_max_threads());
    DistanceL2 metric;  // the CPU path always measures squared L2 (src/search_in_cpu.cpp:52)
    double elapsed = 0.0;
#pragma omp parallel num_threads(T)
    {
        // one byte per node and an 8-bit epoch per thread (src/search_in_cpu.cpp:44-48, 68-71)
        std::vector<uint8_t> seen((size_t)n_nodes, 0);
        uint8_t epoch = 1;
#pragma omp barrier
        const auto t_begin = std::chrono::steady_clock::now();
#pragma omp for schedule(dynamic, 1)
        for (int q = 0; q < Q; ++q) {
            const float* qv = queries + (size_t)q * dim;
            NeighborPriorityQueue pq((size_t)L);
            if (++epoch == 0) {
                std::fill(seen.begin(), seen.end(), 0);
                epoch = 1;
            }
            int32_t evals = 0, expansions = 0;
            for (int s = 0; s < M; ++s) {  // seeds (src/search_in_cpu.cpp:74-79)
                const int node = entry_ids[s];
                pq.insert(Neighbor(node, metric.compare(vectors + (size_t)node * dim, qv, dim), false));
                seen[node] = epoch;
                ++evals;
            }
            while (pq.has_unexpanded_node()) {  // src/search_in_cpu.cpp:83-99
                const int node = pq.closest_unexpanded().id;
                ++expansions;
                const int32_t* row = nbr_table + (size_t)node * R;
                for (int j = 0; j < R && row[j] >= 0; ++j) {
                    const int v = row[j];
                    if (seen[v] == epoch) continue;
                    pq.insert(Neighbor(v, metric.compare(vectors + (size_t)v * dim, qv, dim), false));
                    seen[v] = epoch;
                    ++evals;
                }
            }
            const int filled = std::min<int>(k, (int)pq.size());  // src/search_in_cpu.cpp:103-107
            for (int i = 0; i < filled; ++i) {
                out_ids[(size_t)q * k + i] = pq[i].id;
                if (out_dists) out_dists[(size_t)q * k + i] = pq[i].distance;
            }
            if (stats) {
                int32_t* st = stats + (size_t)q * 4;
                st[0] = M + expansions, st[1] = expansions, st[2] = evals, st[3] = expansions;
            }
        }
        const auto t_end = std::chrono::steady_clock::now();
#pragma omp master
        elapsed = std::chrono::duration<double>(t_end - t_begin).count();
    }
    if (time_s) *time_s = elapsed;
    return 0;
}
}
