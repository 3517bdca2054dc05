// graph_build_api.cpp -- coral_build_*: the query-aware graph construction behind the C ABI.
//   coral_build_graph            IndexGPU::BuildGPU            src/index_gpu.cpp:308-383 (KNNTask :385-499, GraphTask :501-580)
//   coral_build_nap_batch        GPUFuncs::graph_update        src/upd_disk.cu:218-224 -> gpu_neibor_aware, src/upd_gpu.cu:260-303
//   coral_build_connect_enhance  GPUFuncs::gpu_connect_enhance src/enhance.cu:728-861 (enhance_mode 0, isolated nodes)
//   coral_build_enhance_batch    GPUFuncs::enhance_neibor_aware_gpu src/enhance.cu:660-689
//   coral_build_enhance_top_batch  its five-argument form      src/enhance.cu:632-658 (most-hit nodes, :819-856)
//   coral_build_resume           Graph ctor in Mode::CE        include/graph.cuh:252-256 (rows of a saved build)
//   coral_build_test_search      GPUFuncs::test_search         include/gpufuncs.cuh:688-702 (and its calls during a build)
#include <algorithm>
#include <chrono>
#include <climits>
#include <vector>

#include "beam_search.h"
#include "graph_build.h"
#include "index_internal.h"

using coral::fail;

namespace coral {
void free_build_state(coral_index* idx) {
    (void)hipFree(idx->d_nbr_dists), (void)hipFree(idx->d_deg), (void)hipFree(idx->d_owner);
    (void)hipFree(idx->d_new_ids), (void)hipFree(idx->d_new_dists), (void)hipFree(idx->d_new_deg);
    (void)hipFree(idx->d_len), (void)hipFree(idx->d_build_stats), (void)hipFree(idx->d_hits);
    (void)hipFree(idx->d_top_ids_list), (void)hipFree(idx->d_top_dists_list), (void)hipFree(idx->d_rev_len);
    idx->d_nbr_dists = nullptr, idx->d_deg = nullptr, idx->d_owner = nullptr;
    idx->d_new_ids = nullptr, idx->d_new_dists = nullptr, idx->d_new_deg = nullptr;
    idx->d_len = nullptr, idx->d_build_stats = nullptr, idx->d_hits = nullptr;
    idx->d_top_ids_list = nullptr, idx->d_top_dists_list = nullptr, idx->d_rev_len = nullptr;
    idx->stage_rows = 0, idx->len_alloc = 0, idx->top_list_cells = 0, idx->rev_len_alloc = 0;
    idx->building = false;
}
}  // namespace coral

namespace {

double now_s() {
    return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// The sampling repeats an id once every node it can reach is taken (a linked part smaller than the number of
// entry points asked for); the search wants distinct start ids, so repeats are dropped here.
int set_start_ids(coral_index* idx, const int32_t* all_ids, int count) {
    std::vector<int32_t> uniq;
    for (int i = 0; i < count; ++i)
        if (std::find(uniq.begin(), uniq.end(), all_ids[i]) == uniq.end()) uniq.push_back(all_ids[i]);
    const int32_t* ids = uniq.data();
    const int M = (int)uniq.size();
    if (M != idx->M) {
        int32_t* p = nullptr;
        HIP_TRY(hipMalloc(&p, (size_t)M * sizeof(int32_t)));
        (void)hipFree(idx->d_start);
        idx->d_start = p;
        idx->M = M;
        idx->prepared = false;
        idx->noalloc_L = 0;  // (launch plans depend on the number of start ids)
    }
    HIP_TRY(hipMemcpyAsync(idx->d_start, ids, (size_t)M * sizeof(int32_t), hipMemcpyHostToDevice, idx->stream));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    return CORAL_OK;
}

// ids outside [0, n) would be followed into memory that is not there: count them before any kernel uses them
int check_ids(coral_index* idx, const int32_t* d_ids, int64_t count, bool minus_one_ok, const char* what) {
    HIP_TRY(coral::launch_fill_u32((uint32_t*)(idx->d_build_stats + 2), 2, 0u, idx->stream));
    HIP_TRY(coral::launch_count_bad_ids(d_ids, count, idx->n, minus_one_ok ? 1 : 0, idx->d_build_stats + 2, idx->stream));
    unsigned long long bad = 0;
    HIP_TRY(hipMemcpyAsync(&bad, idx->d_build_stats + 2, sizeof(bad), hipMemcpyDeviceToHost, idx->stream));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    if (bad) return fail(CORAL_ERR_GRAPH, "%llu of %lld %s are outside [0,%lld)", bad, (long long)count, what, (long long)idx->n);
    return CORAL_OK;
}

int ensure_stage(coral_index* idx, size_t rows) {
    if (rows <= idx->stage_rows) return CORAL_OK;
    (void)hipFree(idx->d_new_ids), (void)hipFree(idx->d_new_dists), (void)hipFree(idx->d_new_deg);
    idx->d_new_ids = nullptr, idx->d_new_dists = nullptr, idx->d_new_deg = nullptr, idx->stage_rows = 0;
    HIP_TRY(hipMalloc(&idx->d_new_ids, rows * idx->R * sizeof(int32_t)));
    HIP_TRY(hipMalloc(&idx->d_new_dists, rows * idx->R * sizeof(float)));
    HIP_TRY(hipMalloc(&idx->d_new_deg, rows * sizeof(int32_t)));
    idx->stage_rows = rows;
    return CORAL_OK;
}

// GPUFuncs::test_search (include/gpufuncs.cuh:688-702) on the graph as it stands: prepare for (Q, L), one search from
// the index's current start ids, the hit count against the true neighbours, and the caller's report.  With
// fresh_starts (the calls between batches, when the index has no entry points yet) the start ids are sampled first,
// as the enhancement does for its own searches; they are replaced again before the build ends.
int check_monitor(const coral_build_params* prm) {
    const coral_build_monitor* m = prm->monitor;
    if (!m || !m->report) return CORAL_OK;
    if (!m->h_queries || !m->h_gt || m->Q < 1 || m->k < 1 || m->k > m->L || m->L > CORAL_MAX_BEAM)
        return fail(CORAL_ERR_ARG, "build monitor: queries, true neighbours, Q >= 1 and 1 <= k <= L <= %d are needed",
                    CORAL_MAX_BEAM);
    if (prm->test_search_frequency < 0) return fail(CORAL_ERR_ARG, "test_search_frequency must not be negative");
    return CORAL_OK;
}

int monitor_search(coral_index* idx, const coral_build_params* prm, int32_t phase, int64_t done, int64_t total,
                   bool fresh_starts) {
    const coral_build_monitor* m = prm->monitor;
    if (!m || !m->report) return CORAL_OK;
    if (int rc = check_monitor(prm)) return rc;
    if (fresh_starts) {
        std::vector<int32_t> deg((size_t)idx->n), starts((size_t)prm->n_start);
        HIP_TRY(hipMemcpyAsync(deg.data(), idx->d_deg, (size_t)idx->n * sizeof(int32_t), hipMemcpyDeviceToHost, idx->stream));
        HIP_TRY(hipStreamSynchronize(idx->stream));
        int32_t first = prm->first_start_id;
        if (first < 0 || first >= idx->n || deg[first] == 0) {
            first = -1;
            for (int64_t i = 0; i < idx->n && first < 0; ++i)
                if (deg[i] > 0) first = (int32_t)i;
        }
        if (first < 0) return CORAL_OK;  // nothing to search from yet
        if (int rc = coral_start_ids_fps(idx, first, prm->n_start, starts.data())) return rc;
        if (int rc = set_start_ids(idx, starts.data(), prm->n_start)) return rc;
    }
    float* d_q = nullptr;
    int32_t *d_gt = nullptr, *d_res = nullptr;
    const size_t qb = (size_t)m->Q * idx->dim * sizeof(float), rb = (size_t)m->Q * m->k * sizeof(int32_t);
    int rc = CORAL_OK;
    if (hipMalloc(&d_q, qb) != hipSuccess || hipMalloc(&d_gt, rb) != hipSuccess || hipMalloc(&d_res, rb) != hipSuccess) {
        (void)hipGetLastError();
        rc = fail(CORAL_ERR_MEMORY, "build monitor: device allocation failed");
    } else if (hipMemcpy(d_q, m->h_queries, qb, hipMemcpyHostToDevice) != hipSuccess ||
               hipMemcpy(d_gt, m->h_gt, rb, hipMemcpyHostToDevice) != hipSuccess) {
        rc = fail(CORAL_ERR_DEVICE, "build monitor: upload failed");
    }
    coral_stats st{};
    int64_t hits = 0;
    coral_tuning tun{};
    tun.policy = CORAL_POLICY_ROUNDS;
    if (rc == CORAL_OK) rc = coral_search_prepare(idx, m->Q, m->L, &tun);
    if (rc == CORAL_OK) rc = coral_search_gpu(idx, d_q, d_res, nullptr, m->Q, m->k, CORAL_POLICY_ROUNDS, 0, nullptr, &st);
    if (rc == CORAL_OK) rc = coral_search_verify(idx, d_res, d_gt, m->Q, m->k, &hits);
    (void)hipFree(d_q), (void)hipFree(d_gt), (void)hipFree(d_res);
    if (rc == CORAL_OK) m->report(m->user, phase, done, total, &st, hits);
    return rc;
}

}  // namespace

extern "C" {

int coral_build_params_default(coral_build_params* p) {
    if (!p) return fail(CORAL_ERR_ARG, "null argument");
    *p = coral_build_params{};
    p->R = 32, p->k_b = 100, p->batch = 1024, p->need_discard = 1, p->connect_enhance = 1;
    p->enhance_search_batch = 524288, p->enhance_nap_batch = 4096, p->enhance_L = 256;
    p->n_start = 16, p->first_start_id = -1;
    p->test_search_frequency = 100;
    return CORAL_OK;
}

int coral_build_begin(coral_index* idx, int32_t R) {
    if (!idx) return fail(CORAL_ERR_ARG, "null index");
    if (R <= 0 || R > coral::kBuildMaxR) return fail(CORAL_ERR_ARG, "R must be in 1..%d (got %d)", coral::kBuildMaxR, R);
    if (idx->d_nbrs && idx->R != R)
        return fail(CORAL_ERR_ARG, "the index already holds rows of width %d (asked for %d)", idx->R, R);
    HIP_TRY(hipSetDevice(idx->device));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    coral::free_build_state(idx);
    const size_t n = (size_t)idx->n;
    if (!idx->d_nbrs) {
        HIP_TRY(hipMalloc(&idx->d_nbrs, n * R * sizeof(int32_t)));
        idx->R = R;
    }
    idx->prepared = false;
    idx->rows_unique = -1;
    HIP_TRY(hipMalloc(&idx->d_nbr_dists, n * R * sizeof(float)));
    HIP_TRY(hipMalloc(&idx->d_deg, n * sizeof(int32_t)));
    HIP_TRY(hipMalloc(&idx->d_owner, n * sizeof(int32_t)));
    HIP_TRY(hipMalloc(&idx->d_build_stats, 4 * sizeof(unsigned long long)));
    HIP_TRY(hipMalloc(&idx->d_hits, n * sizeof(uint32_t)));
    HIP_TRY(coral::launch_fill_u32(idx->d_hits, n, 0u, idx->stream));
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_nbrs, n * R, 0xffffffffu, idx->stream));
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_nbr_dists, n * R, 0u, idx->stream));
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_deg, n, 0u, idx->stream));
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_owner, n, (uint32_t)INT_MAX, idx->stream));
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_build_stats, 8, 0u, idx->stream));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    idx->building = true;
    return CORAL_OK;
}

int coral_build_end(coral_index* idx) {
    if (!idx) return fail(CORAL_ERR_ARG, "null index");
    HIP_TRY(hipSetDevice(idx->device));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    coral::free_build_state(idx);
    return CORAL_OK;
}

int coral_build_resume(coral_index* idx, int32_t R, const int32_t* h_nbrs, const float* h_dists,
                       const uint32_t* h_hits) {
    if (!idx || !h_nbrs || !h_dists) return fail(CORAL_ERR_ARG, "null argument");
    const int64_t n = idx->n;
    if (R <= 0 || R > coral::kBuildMaxR) return fail(CORAL_ERR_ARG, "R must be in 1..%d (got %d)", coral::kBuildMaxR, R);
    // a row is its first deg cells: every id in range, nothing after the first -1
    std::vector<int32_t> deg((size_t)n);
    int64_t bad = -1;
#pragma omp parallel for schedule(static) reduction(max : bad)
    for (int64_t i = 0; i < n; ++i) {
        const int32_t* row = h_nbrs + (size_t)i * R;
        int d = 0;
        while (d < R && row[d] >= 0) ++d;
        bool ok = true;
        for (int j = 0; j < R; ++j)
            if (j < d ? row[j] >= n : row[j] != -1) ok = false;
        deg[(size_t)i] = d;
        if (!ok) bad = std::max(bad, i);
    }
    if (bad >= 0)
        return fail(CORAL_ERR_GRAPH, "row %lld is not a row of a build (ids in range, -1 only at the end)",
                    (long long)bad);
    if (int rc = coral_build_begin(idx, R)) return rc;
    const size_t cells = (size_t)n * R;
    HIP_TRY(hipMemcpy(idx->d_nbrs, h_nbrs, cells * sizeof(int32_t), hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(idx->d_nbr_dists, h_dists, cells * sizeof(float), hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(idx->d_deg, deg.data(), (size_t)n * sizeof(int32_t), hipMemcpyHostToDevice));
    if (h_hits) HIP_TRY(hipMemcpy(idx->d_hits, h_hits, (size_t)n * sizeof(uint32_t), hipMemcpyHostToDevice));
    return CORAL_OK;
}

int coral_build_nap_batch(coral_index* idx, const int32_t* d_knn_ids, int32_t batch, int32_t k_b, int32_t need_discard) {
    if (!idx || !d_knn_ids) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->building) return fail(CORAL_ERR_STATE, "coral_build_begin has not been called");
    if (batch <= 0) return fail(CORAL_ERR_ARG, "batch must be positive");
    if (k_b < 2 || k_b > coral::kBuildMaxKb)
        return fail(CORAL_ERR_ARG, "k_b must be in 2..%d (got %d)", coral::kBuildMaxKb, k_b);
    if ((int64_t)batch * k_b > INT_MAX / 2) return fail(CORAL_ERR_ARG, "batch * k_b too large");
    HIP_TRY(hipSetDevice(idx->device));
    if (int rc = ensure_stage(idx, (size_t)batch * k_b)) return rc;
    if (int rc = check_ids(idx, d_knn_ids, (int64_t)batch * k_b, false, "cluster ids")) return rc;
    idx->rows_unique = -1;
    HIP_TRY(coral::launch_count_hits(d_knn_ids, (int64_t)batch * k_b, idx->d_hits, idx->stream));
    HIP_TRY(coral::launch_nap_batch(idx->d_vec, idx->dim, idx->metric, idx->R, idx->d_nbrs, idx->d_nbr_dists, idx->d_deg,
                                    idx->d_owner, d_knn_ids, batch, k_b, need_discard, idx->d_new_ids, idx->d_new_dists,
                                    idx->d_new_deg, idx->stream));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    return CORAL_OK;
}

// the common part of the two enhancement batches: lists [batch][kn], of which the first rev_len[b] (all, if null)
// insert reverse edges
static int enhance_lists(coral_index* idx, const int32_t* d_node_ids, const int32_t* d_ids, const float* d_dists,
                         int32_t batch, int32_t kn, const int32_t* d_rev_len, int64_t* reverse_edges,
                         int64_t* reverse_rejected) {
    if ((size_t)batch > idx->len_alloc) {
        (void)hipFree(idx->d_len);
        idx->d_len = nullptr, idx->len_alloc = 0;
        HIP_TRY(hipMalloc(&idx->d_len, (size_t)batch * sizeof(int32_t)));
        idx->len_alloc = (size_t)batch;
    }
    idx->rows_unique = -1;
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_build_stats, 4, 0u, idx->stream));
    HIP_TRY(coral::launch_enhance_batch(idx->d_vec, idx->dim, idx->metric, idx->R, idx->d_nbrs, idx->d_nbr_dists,
                                        idx->d_deg, idx->d_owner, d_node_ids, d_ids, d_dists, batch, kn, idx->d_len,
                                        d_rev_len, idx->d_build_stats, idx->stream));
    unsigned long long st[2] = {0, 0};
    HIP_TRY(hipMemcpyAsync(st, idx->d_build_stats, sizeof(st), hipMemcpyDeviceToHost, idx->stream));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    if (reverse_edges) *reverse_edges = (int64_t)st[0];
    if (reverse_rejected) *reverse_rejected = (int64_t)st[1];
    return CORAL_OK;
}

int coral_build_enhance_batch(coral_index* idx, const int32_t* d_iso_ids, const int32_t* d_knn_ids,
                              const float* d_knn_dists, int32_t batch, int32_t kn, int64_t* reverse_edges,
                              int64_t* reverse_rejected) {
    if (!idx || !d_iso_ids || !d_knn_ids || !d_knn_dists) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->building) return fail(CORAL_ERR_STATE, "coral_build_begin has not been called");
    if (batch <= 0) return fail(CORAL_ERR_ARG, "batch must be positive");
    if (kn < 1 || kn > coral::kBuildMaxKb + coral::kBuildMaxR)
        return fail(CORAL_ERR_ARG, "found-list length must be in 1..%d (got %d)", coral::kBuildMaxKb + coral::kBuildMaxR, kn);
    if ((int64_t)batch * kn > INT_MAX / 2) return fail(CORAL_ERR_ARG, "batch * list length too large");
    HIP_TRY(hipSetDevice(idx->device));
    if (int rc = check_ids(idx, d_iso_ids, batch, false, "isolated ids")) return rc;
    if (int rc = check_ids(idx, d_knn_ids, (int64_t)batch * kn, true, "found ids")) return rc;
    return enhance_lists(idx, d_iso_ids, d_knn_ids, d_knn_dists, batch, kn, nullptr, reverse_edges, reverse_rejected);
}

int coral_build_enhance_top_batch(coral_index* idx, const int32_t* d_top_ids, const int32_t* d_knn_ids,
                                  const float* d_knn_dists, int32_t batch, int32_t k, int64_t* reverse_edges,
                                  int64_t* reverse_rejected) {
    if (!idx || !d_top_ids || !d_knn_ids || !d_knn_dists) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->building) return fail(CORAL_ERR_STATE, "coral_build_begin has not been called");
    if (batch <= 0) return fail(CORAL_ERR_ARG, "batch must be positive");
    if (k < 1 || k > coral::kBuildMaxKb) return fail(CORAL_ERR_ARG, "found-list length must be in 1..%d (got %d)", coral::kBuildMaxKb, k);
    const int kn = k + idx->R;
    if ((int64_t)batch * kn > INT_MAX / 2) return fail(CORAL_ERR_ARG, "batch * list length too large");
    HIP_TRY(hipSetDevice(idx->device));
    if (int rc = check_ids(idx, d_top_ids, batch, false, "node ids")) return rc;
    if (int rc = check_ids(idx, d_knn_ids, (int64_t)batch * k, true, "found ids")) return rc;
    const size_t cells = (size_t)batch * kn;
    if (cells > idx->top_list_cells) {
        (void)hipFree(idx->d_top_ids_list), (void)hipFree(idx->d_top_dists_list);
        idx->d_top_ids_list = nullptr, idx->d_top_dists_list = nullptr, idx->top_list_cells = 0;
        HIP_TRY(hipMalloc(&idx->d_top_ids_list, cells * sizeof(int32_t)));
        HIP_TRY(hipMalloc(&idx->d_top_dists_list, cells * sizeof(float)));
        idx->top_list_cells = cells;
    }
    if ((size_t)batch > idx->rev_len_alloc) {
        (void)hipFree(idx->d_rev_len);
        idx->d_rev_len = nullptr, idx->rev_len_alloc = 0;
        HIP_TRY(hipMalloc(&idx->d_rev_len, (size_t)batch * sizeof(int32_t)));
        idx->rev_len_alloc = (size_t)batch;
    }
    HIP_TRY(coral::launch_enhance_top_lists(idx->R, idx->d_nbrs, idx->d_nbr_dists, idx->d_deg, d_top_ids, d_knn_ids,
                                            d_knn_dists, batch, k, idx->d_top_ids_list, idx->d_top_dists_list,
                                            idx->d_rev_len, idx->stream));
    return enhance_lists(idx, d_top_ids, idx->d_top_ids_list, idx->d_top_dists_list, batch, kn, idx->d_rev_len,
                         reverse_edges, reverse_rejected);
}

int coral_build_top_hit_ids(coral_index* idx, int64_t top_n, int32_t* h_ids, uint32_t* h_hits) {
    if (!idx || (!h_ids && !h_hits)) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->building) return fail(CORAL_ERR_STATE, "coral_build_begin has not been called");
    if (top_n < 0 || top_n > idx->n) return fail(CORAL_ERR_ARG, "top_n must be in 0..n");
    HIP_TRY(hipSetDevice(idx->device));
    std::vector<uint32_t> local;
    uint32_t* hits = h_hits;
    if (!hits) {
        local.resize((size_t)idx->n);
        hits = local.data();
    }
    HIP_TRY(hipMemcpyAsync(hits, idx->d_hits, (size_t)idx->n * sizeof(uint32_t), hipMemcpyDeviceToHost, idx->stream));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    if (!h_ids || top_n == 0) return CORAL_OK;
    // counting sort, most hits first, ids ascending within a count
    uint32_t mx = 0;
    for (int64_t i = 0; i < idx->n; ++i) mx = std::max(mx, hits[i]);
    std::vector<int64_t> at((size_t)mx + 2, 0);  // at[h] = ids with more than h hits = where count h starts
    for (int64_t i = 0; i < idx->n; ++i) ++at[hits[i]];
    int64_t run = 0;
    for (int64_t h = mx; h >= 0; --h) {
        const int64_t c = at[(size_t)h];
        at[(size_t)h] = run;
        run += c;
    }
    for (int64_t i = 0; i < idx->n; ++i) {
        const int64_t pos = at[hits[i]]++;
        if (pos < top_n) h_ids[pos] = (int32_t)i;
    }
    return CORAL_OK;
}

int coral_build_connect_enhance(coral_index* idx, const coral_build_params* prm, coral_build_stats* stats) {
    if (!idx || !prm) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->building) return fail(CORAL_ERR_STATE, "coral_build_begin has not been called");
    if (prm->k_b < 1 || prm->k_b > prm->enhance_L) return fail(CORAL_ERR_ARG, "k_b must be in 1..enhance_L");
    if (prm->n_start < 1 || prm->enhance_search_batch < 1 || prm->enhance_nap_batch < 1)
        return fail(CORAL_ERR_ARG, "n_start and the enhancement batch sizes must be positive");
    if (int rc = check_monitor(prm)) return rc;
    HIP_TRY(hipSetDevice(idx->device));
    hipStream_t st = idx->stream;
    const int64_t n = idx->n;
    const int dim = idx->dim, kb = prm->k_b;
    // load_isolated_nodes (src/enhance.cu:577-611): ids without neighbours, ascending
    std::vector<int32_t> deg((size_t)n);
    HIP_TRY(hipMemcpyAsync(deg.data(), idx->d_deg, (size_t)n * sizeof(int32_t), hipMemcpyDeviceToHost, st));
    HIP_TRY(hipStreamSynchronize(st));
    std::vector<int32_t> iso;
    int32_t first = prm->first_start_id;
    for (int64_t i = 0; i < n; ++i) {
        if (deg[i] == 0)
            iso.push_back((int32_t)i);
        else if (first < 0)
            first = (int32_t)i;
    }
    if (stats) stats->isolated = (int64_t)iso.size();
    if (first < 0 || first >= n) return fail(CORAL_ERR_STATE, "no node has neighbours yet: nothing to search from");
    if (deg[first] == 0) return fail(CORAL_ERR_ARG, "first_start_id %d has no neighbours", first);
    std::vector<int32_t> starts((size_t)prm->n_start);
    const int64_t iso_num = (int64_t)iso.size();
    int rc = CORAL_OK;
    // One phase: per search batch fresh entry points on the graph as it is now (src/enhance.cu:793-795, 843), one
    // search for the nodes' own vectors, then the rewiring per enhance_nap_batch nodes.
    auto phase = [&](const std::vector<int32_t>& ids, bool top) {
        const int64_t count = (int64_t)ids.size();
        const int64_t sb = std::min<int64_t>(prm->enhance_search_batch, count);
        int32_t *d_ids = nullptr, *d_res = nullptr;
        float *d_vecs = nullptr, *d_res_d = nullptr;
        auto ok = [&](hipError_t e, const char* what) {
            if (e == hipSuccess) return true;
            rc = fail(e == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE, "%s failed: %s", what,
                      hipGetErrorString(e));
            return false;
        };
        if (ok(hipMalloc(&d_ids, (size_t)count * sizeof(int32_t)), "hipMalloc") &&
            ok(hipMalloc(&d_vecs, (size_t)sb * dim * sizeof(float)), "hipMalloc") &&
            ok(hipMalloc(&d_res, (size_t)sb * kb * sizeof(int32_t)), "hipMalloc") &&
            ok(hipMalloc(&d_res_d, (size_t)sb * kb * sizeof(float)), "hipMalloc"))
            ok(hipMemcpy(d_ids, ids.data(), (size_t)count * sizeof(int32_t), hipMemcpyHostToDevice), "hipMemcpy");
        for (int64_t i = 0; rc == CORAL_OK && i < count; i += sb) {
            const int batch = (int)std::min<int64_t>(sb, count - i);
            if ((rc = coral_start_ids_fps(idx, first, prm->n_start, starts.data()))) break;
            if ((rc = set_start_ids(idx, starts.data(), prm->n_start))) break;
            if (!ok(coral::launch_gather_rows(idx->d_vec, dim, d_ids + i, batch, d_vecs, st), "gather")) break;
            coral_tuning tun{};
            tun.policy = CORAL_POLICY_ROUNDS;
            if ((rc = coral_search_prepare(idx, batch, prm->enhance_L, &tun))) break;
            if ((rc = coral_search_gpu(idx, d_vecs, d_res, d_res_d, batch, kb, CORAL_POLICY_ROUNDS, 0, nullptr, nullptr)))
                break;
            for (int64_t j = 0; j < batch; j += prm->enhance_nap_batch) {
                const int b1 = (int)std::min<int64_t>(prm->enhance_nap_batch, batch - j);
                int64_t ins = 0, rej = 0;
                rc = top ? coral_build_enhance_top_batch(idx, d_ids + i + j, d_res + (size_t)j * kb, d_res_d + (size_t)j * kb,
                                                         b1, kb, &ins, &rej)
                         : coral_build_enhance_batch(idx, d_ids + i + j, d_res + (size_t)j * kb, d_res_d + (size_t)j * kb, b1,
                                                     kb, &ins, &rej);
                if (rc) break;
                if (stats && top) stats->top_reverse_edges += ins;
                if (stats && !top) stats->reverse_edges += ins, stats->reverse_rejected += rej;
            }
            if (rc == CORAL_OK && top) rc = monitor_search(idx, prm, CORAL_MONITOR_TOP, i + batch, count, false);
        }
        (void)hipFree(d_ids), (void)hipFree(d_res), (void)hipFree(d_vecs), (void)hipFree(d_res_d);
    };
    if (iso_num > 0) phase(iso, false);
    if (rc == CORAL_OK && iso_num > 0) rc = monitor_search(idx, prm, CORAL_MONITOR_ISOLATED, iso_num, iso_num, false);
    // src/enhance.cu:819-856: the nodes most clusters contain, as many as top_hit_num exceeds the isolated ones
    int64_t top_n = rc == CORAL_OK && prm->top_hit_num > iso_num ? std::min<int64_t>(prm->top_hit_num - iso_num, n) : 0;
    if (top_n > 0) {
        if (prm->k_b > coral::kBuildMaxKb) return fail(CORAL_ERR_ARG, "k_b must be at most %d", coral::kBuildMaxKb);
        std::vector<int32_t> top((size_t)top_n);
        if ((rc = coral_build_top_hit_ids(idx, top_n, top.data(), nullptr))) return rc;
        if (stats) stats->top_hit_nodes = top_n;
        phase(top, true);
    }
    if (rc == CORAL_OK && iso_num == 0 && top_n == 0) {
        if ((rc = coral_start_ids_fps(idx, first, prm->n_start, starts.data()))) return rc;
        rc = set_start_ids(idx, starts.data(), prm->n_start);
    }
    return rc;
}

int coral_build_test_search(coral_index* idx, const coral_build_params* prm, int32_t phase, int64_t done, int64_t total) {
    if (!idx || !prm) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->d_nbrs || idx->M < 1) return fail(CORAL_ERR_STATE, "the index has no graph or no start ids to search from");
    HIP_TRY(hipSetDevice(idx->device));
    return monitor_search(idx, prm, phase, done, total, false);
}

// the construction from auxiliary queries (h_aux) or from their precomputed clusters (h_clusters)
static int build_impl(coral_index* idx, const float* h_aux, const int32_t* h_clusters, int64_t A,
                      const coral_build_params* prm, coral_build_stats* stats) {
    if (!idx || (!h_aux && !h_clusters) || !prm) return fail(CORAL_ERR_ARG, "null argument");
    if (A <= 0) return fail(CORAL_ERR_ARG, "no auxiliary queries");
    if (prm->batch <= 0) return fail(CORAL_ERR_ARG, "batch must be positive");
    if (prm->k_b > idx->n) return fail(CORAL_ERR_ARG, "k_b exceeds the number of base vectors");
    if (int rc = check_monitor(prm)) return rc;
    coral_build_stats local{};
    coral_build_stats* S = stats ? stats : &local;
    *S = coral_build_stats{};
    const double t0 = now_s();
    if (int rc = coral_build_begin(idx, prm->R)) return rc;
    HIP_TRY(hipSetDevice(idx->device));
    const int dim = idx->dim, kb = prm->k_b;
    // the exact k_b-NN of a chunk of auxiliary queries at a time (KNNTask), then its batches in order (GraphTask)
    const int64_t chunk = std::min<int64_t>(A, (int64_t)prm->batch * 16);
    float* d_aux = nullptr;
    int32_t* d_knn = nullptr;
    int rc = CORAL_OK;
    if ((h_aux && hipMalloc(&d_aux, (size_t)chunk * dim * sizeof(float)) != hipSuccess) ||
        hipMalloc(&d_knn, (size_t)chunk * kb * sizeof(int32_t)) != hipSuccess)
        rc = fail(CORAL_ERR_MEMORY, "device allocation for the auxiliary queries failed");
    for (int64_t a0 = 0; rc == CORAL_OK && a0 < A; a0 += chunk) {
        const int64_t cq = std::min(chunk, A - a0);
        if (h_clusters) {  // GraphTask's train_gt_file branch, src/index_gpu.cpp:505-524
            if (hipMemcpy(d_knn, h_clusters + (size_t)a0 * kb, (size_t)cq * kb * sizeof(int32_t), hipMemcpyHostToDevice) !=
                hipSuccess) {
                rc = fail(CORAL_ERR_DEVICE, "upload of clusters failed");
                break;
            }
        } else {
            if (hipMemcpy(d_aux, h_aux + (size_t)a0 * dim, (size_t)cq * dim * sizeof(float), hipMemcpyHostToDevice) !=
                hipSuccess) {
                rc = fail(CORAL_ERR_DEVICE, "upload of auxiliary queries failed");
                break;
            }
            double t = 0.0;
            if ((rc = coral_bruteforce_knn_gpu(idx, d_aux, (int32_t)cq, kb, 0, d_knn, nullptr, nullptr, &t))) break;
            S->knn_s += t;
        }
        const double t1 = now_s();
        for (int64_t b0 = 0; b0 < cq; b0 += prm->batch) {
            const int b = (int)std::min<int64_t>(prm->batch, cq - b0);
            if ((rc = coral_build_nap_batch(idx, d_knn + (size_t)b0 * kb, b, kb, prm->need_discard))) break;
            const int64_t batch_id = S->batches++;
            if (prm->monitor && prm->test_search_frequency > 0 && batch_id > 0 &&
                batch_id % prm->test_search_frequency == 0 &&
                (rc = monitor_search(idx, prm, CORAL_MONITOR_BATCHES, a0 + b0 + b, A, true)))
                break;
        }
        S->nap_s += now_s() - t1;
    }
    (void)hipFree(d_aux), (void)hipFree(d_knn);
    if (rc) return rc;
    const double t2 = now_s();
    if (prm->connect_enhance) {
        if ((rc = coral_build_connect_enhance(idx, prm, S))) return rc;
    } else {
        std::vector<int32_t> deg((size_t)idx->n), starts((size_t)prm->n_start);
        HIP_TRY(hipMemcpy(deg.data(), idx->d_deg, (size_t)idx->n * sizeof(int32_t), hipMemcpyDeviceToHost));
        int32_t first = prm->first_start_id;
        int64_t isolated = 0;
        for (int64_t i = 0; i < idx->n; ++i) {
            isolated += deg[i] == 0;
            if (first < 0 && deg[i] > 0) first = (int32_t)i;
        }
        S->isolated = isolated;
        if (first < 0) return fail(CORAL_ERR_STATE, "no node has neighbours");
        if ((rc = coral_start_ids_fps(idx, first, prm->n_start, starts.data()))) return rc;
        if ((rc = set_start_ids(idx, starts.data(), prm->n_start))) return rc;
    }
    S->enhance_s = now_s() - t2;
    if (prm->connect_enhance && (rc = monitor_search(idx, prm, CORAL_MONITOR_DONE, A, A, false))) return rc;
    std::vector<int32_t> deg((size_t)idx->n);
    HIP_TRY(hipMemcpy(deg.data(), idx->d_deg, (size_t)idx->n * sizeof(int32_t), hipMemcpyDeviceToHost));
    for (int32_t d : deg) S->edges += d;
    S->total_s = now_s() - t0;
    return CORAL_OK;
}

int coral_build_graph(coral_index* idx, const float* h_aux, int64_t A, const coral_build_params* prm,
                      coral_build_stats* stats) {
    if (!h_aux) return fail(CORAL_ERR_ARG, "null argument");
    return build_impl(idx, h_aux, nullptr, A, prm, stats);
}

int coral_build_graph_from_clusters(coral_index* idx, const int32_t* h_clusters, int64_t A, const coral_build_params* prm,
                                    coral_build_stats* stats) {
    if (!h_clusters) return fail(CORAL_ERR_ARG, "null argument");
    return build_impl(idx, nullptr, h_clusters, A, prm, stats);
}

int coral_index_get_graph(coral_index* idx, int32_t* h_nbrs, float* h_dists, int32_t* h_deg, int32_t* h_start_ids) {
    if (!idx) return fail(CORAL_ERR_ARG, "null index");
    if (!idx->d_nbrs) return fail(CORAL_ERR_STATE, "the index holds vectors only (no graph was given or built)");
    if ((h_dists || h_deg) && !idx->building)
        return fail(CORAL_ERR_STATE, "distances and degrees exist only between coral_build_begin and coral_build_end");
    HIP_TRY(hipSetDevice(idx->device));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    const size_t cells = (size_t)idx->n * idx->R;
    if (h_nbrs) HIP_TRY(hipMemcpy(h_nbrs, idx->d_nbrs, cells * sizeof(int32_t), hipMemcpyDeviceToHost));
    if (h_dists) HIP_TRY(hipMemcpy(h_dists, idx->d_nbr_dists, cells * sizeof(float), hipMemcpyDeviceToHost));
    if (h_deg) HIP_TRY(hipMemcpy(h_deg, idx->d_deg, (size_t)idx->n * sizeof(int32_t), hipMemcpyDeviceToHost));
    if (h_start_ids && idx->M > 0)
        HIP_TRY(hipMemcpy(h_start_ids, idx->d_start, (size_t)idx->M * sizeof(int32_t), hipMemcpyDeviceToHost));
    return CORAL_OK;
}

}  // extern "C"
