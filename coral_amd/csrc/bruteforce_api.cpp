// bruteforce_api.cpp -- coral_bruteforce_knn*: exact k nearest neighbours of a batch of
// queries among the index's resident vectors (kernels in bruteforce.hip, bruteforce_mfma.hip).
#include <algorithm>
#include <cstring>
#include <vector>

#include "beam_search.h"
#include "bruteforce.h"
#include "graph_build.h"
#include "index_internal.h"

using coral::fail;

namespace {
constexpr int64_t kSegment = (int64_t)1 << 22;   // base points per pass
constexpr int64_t kBufferFloats = (int64_t)1 << 29;  // 2 GiB distance buffer

// the passes over the base: distances of a block of queries to a segment of the base into D, the k best of every row
// of D, and at the end the k best of the per-segment winners.  screen: approximate distances from the matrix cores
// (qn, bn: squared norms) instead of the reference-order ones.
int knn_passes(coral_index* idx, const float* d_queries, int32_t Q, int32_t k, int32_t have_delete, bool screen,
               const float* d_qn, int metric_out, int32_t* d_ids, float* d_dists, hipStream_t stream) {
    const int64_t n = idx->n;
    int64_t seg = std::min(n, kSegment);
    int64_t nseg = (n + seg - 1) / seg;
    while (nseg * k > 8192) {  // the final merge sorts nseg*k keys in LDS
        seg *= 2;
        nseg = (n + seg - 1) / seg;
    }
    const int64_t ld = (seg + 3) & ~(int64_t)3;
    int64_t qc = std::max<int64_t>(128, (kBufferFloats / ld) & ~(int64_t)127);
    qc = std::min<int64_t>(qc, ((int64_t)Q + 127) & ~(int64_t)127);
    float* D = nullptr;
    unsigned long long* part = nullptr;
    int* redo = nullptr;
    auto release = [&]() {
        (void)hipFree(D);
        (void)hipFree(part);
        (void)hipFree(redo);
    };
#define HIP_TRY_R(expr)                                                                  \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess) {                                                          \
            release();                                                                   \
            return fail(e_ == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE, \
                        "%s failed: %s", #expr, hipGetErrorString(e_));                  \
        }                                                                                \
    } while (0)
    HIP_TRY_R(hipMalloc(&D, (size_t)qc * ld * sizeof(float)));
    HIP_TRY_R(hipMalloc(&part, (size_t)Q * nseg * k * sizeof(unsigned long long)));
    HIP_TRY_R(hipMalloc(&redo, (size_t)qc * sizeof(int)));
    for (int64_t q0 = 0; q0 < Q; q0 += qc) {
        const int nq = (int)std::min<int64_t>(qc, Q - q0);
        for (int64_t s = 0; s < nseg; ++s) {
            const int64_t b0 = s * seg, nb = std::min(seg, n - b0);
            const float* qp = d_queries + (size_t)q0 * idx->dim;
            const float* bp = idx->d_vec + (size_t)b0 * idx->dim;
            const uint32_t* del = have_delete ? idx->d_deleted : nullptr;
            if (screen)
                HIP_TRY_R(coral::launch_approx_tile(qp, bp, nq, nb, idx->dim, idx->metric, d_qn + q0, idx->d_bnorm + b0, del,
                                                    b0, D, ld, stream));
            else
                HIP_TRY_R(coral::launch_distance_tile(qp, bp, nq, nb, idx->dim, idx->metric, del, b0, D, ld, stream));
            HIP_TRY_R(coral::launch_row_select(D, ld, nq, nb, k, b0, part + ((size_t)q0 * nseg + s) * k, nseg * k, redo,
                                               stream));
        }
    }
    HIP_TRY_R(coral::launch_merge_segments(part, Q, (int)nseg, k, metric_out, d_ids, d_dists, stream));
    HIP_TRY_R(hipStreamSynchronize(stream));
#undef HIP_TRY_R
    release();
    return CORAL_OK;
}

// |b|^2 of the base, once per index
int ensure_base_norms(coral_index* idx, hipStream_t stream) {
    if (idx->d_bnorm) return CORAL_OK;
    if (!idx->d_bnorm_max) HIP_TRY(hipMalloc(&idx->d_bnorm_max, sizeof(uint32_t)));
    float* norms = nullptr;
    HIP_TRY(hipMalloc(&norms, (size_t)idx->n * sizeof(float)));
    hipError_t e = coral::launch_fill_u32(idx->d_bnorm_max, 1, 0u, stream);
    if (e == hipSuccess) e = coral::launch_row_norms(idx->d_vec, idx->n, idx->dim, norms, idx->d_bnorm_max, stream);
    if (e != hipSuccess) {
        (void)hipFree(norms);
        HIP_TRY(e);
    }
    idx->d_bnorm = norms;  // kept only once its kernel is on the stream
    return CORAL_OK;
}

constexpr int kScreenSlack = 32;  // candidates kept beyond k
constexpr int64_t kListCap = 16384;  // keys a query's candidate list holds in the fused screening

// The screening with the selection inside the matrix-core kernel: no distance matrix goes to memory.  Per block of
// queries: (1) the distances to a sample of the base (every stride-th tile of 128 points) as a small matrix, whose
// kc-th smallest entry per row is a bound tau[q] that at least kc entries of the whole row do not exceed; (2) one
// pass over the whole base that appends the entries up to tau[q] to the query's list (about kc * n / sample of
// them); (3) the kc smallest keys of every list.  The kept candidates are those of knn_passes(screen = true): the
// same approximate values, the kc smallest under (value, id).  *used = false when the shape does not suit (kc beyond
// what list_select_kernel takes, a base too small to sample) or a list overflowed (sample unlike the base, rows of
// equal values, too few live points in the sample): the caller then goes through the matrix.
int knn_screen_fused(coral_index* idx, const float* d_queries, int32_t Q, int32_t kc, int32_t have_delete,
                     const float* d_qn, int32_t* d_cid, float* d_cd, hipStream_t stream, bool* used) {
    *used = false;
    const int64_t n = idx->n, full_tiles = n / 128;
    int64_t tiles = (2 * (int64_t)kc * full_tiles + kListCap - 1) / kListCap;
    tiles = std::max<int64_t>(8, (tiles + 7) & ~(int64_t)7);
    if (kc > 1024 || tiles * 8 > full_tiles || n > 0x7fffffff) return CORAL_OK;
    const int64_t stride = full_tiles / tiles, ns = tiles * 128;
    int64_t qc = std::min<int64_t>(kListCap, (kBufferFloats / ns) & ~(int64_t)127);
    qc = std::min<int64_t>(qc, ((int64_t)Q + 127) & ~(int64_t)127);
    float *D = nullptr, *tau = nullptr;
    unsigned long long *keys = nullptr, *lists = nullptr;
    unsigned int* cnt = nullptr;
    int *redo = nullptr, *overflow = nullptr;
    auto release = [&]() {
        (void)hipFree(D), (void)hipFree(tau), (void)hipFree(keys), (void)hipFree(lists);
        (void)hipFree(cnt), (void)hipFree(redo), (void)hipFree(overflow);
    };
#define HIP_TRY_R(expr)                                                                  \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess) {                                                          \
            release();                                                                   \
            return fail(e_ == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE, \
                        "%s failed: %s", #expr, hipGetErrorString(e_));                  \
        }                                                                                \
    } while (0)
    HIP_TRY_R(hipMalloc(&D, (size_t)qc * ns * sizeof(float)));
    HIP_TRY_R(hipMalloc(&tau, (size_t)qc * sizeof(float)));
    HIP_TRY_R(hipMalloc(&keys, (size_t)qc * kc * sizeof(unsigned long long)));
    HIP_TRY_R(hipMalloc(&lists, (size_t)qc * kListCap * sizeof(unsigned long long)));
    HIP_TRY_R(hipMalloc(&cnt, (size_t)qc * sizeof(unsigned int)));
    HIP_TRY_R(hipMalloc(&redo, (size_t)qc * sizeof(int)));
    HIP_TRY_R(hipMalloc(&overflow, sizeof(int)));
    HIP_TRY_R(coral::launch_fill_u32(reinterpret_cast<uint32_t*>(overflow), 1, 0u, stream));
    const uint32_t* del = have_delete ? idx->d_deleted : nullptr;
    for (int64_t q0 = 0; q0 < Q; q0 += qc) {
        const int nq = (int)std::min<int64_t>(qc, Q - q0);
        const float* qp = d_queries + (size_t)q0 * idx->dim;
        HIP_TRY_R(coral::launch_approx_tile(qp, idx->d_vec, nq, n, idx->dim, idx->metric, d_qn + q0, idx->d_bnorm, del, 0, D,
                                            ns, stream, tiles, stride));
        HIP_TRY_R(coral::launch_row_select(D, ns, nq, ns, kc, 0, keys, kc, redo, stream));
        HIP_TRY_R(coral::launch_bound_from_keys(keys, kc, kc - 1, nq, tau, stream));
        HIP_TRY_R(coral::launch_fill_u32(cnt, (size_t)nq, 0u, stream));
        HIP_TRY_R(coral::launch_approx_filter(qp, idx->d_vec, nq, n, idx->dim, idx->metric, d_qn + q0, idx->d_bnorm, del, tau,
                                              lists, kListCap, cnt, stream));
        HIP_TRY_R(coral::launch_list_select(lists, kListCap, cnt, nq, kc, keys, kc, overflow, stream));
        HIP_TRY_R(coral::launch_merge_segments(keys, nq, 1, kc, /*signed distances*/ 0, d_cid + (size_t)q0 * kc,
                                               d_cd + (size_t)q0 * kc, stream));
    }
    int lost = 0;
    HIP_TRY_R(hipMemcpyAsync(&lost, overflow, sizeof(int), hipMemcpyDeviceToHost, stream));
    HIP_TRY_R(hipStreamSynchronize(stream));
#undef HIP_TRY_R
    release();
    *used = lost == 0;
    return CORAL_OK;
}

}  // namespace

extern "C" {

int coral_bruteforce_set_exact_only(coral_index* idx, int32_t on) {
    if (!idx) return fail(CORAL_ERR_ARG, "null index");
    if (on < 0 || on > 2) return fail(CORAL_ERR_ARG, "on must be 0, 1 or 2 (got %d)", on);
    idx->knn_mode = on;
    return CORAL_OK;
}

int64_t coral_bruteforce_last_redone(coral_index* idx) { return idx ? idx->knn_last_redone : -1; }

int32_t coral_bruteforce_last_fused(coral_index* idx) { return idx ? (int32_t)idx->knn_last_fused : -1; }

int coral_bruteforce_knn_gpu(coral_index* idx, const float* d_queries, int32_t Q, int32_t k,
                             int32_t have_delete, int32_t* d_ids, float* d_dists, void* stream_,
                             double* time_s) {
    if (!idx || !d_queries || !d_ids) return fail(CORAL_ERR_ARG, "null argument");
    if (Q <= 0) return fail(CORAL_ERR_ARG, "Q must be positive");
    if (k <= 0 || k > 2048) return fail(CORAL_ERR_ARG, "k must be in 1..2048 (got %d)", k);
    if (have_delete && !idx->d_deleted)
        return fail(CORAL_ERR_STATE, "have_delete set but no tombstone mask was given");
    HIP_TRY(hipSetDevice(idx->device));
    hipStream_t stream = stream_ ? (hipStream_t)stream_ : idx->stream;
    hipEvent_t ev0, ev1;
    HIP_TRY(hipEventCreate(&ev0));
    HIP_TRY(hipEventCreate(&ev1));
    HIP_TRY(hipEventRecord(ev0, stream));
    int rc = CORAL_OK;
    const int kc = k + kScreenSlack;
    idx->knn_last_redone = 0;
    idx->knn_last_fused = false;
    if (idx->knn_mode == 1 || kc > 2048 || idx->n <= kc) {
        rc = knn_passes(idx, d_queries, Q, k, have_delete, false, nullptr, idx->metric, d_ids, d_dists, stream);
    } else {
        // screening on the matrix cores, exact distances for the kc candidates of each query, the exact passes for
        // the queries whose candidates cannot vouch for the result (bruteforce_mfma.hip)
        float *d_qn = nullptr, *d_cd = nullptr, *d_rq = nullptr, *d_rd = nullptr;
        int32_t *d_cid = nullptr, *d_rows = nullptr, *d_rid = nullptr;
        int* d_redo = nullptr;
        std::vector<int> redo((size_t)Q);
        std::vector<int32_t> rows;
        auto release = [&]() {
            (void)hipFree(d_qn), (void)hipFree(d_cd), (void)hipFree(d_cid), (void)hipFree(d_redo);
            (void)hipFree(d_rows), (void)hipFree(d_rq), (void)hipFree(d_rid), (void)hipFree(d_rd);
        };
        auto ok = [&](hipError_t e, const char* what) {
            if (e == hipSuccess) return true;
            rc = fail(e == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE, "%s failed: %s", what,
                      hipGetErrorString(e));
            return false;
        };
        if ((rc = ensure_base_norms(idx, stream)) == CORAL_OK &&
            ok(hipMalloc(&d_qn, (size_t)Q * sizeof(float)), "hipMalloc") &&
            ok(hipMalloc(&d_cid, (size_t)Q * kc * sizeof(int32_t)), "hipMalloc") &&
            ok(hipMalloc(&d_cd, (size_t)Q * kc * sizeof(float)), "hipMalloc") &&
            ok(hipMalloc(&d_redo, (size_t)Q * sizeof(int)), "hipMalloc") &&
            ok(coral::launch_row_norms(d_queries, Q, idx->dim, d_qn, nullptr, stream), "query norms")) {
            bool fused = false;
            if (idx->knn_mode == 0)
                rc = knn_screen_fused(idx, d_queries, Q, kc, have_delete, d_qn, d_cid, d_cd, stream, &fused);
            idx->knn_last_fused = fused;
            if (rc == CORAL_OK && !fused)
                rc = knn_passes(idx, d_queries, Q, kc, have_delete, true, d_qn, /*signed distances*/ 0, d_cid, d_cd, stream);
        }
        if (rc == CORAL_OK &&
            ok(coral::launch_rerank(d_queries, idx->d_vec, Q, idx->dim, idx->metric, d_cid, d_cd, kc, k, d_qn,
                                    idx->d_bnorm_max, d_ids, d_dists, d_redo, stream), "rerank") &&
            ok(hipMemcpyAsync(redo.data(), d_redo, (size_t)Q * sizeof(int), hipMemcpyDeviceToHost, stream), "hipMemcpy") &&
            ok(hipStreamSynchronize(stream), "synchronize")) {
            for (int32_t q = 0; q < Q; ++q)
                if (redo[(size_t)q]) rows.push_back(q);
        }
        if (rc == CORAL_OK && !rows.empty()) {
            const int m = (int)rows.size();
            if (ok(hipMalloc(&d_rows, (size_t)m * sizeof(int32_t)), "hipMalloc") &&
                ok(hipMalloc(&d_rq, (size_t)m * idx->dim * sizeof(float)), "hipMalloc") &&
                ok(hipMalloc(&d_rid, (size_t)m * k * sizeof(int32_t)), "hipMalloc") &&
                ok(hipMalloc(&d_rd, (size_t)m * k * sizeof(float)), "hipMalloc") &&
                ok(hipMemcpyAsync(d_rows, rows.data(), (size_t)m * sizeof(int32_t), hipMemcpyHostToDevice, stream), "hipMemcpy") &&
                ok(coral::launch_gather_rows(d_queries, idx->dim, d_rows, m, d_rq, stream), "gather"))
                rc = knn_passes(idx, d_rq, m, k, have_delete, false, nullptr, idx->metric, d_rid, d_rd, stream);
            if (rc == CORAL_OK &&
                ok(coral::launch_scatter_results(d_rows, m, k, d_rid, d_rd, d_ids, d_dists, stream), "scatter"))
                ok(hipStreamSynchronize(stream), "synchronize");
        }
        idx->knn_last_redone = (int64_t)rows.size();
        release();
    }
    if (rc == CORAL_OK) {
        HIP_TRY(hipEventRecord(ev1, stream));
        HIP_TRY(hipEventSynchronize(ev1));
        float ms = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms, ev0, ev1));
        if (time_s) *time_s = ms / 1000.0;
    }
    (void)hipEventDestroy(ev0);
    (void)hipEventDestroy(ev1);
    return rc;
}

int coral_bruteforce_knn(coral_index* idx, const float* h_queries, int32_t Q, int32_t k, int32_t have_delete,
                         int32_t* h_ids, float* h_dists, double* time_s) {
    if (!idx || !h_queries || !h_ids) return fail(CORAL_ERR_ARG, "null argument");
    if (Q <= 0 || k <= 0) return fail(CORAL_ERR_ARG, "Q and k must be positive");
    HIP_TRY(hipSetDevice(idx->device));
    float* d_q = nullptr;
    int32_t* d_ids = nullptr;
    float* d_d = nullptr;
    const size_t qb = (size_t)Q * idx->dim * sizeof(float), ib = (size_t)Q * k * sizeof(int32_t);
    int rc = CORAL_OK;
    if (hipMalloc(&d_q, qb) != hipSuccess || hipMalloc(&d_ids, ib) != hipSuccess ||
        (h_dists && hipMalloc(&d_d, ib) != hipSuccess) ||
        hipMemcpy(d_q, h_queries, qb, hipMemcpyHostToDevice) != hipSuccess)
        rc = fail(CORAL_ERR_MEMORY, "device allocation or upload failed");
    if (rc == CORAL_OK) rc = coral_bruteforce_knn_gpu(idx, d_q, Q, k, have_delete, d_ids, d_d, nullptr, time_s);
    if (rc == CORAL_OK && (hipMemcpy(h_ids, d_ids, ib, hipMemcpyDeviceToHost) != hipSuccess ||
                           (h_dists && hipMemcpy(h_dists, d_d, ib, hipMemcpyDeviceToHost) != hipSuccess)))
        rc = fail(CORAL_ERR_DEVICE, "download failed");
    (void)hipFree(d_q);
    (void)hipFree(d_ids);
    (void)hipFree(d_d);
    return rc;
}

}  // extern "C"
