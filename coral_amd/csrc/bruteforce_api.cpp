// bruteforce_api.cpp -- coral_bruteforce_knn*: exact k nearest neighbours of a batch of
// queries among the index's resident vectors (kernels in bruteforce.hip).
#include <algorithm>
#include <cstring>

#include "bruteforce.h"
#include "index_internal.h"

using coral::fail;

namespace {
constexpr int64_t kSegment = (int64_t)1 << 22;   // base points per pass
constexpr int64_t kBufferFloats = (int64_t)1 << 29;  // 2 GiB distance buffer
}  // namespace

extern "C" {

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
    hipEvent_t ev0, ev1;
    HIP_TRY_R(hipEventCreate(&ev0));
    HIP_TRY_R(hipEventCreate(&ev1));
    HIP_TRY_R(hipEventRecord(ev0, stream));
    for (int64_t q0 = 0; q0 < Q; q0 += qc) {
        const int nq = (int)std::min<int64_t>(qc, Q - q0);
        for (int64_t s = 0; s < nseg; ++s) {
            const int64_t b0 = s * seg, nb = std::min(seg, n - b0);
            HIP_TRY_R(coral::launch_distance_tile(d_queries + (size_t)q0 * idx->dim,
                                                  idx->d_vec + (size_t)b0 * idx->dim, nq, nb, idx->dim,
                                                  idx->metric, have_delete ? idx->d_deleted : nullptr, b0, D, ld,
                                                  stream));
            HIP_TRY_R(coral::launch_row_select(D, ld, nq, nb, k, b0, part + ((size_t)q0 * nseg + s) * k,
                                               nseg * k, redo, stream));
        }
    }
    HIP_TRY_R(coral::launch_merge_segments(part, Q, (int)nseg, k, idx->metric, d_ids, d_dists, stream));
    HIP_TRY_R(hipEventRecord(ev1, stream));
    HIP_TRY_R(hipEventSynchronize(ev1));
    float ms = 0.f;
    HIP_TRY_R(hipEventElapsedTime(&ms, ev0, ev1));
#undef HIP_TRY_R
    (void)hipEventDestroy(ev0);
    (void)hipEventDestroy(ev1);
    release();
    if (time_s) *time_s = ms / 1000.0;
    return CORAL_OK;
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
