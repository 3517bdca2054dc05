// graph_build.h -- launchers of the graph construction kernels (graph_build.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace coral {
constexpr int kBuildMaxKb = 128;  // members of a cluster (the reference's k, config.json:3: 100)
constexpr int kBuildMaxR = 32;    // row width (MAX_DEGREE, include/uni.h:60)

size_t nap_lds_bytes(int kb);
// One batch of clusters knn[batch][kb] (device).  owner[n] must hold INT_MAX everywhere and does so again afterwards;
// new_ids / new_dists [batch*kb][R] and new_deg [batch*kb] are staging.
hipError_t launch_nap_batch(const float* vec, int dim, int metric, int R, int32_t* nbrs, float* dists, int32_t* deg,
                            int32_t* owner, const int32_t* knn, int batch, int kb, int need_discard, int32_t* new_ids,
                            float* new_dists, int32_t* new_deg, hipStream_t st);
// One batch of isolated nodes with what the search found for them, knn_ids / knn_dists [batch][kn]; len [batch] is
// scratch; stats (optional) [0] reverse edges inserted, [1] turned away.
hipError_t launch_enhance_batch(const float* vec, int dim, int metric, int R, int32_t* nbrs, float* dists, int32_t* deg,
                                int32_t* owner, const int32_t* iso_ids, const int32_t* knn_ids, const float* knn_dists,
                                int batch, int kn, int32_t* len, const int32_t* rev_len, unsigned long long* stats,
                                hipStream_t st);
// rev_len (optional) [batch]: only the first rev_len[b] entries of list b insert reverse edges.
// The candidate lists of the second enhancement phase: found list (to its first -1) + the node's current row, -1 padded,
// out_ids / out_dists [batch][k + R]; rev_len[b] = entries that came from the found list
hipError_t launch_enhance_top_lists(int R, const int32_t* nbrs, const float* dists, const int32_t* deg,
                                    const int32_t* top_ids, const int32_t* knn_ids, const float* knn_dists, int batch, int k,
                                    int32_t* out_ids, float* out_dists, int32_t* rev_len, hipStream_t st);
// hits[id] += 1 for every id of the list
hipError_t launch_count_hits(const int32_t* ids, int64_t count, uint32_t* hits, hipStream_t st);
// *bad += number of ids outside [0, n) (an id of -1 is let through when minus_one_ok)
hipError_t launch_count_bad_ids(const int32_t* ids, int64_t count, int64_t n, int minus_one_ok, unsigned long long* bad,
                                hipStream_t st);
hipError_t launch_gather_rows(const float* vec, int dim, const int32_t* ids, int count, float* out, hipStream_t st);
}  // namespace coral
