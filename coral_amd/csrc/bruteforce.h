// bruteforce.h -- host-side launchers of the exact kNN kernels (bruteforce.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace coral {
hipError_t launch_distance_tile(const float* queries, const float* base, int nq, int64_t nb, int dim,
                                int metric, const uint32_t* deleted, int64_t base_id0, float* D,
                                int64_t ldD, hipStream_t stream);
// redo: int[nq] scratch for the rows the fast path hands over (null: radix path for every row)
hipError_t launch_row_select(const float* D, int64_t ldD, int nq, int64_t n, int k, int64_t id0,
                             unsigned long long* out, int64_t out_stride, int* redo, hipStream_t stream);
hipError_t launch_merge_segments(const unsigned long long* part, int nq, int nseg, int k, int metric,
                                 int32_t* ids, float* dists, hipStream_t stream);
// --- the screening pass on the matrix cores (bruteforce_mfma.hip) ---
// out[r] = |x_r|^2; *max_bits (optional, zero before) = bit pattern of the largest of them
hipError_t launch_row_norms(const float* x, int64_t n, int dim, float* out, uint32_t* max_bits, hipStream_t stream);
// as launch_distance_tile, with D[q][b] = |q|^2 + |b|^2 - 2 q.b (L2) or -q.b (IP) from fp32 MFMA inner products
// sample_tiles > 0: only that many tiles of 128 base points, every tile_stride-th of the base, side by side in D
hipError_t launch_approx_tile(const float* queries, const float* base, int nq, int64_t nb, int dim, int metric,
                              const float* qn, const float* bn, const uint32_t* deleted, int64_t base_id0, float* D,
                              int64_t ldD, hipStream_t stream, int64_t sample_tiles = 0, int64_t tile_stride = 1);
// the same distances, no matrix: every entry <= tau[q] is appended to lists[q * cap ...] as ord(value) << 32 | id
// (cnt[q] counts them, also those beyond cap that were dropped; zero before)
hipError_t launch_approx_filter(const float* queries, const float* base, int nq, int64_t nb, int dim, int metric,
                                const float* qn, const float* bn, const uint32_t* deleted, const float* tau,
                                unsigned long long* lists, int64_t cap, unsigned int* cnt, hipStream_t stream);
// tau[q] = value of keys[q * stride + j], +inf where that key is the "none" key
hipError_t launch_bound_from_keys(const unsigned long long* keys, int64_t stride, int j, int nq, float* tau,
                                  hipStream_t stream);
// the k (<= 1024) smallest keys of every list, sorted; *overflow (zero before) counts the lists that could not be done
hipError_t launch_list_select(const unsigned long long* lists, int64_t cap, const unsigned int* cnt, int nq, int k,
                              unsigned long long* out, int64_t out_stride, int* overflow, hipStream_t stream);
// cand_ids / cand_d [nq][kc] (ascending approximate signed distance, -1 = none) -> the exact k best per query in the
// reference's summation order; redo[q] = 1 where the candidates cannot vouch for the result
hipError_t launch_rerank(const float* queries, const float* base, int nq, int dim, int metric, const int32_t* cand_ids,
                         const float* cand_d, int kc, int k, const float* qn, const uint32_t* bn_max_bits, int32_t* ids,
                         float* dists, int* redo, hipStream_t stream);
hipError_t launch_scatter_results(const int32_t* rows, int count, int k, const int32_t* src_ids, const float* src_d,
                                  int32_t* dst_ids, float* dst_d, hipStream_t stream);
}  // namespace coral
