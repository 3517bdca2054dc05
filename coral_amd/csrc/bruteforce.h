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
}  // namespace coral
