// start_nodes.h -- launchers of the hop-distance farthest-point sampling kernels and the tombstone marker.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace coral {
// seen: uint32[ceil(n/32)], one bit per node that has its hop count
hipError_t launch_bfs_init(int* hops, uint32_t* seen, int* frontier, int start, int64_t n, hipStream_t st);
hipError_t launch_bfs_expand(const int32_t* nbrs, int R, const int* frontier, int fsize, int* next, int* nsize,
                             int* hops, uint32_t* seen, int level, hipStream_t st);
hipError_t launch_update_min_hop(const int* hops, int* min_hops, int64_t n, hipStream_t st);
hipError_t launch_argmax(const int* v, int64_t n, unsigned long long* partial, int nblocks, hipStream_t st);
hipError_t launch_mark_deleted(const int32_t* ids, int count, int64_t n, uint32_t* deleted, int* bad, hipStream_t st);
hipError_t launch_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t stream);
}  // namespace coral
