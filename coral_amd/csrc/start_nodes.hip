// start_nodes.hip -- the small index-maintenance kernels around the search: farthest-point sampling of
// search entry points by hop distance, the reference's Graph::FPS (src/start.cu:10-145) on the compact
// graph rows, and the tombstone marker (src/update.cu:406-412).
//
//   selected = {first}; repeat until M ids: BFS from the id selected last; min_hops[i] =
//   smallest hop count seen from any selected id (-1 while unreached); the next id is the
//   arg-max of min_hops, lowest id on ties (cub::DeviceReduce::ArgMax keeps the first maximum).
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "start_nodes.h"

namespace coral {

// seen: one bit per node, set when the node gets its hop count.  A frontier node's 32 neighbours are mostly nodes that
// have theirs already (only the first of a node's many in-edges to arrive sets it), and the bitmap is 32 times
// smaller than the hop array: it stays in L2 where the hop array does not.
__global__ void bfs_init_kernel(int* hops, uint32_t* seen, int* frontier, int start, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        hops[i] = i == start ? 0 : -1;
        if ((i & 31) == 0) seen[i >> 5] = (start >> 5) == (i >> 5) ? 1u << (start & 31) : 0u;
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) frontier[0] = start;
}

// half a wavefront per frontier node: lane = neighbour slot of its 128-byte row.  Newly reached nodes are collected
// in LDS and handed to the next frontier a few thousand at a time: one atomic on the frontier's counter per flush
// instead of one per wavefront and step (millions on one address per search otherwise).
constexpr int kBfsStage = 4096;
__global__ __launch_bounds__(256) void bfs_expand_kernel(const int32_t* __restrict__ nbrs, int R,
                                                        const int* __restrict__ frontier, int frontier_size,
                                                        int* __restrict__ next_frontier, int* __restrict__ next_size,
                                                        int* __restrict__ hops, uint32_t* __restrict__ seen, int level) {
    __shared__ int s_buf[kBfsStage];
    __shared__ int s_cnt, s_base;
    const int gtid = blockIdx.x * blockDim.x + threadIdx.x;
    const int group = gtid >> 5, lane32 = gtid & 31, ngroups = (gridDim.x * blockDim.x) >> 5;
    const int lane = threadIdx.x & 63;
    const int rounds = (frontier_size + ngroups - 1) / ngroups;  // uniform trip count for ballots and barriers
    if (threadIdx.x == 0) s_cnt = 0;
    __syncthreads();
    auto flush = [&]() {  // all threads
        const int cnt = s_cnt;
        if (threadIdx.x == 0 && cnt > 0) s_base = atomicAdd(next_size, cnt);
        __syncthreads();
        for (int i = threadIdx.x; i < cnt; i += 256) next_frontier[s_base + i] = s_buf[i];
        __syncthreads();
        if (threadIdx.x == 0) s_cnt = 0;
        __syncthreads();
    };
    for (int r = 0; r < rounds; ++r) {
        const int i = group + r * ngroups;
        bool valid = false;
        int v = -1;
        if (i < frontier_size && lane32 < R) v = nbrs[(size_t)frontier[i] * R + lane32];
        // a row ends at its first negative entry: only the lanes below it hold neighbours
        const unsigned int ends = (unsigned int)(__ballot(v < 0) >> (lane & 32));
        if (lane32 < __ffs((int)ends) - 1 || ends == 0u) {
            const uint32_t bit = 1u << (v & 31);
            // look before the atomic: a set bit stays set
            if ((seen[v >> 5] & bit) == 0u) valid = (atomicOr(seen + (v >> 5), bit) & bit) == 0u;
            if (valid) hops[v] = level;
        }
        const unsigned long long m = __ballot(valid);
        if (m) {
            int base = 0;
            if (lane == __ffsll((long long)m) - 1) base = atomicAdd(&s_cnt, __popcll(m));
            base = __shfl(base, __ffsll((long long)m) - 1, 64);
            if (valid) s_buf[base + __popcll(m & ((1ull << lane) - 1ull))] = v;
        }
        __syncthreads();
        // every thread reads the count before any thread's next step can add to it: a thread that read it later
        // could see more than the others and flush alone
        const int staged = s_cnt;
        __syncthreads();
        if (staged > kBfsStage - 256) flush();  // a step adds at most 256
    }
    flush();
}

// src/start.cu:20-30
__global__ void update_min_hop_kernel(const int* __restrict__ hops, int* __restrict__ min_hops, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const int h = hops[i];
        if (h >= 0) {
            if (h < min_hops[i] || min_hops[i] < 0) min_hops[i] = h;
        } else if (min_hops[i] == INT_MAX) {
            min_hops[i] = -1;
        }
    }
}

// arg-max with the lowest index on ties, packed as (value + 2^31) << 32 | ~index so that one
// unsigned 64-bit max does both; partial[] holds one entry per block
__global__ void argmax_kernel(const int* __restrict__ v, int64_t n, unsigned long long* __restrict__ partial) {
    __shared__ unsigned long long s[256];
    unsigned long long best = 0ull;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const unsigned long long key =
            ((unsigned long long)((uint32_t)v[i] ^ 0x80000000u) << 32) | (uint32_t)(~(uint32_t)i);
        best = key > best ? key : best;
    }
    s[threadIdx.x] = best;
    __syncthreads();
    for (int off = 128; off > 0; off >>= 1) {
        if ((int)threadIdx.x < off && s[threadIdx.x + off] > s[threadIdx.x]) s[threadIdx.x] = s[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) partial[blockIdx.x] = s[0];
}

// del_node_mark (src/update.cu:406-412): bit (id & 31) of word (id >> 5); ids outside [0, n) are counted, not marked
__global__ void mark_deleted_kernel(const int32_t* __restrict__ ids, int count, int64_t n, uint32_t* __restrict__ deleted,
                                    int* __restrict__ bad) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    const int id = ids[i];
    if (id < 0 || id >= n) {
        atomicAdd(bad, 1);
        return;
    }
    atomicOr(deleted + (id >> 5), 1u << (id & 31));
}

hipError_t launch_mark_deleted(const int32_t* ids, int count, int64_t n, uint32_t* deleted, int* bad, hipStream_t st) {
    hipLaunchKernelGGL(mark_deleted_kernel, dim3((count + 255) / 256), dim3(256), 0, st, ids, count, n, deleted, bad);
    return hipGetLastError();
}
hipError_t launch_bfs_init(int* hops, uint32_t* seen, int* frontier, int start, int64_t n, hipStream_t st) {
    hipLaunchKernelGGL(bfs_init_kernel, dim3(1024), dim3(256), 0, st, hops, seen, frontier, start, n);
    return hipGetLastError();
}
hipError_t launch_bfs_expand(const int32_t* nbrs, int R, const int* frontier, int fsize, int* next, int* nsize,
                             int* hops, uint32_t* seen, int level, hipStream_t st) {
    int blocks = (fsize * 32 + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > 2048 ? 2048 : blocks);
    hipLaunchKernelGGL(bfs_expand_kernel, dim3(blocks), dim3(256), 0, st, nbrs, R, frontier, fsize, next, nsize, hops,
                       seen, level);
    return hipGetLastError();
}
hipError_t launch_update_min_hop(const int* hops, int* min_hops, int64_t n, hipStream_t st) {
    hipLaunchKernelGGL(update_min_hop_kernel, dim3(1024), dim3(256), 0, st, hops, min_hops, n);
    return hipGetLastError();
}
hipError_t launch_argmax(const int* v, int64_t n, unsigned long long* partial, int nblocks, hipStream_t st) {
    hipLaunchKernelGGL(argmax_kernel, dim3(nblocks), dim3(256), 0, st, v, n, partial);
    return hipGetLastError();
}

}  // namespace coral
