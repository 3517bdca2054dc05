// start_nodes_api.cpp -- coral_start_ids_fps: Graph::FPS (src/start.cu:74-145) on the resident graph;
// coral_index_mark_deleted: GPUFuncs::del_node_mark (src/update.cu:660-672).
#include <climits>
#include <vector>

#include "index_internal.h"
#include "start_nodes.h"

using coral::fail;

extern "C" int coral_start_ids_fps(coral_index* idx, int32_t first_id, int32_t M, int32_t* out_ids) {
    if (!idx || !out_ids) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->d_nbrs) return fail(CORAL_ERR_STATE, "the index holds vectors only (no graph was given)");
    if (M <= 0) return fail(CORAL_ERR_ARG, "M must be positive");
    if (first_id < 0 || first_id >= idx->n) return fail(CORAL_ERR_ARG, "first id %d out of range", first_id);
    HIP_TRY(hipSetDevice(idx->device));
    hipStream_t st = idx->stream;
    const int64_t n = idx->n;
    const int nblocks = 512;
    int *hops = nullptr, *min_hops = nullptr, *fa = nullptr, *fb = nullptr, *sizes = nullptr;
    uint32_t* seen = nullptr;
    unsigned long long* partial = nullptr;
    auto release = [&]() {
        (void)hipFree(hops), (void)hipFree(min_hops), (void)hipFree(fa), (void)hipFree(fb);
        (void)hipFree(sizes), (void)hipFree(partial), (void)hipFree(seen);
    };
#define TRY_R(expr)                                                                      \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess) {                                                          \
            release();                                                                   \
            return fail(e_ == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE, \
                        "%s failed: %s", #expr, hipGetErrorString(e_));                  \
        }                                                                                \
    } while (0)
    TRY_R(hipMalloc(&hops, n * sizeof(int)));
    TRY_R(hipMalloc(&min_hops, n * sizeof(int)));
    TRY_R(hipMalloc(&fa, n * sizeof(int)));
    TRY_R(hipMalloc(&fb, n * sizeof(int)));
    TRY_R(hipMalloc(&seen, (((size_t)n + 31) / 32 + 1) * sizeof(uint32_t)));
    TRY_R(hipMalloc(&sizes, 2 * sizeof(int)));
    TRY_R(hipMalloc(&partial, nblocks * sizeof(unsigned long long)));
    TRY_R(coral::launch_fill_u32((uint32_t*)min_hops, (size_t)n, (uint32_t)INT_MAX, st));
    std::vector<unsigned long long> h_partial(nblocks);
    int start = first_id, count = 0;
    out_ids[count++] = start;
    while (count < M) {
        // one breadth-first search from the id selected last (src/start.cu:53-72)
        TRY_R(coral::launch_bfs_init(hops, seen, fa, start, n, st));
        int fsize = 1, level = 1;
        int *cur = fa, *next = fb;
        while (fsize > 0) {
            TRY_R(coral::launch_fill_u32((uint32_t*)sizes, 1, 0u, st));
            TRY_R(coral::launch_bfs_expand(idx->d_nbrs, idx->R, cur, fsize, next, sizes, hops, seen, level++, st));
            TRY_R(hipMemcpyAsync(&fsize, sizes, sizeof(int), hipMemcpyDeviceToHost, st));
            TRY_R(hipStreamSynchronize(st));
            std::swap(cur, next);
        }
        TRY_R(coral::launch_update_min_hop(hops, min_hops, n, st));
        TRY_R(coral::launch_argmax(min_hops, n, partial, nblocks, st));
        TRY_R(hipMemcpyAsync(h_partial.data(), partial, nblocks * sizeof(unsigned long long), hipMemcpyDeviceToHost,
                             st));
        TRY_R(hipStreamSynchronize(st));
        unsigned long long best = 0ull;
        for (unsigned long long p : h_partial) best = p > best ? p : best;
        start = (int)(~(uint32_t)best);
        out_ids[count++] = start;
    }
#undef TRY_R
    release();
    return CORAL_OK;
}

// GPUFuncs::del_node_mark (src/update.cu:660-672): upload the ids, OR their bits into the mask.
extern "C" int coral_index_mark_deleted(coral_index* idx, const int32_t* h_ids, int32_t count) {
    if (!idx || (!h_ids && count > 0)) return fail(CORAL_ERR_ARG, "null argument");
    if (count < 0) return fail(CORAL_ERR_ARG, "negative count");
    HIP_TRY(hipSetDevice(idx->device));
    hipStream_t st = idx->stream;
    const size_t words = ((size_t)idx->n + 31) / 32;
    if (!idx->d_deleted) {
        HIP_TRY(hipMalloc(&idx->d_deleted, words * sizeof(uint32_t)));
        hipError_t e = coral::launch_fill_u32(idx->d_deleted, words, 0u, st);
        if (e == hipSuccess) e = hipStreamSynchronize(st);
        if (e != hipSuccess) {
            (void)hipFree(idx->d_deleted);
            idx->d_deleted = nullptr;
            return fail(CORAL_ERR_DEVICE, "clearing the tombstone mask failed: %s", hipGetErrorString(e));
        }
    }
    if (count == 0) return CORAL_OK;
    int32_t* d_ids = nullptr;
    int* d_bad = nullptr;
    int bad = 0;
    hipError_t e = hipMalloc(&d_ids, (size_t)count * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc(&d_bad, sizeof(int));
    if (e == hipSuccess) e = hipMemcpyAsync(d_ids, h_ids, (size_t)count * sizeof(int32_t), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) e = coral::launch_fill_u32((uint32_t*)d_bad, 1, 0u, st);
    if (e == hipSuccess) e = coral::launch_mark_deleted(d_ids, count, idx->n, idx->d_deleted, d_bad, st);
    if (e == hipSuccess) e = hipMemcpyAsync(&bad, d_bad, sizeof(int), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    (void)hipFree(d_ids), (void)hipFree(d_bad);
    if (e != hipSuccess)
        return fail(e == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE, "marking deleted ids failed: %s",
                    hipGetErrorString(e));
    if (bad) return fail(CORAL_ERR_GRAPH, "%d of %d deleted ids are outside [0,%lld); the others were marked", bad, count,
                         (long long)idx->n);
    return CORAL_OK;
}

// The tombstone mask as the device holds it, ceil(n/32) words; all zero when nothing was ever deleted.
extern "C" int coral_index_get_deleted(coral_index* idx, uint32_t* host_mask) {
    if (!idx || !host_mask) return fail(CORAL_ERR_ARG, "null argument");
    HIP_TRY(hipSetDevice(idx->device));
    const size_t words = ((size_t)idx->n + 31) / 32;
    if (!idx->d_deleted) {
        for (size_t i = 0; i < words; ++i) host_mask[i] = 0u;
        return CORAL_OK;
    }
    HIP_TRY(hipStreamSynchronize(idx->stream));
    HIP_TRY(hipMemcpy(host_mask, idx->d_deleted, words * sizeof(uint32_t), hipMemcpyDeviceToHost));
    return CORAL_OK;
}
