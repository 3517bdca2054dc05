/*
 * coral_formats.h -- C ABI for the reference's on-disk formats that the search
 * path reads (and writers for the same, so tests and tools can produce them).
 * Host code only.  All functions return a coral_status (coral_search.h).
 *
 *   .fbin     uint32 n, uint32 dim, float32[n*dim]
 *             (README.md:13; include/efanna2e/util.h:104-128, 182-218)
 *   gt file   uint32 nq, uint32 k, int32 ids[nq*k] (+ optional trailing
 *             distances, ignored) (include/efanna2e/util.h:81-103, 159-180;
 *             tests/comp_gt.cpp:142-175)
 *   index directory
 *             graph.part<p>.idx    node_count x {uint64 offset; uint32 size; int32 pos}
 *                                  (include/disk_graph.h:78-84, src/disk.cpp:155-179)
 *             graph.part<p>.data / .append
 *                                  per node [int32 node_id][uint32 raw_size][LZ4 block of
 *                                  {int32 deg; int32 nbrs[deg]; float dists[deg]}]
 *                                  (src/disk.cpp:22-37, 336-426); size 0 = degree 0
 *             graph.search_start_ids  text "M id0 id1 ..." (src/graph.cpp:316-351)
 *             graph.batch_id       text integer (src/disk.cpp:65-78)
 *             partitions: count = ceil(n / 1e8), nodes per partition = ceil(n / count)
 *             (src/disk.cpp:102-103)
 *   RoarGraph file
 *             uint32 ep, uint32 npts, then per node uint32 deg, uint32 nbrs[deg]
 *             (src/graph.cu:709-735)
 *
 * The LZ4 block codec is this library's own (the reference links the system
 * liblz4, CMakeLists.txt:66-67): any conforming decoder reads what
 * coral_lz4_compress writes, and coral_lz4_decompress reads what
 * LZ4_compress_default writes.
 */
#ifndef CORAL_FORMATS_H
#define CORAL_FORMATS_H

#include "coral_search.h"

#ifdef __cplusplus
extern "C" {
#endif

/* load_meta: header + file-size check (throws in the reference, util.h:120-125) */
CORAL_API int coral_fbin_read_meta(const char* path, int64_t* n, int32_t* dim);
/* load_data: rows are written `stride` floats apart (stride >= dim, the tail of
 * each row zero-filled: the reference pads dim up to a multiple of 4, util.h:194-208) */
CORAL_API int coral_fbin_read(const char* path, float* out, int64_t n, int32_t dim, int32_t stride);
CORAL_API int coral_fbin_write(const char* path, const float* data, int64_t n, int32_t dim);

CORAL_API int coral_gt_read_meta(const char* path, int32_t* nq, int32_t* k);
CORAL_API int coral_gt_read(const char* path, int32_t* ids, int32_t nq, int32_t k);
CORAL_API int coral_gt_write(const char* path, const int32_t* ids, int32_t nq, int32_t k);

/* DiskStorage::load_batch_slots over all nodes -> compact rows nbrs[n][R] (-1
 * padded); dists[n][R] optional (0-filled past deg).  A node whose stored degree
 * exceeds R is an error. */
CORAL_API int coral_graph_dir_read(const char* dir, int64_t n, int32_t R, int32_t* nbrs, float* dists);
/* writes graph.part*.idx/.data (everything in the BASE file, .append left empty),
 * graph.batch_id = 0; dists may be NULL (zeros are stored) */
CORAL_API int coral_graph_dir_write(const char* dir, int64_t n, int32_t R, const int32_t* nbrs,
                                    const float* dists);

CORAL_API int coral_start_ids_read(const char* dir, int32_t* ids, int32_t capacity, int32_t* count);
CORAL_API int coral_start_ids_write(const char* dir, const int32_t* ids, int32_t count);

/* IVFBuilder::save_hits / load_hits (include/ivf.cuh:639-656): <dir>/hits.bin = int64 n, then uint32[n], how many
 * clusters of the build contained each node.  read fails when the file holds fewer than n counts. */
CORAL_API int coral_hits_read(const char* dir, uint32_t* hits, int64_t n);
CORAL_API int coral_hits_write(const char* dir, const uint32_t* hits, int64_t n);

/* Graph::LoadRoarGraph: degrees above R are truncated to R as the reference does */
CORAL_API int coral_roargraph_read(const char* path, int64_t n, int32_t R, int32_t* nbrs, int32_t* ep);
CORAL_API int coral_roargraph_write(const char* path, int64_t n, int32_t R, const int32_t* nbrs,
                                    int32_t ep);

/* LZ4 block format.  decompress returns the number of bytes written or a
 * negative value on malformed input / overflow; compress returns the compressed
 * size or 0 when dst is too small. */
CORAL_API int coral_lz4_compress_bound(int src_len);
CORAL_API int coral_lz4_compress(const void* src, int src_len, void* dst, int dst_cap);
CORAL_API int coral_lz4_decompress(const void* src, int src_len, void* dst, int dst_cap);

/* normalize_L2_omp (src/uni.cpp:38-54) */
CORAL_API void coral_normalize_l2(float* x, int64_t n, int64_t d);

/* ComputeRecall's hit count (tests/test_search_pipeline.cpp:25-39), host arrays;
 * res rows are k apart, gt rows gt_dim apart */
CORAL_API int64_t coral_recall_hits(int32_t q_num, int32_t k, int32_t gt_dim, const int32_t* res,
                                    const int32_t* gt);

#ifdef __cplusplus
}
#endif
#endif
