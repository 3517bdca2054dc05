// index_internal.h -- the library-private state behind a coral_index handle and the
// error-propagation macro shared by the translation units that implement the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "coral_search.h"
#include "error.h"

#define HIP_TRY(expr)                                                                       \
    do {                                                                                    \
        hipError_t e_ = (expr);                                                             \
        if (e_ != hipSuccess)                                                               \
            return coral::fail(e_ == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE,    \
                        "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__,    \
                        __LINE__);                                                          \
    } while (0)


// Launch geometry of the workgroup-per-query search kernel for one beam capacity: what coral_search_prepare works
// out and a search call hands to the kernel.
struct coral_search_plan {
    int L = 0;
    bool big = false;         // beams in global memory (the kernel's BIG form)
    int direct = 0;           // the visited set is a bitmap of all ids in LDS
    int prefetch = 0;         // a chunk's graph rows are requested one chunk ahead
    int screen = 0;           // rows are screened before their fp32 row is read: 1 in half precision, 2 in eight-bit codes
    int slots_log2 = 0, table_words = 0, vis_limit = 0, tcap = 0, ccap = 0, threads = 512, workgroups = 0;
    int id_bits = 0, rem_bits = 0, dmax = 0, ocap = 0;
    int choices = 0;          // 3: the table of cells in its bucket form (three candidate buckets per id)
    size_t lds_bytes = 0;
    size_t spill_words = 0;   // words of one workgroup's overflow bitmap in global memory (0: never used)
    size_t beam_stride = 0;   // 64-bit words of one workgroup's beam block in global memory (0 unless big)
};

struct coral_index {
    int device = 0;
    int64_t n = 0;
    int dim = 0, R = 0, M = 0, metric = 0;
    float* d_vec = nullptr;
    int32_t* d_nbrs = nullptr;
    int32_t* d_start = nullptr;
    uint32_t* d_deleted = nullptr;
    hipStream_t stream = nullptr;
    int num_cu = 0;

    // state of search_prepare
    bool prepared = false;
    int Q = 0, L = 0, prepared_policy = 0;
    coral_search_plan plan;
    uint32_t* d_spill = nullptr;
    size_t spill_alloc_words = 0;
    unsigned char* d_vec16 = nullptr;  // half-precision copy of the vectors for the screening phase (made on first use)
    unsigned char* d_vec8 = nullptr;   // copy in eight-bit codes for the screening phase (made on first use)
    uint64_t* d_beam = nullptr;  // beam blocks of a BIG launch, plan.workgroups x plan.beam_stride words
    size_t beam_alloc_words = 0;
    int32_t* d_counters = nullptr;
    size_t counters_alloc = 0;
    int* d_scalars = nullptr;  // [0] next_qid, [1] spill_count
    unsigned long long* d_hit = nullptr;
    unsigned long long* d_phase = nullptr;  // debug builds only
    int32_t* h_counters = nullptr;  // pinned, counters_alloc entries
    int last_Q = 0;
    // the entry point that allocates nothing: its last plan (kernel attributes and occupancy are looked up once per
    // (Q, L, policy, screening form)), and whether a launch of it may still be in flight on a stream of the caller's
    coral_search_plan noalloc_plan;
    int noalloc_Q = 0, noalloc_L = 0, noalloc_policy = -1, noalloc_screen = -2;
    bool noalloc_in_flight = false;
    hipEvent_t ev[3] = {nullptr, nullptr, nullptr};  // start, kernel end, read-back end of a search
    // device staging of the host-buffer entry point (grow-only)
    float* d_io_q = nullptr;
    int32_t* d_io_ids = nullptr;
    float* d_io_dists = nullptr;
    size_t io_q_bytes = 0, io_ids_bytes = 0, io_dists_bytes = 0;

    // exact kNN: |b|^2 of every base vector and the bit pattern of the largest (made on first use), and whether the
    // matrix-core screening pass is skipped
    float* d_bnorm = nullptr;
    uint32_t* d_bnorm_max = nullptr;
    int knn_mode = 0;             // 0: fused screening, 1: no screening, 2: screening through the distance matrix
    bool knn_last_fused = false;  // the last call's candidates came from the fused screening
    int64_t knn_last_redone = 0;  // queries of the last call that went through the exact passes after screening

    // best-first on one wavefront per query: per-slot visited epochs in global memory
    bool bf_ready = false;
    uint8_t* d_bf_visited = nullptr;
    uint32_t* d_bf_epochs = nullptr;
    size_t bf_stride = 0, bf_alloc_bytes = 0;
    int bf_slots = 0, bf_alloc_slots = 0, bf_rows_in_flight = 8, bf_packed = 0, bf_bloom_log2 = 0;
    int bf_table_log2 = 0, bf_table_rem_bits = 0;
    // ... or, for long beams, with an insert buffer in LDS and the long sorted run of every slot in global memory
    int bf_screen = 0;  // the kernel with the beam in LDS screens rows: 1 in half precision (d_vec16), 2 in eight-bit codes (d_vec8)
    bool bf_long = false;
    uint64_t* d_bf_beams = nullptr;
    size_t bf_beam_alloc_words = 0, bf_beam_stride = 0;
    int bf_bcap = 0, bf_scap = 0, bf_sshift = 0;
    int rows_unique = -1;  // 1: no graph row lists an id twice, 0: some do, -1: not looked at since the rows changed
    // the tuning of the last prepare, and what the searches since have taught about the visited table:
    // at beam capacity bump_L the library's own choice of table size is raised by bump_log2
    coral_tuning tuning{};
    int bump_L = 0, bump_log2 = 0;

    // graph construction (coral_build_*): per-neighbour distances, degrees, the per-batch claim table
    // (INT_MAX when idle) and the staging rows of one batch
    bool building = false;
    float* d_nbr_dists = nullptr;  // [n][R]
    int32_t* d_deg = nullptr;      // [n]
    int32_t* d_owner = nullptr;    // [n]
    int32_t* d_new_ids = nullptr;
    float* d_new_dists = nullptr;
    int32_t* d_new_deg = nullptr;
    size_t stage_rows = 0;
    int32_t* d_len = nullptr;  // found-list lengths of one enhancement batch
    size_t len_alloc = 0;
    uint32_t* d_hits = nullptr;  // [n] clusters of this build that contain the node
    // second enhancement phase: candidate lists (found + current row) of one batch and their found-part lengths
    int32_t* d_top_ids_list = nullptr;
    float* d_top_dists_list = nullptr;
    int32_t* d_rev_len = nullptr;
    size_t top_list_cells = 0, rev_len_alloc = 0;
    unsigned long long* d_build_stats = nullptr;  // [0] reverse edges inserted, [1] turned away, [2] ids out of range
};

namespace coral {
void free_build_state(coral_index* idx);
}

