/*
 * coral_search.h -- C ABI of libcoral_search.so: CORAL's batched graph beam
 * search on one MI355X (gfx950), whole index resident in HBM.
 *
 * The reference's boundary for this path is a C++ class (efanna2e::IndexGPU over
 * GPUFuncs, include/index_gpu.h:42-76, include/gpufuncs.cuh:597-893); it has no C
 * interface.  Each entry point below names the reference member it stands for.
 * include/efanna2e/index_gpu.h in this repository is the C++ class of the same
 * name and signatures, implemented on top of these calls.
 *
 * Conventions
 *   - plain pointers and sizes only; every function returns a coral_status
 *     (0 = success) instead of terminating the process the way the reference's
 *     CUDA_CHECK / fo.eprint do (include/utils.cuh:50-58, src/fileout.cpp:88-98);
 *     coral_last_error() gives the message of the calling thread's last failure.
 *   - metric: CORAL_L2 = squared Euclidean, smaller is closer; CORAL_IP = raw
 *     inner product, larger is closer (include/utils.cuh:380-382, include/uni.h:65-68).
 *   - graph rows are compact: int32 nbrs[n][R], a row's neighbours are its
 *     leading non-negative entries (the deg and nbrs[0..deg) fields of the
 *     reference's 400-byte Slot, include/disk_graph.h:30-52, and nothing else).
 *   - results are ordered closest first; unfilled slots hold id -1 and the
 *     farthest value of the policy's reference path: +-FLT_MAX (L2 / IP) for
 *     CORAL_POLICY_ROUNDS (src/search_gpu.cu:408), +-infinity for
 *     CORAL_POLICY_BEST_FIRST (src/search_in_cpu.cpp:33-35).
 *   - not thread-safe per index, like the reference (src/search.cu:404-408).
 */
#ifndef CORAL_SEARCH_H
#define CORAL_SEARCH_H

#include <stddef.h>
#include <stdint.h>

#if defined(__GNUC__)
#define CORAL_API __attribute__((visibility("default")))
#else
#define CORAL_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    CORAL_OK = 0,
    CORAL_ERR_ARG = 1,      /* null pointer, size out of range, k > L, M > L ... */
    CORAL_ERR_GRAPH = 2,    /* neighbour id or start id out of range, duplicate start ids */
    CORAL_ERR_DEVICE = 3,   /* a HIP call failed; message carries hipGetErrorString */
    CORAL_ERR_MEMORY = 4,   /* host or device allocation failed */
    CORAL_ERR_IO = 5,       /* file missing, short, or malformed */
    CORAL_ERR_STATE = 6     /* call order: search before prepare, and the like */
} coral_status;

enum { CORAL_L2 = 0, CORAL_IP = 1 };

/* Traversal policy.
 * CORAL_POLICY_ROUNDS: every beam entry not yet expanded is expanded in one
 *   round, candidates are pre-filtered against the threshold frozen at the start
 *   of the round, then merged (the CUDA kernel, src/search_gpu.cu:347-580).
 * CORAL_POLICY_BEST_FIRST: one expansion at a time, always the closest entry not
 *   yet expanded (the CPU path, src/search_in_cpu.cpp:63-108). */
enum { CORAL_POLICY_ROUNDS = 0, CORAL_POLICY_BEST_FIRST = 1 };

typedef struct coral_index coral_index;

/* Host-side description of an index; all pointers are borrowed for the duration
 * of coral_index_create only (the data is copied into HBM). */
typedef struct {
    const float* base;        /* [n][dim] fp32 row major; dim % 4 == 0 */
    const int32_t* nbrs;      /* [n][R] compact rows, -1 padded; NULL = vectors only (brute force) */
    int64_t n;
    int32_t dim;
    int32_t R;                /* row width, <= 32 (MAX_DEGREE, include/uni.h:60) */
    const int32_t* start_ids; /* graph.search_start_ids, src/graph.cpp:329-351 */
    int32_t n_start;
    int32_t metric;
    int32_t device;           /* HIP device ordinal; the reference hard-codes 0 */
} coral_index_desc;

/* Counters of one search call.  time_s has the scope of the reference's own
 * timer (src/search_gpu.cu:861-877): the kernel plus the read-back of the
 * per-query counters, measured with a HIP event pair on the search stream. */
typedef struct {
    double time_s;
    double kernel_s;     /* the search kernel alone (HIP event pair around the launch) */
    int64_t hops;        /* what Test_Result.hops holds for this policy */
    int64_t expansions;  /* graph rows read */
    int64_t dist_evals;  /* vector rows read (first visits + start ids) */
    int64_t rounds;      /* merge rounds (ROUNDS) or expansion steps (BEST_FIRST) */
    int64_t spills;      /* queries whose visited set outgrew LDS */
    /* what the launch read, by class (the sums of coral_search_row_counters): */
    int64_t screened_rows;  /* rows measured on the smaller copy of the vectors (codes or half precision) */
    int64_t exact_rows;     /* fp32 vector rows read: dist_evals without screening, a fraction of them with it */
    int64_t beam_words;     /* 32-bit words of beam state (keys, expand lists, long runs) read or written in global
                               memory by passes over a beam that does not live in LDS */
    int64_t visited_requests; /* tests and marks of the visited state that went to global memory */
    int64_t visited_dedupes;  /* lists of new ids that the bucket form of the visited table had searched for repeats
                                 (two threads inserted the same id at the same time) */
} coral_stats;

/* Optional launch tuning; zero-initialise for defaults. */
typedef struct {
    int32_t visited_slots_log2; /* visited set in LDS: log2 of the 16-bit cells of its table, 10..16 (what outgrows the
                                   table goes to a bitmap in global memory); -1 = a plain bitmap of all n ids instead
                                   (n / 8 bytes: up to about a million nodes); 0 = chosen from L and n */
    int32_t workgroups;         /* persistent workgroups (of four query slots each on the wavefront-per-query
                                   best-first kernel); 0 = chosen from Q and the device */
    int32_t threads;            /* threads per workgroup: 128, 256, 512 or 1024; 0 = chosen from the LDS need */
    int32_t policy;             /* the policy the scratch is sized for (CORAL_POLICY_*); best-first visits
                                   fewer nodes per beam entry and works on one graph row at a time */
    int32_t best_first_in_lds;  /* best-first normally runs one wavefront per query with a byte of visited state
                                   per node and query slot in HBM (n bytes x up to 4096 slots); 1 keeps it on the
                                   workgroup-per-query kernel with the visited set in LDS, as it also does by
                                   itself when that memory is not to be had */
    int32_t best_first_packed;  /* that visited state is a byte per node while n bytes x query slots fit a third of
                                   the free memory (and 64 GiB), else a 32-bit word per 24 nodes (8 bits of epoch,
                                   24 flags: n / 6 bytes per slot, about 5 % slower); 1 = the packed form always */
    int32_t best_first_table_log2; /* the wavefront-per-query kernel keeps the first visits of a query in an exact
                                   table of 16-bit cells in LDS (the cells of the ROUNDS kernel's table) and only
                                   what outgrows it in HBM: log2 of the cells per query, 8..14; 0 = chosen from L
                                   where 8192 cells hold most of a query's visits (L <= 409 at up to 2^25 nodes),
                                   none otherwise; -1 = none */
    int32_t beam_in_hbm;        /* 1 = keep the beam in global memory whatever L is (the form beams longer than
                                   CORAL_MAX_LDS_BEAM always take, and shorter ones when that frees the LDS a bitmap of
                                   all ids needs) */
    int32_t prefetch_rows;      /* graph rows of a chunk of beam entries requested one chunk ahead: 1 = yes, -1 = no,
                                   0 = where a workgroup has its CU to itself */
    int32_t cand_cap;           /* capacity of the candidate buffer in LDS (a power of two, at least the todo list's);
                                   0 = chosen */
    int32_t best_first_long;    /* best-first with a wavefront per query keeps beams up to 1280 entries in LDS and longer
                                   ones as a sorted insert buffer in LDS in front of a long run in global memory (two
                                   runs of L keys per query slot): 1 = that form whatever L is, -1 = never (beams
                                   beyond CORAL_MAX_LDS_BEAM then run on the workgroup-per-query kernel), 0 = by L */
    int32_t best_first_buffer;  /* keys of that insert buffer, a multiple of 64 in 64..4096; 0 = 512 */
    int32_t screening;          /* every row is first measured in a smaller copy of the vectors (made on first use) and its
                                   fp32 row is read only if rigorous bounds on the exact distance leave open whether it
                                   is a candidate or a beam entry; results and counters are the same bit for bit.
                                   2 = a copy in eight-bit codes (256 bytes per row at dim 200): rows of 68 .. 2048
                                   floats under the rounds policy, 68 .. 512 under best-first; 1 = a half-precision
                                   copy (512 bytes per row at dim 200): L2 only, rows of more than 128 floats;
                                   -1 = off; 0 = the library's choice where the memory for the copy is there: rows of
                                   more than 128 floats on codes (L2 rows of more than 1024 floats in half precision)
                                   under the rounds policy; under best-first rows of 132 .. 512 floats on codes for
                                   beams of 410 entries and more. */
    int32_t visited_choices;    /* form of the table of 16-bit cells: 1 = open addressing with linear probing (a cell
                                   carries its displacement), 3 = buckets of four cells, three candidate buckets per
                                   id (a cell carries which of the three: 14 bits of the id per cell whatever the
                                   load; ids of up to 12 bits more than the table has cells); 0 = linear probing
                                   unless the ids are so wide that a cell could carry displacements below 30
                                   (beyond 2^24 ids); 4 = form 3 with the bucket picked by the inserting wavefront's
                                   number instead of by the load: same results, for tests of the path that two
                                   threads take when they insert one id at the same time */
} coral_tuning;

CORAL_API const char* coral_last_error(void);

/* Graph ctor, GPU branch (include/graph.cuh:240-261): device allocation and
 * upload of the graph rows and vectors; also validates ids, which the reference
 * does not.  For CORAL_IP the caller has already normalised base, as
 * IndexGPU::LoadVectorData does (src/index_gpu.cpp:641). */
CORAL_API int coral_index_create(const coral_index_desc* desc, coral_index** out);
CORAL_API void coral_index_destroy(coral_index* idx);

/* Replace the graph rows of an existing index (Graph::LoadRoarGraph's upload,
 * src/graph.cu:737-742) and its start ids. */
CORAL_API int coral_index_set_graph(coral_index* idx, const int32_t* nbrs, const int32_t* start_ids,
                          int32_t n_start);

/* Tombstone mask, bit (id & 31) of word (id >> 5) (src/update.cu:406-412);
 * host_mask holds ceil(n/32) words, or NULL to clear. */
CORAL_API int coral_index_set_deleted(coral_index* idx, const uint32_t* host_mask);

/* GPUFuncs::del_node_mark (src/update.cu:406-412, 660-672): ORs the bits of count host ids into the mask
 * (allocated and cleared on first use).  Ids outside [0, n) are skipped and reported as CORAL_ERR_GRAPH
 * after the valid ones were marked; the reference does not check.  coral_index_get_deleted copies the
 * mask back, ceil(n/32) words. */
CORAL_API int coral_index_mark_deleted(coral_index* idx, const int32_t* h_ids, int32_t count);
CORAL_API int coral_index_get_deleted(coral_index* idx, uint32_t* host_mask);

CORAL_API int coral_index_info(const coral_index* idx, int64_t* n, int32_t* dim, int32_t* R,
                     int32_t* n_start, int32_t* metric);

/* Beam capacity L.  Up to CORAL_MAX_LDS_BEAM the beam lives in LDS; longer beams are kept per workgroup in global
 * memory, as the reference keeps every beam (src/search.cu:400-402, include/gpufuncs.cuh:557-564), up to
 * CORAL_MAX_BEAM.  The reference sets no limit; its driver grows L by 128 for at most 51 steps
 * (tests/test_search_pipeline.cpp:278-313) and its config.json defaults to 1024. */
#define CORAL_MAX_LDS_BEAM 2048
#define CORAL_MAX_BEAM 65536

/* GPUFuncs::search_prepare(Q, L) (src/search.cu:400-408): fixes the beam
 * capacity (1..CORAL_MAX_BEAM) and (re)allocates per-workgroup scratch. */
CORAL_API int coral_search_prepare(coral_index* idx, int32_t Q, int32_t L, const coral_tuning* tuning);

/* GPUFuncs::search_gpu (src/search_gpu.cu:835-886): device pointers in and out,
 * one persistent launch.  d_dists may be NULL.  have_delete selects the
 * tombstone-aware output (src/search_gpu.cu:582-833).  stream is a hipStream_t
 * (NULL = the index's own stream, like streams["search"]). */
CORAL_API int coral_search_gpu(coral_index* idx, const float* d_queries, int32_t* d_ids, float* d_dists,
                     int32_t Q, int32_t k, int32_t policy, int32_t have_delete, void* stream,
                     coral_stats* stats);

/* coral_search_gpu for callers that cannot allocate device memory (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc).  No counterpart in the reference, whose search allocates on every call
 * (src/index_gpu.cpp:120-124, src/search_gpu.cu:846-852).  No coral_search_prepare is needed and none of its
 * scratch is used: the work counter, the per-query counters and the per-workgroup overflow bitmaps live in a fixed
 * 32.5 MiB block of device memory inside the library's code object (each GPU that loads the library holds its
 * copy until the process ends).  The call makes no allocation of any kind, records only kernels on `stream`
 * (NULL = the index's own) and returns without waiting for them; both policies run on the workgroup-per-query
 * kernel, with the results of coral_search_gpu bit for bit.  Rows are screened on a smaller copy of the vectors
 * (rounds policy) only where an earlier coral_search_prepare on this index has made that copy.  Limits (CORAL_ERR_ARG beyond them): Q <= 16384,
 * n <= 4194304, L <= CORAL_MAX_LDS_BEAM.  Every call on a GPU shares that GPU's block: calls that overlap on one
 * GPU (two streams, two indexes, two threads) race; order them. */
CORAL_API int coral_search_gpu_noalloc(coral_index* idx, const float* d_queries, int32_t* d_ids, float* d_dists,
                                       int32_t Q, int32_t k, int32_t L, int32_t policy, int32_t have_delete,
                                       void* stream);

/* Per-query counters of the last coral_search_gpu call, int32 [Q][4] on the
 * host: hops, expansions, dist_evals, rounds. */
CORAL_API int coral_search_query_counters(coral_index* idx, int32_t* host_out, int32_t Q);

/* What the last coral_search_gpu call read per query, by class, int32 [Q][4] on the host: rows measured on the
 * smaller copy of the vectors, fp32 vector rows read, 32-bit words of beam state moved in global memory, visited-state
 * requests to global memory.  Every distance evaluation reads one row of one or both kinds: screened_rows +
 * exact_rows >= dist_evals >= exact_rows.  No counterpart in the reference (which reads the fp32 row for every
 * evaluation, include/utils.cuh:254-275); these counts price the launch's memory traffic. */
CORAL_API int coral_search_row_counters(coral_index* idx, int32_t* host_out, int32_t Q);

/* The launch geometry the last coral_search_prepare chose (what a search call on this index runs with). */
typedef struct {
    int32_t kernel;          /* 0 beam_search_kernel (workgroup per query), 1 best_first_wave_kernel, 2 best_first_long_kernel */
    int32_t threads;         /* per workgroup */
    int32_t workgroups;      /* persistent workgroups (the wavefront kernels: query slots / 4) */
    int32_t lds_bytes;       /* per workgroup */
    int32_t screening;       /* 0 none, 1 half precision, 2 eight-bit codes */
    int32_t screen_row_bytes;/* bytes of one row of the smaller copy (0 without screening) */
    int32_t visited_form;    /* 0 table of 16-bit cells in LDS + bitmap in global memory, 1 bitmap of all ids in LDS,
                                2 bytes per node and slot in global memory, 3 packed words in global memory,
                                4 table of 16-bit cells in LDS in front of form 2 or 3, 5 form 0 with the table in
                                its bucket form (three candidate buckets of four cells per id) */
    int32_t visited_slots_log2; /* cells of the LDS table (forms 0 and 4), else 0 */
    int32_t beam_in_hbm;     /* the beam (or the long run) lives in global memory */
    int32_t todo_cap, cand_cap; /* LDS list capacities of the workgroup kernel */
    int32_t query_slots;     /* queries in flight */
    int32_t reserved[4];
} coral_plan_info;
CORAL_API int coral_search_plan_info(const coral_index* idx, coral_plan_info* out);

/* IndexGPU::Search (src/index_gpu.cpp:117-136): host buffers in and out; uploads
 * the queries, prepares for (Q, L), searches, downloads ids (and distances when
 * h_dists is not NULL). */
CORAL_API int coral_search(coral_index* idx, const float* h_queries, int32_t Q, int32_t k, int32_t L,
                 int32_t policy, int32_t have_delete, int32_t* h_ids, float* h_dists,
                 coral_stats* stats);

/* GPUFuncs::search_verify / ids_verify_kernel (src/search_gpu.cu:888-922):
 * hits = sum over queries of |res[q][0..k) n gt[q][0..k)|, both device arrays
 * with row stride k. */
CORAL_API int coral_search_verify(coral_index* idx, const int32_t* d_ids_res, const int32_t* d_ids_gt,
                        int32_t Q, int32_t k, int64_t* hits);

/* Exact k nearest neighbours of Q queries among the index's vectors by brute force:
 * what the reference gets from faiss for ground truth (tests/comp_gt.cpp:119-176) and for
 * the builder's k_b-NN (src/knn.cu:174-193).  Ordered by (distance, id); every distance is
 * accumulated in dimension order by fused multiply-adds, the arithmetic of
 * include/utils.cuh:254-275 / :307-323.  have_delete leaves tombstoned ids out.  Unfilled
 * slots: id -1, +-FLT_MAX.  The *_gpu form takes device pointers (d_dists may be NULL). */
CORAL_API int coral_bruteforce_knn_gpu(coral_index* idx, const float* d_queries, int32_t Q, int32_t k,
                                       int32_t have_delete, int32_t* d_ids, float* d_dists, void* stream,
                                       double* time_s);
CORAL_API int coral_bruteforce_knn(coral_index* idx, const float* h_queries, int32_t Q, int32_t k,
                                   int32_t have_delete, int32_t* h_ids, float* h_dists, double* time_s);
/* The search first screens all pairs with approximate distances from the matrix cores, keeps k + 32 candidates per
 * query, measures those in the reference's summation order and sends the rare query whose candidates cannot vouch
 * for the result through the plain passes: same ids and distance bits either way.  The candidates are selected
 * inside the matrix-core kernel (entries up to a per-query bound, taken from a sample of the base, go to a short
 * list per query; no distance matrix is written); where that does not apply -- k + 32 > 1024, a base of fewer than
 * 64 sample tiles, a list that overflows -- the screening goes through the distance matrix instead.  on = 1 skips
 * the screening (every pair in the reference's order on the vector units); on = 2 keeps the screening and always
 * goes through the distance matrix; on = 0 restores the default.  No counterpart in the reference (faiss does this
 * work there). */
CORAL_API int coral_bruteforce_set_exact_only(coral_index* idx, int32_t on);
/* 1 if the candidates of the last coral_bruteforce_knn* call were selected inside the matrix-core kernel */
CORAL_API int32_t coral_bruteforce_last_fused(coral_index* idx);
/* queries of the last coral_bruteforce_knn* call that went through the plain passes after the screening */
CORAL_API int64_t coral_bruteforce_last_redone(coral_index* idx);

/* Entry points by farthest-point sampling in hop distance, Graph::FPS (src/start.cu:74-145): out_ids[0] =
 * first_id; each further id is the node whose smallest hop count from the ids chosen so far is largest
 * (lowest id on ties; nodes unreachable from them are never chosen).  The reference draws first_id from
 * std::random_device among nodes with a non-empty row; here the caller names it.  Writes M ids. */
CORAL_API int coral_start_ids_fps(coral_index* idx, int32_t first_id, int32_t M, int32_t* out_ids);

/* ---- Graph construction from auxiliary queries (IndexGPU::BuildGPU, src/index_gpu.cpp:308-383) ----
 * Rows under construction live in the index itself, so a search may run at any point of a build (the
 * connectivity enhancement does).  Two outcomes that the reference leaves to thread timing are fixed here:
 * equal distances keep the order in which the candidates were listed (cluster order, then the current row),
 * and a node that several clusters (or several isolated nodes) of one batch claim goes to the first of them. */
/* The search the reference runs on a set of test queries while a graph grows, GPUFuncs::test_search
 * (include/gpufuncs.cuh:688-702: search_prepare(TEST_SEARCH_QUERY_SIZE, test_beam_capacity), Search with the current
 * start ids, search_verify against the test queries' true neighbours): called every test_search_frequency batches
 * (src/index_gpu.cpp:525-570), after the isolated nodes were attached (src/enhance.cu:814), after every search batch
 * of the most-hit nodes (src/enhance.cu:852) and on the finished graph (src/index_gpu.cpp:376-378).  It changes
 * nothing in the graph.  `report` is called once per such search, from the thread that runs the build. */
#define CORAL_MONITOR_BATCHES 0  /* done = auxiliary queries consumed so far, total = all of them */
#define CORAL_MONITOR_ISOLATED 1 /* done = total = isolated nodes attached */
#define CORAL_MONITOR_TOP 2      /* done = most-hit nodes gone over so far, total = all of them */
#define CORAL_MONITOR_DONE 3     /* the finished graph (only with connect_enhance, as in the reference) */
typedef void (*coral_build_report_fn)(void* user, int32_t phase, int64_t done, int64_t total, const coral_stats* search,
                                      int64_t hits);
typedef struct {
    const float* h_queries; /* host [Q][dim]: test_query_data */
    const int32_t* h_gt;    /* host [Q][k]: test_query_knns, the k true nearest of each */
    int32_t Q;              /* TEST_SEARCH_QUERY_SIZE (the reference: config.json "batch") */
    int32_t k;              /* gtk */
    int32_t L;              /* config.json "test_beam_capacity" (512) */
    int32_t reserved;
    coral_build_report_fn report; /* search->hops / Q = Test_Result::avg_hops, 100 hits / (Q k) = calc_recall */
    void* user;
} coral_build_monitor;

typedef struct {
    int32_t R;                    /* row width, <= 32: --M_pjbp, tests/test_build_pipeline.cpp:82 */
    int32_t k_b;                  /* nearest base points per auxiliary query, 2..128: config.json "k" */
    int32_t batch;                /* auxiliary queries per update: config.json "batch" (1024) */
    int32_t need_discard;         /* fill rows with the nearest ruled-out candidates: config.json "need_discard" */
    int32_t connect_enhance;      /* --CE: 0 = leave untouched nodes isolated, 1 = attach them afterwards */
    int32_t enhance_search_batch; /* config.json "enhance_search_batch" (524288) */
    int32_t enhance_nap_batch;    /* config.json "enhance_nap_batch" (4096) */
    int32_t enhance_L;            /* beam capacity of the enhancement search: 256, src/enhance.cu:783 */
    int32_t n_start;              /* entry points: config.json "search_start_nodes_num" (16) */
    int32_t first_start_id;       /* first id of the farthest-point sampling (the reference draws it from
                                     std::random_device, src/start.cu:77-86); -1 = lowest id that has neighbours */
    int32_t top_hit_num;          /* config.json "top_hit_num": after the isolated nodes, the (top_hit_num - isolated)
                                     nodes that most clusters contain are searched for and rewired too; 0 (the code's
                                     default, src/index_gpu.cpp:78) = no such phase */
    int32_t test_search_frequency; /* config.json "test_search_frequency" (100): a monitor search after every batch
                                      whose number (from 0) is a positive multiple of it; 0 = none during the batches */
    const coral_build_monitor* monitor; /* NULL (the default) = no test searches */
    int32_t reserved[2];
} coral_build_params;

typedef struct {
    double knn_s;      /* exact k_b-NN of the auxiliary queries */
    double nap_s;      /* batch updates */
    double enhance_s;  /* connectivity enhancement, entry points included */
    double total_s;
    int64_t batches;
    int64_t isolated;          /* nodes without neighbours after the batch updates */
    int64_t reverse_edges;     /* isolated nodes inserted into rows of the nodes found for them */
    int64_t reverse_rejected;  /* ... turned away by a full row */
    int64_t edges;             /* sum of degrees at the end */
    int64_t top_hit_nodes;     /* nodes the second enhancement phase went over */
    int64_t top_reverse_edges; /* reverse edges of that phase */
} coral_build_stats;

/* the values of the reference's config.json and CLI defaults */
CORAL_API int coral_build_params_default(coral_build_params* p);

/* Graph ctor in construction mode: every row empty.  On a vectors-only index this creates the rows. */
CORAL_API int coral_build_begin(coral_index* idx, int32_t R);
/* frees the per-neighbour distances and the staging; the rows and start ids stay */
CORAL_API int coral_build_end(coral_index* idx);

/* Graph ctor in Mode::CE (include/graph.cuh:252-256, DS.load_batch_slots of every node): construction state from
 * rows of an earlier build, as coral_index_get_graph handed them out before coral_build_end (h_nbrs [n][R] with -1
 * after the last neighbour, h_dists [n][R] the neighbours' distances), and the per-node cluster counts (h_hits [n], or
 * NULL for zeros; IVFBuilder::load_hits, include/ivf.cuh:647-656).  coral_build_connect_enhance can follow. */
CORAL_API int coral_build_resume(coral_index* idx, int32_t R, const int32_t* h_nbrs, const float* h_dists,
                                 const uint32_t* h_hits);

/* GPUFuncs::graph_update -> gpu_neibor_aware (src/upd_disk.cu:218-224, src/upd_gpu.cu:260-303): one batch of
 * clusters, d_knn_ids int32 [batch][k_b] on the device, distinct ids per row.  Every member becomes a pivot:
 * candidates = the other members (pairs where both sides already have neighbours are left out) + its current row;
 * sorted by distance; occlusion rule; write-back (with need_discard, filled up to R with the nearest ruled-out). */
CORAL_API int coral_build_nap_batch(coral_index* idx, const int32_t* d_knn_ids, int32_t batch, int32_t k_b,
                                    int32_t need_discard);

/* GPUFuncs::enhance_neibor_aware_gpu (src/enhance.cu:660-689): d_iso_ids [batch] nodes without neighbours,
 * d_knn_ids / d_knn_dists [batch][kn] what the search found for their vectors (closest first, -1 ends a list).
 * Each found node takes the first isolated node that lists it into its own row (src/enhance.cu:161-207); each
 * isolated node gets its row from its list through the occlusion rule, filled (src/enhance.cu:334-380, 519-575). */
CORAL_API int coral_build_enhance_batch(coral_index* idx, const int32_t* d_iso_ids, const int32_t* d_knn_ids,
                                        const float* d_knn_dists, int32_t batch, int32_t kn, int64_t* reverse_edges,
                                        int64_t* reverse_rejected);

/* GPUFuncs::gpu_connect_enhance, isolated nodes (src/enhance.cu:728-803, enhance_mode 0): per search batch, entry
 * points by coral_start_ids_fps on the graph as it is, one CORAL_POLICY_ROUNDS search (k = k_b, L = enhance_L) for
 * the isolated nodes' own vectors, then coral_build_enhance_batch per enhance_nap_batch.  The entry points of the
 * last search batch stay the index's start ids, as in the reference (fewer than n_start when fewer nodes can be
 * reached: an id is never listed twice).  Second phase (src/enhance.cu:819-856) when params->top_hit_num exceeds the
 * number of isolated nodes: the (top_hit_num - isolated) nodes of coral_build_top_hit_ids, capped at n (the reference
 * reads past its id array beyond that), go through the same search and coral_build_enhance_top_batch. */
CORAL_API int coral_build_connect_enhance(coral_index* idx, const coral_build_params* params, coral_build_stats* stats);

/* GPUFuncs::test_search by itself (include/gpufuncs.cuh:688-702): one search of params->monitor's queries from the
 * index's current start ids on the graph as it stands, reported through params->monitor->report with the phase and
 * progress given.  Does nothing without a monitor.  (IndexGPU::BuildGPU's closing call, src/index_gpu.cpp:376-378,
 * where the enhancement ran on a saved build.) */
CORAL_API int coral_build_test_search(coral_index* idx, const coral_build_params* params, int32_t phase, int64_t done,
                                      int64_t total);

/* The five-argument GPUFuncs::enhance_neibor_aware_gpu (src/enhance.cu:632-658, 58-129): d_top_ids [batch] nodes that
 * have rows, d_knn_ids / d_knn_dists [batch][k] what the search found for their vectors (the node itself included, as
 * in the reference).  A node's candidates are its found list followed by its current row; the found part inserts
 * reverse edges like coral_build_enhance_batch, and the node's row is rebuilt from all candidates.  Rows are read as
 * they were before the batch (the reference reads them while the same kernel changes them). */
CORAL_API int coral_build_enhance_top_batch(coral_index* idx, const int32_t* d_top_ids, const int32_t* d_knn_ids,
                                            const float* d_knn_dists, int32_t batch, int32_t k, int64_t* reverse_edges,
                                            int64_t* reverse_rejected);

/* get_top_hit_nodes (src/knn.cu:140-150): the top_n ids by the number of clusters of this build that contain them
 * (counted by coral_build_nap_batch as src/knn.cu:60-73 does), most first, equal counts by ascending id.  h_hits
 * (optional) receives the n counts. */
CORAL_API int coral_build_top_hit_ids(coral_index* idx, int64_t top_n, int32_t* h_ids, uint32_t* h_hits);

/* IndexGPU::BuildGPU: begin; exact k_b-NN of the A auxiliary queries (host, [A][dim]; what the reference asks faiss
 * for, src/knn.cu:174-193) in order, `batch` at a time through coral_build_nap_batch; then the enhancement (or, with
 * connect_enhance 0, just the entry points).  The index can be searched afterwards; call coral_build_end to drop the
 * construction state. */
CORAL_API int coral_build_graph(coral_index* idx, const float* h_aux, int64_t A, const coral_build_params* params,
                                coral_build_stats* stats);

/* The same with the clusters given instead of computed: h_clusters int32 [A][k_b], row i = the k_b nearest base
 * ids of auxiliary query i, distinct within a row (GraphTask's train_gt_file branch, src/index_gpu.cpp:505-537;
 * the payload of a ground-truth file of the auxiliary queries with k = k_b). */
CORAL_API int coral_build_graph_from_clusters(coral_index* idx, const int32_t* h_clusters, int64_t A,
                                              const coral_build_params* params, coral_build_stats* stats);

/* Download rows [n][R] (-1 padded) and start ids [n_start]; during a build also the per-neighbour distances
 * [n][R] and degrees [n] (the dists and deg fields of the reference's Slot).  Any pointer may be NULL. */
CORAL_API int coral_index_get_graph(coral_index* idx, int32_t* h_nbrs, float* h_dists, int32_t* h_deg,
                                    int32_t* h_start_ids);

/* What the device's memory delivers, for setting the search kernels' rates against (no counterpart in the
 * reference): allocates `bytes` of device memory (use far more than the 256 MB memory-side cache), reads all of it
 * once in 16-byte coalesced requests (*stream_gbps) and then as many bytes as rows of row_bytes from pseudo-random
 * places, one wavefront per row, eight rows in flight per wavefront (*gather_gbps: the access pattern of the distance
 * phase, one vector row per visited node, with no reuse for a cache to find).  Best of `reps` timed passes each
 * (HIP events), GB/s = 1e9 bytes per second.  Either pointer may be NULL. */
CORAL_API int coral_membench(int32_t device, size_t bytes, int32_t row_bytes, int32_t reps, double* stream_gbps,
                             double* gather_gbps);

#ifdef __cplusplus
}
#endif
#endif /* CORAL_SEARCH_H */
