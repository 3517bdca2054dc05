// coral_search.cpp -- the C ABI of include/coral_search.h over the HIP kernels of
// beam_search.hip.  Host code only; every device allocation of the search path
// is made here.  There is no CPU fallback: without a usable HIP device every
// entry point that needs one fails with CORAL_ERR_DEVICE.
#include "coral_search.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <string>
#include <vector>

#include "beam_search.h"
#include "error.h"
#include "index_internal.h"

namespace {
thread_local std::string g_err;
}

namespace coral {
int fail(int code, const char* fmt, ...) {
    char buf[768];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}
}  // namespace coral

namespace {
using coral::fail;

constexpr int kMaxL = CORAL_MAX_BEAM;  // beams beyond CORAL_MAX_LDS_BEAM live in global memory
constexpr int kMaxLdsBytes = 160 * 1024;
constexpr int kStaticLds = 128;  // what the workgroup kernel declares outside its dynamic block (counts, per-wave sums)
constexpr int kLongBeamFrom = 1280;  // best-first: beams longer than this take the long-beam kernel

// bits of a mixed id that a cell of the wavefront kernel's table stores: what the bucket index (a quarter of the
// cells) does not imply; a cell has room for 14
int bf_table_rem_bits(int id_bits, int table_log2) { return std::max(0, id_bits - (table_log2 - 2)); }

// First level of the visited set of the wavefront-per-query best-first kernel: an exact table of 16-bit cells per
// wavefront in LDS, where one that holds most of a query's first visits (20 to 30 per beam entry) still leaves a CU
// eight wavefronts -- what the HBM-resident state costs in requests is worth more than the wavefronts given up.
// Sixteen wavefronts if 24 cells per entry fit with them, else twelve, else eight with 20 cells per entry; no table
// (0) for longer beams, or when the ids are wider than a cell can tell apart.  wanted: the caller's
// coral_tuning.best_first_table_log2.
int choose_bf_table(int L, int id_bits, int wanted, int* table_log2) {
    *table_log2 = 0;
    if (wanted > 0) {
        if (wanted < 8 || wanted > 14 || coral::best_first_wave_lds_bytes(L, 0, wanted) * 4 > (size_t)kMaxLdsBytes)
            return fail(CORAL_ERR_ARG, "best_first_table_log2 must be in 8..14 and fit LDS with the beam");
        if (bf_table_rem_bits(id_bits, wanted) > 14)
            return fail(CORAL_ERR_ARG, "ids of %d bits do not fit the cells of a 2^%d table", id_bits, wanted);
        *table_log2 = wanted;
    } else if (wanted == 0) {
        const struct { int waves, cells_per_entry; } plans[] = {{16, 24}, {12, 24}, {8, 20}};
        for (const auto& pl : plans)
            for (int lg = 14; lg >= 10 && !*table_log2; --lg)
                if (coral::best_first_wave_lds_bytes(L, 0, lg) * pl.waves <= (size_t)kMaxLdsBytes &&
                    (1 << lg) >= pl.cells_per_entry * L && bf_table_rem_bits(id_bits, lg) <= 14)
                    *table_log2 = lg;
    }
    return CORAL_OK;
}

}  // namespace

// Before a buffer that a search kernel reads is freed or rewritten: wait for the index's own stream and, if the entry
// point that returns without waiting has been used, for everything on the device (its launches run on streams of the
// caller's choosing).
static hipError_t quiesce(coral_index* idx) {
    hipError_t e = idx->stream ? hipStreamSynchronize(idx->stream) : hipSuccess;
    if (e == hipSuccess && idx->noalloc_in_flight) {
        e = hipDeviceSynchronize();
        idx->noalloc_in_flight = false;
    }
    return e;
}

extern "C" {

const char* coral_last_error(void) { return g_err.c_str(); }

static int validate_graph(const int32_t* nbrs, int64_t n, int R, const int32_t* start_ids,
                          int n_start) {
    if (n_start <= 0 || !start_ids) return fail(CORAL_ERR_ARG, "no start ids");
    for (int i = 0; i < n_start; ++i) {
        if (start_ids[i] < 0 || start_ids[i] >= n)
            return fail(CORAL_ERR_GRAPH, "start id %d out of range [0,%lld)", start_ids[i],
                        (long long)n);
        for (int j = 0; j < i; ++j)
            if (start_ids[i] == start_ids[j])
                return fail(CORAL_ERR_GRAPH, "duplicate start id %d", start_ids[i]);
    }
    int64_t bad_node = -1;
    int bad_kind = 0;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const int32_t* row = nbrs + i * R;
        bool ended = false;
        for (int j = 0; j < R; ++j) {
            const int32_t v = row[j];
            if (v < 0) {
                ended = true;
            } else if (ended || v >= n) {
#pragma omp critical
                if (bad_node < 0) bad_node = i, bad_kind = ended ? 1 : 2;
            }
        }
    }
    if (bad_node >= 0)
        return fail(CORAL_ERR_GRAPH,
                    bad_kind == 1 ? "node %lld: neighbour after the end-of-row marker"
                                  : "node %lld: neighbour id out of range",
                    (long long)bad_node);
    return CORAL_OK;
}

int coral_index_create(const coral_index_desc* d, coral_index** out) {
    if (!d || !out) return fail(CORAL_ERR_ARG, "null argument");
    *out = nullptr;
    if (!d->base) return fail(CORAL_ERR_ARG, "null base");
    const bool vectors_only = d->nbrs == nullptr;  // enough for coral_bruteforce_knn*
    if (d->n <= 0 || d->n > 0x7fffffffLL) return fail(CORAL_ERR_ARG, "n out of range");
    if (d->dim <= 0 || d->dim % 4 != 0 || d->dim > 2048)
        return fail(CORAL_ERR_ARG, "dim must be a positive multiple of 4, at most 2048 (got %d)",
                    d->dim);
    if (d->metric != CORAL_L2 && d->metric != CORAL_IP) return fail(CORAL_ERR_ARG, "bad metric");
    if (!vectors_only) {
        if (d->R <= 0 || d->R > 32) return fail(CORAL_ERR_ARG, "R must be in 1..32 (got %d)", d->R);
        if (int rc = validate_graph(d->nbrs, d->n, d->R, d->start_ids, d->n_start)) return rc;
    }

    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev <= 0)
        return fail(CORAL_ERR_DEVICE, "no HIP device (%s)", hipGetErrorString(e));
    if (d->device < 0 || d->device >= ndev) return fail(CORAL_ERR_ARG, "device ordinal out of range");
    HIP_TRY(hipSetDevice(d->device));

    coral_index* idx = new (std::nothrow) coral_index();
    if (!idx) return fail(CORAL_ERR_MEMORY, "host allocation failed");
    idx->device = d->device, idx->n = d->n, idx->dim = d->dim, idx->R = vectors_only ? 0 : d->R;
    idx->M = vectors_only ? 0 : d->n_start, idx->metric = d->metric;
    hipDeviceProp_t prop;
    auto cleanup = [&](int rc) {
        coral_index_destroy(idx);
        return rc;
    };
#define HIP_TRY_C(expr)                                                                      \
    do {                                                                                     \
        hipError_t e_ = (expr);                                                              \
        if (e_ != hipSuccess)                                                                \
            return cleanup(fail(e_ == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE, \
                                "%s failed: %s", #expr, hipGetErrorString(e_)));             \
    } while (0)
    HIP_TRY_C(hipGetDeviceProperties(&prop, d->device));
    idx->num_cu = prop.multiProcessorCount;
    HIP_TRY_C(hipStreamCreate(&idx->stream));
    HIP_TRY_C(coral::static_scratch_init(d->device));  // address of the fixed scratch block on this device
    const size_t vec_bytes = (size_t)d->n * d->dim * sizeof(float);
    const size_t nbr_bytes = vectors_only ? 0 : (size_t)d->n * d->R * sizeof(int32_t);
    HIP_TRY_C(hipMalloc(&idx->d_vec, vec_bytes));
    if (!vectors_only) {
        HIP_TRY_C(hipMalloc(&idx->d_nbrs, nbr_bytes));
        HIP_TRY_C(hipMalloc(&idx->d_start, (size_t)d->n_start * sizeof(int32_t)));
    }
    HIP_TRY_C(hipMalloc(&idx->d_scalars, 4 * sizeof(int)));
    HIP_TRY_C(hipMalloc(&idx->d_hit, sizeof(unsigned long long)));
    HIP_TRY_C(hipMemcpy(idx->d_vec, d->base, vec_bytes, hipMemcpyHostToDevice));
    if (!vectors_only) {
        HIP_TRY_C(hipMemcpy(idx->d_nbrs, d->nbrs, nbr_bytes, hipMemcpyHostToDevice));
        HIP_TRY_C(hipMemcpy(idx->d_start, d->start_ids, (size_t)d->n_start * sizeof(int32_t),
                            hipMemcpyHostToDevice));
    }
#undef HIP_TRY_C
    *out = idx;
    return CORAL_OK;
}

void coral_index_destroy(coral_index* idx) {
    if (!idx) return;
    (void)hipSetDevice(idx->device);
    (void)quiesce(idx);
    (void)hipFree(idx->d_vec);
    (void)hipFree(idx->d_nbrs);
    (void)hipFree(idx->d_start);
    (void)hipFree(idx->d_deleted);
    (void)hipFree(idx->d_spill);
    (void)hipFree(idx->d_beam);
    (void)hipFree(idx->d_vec16);
    (void)hipFree(idx->d_vec8);
    (void)hipFree(idx->d_counters);
    (void)hipFree(idx->d_scalars);
    (void)hipFree(idx->d_hit);
    (void)hipFree(idx->d_phase);
    (void)hipFree(idx->d_bf_visited);
    (void)hipFree(idx->d_bf_epochs);
    (void)hipFree(idx->d_bf_beams);
    (void)hipFree(idx->d_bnorm);
    (void)hipFree(idx->d_bnorm_max);
    (void)hipFree(idx->d_io_q);
    (void)hipFree(idx->d_io_ids);
    (void)hipFree(idx->d_io_dists);
    for (hipEvent_t e : idx->ev)
        if (e) (void)hipEventDestroy(e);
    coral::free_build_state(idx);
    if (idx->h_counters) (void)hipHostFree(idx->h_counters);
    if (idx->stream) (void)hipStreamDestroy(idx->stream);
    delete idx;
}

int coral_index_set_graph(coral_index* idx, const int32_t* nbrs, const int32_t* start_ids,
                          int32_t n_start) {
    if (!idx || !nbrs) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->d_nbrs) return fail(CORAL_ERR_STATE, "the index holds vectors only (no graph was given)");
    if (int rc = validate_graph(nbrs, idx->n, idx->R, start_ids, n_start)) return rc;
    HIP_TRY(hipSetDevice(idx->device));
    HIP_TRY(quiesce(idx));
    idx->noalloc_L = 0;  // (a plan depends on the number of start ids)
    if (n_start != idx->M) {
        int32_t* p = nullptr;
        HIP_TRY(hipMalloc(&p, (size_t)n_start * sizeof(int32_t)));
        (void)hipFree(idx->d_start);
        idx->d_start = p;
        idx->M = n_start;
        idx->prepared = false;
    }
    idx->rows_unique = -1;
    HIP_TRY(hipMemcpy(idx->d_nbrs, nbrs, (size_t)idx->n * idx->R * sizeof(int32_t),
                      hipMemcpyHostToDevice));
    HIP_TRY(hipMemcpy(idx->d_start, start_ids, (size_t)n_start * sizeof(int32_t),
                      hipMemcpyHostToDevice));
    return CORAL_OK;
}

int coral_index_set_deleted(coral_index* idx, const uint32_t* host_mask) {
    if (!idx) return fail(CORAL_ERR_ARG, "null index");
    HIP_TRY(hipSetDevice(idx->device));
    HIP_TRY(quiesce(idx));
    if (!host_mask) {
        (void)hipFree(idx->d_deleted);
        idx->d_deleted = nullptr;
        return CORAL_OK;
    }
    const size_t words = ((size_t)idx->n + 31) / 32;
    if (!idx->d_deleted) HIP_TRY(hipMalloc(&idx->d_deleted, words * sizeof(uint32_t)));
    HIP_TRY(hipMemcpy(idx->d_deleted, host_mask, words * sizeof(uint32_t), hipMemcpyHostToDevice));
    return CORAL_OK;
}

int coral_index_info(const coral_index* idx, int64_t* n, int32_t* dim, int32_t* R, int32_t* n_start,
                     int32_t* metric) {
    if (!idx) return fail(CORAL_ERR_ARG, "null index");
    if (n) *n = idx->n;
    if (dim) *dim = idx->dim;
    if (R) *R = idx->R;
    if (n_start) *n_start = idx->M;
    if (metric) *metric = idx->metric;
    return CORAL_OK;
}

// Size (log2 of the cells) of the visited table for ids that leave a 16-bit cell little room: see plan_search.
// want: the size the load asks for; choices: the caller's coral_tuning.visited_choices.
static int size_for_wide_ids(int want, int id_bits, int choices, bool* three) {
    *three = false;
    if (choices != 1) {
        // the bucket form wherever its cells have room for the ids at the size the load asks for (it is the faster
        // form at any load: three reads side by side against a probe sequence: +7 % at L = 256 on a million nodes);
        // at a larger size only for ids that would leave linear probing short displacements, or when asked for
        int w3 = want;
        while (w3 < 16 && id_bits - (w3 - 2) > 14) ++w3;
        if (id_bits - (w3 - 2) <= 14 && (w3 == want || choices == 3 || id_bits - want > 11)) {
            *three = true;
            return w3;
        }
    }
    while (want < 16 && id_bits - want > 11) ++want;
    return want;
}

// Launch geometry of the workgroup-per-query kernel for a beam of capacity L: arithmetic, the kernel's LDS
// attribute and an occupancy query; nothing is allocated.  bump_log2 raises the library's own choice of table size.
static int plan_search(const coral_index* idx, int32_t Q, int32_t L, const coral_tuning& t, int bump_log2,
                       bool lds_beam_only, bool no_screen, coral_search_plan* out) {
    if (Q <= 0) return fail(CORAL_ERR_ARG, "Q must be positive");
    if (L <= 0 || L > kMaxL) return fail(CORAL_ERR_ARG, "L must be in 1..%d (got %d)", kMaxL, L);
    if (idx->M <= 0) return fail(CORAL_ERR_STATE, "the graph has no start ids yet (rows under construction)");
    if (idx->M > L)
        return fail(CORAL_ERR_ARG, "%d start ids do not fit a beam of capacity %d", idx->M, L);
    if (t.policy != CORAL_POLICY_ROUNDS && t.policy != CORAL_POLICY_BEST_FIRST)
        return fail(CORAL_ERR_ARG, "unknown policy %d", t.policy);
    const bool best_first = t.policy == CORAL_POLICY_BEST_FIRST;
    coral_search_plan p;
    p.L = L;
    p.big = L > CORAL_MAX_LDS_BEAM || t.beam_in_hbm != 0;
    // todo / candidate buffers: at least what the start ids and four graph rows need
    int min_cap = 256;
    while (min_cap < idx->M || min_cap < idx->R * 4) min_cap <<= 1;
    int id_bits = 1;
    while (id_bits < 31 && ((int64_t)1 << id_bits) < idx->n) ++id_bits;
    const size_t lds_max = (size_t)kMaxLdsBytes;
    // ---- screening on a smaller copy of the vectors (rounds policy, L2, rows of 132 .. 2048 floats): eight-bit codes
    // (tuning 2; the library's choice up to 512 floats) or half precision (tuning 1); see beam_search.hip
    // (best-first: the wavefront-per-query kernel with the beam in LDS screens too, see coral_search_prepare)
    // (the inner product is screened on codes only)
    const bool codes_possible = idx->dim <= (best_first ? coral::kMaxByteRowDim : coral::kMaxByteRowDimRounds);
    // (the rounds kernel takes codes for rows of more than 64 floats; half precision, and the best-first kernels,
    // need more than 128)
    const bool wide = idx->dim / 4 > 32, codes_wide = idx->dim / 4 > 16;
    const bool screen_possible = !best_first && ((wide && idx->metric == CORAL_L2) || ((wide || codes_wide) && codes_possible));
    if (t.screening > 2 || t.screening < -1) return fail(CORAL_ERR_ARG, "screening must be -1, 0, 1 or 2 (got %d)", t.screening);
    if (t.screening > 0 && !wide && !(t.screening == 2 && codes_wide))
        return fail(CORAL_ERR_ARG, "screening needs more than 128 dimensions (on eight-bit codes: more than 64)");
    if (t.screening == 1 && idx->metric != CORAL_L2)
        return fail(CORAL_ERR_ARG, "screening in half precision needs the L2 metric");
    if (t.screening == 2 && !codes_possible)
        return fail(CORAL_ERR_ARG, "screening on eight-bit codes takes rows of up to %d floats",
                    best_first ? coral::kMaxByteRowDim : coral::kMaxByteRowDimRounds);
    // (by itself the library screens rows of more than 128 floats only: at 128 floats and the short beam of the
    // configuration that has such rows, the codes cost 9 %)
    const bool screen = screen_possible && (t.screening > 0 || (t.screening == 0 && !no_screen && wide));
    // (the library's own choice: codes, except for L2 rows of more than 1024 floats, where the kernel form that keeps
    // eight chunks of codes per lane is no faster than half precision: 103 k against 106 k QPS at 2048 floats, after
    // 382 k against 291 k at 1024)
    p.screen = !screen ? 0 : t.screening > 0 ? t.screening : (codes_possible && (idx->dim <= 1024 || idx->metric != CORAL_L2) ? 2 : 1);
    // ---- the visited structure.  Three forms: a table of 2^s 16-bit cells with an overflow bitmap in global memory
    // (visited_slots_log2 = s, or the library's choice), or a plain bitmap of all n ids in LDS (visited_slots_log2 =
    // -1, or the library's choice): one LDS atomic per test and nothing ever overflows, at n / 8 bytes -- 125 KB for
    // a million nodes, which leaves a CU one workgroup.
    const int bitmap_words = (int)(((idx->n + 31) / 32 + 3) & ~(int64_t)3);
    auto lds_bitmap = [&](bool big, int cap) {
        return coral::search_lds_bytes(L, idx->dim, bitmap_words, cap, cap, 4, big, screen) + kStaticLds;
    };
    auto lds_table = [&](bool big, int lg, int cap) {
        return coral::search_lds_bytes(L, idx->dim, (1 << lg) >> 1, cap, cap, 256, big, screen) + kStaticLds;
    };
    const bool bitmap_possible = idx->n <= ((int64_t)1 << 21);
    if (t.visited_choices != 0 && t.visited_choices != 1 && t.visited_choices != 3 && t.visited_choices != 4)
        return fail(CORAL_ERR_ARG, "visited_choices must be 0, 1, 3 or 4 (got %d)", t.visited_choices);
    const int choices = t.visited_choices == 4 ? 3 : t.visited_choices;  // (4: the bucket form as tests want it)
    bool three = false;  // the table of cells in its bucket form
    int slots_log2 = t.visited_slots_log2;
    if (slots_log2 == -1) {
        if (!bitmap_possible || lds_bitmap(p.big, min_cap) > lds_max)
            return fail(CORAL_ERR_ARG, "a bitmap of %lld ids does not fit LDS beside a beam of %d", (long long)idx->n, L);
        p.direct = 1;
    } else if (slots_log2 == 0 && !best_first) {
        // the table the rounds policy wants: a degree-32 graph over a million nodes sees about 75 first visits per
        // beam entry, 112 cells per entry keep the load factor near 0.65; `bump_log2` doubles that after batches
        // that overflowed (see coral_search_gpu)
        int want = 12;
        while ((1 << want) < 112 * L && want < 20) ++want;
        // A 16-bit cell of a 2^s table keeps id_bits - s bits of the id and has the rest for the displacement: beyond
        // 2^24 ids a table sized for the load alone carries displacements of 14 or fewer, and a few ids of every
        // query would leave LDS for the bitmap in global memory.  Such launches take the table in its bucket form
        // (three candidate buckets of four cells per id: no displacement to carry, 14 bits of the id per cell), at the
        // size the load asks for where the cells have room for the ids; or else the table that carries 30.
        want = size_for_wide_ids(want, id_bits, choices, &three);
        want += bump_log2;
        const bool table_holds = !p.big && want <= 16 && lds_table(false, want, min_cap) <= lds_max;
        const bool table_alone_on_cu = table_holds && lds_table(false, want, min_cap) > lds_max / 2;
        if (bitmap_possible && !p.big && lds_bitmap(false, min_cap) <= lds_max && (!table_holds || table_alone_on_cu)) {
            p.direct = 1;  // one workgroup per CU either way: the bitmap is the cheaper test and cannot overflow
        } else if (bitmap_possible && !table_holds && !lds_beam_only && lds_bitmap(true, 1024) <= lds_max) {
            p.direct = 1, p.big = true;  // the beam gives its LDS to the bitmap (measured: +30 % at L = 1024 and 2048)
        } else {
            slots_log2 = std::min(16, want);
            while (slots_log2 > 12 && lds_table(p.big, slots_log2, min_cap) > lds_max) --slots_log2;
        }
    } else if (slots_log2 == 0) {
        // best-first on this kernel: about 31 first visits per beam entry, 48 cells
        if (p.big && bitmap_possible && lds_bitmap(true, min_cap) <= lds_max) {
            p.direct = 1;
        } else {
            slots_log2 = 12;
            while ((1 << slots_log2) < 48 * L && slots_log2 < 16) ++slots_log2;
            slots_log2 = size_for_wide_ids(slots_log2, id_bits, choices, &three);  // (as above)
            slots_log2 = std::min(16, slots_log2 + bump_log2);
            while (slots_log2 > 12 && lds_table(p.big, slots_log2, min_cap) > lds_max) --slots_log2;
        }
    }
    int ocap = 256;
    if (!p.direct) {
        if (slots_log2 < 10 || slots_log2 > 16)
            return fail(CORAL_ERR_ARG, "visited_slots_log2 must be -1 or in 10..16");
        const int slots = 1 << slots_log2;
        p.slots_log2 = slots_log2, p.table_words = slots >> 1;
        p.rem_bits = std::max(0, id_bits - slots_log2);
        // a cell is 1 + ((d << rem_bits) | remainder) in 16 bits
        p.dmax = p.rem_bits >= 16 ? -1 : std::min(63, (65535 >> p.rem_bits) - 1);
        p.vis_limit = p.dmax < 0 ? 0 : slots - slots / 4;
        // the bucket form: a cell is 1 + ((choice << rem_bits) | remainder), the remainder what the bucket index (a
        // quarter of the cells) does not imply; a lookup costs the same whatever the load, so nothing is frozen
        const int rem3 = std::max(0, id_bits - (slots_log2 - 2));
        if (choices == 3 && t.visited_slots_log2 > 0) three = true;
        if (three && rem3 > 14) {
            if (choices == 3)
                return fail(CORAL_ERR_ARG, "ids of %d bits do not fit the cells of a 2^%d table in its bucket form", id_bits,
                            slots_log2);
            three = false;  // (LDS had no room for the size that was asked for)
        }
        if (three) p.choices = t.visited_choices == 4 ? 4 : 3, p.rem_bits = rem3, p.dmax = 0, p.vis_limit = 0x7fffffff;
        p.spill_words = ((size_t)idx->n + 31) / 32;
    } else {
        p.table_words = bitmap_words, ocap = 4;
        p.dmax = -1, p.vis_limit = 0x7fffffff;
    }
    // ---- todo and candidate buffers (powers of two: the candidates are bitonic-sorted in place).  Larger chunks
    // mean fewer latency-bound steps per round: the largest that does not lower the number of workgroups a CU can
    // hold; a launch that is alone on its CU anyway takes a candidate buffer of twice the size where there is room
    // (half as many merges of a long beam).  Best-first expands one row at a time and needs neither.
    auto lds_for = [&](int tc, int cc) {
        return coral::search_lds_bytes(L, idx->dim, p.table_words, tc, cc, ocap, p.big, screen) + kStaticLds;
    };
    if (lds_for(min_cap, min_cap) > lds_max)
        return fail(CORAL_ERR_ARG, "L=%d with %d words of visited state needs %zu bytes of LDS", L, p.table_words,
                    lds_for(min_cap, min_cap));
    int tcap = min_cap;
    const int wg_fit = (int)(lds_max / lds_for(min_cap, min_cap));
    for (int cap : {2048, 1024, 512}) {
        if (cap <= tcap || best_first) break;
        // (twice the ids of one pass of 1024 threads: a screening collects the ids of several chunks, see
        // beam_search.hip; for beams in global memory only -- with a beam in LDS the candidate buffer would double
        // with the list, the beam's worst entry be refreshed half as often, and a 512-float inner-product search at
        // L = 256 lost 5 %)
        if (cap == 2048 && !(screen && wg_fit == 1 && p.big)) continue;
        if (lds_for(cap, cap) <= lds_max && (int)(lds_max / lds_for(cap, cap)) >= std::min(wg_fit, 2)) {
            tcap = cap;
            break;
        }
    }
    int ccap = tcap;
    if (t.cand_cap > 0) {
        if ((t.cand_cap & (t.cand_cap - 1)) != 0 || t.cand_cap < tcap || lds_for(tcap, t.cand_cap) > lds_max)
            return fail(CORAL_ERR_ARG, "cand_cap must be a power of two, at least %d, that fits LDS", tcap);
        ccap = t.cand_cap;
    } else if (!best_first && p.big && lds_for(tcap, 2 * tcap) <= lds_max) {
        ccap = 2 * tcap;
    }
    int threads = t.threads;
    if (threads == 0)
        threads = p.big ? 1024 : best_first ? 256 : (lds_for(tcap, ccap) > lds_max / 2 ? 1024 : 512);
    if (threads != 128 && threads != 256 && threads != 512 && threads != 1024)
        return fail(CORAL_ERR_ARG, "threads must be 128, 256, 512 or 1024");
    p.lds_bytes = coral::search_lds_bytes(L, idx->dim, p.table_words, tcap, ccap, ocap, p.big, screen);
    int wg_per_cu = 0;
    HIP_TRY(coral::search_kernel_prepare(idx->dim, p.big, p.lds_bytes, threads, &wg_per_cu));
    if (wg_per_cu <= 0) return fail(CORAL_ERR_DEVICE, "kernel does not fit the device");
    // A small batch that the chip cannot take at once in workgroups of 512 threads, but can in workgroups of 256 (twice
    // as many per CU where LDS allows), runs in one go instead of two: 1000 queries on a 100 000-node graph at L = 64
    // take 276 us instead of 312.
    if (t.threads == 0 && threads == 512 && !best_first && Q > (int64_t)wg_per_cu * idx->num_cu) {
        int wg256 = 0;
        if (coral::search_kernel_prepare(idx->dim, p.big, p.lds_bytes, 256, &wg256) == hipSuccess && wg256 > wg_per_cu &&
            Q <= (int64_t)wg256 * idx->num_cu)
            threads = 256, wg_per_cu = wg256;
    }
    int workgroups = t.workgroups > 0 ? t.workgroups : wg_per_cu * idx->num_cu;
    p.workgroups = std::min(workgroups, (int)Q);
    p.tcap = tcap, p.ccap = ccap, p.threads = threads, p.id_bits = id_bits, p.ocap = ocap;
    // graph rows a chunk ahead: pays where a workgroup is alone on its CU (nothing else covers the wait)
    p.prefetch = t.prefetch_rows > 0 || (t.prefetch_rows == 0 && wg_per_cu == 1 && !best_first);
    p.beam_stride = p.big ? coral::search_beam_stride(L) : 0;
    *out = p;
    return CORAL_OK;
}

int coral_search_prepare(coral_index* idx, int32_t Q, int32_t L, const coral_tuning* tuning) {
    if (!idx) return fail(CORAL_ERR_ARG, "null index");
    if (!idx->d_nbrs) return fail(CORAL_ERR_STATE, "the index holds vectors only (no graph was given)");
    coral_tuning t;
    std::memset(&t, 0, sizeof t);
    if (tuning) t = *tuning;
    HIP_TRY(hipSetDevice(idx->device));
    coral_search_plan plan;
    // The screening phase needs a half-precision copy of the vectors (5/8 of their memory at dim 200), made once per
    // index; where the library chooses by itself and the memory is not to be had, the search runs without.
    auto ensure_vec16 = [&]() -> hipError_t {
        if (idx->d_vec16) return hipSuccess;
        const size_t bytes = coral::half_row_stride(idx->dim) * (size_t)idx->n;
        unsigned char* p = nullptr;
        hipError_t e = hipMalloc(&p, bytes);
        if (e != hipSuccess) return e;
        e = hipMemsetAsync(p, 0, bytes, idx->stream);
        if (e == hipSuccess) e = coral::launch_half_rows(idx->d_vec, idx->n, idx->dim, p, idx->stream);
        if (e == hipSuccess)
            idx->d_vec16 = p;
        else
            (void)hipFree(p);
        return e;
    };
    auto ensure_vec8 = [&]() -> hipError_t {
        if (idx->d_vec8) return hipSuccess;
        const size_t bytes = coral::byte_row_stride(idx->dim) * (size_t)idx->n;
        unsigned char* p = nullptr;
        hipError_t e = hipMalloc(&p, bytes);
        if (e != hipSuccess) return e;
        e = hipMemsetAsync(p, 0, bytes, idx->stream);
        if (e == hipSuccess) e = coral::launch_byte_rows(idx->d_vec, idx->n, idx->dim, p, idx->stream);
        if (e == hipSuccess)
            idx->d_vec8 = p;
        else
            (void)hipFree(p);
        return e;
    };
    const int bump = idx->bump_L == L ? idx->bump_log2 : 0;
    if (int rc = plan_search(idx, Q, L, t, bump, false, false, &plan)) return rc;
    if (plan.screen) {
        const hipError_t e = plan.screen == 2 ? ensure_vec8() : ensure_vec16();
        if (e == hipErrorOutOfMemory && t.screening == 0) {
            (void)hipGetLastError();
            if (int rc = plan_search(idx, Q, L, t, bump, false, true, &plan)) return rc;
        } else {
            HIP_TRY(e);
        }
    }
    HIP_TRY(hipStreamSynchronize(idx->stream));
    const bool best_first = t.policy == CORAL_POLICY_BEST_FIRST;
    const int id_bits = plan.id_bits;
    const int workgroups = plan.workgroups;

    // Best-first on one wavefront per query: with the beam in LDS (best_first.hip; four wavefronts of a workgroup must
    // fit) or, for longer beams, with a sorted insert buffer in LDS in front of a long run in global memory
    // (best_first_long.hip).  best_first_in_lds = 1 keeps the policy on the workgroup-per-query kernel.
    if (t.best_first_buffer != 0 && (t.best_first_buffer < 64 || t.best_first_buffer > 4096 || t.best_first_buffer % 64))
        return fail(CORAL_ERR_ARG, "best_first_buffer must be a multiple of 64 in 64..4096");
    // (measured at a million nodes: the two forms cross between L = 1024 and 1536)
    const bool long_form = best_first && !t.best_first_in_lds &&
                           (t.best_first_long > 0 || (t.best_first_long == 0 && L > kLongBeamFrom));
    const bool wave_form = best_first && !t.best_first_in_lds && !long_form && !plan.big &&
                           coral::best_first_wave_lds_bytes(L, 0, 0) * 4 <= (size_t)kMaxLdsBytes;
    // rows of 68 .. 128 floats are screened (on codes) only when the caller asks for it by name; the coded query then
    // takes the LDS a table of visited ids would fill
    const bool narrow_codes = best_first && t.screening == 2 && idx->dim / 4 > 16 && idx->dim / 4 <= 32;
    int table_log2 = 0;
    if (wave_form)
        if (int rc = choose_bf_table(L, id_bits, narrow_codes ? -1 : t.best_first_table_log2, &table_log2)) return rc;
    // from here on buffers are replaced: a failure part-way leaves the index unprepared, not half-prepared
    idx->prepared = false;
    const size_t need_words = plan.spill_words * (size_t)workgroups;
    if (need_words > idx->spill_alloc_words) {
        (void)hipFree(idx->d_spill);
        idx->d_spill = nullptr, idx->spill_alloc_words = 0;
        HIP_TRY(hipMalloc(&idx->d_spill, need_words * sizeof(uint32_t)));
        idx->spill_alloc_words = need_words;
        HIP_TRY(coral::launch_fill_u32(idx->d_spill, need_words, 0u, idx->stream));
    }
    const size_t need_beam = plan.beam_stride * (size_t)workgroups;
    if (need_beam > idx->beam_alloc_words) {
        (void)hipFree(idx->d_beam);
        idx->d_beam = nullptr, idx->beam_alloc_words = 0;
        HIP_TRY(hipMalloc(&idx->d_beam, need_beam * sizeof(uint64_t)));
        idx->beam_alloc_words = need_beam;
    }
    // per query: the four traversal counters, then (behind those of the whole batch) the four counts of what it read
    const size_t need_counters = (size_t)Q * 8;
    if (need_counters > idx->counters_alloc) {
        (void)hipFree(idx->d_counters);
        if (idx->h_counters) (void)hipHostFree(idx->h_counters);
        idx->d_counters = nullptr, idx->h_counters = nullptr, idx->counters_alloc = 0;
        HIP_TRY(hipMalloc(&idx->d_counters, need_counters * sizeof(int32_t)));
        HIP_TRY(hipHostMalloc(&idx->h_counters, need_counters * sizeof(int32_t)));
        idx->counters_alloc = need_counters;
    }
    // Best-first, one wavefront per query: the visited state lives in HBM, n bytes per wavefront (n / 6 in the packed
    // form), up to a third of what is free and 64 GiB.  wg_per_cu: what the chosen kernel's occupancy allows;
    // reprepare(packed): sets that kernel up in the packed form and returns its occupancy.
    idx->bf_ready = false, idx->bf_long = false, idx->bf_screen = 0;
    // Best-first with the beam in LDS screens rows in half precision too, where a CU holds sixteen wavefronts (beams
    // without the LDS table: L > 409): +12 % at L = 512 and 1024.  With the table (eight wavefronts per CU) the extra
    // wait per step costs more than the bytes it spares (L = 256 / 320: -27 %), so those launches go without unless
    // the caller asks for it by name.
    if (long_form && (idx->dim / 4 > 32 || narrow_codes) && idx->dim <= coral::kMaxByteRowDim &&
        (t.screening == 2 || t.screening == 0)) {
        // the kernel of long beams screens on eight-bit codes only.  (The longer the queue, the larger the share of
        // rows that enter it and need their fp32 row after all: a quarter at L = 19 456 on a million isotropic
        // vectors, where the screening still spares a third of the launch's bytes.)
        const hipError_t e = ensure_vec8();
        if (e == hipSuccess) {
            idx->bf_screen = 2;
        } else if (e == hipErrorOutOfMemory && t.screening == 0) {
            (void)hipGetLastError();
        } else {
            HIP_TRY(e);
        }
    }
    // eight-bit codes where they apply; launches with the LDS table (whose size was chosen to fill LDS) and rows of
    // more than 512 floats screen in half precision, which only the L2 metric has
    const int form = t.screening == 1 || idx->dim > coral::kMaxByteRowDim || table_log2 != 0 ? 1 : 2;
    // (rows of more than 512 floats, which this kernel can only screen in half precision, go without unless asked by
    // name: 156 k against 211 k QPS at 1024 floats and L = 512, 51 k against 111 k at 2048)
    if (wave_form && (idx->dim / 4 > 32 || narrow_codes) && (form == 2 || idx->metric == CORAL_L2) &&
        (t.screening > 0 || (t.screening == 0 && table_log2 == 0 && idx->dim <= coral::kMaxByteRowDim))) {
        const hipError_t e = form == 2 ? ensure_vec8() : ensure_vec16();
        if (e == hipSuccess) {
            idx->bf_screen = form;
        } else if (e == hipErrorOutOfMemory && t.screening == 0) {
            (void)hipGetLastError();
        } else {
            HIP_TRY(e);
        }
    }
    auto visited_slots = [&](int bf_wg_per_cu, auto reprepare, int64_t other_bytes_per_slot) -> int {
        size_t free_b = 0, total_b = 0;
        HIP_TRY(hipMemGetInfo(&free_b, &total_b));
        const size_t budget = std::min<size_t>((free_b + idx->bf_alloc_bytes) / 3, (size_t)64 << 30);
        const int64_t want = t.workgroups > 0 ? (int64_t)t.workgroups * 4 : (int64_t)bf_wg_per_cu * idx->num_cu * 4;
        const size_t stride_bytes = ((size_t)idx->n + 15) & ~(size_t)15;
        const size_t stride_packed = ((((size_t)idx->n + 23) / 24 * 4) + 15) & ~(size_t)15;
        // a byte per node while that leaves every wavefront its slot, else the packed words
        const int64_t need = std::min<int64_t>(want, (int64_t)Q);
        const int packed = t.best_first_packed || (int64_t)(budget / (stride_bytes + other_bytes_per_slot)) < need ? 1 : 0;
        const size_t stride = packed ? stride_packed : stride_bytes;
        if (packed != idx->bf_packed) idx->bf_stride = 0;  // forces a fresh, zeroed allocation
        idx->bf_packed = packed;
        if (packed) HIP_TRY(reprepare(&bf_wg_per_cu));
        int slots = (int)std::min<size_t>((size_t)need, budget / (stride + other_bytes_per_slot));
        // below about four wavefronts per CU the workgroup-per-query kernel is the faster one
        if (bf_wg_per_cu > 0 && (slots >= 4 * idx->num_cu || slots >= Q || t.workgroups > 0) && slots > 0) {
            bool have = stride == idx->bf_stride && slots <= idx->bf_alloc_slots;
            if (!have) {
                (void)hipFree(idx->d_bf_visited), (void)hipFree(idx->d_bf_epochs);
                idx->d_bf_visited = nullptr, idx->d_bf_epochs = nullptr;
                idx->bf_alloc_slots = 0, idx->bf_alloc_bytes = 0, idx->bf_stride = 0;
                // a refused allocation is no error: the workgroup-per-query kernel serves the policy then
                hipError_t e = hipMalloc(&idx->d_bf_visited, stride * (size_t)slots);
                if (e == hipSuccess) e = hipMalloc(&idx->d_bf_epochs, (size_t)slots * sizeof(uint32_t));
                if (e == hipSuccess) {
                    HIP_TRY(hipMemsetAsync(idx->d_bf_visited, 0, stride * (size_t)slots, idx->stream));
                    HIP_TRY(hipMemsetAsync(idx->d_bf_epochs, 0, (size_t)slots * sizeof(uint32_t), idx->stream));
                    idx->bf_stride = stride, idx->bf_alloc_slots = slots;
                    idx->bf_alloc_bytes = stride * (size_t)slots;
                    have = true;
                } else {
                    (void)hipGetLastError();
                    (void)hipFree(idx->d_bf_visited);
                    idx->d_bf_visited = nullptr;
                }
            }
            if (have) idx->bf_slots = slots, idx->bf_ready = true;
        }
        return CORAL_OK;
    };
    if (wave_form) {
        int bf_wg_per_cu = 0;
        const int chunks = idx->dim / 4;
        idx->bf_table_log2 = table_log2;
        idx->bf_table_rem_bits = table_log2 ? bf_table_rem_bits(id_bits, table_log2) : 0;
        // 16 rows requested per wavefront before any is added up where that fits 128 registers without spilling; a
        // launch whose LDS leaves a CU eight wavefronts may as well use 256 registers per lane: all 32 rows of a step
        int rif = (chunks > 16 && chunks <= 256) ? 16 : 8;
        if (idx->bf_screen != 0 && table_log2 == 0) rif = 8;  // (the screening leaves few rows to read in fp32)
        if (table_log2 && coral::best_first_wave_lds_bytes(L, 0, table_log2) * 12 > (size_t)kMaxLdsBytes && chunks > 16 &&
            chunks <= 64)
            rif = 32;
        idx->bf_rows_in_flight = rif;
        // with a table the filter would only cover what outgrew it, and its LDS is worth more as cells
        const int coded = idx->bf_screen == 2 ? coral::coded_query_bytes(idx->dim) : 0;
        const int bloom_log2 = table_log2 ? 0 : coral::best_first_bloom_log2(L, coded);
        idx->bf_bloom_log2 = bloom_log2;
        HIP_TRY(coral::best_first_prepare(idx->dim, L, rif, false, idx->bf_screen, bloom_log2, table_log2, &bf_wg_per_cu));
        auto reprepare = [&](int* occ) {
            return coral::best_first_prepare(idx->dim, L, rif, true, idx->bf_screen, bloom_log2, table_log2, occ);
        };
        if (int rc = visited_slots(bf_wg_per_cu, reprepare, 0)) return rc;
    } else if (long_form) {
        // the insert buffer: 512 keys unless the caller names a size; a sample of at most 128 keys of the long run
        const int bcap = t.best_first_buffer ? t.best_first_buffer : 512;
        const int scap = 128;
        int sshift = 0;
        while ((((int64_t)L - 1) >> sshift) + 1 > scap) ++sshift;
        const bool screen = idx->bf_screen == 2;
        if (coral::best_first_long_lds_bytes(bcap, scap, screen ? coral::best_first_long_coded_bytes(idx->dim) : 0) * 4 >
            (size_t)kMaxLdsBytes)
            return fail(CORAL_ERR_ARG, "best_first_buffer = %d does not fit LDS", bcap);
        int bf_wg_per_cu = 0;
        HIP_TRY(coral::best_first_long_prepare(idx->dim, false, screen, bcap, scap, &bf_wg_per_cu));
        auto reprepare = [&](int* occ) { return coral::best_first_long_prepare(idx->dim, true, screen, bcap, scap, occ); };
        const size_t Lp = (size_t)((L + 3) & ~3);
        const size_t beam_stride = (2 * Lp + 15) & ~(size_t)15;  // two runs of Lp keys, a multiple of 128 bytes
        if (int rc = visited_slots(bf_wg_per_cu, reprepare, (int64_t)beam_stride * 8)) return rc;
        if (idx->bf_ready) {
            const size_t need = beam_stride * (size_t)idx->bf_slots;
            if (need > idx->bf_beam_alloc_words) {
                (void)hipFree(idx->d_bf_beams);
                idx->d_bf_beams = nullptr, idx->bf_beam_alloc_words = 0;
                const hipError_t e = hipMalloc(&idx->d_bf_beams, need * sizeof(uint64_t));
                if (e == hipSuccess) {
                    idx->bf_beam_alloc_words = need;
                } else {
                    (void)hipGetLastError();
                    idx->bf_ready = false;  // the workgroup-per-query kernel serves the policy
                }
            }
        }
        idx->bf_long = idx->bf_ready;
        idx->bf_bcap = bcap, idx->bf_scap = scap, idx->bf_sshift = sshift, idx->bf_beam_stride = beam_stride;
    }
    HIP_TRY(hipStreamSynchronize(idx->stream));
    idx->Q = Q, idx->L = L, idx->plan = plan;
    idx->prepared_policy = t.policy;
    idx->tuning = t;
    idx->prepared = true;
    return CORAL_OK;
}

// the kernel's argument block for one call under a plan; scratch pointers are the caller's
static coral::SearchArgs search_args(const coral_index* idx, const coral_search_plan& p, const float* d_queries,
                                     int32_t* d_ids, float* d_dists, int32_t Q, int32_t k, int32_t policy,
                                     int32_t have_delete) {
    coral::SearchArgs a;
    std::memset(&a, 0, sizeof a);
    a.vec = idx->d_vec, a.nbrs = idx->d_nbrs, a.start_ids = idx->d_start;
    a.deleted = have_delete ? idx->d_deleted : nullptr;
    a.queries = d_queries, a.ids_out = d_ids, a.dists_out = d_dists;
    a.spill_words = p.spill_words, a.n = idx->n;
    a.dim = idx->dim, a.R = idx->R, a.M = idx->M, a.Q = Q, a.k = k, a.L = p.L;
    a.metric = idx->metric, a.policy = policy;
    a.slots_log2 = p.slots_log2, a.vis_limit = p.vis_limit;
    a.tcap = p.tcap, a.ccap = p.ccap;
    a.id_bits = p.id_bits, a.rem_bits = p.rem_bits, a.dmax = p.dmax, a.ocap = p.ocap;
    a.beam_stride = p.beam_stride, a.direct_bitmap = p.direct, a.table_words = p.table_words;
    a.prefetch_rows = p.prefetch;
    a.bucket_choices = p.choices;
    a.vec16 = p.screen == 1 ? idx->d_vec16 : nullptr, a.stride16 = coral::half_row_stride(idx->dim);
    a.vec8 = p.screen == 2 ? idx->d_vec8 : nullptr, a.stride8 = coral::byte_row_stride(idx->dim);
    a.tcap2 = p.screen ? coral::search_exact_list_cap(p.tcap) : 0;
    a.scap = p.big ? coral::kBeamSampleKeys : 0;
    return a;
}

int coral_search_gpu(coral_index* idx, const float* d_queries, int32_t* d_ids, float* d_dists,
                     int32_t Q, int32_t k, int32_t policy, int32_t have_delete, void* stream_,
                     coral_stats* stats) {
    if (!idx || !d_queries || !d_ids) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->prepared) return fail(CORAL_ERR_STATE, "coral_search_prepare has not been called");
    if (Q <= 0 || Q > idx->Q)
        return fail(CORAL_ERR_ARG, "Q=%d exceeds the prepared batch of %d", Q, idx->Q);
    if (k <= 0 || k > idx->L) return fail(CORAL_ERR_ARG, "k=%d must be in 1..L=%d", k, idx->L);
    if (policy != CORAL_POLICY_ROUNDS && policy != CORAL_POLICY_BEST_FIRST)
        return fail(CORAL_ERR_ARG, "unknown policy %d", policy);
    if (have_delete && !idx->d_deleted)
        return fail(CORAL_ERR_STATE, "have_delete set but no tombstone mask was given");
    HIP_TRY(hipSetDevice(idx->device));
    hipStream_t stream = stream_ ? (hipStream_t)stream_ : idx->stream;

    const coral_search_plan& plan = idx->plan;
    coral::SearchArgs a = search_args(idx, plan, d_queries, d_ids, d_dists, Q, k, policy, have_delete);
    a.counters = idx->d_counters, a.spill = idx->d_spill, a.beam_scratch = idx->d_beam;
    a.next_qid = idx->d_scalars, a.spill_count = idx->d_scalars + 1;

    const bool wave_kernel = policy == CORAL_POLICY_BEST_FIRST && idx->bf_ready;
    if (wave_kernel && idx->rows_unique < 0) {
        // once per graph: rows without repeated ids let the kernel skip its comparison of a row with itself
        uint32_t flag = 0;
        HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_scalars, 4, 0u, stream));
        HIP_TRY(coral::launch_find_repeated_ids(idx->d_nbrs, idx->n, idx->R, (uint32_t*)idx->d_scalars + 2, stream));
        HIP_TRY(hipMemcpyAsync(&flag, idx->d_scalars + 2, sizeof flag, hipMemcpyDeviceToHost, stream));
        HIP_TRY(hipStreamSynchronize(stream));
        idx->rows_unique = flag ? 0 : 1;
    }

    for (hipEvent_t& e : idx->ev)
        if (!e) HIP_TRY(hipEventCreate(&e));
    hipEvent_t ev0 = idx->ev[0], evk = idx->ev[1], ev1 = idx->ev[2];
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_scalars, 4, 0u, stream));
#ifdef CORAL_PHASE_TIMERS
    if (!idx->d_phase) HIP_TRY(hipMalloc(&idx->d_phase, 8 * sizeof(unsigned long long)));
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_phase, 16, 0u, stream));
    a.phase_ticks = idx->d_phase;
#endif
    // timed region, same scope as the reference: kernel + counter read-back
    HIP_TRY(hipEventRecord(ev0, stream));
    if (wave_kernel && idx->bf_long) {
        coral::BestFirstLongArgs b;
        std::memset(&b, 0, sizeof b);
        b.visited = idx->d_bf_visited, b.epochs = idx->d_bf_epochs, b.stride = idx->bf_stride;
        b.beams = idx->d_bf_beams, b.beam_stride = idx->bf_beam_stride;
        b.slots = std::min(idx->bf_slots, (int)Q);
        b.rows_unique = idx->rows_unique == 1, b.packed = idx->bf_packed;
        b.bcap = idx->bf_bcap, b.scap = idx->bf_scap, b.sshift = idx->bf_sshift;
        b.vec8 = idx->bf_screen == 2 ? idx->d_vec8 : nullptr, b.stride8 = coral::byte_row_stride(idx->dim);
        b.coded_bytes = idx->bf_screen == 2 ? coral::best_first_long_coded_bytes(idx->dim) : 0;
        HIP_TRY(coral::launch_best_first_long(a, b, stream));
    } else if (wave_kernel) {
        coral::BestFirstArgs b;
        b.rows_unique = idx->rows_unique == 1;
        b.packed = idx->bf_packed;
        b.bloom_log2 = idx->bf_bloom_log2;
        b.table_log2 = idx->bf_table_log2;
        b.id_bits = plan.id_bits, b.rem_bits = idx->bf_table_rem_bits;
        b.visited = idx->d_bf_visited, b.epochs = idx->d_bf_epochs, b.stride = idx->bf_stride;
        b.slots = std::min(idx->bf_slots, (int)Q);
        b.rows_in_flight = idx->bf_rows_in_flight;
        b.vec16 = idx->bf_screen == 1 ? idx->d_vec16 : nullptr, b.stride16 = coral::half_row_stride(idx->dim);
        b.vec8 = idx->bf_screen == 2 ? idx->d_vec8 : nullptr, b.stride8 = coral::byte_row_stride(idx->dim);
        b.coded_bytes = idx->bf_screen == 2 ? coral::coded_query_bytes(idx->dim) : 0;
        HIP_TRY(coral::launch_best_first(a, b, stream));
    } else {
        const int wgs = std::min(plan.workgroups, (int)Q);
        HIP_TRY(coral::launch_search(a, plan.big, wgs, plan.threads, plan.lds_bytes, stream));
    }
    HIP_TRY(hipEventRecord(evk, stream));
    HIP_TRY(hipMemcpyAsync(idx->h_counters, idx->d_counters, (size_t)Q * 8 * sizeof(int32_t),
                           hipMemcpyDeviceToHost, stream));
    HIP_TRY(hipEventRecord(ev1, stream));
    HIP_TRY(hipEventSynchronize(ev1));
    float ms = 0.f, ms_kernel = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, ev0, ev1));
    HIP_TRY(hipEventElapsedTime(&ms_kernel, ev0, evk));
    int scal[3] = {0, 0, 0};
    HIP_TRY(hipMemcpyAsync(scal, idx->d_scalars, sizeof scal, hipMemcpyDeviceToHost, stream));
    HIP_TRY(hipStreamSynchronize(stream));
#ifdef CORAL_PHASE_TIMERS
    {
        unsigned long long t[8];
        HIP_TRY(hipMemcpy(t, idx->d_phase, sizeof t, hipMemcpyDeviceToHost));
        double sum = 0;
        for (int i = 0; i < 7; ++i) sum += (double)t[i];
        sum += (double)t[7];
        std::fprintf(stderr, "[phase %%] init %.1f seeds %.1f elist %.1f expand %.1f screening %.1f distance %.1f merge %.1f output %.1f\n",
                     100 * t[0] / sum, 100 * t[1] / sum, 100 * t[2] / sum, 100 * t[3] / sum, 100 * t[7] / sum,
                     100 * t[4] / sum, 100 * t[5] / sum, 100 * t[6] / sum);
    }
#endif
    idx->last_Q = Q;
    coral_stats sum;
    std::memset(&sum, 0, sizeof sum);
    sum.time_s = ms / 1000.0, sum.kernel_s = ms_kernel / 1000.0;
    for (int q = 0; q < Q; ++q) {
        const int32_t* c = idx->h_counters + (size_t)q * 4;
        sum.hops += c[0], sum.expansions += c[1], sum.dist_evals += c[2], sum.rounds += c[3];
        const int32_t* r = idx->h_counters + (size_t)Q * 4 + (size_t)q * 4;
        sum.screened_rows += r[0], sum.exact_rows += r[1], sum.beam_words += r[2], sum.visited_requests += r[3];
    }
    sum.spills = scal[1], sum.visited_dedupes = scal[2];
    // The table size the library picks assumes about 75 first visits per beam entry.  Data on which a query visits
    // more sends queries to the global bitmap (same results, slower): when more than a twentieth of a batch went
    // there, the next launches get a table twice the size.  (The bucket form turns away only the ids that find their
    // three buckets full, a handful per query at a load where linear probing freezes the table: it takes the larger
    // table only when more than a fiftieth of all first visits went to the bitmap.)
    const bool lds_table = !(policy == CORAL_POLICY_BEST_FIRST && idx->bf_ready) && !plan.big;
    bool grow = lds_table && idx->tuning.visited_slots_log2 == 0 && (int64_t)scal[1] * 20 > Q && plan.slots_log2 < 16;
    if (grow && plan.choices != 0 && sum.visited_requests / 2 * 50 <= sum.dist_evals) {
        // few ids left LDS: the larger table is worth taking only if it costs the CU no workgroup
        coral_search_plan peek;
        const int next = (idx->bump_L == idx->L ? idx->bump_log2 : 0) + 1;
        grow = plan_search(idx, idx->Q, idx->L, idx->tuning, next, false, plan.screen == 0, &peek) == CORAL_OK &&
               !peek.direct && peek.workgroups >= plan.workgroups;
    }
    if (grow) {
        const int had = plan.slots_log2;
        idx->bump_log2 = idx->bump_L == idx->L ? idx->bump_log2 + 1 : 1;
        idx->bump_L = idx->L;
        coral_tuning t = idx->tuning;
        if (coral_search_prepare(idx, idx->Q, idx->L, &t) != CORAL_OK || idx->plan.slots_log2 == had) {
            idx->bump_log2 -= 1;  // no room in LDS for more: stay
            if (!idx->prepared) return fail(CORAL_ERR_DEVICE, "could not restore the search scratch");
        }
    }
    if (stats) *stats = sum;
    return CORAL_OK;
}

int coral_search_gpu_noalloc(coral_index* idx, const float* d_queries, int32_t* d_ids, float* d_dists, int32_t Q,
                             int32_t k, int32_t L, int32_t policy, int32_t have_delete, void* stream_) {
    if (!idx || !d_queries || !d_ids) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->d_nbrs) return fail(CORAL_ERR_STATE, "the index holds vectors only (no graph was given)");
    if (Q <= 0 || Q > coral::kStaticMaxQ)
        return fail(CORAL_ERR_ARG, "Q=%d is outside 1..%d, the queries the fixed scratch block has counters for", Q,
                    coral::kStaticMaxQ);
    if (idx->n > coral::kStaticMaxN)
        return fail(CORAL_ERR_ARG, "n=%lld exceeds %lld, the nodes the fixed scratch block has overflow bitmaps for",
                    (long long)idx->n, (long long)coral::kStaticMaxN);
    if (L <= 0 || L > CORAL_MAX_LDS_BEAM)
        return fail(CORAL_ERR_ARG, "L=%d is outside 1..%d: longer beams need scratch in global memory", L,
                    CORAL_MAX_LDS_BEAM);
    if (k <= 0 || k > L) return fail(CORAL_ERR_ARG, "k=%d must be in 1..L=%d", k, L);
    if (have_delete && !idx->d_deleted)
        return fail(CORAL_ERR_STATE, "have_delete set but no tombstone mask was given");
    HIP_TRY(hipSetDevice(idx->device));
    unsigned char* base = static_cast<unsigned char*>(coral::static_scratch(idx->device));
    if (!base) return fail(CORAL_ERR_STATE, "the fixed scratch block of device %d was not set up", idx->device);
    hipStream_t stream = stream_ ? (hipStream_t)stream_ : idx->stream;
    coral_tuning t;
    std::memset(&t, 0, sizeof t);
    t.policy = policy;  // both policies run on the workgroup-per-query kernel here
    // rows are screened on a smaller copy of the vectors only if an earlier coral_search_prepare has made one:
    // nothing is allocated here
    const bool rounds = policy == CORAL_POLICY_ROUNDS;
    t.screening = rounds && idx->d_vec8 && idx->dim / 4 > 16                            ? 2
                  : rounds && idx->d_vec16 && idx->dim / 4 > 32 && idx->metric == CORAL_L2 ? 1
                                                                                           : -1;
    // the launch geometry (kernel attributes, an occupancy query) is worked out on the first call with these
    // arguments and kept: later calls only fill two buffers and launch
    if (idx->noalloc_Q != Q || idx->noalloc_L != L || idx->noalloc_policy != policy || idx->noalloc_screen != t.screening) {
        idx->noalloc_L = 0;
        if (int rc = plan_search(idx, Q, L, t, 0, /*lds_beam_only*/ true, /*no_screen*/ t.screening < 0, &idx->noalloc_plan))
            return rc;
        idx->noalloc_Q = Q, idx->noalloc_L = L, idx->noalloc_policy = policy, idx->noalloc_screen = t.screening;
    }
    const coral_search_plan& plan = idx->noalloc_plan;
    // the block: 256 bytes of scalars, the per-query counters, then one overflow bitmap per workgroup
    int* scal = reinterpret_cast<int*>(base);
    int32_t* counters = reinterpret_cast<int32_t*>(base + 256);
    uint32_t* spill = reinterpret_cast<uint32_t*>(base + 256 + (size_t)coral::kStaticMaxQ * 32);
    int wgs = std::min(plan.workgroups, (int)Q);
    if (plan.spill_words)  // (none when the visited set is a bitmap of all ids in LDS)
        wgs = (int)std::min<size_t>((size_t)wgs, coral::kStaticSpillWords / plan.spill_words);
    // the block keeps what the last call left: the work counter and the bitmaps must start at zero (fill kernels,
    // which a caller may record into a graph)
    HIP_TRY(coral::launch_fill_u32(reinterpret_cast<uint32_t*>(scal), 64, 0u, stream));
    HIP_TRY(coral::launch_fill_u32(spill, plan.spill_words * (size_t)wgs, 0u, stream));
    coral::SearchArgs a = search_args(idx, plan, d_queries, d_ids, d_dists, Q, k, policy, have_delete);
    a.counters = counters, a.spill = spill, a.beam_scratch = nullptr;
    a.next_qid = scal, a.spill_count = scal + 1;
    idx->noalloc_in_flight = true;
    HIP_TRY(coral::launch_search(a, false, wgs, plan.threads, plan.lds_bytes, stream));
    return CORAL_OK;
}

int coral_search_query_counters(coral_index* idx, int32_t* host_out, int32_t Q) {
    if (!idx || !host_out) return fail(CORAL_ERR_ARG, "null argument");
    if (Q <= 0 || Q > idx->last_Q) return fail(CORAL_ERR_ARG, "no counters for %d queries", Q);
    std::memcpy(host_out, idx->h_counters, (size_t)Q * 4 * sizeof(int32_t));
    return CORAL_OK;
}

int coral_search_row_counters(coral_index* idx, int32_t* host_out, int32_t Q) {
    if (!idx || !host_out) return fail(CORAL_ERR_ARG, "null argument");
    if (Q <= 0 || Q > idx->last_Q) return fail(CORAL_ERR_ARG, "no counters for %d queries", Q);
    std::memcpy(host_out, idx->h_counters + (size_t)idx->last_Q * 4, (size_t)Q * 4 * sizeof(int32_t));
    return CORAL_OK;
}

int coral_search_plan_info(const coral_index* idx, coral_plan_info* out) {
    if (!idx || !out) return fail(CORAL_ERR_ARG, "null argument");
    if (!idx->prepared) return fail(CORAL_ERR_STATE, "coral_search_prepare has not been called");
    std::memset(out, 0, sizeof *out);
    const coral_search_plan& p = idx->plan;
    const bool wave = idx->prepared_policy == CORAL_POLICY_BEST_FIRST && idx->bf_ready;
    if (wave) {
        out->kernel = idx->bf_long ? 2 : 1;
        out->threads = 256;
        out->query_slots = std::min(idx->bf_slots, idx->Q);
        out->workgroups = (out->query_slots + 3) / 4;
        const size_t per_wave =
            idx->bf_long
                ? coral::best_first_long_lds_bytes(idx->bf_bcap, idx->bf_scap,
                                                   idx->bf_screen == 2 ? coral::best_first_long_coded_bytes(idx->dim) : 0)
                : coral::best_first_wave_lds_bytes(idx->L, idx->bf_bloom_log2, idx->bf_table_log2,
                                                   idx->bf_screen == 2 ? coral::coded_query_bytes(idx->dim) : 0);
        out->lds_bytes = (int32_t)(per_wave * 4);
        out->screening = idx->bf_screen;
        out->visited_form = !idx->bf_long && idx->bf_table_log2 ? 4 : idx->bf_packed ? 3 : 2;
        out->visited_slots_log2 = idx->bf_long ? 0 : idx->bf_table_log2;
        out->beam_in_hbm = idx->bf_long;
    } else {
        out->kernel = 0;
        out->threads = p.threads, out->workgroups = p.workgroups, out->lds_bytes = (int32_t)p.lds_bytes;
        out->screening = p.screen;
        out->visited_form = p.direct ? 1 : p.choices != 0 ? 5 : 0;
        out->visited_slots_log2 = p.direct ? 0 : p.slots_log2;
        out->beam_in_hbm = p.big;
        out->todo_cap = p.tcap, out->cand_cap = p.ccap;
        out->query_slots = p.workgroups;
    }
    out->screen_row_bytes = out->screening == 2   ? (int32_t)coral::byte_row_stride(idx->dim)
                            : out->screening == 1 ? (int32_t)coral::half_row_stride(idx->dim)
                                                  : 0;
    return CORAL_OK;
}

int coral_search(coral_index* idx, const float* h_queries, int32_t Q, int32_t k, int32_t L,
                 int32_t policy, int32_t have_delete, int32_t* h_ids, float* h_dists,
                 coral_stats* stats) {
    if (!idx || !h_queries || !h_ids) return fail(CORAL_ERR_ARG, "null argument");
    if (Q <= 0) return fail(CORAL_ERR_ARG, "Q must be positive");
    if (k <= 0 || k > L) return fail(CORAL_ERR_ARG, "k=%d must be in 1..L=%d", k, L);
    HIP_TRY(hipSetDevice(idx->device));
    if (!idx->prepared || idx->L != L || idx->Q < Q || idx->prepared_policy != policy) {
        coral_tuning t;
        std::memset(&t, 0, sizeof t);
        t.policy = policy;
        if (int rc = coral_search_prepare(idx, Q, L, &t)) return rc;
    }
    // device copies of the caller's buffers: kept with the index and grown when a call needs more
    auto grow = [](void** p, size_t* have, size_t need) -> hipError_t {
        if (need <= *have) return hipSuccess;
        (void)hipFree(*p);
        *p = nullptr, *have = 0;
        const hipError_t e = hipMalloc(p, need);
        if (e == hipSuccess) *have = need;
        return e;
    };
    const size_t qbytes = (size_t)Q * idx->dim * sizeof(float);
    const size_t ibytes = (size_t)Q * k * sizeof(int32_t), dbytes = (size_t)Q * k * sizeof(float);
    HIP_TRY(grow((void**)&idx->d_io_q, &idx->io_q_bytes, qbytes));
    HIP_TRY(grow((void**)&idx->d_io_ids, &idx->io_ids_bytes, ibytes));
    if (h_dists) HIP_TRY(grow((void**)&idx->d_io_dists, &idx->io_dists_bytes, dbytes));
    HIP_TRY(hipMemcpy(idx->d_io_q, h_queries, qbytes, hipMemcpyHostToDevice));
    const int rc = coral_search_gpu(idx, idx->d_io_q, idx->d_io_ids, h_dists ? idx->d_io_dists : nullptr, Q, k, policy,
                                    have_delete, nullptr, stats);
    if (rc != CORAL_OK) return rc;
    HIP_TRY(hipMemcpy(h_ids, idx->d_io_ids, ibytes, hipMemcpyDeviceToHost));
    if (h_dists) HIP_TRY(hipMemcpy(h_dists, idx->d_io_dists, dbytes, hipMemcpyDeviceToHost));
    return CORAL_OK;
}

int coral_search_verify(coral_index* idx, const int32_t* d_ids_res, const int32_t* d_ids_gt, int32_t Q,
                        int32_t k, int64_t* hits) {
    if (!idx || !d_ids_res || !d_ids_gt || !hits) return fail(CORAL_ERR_ARG, "null argument");
    if (Q <= 0 || k <= 0) return fail(CORAL_ERR_ARG, "Q and k must be positive");
    HIP_TRY(hipSetDevice(idx->device));
    HIP_TRY(coral::launch_fill_u32((uint32_t*)idx->d_hit, 2, 0u, idx->stream));
    HIP_TRY(coral::launch_verify(d_ids_res, d_ids_gt, idx->d_hit, Q, k, idx->stream));
    unsigned long long h = 0;
    HIP_TRY(hipMemcpyAsync(&h, idx->d_hit, sizeof h, hipMemcpyDeviceToHost, idx->stream));
    HIP_TRY(hipStreamSynchronize(idx->stream));
    *hits = (int64_t)h;
    return CORAL_OK;
}

}  // extern "C"
