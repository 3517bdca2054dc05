// beam_search.hip -- batched graph beam search for gfx950 (MI355X), one
// workgroup per in-flight query, persistent workgroups pulling query ids from a
// device counter.
//
// What it computes is the search of the reference's CUDA kernel
// (src/search_gpu.cu:347-580, tombstone variant :582-833) and, with
// policy == CORAL_POLICY_BEST_FIRST, of its CPU path (src/search_in_cpu.cpp:63-108).
// How it computes it is specific to this GPU:
//   * per query the sorted beam (64-bit keys), the exact visited set (open
//     addressing, 32-bit ids), the candidate buffer and the query live in LDS;
//     the reference keeps beam scratch and an N-bit visited bitmap per block in
//     global memory and clears the bitmap for every query (:388);
//   * a graph row is 32 int32 = one 128-byte line, read by half a wavefront;
//   * a vector row is read as float4 by a group of 16/32/64 lanes, eight rows in
//     flight per wave, and reduced across lanes (the reference lets one thread
//     walk a whole row, include/utils.cuh:254-275);
//   * candidates are bitonic-sorted and merged into the beam by rank; the
//     reference replaces the current worst entry one candidate at a time (:530-570);
//   * beams too long for LDS (the reference sets no limit on L, src/search.cu:400-408) run the
//     kernel's BIG form: the two beam buffers move to a per-workgroup block of global memory
//     (read and written in whole coalesced passes by the merge, so they live in L2), and the LDS
//     they leave holds the visited set as a plain bitmap of all n ids where n allows
//     (a million nodes = 125 KB): one LDS atomic per test, nothing ever spills.
//
// Distance summation order (mirrored bit for bit by the test oracle): lane l of a
// group of G lanes accumulates float4 chunks l, l+G, ... with four fused
// multiply-adds per chunk in x,y,z,w order; partials are combined by a butterfly
// p[l] += p[l^off], off = 1, 2, 4, ..., G/2.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <utility>

#include "beam_search.h"
#include "search_device.h"

namespace coral {

// Optional per-phase cycle accounting (debug builds only; thread 0 of each workgroup).
#ifdef CORAL_PHASE_TIMERS
#define PHASE_DECL unsigned long long ph_t = wall_clock64(), ph_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}
#define PHASE_MARK(i)                          \
    do {                                       \
        if (tid == 0) {                        \
            unsigned long long n_ = wall_clock64(); \
            ph_acc[i] += n_ - ph_t;            \
            ph_t = n_;                         \
        }                                      \
    } while (0)
#define PHASE_FLUSH()                                                             \
    do {                                                                          \
        if (tid == 0 && a.phase_ticks)                                            \
            for (int i_ = 0; i_ < 8; ++i_) atomicAdd(&a.phase_ticks[i_], ph_acc[i_]); \
    } while (0)
#else
#define PHASE_DECL
#define PHASE_MARK(i)
#define PHASE_FLUSH()
#endif

constexpr int kSmallMerge = 32;  // candidate counts merged by counting instead of sorting

// The visited set of one query.
//
// First level, in LDS: an open-addressing table of 16-bit cells.  A node id is
// mixed by a bijection on its b = ceil(log2 n) bits; the high bits of the result
// pick the home cell and only the remaining `rb` low bits (the remainder) are
// stored, together with the displacement d of the cell from its home:
//     cell = 1 + ((d << rb) | remainder),   0 = empty.
// (cell index, d, remainder) determine the mixed value and hence the id, so the
// table is exact; it holds twice the ids a table of 32-bit ids would.  Probing is
// linear and bounded by dmax (the largest d the 16 bits can carry).
// Second level, in global memory: this workgroup's n-bit bitmap, used for ids
// that find no cell within dmax and for every new id once the table has been
// frozen (load limit reached).  Ids sent there are remembered in a short LDS list
// so that the bitmap can be cleaned word by word when the query ends.
struct VisitedSet {
    uint32_t* words;   // LDS: slots/2 words
    uint32_t* olist;   // LDS: ids that went to the bitmap
    int* ocount;       // LDS: how many did (may exceed ocap)
    uint32_t* bitmap;  // global
    uint32_t smask, bmask, rmask;
    int rb, xs, dmax, ocap;
    bool direct;       // words is a bitmap of all ids (launches over few enough nodes that have LDS to spare)
    // Third form of the first level, for ids too wide for the displacement a 16-bit cell can carry beside them
    // (beyond 2^24 ids): the cells form buckets of four, an id may sit in any of three buckets -- its home, picked by
    // the high bits of the mixed id, and two more that follow from the home and the remaining bits -- and a cell
    // stores those remaining bits and which of the three it is in: cell = 1 + (choice << rb | remainder).  (bucket,
    // cell) give the mixed id back, so the table is exact; a new id goes to the emptiest of its buckets, which keeps
    // the load so even that a table two thirds full turns practically no id away (linear probing at that load needs
    // displacements far beyond the 14 that 2^27 ids leave room for in 2^15 cells).  The price is that the place of
    // an id depends on what a thread saw of the three buckets: two threads that insert the same id at the same time
    // can each find it absent and put it into different buckets.  Every thread therefore looks at the other two
    // buckets again after its insert; of two such threads at least the later one sees the other's cell, and raises
    // *dupflag: the list of new ids is then searched for repeats before it is used (see the kernel).
    bool buckets;
    uint32_t bkmask;   // buckets - 1
    int* dupflag;      // LDS
    int skew;          // -1; or (a form for tests) the inserting wavefront's number, which then picks the bucket in
                       // place of the load, so that concurrent inserts of one id part as often as they can

    // the three buckets of a mixed id and what its cells would hold
    __device__ __forceinline__ void places(uint32_t h, uint32_t (&bk)[3], uint32_t (&want)[3]) const {
        const uint32_t rem = h & rmask, b0 = (h >> rb) & bkmask;
        // two nonzero offsets that differ, from the remainder alone (so that bucket ^ offset gives the home back)
        uint32_t o1 = ((rem * 0x9E3779B1u + 0x7F4A7C15u) >> 7) & bkmask, o2 = ((rem * 0x85EBCA6Bu + 0x165667B1u) >> 9) & bkmask;
        if (o1 == 0u) o1 = 1u & bkmask;
        if (o2 == 0u || o2 == o1) o2 = (o1 ^ 2u) & bkmask ? (o1 ^ 2u) & bkmask : (o1 + 1u) & bkmask;
        bk[0] = b0, bk[1] = b0 ^ o1, bk[2] = b0 ^ o2;
        want[0] = 1u + rem, want[1] = 1u + ((1u << rb) | rem), want[2] = 1u + ((2u << rb) | rem);
    }

    __device__ __forceinline__ static bool holds(const uint2 w, uint32_t want) {
        return (w.x & 0xffffu) == want || (w.x >> 16) == want || (w.y & 0xffffu) == want || (w.y >> 16) == want;
    }
    __device__ __forceinline__ static int empties(const uint2 w) {
        return ((w.x & 0xffffu) == 0u) + ((w.x >> 16) == 0u) + ((w.y & 0xffffu) == 0u) + ((w.y >> 16) == 0u);
    }

    // 1: id was not in the table and now is; 0: it was; 2: it is not and no bucket has room
    __device__ __forceinline__ int bucket_test_and_set(uint32_t id) {
        uint32_t bk[3], want[3];
        places(mix(id), bk, want);
        const uint2* bks = reinterpret_cast<const uint2*>(words);
        for (;;) {
            const uint2 w0 = bks[bk[0]], w1 = bks[bk[1]], w2 = bks[bk[2]];
            if (holds(w0, want[0]) || holds(w1, want[1]) || holds(w2, want[2])) return 0;
            const int e0 = empties(w0), e1 = empties(w1), e2 = empties(w2);
            if (e0 + e1 + e2 == 0) return 2;
            int c = (e0 >= e1 && e0 >= e2) ? 0 : (e1 >= e2 ? 1 : 2);
            if (skew >= 0) {
                const int cs = skew % 3;
                if ((cs == 0 ? e0 : cs == 1 ? e1 : e2) > 0) c = cs;
            }
            const uint2 w = c == 0 ? w0 : c == 1 ? w1 : w2;
            // the first empty cell of that bucket
            const int cell = (w.x & 0xffffu) == 0u ? 0 : (w.x >> 16) == 0u ? 1 : (w.y & 0xffffu) == 0u ? 2 : 3;
            const uint32_t oldw = cell < 2 ? w.x : w.y;
            uint32_t* word = words + bk[c] * 2u + (uint32_t)(cell >> 1);
            if (atomicCAS(word, oldw, oldw | (want[c] << ((cell & 1) * 16))) != oldw) continue;  // another thread took a cell of that word: look again
            // the same id in another of its buckets: somebody inserted it at the same time
            const int c1 = c == 0 ? 1 : 0, c2 = c == 2 ? 1 : 2;
            if (holds(bks[bk[c1]], want[c1]) || holds(bks[bk[c2]], want[c2])) *dupflag = 1;
            return 1;
        }
    }

    __device__ __forceinline__ uint32_t mix(uint32_t id) const {
        uint32_t h = (id * 0x9E3779B1u) & bmask;
        h ^= h >> xs;
        h = (h * 0x85EBCA6Bu) & bmask;
        h ^= h >> xs;
        return h;
    }

    // 1 if id was not yet in the set (and now is), 0 if it was
    __device__ __forceinline__ int test_and_set(uint32_t id, bool frozen) {
        if (direct) {
            const uint32_t b = 1u << (id & 31);
            return (atomicOr(&words[id >> 5], b) & b) == 0u;
        }
        if (buckets) {
            if (!frozen) {
                const int r = bucket_test_and_set(id);
                if (r != 2) return r;
            } else {
                uint32_t bk[3], want[3];
                places(mix(id), bk, want);
                const uint2* bks = reinterpret_cast<const uint2*>(words);
                if (holds(bks[bk[0]], want[0]) || holds(bks[bk[1]], want[1]) || holds(bks[bk[2]], want[2])) return 0;
            }
            const uint32_t bit = 1u << (id & 31);
            const uint32_t old = atomicOr(&bitmap[id >> 5], bit);
            if (old & bit) return 0;
            const int p = atomicAdd(ocount, 1);
            if (p < ocap) olist[p] = id;
            return 1;
        }
        const uint32_t h = mix(id);
        const uint32_t home = h >> rb, rem = h & rmask;
        const uint16_t* cells = reinterpret_cast<const uint16_t*>(words);
        for (int d = 0; d <= dmax; ++d) {
            const uint32_t s = (home + (uint32_t)d) & smask;
            const uint32_t want = 1u + (((uint32_t)d << rb) | rem);
            uint32_t cur = cells[s];
            if (cur == want) return 0;
            if (cur == 0u) {
                if (frozen) break;
                uint32_t* w = words + (s >> 1);
                const int sh = (int)(s & 1u) * 16;
                uint32_t old = *w;
                for (;;) {
                    cur = (old >> sh) & 0xffffu;
                    if (cur != 0u) break;
                    const uint32_t prev = atomicCAS(w, old, old | (want << sh));
                    if (prev == old) return 1;
                    old = prev;
                }
                if (cur == want) return 0;
            }
        }
        const uint32_t bit = 1u << (id & 31);
        const uint32_t old = atomicOr(&bitmap[id >> 5], bit);
        if (old & bit) return 0;
        const int p = atomicAdd(ocount, 1);
        if (p < ocap) olist[p] = id;
        return 1;
    }
};

struct WgState {
    int nb;           // beam entries
    int cur;          // which LDS beam buffer is current
    uint64_t live;    // key of the worst entry of a full beam, else kKeyMax
};

template <int G, int CPL, bool BIG>
__global__ __launch_bounds__(1024) void beam_search_kernel(const SearchArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int tid = threadIdx.x, NT = blockDim.x;
    const int lane = tid & 63, wave = tid >> 6, NW = NT >> 6;
    const int L = a.L, R = a.R, dim = a.dim, chunks = dim >> 2;
    const int Lp = (L + 3) & ~3;
    const int slots = 1 << a.slots_log2;
    const int TCAP = a.tcap, CCAP = a.ccap;

    uint64_t *beam0, *beam1, *cand, *samp = nullptr;
    uint32_t *table, *todo, *todo2, *elist, *olist;
    if constexpr (BIG) {
        uint64_t* g = a.beam_scratch + (size_t)blockIdx.x * a.beam_stride;
        beam0 = g, beam1 = g + Lp, elist = (uint32_t*)(g + 2 * (size_t)Lp);
        cand = (uint64_t*)smem;
        samp = cand + CCAP;                     // a sample of the beam's keys for the merge's searches
        table = (uint32_t*)(samp + a.scap);     // 16-bit cells, or the bitmap of all ids
        todo = table + a.table_words;
        todo2 = todo + TCAP;
        olist = todo2 + a.tcap2;
    } else {
        beam0 = (uint64_t*)smem;
        beam1 = beam0 + Lp;
        cand = beam1 + Lp;
        table = (uint32_t*)(cand + CCAP);  // slots 16-bit cells
        todo = table + a.table_words;
        todo2 = todo + TCAP;
        elist = todo2 + a.tcap2;
        olist = elist + Lp;
    }
    float* qs = (float*)(olist + a.ocap);

    __shared__ int s_qid, s_ntodo, s_ntodo2, s_ncand, s_nexp, s_cntf, s_cursor, s_nover, s_dup;
    __shared__ int s_wcnt[16];
    // what the query read, by class (thread 0 alone adds to these and writes them out): rows measured on the smaller
    // copy, fp32 rows, words of a beam in global memory
    __shared__ int s_rows_screened, s_rows_exact, s_beam_words;
    __shared__ float s_qq, s_qscale, s_qerr;  // of the query in integer codes: |q~|^2, its scale, |q - q~| rounded up

    VisitedSet vs;
    vs.words = table, vs.olist = olist, vs.ocount = &s_nover;
    vs.bitmap = a.spill + (size_t)blockIdx.x * a.spill_words;
    vs.smask = (uint32_t)slots - 1u, vs.bmask = a.id_bits >= 32 ? 0xffffffffu : (1u << a.id_bits) - 1u;
    vs.rb = a.rem_bits, vs.rmask = (1u << a.rem_bits) - 1u;
    vs.xs = a.id_bits > 1 ? a.id_bits / 2 : 1, vs.dmax = a.dmax, vs.ocap = a.ocap;
    vs.direct = a.direct_bitmap != 0;
    vs.buckets = a.bucket_choices != 0, vs.bkmask = ((uint32_t)slots >> 2) - 1u, vs.dupflag = &s_dup;
    vs.skew = a.bucket_choices == 4 ? wave : -1;
    (void)slots;

    constexpr int GPW = 64 / G;                    // row groups per wave
    constexpr int U = (CPL >= 8) ? 1 : (8 / CPL);  // rows in flight per group
    constexpr int RPI = GPW * U;                   // rows per wave iteration
    const int gl = lane & (G - 1), grp = lane / G;

    for (;;) {
        __syncthreads();
        if (tid == 0) s_qid = atomicAdd(a.next_qid, 1);
        __syncthreads();
        const int qid = s_qid;
        if (qid >= a.Q) break;
        PHASE_DECL;

        for (int i = tid; i < a.table_words; i += NT) table[i] = 0u;
        for (int i = tid; i < dim; i += NT) qs[i] = a.queries[(size_t)qid * dim + i];
        if (tid == 0) s_ncand = 0, s_cntf = 0, s_nover = 0, s_cursor = 0, s_ntodo2 = 0, s_dup = 0;
        if (tid == 0) s_rows_screened = 0, s_rows_exact = 0, s_beam_words = 0;
        __syncthreads();

        float4 qreg[CPL];
#pragma unroll
        for (int t = 0; t < CPL; ++t) {
            const int c = gl + G * t;
            qreg[t] = c < chunks ? reinterpret_cast<const float4*>(qs)[c] : make_float4(0, 0, 0, 0);
        }
        // The query in integer codes for the screening on eight-bit rows (search_device.h).  Written by wave 0 alone;
        // first read after the barriers of the seeds' merge.
        signed char* qh8 = reinterpret_cast<signed char*>(qs + ((dim + 3) & ~3));
        signed char* ql8 = qh8 + ((dim + 15) & ~15);
        if (a.vec8 != nullptr && wave == 0) {
            float qq, sq, eq;
            code_query(qs, dim, lane, qh8, ql8, qq, sq, eq);
            if (lane == 0) s_qq = qq, s_qscale = sq, s_qerr = eq;
        }

        WgState st;
        st.nb = 0, st.cur = 0, st.live = kKeyMax;
        float thr = 3.402823466e+38f;  // signed form of the farthest sentinel
        int hops = 0, nd = 0, ne = 0, rounds = 0;
        // Counts that decide what the whole workgroup does next (merge first? measure the open rows first?) are
        // kept in registers, the same in every thread: each is read from LDS only behind a barrier that no thread's
        // next addition to it can overtake.  A thread that read the LDS count where it decides could see the
        // additions of wavefronts already a step ahead, and the workgroup would part ways.
        int ncand_u = 0, ntodo2_u = 0, nvis = 0;
        bool spill = false;

        // ---- screening phase (launches with a half-precision copy of the vectors): todo[0..T) -> todo2[0..s_ntodo2)
        //
        // Most ids a long search measures fail the round's frozen threshold.  Each row is first measured in its
        // half-precision copy (half the bytes; 512-byte rows that start on a cache line).  From that distance d16, the
        // norm of the row |x| (stored behind it) and the rounding bound of the format, |x - half(x)| <= 2^-11 |x|,
        // the exact distance d lies in [(sqrt(d16) - r)^2, (sqrt(d16) + r)^2], r = 2^-11 |x| + sqrt(dim) 2^-25 (the second
        // term for components below the format's normal range; both taken a little larger, and both ends widened by
        // 1e-4 to cover the fp32 rounding of either computation).  A row whose whole
        // interval lies beyond the frozen threshold is no candidate whatever its exact distance; one whose interval
        // lies below the threshold and beyond the beam's current worst entry is a candidate that is counted and
        // cannot enter the beam.  Only the rest -- possible beam entries and rows within 0.1 % of the threshold --
        // have their fp32 row read, by the distance phase below; results and counters are what they are without
        // the screening, bit for bit.
        auto screening_phase = [&](const uint32_t* list, int T) {
            if constexpr (G == 64) {
                constexpr int RPIH = 2 * U;  // two groups of 32 lanes per wave, U rows in flight per group
                const int glh = lane & 31, grph = lane >> 5;
                const int chunksH = (dim + 7) >> 3;  // 16-byte chunks of eight halves
                float4 qa[CPL][2];
#pragma unroll
                for (int t = 0; t < CPL; ++t) {
                    const int c = 2 * (glh + 32 * t);
                    qa[t][0] = c < chunks ? reinterpret_cast<const float4*>(qs)[c] : make_float4(0, 0, 0, 0);
                    qa[t][1] = c + 1 < chunks ? reinterpret_cast<const float4*>(qs)[c + 1] : make_float4(0, 0, 0, 0);
                }
                const float s_live = st.live == kKeyMax ? 3.402823466e+38f : key_s(st.live);
                // |x - half(x)| <= 2^-11 |x| holds for components that are normal numbers in half precision; one
                // below 6.1e-5 is rounded to a multiple of 2^-24, an absolute error of up to 2^-25: sqrt(dim) 2^-25
                // over a row
                const float r_abs = 1.0e-6f + 3.0e-8f * sqrtf((float)(chunksH * 8));
                int cnt = 0;
                for (int base = wave * RPIH; base < T; base += NW * RPIH) {
                    int vid[U];
                    const int r0 = base + grph * U;
#pragma unroll
                    for (int u = 0; u < U; ++u) vid[u] = (int)list[r0 + u];  // inside the lists' LDS
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (r0 + u >= T) vid[u] = -1;
                    uint4 h[U][CPL];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const uint4* row = reinterpret_cast<const uint4*>(
                            a.vec16 + (uint64_t)(uint32_t)(vid[u] < 0 ? 0 : vid[u]) * a.stride16);
#pragma unroll
                        for (int t = 0; t < CPL; ++t) {
                            const int c = glh + 32 * t;
                            h[u][t] = (vid[u] >= 0 && c < chunksH) ? row[c] : make_uint4(0u, 0u, 0u, 0u);
                        }
                    }
                    // the row this lane will file, and its norm
                    int myid = vid[0];
#pragma unroll
                    for (int u = 1; u < U; ++u)
                        if ((lane & (U - 1)) == u) myid = vid[u];
                    const bool valid = glh < U && myid >= 0;
                    float nx = 0.0f;
                    if (valid)
                        nx = *reinterpret_cast<const float*>(a.vec16 + (uint64_t)(uint32_t)myid * a.stride16 +
                                                             (size_t)chunksH * 16);
                    float acc[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        float sum = 0.0f;
#pragma unroll
                        for (int t = 0; t < CPL; ++t) {
                            const __half2* hp = reinterpret_cast<const __half2*>(&h[u][t]);
                            const float2 x0 = __half22float2(hp[0]), x1 = __half22float2(hp[1]);
                            const float2 x2 = __half22float2(hp[2]), x3 = __half22float2(hp[3]);
                            float d;
                            d = qa[t][0].x - x0.x, sum = __fmaf_rn(d, d, sum);
                            d = qa[t][0].y - x0.y, sum = __fmaf_rn(d, d, sum);
                            d = qa[t][0].z - x1.x, sum = __fmaf_rn(d, d, sum);
                            d = qa[t][0].w - x1.y, sum = __fmaf_rn(d, d, sum);
                            d = qa[t][1].x - x2.x, sum = __fmaf_rn(d, d, sum);
                            d = qa[t][1].y - x2.y, sum = __fmaf_rn(d, d, sum);
                            d = qa[t][1].z - x3.x, sum = __fmaf_rn(d, d, sum);
                            d = qa[t][1].w - x3.y, sum = __fmaf_rn(d, d, sum);
                        }
                        acc[u] = sum;
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        acc[u] = acc[u] + dpp_mov<0xB1>(acc[u]);   // quad_perm [1,0,3,2]
                        acc[u] = acc[u] + dpp_mov<0x4E>(acc[u]);   // quad_perm [2,3,0,1]
                        acc[u] = acc[u] + dpp_mov<0x141>(acc[u]);  // row_half_mirror
                        acc[u] = acc[u] + dpp_mov<0x140>(acc[u]);  // row_mirror
                    }
                    float mine = acc[0];
#pragma unroll
                    for (int u = 1; u < U; ++u)
                        if ((lane & (U - 1)) == u) mine = acc[u];
                    mine = mine + __shfl_xor(mine, 16, 64);
                    const float root = sqrtf(mine), r = 5.0e-4f * nx + r_abs;
                    const float lo_root = fmaxf(root - r, 0.0f), hi_root = root + r;
                    const float lo = lo_root * lo_root * (1.0f - 1.0e-4f), hi = hi_root * hi_root * (1.0f + 1.0e-4f);
                    // (a row with a component beyond the half format has an infinite norm: lo = 0, hi = inf)
                    const bool gone = valid && lo > thr;
                    const bool counted = valid && !gone && hi < thr && lo > s_live;
                    const bool exact = valid && !gone && !counted;
                    cnt += __popcll(__ballot(counted));
                    const uint64_t m = __ballot(exact);
                    if (m) {
                        int pos = 0;
                        if (lane == 0) pos = atomicAdd(&s_ntodo2, __popcll(m));
                        pos = __shfl(pos, 0, 64);
                        if (exact) todo2[pos + prefix_popc(m)] = (uint32_t)myid;
                    }
                }
                if (lane == 0 && cnt) atomicAdd(&s_cntf, cnt);
            }
        };

        // ---- screening phase on eight-bit codes (launches with a.vec8; bounds: search_device.h): the same three
        // classes from a quarter of the bytes.  Sixteen lanes per row (a 256-byte row at dim 200: two cache lines),
        // eight rows in flight per group, four groups per wavefront.
        auto screening_phase8 = [&](const uint32_t* list, int T) {
            if constexpr (G >= 32) {  // dim > 64: a row's code chunks are CPL per lane of its sixteen
                constexpr int CPL8 = CPL, U8 = 8 / CPL8, RPI8 = 4 * U8;
                constexpr bool WIDE8 = CPL8 > 2;  // rows of more than 512 codes: the coded query stays in LDS
                const int gl8 = lane & 15, grp8 = lane >> 4;
                const int nck = (dim + 15) >> 4;  // chunks of sixteen codes; the row's three figures are chunk nck
                CodedQuery<WIDE8 ? 1 : CPL8> cq;
                if constexpr (!WIDE8) load_coded_query<CPL8>(qh8, ql8, nck, gl8, cq);
                const float qq = s_qq, sq = s_qscale, eq = s_qerr;
                const float s_live = st.live == kKeyMax ? 3.402823466e+38f : key_s(st.live);
                const uint32_t st8 = (uint32_t)a.stride8;
                int cnt = 0;
                for (int base = wave * RPI8; base < T; base += NW * RPI8) {
                    int vid[U8];
                    const int r0 = base + grp8 * U8;
#pragma unroll
                    for (int u = 0; u < U8; ++u) vid[u] = (int)list[r0 + u];  // inside the lists' LDS
#pragma unroll
                    for (int u = 0; u < U8; ++u)
                        if (r0 + u >= T) vid[u] = -1;
                    const int mi = r0 + gl8;
                    int myid = (int)list[mi];  // the row this lane files (inside the lists' LDS)
                    if (gl8 >= U8 || mi >= T) myid = -1;
                    const bool valid = myid >= 0;
                    float lo, hi;
                    if constexpr (WIDE8)
                        coded_rows_bounds_wide<CPL8, U8>(a.vec8, st8, nck, gl8, vid, myid, qh8, ql8, qq, sq, eq, a.metric, lo, hi);
                    else
                        coded_rows_bounds<CPL8, U8>(a.vec8, st8, nck, gl8, vid, myid, cq, qq, sq, eq, a.metric, lo, hi);
                    const bool gone = valid && lo > thr;
                    const bool counted = valid && !gone && hi < thr && lo > s_live;
                    const bool exact = valid && !gone && !counted;
                    cnt += __popcll(__ballot(counted));
                    const uint64_t m = __ballot(exact);
                    if (m) {
                        int pos = 0;
                        if (lane == 0) pos = atomicAdd(&s_ntodo2, __popcll(m));
                        pos = __shfl(pos, 0, 64);
                        if (exact) todo2[pos + prefix_popc(m)] = (uint32_t)myid;
                    }
                }
                if (lane == 0 && cnt) atomicAdd(&s_cntf, cnt);
            }
        };

        // ---- distance phase: list[0..T) -> cand[], counting passes of the frozen threshold
        auto distance_phase = [&](const uint32_t* list, int T) {
            int cntf = 0;
            for (int base = wave * RPI; base < T; base += NW * RPI) {
                // all ids of this iteration first (one LDS wait), then all row requests back to back
                int vid[U];
                const int r0 = base + grp * U;
#pragma unroll
                for (int u = 0; u < U; ++u) vid[u] = (int)list[r0 + u];  // inside the list's capacity
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (r0 + u >= T) vid[u] = -1;
                float4 v[U][CPL];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const float4* row = reinterpret_cast<const float4*>(
                        a.vec + (uint64_t)(uint32_t)(vid[u] < 0 ? 0 : vid[u]) * (uint32_t)dim);
#pragma unroll
                    for (int t = 0; t < CPL; ++t) {
                        const int c = gl + G * t;
                        v[u][t] = (vid[u] >= 0 && c < chunks) ? row[c] : make_float4(0, 0, 0, 0);
                    }
                }
                float acc[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    float s = 0.0f;
#pragma unroll
                    for (int t = 0; t < CPL; ++t) {
                        if (a.metric == 0) {
                            float d;
                            d = qreg[t].x - v[u][t].x, s = __fmaf_rn(d, d, s);
                            d = qreg[t].y - v[u][t].y, s = __fmaf_rn(d, d, s);
                            d = qreg[t].z - v[u][t].z, s = __fmaf_rn(d, d, s);
                            d = qreg[t].w - v[u][t].w, s = __fmaf_rn(d, d, s);
                        } else {
                            s = __fmaf_rn(qreg[t].x, v[u][t].x, s);
                            s = __fmaf_rn(qreg[t].y, v[u][t].y, s);
                            s = __fmaf_rn(qreg[t].z, v[u][t].z, s);
                            s = __fmaf_rn(qreg[t].w, v[u][t].w, s);
                        }
                    }
                    acc[u] = s;
                }
                // Cross-lane butterfly p[l] += p[l ^ off], off = 1, 2, 4, ..., G/2.  Inside a row of
                // 16 lanes it runs on DPP (register speed): after off = 1, 2 a quad holds one value,
                // so l ^ 7 (row_half_mirror) stands for l ^ 4 and l ^ 15 (row_mirror) for l ^ 8 with
                // bit-identical results.  Across rows each lane only needs the row it will file, so it
                // first picks that row's partial and the last one or two levels cost one exchange each.
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    acc[u] = acc[u] + dpp_mov<0xB1>(acc[u]);   // quad_perm [1,0,3,2]
                    acc[u] = acc[u] + dpp_mov<0x4E>(acc[u]);   // quad_perm [2,3,0,1]
                    acc[u] = acc[u] + dpp_mov<0x141>(acc[u]);  // row_half_mirror
                    acc[u] = acc[u] + dpp_mov<0x140>(acc[u]);  // row_mirror
                }
                float mine = acc[0];
                int myid = vid[0];
#pragma unroll
                for (int u = 1; u < U; ++u)
                    if ((lane & (U - 1)) == u) mine = acc[u], myid = vid[u];
                if (G >= 32) mine = mine + __shfl_xor(mine, 16, 64);
                if (G >= 64) mine = mine + __shfl_xor(mine, 32, 64);
                const bool valid = gl < U && myid >= 0;
                const float s = a.metric == 0 ? mine : 0.0f - mine;
                const bool pf = valid && (s < thr);
                const uint64_t key = make_key(s, myid, 0u);
                const bool app = pf && key < st.live;
                cntf += __popcll(__ballot(pf));
                const uint64_t m = __ballot(app);
                if (m) {
                    int pos = 0;
                    if (lane == 0) pos = atomicAdd(&s_ncand, __popcll(m));
                    pos = __shfl(pos, 0, 64);
                    if (app) cand[pos + prefix_popc(m)] = key;
                }
            }
            if (lane == 0 && cntf) atomicAdd(&s_cntf, cntf);
        };

        // ---- merge cand[0..s_ncand) into the beam (all threads; barriers inside)
        auto merge = [&]() {
            __syncthreads();
            const int nc = s_ncand;
            if (nc == 0) return;
            if (nc <= kSmallMerge) {
                // few candidates (every best-first step, the late rounds): no sort; a key's place
                // is its own index plus the number of smaller keys in the other list, and the
                // candidates are few enough to be counted by reading them all (broadcast reads)
                const uint64_t* src = st.cur ? beam1 : beam0;
                uint64_t* dst = st.cur ? beam0 : beam1;
                const int nb = st.nb;
                for (int i = tid; i < nb; i += NT) {
                    const uint64_t key = src[i];
                    int below = 0;
                    for (int c = 0; c < nc; ++c) below += cand[c] < key;
                    if (i + below < L) dst[i + below] = key;
                }
                for (int j = tid; j < nc; j += NT) {
                    const uint64_t key = cand[j];
                    int below = 0;
                    for (int c = 0; c < nc; ++c) below += cand[c] < key;
                    const int pos = below + lower_bound_u64(src, nb, key);
                    if (pos < L) dst[pos] = key;
                    if (below == 0 && pos < s_cursor) s_cursor = pos;
                }
                __syncthreads();
                st.nb = min(L, nb + nc);
                st.cur ^= 1;
                st.live = st.nb == L ? dst[L - 1] : kKeyMax;
                if (tid == 0) s_ncand = 0;
                if (BIG && tid == 0) s_beam_words += 2 * (nb + st.nb);  // one pass: nb keys read, st.nb written
                ncand_u = 0;
                __syncthreads();
                return;
            }
            int P = 2;
            while (P < nc) P <<= 1;
            for (int i = nc + tid; i < P; i += NT) cand[i] = kKeyMax;
            __syncthreads();
            // Bitonic sort of cand[0..P).  Blocks of 128 keys belong to one wave each: every
            // step whose partner distance stays inside a block needs no workgroup barrier
            // (LDS operations of one wave complete in order), only the few steps that
            // cross blocks do.
            const int B = P < 128 ? P : 128, nblk = P / B;
            auto exchange = [&](int i, int j, int k2) {
                const int x = i + j;
                const bool asc = (i & k2) == 0;
                const uint64_t ka = cand[i], kb = cand[x];
                if ((ka > kb) == asc) cand[i] = kb, cand[x] = ka;
            };
            auto wave_sync = [&]() {
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            };
            auto block_steps = [&](int k2, int jfrom) {  // steps j = jfrom .. 1 of stage k2, inside blocks
                for (int blk = wave; blk < nblk; blk += NW) {
                    for (int j = jfrom; j > 0; j >>= 1) {
                        if (lane < (B >> 1)) exchange(blk * B + 2 * lane - (lane & (j - 1)), j, k2);
                        wave_sync();
                    }
                }
            };
            for (int k2 = 2; k2 <= B; k2 <<= 1) block_steps(k2, k2 >> 1);
            __syncthreads();
            for (int k2 = 2 * B; k2 <= P; k2 <<= 1) {
                for (int j = k2 >> 1; j >= B; j >>= 1) {
                    for (int t = tid; t < (P >> 1); t += NT) exchange(2 * t - (t & (j - 1)), j, k2);
                    __syncthreads();
                }
                block_steps(k2, B >> 1);
                __syncthreads();
            }
            const uint64_t* src = st.cur ? beam1 : beam0;
            uint64_t* dst = st.cur ? beam0 : beam1;
            const int nb = st.nb;
            if constexpr (BIG) {
                // The beam is in global memory: every access is a trip to L2 or beyond.  Beam keys are fetched eight
                // per thread before the first is placed, and keys outside the candidates' range need no search.
                // A candidate's place is its index plus the number of beam keys below it.  That number is not
                // searched for in the beam (a chain of dependent reads from memory): every beam key has just found
                // its own count b of candidates below it, and the keys below candidate j are exactly those with
                // b <= j.  So the keys are counted per value of b (16-bit counts, two to a word, in the LDS that
                // holds the sample otherwise; one addition per run of equal values among a wavefront's 64
                // consecutive keys) and a prefix sum over the counts gives every candidate its place.  Beams of
                // 65536 keys and more, or more candidates than there are counts, take the search: through an LDS
                // sample of every 2^ss-th beam key, then the last few steps in memory.
                const bool counted = nc <= 4 * a.scap && nb < 65536;
                uint32_t* cnt = reinterpret_cast<uint32_t*>(samp);
                const int ncw = (nc + 1) >> 1;
                int ss = 0, ns = 0;
                if (counted) {
                    for (int w = tid; w < ncw; w += NT) cnt[w] = 0u;
                    __syncthreads();
                } else {
                    while (((nb - 1) >> ss) + 1 > a.scap) ++ss;
                    ns = nb > 0 ? ((nb - 1) >> ss) + 1 : 0;
                    for (int j = tid; j < ns; j += NT) samp[j] = src[(size_t)j << ss];
                }
                const uint64_t c_lo = cand[0], c_hi = cand[nc - 1];
                for (int i0 = tid; i0 < nb; i0 += 8 * NT) {
                    uint64_t key[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) key[u] = i0 + u * NT < nb ? src[i0 + u * NT] : kKeyMax;
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int i = i0 + u * NT;
                        int below = nc;  // (a lane past the beam's end counts nothing)
                        if (i < nb) {
                            below = key[u] < c_lo ? 0 : key[u] > c_hi ? nc : lower_bound_u64(cand, nc, key[u]);
                            if (i + below < L) dst[i + below] = key[u];
                        }
                        if (counted) {
                            // the wavefront's keys ascend with the lane, and so do their counts: the lanes with
                            // below < nc are the first few, and equal counts sit side by side
                            const int prev = __shfl_up(below, 1, 64);
                            const bool in = below < nc;
                            const bool head = in && (lane == 0 || prev != below);
                            const uint64_t hm = __ballot(head);
                            const int nin = __popcll(__ballot(in));
                            if (head) {
                                const uint64_t after = hm & ~((2ull << lane) - 1ull);  // heads in the lanes above
                                const int end = after ? min(__ffsll((long long)after) - 1, nin) : nin;
                                atomicAdd(&cnt[below >> 1], (uint32_t)(end - lane) << (16 * (below & 1)));
                            }
                        }
                    }
                }
                __syncthreads();  // the counts (or the sample) are complete
                if (counted) {
                    int base = 0;  // beam keys below the candidates of the passes before
                    for (int w0 = 0; w0 < ncw; w0 += NT) {
                        const int w = w0 + tid;
                        const uint32_t c2 = w < ncw ? cnt[w] : 0u;
                        const int c_even = (int)(c2 & 0xffffu), c_odd = (int)(c2 >> 16);
                        const int incl = wave_inclusive_sum(c_even + c_odd);
                        if (lane == 63) s_wcnt[wave] = incl;
                        __syncthreads();
                        int before = base, total = 0;
                        for (int x = 0; x < NW; ++x) {
                            const int c = s_wcnt[x];
                            before += x < wave ? c : 0;
                            total += c;
                        }
                        const int excl = before + incl - (c_even + c_odd);
                        const int j = 2 * w;
                        if (j < nc) {
                            const int pos = j + excl + c_even;
                            if (pos < L) dst[pos] = cand[j];
                            if (j == 0 && pos < s_cursor) s_cursor = pos;  // entries before the cursor are all expanded
                        }
                        if (j + 1 < nc) {
                            const int pos = j + 1 + excl + c_even + c_odd;
                            if (pos < L) dst[pos] = cand[j + 1];
                        }
                        base += total;
                        __syncthreads();  // the wavefronts' totals are read before the next pass posts its own
                    }
                } else {
                    for (int j = tid; j < nc; j += NT) {
                        const uint64_t key = cand[j];
                        const int js = lower_bound_u64(samp, ns, key);
                        int lo = js == 0 ? 0 : ((js - 1) << ss) + 1, hi = js == ns ? nb : (js << ss);
                        while (lo < hi) {
                            const int mid = (lo + hi) >> 1;
                            if (src[mid] < key)
                                lo = mid + 1;
                            else
                                hi = mid;
                        }
                        const int pos = j + lo;
                        if (pos < L) dst[pos] = key;
                        if (j == 0 && pos < s_cursor) s_cursor = pos;  // entries before the cursor are all expanded
                    }
                }
            } else {
                for (int i = tid; i < nb; i += NT) {
                    const uint64_t key = src[i];
                    const int pos = i + lower_bound_u64(cand, nc, key);
                    if (pos < L) dst[pos] = key;
                }
                for (int j = tid; j < nc; j += NT) {
                    const uint64_t key = cand[j];
                    const int pos = j + lower_bound_u64(src, nb, key);
                    if (pos < L) dst[pos] = key;
                    if (j == 0 && pos < s_cursor) s_cursor = pos;  // entries before the cursor are all expanded
                }
            }
            __syncthreads();
            st.nb = min(L, nb + nc);
            st.cur ^= 1;
            st.live = st.nb == L ? dst[L - 1] : kKeyMax;
            if (tid == 0) s_ncand = 0;
            if (BIG && tid == 0) s_beam_words += 2 * (nb + st.nb);  // one pass: nb keys read, st.nb written
            ncand_u = 0;
            __syncthreads();
        };

        // ---- the rows the screening left open, todo2[0..s_ntodo2): exact distances (entered by every thread after a
        // barrier; the candidates they add must fit the buffer)
        const bool screening = (a.vec16 != nullptr || a.vec8 != nullptr) && a.policy == 0;
        auto flush_exact = [&]() {
            const int n2 = ntodo2_u;
            if (n2 == 0) return;
            if (ncand_u + n2 > CCAP) merge();  // merge() starts and ends with a barrier
            PHASE_MARK(5);
            distance_phase(todo2, n2);
            __syncthreads();
            if (tid == 0) s_ntodo2 = 0, s_rows_exact += n2;
            ncand_u = s_ncand, ntodo2_u = 0;  // (the next additions to either lie behind the barrier below)
            __syncthreads();
            PHASE_MARK(4);
        };

        // ---- the screening of todo[0..T): in pieces that the list for the exact pass has room for whatever the
        // screening leaves (entered by every thread after a barrier, ends with one)
        auto screen_list = [&](int T) {
            for (int off = 0; off < T;) {
                // (what is left goes in one piece where the emptied list could take it whole: a small second piece
                // is one more exposed wait)
                int n = min(T - off, a.tcap2 - ntodo2_u);
                if (n < (T - off <= a.tcap2 ? T - off : a.tcap2 / 2)) {
                    flush_exact();
                    n = min(T - off, a.tcap2);
                }
                if (a.vec8 != nullptr)
                    screening_phase8(todo + off, n);
                else
                    screening_phase(todo + off, n);
                __syncthreads();
                ntodo2_u = s_ntodo2;
                if (tid == 0) s_rows_screened += n;
                PHASE_MARK(7);
                off += n;
                if (off < T) __syncthreads();  // every thread has the count before the next piece adds to it
            }
        };

        PHASE_MARK(0);
        // ---- seeds: every start id is visited and measured, none counts as a hop
        const int M = a.M;
        for (int i = tid; i < M; i += NT) {
            const uint32_t id = (uint32_t)a.start_ids[i];
            vs.test_and_set(id, false);
            todo[i] = id;
        }
        __syncthreads();
        distance_phase(todo, M);
        merge();
        PHASE_MARK(1);
        if (tid == 0) s_cntf = 0, s_rows_exact += M;
        nd = M, nvis = M;
        if (a.policy == 1) hops = M;

        // ---- rounds
        for (;;) {
            uint64_t* beam = st.cur ? beam1 : beam0;
            const int nb0 = st.nb;
            if (tid == 0) s_nexp = 0;
            __syncthreads();
            if (a.policy == 0) {
                for (int i0 = 0; i0 < nb0; i0 += NT) {
                    const int i = i0 + tid;
                    uint64_t key = 0;
                    bool un = false;
                    if (i < nb0) key = beam[i], un = (key & 1ull) == 0;
                    const uint64_t m = __ballot(un);
                    if (m) {
                        int pos = 0;
                        if (lane == 0) pos = atomicAdd(&s_nexp, __popcll(m));
                        pos = __shfl(pos, 0, 64);
                        if (un) {
                            elist[pos + prefix_popc(m)] = (uint32_t)key_id(key);
                            beam[i] = key | 1ull;
                        }
                    }
                }
            } else if (wave == 0) {
                // best first: the closest entry not yet expanded.  s_cursor is a lower bound of
                // its index (kept by the merge); wave 0 scans on from there 64 entries at a time
                int c = s_cursor, found = nb0;
                while (c < nb0) {
                    const int i = c + lane;
                    const bool un = i < nb0 && (beam[i] & 1ull) == 0;
                    const uint64_t m = __ballot(un);
                    if (m) {
                        found = c + (__ffsll((long long)m) - 1);
                        break;
                    }
                    c += 64;
                }
                if (lane == 0) {
                    if (found < nb0) {
                        const uint64_t key = beam[found];
                        elist[0] = (uint32_t)key_id(key);
                        beam[found] = key | 1ull;
                        s_nexp = 1;
                        s_cursor = found + 1;
                    } else {
                        s_cursor = nb0;
                    }
                }
            }
            __syncthreads();
            const int nexp = s_nexp;
            // (rounds: the scan read the beam's nb0 keys and flagged nexp of them; the expand list is written, then read)
            if (BIG && tid == 0) s_beam_words += (a.policy == 0 ? 2 * nb0 : 128) + 4 * nexp;
            PHASE_MARK(2);
            if (nexp == 0) {
                // a round that finds every entry expanded still counts: the candidates of the round that first
                // overfilled the beam can all have fallen behind its L entries
                if (a.policy == 0) ++rounds;
                break;
            }

            // The round's rows are taken in chunks of `ech` beam entries (what the todo list holds).  Where one
            // pass of the workgroup covers a chunk's ids (ech * R <= threads) and the launch asks for it, a chunk's
            // ids are requested one chunk ahead -- and the entry whose row they come from two chunks ahead -- so
            // that both waits pass while the chunk before is being measured.  With two workgroups per CU the other
            // workgroup covers those waits and the look-ahead only costs (measured); with one it pays.
            const int ech = (screening ? min(TCAP, NT) : TCAP) / R;
            ne += nexp;
            const bool ahead = a.prefetch_rows != 0 && ech * R <= NT;
            const int pe = tid / R, pj = tid - pe * R;  // this thread's entry of a chunk and neighbour slot
            int vpre = -1;
            uint32_t epre = 0;
            if (ahead) {
                if (pe < min(ech, nexp)) vpre = a.nbrs[(size_t)elist[pe] * R + pj];
                if (pe < ech && ech + pe < nexp) epre = elist[ech + pe];
            }
            // With a screening, the ids of several chunks collect in the todo list (while the next chunk's could
            // all still join it) and are screened together: a screening of a few hundred rows is one exposed
            // memory wait, of a thousand and more the same wait and some work under it.  (Screening only
            // whole passes of the workgroup, the rest waiting in the list for the next ids, gains nothing: measured.)
            int tprev = 0;  // ids in the todo list from the chunks before, not yet screened
            for (int e0 = 0; e0 < nexp; e0 += ech) {
                if (!spill && nvis > a.vis_limit) spill = true;
                if (tid == 0 && tprev == 0) s_ntodo = 0;
                __syncthreads();
                const int total = min(ech, nexp - e0) * R;
                for (int f0 = 0; f0 < total; f0 += NT) {
                    const int f = f0 + tid;
                    int v = -1;
                    if (ahead) {
                        v = vpre;
                    } else if (f < total) {
                        const int e = f / R;
                        v = a.nbrs[(size_t)elist[e0 + e] * R + (f - e * R)];
                    }
                    bool isnew = false;
                    if (v >= 0) isnew = vs.test_and_set((uint32_t)v, spill) != 0;
                    const uint64_t m = __ballot(isnew);
                    if (m) {
                        int pos = 0;
                        if (lane == 0) pos = atomicAdd(&s_ntodo, __popcll(m));
                        pos = __shfl(pos, 0, 64);
                        if (isnew) todo[pos + prefix_popc(m)] = (uint32_t)v;
                    }
                }
                __syncthreads();
                int tall = s_ntodo;
                if (vs.buckets) {
                    // (read by every thread behind the barrier above; the next chunk's inserts lie behind the barrier
                    // at its start)
                    if (s_dup != 0) {
                        // Two threads may have inserted the same id at the same time (see VisitedSet): an id of this
                        // chunk that stands in the list before is struck out, and the list closed up.  An id's first
                        // entry is never struck, so the later ones find it whatever else is struck meanwhile.
                        for (int i = tprev + tid; i < tall; i += NT) {
                            const uint32_t id = todo[i];
                            bool rep = false;
                            for (int j = tprev; j < i && !rep; ++j) rep = todo[j] == id;
                            if (rep) todo[i] = 0xffffffffu;
                        }
                        __syncthreads();
                        if (wave == 0) {
                            int out = tprev;
                            for (int i0 = tprev; i0 < tall; i0 += 64) {
                                const int i = i0 + lane;
                                const uint32_t id = i < tall ? todo[i] : 0xffffffffu;
                                const uint64_t m = __ballot(id != 0xffffffffu);
                                if (id != 0xffffffffu) todo[out + prefix_popc(m)] = id;  // (out + rank <= i: the chunk was read whole before)
                                out += __popcll(m);
                            }
                            if (lane == 0) s_ntodo = out, s_dup = 0, atomicAdd(a.spill_count + 1, 1);
                        }
                        __syncthreads();
                        tall = s_ntodo;
                    }
                }
                const int T = tall - tprev;
                nd += T;
                PHASE_MARK(3);
                if (!screening && ncand_u + T > CCAP) merge();  // merge() starts and ends with a barrier
                PHASE_MARK(5);
                nvis += T;
                if (ahead) {
                    // the next chunk's ids (their entries arrived a chunk ago) and the entries of the chunk after
                    vpre = -1;
                    const int e1 = e0 + ech, e2 = e0 + 2 * ech;
                    if (pe < ech && e1 + pe < nexp) vpre = a.nbrs[(size_t)epre * R + pj];
                    if (pe < ech && e2 + pe < nexp) epre = elist[e2 + pe];
                }
                if (screening) {
                    // what the screening leaves for the exact pass collects over the chunks of a round (the round's
                    // threshold does not move) and is measured when the list could overflow, and at the round's end
                    if (e0 + ech >= nexp || tall + ech * R > TCAP) {
                        screen_list(tall);
                        tprev = 0;
                    } else {
                        tprev = tall;
                    }
                } else {
                    distance_phase(todo, T);
                    __syncthreads();
                    if (tid == 0) s_rows_exact += T;
                    ncand_u = s_ncand;  // (the next chunk's additions lie behind the barrier at its start)
                }
                PHASE_MARK(4);
            }
            if (screening) flush_exact();
            ++rounds;
            const int cntf = s_cntf;
            if (a.policy == 0) {
                if (cntf == 0) break;
                hops += cntf;
            } else {
                hops += 1;
            }
            merge();
            PHASE_MARK(5);
            if (tid == 0) s_cntf = 0;
            if (a.policy == 0 && nb0 + cntf > L) thr = key_s((st.cur ? beam1 : beam0)[L - 1]);
        }

        // ---- output: the k closest live entries, closest first
        {
            __syncthreads();
            const uint64_t* beam = st.cur ? beam1 : beam0;
            int32_t* ids_out = a.ids_out + (size_t)qid * a.k;
            float* dists_out = a.dists_out ? a.dists_out + (size_t)qid * a.k : nullptr;
            // ordered compaction: every wave posts how many live entries it holds, and each finds its place
            // from the counts of the waves before it; outpos is the same in every thread
            int outpos = 0;
            for (int i0 = 0; i0 < st.nb && outpos < a.k; i0 += NT) {
                const int i = i0 + tid;
                uint64_t key = 0;
                bool livee = false;
                if (i < st.nb) {
                    key = beam[i];
                    livee = true;
                    if (a.deleted) {
                        const int32_t id = key_id(key);
                        livee = ((a.deleted[id >> 5] >> (id & 31)) & 1u) == 0;
                    }
                }
                const uint64_t m = __ballot(livee);
                if (lane == 0) s_wcnt[wave] = __popcll(m);
                __syncthreads();
                int before = 0, total = 0;
                for (int w = 0; w < NW; ++w) {
                    const int c = s_wcnt[w];
                    before += w < wave ? c : 0;
                    total += c;
                }
                const int pos = outpos + before + prefix_popc(m);
                if (livee && pos < a.k) {
                    ids_out[pos] = key_id(key);
                    if (dists_out) {
                        const float s = key_s(key);
                        dists_out[pos] = a.metric == 0 ? s : 0.0f - s;
                    }
                }
                outpos += total;
                __syncthreads();  // the counts are read before the next chunk posts its own
            }
            for (int i = outpos + tid; i < a.k; i += NT) {
                ids_out[i] = -1;
                // unfilled slots: the farthest sentinel (rounds: +-FLT_MAX as the CUDA kernel pads its
                // beam, src/search_gpu.cu:408; best-first: +-infinity, src/search_in_cpu.cpp:33-35)
                if (dists_out) {
                    const float far = a.policy == 1 ? __int_as_float(0x7f800000) : 3.402823466e+38f;
                    dists_out[i] = a.metric == 0 ? far : -far;
                }
            }
            if (tid == 0) {
                int32_t* c = a.counters + (size_t)qid * 4;
                c[0] = hops, c[1] = ne, c[2] = nd, c[3] = rounds;
                {
                    int32_t* rc = a.counters + ((size_t)a.Q + qid) * 4;
                    // (ids sent to the bitmap in global memory: one atomic each; the clean-up writes them once more)
                    rc[0] = s_rows_screened, rc[1] = s_rows_exact, rc[2] = s_beam_words, rc[3] = 2 * s_nover;
                }
                if (s_nover > 0) atomicAdd(a.spill_count, 1);
            }
            // leave the global bitmap clean: word by word from the list, or all of it
            const int nover = s_nover;
            if (nover > a.ocap) {
                for (size_t i = tid; i < a.spill_words; i += NT) vs.bitmap[i] = 0u;
            } else {
                for (int i = tid; i < nover; i += NT) atomicExch(&vs.bitmap[olist[i] >> 5], 0u);
            }
            if (nover > 0) __threadfence();
            PHASE_MARK(6);
            PHASE_FLUSH();
        }
    }
}

// hits = sum_q |res[q][0..k) n gt[q][0..k)| (src/search_gpu.cu:888-907)
__global__ void ids_verify_kernel(const int32_t* __restrict__ res, const int32_t* __restrict__ gt,
                                  unsigned long long* hit, int Q, int k) {
    __shared__ int s_hit;
    for (int q = blockIdx.x; q < Q; q += gridDim.x) {
        if (threadIdx.x == 0) s_hit = 0;
        __syncthreads();
        const int32_t* g = gt + (size_t)q * k;
        int mine = 0;
        for (int i = threadIdx.x; i < k; i += blockDim.x) {
            const int32_t id = res[(size_t)q * k + i];
            for (int j = 0; j < k; ++j)
                if (g[j] == id) {
                    ++mine;
                    break;
                }
        }
        if (mine) atomicAdd(&s_hit, mine);
        __syncthreads();
        if (threadIdx.x == 0 && s_hit) atomicAdd(hit, (unsigned long long)s_hit);
        __syncthreads();
    }
}

__global__ void fill_u32_kernel(uint32_t* p, size_t n, uint32_t v) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (size_t)gridDim.x * blockDim.x)
        p[i] = v;
}

// ------------------------------------------------------------------ launchers

typedef void (*kernel_fn)(const SearchArgs);

template <bool BIG>
static kernel_fn pick_kernel_form(int chunks) {
    if (chunks <= 16) return beam_search_kernel<16, 1, BIG>;
    if (chunks <= 32) return beam_search_kernel<32, 1, BIG>;
    if (chunks <= 64) return beam_search_kernel<64, 1, BIG>;
    if (chunks <= 128) return beam_search_kernel<64, 2, BIG>;
    if (chunks <= 256) return beam_search_kernel<64, 4, BIG>;
    if (chunks <= 512) return beam_search_kernel<64, 8, BIG>;
    return nullptr;
}

static kernel_fn pick_kernel(int dim, bool big) {
    return big ? pick_kernel_form<true>(dim / 4) : pick_kernel_form<false>(dim / 4);
}

size_t search_lds_bytes(int L, int dim, int table_words, int tcap, int ccap, int ocap, bool big, bool screening) {
    const size_t Lp = (size_t)((L + 3) & ~3);
    if (screening) tcap += search_exact_list_cap(tcap);  // the list of rows the screening leaves for the exact pass
    const size_t beams = big ? (size_t)kBeamSampleKeys * 8 : Lp * 8 * 2 + Lp * 4;  // (big: the merge's sample) two key buffers and the expand list
    const size_t coded_query = screening ? 2 * (size_t)((dim + 15) & ~15) : 0;  // two bytes per dimension
    return beams + (size_t)ccap * 8 + (size_t)table_words * 4 + (size_t)tcap * 4 + (size_t)ocap * 4 +
           (size_t)((dim + 3) & ~3) * 4 + coded_query;
}

size_t search_beam_stride(int L) {
    const size_t Lp = (size_t)((L + 3) & ~3);
    return (2 * Lp + Lp / 2 + 15) & ~(size_t)15;  // [2][Lp] keys + Lp 32-bit ids, a multiple of 128 bytes
}

hipError_t search_kernel_prepare(int dim, bool big, size_t lds_bytes, int threads, int* max_wg_per_cu) {
    kernel_fn fn = pick_kernel(dim, big);
    if (!fn) return hipErrorInvalidValue;
    // The limit on a kernel's dynamic LDS is only ever raised: a launch planned earlier (the entry point that
    // allocates nothing keeps its plan) must stay valid after a later plan for a shorter beam.
    static std::mutex mu;
    static std::map<std::pair<const void*, int>, size_t> limit;
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    {
        std::lock_guard<std::mutex> lock(mu);
        size_t& have = limit[{reinterpret_cast<const void*>(fn), device}];
        if (lds_bytes > have) {
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds_bytes);
            if (e != hipSuccess) return e;
            have = lds_bytes;
        }
    }
    int nb = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, reinterpret_cast<const void*>(fn), threads,
                                                     lds_bytes);
    if (e != hipSuccess) return e;
    *max_wg_per_cu = nb;
    return hipSuccess;
}

hipError_t launch_search(const SearchArgs& a, bool big, int workgroups, int threads, size_t lds_bytes,
                         hipStream_t stream) {
    kernel_fn fn = pick_kernel(a.dim, big);
    if (!fn) return hipErrorInvalidValue;
    hipLaunchKernelGGL(fn, dim3(workgroups), dim3(threads), lds_bytes, stream, a);
    return hipGetLastError();
}

// ---- the block of device memory for callers that must not allocate
//
// `scratch` lives in the code object; in host code its name is only a handle for hipGetSymbolAddress, never an
// address a kernel could use.  Every device that loads the library holds its own copy at its own address.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];
}  // namespace

hipError_t static_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    if (__atomic_load_n(&g_scratch_ptr[device], __ATOMIC_ACQUIRE)) return hipSuccess;
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    __atomic_store_n(&g_scratch_ptr[device], p, __ATOMIC_RELEASE);  // (two racing threads store the same address)
    return hipSuccess;
}

void* static_scratch(int device) {
    if (device < 0 || device >= kMaxDevices) return nullptr;
    return __atomic_load_n(&g_scratch_ptr[device], __ATOMIC_ACQUIRE);
}

// Half-precision copy of the vectors for the screening phase: row i = dim halves (round to nearest), zero padding up
// to a whole 16-byte chunk, then |x_i| as a float (rounded up a little; infinite when a component does not fit the
// format, which sends the row to the exact pass every time), rows `stride` bytes apart.
__global__ __launch_bounds__(256) void half_rows_kernel(const float* __restrict__ vec, int64_t n, int dim,
                                                        unsigned char* __restrict__ out, size_t stride) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    const int padded = (dim + 7) & ~7;
    for (int64_t row = wave; row < n; row += nwaves) {
        const float* x = vec + row * dim;
        __half* h = reinterpret_cast<__half*>(out + (size_t)row * stride);
        float sum = 0.0f;
        bool bad = false;
        for (int j = lane; j < padded; j += 64) {
            const float v = j < dim ? x[j] : 0.0f;
            h[j] = __float2half_rn(v);
            sum = __fmaf_rn(v, v, sum);
            bad |= !(fabsf(v) <= 65504.0f);
        }
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
        bad = __ballot(bad) != 0ull;
        if (lane == 0)
            *reinterpret_cast<float*>(out + (size_t)row * stride + (size_t)padded * 2) =
                bad ? __int_as_float(0x7f800000) : sqrtf(sum) * (1.0f + 1.0e-5f);
    }
}

// Eight-bit copy of the vectors for the screening phase: row i = codes k_j = round(x_j / s), s = max |x_j| / 127, as
// signed bytes, zero padding up to a whole 16-byte chunk, then three floats: s, |x~|^2 and e >= |x - x~| for
// x~ = s k (both from sums in double precision, e rounded up).  A row whose largest component is not in
// [1e-18, 1e17] (or not finite) gets e = inf, which sends it to the exact pass every time; a zero row is exact.
__global__ __launch_bounds__(256) void byte_rows_kernel(const float* __restrict__ vec, int64_t n, int dim,
                                                        unsigned char* __restrict__ out, size_t stride) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    const int padded = (dim + 15) & ~15;
    for (int64_t row = wave; row < n; row += nwaves) {
        const float* x = vec + row * dim;
        signed char* codes = reinterpret_cast<signed char*>(out + (size_t)row * stride);
        float amax = 0.0f;
        bool bad = false;
        for (int j = lane; j < dim; j += 64) {
            const float v = fabsf(x[j]);
            bad |= !(v <= 3.0e38f);
            amax = fmaxf(amax, v);
        }
        for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
        bad = __ballot(bad) != 0ull || (amax != 0.0f && !(amax >= 1.0e-18f && amax <= 1.0e17f));
        const float s = bad ? 0.0f : amax / 127.0f;
        double se = 0.0, sx = 0.0;
        for (int j = lane; j < padded; j += 64) {
            const float v = j < dim ? x[j] : 0.0f;
            int k = 0;
            if (s > 0.0f) {
                k = (int)rintf(v / s);
                k = k > 127 ? 127 : (k < -127 ? -127 : k);
            }
            codes[j] = (signed char)k;
            const double xt = (double)s * (double)k, dv = (double)v - xt;
            se += dv * dv, sx += xt * xt;
        }
        for (int off = 32; off > 0; off >>= 1) se += __shfl_xor(se, off, 64), sx += __shfl_xor(sx, off, 64);
        if (lane == 0) {
            float* fig = reinterpret_cast<float*>(out + (size_t)row * stride + (size_t)padded);
            fig[0] = s, fig[1] = (float)sx;
            fig[2] = bad ? __int_as_float(0x7f800000) : (float)(sqrt(se) * 1.000001) * (1.0f + 2.0e-7f);
            fig[3] = 0.0f;
        }
    }
}

size_t byte_row_stride(int dim) { return ((size_t)((dim + 15) & ~15) + 16 + 127) & ~(size_t)127; }

hipError_t launch_byte_rows(const float* vec, int64_t n, int dim, unsigned char* out, hipStream_t stream) {
    hipLaunchKernelGGL(byte_rows_kernel, dim3(4096), dim3(256), 0, stream, vec, n, dim, out, byte_row_stride(dim));
    return hipGetLastError();
}

size_t half_row_stride(int dim) { return ((size_t)((dim + 7) & ~7) * 2 + 4 + 127) & ~(size_t)127; }

hipError_t launch_half_rows(const float* vec, int64_t n, int dim, unsigned char* out, hipStream_t stream) {
    hipLaunchKernelGGL(half_rows_kernel, dim3(4096), dim3(256), 0, stream, vec, n, dim, out, half_row_stride(dim));
    return hipGetLastError();
}

hipError_t launch_verify(const int32_t* res, const int32_t* gt, unsigned long long* hit, int Q, int k,
                         hipStream_t stream) {
    hipLaunchKernelGGL(ids_verify_kernel, dim3(Q < 1024 ? Q : 1024), dim3(64), 0, stream, res, gt, hit,
                       Q, k);
    return hipGetLastError();
}

hipError_t launch_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    size_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p, n, v);
    return hipGetLastError();
}

}  // namespace coral
