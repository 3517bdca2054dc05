// best_first.hip -- the best-first traversal (the reference's CPU search, src/search_in_cpu.cpp:63-108) with one
// WAVEFRONT per in-flight query.
//
// Best-first expands one beam entry at a time: read its graph row, test its neighbours against the visited set,
// measure the new ones, insert them, pick the closest entry not yet expanded.  Every step is a chain of dependent
// memory accesses; what makes it fast on this GPU is how many such chains run side by side.  A workgroup per query
// with the visited set in LDS (the form beam_search.hip gives this policy) holds two queries per CU.  Here a query
// needs one wavefront and 9.1 KB of LDS at L = 512 (its sorted beam, merged in place, and a filter over its visited
// ids): sixteen queries per CU, as many as 128 registers per lane allow, enough to keep HBM busy (2.8 times the
// throughput of the other form at a million nodes; more wavefronts add nothing).
//
// The visited set has two levels.  In global memory, the form the CPU path itself uses (src/search_in_cpu.cpp:44-48,
// 68-71): one byte per node and query slot holding the epoch of the query that last visited the node, so nothing
// is cleared between queries (every 255th query of a slot wipes its array).  With 288 GB of HBM four thousand such
// arrays are cheap (4 GB at a million nodes); each test costs a 128-byte line of HBM traffic and each mark a
// 32-byte write.  For indexes too large for a byte per node and slot the same state is packed into 32-bit words of
// 8 epoch bits over 24 node flags (template parameter PACKED).  A Bloom filter over the query's visited ids in LDS
// (4 KB at L = 512) answers most tests without that line: an id it does not know is new for certain.
// Those single-line requests cost the memory system more than their bytes say (a launch without them moves its
// vectors 1.4 times as fast on data whose neighbourhoods overlap), so where the beam leaves room -- L <= 409 -- the
// first level is an exact table of 16-bit cells in LDS, in buckets of four with two candidate buckets per id: a
// test is two 8-byte LDS reads whatever the load, and only ids that find both buckets full go to the state in HBM.
// 8192 cells (16 KB) per query leave a CU eight wavefronts, which this kernel needs anyway to saturate memory.
//
// The arithmetic is that of beam_search.hip (same lane-strided accumulation, same butterfly, same 64-bit keys), so
// results and counters are identical bit for bit; a wavefront needs no workgroup barrier anywhere.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "beam_search.h"
#include "search_device.h"

namespace coral {

namespace {

constexpr int kWavesPerWg = 4;
constexpr int kBatch = 32;  // ids measured and merged at a time (a graph row has at most 32)
constexpr int kScreenRows = 8;  // half-precision rows in flight per group of 32 lanes in the screening phase

__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// PACKED: the visited state of a slot is one 32-bit word per 24 nodes (8 bits of epoch, 24 flags) instead of one
// byte per node: a sixth of the memory, the same one line per test.
// SCREEN: rows are first measured in a smaller copy of the vectors: 1 the half-precision copy (b.vec16; rows of more
// than 128 floats), 2 the copy in eight-bit codes (b.vec8; rows of 68 .. 512 floats).
// WGS: workgroups a CU is to hold, which sets the registers a lane may use: what the rows in flight allow (two for a
// whole step's rows at once, four for 16, five for 8), or three where the beam leaves LDS for no more than three anyway
// (L beyond about 1000: +14 % at L = 1280 against squeezing into the registers of four).
template <int G, int CPL, int RIF, bool PACKED, int SCREEN, int WGS>
__global__ __launch_bounds__(kWavesPerWg * 64, WGS) void best_first_wave_kernel(const SearchArgs a, const BestFirstArgs b) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slot = blockIdx.x * kWavesPerWg + wave;
    if (slot >= b.slots) return;  // the whole wavefront; no workgroup barrier is used below
    const int L = a.L, R = a.R, dim = a.dim, chunks = dim >> 2, M = a.M;
    const int Lp = (L + 3) & ~3;
    unsigned char* mine_lds = smem + (size_t)wave * best_first_wave_lds_bytes(L, b.bloom_log2, b.table_log2, b.coded_bytes);
    uint64_t* beam = reinterpret_cast<uint64_t*>(mine_lds);      // L keys, sorted
    uint64_t* cand = beam + Lp;                                   // kBatch keys
    uint32_t* todo = reinterpret_cast<uint32_t*>(cand + kBatch);  // kBatch ids
    uint32_t* todo2 = todo + kBatch;                              // kBatch ids: what the screening leaves to measure
    uint32_t* table = todo2 + kBatch;                             // 2^table_log2 16-bit cells, or none (8-byte aligned)
    uint32_t* marks = table + (b.table_log2 ? (1 << b.table_log2) >> 1 : 0);  // Lp byte counters, zero between merges
    uint32_t* bloom = marks + (Lp >> 2);                          // 2^bloom_log2 bits, or none
    for (int i = lane; i < (Lp >> 2); i += 64) marks[i] = 0u;
    // The Bloom filter holds every id the query has visited.  An id it does not know is new for certain and needs no
    // look at the visited state in HBM (most tests: a query sees far more new ids than old ones); an id it may know
    // is looked up as before.  Two multiplicative hashes.
    const int bl = b.bloom_log2;
    const int bloom_words = bl ? (1 << bl) >> 5 : 0;
    signed char* qh8 = reinterpret_cast<signed char*>(bloom + bloom_words);  // the query in integer codes (SCREEN == 2)
    signed char* ql8 = qh8 + ((dim + 15) & ~15);
    auto bloom_bits = [&](uint32_t id, uint32_t& h1, uint32_t& h2) {
        h1 = (id * 0x9E3779B1u) >> (32 - bl);
        h2 = (id * 0x85EBCA77u + 0x3C6EF372u) >> (32 - bl);
    };
    auto bloom_may_hold = [&](uint32_t id) -> bool {
        uint32_t h1, h2;
        bloom_bits(id, h1, h2);
        return ((bloom[h1 >> 5] >> (h1 & 31)) & (bloom[h2 >> 5] >> (h2 & 31)) & 1u) != 0u;
    };
    auto bloom_add = [&](uint32_t id) {
        uint32_t h1, h2;
        bloom_bits(id, h1, h2);
        atomicOr(&bloom[h1 >> 5], 1u << (h1 & 31));
        atomicOr(&bloom[h2 >> 5], 1u << (h2 & 31));
    };

    // First level of the visited set, when the launch has one: an exact table of 16-bit cells in LDS, in buckets of
    // four.  A bijection mixes the id; the high bits of the result pick a bucket, a second bucket follows from that
    // one and the remaining bits (the remainder), and a cell stores the remainder and which of the two buckets it is
    // in: cell = 1 + ((second << rb) | remainder), 0 = empty.  (bucket, cell) determine the mixed value and hence the
    // id, so the table is exact.  A test reads the two buckets (two 8-byte reads, whatever the load); an id goes to
    // the emptier one.  0: the id was there; 1: it is now; 2: it is not and cannot be (both buckets are full): such
    // ids are settled against the state in HBM.
    // One call handles distinct ids in its lanes (the caller has removed repeats).
    const int tl = b.table_log2;
    const uint32_t t_bkmask = tl ? (1u << (tl - 2)) - 1u : 0u;
    const uint32_t t_bmask = b.id_bits >= 32 ? 0xffffffffu : (1u << b.id_bits) - 1u;
    const int t_rb = b.rem_bits, t_xs = b.id_bits > 1 ? b.id_bits / 2 : 1;
    const uint32_t t_rmask = (1u << t_rb) - 1u;
    auto table_test_and_set = [&](uint32_t id) -> int {
        uint32_t h = (id * 0x9E3779B1u) & t_bmask;
        h ^= h >> t_xs;
        h = (h * 0x85EBCA6Bu) & t_bmask;
        h ^= h >> t_xs;
        const uint32_t rem = h & t_rmask;
        const uint32_t b1 = (h >> t_rb) & t_bkmask;
        const uint32_t b2 = (b1 ^ (((rem + 1u) * 0x5BD1E995u) >> 15)) & t_bkmask;
        const uint32_t want1 = 1u + rem, want2 = 1u + ((1u << t_rb) | rem);
        const uint2* buckets = reinterpret_cast<const uint2*>(table);
        for (int attempt = 0; attempt < 8; ++attempt) {
            const uint2 w1 = buckets[b1], w2 = buckets[b2];
            const uint32_t c1[4] = {w1.x & 0xffffu, w1.x >> 16, w1.y & 0xffffu, w1.y >> 16};
            const uint32_t c2[4] = {w2.x & 0xffffu, w2.x >> 16, w2.y & 0xffffu, w2.y >> 16};
            int e1 = 0, e2 = 0, f1 = -1, f2 = -1;  // empty cells and the first of them, per bucket
            bool present = false;
#pragma unroll
            for (int i = 3; i >= 0; --i) {
                present |= c1[i] == want1 || c2[i] == want2;
                if (c1[i] == 0u) ++e1, f1 = i;
                if (c2[i] == 0u) ++e2, f2 = i;
            }
            if (present) return 0;
            if (e1 == 0 && e2 == 0) return 2;
            const bool second = e2 > e1;
            const uint32_t bk = second ? b2 : b1, want = second ? want2 : want1;
            const int cell = second ? f2 : f1;
            const uint32_t oldw = second ? (cell < 2 ? w2.x : w2.y) : (cell < 2 ? w1.x : w1.y);
            const int sh = (cell & 1) * 16;
            if (atomicCAS(table + bk * 2u + (uint32_t)(cell >> 1), oldw, oldw | (want << sh)) == oldw) return 1;
            // another lane took a cell of that word: look again
        }
        return 2;
    };

    uint8_t* vis = b.visited + (size_t)slot * b.stride;
    uint32_t epoch = b.epochs[slot];

    constexpr int GPW = 64 / G;                    // row groups per wavefront
    constexpr int U = (CPL >= RIF) ? 1 : (RIF / CPL);  // rows in flight per group
    constexpr int RPI = GPW * U;                   // rows per iteration
    const int gl = lane & (G - 1), grp = lane / G;

    for (;;) {
        int qid = 0;
        if (lane == 0) qid = atomicAdd(a.next_qid, 1);
        qid = __shfl(qid, 0, 64);
        if (qid >= a.Q) break;

        // a new epoch; the byte wraps after 255 queries of this slot, then the array starts over
        if (++epoch == 256u) {
            uint4* p = reinterpret_cast<uint4*>(vis);
            for (size_t i = lane; i < b.stride / 16; i += 64) p[i] = make_uint4(0u, 0u, 0u, 0u);
            __threadfence();
            epoch = 1u;
        }
        const uint8_t tag = (uint8_t)epoch;
        for (int i = lane; i < bloom_words; i += 64) bloom[i] = 0u;
        for (int i = lane; i < (tl ? (1 << tl) >> 1 : 0); i += 64) table[i] = 0u;
        bool any_over = tl == 0;  // has an id of this query gone to the state in HBM?
        uint32_t* visw = reinterpret_cast<uint32_t*>(vis);
        // first visit?  (every lane passes its own id; ids of one call are distinct, or told apart by the caller)
        auto unvisited = [&](uint32_t id) -> bool {
            if (!PACKED) return __hip_atomic_load(vis + id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != tag;
            const uint32_t w = __hip_atomic_load(visw + id / 24u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return (w >> 24) != epoch || ((w >> (id % 24u)) & 1u) == 0u;
        };
        // Mark a visit.  Packed: bring the word to this epoch (a maximum: words of older epochs lose their flags, a
        // word of this epoch keeps them), then set the flag; both without a return value, and any interleaving of the
        // two operations of several lanes on one word ends with all their flags set.
        auto mark = [&](uint32_t id) {
            if (!PACKED) {
                __hip_atomic_store(vis + id, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            } else {
                __hip_atomic_fetch_max(visw + id / 24u, epoch << 24, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_fetch_or(visw + id / 24u, 1u << (id % 24u), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        };

        float4 qreg[CPL];
        {
            const float4* q4 = reinterpret_cast<const float4*>(a.queries + (size_t)qid * dim);
#pragma unroll
            for (int t = 0; t < CPL; ++t) {
                const int c = gl + G * t;
                qreg[t] = c < chunks ? q4[c] : make_float4(0, 0, 0, 0);
            }
        }

        // The query in integer codes for the screening on eight-bit rows (search_device.h): bytes in LDS; |q~|^2, the
        // scale and |q - q~| in registers.
        float c_qq = 0.0f, c_sq = 0.0f, c_eq = 0.0f;
        if constexpr (SCREEN == 2) {
            code_query(a.queries + (size_t)qid * dim, dim, lane, qh8, ql8, c_qq, c_sq, c_eq);
            wave_sync();
        }

        int nb = 0, cursor = 0;
        uint64_t live = kKeyMax;
        int hops = M, nd = M, ne = 0, rounds = 0;
        int n_screened = 0, n_exact = 0, n_vreq = 0;  // rows measured on the smaller copy, fp32 rows, visited-state requests to HBM

        // todo[0..T) -> distances -> the beam
        auto measure_and_merge = [&](int T) {
            const uint32_t* list = todo;
            // Screening (see beam_search.hip): each row is first measured in the half-precision copy of the vectors;
            // a row whose exact distance is certainly beyond the beam's worst entry is dropped without reading its
            // fp32 row -- most of what a search measures once its beam is full.
            if (SCREEN == 1 && G == 64 && nb == L) {
                constexpr int UH = U > kScreenRows ? kScreenRows : U;
                constexpr int RPIH = 2 * UH;
                const int glh = lane & 31, grph = lane >> 5;
                const int chunksH = (dim + 7) >> 3;
                const float s_live = key_s(live);
                // the lane's share of the query: the eight dimensions of each 16-byte chunk of halves it reads
                // (fetched with the rows rather than kept in registers for the whole query)
                float4 qa[CPL][2];
                {
                    const float4* q4 = reinterpret_cast<const float4*>(a.queries + (size_t)qid * dim);
#pragma unroll
                    for (int t = 0; t < CPL; ++t) {
                        const int c = 2 * (glh + 32 * t);
                        qa[t][0] = c < chunks ? q4[c] : make_float4(0, 0, 0, 0);
                        qa[t][1] = c + 1 < chunks ? q4[c + 1] : make_float4(0, 0, 0, 0);
                    }
                }
                int n2 = 0;
                for (int base = 0; base < T; base += RPIH) {
                    int vid[UH];
                    const int r0 = base + grph * UH;
#pragma unroll
                    for (int u = 0; u < UH; ++u) vid[u] = r0 + u < T ? (int)todo[r0 + u] : -1;
                    uint4 h[UH][CPL];
#pragma unroll
                    for (int u = 0; u < UH; ++u) {
                        const uint4* row = reinterpret_cast<const uint4*>(
                            b.vec16 + (uint64_t)(uint32_t)(vid[u] < 0 ? 0 : vid[u]) * b.stride16);
#pragma unroll
                        for (int t = 0; t < CPL; ++t) {
                            const int c = glh + 32 * t;
                            h[u][t] = (vid[u] >= 0 && c < chunksH) ? row[c] : make_uint4(0u, 0u, 0u, 0u);
                        }
                    }
                    int myid = vid[0];
#pragma unroll
                    for (int u = 1; u < UH; ++u)
                        if ((lane & (UH - 1)) == u) myid = vid[u];
                    const bool valid = glh < UH && myid >= 0;
                    float nx = 0.0f;
                    if (valid)
                        nx = *reinterpret_cast<const float*>(b.vec16 + (uint64_t)(uint32_t)myid * b.stride16 +
                                                             (size_t)chunksH * 16);
                    float acc[UH];
#pragma unroll
                    for (int u = 0; u < UH; ++u) {
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
                    for (int u = 0; u < UH; ++u) {
                        acc[u] = acc[u] + dpp_mov<0xB1>(acc[u]);   // quad_perm [1,0,3,2]
                        acc[u] = acc[u] + dpp_mov<0x4E>(acc[u]);   // quad_perm [2,3,0,1]
                        acc[u] = acc[u] + dpp_mov<0x141>(acc[u]);  // row_half_mirror
                        acc[u] = acc[u] + dpp_mov<0x140>(acc[u]);  // row_mirror
                    }
                    float mine = acc[0];
#pragma unroll
                    for (int u = 1; u < UH; ++u)
                        if ((lane & (UH - 1)) == u) mine = acc[u];
                    mine = mine + __shfl_xor(mine, 16, 64);
                    // (2^-11 |x| for components that are normal in half precision, 2^-25 each for smaller ones)
                    const float root = sqrtf(mine), r = 5.0e-4f * nx + 1.0e-6f + 3.0e-8f * sqrtf((float)(chunksH * 8));
                    const float lo_root = fmaxf(root - r, 0.0f);
                    const float lo = lo_root * lo_root * (1.0f - 1.0e-4f);
                    const bool exact = valid && !(lo > s_live);
                    const uint64_t m = __ballot(exact);
                    if (exact) todo2[n2 + prefix_popc(m)] = (uint32_t)myid;
                    n2 += __popcll(m);
                }
                wave_sync();
                list = todo2;
                n_screened += T;
                T = n2;
            }
            if constexpr (SCREEN == 2 && G >= 32 && CPL <= 2) {
                if (nb == L) {
                    // the same on eight-bit codes: sixteen lanes per row, all 32 rows of a step in one round of requests
                    constexpr int CPL8 = CPL, U8 = 8 / CPL8, RPI8 = 4 * U8;
                    const int gl8 = lane & 15, grp8 = lane >> 4;
                    const int nck = (dim + 15) >> 4;
                    const float s_live = key_s(live);
                    CodedQuery<CPL8> cq;
                    load_coded_query<CPL8>(qh8, ql8, nck, gl8, cq);
                    int n2 = 0;
                    for (int base = 0; base < T; base += RPI8) {
                        int vid[U8];
                        const int r0 = base + grp8 * U8;
#pragma unroll
                        for (int u = 0; u < U8; ++u) vid[u] = r0 + u < T ? (int)todo[r0 + u] : -1;
                        const int mi = r0 + gl8;
                        const int myid = (gl8 < U8 && mi < T) ? (int)todo[mi] : -1;  // the row this lane files
                        const bool valid = myid >= 0;
                        float lo, hi;
                        coded_rows_bounds<CPL8, U8>(b.vec8, (uint32_t)b.stride8, nck, gl8, vid, myid, cq, c_qq, c_sq, c_eq, a.metric, lo, hi);
                        const bool exact = valid && !(lo > s_live);
                        const uint64_t m = __ballot(exact);
                        if (exact) todo2[n2 + prefix_popc(m)] = (uint32_t)myid;
                        n2 += __popcll(m);
                    }
                    wave_sync();
                    list = todo2;
                    n_screened += T;
                    T = n2;
                }
            }
            n_exact += T;
            int nc = 0;
            for (int base = 0; base < T; base += RPI) {
                int vid[U];
                const int r0 = base + grp * U;
#pragma unroll
                for (int u = 0; u < U; ++u) vid[u] = r0 + u < T ? (int)list[r0 + u] : -1;
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
                // butterfly p[l] += p[l ^ off], off = 1, 2, 4, ..., G/2 (the in-row levels on DPP)
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    acc[u] = acc[u] + dpp_mov<0xB1>(acc[u]);   // quad_perm [1,0,3,2]
                    acc[u] = acc[u] + dpp_mov<0x4E>(acc[u]);   // quad_perm [2,3,0,1]
                    acc[u] = acc[u] + dpp_mov<0x141>(acc[u]);  // row_half_mirror
                    acc[u] = acc[u] + dpp_mov<0x140>(acc[u]);  // row_mirror
                }
                // lane l of a group takes the sum of row l: the levels across the 16-lane rows add lanes 16 and 32
                // apart, which have chosen the same row as long as at most 16 rows are dealt out at a time
                constexpr int UH = U > 16 ? 16 : U;
#pragma unroll
                for (int h = 0; h < U; h += UH) {
                    float mine = acc[h];
                    int myid = vid[h];
#pragma unroll
                    for (int u = 1; u < UH; ++u)
                        if ((lane & (UH - 1)) == u) mine = acc[h + u], myid = vid[h + u];
                    if (G >= 32) mine = mine + __shfl_xor(mine, 16, 64);
                    if (G >= 64) mine = mine + __shfl_xor(mine, 32, 64);
                    const bool valid = gl < UH && myid >= 0;
                    const float s = a.metric == 0 ? mine : 0.0f - mine;
                    const uint64_t key = make_key(s, myid, 0u);
                    // the queue turns away what is not better than its worst entry once it is full
                    // (include/efanna2e/neighbor.h:162-166)
                    const bool app = valid && s < 3.402823466e+38f && key < live;
                    const uint64_t m = __ballot(app);
                    if (app) cand[nc + prefix_popc(m)] = key;
                    nc += __popcll(m);
                }
            }
            wave_sync();
            if (nc == 0) return;
            // In place: a candidate's place is its rank among the candidates plus the number of beam keys below it
            // (p); a beam key moves up by the number of candidates with p at or below its index.  Those counts come
            // from one byte counter per beam position and a prefix sum, chunk by chunk from the top, so that what a
            // chunk overwrites has been read already; nothing below the first insertion moves.
            uint64_t ck = 0;
            int p = 0x7fffffff, rank = 0;
            if (lane < nc) {
                ck = cand[lane];
                for (int c = 0; c < nc; ++c) rank += cand[c] < ck;
                p = lower_bound_u64(beam, nb, ck);
                if (p < nb) atomicAdd(&marks[p >> 2], 1u << ((p & 3) * 8));
            }
            const uint64_t mz = __ballot(lane < nc && rank == 0);  // the closest candidate: exactly one lane
            const int fp = __builtin_amdgcn_readlane(p, __ffsll((long long)mz) - 1);
            // entries before the cursor are all expanded: the closest new key may land before it
            if (fp < L && fp < cursor) cursor = fp;
            wave_sync();
            if (fp < nb) {
                for (int base = (nb - 1) & ~63; base >= (fp & ~63); base -= 64) {
                    const int i = base + lane;
                    const bool act = i < nb;
                    const uint64_t key = act ? beam[i] : 0ull;
                    const int m = act ? (int)((marks[i >> 2] >> ((i & 3) * 8)) & 0xffu) : 0;
                    const int carry = __popcll(__ballot(lane < nc && p < base));
                    const int shift = carry + wave_inclusive_sum(m);
                    wave_sync();  // every read of this chunk before its writes
                    if (act && shift > 0 && i + shift < L) beam[i + shift] = key;
                }
            }
            wave_sync();
            if (lane < nc) {
                if (p + rank < L) beam[p + rank] = ck;
                if (p < nb) marks[p >> 2] = 0u;
            }
            wave_sync();
            nb = nb + nc < L ? nb + nc : L;
            live = nb == L ? beam[L - 1] : kKeyMax;
        };

        // ---- seeds: every start id is visited and measured (src/search_in_cpu.cpp:74-79)
        for (int s0 = 0; s0 < M; s0 += kBatch) {
            const int T = M - s0 < kBatch ? M - s0 : kBatch;
            bool over = false;
            if (lane < T) {
                const uint32_t id = (uint32_t)a.start_ids[s0 + lane];
                over = tl == 0 || table_test_and_set(id) == 2;
                if (over) {
                    mark(id);
                    if (bl) bloom_add(id);
                }
                todo[lane] = id;
            }
            any_over = any_over || __ballot(over) != 0ull;
            n_vreq += __popcll(__ballot(over)) * (PACKED ? 2 : 1);
            wave_sync();
            measure_and_merge(T);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");

        // ---- one expansion per step
        for (;;) {
            int c = cursor, found = nb;
            while (c < nb) {
                const int i = c + lane;
                const bool un = i < nb && (beam[i] & 1ull) == 0;
                const uint64_t m = __ballot(un);
                if (m) {
                    found = c + (__ffsll((long long)m) - 1);
                    break;
                }
                c += 64;
            }
            if (found >= nb) break;
            const uint64_t ekey = beam[found];
            wave_sync();
            if (lane == 0) beam[found] = ekey | 1ull;
            cursor = found + 1;
            const uint32_t eid = (uint32_t)key_id(ekey);
            ++hops, ++ne, ++rounds;

            int v = -1;
            if (lane < R) v = a.nbrs[(size_t)eid * R + lane];
            if (!b.rows_unique) {
                // an id listed twice in the row counts once (the first listing)
                const int v0 = v;
                for (int k = 0; k < R; ++k) {
                    const int vk = __builtin_amdgcn_readlane(v0, k);
                    if (k < lane && vk == v0) v = -1;
                }
            }
            // the table first; what it has no room for is settled against the state in HBM, which holds nothing
            // before the first id went there, and whose filter knows every id that did
            bool isnew = false, over = false, tested = false;
            if (v >= 0) {
                if (tl) {
                    const int r = table_test_and_set((uint32_t)v);
                    isnew = r == 1, over = r == 2;
                } else {
                    over = true;
                }
                if (over) {
                    const bool settled = !any_over || (bl && !bloom_may_hold((uint32_t)v));
                    isnew = settled || unvisited((uint32_t)v);
                    tested = !settled;
                }
            }
            if (isnew && over) {
                mark((uint32_t)v);
                if (bl) bloom_add((uint32_t)v);
            }
            n_vreq += __popcll(__ballot(tested)) + __popcll(__ballot(isnew && over)) * (PACKED ? 2 : 1);
            const uint64_t m = __ballot(isnew);
            any_over = any_over || __ballot(isnew && over) != 0ull;
            const int T = __popcll(m);
            if (isnew) todo[prefix_popc(m)] = (uint32_t)v;
            nd += T;
            wave_sync();
            measure_and_merge(T);
            // The tags written in this step are read by later steps of this wavefront through other lanes.  Tag loads
            // and stores are agent-scope atomics, so both go to L2 past the CU's cache; the fence makes the wavefront
            // wait for its stores to be acknowledged before it issues the next step's loads.  (A fence of agent scope
            // would also write the whole L2 back each step, which no other wavefront needs: slots are private.)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        }

        // ---- output: the k closest live entries, closest first
        {
            int32_t* ids_out = a.ids_out + (size_t)qid * a.k;
            float* dists_out = a.dists_out ? a.dists_out + (size_t)qid * a.k : nullptr;
            int outpos = 0;
            for (int i0 = 0; i0 < nb && outpos < a.k; i0 += 64) {
                const int i = i0 + lane;
                uint64_t key = 0;
                bool livee = false;
                if (i < nb) {
                    key = beam[i];
                    livee = true;
                    if (a.deleted) {
                        const int32_t id = key_id(key);
                        livee = ((a.deleted[id >> 5] >> (id & 31)) & 1u) == 0;
                    }
                }
                const uint64_t m = __ballot(livee);
                const int pos = outpos + prefix_popc(m);
                if (livee && pos < a.k) {
                    ids_out[pos] = key_id(key);
                    if (dists_out) {
                        const float s = key_s(key);
                        dists_out[pos] = a.metric == 0 ? s : 0.0f - s;
                    }
                }
                outpos += __popcll(m);
            }
            for (int i = outpos + lane; i < a.k; i += 64) {
                ids_out[i] = -1;
                if (dists_out) {
                    const float far = __int_as_float(0x7f800000);  // src/search_in_cpu.cpp:33-35
                    dists_out[i] = a.metric == 0 ? far : -far;
                }
            }
            if (lane == 0) {
                int32_t* c = a.counters + (size_t)qid * 4;
                c[0] = hops, c[1] = ne, c[2] = nd, c[3] = rounds;
                {
                    int32_t* rc = a.counters + ((size_t)a.Q + qid) * 4;
                    rc[0] = n_screened, rc[1] = n_exact, rc[2] = 0, rc[3] = n_vreq;
                }
            }
        }
        wave_sync();
    }
    if (lane == 0) b.epochs[slot] = epoch;
}

// one thread per graph row: does it list an id twice?
__global__ __launch_bounds__(256) void find_repeated_ids_kernel(const int32_t* __restrict__ nbrs, int64_t n, int R,
                                                                uint32_t* flag) {
    const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= n) return;
    const int32_t* r = nbrs + row * R;
    bool rep = false;
    for (int i = 1; i < R; ++i) {
        const int32_t v = r[i];
        if (v < 0) break;  // rows end at their first -1
        for (int j = 0; j < i; ++j) rep |= r[j] == v;
    }
    if (rep) atomicOr(flag, 1u);
}

using bf_kernel_fn = void (*)(const SearchArgs, const BestFirstArgs);

// RIF float4 registers of row data per lane are requested before any is added up: 16 halves the number of
// dependent memory waits of a step against 8 and needs 128 registers; 32 (a whole step at once, 212 registers) is
// for launches whose LDS holds a CU to eight wavefronts anyway (+2..3 %)
template <int RIF, bool PACKED, int SCREEN, int WGS>
bf_kernel_fn pick_bf_kernel_rif(int chunks) {
    constexpr int WIDE = SCREEN == 2 ? 1 : SCREEN;  // rows of more than 512 floats have no copy in eight-bit codes
    if (chunks <= 16) return best_first_wave_kernel<16, 1, RIF, PACKED, 0, WGS>;
    if (chunks <= 32) return best_first_wave_kernel<32, 1, RIF, PACKED, (SCREEN == 2 ? 2 : 0), WGS>;  // (codes only)
    if (chunks <= 64) return best_first_wave_kernel<64, 1, RIF, PACKED, SCREEN, WGS>;
    if (chunks <= 128) return best_first_wave_kernel<64, 2, RIF, PACKED, SCREEN, WGS>;
    if (chunks <= 256) return best_first_wave_kernel<64, 4, RIF, PACKED, WIDE, WGS>;
    if (chunks <= 512) return best_first_wave_kernel<64, 8, RIF, PACKED, WIDE, WGS>;
    return nullptr;
}

template <int SCREEN>
bf_kernel_fn pick_bf_kernel_screen(int dim, int rif, bool packed, bool three) {
    // 32: for launches that hold eight wavefronts per CU or fewer (256 registers per lane); rows of 17..64 chunks
    if (rif >= 32 && dim / 4 > 16 && dim / 4 <= 64)
        return packed ? pick_bf_kernel_rif<32, true, SCREEN, 2>(dim / 4) : pick_bf_kernel_rif<32, false, SCREEN, 2>(dim / 4);
    if (three) {
        if (packed)
            return rif >= 16 ? pick_bf_kernel_rif<16, true, SCREEN, 3>(dim / 4) : pick_bf_kernel_rif<8, true, SCREEN, 3>(dim / 4);
        return rif >= 16 ? pick_bf_kernel_rif<16, false, SCREEN, 3>(dim / 4) : pick_bf_kernel_rif<8, false, SCREEN, 3>(dim / 4);
    }
    // with a screening few rows of a step are left to read in fp32: eight in flight are enough, and sixteen would
    // spill two dozen of the 128 registers that sixteen wavefronts per CU leave a lane (L = 512: 773 k -> 878 k QPS)
    if (SCREEN != 0 && rif < 16)
        return packed ? pick_bf_kernel_rif<8, true, SCREEN, 4>(dim / 4) : pick_bf_kernel_rif<8, false, SCREEN, 4>(dim / 4);
    if (packed)
        return rif >= 16 ? pick_bf_kernel_rif<16, true, SCREEN, 4>(dim / 4) : pick_bf_kernel_rif<8, true, SCREEN, 5>(dim / 4);
    return rif >= 16 ? pick_bf_kernel_rif<16, false, SCREEN, 4>(dim / 4) : pick_bf_kernel_rif<8, false, SCREEN, 5>(dim / 4);
}

// lds: bytes of one workgroup; a CU that has room for three workgroups at most runs the form compiled for three
bf_kernel_fn pick_bf_kernel(int dim, int rif, bool packed, int screen, size_t lds) {
    const bool three = lds * 4 > (size_t)160 * 1024;
    return screen == 2   ? pick_bf_kernel_screen<2>(dim, rif, packed, three)
           : screen == 1 ? pick_bf_kernel_screen<1>(dim, rif, packed, three)
                         : pick_bf_kernel_screen<0>(dim, rif, packed, three);
}

}  // namespace

hipError_t best_first_prepare(int dim, int L, int rows_in_flight, bool packed, int screen, int bloom_log2,
                              int table_log2, int* max_wg_per_cu) {
    if (screen == 2 && dim > kMaxByteRowDim) return hipErrorInvalidValue;
    const size_t lds = best_first_wave_lds_bytes(L, bloom_log2, table_log2, screen == 2 ? coded_query_bytes(dim) : 0) * kWavesPerWg;
    bf_kernel_fn fn = pick_bf_kernel(dim, rows_in_flight, packed, screen, lds);
    if (!fn) return hipErrorInvalidValue;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds);
    if (e != hipSuccess) return e;
    int nb = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, reinterpret_cast<const void*>(fn), kWavesPerWg * 64, lds);
    if (e != hipSuccess) return e;
    *max_wg_per_cu = nb;
    return hipSuccess;
}

hipError_t launch_best_first(const SearchArgs& a, const BestFirstArgs& b, hipStream_t stream) {
    const int screen = b.vec8 != nullptr ? 2 : b.vec16 != nullptr ? 1 : 0;
    if (screen == 2 && (a.dim > kMaxByteRowDim || b.coded_bytes != coded_query_bytes(a.dim))) return hipErrorInvalidValue;
    const size_t lds = best_first_wave_lds_bytes(a.L, b.bloom_log2, b.table_log2, b.coded_bytes) * kWavesPerWg;
    bf_kernel_fn fn = pick_bf_kernel(a.dim, b.rows_in_flight, b.packed != 0, screen, lds);
    if (!fn) return hipErrorInvalidValue;
    const int wgs = (b.slots + kWavesPerWg - 1) / kWavesPerWg;
    hipLaunchKernelGGL(fn, dim3(wgs), dim3(kWavesPerWg * 64), lds, stream, a, b);
    return hipGetLastError();
}

hipError_t launch_find_repeated_ids(const int32_t* nbrs, int64_t n, int R, uint32_t* flag, hipStream_t stream) {
    const int64_t blocks = (n + 255) / 256;
    if (blocks <= 0 || blocks > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(find_repeated_ids_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, nbrs, n, R, flag);
    return hipGetLastError();
}

}  // namespace coral
