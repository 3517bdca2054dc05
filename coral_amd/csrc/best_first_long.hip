// best_first_long.hip -- the best-first traversal (the reference's CPU search, src/search_in_cpu.cpp:63-108) for
// beams too long for a wavefront's share of LDS, still with one WAVEFRONT per in-flight query.
//
// The reference's queue is one sorted array: an insert shifts everything behind it (memmove of up to L entries,
// include/efanna2e/neighbor.h:162-195).  At the beam lengths isotropic data needs for recall 0.9 (L near 20 000,
// 20 000 sequential expansions per query) the traversal is a chain of dependent memory waits with little work per
// step, so throughput comes from the number of chains in flight: a wavefront per query, up to sixteen per CU.
// The queue is kept in two levels:
//   * `g`, the long sorted run, in global memory (two buffers per query slot; it lives in L2 / the memory-side
//     cache), touched only when the short level is merged into it;
//   * `buf`, a sorted insert buffer of `bcap` keys in LDS.  A step's new keys are merged into buf in place; when buf
//     could overflow it is merged into g in one coalesced pass (buf's places in g are found through an LDS sample of
//     every 2^ss-th key of g, so only the last steps of a search go to memory).
// The queue's content is the union of the two.  The closest entry not yet expanded is the closer of buf's first and
// g's first unflagged key (g's through a window of 64 keys held in registers).  A full queue drops its largest keys:
// they sit at the end of g or of buf, so dropping is a decrement of one of two counters, decided against an LDS copy
// of g's last keys; the key a newcomer has to beat is the larger of the two last keys.
// The visited set is the CPU path's own: a byte (or a packed flag) per node and query slot in global memory, tagged
// with the slot's query epoch (see best_first.hip).
//
// The arithmetic is that of beam_search.hip (same lane-strided accumulation, same butterfly, same 64-bit keys):
// results and counters are identical bit for bit to the other forms of this policy and to the test oracle.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "beam_search.h"
#include "search_device.h"

namespace coral {

namespace {

constexpr int kWavesPerWg = 4;
constexpr int kBatch = 32;  // ids measured and merged at a time (a graph row has at most 32)

__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The long run is written by some lanes and read by others of the same wavefront: both go past the CU's cache
// (agent-scope atomics), ordered by the fences of the steps that separate them.
__device__ __forceinline__ uint64_t gload(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void gstore(uint64_t* p, uint64_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void memory_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // waits for the wavefront's stores to be acknowledged
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// SCREEN: once the queue is full, rows are first measured in the copy in eight-bit codes (b.vec8; rows of 68 .. 512
// floats) and only those that may enter the queue are read in fp32 (search_device.h).
// WGS: workgroups a CU is to hold.  The insert buffer decides how many fit its LDS (three at 512 keys); the registers
// a lane may use follow from that number, and a launch that LDS holds to three workgroups per CU need not squeeze into
// the 128 registers that four would leave.
template <int G, int CPL, int RIF, bool PACKED, bool SCREEN, int WGS>
__global__ __launch_bounds__(kWavesPerWg * 64, WGS) void best_first_long_kernel(const SearchArgs a,
                                                                                   const BestFirstLongArgs b) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slot = blockIdx.x * kWavesPerWg + wave;
    if (slot >= b.slots) return;  // the whole wavefront; no workgroup barrier is used below
    const int L = a.L, R = a.R, dim = a.dim, chunks = dim >> 2, M = a.M;
    const int Lp = (L + 3) & ~3;
    const int bcap = b.bcap, tcap = b.bcap + kBatch, scap = b.scap, ss = b.sshift;
    unsigned char* mine_lds = smem + (size_t)wave * best_first_long_lds_bytes(bcap, scap, b.coded_bytes);
    uint64_t* buf = reinterpret_cast<uint64_t*>(mine_lds);  // bcap keys, sorted: the insert buffer
    uint64_t* tail = buf + bcap;                             // tcap keys: the last keys of g as of the last merge
    uint64_t* samp0 = tail + tcap;                           // scap keys: every 2^ss-th key of g (two copies: the
    uint64_t* samp1 = samp0 + scap;                          //   merge reads one while it writes the other)
    uint64_t* cand = samp1 + scap;                           // kBatch keys
    uint32_t* todo = reinterpret_cast<uint32_t*>(cand + kBatch);  // kBatch ids
    uint32_t* marks = todo + kBatch;                         // bcap byte counters, zero between merges
    uint32_t* todo2 = marks + (bcap >> 2);                   // (SCREEN) kBatch ids: what the screening leaves to measure
    signed char* qh8 = reinterpret_cast<signed char*>(todo2 + kBatch);  // (SCREEN) the query in integer codes
    signed char* ql8 = qh8 + ((dim + 15) & ~15);
    for (int i = lane; i < (bcap >> 2); i += 64) marks[i] = 0u;

    uint64_t* gbuf0 = b.beams + (size_t)slot * b.beam_stride;
    uint64_t* gbuf1 = gbuf0 + Lp;
    uint8_t* vis = b.visited + (size_t)slot * b.stride;
    uint32_t epoch = b.epochs[slot];

    constexpr int GPW = 64 / G;                        // row groups per wavefront
    constexpr int U = (CPL >= RIF) ? 1 : (RIF / CPL);  // rows in flight per group
    constexpr int RPI = GPW * U;                       // rows per iteration
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
        uint32_t* visw = reinterpret_cast<uint32_t*>(vis);
        auto unvisited = [&](uint32_t id) -> bool {
            if (!PACKED) return __hip_atomic_load(vis + id, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != tag;
            const uint32_t w = __hip_atomic_load(visw + id / 24u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return (w >> 24) != epoch || ((w >> (id % 24u)) & 1u) == 0u;
        };
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

        float c_qq = 0.0f, c_sq = 0.0f, c_eq = 0.0f;
        if constexpr (SCREEN) {
            code_query(a.queries + (size_t)qid * dim, dim, lane, qh8, ql8, c_qq, c_sq, c_eq);
            wave_sync();
        }

        // ---- the queue: g[0..ng) in global memory, buf[0..nbuf) in LDS, ng + nbuf <= L
        uint64_t* g = gbuf0;
        uint64_t* galt = gbuf1;
        uint64_t* samp = samp0;
        uint64_t* salt = samp1;
        int ng = 0, nbuf = 0, bcur = 0;
        int tbase = 0;            // tail[i - tbase] = g[i] for the last keys of g as of the last merge
        int wbase = 0;            // the window: wkey = g[wbase + lane]; every key of g before wbase is expanded
        uint64_t wkey = kKeyMax;  // (kKeyMax has its flag set: nothing to expand)
        uint64_t live = kKeyMax;
        int hops = M, nd = M, ne = 0, rounds = 0;
        // rows measured on the smaller copy, fp32 rows, words of the long run moved, visited-state requests to HBM
        int n_screened = 0, n_exact = 0, n_words = 0, n_vreq = 0;

        // ---- buf into g: one coalesced pass over g, buf's places found through the sample
        auto flush = [&]() {
            if (nbuf == 0) return;
            memory_sync();  // the flags stored into g since the last merge
            const int nn = ng + nbuf;  // <= L
            n_words += 2 * (ng + nn);  // one pass: ng keys read, nn written
            const int ntb = nn > tcap ? nn - tcap : 0;
            const int ns = ng > 0 ? ((ng - 1) >> ss) + 1 : 0;
            const uint64_t b_lo = buf[0], b_hi = buf[nbuf - 1];
            int minun = nn;  // lowest new position of a key not yet expanded
            auto place = [&](int pos, uint64_t key) {
                gstore(galt + pos, key);
                if (pos >= ntb) tail[pos - ntb] = key;
                if ((pos & ((1 << ss) - 1)) == 0) salt[pos >> ss] = key;
                if ((key & 1ull) == 0 && pos < minun) minun = pos;
            };
            for (int i0 = 0; i0 < ng; i0 += 4 * 64) {
                uint64_t key[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int i = i0 + u * 64 + lane;
                    key[u] = i < ng ? gload(g + i) : kKeyMax;
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int i = i0 + u * 64 + lane;
                    if (i < ng) {
                        const int below = key[u] < b_lo ? 0 : key[u] > b_hi ? nbuf : lower_bound_u64(buf, nbuf, key[u]);
                        place(i + below, key[u]);
                    }
                }
            }
            for (int j = lane; j < nbuf; j += 64) {
                const uint64_t key = buf[j];
                const int js = lower_bound_u64(samp, ns, key);
                int lo = js == 0 ? 0 : ((js - 1) << ss) + 1, hi = js == ns ? ng : (js << ss);
                while (lo < hi) {
                    const int mid = (lo + hi) >> 1;
                    if (gload(g + mid) < key)
                        lo = mid + 1;
                    else
                        hi = mid;
                }
                place(j + lo, key);
            }
            // the lowest unexpanded position over the wavefront
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) minun = min(minun, __shfl_xor(minun, off, 64));
            memory_sync();
            uint64_t* t = g;
            g = galt, galt = t;
            t = samp, samp = salt, salt = t;
            ng = nn, nbuf = 0, bcur = 0, tbase = ntb;
            wbase = minun;
            wkey = wbase + lane < ng ? gload(g + wbase + lane) : kKeyMax;
        };

        // the i-th key of g from the copy of its end in LDS (i >= tbase by construction)
        auto gtail = [&](int i) -> uint64_t { return tail[i - tbase]; };

        // todo[0..T) -> distances -> the queue
        auto measure_and_merge = [&](int T) {
            const uint32_t* list = todo;
            if constexpr (SCREEN && G >= 32 && CPL <= 2) {
                if (live != kKeyMax) {
                    // a row whose exact distance is certainly beyond the queue's worst entry is dropped on its codes
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
            // ---- the new keys into buf, in place (the merge of best_first.hip; buf has room for them)
            uint64_t ck = 0;
            int p = 0x7fffffff, rank = 0;
            if (lane < nc) {
                ck = cand[lane];
                for (int c = 0; c < nc; ++c) rank += cand[c] < ck;
                p = lower_bound_u64(buf, nbuf, ck);
                if (p < nbuf) atomicAdd(&marks[p >> 2], 1u << ((p & 3) * 8));
            }
            const uint64_t mz = __ballot(lane < nc && rank == 0);  // the closest candidate: exactly one lane
            const int fp = __builtin_amdgcn_readlane(p, __ffsll((long long)mz) - 1);
            if (fp < bcur) bcur = fp;  // keys of buf before bcur are all expanded: the closest new key may land before it
            wave_sync();
            if (fp < nbuf) {
                for (int base = (nbuf - 1) & ~63; base >= (fp & ~63); base -= 64) {
                    const int i = base + lane;
                    const bool act = i < nbuf;
                    const uint64_t key = act ? buf[i] : 0ull;
                    const int m = act ? (int)((marks[i >> 2] >> ((i & 3) * 8)) & 0xffu) : 0;
                    const int carry = __popcll(__ballot(lane < nc && p < base));
                    const int shift = carry + wave_inclusive_sum(m);
                    wave_sync();  // every read of this chunk before its writes
                    if (act && shift > 0) buf[i + shift] = key;
                }
            }
            wave_sync();
            if (lane < nc) {
                buf[p + rank] = ck;
                if (p < nbuf) marks[p >> 2] = 0u;
            }
            wave_sync();
            nbuf += nc;
            // ---- a queue over its capacity drops its largest keys: the last of g or the last of buf, e of them
            const int e = ng + nbuf - L;
            if (e > 0) {
                // lane j holds the j-th key from the end of g; it goes if fewer than e keys of the two ends are
                // larger: the j keys of g behind it and those of buf's last e that exceed it
                const bool have = lane < e && lane < ng;
                const uint64_t tg = have ? gtail(ng - 1 - lane) : 0ull;
                int larger = lane;
                for (int i = 0; i < e && i < nbuf; ++i) larger += buf[nbuf - 1 - i] > tg;
                const int dg = __popcll(__ballot(have && larger < e));
                ng -= dg;
                nbuf -= e - dg;
                if (bcur > nbuf) bcur = nbuf;
            }
            if (ng + nbuf == L) {
                const uint64_t lg = ng > 0 ? gtail(ng - 1) : 0ull, lb = nbuf > 0 ? buf[nbuf - 1] : 0ull;
                live = lg > lb ? lg : lb;
            } else {
                live = kKeyMax;
            }
        };

        // ---- seeds: every start id is visited and measured (src/search_in_cpu.cpp:74-79)
        for (int s0 = 0; s0 < M; s0 += kBatch) {
            const int T = M - s0 < kBatch ? M - s0 : kBatch;
            if (nbuf + kBatch > bcap) flush();
            if (lane < T) {
                const uint32_t id = (uint32_t)a.start_ids[s0 + lane];
                mark(id);
                todo[lane] = id;
            }
            n_vreq += T * (PACKED ? 2 : 1);
            wave_sync();
            measure_and_merge(T);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");

        // ---- one expansion per step
        for (;;) {
            if (nbuf + kBatch > bcap) flush();
            // the closest unexpanded key of buf ...
            int bi = nbuf;
            for (int c = bcur; c < nbuf; c += 64) {
                const int i = c + lane;
                const bool un = i < nbuf && (buf[i] & 1ull) == 0;
                const uint64_t m = __ballot(un);
                if (m) {
                    bi = c + (__ffsll((long long)m) - 1);
                    break;
                }
            }
            bcur = bi;
            // ... and of g, through the window
            int gi = ng;
            for (;;) {
                const bool un = wbase + lane < ng && (wkey & 1ull) == 0;
                const uint64_t m = __ballot(un);
                if (m) {
                    gi = wbase + (__ffsll((long long)m) - 1);
                    break;
                }
                if (wbase + 64 >= ng) break;
                wbase += 64;
                wkey = wbase + lane < ng ? gload(g + wbase + lane) : kKeyMax;
            }
            if (bi >= nbuf && gi >= ng) break;
            const uint64_t bkey = bi < nbuf ? buf[bi] : kKeyMax;
            const uint64_t gkey = gi < ng ? (uint64_t)__shfl((unsigned long long)wkey, gi - wbase, 64) : kKeyMax;
            uint64_t ekey;
            wave_sync();
            if (bkey < gkey) {
                ekey = bkey;
                if (lane == 0) buf[bi] = bkey | 1ull;
                bcur = bi + 1;
            } else {
                ekey = gkey;
                if (lane == gi - wbase) {
                    wkey |= 1ull;
                    gstore(g + gi, gkey | 1ull);
                }
            }
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
            const bool isnew = v >= 0 && unvisited((uint32_t)v);
            if (isnew) mark((uint32_t)v);
            const uint64_t m = __ballot(isnew);
            const int T = __popcll(m);
            if (isnew) todo[prefix_popc(m)] = (uint32_t)v;
            nd += T;
            n_vreq += __popcll(__ballot(v >= 0)) + T * (PACKED ? 2 : 1);  // a test per listed id, a mark per first visit
            wave_sync();
            measure_and_merge(T);
            // the tags written in this step are read by later steps through other lanes (see best_first.hip)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        }

        // ---- output: the k closest live entries, closest first
        flush();
        {
            int32_t* ids_out = a.ids_out + (size_t)qid * a.k;
            float* dists_out = a.dists_out ? a.dists_out + (size_t)qid * a.k : nullptr;
            int outpos = 0;
            for (int i0 = 0; i0 < ng && outpos < a.k; i0 += 64) {
                const int i = i0 + lane;
                uint64_t key = 0;
                bool livee = false;
                if (i < ng) {
                    key = gload(g + i);
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
                    rc[0] = n_screened, rc[1] = n_exact, rc[2] = n_words, rc[3] = n_vreq;
                }
            }
        }
        wave_sync();
    }
    if (lane == 0) b.epochs[slot] = epoch;
}

using bfl_kernel_fn = void (*)(const SearchArgs, const BestFirstLongArgs);

template <int RIF, bool PACKED, bool SCREEN, int WGS>
bfl_kernel_fn pick_rif(int chunks) {
    if (chunks <= 16) return best_first_long_kernel<16, 1, RIF, PACKED, false, WGS>;
    if (chunks <= 32) return best_first_long_kernel<32, 1, RIF, PACKED, SCREEN, WGS>;
    if (chunks <= 64) return best_first_long_kernel<64, 1, RIF, PACKED, SCREEN, WGS>;
    if (chunks <= 128) return best_first_long_kernel<64, 2, RIF, PACKED, SCREEN, WGS>;
    if (chunks <= 256) return best_first_long_kernel<64, 4, RIF, PACKED, false, WGS>;
    if (chunks <= 512) return best_first_long_kernel<64, 8, RIF, PACKED, false, WGS>;
    return nullptr;
}

template <bool SCREEN, int WGS>
bfl_kernel_fn pick_screen(int dim, bool packed) {
    const int chunks = dim / 4;
    // 16 rows requested per wavefront before any is added up where that fits the registers, else 8; with the
    // screening few rows of a step are left to read in fp32, and the registers are worth more to its own requests
    const bool wide = chunks > 16 && chunks <= 256 && !SCREEN;
    if (packed) return wide ? pick_rif<16, true, SCREEN, WGS>(chunks) : pick_rif<8, true, SCREEN, WGS>(chunks);
    return wide ? pick_rif<16, false, SCREEN, WGS>(chunks) : pick_rif<8, false, SCREEN, WGS>(chunks);
}

// workgroups per CU that LDS leaves room for, in the steps the kernel is compiled for: 2, 3 or 4 and more
int wgs_class(size_t lds_per_wg) {
    const size_t fit = (size_t)160 * 1024 / lds_per_wg;
    return fit >= 4 ? 4 : fit >= 3 ? 3 : 2;
}

bfl_kernel_fn pick(int dim, bool packed, bool screen, int wgs) {
    if (wgs >= 4) return screen ? pick_screen<true, 4>(dim, packed) : pick_screen<false, 4>(dim, packed);
    if (wgs == 3) return screen ? pick_screen<true, 3>(dim, packed) : pick_screen<false, 3>(dim, packed);
    return screen ? pick_screen<true, 2>(dim, packed) : pick_screen<false, 2>(dim, packed);
}

}  // namespace

hipError_t best_first_long_prepare(int dim, bool packed, bool screen, int bcap, int scap, int* max_wg_per_cu) {
    if (screen && (dim > kMaxByteRowDim || dim / 4 <= 16)) return hipErrorInvalidValue;
    const size_t lds = best_first_long_lds_bytes(bcap, scap, screen ? best_first_long_coded_bytes(dim) : 0) * kWavesPerWg;
    bfl_kernel_fn fn = pick(dim, packed, screen, wgs_class(lds));
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

hipError_t launch_best_first_long(const SearchArgs& a, const BestFirstLongArgs& b, hipStream_t stream) {
    const bool screen = b.vec8 != nullptr;
    if (screen && (a.dim > kMaxByteRowDim || a.dim / 4 <= 16 || b.coded_bytes != best_first_long_coded_bytes(a.dim)))
        return hipErrorInvalidValue;
    const size_t lds = best_first_long_lds_bytes(b.bcap, b.scap, b.coded_bytes) * kWavesPerWg;
    bfl_kernel_fn fn = pick(a.dim, b.packed != 0, screen, wgs_class(lds));
    if (!fn) return hipErrorInvalidValue;
    const int wgs = (b.slots + kWavesPerWg - 1) / kWavesPerWg;
    hipLaunchKernelGGL(fn, dim3(wgs), dim3(kWavesPerWg * 64), lds, stream, a, b);
    return hipGetLastError();
}

}  // namespace coral
