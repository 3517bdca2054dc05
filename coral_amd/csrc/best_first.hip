// best_first.hip -- the best-first traversal (the reference's CPU search, src/search_in_cpu.cpp:63-108) with one
// WAVEFRONT per in-flight query.
//
// Best-first expands one beam entry at a time: read its graph row, test its neighbours against the visited set,
// measure the new ones, insert them, pick the closest entry not yet expanded.  Every step is a chain of dependent
// memory accesses; what makes it fast on this GPU is how many such chains run side by side.  A workgroup per query
// with the visited set in LDS (the form beam_search.hip gives this policy) holds two queries per CU.  Here a query
// needs one wavefront and 9 KB of LDS at L = 512 (its sorted beam, twice, for the merge): sixteen queries per CU,
// enough to keep HBM busy (2.4 times the throughput of the other form at a million nodes).  The visited set moves to
// global memory in the form the CPU path itself uses (src/search_in_cpu.cpp:44-48, 68-71): one byte per node and
// query slot holding the epoch of the query that last visited the node, so nothing is cleared between queries
// (every 255th query of a slot wipes its array).  With 288 GB of HBM four thousand such arrays are cheap (4 GB at a
// million nodes); each test costs a 128-byte line of HBM traffic, about a sixth of what the vectors cost.
//
// The arithmetic is that of beam_search.hip (same lane-strided accumulation, same butterfly, same 64-bit keys), so
// results and counters are identical bit for bit; a wavefront needs no workgroup barrier anywhere.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "beam_search.h"
#include "search_device.h"

namespace coral {

namespace {

constexpr int kWavesPerWg = 4;
constexpr int kBatch = 64;  // ids measured and merged at a time (a graph row has at most 32)

__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int G, int CPL, int RIF>
__global__ __launch_bounds__(kWavesPerWg * 64, 4) void best_first_wave_kernel(const SearchArgs a, const BestFirstArgs b) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slot = blockIdx.x * kWavesPerWg + wave;
    if (slot >= b.slots) return;  // the whole wavefront; no workgroup barrier is used below
    const int L = a.L, R = a.R, dim = a.dim, chunks = dim >> 2, M = a.M;
    const int Lp = (L + 3) & ~3;
    unsigned char* mine_lds = smem + (size_t)wave * best_first_wave_lds_bytes(L);
    uint64_t* beam0 = reinterpret_cast<uint64_t*>(mine_lds);
    uint64_t* beam1 = beam0 + Lp;
    uint64_t* cand = beam1 + Lp;                                 // kBatch keys
    uint32_t* todo = reinterpret_cast<uint32_t*>(cand + kBatch);  // kBatch ids

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

        float4 qreg[CPL];
        {
            const float4* q4 = reinterpret_cast<const float4*>(a.queries + (size_t)qid * dim);
#pragma unroll
            for (int t = 0; t < CPL; ++t) {
                const int c = gl + G * t;
                qreg[t] = c < chunks ? q4[c] : make_float4(0, 0, 0, 0);
            }
        }

        int nb = 0, cur = 0, cursor = 0;
        uint64_t live = kKeyMax;
        int hops = M, nd = M, ne = 0, rounds = 0;

        // todo[0..T) -> distances -> the beam
        auto measure_and_merge = [&](int T) {
            int nc = 0;
            for (int base = 0; base < T; base += RPI) {
                int vid[U];
                const int r0 = base + grp * U;
#pragma unroll
                for (int u = 0; u < U; ++u) vid[u] = r0 + u < T ? (int)todo[r0 + u] : -1;
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
                float mine = acc[0];
                int myid = vid[0];
#pragma unroll
                for (int u = 1; u < U; ++u)
                    if ((lane & (U - 1)) == u) mine = acc[u], myid = vid[u];
                if (G >= 32) mine = mine + __shfl_xor(mine, 16, 64);
                if (G >= 64) mine = mine + __shfl_xor(mine, 32, 64);
                const bool valid = gl < U && myid >= 0;
                const float s = a.metric == 0 ? mine : 0.0f - mine;
                const uint64_t key = make_key(s, myid, 0u);
                // the queue turns away what is not better than its worst entry once it is full
                // (include/efanna2e/neighbor.h:162-166)
                const bool app = valid && s < 3.402823466e+38f && key < live;
                const uint64_t m = __ballot(app);
                if (app) cand[nc + prefix_popc(m)] = key;
                nc += __popcll(m);
            }
            wave_sync();
            if (nc == 0) return;
            // few keys: a key's place is its own index plus the number of smaller keys in the other list
            const uint64_t* src = cur ? beam1 : beam0;
            uint64_t* dst = cur ? beam0 : beam1;
            for (int i = lane; i < nb; i += 64) {
                const uint64_t key = src[i];
                int below = 0;
                for (int c = 0; c < nc; ++c) below += cand[c] < key;
                if (i + below < L) dst[i + below] = key;
            }
            int first_pos = L;
            if (lane < nc) {
                const uint64_t key = cand[lane];
                int below = 0;
                for (int c = 0; c < nc; ++c) below += cand[c] < key;
                const int pos = below + lower_bound_u64(src, nb, key);
                if (pos < L) dst[pos] = key;
                if (below == 0) first_pos = pos;
            }
            // entries before the cursor are all expanded: the closest new key may land before it
            const uint64_t mf = __ballot(first_pos < L);
            if (mf) {
                const int fp = __shfl(first_pos, __ffsll((long long)mf) - 1, 64);
                cursor = fp < cursor ? fp : cursor;
            }
            wave_sync();
            nb = nb + nc < L ? nb + nc : L;
            cur ^= 1;
            live = nb == L ? dst[L - 1] : kKeyMax;
        };

        // ---- seeds: every start id is visited and measured (src/search_in_cpu.cpp:74-79)
        for (int s0 = 0; s0 < M; s0 += kBatch) {
            const int T = M - s0 < kBatch ? M - s0 : kBatch;
            if (lane < T) {
                const uint32_t id = (uint32_t)a.start_ids[s0 + lane];
                __hip_atomic_store(vis + id, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                todo[lane] = id;
            }
            wave_sync();
            measure_and_merge(T);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");

        // ---- one expansion per step
        for (;;) {
            uint64_t* beam = cur ? beam1 : beam0;
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
            bool isnew = false;
            if (v >= 0) isnew = __hip_atomic_load(vis + v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != tag;
            if (__ballot(isnew)) {
                // an id listed twice in the row counts once (the first listing)
                for (int k = 0; k < R; ++k) {
                    const int vk = __builtin_amdgcn_readlane(v, k);
                    if (k < lane && vk == v) isnew = false;
                }
                if (isnew) __hip_atomic_store(vis + v, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            const uint64_t m = __ballot(isnew);
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
            const uint64_t* beam = cur ? beam1 : beam0;
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
            }
        }
        wave_sync();
    }
    if (lane == 0) b.epochs[slot] = epoch;
}

using bf_kernel_fn = void (*)(const SearchArgs, const BestFirstArgs);

// RIF float4 registers of row data per lane are requested before any is added up: 16 halves the number of
// dependent memory waits of a step against 8 and needs 128 registers
template <int RIF>
bf_kernel_fn pick_bf_kernel_rif(int chunks) {
    if (chunks <= 16) return best_first_wave_kernel<16, 1, RIF>;
    if (chunks <= 32) return best_first_wave_kernel<32, 1, RIF>;
    if (chunks <= 64) return best_first_wave_kernel<64, 1, RIF>;
    if (chunks <= 128) return best_first_wave_kernel<64, 2, RIF>;
    if (chunks <= 256) return best_first_wave_kernel<64, 4, RIF>;
    if (chunks <= 512) return best_first_wave_kernel<64, 8, RIF>;
    return nullptr;
}

bf_kernel_fn pick_bf_kernel(int dim, int rif) {
    return rif >= 16 ? pick_bf_kernel_rif<16>(dim / 4) : pick_bf_kernel_rif<8>(dim / 4);
}

}  // namespace

hipError_t best_first_prepare(int dim, int L, int rows_in_flight, int* max_wg_per_cu) {
    bf_kernel_fn fn = pick_bf_kernel(dim, rows_in_flight);
    if (!fn) return hipErrorInvalidValue;
    const size_t lds = best_first_wave_lds_bytes(L) * kWavesPerWg;
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
    bf_kernel_fn fn = pick_bf_kernel(a.dim, b.rows_in_flight);
    if (!fn) return hipErrorInvalidValue;
    const int wgs = (b.slots + kWavesPerWg - 1) / kWavesPerWg;
    hipLaunchKernelGGL(fn, dim3(wgs), dim3(kWavesPerWg * 64), best_first_wave_lds_bytes(a.L) * kWavesPerWg, stream, a, b);
    return hipGetLastError();
}

}  // namespace coral
