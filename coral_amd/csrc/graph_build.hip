// graph_build.hip -- the query-aware graph construction on the device.
//
// The reference builds its graph batch by batch (GPUFuncs::gpu_neibor_aware, src/upd_gpu.cu:260-303): the k_b
// nearest base points of an auxiliary query form a cluster, every member is a pivot whose candidates are the
// other members plus its current row, sorted by distance, thinned by an occlusion rule and written back.  Nodes
// that no cluster ever touched are attached afterwards through a beam search for their own vector
// (GPUFuncs::enhance_neibor_aware_gpu, src/enhance.cu:660-689).  There one thread walks a pivot's whole
// candidate list and evaluates every distance by itself; the sort is a device-wide segmented sort over
// 48-byte records in global memory.
//
// Here one workgroup owns one cluster: the member-pair distances are computed once into LDS (every pivot of the
// cluster reuses them), and one wavefront per pivot keeps its candidate list in LDS from assembly to the final
// row: rank-by-counting sort, occlusion loop with the later candidates spread over the lanes, ballot-prefix
// emission.  Only distances to a pivot's current neighbours are evaluated on the fly.  Every distance is the
// sequential fp32 chain of include/utils.cuh:254-275 / :307-323, so rows are bit-identical to a CPU statement
// of the same rules.
//
// Two outcomes that the reference leaves to thread timing are fixed: ties of the sort keep column order (its
// cub::DeviceSegmentedSort::SortPairs is not stable), and a base id that several clusters of one batch contain
// takes its row from the lowest pivot index (its atomicTestAndSetBit race, src/upd_gpu.cu:101; the same for the
// reverse edges of src/enhance.cu:161).  Rows are written by a separate kernel after all pivots have read.
#include <hip/hip_runtime.h>
#include <limits.h>
#include <stdint.h>

#include "coral_search.h"
#include "graph_build.h"

namespace coral {

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kChunk = 32;                         // dimensions staged per step of the member-pair distances
constexpr int kMaxCand = kBuildMaxKb + kBuildMaxR;  // candidates of one pivot

enum : uint8_t { ST_INITIAL = 0, ST_RETAINED = 1, ST_DISCARDED = 2, ST_REPEATED = 3 };  // include/uni.h:140-147

__device__ __forceinline__ uint32_t ord32(float s) {
    const uint32_t u = __float_as_uint(s);
    return u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
}
// include/utils.cuh:380-382: "d1 is closer than d0"
__device__ __forceinline__ bool closer(float d0, float d1, int metric) { return metric == CORAL_L2 ? d0 > d1 : d0 < d1; }

__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// one lane walks both rows: the accumulation order of include/utils.cuh:254-275 (L2) and :307-323 (IP).  The rows
// are fetched eight float4 at a time ahead of the additions, so a lane waits for memory once per 32 dimensions
// instead of once per 4; the chain of additions itself stays strictly in dimension order.
__device__ __forceinline__ float seq_dist(const float* __restrict__ a, const float* __restrict__ b, int dim, int metric) {
    constexpr int kAhead = 8;
    const float4* a4 = reinterpret_cast<const float4*>(a);
    const float4* b4 = reinterpret_cast<const float4*>(b);
    const int n4 = dim / 4;
    float acc = 0.0f;
    for (int i0 = 0; i0 < n4; i0 += kAhead) {
        float4 x[kAhead], y[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int i = i0 + u < n4 ? i0 + u : n4 - 1;
            x[u] = a4[i];
            y[u] = b4[i];
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            if (i0 + u < n4) {
                if (metric == CORAL_L2) {
                    float t = x[u].x - y[u].x;
                    acc = fmaf(t, t, acc);
                    t = x[u].y - y[u].y;
                    acc = fmaf(t, t, acc);
                    t = x[u].z - y[u].z;
                    acc = fmaf(t, t, acc);
                    t = x[u].w - y[u].w;
                    acc = fmaf(t, t, acc);
                } else {
                    acc = fmaf(x[u].x, y[u].x, acc);
                    acc = fmaf(x[u].y, y[u].y, acc);
                    acc = fmaf(x[u].z, y[u].z, acc);
                    acc = fmaf(x[u].w, y[u].w, acc);
                }
            }
        }
    }
    return acc;
}

// Member-pair distances are kept once per unordered pair: entry (r, q), r < q, of a kb x kb matrix.
__device__ __forceinline__ int tri_index(int r, int q, int kb) { return r * (2 * kb - r - 1) / 2 + (q - r - 1); }
__device__ __forceinline__ int pair_index(int a, int b, int kb) { return a < b ? tri_index(a, b, kb) : tri_index(b, a, kb); }

// The candidate list of one pivot, private to one wavefront.
struct WaveCands {
    unsigned long long ukey[kMaxCand];  // as assembled: order key << 32 | column; all ones = no candidate
    int32_t uid[kMaxCand];
    float udist[kMaxCand];
    float dist[kMaxCand];  // sorted, closest first
    int32_t id[kMaxCand];
    int16_t col[kMaxCand];
    uint8_t st[kMaxCand];
};

// bytes of the region that holds the staging rows first and the candidate lists afterwards
__host__ __device__ inline size_t nap_union_bytes(int kb) {
    const size_t a = (size_t)kb * (kChunk + 4) * sizeof(float), b = sizeof(WaveCands) * kWaves;
    return ((a > b ? a : b) + 15) & ~(size_t)15;
}

__device__ __forceinline__ unsigned long long cand_key(float dist, int col, int metric) {
    const uint32_t o = ord32(dist);
    return ((unsigned long long)(metric == CORAL_L2 ? o : ~o) << 32) | (uint32_t)col;
}

// rank-by-counting sort of the C assembled entries; returns the number of candidates (invalid ones drop out)
__device__ int sort_cands(WaveCands& S, int C, int lane) {
    wave_sync();
    int m = 0;
    for (int e0 = 0; e0 < C; e0 += 64) {
        const int e = e0 + lane;
        const unsigned long long k = e < C ? S.ukey[e] : ~0ull;
        const bool valid = k != ~0ull;
        m += __popcll(__ballot(valid));
        if (valid) {
            int rank = 0;
            for (int f = 0; f < C; ++f) rank += S.ukey[f] < k;
            S.dist[rank] = S.udist[e];
            S.id[rank] = S.uid[e];
            S.col[rank] = (int16_t)(uint32_t)k;
            S.st[rank] = ST_INITIAL;
        }
    }
    wave_sync();
    return m;
}

// candidate_ignore_kernel (src/upd_gpu.cu:203-247, src/enhance.cu:334-380): in order of distance a candidate not yet
// ruled out is retained and rules out every later one that is closer to it than to the pivot; duplicates of an id
// are marked.  Stops once R are retained.  G (optional) holds the member-pair distances by pair of columns.
template <bool HAVE_G>
__device__ void prune_cands(WaveCands& S, int m, int lane, const float* __restrict__ vec, int dim, int metric, int R,
                            const float* G, int kb) {
    int nbr_num = 0;
    for (int i = 0; i < m && nbr_num < R; ++i) {
        const uint8_t st = S.st[i];
        const int32_t idi = S.id[i];
        if (st == ST_INITIAL) {
            ++nbr_num;
            const int coli = S.col[i];
            const float* vi = vec + (size_t)idi * dim;
            for (int j = i + 1 + lane; j < m; j += 64) {
                const int32_t idj = S.id[j];
                if (idj == idi) {
                    S.st[j] = ST_REPEATED;
                } else if (S.st[j] == ST_INITIAL) {
                    const int colj = S.col[j];
                    float d;
                    if (HAVE_G && coli < kb && colj < kb)
                        d = G[pair_index(coli, colj, kb)];
                    else
                        d = seq_dist(vi, vec + (size_t)idj * dim, dim, metric);
                    if (closer(S.dist[j], d, metric)) S.st[j] = ST_DISCARDED;
                }
            }
            if (lane == 0) S.st[i] = ST_RETAINED;
        } else if (st == ST_DISCARDED) {
            for (int j = i + 1 + lane; j < m; j += 64)
                if (S.id[j] == idi) S.st[j] = ST_REPEATED;
        }
        wave_sync();
    }
}

// update_new_nbrs_kernel (src/upd_gpu.cu:102-156) / update_iso_nbrs_kernel (src/enhance.cu:528-568): the retained
// candidates and, with fill, the nearest discarded ones up to R, in order of distance.  Returns the row length.
__device__ int emit_row(const WaveCands& S, int m, int lane, int R, bool fill, int32_t* __restrict__ out_ids,
                        float* __restrict__ out_dists) {
    const unsigned long long below = (1ull << lane) - 1ull;
    int retained = 0;
    for (int j0 = 0; j0 < m; j0 += 64) {
        const int j = j0 + lane;
        retained += __popcll(__ballot(j < m && S.st[j] == ST_RETAINED));
    }
    const int need = fill ? R - retained : 0;
    int outn = 0, disc_seen = 0;
    for (int j0 = 0; j0 < m; j0 += 64) {
        const int j = j0 + lane;
        const uint8_t st = j < m ? S.st[j] : (uint8_t)ST_REPEATED;
        const unsigned long long mdisc = __ballot(st == ST_DISCARDED);
        const bool keep = st == ST_RETAINED || (st == ST_DISCARDED && disc_seen + __popcll(mdisc & below) < need);
        const unsigned long long mkeep = __ballot(keep);
        const int pos = outn + __popcll(mkeep & below);
        if (keep && pos < R) {
            out_ids[pos] = S.id[j];
            out_dists[pos] = S.dist[j];
        }
        outn += __popcll(mkeep);
        disc_seen += __popcll(mdisc);
    }
    return outn < R ? outn : R;
}

// ------------------------------------------------------------------------------------------------ NAP batch

__global__ void claim_kernel(const int32_t* __restrict__ ids, int64_t count, int32_t* __restrict__ owner) {
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < count; p += (int64_t)gridDim.x * blockDim.x)
        atomicMin(owner + ids[p], (int32_t)p);
}

// one workgroup per cluster; dynamic LDS: G[kb(kb-1)/2] | stage[kb][kChunk+4] or WaveCands[kWaves] | ids[kb] | deg[kb]
// (the staging rows of the distance phase and the candidate lists of the pivot phase are never live together)
__global__ void __launch_bounds__(kThreads)
nap_cluster_kernel(const float* __restrict__ vec, int dim, int metric, int R, const int32_t* __restrict__ nbrs,
                   const float* __restrict__ dists, const int32_t* __restrict__ deg, const int32_t* __restrict__ owner,
                   const int32_t* __restrict__ knn, int batch, int kb, int need_discard, int32_t* __restrict__ new_ids,
                   float* __restrict__ new_dists, int32_t* __restrict__ new_deg) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int lds = kChunk + 4;  // stage rows stay 16-byte aligned
    const int npairs = kb * (kb - 1) / 2;
    float* G = reinterpret_cast<float*>(smem);
    float* stage = G + ((npairs + 3) & ~3);
    WaveCands* cands = reinterpret_cast<WaveCands*>(stage);
    const size_t shared_bytes = nap_union_bytes(kb);
    int32_t* s_ids = reinterpret_cast<int32_t*>(reinterpret_cast<unsigned char*>(stage) + shared_bytes);
    int32_t* s_deg = s_ids + kb;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int C = kb + R;

    for (int b = blockIdx.x; b < batch; b += gridDim.x) {
        __syncthreads();
        for (int r = tid; r < kb; r += kThreads) {
            const int32_t id = knn[(size_t)b * kb + r];
            s_ids[r] = id;
            s_deg[r] = deg[id];
        }
        // member-pair distances, pair t of the folded enumeration to thread t % kThreads; between two chunks of
        // dimensions the running sum of a pair waits in G, so the chain of additions is the sequential one
        const int half = (kb + 1) / 2, rowlen = kb - 1;
        for (int d0 = 0; d0 < dim; d0 += kChunk) {
            const int cw = dim - d0 < kChunk ? dim - d0 : kChunk;
            __syncthreads();
            for (int t = tid; t < kb * cw; t += kThreads) {
                const int r = t / cw, c = t - r * cw;
                stage[r * lds + c] = vec[(size_t)s_ids[r] * dim + d0 + c];
            }
            __syncthreads();
            for (int t = tid; t < half * rowlen; t += kThreads) {
                // folded enumeration of the pairs r < q: row fr and row kb-1-fr together hold kb-1 of them
                const int fr = t / rowlen, c = t - fr * rowlen;
                int r = fr, q = fr + 1 + c;
                if (c >= rowlen - fr) {
                    r = kb - 1 - fr;
                    q = r + 1 + (c - (rowlen - fr));
                    if (r == fr) continue;  // odd kb: the middle row is its own partner
                }
                const int g = tri_index(r, q, kb);
                const float4* a = reinterpret_cast<const float4*>(stage + r * lds);
                const float4* bq = reinterpret_cast<const float4*>(stage + q * lds);
                float x = d0 ? G[g] : 0.0f;
                if (metric == CORAL_L2) {
                    for (int c = 0; c < cw / 4; ++c) {
                        const float4 u = a[c], w = bq[c];
                        float dlt = u.x - w.x;
                        x = fmaf(dlt, dlt, x);
                        dlt = u.y - w.y;
                        x = fmaf(dlt, dlt, x);
                        dlt = u.z - w.z;
                        x = fmaf(dlt, dlt, x);
                        dlt = u.w - w.w;
                        x = fmaf(dlt, dlt, x);
                    }
                } else {
                    for (int c = 0; c < cw / 4; ++c) {
                        const float4 u = a[c], w = bq[c];
                        x = fmaf(u.x, w.x, x);
                        x = fmaf(u.y, w.y, x);
                        x = fmaf(u.z, w.z, x);
                        x = fmaf(u.w, w.w, x);
                    }
                }
                G[g] = x;
            }
        }
        __syncthreads();

        // pivots of the cluster, one wavefront each
        int n_new = 0;  // members still without neighbours
        for (int r0 = 0; r0 < kb; r0 += 64) n_new += __popcll(__ballot(r0 + lane < kb && s_deg[r0 + lane] == 0));
        WaveCands& S = cands[wave];
        for (int r = wave; r < kb; r += kWaves) {
            const int64_t p = (int64_t)b * kb + r;
            const int32_t pid = s_ids[r];
            if (owner[pid] != (int32_t)p) continue;  // uniform in the wavefront
            const int rdeg = s_deg[r];
            if (rdeg > 0 && n_new == 0 && need_discard) {
                // no member is new, so the candidates are the pivot's own row (at most R entries, sorted, no
                // duplicates): whatever the occlusion rule retains, the fill puts the rest back in the same order.
                // The row comes out as it went in: nothing to compute, nothing to write.
                if (lane == 0) new_deg[p] = -1;
                continue;
            }
            for (int q = lane; q < C; q += 64) {
                unsigned long long key = ~0ull;
                int32_t id = -1;
                float d = 0.0f;
                if (q < kb) {
                    // src/upd_gpu.cu:45-73: not itself, and one of the two must still be without neighbours
                    if (q != r && s_ids[q] != pid && !(rdeg > 0 && s_deg[q] > 0)) {
                        id = s_ids[q];
                        d = G[pair_index(r, q, kb)];
                        key = cand_key(d, q, metric);
                    }
                } else if (q - kb < rdeg) {  // src/upd_gpu.cu:48-52: the current row
                    id = nbrs[(size_t)pid * R + (q - kb)];
                    d = dists[(size_t)pid * R + (q - kb)];
                    key = cand_key(d, q, metric);
                }
                S.ukey[q] = key;
                S.uid[q] = id;
                S.udist[q] = d;
            }
            const int m = sort_cands(S, C, lane);
            prune_cands<true>(S, m, lane, vec, dim, metric, R, G, kb);
            const int nd = emit_row(S, m, lane, R, need_discard != 0, new_ids + (size_t)p * R, new_dists + (size_t)p * R);
            if (lane == 0) new_deg[p] = nd;
            wave_sync();
        }
    }
}

// half a wavefront per pivot: the winner's staged row replaces the node's row
__global__ void nap_commit_kernel(const int32_t* __restrict__ knn, int64_t count, int R, int32_t* __restrict__ owner,
                                  const int32_t* __restrict__ new_ids, const float* __restrict__ new_dists,
                                  const int32_t* __restrict__ new_deg, int32_t* __restrict__ nbrs,
                                  float* __restrict__ dists, int32_t* __restrict__ deg) {
    const int64_t gtid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t p = gtid >> 5;
    const int l = (int)(gtid & 31);
    if (p >= count) return;
    const int32_t id = knn[p];
    if (owner[id] != (int32_t)p) return;
    const int nd = new_deg[p];
    if (nd >= 0 && l < R) {
        nbrs[(size_t)id * R + l] = l < nd ? new_ids[(size_t)p * R + l] : -1;
        dists[(size_t)id * R + l] = l < nd ? new_dists[(size_t)p * R + l] : 0.0f;
    }
    __builtin_amdgcn_wave_barrier();
    if (l == 0) {
        if (nd >= 0) deg[id] = nd;  // negative: the row stays as it is
        owner[id] = INT_MAX;
    }
}

// ------------------------------------------------------------------------------------- connectivity enhancement

// one wavefront per isolated node: length of its found list (an id of -1 ends it) and the claims on the found nodes
__global__ void enh_claim_kernel(const int32_t* __restrict__ knn_ids, int batch, int kn, int32_t* __restrict__ len,
                                 const int32_t* __restrict__ rev_len, int32_t* __restrict__ owner) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    for (int b = wave; b < batch; b += nwaves) {
        int n = kn;
        for (int i0 = 0; i0 < kn; i0 += 64) {
            const int i = i0 + lane;
            const unsigned long long neg = __ballot(i < kn && knn_ids[(size_t)b * kn + i] < 0);
            if (neg) {
                n = i0 + __ffsll((long long)neg) - 1;
                break;
            }
        }
        if (lane == 0) len[b] = n;
        if (rev_len) n = min(n, rev_len[b]);  // only these entries insert reverse edges
        for (int i = lane; i < n; i += 64) atomicMin(owner + knn_ids[(size_t)b * kn + i], b * kn + i);
    }
}

// build_candidate_kernel's reverse edge (src/enhance.cu:161-207).  Half a wavefront per (isolated node, found node)
// pair; lane = position in the found node's row.  stats: [0] inserted, [1] turned away by a full row.
__global__ void enh_reverse_kernel(const float* __restrict__ vec, int dim, int metric, int R, int32_t* __restrict__ nbrs,
                                   float* __restrict__ dists, int32_t* __restrict__ deg, int32_t* __restrict__ owner,
                                   const int32_t* __restrict__ iso_ids, const int32_t* __restrict__ knn_ids,
                                   const float* __restrict__ knn_dists, const int32_t* __restrict__ len,
                                   const int32_t* __restrict__ rev_len, int batch, int kn,
                                   unsigned long long* __restrict__ stats) {
    const int gtid = blockIdx.x * blockDim.x + threadIdx.x;
    const int l = gtid & 31, shift = threadIdx.x & 32;
    const int half = gtid >> 5, nhalf = (gridDim.x * blockDim.x) >> 5;
    const int total = batch * kn;
    const int rounds = (total + nhalf - 1) / nhalf;  // the same trip count for both halves of a wavefront
    unsigned int n_in = 0u, n_out = 0u;
    for (int rd_i = 0; rd_i < rounds; ++rd_i) {
        const int pair = half + rd_i * nhalf;
        bool active = pair < total;
        int b = 0, v = -1;
        if (active) {
            b = pair / kn;
            active = pair - b * kn < (rev_len ? min(len[b], rev_len[b]) : len[b]);
        }
        if (active) {
            v = knn_ids[pair];
            active = owner[v] == pair;
        }
        const int32_t iso = active ? iso_ids[b] : 0;
        const float vd = active ? knn_dists[pair] : 0.0f;
        const int d = active ? deg[v] : 0;
        const bool have = l < d;
        int32_t nb = -1;
        float rd = 0.0f, dij = 0.0f;
        if (have) {
            nb = nbrs[(size_t)v * R + l];
            rd = dists[(size_t)v * R + l];
            dij = seq_dist(vec + (size_t)iso * dim, vec + (size_t)nb * dim, dim, metric);
        }
        // the newcomer goes in front of the first entry that is not strictly closer than it
        const uint32_t ahead = (uint32_t)(__ballot(have && closer(vd, rd, metric)) >> shift);
        const int pos = ahead == 0xffffffffu ? 32 : __ffs((int)~ahead) - 1;
        // an entry in front that is closer to the newcomer than the row's owner is: the newcomer is occluded
        const uint32_t occl = (uint32_t)(__ballot(have && l < pos && closer(vd, dij, metric)) >> shift);
        // entries behind that the newcomer occludes
        const uint32_t evict = (uint32_t)(__ballot(have && l >= pos && closer(rd, dij, metric)) >> shift);
        bool accept = active;
        int out_pos = d, newdeg = d + 1;
        if (d == R) {
            newdeg = d;
            if (occl != 0u || pos >= d)
                accept = false;
            else
                out_pos = evict ? 31 - __clz((int)evict) : d - 1;
        }
        const int32_t nb_prev = __shfl_up(nb, 1, 32);
        const float rd_prev = __shfl_up(rd, 1, 32);
        if (accept) {
            if (l == pos) {
                nbrs[(size_t)v * R + l] = iso;
                dists[(size_t)v * R + l] = vd;
            } else if (l > pos && l <= out_pos) {
                nbrs[(size_t)v * R + l] = nb_prev;
                dists[(size_t)v * R + l] = rd_prev;
            }
        }
        if (active && l == 0) {
            if (accept) deg[v] = newdeg;
            owner[v] = INT_MAX;
            n_in += accept ? 1 : 0, n_out += accept ? 0 : 1;
        }
    }
    // the two counts of the whole workgroup in one atomic each (millions of pairs would otherwise queue on two words)
    __shared__ unsigned int s_in, s_out;
    if (threadIdx.x == 0) s_in = 0u, s_out = 0u;
    __syncthreads();
    if (n_in) atomicAdd(&s_in, n_in);
    if (n_out) atomicAdd(&s_out, n_out);
    __syncthreads();
    if (stats && threadIdx.x == 0) {
        if (s_in) atomicAdd(stats + 0, (unsigned long long)s_in);
        if (s_out) atomicAdd(stats + 1, (unsigned long long)s_out);
    }
}

// the isolated node's own row from its found list (src/enhance.cu:334-380, 519-575); one wavefront per node
__global__ void __launch_bounds__(kThreads)
enh_rows_kernel(const float* __restrict__ vec, int dim, int metric, int R, int32_t* __restrict__ nbrs,
                float* __restrict__ dists, int32_t* __restrict__ deg, const int32_t* __restrict__ iso_ids,
                const int32_t* __restrict__ knn_ids, const float* __restrict__ knn_dists,
                const int32_t* __restrict__ len, int batch, int kn) {
    __shared__ WaveCands cands[kWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    WaveCands& S = cands[wave];
    for (int b = blockIdx.x * kWaves + wave; b < batch; b += gridDim.x * kWaves) {
        const int n = len[b];
        const int32_t iso = iso_ids[b];
        for (int q = lane; q < kn; q += 64) {
            const bool ok = q < n;
            const float d = ok ? knn_dists[(size_t)b * kn + q] : 0.0f;
            S.ukey[q] = ok ? cand_key(d, q, metric) : ~0ull;
            S.uid[q] = ok ? knn_ids[(size_t)b * kn + q] : -1;
            S.udist[q] = d;
        }
        const int m = sort_cands(S, kn, lane);
        prune_cands<false>(S, m, lane, vec, dim, metric, R, nullptr, 0);
        int32_t* row = nbrs + (size_t)iso * R;
        float* rowd = dists + (size_t)iso * R;
        const int nd = emit_row(S, m, lane, R, true, row, rowd);
        for (int j = nd + lane; j < R; j += 64) row[j] = -1, rowd[j] = 0.0f;
        if (lane == 0) deg[iso] = nd;
        wave_sync();
    }
}

// build_candidate_kernel of the second phase (src/enhance.cu:58-129), the part that lists the candidates: what the
// search found for the node (up to the first -1), then the node's current row with its stored distances; -1 pads.
// One wavefront per node; out lists are [batch][k + R], rev_len[b] = number of found entries.
__global__ void enh_top_lists_kernel(int R, const int32_t* __restrict__ nbrs, const float* __restrict__ dists,
                                     const int32_t* __restrict__ deg, const int32_t* __restrict__ top_ids,
                                     const int32_t* __restrict__ knn_ids, const float* __restrict__ knn_dists, int batch,
                                     int k, int32_t* __restrict__ out_ids, float* __restrict__ out_dists,
                                     int32_t* __restrict__ rev_len) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, nwaves = (gridDim.x * blockDim.x) >> 6;
    const int kn = k + R;
    for (int b = wave; b < batch; b += nwaves) {
        int nf = k;
        for (int i0 = 0; i0 < k; i0 += 64) {
            const int i = i0 + lane;
            const unsigned long long neg = __ballot(i < k && knn_ids[(size_t)b * k + i] < 0);
            if (neg) {
                nf = i0 + __ffsll((long long)neg) - 1;
                break;
            }
        }
        const int32_t t = top_ids[b];
        const int d = deg[t];
        for (int q = lane; q < kn; q += 64) {
            int32_t id = -1;
            float dist = 0.0f;
            if (q < nf) {
                id = knn_ids[(size_t)b * k + q], dist = knn_dists[(size_t)b * k + q];
            } else if (q - nf < d) {
                id = nbrs[(size_t)t * R + (q - nf)], dist = dists[(size_t)t * R + (q - nf)];
            }
            out_ids[(size_t)b * kn + q] = id;
            out_dists[(size_t)b * kn + q] = dist;
        }
        if (lane == 0) rev_len[b] = nf;
    }
}

// hits_update_kernel (src/knn.cu:60-73): one more cluster contains these nodes
__global__ void count_hits_kernel(const int32_t* __restrict__ ids, int64_t count, uint32_t* __restrict__ hits) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < count; t += (int64_t)gridDim.x * blockDim.x)
        atomicAdd(hits + ids[t], 1u);
}

__global__ void count_bad_ids_kernel(const int32_t* __restrict__ ids, int64_t count, int64_t n, int minus_one_ok,
                                     unsigned long long* __restrict__ bad) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < count; t += (int64_t)gridDim.x * blockDim.x) {
        const int32_t id = ids[t];
        if (!((id >= 0 && id < n) || (minus_one_ok && id == -1))) atomicAdd(bad, 1ull);
    }
}

__global__ void gather_rows_kernel(const float* __restrict__ vec, int dim, const int32_t* __restrict__ ids, int count,
                                   float* __restrict__ out) {
    const int per = dim / 4;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < (int64_t)count * per;
         t += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(t / per), c = (int)(t - (int64_t)i * per);
        reinterpret_cast<float4*>(out)[t] = reinterpret_cast<const float4*>(vec + (size_t)ids[i] * dim)[c];
    }
}

}  // namespace

size_t nap_lds_bytes(int kb) {
    const size_t g = ((size_t)(kb * (kb - 1) / 2 + 3) & ~(size_t)3) * sizeof(float);
    return g + nap_union_bytes(kb) + (size_t)kb * 8;
}

hipError_t launch_nap_batch(const float* vec, int dim, int metric, int R, int32_t* nbrs, float* dists, int32_t* deg,
                            int32_t* owner, const int32_t* knn, int batch, int kb, int need_discard, int32_t* new_ids,
                            float* new_dists, int32_t* new_deg, hipStream_t st) {
    const int64_t P = (int64_t)batch * kb;
    const size_t lds = nap_lds_bytes(kb);
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(nap_cluster_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    int blocks = (int)((P + 255) / 256);
    hipLaunchKernelGGL(claim_kernel, dim3(blocks > 2048 ? 2048 : blocks), dim3(256), 0, st, knn, P, owner);
    hipLaunchKernelGGL(nap_cluster_kernel, dim3(batch), dim3(kThreads), lds, st, vec, dim, metric, R, nbrs, dists, deg,
                       owner, knn, batch, kb, need_discard, new_ids, new_dists, new_deg);
    hipLaunchKernelGGL(nap_commit_kernel, dim3((unsigned)((P * 32 + 255) / 256)), dim3(256), 0, st, knn, P, R, owner,
                       new_ids, new_dists, new_deg, nbrs, dists, deg);
    return hipGetLastError();
}

hipError_t launch_enhance_batch(const float* vec, int dim, int metric, int R, int32_t* nbrs, float* dists, int32_t* deg,
                                int32_t* owner, const int32_t* iso_ids, const int32_t* knn_ids, const float* knn_dists,
                                int batch, int kn, int32_t* len, const int32_t* rev_len, unsigned long long* stats,
                                hipStream_t st) {
    const int waves_per_block = 4;
    int blocks = (batch + waves_per_block - 1) / waves_per_block;
    hipLaunchKernelGGL(enh_claim_kernel, dim3(blocks), dim3(256), 0, st, knn_ids, batch, kn, len, rev_len, owner);
    const int64_t pairs = (int64_t)batch * kn;
    int64_t rb = (pairs * 32 + 255) / 256;
    rb = rb > 8192 ? 8192 : rb;
    hipLaunchKernelGGL(enh_reverse_kernel, dim3((unsigned)rb), dim3(256), 0, st, vec, dim, metric, R, nbrs, dists, deg,
                       owner, iso_ids, knn_ids, knn_dists, len, rev_len, batch, kn, stats);
    hipLaunchKernelGGL(enh_rows_kernel, dim3(blocks), dim3(kThreads), 0, st, vec, dim, metric, R, nbrs, dists, deg,
                       iso_ids, knn_ids, knn_dists, len, batch, kn);
    return hipGetLastError();
}

hipError_t launch_enhance_top_lists(int R, const int32_t* nbrs, const float* dists, const int32_t* deg,
                                    const int32_t* top_ids, const int32_t* knn_ids, const float* knn_dists, int batch, int k,
                                    int32_t* out_ids, float* out_dists, int32_t* rev_len, hipStream_t st) {
    hipLaunchKernelGGL(enh_top_lists_kernel, dim3((batch + 3) / 4), dim3(256), 0, st, R, nbrs, dists, deg, top_ids, knn_ids,
                       knn_dists, batch, k, out_ids, out_dists, rev_len);
    return hipGetLastError();
}

hipError_t launch_count_hits(const int32_t* ids, int64_t count, uint32_t* hits, hipStream_t st) {
    int64_t blocks = (count + 255) / 256;
    blocks = blocks > 2048 ? 2048 : (blocks < 1 ? 1 : blocks);
    hipLaunchKernelGGL(count_hits_kernel, dim3((unsigned)blocks), dim3(256), 0, st, ids, count, hits);
    return hipGetLastError();
}

hipError_t launch_count_bad_ids(const int32_t* ids, int64_t count, int64_t n, int minus_one_ok, unsigned long long* bad,
                                hipStream_t st) {
    int64_t blocks = (count + 255) / 256;
    blocks = blocks > 2048 ? 2048 : (blocks < 1 ? 1 : blocks);
    hipLaunchKernelGGL(count_bad_ids_kernel, dim3((unsigned)blocks), dim3(256), 0, st, ids, count, n, minus_one_ok, bad);
    return hipGetLastError();
}

hipError_t launch_gather_rows(const float* vec, int dim, const int32_t* ids, int count, float* out, hipStream_t st) {
    int64_t blocks = ((int64_t)count * (dim / 4) + 255) / 256;
    blocks = blocks > 4096 ? 4096 : (blocks < 1 ? 1 : blocks);
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, st, vec, dim, ids, count, out);
    return hipGetLastError();
}

}  // namespace coral
