// bruteforce_mfma.hip -- the screening pass of the exact k-nearest-neighbour search on the matrix cores.
//
// The exact search (bruteforce.hip) accumulates every (query, base) pair in the reference's order, one fused
// multiply-add per dimension on the vector units, because ids and distances must be reproducible bit for bit.  Almost
// all of that work goes into pairs that are nowhere near the k best.  Here the same pairs are first measured
// approximately, as |q|^2 + |b|^2 - 2 q.b with the inner products on fp32 MFMA (v_mfma_f32_32x32x2_f32: full
// fp32 operands and accumulation, only the order of the additions differs), k + 32 candidates per query are kept,
// and rerank_kernel measures just those in the reference's order.  The result is exact, not approximately exact: a
// query is accepted only if its k-th exact distance lies below the worst kept approximate distance by more than a
// bound on what the two ways of rounding can differ by; otherwise it is flagged and goes through the exact search.
//
// Error bound.  With u = 2^-24 and any order of fp32 fused multiply-adds, a sum of dim products q_i b_i is within
// dim u |q| |b| of the true value (first order), the two norms within dim u of themselves, the two final additions
// add 4 u (|q|^2 + |b|^2); the reference-order distance itself is within (dim + 2) u of the true one.  Together the
// approximate and the reference-order value of a pair differ by less than 4 (dim + 2) u (|q|^2 + |b|^2); the check
// uses twice that, with the largest |b|^2 of the index.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bruteforce.h"

namespace coral {

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

#ifndef CORAL_MFMA_BK
#define CORAL_MFMA_BK 8
#endif
constexpr int MT = 128, NT = 128, BK = CORAL_MFMA_BK;  // tile of queries x base points per workgroup, dimensions per LDS stage
constexpr int NS = BK / 8;                              // 16-byte pieces per thread, operand and stage
constexpr int RS = BK == 8 ? 8 : BK + 4;                // floats from one row to the next in LDS


__device__ __forceinline__ uint32_t mf_ord32(float s) {
    const uint32_t u = __float_as_uint(s);
    return u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
}
__device__ __forceinline__ float mf_unord32(uint32_t o) {
    const uint32_t u = (o & 0x80000000u) ? (o ^ 0x80000000u) : ~o;
    return __uint_as_float(u);
}

// |x|^2 per row, and the largest of them (as the bit pattern of a non-negative float)
__global__ __launch_bounds__(256) void row_norms_kernel(const float* __restrict__ x, int64_t n, int dim,
                                                       float* __restrict__ out, uint32_t* __restrict__ max_bits) {
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    float s = 0.0f;
    if (r < n) {
        const float4* p = reinterpret_cast<const float4*>(x + (size_t)r * dim);
        for (int c = 0; c < dim / 4; ++c) {
            const float4 v = p[c];
            s = __fmaf_rn(v.x, v.x, s), s = __fmaf_rn(v.y, v.y, s), s = __fmaf_rn(v.z, v.z, s), s = __fmaf_rn(v.w, v.w, s);
        }
        out[r] = s;
    }
    if (max_bits) {
        float m = s;
        for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
        if ((threadIdx.x & 63) == 0) atomicMax(max_bits, __float_as_uint(m));
    }
}

// D[q][b] ~ signed distance (smaller is closer): |q|^2 + |b|^2 - 2 q.b for L2, -q.b for IP; +inf for tombstoned
// ids.  One workgroup per 128 x 128 tile (the mapping of blockIdx to tiles is at the head of the kernel), 256
// threads = 4 wavefronts in 2 x 2, each 64 x 64 of the tile as 2 x 2 MFMA blocks of 32 x 32.  Operands go through
// LDS dimension-major, so that the 32 lanes of an MFMA operand read consecutive words.
#ifndef CORAL_MFMA_WAVES
#define CORAL_MFMA_WAVES 4
#endif
// FUSED = false writes the tile into D (column bt * 128 + ..., where bt counts the tiles this launch computes:
// tile_stride > 1 takes every tile_stride-th tile of the base, a sample whose columns lie side by side in D).
// FUSED = true writes no matrix: an entry goes, as the key ord(value) << 32 | id, to the list of its query if it does
// not exceed the query's bound tau[q] -- cnt[q] entries so far, at most cap kept (a count beyond cap tells the
// caller that the list is incomplete).  A tile's entries are first gathered in LDS, so that the global counters see
// one round of atomics per tile instead of one per accumulator register.
template <bool FUSED, bool L2>
__global__ __launch_bounds__(256, CORAL_MFMA_WAVES) void approx_tile_mfma_kernel(const float* __restrict__ queries,
                                                              const float* __restrict__ base, int nq, int64_t nb,
                                                              int dim, const float* __restrict__ qn,
                                                              const float* __restrict__ bn,
                                                              const uint32_t* __restrict__ deleted, int64_t base_id0,
                                                              int64_t ntiles, int64_t tile_stride, int hq,
                                                              float* __restrict__ D, int64_t ldD,
                                                              const float* __restrict__ tau,
                                                              unsigned long long* __restrict__ lists, int64_t cap,
                                                              unsigned int* __restrict__ cnt) {
    // Operands in LDS row-major, the BK = 8 dimensions of a row side by side (32 bytes): a thread parks the 16 bytes
    // it fetched with one write, and the 16 bytes a lane reads hold its operands of four multiplications -- lane
    // (kh, m) supplies row m's dimension kh * 4 + j to step j, so a step multiplies the dimension pair (j, 4 + j) of
    // the stage.  The 64 lanes of either access cover consecutive addresses: no bank conflicts, no padding.
    __shared__ __align__(16) float sa[2][MT][RS];
    __shared__ __align__(16) float sb[2][NT][RS];
    static_assert(BK % 8 == 0, "a stage is made of 16-byte pieces, one per thread, operand and eight dimensions");
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    // Workgroups go to the eight XCDs in turn, each with an L2 of its own (4 MB).  An XCD takes every eighth tile of
    // base points and walks, for one block of hq query tiles after the other, through all its base tiles: the
    // workgroups in flight on it share those hq query tiles (hq x 100 KB at dim 200) and a handful of base tiles,
    // so both operands come from that L2 and each base tile from memory once per block of queries.
    // grid.x = 8 x ceil(base tiles / 8) x query blocks x hq.
    const int nqt = (nq + MT - 1) / MT;
    const unsigned xcd = blockIdx.x & 7u, place = blockIdx.x >> 3;
    const unsigned nbt8 = (unsigned)((ntiles + 7) >> 3);
    const unsigned qb = place / (nbt8 * (unsigned)hq), rem = place - qb * nbt8 * (unsigned)hq;
    const int64_t bt = (int64_t)(rem / (unsigned)hq) * 8 + xcd;
    const int qt = (int)(qb * (unsigned)hq + rem % (unsigned)hq);
    const int64_t b0 = bt * tile_stride * NT;
    const int q0 = qt * MT;
    if (bt >= ntiles || b0 >= nb || qt >= nqt) return;  // padding: the last group of eight base tiles, the last query block
    const int lrow = tid >> 1, lk = (tid & 1) * 4;  // staging: thread t loads row t/2, dimensions (t&1)*4 .. +4
    // rows beyond the end read the last row instead: their results are never written
    const float* pa = queries + (size_t)min(q0 + lrow, nq - 1) * dim + lk;
    const float* pb = base + (size_t)min(b0 + lrow, nb - 1) * dim + lk;
    float4 va[NS], vb[NS];
    auto park = [&](int buf) {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            *reinterpret_cast<float4*>(&sa[buf][lrow][8 * u + lk]) = va[u];
            *reinterpret_cast<float4*>(&sb[buf][lrow][8 * u + lk]) = vb[u];
        }
    };
    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    const int kh = lane >> 5, m = lane & 31;  // an MFMA operand: lane = row (or column) m of dimension kh
    // the last stage may hold half a row (dim is a multiple of 4): its missing half is zero
    const int full = dim / BK, tail = dim % BK;
    auto fetch = [&](int st) {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            va[u] = *reinterpret_cast<const float4*>(pa + st * BK + 8 * u);
            vb[u] = *reinterpret_cast<const float4*>(pb + st * BK + 8 * u);
        }
    };
    auto fetch_tail = [&]() {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            va[u] = make_float4(0, 0, 0, 0), vb[u] = make_float4(0, 0, 0, 0);
            if (8 * u + lk < tail) {
                va[u] = *reinterpret_cast<const float4*>(pa + full * BK + 8 * u);
                vb[u] = *reinterpret_cast<const float4*>(pb + full * BK + 8 * u);
            }
        }
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int u = 0; u < NS; ++u) {
            const float4 a0 = *reinterpret_cast<const float4*>(&sa[buf][wr * 64 + m][8 * u + kh * 4]);
            const float4 a1 = *reinterpret_cast<const float4*>(&sa[buf][wr * 64 + 32 + m][8 * u + kh * 4]);
            const float4 c0 = *reinterpret_cast<const float4*>(&sb[buf][wc * 64 + m][8 * u + kh * 4]);
            const float4 c1 = *reinterpret_cast<const float4*>(&sb[buf][wc * 64 + 32 + m][8 * u + kh * 4]);
#define CORAL_MFMA_STEP(X)                                                                  \
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.X, c0.X, acc[0][0], 0, 0, 0); \
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.X, c1.X, acc[0][1], 0, 0, 0); \
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.X, c0.X, acc[1][0], 0, 0, 0); \
        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.X, c1.X, acc[1][1], 0, 0, 0);
            CORAL_MFMA_STEP(x)
            CORAL_MFMA_STEP(y)
            CORAL_MFMA_STEP(z)
            CORAL_MFMA_STEP(w)
#undef CORAL_MFMA_STEP
        }
    };
    const int stages = full + (tail ? 1 : 0);
    if (full > 0)
        fetch(0);
    else
        fetch_tail();
    park(0);
    __syncthreads();
    int cur = 0;
    for (int st = 0; st < stages; ++st) {
        const bool more = st + 1 < stages;
        if (st + 1 < full)
            fetch(st + 1);
        else if (more)
            fetch_tail();
        multiply(cur);
        if (more) park(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    // a 32 x 32 block's 16 registers: register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4, column l % 32.
    // The norms of the tile's rows and columns (+inf for a tombstoned column) come through LDS, fetched once per
    // workgroup instead of by 64 dependent global loads per lane.
    float* srow = &sa[0][0][0];  // the operand buffers are free after the last barrier of the loop
    float* scol = &sb[0][0][0];
    float* stau = srow + MT;
    // (FUSED) the tile's entries that pass: ord(value) << 32 | place, where place = accumulator register << 8 |
    // thread names the entry's row and column; they lie behind the norms
    unsigned long long* shit = reinterpret_cast<unsigned long long*>(scol + NT);
    constexpr int kHitCap = (2 * NT * RS - NT) / 2;
    unsigned int& s_nhit = *reinterpret_cast<unsigned int*>(stau + MT);
    const float inf = __int_as_float(0x7f800000), nan = __int_as_float(0x7fc00000);
    if (tid < MT) {
        const int r = q0 + tid;
        srow[tid] = (L2 && r < nq) ? qn[r] : 0.0f;
        if constexpr (FUSED) stau[tid] = r < nq ? tau[r] : -inf;
    } else if (tid < MT + NT) {
        // what a column adds to its entries: |b|^2 (L2) or 0, +inf for a tombstoned id; (FUSED) NaN beyond the end of
        // the base, which no comparison passes
        const int64_t c = b0 + (tid - MT);
        float v = FUSED ? nan : 0.0f;
        if (c < nb) {
            v = L2 ? bn[c] : 0.0f;
            if (deleted) {
                const int64_t id = base_id0 + c;
                if ((deleted[id >> 5] >> (id & 31)) & 1u) v = inf;
            }
        }
        scol[tid - MT] = v;
    }
    if (tid == 0) s_nhit = 0u;
    __syncthreads();
    // register v of block (ti, tj) in thread t: row and column inside the tile
    auto row_of = [&](int t, int ti, int v) { return ((t >> 6) >> 1) * 64 + ti * 32 + 8 * (v >> 2) + 4 * ((t & 63) >> 5) + (v & 3); };
    auto col_of = [&](int t, int tj) { return ((t >> 6) & 1) * 64 + tj * 32 + (t & 31); };
    auto emit = [&](int rl, int cl, float sv) {
        const int r = q0 + rl;
        const unsigned pos = atomicAdd(&cnt[r], 1u);
        if (pos < (unsigned)cap)
            lists[(size_t)r * cap + pos] = ((unsigned long long)mf_ord32(sv) << 32) | (uint32_t)(base_id0 + b0 + cl);
    };
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
        float4 rown[4];  // |q|^2 of the 16 rows this lane holds of a block: four runs of four
        float4 taun[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            rown[g] = *reinterpret_cast<const float4*>(srow + wr * 64 + ti * 32 + 8 * g + 4 * kh);
            if constexpr (FUSED) taun[g] = *reinterpret_cast<const float4*>(stau + wr * 64 + ti * 32 + 8 * g + 4 * kh);
        }
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) {
            const int cl = wc * 64 + tj * 32 + m;
            const int64_t c = b0 + cl;
            const float bnc = scol[cl];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float4 rn4 = rown[v >> 2];
                const float rn = (v & 3) == 0 ? rn4.x : (v & 3) == 1 ? rn4.y : (v & 3) == 2 ? rn4.z : rn4.w;
                const float dot = acc[ti][tj][v];
                // (|q|^2 + |b|^2) - 2 q.b, or -q.b; a tombstoned column's +inf survives both forms
                const float sv = L2 ? __fmaf_rn(-2.0f, dot, rn + bnc) : bnc - dot;
                if constexpr (FUSED) {
                    const float4 t4 = taun[v >> 2];
                    const float tq = (v & 3) == 0 ? t4.x : (v & 3) == 1 ? t4.y : (v & 3) == 2 ? t4.z : t4.w;
                    if (sv <= tq) {  // rows beyond nq have tau = -inf, columns beyond nb give NaN
                        const unsigned pos = atomicAdd(&s_nhit, 1u);
                        if (pos < (unsigned)kHitCap)
                            shit[pos] = ((unsigned long long)mf_ord32(sv) << 32) | (unsigned)(((ti * 2 + tj) * 16 + v) << 8) | (unsigned)tid;
                        else  // more hits than the tile's buffer holds: straight to the list
                            emit(row_of(tid, ti, v), cl, sv);
                    }
                } else {
                    const int r = q0 + row_of(tid, ti, v);
                    if (r < nq && c < nb) D[(size_t)r * ldD + bt * NT + cl] = sv;
                }
            }
        }
    }
    if constexpr (FUSED) {
        __syncthreads();
        const int nhit = (int)min(s_nhit, (unsigned)kHitCap);
        for (int i = tid; i < nhit; i += 256) {
            const unsigned long long h = shit[i];
            const int t = (int)(h & 0xffu), reg = (int)((h >> 8) & 0x3fu);
            emit(row_of(t, reg >> 5, reg & 15), col_of(t, (reg >> 4) & 1), mf_unord32((uint32_t)(h >> 32)));
        }
    }
}

// tau[q] = value of the key keys[q * stride + j] (the j-th smallest of a sample of the row), +inf where the sample
// has no j-th entry
__global__ void bound_from_keys_kernel(const unsigned long long* __restrict__ keys, int64_t stride, int j, int nq,
                                       float* __restrict__ tau) {
    const int q = blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= nq) return;
    const unsigned long long key = keys[(size_t)q * stride + j];
    tau[q] = key == ~0ull ? __int_as_float(0x7f800000) : mf_unord32((uint32_t)(key >> 32));
}

// One workgroup per query: the kc candidates (ids, -1 = none; approximate signed distances, ascending) are measured
// in the reference's order (one thread walks the dimensions of one candidate with one fused multiply-add each,
// include/utils.cuh:254-275, 307-323: the arithmetic of distance_tile_kernel), sorted by (distance, id), and the k
// best written.  redo[q] = 1 when the result cannot be vouched for (see the head of this file).
__global__ __launch_bounds__(256) void rerank_kernel(const float* __restrict__ queries, const float* __restrict__ base,
                                                    int dim, int metric, const int32_t* __restrict__ cand_ids,
                                                    const float* __restrict__ cand_d, int kc, int k,
                                                    const float* __restrict__ qn, const uint32_t* __restrict__ bn_max_bits,
                                                    int32_t* __restrict__ ids, float* __restrict__ dists,
                                                    int* __restrict__ redo) {
    extern __shared__ unsigned long long rkeys[];
    const int q = blockIdx.x, tid = threadIdx.x;
    int P = 2;
    while (P < kc) P <<= 1;
    const float* qv = queries + (size_t)q * dim;
    for (int i = tid; i < P; i += 256) {
        unsigned long long key = ~0ull;
        const int32_t id = i < kc ? cand_ids[(size_t)q * kc + i] : -1;
        if (id >= 0) {
            const float4* b4 = reinterpret_cast<const float4*>(base + (size_t)id * dim);
            const float4* q4 = reinterpret_cast<const float4*>(qv);
            float s = 0.0f;
            if (metric == 0) {
                for (int c = 0; c < dim / 4; ++c) {
                    const float4 a = q4[c], b = b4[c];
                    float t;
                    t = a.x - b.x, s = __fmaf_rn(t, t, s);
                    t = a.y - b.y, s = __fmaf_rn(t, t, s);
                    t = a.z - b.z, s = __fmaf_rn(t, t, s);
                    t = a.w - b.w, s = __fmaf_rn(t, t, s);
                }
            } else {
                for (int c = 0; c < dim / 4; ++c) {
                    const float4 a = q4[c], b = b4[c];
                    s = __fmaf_rn(a.x, b.x, s), s = __fmaf_rn(a.y, b.y, s), s = __fmaf_rn(a.z, b.z, s), s = __fmaf_rn(a.w, b.w, s);
                }
                s = 0.0f - s;
            }
            key = ((unsigned long long)mf_ord32(s) << 32) | (uint32_t)id;
        }
        rkeys[i] = key;
    }
    __syncthreads();
    for (int k2 = 2; k2 <= P; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            for (int t = tid; t < (P >> 1); t += 256) {
                const int i = 2 * t - (t & (j - 1)), x = i + j;
                const bool asc = (i & k2) == 0;
                const unsigned long long ka = rkeys[i], kb = rkeys[x];
                if ((ka > kb) == asc) rkeys[i] = kb, rkeys[x] = ka;
            }
            __syncthreads();
        }
    for (int i = tid; i < k; i += 256) {
        const unsigned long long key = rkeys[i];
        const bool none = key == ~0ull;
        ids[(size_t)q * k + i] = none ? -1 : (int32_t)(uint32_t)key;
        if (dists) {
            const float s = mf_unord32((uint32_t)(key >> 32));
            const float far = 3.402823466e+38f;
            dists[(size_t)q * k + i] = none ? (metric == 0 ? far : -far) : (metric == 0 ? s : 0.0f - s);
        }
    }
    if (tid == 0) {
        int bad = 0;
        // every live point is a candidate unless the list is full; a full list vouches for the k best only if the
        // k-th of them lies clear of the worst candidate's approximate distance
        if (cand_ids[(size_t)q * kc + kc - 1] >= 0) {
            const float worst = cand_d[(size_t)q * kc + kc - 1];
            const float delta = 8.0f * (float)(dim + 2) * 5.9604645e-8f * (qn[q] + __uint_as_float(*bn_max_bits));
            const unsigned long long kth = rkeys[k - 1];
            const float sk = mf_unord32((uint32_t)(kth >> 32));
            if (kth == ~0ull || !(sk < worst - delta)) bad = 1;
        }
        redo[q] = bad;
    }
}

// dst[rows[i]][0..k) = src[i][0..k)
__global__ void scatter_results_kernel(const int32_t* __restrict__ rows, int count, int k, const int32_t* __restrict__ src_ids,
                                       const float* __restrict__ src_d, int32_t* __restrict__ dst_ids,
                                       float* __restrict__ dst_d) {
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < (int64_t)count * k;
         t += (int64_t)gridDim.x * blockDim.x) {
        const int i = (int)(t / k), j = (int)(t - (int64_t)i * k);
        dst_ids[(size_t)rows[i] * k + j] = src_ids[t];
        if (dst_d) dst_d[(size_t)rows[i] * k + j] = src_d[t];
    }
}

}  // namespace

hipError_t launch_row_norms(const float* x, int64_t n, int dim, float* out, uint32_t* max_bits, hipStream_t stream) {
    const int64_t blocks = (n + 255) / 256;
    if (blocks <= 0 || blocks > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(row_norms_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, n, dim, out, max_bits);
    return hipGetLastError();
}

#ifndef CORAL_MFMA_HQ
#define CORAL_MFMA_HQ 16
#endif
constexpr int64_t kQueryTilesPerBlock = CORAL_MFMA_HQ;  // query tiles an XCD keeps in its L2 while it walks the base

hipError_t launch_approx_tile(const float* queries, const float* base, int nq, int64_t nb, int dim, int metric,
                              const float* qn, const float* bn, const uint32_t* deleted, int64_t base_id0, float* D,
                              int64_t ldD, hipStream_t stream, int64_t sample_tiles, int64_t tile_stride) {
    const int64_t nbt = sample_tiles > 0 ? sample_tiles : (nb + NT - 1) / NT, nqt = (nq + MT - 1) / MT;
    const int64_t qblocks = (nqt + kQueryTilesPerBlock - 1) / kQueryTilesPerBlock, hq = (nqt + qblocks - 1) / qblocks;
    const int64_t wgs = (nbt + 7) / 8 * 8 * qblocks * hq;
    if (wgs <= 0 || wgs > 0x7fffffff || tile_stride < 1) return hipErrorInvalidValue;
    dim3 grid((unsigned)wgs);
    auto kernel = metric == 0 ? approx_tile_mfma_kernel<false, true> : approx_tile_mfma_kernel<false, false>;
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, queries, base, nq, nb, dim, qn, bn, deleted, base_id0, nbt,
                       tile_stride, (int)hq, D, ldD, (const float*)nullptr, (unsigned long long*)nullptr, (int64_t)0,
                       (unsigned int*)nullptr);
    return hipGetLastError();
}

hipError_t launch_approx_filter(const float* queries, const float* base, int nq, int64_t nb, int dim, int metric,
                                const float* qn, const float* bn, const uint32_t* deleted, const float* tau,
                                unsigned long long* lists, int64_t cap, unsigned int* cnt, hipStream_t stream) {
    const int64_t nbt = (nb + NT - 1) / NT, nqt = (nq + MT - 1) / MT;
    const int64_t qblocks = (nqt + kQueryTilesPerBlock - 1) / kQueryTilesPerBlock, hq = (nqt + qblocks - 1) / qblocks;
    const int64_t wgs = (nbt + 7) / 8 * 8 * qblocks * hq;
    if (wgs <= 0 || wgs > 0x7fffffff || nb > 0x7fffffff) return hipErrorInvalidValue;
    dim3 grid((unsigned)wgs);
    auto kernel = metric == 0 ? approx_tile_mfma_kernel<true, true> : approx_tile_mfma_kernel<true, false>;
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, queries, base, nq, nb, dim, qn, bn, deleted, (int64_t)0, nbt,
                       (int64_t)1, (int)hq, (float*)nullptr, (int64_t)0, tau, lists, cap, cnt);
    return hipGetLastError();
}

hipError_t launch_bound_from_keys(const unsigned long long* keys, int64_t stride, int j, int nq, float* tau,
                                  hipStream_t stream) {
    hipLaunchKernelGGL(bound_from_keys_kernel, dim3((nq + 255) / 256), dim3(256), 0, stream, keys, stride, j, nq, tau);
    return hipGetLastError();
}

hipError_t launch_rerank(const float* queries, const float* base, int nq, int dim, int metric, const int32_t* cand_ids,
                         const float* cand_d, int kc, int k, const float* qn, const uint32_t* bn_max_bits, int32_t* ids,
                         float* dists, int* redo, hipStream_t stream) {
    int P = 2;
    while (P < kc) P <<= 1;
    hipLaunchKernelGGL(rerank_kernel, dim3(nq), dim3(256), (size_t)P * 8, stream, queries, base, dim, metric, cand_ids,
                       cand_d, kc, k, qn, bn_max_bits, ids, dists, redo);
    return hipGetLastError();
}

hipError_t launch_scatter_results(const int32_t* rows, int count, int k, const int32_t* src_ids, const float* src_d,
                                  int32_t* dst_ids, float* dst_d, hipStream_t stream) {
    int64_t blocks = ((int64_t)count * k + 255) / 256;
    blocks = blocks > 4096 ? 4096 : (blocks < 1 ? 1 : blocks);
    hipLaunchKernelGGL(scatter_results_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, rows, count, k, src_ids, src_d,
                       dst_ids, dst_d);
    return hipGetLastError();
}

}  // namespace coral
