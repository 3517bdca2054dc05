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
constexpr int NLD = BK / 8;                             // float4 loads per thread, operand and stage

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
__global__ __launch_bounds__(256, CORAL_MFMA_WAVES) void approx_tile_mfma_kernel(const float* __restrict__ queries,
                                                              const float* __restrict__ base, int nq, int64_t nb,
                                                              int dim, int metric, const float* __restrict__ qn,
                                                              const float* __restrict__ bn,
                                                              const uint32_t* __restrict__ deleted, int64_t base_id0,
                                                              float* __restrict__ D, int64_t ldD) {
    __shared__ float sa[2][BK][MT + 4];
    __shared__ float sb[2][BK][NT + 4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    // Workgroups go to the eight XCDs in turn, each with an L2 of its own: the workgroups that share a tile of
    // base points (one per tile of queries) are given consecutive places on one XCD, so that the base tile comes
    // from memory once and from that L2 afterwards.  grid.x = 8 x ceil(base tiles / 8) x query tiles.
    const int nqt = (nq + MT - 1) / MT;
    const unsigned xcd = blockIdx.x & 7u, place = blockIdx.x >> 3;
    const int64_t bt = (int64_t)(place / (unsigned)nqt) * 8 + xcd;
    const int64_t b0 = bt * NT;
    const int q0 = (int)(place % (unsigned)nqt) * MT;
    if (b0 >= nb) return;  // the padding of the last group of eight base tiles
    const int lrow = tid >> 1, lk = (tid & 1) * 4;  // staging: thread t loads row t/2, dimensions (t&1)*4 .. +4
    float4 va[NLD], vb[NLD];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            va[u] = make_float4(0, 0, 0, 0), vb[u] = make_float4(0, 0, 0, 0);
            const int kd = k0 + lk + 8 * u;
            if (kd < dim) {
                if (q0 + lrow < nq) va[u] = *reinterpret_cast<const float4*>(queries + (size_t)(q0 + lrow) * dim + kd);
                if (b0 + lrow < nb) vb[u] = *reinterpret_cast<const float4*>(base + (size_t)(b0 + lrow) * dim + kd);
            }
        }
    };
    auto park = [&](int buf) {
#pragma unroll
        for (int u = 0; u < NLD; ++u) {
            const int r = lk + 8 * u;
            sa[buf][r + 0][lrow] = va[u].x, sa[buf][r + 1][lrow] = va[u].y, sa[buf][r + 2][lrow] = va[u].z, sa[buf][r + 3][lrow] = va[u].w;
            sb[buf][r + 0][lrow] = vb[u].x, sb[buf][r + 1][lrow] = vb[u].y, sb[buf][r + 2][lrow] = vb[u].z, sb[buf][r + 3][lrow] = vb[u].w;
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
    fetch(0);
    park(0);
    __syncthreads();
    int cur = 0;
    for (int k0 = 0; k0 < dim; k0 += BK) {
        const bool more = k0 + BK < dim;
        if (more) fetch(k0 + BK);
        // the operands of a pair of dimensions are read while the pair before is multiplied
        float a0 = sa[cur][kh][wr * 64 + m], a1 = sa[cur][kh][wr * 64 + 32 + m];
        float c0 = sb[cur][kh][wc * 64 + m], c1 = sb[cur][kh][wc * 64 + 32 + m];
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float a0n = 0.0f, a1n = 0.0f, c0n = 0.0f, c1n = 0.0f;
            if (kk + 2 < BK) {
                a0n = sa[cur][kk + 2 + kh][wr * 64 + m], a1n = sa[cur][kk + 2 + kh][wr * 64 + 32 + m];
                c0n = sb[cur][kk + 2 + kh][wc * 64 + m], c1n = sb[cur][kk + 2 + kh][wc * 64 + 32 + m];
            }
            __builtin_amdgcn_sched_barrier(0);  // keeps the reads above ahead of the multiplications below
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, c0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, c1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, c0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, c1, acc[1][1], 0, 0, 0);
            a0 = a0n, a1 = a1n, c0 = c0n, c1 = c1n;
        }
        if (more) park(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    // a 32 x 32 block's 16 registers: register v of lane l holds row 8 (v / 4) + 4 (l / 32) + v % 4, column l % 32.
    // The norms of the tile's rows and columns (+inf for a tombstoned column) come through LDS, fetched once per
    // workgroup instead of by 64 dependent global loads per lane.
    float* srow = &sa[0][0][0];  // the operand buffers are free after the last barrier of the loop
    float* scol = &sb[0][0][0];
    const float inf = __int_as_float(0x7f800000);
    if (tid < MT) {
        const int r = q0 + tid;
        srow[tid] = (metric == 0 && r < nq) ? qn[r] : 0.0f;
    } else if (tid < MT + NT) {
        const int64_t c = b0 + (tid - MT);
        float v = 0.0f;
        if (c < nb) {
            if (metric == 0) v = bn[c];
            if (deleted) {
                const int64_t id = base_id0 + c;
                if ((deleted[id >> 5] >> (id & 31)) & 1u) v = inf;
            }
        }
        scol[tid - MT] = v;
    }
    __syncthreads();
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
        float4 rown[4];  // |q|^2 of the 16 rows this lane holds of a block: four runs of four
#pragma unroll
        for (int g = 0; g < 4; ++g) rown[g] = *reinterpret_cast<const float4*>(srow + wr * 64 + ti * 32 + 8 * g + 4 * kh);
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) {
            const int cl = wc * 64 + tj * 32 + m;
            const int64_t c = b0 + cl;
            const float bnc = scol[cl];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = q0 + wr * 64 + ti * 32 + 8 * (v >> 2) + 4 * kh + (v & 3);
                const float4 rn4 = rown[v >> 2];
                const float rn = (v & 3) == 0 ? rn4.x : (v & 3) == 1 ? rn4.y : (v & 3) == 2 ? rn4.z : rn4.w;
                const float dot = acc[ti][tj][v];
                // (|q|^2 + |b|^2) - 2 q.b; a tombstoned column's +inf survives both forms
                const float s = metric == 0 ? (rn + bnc) - 2.0f * dot : (bnc == inf ? inf : 0.0f - dot);
                if (r < nq && c < nb) D[(size_t)r * ldD + c] = s;
            }
        }
    }
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

hipError_t launch_approx_tile(const float* queries, const float* base, int nq, int64_t nb, int dim, int metric,
                              const float* qn, const float* bn, const uint32_t* deleted, int64_t base_id0, float* D,
                              int64_t ldD, hipStream_t stream) {
    const int64_t nbt = (nb + NT - 1) / NT, nqt = (nq + MT - 1) / MT;
    const int64_t wgs = (nbt + 7) / 8 * 8 * nqt;
    if (wgs <= 0 || wgs > 0x7fffffff) return hipErrorInvalidValue;
    dim3 grid((unsigned)wgs);
    hipLaunchKernelGGL(approx_tile_mfma_kernel, grid, dim3(256), 0, stream, queries, base, nq, nb, dim, metric, qn, bn,
                       deleted, base_id0, D, ldD);
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
