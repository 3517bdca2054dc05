// bruteforce.hip -- exact k-nearest-neighbour search by brute force on gfx950.
//
// Stands where the reference uses faiss: the ground-truth tool (tests/comp_gt.cpp:119-176,
// GpuIndexFlatL2/IP) and the builder's exact k_b-NN of auxiliary queries
// (src/knn.cu:174-193).  Output order and file layout are the gt file's
// (uint32 nq, uint32 k, int32 ids[nq*k], include/efanna2e/util.h:81-103).
//
// The search screens all pairs on the matrix cores first and re-ranks a few candidates per query exactly
// (bruteforce_mfma.hip); the kernels here are the selection both ways share, and the plain distance pass that
// defines the result and takes over where the screening cannot vouch for it:
//   distance_tile_kernel  a 128 x 128 tile of (query, base) pairs per workgroup, 8 x 8 pairs per
//                         thread, operands staged through LDS.  Every pair is accumulated by ONE
//                         thread walking the dimensions in order with one fused multiply-add per
//                         dimension -- the arithmetic of the reference's l2_distance / ip_distance
//                         (include/utils.cuh:254-275, 307-323) -- so the distances, and hence the
//                         ids, are reproducible bit for bit on a CPU.
//   row_select_kernel     per query row: a threshold from the per-thread minima, one more pass that
//                         collects the entries up to it into LDS, a sort by (value, id).  Rows with too
//                         many ties at the threshold go to row_select_radix_kernel: exact k-th smallest by
//                         an 8-bit radix select over the order-preserving bit pattern, ordered compaction.
//   merge_segments_kernel per query: the k best of the per-segment winners (large bases are
//                         processed in segments so the distance buffer stays bounded).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bruteforce.h"

namespace coral {

namespace {

__device__ __forceinline__ uint32_t bf_ord32(float s) {
    const uint32_t u = __float_as_uint(s);
    return u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
}
__device__ __forceinline__ float bf_unord32(uint32_t o) {
    const uint32_t u = (o & 0x80000000u) ? (o ^ 0x80000000u) : ~o;
    return __uint_as_float(u);
}

constexpr int TQ = 128, TB = 128, KC = 8;  // tile of queries x base points, dimensions per LDS stage

}  // namespace

// D[q][b] = signed distance (smaller is closer): sum (q-b)^2 for L2, 0 - sum q*b for IP;
// +inf for tombstoned base ids.  grid = (ceil(nb/TB), ceil(nq/TQ)), 256 threads.
__global__ __launch_bounds__(256) void distance_tile_kernel(const float* __restrict__ queries,
                                                           const float* __restrict__ base, int nq,
                                                           int64_t nb, int dim, int metric,
                                                           const uint32_t* __restrict__ deleted,
                                                           int64_t base_id0, float* __restrict__ D,
                                                           int64_t ldD) {
    __shared__ float sq2[2][KC][TQ + 4];
    __shared__ float sb2[2][KC][TB + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;  // thread (ty, tx) owns queries ty*8.. and base tx*8..
    const int64_t b0 = (int64_t)blockIdx.x * TB;
    const int q0 = blockIdx.y * TQ;
    float acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = 0.0f;

    // staging: 128 rows x KC dims per operand = 32*KC float4, KC/8 per thread: thread t loads row t/2, dims
    // (t&1)*4 + 8*u
    constexpr int NL = KC / 8;
    const int lrow = tid >> 1, lk = (tid & 1) * 4;
    float4 vq[NL], vb[NL];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int u = 0; u < NL; ++u) {
            vq[u] = make_float4(0, 0, 0, 0), vb[u] = make_float4(0, 0, 0, 0);
            const int kd = k0 + lk + 8 * u;
            if (kd < dim) {
                if (q0 + lrow < nq) vq[u] = *reinterpret_cast<const float4*>(queries + (size_t)(q0 + lrow) * dim + kd);
                if (b0 + lrow < nb) vb[u] = *reinterpret_cast<const float4*>(base + (size_t)(b0 + lrow) * dim + kd);
            }
        }
    };
    // two staging buffers, one barrier per stage: while a stage is consumed the next one is fetched into registers
    // and parked in the other buffer
    auto park = [&](int buf) {
#pragma unroll
        for (int u = 0; u < NL; ++u) {
            const int r = lk + 8 * u;
            sq2[buf][r + 0][lrow] = vq[u].x, sq2[buf][r + 1][lrow] = vq[u].y, sq2[buf][r + 2][lrow] = vq[u].z, sq2[buf][r + 3][lrow] = vq[u].w;
            sb2[buf][r + 0][lrow] = vb[u].x, sb2[buf][r + 1][lrow] = vb[u].y, sb2[buf][r + 2][lrow] = vb[u].z, sb2[buf][r + 3][lrow] = vb[u].w;
        }
    };
    auto consume = [&](int buf, int kk) {
        float a[8], b[8];
        const float4 a0 = *reinterpret_cast<const float4*>(&sq2[buf][kk][ty * 8]);
        const float4 a1 = *reinterpret_cast<const float4*>(&sq2[buf][kk][ty * 8 + 4]);
        const float4 c0 = *reinterpret_cast<const float4*>(&sb2[buf][kk][tx * 8]);
        const float4 c1 = *reinterpret_cast<const float4*>(&sb2[buf][kk][tx * 8 + 4]);
        a[0] = a0.x, a[1] = a0.y, a[2] = a0.z, a[3] = a0.w, a[4] = a1.x, a[5] = a1.y, a[6] = a1.z, a[7] = a1.w;
        b[0] = c0.x, b[1] = c0.y, b[2] = c0.z, b[3] = c0.w, b[4] = c1.x, b[5] = c1.y, b[6] = c1.z, b[7] = c1.w;
        if (metric == 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float t = a[i] - b[j];
                    acc[i][j] = __fmaf_rn(t, t, acc[i][j]);
                }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[i][j] = __fmaf_rn(a[i], b[j], acc[i][j]);
        }
    };
    fetch(0);
    park(0);
    __syncthreads();
    int cur = 0;
    for (int k0 = 0; k0 < dim; k0 += KC) {
        const bool more = k0 + KC < dim;
        if (more) fetch(k0 + KC);
        if (dim - k0 >= KC) {
#pragma unroll
            for (int kk = 0; kk < KC; ++kk) consume(cur, kk);
        } else {
            for (int kk = 0; kk < dim - k0; ++kk) consume(cur, kk);
        }
        if (more) park(cur ^ 1);
        __syncthreads();
        cur ^= 1;
    }
    const float inf = __int_as_float(0x7f800000);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int q = q0 + ty * 8 + i;
        if (q >= nq) continue;
        float out[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t b = b0 + tx * 8 + j;
            float s = metric == 0 ? acc[i][j] : 0.0f - acc[i][j];
            if (b < nb && deleted) {
                const int64_t id = base_id0 + b;
                if ((deleted[id >> 5] >> (id & 31)) & 1u) s = inf;
            }
            out[j] = s;
        }
        float* dst = D + (size_t)(q - q0 + (int64_t)blockIdx.y * TQ) * ldD + b0 + tx * 8;
        if (b0 + tx * 8 + 7 < nb && (((uintptr_t)dst) & 15) == 0) {
            *reinterpret_cast<float4*>(dst) = make_float4(out[0], out[1], out[2], out[3]);
            *reinterpret_cast<float4*>(dst + 4) = make_float4(out[4], out[5], out[6], out[7]);
        } else {
            for (int j = 0; j < 8; ++j)
                if (b0 + tx * 8 + j < nb) dst[j] = out[j];
        }
    }
}

// One workgroup per row of n floats: the k smallest under (value, index), sorted, as
// keys ord32(value) << 32 | (id0 + index).  Fewer than k finite entries: padded with ~0.
// Entries equal to +inf (tombstones) never win over finite ones and are dropped at the end.
//
// row_select_kernel is the fast path.  Every thread keeps the smallest value of the entries it reads; the k-th
// smallest of those 1024 minima is a value that at least k entries of the row do not exceed (the minima are
// distinct entries), and in a row of independent values hardly more than k do (about k + k^2/2048).  A second pass
// collects the entries up to that value into LDS, a sort by (value, index) finishes.  Two coalesced reads of the
// row, no atomics on the way.  A row with so many ties at the threshold that the candidates outgrow LDS is
// flagged and left to row_select_radix_kernel, which makes no such assumption.
constexpr int kSelThreads = 1024;
constexpr int kSelCap = 4096;  // candidate keys in LDS

__global__ __launch_bounds__(kSelThreads) void row_select_kernel(const float* __restrict__ D, int64_t ldD, int64_t n,
                                                                 int k, int64_t id0,
                                                                 unsigned long long* __restrict__ out,
                                                                 int64_t out_stride, int* __restrict__ redo) {
    __shared__ unsigned long long skeys[kSelCap];
    __shared__ uint32_t smin[kSelThreads];
    __shared__ unsigned int s_count;
    const int tid = threadIdx.x;
    const float* row = D + (size_t)blockIdx.x * ldD;
    const int kk = (int)min((int64_t)k, n);
    const int64_t n4 = n >> 2;
    const float4* row4 = reinterpret_cast<const float4*>(row);  // rows start 16-byte aligned (ldD % 4 == 0)
    // pass 1: per-thread minimum
    uint32_t m = 0xffffffffu;
    for (int64_t i = tid; i < n4; i += 2 * kSelThreads) {
        const float4 v0 = row4[i];
        const float4 v1 = i + kSelThreads < n4 ? row4[i + kSelThreads] : v0;
        m = min(m, min(min(bf_ord32(v0.x), bf_ord32(v0.y)), min(bf_ord32(v0.z), bf_ord32(v0.w))));
        m = min(m, min(min(bf_ord32(v1.x), bf_ord32(v1.y)), min(bf_ord32(v1.z), bf_ord32(v1.w))));
    }
    for (int64_t i = (n4 << 2) + tid; i < n; i += kSelThreads) m = min(m, bf_ord32(row[i]));
    smin[tid] = m;
    if (tid == 0) s_count = 0u;
    __syncthreads();
    // the kk-th smallest of the minima: bitonic sort of 1024 values
    for (int k2 = 2; k2 <= kSelThreads; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            if (tid < kSelThreads / 2) {
                const int i = 2 * tid - (tid & (j - 1)), x = i + j;
                const bool asc = (i & k2) == 0;
                const uint32_t a = smin[i], b = smin[x];
                if ((a > b) == asc) smin[i] = b, smin[x] = a;
            }
            __syncthreads();
        }
    const uint32_t thr = kk <= kSelThreads ? smin[kk - 1] : 0xffffffffu;
    // pass 2: everything up to the threshold
    for (int64_t i0 = 0; i0 < n4; i0 += kSelThreads) {
        const int64_t i = i0 + tid;
        float4 v = make_float4(0, 0, 0, 0);
        bool hit = false;
        uint32_t o[4] = {0, 0, 0, 0};
        if (i < n4) {
            v = row4[i];
            o[0] = bf_ord32(v.x), o[1] = bf_ord32(v.y), o[2] = bf_ord32(v.z), o[3] = bf_ord32(v.w);
            hit = o[0] <= thr || o[1] <= thr || o[2] <= thr || o[3] <= thr;
        }
        if (__ballot(hit) == 0ull) continue;  // uniform in the wavefront
        if (hit) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (o[j] <= thr) {
                    const unsigned pos = atomicAdd(&s_count, 1u);
                    if (pos < (unsigned)kSelCap)
                        skeys[pos] = ((unsigned long long)o[j] << 32) | (unsigned long long)(uint32_t)(id0 + 4 * i + j);
                }
        }
    }
    for (int64_t i = (n4 << 2) + tid; i < n; i += kSelThreads) {
        const uint32_t o = bf_ord32(row[i]);
        if (o <= thr) {
            const unsigned pos = atomicAdd(&s_count, 1u);
            if (pos < (unsigned)kSelCap) skeys[pos] = ((unsigned long long)o << 32) | (unsigned long long)(uint32_t)(id0 + i);
        }
    }
    __syncthreads();
    const unsigned count = s_count;
    if (count > (unsigned)kSelCap) {  // too many ties at the threshold: the radix kernel takes this row
        if (tid == 0) redo[blockIdx.x] = 1;
        return;
    }
    if (tid == 0) redo[blockIdx.x] = 0;
    int P = 2;
    while (P < (int)count) P <<= 1;
    for (int i = (int)count + tid; i < P; i += kSelThreads) skeys[i] = ~0ull;
    __syncthreads();
    for (int k2 = 2; k2 <= P; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            for (int t = tid; t < (P >> 1); t += kSelThreads) {
                const int i = 2 * t - (t & (j - 1)), x = i + j;
                const bool asc = (i & k2) == 0;
                const unsigned long long ka = skeys[i], kb = skeys[x];
                if ((ka > kb) == asc) skeys[i] = kb, skeys[x] = ka;
            }
            __syncthreads();
        }
    unsigned long long* dst = out + (size_t)blockIdx.x * out_stride;
    for (int i = tid; i < k; i += kSelThreads) {
        unsigned long long key = i < kk ? skeys[i] : ~0ull;
        if ((uint32_t)(key >> 32) == bf_ord32(__int_as_float(0x7f800000))) key = ~0ull;  // tombstoned
        dst[i] = key;
    }
}

// One workgroup per query: the k smallest of the cnt[q] keys in lists[q * cap ...] (distinct: every key carries its
// id), sorted, into out.  The scheme of row_select_kernel on keys: the k-th smallest of the per-thread minima bounds
// the k-th smallest key from above, a second pass collects what lies up to it, a sort finishes.  *overflow is raised
// when a list lost entries (cnt[q] > cap) or the collection outgrows LDS; the caller then takes another path.
__global__ __launch_bounds__(kSelThreads) void list_select_kernel(const unsigned long long* __restrict__ lists,
                                                                  int64_t cap, const unsigned int* __restrict__ cnt,
                                                                  int k, unsigned long long* __restrict__ out,
                                                                  int64_t out_stride, int* __restrict__ overflow) {
    __shared__ unsigned long long skeys[kSelCap];
    __shared__ unsigned long long smin[kSelThreads];
    __shared__ unsigned int s_count;
    const int tid = threadIdx.x;
    const unsigned int have = cnt[blockIdx.x];
    if (have > (unsigned)cap) {
        if (tid == 0) atomicAdd(overflow, 1);
        return;
    }
    const int n = (int)have;
    const unsigned long long* list = lists + (size_t)blockIdx.x * cap;
    const int kk = min(k, n);
    unsigned long long m = ~0ull;
    for (int i = tid; i < n; i += kSelThreads) m = min(m, list[i]);
    smin[tid] = m;
    if (tid == 0) s_count = 0u;
    __syncthreads();
    for (int k2 = 2; k2 <= kSelThreads; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            if (tid < kSelThreads / 2) {
                const int i = 2 * tid - (tid & (j - 1)), x = i + j;
                const bool asc = (i & k2) == 0;
                const unsigned long long a = smin[i], b = smin[x];
                if ((a > b) == asc) smin[i] = b, smin[x] = a;
            }
            __syncthreads();
        }
    const unsigned long long thr = kk > 0 ? smin[kk - 1] : 0ull;  // k <= kSelThreads (launcher)
    for (int i = tid; i < n; i += kSelThreads) {
        const unsigned long long key = list[i];
        if (kk > 0 && key <= thr) {
            const unsigned pos = atomicAdd(&s_count, 1u);
            if (pos < (unsigned)kSelCap) skeys[pos] = key;
        }
    }
    __syncthreads();
    const unsigned count = s_count;
    if (count > (unsigned)kSelCap) {
        if (tid == 0) atomicAdd(overflow, 1);
        return;
    }
    int P = 2;
    while (P < (int)count) P <<= 1;
    for (int i = (int)count + tid; i < P; i += kSelThreads) skeys[i] = ~0ull;
    __syncthreads();
    for (int k2 = 2; k2 <= P; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            for (int t = tid; t < (P >> 1); t += kSelThreads) {
                const int i = 2 * t - (t & (j - 1)), x = i + j;
                const bool asc = (i & k2) == 0;
                const unsigned long long ka = skeys[i], kb = skeys[x];
                if ((ka > kb) == asc) skeys[i] = kb, skeys[x] = ka;
            }
            __syncthreads();
        }
    unsigned long long* dst = out + (size_t)blockIdx.x * out_stride;
    for (int i = tid; i < k; i += kSelThreads) {
        unsigned long long key = i < kk ? skeys[i] : ~0ull;
        if ((uint32_t)(key >> 32) == bf_ord32(__int_as_float(0x7f800000))) key = ~0ull;  // tombstoned
        dst[i] = key;
    }
}

// The general path: exact k-th smallest by an 8-bit radix select, then ordered compaction.  Only rows flagged in
// redo (or all rows when redo is null) are processed.
__global__ __launch_bounds__(256) void row_select_radix_kernel(const float* __restrict__ D, int64_t ldD,
                                                               int64_t n, int k, int64_t id0,
                                                               unsigned long long* __restrict__ out,
                                                               int64_t out_stride, const int* __restrict__ redo) {
    extern __shared__ unsigned long long skeys[];  // pow2 >= k keys
    __shared__ unsigned int hist[256];
    __shared__ unsigned int s_prefix, s_need, s_count, s_base;
    const int tid = threadIdx.x;
    if (redo && !redo[blockIdx.x]) return;
    const float* row = D + (size_t)blockIdx.x * ldD;
    const int kk = (int)min((int64_t)k, n);

    // radix select: after the loop s_prefix is the bit pattern of the kk-th smallest value and
    // s_need how many entries equal to it belong to the answer
    if (tid == 0) s_prefix = 0u, s_need = (unsigned)kk;
    __syncthreads();
    for (int shift = 24; shift >= 0; shift -= 8) {
        hist[tid] = 0u;
        __syncthreads();
        const uint32_t prefix = s_prefix;
        const uint32_t himask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
        // rows start 16-byte aligned (ldD is a multiple of 4): float4 loads, two per thread in flight
        const int64_t n4 = n >> 2;
        const float4* row4 = reinterpret_cast<const float4*>(row);
        for (int64_t i = tid; i < n4; i += 512) {
            const float4 v0 = row4[i];
            const bool two = i + 256 < n4;
            const float4 v1 = two ? row4[i + 256] : v0;
            const float e[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if (j >= 4 && !two) break;
                const uint32_t o = bf_ord32(e[j]);
                if ((o & himask) == prefix) atomicAdd(&hist[(o >> shift) & 255u], 1u);
            }
        }
        for (int64_t i = (n4 << 2) + tid; i < n; i += 256) {
            const uint32_t o = bf_ord32(row[i]);
            if ((o & himask) == prefix) atomicAdd(&hist[(o >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (tid == 0) {
            unsigned need = s_need, run = 0;
            int d = 0;
            for (; d < 256; ++d) {
                if (run + hist[d] >= need) break;
                run += hist[d];
            }
            s_prefix = prefix | ((uint32_t)d << shift);
            s_need = need - run;
        }
        __syncthreads();
    }
    const uint32_t vk = s_prefix;
    const unsigned need_eq = s_need;  // entries == vk to take, lowest indices first
    // ordered compaction: everything below vk, and the first need_eq entries equal to vk
    if (tid == 0) s_count = 0u, s_base = 0u;
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6;
    __shared__ unsigned int w_eq[4];
    for (int64_t i0 = 0; i0 < n; i0 += 256) {
        // almost every stretch of the row holds no winner: look at 1024 entries at a time with
        // float4 loads and step over the stretches without any
        if ((i0 & 1023) == 0 && i0 + 1024 <= n) {
            const float4 v = reinterpret_cast<const float4*>(row + i0)[tid];
            const bool hit = bf_ord32(v.x) <= vk || bf_ord32(v.y) <= vk || bf_ord32(v.z) <= vk || bf_ord32(v.w) <= vk;
            if (!__syncthreads_or(hit)) {
                i0 += 768;  // the loop adds the last 256
                continue;
            }
        }
        const int64_t i = i0 + tid;
        uint32_t o = 0xffffffffu;
        bool lt = false, eq = false;
        if (i < n) {
            o = bf_ord32(row[i]);
            lt = o < vk, eq = o == vk;
        }
        const unsigned long long meq = __ballot(eq);
        if (lane == 0) w_eq[wave] = (unsigned)__popcll(meq);
        __syncthreads();
        unsigned eq_before = 0, eq_total = 0;
        for (int w = 0; w < 4; ++w) {
            if (w < wave) eq_before += w_eq[w];
            eq_total += w_eq[w];
        }
        const unsigned long long below = (1ull << lane) - 1ull;
        const unsigned eq_rank = s_base + eq_before + (unsigned)__popcll(meq & below);  // among equals, by index
        const bool take = lt || (eq && eq_rank < need_eq);
        // position: entries taken so far + taken before me in this tile
        const unsigned long long mtake = __ballot(take);
        __shared__ unsigned int w_take[4];
        if (lane == 0) w_take[wave] = (unsigned)__popcll(mtake);
        __syncthreads();
        unsigned take_before = 0, take_total = 0;
        for (int w = 0; w < 4; ++w) {
            if (w < wave) take_before += w_take[w];
            take_total += w_take[w];
        }
        if (take) {
            const unsigned pos = s_count + take_before + (unsigned)__popcll(mtake & below);
            skeys[pos] = ((unsigned long long)o << 32) | (unsigned long long)(uint32_t)(id0 + i);
        }
        __syncthreads();
        if (tid == 0) s_count += take_total, s_base += eq_total;
        __syncthreads();
    }
    // sort the kk winners
    int P = 2;
    while (P < kk) P <<= 1;
    for (int i = kk + tid; i < P; i += 256) skeys[i] = ~0ull;
    __syncthreads();
    for (int k2 = 2; k2 <= P; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            for (int t = tid; t < (P >> 1); t += 256) {
                const int i = 2 * t - (t & (j - 1)), x = i + j;
                const bool asc = (i & k2) == 0;
                const unsigned long long ka = skeys[i], kb = skeys[x];
                if ((ka > kb) == asc) skeys[i] = kb, skeys[x] = ka;
            }
            __syncthreads();
        }
    unsigned long long* dst = out + (size_t)blockIdx.x * out_stride;
    for (int i = tid; i < k; i += 256) {
        unsigned long long key = i < kk ? skeys[i] : ~0ull;
        if ((uint32_t)(key >> 32) == bf_ord32(__int_as_float(0x7f800000))) key = ~0ull;  // tombstoned
        dst[i] = key;
    }
}

// per query: the k smallest of nseg*k sorted-per-segment keys -> ids and values
__global__ __launch_bounds__(256) void merge_segments_kernel(const unsigned long long* __restrict__ part,
                                                             int nseg, int k, int metric,
                                                             int32_t* __restrict__ ids,
                                                             float* __restrict__ dists) {
    extern __shared__ unsigned long long skeys[];
    const int tid = threadIdx.x, total = nseg * k;
    const unsigned long long* src = part + (size_t)blockIdx.x * total;
    int P = 2;
    while (P < total) P <<= 1;
    for (int i = tid; i < P; i += 256) skeys[i] = i < total ? src[i] : ~0ull;
    __syncthreads();
    for (int k2 = 2; k2 <= P; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1) {
            for (int t = tid; t < (P >> 1); t += 256) {
                const int i = 2 * t - (t & (j - 1)), x = i + j;
                const bool asc = (i & k2) == 0;
                const unsigned long long ka = skeys[i], kb = skeys[x];
                if ((ka > kb) == asc) skeys[i] = kb, skeys[x] = ka;
            }
            __syncthreads();
        }
    for (int i = tid; i < k; i += 256) {
        const unsigned long long key = skeys[i];
        const bool none = key == ~0ull;
        ids[(size_t)blockIdx.x * k + i] = none ? -1 : (int32_t)(uint32_t)key;
        if (dists) {
            const float s = bf_unord32((uint32_t)(key >> 32));
            const float far = 3.402823466e+38f;
            dists[(size_t)blockIdx.x * k + i] = none ? (metric == 0 ? far : -far) : (metric == 0 ? s : 0.0f - s);
        }
    }
}

hipError_t launch_distance_tile(const float* queries, const float* base, int nq, int64_t nb, int dim,
                                int metric, const uint32_t* deleted, int64_t base_id0, float* D,
                                int64_t ldD, hipStream_t stream) {
    dim3 grid((unsigned)((nb + TB - 1) / TB), (unsigned)((nq + TQ - 1) / TQ));
    hipLaunchKernelGGL(distance_tile_kernel, grid, dim3(256), 0, stream, queries, base, nq, nb, dim, metric,
                       deleted, base_id0, D, ldD);
    return hipGetLastError();
}

hipError_t launch_row_select(const float* D, int64_t ldD, int nq, int64_t n, int k, int64_t id0,
                             unsigned long long* out, int64_t out_stride, int* redo, hipStream_t stream) {
    int P = 2;
    while (P < k) P <<= 1;
    const bool fast = redo != nullptr && k <= kSelThreads;
    if (fast)
        hipLaunchKernelGGL(row_select_kernel, dim3(nq), dim3(kSelThreads), 0, stream, D, ldD, n, k, id0, out, out_stride,
                           redo);
    hipLaunchKernelGGL(row_select_radix_kernel, dim3(nq), dim3(256), (size_t)P * 8, stream, D, ldD, n, k, id0, out,
                       out_stride, fast ? redo : nullptr);
    return hipGetLastError();
}

hipError_t launch_list_select(const unsigned long long* lists, int64_t cap, const unsigned int* cnt, int nq, int k,
                              unsigned long long* out, int64_t out_stride, int* overflow, hipStream_t stream) {
    if (k > kSelThreads) return hipErrorInvalidValue;
    hipLaunchKernelGGL(list_select_kernel, dim3(nq), dim3(kSelThreads), 0, stream, lists, cap, cnt, k, out, out_stride,
                       overflow);
    return hipGetLastError();
}

hipError_t launch_merge_segments(const unsigned long long* part, int nq, int nseg, int k, int metric,
                                 int32_t* ids, float* dists, hipStream_t stream) {
    int P = 2;
    while (P < nseg * k) P <<= 1;
    hipLaunchKernelGGL(merge_segments_kernel, dim3(nq), dim3(256), (size_t)P * 8, stream, part, nseg, k, metric,
                       ids, dists);
    return hipGetLastError();
}

}  // namespace coral
