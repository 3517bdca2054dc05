// search_device.h -- small device functions shared by the search kernels (beam_search.hip, best_first.hip):
// the 64-bit beam key, the order-preserving float mapping, DPP lane exchange, prefix counts, binary search.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace coral {

constexpr uint64_t kKeyMax = ~0ull;

// float -> uint32 whose unsigned order is the float order
__device__ __forceinline__ uint32_t ord32(float s) {
    const uint32_t u = __float_as_uint(s);
    return u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
}
__device__ __forceinline__ float unord32(uint32_t o) {
    const uint32_t u = (o & 0x80000000u) ? (o ^ 0x80000000u) : ~o;
    return __uint_as_float(u);
}
// key order = (signed distance, id, expanded flag)
__device__ __forceinline__ uint64_t make_key(float s, int32_t id, uint32_t flag) {
    return ((uint64_t)ord32(s) << 32) | ((uint64_t)((uint32_t)id << 1)) | flag;
}
__device__ __forceinline__ int32_t key_id(uint64_t k) { return (int32_t)((uint32_t)k >> 1); }
__device__ __forceinline__ float key_s(uint64_t k) { return unord32((uint32_t)(k >> 32)); }

// the value of x in the lane a DPP control selects (all rows and banks enabled)
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}

template <int CTRL>
__device__ __forceinline__ int dpp_mov_i(int x) {
    return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xF, 0xF, true);
}

// ---- Screening on rows in eight-bit codes (the copy byte_rows_kernel makes).  Row x is stored as codes k_i in
// [-127, 127] with x~_i = s k_i, s = max |x_i| / 127, followed by s, |x~|^2 and e >= |x - x~| (rounded up; infinite for
// rows that take no part).  The query is coded as q~_i = sq (128 h_i + l_i), bytes h_i in [-127, 127] and l_i in
// [-64, 63], sq = max |q_i| / 16256, with eq >= |q - q~|.  D = |q~ - x~|^2 = |q~|^2 + |x~|^2 - 2 sq s sum (128 h_i + l_i) k_i
// needs integer dot products only (v_dot4_i32_i8, exact), and the exact distance d = |q - x|^2 satisfies
// (sqrt(D) - e - eq)^2 <= d <= (sqrt(D) + e + eq)^2.  The computed D is within delta = 16 * 2^-24 (|q~|^2 + |x~|^2) of its
// true value (the conversion of the integer sum, the product of the scales, the two stored norms and the two final
// additions: each relative 2^-24 of a quantity no larger than |q~|^2 + |x~|^2; taken twice); both ends are widened by
// 1e-4 for the fp32 rounding of the exact distance that the bounds are compared with.

// The query in integer codes, by one whole wavefront: bytes h_i to qh8, l_i to ql8 (zero up to a multiple of 16
// dimensions); qq = |q~|^2, sq, eq (sums in double precision, eq rounded up).  A query with a component that is not
// finite, or whose largest lies outside [1e-18, 1e17], gets eq = inf: every row then goes to the exact pass.
__device__ __forceinline__ void code_query(const float* q, int dim, int lane, signed char* qh8, signed char* ql8,
                                           float& qq, float& sq, float& eq) {
    float amax = 0.0f;
    bool bad = false;
    for (int i = lane; i < dim; i += 64) {
        const float v = fabsf(q[i]);
        bad |= !(v <= 3.0e38f);
        amax = fmaxf(amax, v);
    }
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    bad = __ballot(bad) != 0ull || (amax != 0.0f && !(amax >= 1.0e-18f && amax <= 1.0e17f));
    sq = bad ? 0.0f : amax / 16256.0f;
    double se = 0.0, sx = 0.0;
    for (int i = lane; i < ((dim + 15) & ~15); i += 64) {
        const float v = i < dim ? q[i] : 0.0f;
        int code = 0;
        if (sq > 0.0f) {
            code = (int)rintf(v / sq);
            code = code > 16256 ? 16256 : (code < -16256 ? -16256 : code);
        }
        const int h = (code + 64) >> 7, l = code - 128 * h;
        qh8[i] = (signed char)h, ql8[i] = (signed char)l;
        const double qt = (double)sq * (double)code, dv = (double)v - qt;
        se += dv * dv, sx += qt * qt;
    }
    for (int off = 32; off > 0; off >>= 1) se += __shfl_xor(se, off, 64), sx += __shfl_xor(sx, off, 64);
    qq = (float)sx;
    eq = bad ? __int_as_float(0x7f800000) : (float)(sqrt(se) * 1.000001) * (1.0f + 2.0e-7f);
}

// the coded query of the lane: sixteen lanes share a row, lane gl8 of them takes the 16-byte chunks gl8 + 16 t
template <int CPL8>
struct CodedQuery {
    int h[CPL8][4], l[CPL8][4];
};
template <int CPL8>
__device__ __forceinline__ void load_coded_query(const signed char* qh8, const signed char* ql8, int nck, int gl8,
                                                 CodedQuery<CPL8>& q) {
#pragma unroll
    for (int t = 0; t < CPL8; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = gl8 + 16 * t;
            q.h[t][j] = c < nck ? reinterpret_cast<const int*>(qh8)[4 * c + j] : 0;
            q.l[t][j] = c < nck ? reinterpret_cast<const int*>(ql8)[4 * c + j] : 0;
        }
}

// Rows vid[0..U8) (-1: none) of one group of sixteen lanes, in three steps so that a caller with more rows to come can
// request the next ones before it finishes these: request (all loads back to back), dots (the integer sums, which
// wait for the loads and leave their registers free), finish (the lane that files a row gets the bounds
// lo <= d <= hi of its exact distance).  Lane gl8 < U8 of the group files row vid[gl8]; the caller hands it that id as
// myid (-1: the lane files none; lo and hi are then worthless).  A row that takes no part has lo = 0 and hi = inf; a
// NaN anywhere fails every comparison a caller makes with the bounds.
//
// Inner product (metric 1; the signed distance is -q.x): q.x = q~.x~ + q~.(x - x~) + (q - q~).x, so
// |q.x - q~.x~| <= |q~| e + eq (|x~| + e); the bound is widened by 2e-4 (|q~| + eq)(|x~| + e) for the fp32 rounding of
// the exact inner product and of the computed q~.x~ (each at most dim 2^-24 |q| |x|; rows of up to 512 floats: 6e-5;
// 6e-4 for rows of up to 2048).
template <int CPL8, int U8>
struct CodedRows {
    uint4 hb[U8][CPL8];
    float4 fig;  // s, |x~|^2, e of the row this lane files
};

// Every lane requests a chunk of every row, with no condition: a lane whose chunk lies past the codes takes the row's
// figures instead (its query codes are zero, so whatever it reads adds nothing), a row that is none takes row 0 (and
// is dropped by its lane).  One 32 x 32 -> 64 bit multiply-add per address.
template <int CPL8, int U8>
__device__ __forceinline__ void coded_rows_request(const unsigned char* vec8, uint32_t st8, int nck, int gl8,
                                                   const int (&vid)[U8], int myid, CodedRows<CPL8, U8>& r) {
#pragma unroll
    for (int u = 0; u < U8; ++u) {
        const uint4* row = reinterpret_cast<const uint4*>(vec8 + (uint64_t)(uint32_t)(vid[u] < 0 ? 0 : vid[u]) * st8);
#pragma unroll
        for (int t = 0; t < CPL8; ++t) {
            const int c = gl8 + 16 * t;
            r.hb[u][t] = row[c < nck ? c : nck];
        }
    }
    r.fig = make_float4(0, 0, 0, 0);
    if (myid >= 0) r.fig = *reinterpret_cast<const float4*>(vec8 + (uint64_t)(uint32_t)myid * st8 + (uint32_t)nck * 16u);
}

template <int CPL8, int U8>
__device__ __forceinline__ void coded_rows_dots(const CodedRows<CPL8, U8>& r, const CodedQuery<CPL8>& q, int (&acc)[U8]) {
    static_assert(CPL8 <= 4, "the combined sum 128 dh + dl fits 32 bits for rows of up to 1024 codes");
#pragma unroll
    for (int u = 0; u < U8; ++u) {
        int dh = 0, dl = 0;
#pragma unroll
        for (int t = 0; t < CPL8; ++t) {
            const int w[4] = {(int)r.hb[u][t].x, (int)r.hb[u][t].y, (int)r.hb[u][t].z, (int)r.hb[u][t].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                dh = __builtin_amdgcn_sdot4(w[j], q.h[t][j], dh, false);
                dl = __builtin_amdgcn_sdot4(w[j], q.l[t][j], dl, false);
            }
        }
        acc[u] = 128 * dh + dl;  // below 2^31 for 1024 dimensions: 1024 * 127 * 16256
    }
}

// The same for rows of more than 512 codes (CPL8 = 4 or 8 chunks per lane): the coded query would take 8 CPL8
// registers, so its chunks are read from LDS as they are used; and beyond 1024 codes 128 dh + dl no longer fits 32
// bits, so the two sums stay apart (each below 2^26) until they are floats.
template <int CPL8, int U8>
__device__ __forceinline__ void coded_rows_dots_wide(const CodedRows<CPL8, U8>& r, const signed char* qh8,
                                                     const signed char* ql8, int nck, int gl8, int (&acch)[U8],
                                                     int (&accl)[U8]) {
#pragma unroll
    for (int u = 0; u < U8; ++u) acch[u] = 0, accl[u] = 0;
#pragma unroll
    for (int t = 0; t < CPL8; ++t) {
        const int c = gl8 + 16 * t;
        int4 qh = make_int4(0, 0, 0, 0), ql = make_int4(0, 0, 0, 0);
        if (c < nck) qh = reinterpret_cast<const int4*>(qh8)[c], ql = reinterpret_cast<const int4*>(ql8)[c];
        const int hq[4] = {qh.x, qh.y, qh.z, qh.w}, lq[4] = {ql.x, ql.y, ql.z, ql.w};
#pragma unroll
        for (int u = 0; u < U8; ++u) {
            const int w[4] = {(int)r.hb[u][t].x, (int)r.hb[u][t].y, (int)r.hb[u][t].z, (int)r.hb[u][t].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acch[u] = __builtin_amdgcn_sdot4(w[j], hq[j], acch[u], false);
                accl[u] = __builtin_amdgcn_sdot4(w[j], lq[j], accl[u], false);
            }
        }
    }
}

// the sum over the sixteen lanes of a row, for the lane that files it
template <int U8>
__device__ __forceinline__ int coded_rows_reduce(int (&acc)[U8], int gl8) {
#pragma unroll
    for (int u = 0; u < U8; ++u) {
        acc[u] = acc[u] + dpp_mov_i<0xB1>(acc[u]);   // quad_perm [1,0,3,2]
        acc[u] = acc[u] + dpp_mov_i<0x4E>(acc[u]);   // quad_perm [2,3,0,1]
        acc[u] = acc[u] + dpp_mov_i<0x141>(acc[u]);  // row_half_mirror
        acc[u] = acc[u] + dpp_mov_i<0x140>(acc[u]);  // row_mirror
    }
    int mine = acc[0];
#pragma unroll
    for (int u = 1; u < U8; ++u)
        if (gl8 == u) mine = acc[u];
    return mine;
}

// bounds from the integer sum as a float; WIDE: rows of more than 512 codes (two more roundings on the way to the
// sum, and a longer exact inner product to allow for)
template <bool WIDE>
__device__ __forceinline__ void coded_bounds(float isum, const float4& fig, float qq, float sq, float eq, int metric,
                                             float& lo, float& hi) {
    if (metric == 0) {
        const float both = qq + fig.y;
        const float d8 = both - (2.0f * sq * fig.x) * isum, delta = (WIDE ? 24.0f : 16.0f) * 5.9604645e-8f * both, e = fig.z + eq;
        // (the hardware's square root, good to one unit in the last place and only trusted on normal numbers: below
        // 1e-36 the lower end takes 0 and the upper end the root of 1e-36; the 1e-4 covers the last place)
        const float under = d8 - delta, over = fmaxf(d8 + delta, 1.0e-36f);
        const float lo_root = fmaxf((under < 1.0e-36f ? 0.0f : __builtin_amdgcn_sqrtf(under)) - e, 0.0f);
        const float hi_root = __builtin_amdgcn_sqrtf(over) + e;
        lo = lo_root * lo_root * (1.0f - 1.0e-4f), hi = hi_root * hi_root * (1.0f + 1.0e-4f);
    } else {
        const float p = (sq * fig.x) * isum;  // q~.x~
        const float nq = sqrtf(qq) * (1.0f + 1.0e-6f), e = fig.z;
        const float nx = __builtin_amdgcn_sqrtf(fmaxf(fig.y, 1.0e-36f)) * (1.0f + 1.0e-6f);
        const float bound = (nq * e + eq * (nx + e) + (WIDE ? 6.0e-4f : 2.0e-4f) * (nq + eq) * (nx + e)) * (1.0f + 1.0e-5f);
        lo = (0.0f - p) - bound, hi = (0.0f - p) + bound;  // e = inf or eq = inf: lo = -inf, hi = inf (or NaN)
    }
}

template <int U8>
__device__ __forceinline__ void coded_rows_finish(int (&acc)[U8], int gl8, const float4& fig, float qq, float sq, float eq,
                                                  int metric, float& lo, float& hi) {
    const int mine = coded_rows_reduce<U8>(acc, gl8);
    coded_bounds<false>((float)mine, fig, qq, sq, eq, metric, lo, hi);
}

// the three steps in one go
template <int CPL8, int U8>
__device__ __forceinline__ void coded_rows_bounds(const unsigned char* vec8, uint32_t st8, int nck, int gl8,
                                                  const int (&vid)[U8], int myid, const CodedQuery<CPL8>& q, float qq,
                                                  float sq, float eq, int metric, float& lo, float& hi) {
    CodedRows<CPL8, U8> r;
    coded_rows_request<CPL8, U8>(vec8, st8, nck, gl8, vid, myid, r);
    int acc[U8];
    coded_rows_dots<CPL8, U8>(r, q, acc);
    coded_rows_finish<U8>(acc, gl8, r.fig, qq, sq, eq, metric, lo, hi);
}

// rows of more than 512 codes: the query's codes come from LDS (qh8, ql8)
template <int CPL8, int U8>
__device__ __forceinline__ void coded_rows_bounds_wide(const unsigned char* vec8, uint32_t st8, int nck, int gl8,
                                                       const int (&vid)[U8], int myid, const signed char* qh8,
                                                       const signed char* ql8, float qq, float sq, float eq, int metric,
                                                       float& lo, float& hi) {
    CodedRows<CPL8, U8> r;
    coded_rows_request<CPL8, U8>(vec8, st8, nck, gl8, vid, myid, r);
    int acch[U8], accl[U8];
    coded_rows_dots_wide<CPL8, U8>(r, qh8, ql8, nck, gl8, acch, accl);
    const int mh = coded_rows_reduce<U8>(acch, gl8), ml = coded_rows_reduce<U8>(accl, gl8);
    coded_bounds<true>(128.0f * (float)mh + (float)ml, r.fig, qq, sq, eq, metric, lo, hi);
}

// inclusive prefix sum over the 64 lanes: four steps inside the rows of 16 lanes, then the totals of the rows
// before (row_bcast15 into rows 1 and 3, row_bcast31 into rows 2 and 3); lanes without a source add 0
__device__ __forceinline__ int wave_inclusive_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);  // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);  // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);  // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);  // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);  // row_bcast15
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast31
    return v;
}

// number of set bits of m below the calling lane
__device__ __forceinline__ int prefix_popc(uint64_t m) {
    const uint32_t lane = threadIdx.x & 63;
    return __popcll(m & ((1ull << lane) - 1ull));
}

__device__ __forceinline__ int lower_bound_u64(const uint64_t* a, int n, uint64_t key) {
    int lo = 0, hi = n;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (a[mid] < key)
            lo = mid + 1;
        else
            hi = mid;
    }
    return lo;
}

}  // namespace coral
