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
