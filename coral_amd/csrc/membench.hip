// membench.hip -- what this GPU's memory delivers, measured with two plain kernels, so that the search kernels'
// achieved rates can be set against something the machine actually does and not only against the 8 TB/s of the
// data sheet:
//   stream: every byte of a large buffer read once, 16 bytes per lane per request, fully coalesced;
//   gather: rows of row_bytes read from pseudo-random places of the buffer, a group of lanes per row -- the access
//           pattern of the search kernels' distance phase (an 800-byte vector row per visited node) with nothing
//           else going on and no reuse for any cache to find (the buffer is far larger than L2 and the memory-side cache).
// No counterpart in the reference.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "coral_search.h"
#include "error.h"
#include "index_internal.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* __restrict__ p, size_t n16, uint32_t* sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t acc = 0;
    // eight independent 16-byte requests per lane in flight
    for (; i + 7 * stride < n16; i += 8 * stride) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) {
        const u32x4 v = __builtin_nontemporal_load(p + i);
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9E3779B9u) *sink = acc;  // keeps the loads alive; the buffer holds no such pattern
}

// A group of LPG lanes per row (16, 32 or 64: the smallest that covers the row with 16 bytes per lane, as the search
// kernels read their rows), eight rows in flight per group; rows chosen by a hash of the row counter
template <int LPG>
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint4* __restrict__ p, size_t rows_in_buffer,
                                                          int row16, size_t rows_to_read, uint32_t seed, uint32_t* sink) {
    const int lig = threadIdx.x % LPG;
    const size_t grp = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) / LPG;
    const size_t ngrp = ((size_t)gridDim.x * blockDim.x) / LPG;
    uint32_t acc = 0;
    for (size_t r = grp * 8; r < rows_to_read; r += ngrp * 8) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            uint64_t h = (r + u + seed) * 0x9E3779B97F4A7C15ull;
            h ^= h >> 29;
            h *= 0xBF58476D1CE4E5B9ull;
            h ^= h >> 32;
            const size_t row = (size_t)(h % rows_in_buffer);
            v[u] = lig < row16 ? p[row * row16 + lig] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (acc == 0x9E3779B9u) *sink = acc;
}

__global__ void fill_pattern_kernel(uint32_t* p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        p[i] = (uint32_t)i * 2654435761u | 1u;
}

}  // namespace

extern "C" int coral_membench(int32_t device, size_t bytes, int32_t row_bytes, int32_t reps, double* stream_gbps,
                              double* gather_gbps) {
    using coral::fail;
    if (bytes < ((size_t)1 << 20) || reps <= 0 || row_bytes <= 0 || row_bytes % 16 != 0 || row_bytes > 1024)
        return fail(CORAL_ERR_ARG, "bytes >= 1 MiB, reps > 0, row_bytes a multiple of 16 up to 1024");
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    void* buf = nullptr;
    uint32_t* sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = CORAL_OK;
#define MB_TRY(expr)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (expr);                                                                       \
        if (e_ != hipSuccess && rc == CORAL_OK)                                                       \
            rc = fail(e_ == hipErrorOutOfMemory ? CORAL_ERR_MEMORY : CORAL_ERR_DEVICE, "%s failed: %s", #expr, \
                      hipGetErrorString(e_));                                                         \
    } while (0)
    MB_TRY(hipMalloc(&buf, bytes));
    MB_TRY(hipMalloc(&sink, 256));
    MB_TRY(hipEventCreate(&e0));
    MB_TRY(hipEventCreate(&e1));
    if (rc == CORAL_OK) {
        const int grid = prop.multiProcessorCount * 8;
        hipLaunchKernelGGL(fill_pattern_kernel, dim3(grid), dim3(256), 0, 0, (uint32_t*)buf, bytes / 4);
        const size_t n16 = bytes / 16;
        const int row16 = row_bytes / 16;
        const size_t rows_in_buffer = n16 / row16, rows_to_read = rows_in_buffer;  // as many bytes as the stream pass
        for (int which = 0; which < 2 && rc == CORAL_OK; ++which) {
            float best_ms = 0.f;
            for (int r = 0; r < reps + 1 && rc == CORAL_OK; ++r) {  // the first pass warms up
                MB_TRY(hipEventRecord(e0, 0));
                if (which == 0)
                    hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(256), 0, 0, (const u32x4*)buf, n16, sink);
                else if (row16 <= 16)
                    hipLaunchKernelGGL(gather_rows_kernel<16>, dim3(grid), dim3(256), 0, 0, (const uint4*)buf, rows_in_buffer,
                                       row16, rows_to_read, (uint32_t)r * 7919u, sink);
                else if (row16 <= 32)
                    hipLaunchKernelGGL(gather_rows_kernel<32>, dim3(grid), dim3(256), 0, 0, (const uint4*)buf, rows_in_buffer,
                                       row16, rows_to_read, (uint32_t)r * 7919u, sink);
                else
                    hipLaunchKernelGGL(gather_rows_kernel<64>, dim3(grid), dim3(256), 0, 0, (const uint4*)buf, rows_in_buffer,
                                       row16, rows_to_read, (uint32_t)r * 7919u, sink);
                MB_TRY(hipGetLastError());
                MB_TRY(hipEventRecord(e1, 0));
                MB_TRY(hipEventSynchronize(e1));
                float ms = 0.f;
                MB_TRY(hipEventElapsedTime(&ms, e0, e1));
                if (r > 0 && (best_ms == 0.f || ms < best_ms)) best_ms = ms;
            }
            const double moved = which == 0 ? (double)n16 * 16.0 : (double)rows_to_read * row_bytes;
            double* out = which == 0 ? stream_gbps : gather_gbps;
            if (out && best_ms > 0.f) *out = moved / (best_ms * 1e-3) / 1e9;
        }
    }
#undef MB_TRY
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(sink);
    (void)hipFree(buf);
    return rc;
}
