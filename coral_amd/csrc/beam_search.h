// beam_search.h -- kernel argument block and host-side launchers shared by
// beam_search.hip (device code) and coral_search.cpp (the C ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace coral {

// Everything the search kernel reads, passed by value like the reference passes
// its BP block (include/uni.h:323-354).
struct SearchArgs {
    const float* vec;          // [n][dim]
    const int32_t* nbrs;       // [n][R], -1 padded
    const int32_t* start_ids;  // [M]
    const uint32_t* deleted;   // tombstone mask or nullptr
    const float* queries;      // [Q][dim]
    int32_t* ids_out;          // [Q][k]
    float* dists_out;          // [Q][k] or nullptr
    int32_t* counters;         // [2 Q][4]: per query hops, expansions, dist_evals, rounds; then, behind those of all Q
                               // queries, what each read: rows measured on the smaller copy, fp32 rows, 32-bit words
                               // of beam state moved in global memory, visited-state requests to global memory
    uint32_t* spill;           // [workgroups][spill_words] zeroed bitmaps
    int* next_qid;             // work counter, zero at launch
    int* spill_count;          // [0] queries that left LDS, [1] lists of new ids searched for repeats; zero at launch
    unsigned long long* phase_ticks;  // debug builds: 8 per-phase tick sums, else nullptr
    size_t spill_words;        // ceil(n/32)
    int64_t n;
    int32_t dim, R, M, Q, k, L;
    int32_t metric;            // 0 = L2, 1 = IP
    int32_t policy;            // 0 = rounds, 1 = best first
    int32_t slots_log2;        // LDS visited table: number of 16-bit cells
    int32_t vis_limit;         // first visits after which the table takes no more inserts
    int32_t id_bits;           // ceil(log2 n): width of the id mixing bijection
    int32_t rem_bits;          // low bits of the mixed id kept in a cell
    int32_t dmax;              // largest displacement a cell can encode (-1: table unused)
    int32_t ocap;              // LDS list of ids sent to the global bitmap (multiple of 4)
    int32_t tcap, ccap;        // LDS todo / candidate capacities (multiples of 4, ccap >= tcap)
    // Beams too long for LDS (launches of the kernel's BIG form): the two beam buffers and the list of entries to
    // expand live in global memory, beam_stride 64-bit words per workgroup ([2][Lp] keys, then Lp ids).
    uint64_t* beam_scratch;
    size_t beam_stride;
    // the visited set is a plain bitmap of the n ids in LDS (table_words 32-bit words) instead of the table of
    // 16-bit cells; no id ever goes to the bitmap in global memory then
    int32_t direct_bitmap;
    // screening: a half-precision copy of the vectors (rows stride16 bytes apart, the row's norm behind its halves), or
    // nullptr; tcap2 = entries of the list of rows it leaves for the exact pass (search_exact_list_cap(tcap), or 0 without screening)
    const unsigned char* vec16;
    size_t stride16;
    // the same screening on a copy in eight-bit codes (rows stride8 bytes apart: codes, then scale, squared norm of
    // the coded row and a bound of its distance to the row), or nullptr; taken when both are given
    const unsigned char* vec8;
    size_t stride8;
    int32_t tcap2;
    int32_t scap;              // BIG form: keys of the LDS sample of the beam that the merge searches first
    int32_t prefetch_rows;     // request a chunk's graph rows one chunk ahead (launches with one workgroup per CU)
    int32_t table_words;       // 32-bit words of LDS the visited structure takes (cells / 2, or ceil(n / 32) rounded up to 4)
    // the table of 16-bit cells in its bucket form (0 or 3): buckets of four cells, three candidate buckets per id;
    // rem_bits is then id_bits - (slots_log2 - 2), at most 14, and dmax is unused.  4: the same with the bucket picked
    // by the inserting wavefront's number instead of by load (for tests of what follows concurrent inserts of one id)
    int32_t bucket_choices;
};

// What the wavefront-per-query best-first kernel (best_first.hip) needs beyond SearchArgs.
struct BestFirstArgs {
    uint8_t* visited;   // [slots][stride]: the epoch of the query that last visited the node, 0 = never
    uint32_t* epochs;   // [slots]: last epoch used by the slot (kept across launches)
    size_t stride;      // bytes per slot, a multiple of 16: n, or 4 * ceil(n / 24) when packed
    int32_t slots;      // wavefronts = queries in flight
    int32_t rows_in_flight;  // 8, 16 or 32: float4 registers of vector data a lane requests before it adds them up
    int32_t rows_unique;     // no graph row lists an id twice (checked by launch_find_repeated_ids)
    int32_t packed;          // visited is [slots][stride] of 32-bit words, 8 bits of epoch over 24 node flags each
    int32_t bloom_log2;      // log2 of the bits of the per-wavefront Bloom filter in LDS, 0 = none
    // first level of the visited set: an exact table of 2^table_log2 16-bit cells per wavefront in LDS (0 = none) in
    // buckets of four; rem_bits = the bits of the mixed id (id_bits wide) that a cell stores, at most 14; what
    // finds its two buckets full goes to the state in HBM
    int32_t table_log2, id_bits, rem_bits;
    // screening: the half-precision copy of the vectors, or the copy in eight-bit codes (see SearchArgs); one of them
    // or neither.  coded_bytes: LDS a wavefront keeps for its query in integer codes (with vec8; else 0)
    const unsigned char* vec16;
    size_t stride16;
    const unsigned char* vec8;
    size_t stride8;
    int32_t coded_bytes;
};

// LDS bytes of one wavefront: a beam of L keys, 32 candidate keys, two lists of 32 ids, L byte counters, a Bloom filter of
// 2^bloom_log2 bits over the visited ids in HBM (bloom_log2 = 0: none) and a table of 2^table_log2 16-bit cells
// (table_log2 = 0: none)
__host__ __device__ inline size_t best_first_wave_lds_bytes(int L, int bloom_log2, int table_log2 = 0, int coded_bytes = 0) {
    const size_t bloom = bloom_log2 ? ((size_t)1 << bloom_log2) / 8 : 0;
    const size_t table = table_log2 ? (size_t)2 << table_log2 : 0;
    return ((size_t)((L + 3) & ~3) * 9 + 32 * 8 + 2 * 32 * 4 + bloom + table + (size_t)coded_bytes + 15) & ~(size_t)15;
}
// LDS of a wavefront's query in integer codes for the screening on eight-bit rows: two bytes per dimension
__host__ __device__ inline int coded_query_bytes(int dim) { return 2 * ((dim + 15) & ~15); }
// the filter size for a beam of L: 128 bits per beam entry rounded up to a power of two, halved while that would leave
// a CU fewer than sixteen wavefronts; none below 4096 bits
__host__ inline int best_first_bloom_log2(int L, int coded_bytes = 0) {
    int lg = 12;
    while (((size_t)1 << lg) < (size_t)128 * L && lg < 17) ++lg;
    while (lg >= 12 && best_first_wave_lds_bytes(L, lg, 0, coded_bytes) > (size_t)10 * 1024) --lg;
    return lg >= 12 ? lg : 0;
}
// screen: 0 none, 1 rows are first measured in half precision, 2 in eight-bit codes (rows of up to 512 floats)
hipError_t best_first_prepare(int dim, int L, int rows_in_flight, bool packed, int screen, int bloom_log2,
                              int table_log2, int* max_wg_per_cu);
hipError_t launch_best_first(const SearchArgs& a, const BestFirstArgs& b, hipStream_t stream);
// *flag (a device word, zero before) becomes nonzero if a row of nbrs [n][R] holds the same id twice
hipError_t launch_find_repeated_ids(const int32_t* nbrs, int64_t n, int R, uint32_t* flag, hipStream_t stream);

constexpr int kBeamSampleKeys = 512;  // LDS sample of a beam in global memory (4 KB)

// LDS bytes of one workgroup.  big: the beams and the expand list are in global memory, LDS holds the candidate
// buffer, the visited structure (table_words 32-bit words), the todo list, the overflow list and the query.
// What the wavefront-per-query best-first kernel for long beams (best_first_long.hip) needs beyond SearchArgs: the
// visited state of BestFirstArgs, and per query slot two buffers of Lp keys in global memory for the long sorted run.
struct BestFirstLongArgs {
    uint8_t* visited;    // [slots][stride], as BestFirstArgs
    uint32_t* epochs;    // [slots]
    size_t stride;
    uint64_t* beams;     // [slots][beam_stride]: two runs of Lp keys each
    size_t beam_stride;  // 64-bit words per slot
    int32_t slots;
    int32_t rows_unique;
    int32_t packed;
    int32_t bcap;        // keys of the sorted insert buffer in LDS, a multiple of 64
    int32_t scap;        // keys of the LDS sample of the long run
    int32_t sshift;      // the sample holds every 2^sshift-th key: ((L - 1) >> sshift) + 1 <= scap
    // screening: the copy of the vectors in eight-bit codes (see SearchArgs), or nullptr; coded_bytes: LDS a wavefront
    // keeps for its query in integer codes and the list the screening leaves (with vec8; else 0)
    const unsigned char* vec8;
    size_t stride8;
    int32_t coded_bytes;
};
// LDS bytes of one wavefront: the insert buffer, a copy of the long run's last bcap + 32 keys, two samples, 32 candidate
// keys, 32 ids, bcap byte counters
__host__ __device__ inline size_t best_first_long_lds_bytes(int bcap, int scap, int coded_bytes = 0) {
    return ((size_t)bcap * 8 + (size_t)(bcap + 32) * 8 + (size_t)scap * 16 + 32 * 8 + 32 * 4 + (size_t)bcap +
            (size_t)coded_bytes + 15) & ~(size_t)15;
}
// with screening on eight-bit codes: the coded query and a second list of 32 ids
__host__ __device__ inline int best_first_long_coded_bytes(int dim) { return coded_query_bytes(dim) + 32 * 4; }
hipError_t best_first_long_prepare(int dim, bool packed, bool screen, int bcap, int scap, int* max_wg_per_cu);
hipError_t launch_best_first_long(const SearchArgs& a, const BestFirstLongArgs& b, hipStream_t stream);

// entries of the list of rows a screening leaves for the exact pass, beside a todo list of tcap
constexpr int search_exact_list_cap(int tcap) { return tcap < 1024 ? tcap : 1024; }
size_t search_lds_bytes(int L, int dim, int table_words, int tcap, int ccap, int ocap, bool big, bool screening);
// the half-precision copy of the vectors that the screening phase reads: bytes per row, and its construction
size_t half_row_stride(int dim);
// the copy in eight-bit codes (a row's chunks of sixteen codes are read by sixteen lanes: up to two each for rows of
// up to 512 floats, four or eight for longer ones)
size_t byte_row_stride(int dim);
hipError_t launch_byte_rows(const float* vec, int64_t n, int dim, unsigned char* out, hipStream_t stream);
constexpr int kMaxByteRowDim = 512;         // ... in the wavefront-per-query best-first kernels
constexpr int kMaxByteRowDimRounds = 2048;  // ... in the workgroup-per-query kernel (rounds policy)
hipError_t launch_half_rows(const float* vec, int64_t n, int dim, unsigned char* out, hipStream_t stream);
// 64-bit words of global scratch one workgroup of a BIG launch needs for a beam of capacity L
size_t search_beam_stride(int L);
hipError_t search_kernel_prepare(int dim, bool big, size_t lds_bytes, int threads, int* max_wg_per_cu);
hipError_t launch_search(const SearchArgs& a, bool big, int workgroups, int threads, size_t lds_bytes,
                         hipStream_t stream);

// A fixed block of device memory inside the library's code object (no allocation call ever made for it): the
// scratch of the entry point that must not allocate.  Layout: 256 bytes of scalars, kStaticMaxQ x 8 per-query
// counters, kStaticSpillWords words of per-workgroup overflow bitmaps.  static_scratch_init(device) looks the
// block's address up once per device (that device must be current) and static_scratch(device) returns it, or
// nullptr before that.
constexpr int kStaticMaxQ = 16384;
constexpr size_t kStaticSpillWords = (size_t)8 << 20;  // 32 MiB
constexpr int64_t kStaticMaxN = (int64_t)1 << 22;      // leaves at least 64 workgroups a bitmap each
constexpr size_t kStaticScratchBytes = 256 + (size_t)kStaticMaxQ * 32 + kStaticSpillWords * 4;
hipError_t static_scratch_init(int device);
void* static_scratch(int device);
hipError_t launch_verify(const int32_t* res, const int32_t* gt, unsigned long long* hit, int Q, int k,
                         hipStream_t stream);
hipError_t launch_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t stream);

}  // namespace coral
