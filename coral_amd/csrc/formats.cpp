// formats.cpp -- readers and writers for the reference's file formats
// (include/coral_formats.h lists each layout with its reference citation) and an
// LZ4 block codec written for this library.  Host code only.
#include "coral_formats.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "error.h"

using coral::fail;

namespace {

struct File {
    FILE* f = nullptr;
    explicit File(const char* path, const char* mode) { f = std::fopen(path, mode); }
    ~File() {
        if (f) std::fclose(f);
    }
    File(const File&) = delete;
    File& operator=(const File&) = delete;
};

int64_t file_size(const char* path) {
    struct stat st;
    if (stat(path, &st) != 0) return -1;
    return (int64_t)st.st_size;
}

// read-only mapping of a whole file (empty files map to nullptr / size 0)
struct Mapping {
    const unsigned char* p = nullptr;
    size_t size = 0;
    bool ok = false;
    explicit Mapping(const std::string& path) {
        int fd = open(path.c_str(), O_RDONLY);
        if (fd < 0) return;
        struct stat st;
        if (fstat(fd, &st) != 0) {
            close(fd);
            return;
        }
        size = (size_t)st.st_size;
        if (size == 0) {
            ok = true;
            close(fd);
            return;
        }
        void* m = mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
        close(fd);
        if (m == MAP_FAILED) return;
        p = (const unsigned char*)m;
        ok = true;
    }
    ~Mapping() {
        if (p) munmap((void*)p, size);
    }
    Mapping(const Mapping&) = delete;
    Mapping& operator=(const Mapping&) = delete;
};

// entry of graph.part<p>.idx (include/disk_graph.h:78-84)
struct NodeDiskIndex {
    uint64_t offset;
    uint32_t size;
    int32_t pos;  // 0 = .data, 1 = .append
};
static_assert(sizeof(NodeDiskIndex) == 16, "index entries are 16 bytes on disk");

constexpr int64_t kNodesPerPartitionMax = 100000000;  // CPU_N, include/uni.h:71

void partitioning(int64_t n, int64_t* count, int64_t* per) {
    *count = (n + kNodesPerPartitionMax - 1) / kNodesPerPartitionMax;
    if (*count < 1) *count = 1;
    *per = (n + *count - 1) / *count;
}

std::string part_path(const char* dir, int64_t p, const char* ext) {
    return std::string(dir) + "/graph.part" + std::to_string(p) + ext;
}

// ------------------------------------------------------------------ LZ4 block
inline uint32_t read32(const unsigned char* p) {
    uint32_t v;
    std::memcpy(&v, p, 4);
    return v;
}

int lz4_decompress(const unsigned char* src, int src_len, unsigned char* dst, int dst_cap) {
    if (src_len <= 0 || dst_cap < 0) return -1;
    const unsigned char *ip = src, *iend = src + src_len;
    unsigned char *op = dst, *oend = dst + dst_cap;
    for (;;) {
        if (ip >= iend) return -1;
        const unsigned token = *ip++;
        size_t lit = token >> 4;
        if (lit == 15) {
            unsigned s;
            do {
                if (ip >= iend) return -1;
                s = *ip++;
                lit += s;
            } while (s == 255);
        }
        if ((size_t)(iend - ip) < lit || (size_t)(oend - op) < lit) return -1;
        std::memcpy(op, ip, lit);
        ip += lit, op += lit;
        if (ip == iend) break;  // the last sequence carries literals only
        if (iend - ip < 2) return -1;
        const size_t offset = (size_t)ip[0] | ((size_t)ip[1] << 8);
        ip += 2;
        if (offset == 0 || offset > (size_t)(op - dst)) return -1;
        size_t mlen = token & 15;
        if (mlen == 15) {
            unsigned s;
            do {
                if (ip >= iend) return -1;
                s = *ip++;
                mlen += s;
            } while (s == 255);
        }
        mlen += 4;
        if ((size_t)(oend - op) < mlen) return -1;
        const unsigned char* m = op - offset;
        for (size_t i = 0; i < mlen; ++i) op[i] = m[i];  // overlapping copies are the point
        op += mlen;
    }
    return (int)(op - dst);
}

int lz4_bound(int n) { return n < 0 ? 0 : n + n / 255 + 16; }

// greedy single-pass compressor: 4-byte hash, 64 KiB window, block end rules of
// the format (last 5 bytes literal, no match starting in the last 12 bytes)
int lz4_compress(const unsigned char* src, int n, unsigned char* dst, int cap) {
    if (n < 0 || cap < lz4_bound(n)) return 0;
    unsigned char* op = dst;
    const unsigned char* anchor = src;
    auto emit = [&](const unsigned char* lit_end, size_t mlen, size_t offset, bool last) {
        const size_t lit = (size_t)(lit_end - anchor);
        unsigned char* token = op++;
        if (lit >= 15) {
            *token = 15u << 4;
            size_t r = lit - 15;
            for (; r >= 255; r -= 255) *op++ = 255;
            *op++ = (unsigned char)r;
        } else {
            *token = (unsigned char)(lit << 4);
        }
        std::memcpy(op, anchor, lit);
        op += lit;
        if (last) return;
        *op++ = (unsigned char)(offset & 255);
        *op++ = (unsigned char)(offset >> 8);
        size_t m = mlen - 4;
        if (m >= 15) {
            *token |= 15;
            m -= 15;
            for (; m >= 255; m -= 255) *op++ = 255;
            *op++ = (unsigned char)m;
        } else {
            *token |= (unsigned char)m;
        }
    };
    if (n >= 13) {
        std::vector<int32_t> table(1 << 12, -1);
        const unsigned char* ip = src;
        const unsigned char* const mflimit = src + n - 12;
        const unsigned char* const matchlimit = src + n - 5;
        while (ip < mflimit) {
            const uint32_t h = (read32(ip) * 2654435761u) >> 20;
            const int32_t cand = table[h];
            table[h] = (int32_t)(ip - src);
            if (cand >= 0 && (ip - src) - cand <= 65535 && read32(src + cand) == read32(ip)) {
                const unsigned char* m = src + cand;
                size_t len = 4;
                while (ip + len < matchlimit && ip[len] == m[len]) ++len;
                emit(ip, len, (size_t)(ip - m), false);
                ip += len;
                anchor = ip;
            } else {
                ++ip;
            }
        }
    }
    emit(src + n, 0, 0, true);
    return (int)(op - dst);
}

}  // namespace

extern "C" {

int coral_lz4_compress_bound(int src_len) { return lz4_bound(src_len); }
int coral_lz4_compress(const void* src, int src_len, void* dst, int dst_cap) {
    return lz4_compress((const unsigned char*)src, src_len, (unsigned char*)dst, dst_cap);
}
int coral_lz4_decompress(const void* src, int src_len, void* dst, int dst_cap) {
    return lz4_decompress((const unsigned char*)src, src_len, (unsigned char*)dst, dst_cap);
}

// ---------------------------------------------------------------------- fbin
int coral_fbin_read_meta(const char* path, int64_t* n, int32_t* dim) {
    if (!path || !n || !dim) return fail(CORAL_ERR_ARG, "null argument");
    File f(path, "rb");
    if (!f.f) return fail(CORAL_ERR_IO, "open file error: %s", path);
    int32_t hdr[2];
    if (std::fread(hdr, 4, 2, f.f) != 2) return fail(CORAL_ERR_IO, "%s: short header", path);
    if (hdr[0] < 0 || hdr[1] <= 0) return fail(CORAL_ERR_IO, "%s: bad header (%d, %d)", path, hdr[0], hdr[1]);
    const int64_t sz = file_size(path);
    const int64_t contained = (sz - 8) / hdr[1] / 4;
    if (hdr[0] > contained)
        return fail(CORAL_ERR_IO, "Data file size wrong! %s holds %lld points but should have %d", path,
                    (long long)contained, hdr[0]);
    *n = hdr[0], *dim = hdr[1];
    return CORAL_OK;
}

int coral_fbin_read(const char* path, float* out, int64_t n, int32_t dim, int32_t stride) {
    if (!path || !out || n < 0 || dim <= 0 || stride < dim) return fail(CORAL_ERR_ARG, "bad argument");
    File f(path, "rb");
    if (!f.f) return fail(CORAL_ERR_IO, "open file error: %s", path);
    if (std::fseek(f.f, 8, SEEK_SET) != 0) return fail(CORAL_ERR_IO, "%s: seek failed", path);
    if (stride == dim) {
        const size_t want = (size_t)n * dim;
        size_t got = 0;
        while (got < want) {  // chunked so that a single read stays below 2 GiB
            const size_t chunk = std::min(want - got, (size_t)1 << 28);
            const size_t r = std::fread(out + got, 4, chunk, f.f);
            got += r;
            if (r != chunk) break;
        }
        if (got != want) return fail(CORAL_ERR_IO, "Read file incompleted! filename: %s", path);
    } else {
        for (int64_t i = 0; i < n; ++i) {
            float* row = out + (size_t)i * stride;
            if (std::fread(row, 4, (size_t)dim, f.f) != (size_t)dim)
                return fail(CORAL_ERR_IO, "Read file incompleted! filename: %s", path);
            std::memset(row + dim, 0, (size_t)(stride - dim) * 4);
        }
    }
    return CORAL_OK;
}

int coral_fbin_write(const char* path, const float* data, int64_t n, int32_t dim) {
    if (!path || (!data && n > 0) || n < 0 || n > 0x7fffffff || dim <= 0)
        return fail(CORAL_ERR_ARG, "bad argument");
    File f(path, "wb");
    if (!f.f) return fail(CORAL_ERR_IO, "cannot create %s", path);
    const int32_t hdr[2] = {(int32_t)n, dim};
    if (std::fwrite(hdr, 4, 2, f.f) != 2) return fail(CORAL_ERR_IO, "%s: write failed", path);
    const size_t want = (size_t)n * dim;
    size_t done = 0;
    while (done < want) {
        const size_t chunk = std::min(want - done, (size_t)1 << 28);
        if (std::fwrite(data + done, 4, chunk, f.f) != chunk) return fail(CORAL_ERR_IO, "%s: write failed", path);
        done += chunk;
    }
    return CORAL_OK;
}

// ------------------------------------------------------------------------ gt
int coral_gt_read_meta(const char* path, int32_t* nq, int32_t* k) {
    if (!path || !nq || !k) return fail(CORAL_ERR_ARG, "null argument");
    File f(path, "rb");
    if (!f.f) return fail(CORAL_ERR_IO, "open file error: %s", path);
    int32_t hdr[2];
    if (std::fread(hdr, 4, 2, f.f) != 2) return fail(CORAL_ERR_IO, "%s: short header", path);
    if (hdr[0] < 0 || hdr[1] <= 0) return fail(CORAL_ERR_IO, "%s: bad header", path);
    *nq = hdr[0], *k = hdr[1];
    return CORAL_OK;
}

int coral_gt_read(const char* path, int32_t* ids, int32_t nq, int32_t k) {
    if (!path || !ids || nq < 0 || k <= 0) return fail(CORAL_ERR_ARG, "bad argument");
    File f(path, "rb");
    if (!f.f) return fail(CORAL_ERR_IO, "open file error: %s", path);
    if (std::fseek(f.f, 8, SEEK_SET) != 0) return fail(CORAL_ERR_IO, "%s: seek failed", path);
    const size_t want = (size_t)nq * k;
    if (std::fread(ids, 4, want, f.f) != want) return fail(CORAL_ERR_IO, "Read file incompleted! filename: %s", path);
    return CORAL_OK;
}

int coral_gt_write(const char* path, const int32_t* ids, int32_t nq, int32_t k) {
    if (!path || !ids || nq < 0 || k <= 0) return fail(CORAL_ERR_ARG, "bad argument");
    File f(path, "wb");
    if (!f.f) return fail(CORAL_ERR_IO, "cannot create %s", path);
    const int32_t hdr[2] = {nq, k};
    const size_t want = (size_t)nq * k;
    if (std::fwrite(hdr, 4, 2, f.f) != 2 || std::fwrite(ids, 4, want, f.f) != want)
        return fail(CORAL_ERR_IO, "%s: write failed", path);
    return CORAL_OK;
}

// ----------------------------------------------------------------- index dir
int coral_graph_dir_read(const char* dir, int64_t n, int32_t R, int32_t* nbrs, float* dists) {
    if (!dir || !nbrs || n <= 0 || R <= 0) return fail(CORAL_ERR_ARG, "bad argument");
    int64_t count, per;
    partitioning(n, &count, &per);
    for (int64_t p = 0; p < count; ++p) {
        const int64_t start = p * per;
        const int64_t cnt = std::max<int64_t>(0, std::min(per, n - start));
        const std::string idx_path = part_path(dir, p, ".idx");
        Mapping idx(idx_path), data(part_path(dir, p, ".data")), app(part_path(dir, p, ".append"));
        if (!idx.ok) return fail(CORAL_ERR_IO, "cannot open %s", idx_path.c_str());
        if (!data.ok) return fail(CORAL_ERR_IO, "cannot open %s", part_path(dir, p, ".data").c_str());
        if (idx.size < (size_t)cnt * sizeof(NodeDiskIndex))
            return fail(CORAL_ERR_IO, "%s holds %zu entries, %lld expected", idx_path.c_str(),
                        idx.size / sizeof(NodeDiskIndex), (long long)cnt);
        const NodeDiskIndex* table = (const NodeDiskIndex*)idx.p;
        std::atomic<int64_t> bad(-1);
        std::atomic<int> bad_kind(0);
#pragma omp parallel
        {
            std::vector<unsigned char> raw;
#pragma omp for schedule(static)
            for (int64_t i = 0; i < cnt; ++i) {
                int32_t* row = nbrs + (size_t)(start + i) * R;
                float* drow = dists ? dists + (size_t)(start + i) * R : nullptr;
                for (int j = 0; j < R; ++j) row[j] = -1;
                if (drow) std::memset(drow, 0, (size_t)R * 4);
                const NodeDiskIndex e = table[i];
                if (e.size == 0) continue;  // no block: degree 0 (src/disk.cpp:343-347)
                auto flag = [&](int kind) {
                    int64_t expect = -1;
                    if (bad.compare_exchange_strong(expect, start + i)) bad_kind = kind;
                };
                const Mapping& src = e.pos == 0 ? data : app;
                if (!src.ok || e.size < 8 || e.offset + e.size > src.size) {
                    flag(1);
                    continue;
                }
                const unsigned char* blk = src.p + e.offset;
                const uint32_t raw_size = read32(blk + 4);
                if (raw_size < 4 || raw_size > 4u + 8u * 64u) {
                    flag(2);
                    continue;
                }
                raw.resize(raw_size);
                const int dec = lz4_decompress(blk + 8, (int)e.size - 8, raw.data(), (int)raw_size);
                if (dec != (int)raw_size) {
                    flag(3);
                    continue;
                }
                int32_t deg;
                std::memcpy(&deg, raw.data(), 4);
                if (deg < 0 || (uint32_t)(4 + 8 * deg) != raw_size) {
                    flag(2);
                    continue;
                }
                if (deg > R) {
                    flag(4);
                    continue;
                }
                std::memcpy(row, raw.data() + 4, (size_t)deg * 4);
                if (drow) std::memcpy(drow, raw.data() + 4 + (size_t)deg * 4, (size_t)deg * 4);
            }
        }
        if (bad >= 0) {
            static const char* what[] = {"", "block outside its file", "corrupted block header",
                                         "LZ4 decompress failed", "degree exceeds max_degree"};
            return fail(CORAL_ERR_IO, "%s: node %lld: %s", dir, (long long)bad.load(), what[bad_kind.load()]);
        }
    }
    return CORAL_OK;
}

int coral_graph_dir_write(const char* dir, int64_t n, int32_t R, const int32_t* nbrs, const float* dists) {
    if (!dir || !nbrs || n <= 0 || R <= 0 || R > 64) return fail(CORAL_ERR_ARG, "bad argument");
    if (mkdir(dir, 0755) != 0 && errno != EEXIST) return fail(CORAL_ERR_IO, "cannot create directory %s", dir);
    int64_t count, per;
    partitioning(n, &count, &per);
    for (int64_t p = 0; p < count; ++p) {
        const int64_t start = p * per;
        const int64_t cnt = std::max<int64_t>(0, std::min(per, n - start));
        File fd(part_path(dir, p, ".data").c_str(), "wb"), fi(part_path(dir, p, ".idx").c_str(), "wb"),
            fa(part_path(dir, p, ".append").c_str(), "wb");
        if (!fd.f || !fi.f || !fa.f) return fail(CORAL_ERR_IO, "cannot create partition files in %s", dir);
        std::vector<NodeDiskIndex> table((size_t)cnt);
        std::vector<unsigned char> raw(4 + 8 * (size_t)R), comp(8 + (size_t)lz4_bound(4 + 8 * R));
        uint64_t off = 0;
        for (int64_t i = 0; i < cnt; ++i) {
            const int64_t id = start + i;
            const int32_t* row = nbrs + (size_t)id * R;
            int32_t deg = 0;
            while (deg < R && row[deg] >= 0) ++deg;
            if (deg == 0) {
                table[(size_t)i] = {0, 0, 0};
                continue;
            }
            const int32_t raw_size = 4 + 8 * deg;
            std::memcpy(raw.data(), &deg, 4);
            std::memcpy(raw.data() + 4, row, (size_t)deg * 4);
            if (dists)
                std::memcpy(raw.data() + 4 + (size_t)deg * 4, dists + (size_t)id * R, (size_t)deg * 4);
            else
                std::memset(raw.data() + 4 + (size_t)deg * 4, 0, (size_t)deg * 4);
            const int32_t node_id = (int32_t)id;
            std::memcpy(comp.data(), &node_id, 4);
            std::memcpy(comp.data() + 4, &raw_size, 4);
            const int csz = lz4_compress(raw.data(), raw_size, comp.data() + 8, (int)comp.size() - 8);
            if (csz <= 0) return fail(CORAL_ERR_IO, "LZ4 compression failed for node %lld", (long long)id);
            const uint32_t total = (uint32_t)csz + 8;
            if (std::fwrite(comp.data(), 1, total, fd.f) != total) return fail(CORAL_ERR_IO, "%s: write failed", dir);
            table[(size_t)i] = {off, total, 0};
            off += total;
        }
        if (cnt && std::fwrite(table.data(), sizeof(NodeDiskIndex), (size_t)cnt, fi.f) != (size_t)cnt)
            return fail(CORAL_ERR_IO, "%s: index write failed", dir);
    }
    File fb((std::string(dir) + "/graph.batch_id").c_str(), "w");
    if (!fb.f) return fail(CORAL_ERR_IO, "cannot create graph.batch_id in %s", dir);
    std::fputs("0", fb.f);
    return CORAL_OK;
}

// Graph::load_search_start_nodes (src/graph.cpp:329-351): a missing file or a
// list that ends early leaves no start ids; neither is an error there.
int coral_start_ids_read(const char* dir, int32_t* ids, int32_t capacity, int32_t* count) {
    if (!dir || !count) return fail(CORAL_ERR_ARG, "null argument");
    *count = 0;
    File f((std::string(dir) + "/graph.search_start_ids").c_str(), "r");
    if (!f.f) return CORAL_OK;
    int M = -1;
    if (std::fscanf(f.f, "%d", &M) != 1 || M <= 0) return CORAL_OK;
    if (!ids || M > capacity) return fail(CORAL_ERR_ARG, "%d start ids do not fit a buffer of %d", M, capacity);
    for (int i = 0; i < M; ++i)
        if (std::fscanf(f.f, "%d", &ids[i]) != 1) return CORAL_OK;
    *count = M;
    return CORAL_OK;
}

int coral_start_ids_write(const char* dir, const int32_t* ids, int32_t count) {
    if (!dir || (!ids && count > 0) || count < 0) return fail(CORAL_ERR_ARG, "bad argument");
    File f((std::string(dir) + "/graph.search_start_ids").c_str(), "w");
    if (!f.f) return fail(CORAL_ERR_IO, "cannot create graph.search_start_ids in %s", dir);
    std::fprintf(f.f, "%d ", count);
    for (int i = 0; i < count; ++i) std::fprintf(f.f, "%d ", ids[i]);
    return CORAL_OK;
}

// ----------------------------------------------------------------- hit counts
int coral_hits_read(const char* dir, uint32_t* hits, int64_t n) {
    if (!dir || !hits || n <= 0) return fail(CORAL_ERR_ARG, "bad argument");
    const std::string path = std::string(dir) + "/hits.bin";
    File f(path.c_str(), "rb");
    if (!f.f) return fail(CORAL_ERR_IO, "open file error: %s", path.c_str());
    int64_t stored = 0;
    if (std::fread(&stored, sizeof stored, 1, f.f) != 1) return fail(CORAL_ERR_IO, "%s: short header", path.c_str());
    if (stored < n)
        return fail(CORAL_ERR_IO, "%s holds %lld counts, the index has %lld nodes", path.c_str(), (long long)stored,
                    (long long)n);
    if (std::fread(hits, sizeof(uint32_t), (size_t)n, f.f) != (size_t)n)
        return fail(CORAL_ERR_IO, "%s: truncated", path.c_str());
    return CORAL_OK;
}

int coral_hits_write(const char* dir, const uint32_t* hits, int64_t n) {
    if (!dir || !hits || n <= 0) return fail(CORAL_ERR_ARG, "bad argument");
    const std::string path = std::string(dir) + "/hits.bin";
    File f(path.c_str(), "wb");
    if (!f.f) return fail(CORAL_ERR_IO, "cannot create %s", path.c_str());
    if (std::fwrite(&n, sizeof n, 1, f.f) != 1 || std::fwrite(hits, sizeof(uint32_t), (size_t)n, f.f) != (size_t)n)
        return fail(CORAL_ERR_IO, "%s: short write", path.c_str());
    return CORAL_OK;
}

// ----------------------------------------------------------------- RoarGraph
int coral_roargraph_read(const char* path, int64_t n, int32_t R, int32_t* nbrs, int32_t* ep) {
    if (!path || !nbrs || !ep || n <= 0 || R <= 0) return fail(CORAL_ERR_ARG, "bad argument");
    File f(path, "rb");
    if (!f.f) return fail(CORAL_ERR_IO, "open file error: %s", path);
    uint32_t hdr[2];
    if (std::fread(hdr, 4, 2, f.f) != 2) return fail(CORAL_ERR_IO, "%s: short header", path);
    if ((int64_t)hdr[1] > n) return fail(CORAL_ERR_IO, "%s holds %u nodes, index has %lld", path, hdr[1], (long long)n);
    for (size_t i = 0; i < (size_t)n * R; ++i) nbrs[i] = -1;
    std::vector<uint32_t> row;
    for (uint32_t i = 0; i < hdr[1]; ++i) {
        uint32_t deg;
        if (std::fread(&deg, 4, 1, f.f) != 1) return fail(CORAL_ERR_IO, "%s: truncated at node %u", path, i);
        row.resize(deg);
        if (deg && std::fread(row.data(), 4, deg, f.f) != deg) return fail(CORAL_ERR_IO, "%s: truncated at node %u", path, i);
        const uint32_t keep = std::min<uint32_t>(deg, (uint32_t)R);
        for (uint32_t j = 0; j < keep; ++j) nbrs[(size_t)i * R + j] = (int32_t)row[j];
    }
    *ep = (int32_t)hdr[0];
    return CORAL_OK;
}

int coral_roargraph_write(const char* path, int64_t n, int32_t R, const int32_t* nbrs, int32_t ep) {
    if (!path || !nbrs || n <= 0 || R <= 0) return fail(CORAL_ERR_ARG, "bad argument");
    File f(path, "wb");
    if (!f.f) return fail(CORAL_ERR_IO, "cannot create %s", path);
    const uint32_t hdr[2] = {(uint32_t)ep, (uint32_t)n};
    if (std::fwrite(hdr, 4, 2, f.f) != 2) return fail(CORAL_ERR_IO, "%s: write failed", path);
    for (int64_t i = 0; i < n; ++i) {
        const int32_t* row = nbrs + (size_t)i * R;
        uint32_t deg = 0;
        while (deg < (uint32_t)R && row[deg] >= 0) ++deg;
        if (std::fwrite(&deg, 4, 1, f.f) != 1 || (deg && std::fwrite(row, 4, deg, f.f) != deg))
            return fail(CORAL_ERR_IO, "%s: write failed", path);
    }
    return CORAL_OK;
}

void coral_normalize_l2(float* x, int64_t n, int64_t d) {
#pragma omp parallel for
    for (int64_t i = 0; i < n; ++i) {
        float* row = x + i * d;
        float norm2 = 0.0f;
        for (int64_t j = 0; j < d; ++j) norm2 += row[j] * row[j];
        const float norm = std::sqrt(norm2);
        if (norm > 0.0f) {
            const float inv = 1.0f / norm;
            for (int64_t j = 0; j < d; ++j) row[j] *= inv;
        }
    }
}

int64_t coral_recall_hits(int32_t q_num, int32_t k, int32_t gt_dim, const int32_t* res, const int32_t* gt) {
    int64_t total = 0;
    for (int32_t i = 0; i < q_num; ++i) {
        const int32_t* g = gt + (size_t)i * gt_dim;
        const int32_t* r = res + (size_t)i * k;
        for (int a = 0; a < k; ++a)
            if (std::find(r, r + k, g[a]) != r + k) ++total;
    }
    return total;
}

}  // extern "C"
