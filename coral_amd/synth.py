"""Seeded synthetic inputs for the benchmark configurations.

Every stream is counter based: value i of stream `seed` is a pure function of
(seed, i), so any slice can be generated on its own and a CPU box and a GPU box
produce identical bytes.  Uniforms come from SplitMix64, normals from Box-Muller
on pairs of uniforms (float64 arithmetic, rounded to float32 at the end).
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def splitmix64(seed, idx):
    """SplitMix64 output number idx (array of uint64 counters) of stream `seed`."""
    with np.errstate(over="ignore"):
        z = (np.uint64(seed) + (idx.astype(np.uint64) + np.uint64(1)) * _GOLDEN)
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def uniform01(seed, start, count):
    """count float64 uniforms in (0,1), positions start..start+count of the stream."""
    idx = np.arange(start, start + count, dtype=np.uint64)
    bits = splitmix64(seed, idx) >> np.uint64(11)
    return (bits.astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def normal(seed, start, count):
    """count float64 standard normals, positions start..start+count of the stream.
    Normal number j uses uniforms 2*(j//2) and 2*(j//2)+1 (cos branch for even j)."""
    first = start // 2
    last = (start + count + 1) // 2
    u = uniform01(seed, 2 * first, 2 * (last - first)).reshape(-1, 2)
    r = np.sqrt(-2.0 * np.log(u[:, 0]))
    t = 2.0 * np.pi * u[:, 1]
    z = np.empty((last - first, 2), dtype=np.float64)
    z[:, 0] = r * np.cos(t)
    z[:, 1] = r * np.sin(t)
    z = z.reshape(-1)
    off = start - 2 * first
    return z[off:off + count]


def gaussian_matrix(seed, n, dim, row0=0, chunk_rows=1 << 16, out=None):
    """float32 [n][dim] of N(0,1), rows row0..row0+n of the stream."""
    if out is None:
        out = np.empty((n, dim), dtype=np.float32)
    for r in range(0, n, chunk_rows):
        m = min(chunk_rows, n - r)
        out[r:r + m] = normal(seed, (row0 + r) * dim, m * dim).reshape(m, dim)
    return out


def shifted_queries(n, dim, seed_mu, seed_s, seed_z):
    """q = mu + s * z with mu ~ N(0, 0.5^2 I), s ~ U[0.5, 1.5] per dim, z ~ N(0, I):
    a shifted, anisotropic query law (the modality gap of the configurations)."""
    mu = 0.5 * normal(seed_mu, 0, dim)
    s = 0.5 + uniform01(seed_s, 0, dim)
    z = normal(seed_z, 0, n * dim).reshape(n, dim)
    return (mu[None, :] + s[None, :] * z).astype(np.float32)


def normalize_rows(x):
    """Row-wise L2 normalisation with the arithmetic of the reference loader
    (src/uni.cpp:38-54): float32 running sum, inv = 1/sqrt, multiply; zero rows stay."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    n2 = np.zeros(x.shape[0], dtype=np.float32)
    for j in range(x.shape[1]):
        n2 = (n2 + x[:, j] * x[:, j]).astype(np.float32)
    norm = np.sqrt(n2).astype(np.float32)
    inv = np.where(norm > 0, (np.float32(1.0) / np.where(norm > 0, norm, 1)).astype(np.float32), np.float32(1.0))
    return (x * inv[:, None]).astype(np.float32)


def cone_queries(n, dim, seed_v, seed_z):
    """normalise(v + 0.6 z), v = 1.5 * unit(N(0,I)): the text/image cone gap."""
    v = normal(seed_v, 0, dim)
    v = 1.5 * v / np.sqrt((v * v).sum())
    z = normal(seed_z, 0, n * dim).reshape(n, dim)
    return normalize_rows((v[None, :] + 0.6 * z).astype(np.float32))


def tombstone_mask(n, seed, modulo=10):
    """uint32 words, bit (id&31) of word id>>5 set iff splitmix64(seed, id) % modulo == 0."""
    words = np.zeros((n + 31) // 32, dtype=np.uint32)
    step = 1 << 22
    for s in range(0, n, step):
        ids = np.arange(s, min(n, s + step), dtype=np.uint64)
        dead = (splitmix64(seed, ids) % np.uint64(modulo)) == 0
        d = ids[dead].astype(np.int64)
        np.bitwise_or.at(words, d >> 5, (np.uint32(1) << (d & 31).astype(np.uint32)))
    return words


def exact_knn_graph(base, R=32, metric="l2", block=2048, device=None):
    """Exact R-nearest-neighbour graph (self excluded, ties by id): int32 [n][R].
    Plain brute force; on a GPU box pass device="cuda" to run the matmuls in torch
    (data plumbing for the benchmark, not part of the search path)."""
    n, dim = base.shape
    out = np.empty((n, R), dtype=np.int32)
    if device is not None:
        import torch
        xb = torch.from_numpy(base).to(device)
        nb = (xb * xb).sum(1)
        for s in range(0, n, block):
            xq = xb[s:s + block]
            ip = xq @ xb.T
            d = (nb[None, :] - 2.0 * ip) if metric == "l2" else -ip
            rows = torch.arange(xq.shape[0], device=device)
            d[rows, rows + s] = float("inf")
            idx = torch.topk(d, R, dim=1, largest=False, sorted=True).indices
            out[s:s + block] = idx.to(torch.int32).cpu().numpy()
        return out
    nb = (base.astype(np.float64) ** 2).sum(1)
    for s in range(0, n, block):
        xq = base[s:s + block]
        ip = xq.astype(np.float64) @ base.T.astype(np.float64)
        d = (nb[None, :] - 2.0 * ip) if metric == "l2" else -ip
        d[np.arange(xq.shape[0]), np.arange(xq.shape[0]) + s] = np.inf
        part = np.argpartition(d, R, axis=1)[:, :R]
        pd = np.take_along_axis(d, part, axis=1)
        order = np.lexsort((part, pd), axis=1)
        out[s:s + block] = np.take_along_axis(part, order, axis=1).astype(np.int32)
    return out


def medoid_start(base):
    """Index of the base vector nearest the mean (the single entry point of config 1)."""
    mean = base.mean(axis=0, dtype=np.float64)
    d = ((base.astype(np.float64) - mean[None, :]) ** 2).sum(1)
    return int(np.argmin(d))


def block_graph(base, R=32, block=4096, long_links=8, seed=7, device="cuda"):
    """A cheap degree-R graph for very large bases where neither an exact kNN graph
    nor the query-aware builder is affordable: consecutive ids form blocks; a node
    links to its R - long_links nearest nodes inside its block and to long_links
    pseudo-random nodes anywhere (SplitMix64 of (seed, id, j)), which keeps the graph
    connected.  Rows are sorted block links first.  Test/benchmark data only."""
    import torch
    n = base.shape[0]
    near = R - long_links
    out = np.empty((n, R), dtype=np.int32)
    for s in range(0, n, block * 64):
        e = min(n, s + block * 64)
        xb = torch.from_numpy(base[s:e]).to(device)
        for b0 in range(0, e - s, block):
            x = xb[b0:b0 + block]
            m = x.shape[0]
            sq = (x * x).sum(1)
            d = sq[:, None] + sq[None, :] - 2.0 * (x @ x.T)
            d.fill_diagonal_(float("inf"))
            kk = min(near, m - 1)
            idx = torch.topk(d, kk, dim=1, largest=False, sorted=True).indices + (s + b0)
            out[s + b0:s + b0 + m, :kk] = idx.to(torch.int32).cpu().numpy()
            if kk < near:
                out[s + b0:s + b0 + m, kk:near] = -1
    ids = np.arange(n, dtype=np.uint64)
    for j in range(long_links):
        r = (splitmix64(seed + j, ids) % np.uint64(n)).astype(np.int64)
        r = np.where(r == np.arange(n), (r + 1) % n, r)
        out[:, near + j] = r.astype(np.int32)
    # a row's neighbours are its leading non-negative entries: compact rows that got -1 in the middle
    if (out[:, :near] < 0).any():
        for i in np.where((out[:, :near] < 0).any(axis=1))[0]:
            row = out[i][out[i] >= 0]
            out[i] = -1
            out[i, :row.size] = row
    return out
