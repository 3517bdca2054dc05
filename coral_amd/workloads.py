"""The benchmark configurations as seeded synthetic workloads (base vectors,
queries, auxiliary queries, graph, start ids, ground truth).

Generation runs on the host (coral_amd.synth); the graphs of configurations 2 and 3
are built by the library's own construction path (coral_build_graph: the reference's
IndexGPU::BuildGPU with its config.json defaults) and ground truth comes from the
library's brute-force kernels."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np

from . import synth


def gaussian_base(seed, n, dim, threads=16):
    out = np.empty((n, dim), dtype=np.float32)
    step = 1 << 15
    with ThreadPoolExecutor(threads) as ex:
        list(ex.map(lambda r: synth.gaussian_matrix(seed, min(step, n - r), dim, row0=r, out=out[r:r + step]),
                    range(0, n, step)))
    return out


def build_query_aware_graph(base, aux, metric="l2", **params):
    """(nbrs, start_ids, info) from the library's builder with the reference's defaults (R=32, k_b=100, batch=1024,
    need_discard, connectivity enhancement, 16 entry points)."""
    from . import capi
    idx = capi.Index(base, None, None, metric=capi.IP if metric == "ip" else capi.L2)
    st = idx.build_graph(aux, capi.build_params(**params))
    nbrs, starts = idx.get_graph()
    idx.close()
    info = st.as_dict()
    info["avg_degree"] = info["edges"] / base.shape[0]
    return nbrs, starts, info


def exact_knn_graph(base, R=32, metric="l2", batch=1 << 17):
    """Exact R-nearest-neighbour graph of the base, int32 [n][R], by the library's own brute-force kernels
    (coral_bruteforce_knn, the stand-in for the reference's faiss calls, tests/comp_gt.cpp:119-176): every vector's
    R + 1 nearest under (distance, id), the vector itself dropped.  n <= R gives rows padded with -1."""
    from . import capi
    base = np.ascontiguousarray(base, dtype=np.float32)
    n = base.shape[0]
    idx = capi.Index(base, None, None, metric=capi.IP if metric == "ip" else capi.L2)
    kk = min(R + 1, n)
    out = np.full((n, R), -1, np.int32)
    for s in range(0, n, batch):
        ids, _, _ = idx.bruteforce(base[s:s + batch], kk, want_dists=False)
        own = np.arange(s, s + ids.shape[0], dtype=np.int32)[:, None]
        # the vector itself is among its R + 1 nearest (first, unless an exact duplicate with a lower id comes before
        # it); where it is not -- more than R duplicates -- the last entry goes instead
        is_self = ids == own
        is_self[~is_self.any(1), -1] = True
        keep = ids[~is_self].reshape(ids.shape[0], kk - 1)
        out[s:s + ids.shape[0], :kk - 1] = keep
    idx.close()
    return out


def config1(device="cuda"):
    """100k x 128 N(0,I); 1k shifted queries; exact 32-NN graph; entry = medoid; k=10, L=64, L2."""
    base = gaussian_base(1001, 100000, 128)
    queries = synth.shifted_queries(1000, 128, 1002, 1003, 1004)
    nbrs = exact_knn_graph(base, 32)
    starts = np.array([synth.medoid_start(base)], np.int32)
    return dict(name="100k x 128 fp32 L2, exact 32-NN graph, k=10, L=64", base=base, queries=queries, nbrs=nbrs,
                starts=starts, metric="l2", k=10, Ls=(64,))


def config2(n=1000000, dim=200, Q=10000, A=100000, device="cuda", verbose=False):
    """1M x 200 N(0,I); 10k shifted queries; graph from 100k auxiliary queries (R=32, k_b=100); k=100."""
    base = gaussian_base(2001, n, dim)
    queries = synth.shifted_queries(Q, dim, 2002, 2003, 2004)
    aux = synth.shifted_queries(A, dim, 2002, 2003, 2005)
    nbrs, starts, info = build_query_aware_graph(base, aux, "l2")
    return dict(name="%dx%d fp32 L2, R=32 query-aware graph (k_b=100, %d aux queries), %d queries, k=100" %
                (n, dim, A, Q), base=base, queries=queries, aux=aux, nbrs=nbrs, starts=starts, metric="l2", k=100,
                Ls=(256, 512), build=info)


def structured(n=1000000, dim=200, latent=16, Q=10000, A=100000, noise=0.1, seed=6001):
    """Data with neighbourhood structure, unlike the isotropic configurations: points near a `latent`-dimensional
    subspace of R^dim (x = z P + noise * e, z ~ N(0, I_latent), P a fixed latent x dim Gaussian matrix scaled to unit
    column variance, e ~ N(0, I_dim)); base, queries and auxiliary queries follow the same law.  Same graph
    construction and k as configuration 2.  Not a configuration of the benchmark: it shows what beam the graph
    search needs for recall@100 >= 0.90 when the data lets a degree-32 graph work."""
    proj = (synth.gaussian_matrix(seed, latent, dim) / np.sqrt(latent)).astype(np.float32)

    def draw(count, seed_z, seed_e):
        out = gaussian_base(seed_e, count, dim)
        out *= np.float32(noise)
        step = 1 << 16
        for r in range(0, count, step):
            z = synth.gaussian_matrix(seed_z, min(step, count - r), latent, row0=r)
            out[r:r + step] += z @ proj
        return out

    base = draw(n, seed + 1, seed + 2)
    queries = draw(Q, seed + 3, seed + 4)
    aux = draw(A, seed + 5, seed + 6)
    nbrs, starts, info = build_query_aware_graph(base, aux, "l2")
    return dict(name="%dx%d fp32 L2 near a %d-dimensional subspace, R=32 query-aware graph (k_b=100, %d aux queries), "
                     "%d queries, k=100" % (n, dim, latent, A, Q), base=base, queries=queries, nbrs=nbrs,
                starts=starts, metric="l2", k=100, Ls=(128, 256, 512), build=info)


def config3(n=1000000, dim=512, Q=10000, A=100000, device="cuda", verbose=False):
    """Inner product: unit-normalised 1M x 512 base, cone-gap queries, k=100, L=256."""
    base = synth.normalize_rows(gaussian_base(3001, n, dim))
    queries = synth.cone_queries(Q, dim, 3002, 3003)
    aux = synth.cone_queries(A, dim, 3002, 3004)
    nbrs, starts, info = build_query_aware_graph(base, aux, "ip")
    return dict(name="%dx%d fp32 IP, R=32 query-aware graph, %d queries, k=100" % (n, dim, Q), base=base,
                queries=queries, nbrs=nbrs, starts=starts, metric="ip", k=100, Ls=(256,), build=info)


def ground_truth(base, queries, k, metric="l2", device="cuda", deleted_words=None):
    """Exact top-k ids (int32 [Q][k]) by the library's brute-force kernels; tombstoned ids are left out."""
    from . import capi
    idx = capi.Index(base, None, None, metric=capi.IP if metric == "ip" else capi.L2)
    if deleted_words is not None:
        idx.set_deleted(deleted_words)
    ids, _, _ = idx.bruteforce(queries, k, have_delete=deleted_words is not None, want_dists=False)
    idx.close()
    return ids
