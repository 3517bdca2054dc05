"""The benchmark configurations as seeded synthetic workloads (base vectors,
queries, auxiliary queries, graph, start ids, ground truth).

Everything here is data preparation around the search path: generation runs on
the host (coral_amd.synth), graph construction and brute-force ground truth use
torch on the GPU as plumbing (coral_amd.builder)."""
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


def config1(device="cuda"):
    """100k x 128 N(0,I); 1k shifted queries; exact 32-NN graph; entry = medoid; k=10, L=64, L2."""
    base = gaussian_base(1001, 100000, 128)
    queries = synth.shifted_queries(1000, 128, 1002, 1003, 1004)
    nbrs = synth.exact_knn_graph(base, 32, device=device)
    starts = np.array([synth.medoid_start(base)], np.int32)
    return dict(name="100k x 128 fp32 L2, exact 32-NN graph, k=10, L=64", base=base, queries=queries, nbrs=nbrs,
                starts=starts, metric="l2", k=10, Ls=(64,))


def config2(n=1000000, dim=200, Q=10000, A=100000, device="cuda", verbose=False):
    """1M x 200 N(0,I); 10k shifted queries; graph from 100k auxiliary queries (R=32, k_b=100); k=100."""
    from . import builder
    base = gaussian_base(2001, n, dim)
    queries = synth.shifted_queries(Q, dim, 2002, 2003, 2004)
    aux = synth.shifted_queries(A, dim, 2002, 2003, 2005)
    nbrs, starts, info = builder.build_graph(base, aux, 32, 100, "l2", device=device, verbose=verbose)
    return dict(name="%dx%d fp32 L2, R=32 query-aware graph (k_b=100, %d aux queries), %d queries, k=100" %
                (n, dim, A, Q), base=base, queries=queries, nbrs=nbrs, starts=starts, metric="l2", k=100,
                Ls=(256, 512), build=info)


def config3(n=1000000, dim=512, Q=10000, A=100000, device="cuda", verbose=False):
    """Inner product: unit-normalised 1M x 512 base, cone-gap queries, k=100, L=256."""
    from . import builder
    base = synth.normalize_rows(gaussian_base(3001, n, dim))
    queries = synth.cone_queries(Q, dim, 3002, 3003)
    aux = synth.cone_queries(A, dim, 3002, 3004)
    nbrs, starts, info = builder.build_graph(base, aux, 32, 100, "ip", device=device, verbose=verbose)
    return dict(name="%dx%d fp32 IP, R=32 query-aware graph, %d queries, k=100" % (n, dim, Q), base=base,
                queries=queries, nbrs=nbrs, starts=starts, metric="ip", k=100, Ls=(256,), build=info)


def ground_truth(base, queries, k, metric="l2", device="cuda", deleted_words=None):
    """Exact top-k ids (int32 [Q][k]) by brute force on the GPU."""
    import torch
    from . import builder
    tb = torch.from_numpy(base).to(device)
    tq = torch.from_numpy(queries).to(device)
    if deleted_words is None:
        return builder.exact_topk(tb, tq, k, metric).to(torch.int32).cpu().numpy()
    dead = torch.from_numpy(np.unpackbits(deleted_words.view(np.uint8), bitorder="little")[:base.shape[0]]
                            .astype(bool)).to(device)
    nb = (tb * tb).sum(1)
    out = np.empty((queries.shape[0], k), np.int32)
    for s in range(0, queries.shape[0], 2048):
        ip = tq[s:s + 2048] @ tb.T
        d = (nb[None, :] - 2.0 * ip) if metric == "l2" else -ip
        d[:, dead] = float("inf")
        out[s:s + 2048] = torch.topk(d, k, dim=1, largest=False).indices.to(torch.int32).cpu().numpy()
    return out
