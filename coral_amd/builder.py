"""Query-aware graph construction for the synthetic benchmark configurations.

The reference builds its graph from auxiliary queries: the exact k_b nearest
base points of every auxiliary query form a cluster; inside a cluster every
member takes the other members as neighbour candidates, sorted by distance and
thinned by an occlusion rule ("neighbour-aware pruning", src/upd_gpu.cu:12-303),
and base points that no auxiliary query ever selected are attached afterwards
("connectivity enhancement", src/enhance.cu:728-861).  That builder needs
faiss-gpu and CUDA, is order dependent and seeds itself from std::random_device
(src/start.cu:77-79), so its exact output cannot be reproduced anywhere.

This module is a deterministic, batch-at-once restatement of the same idea in
torch tensor operations.  It exists to give the search benchmark a graph of the
right kind (degree 32, navigable for out-of-distribution queries); it is data
preparation, not part of the search path, and makes no parity claim:

  1. clusters: exact top-k_b base ids per auxiliary query (src/knn.cu:174-193);
  2. candidates of node v: the members of the first cluster that contains v,
     plus every node whose own first cluster contains v (the reference only
     pairs two nodes while at least one of them has no neighbours yet,
     src/upd_gpu.cu:61-66); the nearest `cand_cap` are kept;
  3. occlusion pruning in order of distance: a candidate is retained unless a
     retained one is closer to it than v is (src/upd_gpu.cu:203-247); rows are
     then filled with the nearest discarded candidates (need_discard,
     src/upd_gpu.cu:103-132);
  4. nodes in no cluster take their candidates from their exact nearest
     neighbours, and are inserted as candidates of the neighbours they chose
     (the reverse-edge insertion of src/enhance.cu:131-208);
  5. start ids: farthest-point sampling in vector space from the node nearest
     the auxiliary queries' mean (the reference samples farthest points in hop
     distance, src/start.cu:10-145).
"""
import numpy as np
import torch


def _dist_matrix(xq, xb, nb, metric):
    ip = xq @ xb.T
    return (nb[None, :] - 2.0 * ip) if metric == "l2" else -ip


def exact_topk(base, queries, k, metric="l2", block=4096, exclude_self_offset=None):
    """ids [Q][k] nearest first.  With exclude_self_offset = s, query i is base row s+i and skips itself."""
    nb = (base * base).sum(1)
    out = torch.empty((queries.shape[0], k), dtype=torch.int64, device=base.device)
    for s in range(0, queries.shape[0], block):
        d = _dist_matrix(queries[s:s + block], base, nb, metric)
        if exclude_self_offset is not None:
            rows = torch.arange(d.shape[0], device=base.device)
            d[rows, rows + s + exclude_self_offset] = float("inf")
        out[s:s + block] = torch.topk(d, k, dim=1, largest=False, sorted=True).indices
    return out


def _prune_rows(base, node_ids, cand, cand_d, R, metric, chunk):
    """Occlusion pruning + fill.  cand [n][C] ids sorted by distance to the node (-1 padded),
    cand_d their distances.  Returns int32 [n][R], -1 padded."""
    n, C = cand.shape
    out = torch.full((n, R), -1, dtype=torch.int32, device=base.device)
    for s in range(0, n, chunk):
        c = cand[s:s + chunk]
        dv = cand_d[s:s + chunk]
        valid = c >= 0
        vec = base[c.clamp(min=0)]  # [m][C][d]
        if metric == "l2":
            sq = (vec * vec).sum(-1)
            D = sq[:, :, None] + sq[:, None, :] - 2.0 * torch.bmm(vec, vec.transpose(1, 2))
        else:
            D = -torch.bmm(vec, vec.transpose(1, 2))
        del vec
        m = c.shape[0]
        discarded = torch.zeros((m, C), dtype=torch.bool, device=base.device)
        kept = torch.zeros((m, C), dtype=torch.bool, device=base.device)
        nkept = torch.zeros(m, dtype=torch.int32, device=base.device)
        for i in range(C):
            take = valid[:, i] & ~discarded[:, i] & (nkept < R)
            kept[:, i] = take
            nkept += take.to(torch.int32)
            if i + 1 < C:
                occl = D[:, i, i + 1:] < dv[:, i + 1:]
                discarded[:, i + 1:] |= take[:, None] & occl
        # fill: retained entries plus the nearest discarded ones, in distance order
        need = (R - nkept).clamp(min=0)
        disc_rank = torch.cumsum((valid & ~kept).to(torch.int32), dim=1)
        chosen = kept | (valid & ~kept & (disc_rank <= need[:, None]))
        pos = torch.cumsum(chosen.to(torch.int32), dim=1) - 1
        sel = chosen & (pos < R)
        rows = torch.arange(m, device=base.device)[:, None].expand(m, C)
        out[s:s + chunk][rows[sel], pos[sel].long()] = c[sel].to(torch.int32)
        del D
    return out


def _topc_by_node(src, dst, dist, n, C):
    """Group (src, dst, dist) pairs by src, drop duplicate dst, keep the C nearest.
    Returns cand [n][C] int64 (-1 padded) and their distances (inf padded)."""
    dev = src.device
    # order by (src, dist); distances are compared through their order-preserving bit pattern
    bits = dist.view(torch.int32).to(torch.int64)
    bits = torch.where(bits < 0, bits ^ 0x7FFFFFFF, bits) + (1 << 31)
    order = torch.argsort(src * (1 << 32) + bits)
    src, dst, dist = src[order], dst[order], dist[order]
    del order, bits
    # duplicates of (src, dst) carry the same distance, so they sit next to each other
    # only up to ties; remove them with a second stable pass keyed on (src, dst)
    key = src * (1 << 31) + dst
    uniq_order = torch.argsort(key, stable=True)
    ks = key[uniq_order]
    first = torch.ones_like(ks, dtype=torch.bool)
    first[1:] = ks[1:] != ks[:-1]
    keep = torch.zeros_like(first)
    keep[uniq_order[first]] = True
    src, dst, dist = src[keep], dst[keep], dist[keep]
    del key, uniq_order, ks, first, keep
    start = torch.searchsorted(src, torch.arange(n, device=dev))
    rank = torch.arange(src.numel(), device=dev) - start[src]
    ok = rank < C
    cand = torch.full((n, C), -1, dtype=torch.int64, device=dev)
    cd = torch.full((n, C), float("inf"), dtype=torch.float32, device=dev)
    cand[src[ok], rank[ok]] = dst[ok]
    cd[src[ok], rank[ok]] = dist[ok]
    return cand, cd


def build_graph(base_np, aux_np, R=32, k_b=100, metric="l2", n_start=16, cand_cap=128, device="cuda",
                cluster_chunk=4096, prune_chunk=32768, verbose=False):
    """Returns (nbrs int32 [n][R] numpy, start_ids int32 [n_start] numpy, info dict)."""
    import time
    t0 = time.time()
    dev = torch.device(device)
    base = torch.from_numpy(np.ascontiguousarray(base_np, dtype=np.float32)).to(dev)
    aux = torch.from_numpy(np.ascontiguousarray(aux_np, dtype=np.float32)).to(dev)
    n, A = base.shape[0], aux.shape[0]

    def log(msg):
        if verbose:
            if dev.type == "cuda":
                torch.cuda.synchronize()
            print("[builder %6.1fs] %s" % (time.time() - t0, msg), flush=True)

    knn = exact_topk(base, aux, k_b, metric)  # [A][k_b]
    log("cluster ids")
    first = torch.full((n,), A, dtype=torch.int64, device=dev)
    aidx = torch.arange(A, device=dev)[:, None].expand(A, k_b).reshape(-1)
    first.scatter_reduce_(0, knn.reshape(-1), aidx, reduce="amin")
    covered = first < A
    log("%d of %d nodes appear in a cluster" % (int(covered.sum()), n))

    srcs, dsts, dds = [], [], []
    for s in range(0, A, cluster_chunk):
        m = knn[s:s + cluster_chunk]  # [c][k_b]
        c = m.shape[0]
        vec = base[m]
        if metric == "l2":
            sq = (vec * vec).sum(-1)
            D = sq[:, :, None] + sq[:, None, :] - 2.0 * torch.bmm(vec, vec.transpose(1, 2))
            D.clamp_(min=0)
        else:
            D = -torch.bmm(vec, vec.transpose(1, 2))
        del vec
        new = first[m] == (torch.arange(s, s + c, device=dev)[:, None])  # node is new in this cluster
        ok = new[:, :, None] | new[:, None, :]
        eye = torch.eye(k_b, dtype=torch.bool, device=dev)[None]
        ok &= ~eye
        ci, ii, jj = ok.nonzero(as_tuple=True)
        srcs.append(m[ci, ii])
        dsts.append(m[ci, jj])
        dds.append(D[ci, ii, jj])
        del D, ok
    src, dst, dd = torch.cat(srcs), torch.cat(dsts), torch.cat(dds)
    del srcs, dsts, dds
    log("%d candidate pairs" % src.numel())
    cand, cd = _topc_by_node(src, dst, dd, n, cand_cap)
    del src, dst, dd
    nbrs = _prune_rows(base, None, cand, cd, R, metric, prune_chunk)
    del cand, cd
    log("pruned covered nodes")

    iso = (~covered).nonzero(as_tuple=True)[0]
    if iso.numel():
        # nodes outside every cluster: candidates from their exact neighbours ...
        nb = (base * base).sum(1)
        iso_knn = torch.empty((iso.numel(), k_b), dtype=torch.int64, device=dev)
        iso_d = torch.empty((iso.numel(), k_b), dtype=torch.float32, device=dev)
        for s in range(0, iso.numel(), 4096):
            ids = iso[s:s + 4096]
            d = _dist_matrix(base[ids], base, nb, metric)
            d[torch.arange(ids.numel(), device=dev), ids] = float("inf")
            tv, ti = torch.topk(d, k_b, dim=1, largest=False, sorted=True)
            iso_knn[s:s + 4096], iso_d[s:s + 4096] = ti, tv
        iso_rows = _prune_rows(base, None, iso_knn, iso_d, R, metric, prune_chunk)
        nbrs[iso] = iso_rows
        log("attached %d uncovered nodes" % iso.numel())
        # ... and they become candidates of the neighbours they chose
        sel = iso_rows >= 0
        r_src = iso_rows[sel].to(torch.int64)  # the chosen neighbour receives ...
        r_dst = iso[:, None].expand(-1, R)[sel]  # ... the uncovered node as a candidate
        vb, vd = base[r_src], base[r_dst]
        r_d = ((vb - vd) ** 2).sum(1) if metric == "l2" else -(vb * vd).sum(1)
        del vb, vd
        touched = torch.unique(r_src)
        old = nbrs[touched].to(torch.int64)  # current rows of the receiving nodes
        o_valid = old >= 0
        o_src = touched[:, None].expand(-1, R)[o_valid]
        o_dst = old[o_valid]
        vb, vd = base[o_src], base[o_dst]
        o_d = ((vb - vd) ** 2).sum(1) if metric == "l2" else -(vb * vd).sum(1)
        del vb, vd
        # compact the touched nodes to 0..t-1 for the grouping step
        remap = torch.full((n,), -1, dtype=torch.int64, device=dev)
        remap[touched] = torch.arange(touched.numel(), device=dev)
        cand, cd = _topc_by_node(torch.cat([remap[o_src], remap[r_src]]), torch.cat([o_dst, r_dst]),
                                 torch.cat([o_d, r_d]), touched.numel(), cand_cap)
        nbrs[touched] = _prune_rows(base, None, cand, cd, R, metric, prune_chunk)
        log("re-pruned %d nodes that received reverse edges" % touched.numel())

    # start ids: farthest-point sampling among covered nodes
    pool = covered.nonzero(as_tuple=True)[0]
    if pool.numel() < n_start:
        pool = torch.arange(n, device=dev)
    mean = aux.mean(0, keepdim=True)
    pv = base[pool]
    d0 = ((pv - mean) ** 2).sum(1)
    picks = [int(torch.argmin(d0))]
    mind = ((pv - pv[picks[0]][None]) ** 2).sum(1)
    for _ in range(1, n_start):
        nxt = int(torch.argmax(mind))
        picks.append(nxt)
        mind = torch.minimum(mind, ((pv - pv[nxt][None]) ** 2).sum(1))
    starts = pool[torch.tensor(picks, device=dev)].to(torch.int32).cpu().numpy()
    deg = (nbrs >= 0).sum(1).float()
    info = {"covered": int(covered.sum()), "uncovered": int(iso.numel()), "avg_degree": float(deg.mean()),
            "min_degree": int(deg.min()), "build_s": time.time() - t0}
    log("done: %s" % info)
    return nbrs.cpu().numpy(), starts, info
