"""TEST INFRASTRUCTURE ONLY: CPU restatement of the reference's structure learning.

Restated (paths relative to VariationalJuice.jl/):
  * src/utils/information.jl:43-95   -- `single_and_pairwise_marginal`: cell counts start at
        pseudocount / C^2 (pairs) and pseudocount / C (singles) and are divided by Z = N + pseudocount
  * src/utils/information.jl:97-141  -- `pairwise_MI_chunked`:
        MI[u, v] = sum_{a,b} xlogx(P_uv[a,b]) - xlogy(P_uv[a,b], P_u[a] * P_v[b])
  * src/structures/hclts.jl:17-18    -- `learn_chow_liu_tree` + `clt_edges2graphs(...; shape = :directed)`

The last two live in the un-vendored dependencies ChowLiuTrees.jl and ProbabilisticCircuits.jl
(no manifest, versions unpinned).  Their published behaviour is restated: a maximum spanning
tree of the MI matrix, directed by breadth-first search from `center(tree)[1]`, the
lowest-numbered vertex of least eccentricity (Graphs.jl).  Which of several equal-weight
trees ChowLiuTrees.jl returns and the order of a node's children are PARITY UNPINNED: no file
of the reference fixes them; the tests check tree weight and validity, not edge identity.

`pairwise_mi` is pinned by sklearn.metrics.mutual_info_score (pseudocount 0), by
MI(x, x) = H(x), MI of independent columns -> 0, and symmetry; `chow_liu_tree` by
scipy.sparse.csgraph.minimum_spanning_tree (total weight) and a brute-force eccentricity.
Nothing in the product imports this module.
"""
import numpy as np


def marginals(data, C, pseudocount):
    """[V, V, C, C] pair marginals and [V, C] single marginals, float64 (small inputs only)."""
    N, V = data.shape
    Z = N + pseudocount
    single = np.full((V, C), pseudocount / C, np.float64)
    for v in range(V):
        np.add.at(single[v], data[:, v], 1.0)
    pair = np.full((V, V, C, C), pseudocount / C / C, np.float64)
    for u in range(V):
        for v in range(V):
            np.add.at(pair[u, v], (data[:, u], data[:, v]), 1.0)
    return pair / Z, single / Z


def pairwise_mi(data, C, pseudocount=0.1):
    """MI matrix [V, V], float64, the formula of information.jl:124-127 term by term."""
    data = np.asarray(data).astype(np.int64)
    pair, single = marginals(data, C, pseudocount)
    V = data.shape[1]
    mi = np.zeros((V, V))
    for u in range(V):
        for v in range(V):
            p = pair[u, v]
            q = np.outer(single[u], single[v])
            nz = p > 0
            mi[u, v] = (p[nz] * np.log(p[nz])).sum() - (p[nz] * np.log(q[nz])).sum()
    return mi


def chow_liu_tree(mi):
    """Parent array (root -1) of the maximum spanning tree of `mi`, rooted at the
    lowest-numbered vertex of least eccentricity.  Prim from vertex 0, ties to the lowest index."""
    mi = np.asarray(mi, np.float64)
    V = mi.shape[0]
    in_tree = np.zeros(V, bool)
    in_tree[0] = True
    best, link = mi[0].copy(), np.zeros(V, np.int64)
    adj = [[] for _ in range(V)]
    for _ in range(V - 1):
        cand = np.where(~in_tree)[0]
        pick = cand[np.argmax(best[cand])]
        in_tree[pick] = True
        adj[pick].append(int(link[pick]))
        adj[int(link[pick])].append(int(pick))
        upd = (~in_tree) & (mi[pick] > best)
        best[upd] = mi[pick][upd]
        link[upd] = pick

    def bfs(src):
        dist = np.full(V, -1)
        dist[src] = 0
        order = [src]
        for x in order:
            for y in sorted(adj[x]):
                if dist[y] < 0:
                    dist[y] = dist[x] + 1
                    order.append(y)
        return dist, order

    ecc = np.array([bfs(v)[0].max() for v in range(V)])
    root = int(np.argmin(ecc))
    parent = np.full(V, -1, np.int32)
    dist, order = bfs(root)
    for x in order:
        for y in adj[x]:
            if dist[y] == dist[x] + 1:
                parent[y] = x
    return parent


def tree_weight(mi, parent):
    return float(sum(mi[v, p] for v, p in enumerate(parent) if p >= 0))
