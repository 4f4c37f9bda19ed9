"""Structure learning: the step before `hclt_from_clt`, named after the reference functions."""
import numpy as np
import torch

from ._lib import lib, check, np_ptr
from .circuits import hclt_from_clt


def pairwise_MI(data, num_cats=None, pseudocount=0.1):
    """`pairwise_MI_chunked(data; num_cats, pseudocount)` (src/utils/information.jl:97-141):
    mutual information of every pair of variables of a uint8 device tensor [N, V]; returns a
    float32 device tensor [V, V] (symmetric, diagonal included).  Any number of examples in one
    call: a pair's table never leaves the workgroup that counts it (16-bit cells up to 65535
    examples, 32-bit cells walked in bands of rows beyond)."""
    if not (isinstance(data, torch.Tensor) and data.is_cuda and data.dtype == torch.uint8 and data.dim() == 2):
        raise ValueError("data must be a 2-D uint8 tensor on the GPU (examples x variables)")
    n, v = data.shape
    if num_cats is None:
        num_cats = int(data.max().item()) + 1
    mi = torch.empty((v, v), dtype=torch.float32, device=data.device)
    check(lib.pcm_pairwise_mi(data.data_ptr(), data.stride(0), data.stride(1), n, v, int(num_cats), float(pseudocount),
                              mi.data_ptr(), torch.cuda.current_stream(data.device).cuda_stream))
    return mi


def chow_liu_tree(mi):
    """Maximum spanning tree of a mutual-information matrix, directed away from the centre of
    the tree (what `learn_chow_liu_tree` followed by `clt_edges2graphs(...; shape = :directed)`
    gives src/structures/hclts.jl:17-18), as the parent array `hclt_from_clt` takes."""
    m = np.ascontiguousarray(mi.detach().cpu().numpy() if isinstance(mi, torch.Tensor) else mi, dtype=np.float32)
    if m.ndim != 2 or m.shape[0] != m.shape[1]:
        raise ValueError("mi must be a square matrix")
    parent = np.empty(m.shape[0], np.int32)
    check(lib.pcm_chow_liu_tree(np_ptr(m), m.shape[0], np_ptr(parent)))
    return parent


def learn_chow_liu_tree(data, num_cats=None, pseudocount=0.1):
    """`learn_chow_liu_tree(data; pseudocount)` as src/structures/hclts.jl:17 calls it, returning
    the rooted tree as a parent array."""
    return chow_liu_tree(pairwise_MI(data, num_cats, pseudocount))


def hclt(data, num_hidden_cats, variable_groups=None, num_cats=None, pseudocount=0.1, get_leaves=False):
    """`hclt(data, num_hidden_cats, variable_groups; num_cats, pseudocount)` (src/structures/hclts.jl:7-24): the
    Chow-Liu tree of the groups' first variables, then the hidden Chow-Liu tree circuit over the groups.  Without
    groups (one variable per tree node) the circuit is built on the block kernels (`hclt_from_clt`); with groups
    it is the DAG of `hclt_pc`, to be compiled with `CuBitsProbCircuit` (with `get_leaves` also the tree nodes'
    leaf circuits, as `hclt_from_clt(...; get_leaves = true)` returns them)."""
    if num_cats is None:
        num_cats = int(data.max().item()) + 1
    if variable_groups is None:
        return hclt_from_clt(learn_chow_liu_tree(data, num_cats, pseudocount), int(num_cats), int(num_hidden_cats))
    firsts = [int(g[0]) for g in variable_groups]
    mapped = data[:, firsts].contiguous()            # mapped_data[:, idx] = data[:, variable_groups[idx][1]] (:14)
    clt = learn_chow_liu_tree(mapped, num_cats, pseudocount)
    return hclt_pc(clt, int(num_cats), int(num_hidden_cats), variable_groups, get_leaves=get_leaves)


def hclt_for_colored_images(data, nc, height, width, num_hidden_cats, num_cats=None, pseudocount=0.1, mode="red_only",
                            patch_size=2):
    """`hclt_for_colored_images` (src/structures/hclts.jl:26-98): an HCLT over patch_size x patch_size groups of the
    pixels of one channel ("red_only", "green_only", "blue_only": the channel's plane of the [N, nc * height * width]
    data) or of all channels of a patch ("cat_channels").  Returns (circuit, leaves) as the reference does."""
    plane = height * width
    if mode in ("red_only", "green_only", "blue_only"):
        offset = {"red_only": 0, "green_only": plane, "blue_only": 2 * plane}[mode]
        groups = group_vars_by_grid(height, width, 1, patch_h=patch_size, patch_w=patch_size, global_offset=offset)
    elif mode == "cat_channels":
        groups = group_vars_by_cgrid(height, width, nc, patch_h=patch_size, patch_w=patch_size, global_offset=0)
    else:
        raise ValueError("Not implemented")           # hclts.jl:94
    if num_cats is None:
        num_cats = int(data.max().item()) + 1
    return hclt(data, num_hidden_cats, groups, num_cats=num_cats, pseudocount=pseudocount, get_leaves=True)


# ---- trees ---------------------------------------------------------------------------------

def clt_edges2parent(clt_edges, num_vars=None):
    """`clt_edges2graphs(clt_edges; shape = :directed)` / `edges2graphs`
    (src/structures/customizable_hclt.jl:104-125): the undirected tree given by its edges,
    rooted at its lowest-numbered centre and directed away from it; returned as a parent array
    (root: -1).  Variables are 0-based and must be 0..num_vars-1."""
    edges = [(int(a), int(b)) for a, b in clt_edges]
    if num_vars is None:
        num_vars = max(max(e) for e in edges) + 1 if edges else 1
    if len(edges) != num_vars - 1:
        raise ValueError(f"a tree over {num_vars} variables has {num_vars - 1} edges, got {len(edges)}")
    adj = [[] for _ in range(num_vars)]
    for a, b in edges:
        if not (0 <= a < num_vars and 0 <= b < num_vars) or a == b:
            raise ValueError(f"bad edge ({a}, {b})")
        adj[a].append(b)
        adj[b].append(a)
    # centre by peeling leaves; of two centres the lower-numbered one
    deg = [len(a) for a in adj]
    alive = num_vars
    layer = [v for v in range(num_vars) if deg[v] <= 1]
    removed = [False] * num_vars
    while alive > 2:
        nxt = []
        for v in layer:
            removed[v] = True
            alive -= 1
            for u in adj[v]:
                if not removed[u]:
                    deg[u] -= 1
                    if deg[u] == 1:
                        nxt.append(u)
        if not nxt:
            raise ValueError("the edges do not form a tree")
        layer = nxt
    root = min(v for v in range(num_vars) if not removed[v])
    parent = np.full(num_vars, -2, np.int32)
    parent[root] = -1
    queue = [root]
    for v in queue:
        for u in sorted(adj[v]):
            if parent[u] == -2:
                parent[u] = v
                queue.append(u)
    if (parent == -2).any():
        raise ValueError("the edges do not form a tree")
    return parent


def _tree_children(parent):
    parent = np.asarray(parent, np.int64)
    ch = [[] for _ in parent]
    root = -1
    for v, p in enumerate(parent):
        if p < 0:
            root = v
        else:
            ch[p].append(v)
    order, stack = [], [root]
    while stack:                       # parents first; reversed: a bottom-up order
        v = stack.pop()
        order.append(v)
        stack.extend(reversed(ch[v]))
    return ch, root, order[::-1]


def group_vars_by_grid(height, width, cdepth, patch_h=2, patch_w=2, global_offset=0):
    """`group_vars_by_grid` (src/structures/hclts.jl:189-221): per channel, patch_h x patch_w
    blocks of pixels; returns [(first variable, sorted variables of the group)], 0-based."""
    if height % patch_h or width % patch_w:
        raise ValueError("the patch must divide the image")
    groups = []
    for c in range(cdepth):
        off = height * width * c + global_offset
        for h in range(0, height, patch_h):
            for w in range(0, width, patch_w):
                vs = [(h + x) * width + (w + y) + off for x in range(patch_h) for y in range(patch_w)]
                groups.append((h * width + w + off, sorted(vs)))
    return groups


def group_vars_by_cgrid(height, width, cdepth, patch_h=2, patch_w=2, global_offset=0):
    """`group_vars_by_cgrid` (src/structures/hclts.jl:223-257): patch_h x patch_w blocks of
    pixels with all their channels in one group."""
    if height % patch_h or width % patch_w:
        raise ValueError("the patch must divide the image")
    groups = []
    for h in range(0, height, patch_h):
        for w in range(0, width, patch_w):
            vs = [(h + x) * width + (w + y) + height * width * c + global_offset
                  for x in range(patch_h) for y in range(patch_w) for c in range(cdepth)]
            groups.append((h * width + w + global_offset, sorted(vs)))
    return groups


# ---- circuits as DAGs ------------------------------------------------------------------------

def hclt_pc(clt_parent, num_cats, num_hidden_cats, variable_groups=None, get_leaves=False):
    """`hclt_from_clt(clt, num_cats, num_hidden_cats, variable_groups; input_type = Categorical)`
    (src/structures/hclts.jl:100-145) as a DAG of `pcmi355.nodes`: tree node i stands for the
    observed variables `variable_groups[i][1]` (default: variable i alone), whose joint leaf is
    the product of one categorical per variable (`categorical_leaves`, hclts.jl:146-155).
    Compile with `CuBitsProbCircuit`; with one variable per group `hclt_from_clt` builds the
    same circuit on the block kernels."""
    from . import nodes as N
    K = int(num_hidden_cats)
    ch, root, order = _tree_children(clt_parent)
    if variable_groups is None:
        variable_groups = [(v, [v]) for v in range(len(ch))]
    if len(variable_groups) != len(ch):
        raise ValueError("one variable group per tree node is needed")

    def leaf(i):
        return N.summate(N.multiply([N.categorical(v, num_cats) for v in variable_groups[i][1]]))

    leaves = [[leaf(i) for _ in range(K)] for i in range(len(ch))]
    circuits = {}
    for v in order:
        if not ch[v]:
            circuits[v] = leaves[v]
            continue
        cc = [circuits[c] for c in ch[v]]
        cc = [N.summate(N.multiply([c[j] for c in cc])) for j in range(K)] if len(cc) > 1 else cc[0]
        circuits[v] = [N.summate([N.multiply(cc[j], leaves[v][j]) for j in range(K)]) for _ in range(K)]
    return (circuits[root][0], leaves) if get_leaves else circuits[root][0]


def customized_hclt(clt, num_hidden_cats, get_leaf_pcs, get_edge_params=None, parameterize_leaf_edge=True,
                    variables=None):
    """`customized_hclt(clt_edges, num_hidden_cats; get_leaf_pcs, get_edge_params,
    parameterize_leaf_edge)` (src/structures/customizable_hclt.jl:4-50), the builder of the
    top-level circuit (exps/LVD_for_imagenet/src/train_PG_top_level_pcs.jl:153-170): every tree
    node's K circuits are the products of its children's circuits and its own K leaf circuits
    `get_leaf_pcs(var, num_hidden_cats)`; the edge to a child is a K x K block of sum nodes over
    the child's circuits (also over a leaf child's when `parameterize_leaf_edge`), initialised
    from `get_edge_params(var, child_var, num_hidden_cats)` [K, K] (rows normalised) when given.
    `clt`: a parent array or a list of undirected edges; `variables[i]`: what tree node i is
    called in the two callbacks (default i)."""
    from . import nodes as N
    K = int(num_hidden_cats)
    parent = np.asarray(clt, np.int32) if np.ndim(clt) == 1 and not isinstance(clt[0], (tuple, list)) else clt_edges2parent(clt)
    ch, root, order = _tree_children(parent)
    name = (lambda i: i) if variables is None else (lambda i: variables[i])
    pcs = {}
    for v in order:
        own = list(get_leaf_pcs(name(v), K))
        if len(own) != K:
            raise ValueError("get_leaf_pcs must return num_hidden_cats circuits")
        if not ch[v]:
            pcs[v] = own
            continue
        ch_pcs = []
        for c in ch[v]:
            cp = pcs[c]
            if parameterize_leaf_edge or ch[c]:
                cp = [N.summate(cp) for _ in range(K)]
                if get_edge_params is not None:
                    w = np.asarray(get_edge_params(name(v), name(c), K), np.float64)
                    for i in range(K):
                        cp[i].params = np.log(w[i] / w[i].sum()).astype(np.float32)
            ch_pcs.append(cp)
        ch_pcs.append(own)
        pcs[v] = [N.multiply([cp[j] for cp in ch_pcs]) for j in range(K)]
    return N.summate(pcs[root])


class _Region:
    __slots__ = ("scope", "partitions", "var")

    def __init__(self, scope, var=None):
        self.scope, self.partitions, self.var = scope, [], var


def joined_hclt_from_clts(clt_parents, num_hidden_cats, num_cats):
    """The circuit of `joined_hclt` (src-jl/structures/joined_hclt.jl:16-104) for trees already
    learned: the trees' regions (a tree node with everything below it) are merged by scope, a
    region keeps one partition per distinct way of splitting it (`myhash`: the children's
    scopes), every partition is K products taking the j-th circuit of each child region and of
    the node's own input region, every region K sum nodes over all its partitions' products.
    Returns the K circuits of the full scope (the reference returns the same vector)."""
    from . import nodes as N
    K = int(num_hidden_cats)
    regions = {}

    def input_region(v):
        s = frozenset([v])
        if s not in regions:
            regions[s] = _Region(s, var=v)
        return regions[s]

    num_vars = len(clt_parents[0])
    for parent in clt_parents:
        if len(parent) != num_vars:
            raise ValueError("the trees must span the same variables")
        ch, root, order = _tree_children(parent)
        rnode = {}
        for v in order:
            if not ch[v]:
                rnode[v] = input_region(v)
                continue
            kids = [rnode[c] for c in ch[v]] + [input_region(v)]
            scope = frozenset().union(*[k.scope for k in kids])
            key = tuple(sorted((k.scope for k in kids), key=min))
            r = regions.get(scope)
            if r is None:
                r = regions[scope] = _Region(scope)
            if r.var is not None:
                raise ValueError("a tree node's region coincides with a single variable")
            if all(k != key for k, _ in r.partitions):
                r.partitions.append((key, kids))
            rnode[v] = r
    full = regions.get(frozenset(range(num_vars)))
    if full is None:
        raise ValueError("the trees do not span all variables")

    built = {}
    order, stack, seen = [], [(full, 0)], {id(full)}
    flat_kids = lambda r: [k for _, kids in r.partitions for k in kids]
    while stack:                                    # regions bottom-up
        r, i = stack[-1]
        kids = flat_kids(r)
        if i < len(kids):
            stack[-1] = (r, i + 1)
            if id(kids[i]) not in seen:
                seen.add(id(kids[i]))
                stack.append((kids[i], 0))
        else:
            order.append(r)
            stack.pop()
    for r in order:
        if r.var is not None:
            built[id(r)] = [N.categorical(r.var, num_cats) for _ in range(K)]
        else:
            prods = [N.multiply([built[id(k)][j] for k in kids]) for _, kids in r.partitions for j in range(K)]
            built[id(r)] = [N.summate(prods) for _ in range(K)]
    return built[id(full)]


def joined_hclt(datasets, num_hidden_cats, num_cats=None, pseudocount=0.1):
    """`joined_hclt(datasets, num_hidden_cats; num_cats, pseudocount)`
    (src-jl/structures/joined_hclt.jl:65-104): one Chow-Liu tree per dataset (uint8 device
    tensors over the same variables), merged into one circuit."""
    if num_cats is None:
        num_cats = max(int(d.max().item()) for d in datasets) + 1
    trees = [learn_chow_liu_tree(d, num_cats, pseudocount) for d in datasets]
    return joined_hclt_from_clts(trees, num_hidden_cats, num_cats)
