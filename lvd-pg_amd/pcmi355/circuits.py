"""Compiled circuits: thin owners of a `pcm_circuit*` handle."""
import ctypes

import numpy as np

from ._lib import lib, check, np_ptr, H, c_i64

_SIZE = dict(parameters=0, sum_parameters=1, nodes=2, edges=3, input_parameters=4, variables=5,
             categories=6, hidden_categories=7, inner_tree_nodes=8, layers=9, groups=10, input_nodes=11, heads=12,
             description_nodes=13, walk_kernels=14, trees=15, dense_groups=16, layer_nodes=17, walk_levels=18)
_TABLE = dict(edge2param=(0, "edges"), param2edge=(1, "sum_parameters"), param2group=(2, "sum_parameters"),
              pargroup_sizes=(3, "groups"), innode2ncumparam=(4, "input_nodes"), layer_ends=(5, "layers"),
              edge_parent=(6, "edges"), edge_prime=(7, "edges"), edge_sub=(8, "edges"), heads=(9, "heads"),
              description2node=(10, "description_nodes"), input_node_ids=(11, "input_nodes"))


class BitsCircuit:
    """Counterpart of `CuMetaBitsProbCircuit` (src/bits_circuit.jl:5-37): the flattened
    circuit lives on the device inside the library; index tables are served on request."""

    def __init__(self, handle):
        self._h = handle

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            lib.pcm_free(h)

    @property
    def handle(self):
        if not self._h:
            raise ValueError("circuit has been freed")
        return self._h

    def size(self, what):
        r = lib.pcm_size(self.handle, _SIZE[what])
        if r < 0:
            check(-1)
        return int(r)

    def set_flow_scale(self, fscale):
        """`fscale` of `mini_batch_em_beta` (src-jl/learning/em.jl:293, flow.jl:120-373): flows that feed the statistics
        hand a sum node's flow down in shares proportional to (posterior share)^(1 / fscale).  1 switches it off."""
        check(lib.pcm_set_flow_scale(self.handle, float(fscale)))

    # src/bits_circuit.jl:119-131
    def num_parameters(self):
        return self.size("parameters")

    def num_nodes(self):
        return self.size("nodes")

    def num_edges(self):
        return self.size("edges")

    def num_input_params(self):
        return self.size("input_parameters")

    def num_inner_params(self):
        return self.size("sum_parameters")

    def table(self, name):
        """1-based index tables named as the fields of `CuMetaBitsProbCircuit`."""
        which, length = _TABLE[name]
        out = np.empty(self.size(length), dtype=np.int64)
        check(lib.pcm_index_table(self.handle, which, np_ptr(out), c_i64(len(out))))
        return out

    def set_stream(self, stream):
        check(lib.pcm_set_stream(self.handle, ctypes.c_void_p(stream)))

    def get_node_values(self, batch, flows=True):
        """Host copies of `mars` (and `flows`) of the last batch, [num_nodes, batch]
        (circuits from compile_circuit only)."""
        n = self.num_nodes()
        mars = np.empty((n, batch), np.float32)
        fl = np.empty((n, batch), np.float32) if flows else None
        check(lib.pcm_get_node_values(self.handle, np_ptr(mars), np_ptr(fl), c_i64(n * batch)))
        return (mars, fl) if flows else mars

    def node_flow_sums(self):
        """Flow of every node summed over the examples of the last flow pass, [num_nodes]."""
        out = np.empty(self.num_nodes(), np.float32)
        check(lib.pcm_node_flow_sums(self.handle, np_ptr(out), c_i64(len(out))))
        return out

    def get_aggregates(self):
        """(edge_aggr [edges, up order], leaf flows [input parameters]) accumulated so far."""
        ea = np.empty(self.num_edges(), np.float32)
        lf = np.empty(self.num_input_params(), np.float32)
        check(lib.pcm_get_aggregates(self.handle, np_ptr(ea), c_i64(len(ea)), np_ptr(lf), c_i64(len(lf))))
        return ea, lf


class HcltCircuit(BitsCircuit):
    def __init__(self, handle, clt_parent, num_cats, num_hidden_cats):
        super().__init__(handle)
        self.clt_parent = np.asarray(clt_parent, dtype=np.int32).copy()
        self.num_vars = len(self.clt_parent)
        self.num_cats = num_cats
        self.num_hidden_cats = num_hidden_cats

    def set_params(self, theta=None, leaf=None):
        """theta [V, K, K], leaf [V, K, C] log-parameters (block form)."""
        V, K, C = self.num_vars, self.num_hidden_cats, self.num_cats
        if theta is not None:
            theta = np.ascontiguousarray(theta, dtype=np.float32)
            assert theta.shape == (V, K, K), theta.shape
        if leaf is not None:
            leaf = np.ascontiguousarray(leaf, dtype=np.float32)
            assert leaf.shape == (V, K, C), leaf.shape
        check(lib.pcm_hclt_set_params(self.handle, np_ptr(theta), np_ptr(leaf)))

    def get_params(self):
        V, K, C = self.num_vars, self.num_hidden_cats, self.num_cats
        theta = np.empty((V, K, K), np.float32)
        leaf = np.empty((V, K, C), np.float32)
        check(lib.pcm_hclt_get_params(self.handle, np_ptr(theta), np_ptr(leaf)))
        return theta, leaf

    def get_flows(self):
        V, K, C = self.num_vars, self.num_hidden_cats, self.num_cats
        ea = np.empty((V, K, K), np.float32)
        lf = np.empty((V, K, C), np.float32)
        check(lib.pcm_hclt_get_flows(self.handle, np_ptr(ea), np_ptr(lf)))
        return ea, lf

    def set_soft_reg(self, soft_reg, soft_reg_width=1, as_written=False):
        """`soft_reg` / `soft_reg_width` smoothing of categorical batches inside the block kernels
        (src/regularization/reg_likelihood.jl:4-14, reg_flow.jl:3-22); `as_written`: leaf statistics as `soft_flow`
        computes them.  0 switches it off.  `mini_batch_em_with_reg` sets and clears it around its loop."""
        check(lib.pcm_set_soft_reg(self.handle, float(soft_reg), int(soft_reg_width), int(bool(as_written))))

    def set_missing_category(self, on=True):
        """Declares the last category (num_cats - 1) the marker of a missing value: data carry it where the
        reference's data hold `missing` (src/regularization/reg_likelihood.jl:40-47); the leaf then counts as
        probability 1 and the update treats the marker's flow as `missing_flow`
        (src/nodes/fixable_categorical_dist.jl:223-248).  Create the circuit with one category more than the data has."""
        check(lib.pcm_set_missing_category(self.handle, int(bool(on))))

    def set_timing(self, on):
        """0 / False: off; 1 / True: the forward, backward and statistics kernels of every flows call carry timing
        events; 2, 4, 8 (or a sum of them): only the forward / backward / statistics kernel does."""
        check(lib.pcm_set_timing(self.handle, int(on)))

    def get_timing(self):
        ms = np.zeros(4, np.float32)
        check(lib.pcm_get_timing(self.handle, np_ptr(ms), 4))
        return dict(forward=float(ms[0]), backward=float(ms[1]), statistics=float(ms[2]))


class HcltForest(HcltCircuit):
    """Many multi-head HCLTs over the same batch behind one handle (`pcm_hclt_create_forest`): the patch circuits
    of exps/progressive_growing/parallel_PG.jl:214-225, trained together instead of one
    `mini_batch_em_for_multihead_pc` call each.  Tree t is the t-th root of `clt_parent` in variable order."""

    @property
    def num_trees(self):
        return self.size("trees")

    def tree_of_var(self):
        """[num_vars] index of the tree every variable belongs to."""
        par = self.clt_parent
        roots = np.flatnonzero(par < 0)
        tree = np.full(len(par), -1, np.int64)
        tree[roots] = np.arange(len(roots))
        pending = np.flatnonzero(tree < 0)
        while len(pending):
            tree[pending] = tree[par[pending]]
            pending = pending[tree[pending] < 0]
        return tree


def _set_heads(self, heads):
    """Head log-parameters [num_trees, num_heads, K] ([num_heads, K] for a single multi-head circuit)."""
    h = np.ascontiguousarray(heads, dtype=np.float32)
    assert h.size == self.size("trees") * self.num_heads * self.num_hidden_cats, h.shape
    check(lib.pcm_hclt_set_heads(self.handle, np_ptr(h)))


def _get_heads(self):
    T = self.size("trees")
    h = np.empty((T, self.num_heads, self.num_hidden_cats), np.float32)
    check(lib.pcm_hclt_get_heads(self.handle, np_ptr(h)))
    return h if isinstance(self, HcltForest) else h[0]


HcltCircuit.set_heads = _set_heads
HcltCircuit.get_heads = _get_heads


def hclt_forest_from_clts(clt_parent, num_cats, num_hidden_cats, num_heads):
    """A forest handle: `clt_parent` over all variables of the batch, one -1 entry per tree; every tree becomes a
    multi-head HCLT with `num_heads` heads (see HcltForest)."""
    par = np.ascontiguousarray(clt_parent, dtype=np.int32)
    h = H()
    check(lib.pcm_hclt_create_forest(np_ptr(par), len(par), int(num_hidden_cats), int(num_cats), int(num_heads),
                                     ctypes.byref(h)))
    c = HcltForest(h, par, int(num_cats), int(num_hidden_cats))
    c.num_heads = int(num_heads)
    return c


def multihead_hclt_from_clt(clt_parent, num_cats, num_hidden_cats, num_heads):
    """A multi-head HCLT on the block engine: `num_heads` root sum nodes over the K products of one
    HCLT body, what `CuMultiHeadBitsProbCircuit(pcs)` (src-jl/multi_head_pc/bit_circuit.jl:14-56) is
    given by exps/progressive_growing/parallel_PG.jl:214-225.  Raises PcmError (unsupported) for
    hidden sizes or trees without block kernels: use `compile_multihead` then."""
    par = np.ascontiguousarray(clt_parent, dtype=np.int32)
    h = ctypes.c_void_p()
    check(lib.pcm_hclt_create_multihead(np_ptr(par), len(par), int(num_hidden_cats), int(num_cats), int(num_heads),
                                        ctypes.byref(h)))
    c = HcltCircuit(h, par, int(num_cats), int(num_hidden_cats))
    c.num_heads = int(num_heads)
    return c


def hclt_from_clt(clt_parent, num_cats, num_hidden_cats):
    """`hclt_from_clt(clt, num_cats, num_hidden_cats, variable_groups; input_type = Categorical)`
    (src/structures/hclts.jl:100-145) followed by `CuMetaBitsProbCircuit(pc)`; the tree is
    given as a parent array (root: -1), one observed variable per tree node."""
    par = np.ascontiguousarray(clt_parent, dtype=np.int32)
    h = H()
    check(lib.pcm_hclt_create(np_ptr(par), len(par), int(num_hidden_cats), int(num_cats), ctypes.byref(h)))
    return HcltCircuit(h, par, int(num_cats), int(num_hidden_cats))


def compile_circuit(node_type, child_ptr, child_idx, sum_logp, input_var, input_logp, num_vars, num_cats,
                    num_heads=0):
    """`CuMetaBitsProbCircuit(pc)` (src/bits_circuit.jl:39) for a DAG in flat form."""
    node_type = np.ascontiguousarray(node_type, np.uint8)
    child_ptr = np.ascontiguousarray(child_ptr, np.int32)
    child_idx = np.ascontiguousarray(child_idx, np.int32)
    sum_logp = np.ascontiguousarray(sum_logp, np.float32)
    input_var = np.ascontiguousarray(input_var, np.int32)
    input_logp = np.ascontiguousarray(input_logp, np.float32)
    h = H()
    check(lib.pcm_circuit_create(len(node_type), np_ptr(node_type), np_ptr(child_ptr), np_ptr(child_idx),
                                 np_ptr(sum_logp), np_ptr(input_var), np_ptr(input_logp), int(num_vars),
                                 int(num_cats), int(num_heads), ctypes.byref(h)))
    c = BitsCircuit(h)
    c.num_vars, c.num_cats, c.num_heads = int(num_vars), int(num_cats), int(num_heads)
    return c


def compile_multihead(node_type, child_ptr, child_idx, sum_logp, input_var, input_logp, num_vars, num_cats,
                      num_heads):
    """`CuMultiHeadBitsProbCircuit(pcs)` (src-jl/multi_head_pc/bit_circuit.jl:14-56): the
    last `num_heads` nodes of the description are the heads."""
    return compile_circuit(node_type, child_ptr, child_idx, sum_logp, input_var, input_logp, num_vars,
                           num_cats, num_heads)


def _compile_nodes(pcs, num_vars, heads):
    from . import nodes as N
    desc, order = N.describe(pcs)
    if num_vars is None:
        num_vars = int(desc["input_var"].max()) + 1
    c = compile_circuit(desc["node_type"], desc["child_ptr"], desc["child_idx"], desc["sum_logp"], desc["input_var"],
                        desc["input_logp"], num_vars, desc["num_cats"], heads)
    c.nodes = order            # description order: c.table("description2node")[i] is the node id of c.nodes[i]
    c.pcs = list(pcs) if heads else pcs
    return c


def CuBitsProbCircuit(pc, num_vars=None):
    """`CuBitsProbCircuit(pc)` / `CuMetaBitsProbCircuit(pc)` (src/bits_circuit.jl:39) for a
    circuit given as a DAG of `pcmi355.nodes`."""
    return _compile_nodes(pc, num_vars, 0)


def CuMultiHeadBitsProbCircuit(pcs, num_vars=None):
    """`CuMultiHeadBitsProbCircuit(pcs)` (src-jl/multi_head_pc/bit_circuit.jl:14-56): the roots
    `pcs` share one body and become the heads, in order."""
    pcs = list(pcs)
    if not pcs:
        raise ValueError("no heads given")
    return _compile_nodes(pcs, num_vars, len(pcs))


def node_maps(bpc):
    """(node id -> DAG node, DAG node -> node id) of a circuit compiled from `pcmi355.nodes`
    (`bpc.nodes_map` and its inverse, src-jl/multi_head_pc/transformation.jl:132-135).  Node ids
    are 1-based; DAG nodes that were folded into an edge have none, and of the DAG nodes that
    share an id (a node and its only child) the map keeps the one that owns the edges."""
    d2n = bpc.table("description2node")
    node2id, nodes_map = {}, {}
    for n, f in zip(bpc.nodes, d2n):
        if f > 0:
            node2id[id(n)] = int(f)
            if int(f) not in nodes_map or len(n.inputs) > 1:
                nodes_map[int(f)] = n
    return nodes_map, node2id


def write_back_parameters(bpc):
    """`update_parameters(bpc)` of ProbabilisticCircuits.jl as
    exps/LVD_for_imagenet/src/train_PG_top_level_pcs.jl:186 calls it: copies the device
    parameters into the DAG nodes the circuit was compiled from."""
    from .queries import vectorize_parameters
    pv = vectorize_parameters(bpc)
    nodes_map, _ = node_maps(bpc)
    e2p = bpc.table("edge2param")
    parent = bpc.table("edge_parent")
    pos = 0
    while pos < len(parent):
        end = pos
        while end < len(parent) and parent[end] == parent[pos]:
            end += 1
        n = nodes_map.get(int(parent[pos]))
        if n is not None and n.kind == 1 and e2p[pos] > 0:      # a run of product edges can carry the id of a one-child sum
            if len(n.params) != end - pos:
                raise RuntimeError("edge run does not match the sum node's children")
            n.params = pv[e2p[pos:end] - 1].astype(np.float32)
        pos = end
    ns = bpc.num_inner_params()
    C = bpc.num_cats
    for i, f in enumerate(bpc.table("input_node_ids")):
        n = nodes_map[int(f)]
        n.logps = pv[ns + i * C: ns + (i + 1) * C].astype(np.float32)
