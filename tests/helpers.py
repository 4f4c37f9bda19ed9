"""Shared builders for the parity tests (CPU side only: numpy + the oracle)."""
import numpy as np

import pc_oracle as O


def block_theta(parent, K, theta_dict):
    """{v: [K, K]} -> dense [V, K, K] (zeros for leaf tree nodes)."""
    V = len(parent)
    out = np.zeros((V, K, K), np.float32)
    for v, t in theta_dict.items():
        out[v] = t
    return out


def make_hclt(V, K, C, seed, kind="dirichlet", max_children=3, parent=None):
    rng = np.random.default_rng(seed)
    if parent is None:
        parent = O.random_tree(V, rng, max_children)
    theta, leaf = O.random_hclt_params(parent, K, C, rng, kind)
    fc = O.hclt_flat(parent, K, C, theta, leaf)
    return parent, theta, leaf, fc


def correlated_data(N, V, C, seed, parent=None):
    """uint8 data with tree-shaped dependence so flows are not uniform."""
    rng = np.random.default_rng(seed)
    x = np.zeros((N, V), np.int64)
    if parent is None:
        parent = np.arange(-1, V - 1)
    order = O.clt_bottom_up(parent)[::-1]
    for v in order:
        if parent[v] < 0:
            x[:, v] = rng.integers(0, C, N)
        else:
            step = rng.integers(-2, 3, N)
            fresh = rng.random(N) < 0.15
            x[:, v] = np.where(fresh, rng.integers(0, C, N), (x[:, parent[v]] + step) % C)
    return x.astype(np.uint8)


def oracle_em_reference(fc, data, idx, pseudocount, inertia, double=False):
    """One EM step on the oracle; returns LL, theta blocks, leaf [V,K,C], edge_aggr blocks, leaf flows."""
    ll, logp, leaf, ea, lf = O.em_step(fc, data, idx, pseudocount, inertia, double=double)
    K, C, V = fc.meta["K"], fc.C, fc.V
    new = fc.copy()
    new.logp = logp
    new.leaf_logp = leaf
    th, lf_new = O.hclt_block_params(new)
    return ll, th, lf_new, O.hclt_block_aggr(fc, ea), lf.reshape(V, K, C)


def rel_err(a, b, floor=1e-30):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return np.abs(a - b) / np.maximum(np.abs(b), floor)


def three_way(got, exact, single):
    """Worst relative distances, as probabilities, between three sets of log-parameters: (library vs float64
    oracle, float32 oracle vs float64 oracle, library vs float32 oracle).  Each argument is (theta blocks by
    tree node -- the library's as a dense array --, leaf tables)."""
    def rel(a, b):
        a, b = np.exp(np.asarray(a, np.float64)), np.exp(np.asarray(b, np.float64))
        return float((np.abs(a - b) / b).max())
    (th, lf), (th64, lf64), (th32, lf32) = got, exact, single
    sums = (max(rel(th[v][:b.shape[0]], b) for v, b in th64.items()),
            max(rel(th32[v], b) for v, b in th64.items()),
            max(rel(th[v][:b.shape[0]], th32[v]) for v, b in th64.items()))
    leaves = (rel(lf, lf64), rel(lf32, lf64), rel(lf, lf32))
    return sums, leaves


def assert_three_way(got, exact, single, bar, label=""):
    """The library must be within `bar` of the exact (float64) result, whatever the float32 oracle -- the
    reference's arithmetic, whose log-values lose absolute precision with the depth of the circuit -- manages, and
    where the two float32 results are further apart than `bar`, the float32 oracle's own error must account for
    it (the distances obey the triangle inequality up to the different denominators)."""
    sums, leaves = three_way(got, exact, single)
    print(f"\n{label}: sum parameters library/f64 {sums[0]:.2e} f32/f64 {sums[1]:.2e} library/f32 {sums[2]:.2e}; "
          f"leaf parameters {leaves[0]:.2e} {leaves[1]:.2e} {leaves[2]:.2e}")
    for e_gpu, e_f32, e_gpu32 in (sums, leaves):
        assert e_gpu < bar, (label, sums, leaves)
        assert e_gpu32 < max(bar, 1.01 * (e_gpu + e_f32)), (label, sums, leaves)
    return sums, leaves


def describe_dag(roots):
    """Oracle DAG (pc_oracle.Node) -> the flat description pcm_circuit_create takes:
    children before parents, the given roots last (several roots = heads of a multi-head
    circuit).  Returns a dict of numpy arrays."""
    roots = list(roots)
    root_ids = {id(r) for r in roots}
    order, seen = [], set()

    def visit(n):
        if id(n) in seen:
            return
        seen.add(id(n))
        for c in n.children:
            visit(c)
        if id(n) not in root_ids:
            order.append(n)

    for r in roots:
        visit(r)
    order += roots
    index = {id(n): i for i, n in enumerate(order)}
    node_type = np.array([n.kind for n in order], np.uint8)
    child_ptr = np.zeros(len(order) + 1, np.int32)
    child_idx, sum_logp, input_var, input_logp = [], [], [], []
    for i, n in enumerate(order):
        for q, c in enumerate(n.children):
            child_idx.append(index[id(c)])
            sum_logp.append(float(n.logps[q]) if n.kind == O.SUM else 0.0)
        child_ptr[i + 1] = len(child_idx)
        input_var.append(n.var if n.kind == O.INPUT else -1)
        if n.kind == O.INPUT:
            input_logp.append(np.asarray(n.logps, np.float32))
    return dict(node_type=node_type, child_ptr=child_ptr, child_idx=np.array(child_idx, np.int32),
                sum_logp=np.array(sum_logp, np.float32), input_var=np.array(input_var, np.int32),
                input_logp=np.concatenate(input_logp).astype(np.float32))


def log_dirichlet(rng, n):
    x = rng.exponential(size=n) + 1e-3
    return np.log(x / x.sum()).astype(np.float32)


def simple_3vars_circuit(C, rng=None, weights=None):
    """test/helpers/simple_circuits.jl:4-14: summate(multiply(n11, n21, n31), multiply(n12, n22, n32))."""
    def leaf(v):
        lp = np.full(C, -np.log(C), np.float32) if rng is None else log_dirichlet(rng, C)
        return O.input_node(v, lp)
    n11, n21, n31 = leaf(0), leaf(1), leaf(2)
    n12, n22, n32 = leaf(0), leaf(1), leaf(2)
    w = None if weights is None else np.log(np.asarray(weights, np.float32))
    return O.summate(O.multiply(n11, n21, n31), O.multiply(n12, n22, n32), logps=w)


def simple_multihead_circuit(C, rng=None):
    """test/helpers/simple_circuits.jl:54-66: two sum heads over the same two 3-way products."""
    def leaf(v):
        lp = np.full(C, -np.log(C), np.float32) if rng is None else log_dirichlet(rng, C)
        return O.input_node(v, lp)
    n11, n21, n31 = leaf(0), leaf(1), leaf(2)
    n12, n22, n32 = leaf(0), leaf(1), leaf(2)
    n1, n2 = O.multiply(n11, n21, n31), O.multiply(n12, n22, n32)
    return [O.summate(n1, n2), O.summate(n1, n2)]


def random_dag(V, C, rng, width=4, depth=3):
    """A random smooth & decomposable circuit with shared sub-circuits: a balanced
    variable-partition tree; each region holds `width` sum nodes over products that pair
    (or triple) children regions' nodes; region nodes are reused by several parents."""
    def region(vars_, d):
        if len(vars_) == 1:
            return [O.input_node(int(vars_[0]), log_dirichlet(rng, C)) for _ in range(width)]
        nparts = 3 if (len(vars_) >= 3 and rng.random() < 0.4) else 2
        parts = np.array_split(vars_, nparts)
        kids = [region(p, d + 1) for p in parts]
        outs = []
        nsum = 1 if d == 0 else width
        prods = []
        for _ in range(width + 1):
            prods.append(O.multiply(*[k[rng.integers(len(k))] for k in kids]))
        for _ in range(nsum):
            m = int(rng.integers(1, len(prods) + 1))
            sel = rng.choice(len(prods), size=m, replace=False)
            outs.append(O.summate(*[prods[q] for q in sel], logps=log_dirichlet(rng, m)))
        return outs
    return region(np.arange(V), 0)[0]


def multihead_hclt(parent, K, C, H, rng):
    """A multi-head HCLT as the patch circuits of the progressive-growing experiments use it:
    one HCLT body, H head sum nodes over the K products under the root
    (exps/progressive_growing/parallel_PG.jl:214-225 builds such circuits for
    CuMultiHeadBitsProbCircuit).  Returns (heads, body root)."""
    theta, leaf = O.random_hclt_params(parent, K, C, rng)
    root = O.hclt_dag(parent, K, C, theta, leaf)
    prods = root.children
    heads = [O.summate(*prods, logps=log_dirichlet(rng, len(prods))) for _ in range(H)]
    return heads, root


def to_oracle_dag(pcs):
    """pcmi355.nodes DAG -> pc_oracle.Node DAG (shared nodes stay shared).  Returns the list of
    converted roots and the map id(product node) -> oracle node."""
    from pcmi355 import nodes as N
    roots = list(pcs) if isinstance(pcs, (list, tuple)) else [pcs]
    conv = {}
    for n in N.linearize(roots):
        if n.kind == N.INPUT:
            conv[id(n)] = O.input_node(n.var, n.logps)
        elif n.kind == N.MUL:
            conv[id(n)] = O.multiply(*[conv[id(c)] for c in n.inputs])
        else:
            conv[id(n)] = O.summate(*[conv[id(c)] for c in n.inputs], logps=n.params)
    return [conv[id(r)] for r in roots], conv


def from_oracle_dag(roots):
    """pc_oracle.Node DAG -> pcmi355.nodes DAG.  Returns (converted roots, map id(oracle node) -> node)."""
    import dag_oracle
    from pcmi355 import nodes as N
    conv = {}
    for n in dag_oracle.topo(list(roots)):
        if n.kind == O.INPUT:
            conv[id(n)] = N.input_node(n.var, n.logps)
        elif n.kind == O.MUL:
            conv[id(n)] = N.multiply([conv[id(c)] for c in n.children])
        else:
            conv[id(n)] = N.summate([conv[id(c)] for c in n.children], params=n.logps)
    return [conv[id(r)] for r in roots], conv
