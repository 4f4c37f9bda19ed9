"""Host-side circuit DAGs, the structure builders around the HCLT, and the flow-driven
structure changes (`prune_pc`, `grow_heads_by_flows`) against the DAG-level oracle."""
import itertools

import numpy as np
import pytest

from helpers import (random_dag, describe_dag, multihead_hclt, simple_multihead_circuit, log_dirichlet,
                     to_oracle_dag, from_oracle_dag)


def _all_assignments(V, C):
    return np.array(list(itertools.product(range(C), repeat=V)), np.uint8)


# ---- the DAG oracle itself ---------------------------------------------------------------------

def test_dag_oracle_values_equal_the_flat_oracle(oracle):
    import dag_oracle as D
    O = oracle
    rng = np.random.default_rng(3)
    for V, C in ((5, 3), (7, 4)):
        root = random_dag(V, C, rng)
        data = rng.integers(0, C, size=(40, V)).astype(np.uint8)
        fc = O.bits_compile(root, C, V)
        want = O.forward(fc, data, double=True)[-1]
        np.testing.assert_allclose(D.values([root], data)[id(root)], want, rtol=1e-10)


def test_dag_oracle_flows_are_derivatives_and_balance(oracle):
    import dag_oracle as D
    O = oracle
    rng = np.random.default_rng(4)
    V, C, B = 5, 3, 25
    heads = simple_multihead_circuit(C, rng) if False else None
    root = random_dag(V, C, rng)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    F, E, val = D.flows([root], data, np.ones((B, 1)))
    sums = [n for n in D.topo([root]) if n.kind == O.SUM]
    for n in sums:                                              # a sum node's edge flows add up to its flow
        np.testing.assert_allclose(sum(E[(id(n), i)] for i in range(len(n.children))), F[id(n)], rtol=1e-10, atol=1e-14)
    np.testing.assert_allclose(F[id(root)], 1.0)
    eps = 1e-6
    checked = 0
    for n in sums[:6]:
        for i in range(len(n.children)):
            keep = float(n.logps[i])
            lp = n.logps.astype(np.float64)
            n.logps = lp.copy(); n.logps[i] = keep + eps
            up = D.values([root], data)[id(root)].sum()
            n.logps = lp.copy(); n.logps[i] = keep - eps
            dn = D.values([root], data)[id(root)].sum()
            n.logps = lp.astype(np.float32)
            np.testing.assert_allclose(E[(id(n), i)].sum(), (up - dn) / (2 * eps), rtol=2e-4, atol=1e-6)
            checked += 1
    assert checked > 5


def test_dag_oracle_prune_properties(oracle):
    import dag_oracle as D
    O = oracle
    rng = np.random.default_rng(5)
    V, C, B = 4, 3, 60
    root = random_dag(V, C, rng, width=3)
    prods = root.children
    heads = [O.summate(*prods, logps=log_dirichlet(rng, len(prods))) for _ in range(3)]
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    mask = np.zeros((B, 3)); mask[np.arange(B), rng.integers(0, 3, B)] = 1
    F, E, val = D.flows(heads, data, mask)
    sums = {k: v.sum() for k, v in E.items()}
    same = D.prune(heads, sums, -1.0)
    v2 = D.values(same, data)
    for h, s in zip(heads, same):
        np.testing.assert_allclose(v2[id(s)], val[id(h)], rtol=1e-6)
    thr = np.median(list(sums.values()))
    pruned = D.prune(heads, sums, thr)
    allx = _all_assignments(V, C)
    pv = D.values(pruned, allx)
    for p in pruned:                                            # still a distribution
        np.testing.assert_allclose(np.exp(pv[id(p)]).sum(), 1.0, rtol=1e-5)
    old = {id(n): n for n in D.topo(heads)}
    n_old = sum(len(n.children) for n in old.values() if n.kind == O.SUM)
    n_new = sum(len(n.children) for n in D.topo(pruned) if n.kind == O.SUM)
    assert n_new < n_old
    for h, p in zip(heads, pruned):                             # exactly the edges above the threshold survive
        want = [i for i in range(len(h.children)) if sums[(id(h), i)] > thr] or [int(np.argmax(h.logps))]
        if len(want) > 1:
            assert len(p.children) == len(want)


# ---- host DAGs and structure builders ------------------------------------------------------------

def test_describe_matches_the_flat_description_of_the_same_dag(oracle):
    from pcmi355 import nodes as N
    rng = np.random.default_rng(6)
    root = random_dag(6, 4, rng)
    heads = [oracle.summate(*root.children, logps=log_dirichlet(rng, len(root.children))) for _ in range(2)]
    mine, _ = from_oracle_dag(heads)
    desc, order = N.describe(mine)
    want = describe_dag(heads)
    for k in ("node_type", "child_ptr", "child_idx", "sum_logp", "input_var", "input_logp"):
        np.testing.assert_array_equal(desc[k], want[k], err_msg=k)
    assert desc["num_cats"] == 4 and len(order) == len(desc["node_type"])
    assert N.num_nodes(mine) == len(order) and N.num_edges(mine) == len(desc["child_idx"])
    back, _ = to_oracle_dag(mine)
    for k, v in describe_dag(back).items():
        np.testing.assert_array_equal(v, want[k])
    with pytest.raises(ValueError):
        N.describe([mine[0], mine[0]])
    with pytest.raises(ValueError):
        N.summate([])
    with pytest.raises(ValueError):
        N.summate(mine, params=[0.0])


def test_init_parameters_and_counts():
    from pcmi355 import nodes as N
    a, b = N.categorical(0, 4), N.categorical(1, 4)
    pc = N.summate(N.multiply(a, b), N.multiply(N.categorical(0, 4), N.categorical(1, 4)))
    assert N.num_parameters(pc) == 1 + 4 * 3
    N.init_parameters(pc, perturbation=0.4, rng=np.random.default_rng(0))
    for n in N.linearize(pc):
        lp = n.params if N.issum(n) else n.logps if N.isinput(n) else None
        if lp is not None:
            np.testing.assert_allclose(np.exp(lp.astype(np.float64)).sum(), 1.0, rtol=1e-6)
            w = np.exp(lp - lp.max())
            assert w.min() / w.max() >= 0.6 / 1.4 - 1e-6            # uniform(0.6, 1.4) before normalising
    seen = []
    N.foreach_down(lambda n: seen.append(n), pc)
    assert seen[0] is pc and N.variables(pc) == [0, 1]


def test_clt_edges2parent_roots_at_the_lowest_centre():
    from pcmi355 import structures as S
    np.testing.assert_array_equal(S.clt_edges2parent([(0, 1), (1, 2), (2, 3), (3, 4)]), [1, 2, -1, 2, 3])
    np.testing.assert_array_equal(S.clt_edges2parent([(3, 2), (0, 1), (2, 1)]), [1, -1, 1, 2])       # centres 1 and 2
    np.testing.assert_array_equal(S.clt_edges2parent([(0, 3), (1, 3), (2, 3)]), [3, 3, 3, -1])      # a star
    with pytest.raises(ValueError):
        S.clt_edges2parent([(0, 1), (2, 3), (0, 1)], 4)
    with pytest.raises(ValueError):
        S.clt_edges2parent([(0, 1)], 3)


def test_hclt_pc_is_the_hclt_of_the_block_engine(oracle):
    """Same flat sizes as the oracle's HCLT DAG, and a distribution (brute force)."""
    import dag_oracle as D
    from pcmi355 import nodes as N, structures as S
    O = oracle
    rng = np.random.default_rng(7)
    parent = O.random_tree(6, rng, 3)
    K, C = 3, 4
    pc = S.hclt_pc(parent, C, K)
    N.init_parameters(pc, 0.4, rng)
    (root,), _ = to_oracle_dag(pc)
    theta, leaf = O.random_hclt_params(parent, K, C, rng)
    ref = O.bits_compile(O.hclt_dag(parent, K, C, theta, leaf), C, 6)
    got = O.bits_compile(root, C, 6)
    assert (got.n_nodes, got.n_edges) == (ref.n_nodes, ref.n_edges)
    np.testing.assert_array_equal(got.edge_parent(), ref.edge_parent())
    np.testing.assert_array_equal(got.type, ref.type)
    small = S.hclt_pc(np.array([-1, 0, 0, 1], np.int32), 2, 2)
    N.init_parameters(small, 0.4, rng)
    (r,), _ = to_oracle_dag(small)
    np.testing.assert_allclose(np.exp(D.values([r], _all_assignments(4, 2))[id(r)]).sum(), 1.0, rtol=1e-6)
    # variable groups: tree node i covers two observed variables
    groups = S.group_vars_by_grid(2, 4, 1, patch_h=1, patch_w=2)
    assert groups == [(0, [0, 1]), (2, [2, 3]), (4, [4, 5]), (6, [6, 7])]
    assert S.group_vars_by_cgrid(2, 2, 2, patch_h=2, patch_w=1) == [(0, [0, 2, 4, 6]), (1, [1, 3, 5, 7])]
    g = S.hclt_pc(np.array([-1, 0, 0], np.int32), 2, 2, variable_groups=[(0, [0, 1]), (2, [2, 3]), (4, [4, 5])])
    N.init_parameters(g, 0.4, rng)
    (r,), _ = to_oracle_dag(g)
    assert N.variables(g) == list(range(6))
    np.testing.assert_allclose(np.exp(D.values([r], _all_assignments(6, 2))[id(r)]).sum(), 1.0, rtol=1e-6)


def test_customized_hclt_shape_and_edge_parameters(oracle):
    import dag_oracle as D
    from pcmi355 import nodes as N, structures as S
    rng = np.random.default_rng(8)
    K = C = 3
    edges = [(0, 1), (1, 2), (1, 3)]

    def leaf_pcs(v, K):
        out = []
        for i in range(K):
            ps = rng.random(K) * 0.01
            ps[i] += 1.0
            out.append(N.input_node(v, np.log(ps / ps.sum())))
        return out

    w = np.array([[1.0, 1, 2], [2, 1, 1], [1, 3, 1]])
    pc = S.customized_hclt(edges, K, leaf_pcs, lambda a, b, K: w)
    sums = [n for n in N.linearize(pc) if N.issum(n)]
    assert len(sums) == 3 * K + 1                                   # a K x K block per edge, and the root
    for n in sums[:-1]:
        assert any(np.allclose(np.exp(n.params), w[i] / w[i].sum(), rtol=1e-6) for i in range(K))
    (r,), _ = to_oracle_dag(pc)
    np.testing.assert_allclose(np.exp(D.values([r], _all_assignments(4, C))[id(r)]).sum(), 1.0, rtol=1e-5)
    bare = S.customized_hclt(edges, K, leaf_pcs, parameterize_leaf_edge=False)
    assert len([n for n in N.linearize(bare) if N.issum(n)]) == 0 * K + 1   # root 1 has only leaf children
    with pytest.raises(ValueError):
        S.customized_hclt(edges, K, lambda v, K: leaf_pcs(v, K)[:2])


def test_joined_hclt_merges_regions(oracle):
    import dag_oracle as D
    from pcmi355 import nodes as N, structures as S
    rng = np.random.default_rng(9)
    t1 = S.clt_edges2parent([(0, 1), (1, 2), (2, 3), (3, 4)])
    t2 = S.clt_edges2parent([(0, 2), (2, 1), (1, 3), (3, 4)])
    one = S.joined_hclt_from_clts([t1], 2, 3)
    twice = S.joined_hclt_from_clts([t1, t1.copy()], 2, 3)
    assert len(one) == 2 and N.num_nodes(twice) == N.num_nodes(one) and N.num_edges(twice) == N.num_edges(one)
    both = S.joined_hclt_from_clts([t1, t2], 2, 3)
    assert N.num_nodes(both) > N.num_nodes(one)
    N.init_parameters(both, 0.4, rng)
    rs, _ = to_oracle_dag(both)
    v = D.values(rs, _all_assignments(5, 3))
    for r in rs:
        np.testing.assert_allclose(np.exp(v[id(r)]).sum(), 1.0, rtol=1e-5)
    top = [n for n in N.linearize(both) if N.issum(n)][-1]
    assert top is both[-1] and len(top.inputs) >= 2


# ---- on the GPU ----------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355
    return torch, pcmi355


def _heads_and_data(oracle, rng, V=6, C=4, H=3, B=96):
    root = random_dag(V, C, rng, width=3)
    while len(root.children) < 3:
        root = random_dag(V, C, rng, width=3)
    heads = [oracle.summate(*root.children, logps=log_dirichlet(rng, len(root.children))) for _ in range(H)]
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    mask = np.zeros((B, H), np.float32)
    mask[np.arange(B), rng.integers(0, H, B)] = 1.0
    return heads, data, mask


@pytest.mark.gpu
def test_compiled_dag_node_maps_and_node_flow_sums(gpu, oracle):
    import dag_oracle as D
    torch, P = gpu
    rng = np.random.default_rng(11)
    heads, data, mask = _heads_and_data(oracle, rng)
    pcs, conv = from_oracle_dag(heads)
    bpc = P.CuMultiHeadBitsProbCircuit(pcs)
    assert bpc.size("description_nodes") == len(bpc.nodes) and bpc.size("heads") == 3
    d, hm = torch.from_numpy(data).cuda(), torch.from_numpy(mask).cuda()
    ll = P.loglikelihoods(bpc, d).cpu().numpy()
    F, E, val = D.flows(heads, data, mask.astype(np.float64))
    np.testing.assert_allclose(ll, np.stack([val[id(h)] for h in heads], 1), rtol=2e-5)
    with pytest.raises(P.PcmError):
        bpc.node_flow_sums()                                        # no flows yet
    P.probs_flows_circuit(bpc, d, head_mask=hm)
    sums = bpc.node_flow_sums()
    nodes_map, node2id = P.node_maps(bpc)
    back = {id(v): k for k, v in conv.items()}                      # product node -> oracle node
    checked = 0
    for n in bpc.nodes:
        f = node2id.get(id(n))
        if f is None or nodes_map[f] is not n:
            continue
        np.testing.assert_allclose(sums[f - 1], F[back[id(n)]].sum(), rtol=2e-4, atol=1e-4)
        checked += 1
    assert checked >= 15
    heads_tab = bpc.table("heads")
    assert [node2id[id(p)] for p in pcs] == list(heads_tab)
    # edge statistics per (sum node, child): an edge's rank in its parent's run is the child's index
    ea, _ = bpc.get_aggregates()
    parent = bpc.table("edge_parent")
    first = {}
    for e, p in enumerate(parent):
        first.setdefault(int(p), e)
    for n in bpc.nodes:
        f = node2id.get(id(n))
        if f is not None and nodes_map[f] is n and n.kind == 1 and len(n.inputs) > 1:
            for i in range(len(n.inputs)):
                np.testing.assert_allclose(ea[first[f] + i], E[(back[id(n)], i)].sum(), rtol=2e-4, atol=1e-4)
    hc = P.hclt_from_clt(np.array([-1, 0], np.int32), 4, 16)
    with pytest.raises(P.PcmError):
        hc.node_flow_sums()


@pytest.mark.gpu
def test_structure_builders_compile_and_run(gpu, oracle):
    """hclt_pc with variable groups, customized_hclt and joined_hclt through the layered engine
    against the DAG oracle; hclt_pc with one variable per group against the block engine."""
    import dag_oracle as D
    torch, P = gpu
    N, S = P.nodes, P
    rng = np.random.default_rng(21)
    B = 40
    # variable groups: 4 tree nodes over 8 observed variables
    groups = S.group_vars_by_grid(2, 4, 1, patch_h=1, patch_w=2)
    pc = S.hclt_pc(np.array([-1, 0, 0, 1], np.int32), 5, 4, variable_groups=groups)
    N.init_parameters(pc, 0.4, rng)
    data = rng.integers(0, 5, size=(B, 8)).astype(np.uint8)
    bpc = P.CuBitsProbCircuit(pc)
    (ro,), _ = to_oracle_dag(pc)
    np.testing.assert_allclose(P.loglikelihoods(bpc, torch.from_numpy(data).cuda()).cpu().numpy(),
                               D.values([ro], data)[id(ro)], rtol=2e-5)
    # one variable per group: the same function as the block engine's HCLT with these parameters
    parent = oracle.random_tree(7, rng, 3)
    pc1 = S.hclt_pc(parent, 6, 16)
    N.init_parameters(pc1, 0.4, rng)
    gen = P.CuBitsProbCircuit(pc1)
    blk = P.hclt_from_clt(parent, 6, 16)
    assert blk.num_parameters() == gen.num_parameters() and blk.num_nodes() == gen.num_nodes()
    P.update_parameters(blk, P.vectorize_parameters(gen))
    d1 = torch.from_numpy(rng.integers(0, 6, size=(B, 7)).astype(np.uint8)).cuda()
    np.testing.assert_allclose(P.loglikelihoods(blk, d1).cpu().numpy(), P.loglikelihoods(gen, d1).cpu().numpy(), rtol=2e-5)
    for t in ("edge2param", "edge_parent", "edge_prime", "edge_sub"):
        np.testing.assert_array_equal(blk.table(t), gen.table(t), err_msg=t)
    # joined trees: K heads over the full scope; EM on the multi-head circuit raises the mixture likelihood
    t1 = S.clt_edges2parent([(0, 1), (1, 2), (2, 3), (3, 4)])
    t2 = S.clt_edges2parent([(0, 2), (2, 1), (1, 3), (3, 4)])
    roots = S.joined_hclt_from_clts([t1, t2], 3, 4)
    N.init_parameters(roots, 0.4, rng)
    dj = rng.integers(0, 4, size=(B, 5)).astype(np.uint8)
    mh = P.CuMultiHeadBitsProbCircuit(roots)
    ro, _ = to_oracle_dag(roots)
    vals = D.values(ro, dj)
    np.testing.assert_allclose(P.loglikelihoods(mh, torch.from_numpy(dj).cuda()).cpu().numpy(),
                               np.stack([vals[id(r)] for r in ro], 1), rtol=2e-5)
    hm = torch.ones((B, 3), device="cuda")
    lls = P.mini_batch_em_for_multihead_pc(mh, torch.from_numpy(dj).cuda(), hm, 3, batch_size=B, pseudocount=0.1,
                                           param_inertia=0.5, shuffle="none")
    assert lls[-1] > lls[0]
    # joined_hclt end to end: trees learned on the device from two datasets
    ds = [torch.from_numpy(rng.integers(0, 4, size=(200, 5)).astype(np.uint8)).cuda() for _ in range(2)]
    jr = S.joined_hclt(ds, 2, num_cats=4)
    assert len(jr) == 2 and N.variables(jr) == [0, 1, 2, 3, 4]


@pytest.mark.gpu
@pytest.mark.parametrize("threshold", [-1.0, 0.02, 0.15])
def test_prune_pc_matches_the_oracle(gpu, oracle, threshold):
    import dag_oracle as D
    torch, P = gpu
    rng = np.random.default_rng(12)
    heads, data, mask = _heads_and_data(oracle, rng, B=128)
    pcs, _ = from_oracle_dag(heads)
    d, hm = torch.from_numpy(data).cuda(), torch.from_numpy(mask).cuda()
    got = P.prune_pc(pcs, d, hm, batch_size=48, prune_threshold=threshold)       # 2 full batches, 32 examples left out
    used = 96
    F, E, val = D.flows(heads, data[:used], mask[:used].astype(np.float64))
    want = D.prune(heads, {k: v.sum() for k, v in E.items()}, threshold * len(data))
    got_o, _ = to_oracle_dag(got)
    probe = rng.integers(0, 4, size=(50, 6)).astype(np.uint8)
    vg, vw = D.values(got_o, probe), D.values(want, probe)
    for g, w in zip(got_o, want):
        np.testing.assert_allclose(vg[id(g)], vw[id(w)], rtol=1e-5)
    count = lambda rs: (len(D.topo(rs)), sum(len(n.children) for n in D.topo(rs)))
    assert count(got_o) == count(want)
    if threshold < 0:
        assert count(got_o) == count(heads)
    bpc = P.CuMultiHeadBitsProbCircuit(got)                                       # the result compiles and runs
    np.testing.assert_allclose(P.loglikelihoods(bpc, torch.from_numpy(probe).cuda()).cpu().numpy(),
                               np.stack([vw[id(w)] for w in want], 1), rtol=2e-5)


@pytest.mark.gpu
def test_grow_heads_by_flows(gpu, oracle):
    import dag_oracle as D
    torch, P = gpu
    N = P.nodes
    rng = np.random.default_rng(13)
    heads, data, mask = _heads_and_data(oracle, rng, B=100)
    mask[:, 2] = 0.0                                                             # head 2 sees no data
    mask[mask.sum(1) == 0, 0] = 1.0
    pcs, _ = from_oracle_dag(heads)
    d, hm = torch.from_numpy(data).cuda(), torch.from_numpy(mask).cuda()
    probe = rng.integers(0, 4, size=(60, 6)).astype(np.uint8)
    old = D.values(heads, probe)
    # without noise every copy computes what its original did
    grown = P.grow_heads_by_flows(pcs, d, hm, batch_size=32, sigma=0.0, node_selection_args={"grow_frac": 0.5},
                                  rng=np.random.default_rng(1))
    assert len(pcs) < len(grown) <= 2 * len(pcs)
    go, _ = to_oracle_dag(grown)
    new = D.values(go, probe)
    for i, h in enumerate(heads):
        np.testing.assert_allclose(new[id(go[i])], old[id(h)], rtol=1e-5)
    aggr = P.aggregate_node_flows(P.CuMultiHeadBitsProbCircuit(pcs), d, hm, 32)
    assert N.num_nodes(grown) > N.num_nodes(pcs)
    for extra in go[len(pcs):]:                                                  # a split head's second copy
        assert any(np.allclose(new[id(extra)], old[id(h)], rtol=1e-5) for h in heads)
    # everything split
    full = P.grow_heads_by_flows(pcs, d, hm, batch_size=100, sigma=0.0, node_selection_args={"grow_frac": 1.0})
    n_flow = int((aggr >= 1e-8).sum())
    assert len(full) == len(pcs) + sum(1 for p in pcs if aggr[P.node_maps(P.CuMultiHeadBitsProbCircuit(pcs))[1][id(p)] - 1] >= 1e-8)
    assert n_flow > 0
    # with noise: still normalised, and it runs
    noisy = P.grow_heads_by_flows(pcs, d, hm, batch_size=32, sigma=0.2, cross_term_discount=0.2,
                                  node_selection_args={"grow_frac": 0.3}, rng=np.random.default_rng(2))
    for n in N.linearize(noisy):
        if N.issum(n):
            np.testing.assert_allclose(np.exp(n.params.astype(np.float64)).sum(), 1.0, rtol=1e-5)
        elif N.isinput(n):
            np.testing.assert_allclose(np.exp(n.logps.astype(np.float64)).sum(), 1.0, rtol=1e-5)
    bpc = P.CuMultiHeadBitsProbCircuit(noisy)
    no, _ = to_oracle_dag(noisy)
    vn = D.values(no, probe)
    np.testing.assert_allclose(P.loglikelihoods(bpc, torch.from_numpy(probe).cuda()).cpu().numpy(),
                               np.stack([vn[id(r)] for r in no], 1), rtol=2e-5)
    with pytest.raises(ValueError):
        P.grow_heads_by_flows(pcs, d, hm, batch_size=32, node_selection_method="top", node_selection_args={})


@pytest.mark.gpu
def test_write_back_parameters_after_em(gpu, oracle):
    import dag_oracle as D
    torch, P = gpu
    rng = np.random.default_rng(14)
    heads, data, mask = _heads_and_data(oracle, rng, B=128)
    pcs, _ = from_oracle_dag(heads)
    bpc = P.CuMultiHeadBitsProbCircuit(pcs)
    d, hm = torch.from_numpy(data).cuda(), torch.from_numpy(mask).cuda()
    P.mini_batch_em_for_multihead_pc(bpc, d, hm, 2, batch_size=64, pseudocount=0.1, param_inertia=0.5, shuffle="none")
    before, _ = to_oracle_dag(pcs)
    P.write_back_parameters(bpc)
    after, _ = to_oracle_dag(pcs)
    ll = P.loglikelihoods(bpc, d).cpu().numpy()
    va = D.values(after, data)
    np.testing.assert_allclose(ll, np.stack([va[id(r)] for r in after], 1), rtol=2e-5)
    vb = D.values(before, data)
    assert np.abs(np.stack([vb[id(r)] for r in before], 1) - ll).max() > 1e-3    # the parameters did move


@pytest.mark.gpu
def test_trained_heads_through_a_jpc_file(gpu, oracle, tmp_path):
    """write_mhpc / read_mhpc (src-jl/multi_head_pc/io.jl:2-9) around a trained circuit: the heads read back
    compile to a circuit with the same likelihoods, to the bit."""
    torch, P = gpu
    rng = np.random.default_rng(15)
    heads, data, mask = _heads_and_data(oracle, rng, B=96)
    pcs, _ = from_oracle_dag(heads)
    bpc = P.CuMultiHeadBitsProbCircuit(pcs)
    d, hm = torch.from_numpy(data).cuda(), torch.from_numpy(mask).cuda()
    P.mini_batch_em_for_multihead_pc(bpc, d, hm, 1, batch_size=48, pseudocount=0.1, param_inertia=0.5, shuffle="none")
    P.write_back_parameters(bpc)
    path = tmp_path / "heads.jpc.gz"
    P.write_mhpc(path, pcs)
    back = P.read_mhpc(path)
    assert len(back) == len(pcs)
    bpc2 = P.CuMultiHeadBitsProbCircuit(back)
    np.testing.assert_array_equal(P.loglikelihoods(bpc2, d).cpu().numpy(), P.loglikelihoods(bpc, d).cpu().numpy())
    again = P.CuMultiHeadBitsProbCircuit(pcs)
    np.testing.assert_array_equal(P.vectorize_parameters(again), P.vectorize_parameters(bpc))


@pytest.mark.gpu
def test_patch_circuits_feed_the_top_level_circuit(gpu, oracle):
    """exps/LVD_for_imagenet/src/train_PG_top_level_pcs.jl:82-195 in small: per-head patch
    log-likelihoods become the soft evidence of a customized HCLT over the patches."""
    import dag_oracle as D
    torch, P = gpu
    N = P.nodes
    O = oracle
    rng = np.random.default_rng(15)
    Vp, C, K, n_patches, B = 5, 6, 16, 4, 64
    parent = O.random_tree(Vp, rng, 3)
    circuits, heads_o = [], []
    for H in (3, 2):
        hs, _ = multihead_hclt(parent, K, C, H, rng)
        pcs, _ = from_oracle_dag(hs)
        circuits.append(P.CuMultiHeadBitsProbCircuit(pcs, num_vars=Vp))
        heads_o.append(hs)
    patches = [rng.integers(0, C, size=(B, Vp)).astype(np.uint8) for _ in range(n_patches)]
    ev = P.patch_level_evidence(circuits, [torch.from_numpy(p).cuda() for p in patches], batch_size=24)
    assert ev.shape == (B, n_patches, 5)
    want = np.stack([np.concatenate([np.stack([D.values(hs, p)[id(h)] for h in hs], 1) for hs in heads_o], 1) for p in patches], 1)
    np.testing.assert_allclose(ev.cpu().numpy(), want, rtol=2e-5)
    n_clusters = 5

    def leaf_pcs(v, K):
        out = []
        for i in range(K):
            ps = rng.random(K).astype(np.float32) * 0.01
            ps[i] += 1.0
            out.append(N.input_node(v, np.log(ps / ps.sum())))
        return out

    top = P.customized_hclt([(0, 1), (1, 2), (2, 3)], n_clusters, leaf_pcs, lambda a, b, K: np.full((K, K), 0.2))
    N.init_parameters([n for n in [top]], perturbation=0.0)                       # uniform sums; leaves rebuilt below
    for n in N.linearize(top):
        if N.isinput(n):
            n.logps = log_dirichlet(rng, n_clusters)
        elif N.issum(n):
            n.params = log_dirichlet(rng, len(n.params))
    bpc = P.CuBitsProbCircuit(top)
    ll = P.loglikelihoods(bpc, ev).cpu().numpy()
    (ro,), _ = to_oracle_dag(top)
    fc = O.bits_compile(ro, n_clusters, n_patches)
    np.testing.assert_allclose(ll, O.forward_soft(fc, want.astype(np.float32))[-1], rtol=2e-5)
    lls = P.mini_batch_em_with_reg(bpc, ev, 4, batch_size=32, pseudocount=0.1, param_inertia=0.5, shuffle="none")
    assert lls[-1] > lls[0]
    P.write_back_parameters(bpc)
    (ro2,), _ = to_oracle_dag(top)
    fc2 = O.bits_compile(ro2, n_clusters, n_patches)
    np.testing.assert_allclose(P.loglikelihoods(bpc, ev).cpu().numpy(), O.forward_soft(fc2, want.astype(np.float32))[-1], rtol=2e-5)
