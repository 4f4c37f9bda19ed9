"""Pins the CPU oracle (test infrastructure) against facts that do not depend on it:
brute-force enumeration of latent states, closed forms and known answers quoted from the
reference's own tests, finite differences in float64, textbook EM properties, and the
statistics of exact samples.  A dropped term, a transposed parameter block, a wrong child
or a wrong sign fails at least one of these."""
import itertools

import numpy as np
import pytest
from scipy.special import logsumexp

import pc_oracle as O
from helpers import (make_hclt, correlated_data, simple_3vars_circuit, simple_multihead_circuit, random_dag,
                     log_dirichlet)


# ------------------------------------------------------------------------------------
# forward
# ------------------------------------------------------------------------------------

def brute_force_hclt_ll(parent, K, theta, leaf, x):
    """log p(x) of the HCLT of src/structures/hclts.jl:100-145 by summing the joint over
    every assignment of the inner tree nodes' hidden states (float64).  Hidden state of
    tree node v: j_v; its sum parameters are theta_v[j_parent(v), j_v] (the root's parent
    state is 0, :137 keeps circuits[1]); observed leaf of v: leaf[v, j_v, x_v]; a leaf
    tree node c has no state of its own and contributes leaf[c, j_parent(c), x_c]."""
    ch, root = O.clt_children(parent)
    inner = [v for v in range(len(parent)) if ch[v]]
    total = -np.inf
    for states in itertools.product(range(K), repeat=len(inner)):
        j = dict(zip(inner, states))
        lp = 0.0
        for v in inner:
            jp = 0 if v == root else j[parent[v]]
            lp += float(theta[v][jp, j[v]]) + float(leaf[v, j[v], x[v]])
            for c in ch[v]:
                if not ch[c]:
                    lp += float(leaf[c, j[v], x[c]])
        total = np.logaddexp(total, lp)
    return total


@pytest.mark.parametrize("tree,K,C", [([-1, 0], 3, 4), ([-1, 0, 0], 2, 3), ([-1, 0, 1, 1], 3, 2), ([1, -1, 1, 0, 0, 0], 2, 3),
                                      ([-1, 0, 1, 2, 3], 3, 3), ([-1, 0, 0, 1, 1, 2], 2, 2)])
def test_forward_equals_latent_enumeration(tree, K, C):
    parent = np.array(tree, np.int32)
    V = len(parent)
    rng = np.random.default_rng(V * 10 + K)
    theta, leaf = O.random_hclt_params(parent, K, C, rng)
    data = rng.integers(0, C, size=(12, V)).astype(np.uint8)
    want = np.array([brute_force_hclt_ll(parent, K, theta, leaf, x) for x in data])
    for fc in (O.hclt_flat(parent, K, C, theta, leaf), O.bits_compile(O.hclt_dag(parent, K, C, theta, leaf), C, V)):
        got64 = O.forward(fc, data, double=True)[-1]
        np.testing.assert_allclose(got64, want, rtol=1e-6)          # parameters are float32 draws
        got32 = O.forward(fc, data)[-1]
        np.testing.assert_allclose(got32, want, rtol=2e-6)


def test_forward_is_a_normalised_distribution():
    for parent, K, C in [([-1, 0, 0, 1], 3, 3), ([-1, 0, 1, 1, 3], 2, 2)]:
        parent = np.array(parent, np.int32)
        V = len(parent)
        _, _, _, fc = make_hclt(V, K, C, 4, parent=parent)
        allx = np.array(list(itertools.product(range(C), repeat=V)), np.uint8)
        assert abs(np.exp(O.forward(fc, allx, double=True)[-1]).sum() - 1) < 1e-6
    root = random_dag(5, 3, np.random.default_rng(1), width=3)
    fc = O.bits_compile(root, 3, 5)
    allx = np.array(list(itertools.product(range(3), repeat=5)), np.uint8)
    assert abs(np.exp(O.forward(fc, allx, double=True)[-1]).sum() - 1) < 1e-6


def test_pairwise_logsumexp_matches_scipy():
    """Sum nodes fold their edges with the pairwise logsumexp (src/queries/likelihood.jl:101-102)."""
    rng = np.random.default_rng(0)
    C = 2
    for m in (2, 3, 9):
        w = log_dirichlet(rng, m)
        leaves = [O.input_node(0, log_dirichlet(rng, C)) for _ in range(m)]
        fc = O.bits_compile(O.summate(*leaves, logps=w), C, 1)
        data = np.array([[0], [1]], np.uint8)
        got = O.forward(fc, data)[-1]
        for b in range(2):
            want = logsumexp([w[i] + leaves[i].logps[data[b, 0]] for i in range(m)])
            assert abs(got[b] - want) < 1e-6


def test_three_var_fixture_likelihood():
    """test/queries/likelihood_tests.jl:24-37: with uniform leaves over 5 categories the
    product nodes evaluate to 3*log(1/5) and the root to logsumexp of the two branches."""
    root = simple_3vars_circuit(5, weights=[0.25, 0.75])
    fc = O.bits_compile(root, 5, 3)
    data = np.array([[0, 1, 2], [4, 4, 4]], np.uint8)
    mars = O.forward(fc, data)
    np.testing.assert_allclose(mars[-1], 3 * np.log(0.2), rtol=1e-6)
    assert fc.n_nodes == 9 and (fc.type == O.MUL).sum() == 2
    for n in np.nonzero(fc.type == O.MUL)[0]:
        np.testing.assert_allclose(mars[n], 3 * np.log(0.2), rtol=1e-6)


# ------------------------------------------------------------------------------------
# flattening and index tables: known answers held by the reference's tests
# ------------------------------------------------------------------------------------

def test_three_var_fixture_index_tables():
    """test/bits_circuit_tests.jl:13-24 and test/misc_tests.jl:39-62."""
    fc = O.bits_compile(simple_3vars_circuit(5), 5, 3)
    t = fc.param_tables()
    assert fc.n_nodes == 9 and fc.n_edges == 6
    assert t["edge2param"].tolist() == [0, 0, 0, 0, 1, 2]
    assert t["param2edge"].tolist() == [5, 6]
    assert t["param2group"].tolist() == [1, 1]
    assert t["pargroup_sizes"].tolist() == [2]
    assert t["innode2ncumparam"].tolist() == [5, 10, 15, 20, 25, 30]
    assert t["num_input_params"] == 30
    assert len(fc.vectorize_parameters()) == 32


def test_vectorize_update_roundtrip():
    """test/misc_tests.jl:14-36: update_parameters(vectorize_parameters()) is the identity and
    a changed vector lands in the circuit."""
    rng = np.random.default_rng(2)
    fc = O.bits_compile(random_dag(6, 4, rng, width=3), 4, 6)
    p = fc.vectorize_parameters()
    q = rng.normal(size=len(p)).astype(np.float32)
    g = fc.copy()
    g.update_parameters(q)
    assert np.array_equal(g.vectorize_parameters(), q)
    g.update_parameters(p)
    assert np.array_equal(g.logp, fc.logp) and np.array_equal(g.leaf_logp, fc.leaf_logp)


def test_multihead_node_numbering_and_closed_forms():
    """test/multi_head_pc/multi_head_pc_learning_tests.jl:11-47: shared products become nodes
    4 and 8, heads 9 and 10, fake root 11 (1-based); LL closed forms."""
    heads = simple_multihead_circuit(5)
    heads[0].children[0].children[0].logps = np.log(np.array([0.1, 0.2, 0.3, 0.3, 0.1], np.float32))
    heads[0].logps = np.log(np.array([0.2, 0.8], np.float32))
    heads[1].logps = np.log(np.array([0.6, 0.4], np.float32))
    fc = O.bits_compile(O.summate(*heads), 5, 3)
    assert fc.n_nodes == 11
    assert fc.type.tolist() == [0, 0, 0, 2, 0, 0, 0, 2, 1, 1, 1]
    data = np.array([[0, 0, 0], [2, 0, 0]], np.uint8)
    mars = O.forward(fc, data)
    np.testing.assert_allclose(mars[8, 0], np.log(0.1 * 0.2 * 0.2 * 0.2 + 0.2 ** 3 * 0.8), rtol=1e-6)
    np.testing.assert_allclose(mars[9, 1], np.log(0.3 * 0.2 * 0.2 * 0.6 + 0.2 ** 3 * 0.4), rtol=1e-6)
    skip = (fc.edge_parent() == 10).astype(np.uint8)
    mask = np.array([[1.0, 0.0], [0.0, 1.0]], np.float32)       # [head, example]
    flows, _ = O.backward(fc, mars, skip=skip, root_ids=np.array([8, 9], np.int32), root_flow=mask)
    assert flows[8, 0] == 1 and flows[9, 0] == 0 and flows[8, 1] == 0 and flows[9, 1] == 1
    assert (flows[10] == 0).all()
    f32 = np.float32
    np.testing.assert_allclose(flows[3, 0], np.exp(mars[0, 0] + mars[1, 0] + mars[2, 0] + np.log(f32(0.2)) - mars[8, 0]), rtol=1e-5)
    np.testing.assert_allclose(flows[7, 0], np.exp(mars[4, 0] + mars[5, 0] + mars[6, 0] + np.log(f32(0.8)) - mars[8, 0]), rtol=1e-5)
    np.testing.assert_allclose(flows[3, 1], np.exp(mars[0, 1] + mars[1, 1] + mars[2, 1] + np.log(f32(0.6)) - mars[9, 1]), rtol=1e-5)
    np.testing.assert_allclose(flows[7, 1], np.exp(mars[4, 1] + mars[5, 1] + mars[6, 1] + np.log(f32(0.4)) - mars[9, 1]), rtol=1e-5)


def test_hclt_flat_is_the_flattened_dag():
    """The direct HCLT builder and the generic flattening give the same function and the
    same multiset of parameters (node numbering differs)."""
    parent, theta, leaf, flat = make_hclt(7, 3, 4, 8)
    dag = O.bits_compile(O.hclt_dag(parent, 3, 4, theta, leaf), 4, 7)
    assert flat.n_nodes == dag.n_nodes and flat.n_edges == dag.n_edges
    data = correlated_data(40, 7, 4, 9, parent)
    np.testing.assert_allclose(O.forward(flat, data)[-1], O.forward(dag, data)[-1], rtol=1e-6)
    assert np.array_equal(np.sort(flat.vectorize_parameters()), np.sort(dag.vectorize_parameters()))


# ------------------------------------------------------------------------------------
# flows
# ------------------------------------------------------------------------------------

def _total_ll(fc, data):
    return O.forward(fc, data, double=True)[-1].sum()


@pytest.mark.parametrize("kind", ["hclt", "dag"])
def test_flows_are_the_gradient_of_the_log_likelihood(kind):
    """edge_aggr[e] = sum_b d log p(x_b) / d logp_e and leaf_flow[n, c] = sum_b d log p(x_b) /
    d leaf_logp[n, c], checked by central differences in float64 on every parameter."""
    if kind == "hclt":
        parent, theta, leaf, fc = make_hclt(5, 3, 3, 12)
        data = correlated_data(9, 5, 3, 13, parent)
    else:
        fc = O.bits_compile(random_dag(5, 3, np.random.default_rng(3), width=2), 3, 5)
        data = np.random.default_rng(4).integers(0, 3, size=(9, 5)).astype(np.uint8)
    fc.logp = fc.logp.astype(np.float64)
    fc.leaf_logp = fc.leaf_logp.astype(np.float64)
    mars = O.forward(fc, data, double=True)
    flows, ea = O.backward(fc, mars, double=True)
    lf = O.input_flows(fc, data, flows, double=True)
    h = 1e-6
    par = fc.edge_parent()
    for e in range(fc.n_edges):
        if fc.type[par[e]] != O.SUM:
            continue
        g = fc.copy()
        g.logp[e] += h
        up = _total_ll(g, data)
        g.logp[e] -= 2 * h
        fd = (up - _total_ll(g, data)) / (2 * h)
        assert abs(fd - ea[e]) < 1e-6 * max(1.0, abs(ea[e])), e
    for i in range(len(fc.leaf_logp)):
        g = fc.copy()
        g.leaf_logp[i] += h
        up = _total_ll(g, data)
        g.leaf_logp[i] -= 2 * h
        fd = (up - _total_ll(g, data)) / (2 * h)
        assert abs(fd - lf[i]) < 1e-6 * max(1.0, abs(lf[i])), i


def test_flow_invariants():
    """test/queries/flow_tests.jl:44-64, 97-114: the root's flow is 1, a sum node's edge flows
    are flow * exp(edge_mar - node_mar) and add up to the node's flow; in an HCLT the K sum
    nodes of a tree node share one unit of flow per example; edge_aggr is the batch sum."""
    parent, theta, leaf, fc = make_hclt(8, 4, 5, 15)
    data = correlated_data(30, 8, 5, 16, parent)
    mars = O.forward(fc, data)
    flows, ea = O.backward(fc, mars)
    assert np.all(flows[-1] == 1)
    for v, ids in fc.meta["sum_node"].items():
        np.testing.assert_allclose(flows[ids].sum(axis=0), 1.0, rtol=2e-5)
    par = fc.edge_parent()
    for n in np.nonzero(fc.type == O.SUM)[0]:
        tot = np.zeros(30)
        for e in range(fc.edge_ptr[n], fc.edge_ptr[n + 1]):
            em = mars[fc.prime[e]] + (mars[fc.sub[e]] if fc.sub[e] >= 0 else 0) + fc.logp[e]
            ef = flows[n] * np.exp(em - mars[n])
            np.testing.assert_allclose(ea[e], ef.sum(), rtol=1e-4, atol=1e-6)
            tot += ef
        np.testing.assert_allclose(tot, flows[n], rtol=1e-4, atol=1e-7)
    lf = O.input_flows(fc, data, flows)
    np.testing.assert_allclose(lf.reshape(8, -1).sum(axis=1), 30.0, rtol=1e-4)


def test_tempered_flows_by_hand_and_in_their_limits():
    """fscale of mini_batch_em_beta (src-jl/learning/flow.jl:120-175, :204-300): a sum node hands its flow down in
    shares proportional to (posterior share)^(1 / fscale).  One sum node over two leaves by hand; fscale = 1 is the
    ordinary pass; a very large fscale splits evenly; whatever the scale a sum's edge flows add up to its flow and a
    product hands its flow on unchanged."""
    C = 3
    pa, pb = np.array([0.5, 0.25, 0.25], np.float32), np.array([0.1, 0.1, 0.8], np.float32)
    root = O.summate(O.input_node(0, np.log(pa)), O.input_node(0, np.log(pb)), logps=np.log(np.float32([0.2, 0.8])))
    fc = O.bits_compile(root, C, 1)
    data = np.array([[0], [2]], np.uint8)
    mars = O.forward(fc, data, double=True)
    flows, ea = O.backward(fc, mars, double=True, fscale=2.0)
    # example 0: terms 0.2 * 0.5 = 0.1 and 0.8 * 0.1 = 0.08 -> square roots 0.31623, 0.28284 -> shares 0.52786, 0.47214
    # example 1: terms 0.2 * 0.25 = 0.05 and 0.8 * 0.8 = 0.64 -> 0.22361, 0.8 -> shares 0.218450, 0.781550
    np.testing.assert_allclose(flows[0], [0.527864, 0.218450], rtol=2e-6)
    np.testing.assert_allclose(flows[1], [0.472136, 0.781550], rtol=2e-6)
    np.testing.assert_allclose(ea, [0.527864 + 0.218450, 0.472136 + 0.781550], rtol=2e-6)

    parent, theta, leaf, fc = make_hclt(9, 4, 5, 25)
    data = correlated_data(20, 9, 5, 26, parent)
    mars = O.forward(fc, data, double=True)
    plain, ea_plain = O.backward(fc, mars, double=True)
    one, ea_one = O.backward(fc, mars, double=True, fscale=1.0 + 1e-12)      # through the tempered code
    np.testing.assert_allclose(one, plain, rtol=1e-9, atol=1e-300)
    np.testing.assert_allclose(ea_one, ea_plain, rtol=1e-9)
    for fscale in (0.5, 3.0, 1e9):
        flows, ea = O.backward(fc, mars, double=True, fscale=fscale)
        par = fc.edge_parent()
        for n in np.nonzero(fc.type != O.INPUT)[0]:
            es = np.arange(fc.edge_ptr[n], fc.edge_ptr[n + 1])
            if fc.type[n] == O.SUM:
                np.testing.assert_allclose(ea[es].sum(), flows[n].sum(), rtol=1e-9)
                if fscale == 1e9:
                    np.testing.assert_allclose(ea[es], flows[n].sum() / len(es), rtol=1e-6)
            else:
                np.testing.assert_allclose(ea[es], flows[n].sum(), rtol=1e-9)
        np.testing.assert_allclose(flows[fc.type == O.INPUT].reshape(9, -1, 20).sum(axis=1), 1.0, rtol=1e-9)
    # sharper than the posterior: fscale < 1 moves flow towards the larger share
    sharp, _ = O.backward(fc, mars, double=True, fscale=0.5)
    top = fc.meta["sum_node"][int(np.nonzero(np.asarray(parent) < 0)[0][0])]
    es = np.arange(fc.edge_ptr[top[0]], fc.edge_ptr[top[0] + 1])
    kids = fc.prime[es]
    assert (sharp[kids].max(axis=0) >= plain[kids].max(axis=0) - 1e-12).all()


# ------------------------------------------------------------------------------------
# EM update
# ------------------------------------------------------------------------------------

def test_em_update_formulas_by_hand():
    """add_pseudocount / aggr_node_flows / update_params (src/pretrain/mini_batch_warmup.jl:4-17,
    :54-70) and the leaf update (src/nodes/fixable_categorical_dist.jl:223-248) on one sum
    node over three leaves, computed by hand."""
    C = 4
    w = np.array([0.5, 0.3, 0.2], np.float32)
    lps = [np.log(np.array(p, np.float32)) for p in ([0.1, 0.2, 0.3, 0.4], [0.25, 0.25, 0.25, 0.25], [0.7, 0.1, 0.1, 0.1])]
    fc = O.bits_compile(O.summate(*[O.input_node(0, lp) for lp in lps], logps=np.log(w)), C, 1)
    ea = np.array([3.0, 1.0, 0.5], np.float32)
    lf = np.array([[1, 0, 2, 0], [0, 0.5, 0, 0.5], [0.25, 0.25, 0, 0]], np.float32)
    pc, inertia = 0.6, 0.3
    logp, leaf = O.em_update(fc, ea, lf.reshape(-1), pc, inertia)
    e = ea.astype(np.float64) + pc / 3
    want = inertia * w + (1 - inertia) * e / e.sum()
    np.testing.assert_allclose(np.exp(logp), want, rtol=1e-6)
    for i in range(3):
        nf = lf[i].sum() + pc
        want = inertia * np.exp(lps[i]) + (1 - inertia) * (lf[i] + pc / C) / nf
        np.testing.assert_allclose(np.exp(leaf[i * C:(i + 1) * C]), want, rtol=1e-6)


def test_em_is_convex_mix_and_exact_m_step():
    """test/regularization custom_em_tests.jl:207 (new = inertia*old + (1-inertia)*target);
    with pseudocount 0 and inertia 0 the step is the exact M-step: the full-batch
    log-likelihood never decreases and parameters stay normalised."""
    parent, theta, leaf, fc = make_hclt(6, 3, 4, 18)
    data = correlated_data(200, 6, 4, 19, parent)
    idx = np.arange(200, dtype=np.int32)
    _, logp0, leaf0, ea, lf = O.em_step(fc, data, idx, 0.1, 0.0, double=True)
    _, logp3, leaf3, _, _ = O.em_step(fc, data, idx, 0.1, 0.3, double=True)
    par = fc.edge_parent()
    issum = fc.type[par] == O.SUM
    np.testing.assert_allclose(np.exp(logp3[issum]), 0.3 * np.exp(fc.logp[issum].astype(np.float64)) + 0.7 * np.exp(logp0[issum]), rtol=1e-9)
    np.testing.assert_allclose(np.exp(leaf3), 0.3 * np.exp(fc.leaf_logp.astype(np.float64)) + 0.7 * np.exp(leaf0), rtol=1e-9)
    cur = fc.copy()
    cur.logp = cur.logp.astype(np.float64)
    cur.leaf_logp = cur.leaf_logp.astype(np.float64)
    prev = -np.inf
    for _ in range(6):
        ll, logp, lf_new, _, _ = O.em_step(cur, data, idx, 0.0, 0.0, double=True)
        assert ll.sum() >= prev - 1e-9
        prev = ll.sum()
        cur.logp, cur.leaf_logp = logp, lf_new
    for n in np.nonzero(fc.type == O.SUM)[0]:
        s = np.exp(cur.logp[fc.edge_ptr[n]:fc.edge_ptr[n + 1]]).sum()
        assert abs(s - 1) < 1e-9
    assert np.abs(np.exp(cur.leaf_logp).reshape(-1, 4).sum(axis=1) - 1).max() < 1e-9


# ------------------------------------------------------------------------------------
# KL recursion
# ------------------------------------------------------------------------------------

def _three_var_pair(seed=0):
    root = simple_3vars_circuit(5, np.random.default_rng(seed), weights=[0.45, 0.55])
    fc = O.bits_compile(root, 5, 3)
    return fc, fc.vectorize_parameters()


def test_kld_closed_forms():
    """test/queries/kld_tests.jl:9-70."""
    fc, pars = _three_var_pair()
    klds, ek = O.kld(fc, fc.copy())
    assert np.allclose(klds, 0) and np.allclose(ek, 0)
    for a, b in [((0.2, 0.8), (0.4, 0.6)), ((0.5, 0.5), (0.9, 0.1))]:
        f1, f2 = fc.copy(), fc.copy()
        p1, p2 = pars.copy(), pars.copy()
        p1[:2], p2[:2] = np.log(np.float32(a)), np.log(np.float32(b))
        f1.update_parameters(p1)
        f2.update_parameters(p2)
        want = a[0] * np.log(a[0] / b[0]) + a[1] * np.log(a[1] / b[1])
        np.testing.assert_allclose(O.kld(f1, f2)[0][-1], want, rtol=1e-5)
    for w, l1, l2 in [(0.2, [0.1, 0.2, 0.3, 0.2, 0.2], [0.2, 0.1, 0.1, 0.3, 0.3]),
                      (0.5, [0.1, 0.2, 0.3, 0.2, 0.2], [0.2, 0.1, 0.2, 0.3, 0.2])]:
        f1, f2 = fc.copy(), fc.copy()
        p1, p2 = pars.copy(), pars.copy()
        p1[:2] = p2[:2] = np.log(np.float32([w, 1 - w]))
        p1[2:7], p2[2:7] = np.log(np.float32(l1)), np.log(np.float32(l2))
        f1.update_parameters(p1)
        f2.update_parameters(p2)
        want = np.sum(np.exp(p1[2:7]) * (p1[2:7] - p2[2:7])) * w
        np.testing.assert_allclose(O.kld(f1, f2)[0][-1], want, rtol=1e-5)


def test_kld_backward_closed_forms():
    """test/queries/kld_tests.jl:101-131 (edges 5 and 6 are the root's sum edges)."""
    fc, pars = _three_var_pair(1)
    klds, ek = O.kld(fc, fc.copy())
    _, eg1, eg2, _, _ = O.kld_backward(fc, fc.copy(), ek)
    order = fc.up_order()
    eg1, eg2 = eg1[order], eg2[order]
    np.testing.assert_allclose(eg1[4:6], np.exp(pars[:2]), rtol=1e-6)
    np.testing.assert_allclose(eg2[4:6], -eg1[4:6], rtol=1e-6)
    assert np.all(eg1[:4] == 0) and np.all(eg2[:4] == 0)
    f1, f2 = fc.copy(), fc.copy()
    p1, p2 = pars.copy(), pars.copy()
    p1[:2], p2[:2] = np.log(np.float32([0.2, 0.8])), np.log(np.float32([0.4, 0.6]))
    f1.update_parameters(p1)
    f2.update_parameters(p2)
    klds, ek = O.kld(f1, f2)
    _, eg1, eg2, _, _ = O.kld_backward(f1, f2, ek)
    eg1, eg2 = eg1[order], eg2[order]
    np.testing.assert_allclose(eg1[4], 0.2 * (np.log(0.2) - np.log(0.4) + 1), rtol=1e-5)
    np.testing.assert_allclose(eg2[4], -0.2, rtol=1e-6)
    np.testing.assert_allclose(eg1[5], 0.8 * (np.log(0.8) - np.log(0.6) + 1), rtol=1e-5)
    np.testing.assert_allclose(eg2[5], -0.8, rtol=1e-6)


def test_kld_equals_brute_force_on_a_deterministic_circuit():
    """A fully factorised circuit: KL is the sum of the per-variable KLs; and a mixture whose
    branches have disjoint support (deterministic): KL = sum_x p log(p/q) by enumeration."""
    rng = np.random.default_rng(6)
    C, V = 3, 3
    # deterministic mixture: branch i puts variable 0 on category i only
    def circuit():
        branches = []
        for i in range(C):
            lp0 = np.full(C, -80.0, np.float32)
            lp0[i] = 0.0
            branches.append(O.multiply(O.input_node(0, lp0), O.input_node(1, log_dirichlet(rng, C)),
                                       O.input_node(2, log_dirichlet(rng, C))))
        return O.summate(*branches, logps=log_dirichlet(rng, C))
    f1 = O.bits_compile(circuit(), C, V)
    f2 = O.bits_compile(circuit(), C, V)
    allx = np.array(list(itertools.product(range(C), repeat=V)), np.uint8)
    lp = O.forward(f1, allx, double=True)[-1]
    lq = O.forward(f2, allx, double=True)[-1]
    want = np.sum(np.exp(lp) * (lp - lq))
    got = O.kld(f1, f2, double=True)[0][-1]
    np.testing.assert_allclose(got, want, rtol=1e-6)


def test_kld_gradient_by_finite_differences():
    """The recursion's reverse pass against central differences of the forward recursion in
    float64 (sum edges; leaves with the analytic leaf derivative)."""
    rng = np.random.default_rng(7)
    root = random_dag(4, 3, rng, width=2)
    f1 = O.bits_compile(root, 3, 4)
    f2 = f1.copy()
    f2.update_parameters((f1.vectorize_parameters() + rng.normal(0, 0.3, len(f1.vectorize_parameters()))).astype(np.float32))
    for f in (f1, f2):
        f.logp = f.logp.astype(np.float64)
        f.leaf_logp = f.leaf_logp.astype(np.float64)
    klds, ek = O.kld(f1, f2, double=True)
    _, eg1, eg2, lg1, lg2 = O.kld_backward(f1, f2, ek, analytic=True, double=True)
    h = 1e-6
    par = f1.edge_parent()

    def val(a, b):
        return O.kld(a, b, double=True)[0][-1]

    for e in range(f1.n_edges):
        if f1.type[par[e]] != O.SUM:
            assert eg1[e] == 0 and eg2[e] == 0
            continue
        for which, want in ((0, eg1[e]), (1, eg2[e])):
            a, b = f1.copy(), f2.copy()
            t = (a, b)[which]
            t.logp[e] += h
            up = val(a, b)
            t.logp[e] -= 2 * h
            fd = (up - val(a, b)) / (2 * h)
            assert abs(fd - want) < 1e-6 * max(1, abs(want)), (e, which)
    for i in range(len(f1.leaf_logp)):
        for which, want in ((0, lg1[i]), (1, lg2[i])):
            a, b = f1.copy(), f2.copy()
            t = (a, b)[which]
            t.leaf_logp[i] += h
            up = val(a, b)
            t.leaf_logp[i] -= 2 * h
            fd = (up - val(a, b)) / (2 * h)
            assert abs(fd - want) < 1e-6 * max(1, abs(want)), (i, which)


def test_kld_backward_leaf_lines_as_written():
    """src/nodes/fixable_categorical_dist.jl:219 (norm_params = false) returns, per category,
    grad1 = g * (p1 - p2 + 1) and grad2 = g * exp(p1 - p2) -- not the analytic derivatives
    g * exp(p1) * (p1 - p2 + 1) and -g * exp(p1), which central differences pin above.  The two
    forms differ by a known factor each: written1 * exp(p1) = analytic1 and
    written2 * exp(p2) = -analytic2.  Plus one literal worked by hand on the three-variable
    fixture: a leaf under the branch of weight 0.2 receives node gradient 0.2, so a category
    with p1 = log 0.1 against p2 = log 0.2 gets 0.2 * (1 - log 2) and 0.2 * 0.5."""
    rng = np.random.default_rng(21)
    root = random_dag(4, 3, rng, width=2)
    f1 = O.bits_compile(root, 3, 4)
    f2 = f1.copy()
    f2.update_parameters((f1.vectorize_parameters() + rng.normal(0, 0.3, len(f1.vectorize_parameters()))).astype(np.float32))
    for dbl in (True, False):
        _, ek = O.kld(f1, f2, double=dbl)
        _, _, _, a1, a2 = O.kld_backward(f1, f2, ek, analytic=True, double=dbl)
        _, _, _, w1, w2 = O.kld_backward(f1, f2, ek, analytic=False, double=dbl)
        tol = 1e-12 if dbl else 1e-5
        assert np.abs(a1).max() > 1e-3 and np.abs(a2).max() > 1e-3
        np.testing.assert_allclose(w1 * np.exp(f1.leaf_logp.astype(np.float64)), a1, rtol=tol, atol=tol * 1e-3)
        np.testing.assert_allclose(w2 * np.exp(f2.leaf_logp.astype(np.float64)), -a2, rtol=tol, atol=tol * 1e-3)
    # literal on the fixture of test/helpers/simple_circuits.jl:4-14
    fc, pars = _three_var_pair(2)
    g1c, g2c = fc.copy(), fc.copy()
    p1, p2 = pars.copy(), pars.copy()
    p1[:2] = p2[:2] = np.log(np.float32([0.2, 0.8]))
    p1[2:7] = np.log(np.float32([0.1, 0.2, 0.3, 0.2, 0.2]))      # first input node: variable 0 of branch 1
    p2[2:7] = np.log(np.float32([0.2, 0.1, 0.3, 0.3, 0.1]))
    g1c.update_parameters(p1)
    g2c.update_parameters(p2)
    _, ek = O.kld(g1c, g2c)
    grads, _, _, w1, w2 = O.kld_backward(g1c, g2c, ek)
    first = int(g1c.input_nodes()[0])
    np.testing.assert_allclose(grads[first], 0.2, rtol=1e-6)
    off = g1c.in_off[first]
    np.testing.assert_allclose(w1[off:off + 5], 0.2 * (1 + np.log([0.5, 2.0, 1.0, 2 / 3, 2.0])), rtol=1e-5)
    np.testing.assert_allclose(w2[off:off + 5], 0.2 * np.array([0.5, 2.0, 1.0, 2 / 3, 2.0]), rtol=1e-5)
    np.testing.assert_allclose(w1[off], 0.2 * (1 - np.log(2)), rtol=1e-5)
    np.testing.assert_allclose(w2[off], 0.1, rtol=1e-5)


def test_probability_valued_leaf_parameters():
    """norm_params = true: leaf parameters are probabilities (src/nodes/fixable_categorical_dist.jl:182-186,
    :216-217; src/queries/sample.jl:265-268), sum edges stay in log space.  The KL equals the
    log-parameter form on the logarithms and scipy's entropy leaf by leaf; grad1 as written IS the
    derivative with respect to p1 (central differences), grad2 as written is minus the derivative
    with respect to p2; the relaxed sampler's output equals the log-parameter form's."""
    from scipy.stats import entropy
    rng = np.random.default_rng(41)
    root = random_dag(4, 3, rng, width=2)
    f1 = O.bits_compile(root, 3, 4)
    f2 = f1.copy()
    f2.update_parameters((f1.vectorize_parameters() + rng.normal(0, 0.3, len(f1.vectorize_parameters()))).astype(np.float32))
    f2.leaf_logp = np.log(np.exp(f2.leaf_logp.reshape(-1, 3)) / np.exp(f2.leaf_logp.reshape(-1, 3)).sum(1, keepdims=True)).reshape(-1)
    n1, n2 = f1.copy(), f2.copy()
    for a, b in ((n1, f1), (n2, f2)):
        a.logp = b.logp.astype(np.float64)
        a.leaf_logp = np.exp(b.leaf_logp.astype(np.float64))
    want, _ = O.kld(f1, f2, double=True)
    got, ek = O.kld(n1, n2, double=True, norm_params=True)
    np.testing.assert_allclose(got[-1], want[-1], rtol=1e-6)            # the 1e-8 inside the logarithms
    for n in f1.input_nodes():
        o = f1.in_off[n]
        # (scipy renormalises its arguments; float32 draws add up to 1 within 1e-7)
        np.testing.assert_allclose(got[n], entropy(n1.leaf_logp[o:o + 3], n2.leaf_logp[o:o + 3]), rtol=1e-5, atol=1e-6)
    _, _, _, w1, w2 = O.kld_backward(n1, n2, ek, double=True, norm_params=True)
    h = 1e-7
    for i in range(len(n1.leaf_logp)):
        for which, wantg in ((0, w1[i]), (1, -w2[i])):
            a, b = n1.copy(), n2.copy()
            t = (a, b)[which]
            t.leaf_logp = t.leaf_logp.copy()
            t.leaf_logp[i] += h
            up = O.kld(a, b, double=True, norm_params=True)[0][-1]
            t.leaf_logp[i] -= 2 * h
            fd = (up - O.kld(a, b, double=True, norm_params=True)[0][-1]) / (2 * h)
            assert abs(fd - wantg) < 1e-5 * max(1, abs(wantg)), (i, which)
    g = _gumbel(rng, f1.n_edges)
    _, out_log = O.gumbel_soft(f1, g, 0.7, double=True)
    _, out_prob = O.gumbel_soft(n1, g, 0.7, double=True, norm_params=True)
    np.testing.assert_allclose(out_prob, out_log, rtol=1e-6)


# ------------------------------------------------------------------------------------
# sampling
# ------------------------------------------------------------------------------------

def _gumbel(rng, shape):
    return -np.log(-np.log(rng.random(shape).clip(1e-12, 1 - 1e-12)))


def test_gumbel_max_samples_follow_the_circuit():
    rng = np.random.default_rng(8)
    V, C, B = 3, 3, 40000
    fc = O.bits_compile(random_dag(V, C, rng, width=2), C, V)
    allx = np.array(list(itertools.product(range(C), repeat=V)), np.uint8)
    prob = np.exp(O.forward(fc, allx, double=True)[-1])
    s = O.sample(fc, _gumbel(rng, (B, fc.n_edges)), _gumbel(rng, (B, V, C))).astype(np.int64)
    assert (s < C).all()
    code = (s * (C ** np.arange(V - 1, -1, -1))).sum(axis=1)
    freq = np.bincount(code, minlength=C ** V) / B
    assert np.abs(freq - prob).max() < 5 * np.sqrt(prob.max() / B) + 1e-3


def test_zero_noise_sampling_is_greedy_descent():
    """Without noise each sum node takes its heaviest edge and each leaf its mode."""
    w = np.log(np.array([0.2, 0.5, 0.3], np.float32))
    leaves = [O.input_node(0, np.log(np.array(p, np.float32))) for p in ([0.9, 0.1], [0.3, 0.7], [0.5, 0.5])]
    fc = O.bits_compile(O.summate(*leaves, logps=w), 2, 1)
    out = O.sample(fc, np.zeros((1, fc.n_edges), np.float32), np.zeros((1, 1, 2), np.float32))
    assert out.tolist() == [[1]]
    # ties: the first maximum wins
    fc2 = O.bits_compile(O.summate(*leaves, logps=np.log(np.array([0.4, 0.4, 0.2], np.float32))), 2, 1)
    assert O.sample(fc2, np.zeros((1, 3), np.float32), np.zeros((1, 1, 2), np.float32)).tolist() == [[0]]


def test_soft_sampling_invariants():
    """test/queries/sample_tests.jl:34-53: top-down probabilities of a sum node's children add
    up to the node's; per variable the soft output is a distribution; at temperature 1 without
    noise the output is the circuit's marginal."""
    rng = np.random.default_rng(10)
    V, C = 4, 3
    parent, theta, leaf, fc = make_hclt(V, 3, C, 11)
    td, out = O.gumbel_soft(fc, None, 1.0, double=True)
    assert abs(td[-1] - 1) < 1e-12
    np.testing.assert_allclose(out.sum(axis=1), 1.0, rtol=1e-6)
    allx = np.array(list(itertools.product(range(C), repeat=V)), np.uint8)
    p = np.exp(O.forward(fc, allx, double=True)[-1])
    for v in range(V):
        marg = np.array([p[allx[:, v] == c].sum() for c in range(C)])
        np.testing.assert_allclose(out[v], marg, rtol=1e-5)
    g = _gumbel(rng, fc.n_edges)
    td, out = O.gumbel_soft(fc, g, 0.5, double=True)
    np.testing.assert_allclose(out.sum(axis=1), 1.0, rtol=1e-6)
    for ids in fc.meta["sum_node"].values():
        assert abs(td[ids].sum() - 1) < 1e-9


@pytest.mark.parametrize("T", [0.5, 2.0])
def test_soft_sampling_temperature_closed_form(T):
    """src/queries/sample.jl:47-51: an edge's weight is exp((logp + g)/T) over the sum node's
    total.  Without noise a single sum node over m leaves therefore hands leaf i the share
    theta_i^(1/T) / sum_j theta_j^(1/T) (a product, or T in place of 1/T, gives another number)."""
    C = 3
    w = np.array([0.5, 0.3, 0.15, 0.05])
    rng = np.random.default_rng(31)
    lps = [log_dirichlet(rng, C) for _ in w]
    fc = O.bits_compile(O.summate(*[O.input_node(0, lp) for lp in lps], logps=np.log(w).astype(np.float32)), C, 1)
    want = w ** (1 / T) / (w ** (1 / T)).sum()
    for dbl, tol in ((True, 1e-6), (False, 1e-5)):
        td, out = O.gumbel_soft(fc, None, T, double=dbl)
        np.testing.assert_allclose(td[:4], want, rtol=tol)
        np.testing.assert_allclose(out[0], sum(want[i] * np.exp(lps[i].astype(np.float64)) for i in range(4)), rtol=tol)
    # with noise: the same closed form on the tilted weights theta_i * exp(g_i)
    g = _gumbel(rng, 4)
    tilt = (w * np.exp(g)) ** (1 / T)
    td, _ = O.gumbel_soft(fc, g, T, double=True)
    np.testing.assert_allclose(td[:4], tilt / tilt.sum(), rtol=1e-6)


@pytest.mark.parametrize("T", [0.3, 1.7])
def test_soft_sampling_is_a_softmax_per_sum_node(T):
    """Every sum node shares its top-down probability among its edges as
    scipy.special.softmax((logp + g)/T); products pass theirs on to prime and sub; an input node's
    share goes to its variable weighted by its distribution (src/queries/sample.jl:105-140, :262-284).
    Recomputed here node by node with scipy on a DAG with shared sub-circuits."""
    from scipy.special import softmax
    rng = np.random.default_rng(32)
    V, C = 5, 3
    fc = O.bits_compile(random_dag(V, C, rng, width=3), C, V)
    g = _gumbel(rng, fc.n_edges)
    td, out = O.gumbel_soft(fc, g, T, double=True)
    want = np.zeros(fc.n_nodes)
    want[-1] = 1.0
    want_out = np.zeros((V, C))
    for n in range(fc.n_nodes - 1, -1, -1):
        e0, e1 = fc.edge_ptr[n], fc.edge_ptr[n + 1]
        if fc.type[n] == O.INPUT:
            want_out[fc.in_var[n]] += want[n] * np.exp(fc.leaf_logp[fc.in_off[n]:fc.in_off[n] + C].astype(np.float64))
            continue
        share = softmax((fc.logp[e0:e1].astype(np.float64) + g[e0:e1]) / T) if fc.type[n] == O.SUM else np.ones(e1 - e0)
        for e, s in zip(range(e0, e1), share):
            want[fc.prime[e]] += want[n] * s
            if fc.sub[e] >= 0:
                want[fc.sub[e]] += want[n] * s
    np.testing.assert_allclose(td, want, rtol=1e-9, atol=1e-15)
    np.testing.assert_allclose(out, want_out, rtol=1e-9)


def test_soft_sampling_cold_limit_is_the_gumbel_max_sample():
    """As T -> 0 the relaxed sampler concentrates on the edge maximising logp + g, i.e. on what
    orc_sample (pinned by the statistics of its draws above) picks from the same noise.  With
    leaves that put all mass on one category the soft output is then the one-hot of the sample."""
    rng = np.random.default_rng(33)
    V, C, T = 5, 4, 0.01
    fc = O.bits_compile(random_dag(V, C, rng, width=3), C, V)
    for n in fc.input_nodes():                      # deterministic leaves
        lp = np.full(C, -80.0, np.float32)
        lp[rng.integers(C)] = 0.0
        fc.leaf_logp[fc.in_off[n]:fc.in_off[n] + C] = lp
    checked = 0
    for trial in range(40):
        g = _gumbel(rng, fc.n_edges)
        # leave out draws whose visited sum nodes do not separate their two best edges by 0.2
        # (exp(-0.2/T) = 2e-9 is what the runner-up keeps at this temperature)
        hard = O.sample(fc, g[None, :], np.zeros((1, V, C)), double=True)[0]
        td, out = O.gumbel_soft(fc, g, T, double=True)
        gaps = []
        for n in np.nonzero(fc.type == O.SUM)[0]:
            if td[n] < 0.5:
                continue
            s = np.sort(fc.logp[fc.edge_ptr[n]:fc.edge_ptr[n + 1]].astype(np.float64) + g[fc.edge_ptr[n]:fc.edge_ptr[n + 1]])
            if len(s) > 1:
                gaps.append(s[-1] - s[-2])
        if min(gaps) < 0.2:
            continue
        onehot = np.zeros((V, C))
        onehot[np.arange(V), hard] = 1.0
        assert np.abs(out - onehot).max() < 1e-6, trial
        checked += 1
    assert checked >= 10


@pytest.mark.parametrize("T,noise", [(1.0, False), (0.6, True), (1.8, True)])
def test_soft_sampling_reverse_pass_is_the_derivative_of_the_soft_output(T, noise):
    """src/queries/sample.jl:389-650.  For a loss L = sum(out * G) the reverse pass must return dL/d(log
    parameter) on the sum edges, and on the leaves dL/d(probability of the category), i.e. the log-parameter
    derivative divided by that probability (the source leaves the factor p out, :566).  Checked against
    float64 central differences of orc_gumbel_soft, itself pinned above, on a DAG with shared sub-circuits;
    a wrong sign, a missing 1/T, a dropped normaliser term or td taken from the wrong end each fail it."""
    rng = np.random.default_rng(41)
    V, C = 5, 3
    fc = O.bits_compile(random_dag(V, C, rng, width=3), C, V)
    g = _gumbel(rng, fc.n_edges) if noise else None
    G = rng.normal(size=(V, C))
    eg, lg = O.gumbel_soft_backward(fc, g, T, G, double=True)

    def loss():
        return float((O.gumbel_soft(fc, g, T, double=True)[1] * G).sum())

    h = 1e-5
    logp0, leaf0 = fc.logp.copy(), fc.leaf_logp.copy()
    fc.logp = logp0.astype(np.float64)
    fc.leaf_logp = leaf0.astype(np.float64)
    sum_edges = np.nonzero(fc.type[fc.edge_parent()] == O.SUM)[0]
    for e in rng.choice(sum_edges, size=min(25, len(sum_edges)), replace=False):
        keep = fc.logp[e]
        fc.logp[e] = keep + h
        up = loss()
        fc.logp[e] = keep - h
        dn = loss()
        fc.logp[e] = keep
        assert abs(eg[e] - (up - dn) / (2 * h)) < 1e-6 * max(1.0, abs(eg[e])), e
    assert np.all(eg[fc.type[fc.edge_parent()] != O.SUM] == 0)
    for i in rng.choice(len(fc.leaf_logp), size=25, replace=False):
        keep = fc.leaf_logp[i]
        fc.leaf_logp[i] = keep + h
        up = loss()
        fc.leaf_logp[i] = keep - h
        dn = loss()
        fc.leaf_logp[i] = keep
        assert abs(lg[i] * np.exp(keep) - (up - dn) / (2 * h)) < 1e-6 * max(1.0, abs(lg[i])), i
    # grad_wrt_logparams = false drops the factor w = softmax weight of the edge (:466-469)
    eg_p, _ = O.gumbel_soft_backward(fc, g, T, G, double=True, grad_wrt_logparams=False)
    td, _ = O.gumbel_soft(fc, g, T, double=True)
    par = fc.edge_parent()
    for n in np.nonzero(fc.type == O.SUM)[0]:
        e0, e1 = fc.edge_ptr[n], fc.edge_ptr[n + 1]
        z = (fc.logp[e0:e1] + (g[e0:e1] if noise else 0.0)) / T
        w = np.exp(z - z.max())
        w /= w.sum()
        np.testing.assert_allclose(eg_p[e0:e1] * w, eg[e0:e1], rtol=1e-9, atol=1e-14)
    # probability-valued leaves (norm_params): the leaf gradient is then the plain derivative
    fc.leaf_logp = np.exp(fc.leaf_logp)
    _, lgn = O.gumbel_soft_backward(fc, g, T, G, double=True, norm_params=True)
    for i in rng.choice(len(fc.leaf_logp), size=15, replace=False):
        keep = fc.leaf_logp[i]
        vals = []
        for d in (h, -h):
            fc.leaf_logp[i] = keep + d
            vals.append(float((O.gumbel_soft(fc, g, T, double=True, norm_params=True)[1] * G).sum()))
        fc.leaf_logp[i] = keep
        assert abs(lgn[i] - (vals[0] - vals[1]) / (2 * h)) < 1e-6 * max(1.0, abs(lgn[i])), i
    fc.logp, fc.leaf_logp = logp0, leaf0


def test_soft_sampling_reverse_pass_single_sum_node_closed_form():
    """One sum node over m leaves, no noise: out = sum_i w_i p_i with w = softmax(logp / T), so
    dL/dlogp_i = w_i (a_i - sum_j w_j a_j) / T with a_i = <p_i, G>  (softmax derivative, worked by hand)."""
    rng = np.random.default_rng(42)
    C, T = 4, 0.7
    w = np.array([0.4, 0.3, 0.2, 0.1])
    lps = [log_dirichlet(rng, C) for _ in w]
    fc = O.bits_compile(O.summate(*[O.input_node(0, lp) for lp in lps], logps=np.log(w).astype(np.float32)), C, 1)
    G = rng.normal(size=(1, C))
    eg, lg = O.gumbel_soft_backward(fc, None, T, G, double=True)
    sm = w ** (1 / T) / (w ** (1 / T)).sum()
    a = np.array([(np.exp(lp.astype(np.float64)) * G[0]).sum() for lp in lps])
    np.testing.assert_allclose(eg, sm * (a - (sm * a).sum()) / T, rtol=1e-6)
    np.testing.assert_allclose(lg.reshape(4, C), sm[:, None] * G, rtol=1e-6)


# ------------------------------------------------------------------------------------
# Adam
# ------------------------------------------------------------------------------------

def test_adam_first_step_closed_form():
    """At t = 1 with zero moments mhat = g and vhat = g^2, so params move by
    lr * g / (|g| + eps); groups are normalised into logp_out, params stay unnormalised."""
    rng = np.random.default_rng(12)
    n = 10
    params = rng.normal(size=n).astype(np.float32)
    p0 = params.copy()
    grad = rng.normal(size=n).astype(np.float32)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    logp = np.full(n, 7.0, np.float32)
    gp = np.array([0, 4, 5, 10])
    O.adam_step(params, grad, m, v, 1e-2, 0.9, 0.999, 1e-8, 1, gp, logp)
    np.testing.assert_allclose(params, p0 + 1e-2 * grad / (np.abs(grad) + 1e-8), rtol=1e-5)
    np.testing.assert_allclose(m, 0.1 * grad, rtol=1e-6)
    np.testing.assert_allclose(v, 0.001 * grad * grad, rtol=5e-5)     # 1 - 0.999 in float32
    for a, b in ((0, 4), (5, 10)):
        np.testing.assert_allclose(np.exp(logp[a:b].astype(np.float64)).sum(), 1.0, rtol=1e-6)
        np.testing.assert_allclose(logp[a:b] - params[a:b], (logp[a] - params[a]), rtol=1e-5)
    assert logp[4] == 7.0          # a sum node with one edge keeps its parameter


def test_flow_gradient_is_the_derivative_of_the_mean_log_likelihood():
    """src/sgd/adam.jl:27-61 with :305: edge flows / B minus exp(logp) times their sum over the sum
    node is d(mean LL)/d(unnormalised log-parameter) when logp = params - logsumexp(params) per sum
    node; checked by central differences in float64 on every sum edge."""
    rng = np.random.default_rng(51)
    fc = O.bits_compile(random_dag(5, 3, rng, width=3), 3, 5)
    fc.logp = fc.logp.astype(np.float64)
    fc.leaf_logp = fc.leaf_logp.astype(np.float64)
    data = rng.integers(0, 3, size=(11, 5)).astype(np.uint8)
    B = len(data)
    mars = O.forward(fc, data, double=True)
    _, ea = O.backward(fc, mars, double=True)
    grad = O.flow_gradients(fc, ea, B, double=True)
    par = fc.edge_parent()
    params = fc.logp.copy()                      # normalised already: logsumexp of a group is 0

    def mean_ll(p):
        g = fc.copy()
        lp = p.copy()
        for n in np.nonzero(fc.type == O.SUM)[0]:
            e0, e1 = fc.edge_ptr[n], fc.edge_ptr[n + 1]
            lp[e0:e1] = p[e0:e1] - logsumexp(p[e0:e1])
        g.logp = lp
        return O.forward(g, data, double=True)[-1].mean()

    h = 1e-6
    checked = 0
    for e in range(fc.n_edges):
        if fc.type[par[e]] != O.SUM:
            assert grad[e] == ea[e]               # product edges keep their flow
            continue
        up, dn = params.copy(), params.copy()
        up[e] += h
        dn[e] -= h
        fd = (mean_ll(up) - mean_ll(dn)) / (2 * h)
        assert abs(fd - grad[e]) < 1e-6 * max(1, abs(grad[e])), e
        checked += 1
    assert checked > 10
    # float build agrees
    g32 = O.flow_gradients(fc, ea.astype(np.float32), B)
    np.testing.assert_allclose(g32, grad, rtol=1e-4, atol=1e-6)


def test_leaf_adam_as_the_source_writes_it():
    """src/sgd/adam.jl:218-242 by hand at t = 1 with zero moments: g_i = flow_i + p_i * sum(flow) (a
    plus, as written), the auxiliary parameter copy moves by lr * g / (|g| + eps), the moments become
    (1 - beta) * g and (1 - beta2) * g^2, and the circuit's own leaves stay as they are."""
    C = 4
    lp = np.log(np.array([0.1, 0.2, 0.3, 0.4]))
    fc = O.bits_compile(O.summate(O.input_node(0, lp.astype(np.float32)), O.input_node(0, lp[::-1].astype(np.float32).copy())), C, 1)
    fc.leaf_logp = fc.leaf_logp.astype(np.float64)
    flow = np.array([1.0, 0.0, 2.0, 1.0, 0.5, 0.5, 0.0, 0.0])
    aux_p = fc.leaf_logp.copy()
    aux_m, aux_v = np.zeros(8), np.zeros(8)
    before = fc.leaf_logp.copy()
    O.leaf_adam(fc, flow, aux_p, aux_m, aux_v, 1e-2, 0.9, 0.999, 1e-8, 1, double=True)
    g = np.concatenate([flow[:4] + np.exp(before[:4]) * 4.0, flow[4:] + np.exp(before[4:]) * 1.0])
    np.testing.assert_allclose(aux_m, 0.1 * g, rtol=1e-12)
    np.testing.assert_allclose(aux_v, 0.001 * g * g, rtol=1e-9)
    np.testing.assert_allclose(aux_p, before + 1e-2 * g / (np.abs(g) + 1e-8), rtol=1e-9)
    assert np.array_equal(fc.leaf_logp, before)
    np.testing.assert_allclose(g[0], 1.0 + 0.1 * 4.0)          # the literal: flow 1, p 0.1, node flow 4


# ---- missing values --------------------------------------------------------------------------------

def _marker_case(seed=3, V=4, K=2, C_real=3, N=6):
    """A small HCLT twice: over the C_real categories, and with one table row more, pinned to log 1, whose
    category (C_real) marks a missing value in the data."""
    rng = np.random.default_rng(seed)
    parent = O.random_tree(V, rng, 3)
    theta, leaf = O.random_hclt_params(parent, K, C_real, rng, "dirichlet")
    real = O.hclt_flat(parent, K, C_real, theta, leaf)
    leaf_m = np.concatenate([leaf, np.zeros((V, K, 1), leaf.dtype)], axis=2)
    marked = O.hclt_flat(parent, K, C_real + 1, theta, leaf_m)
    data = rng.integers(0, C_real, size=(N, V)).astype(np.uint8)
    hole = rng.random((N, V)) < 0.35
    hole[0] = False                                   # one complete example
    hole[1] = True
    hole[1, 0] = False                                # one with a single observed variable
    data_m = np.where(hole, C_real, data).astype(np.uint8)
    return real, marked, data_m, hole, C_real


def _completions(row, hole_row, C_real):
    """Every way of filling the holes of one example."""
    holes = np.flatnonzero(hole_row)
    for fill in itertools.product(range(C_real), repeat=len(holes)):
        x = row.copy()
        x[holes] = fill
        yield x


def test_missing_marker_marginalises_the_variable():
    """A table row of log-probability 0 for the marker makes the leaf count as 1
    (src/regularization/reg_likelihood.jl:40-47): the likelihood of an example with holes is then the sum of the
    likelihoods of all its completions."""
    real, marked, data_m, hole, C_real = _marker_case()
    ll = O.forward(marked, data_m, double=True)[-1]
    for b in range(len(data_m)):
        comp = np.array(list(_completions(data_m[b], hole[b], C_real)), np.uint8)
        want = logsumexp(O.forward(real, comp, double=True)[-1])
        assert abs(ll[b] - want) < 1e-6, b        # (the float32 parameters sum to 1 to seven digits only)


def test_missing_flow_update_is_the_m_step_on_expected_counts():
    """The update with missing_flow (src/nodes/fixable_categorical_dist.jl:223-248) is the EM step for
    incomplete data: the same numbers as the ordinary update applied to the flows of all completions of
    every example, each weighted by its posterior probability given what was observed."""
    real, marked, data_m, hole, C_real = _marker_case()
    pc, inertia = 0.3, 0.6
    mars = O.forward(marked, data_m, double=True)
    flows, ea = O.backward(marked, mars, double=True)
    lf = O.input_flows(marked, data_m, flows, double=True)
    logp_m, leaf_m = O.em_update(marked, ea, lf, pc, inertia, double=True, missing=True)
    # expected complete-data statistics by enumeration, on the circuit without the marker
    ea_x = np.zeros(real.n_edges)
    lf_x = np.zeros(len(real.leaf_logp))
    for b in range(len(data_m)):
        comp = np.array(list(_completions(data_m[b], hole[b], C_real)), np.uint8)
        m = O.forward(real, comp, double=True)
        w = np.exp(m[-1] - logsumexp(m[-1]))                     # posterior of every completion
        fl, _ = O.backward(real, m, double=True)
        for i in range(len(comp)):
            _, ea_i = O.backward(real, m[:, i:i + 1].copy(), double=True)
            lf_i = O.input_flows(real, comp[i:i + 1], fl[:, i:i + 1].copy(), double=True)
            ea_x += w[i] * ea_i
            lf_x += w[i] * lf_i
    logp_x, leaf_x = O.em_update(real, ea_x, lf_x, pc, inertia, double=True)
    # (to seven digits: the float32 parameters the circuits start from are normalised no better)
    np.testing.assert_allclose(logp_m, logp_x, rtol=1e-7, atol=1e-7)
    C = C_real + 1
    got = leaf_m.reshape(-1, C)
    np.testing.assert_allclose(got[:, :C_real], leaf_x.reshape(-1, C_real), rtol=1e-7, atol=1e-7)
    assert (got[:, C_real] == 0).all()                           # the marker's row stays log 1
    np.testing.assert_allclose(np.exp(got[:, :C_real]).sum(axis=1), 1.0, rtol=1e-6)


# ------------------------------------------------------------------------------------
# per-example normalised flows (src/queries/flow.jl:417-593) and normalize_params (src/misc.jl:448-498)
# ------------------------------------------------------------------------------------

def _hclt_joint(parent, K, theta, leaf, x):
    """log of the joint of x and every assignment of the inner tree nodes' hidden states, as a dict
    states -> log-probability (the terms of brute_force_hclt_ll)."""
    ch, root = O.clt_children(parent)
    inner = [v for v in range(len(parent)) if ch[v]]
    out = {}
    for states in itertools.product(range(K), repeat=len(inner)):
        j = dict(zip(inner, states))
        lp = 0.0
        for v in inner:
            jp = 0 if v == root else j[parent[v]]
            lp += float(theta[v][jp, j[v]]) + float(leaf[v, j[v], x[v]])
            for c in ch[v]:
                if not ch[c]:
                    lp += float(leaf[c, j[v], x[c]])
        out[states] = lp
    return inner, out


@pytest.mark.parametrize("tree,K,C", [([-1, 0, 1, 1], 3, 2), ([1, -1, 1, 0, 0, 0], 2, 3), ([-1, 0, 1, 2, 3], 2, 3)])
def test_normalized_flows_are_posteriors_of_the_hidden_states(tree, K, C):
    """A sum parameter's normalised flow is the posterior of its child's hidden state given its own node's (the
    parent tree node's state) and the example: exp(entry of (v, k, j)) = P(z_v = j | z_parent(v) = k, x), summed
    out of the joint over all hidden-state assignments in float64; and the entries of a sum node add up to 1."""
    parent = np.array(tree, np.int32)
    V = len(parent)
    rng = np.random.default_rng(V + K)
    theta, leaf = O.random_hclt_params(parent, K, C, rng)
    fc = O.hclt_flat(parent, K, C, theta, leaf)
    data = rng.integers(0, C, size=(5, V)).astype(np.uint8)
    nf = O.normalized_flows(fc, data, double=True)
    pe = fc.sum_param_edges()
    pos_of_edge = {int(e): i for i, e in enumerate(pe)}
    ch, root = O.clt_children(parent)
    for b, x in enumerate(data):
        inner, joint = _hclt_joint(parent, K, theta, leaf, x)
        at = {v: i for i, v in enumerate(inner)}
        for v in inner:
            nk = len(fc.meta["sum_node"][v])
            for k in range(nk):
                num = np.full(K, -np.inf)
                for states, lp in joint.items():
                    if v != root and states[at[parent[v]]] != k:
                        continue
                    num[states[at[v]]] = np.logaddexp(num[states[at[v]]], lp)
                post = np.exp(num - logsumexp(num))
                got = np.array([nf[b, pos_of_edge[fc.meta["edge_of"][v] + k * K + j]] for j in range(K)])
                np.testing.assert_allclose(np.exp(got), post, rtol=1e-5, atol=1e-7)
                assert abs(np.exp(got).sum() - 1) < 1e-5


def test_normalized_flows_are_derivatives_of_the_parent_value():
    """On a DAG with shared sub-circuits: edge flow / node flow = d(log-value of the sum node) / d(logp of the
    edge), by central differences in float64, for every sum parameter whose node has flow."""
    fc = O.bits_compile(random_dag(5, 3, np.random.default_rng(8), width=3), 3, 5)
    fc.logp = fc.logp.astype(np.float64)
    fc.leaf_logp = fc.leaf_logp.astype(np.float64)
    data = np.random.default_rng(9).integers(0, 3, size=(4, 5)).astype(np.uint8)
    nf = O.normalized_flows(fc, data, double=True)
    mars = O.forward(fc, data, double=True)
    flows, _ = O.backward(fc, mars, double=True)
    pe = fc.sum_param_edges()
    par = fc.edge_parent()
    h = 1e-6
    seen = 0
    for i, e in enumerate(pe):
        g = fc.copy()
        g.logp[e] += h
        up = O.forward(g, data, double=True)[par[e]]
        g.logp[e] -= 2 * h
        fd = (up - O.forward(g, data, double=True)[par[e]]) / (2 * h)
        live = flows[par[e]] > 1e-3
        seen += int(live.sum())
        np.testing.assert_allclose(np.exp(nf[live, i]), fd[live], rtol=1e-5, atol=1e-7)
    assert seen > 20


def test_normalized_flows_guards_and_input_slots_as_written():
    """The 1e-8 guards of map_flows (flow.jl:525, :535) on a sum node that no flow reaches: log(0 / 1e-8 + 1e-8);
    and the input entries as written: the node's flow in the slot get_edge_flow picks, the literal of
    test/queries/flow_tests.jl:54-64 (data value 1 -> slot 1 of 5, i.e. the first), -inf elsewhere, NaN throughout
    where nothing lands (category 0) -- against the corrected placement with as_written = False."""
    C = 5
    lp = lambda: np.log(np.full(C, 1.0 / C, np.float32))
    dead = O.summate(O.input_node(1, lp()), O.input_node(1, lp()), logps=np.log(np.float32([0.3, 0.7])))
    root = O.summate(O.multiply(O.input_node(0, lp()), O.input_node(1, lp())),
                     O.multiply(O.input_node(0, lp()), dead), logps=np.float32([0.0, -np.inf]))
    fc = O.bits_compile(root, C, 2)
    data = np.array([[1, 2], [0, 4]], np.uint8)
    for dbl in (False, True):
        nf = O.normalized_flows(fc, data, double=dbl)
        pe = fc.sum_param_edges()
        par = fc.edge_parent()[pe]
        dead_rows = np.nonzero(par != fc.n_nodes - 1)[0]
        assert len(dead_rows) == 2
        np.testing.assert_allclose(nf[:, dead_rows], np.log(1e-8), rtol=1e-6)
        top = np.nonzero(par == fc.n_nodes - 1)[0]
        np.testing.assert_allclose(nf[:, top[0]], np.log(1.0 / (1 + 1e-8) + 1e-8), atol=1e-7)
        np.testing.assert_allclose(nf[:, top[1]], np.log(1e-8), rtol=1e-6)
    nf = O.normalized_flows(fc, data, double=True)
    ns = len(fc.sum_param_edges())
    inputs = fc.input_nodes()
    first_var0 = [i for i, n in enumerate(inputs) if fc.in_var[n] == 0][0]     # an input node of variable 0 that has flow
    blk = nf[:, ns + first_var0 * C: ns + (first_var0 + 1) * C]
    with np.errstate(invalid="ignore"):
        assert blk[0].tolist() == [0.0, -np.inf, -np.inf, -np.inf, -np.inf]        # value 1: the first slot
    assert np.isnan(blk[1]).all()                                                  # value 0: no slot, 0 / 0
    fixed = O.normalized_flows(fc, data, double=True, as_written=False)
    blk = fixed[:, ns + first_var0 * C: ns + (first_var0 + 1) * C]
    assert blk[0].tolist() == [-np.inf, 0.0, -np.inf, -np.inf, -np.inf]
    assert blk[1].tolist() == [0.0, -np.inf, -np.inf, -np.inf, -np.inf]
    np.testing.assert_array_equal(fixed[:, :ns], nf[:, :ns])


def test_normalize_params_against_scipy():
    """normalize_params (src/misc.jl:448-498): input entries -> scipy's softmax per input node, sum parameters ->
    scipy's log_softmax per sum node; undo: log(p + 1e-6) where p > 0 (:380-393)."""
    from scipy.special import softmax, log_softmax
    fc = O.bits_compile(random_dag(4, 3, np.random.default_rng(2), width=3), 3, 4)
    rng = np.random.default_rng(3)
    n = len(fc.vectorize_parameters())
    p = rng.normal(0, 2, size=(3, n)).astype(np.float32)
    got = O.normalize_params(fc, p, double=True)
    pe = fc.sum_param_edges()
    ns = len(pe)
    par = fc.edge_parent()[pe]
    for node in np.unique(par):
        cols = np.nonzero(par == node)[0]
        assert (np.diff(cols) == 1).all()                       # a sum node's parameters sit side by side
        np.testing.assert_allclose(got[:, cols], log_softmax(p[:, cols].astype(np.float64), axis=1), rtol=1e-6, atol=1e-9)
    nin = len(fc.input_nodes())
    np.testing.assert_allclose(got[:, ns:].reshape(3, nin, 3), softmax(p[:, ns:].astype(np.float64).reshape(3, nin, 3), axis=2),
                               rtol=1e-6)
    back = O.normalize_params(fc, got, undo=True, double=True)
    np.testing.assert_allclose(back[:, ns:], np.log(got[:, ns:] + 1e-6), rtol=1e-6)
    np.testing.assert_allclose(back[:, :ns], got[:, :ns], atol=1e-6)     # already normalised: unchanged


# ---- soft_flow: the leaf statistics under soft_reg (src/regularization/reg_flow.jl:3-22) ----------------------

def test_soft_flow_as_written_by_hand():
    """One leaf, worked by hand from the source lines.  p = (0.5, 0.3, 0.2), x = 1, soft_reg = 0.1, width 3, node flow 2:
    window 0..2, sp = 1/3, base = 0.9 ln 0.3 + 0.1 / 3 = -1.08357552 + 0.03333333 = -1.05024219;
    counts[1] = (0.9 ln 0.3 + (0.1 / 3) ln 0.3) * 2 / base = -2.2474159 / -1.05024219 = 2.139903,
    counts[0] = (0.1 / 3) ln 0.5 * 2 / base = -0.04620981 / -1.05024219 = 0.0439992,
    counts[2] = (0.1 / 3) ln 0.2 * 2 / base = -0.1072959 / -1.05024219 = 0.1021630.
    Then a window cut by the end of the range: p = (0.1, 0.2, 0.3, 0.4), x = 3: c_start = 2, c_end = min(4, 3) = 3, n = 2,
    sp = 0.35, base = 0.9 ln 0.4 + 0.035 = -0.78966166: counts = (0, 0, 0.05 ln 0.3 * 2 / base, 0.95 ln 0.4 * 2 / base)
    = (0, 0, 0.1524669, 2.2046814).  With probabilities in place of the logarithms (as_written = False) the shares of
    a leaf add up to its flow; as written they do not."""
    from types import SimpleNamespace

    def leaf(p):
        return SimpleNamespace(n_nodes=1, type=np.array([O.INPUT], np.uint8), in_var=np.array([0], np.int32),
                               in_off=np.array([0], np.int64), leaf_logp=np.log(np.array(p)), C=len(p))
    flows = np.array([[2.0]])
    got = O.soft_flow_counts(leaf([0.5, 0.3, 0.2]), np.array([[1]]), flows, 0.1, 3, as_written=True, double=True)
    np.testing.assert_allclose(got, [0.0439992, 2.139903, 0.1021630], rtol=2e-6)
    got = O.soft_flow_counts(leaf([0.1, 0.2, 0.3, 0.4]), np.array([[3]]), flows, 0.1, 3, as_written=True, double=True)
    np.testing.assert_allclose(got, [0.0, 0.0, 0.1524669, 2.2046814], rtol=2e-6, atol=1e-12)
    assert abs(got.sum() - 2.0) > 0.1
    der = O.soft_flow_counts(leaf([0.1, 0.2, 0.3, 0.4]), np.array([[3]]), flows, 0.1, 3, as_written=False, double=True)
    assert abs(der.sum() - 2.0) < 1e-12
    np.testing.assert_allclose(der, [0, 0, 0.05 * 0.3 * 2 / (0.9 * 0.4 + 0.035), 0.95 * 0.4 * 2 / (0.9 * 0.4 + 0.035)], rtol=1e-12)


def test_soft_flow_derivative_form_is_the_soft_evidence_flow():
    """With probabilities where the source has heap entries, soft_flow is the leaf flow of the soft evidence that gives
    the leaves the smoothed value -- `orc_input_flows_soft`, pinned by central differences in tests/test_soft_evidence.py
    -- on a whole HCLT, windows cut at both ends included."""
    V, K, C, B, s, width = 6, 3, 7, 9, 0.15, 4
    parent, theta, leaf, fc = make_hclt(V, K, C, 5)
    rng = np.random.default_rng(3)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    data[0, :] = 0
    data[1, :] = C - 1
    ev = np.full((B, V, C), -np.inf)
    for b in range(B):
        for v in range(V):
            x = int(data[b, v])
            c0 = max(0, x - width // 2)
            c1 = min(c0 + width - 1, C - 1)
            ev[b, v, c0:c1 + 1] = np.log(s / (c1 - c0 + 1))
            ev[b, v, x] = np.log(np.exp(ev[b, v, x]) + 1 - s)
    mars = O.forward_soft(fc, ev, double=True)
    fl, _ = O.backward(fc, mars, double=True)
    want = O.input_flows_soft(fc, ev, mars, fl, double=True)
    got = O.soft_flow_counts(fc, data, fl, s, width, as_written=False, double=True)
    np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-12)
    written = O.soft_flow_counts(fc, data, fl, s, width, as_written=True, double=True)
    assert np.abs(written - want).max() > 1e-3        # the two forms are not the same numbers
