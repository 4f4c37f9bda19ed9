"""GPU parity of the general (layered) engine against the CPU oracle, through the C ABI:
the reference's fixture circuits, random DAGs with shared sub-circuits, multi-head circuits,
and the HCLT in its general form against the dense-block engine."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

LL_RTOL = 1e-4
PARAM_RTOL = 1e-4
FLOW_RTOL = 2e-4


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355
    return torch, pcmi355


def _compile(P, roots, V, C, heads=0):
    from helpers import describe_dag
    d = describe_dag(roots)
    return P.compile_circuit(d["node_type"], d["child_ptr"], d["child_idx"], d["sum_logp"], d["input_var"],
                             d["input_logp"], V, C, heads)


def _check_tables(bpc, fc):
    """Index tables and parameter vector of the compiled circuit against the oracle's flattening."""
    import pcmi355 as P
    t = fc.param_tables()
    order = fc.up_order()
    assert bpc.num_nodes() == fc.n_nodes and bpc.num_edges() == fc.n_edges
    for name in ("edge2param", "param2edge", "param2group", "pargroup_sizes", "innode2ncumparam"):
        assert np.array_equal(bpc.table(name), t[name]), name
    assert np.array_equal(bpc.table("edge_parent") - 1, fc.edge_parent()[order])
    assert np.array_equal(bpc.table("edge_prime") - 1, fc.prime[order])
    assert np.array_equal(bpc.table("edge_sub") - 1, fc.sub[order])
    assert np.array_equal(P.vectorize_parameters(bpc), fc.vectorize_parameters())
    return order


def _check_em_step(gpu, O, root, V, C, B, seed, pseudocount=0.1, inertia=0.9):
    torch, P = gpu
    from helpers import rel_err
    fc = O.bits_compile(root, C, V)
    bpc = _compile(P, [root], V, C)
    order = _check_tables(bpc, fc)
    rng = np.random.default_rng(seed)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    d = torch.from_numpy(data).cuda()

    mars_ref = O.forward(fc, data)
    ll = P.loglikelihoods(bpc, d).cpu().numpy()
    assert rel_err(ll, mars_ref[-1]).max() < LL_RTOL
    ll2 = P.probs_flows_circuit(bpc, d).cpu().numpy()
    assert np.array_equal(ll, ll2)

    flows_ref, ea_ref = O.backward(fc, mars_ref)
    lf_ref = O.input_flows(fc, data, flows_ref)
    mars, flows = bpc.get_node_values(B)
    assert np.abs(mars - mars_ref).max() < LL_RTOL * np.abs(mars_ref).max()
    assert np.abs(flows - flows_ref).max() < FLOW_RTOL
    ea, lf = bpc.get_aggregates()
    assert np.abs(ea - ea_ref[order]).max() < FLOW_RTOL * max(ea_ref.max(), 1.0)
    assert np.abs(lf - lf_ref).max() < FLOW_RTOL * max(lf_ref.max(), 1.0)

    import pcmi355._lib as L
    L.check(L.lib.pcm_em_update(bpc.handle, pseudocount, inertia))
    logp, leaf = O.em_update(fc, ea_ref, lf_ref, pseudocount, inertia)
    new = fc.copy()
    new.logp, new.leaf_logp = logp, leaf
    got = P.vectorize_parameters(bpc)
    assert rel_err(np.exp(got), np.exp(new.vectorize_parameters())).max() < PARAM_RTOL
    return bpc, fc


def test_three_var_fixture_known_answers(gpu, oracle):
    """test/bits_circuit_tests.jl:13-24 and test/misc_tests.jl:39-62 on simple_3vars_circuit."""
    torch, P = gpu
    from helpers import simple_3vars_circuit
    root = simple_3vars_circuit(5, np.random.default_rng(3))
    bpc = _compile(P, [root], 3, 5)
    assert bpc.num_nodes() == 9 and bpc.num_edges() == 6
    assert bpc.num_parameters() == 32 and bpc.num_input_params() == 30
    assert bpc.table("edge2param").tolist() == [0, 0, 0, 0, 1, 2]
    assert bpc.table("param2edge").tolist() == [5, 6]
    assert bpc.table("param2group").tolist() == [1, 1]
    assert bpc.table("pargroup_sizes").tolist() == [2]
    assert bpc.table("innode2ncumparam").tolist() == [5, 10, 15, 20, 25, 30]


@pytest.mark.parametrize("B", [1, 7, 64, 200])
def test_three_var_fixture_em_step(gpu, oracle, B):
    from helpers import simple_3vars_circuit
    root = simple_3vars_circuit(5, np.random.default_rng(11), weights=[0.3, 0.7])
    _check_em_step(gpu, oracle, root, 3, 5, B, seed=B)


@pytest.mark.parametrize("V,C,width,seed", [(4, 3, 2, 0), (9, 6, 4, 1), (17, 11, 5, 2), (6, 256, 3, 3)])
def test_random_dag_em_step(gpu, oracle, V, C, width, seed):
    from helpers import random_dag
    root = random_dag(V, C, np.random.default_rng(seed), width=width)
    _check_em_step(gpu, oracle, root, V, C, 96, seed=seed + 50)


def test_random_dag_em_step_on_a_large_batch(gpu, oracle):
    """Layers of many nodes with few edges each take the layer kernels with four examples per lane
    (at least 16384 (node, 64 examples) pairs): 96 input nodes and 16000 examples."""
    from helpers import random_dag
    root = random_dag(12, 5, np.random.default_rng(21), width=8)
    _check_em_step(gpu, oracle, root, 12, 5, 16000, seed=77)


def test_layered_engine_on_a_batch_that_saturates_the_device(gpu, oracle):
    """Layers of many-edged nodes with at least 32768 (node, 64 examples) pairs take two examples per lane: an HCLT
    with K = 32 compiled as a general circuit, 8192 examples, against the block engine on the same tree and
    parameters (itself checked against the oracle elsewhere) and against the oracle on the head of the batch."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta, describe_dag, rel_err
    V, K, C, B = 30, 32, 16, 8192
    rng = np.random.default_rng(31)
    parent = np.full(V, -1, np.int32)
    for v in range(1, V):
        parent[v] = rng.integers(max(0, v - 4), v)
    parent, theta, leaf, fc = make_hclt(V, K, C, 31, parent=parent)
    a = P.hclt_from_clt(parent, C, K)
    a.set_params(block_theta(parent, K, theta), leaf)
    d = describe_dag([O.hclt_dag(parent, K, C, theta, leaf)])
    g = P.compile_circuit(d["node_type"], d["child_ptr"], d["child_idx"], d["sum_logp"], d["input_var"], d["input_logp"], V, C)
    np.testing.assert_allclose(P.vectorize_parameters(a), P.vectorize_parameters(g), atol=1e-6)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    dd = torch.from_numpy(data).cuda()
    la, lg = P.loglikelihoods(a, dd).cpu().numpy(), P.loglikelihoods(g, dd).cpu().numpy()
    assert rel_err(lg, la).max() < LL_RTOL
    assert rel_err(lg[:64], O.forward(fc, data[:64])[-1]).max() < LL_RTOL
    for c in (a, g):
        P.mini_batch_em(c, dd, 1, batch_size=B, pseudocount=0.1, param_inertia=0.3)
    pa, pg = P.vectorize_parameters(a), P.vectorize_parameters(g)
    assert rel_err(np.exp(pg), np.exp(pa)).max() < PARAM_RTOL


def test_layered_engine_with_value_arrays_beyond_two_gigabytes(gpu, oracle):
    """From 2 GiB of node values on, the layer kernels address rows through pointers instead of buffer descriptors:
    a circuit of about 7900 nodes (K = 32 HCLT over 128 variables) on 73728 examples, 96 copies of 768 distinct ones.  The
    likelihood of a copy is that of its original in a 768-example batch (the descriptor path) and the same bits in
    every copy, and with no
    pseudocount the EM update of the large batch is the update of the small one up to rounding."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, describe_dag, rel_err
    V, K, C, base, copies = 128, 32, 6, 768, 96
    rng = np.random.default_rng(41)
    parent = np.full(V, -1, np.int32)
    for v in range(1, V):
        parent[v] = rng.integers(max(0, v - 3), v)
    parent, theta, leaf, fc = make_hclt(V, K, C, 41, parent=parent)
    d = describe_dag([O.hclt_dag(parent, K, C, theta, leaf)])

    def compiled():
        return P.compile_circuit(d["node_type"], d["child_ptr"], d["child_idx"], d["sum_logp"], d["input_var"],
                                 d["input_logp"], V, C)
    small, large = compiled(), compiled()
    assert small.num_nodes() * base * 4 < 2 ** 31 <= large.num_nodes() * base * copies * 4
    data = rng.integers(0, C, size=(base, V)).astype(np.uint8)
    ds = torch.from_numpy(data).cuda()
    dl = torch.from_numpy(np.tile(data, (copies, 1))).cuda()
    ll_s = P.loglikelihoods(small, ds).cpu().numpy()
    assert rel_err(ll_s[:32], O.forward(fc, data[:32])[-1]).max() < LL_RTOL
    ll_l = P.loglikelihoods(large, dl).cpu().numpy().reshape(copies, base)
    # (which build of the layer kernels a layer takes depends on the batch, and they fold a node's edges in
    # different groupings: equal to rounding, not to the bit)
    np.testing.assert_allclose(ll_l, np.broadcast_to(ll_s, (copies, base)), rtol=2e-6)
    np.testing.assert_array_equal(ll_l, np.broadcast_to(ll_l[0], (copies, base)))   # a copy is a copy
    P.mini_batch_em(small, ds, 1, batch_size=base, pseudocount=0.0, param_inertia=0.0)
    P.mini_batch_em(large, dl, 1, batch_size=base * copies, pseudocount=0.0, param_inertia=0.0)
    ps, pl = np.exp(P.vectorize_parameters(small)), np.exp(P.vectorize_parameters(large))
    assert np.abs(pl - ps).max() < 2e-5


def test_per_example_weights(gpu, oracle):
    """`weights` of probs_flows_circuit_with_reg / mini_batch_em_with_reg (reg_flow.jl:38-39,190-191: an example's
    edge and leaf flows times its weight), as the flow the example starts with at the root: a single-root circuit
    of the layered engine against the oracle seeded with the weights, the driver against the same loop written
    out."""
    torch, P = gpu
    O = oracle
    import pcmi355._lib as L
    from helpers import random_dag
    V, C, B = 8, 4, 150
    rng = np.random.default_rng(61)
    root = random_dag(V, C, rng, width=3)
    fc = O.bits_compile(root, C, V)
    bpc = _compile(P, [root], V, C)
    order = fc.up_order()
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    w = rng.uniform(0.0, 3.0, size=B).astype(np.float32)
    w[::7] = 0.0
    d = torch.from_numpy(data).cuda()
    ll = P.probs_flows_circuit(bpc, d, weights=w).cpu().numpy()
    mars = O.forward(fc, data)
    assert np.abs(ll - mars[-1]).max() < LL_RTOL * np.abs(mars[-1]).max()      # likelihoods are not weighted
    flows, ea_ref = O.backward(fc, mars, root_ids=np.array([fc.n_nodes - 1], np.int32), root_flow=w[None, :])
    lf_ref = O.input_flows(fc, data, flows)
    ea, lf = bpc.get_aggregates()
    assert np.abs(ea - ea_ref[order]).max() < FLOW_RTOL * max(ea_ref.max(), 1.0)
    assert np.abs(lf - lf_ref).max() < FLOW_RTOL * max(lf_ref.max(), 1.0)
    # the weighted mean of the data set's log-likelihoods, with chunks that do not divide the data set
    assert abs(P.loglikelihood(bpc, d, w, batch_size=64) - (mars[-1].astype(np.float64) * w).sum() / w.astype(np.float64).sum()) < 1e-5
    assert abs(P.loglikelihood(bpc, d) - mars[-1].astype(np.float64).mean()) < 1e-5
    # weights of one are no weights
    P.probs_flows_circuit(bpc, d, weights=np.ones(B, np.float32))
    ea1, lf1 = bpc.get_aggregates()
    P.probs_flows_circuit(bpc, d)
    ea0, lf0 = bpc.get_aggregates()
    np.testing.assert_array_equal(ea1, ea0)
    np.testing.assert_array_equal(lf1, lf0)
    # the driver: two circuits, one through mini_batch_em_with_reg(weights=...), one through the loop written out
    a, b = _compile(P, [root], V, C), _compile(P, [root], V, C)
    lls = P.mini_batch_em_with_reg(a, d, 2, batch_size=50, pseudocount=0.1, param_inertia=0.4, shuffle="none", weights=w)
    for _ in range(2):
        for s0 in range(0, B, 50):
            ids = np.arange(s0, s0 + 50, dtype=np.int32)
            P.probs_flows_circuit(b, d, example_ids=ids, weights=w)
            L.check(L.lib.pcm_em_update(b.handle, 0.1, 0.4))
    np.testing.assert_array_equal(P.vectorize_parameters(a), P.vectorize_parameters(b))
    assert len(lls) == 2 and lls[1] > lls[0]
    with pytest.raises(ValueError):
        P.mini_batch_em_with_reg(a, d, 1, batch_size=50, pseudocount=0.1, param_inertia=0.4, weights=w[:10])


def test_driver_called_again_without_clearing_its_flow_memory(gpu, oracle):
    """`init_clear_mem = false` (src-jl/multi_head_pc/em.jl:6,28-31): two calls of one epoch, the second keeping the
    accumulators, are one call of two epochs; with the default the second call starts from cleared ones."""
    torch, P = gpu
    from helpers import random_dag
    V, C, B = 7, 4, 120
    rng = np.random.default_rng(71)
    root = random_dag(V, C, rng, width=3)
    d = torch.from_numpy(rng.integers(0, C, size=(B, V)).astype(np.uint8)).cuda()
    kw = dict(batch_size=40, pseudocount=0.1, param_inertia=0.6, flow_memory=150.0, shuffle="none")
    one, two, cleared = (_compile(P, [root], V, C) for _ in range(3))
    P.mini_batch_em_with_reg(one, d, 2, **kw)
    for c, keep in ((two, False), (cleared, True)):
        P.mini_batch_em_with_reg(c, d, 1, **kw)
        P.mini_batch_em_with_reg(c, d, 1, init_clear_mem=keep, **kw)
    np.testing.assert_array_equal(P.vectorize_parameters(two), P.vectorize_parameters(one))
    assert np.abs(P.vectorize_parameters(cleared) - P.vectorize_parameters(one)).max() > 1e-6


def test_example_ids_and_flow_memory(gpu, oracle):
    """Batches picked by example ids; accumulators scaled by `rate` before a batch
    (src/regularization/reg_em.jl:276-284)."""
    torch, P = gpu
    O = oracle
    from helpers import random_dag
    V, C = 7, 5
    root = random_dag(V, C, np.random.default_rng(5), width=3)
    fc = O.bits_compile(root, C, V)
    bpc = _compile(P, [root], V, C)
    order = fc.up_order()
    rng = np.random.default_rng(6)
    data = rng.integers(0, C, size=(300, V)).astype(np.uint8)
    d = torch.from_numpy(data).cuda()
    ids1 = rng.permutation(300)[:70].astype(np.int32)
    ids2 = rng.permutation(300)[:33].astype(np.int32)
    P.probs_flows_circuit(bpc, d, example_ids=ids1)
    P.probs_flows_circuit(bpc, d, example_ids=ids2, rate=0.25)
    ea, lf = bpc.get_aggregates()
    m1 = O.forward(fc, data, ids1)
    f1, ea1 = O.backward(fc, m1)
    lf1 = O.input_flows(fc, data, f1, ids1)
    m2 = O.forward(fc, data, ids2)
    f2, ea2 = O.backward(fc, m2)
    lf2 = O.input_flows(fc, data, f2, ids2)
    ea_ref = 0.25 * ea1 + ea2
    lf_ref = 0.25 * lf1 + lf2
    assert np.abs(ea - ea_ref[order]).max() < FLOW_RTOL * ea_ref.max()
    assert np.abs(lf - lf_ref).max() < FLOW_RTOL * lf_ref.max()


def test_multihead_closed_forms(gpu, oracle):
    """test/multi_head_pc/multi_head_pc_learning_tests.jl:11-47."""
    torch, P = gpu
    from helpers import simple_multihead_circuit
    heads = simple_multihead_circuit(5)
    heads[0].children[0].children[0].logps = np.log(np.array([0.1, 0.2, 0.3, 0.3, 0.1], np.float32))
    heads[0].logps = np.log(np.array([0.2, 0.8], np.float32))
    heads[1].logps = np.log(np.array([0.6, 0.4], np.float32))
    bpc = _compile(P, heads, 3, 5, heads=2)
    assert bpc.size("heads") == 2
    assert bpc.table("heads").tolist() == [9, 10]          # the reference's root_ids (fake root would be 11)
    data = torch.tensor([[0, 0, 0], [2, 0, 0]], dtype=torch.uint8).cuda()
    head_mask = torch.tensor([[1.0, 0.0], [0.0, 1.0]]).cuda()
    want = [np.log(0.1 * 0.2 * 0.2 * 0.2 + 0.2 ** 3 * 0.8), np.log(0.3 * 0.2 * 0.2 * 0.6 + 0.2 ** 3 * 0.4)]
    lls = P.multihead_loglikelihoods(bpc, data, head_mask).cpu().numpy()
    np.testing.assert_allclose(lls, want, rtol=1e-5)
    per_head = P.loglikelihoods(bpc, data).cpu().numpy()
    assert per_head.shape == (2, 2)
    np.testing.assert_allclose([per_head[0, 0], per_head[1, 1]], want, rtol=1e-5)

    # the means over the data set (reg_likelihood.jl:164-173, reg_em.jl:191-197), against the closed forms above
    assert abs(P.loglikelihood(bpc, data, head_mask=head_mask) - np.mean(want)) < 1e-5
    assert abs(P.weighted_ll(bpc, data, np.float32([3.0, 1.0]), head_mask=head_mask) - (3 * want[0] + want[1]) / 4) < 1e-5
    assert P.loglikelihood_probcat is P.loglikelihood and P.loglikelihoods_probcat is P.loglikelihoods
    # weighted_ll without weights: the per-example vector, as reg_em.jl:191-197 returns it (here: one row per head)
    np.testing.assert_array_equal(P.weighted_ll(bpc, data).cpu().numpy(), per_head)
    np.testing.assert_array_equal(P.weighted_ll(bpc, data, head_mask=head_mask).cpu().numpy(), lls)
    for bad in ([1.0, -0.5], [np.inf, 1.0], [np.nan, 1.0]):
        with pytest.raises(ValueError, match="finite and >= 0"):
            P.probs_flows_circuit(bpc, data, head_mask=head_mask, weights=np.float32(bad))
    with pytest.raises(ValueError, match="head_mask"):
        P.loglikelihood(bpc, data)
    with pytest.raises(ValueError, match="3 weights for 2 examples"):
        P.loglikelihood(bpc, data, np.ones(3, np.float32), head_mask=head_mask)

    ll = P.probs_flows_circuit(bpc, data, head_mask=head_mask).cpu().numpy()
    np.testing.assert_allclose(ll, want, rtol=1e-5)
    mars, flows = bpc.get_node_values(2)
    mars, flows = mars.T, flows.T        # [example, node] like the reference
    n = lambda i: i - 1                  # the reference's 1-based node ids
    assert flows[0, n(9)] == 1.0 and flows[0, n(10)] == 0.0
    assert flows[1, n(9)] == 0.0 and flows[1, n(10)] == 1.0
    f32 = np.float32
    np.testing.assert_allclose(flows[0, n(4)], np.exp(mars[0, 0] + mars[0, 1] + mars[0, 2] + np.log(f32(0.2)) - mars[0, n(9)]), rtol=1e-5)
    np.testing.assert_allclose(flows[0, n(8)], np.exp(mars[0, 4] + mars[0, 5] + mars[0, 6] + np.log(f32(0.8)) - mars[0, n(9)]), rtol=1e-5)
    np.testing.assert_allclose(flows[1, n(4)], np.exp(mars[1, 0] + mars[1, 1] + mars[1, 2] + np.log(f32(0.6)) - mars[1, n(10)]), rtol=1e-5)
    np.testing.assert_allclose(flows[1, n(8)], np.exp(mars[1, 4] + mars[1, 5] + mars[1, 6] + np.log(f32(0.4)) - mars[1, n(10)]), rtol=1e-5)


def test_multihead_soft_mask_em_matches_oracle(gpu, oracle):
    """Soft head masks: flows seeded by head_mask[b, h] (src-jl/multi_head_pc/flow.jl:141-176),
    mixture LL (likelihood.jl:3-12), then the four update calls (em.jl:77-81).  The oracle
    runs the reference's construction: a fake root over the heads whose edges are skipped."""
    torch, P = gpu
    O = oracle
    from helpers import random_dag, rel_err
    V, C, H, B = 6, 4, 3, 80
    rng = np.random.default_rng(21)
    body = random_dag(V, C, rng, width=3)
    # heads: H sums over the products feeding the body's root
    prods = body.children
    heads = [O.summate(*prods, logps=np.log(rng.dirichlet(np.ones(len(prods)))).astype(np.float32)) for _ in range(H)]
    bpc = _compile(P, heads, V, C, heads=H)
    fake = O.summate(*heads)
    fc = O.bits_compile(fake, C, V)
    n_real = fc.n_nodes - 1
    assert bpc.num_nodes() == n_real
    root_ids = (bpc.table("heads") - 1).astype(np.int32)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    mask = rng.random((B, H)).astype(np.float32) + 0.05
    mask[::7, 1] = 0.0     # hard zeros: log(0) = -inf must fold away
    d = torch.from_numpy(data).cuda()
    hm = torch.from_numpy(mask).cuda()

    ll = P.probs_flows_circuit(bpc, d, head_mask=hm).cpu().numpy()
    mars_ref = O.forward(fc, data)
    with np.errstate(divide="ignore"):
        mix = np.logaddexp.reduce(mars_ref[root_ids].astype(np.float64) + np.log(mask.T.astype(np.float64)), axis=0) \
            - np.log(mask.sum(axis=1, dtype=np.float64))
    assert rel_err(ll, mix).max() < LL_RTOL
    skip = (fc.edge_parent() == fc.n_nodes - 1).astype(np.uint8)
    flows_ref, ea_ref = O.backward(fc, mars_ref, skip=skip, root_ids=root_ids, root_flow=np.ascontiguousarray(mask.T))
    lf_ref = O.input_flows(fc, data, flows_ref)
    mars, flows = bpc.get_node_values(B)
    assert np.abs(flows - flows_ref[:n_real]).max() < FLOW_RTOL
    ea, lf = bpc.get_aggregates()
    order = fc.up_order()
    order = order[fc.edge_parent()[order] != fc.n_nodes - 1]
    assert np.abs(ea - ea_ref[order]).max() < FLOW_RTOL * ea_ref.max()
    assert np.abs(lf - lf_ref).max() < FLOW_RTOL * lf_ref.max()

    lls = P.mini_batch_em_for_multihead_pc(bpc, d, hm, 2, batch_size=40, pseudocount=0.1, param_inertia=0.5,
                                           shuffle="none")
    assert len(lls) == 2 and lls[1] > lls[0]


def test_config_patch_circuit_with_128_heads_and_top_hclt(gpu, oracle):
    """Patch-clustered configuration at its real shape: one 8x8x3 patch circuit (192 variables,
    K = 32) with 128 heads selected by a cluster id, and the top HCLT over 64 cluster indices
    (K = 64, 128 categories), batch 1024.  Oracle on a subset; on the whole batch the flows
    obey conservation and EM raises the likelihood."""
    torch, P = gpu
    O = oracle
    import sys
    from pcmi355 import workloads
    from helpers import multihead_hclt, rel_err
    sys.setrecursionlimit(20000)
    V, K, C, H, B = 192, 32, 256, 128, 1024
    rng = np.random.default_rng(1004)
    data = workloads.grf_images(B, 8, 8, 3, 3.0, 0.8, seed=1004)
    parent = workloads.chow_liu_parent(data)
    heads, _ = multihead_hclt(parent, K, C, H, rng)
    bpc = _compile(P, heads, V, C, heads=H)
    assert bpc.size("heads") == H
    cluster = rng.integers(0, H, size=B)
    mask = np.zeros((B, H), np.float32)
    mask[np.arange(B), cluster] = 1.0
    d = torch.from_numpy(data).cuda()
    hm = torch.from_numpy(mask).cuda()
    ll = P.probs_flows_circuit(bpc, d, head_mask=hm).cpu().numpy()
    sub = 24
    fc = O.bits_compile(O.summate(*heads), C, V)
    root_ids = (bpc.table("heads") - 1).astype(np.int32)
    mars = O.forward(fc, data[:sub])
    want = mars[root_ids[cluster[:sub]], np.arange(sub)]
    assert rel_err(ll[:sub], want).max() < LL_RTOL
    per_head = P.loglikelihoods(bpc, d[:sub].contiguous()).cpu().numpy()
    assert per_head.shape == (sub, H)
    assert rel_err(per_head, mars[root_ids].T).max() < LL_RTOL
    ea, lf = bpc.get_aggregates()
    np.testing.assert_allclose(lf.sum(), B * V, rtol=1e-4)     # one unit of flow per example and variable
    lls = P.mini_batch_em_for_multihead_pc(bpc, d, hm, 3, batch_size=B, pseudocount=0.1, param_inertia=0.9, shuffle="none")
    assert lls[2] > lls[1] > lls[0]

    # top circuit: hard cluster ids of the 64 patches as uint8 data with 128 categories
    Vt, Kt, Ct = 64, 64, 128
    ids = rng.integers(0, Ct, size=(B, Vt)).astype(np.uint8)
    ids[:, 1:] = (ids[:, :-1] + rng.integers(0, 3, size=(B, Vt - 1))) % Ct      # some dependence
    tp = workloads.chow_liu_parent(ids)
    theta, leaf = workloads.init_params(tp, Kt, Ct, 2004)
    top = P.hclt_from_clt(tp, Ct, Kt)
    top.set_params(theta, leaf)
    dt = torch.from_numpy(ids).cuda()
    ch, _ = O.clt_children(tp)
    ft = O.hclt_flat(tp, Kt, Ct, {v: theta[v] for v in range(Vt) if ch[v]}, leaf)
    llt = P.loglikelihoods(top, dt).cpu().numpy()
    assert rel_err(llt[:sub], O.forward(ft, ids[:sub])[-1]).max() < LL_RTOL
    lls = P.mini_batch_em_with_reg(top, dt, 3, batch_size=B, pseudocount=0.1, param_inertia=0.9, shuffle="none")
    assert lls[2] > lls[1] > lls[0]


def test_patch_circuit_on_the_block_engine_at_its_real_shape(gpu, oracle):
    """The patch circuit of the patch-clustered configuration as the benchmark runs it: built from its
    tree with pcm_hclt_create_multihead (body on the walk kernels, 128 heads in the head kernels), 192
    variables, K = 32, 256 categories, batch 1024.  Against the layered engine on the equivalent
    description over the whole batch (per-head values, mixtures and EM updates under a one-hot and a soft
    head mask) and against the oracle on a subset."""
    torch, P = gpu
    O = oracle
    import sys
    from pcmi355 import workloads
    from pcmi355._lib import lib, check
    from helpers import multihead_hclt, rel_err
    sys.setrecursionlimit(20000)
    V, K, C, H, B = 192, 32, 256, 128, 1024
    rng = np.random.default_rng(1004)
    data = workloads.grf_images(B, 8, 8, 3, 3.0, 0.8, seed=1004)
    parent = workloads.chow_liu_parent(data)
    heads, _ = multihead_hclt(parent, K, C, H, rng)
    gen = _compile(P, heads, V, C, heads=H)
    blk = P.multihead_hclt_from_clt(parent, C, K, H)
    assert blk.size("walk_kernels") in (1, 2)
    pv = P.vectorize_parameters(gen)
    P.update_parameters(blk, pv)
    np.testing.assert_array_equal(P.vectorize_parameters(blk), pv)
    d = torch.from_numpy(data).cuda()
    ll_g = P.loglikelihoods(gen, d).cpu().numpy()
    ll_b = P.loglikelihoods(blk, d).cpu().numpy()
    assert ll_b.shape == (B, H) and rel_err(ll_b, ll_g).max() < LL_RTOL
    sub = 24
    fc = O.bits_compile(O.summate(*heads), C, V)
    root_ids = (blk.table("heads") - 1).astype(np.int64)
    mars = O.forward(fc, data[:sub])
    assert rel_err(ll_b[:sub], mars[root_ids].T).max() < LL_RTOL
    cluster = rng.integers(0, H, size=B)
    for soft in (False, True):
        mask = np.zeros((B, H), np.float32)
        mask[np.arange(B), cluster] = 1.0
        if soft:
            mask = (mask + rng.random((B, H)).astype(np.float32) * (rng.random((B, H)) < 0.1)).astype(np.float32)
        hm = torch.from_numpy(mask).cuda()
        P.update_parameters(gen, pv)
        P.update_parameters(blk, pv)
        mix_g = P.probs_flows_circuit(gen, d, head_mask=hm).cpu().numpy()
        mix_b = P.probs_flows_circuit(blk, d, head_mask=hm).cpu().numpy()
        assert rel_err(mix_b, mix_g).max() < LL_RTOL
        with np.errstate(divide="ignore"):
            want = np.logaddexp.reduce(mars[root_ids].astype(np.float64) + np.log(mask[:sub].T.astype(np.float64)), axis=0) \
                - np.log(mask[:sub].sum(axis=1, dtype=np.float64))
        assert rel_err(mix_b[:sub], want).max() < LL_RTOL
        check(lib.pcm_em_update(gen.handle, 0.1, 0.9))
        check(lib.pcm_em_update(blk.handle, 0.1, 0.9))
        a, b = np.exp(P.vectorize_parameters(gen).astype(np.float64)), np.exp(P.vectorize_parameters(blk).astype(np.float64))
        assert (np.abs(a - b) / np.maximum(a, 1e-6)).max() < 2e-4          # two float32 engines, as in the random-shape test
    # the same EM step on the subset against the oracle (one-hot mask)
    P.update_parameters(blk, pv)
    mask = np.zeros((sub, H), np.float32)
    mask[np.arange(sub), cluster[:sub]] = 1.0
    P.probs_flows_circuit(blk, d[:sub].contiguous(), head_mask=torch.from_numpy(mask).cuda())
    check(lib.pcm_em_update(blk.handle, 0.1, 0.9))
    skip = (fc.edge_parent() == fc.n_nodes - 1).astype(np.uint8)

    def oracle_step(double):
        m = O.forward(fc, data[:sub], double=double)
        fl, ea = O.backward(fc, m, skip=skip, root_ids=root_ids.astype(np.int32), root_flow=np.ascontiguousarray(mask.T),
                            double=double)
        lf = O.input_flows(fc, data[:sub], fl, double=double)
        logp_new, leaf_new = O.em_update(fc, ea, lf, 0.1, 0.9, double=double)
        ref = fc.copy()
        ref.logp, ref.leaf_logp = logp_new, leaf_new
        return np.exp(ref.vectorize_parameters().astype(np.float64)) if not double else \
            np.exp(np.concatenate([logp_new[ref.sum_param_edges()]] +
                                  [leaf_new[ref.in_off[n]:ref.in_off[n] + C] for n in ref.input_nodes()]))

    want64, want32 = oracle_step(True), oracle_step(False)
    n_real = len(pv)
    # (the oracle's circuit has the fake root's H edges as extra sum parameters at the end of the sum block)
    ns = blk.num_inner_params()
    got = np.exp(P.vectorize_parameters(blk).astype(np.float64))
    # 24 examples leave most edges little more than their pseudocount share, and the body is 60 levels deep:
    # where the float32 oracle (the reference's arithmetic) cannot hold 1e-4 against float64, the library
    # may be as far from the exact result as twice the float32 oracle is
    for lo_g, hi_g, lo_w, hi_w in ((0, ns, 0, ns), (ns, n_real, len(want64) - (n_real - ns), len(want64))):
        e_gpu = rel_err(got[lo_g:hi_g], want64[lo_w:hi_w]).max()
        e_f32 = rel_err(want32[lo_w:hi_w], want64[lo_w:hi_w]).max()
        print(f"patch circuit, block engine vs float64 {e_gpu:.2e}, float32 oracle vs float64 {e_f32:.2e}")
        assert e_gpu < max(PARAM_RTOL, 2 * e_f32)


def test_hclt_general_form_matches_block_engine(gpu, oracle):
    """The same HCLT through both engines: LL, parameter vector after an EM step."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, correlated_data, block_theta, rel_err
    V, K, C, B = 11, 16, 9, 128
    parent, theta, leaf, fc = make_hclt(V, K, C, 77)
    dense = P.hclt_from_clt(parent, C, K)
    dense.set_params(block_theta(parent, K, theta), leaf)
    general = _compile(P, [O.hclt_dag(parent, K, C, theta, leaf)], V, C)
    for name in ("edge2param", "param2edge", "param2group", "pargroup_sizes", "edge_parent", "edge_prime", "edge_sub"):
        assert np.array_equal(dense.table(name), general.table(name)), name
    p0 = P.vectorize_parameters(dense)
    assert np.array_equal(p0, P.vectorize_parameters(general))
    data = correlated_data(B, V, C, 78, parent)
    d = torch.from_numpy(data).cuda()
    import pcmi355._lib as L
    lls = []
    for bpc in (dense, general):
        ll = torch.empty(B, device="cuda")
        L.check(L.lib.pcm_em_step(bpc.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, 0.1, 0.9, ll.data_ptr()))
        lls.append(ll.cpu().numpy())
    assert rel_err(lls[0], lls[1]).max() < LL_RTOL
    assert rel_err(np.exp(P.vectorize_parameters(dense)), np.exp(P.vectorize_parameters(general))).max() < PARAM_RTOL


def test_error_paths(gpu):
    torch, P = gpu
    import pcmi355._lib as L
    nt = np.array([0, 0, 1], np.uint8)
    ok = dict(child_ptr=[0, 0, 0, 2], child_idx=[0, 1], sum_logp=np.log([0.5, 0.5]), input_var=[0, 0, -1],
              input_logp=np.log(np.full(8, 0.25)))
    P.compile_circuit(nt, ok["child_ptr"], ok["child_idx"], ok["sum_logp"], ok["input_var"], ok["input_logp"], 1, 4)
    with pytest.raises(L.PcmError):      # child that is not an earlier node
        P.compile_circuit(nt, ok["child_ptr"], [0, 2], ok["sum_logp"], ok["input_var"], ok["input_logp"], 1, 4)
    with pytest.raises(L.PcmError):      # variable out of range
        P.compile_circuit(nt, ok["child_ptr"], ok["child_idx"], ok["sum_logp"], [0, 3, -1], ok["input_logp"], 1, 4)
    with pytest.raises(L.PcmError):      # inner node without children
        P.compile_circuit(nt, [0, 0, 0, 0], [], [], ok["input_var"], ok["input_logp"], 1, 4)
    bpc = P.compile_circuit(nt, ok["child_ptr"], ok["child_idx"], ok["sum_logp"], ok["input_var"], ok["input_logp"], 1, 4)
    with pytest.raises(L.PcmError):      # update before any flows
        L.check(L.lib.pcm_em_update(bpc.handle, 0.1, 0.9))
    with pytest.raises(ValueError):      # wrong number of variables
        P.loglikelihoods(bpc, torch.zeros((4, 2), dtype=torch.uint8, device="cuda"))


def test_statistics_are_the_same_bits_on_every_run(gpu, oracle):
    """No floating-point atomics anywhere on the path: the accumulated edge and leaf statistics of a batch
    are identical, bit for bit, however often the pass is repeated -- layered engine with heads, block
    engine with heads, and the block engine on soft evidence."""
    torch, P = gpu
    from helpers import multihead_hclt
    rng = np.random.default_rng(11)
    V, K, C, H, B = 24, 16, 32, 12, 700
    parent = np.array([-1] + [int(rng.integers(0, v)) for v in range(1, V)], np.int32)
    heads, _ = multihead_hclt(parent, K, C, H, rng)
    data = torch.from_numpy(rng.integers(0, C, size=(B, V)).astype(np.uint8)).cuda()
    mask = torch.from_numpy(rng.dirichlet(np.ones(H), size=B).astype(np.float32)).cuda()
    layered = _compile(P, heads, V, C, H)
    assert layered.size("dense_groups") == len(set(parent[1:].tolist()))    # every inner tree node's sums (the root's: the heads) run as blocks
    block = P.multihead_hclt_from_clt(parent, C, K, H)
    P.update_parameters(block, P.vectorize_parameters(layered))
    soft = P.hclt_from_clt(parent, C, K)
    ev = torch.from_numpy((rng.normal(-30, 3, (B, V, 1)) + rng.gumbel(0, 2, (B, V, C))).astype(np.float32)).cuda()

    from pcmi355._lib import lib, check

    def stats(c, x, hm):
        P.update_parameters(c, start[id(c)])
        P.probs_flows_circuit(c, x, head_mask=hm)
        agg = c.get_aggregates() if c is layered else c.get_flows()
        check(lib.pcm_em_update(c.handle, 0.1, 0.9))            # the head statistics show in the updated parameters
        return (*agg, P.vectorize_parameters(c))

    start = {id(c): P.vectorize_parameters(c) for c in (layered, block, soft)}
    for c, x, hm in ((layered, data, mask), (block, data, mask), (soft, ev, None)):
        first = stats(c, x, hm)
        for _ in range(4):
            again = stats(c, x, hm)
            for a, b in zip(first, again):
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert all(np.isfinite(a).all() for a in first) and first[0].sum() > 0 and first[1].sum() > 0


def _with_and_without_groups(P, heads, V, C):
    """The circuit compiled twice: sums with one list of children as blocks on the matrix cores, and (the switch the
    library reads when a circuit is created) every sum edge by edge on the layer kernels."""
    import os
    grouped = _compile(P, heads, V, C, len(heads))
    os.environ["PCMI355_DENSE_GROUPS"] = "0"
    try:
        plain = _compile(P, heads, V, C, len(heads))
    finally:
        del os.environ["PCMI355_DENSE_GROUPS"]
    assert plain.size("dense_groups") == 0 and plain.size("layer_nodes") == plain.num_nodes()
    return grouped, plain


def _without_group_walks(P, heads, V, C):
    """... and with its groups, but a launch per layer where runs of layers would go as one walk launch."""
    import os
    os.environ["PCMI355_GROUP_WALK"] = "0"
    try:
        c = _compile(P, heads, V, C, len(heads))
    finally:
        del os.environ["PCMI355_GROUP_WALK"]
    assert c.size("walk_levels") == 0
    return c


def _check_grouped_multihead(gpu, O, heads, V, C, B, seed, min_groups):
    """Values, flows, statistics and updated parameters of a multi-head circuit whose dense groups run on the block
    kernels, against the oracle and against the same circuit on the layer kernels alone."""
    torch, P = gpu
    from helpers import rel_err
    import pcmi355._lib as L
    rng = np.random.default_rng(seed)
    H = len(heads)
    grouped, plain = _with_and_without_groups(P, heads, V, C)
    assert grouped.size("dense_groups") >= min_groups
    assert grouped.size("layer_nodes") < grouped.num_nodes() or grouped.size("dense_groups") == 0
    fc = O.bits_compile(O.summate(*heads), C, V)
    n_real = fc.n_nodes - 1
    assert grouped.num_nodes() == n_real
    start = P.vectorize_parameters(grouped)
    assert np.array_equal(start, P.vectorize_parameters(plain))
    root_ids = (grouped.table("heads") - 1).astype(np.int32)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    mask = rng.random((B, H)).astype(np.float32) + 0.05
    mask[::5, 0] = 0.0
    d, hm = torch.from_numpy(data).cuda(), torch.from_numpy(mask).cuda()
    mars_ref = O.forward(fc, data)
    skip = (fc.edge_parent() == fc.n_nodes - 1).astype(np.uint8)
    flows_ref, ea_ref = O.backward(fc, mars_ref, skip=skip, root_ids=root_ids, root_flow=np.ascontiguousarray(mask.T))
    lf_ref = O.input_flows(fc, data, flows_ref)
    order = fc.up_order()
    order = order[fc.edge_parent()[order] != fc.n_nodes - 1]
    got = []
    layered = _without_group_walks(P, heads, V, C)
    assert layered.size("dense_groups") == grouped.size("dense_groups")
    for bpc in (grouped, plain, layered):
        per_head = P.loglikelihoods(bpc, d).cpu().numpy()
        assert rel_err(per_head, mars_ref[root_ids].T).max() < LL_RTOL
        ll = P.probs_flows_circuit(bpc, d, head_mask=hm).cpu().numpy()
        mars, flows = bpc.get_node_values(B)
        finite = np.isfinite(mars_ref[:n_real])
        assert np.array_equal(np.isfinite(mars), finite)
        assert np.abs(mars[finite] - mars_ref[:n_real][finite]).max() < LL_RTOL * np.abs(mars_ref[:n_real][finite]).max()
        assert np.abs(flows - flows_ref[:n_real]).max() < FLOW_RTOL * max(flows_ref.max(), 1.0)   # (an example's flow: the sum of its mask)
        ea, lf = bpc.get_aggregates()
        assert np.abs(ea - ea_ref[order]).max() < FLOW_RTOL * ea_ref.max()
        assert np.abs(lf - lf_ref).max() < FLOW_RTOL * lf_ref.max()
        L.check(L.lib.pcm_em_update(bpc.handle, 0.1, 0.7))
        got.append((ll, mars, flows, ea, lf, P.vectorize_parameters(bpc)))
    for a, b, c in zip(*got):                                # the two paths round differently, no more
        fa, fb = np.isfinite(a), np.isfinite(b)
        assert np.array_equal(fa, fb)
        assert np.abs(a[fa] - b[fb]).max() <= 2e-4 * max(np.abs(b[fb]).max(), 1.0)
        assert np.array_equal(a.view(np.uint32), c.view(np.uint32))   # a walk and a launch per layer: the same arithmetic
    # a smaller batch afterwards finds the arrays of the larger one (rows of 64 examples, the last one partly filled)
    small = d[: B // 3]
    for bpc in (grouped, plain):
        P.update_parameters(bpc, start)
    a, b = (P.loglikelihoods(bpc, small).cpu().numpy() for bpc in (grouped, plain))
    assert rel_err(a, mars_ref[root_ids][:, : B // 3].T).max() < LL_RTOL and rel_err(a, b).max() < LL_RTOL
    return grouped, fc


@pytest.mark.parametrize("V,K,C,H,B,max_children,seed", [(20, 8, 5, 9, 150, 5, 31), (9, 32, 4, 40, 64, 2, 32),
                                                         (33, 12, 3, 6, 333, 3, 33), (40, 16, 4, 7, 100, 3, 34),
                                                         (12, 64, 3, 5, 50, 2, 35),
                                                         (130, 32, 4, 6, 101, 3, 36)])   # 4160 input nodes: a wave per node
def test_dense_groups_of_a_multihead_hclt(gpu, oracle, V, K, C, H, B, max_children, seed):
    """An HCLT's K sums per tree node and the heads over the root's products are groups; products of up to three
    children are taken apart by the groups above them, those of more stay nodes of a layer."""
    from helpers import multihead_hclt
    rng = np.random.default_rng(seed)
    parent = np.full(V, -1, np.int32)
    n_children = np.zeros(V, int)
    for v in range(1, V):
        free = [u for u in range(v) if n_children[u] < max_children]
        parent[v] = free[int(rng.integers(0, len(free)))] if v > max_children + 1 else 0   # the root takes max_children + 1
        n_children[parent[v]] += 1
    heads, _ = multihead_hclt(parent, K, C, H, rng)
    inner = len(set(parent[1:].tolist()))                    # (the K sums of an inner tree node; the root's are the heads)
    grouped, _ = _check_grouped_multihead(gpu, oracle, heads, V, C, B, seed, min_groups=inner)
    assert grouped.size("dense_groups") == inner
    if max_children <= 3 and K in (16, 32, 64):
        # every level of the tree below the root's is a layer of K x K groups and nothing else: one walk launch
        assert grouped.size("walk_levels") >= 2
    if max_children <= 3:
        # nothing but the inputs and the product of the root's children is left to the layer kernels going up
        assert grouped.size("layer_nodes") == grouped.size("input_nodes") + K


def test_dense_groups_after_pruning_and_growing(gpu, oracle):
    """prune_pc takes edges out of some of a group's sums (their lists of children differ from then on) and
    grow_heads_by_flows doubles sums and products: what is left of the groups, and the new ones, still compute what
    the oracle does."""
    torch, P = gpu
    from helpers import multihead_hclt, from_oracle_dag, to_oracle_dag
    rng = np.random.default_rng(41)
    V, K, C, H, B = 8, 12, 4, 8, 200
    parent = np.array([-1, 0, 0, 1, 1, 2, 5, 5], np.int32)
    heads, _ = multihead_hclt(parent, K, C, H, rng)
    pcs, _ = from_oracle_dag(heads)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    mask = rng.dirichlet(np.ones(H), size=B).astype(np.float32)
    d, hm = torch.from_numpy(data).cuda(), torch.from_numpy(mask).cuda()
    for threshold in (1e-4, 3e-4, 1e-3, 3e-3):               # the first that takes some edges, and not too many
        pruned = P.prune_pc(pcs, d, hm, batch_size=100, prune_threshold=threshold)
        if P.nodes.num_edges(pruned) < P.nodes.num_edges(pcs):
            break
    assert P.nodes.num_edges(pruned) < P.nodes.num_edges(pcs)
    po, _ = to_oracle_dag(pruned)
    _check_grouped_multihead(gpu, oracle, po, V, C, 90, 42, min_groups=1)
    grown = P.grow_heads_by_flows(pcs, d, hm, batch_size=100, sigma=0.1, node_selection_args={"grow_frac": 0.5},
                                  rng=np.random.default_rng(3))
    go, _ = to_oracle_dag(grown)
    assert len(go) > H
    # (a split sum and its copy share their products, which then are nodes; an unsplit sum's are folded into its
    # edges: the sums of one tree node fall into several sets of children, of which those with four sums are groups)
    _check_grouped_multihead(gpu, oracle, go, V, C, 90, 43, min_groups=1)


def test_dense_groups_beside_ordinary_edges(gpu, oracle):
    """A group whose children other sums use too (their rows of flow are added to what those sums send), beside a
    group whose products nothing else uses (taken apart, written by the group), under one root."""
    O = oracle
    from helpers import log_dirichlet
    rng = np.random.default_rng(51)
    C, G, J = 5, 6, 12
    leaf = lambda v: O.input_node(v, log_dirichlet(rng, C))
    p = [O.multiply(leaf(0), leaf(1)) for _ in range(J)]
    q = [O.multiply(leaf(2), leaf(3)) for _ in range(J)]
    s = [O.summate(*p, logps=log_dirichlet(rng, J)) for _ in range(G)]
    t = O.summate(*p[:3], logps=log_dirichlet(rng, 3))
    t2 = O.summate(*p[2:9], logps=log_dirichlet(rng, 7))
    u = [O.summate(*q, logps=log_dirichlet(rng, J)) for _ in range(G)]
    tops = [O.multiply(s[i], u[i]) for i in range(G)] + [O.multiply(t, u[0]), O.multiply(t2, u[3])]
    heads = [O.summate(*tops, logps=log_dirichlet(rng, len(tops))) for _ in range(2)]
    grouped, _ = _check_grouped_multihead(gpu, oracle, heads, 4, C, 130, 52, min_groups=2)
    assert grouped.size("dense_groups") == 2


@pytest.mark.parametrize("fscale", [0.5, 2.5])
def test_tempered_flows_match_the_oracle(gpu, oracle, fscale):
    """`fscale` of mini_batch_em_beta (src-jl/learning/flow.jl:120-373, `pcm_set_flow_scale`): node flows, edge and leaf
    statistics of the tempered pass on a random DAG (layer kernels), on a multi-head HCLT whose sums run as dense
    groups (and the same circuit without them), and on an HCLT handle of the block engine, which hands such passes to
    its layered form; likelihoods are not touched and fscale = 1 afterwards is the ordinary pass again."""
    torch, P = gpu
    O = oracle
    import pcmi355._lib as L
    from helpers import random_dag, multihead_hclt, make_hclt, block_theta, correlated_data, rel_err
    rng = np.random.default_rng(61)
    # (1) a single-root DAG
    V, C, B = 6, 4, 90
    root = random_dag(V, C, rng, width=3)
    fc = O.bits_compile(root, C, V)
    bpc = _compile(P, [root], V, C)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    d = torch.from_numpy(data).cuda()
    order = fc.up_order()
    mars_ref = O.forward(fc, data)
    plain_ll = P.probs_flows_circuit(bpc, d).cpu().numpy()
    plain_ea, _ = bpc.get_aggregates()
    bpc.set_flow_scale(fscale)
    ll = P.probs_flows_circuit(bpc, d).cpu().numpy()
    assert np.array_equal(ll, plain_ll)
    flows_ref, ea_ref = O.backward(fc, mars_ref, fscale=fscale)
    lf_ref = O.input_flows(fc, data, flows_ref)
    _, flows = bpc.get_node_values(B)
    ea, lf = bpc.get_aggregates()
    assert np.abs(flows - flows_ref).max() < FLOW_RTOL
    assert np.abs(ea - ea_ref[order]).max() < FLOW_RTOL * ea_ref.max()
    assert np.abs(lf - lf_ref).max() < FLOW_RTOL * lf_ref.max()
    assert np.abs(ea - plain_ea).max() > 1e-2 * ea_ref.max()           # (and it is not the ordinary pass)
    with pytest.raises(L.PcmError):
        bpc.set_flow_scale(0.0)
    bpc.set_flow_scale(1.0)
    P.probs_flows_circuit(bpc, d)
    assert np.array_equal(bpc.get_aggregates()[0], plain_ea)

    # (2) dense groups, heads, a soft head mask
    V, K, C, H, B = 12, 8, 5, 9, 150
    parent = np.array([-1] + [int(rng.integers(max(0, v - 3), v)) for v in range(1, V)], np.int32)
    heads, _ = multihead_hclt(parent, K, C, H, rng)
    grouped, plain = _with_and_without_groups(P, heads, V, C)
    assert grouped.size("dense_groups") > 0
    fc = O.bits_compile(O.summate(*heads), C, V)
    n_real = fc.n_nodes - 1
    root_ids = (grouped.table("heads") - 1).astype(np.int32)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    mask = rng.random((B, H)).astype(np.float32) + 0.05
    d, hm = torch.from_numpy(data).cuda(), torch.from_numpy(mask).cuda()
    mars_ref = O.forward(fc, data)
    skip = (fc.edge_parent() == fc.n_nodes - 1).astype(np.uint8)
    flows_ref, ea_ref = O.backward(fc, mars_ref, skip=skip, root_ids=root_ids, root_flow=np.ascontiguousarray(mask.T),
                                   fscale=fscale)
    lf_ref = O.input_flows(fc, data, flows_ref)
    order = fc.up_order()
    order = order[fc.edge_parent()[order] != fc.n_nodes - 1]
    for c in (grouped, plain):
        c.set_flow_scale(fscale)
        P.probs_flows_circuit(c, d, head_mask=hm)
        _, flows = c.get_node_values(B)
        ea, lf = c.get_aggregates()
        assert np.abs(flows - flows_ref[:n_real]).max() < FLOW_RTOL
        assert np.abs(ea - ea_ref[order]).max() < FLOW_RTOL * ea_ref.max()
        assert np.abs(lf - lf_ref).max() < FLOW_RTOL * lf_ref.max()

    # (3) an HCLT handle of the block engine: EM step with tempered flows, then an ordinary one
    V, K, C, B = 11, 16, 7, 200
    parent, theta, leaf, fc = make_hclt(V, K, C, 62)
    data = correlated_data(B, V, C, 63, parent)
    d = torch.from_numpy(data).cuda()
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    cur = fc
    for f in (fscale, 1.0):
        bpc.set_flow_scale(f)
        ll = torch.empty(B, device="cuda")
        L.check(L.lib.pcm_em_step(bpc.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, 0.1, 0.8, ll.data_ptr()))
        mars = O.forward(cur, data, double=True)
        assert rel_err(ll.cpu().numpy(), mars[-1]).max() < LL_RTOL
        flows, ea = O.backward(cur, mars, double=True, fscale=f)
        lf = O.input_flows(cur, data, flows, double=True)
        logp, new_leaf = O.em_update(cur, ea, lf, 0.1, 0.8, True)
        cur = cur.copy()
        cur.logp, cur.leaf_logp = logp.astype(np.float32), new_leaf.astype(np.float32)
        th_ref, leaf_ref = O.hclt_block_params(cur)
        th, lf_new = bpc.get_params()
        for v, blk in th_ref.items():
            assert rel_err(np.exp(th[v][:blk.shape[0]]), np.exp(blk)).max() < 5e-4
        assert rel_err(np.exp(lf_new), np.exp(leaf_ref)).max() < 5e-4
    forest = P.hclt_forest_from_clts(np.array([-1, 0, -1, 2], np.int32), 4, 16, 2)
    with pytest.raises(L.PcmError):               # (a forest has no layered form)
        forest.set_flow_scale(2.0)


def test_forest_of_patch_circuits_at_their_real_shape(gpu, oracle):
    """Sixteen patch circuits of the patch-clustered configuration (8 x 8 x 3 patches of 64 x 64 x 3 images: 192
    variables, K = 32, 256 categories, 128 heads, batch 1024) as one forest handle over the image's pixels, against a
    handle per patch (the path the test above pins to the layered engine and the oracle): per-head values, mixtures,
    flows and the EM update under a one-hot and a soft head mask.  Some of the sixteen Chow-Liu trees have nodes with
    four children, which the forest splits; two groups of trees walk side by side."""
    torch, P = gpu
    from pcmi355 import workloads
    from pcmi355._lib import lib, check
    from helpers import rel_err
    V, K, C, H, B, NP = 192, 32, 256, 128, 1024, 16
    rng = np.random.default_rng(1004)
    img = workloads.grf_images(B, 64, 64, 3, 3.0, 0.8, seed=1004).reshape(B, 3, 64, 64)
    flat = np.ascontiguousarray(img.reshape(B, -1))
    pixel = np.arange(3 * 64 * 64).reshape(3, 64, 64)
    pvars = [pixel[:, 8 * (p // 8):8 * (p // 8) + 8, 8 * (p % 8):8 * (p % 8) + 8].reshape(V) for p in range(NP)]
    used = np.sort(np.concatenate(pvars))                       # the forest's variables: the pixels of these patches
    col = np.full(flat.shape[1], -1, np.int64)
    col[used] = np.arange(len(used))
    parents = [workloads.chow_liu_parent(np.ascontiguousarray(flat[:, pv])) for pv in pvars]
    assert max(np.bincount(par[par >= 0]).max() for par in parents) > 3
    fparent = np.empty(len(used), np.int32)
    theta = np.empty((len(used), K, K), np.float32)
    leaf = np.empty((len(used), K, C), np.float32)
    heads = np.log(rng.dirichlet(np.ones(K), size=(NP, H))).astype(np.float32)
    singles = []
    for p, (pv, par) in enumerate(zip(pvars, parents)):
        th, lf = workloads.init_params(par, K, C, 2000 + p, kind="dirichlet")
        fparent[col[pv]] = np.where(par < 0, -1, col[pv][np.maximum(par, 0)])
        theta[col[pv]], leaf[col[pv]] = th, lf
        c = P.multihead_hclt_from_clt(par, C, K, H)
        c.set_params(th, lf)
        singles.append((c, torch.from_numpy(np.ascontiguousarray(flat[:, pv])).cuda()))
    order = np.argsort([col[pv][np.flatnonzero(par < 0)[0]] for pv, par in zip(pvars, parents)])   # tree t = patch order[t]
    forest = P.hclt_forest_from_clts(fparent, C, K, H)
    assert forest.num_trees == NP and forest.size("walk_kernels") == 1 and forest.size("variables") == len(used)
    forest.set_params(theta, leaf)
    forest.set_heads(heads[order])
    for p, (c, _) in enumerate(singles):
        c.set_heads(heads[p])
    d = torch.from_numpy(np.ascontiguousarray(flat[:, used])).cuda()
    ll_f = P.forest_loglikelihoods(forest, d).cpu().numpy()
    for t, p in enumerate(order):
        c, dp = singles[p]
        assert rel_err(ll_f[t].T, P.loglikelihoods(c, dp).cpu().numpy()).max() < 1e-5, f"patch {p}"
    cluster = rng.integers(0, H, size=(NP, B))
    for soft in (False, True):
        mask = np.zeros((NP, H, B), np.float32)
        for p in range(NP):
            mask[p, cluster[p], np.arange(B)] = 1.0
        if soft:
            mask = (mask + rng.random(mask.shape).astype(np.float32) * (rng.random(mask.shape) < 0.1)).astype(np.float32)
        mix_f = P.forest_flows(forest, d, torch.from_numpy(mask[order]).cuda()).cpu().numpy()
        ea_f, lf_f = forest.get_flows()
        check(lib.pcm_em_update(forest.handle, 0.1, 0.9))
        th_f, leaf_f = forest.get_params()
        heads_f = forest.get_heads()
        worst = 0.0
        for t, p in enumerate(order):
            c, dp = singles[p]
            mix = P.probs_flows_circuit(c, dp, head_mask=torch.from_numpy(mask[p].T.copy()).cuda()).cpu().numpy()
            assert rel_err(mix_f[t], mix).max() < 1e-5, f"patch {p} mixture"
            ea, lf = c.get_flows()
            gv = col[pvars[p]]
            assert np.abs(ea_f[gv] - ea).max() < FLOW_RTOL * ea.max() and np.abs(lf_f[gv] - lf).max() < FLOW_RTOL * lf.max()
            check(lib.pcm_em_update(c.handle, 0.1, 0.9))
            th, lp = c.get_params()
            inner = np.flatnonzero(np.bincount(parents[p][parents[p] >= 0], minlength=V) > 0)
            inner = inner[parents[p][inner] >= 0]                # (the root's block is the identity in both)
            for a, b in ((th_f[gv][inner], th[inner]), (leaf_f[gv], lp), (heads_f[t], c.get_heads())):
                worst = max(worst, float((np.abs(np.exp(a.astype(np.float64)) - np.exp(b.astype(np.float64)))
                                          / np.maximum(np.exp(b.astype(np.float64)), 1e-6)).max()))
        print(f"forest vs one handle per patch, {'soft' if soft else 'one-hot'} mask: parameters differ by {worst:.2e}")
        assert worst < 2e-4
