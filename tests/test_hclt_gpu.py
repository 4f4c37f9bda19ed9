"""GPU parity of the dense-block HCLT engine against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

LL_RTOL = 1e-4      # relative, per-example log-likelihoods (fp32)
PARAM_RTOL = 1e-4   # relative, updated parameters compared as probabilities
FLOW_RTOL = 2e-4    # relative to the largest entry of the block, aggregated flows


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355
    return torch, pcmi355


def _compare_step(gpu, oracle, V, K, C, B, seed, idx=None, N=None, tree=None):
    torch, P = gpu
    from helpers import make_hclt, correlated_data, oracle_em_reference, block_theta, rel_err
    parent, theta, leaf, fc = make_hclt(V, K, C, seed, parent=None if tree is None else np.array(tree, np.int32))
    N = N or B
    data = correlated_data(N, V, C, seed + 1, parent)
    ids = np.arange(B, dtype=np.int32) if idx is None else idx
    # statistics and updated parameters against the float64 oracle: the exact result of the reference's
    # formulas (its own float32 arithmetic, the float32 oracle, loses up to 1e-4 on trees a few hundred
    # variables deep; test_deep_trees_three_way); log-likelihoods against both
    ll_ref, th_ref, leaf_ref, ea_ref, lf_ref = oracle_em_reference(fc, data, ids, 0.1, 0.9, double=True)
    ll32 = oracle.forward(fc, data, ids)[-1]

    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    d = torch.from_numpy(data).cuda()
    ll = P.loglikelihoods(bpc, d, example_ids=None if idx is None else idx)
    ll = ll.cpu().numpy()
    assert rel_err(ll, ll_ref).max() < LL_RTOL and rel_err(ll, ll32).max() < LL_RTOL

    ll2 = P.probs_flows_circuit(bpc, d, example_ids=None if idx is None else idx).cpu().numpy()
    assert np.array_equal(ll, ll2)
    ea, lf = bpc.get_flows()
    for v, blk in ea_ref.items():
        nk = blk.shape[0]
        assert np.abs(ea[v][:nk] - blk).max() < FLOW_RTOL * max(blk.max(), 1e-3), f"edge_aggr block {v}"
        # invariant: flows into the K sum nodes sum to the batch size (root: row 0 only)
    assert np.abs(lf - lf_ref).max() < FLOW_RTOL * max(lf_ref.max(), 1e-3)
    np.testing.assert_allclose(lf.sum(axis=(1, 2)), B, rtol=1e-4)   # every example passes every variable once

    import pcmi355._lib as L
    L.check(L.lib.pcm_em_update(bpc.handle, 0.1, 0.9))
    th, lf_new = bpc.get_params()
    for v, blk in th_ref.items():
        nk = blk.shape[0]
        assert rel_err(np.exp(th[v][:nk]), np.exp(blk)).max() < PARAM_RTOL, f"theta block {v}"
    assert rel_err(np.exp(lf_new), np.exp(leaf_ref)).max() < PARAM_RTOL
    return bpc


@pytest.mark.parametrize("V,K,C,B", [(2, 16, 5, 16), (7, 16, 8, 48), (12, 32, 256, 64), (9, 64, 17, 32),
                                     (2, 128, 5, 16), (10, 128, 256, 70)])
def test_em_step_matches_oracle(gpu, oracle, V, K, C, B):
    _compare_step(gpu, oracle, V, K, C, B, seed=100 + V)


@pytest.mark.parametrize("tree", [[-1, 0, 0, 0, 0, 0, 0],                      # star: six leaf children
                                  [-1, 0, 0, 0, 0, 0, 1, 2, 3, 4, 5],        # five inner children
                                  [-1, 0, 1, 1, 1, 1, 2, 3, 0, 8, 8, 8, 8]])  # mixed, four children twice
def test_em_step_on_wide_trees(gpu, oracle, tree):
    """Nodes with more than three children take the general walk kernels (operands beyond the
    inline ones, schedule items read from memory)."""
    _compare_step(gpu, oracle, len(tree), 16, 7, 40, seed=len(tree), tree=tree)
    _compare_step(gpu, oracle, len(tree), 32, 12, 33, seed=len(tree) + 1, tree=tree)
    _compare_step(gpu, oracle, len(tree), 128, 9, 21, seed=len(tree) + 2, tree=tree)   # the wide block kernels


def test_every_walk_kernel_family_is_exercised(gpu, oracle):
    """Which kernels a circuit gets: lean walks (K <= 32; a node with more than three children is split for them),
    general walks (K = 64 on bushy trees), wide block kernels (K = 128; K = 64 on small trees), per-layer kernels
    (other hidden sizes) -- and the bushy K = 64 case against the oracle."""
    torch, P = gpu
    rng = np.random.default_rng(1)
    kind = lambda parent, K: P.hclt_from_clt(np.asarray(parent, np.int32), 4, K).size("walk_kernels")
    chain = [-1] + list(range(9))
    assert kind(chain, 32) == 1 and kind([-1, 0, 0, 0, 0, 0], 16) == 1 and kind(chain, 128) == 3 and kind(chain, 8) == 0
    assert kind(chain, 64) == 3 and kind([-1, 0, 0, 0, 0, 0], 64) == 3
    star = P.hclt_from_clt(np.array([-1, 0, 0, 0, 0, 0], np.int32), 4, 16)       # what the caller sees is the caller's tree
    assert star.size("variables") == 6 and star.size("inner_tree_nodes") == 1 and star.size("input_nodes") == 6 * 16
    bushy = oracle.random_tree(600, rng, 3)
    assert kind(bushy, 64) == 2
    bpc = _compare_step(gpu, oracle, 600, 64, 4, 16, seed=5, tree=list(bushy))
    assert bpc.size("walk_kernels") == 2


def test_ragged_batch_and_example_ids(gpu, oracle):
    rng = np.random.default_rng(5)
    idx = rng.permutation(200)[:37].astype(np.int32)
    _compare_step(gpu, oracle, 10, 32, 11, 37, seed=7, idx=idx, N=200)


@pytest.mark.parametrize("K", [16, 32])
def test_batches_larger_than_the_device_go_through_in_chunks(gpu, oracle, K):
    """More examples than one 16-example workgroup per compute unit (4096 on 256 units): likelihoods, flows and the
    EM update of the whole batch, contiguous and through example ids, with flow memory on the second call."""
    torch, P = gpu
    import pcmi355._lib as L
    _compare_step(gpu, oracle, 6, K, 5, 9000, seed=21)
    rng = np.random.default_rng(3)
    idx = rng.permutation(12000)[:8200].astype(np.int32)
    bpc = _compare_step(gpu, oracle, 5, K, 7, 8200, seed=22, idx=idx, N=12000)
    # flow memory: a second, smaller batch on top of 0.5 x the first equals the two halves of it added by hand
    from helpers import correlated_data
    data = torch.from_numpy(correlated_data(12000, 5, 7, 23, bpc.clt_parent)).cuda()
    P.probs_flows_circuit(bpc, data[:8200].contiguous())
    ea1, lf1 = bpc.get_flows()
    P.probs_flows_circuit(bpc, data[8200:].contiguous(), rate=0.5)
    ea2, lf2 = bpc.get_flows()
    P.probs_flows_circuit(bpc, data[8200:].contiguous())
    ea3, lf3 = bpc.get_flows()
    np.testing.assert_allclose(lf2, 0.5 * lf1 + lf3, rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(ea2, 0.5 * ea1 + ea3, rtol=1e-5, atol=1e-4)


def test_degenerate_inputs(gpu, oracle):
    """No examples, one example, the smallest tree; a tree of one variable has no sum node and is refused."""
    torch, P = gpu
    c = P.hclt_from_clt(np.array([-1, 0], np.int32), 5, 16)
    empty = P.loglikelihoods(c, torch.zeros((0, 2), dtype=torch.uint8, device="cuda"))
    assert tuple(empty.shape) == (0,)
    one = P.loglikelihoods(c, torch.tensor([[1, 2]], dtype=torch.uint8, device="cuda")).cpu().numpy()
    np.testing.assert_allclose(one, [np.log(1 / 25)], rtol=1e-6)          # uniform parameters
    lls = P.mini_batch_em_with_reg(c, torch.tensor([[1, 2]], dtype=torch.uint8, device="cuda"), 2, batch_size=1,
                                   pseudocount=0.1, param_inertia=0.5, shuffle="none")
    assert lls[1] > lls[0]
    with pytest.raises(P.PcmError):
        P.hclt_from_clt(np.array([-1], np.int32), 5, 16)
    with pytest.raises(ValueError):
        P.mini_batch_em_with_reg(c, torch.zeros((3, 2), dtype=torch.uint8, device="cuda"), 1, batch_size=4, pseudocount=0.1,
                                 param_inertia=0.5)


def test_a_freed_handle_is_refused(gpu):
    """The C ABI keeps a table of live handles: a second free, or any call on a freed handle, comes
    back as an argument error instead of touching freed memory."""
    import ctypes
    torch, P = gpu
    from pcmi355._lib import lib
    par = (ctypes.c_int32 * 3)(-1, 0, 0)
    h = ctypes.c_void_p()
    assert lib.pcm_hclt_create(par, 3, 16, 8, ctypes.byref(h)) == 0
    assert lib.pcm_size(h, 0) > 0
    assert lib.pcm_free(h) == 0
    assert lib.pcm_free(h) == -1
    assert lib.pcm_size(h, 0) < 0
    assert lib.pcm_em_update(h, ctypes.c_float(0.1), ctypes.c_float(0.9)) == -1


@pytest.mark.parametrize("K", [16, 32, 64, 128, 8])
def test_examples_of_probability_zero_carry_no_flow(gpu, oracle, K):
    """A leaf that forbids a category makes the examples showing it impossible: their value is
    -inf and they leave no trace in the statistics (the reference's flows turn NaN there:
    exp(-inf - -inf) in src/queries/flow.jl:49-60); every walk engine behaves the same."""
    torch, P = gpu
    from helpers import make_hclt, block_theta
    V, C, B = 5, 4, 40
    parent, theta, leaf, fc = make_hclt(V, K, C, 3)
    leaf = leaf.copy()
    leaf[2, :, 1] = -np.inf
    leaf[2] -= np.log(np.exp(leaf[2].astype(np.float64)).sum(-1, keepdims=True)).astype(np.float32)
    data = np.random.default_rng(K).integers(0, C, (B, V)).astype(np.uint8)
    bad = data[:, 2] == 1
    assert bad.any() and not bad.all()
    a, b = P.hclt_from_clt(parent, C, K), P.hclt_from_clt(parent, C, K)
    for c in (a, b):
        c.set_params(block_theta(parent, K, theta), leaf)
    ll = P.probs_flows_circuit(a, torch.from_numpy(data).cuda()).cpu().numpy()
    ll_good = P.probs_flows_circuit(b, torch.from_numpy(np.ascontiguousarray(data[~bad])).cuda()).cpu().numpy()
    assert np.isneginf(ll[bad]).all()
    np.testing.assert_allclose(ll[~bad], ll_good, rtol=1e-6)
    (ea, lf), (ea2, lf2) = a.get_flows(), b.get_flows()
    assert np.isfinite(ea).all() and np.isfinite(lf).all()
    np.testing.assert_allclose(ea, ea2, atol=2e-4 * ea2.max())
    np.testing.assert_allclose(lf, lf2, atol=2e-4 * lf2.max())


def test_config1_shape(gpu, oracle):
    """64 variables, K=16, 256 categories, batch 1024 (the reference's CPU-runnable case)."""
    _compare_step(gpu, oracle, 64, 16, 256, 1024, seed=11)


@pytest.mark.parametrize("K", [32, 128])
def test_kernel_timing_does_not_change_results(gpu, oracle, K):
    """pcm_set_timing / pcm_get_timing: the three phases report a positive time each, the flows of a timed call are
    the bits of an untimed one, and a second read without a call in between reports nothing."""
    torch, P = gpu
    from helpers import make_hclt, correlated_data, block_theta
    parent, theta, leaf, _ = make_hclt(20, K, 16, 5)
    data = torch.from_numpy(correlated_data(200, 20, 16, 6, parent)).cuda()
    bpc = P.hclt_from_clt(parent, 16, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    ll0 = P.probs_flows_circuit(bpc, data).cpu().numpy()
    ea0, lf0 = bpc.get_flows()
    bpc.set_timing(True)
    for _ in range(3):
        ll1 = P.probs_flows_circuit(bpc, data).cpu().numpy()
    ms = bpc.get_timing()
    assert all(0.0 < ms[k] < 50.0 for k in ("forward", "backward", "statistics")), ms
    ea1, lf1 = bpc.get_flows()
    assert np.array_equal(ll0, ll1) and np.array_equal(lf0, lf1) and np.array_equal(ea0, ea1)
    assert all(v == 0.0 for v in bpc.get_timing().values())
    bpc.set_timing(8)   # the statistics kernel only
    P.probs_flows_circuit(bpc, data)
    ms = bpc.get_timing()
    assert ms["forward"] == 0.0 and ms["backward"] == 0.0 and 0.0 < ms["statistics"] < 50.0, ms
    bpc.set_timing(False)


@pytest.mark.parametrize("tree", [None, [-1, 0, 0], [-1, 0, 1, 1], [-1, 0, 0, 0, 0], [1, -1, 1, 2, 2, 0, 0, 3],
                                  [-1, 0, 0, 2, 2, 2, 4, 1, 6, 3, 9]])
def test_param_vector_roundtrip(gpu, oracle, tree):
    """Parameter vector and index tables follow the numbering of the flattened DAG, on
    trees whose nodes have one, two, three and four children."""
    torch, P = gpu
    from helpers import make_hclt, block_theta
    V = 9 if tree is None else len(tree)
    parent, theta, leaf, fc = make_hclt(V, 16, 6, 3, parent=None if tree is None else np.array(tree, np.int32))
    bpc = P.hclt_from_clt(parent, 6, 16)
    bpc.set_params(block_theta(parent, 16, theta), leaf)
    dag = oracle.bits_compile(oracle.hclt_dag(parent, 16, 6, theta, leaf), 6, V)
    ref = dag.vectorize_parameters()
    got = P.vectorize_parameters(bpc)
    assert got.shape == ref.shape
    np.testing.assert_array_equal(got, ref)
    P.update_parameters(bpc, got[::-1].copy() * 0 + got)   # write back the same vector
    np.testing.assert_array_equal(P.vectorize_parameters(bpc), ref)
    t = dag.param_tables()
    assert bpc.num_nodes() == dag.n_nodes and bpc.num_edges() == dag.n_edges
    np.testing.assert_array_equal(bpc.table("edge2param"), t["edge2param"])
    np.testing.assert_array_equal(bpc.table("param2edge"), t["param2edge"])
    np.testing.assert_array_equal(bpc.table("param2group"), t["param2group"])
    np.testing.assert_array_equal(bpc.table("pargroup_sizes"), t["pargroup_sizes"])
    order = dag.up_order()
    np.testing.assert_array_equal(bpc.table("edge_parent") - 1, dag.edge_parent()[order])
    np.testing.assert_array_equal(bpc.table("edge_prime") - 1, dag.prime[order])
    np.testing.assert_array_equal(bpc.table("edge_sub") - 1, dag.sub[order])


def test_ten_em_steps_track_oracle(gpu, oracle):
    """Ten mini-batch EM steps (step size 0.1 == inertia 0.9, pseudocount 0.1) stay on the
    oracle's trajectory."""
    torch, P = gpu
    from helpers import make_hclt, correlated_data, block_theta, rel_err
    V, K, C, B = 12, 16, 32, 256
    parent, theta, leaf, fc = make_hclt(V, K, C, 21)
    data = correlated_data(B, V, C, 22, parent)
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    d = torch.from_numpy(data).cuda()
    import pcmi355._lib as L
    ll = torch.empty(B, device="cuda")
    cur = fc
    for step in range(10):
        ll_ref, logp, lf, _, _ = oracle.em_step(cur, data, np.arange(B, dtype=np.int32), 0.1, 0.9)
        cur = cur.copy()
        cur.logp, cur.leaf_logp = logp, lf
        L.check(L.lib.pcm_em_step(bpc.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, 0.1, 0.9,
                                  ll.data_ptr()))
        assert rel_err(ll.cpu().numpy(), ll_ref).max() < LL_RTOL, step
    th_ref, leaf_ref = oracle.hclt_block_params(cur)
    th, lf_new = bpc.get_params()
    for v, blk in th_ref.items():
        assert rel_err(np.exp(th[v][:blk.shape[0]]), np.exp(blk)).max() < 5e-4
    assert rel_err(np.exp(lf_new), np.exp(leaf_ref)).max() < 5e-4


@pytest.mark.parametrize("V,K,C,B", [(6, 8, 5, 40), (5, 128, 7, 33), (9, 3, 4, 70)])
def test_hidden_sizes_without_block_kernels(gpu, oracle, V, K, C, B):
    """Hidden sizes without walk kernels: 128 has the wide block kernels for likelihoods, flows
    and EM and the layered engine for the other queries, the rest run entirely on the layered
    engine, all behind the same HCLT interface (block-form parameters and flows, EM step, KL,
    sampling)."""
    torch, P = gpu
    bpc = _compare_step(gpu, oracle, V, K, C, B, seed=7 * K + V)
    assert bpc.size("hidden_categories") == K
    theta, leaf = bpc.get_params()
    q = P.hclt_from_clt(bpc.clt_parent, C, K)          # uniform parameters
    assert P.kld(bpc, bpc) < 1e-5 and P.kld(bpc, q) > 0
    n_inner = bpc.size("inner_tree_nodes")
    g = torch.Generator(device="cuda").manual_seed(K)
    u1 = torch.rand((16, n_inner * K), device="cuda", generator=g).clamp_(1e-9, 1 - 1e-7)
    u2 = torch.rand((16, V, C), device="cuda", generator=g).clamp_(1e-9, 1 - 1e-7)
    s = P.sample(bpc, -torch.log(-torch.log(u1)), -torch.log(-torch.log(u2))).cpu().numpy()
    assert s.shape == (16, V) and (s < C).all()


def test_config_hclt48_k128(gpu, oracle):
    """Benchmark configuration with K = 128 (48 variables = one 4x4x3 patch, 256 categories,
    Dirichlet(1) parameters, batch 4096): ten mini-batch EM steps with step size 0.1 and
    pseudocount 0.1; the first step is checked against the oracle on a subset, the run for a
    rising likelihood."""
    torch, P = gpu
    O = oracle
    from pcmi355 import workloads
    from helpers import rel_err
    V, K, C, B = 48, 128, 256, 4096
    data = workloads.grf_images(B, 4, 4, 3, 2.0, 0.8, seed=1002)
    parent = workloads.chow_liu_parent(data)
    theta, leaf = workloads.init_params(parent, K, C, 1102, kind="dirichlet")
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(theta, leaf)
    d = torch.from_numpy(data).cuda()
    sub = 48
    ch, _ = O.clt_children(parent)
    fc = O.hclt_flat(parent, K, C, {v: theta[v] for v in range(V) if ch[v]}, leaf)
    ll_ref = O.forward(fc, data[:sub])[-1]
    ll = P.loglikelihoods(bpc, d).cpu().numpy()
    assert rel_err(ll[:sub], ll_ref).max() < LL_RTOL
    lls = P.mini_batch_em_with_reg(bpc, d, 10, batch_size=B, pseudocount=0.1, param_inertia=0.9, shuffle="none")
    assert all(b > a for a, b in zip(lls, lls[1:])), lls
    np.testing.assert_allclose(lls[0], ll.mean(), rtol=1e-5)


@pytest.mark.parametrize("V,K,C,H,B,tree", [(7, 16, 5, 3, 40, None), (12, 32, 9, 128, 70, None), (2, 16, 4, 16, 16, [-1, 0]),
                                            (9, 32, 256, 40, 33, [-1, 0, 0, 1, 1, 2, 2, 3, 3]),
                                            (13, 16, 7, 20, 50, [-1, 0, 1, 1, 1, 1, 2, 3, 0, 8, 8, 8, 8]),     # four children twice
                                            (7, 32, 6, 5, 30, [-1, 0, 0, 0, 0, 0, 0])])                        # a star
def test_multihead_hclt_on_the_block_engine(gpu, oracle, V, K, C, H, B, tree):
    """H heads over the root's products (src-jl/multi_head_pc/bit_circuit.jl:14-56): the block
    engine (body through the walk kernels, heads in two small kernels) against the layered engine
    on the equivalent description and against the oracle: parameter order, per-head likelihoods,
    mask-weighted mixture, flows with one-hot and soft masks, EM update."""
    torch, P = gpu
    O = oracle
    from helpers import multihead_hclt, describe_dag, correlated_data
    from pcmi355._lib import lib, check
    rng = np.random.default_rng(V * 100 + H)
    parent = O.random_tree(V, rng, 3) if tree is None else np.array(tree, np.int32)
    heads, _ = multihead_hclt(parent, K, C, H, rng)
    g = describe_dag(heads)
    gen = P.compile_circuit(g["node_type"], g["child_ptr"], g["child_idx"], g["sum_logp"], g["input_var"], g["input_logp"],
                            V, C, H)
    blk = P.multihead_hclt_from_clt(parent, C, K, H)
    pv = P.vectorize_parameters(gen)
    assert blk.num_parameters() == len(pv) and blk.size("heads") == H
    P.update_parameters(blk, pv)
    np.testing.assert_array_equal(P.vectorize_parameters(blk), pv)
    for t in ("edge2param", "param2edge", "pargroup_sizes", "edge_parent", "edge_prime", "edge_sub", "heads"):
        np.testing.assert_array_equal(blk.table(t), gen.table(t), err_msg=t)
    data = correlated_data(B, V, C, 5, parent)
    d = torch.from_numpy(data).cuda()
    ll_g = P.loglikelihoods(gen, d).cpu().numpy()
    ll_b = P.loglikelihoods(blk, d).cpu().numpy()
    assert ll_b.shape == (B, H)
    np.testing.assert_allclose(ll_b, ll_g, rtol=2e-5)
    fc = O.bits_compile(O.summate(*heads), C, V)                      # the oracle on the same description
    mars = O.forward(fc, data)
    np.testing.assert_allclose(ll_b, mars[(blk.table("heads") - 1).astype(np.int64)].T, rtol=2e-5)
    for soft in (False, True):
        mask = np.zeros((B, H), np.float32)
        mask[np.arange(B), rng.integers(0, H, B)] = 1.0
        if soft:
            mask = (mask + rng.random((B, H)).astype(np.float32) * (rng.random((B, H)) < 0.3)).astype(np.float32)
        hm = torch.from_numpy(mask).cuda()
        mix_g = P.probs_flows_circuit(gen, d, head_mask=hm, rate=0.25 if soft else 0.0).cpu().numpy()
        mix_b = P.probs_flows_circuit(blk, d, head_mask=hm, rate=0.25 if soft else 0.0).cpu().numpy()
        np.testing.assert_allclose(mix_b, mix_g, rtol=2e-5)
        np.testing.assert_allclose(mix_b, P.multihead_loglikelihoods(blk, d, hm).cpu().numpy(), rtol=2e-5)
        check(lib.pcm_em_update(gen.handle, 0.1, 0.7))
        check(lib.pcm_em_update(blk.handle, 0.1, 0.7))
        a, b = P.vectorize_parameters(gen), P.vectorize_parameters(blk)
        assert np.abs(np.exp(a) - np.exp(b)).max() < 5e-4 * np.exp(a).max()
    P.update_parameters(blk, pv)
    lls = P.mini_batch_em_for_multihead_pc(blk, d, hm, 3, batch_size=B, pseudocount=0.1, param_inertia=0.9, shuffle="none")
    assert lls[2] > lls[1] > lls[0]
    with pytest.raises(P.PcmError):
        P.kld(blk, blk)
    with pytest.raises(P.PcmError):                                    # no head kernels for this hidden size
        P.multihead_hclt_from_clt(np.array([-1, 0, 0, 0, 0, 1], np.int32), C, 64, H)


def _random_tree(rng, V):
    """A tree over V variables in one of three shapes: uniform attachment (bushy, large fan-out
    near the root), mostly a chain, attachment to one of the last six nodes."""
    parent = np.full(V, -1, np.int32)
    style = int(rng.integers(0, 3))
    for v in range(1, V):
        if style == 0:
            parent[v] = rng.integers(0, v)
        elif style == 1 and rng.random() < 0.8:
            parent[v] = v - 1
        else:
            parent[v] = rng.integers(max(0, v - 6), v)
    return parent


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_block_engine_against_layered_engine(gpu, oracle, seed):
    """Randomly drawn trees, hidden sizes, category counts and ragged batches: the block engines
    (lean / general / wide walks, KL chains, Gumbel-max sampler) against the layered engine on the
    equivalent description -- two independent implementations, the second checked against the
    oracle elsewhere -- and, for the samples, against the oracle itself.  Tolerances: 1e-4
    relative on likelihoods, KL and its gradient, 2e-4 on updated parameters; samples equal."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta, describe_dag
    rng = np.random.default_rng(9000 + seed)
    V = int(rng.integers(2, 70))
    K = int(rng.choice([16, 32, 64, 128]))
    C = int(rng.choice([2, 3, 7, 16, 33, 100, 255, 256]))
    B = int(rng.integers(1, 200))
    parent, theta, leaf, fc = make_hclt(V, K, C, seed, parent=_random_tree(rng, V))
    a = P.hclt_from_clt(parent, C, K)
    a.set_params(block_theta(parent, K, theta), leaf)
    d = describe_dag([O.hclt_dag(parent, K, C, theta, leaf)])
    g = P.compile_circuit(d["node_type"], d["child_ptr"], d["child_idx"], d["sum_logp"], d["input_var"], d["input_logp"], V, C)
    np.testing.assert_allclose(P.vectorize_parameters(a), P.vectorize_parameters(g), atol=1e-6)
    data = torch.from_numpy(rng.integers(0, C, (B, V)).astype(np.uint8)).cuda()
    np.testing.assert_allclose(P.loglikelihoods(a, data).cpu().numpy(), P.loglikelihoods(g, data).cpu().numpy(), rtol=1e-4)
    # KL and its gradient against a second parameter set
    _, theta2, leaf2, _ = make_hclt(V, K, C, seed + 1000, parent=parent)
    a2 = P.hclt_from_clt(parent, C, K)
    a2.set_params(block_theta(parent, K, theta2), leaf2)
    g2 = P.compile_circuit(d["node_type"], d["child_ptr"], d["child_idx"], d["sum_logp"], d["input_var"], d["input_logp"], V, C)
    P.update_parameters(g2, P.vectorize_parameters(a2))
    ka, kg = P.kld(a, a2), P.kld(g, g2)
    assert abs(ka - kg) <= 1e-4 * abs(kg)
    for x, y in zip(P.kld_backward(a, a2), P.kld_backward(g, g2)):
        assert np.abs(x - y).max() <= 1e-4 * np.abs(y).max()
    # Gumbel-max samples against the oracle (compact noise: one draw per tree node and hidden state)
    if K <= 64 and V * K * K < 150_000:
        ch, _ = O.clt_children(parent)
        inner = [v for v in O.clt_bottom_up(parent) if ch[v]]
        nb = min(B, 40)
        u = rng.random((nb, len(inner) * K)), rng.random((nb, V, C))
        nn, ln = [(-np.log(-np.log(np.clip(x, 1e-12, 1 - 1e-12)))).astype(np.float32) for x in u]
        slot = np.zeros(fc.n_edges, np.int64)
        for r, v in enumerate(inner):
            nk = len(fc.meta["sum_node"][v])
            e0 = fc.meta["edge_of"][v]
            slot[e0:e0 + nk * K] = np.tile(r * K + np.arange(K), nk)
        want = O.sample(fc, nn, ln, noise_slot=slot)
        got = P.sample(a, torch.from_numpy(nn).cuda(), torch.from_numpy(ln).cuda()).cpu().numpy()
        assert np.array_equal(got, want)
    # one EM step
    for c in (a, g):
        P.mini_batch_em(c, data, 1, batch_size=B, pseudocount=0.1, param_inertia=0.3)
    pa, pg = np.exp(P.vectorize_parameters(a)), np.exp(P.vectorize_parameters(g))
    assert np.max(np.abs(pa - pg) / np.maximum(pg, 1e-6)) < 2e-4


def _forest_case(P, O, rng, T, Vt, K, C, H, max_children=3):
    """T random trees over interleaved variables of one batch."""
    from helpers import block_theta
    V = sum(Vt)
    owner = rng.permutation(np.repeat(np.arange(T), Vt))           # tree of every global variable
    gvars = [np.flatnonzero(owner == t) for t in range(T)]          # a tree's variables keep their relative order: the
    # children of a node are added up in variable order, so only then are the sums the same bits
    parent = np.full(V, -2, np.int32)
    trees = []
    for t in range(T):
        par_t = O.random_tree(Vt[t], rng, max_children)
        theta_t = np.log(rng.dirichlet(np.ones(K), size=(Vt[t], K))).astype(np.float32)
        leaf_t = np.log(rng.dirichlet(np.ones(C), size=(Vt[t], K))).astype(np.float32)
        heads_t = np.log(rng.dirichlet(np.ones(K), size=H)).astype(np.float32)
        trees.append((par_t, theta_t, leaf_t, heads_t))
        for v in range(Vt[t]):
            parent[gvars[t][v]] = -1 if par_t[v] < 0 else gvars[t][par_t[v]]
    # trees are numbered by their root's variable index
    order = np.argsort([gvars[t][np.flatnonzero(trees[t][0] < 0)[0]] for t in range(T)])
    return V, parent, [gvars[t] for t in order], [trees[t] for t in order]


@pytest.mark.parametrize("T,Vt,K,C,H,B,wide", [(3, [5, 9, 2], 16, 6, 4, 40, 3), (5, [12, 7, 20, 3, 9], 32, 256, 128, 100, 3),
                                               (16, [24] * 16, 32, 17, 40, 256, 3), (6, [30, 9, 14, 40, 8, 21], 32, 9, 7, 90, 7),
                                               (2, [8, 7], 16, 5, 3, 33, 6)])
def test_forest_handle_gives_the_bits_of_one_handle_per_tree(gpu, oracle, T, Vt, K, C, H, B, wide):
    """pcm_hclt_create_forest: per tree, likelihoods, flows and the EM update are those of a multi-head handle over
    that tree's variables (parallel_PG.jl:214-225 runs one such circuit per patch), to the bit where the trees have at
    most three children per node and within rounding where nodes are split."""
    torch, P = gpu
    from pcmi355._lib import lib, check
    rng = np.random.default_rng(T * 1000 + K)
    V, parent, gvars, trees = _forest_case(P, oracle, rng, T, Vt, K, C, H, max_children=wide)
    if wide > 3:
        assert max(np.bincount(t[0][t[0] >= 0]).max() for t in trees) > 3
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    d = torch.from_numpy(data).cuda()
    forest = P.hclt_forest_from_clts(parent, C, K, H)
    assert forest.num_trees == T and forest.size("walk_kernels") == 1
    theta = np.zeros((V, K, K), np.float32)
    leaf = np.zeros((V, K, C), np.float32)
    for gv, (par_t, theta_t, leaf_t, _) in zip(gvars, trees):
        theta[gv], leaf[gv] = theta_t, leaf_t
    forest.set_params(theta, leaf)
    forest.set_heads(np.stack([t[3] for t in trees]))
    np.testing.assert_array_equal(forest.get_heads(), np.stack([t[3] for t in trees]))
    singles = []
    for gv, (par_t, theta_t, leaf_t, heads_t) in zip(gvars, trees):
        c = P.multihead_hclt_from_clt(par_t, C, K, H)
        c.set_params(theta_t, leaf_t)
        c.set_heads(heads_t)
        singles.append((c, torch.from_numpy(np.ascontiguousarray(data[:, gv])).cuda()))
    ll_f = P.forest_loglikelihoods(forest, d).cpu().numpy()
    for t, (c, dt) in enumerate(singles):
        if wide <= 3:
            np.testing.assert_array_equal(ll_f[t].T, P.loglikelihoods(c, dt).cpu().numpy(), err_msg=f"tree {t}")
        else:
            np.testing.assert_allclose(ll_f[t].T, P.loglikelihoods(c, dt).cpu().numpy(), rtol=2e-6, err_msg=f"tree {t}")
    for soft in (False, True):
        mask = np.zeros((T, H, B), np.float32)
        for t in range(T):
            mask[t, rng.integers(0, H, B), np.arange(B)] = 1.0
        if soft:   # the trees share one bound on an example's total mask, so their fixed-point grids may differ
            mask = (mask + rng.random((T, H, B)).astype(np.float32) * (rng.random((T, H, B)) < 0.3)).astype(np.float32)
        rate = 0.25 if soft else 0.0
        mix_f = P.forest_flows(forest, d, torch.from_numpy(mask).cuda(), rate=rate).cpu().numpy()
        ea_f, lf_f = forest.get_flows()
        check(lib.pcm_em_update(forest.handle, 0.1, 0.7))
        th_f, leaf_f = forest.get_params()
        heads_f = forest.get_heads()
        for t, (c, dt) in enumerate(singles):
            mix = P.probs_flows_circuit(c, dt, head_mask=torch.from_numpy(mask[t].T.copy()).cuda(), rate=rate).cpu().numpy()
            ea, lf = c.get_flows()
            check(lib.pcm_em_update(c.handle, 0.1, 0.7))
            th, lp = c.get_params()
            exact = not soft and wide <= 3
            cmp = np.testing.assert_array_equal if exact else (
                lambda a, b, err_msg="": np.testing.assert_allclose(a, b, rtol=2e-5, atol=2e-6 * max(1.0, float(np.abs(b).max())), err_msg=err_msg))
            cmp(mix_f[t], mix, err_msg=f"tree {t} mixture")
            cmp(ea_f[gvars[t]], ea, err_msg=f"tree {t} edge flows")
            cmp(lf_f[gvars[t]], lf, err_msg=f"tree {t} leaf flows")
            cmp(th_f[gvars[t]], th, err_msg=f"tree {t} sum parameters")
            cmp(leaf_f[gvars[t]], lp, err_msg=f"tree {t} leaf parameters")
            cmp(heads_f[t], c.get_heads(), err_msg=f"tree {t} heads")


def test_forest_handle_with_example_ids_and_flow_memory(gpu, oracle):
    """Flows and EM update of a forest with example ids and flow memory, two batches in a row, against one handle per
    tree."""
    torch, P = gpu
    from pcmi355._lib import lib, check
    T, Vt, K, C, H, N = 9, [11, 6, 14, 9, 5, 17, 8, 12, 7], 16, 12, 5, 150
    rng = np.random.default_rng(77)
    V, parent, gvars, trees = _forest_case(P, oracle, rng, T, Vt, K, C, H)
    data = rng.integers(0, C, size=(N, V)).astype(np.uint8)
    d = torch.from_numpy(data).cuda()
    forest = P.hclt_forest_from_clts(parent, C, K, H)
    theta = np.zeros((V, K, K), np.float32)
    leaf = np.zeros((V, K, C), np.float32)
    for gv, (par_t, theta_t, leaf_t, _) in zip(gvars, trees):
        theta[gv], leaf[gv] = theta_t, leaf_t
    forest.set_params(theta, leaf)
    forest.set_heads(np.stack([t[3] for t in trees]))
    singles = []
    for gv, (par_t, theta_t, leaf_t, heads_t) in zip(gvars, trees):
        c = P.multihead_hclt_from_clt(par_t, C, K, H)
        c.set_params(theta_t, leaf_t)
        c.set_heads(heads_t)
        singles.append((c, torch.from_numpy(np.ascontiguousarray(data[:, gv])).cuda()))
    for it, (B, rate) in enumerate([(70, 0.0), (45, 0.6)]):
        ids = torch.from_numpy(rng.choice(N, size=B, replace=False).astype(np.int32)).cuda()
        mask = np.zeros((T, H, B), np.float32)
        for t in range(T):
            mask[t, rng.integers(0, H, B), np.arange(B)] = 1.0
        hm = torch.from_numpy(mask).cuda()
        ll = torch.empty((T, B), device="cuda")
        check(lib.pcm_flows(forest.handle, d.data_ptr(), d.stride(0), d.stride(1), ids.data_ptr(), B, rate, hm.data_ptr(),
                            ll.data_ptr()))
        check(lib.pcm_em_update(forest.handle, 0.1, 0.8))
        th_f, leaf_f = forest.get_params()
        heads_f = forest.get_heads()
        for t, (c, dt) in enumerate(singles):
            hm_t = torch.from_numpy(np.ascontiguousarray(mask[t])).cuda()
            ll_t = torch.empty(B, device="cuda")
            check(lib.pcm_flows(c.handle, dt.data_ptr(), dt.stride(0), dt.stride(1), ids.data_ptr(), B, rate, hm_t.data_ptr(),
                                ll_t.data_ptr()))
            check(lib.pcm_em_update(c.handle, 0.1, 0.8))
            th, lp = c.get_params()
            np.testing.assert_array_equal(ll[t].cpu().numpy(), ll_t.cpu().numpy(), err_msg=f"batch {it} tree {t}")
            np.testing.assert_array_equal(th_f[gvars[t]], th, err_msg=f"batch {it} tree {t}")
            np.testing.assert_array_equal(leaf_f[gvars[t]], lp, err_msg=f"batch {it} tree {t}")
            np.testing.assert_array_equal(heads_f[t], c.get_heads(), err_msg=f"batch {it} tree {t}")


def test_em_driver_of_a_forest_follows_the_driver_of_every_tree(gpu, oracle):
    """mini_batch_em_for_forest against mini_batch_em_for_multihead_pc on a handle per tree: three epochs in the
    given order of examples, rising inertia, flow memory."""
    torch, P = gpu
    T, Vt, K, C, H, N = 4, [9, 13, 6, 10], 16, 8, 6, 96
    rng = np.random.default_rng(5)
    V, parent, gvars, trees = _forest_case(P, oracle, rng, T, Vt, K, C, H)
    data = rng.integers(0, C, size=(N, V)).astype(np.uint8)
    d = torch.from_numpy(data).cuda()
    masks = np.zeros((T, N, H), np.float32)
    for t in range(T):
        masks[t, np.arange(N), rng.integers(0, H, N)] = 1.0
    forest = P.hclt_forest_from_clts(parent, C, K, H)
    theta = np.zeros((V, K, K), np.float32)
    leaf = np.zeros((V, K, C), np.float32)
    for gv, (par_t, theta_t, leaf_t, _) in zip(gvars, trees):
        theta[gv], leaf[gv] = theta_t, leaf_t
    forest.set_params(theta, leaf)
    forest.set_heads(np.stack([t[3] for t in trees]))
    kw = dict(batch_size=32, pseudocount=0.1, param_inertia=0.8, param_inertia_end=0.95, flow_memory=200.0, shuffle="none")
    lls_f = P.mini_batch_em_for_forest(forest, d, torch.from_numpy(masks), 3, **kw)
    assert lls_f.shape == (3, T) and (lls_f[2] > lls_f[0]).all()
    for t, (gv, (par_t, theta_t, leaf_t, heads_t)) in enumerate(zip(gvars, trees)):
        c = P.multihead_hclt_from_clt(par_t, C, K, H)
        c.set_params(theta_t, leaf_t)
        c.set_heads(heads_t)
        dt = torch.from_numpy(np.ascontiguousarray(data[:, gv])).cuda()
        lls = P.mini_batch_em_for_multihead_pc(c, dt, torch.from_numpy(masks[t]).cuda(), 3, **kw)
        np.testing.assert_allclose(lls_f[:, t], lls, rtol=1e-12)
        np.testing.assert_array_equal(forest.get_heads()[t], c.get_heads())


def test_forest_handle_refuses_what_only_one_circuit_defines(gpu, oracle):
    torch, P = gpu
    parent = np.array([-1, 0, 0, -1, 3], np.int32)
    forest = P.hclt_forest_from_clts(parent, 4, 16, 2)
    with pytest.raises(P.PcmError, match="forest"):
        P.vectorize_parameters(forest)
    with pytest.raises(P.PcmError, match="forest"):
        forest.table("edge2param")
    data = torch.zeros((8, 5), dtype=torch.uint8, device="cuda")
    noise = torch.zeros((8, 64), device="cuda")
    other = P.hclt_from_clt(np.array([-1, 0, 0], np.int32), 4, 16)
    marked = P.hclt_from_clt(np.array([-1, 0, 0], np.int32), 4, 16)
    marked.set_missing_category()
    for bad, what in ((forest, "forest"), (marked, "missing-value")):
        for call in (lambda: P.kld(bad, bad), lambda: P.kld(other, bad) if bad is marked else P.kld(bad, bad),
                     lambda: P.kld_backward(bad, bad),
                     lambda: P.sample(bad, noise, torch.zeros((8, 5, 4), device="cuda")),
                     lambda: P.gumbel_sample(bad, 8, temperature=1.0),
                     lambda: P.flow_gradients(bad, 8),
                     lambda: P.loglikelihoods(bad, torch.zeros((8, bad.num_vars, 4), device="cuda")),
                     lambda: P.kld(bad, np.zeros((2, 10), np.float32), np.zeros((2, 10), np.float32))):
            with pytest.raises((P.PcmError, ValueError)) as e:
                call()
            assert what in str(e.value) or isinstance(e.value, ValueError), str(e.value)
    with pytest.raises(P.PcmError, match="head_mask"):      # pcm_em_step carries no head mask
        from pcmi355._lib import lib, check
        check(lib.pcm_em_step(forest.handle, data.data_ptr(), data.stride(0), data.stride(1), None, 8, 0.0, 0.1, 0.9,
                              torch.empty(16, device="cuda").data_ptr()))
    with pytest.raises(P.PcmError, match="tree of its own"):
        P.hclt_forest_from_clts(np.array([-1, 0, -1], np.int32), 4, 16, 2)
    with pytest.raises(P.PcmError, match="more than one root"):
        P.multihead_hclt_from_clt(parent, 4, 16, 2)


@pytest.mark.parametrize("V,K,C,B,heads", [(9, 16, 6, 70, 0), (14, 32, 256, 100, 0), (6, 128, 9, 48, 0), (11, 64, 5, 33, 0),
                                           (8, 32, 7, 50, 3)])
def test_missing_values_as_a_marker_category(gpu, oracle, V, K, C, B, heads):
    """pcm_set_missing_category: the last category marks a missing value (src/regularization/reg_likelihood.jl:40-47,
    src/nodes/fixable_categorical_dist.jl:223-248).  Likelihoods, flows (the marker's row = missing_flow) and the EM
    update against the oracle, whose treatment of the marker is pinned by enumeration of completions."""
    torch, P = gpu
    O = oracle
    from helpers import block_theta, rel_err
    from pcmi355._lib import lib, check
    rng = np.random.default_rng(V * K + C)
    parent = O.random_tree(V, rng, 3)
    theta, leaf = O.random_hclt_params(parent, K, C - 1, rng, "dirichlet")
    leaf = np.concatenate([leaf, np.zeros((V, K, 1), np.float32)], axis=2)          # the marker's row: log 1
    data = rng.integers(0, C - 1, size=(B, V)).astype(np.uint8)
    data[rng.random((B, V)) < 0.25] = C - 1
    data[0] = C - 1                                                                  # an example with nothing observed
    d = torch.from_numpy(data).cuda()
    if heads:
        bpc = P.multihead_hclt_from_clt(parent, C, K, heads)
        head_logp = np.log(rng.dirichlet(np.ones(K), size=heads)).astype(np.float32)
        bpc.set_heads(head_logp)
    else:
        bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_missing_category()
    noisy = leaf.copy()
    noisy[:, :, C - 1] = -3.0                                                        # whatever the caller puts there
    bpc.set_params(block_theta(parent, K, theta), noisy)
    assert (bpc.get_params()[1][:, :, C - 1] == 0).all()
    fc = O.hclt_flat(parent, K, C, theta, leaf)
    if heads:
        # the oracle's single root row stands for head 0: give it that head's parameters over the root's products
        mask = np.zeros((B, heads), np.float32)
        mask[:, 0] = 1.0
        th0 = {v: t.copy() for v, t in theta.items()}
        root = int(np.flatnonzero(parent < 0)[0])
        th0[root] = np.vstack([head_logp[0][None, :], theta[root][1:]]) if theta[root].shape[0] > 1 else head_logp[0][None, :]
        fc = O.hclt_flat(parent, K, C, th0, leaf)
        ll = P.probs_flows_circuit(bpc, d, head_mask=torch.from_numpy(mask).cuda()).cpu().numpy()
    else:
        ll = P.probs_flows_circuit(bpc, d).cpu().numpy()
    mars = O.forward(fc, data)
    assert rel_err(ll[1:], mars[-1][1:]).max() < LL_RTOL
    assert abs(ll[0]) < 1e-4 and abs(mars[-1][0]) < 1e-4                             # nothing observed: probability 1
    if heads:
        return                                                                       # (flows of the body as below)
    flows, ea = O.backward(fc, mars)
    lf_ref = O.input_flows(fc, data, flows).reshape(V, K, C)
    _, lf = bpc.get_flows()
    assert np.abs(lf - lf_ref).max() < FLOW_RTOL * max(lf_ref.max(), 1e-3)
    np.testing.assert_allclose(lf.sum(axis=(1, 2)), B, rtol=1e-4)                    # marker's row included
    logp_new, leaf_new = O.em_update(fc, ea, lf_ref.reshape(-1), 0.1, 0.9, missing=True)
    check(lib.pcm_em_update(bpc.handle, 0.1, 0.9))
    new = fc.copy()
    new.logp, new.leaf_logp = logp_new, leaf_new
    th_ref, leaf_ref = O.hclt_block_params(new)
    th, lp = bpc.get_params()
    for v, blk in th_ref.items():
        assert rel_err(np.exp(th[v][:blk.shape[0]]), np.exp(blk)).max() < PARAM_RTOL
    assert rel_err(np.exp(lp), np.exp(leaf_ref)).max() < PARAM_RTOL
    assert (lp[:, :, C - 1] == 0).all()
    np.testing.assert_allclose(np.exp(lp[:, :, :C - 1]).sum(axis=2), 1.0, rtol=1e-5)
    # a second step keeps going up; what only complete data define is refused
    ll2 = P.probs_flows_circuit(bpc, d).cpu().numpy()
    assert ll2.mean() > ll.mean()
    with pytest.raises(P.PcmError, match="missing-value"):
        P.kld(bpc, bpc)


@pytest.mark.parametrize("V,K,C,B,bushy", [(9, 16, 5, 70, False), (40, 32, 256, 300, False), (600, 64, 4, 40, True),
                                            (11, 128, 9, 50, False), (8, 64, 256, 33, False)])
def test_per_example_weights_on_single_head_block_circuits(gpu, oracle, V, K, C, B, bushy):
    """`weights` of probs_flows_circuit_with_reg (reg_flow.jl:38-39,190-191) on the walk kernels: the flow an example
    starts with at the root.  Edge and leaf statistics against the oracle seeded with the weights (some of them
    zero, some above one: the fixed-point counters scale by their bound), likelihoods unweighted; on the lean
    kernels (K = 16, 32), the general walk kernels (K = 64 on a bushy tree) and the wide kernels (K = 128, K = 64 on
    a small tree)."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta
    rng = np.random.default_rng(V * 100 + K)
    if bushy:
        parent = np.asarray(O.random_tree(V, rng, 3), np.int32)
    else:
        parent = np.full(V, -1, np.int32)
        for v in range(1, V):
            parent[v] = rng.integers(max(0, v - 3), v)
    parent, theta, leaf, fc = make_hclt(V, K, C, V + K, parent=parent)
    c = P.hclt_from_clt(parent, C, K)
    c.set_params(block_theta(parent, K, theta), leaf)
    assert c.size("walk_kernels") == (2 if bushy else 3 if K >= 64 else 1)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    w = rng.uniform(0.0, 5.0, size=B).astype(np.float32)
    w[::5] = 0.0
    d = torch.from_numpy(data).cuda()
    ll = P.probs_flows_circuit(c, d, weights=w).cpu().numpy()
    mars = O.forward(fc, data)
    assert np.abs(ll - mars[-1]).max() < 1e-4 * np.abs(mars[-1]).max()
    flows, ea_ref = O.backward(fc, mars, root_ids=np.array([fc.n_nodes - 1], np.int32), root_flow=w[None, :])
    lf_ref = O.input_flows(fc, data, flows).reshape(V, K, C)
    ea, lf = c.get_flows()
    for v, blk in O.hclt_block_aggr(fc, ea_ref).items():
        nk = blk.shape[0]
        assert np.abs(ea[v][:nk] - blk).max() < 2e-4 * max(blk.max(), 1e-3), f"edge_aggr block {v}"
    assert np.abs(lf - lf_ref).max() < 2e-4 * max(lf_ref.max(), 1e-3)
    np.testing.assert_allclose(lf.sum(axis=(1, 2)), w.sum(), rtol=1e-4)   # every example passes every variable with its weight
    ref = fc.copy()
    ref.logp, ref.leaf_logp = O.em_update(fc, ea_ref, lf_ref.reshape(-1), 0.1, 0.9)
    th_ref, leaf_ref = O.hclt_block_params(ref)
    import pcmi355._lib as L
    from helpers import rel_err
    L.check(L.lib.pcm_em_update(c.handle, 0.1, 0.9))
    th, lf_new = c.get_params()
    tol = 3e-4 if bushy else 1e-4   # (600 variables deep in float32 on both sides: rounding, not method)
    for v, blk in th_ref.items():
        nk = blk.shape[0]
        assert rel_err(np.exp(th[v][:nk]), np.exp(blk)).max() < tol, f"theta block {v}"
    assert rel_err(np.exp(lf_new), np.exp(leaf_ref)).max() < tol
    # unit weights are no weights, to the bit
    c.set_params(block_theta(parent, K, theta), leaf)
    P.probs_flows_circuit(c, d, weights=np.ones(B, np.float32))
    a1 = c.get_flows()
    P.probs_flows_circuit(c, d)
    a0 = c.get_flows()
    for x, y in zip(a1, a0):
        np.testing.assert_array_equal(x, y)


def test_forest_driver_with_per_example_weights(gpu, oracle):
    """`weights` of the multi-head EM driver (src-jl/multi_head_pc/em.jl:5,20,72) over a forest: the same as masks
    that carry the weights, to the bit, and different from the unweighted run."""
    torch, P = gpu
    rng = np.random.default_rng(77)
    T, Vt, K, C, H, B = 3, [6, 9, 4], 16, 5, 4, 96
    V, parent, gvars, trees = _forest_case(P, oracle, rng, T, Vt, K, C, H)
    data = torch.from_numpy(rng.integers(0, C, size=(B, V)).astype(np.uint8)).cuda()
    masks = torch.from_numpy(rng.random((T, B, H)).astype(np.float32)).cuda()
    w = torch.from_numpy(rng.uniform(0.0, 4.0, size=B).astype(np.float32)).cuda()

    def run(m, weights):
        f = P.hclt_forest_from_clts(parent, C, K, H)
        theta = np.zeros((V, K, K), np.float32)
        leaf = np.zeros((V, K, C), np.float32)
        for gv, (par_t, theta_t, leaf_t, _) in zip(gvars, trees):
            theta[gv], leaf[gv] = theta_t, leaf_t
        f.set_params(theta, leaf)
        f.set_heads(np.stack([t[3] for t in trees]))
        P.mini_batch_em_for_forest(f, data, m, 2, batch_size=48, pseudocount=0.1, param_inertia=0.5, shuffle="none",
                                   weights=weights)
        return f.get_params() + (f.get_heads(),)
    a = run(masks, w)
    b = run(masks * w[None, :, None], None)
    c = run(masks, None)
    for x, y in zip(a, b):
        np.testing.assert_array_equal(x, y)
    assert np.abs(np.exp(a[1]) - np.exp(c[1])).max() > 1e-3   # (leaf tables)


def _deep_tree(rng, V, chain):
    """A tree that is mostly one long chain (every node hangs on its predecessor with probability `chain`,
    else on one of the six before it): hundreds of levels deep at a few hundred variables."""
    parent = np.full(V, -1, np.int32)
    for v in range(1, V):
        parent[v] = v - 1 if rng.random() < chain else rng.integers(max(0, v - 6), v)
    return parent


@pytest.mark.parametrize("V,K,C,B,chain,weighted", [(128, 16, 33, 96, 0.8, False), (128, 32, 255, 120, 0.8, True),
                                                    (200, 32, 256, 150, 0.8, False), (200, 16, 255, 300, 0.5, True),
                                                    (263, 32, 33, 200, 0.8, False), (263, 16, 256, 260, 0.9, True),
                                                    (263, 32, 256, 64, 0.0, False)])
def test_deep_trees_three_way(gpu, oracle, V, K, C, B, chain, weighted):
    """Trees of 128-263 variables, 80-200 levels deep, one EM step (pseudocount 0.1, inertia 0.3 so that the
    statistics dominate the new parameters), with and without per-example weights.  At these depths the reference's
    float32 log-values (several hundred to a thousand nats, one ulp = 6e-5) make its own flows good to a few 1e-4
    only, so the comparison is three-way: library vs float64 oracle, float32 oracle (the reference's arithmetic)
    vs float64 oracle, library vs float32 oracle.  The library keeps a node's value as a tile of order-one numbers
    plus per-example scalars and must meet the 1e-4 bar against the exact result at every depth; its distance to
    the float32 oracle must be the float32 oracle's own error."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta, assert_three_way
    rng = np.random.default_rng(V * 1000 + K * 10 + C)
    parent = _deep_tree(rng, V, chain)
    parent, theta, leaf, fc = make_hclt(V, K, C, V + K + C, parent=parent)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    w = None
    if weighted:
        w = rng.uniform(0.0, 5.0, size=B).astype(np.float32)
        w[::3] = 0.0
    pc, inertia = 0.1, 0.3
    c = P.hclt_from_clt(parent, C, K)
    c.set_params(block_theta(parent, K, theta), leaf)
    assert c.size("walk_kernels") == 1
    d = torch.from_numpy(data).cuda()
    ll = P.probs_flows_circuit(c, d, weights=w).cpu().numpy()
    import pcmi355._lib as L
    L.check(L.lib.pcm_em_update(c.handle, pc, inertia))
    th, lf_new = c.get_params()

    def oracle_step(double):
        mars = O.forward(fc, data, double=double)
        root_flow = None if w is None else w[None, :].astype(np.float64 if double else np.float32)
        flows, ea = O.backward(fc, mars, root_ids=np.array([fc.n_nodes - 1], np.int32),
                               root_flow=np.ones((1, B)) if root_flow is None else root_flow, double=double)
        lfl = O.input_flows(fc, data, flows, double=double)
        new = fc.copy()
        new.logp, new.leaf_logp = O.em_update(fc, ea, lfl, pc, inertia, double=double)
        return mars[-1], O.hclt_block_params(new)

    ll64, (th64, lf64) = oracle_step(True)
    ll32, (th32, lf32) = oracle_step(False)
    assert (np.abs(ll - ll32) / np.abs(ll32)).max() < LL_RTOL
    assert (np.abs(ll - ll64) / np.abs(ll64)).max() < LL_RTOL
    depth = 0
    for v in range(V):
        n, u = 0, v
        while parent[u] >= 0:
            u, n = parent[u], n + 1
        depth = max(depth, n)
    assert_three_way((th, lf_new), (th64, lf64), (th32, lf32), PARAM_RTOL,
                     f"V={V} K={K} C={C} B={B} depth={depth} weighted={weighted}")


@pytest.mark.parametrize("update_interval,flow_memory,fscale", [(2, 0.0, 1.0), (3, 400.0, 1.0), (1, 0.0, 1.0), (2, 300.0, 2.0),
                                                                (1, 0.0, 0.6)])
def test_em_beta_driver_collects_statistics_over_an_interval(gpu, oracle, update_interval, flow_memory, fscale):
    """`mini_batch_em_beta` (src-jl/learning/em.jl:289-409): statistics collect over `update_interval` batches, are
    cleared (or decayed by the flow memory) at a batch with batch_id % update_interval == 1, and the parameters move
    after a batch with batch_id % update_interval == 0 -- replayed on the float64 oracle batch by batch, including the
    source's behaviour at update_interval = 1 (the clearing condition never holds, the statistics of an epoch pile up).
    fscale != 1: the flows of the tempered posterior (src-jl/learning/flow.jl:120-373), which an HCLT handle runs on
    its layered form."""
    torch, P = gpu
    from helpers import make_hclt, correlated_data, block_theta, rel_err
    V, K, C, B, nb, pc, inertia = 10, 16, 12, 64, 6, 0.1, 0.7
    parent, theta, leaf, fc = make_hclt(V, K, C, 5)
    data = correlated_data(B * nb, V, C, 6, parent)
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    lls = P.mini_batch_em_beta(bpc, torch.from_numpy(data).cuda(), 2, batch_size=B, pseudocount=pc, param_inertia=inertia,
                               param_inertia_end=0.9, flow_memory=flow_memory, flow_memory_end=flow_memory * 2,
                               shuffle="none", update_interval=update_interval, fscale=fscale)
    cur, want, inr, fm = fc.copy(), [], inertia, flow_memory
    for epoch in range(2):
        ea = lf = None
        tot = 0.0
        for batch_id in range(1, nb + 1):
            idx = np.arange((batch_id - 1) * B, batch_id * B, dtype=np.int32)
            if ea is not None and batch_id % update_interval == 1:
                rate = 0.0 if fm == 0 else max(0.0, 1.0 - (B + pc) / fm)
                ea, lf = ea * rate, lf * rate
            mars = oracle.forward(cur, data, idx, True)
            flows, ea_b = oracle.backward(cur, mars, double=True, fscale=fscale)
            lf_b = oracle.input_flows(cur, data, flows, idx, double=True)
            ea = ea_b if ea is None else ea + ea_b
            lf = lf_b if lf is None else lf + lf_b
            tot += mars[-1].sum()
            if batch_id % update_interval == 0:
                logp, new_leaf, ea = oracle.em_update(cur, ea, lf, pc, inr, True, return_aggr=True)   # (the pseudocount stays in)
                cur = cur.copy()
                cur.logp, cur.leaf_logp = logp.astype(np.float32), new_leaf.astype(np.float32)
        want.append(tot / B / nb)
        inr += (0.9 - inertia) / 2
        fm += flow_memory / 2
    assert np.abs(np.array(lls) - np.array(want)).max() < 2e-5 * abs(want[0])
    th_ref, leaf_ref = oracle.hclt_block_params(cur)
    th, lf_new = bpc.get_params()
    for v, blk in th_ref.items():
        assert rel_err(np.exp(th[v][:blk.shape[0]]), np.exp(blk)).max() < 5e-4
    assert rel_err(np.exp(lf_new), np.exp(leaf_ref)).max() < 5e-4
    # the loop leaves the handle as it found it: an ordinary step afterwards runs on the block kernels again
    ll = P.probs_flows_circuit(bpc, torch.from_numpy(data[:B]).cuda()).cpu().numpy()
    assert rel_err(ll, oracle.forward(cur, data[:B], double=True)[-1]).max() < 1e-4
