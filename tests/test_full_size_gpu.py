"""Benchmark-size checks (3072-variable HCLT, K = 32, 256 categories, batch 4096): the oracle
on a subset it finishes in seconds, and size-independent properties on the whole batch."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

LL_RTOL = 1e-4
PARAM_RTOL = 1e-4


@pytest.fixture(scope="module")
def c3():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355 as P
    from pcmi355 import workloads
    cfg = workloads.make_config("c3_hclt3072_k32")
    bpc = P.hclt_from_clt(cfg["parent"], cfg["C"], cfg["K"])
    bpc.set_params(cfg["theta"], cfg["leaf"])
    data = torch.from_numpy(cfg["data"]).cuda()
    return torch, P, cfg, bpc, data


def _oracle_circuit(O, cfg, theta=None, leaf=None):
    parent, K, C = cfg["parent"], cfg["K"], cfg["C"]
    theta = cfg["theta"] if theta is None else theta
    leaf = cfg["leaf"] if leaf is None else leaf
    ch, _ = O.clt_children(parent)
    return O.hclt_flat(parent, K, C, {v: theta[v] for v in range(len(parent)) if ch[v]}, leaf)


def test_full_batch_step_properties_and_oracle_subset(c3, oracle):
    torch, P, cfg, bpc, data = c3
    import pcmi355._lib as L
    O = oracle
    V, K, C, B = cfg["V"], cfg["K"], cfg["C"], cfg["B"]
    fc = _oracle_circuit(O, cfg)
    sub = 96
    ll_ref = O.forward(fc, cfg["data"][:sub])[-1]
    ll = P.loglikelihoods(bpc, data).cpu().numpy()
    assert np.isfinite(ll).all()
    assert (np.abs(ll[:sub] - ll_ref) / np.abs(ll_ref)).max() < LL_RTOL

    # flows of the whole batch: every example sends one unit of flow through every variable
    # and through every inner tree node (root: its single sum node)
    ll2 = P.probs_flows_circuit(bpc, data).cpu().numpy()
    assert np.array_equal(ll, ll2)
    ea, lf = bpc.get_flows()
    np.testing.assert_allclose(lf.sum(axis=(1, 2)), B, rtol=1e-4)
    ch, root = O.clt_children(cfg["parent"])
    inner = np.array([v for v in range(V) if ch[v]])
    np.testing.assert_allclose(ea[inner].sum(axis=(1, 2)), B, rtol=1e-4)
    assert (ea >= 0).all() and (lf >= 0).all()

    # one EM step on the first `sub` examples against the oracle
    ids = torch.arange(sub, dtype=torch.int32, device="cuda")
    llb = torch.empty(sub, device="cuda")
    L.check(L.lib.pcm_em_step(bpc.handle, data.data_ptr(), data.stride(0), data.stride(1), ids.data_ptr(), sub, 0.0,
                              0.1, 0.9, llb.data_ptr()))
    # At this depth (132 tree levels, sub-circuit log-values of several thousand) float32 log-values, the reference's
    # arithmetic, are only good to ~1e-3 absolute, which is a relative error of 1e-3 on the smallest flows: the
    # float32 oracle misses the float64 result by 2.5e-3 on a few of the 27 M parameters.  The library keeps node
    # values in two parts (order-one tiles + per-example maxima) and must be within 1e-4 of the float64 result;
    # what separates it from the float32 oracle must be that oracle's own error.
    ids_np = np.arange(sub, dtype=np.int32)
    _, logp64, leaf64, _, _ = O.em_step(fc, cfg["data"], ids_np, 0.1, 0.9, double=True)
    _, logp32, leaf32, _, _ = O.em_step(fc, cfg["data"], ids_np, 0.1, 0.9)
    th, lf_new = bpc.get_params()

    def blocks(logp, leaf):
        new = fc.copy()
        new.logp, new.leaf_logp = logp, leaf
        return O.hclt_block_params(new)

    from helpers import assert_three_way
    th64, lf64 = blocks(logp64, leaf64)
    th32, lf32 = blocks(logp32, leaf32)
    assert_three_way((th, lf_new), (th64, lf64), (th32, lf32), PARAM_RTOL, "3072 variables, 96 examples")
    # the per-example log-likelihoods of the step against the float32 oracle, at the bar itself
    ll32 = O.forward(fc, cfg["data"][:sub])[-1]
    assert (np.abs(llb.cpu().numpy() - ll32) / np.abs(ll32)).max() < LL_RTOL
    bpc.set_params(cfg["theta"], cfg["leaf"])


def test_em_on_the_full_batch_raises_the_likelihood(c3):
    torch, P, cfg, bpc, data = c3
    bpc.set_params(cfg["theta"], cfg["leaf"])
    lls = P.mini_batch_em_with_reg(bpc, data, 4, batch_size=cfg["B"], pseudocount=0.1, param_inertia=0.9, shuffle="none")
    assert all(b > a for a, b in zip(lls, lls[1:])), lls
    th, lf = bpc.get_params()
    np.testing.assert_allclose(np.exp(lf.astype(np.float64)).sum(-1), 1.0, rtol=1e-4)
    bpc.set_params(cfg["theta"], cfg["leaf"])


def test_kld_on_the_benchmark_circuit(c3, oracle):
    torch, P, cfg, bpc, data = c3
    O = oracle
    from pcmi355 import workloads
    bpc.set_params(cfg["theta"], cfg["leaf"])
    theta2, leaf2 = workloads.init_params(cfg["parent"], cfg["K"], cfg["C"], 4242)
    q = P.hclt_from_clt(cfg["parent"], cfg["C"], cfg["K"])
    q.set_params(theta2, leaf2)
    assert abs(P.kld(bpc, bpc)) < 1e-3
    got = P.kld(bpc, q)
    f1, f2 = _oracle_circuit(O, cfg), _oracle_circuit(O, cfg, theta2, leaf2)
    want = O.kld(f1, f2, double=True)[0][-1]
    assert want > 0 and abs(got - want) < 1e-4 * want
    g1, g2 = P.kld_backward(bpc, q)
    assert np.isfinite(g1).all() and np.isfinite(g2).all()
    n_sum = bpc.num_inner_params()
    # the gradient with respect to q's sum log-parameters is -g * p1 <= 0
    assert (g2[:n_sum] <= 0).all()
    # both gradient vectors, all 27.7 M entries, against the float64 oracle at the tolerance of the
    # small circuits (1e-4 of the largest entry).  The oracle works on the direct flat form, whose
    # numbering is its own: a third circuit whose parameters are their own block coordinates tells
    # where every block entry sits in the parameter vector.
    V, K, C = cfg["V"], cfg["K"], cfg["C"]
    ids = P.hclt_from_clt(cfg["parent"], C, K)
    ch, root = O.clt_children(cfg["parent"])
    inner = [v for v in range(V) if ch[v]]
    code = np.zeros((V, K, K), np.float32)
    for r, v in enumerate(inner):
        code[v] = (r * K * K + np.arange(K * K)).reshape(K, K)
    leaf_code = np.broadcast_to((np.arange(V * K, dtype=np.float32)).reshape(V, K, 1), (V, K, C))
    ids.set_params(code, np.ascontiguousarray(leaf_code))
    where = P.vectorize_parameters(ids)
    sum_at = where[:n_sum].astype(np.int64)                      # -> inner rank * K*K + k*K + j
    leaf_at = where[n_sum::C].astype(np.int64)                   # -> v*K + j of every input node, in vector order
    assert len(np.unique(sum_at)) == n_sum and len(np.unique(leaf_at)) == V * K
    _, ek = O.kld(f1, f2, double=True)
    _, eg1, eg2, lg1, lg2 = O.kld_backward(f1, f2, ek, double=True)
    for got_vec, eg, lg in ((g1, eg1, lg1), (g2, eg2, lg2)):
        blocks = np.zeros((len(inner), K, K))
        for r, v in enumerate(inner):
            nk = len(f1.meta["sum_node"][v])
            e0 = f1.meta["edge_of"][v]
            blocks[r, :nk] = eg[e0:e0 + nk * K].reshape(nk, K)
        want_vec = np.concatenate([blocks.reshape(-1)[sum_at], lg.reshape(V * K, C)[leaf_at].reshape(-1)])
        assert np.abs(got_vec - want_vec).max() < 1e-4 * np.abs(want_vec).max()


def test_sampling_on_the_benchmark_circuit(c3, oracle):
    """4096 samples from device-generated noise; the first 24 are checked bit-for-bit against
    the oracle, all of them for range and completeness."""
    torch, P, cfg, bpc, data = c3
    O = oracle
    bpc.set_params(cfg["theta"], cfg["leaf"])
    V, K, C, B = cfg["V"], cfg["K"], cfg["C"], cfg["B"]
    n_inner = bpc.size("inner_tree_nodes")
    g = torch.Generator(device="cuda").manual_seed(7)
    u1 = torch.rand((B, n_inner * K), device="cuda", generator=g).clamp_(1e-10, 1 - 1e-7)
    node_noise = -torch.log(-torch.log(u1))
    del u1
    leaf_noise = torch.empty((B, V, C), device="cuda")
    for s in range(0, B, 512):
        u2 = torch.rand((512, V, C), device="cuda", generator=g).clamp_(1e-10, 1 - 1e-7)
        leaf_noise[s:s + 512] = -torch.log(-torch.log(u2))
    del u2
    out = P.sample(bpc, node_noise, leaf_noise).cpu().numpy()
    assert out.shape == (B, V) and out.dtype == np.uint8
    assert (out < C).all()                     # every variable was reached (unreached ones keep 255 >= C)
    sub = 24
    fc = _oracle_circuit(O, cfg)
    ch, root = O.clt_children(cfg["parent"])
    inner = [v for v in O.clt_bottom_up(cfg["parent"]) if ch[v]]
    slot = np.zeros(fc.n_edges, np.int64)
    for r, v in enumerate(inner):
        nk = len(fc.meta["sum_node"][v])
        e0 = fc.meta["edge_of"][v]
        slot[e0:e0 + nk * K] = np.tile(r * K + np.arange(K), nk)
    want = O.sample(fc, node_noise[:sub].cpu().numpy(), leaf_noise[:sub].cpu().numpy(), noise_slot=slot)
    assert np.array_equal(out[:sub], want)
    assert out.std() > 10                      # not collapsed; distributional checks are on small circuits


def test_kl_gradient_feeds_an_adam_step_on_the_benchmark_circuit(c3, oracle):
    """Variational configuration: the gradient of KL(p || q) with respect to q's sum parameters
    drives one Adam step (lr 1e-3, descent on the KL = ascent on its negative) on q; the
    optimiser state and the renormalised parameters match the oracle."""
    torch, P, cfg, bpc, data = c3
    O = oracle
    from pcmi355 import workloads
    bpc.set_params(cfg["theta"], cfg["leaf"])
    theta2, leaf2 = workloads.init_params(cfg["parent"], cfg["K"], cfg["C"], 4243, kind="dirichlet")
    q = P.hclt_from_clt(cfg["parent"], cfg["C"], cfg["K"])
    q.set_params(theta2, leaf2)
    before = P.kld(bpc, q)
    _, g2 = P.kld_backward(bpc, q)
    n_sum = q.num_inner_params()
    grad = (-g2[:n_sum]).astype(np.float32)
    params = P.vectorize_parameters(q)[:n_sum].copy()
    m = np.zeros(n_sum, np.float32)
    v = np.zeros(n_sum, np.float32)
    dp, dm, dv = (torch.from_numpy(x.copy()).cuda() for x in (params, m, v))
    lr = 1e-3
    P.adam_step(q, torch.from_numpy(grad).cuda(), dp, dm, dv, lr=lr, t=1)
    sizes = q.table("pargroup_sizes")
    logp_ref = params.copy()
    O.adam_step(params, grad, m, v, lr, 0.9, 0.999, 1e-8, 1, np.concatenate([[0], np.cumsum(sizes)]), logp_ref)
    np.testing.assert_allclose(dp.cpu().numpy(), params, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(dm.cpu().numpy(), m, rtol=1e-5, atol=1e-9)
    got = P.vectorize_parameters(q)[:n_sum]
    assert (np.abs(np.exp(got) - np.exp(logp_ref)) / np.exp(logp_ref)).max() < 1e-5
    # (the derivative with respect to every sum log-parameter of q is -g * p1 < 0, so at t = 1
    # Adam moves all of them by the same +lr and the per-node normalisation takes it back: the
    # divergence must come out unchanged, which checks the normalisation at full size)
    after = P.kld(bpc, q)
    assert abs(after - before) < 1e-5 * before


def test_c2_em_step_at_its_real_shape(oracle):
    """The K = 128 configuration at its real shape (48 variables, 256 categories, batch 4096, wide block kernels):
    one EM step on the first 128 examples against the oracle -- log-likelihoods, `edge_aggr`, leaf flows and the
    updated parameters in the order of reg_em.jl:276-299 -- and on the whole batch the flow every example sends
    through every variable and every tree node."""
    import torch
    import pcmi355 as P
    import pcmi355._lib as L
    from pcmi355 import workloads
    from helpers import rel_err, assert_three_way
    O = oracle
    c2 = workloads.c2_config()
    V, K, C, B, data, parent = (c2[k] for k in ("V", "K", "C", "B", "data", "parent"))
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(c2["theta"], c2["leaf"])
    assert bpc.size("walk_kernels") == 3
    ch, _ = O.clt_children(parent)
    fc = O.hclt_flat(parent, K, C, {v: c2["theta"][v] for v in range(V) if ch[v]}, c2["leaf"])
    d = torch.from_numpy(data).cuda()
    sub = 128
    ids = np.arange(sub, dtype=np.int32)
    ll_ref, logp, leaf_new, ea_ref, lf_ref = O.em_step(fc, data, ids, 0.1, 0.9)
    ll = P.probs_flows_circuit(bpc, d[:sub].contiguous()).cpu().numpy()
    assert rel_err(ll, ll_ref).max() < LL_RTOL
    ea, lf = bpc.get_flows()
    for v, blk in O.hclt_block_aggr(fc, ea_ref).items():
        nk = blk.shape[0]
        assert np.abs(ea[v][:nk] - blk).max() < 2e-4 * max(blk.max(), 1e-3), f"edge_aggr block {v}"
    lf_ref = lf_ref.reshape(V, K, C)
    assert np.abs(lf - lf_ref).max() < 2e-4 * max(lf_ref.max(), 1e-3)
    L.check(L.lib.pcm_em_update(bpc.handle, 0.1, 0.9))
    th, lp = bpc.get_params()
    # updated parameters, three-way: with Dirichlet(1) parameters and 128 hidden states most leaf counts of 128
    # examples are tiny, and float32 flows (the reference's type) are themselves a little over 1e-4 from exact there
    def blocks(lg, lf_):
        new = fc.copy()
        new.logp, new.leaf_logp = lg, lf_
        return O.hclt_block_params(new)
    _, logp64, leaf64, _, _ = O.em_step(fc, data, ids, 0.1, 0.9, double=True)
    assert_three_way((th, lp), blocks(logp64, leaf64), blocks(logp, leaf_new), PARAM_RTOL, "C2, 128 examples")
    # the whole batch
    bpc.set_params(c2["theta"], c2["leaf"])
    ll_all = P.probs_flows_circuit(bpc, d).cpu().numpy()
    np.testing.assert_array_equal(ll_all[:sub], ll)
    ea, lf = bpc.get_flows()
    np.testing.assert_allclose(lf.sum(axis=(1, 2)), B, rtol=1e-4)
    inner = np.array([v for v in range(V) if ch[v]])
    np.testing.assert_allclose(ea[inner].sum(axis=(1, 2)), B, rtol=1e-4)
    assert (ea >= 0).all() and (lf >= 0).all()


def test_c4_forest_as_the_benchmark_builds_it(oracle):
    """The patch layer of the patch-clustered configuration exactly as `bench.py --workload c4_full` runs it: 64
    patch circuits (192 variables, K = 32, 128 cluster heads) as one forest handle over the 12288 pixels, four walk
    groups, one-hot cluster masks, batch 1024.  On the whole batch: every example sends one unit of flow through
    every variable, every tree node and the heads of every tree; four sampled trees give the bits of a handle of
    their own (likelihoods, flows, updated parameters, heads), and one of them matches the oracle on a subset."""
    import torch
    import pcmi355 as P
    from pcmi355 import workloads
    from pcmi355._lib import lib, check
    from helpers import rel_err
    O = oracle
    c4 = workloads.c4_config()
    V, K, C, H, B, NP = c4["V"], c4["K"], c4["C"], c4["H"], c4["B"], c4["patches"]
    forest = P.hclt_forest_from_clts(c4["fparent"], C, K, H)
    forest.set_params(c4["theta"], c4["leaf"])
    rng = np.random.default_rng(5)
    heads = np.log(rng.dirichlet(np.ones(K), size=(NP, H))).astype(np.float32)     # tree order
    forest.set_heads(heads)
    assert forest.num_trees == NP and forest.size("walk_kernels") == 1
    d = torch.from_numpy(c4["data"]).cuda()
    dmask = torch.from_numpy(c4["mask"]).cuda()
    mix_f = P.forest_flows(forest, d, dmask).cpu().numpy()
    assert mix_f.shape == (NP, B) and np.isfinite(mix_f).all()
    ea_f, lf_f = forest.get_flows()
    assert (ea_f >= 0).all() and (lf_f >= 0).all()
    np.testing.assert_allclose(lf_f.sum(axis=(1, 2)), B, rtol=1e-4)                 # every variable of every tree
    fparent = c4["fparent"]
    has_child = np.bincount(fparent[fparent >= 0], minlength=len(fparent)) > 0
    inner_not_root = has_child & (fparent >= 0)
    np.testing.assert_allclose(ea_f[inner_not_root].sum(axis=(1, 2)), B, rtol=1e-4)
    check(lib.pcm_em_update(forest.handle, 0.1, 0.9))
    th_f, leaf_f = forest.get_params()
    heads_f = forest.get_heads()
    np.testing.assert_allclose(np.exp(heads_f.astype(np.float64)).sum(-1), 1.0, rtol=1e-5)
    np.testing.assert_allclose(np.exp(leaf_f.astype(np.float64)).sum(-1), 1.0, rtol=1e-4)
    sampled = [0, 21, 42, 63]
    for t in sampled:
        p = int(c4["tree_patch"][t])
        pv, par = c4["pvars"][p], c4["parents"][p]
        c = P.multihead_hclt_from_clt(par, C, K, H)
        c.set_params(*c4["params"][p])
        c.set_heads(heads[t])
        dp = torch.from_numpy(np.ascontiguousarray(c4["data"][:, pv])).cuda()
        mix = P.probs_flows_circuit(c, dp, head_mask=torch.from_numpy(c4["mask"][t].T.copy()).cuda()).cpu().numpy()
        ea, lf = c.get_flows()
        check(lib.pcm_em_update(c.handle, 0.1, 0.9))
        th, lp = c.get_params()
        split = np.bincount(par[par >= 0]).max() > 3       # to the bit, or within rounding where a node is split
        cmp = np.testing.assert_array_equal if not split else (
            lambda a, b, err_msg="": np.testing.assert_allclose(a, b, rtol=2e-5, atol=2e-6 * max(1.0, float(np.abs(b).max())),
                                                                 err_msg=err_msg))
        cmp(mix_f[t], mix, err_msg=f"tree {t} mixture")
        cmp(ea_f[pv], ea, err_msg=f"tree {t} edge flows (split={split})")
        cmp(lf_f[pv], lf, err_msg=f"tree {t} leaf flows")
        cmp(th_f[pv], th, err_msg=f"tree {t} sum parameters")
        cmp(leaf_f[pv], lp, err_msg=f"tree {t} leaf parameters")
        cmp(heads_f[t], c.get_heads(), err_msg=f"tree {t} heads")
    # one tree against the oracle on a subset: the mixture likelihood under the one-hot mask is the
    # chosen head's value
    t = 21
    p = int(c4["tree_patch"][t])
    pv, par = c4["pvars"][p], c4["parents"][p]
    th0, lf0 = c4["params"][p]
    ch, root = O.clt_children(par)
    sub = 24
    heads_dag = []
    body = O.hclt_dag(par, K, C, {v: th0[v] for v in range(V) if ch[v]}, lf0)
    for h in range(H):
        heads_dag.append(O.summate(*body.children, logps=heads[t][h]))
    fc = O.bits_compile(O.summate(*heads_dag), C, V)
    mars = O.forward(fc, np.ascontiguousarray(c4["data"][:sub, pv]))
    n_heads_first = fc.n_nodes - 1 - H
    cl = c4["cluster"][:sub, p].astype(np.int64)
    want = mars[n_heads_first + cl, np.arange(sub)]
    assert rel_err(mix_f[t][:sub], want).max() < LL_RTOL
