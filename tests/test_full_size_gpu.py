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
    # At this depth (114 tree levels, sub-circuit log-values of several thousand) float32 log-space
    # arithmetic itself is only good to ~1e-3 relative on the smallest flows: the float32 oracle,
    # i.e. the reference's arithmetic, misses the float64 result by that much on a few of the
    # 27 M parameters.  The library must be within 1e-4 of the float64 result or, where float32
    # cannot be, no further from it than twice the float32 oracle is.
    ids_np = np.arange(sub, dtype=np.int32)
    _, logp64, leaf64, _, _ = O.em_step(fc, cfg["data"], ids_np, 0.1, 0.9, double=True)
    _, logp32, leaf32, _, _ = O.em_step(fc, cfg["data"], ids_np, 0.1, 0.9)
    th, lf_new = bpc.get_params()

    def blocks(logp, leaf):
        new = fc.copy()
        new.logp, new.leaf_logp = logp, leaf
        return O.hclt_block_params(new)

    th64, lf64 = blocks(logp64, leaf64)
    th32, lf32 = blocks(logp32, leaf32)
    rel = lambda a, b: (np.abs(np.exp(np.asarray(a, np.float64)) - np.exp(b)) / np.exp(b)).max()
    e_gpu = max(rel(th[v][:b.shape[0]], b) for v, b in th64.items())
    e_f32 = max(rel(th32[v], b) for v, b in th64.items())
    e_gpu32 = max(rel(th[v][:b.shape[0]], th32[v].astype(np.float64)) for v, b in th64.items())
    print(f"sum parameters: library vs float64 {e_gpu:.2e}, float32 oracle vs float64 {e_f32:.2e}, "
          f"library vs float32 oracle {e_gpu32:.2e}")
    assert e_gpu < max(PARAM_RTOL, 2 * e_f32)
    # against the float32 oracle -- the reference's own arithmetic -- the two float32 results may be
    # apart by the sum of their distances from the exact one and no more
    assert e_gpu32 < max(PARAM_RTOL, e_gpu + e_f32)
    e_gpu, e_f32 = rel(lf_new, lf64), rel(lf32, lf64)
    e_gpu32 = rel(lf_new, lf32.astype(np.float64))
    print(f"leaf parameters: library vs float64 {e_gpu:.2e}, float32 oracle vs float64 {e_f32:.2e}, "
          f"library vs float32 oracle {e_gpu32:.2e}")
    assert e_gpu < max(PARAM_RTOL, 2 * e_f32)
    assert e_gpu32 < max(PARAM_RTOL, e_gpu + e_f32)
    # the per-example log-likelihoods of the step against the float32 oracle, at the bar itself
    ll32 = O.forward(fc, cfg["data"][:sub])[-1]
    assert (np.abs(llb.cpu().numpy() - ll32) / np.abs(ll32)).max() < LL_RTOL
    # (log-values near the root are ~ -14000, where one float32 ulp is 1e-3: a sizeable share of
    # the flows carries that error in any float32 implementation)
    frac = lambda a: (np.abs(np.exp(np.asarray(a, np.float64)) - np.exp(lf64)) / np.exp(lf64) > PARAM_RTOL).mean()
    f_gpu, f_f32 = frac(lf_new), frac(lf32)
    print(f"share of leaf parameters off by more than 1e-4: library {f_gpu:.3f}, float32 oracle {f_f32:.3f}")
    assert f_gpu < 1.5 * f_f32 + 1e-4
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
