"""Soft evidence (3-D log-evidence data): the oracle against what the mathematics fixes (CPU),
the HIP path against the oracle (GPU).
Reference: src/regularization/reg_likelihood.jl:51-91, src/regularization/reg_flow.jl:50-82."""
import itertools
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.join(ROOT, "lvd-pg_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import pc_oracle as O  # noqa: E402
from helpers import make_hclt, block_theta, random_dag, describe_dag  # noqa: E402


def _one_hot_evidence(data, C):
    ev = np.full(data.shape + (C,), -np.inf, np.float32)
    np.put_along_axis(ev, data[..., None].astype(np.int64), 0.0, axis=2)
    return ev


# ---- the oracle, pinned ------------------------------------------------------------------

def test_oracle_one_hot_evidence_is_hard_evidence():
    parent, theta, leaf, fc = make_hclt(6, 3, 4, 5)
    data = np.random.default_rng(0).integers(0, 4, (20, 6)).astype(np.uint8)
    ev = _one_hot_evidence(data, 4)
    m_hard = O.forward(fc, data, double=True)
    m_soft = O.forward_soft(fc, ev, double=True)
    assert np.allclose(m_soft, m_hard, rtol=0, atol=1e-12)
    fl, _ = O.backward(fc, m_hard, double=True)
    assert np.allclose(O.input_flows_soft(fc, ev, m_soft, fl, double=True), O.input_flows(fc, data, fl, double=True), atol=1e-12)


def test_oracle_soft_likelihood_is_the_weighted_sum_over_assignments():
    """LL_soft = log sum_x prod_v w[v, x_v] p(x): brute force over all assignments of a tiny circuit;
    all-zero evidence marginalises every variable: LL = 0."""
    V, C = 4, 3
    parent, theta, leaf, fc = make_hclt(V, 2, C, 9)
    rng = np.random.default_rng(1)
    ev = rng.normal(0, 1, (3, V, C))
    xs = np.array(list(itertools.product(range(C), repeat=V)), np.uint8)
    logp = O.forward(fc, xs, double=True)[-1]
    want = [np.log(np.sum(np.exp(logp + ev[b][np.arange(V), xs].sum(axis=1)))) for b in range(3)]
    got = O.forward_soft(fc, ev, double=True)[-1]
    assert np.allclose(got, want, atol=1e-10)
    assert np.allclose(O.forward_soft(fc, np.zeros((2, V, C)), double=True)[-1], 0, atol=1e-6)   # parameters are normalised in float32


def test_oracle_soft_leaf_flows_are_the_gradient_of_the_likelihood():
    """d LL / d logp_leaf[c] = the soft count of category c (central differences, float64)."""
    V, C = 4, 3
    parent, theta, leaf, fc = make_hclt(V, 2, C, 12)
    ev = np.random.default_rng(2).normal(0, 1, (5, V, C))
    mars = O.forward_soft(fc, ev, double=True)
    fl, _ = O.backward(fc, mars, double=True)
    counts = O.input_flows_soft(fc, ev, mars, fl, double=True)
    base = np.asarray(fc.leaf_logp, np.float64).copy()
    h = 1e-6
    for i in np.random.default_rng(3).choice(len(base), 12, replace=False):
        g = fc.copy()
        up, dn = base.copy(), base.copy()
        up[i] += h
        dn[i] -= h
        g.leaf_logp = up
        a = O.forward_soft(g, ev, double=True)[-1].sum()
        g.leaf_logp = dn
        b = O.forward_soft(g, ev, double=True)[-1].sum()
        assert abs((a - b) / (2 * h) - counts[i]) < 1e-6


# ---- the HIP path -------------------------------------------------------------------------

@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355
    return torch, pcmi355


LL_RTOL, FLOW_RTOL = 1e-5, 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("V,K,C,B,tree", [(7, 16, 5, 70, None), (9, 64, 128, 33, None), (6, 8, 4, 64, None), (5, 128, 6, 20, None),
                                          (11, 16, 6, 40, [-1, 0, 0, 0, 0, 0, 1, 2, 3, 4, 5])])   # a node the walks split
def test_hclt_soft_evidence_matches_oracle(gpu, V, K, C, B, tree):
    torch, P = gpu
    parent, theta, leaf, fc = make_hclt(V, K, C, 50 + V, parent=None if tree is None else np.array(tree, np.int32))
    rng = np.random.default_rng(V)
    ev = rng.normal(0, 2, (B, V, C)).astype(np.float32)
    ev[rng.random((B, V, C)) < 0.1] = -np.inf                # impossible categories
    ev[:, :, 0] = np.where(np.isinf(ev).all(axis=2), 0.0, ev[:, :, 0])
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    mars = O.forward_soft(fc, ev, double=True)
    d = torch.from_numpy(ev).cuda()
    ll = P.loglikelihoods(bpc, d).cpu().numpy()
    assert np.abs(ll - mars[-1]).max() < LL_RTOL * np.abs(mars[-1]).max()
    # Julia's layout: examples fastest
    dj = torch.from_numpy(np.ascontiguousarray(ev.transpose(2, 1, 0))).cuda().permute(2, 1, 0)
    assert np.array_equal(P.loglikelihoods(bpc, dj, batch_size=16).cpu().numpy(), ll)
    # flows and the EM update
    ll2 = P.probs_flows_circuit(bpc, d).cpu().numpy()
    assert np.array_equal(ll, ll2)
    fl, ea = O.backward(fc, mars, double=True)
    counts = O.input_flows_soft(fc, ev, mars, fl, double=True)
    ea_blk, lf_blk = bpc.get_flows()
    ref_ea = O.hclt_block_aggr(fc, ea)
    for v, blk in ref_ea.items():
        assert np.abs(ea_blk[v][:blk.shape[0]] - blk).max() < FLOW_RTOL * max(blk.max(), 1e-3)
    want = counts.reshape(V, K, C)                                       # the oracle's HCLT holds its leaves as [V][K][C]
    assert np.abs(lf_blk - want).max() < FLOW_RTOL * max(want.max(), 1e-3)
    np.testing.assert_allclose(lf_blk.sum(axis=(1, 2)), B, rtol=1e-4)      # every example passes every variable once
    import pcmi355._lib as L
    L.check(L.lib.pcm_em_update(bpc.handle, 0.1, 0.9))
    new_logp, new_leaf = O.em_update(fc, ea, counts, 0.1, 0.9, double=True)
    _, leaf_after = bpc.get_params()
    assert np.abs(np.exp(leaf_after) - np.exp(new_leaf.reshape(V, K, C))).max() < 5e-4 * np.exp(new_leaf).max()


@pytest.mark.gpu
@pytest.mark.parametrize("K", [16, 64])
def test_hclt_soft_evidence_far_from_the_favoured_category(gpu, K):
    """Evidence that favours, by 150 nats, a category some leaves all but forbid (log-probability
    -100 or -inf): the factored sums of the block kernels lose their footing there and the exact
    paths must take over.  Also example ids and the flow memory rate."""
    torch, P = gpu
    V, C, B = 6, 7, 50
    parent, theta, leaf, fc = make_hclt(V, K, C, 77)
    rng = np.random.default_rng(K)
    leaf = leaf.copy()
    hard = rng.random((V, K)) < 0.4
    leaf[hard, 0] = np.where(rng.random(hard.sum()) < 0.5, -100.0, -np.inf)
    leaf -= np.log(np.exp(leaf.astype(np.float64)).sum(-1, keepdims=True)).astype(np.float32)
    fc = O.hclt_flat(parent, K, C, theta, leaf)
    ev = rng.normal(-150, 3, (B, V, C)).astype(np.float32)
    ev[:, :, 0] = rng.normal(0, 1, (B, V))
    ev[rng.random((B, V)) < 0.3, 0] = -160.0                          # ... and examples where it does not
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    ids = rng.permutation(B)[:37].astype(np.int32)
    sub = np.ascontiguousarray(ev[ids])
    mars = O.forward_soft(fc, sub, double=True)
    d = torch.from_numpy(ev).cuda()
    ll = P.probs_flows_circuit(bpc, d, example_ids=ids).cpu().numpy()
    assert np.isfinite(mars[-1]).all()
    assert np.abs(ll - mars[-1]).max() < LL_RTOL * np.abs(mars[-1]).max()
    fl, ea = O.backward(fc, mars, double=True)
    counts = O.input_flows_soft(fc, sub, mars, fl, double=True).reshape(V, K, C)
    _, lf = bpc.get_flows()
    assert np.abs(lf - counts).max() < FLOW_RTOL * counts.max()
    np.testing.assert_allclose(lf.sum(axis=(1, 2)), len(ids), rtol=1e-4)
    P.probs_flows_circuit(bpc, d, example_ids=ids, rate=0.5)          # flow memory: half of the old statistics stay
    _, lf2 = bpc.get_flows()
    assert np.abs(lf2 - 1.5 * counts).max() < FLOW_RTOL * 1.5 * counts.max()


@pytest.mark.gpu
def test_general_circuit_soft_evidence_and_one_hot_limit(gpu):
    torch, P = gpu
    V, C, B = 8, 5, 90
    rng = np.random.default_rng(4)
    root = random_dag(V, C, rng, width=4)
    g = describe_dag([root])
    bpc = P.compile_circuit(g["node_type"], g["child_ptr"], g["child_idx"], g["sum_logp"], g["input_var"], g["input_logp"], V, C)
    fc = O.bits_compile(root, C, V)
    ev = rng.normal(0, 1.5, (B, V, C)).astype(np.float32)
    mars = O.forward_soft(fc, ev, double=True)
    d = torch.from_numpy(ev).cuda()
    ids = rng.permutation(B)[:37].astype(np.int32)
    ll = P.loglikelihoods(bpc, d, example_ids=ids).cpu().numpy()
    assert np.abs(ll - mars[-1][ids]).max() < LL_RTOL * np.abs(mars[-1]).max()
    # one-hot evidence gives exactly the categorical answer of the same engine
    data = rng.integers(0, C, (B, V)).astype(np.uint8)
    hard = P.loglikelihoods(bpc, torch.from_numpy(data).cuda()).cpu().numpy()
    soft = P.loglikelihoods(bpc, torch.from_numpy(_one_hot_evidence(data, C)).cuda()).cpu().numpy()
    np.testing.assert_allclose(soft, hard, rtol=1e-6)
    # EM on soft evidence raises the soft likelihood
    lls = P.mini_batch_em_with_reg(bpc, d, 4, batch_size=45, pseudocount=0.1, param_inertia=0.5, shuffle="none")
    assert lls[-1] > lls[0]


@pytest.mark.gpu
def test_top_level_circuit_shape(gpu):
    """The top-level circuit of the patch experiments: 64 variables (patches), 128 categories
    (clusters), K = 64, fed per-cluster patch log-likelihoods; oracle on a subset, then training."""
    torch, P = gpu
    V, K, C, B = 64, 64, 128, 512
    parent, theta, leaf, fc = make_hclt(V, K, C, 3)
    rng = np.random.default_rng(8)
    ev = (rng.normal(-600, 30, (B, V, 1)) + rng.gumbel(0, 8, (B, V, C))).astype(np.float32)   # patch LLs per cluster
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    d = torch.from_numpy(ev).cuda()
    ll = P.loglikelihoods(bpc, d, batch_size=256).cpu().numpy()
    want = O.forward_soft(fc, ev[:24], double=True)[-1]
    assert np.abs(ll[:24] - want).max() < LL_RTOL * np.abs(want).max()
    lls = P.mini_batch_em_with_reg(bpc, d, 3, batch_size=256, pseudocount=0.1, param_inertia=0.9, shuffle="none")
    assert lls[-1] > lls[0]


def _soft_ll_as_written(logp, x, s, width):
    """`soft_loglikelihood` of src/regularization/reg_likelihood.jl:4-14, line by line."""
    C = len(logp)
    c_start = max(0, x - width // 2)
    c_end = min(c_start + width - 1, C - 1)
    sp = sum(np.exp(logp[c]) for c in range(c_start, c_end + 1)) / (c_end - c_start + 1)
    return np.logaddexp(logp[x] + np.log(1 - s), np.log(sp) + np.log(s))


@pytest.mark.parametrize("C,width", [(7, 3), (7, 5), (4, 7), (9, 1)])
def test_soft_reg_is_soft_evidence(C, width):
    """soft_reg smoothing of categorical data (reg_likelihood.jl:4-14) is the soft evidence
    `soft_reg_evidence` builds: for every observed category, also at both ends of the range where the window
    is cut, log sum_c exp(ev[c]) p[c] equals the reference's leaf value worked out line by line; and the leaf
    flows of that evidence are the shares (1 - s) p[x] / base and s / n p[c] / base of `soft_flow_params`
    (src/nodes/fixable_categorical_dist.jl:141-160)."""
    import sys
    import torch
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lvd-pg_amd"))
    from pcmi355.queries import soft_reg_evidence
    rng = np.random.default_rng(C * 10 + width)
    s = 0.07
    logp = np.log(rng.dirichlet(np.ones(C)))
    rows = torch.arange(C, dtype=torch.uint8).view(C, 1)              # one variable, every category once
    ev = soft_reg_evidence(rows, C, s, width).numpy()[:, 0, :].astype(np.float64)
    for x in range(C):
        got = np.log(np.exp(ev[x] + logp).sum())
        assert abs(got - _soft_ll_as_written(logp, x, s, width)) < 1e-6
        c_start = max(0, x - width // 2)
        c_end = min(c_start + width - 1, C - 1)
        n = c_end - c_start + 1
        base = (1 - s) * np.exp(logp[x]) + s * np.exp(logp[c_start:c_end + 1]).sum() / n
        want = np.zeros(C)
        want[x] += (1 - s) * np.exp(logp[x]) / base
        want[c_start:c_end + 1] += s / n * np.exp(logp[c_start:c_end + 1]) / base
        share = np.exp(ev[x] + logp - got)
        np.testing.assert_allclose(share, want, rtol=1e-6, atol=1e-12)


@pytest.mark.gpu
def test_em_with_soft_reg_matches_oracle(gpu):
    """mini_batch_em_with_reg(...; soft_reg = 0.02, soft_reg_width = 5) as test/regularization/reg_em_tests.jl:20-21
    calls it: the likelihoods and the parameters after two batches against the oracle's EM on the evidence
    worked out line by line from reg_likelihood.jl:4-14."""
    torch, P = gpu
    V, K, C, B, s, width = 8, 16, 11, 48, 0.02, 5
    parent, theta, leaf, fc = make_hclt(V, K, C, 77)
    rng = np.random.default_rng(7)
    data = rng.integers(0, C, size=(2 * B, V)).astype(np.uint8)
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    lls = P.mini_batch_em_with_reg(bpc, torch.from_numpy(data).cuda(), 1, batch_size=B, pseudocount=0.01, soft_reg=s,
                                   soft_reg_width=width, param_inertia=0.9, shuffle="none")
    want_ll = []
    for b0 in (0, B):
        ev = np.full((B, V, C), -np.inf)
        for i in range(B):
            for v in range(V):
                x = int(data[b0 + i, v])
                c_start = max(0, x - width // 2)
                c_end = min(c_start + width - 1, C - 1)
                ev[i, v, c_start:c_end + 1] = np.log(s / (c_end - c_start + 1))
                ev[i, v, x] = np.log(np.exp(ev[i, v, x]) + 1 - s)
        mars = O.forward_soft(fc, ev.astype(np.float32), double=True)
        want_ll.append(mars[-1].mean())
        fl, ea = O.backward(fc, mars, double=True)
        counts = O.input_flows_soft(fc, ev.astype(np.float32), mars, fl, double=True)
        new_logp, new_leaf = O.em_update(fc, ea, counts, 0.01, 0.9, double=True)
        fc.logp, fc.leaf_logp = new_logp.astype(np.float32), new_leaf.astype(np.float32)
    assert abs(lls[0] - np.mean(want_ll)) < 1e-5 * abs(np.mean(want_ll))
    _, leaf_after = bpc.get_params()
    assert np.abs(np.exp(leaf_after) - np.exp(fc.leaf_logp.reshape(V, K, C))).max() < 5e-4 * np.exp(fc.leaf_logp).max()
    with pytest.raises(NotImplementedError):
        P.mini_batch_em_with_reg(bpc, torch.from_numpy(data).cuda(), 1, batch_size=B, pseudocount=0.01, ent_reg=0.1,
                                 param_inertia=0.9)


def _soft_reg_oracle_step(fc, batch, s, width, pseudocount, inertia, as_written):
    """One batch of mini_batch_em_with_reg with soft_reg on the float64 oracle: values and inner flows from the evidence
    worked out line by line, leaf statistics from `soft_flow` (reg_flow.jl:3-22) in the form asked for."""
    B, V = batch.shape
    C = fc.C
    ev = np.full((B, V, C), -np.inf)
    for i in range(B):
        for v in range(V):
            x = int(batch[i, v])
            c0 = max(0, x - width // 2)
            c1 = min(c0 + width - 1, C - 1)
            ev[i, v, c0:c1 + 1] = np.log(s / (c1 - c0 + 1))
            ev[i, v, x] = np.log(np.exp(ev[i, v, x]) + 1 - s)
    mars = O.forward_soft(fc, ev, double=True)
    fl, ea = O.backward(fc, mars, double=True)
    counts = O.soft_flow_counts(fc, batch, fl, s, width, as_written=as_written, double=True)
    new_logp, new_leaf = O.em_update(fc, ea, counts, pseudocount, inertia, double=True)
    return mars[-1], ea, counts, new_logp, new_leaf


@pytest.mark.gpu
@pytest.mark.parametrize("K,V,max_children,form", [(16, 9, 3, "as_written"), (16, 9, 3, "derivative"), (32, 12, 5, "as_written"),
                                                   (64, 7, 5, "as_written"), (128, 6, 3, "as_written"), (128, 6, 3, "derivative")])
def test_soft_reg_in_the_kernels_matches_oracle(gpu, K, V, max_children, form):
    """soft_reg smoothing inside the block kernels (pcm_set_soft_reg): likelihoods, sum-edge statistics and the leaf
    statistics in both forms -- `soft_flow` as written (reg_flow.jl:12-17, pinned by a hand-worked literal) and the
    derivative of the smoothed value -- and the parameters after two batches, against the float64 oracle; on the lean
    walks (K = 16), a tree whose wide nodes are split (K = 32, five children), the general statistics kernel (K = 64)
    and the wide kernels (K = 128).  Flow memory carries the first batch's statistics into the second."""
    torch, P = gpu
    from pcmi355._lib import lib, check
    C, B, s, width, pc, inertia = 13, 40, 0.05, 5, 0.02, 0.8
    parent, theta, leaf, fc = make_hclt(V, K, C, 31 + K, max_children=max_children)
    rng = np.random.default_rng(K)
    data = rng.integers(0, C, size=(2 * B, V)).astype(np.uint8)
    data[0, :] = 0
    data[1, :] = C - 1
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    d = torch.from_numpy(data).cuda()
    ll = torch.empty(B, device="cuda")
    print(f"soft_reg in kernels: K={K} V={V} form={form}", flush=True)
    check(lib.pcm_set_soft_reg(bpc.handle, s, width, int(form == "as_written")))
    # one batch: statistics against the oracle's
    check(lib.pcm_flows(bpc.handle, d.data_ptr(), d.stride(0), d.stride(1), None, B, 0.0, None, ll.data_ptr()))
    want_ll, want_ea, want_counts, _, _ = _soft_reg_oracle_step(fc, data[:B], s, width, pc, inertia, form == "as_written")
    np.testing.assert_allclose(ll.cpu().numpy(), want_ll, rtol=1e-5, atol=1e-5)
    _, leaf_flow = bpc.get_flows()                                         # [V, K, C]
    want = want_counts.reshape(V, K, C)
    assert np.abs(leaf_flow - want).max() < 2e-5 * np.abs(want).max(), np.abs(leaf_flow - want).max()
    check(lib.pcm_set_soft_reg(bpc.handle, 0.0, 1, 0))
    # the driver: two batches with flow memory, parameters against the oracle's
    lls = P.mini_batch_em_with_reg(bpc, d, 1, batch_size=B, pseudocount=pc, soft_reg=s, soft_reg_width=width,
                                   param_inertia=inertia, shuffle="none", flow_memory=0.0, soft_flow=form, soft_reg_route="kernels")
    want_lls = []
    for b0 in (0, B):
        wl, _, _, new_logp, new_leaf = _soft_reg_oracle_step(fc, data[b0:b0 + B], s, width, pc, inertia, form == "as_written")
        want_lls.append(wl.mean())
        fc.logp, fc.leaf_logp = new_logp.astype(np.float32), new_leaf.astype(np.float32)
    assert abs(lls[0] - np.mean(want_lls)) < 1e-5 * abs(np.mean(want_lls))
    _, leaf_after = bpc.get_params()
    want_leaf = fc.leaf_logp.reshape(V, K, C)
    assert np.abs(np.exp(leaf_after) - np.exp(want_leaf)).max() < 1e-4 * np.exp(want_leaf).max()
    # the smoothing is off again: plain likelihoods
    plain = P.loglikelihoods(bpc, d[:B]).cpu().numpy()
    mars = O.forward(fc, data[:B], double=True)
    np.testing.assert_allclose(plain, mars[-1], rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
def test_soft_reg_routes_agree_and_as_written_needs_the_kernels(gpu):
    """The kernel route and the soft-evidence route of mini_batch_em_with_reg(soft_reg > 0) train the same parameters
    (derivative form); a circuit without block kernels takes the evidence route by itself and refuses `as_written`."""
    torch, P = gpu
    V, K, C, B, s, width = 8, 16, 11, 48, 0.02, 5
    parent, theta, leaf, fc = make_hclt(V, K, C, 77)
    data = torch.from_numpy(np.random.default_rng(7).integers(0, C, size=(2 * B, V)).astype(np.uint8)).cuda()
    out = []
    for route in ("kernels", "evidence"):
        bpc = P.hclt_from_clt(parent, C, K)
        bpc.set_params(block_theta(parent, K, theta), leaf)
        lls = P.mini_batch_em_with_reg(bpc, data, 2, batch_size=B, pseudocount=0.01, soft_reg=s, soft_reg_width=width,
                                       param_inertia=0.9, shuffle="none", soft_reg_route=route)
        out.append((lls, bpc.get_params()))
    np.testing.assert_allclose(out[0][0], out[1][0], rtol=1e-5)
    np.testing.assert_allclose(np.exp(out[0][1][1]), np.exp(out[1][1][1]), rtol=2e-4, atol=1e-7)
    np.testing.assert_allclose(np.exp(out[0][1][0]), np.exp(out[1][1][0]), rtol=2e-4, atol=1e-7)
    parent5, theta5, leaf5, _ = make_hclt(6, 5, C, 3)
    odd = P.hclt_from_clt(parent5, C, 5)                                   # K = 5: no block kernels
    odd.set_params(block_theta(parent5, 5, theta5), leaf5)
    P.mini_batch_em_with_reg(odd, data[:, :6].contiguous(), 1, batch_size=B, pseudocount=0.01, soft_reg=s, soft_reg_width=width,
                             param_inertia=0.9, shuffle="none")
    with pytest.raises(Exception):
        P.mini_batch_em_with_reg(odd, data[:, :6].contiguous(), 1, batch_size=B, pseudocount=0.01, soft_reg=s,
                                 soft_reg_width=width, param_inertia=0.9, shuffle="none", soft_flow="as_written")


def _soft_reg_evidence_rows(batch, C, s, width):
    """The log-evidence of a categorical batch under soft_reg (reg_likelihood.jl:4-14), category by category."""
    B, V = batch.shape
    ev = np.full((B, V, C), -np.inf)
    for i in range(B):
        for v in range(V):
            x = int(batch[i, v])
            c0 = max(0, x - width // 2)
            c1 = min(c0 + width - 1, C - 1)
            ev[i, v, c0:c1 + 1] = np.log(s / (c1 - c0 + 1))
            ev[i, v, x] = np.log(np.exp(ev[i, v, x]) + 1 - s)
    return ev


@pytest.mark.gpu
@pytest.mark.parametrize("fscale,update_interval", [(2.0, 2), (0.7, 1)])
def test_em_beta_with_soft_reg_and_tempered_flows_matches_oracle(gpu, fscale, update_interval):
    """`mini_batch_em_beta(...; soft_reg, soft_reg_width, fscale)` with both at once (src-jl/learning/em.jl:366-368 ->
    flow.jl:366-372): the leaves take their smoothed values on the way up, the inner flows are those of the tempered
    posterior, the leaves share their flow out as `soft_flow_params` does -- replayed on the float64 oracle batch by
    batch.  `soft_flow = "as_written"` is the block kernels' form and is refused beside fscale != 1."""
    torch, P = gpu
    from helpers import correlated_data, rel_err
    V, K, C, B, nb, pc, inertia, s, width = 9, 16, 12, 48, 4, 0.1, 0.8, 0.05, 3
    parent, theta, leaf, fc = make_hclt(V, K, C, 21)
    data = correlated_data(B * nb, V, C, 22, parent)
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    lls = P.mini_batch_em_beta(bpc, torch.from_numpy(data).cuda(), 1, batch_size=B, pseudocount=pc, param_inertia=inertia,
                               shuffle="none", update_interval=update_interval, fscale=fscale, soft_reg=s,
                               soft_reg_width=width)
    cur, ea, lf, tot = fc.copy(), None, None, 0.0
    for batch_id in range(1, nb + 1):
        batch = data[(batch_id - 1) * B:batch_id * B]
        if ea is not None and batch_id % update_interval == 1:
            ea, lf = ea * 0.0, lf * 0.0                                     # flow_memory = 0
        mars = O.forward_soft(cur, _soft_reg_evidence_rows(batch, C, s, width), double=True)
        flows, ea_b = O.backward(cur, mars, double=True, fscale=fscale)
        lf_b = O.soft_flow_counts(cur, batch, flows, s, width, as_written=False, double=True)
        ea = ea_b if ea is None else ea + ea_b
        lf = lf_b if lf is None else lf + lf_b
        tot += mars[-1].sum()
        if batch_id % update_interval == 0:
            logp, new_leaf, ea = O.em_update(cur, ea, lf, pc, inertia, True, return_aggr=True)
            cur = cur.copy()
            cur.logp, cur.leaf_logp = logp.astype(np.float32), new_leaf.astype(np.float32)
    assert abs(lls[0] - tot / B / nb) < 2e-5 * abs(tot / B / nb)
    th_ref, leaf_ref = O.hclt_block_params(cur)
    th, lf_new = bpc.get_params()
    for v, blk in th_ref.items():
        assert rel_err(np.exp(th[v][:blk.shape[0]]), np.exp(blk)).max() < 5e-4
    assert rel_err(np.exp(lf_new), np.exp(leaf_ref)).max() < 5e-4
    with pytest.raises(NotImplementedError):
        P.mini_batch_em_beta(bpc, torch.from_numpy(data).cuda(), 1, batch_size=B, pseudocount=pc, param_inertia=inertia,
                             fscale=fscale, soft_reg=s, soft_reg_width=width, soft_flow="as_written")
    # the loop leaves the handle as it found it: an ordinary pass afterwards runs on the block kernels again
    ll = P.probs_flows_circuit(bpc, torch.from_numpy(data[:B]).cuda()).cpu().numpy()
    assert rel_err(ll, O.forward(cur, data[:B], double=True)[-1]).max() < 1e-4
