"""GPU parity of the parameter-space queries (KL recursion and its gradient, Gumbel-max
sampling from supplied noise, Adam) against the CPU oracle and the reference tests' closed
forms, through the C ABI, on general circuits and on HCLTs."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

KLD_RTOL = 1e-4
GRAD_RTOL = 1e-4
ADAM_RTOL = 1e-5


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355
    return torch, pcmi355


def _compile(P, root, V, C):
    from helpers import describe_dag
    d = describe_dag([root])
    return P.compile_circuit(d["node_type"], d["child_ptr"], d["child_idx"], d["sum_logp"], d["input_var"],
                             d["input_logp"], V, C)


def _perturbed(params, C, n_sum, rng):
    """Another normalised parameter vector for the same structure (sum groups are passed in
    by the caller as whole-vector renormalisation is wrong: only the leaves are redrawn here)."""
    out = params.copy()
    leaves = out[n_sum:].reshape(-1, C)
    x = np.exp(leaves) * rng.uniform(0.5, 1.5, size=leaves.shape)
    out[n_sum:] = np.log(x / x.sum(axis=1, keepdims=True)).reshape(-1)
    return out.astype(np.float32)


def _grads_in_param_order(fc, eg, lg):
    pe = fc.sum_param_edges()
    leaf = [lg[fc.in_off[n]:fc.in_off[n] + fc.C] for n in fc.input_nodes()]
    return np.concatenate([eg[pe]] + leaf)


def test_kld_closed_forms_three_var_fixture(gpu):
    """test/queries/kld_tests.jl:9-70 and :106-131, one parameter row at a time."""
    torch, P = gpu
    from helpers import simple_3vars_circuit
    rng = np.random.default_rng(0)
    root = simple_3vars_circuit(5, rng, weights=[0.45, 0.55])
    p = _compile(P, root, 3, 5)
    q = _compile(P, root, 3, 5)
    pars = P.vectorize_parameters(p)
    assert len(pars) == 32
    assert abs(P.kld(p, q)) < 1e-7

    for (a, b) in [((0.2, 0.8), (0.4, 0.6)), ((0.5, 0.5), (0.9, 0.1))]:
        p1, p2 = pars.copy(), pars.copy()
        p1[:2] = np.log(np.float32(a))
        p2[:2] = np.log(np.float32(b))
        P.update_parameters(p, p1)
        P.update_parameters(q, p2)
        want = a[0] * np.log(a[0] / b[0]) + a[1] * np.log(a[1] / b[1])
        np.testing.assert_allclose(P.kld(p, q), want, rtol=1e-5)
        g1, g2 = P.kld_backward(p, q)
        np.testing.assert_allclose(g1[:2], [a[0] * (np.log(a[0]) - np.log(b[0]) + 1), a[1] * (np.log(a[1]) - np.log(b[1]) + 1)], rtol=1e-5)
        np.testing.assert_allclose(g2[:2], [-a[0], -a[1]], rtol=1e-6)

    for w, l1, l2 in [(0.2, [0.1, 0.2, 0.3, 0.2, 0.2], [0.2, 0.1, 0.1, 0.3, 0.3]),
                      (0.5, [0.1, 0.2, 0.3, 0.2, 0.2], [0.2, 0.1, 0.2, 0.3, 0.2])]:
        p1, p2 = pars.copy(), pars.copy()
        p1[:2] = p2[:2] = np.log(np.float32([w, 1 - w]))
        p1[2:7] = np.log(np.float32(l1))
        p2[2:7] = np.log(np.float32(l2))
        P.update_parameters(p, p1)
        P.update_parameters(q, p2)
        want = float(np.sum(np.exp(p1[2:7]) * (p1[2:7] - p2[2:7])) * w)
        np.testing.assert_allclose(P.kld(p, q), want, rtol=1e-4)

    # equal parameters: the gradient of the sum edges is +-exp(logp) (kld_tests.jl:101-108)
    P.update_parameters(p, pars)
    P.update_parameters(q, pars)
    g1, g2 = P.kld_backward(p, q)
    np.testing.assert_allclose(g1[:2], np.exp(pars[:2]), rtol=1e-6)
    np.testing.assert_allclose(g2[:2], -np.exp(pars[:2]), rtol=1e-6)


@pytest.mark.parametrize("V,C,width,seed", [(5, 4, 3, 0), (12, 7, 4, 1)])
def test_kld_and_gradient_match_oracle_random_dag(gpu, oracle, V, C, width, seed):
    torch, P = gpu
    O = oracle
    from helpers import random_dag, rel_err
    rng = np.random.default_rng(seed)
    root = random_dag(V, C, rng, width=width)
    fc1 = O.bits_compile(root, C, V)
    p = _compile(P, root, V, C)
    q = _compile(P, root, V, C)
    pars = P.vectorize_parameters(p)
    n_sum = p.num_inner_params()
    # second parameterisation: perturbed leaves, re-drawn sum weights per group
    p2 = _perturbed(pars, C, n_sum, rng)
    sizes = p.table("pargroup_sizes")
    pos = 0
    for s in sizes:
        w = rng.dirichlet(np.ones(s)) if s > 1 else np.ones(1)
        p2[pos:pos + s] = np.log(w)
        pos += s
    P.update_parameters(q, p2)
    fc2 = fc1.copy()
    fc2.update_parameters(p2)
    klds, ek = O.kld(fc1, fc2, double=True)
    got = P.kld(p, q)
    assert abs(got - klds[-1]) < KLD_RTOL * abs(klds[-1])
    _, eg1, eg2, lg1, lg2 = O.kld_backward(fc1, fc2, ek, double=True)
    g1, g2 = P.kld_backward(p, q)
    w1, w2 = _grads_in_param_order(fc1, eg1, lg1), _grads_in_param_order(fc1, eg2, lg2)
    assert np.abs(g1 - w1).max() < GRAD_RTOL * np.abs(w1).max()
    assert np.abs(g2 - w2).max() < GRAD_RTOL * np.abs(w2).max()


def _hclt_pair(P, O, V, K, C, seed, tree=None):
    from helpers import make_hclt, block_theta
    parent, theta, leaf, fc = make_hclt(V, K, C, seed, parent=None if tree is None else np.array(tree, np.int32))
    rng = np.random.default_rng(seed + 1)
    theta2, leaf2 = O.random_hclt_params(parent, K, C, rng)
    a = P.hclt_from_clt(parent, C, K)
    a.set_params(block_theta(parent, K, theta), leaf)
    b = P.hclt_from_clt(parent, C, K)
    b.set_params(block_theta(parent, K, theta2), leaf2)
    return parent, (theta, leaf), (theta2, leaf2), a, b


@pytest.mark.parametrize("V,K,C,tree", [
    (9, 16, 6, None), (30, 32, 70, None), (14, 64, 9, None), (40, 32, 256, None),
    (2, 16, 5, [-1, 0]),                                           # the root is the only tree node with a block
    (11, 16, 7, [-1, 0, 0, 0, 0, 0, 1, 2, 3, 4, 5]),               # five non-leaf children under one node
    (13, 32, 12, [-1, 0, 1, 1, 1, 1, 2, 3, 0, 8, 8, 8, 8]),
    (541, 64, 4, [-1] + [0] * 270 + list(range(1, 271))),          # a level too wide for the chains' LDS ring
    (9, 8, 6, None)])                                              # a hidden size without block kernels
def test_hclt_kld_and_gradient_match_oracle(gpu, oracle, V, K, C, tree):
    """KL recursion and its reverse pass on the block form (chains up and down the tree plus the
    data-parallel gradient kernels), against the oracle on the flattened DAG."""
    torch, P = gpu
    O = oracle
    parent, (t1, l1), (t2, l2), a, b = _hclt_pair(P, O, V, K, C, 31 + V, tree)
    fc1 = O.bits_compile(O.hclt_dag(parent, K, C, t1, l1), C, V)
    fc2 = O.bits_compile(O.hclt_dag(parent, K, C, t2, l2), C, V)
    klds, ek = O.kld(fc1, fc2, double=True)
    got = P.kld(a, b)
    assert got > 0 and abs(got - klds[-1]) < KLD_RTOL * abs(klds[-1])
    assert abs(P.kld(a, a)) < 1e-5
    _, eg1, eg2, lg1, lg2 = O.kld_backward(fc1, fc2, ek, double=True)
    g1, g2 = P.kld_backward(a, b)
    w1, w2 = _grads_in_param_order(fc1, eg1, lg1), _grads_in_param_order(fc1, eg2, lg2)
    assert np.abs(g1 - w1).max() < GRAD_RTOL * np.abs(w1).max()
    assert np.abs(g2 - w2).max() < GRAD_RTOL * np.abs(w2).max()
    d1, d2 = P.kld_backward(a, b, device=True)       # the same vectors left on the device
    assert np.array_equal(d1.cpu().numpy(), g1) and np.array_equal(d2.cpu().numpy(), g2)


def _gumbel(rng, shape):
    u = rng.random(shape)
    return (-np.log(-np.log(np.clip(u, 1e-12, 1 - 1e-12)))).astype(np.float32)


@pytest.mark.parametrize("V,C,width,B,seed", [(5, 4, 3, 100, 0), (12, 7, 4, 257, 1), (6, 256, 3, 64, 2)])
def test_sampling_bit_exact_random_dag(gpu, oracle, V, C, width, B, seed):
    torch, P = gpu
    O = oracle
    from helpers import random_dag
    rng = np.random.default_rng(seed)
    root = random_dag(V, C, rng, width=width)
    fc = O.bits_compile(root, C, V)
    bpc = _compile(P, root, V, C)
    n_sum = bpc.num_inner_params()
    node_noise = _gumbel(rng, (B, n_sum))
    leaf_noise = _gumbel(rng, (B, V, C))
    # oracle edges are in CSR order: slot of an edge = its parameter index
    slot = np.zeros(fc.n_edges, np.int64)
    slot[fc.sum_param_edges()] = np.arange(n_sum)
    want = O.sample(fc, node_noise, leaf_noise, noise_slot=slot)
    got = P.sample(bpc, torch.from_numpy(node_noise).cuda(), torch.from_numpy(leaf_noise).cuda()).cpu().numpy()
    assert got.dtype == np.uint8 and got.shape == (B, V)
    assert np.array_equal(got, want)
    assert (got < C).all()


@pytest.mark.parametrize("V,K,C,B,tree", [
    (7, 16, 8, 130, None), (12, 32, 256, 64, None), (10, 64, 5, 70, None), (9, 4, 6, 50, None), (6, 2, 3, 40, None),
    (6, 16, 36, 1030, None),                                     # three blocks of examples, the last one ragged
    (7, 128, 8, 45, None), (5, 128, 128, 20, None),              # K = 128: block sampler; 6 KB and 68 KB of leaf table in LDS
    (5, 64, 256, 70, None), (3, 128, 252, 30, None),             # 67 KB and 131 KB
    (141, 8, 3, 33, [-1] + [0] * 70 + list(range(1, 71))),       # a level of more than 64 tree nodes
    (13, 16, 6, 50, [-1, 0, 1, 1, 1, 1, 2, 3, 0, 8, 8, 8, 8]),   # four children twice: split for the walks, the noise
    (11, 32, 5, 40, [-1, 0, 0, 0, 0, 0, 1, 2, 3, 4, 5])])        # stays indexed by the caller's tree nodes
def test_sampling_bit_exact_hclt(gpu, oracle, V, K, C, B, tree):
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta
    parent, theta, leaf, fc = make_hclt(V, K, C, 5 + V, parent=None if tree is None else np.array(tree, np.int32))
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    ch, root = O.clt_children(parent)
    inner = [v for v in O.clt_bottom_up(parent) if ch[v]]
    rng = np.random.default_rng(V)
    node_noise = _gumbel(rng, (B, len(inner) * K))
    leaf_noise = _gumbel(rng, (B, V, C))
    slot = np.zeros(fc.n_edges, np.int64)
    for r, v in enumerate(inner):
        nk = len(fc.meta["sum_node"][v])
        e0 = fc.meta["edge_of"][v]
        slot[e0:e0 + nk * K] = np.tile(r * K + np.arange(K), nk)
    want = O.sample(fc, node_noise, leaf_noise, noise_slot=slot)
    got = P.sample(bpc, torch.from_numpy(node_noise).cuda(), torch.from_numpy(leaf_noise).cuda()).cpu().numpy()
    assert np.array_equal(got, want)


def test_sampling_follows_the_circuit_distribution(gpu, oracle):
    """With Gumbel noise the samples are exact draws: empirical frequencies of the joint on a
    tiny circuit approach the circuit's probabilities."""
    torch, P = gpu
    O = oracle
    import itertools
    from helpers import random_dag
    V, C, B = 3, 3, 60000
    rng = np.random.default_rng(9)
    root = random_dag(V, C, rng, width=2)
    fc = O.bits_compile(root, C, V)
    bpc = _compile(P, root, V, C)
    allx = np.array(list(itertools.product(range(C), repeat=V)), np.uint8)
    prob = np.exp(O.forward(fc, allx, double=True)[-1])
    g = torch.Generator(device="cuda").manual_seed(1)
    u1 = torch.rand((B, bpc.num_inner_params()), device="cuda", generator=g).clamp_(1e-10, 1 - 1e-7)
    u2 = torch.rand((B, V, C), device="cuda", generator=g).clamp_(1e-10, 1 - 1e-7)
    s = P.sample(bpc, -torch.log(-torch.log(u1)), -torch.log(-torch.log(u2))).cpu().numpy().astype(np.int64)
    code = (s * (C ** np.arange(V - 1, -1, -1))).sum(axis=1)
    freq = np.bincount(code, minlength=C ** V) / B
    assert np.abs(freq - prob).max() < 5 * np.sqrt(prob.max() / B) + 1e-3


def test_adam_step_matches_oracle(gpu, oracle):
    """src/sgd/adam.jl:318-319, :63-76, :88-127 on an HCLT and on a general circuit."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta, random_dag, rel_err
    V, C = 6, 5
    hcs = []
    for K in (16, 32, 64, 128, 8):
        parent, theta, leaf, fc = make_hclt(V, K, C, 41)
        hc = P.hclt_from_clt(parent, C, K)
        hc.set_params(block_theta(parent, K, theta), leaf)
        hcs.append(hc)
    hc = hcs[0]
    gc = _compile(P, random_dag(8, 4, np.random.default_rng(3), width=4), 8, 4)
    for bpc in (*hcs, gc):
        n_sum = bpc.num_inner_params()
        rng = np.random.default_rng(n_sum)
        before = P.vectorize_parameters(bpc)
        params = before[:n_sum].copy() + rng.normal(0, 0.1, n_sum).astype(np.float32)
        m = rng.normal(0, 0.01, n_sum).astype(np.float32)
        v = (rng.random(n_sum) * 1e-3).astype(np.float32)
        sizes = bpc.table("pargroup_sizes")
        group_ptr = np.concatenate([[0], np.cumsum(sizes)])
        dp, dm, dv = (torch.from_numpy(x.copy()).cuda() for x in (params, m, v))
        rp, rm, rv = params.copy(), m.copy(), v.copy()
        logp_ref = before[:n_sum].copy()
        for t in (1, 2, 3):
            grad = rng.normal(0, 1, n_sum).astype(np.float32)
            P.adam_step(bpc, torch.from_numpy(grad).cuda(), dp, dm, dv, lr=1e-2, t=t)
            O.adam_step(rp, grad, rm, rv, 1e-2, 0.9, 0.999, 1e-8, t, group_ptr, logp_ref)
        np.testing.assert_allclose(dp.cpu().numpy(), rp, rtol=ADAM_RTOL, atol=1e-6)
        np.testing.assert_allclose(dm.cpu().numpy(), rm, rtol=ADAM_RTOL, atol=1e-7)   # sums of terms ~0.1 that may cancel
        np.testing.assert_allclose(dv.cpu().numpy(), rv, rtol=ADAM_RTOL, atol=1e-10)
        after = P.vectorize_parameters(bpc)
        assert rel_err(np.exp(after[:n_sum]), np.exp(logp_ref)).max() < 1e-5
        assert np.array_equal(after[n_sum:], before[n_sum:])        # leaves untouched
        # every sum node with more than one edge is normalised
        pos = 0
        for s in sizes:
            if s > 1:
                assert abs(np.exp(after[pos:pos + s].astype(np.float64)).sum() - 1) < 1e-5
            pos += s
    # the dense engine sees the new parameters too
    th, _ = hc.get_params()
    ch, root = O.clt_children(parent)
    v0 = next(v for v in range(V) if ch[v] and v != root)
    assert np.abs(np.exp(th[v0].astype(np.float64)).sum(axis=1) - 1).max() < 1e-5
    # ... in its likelihood kernels as well: a fresh circuit loaded with the same vector agrees
    data = torch.from_numpy(np.random.default_rng(5).integers(0, C, (48, V)).astype(np.uint8)).cuda()
    for h in hcs:
        fresh = P.hclt_from_clt(parent, C, h.num_hidden_cats)
        P.update_parameters(fresh, P.vectorize_parameters(h))
        np.testing.assert_allclose(P.loglikelihoods(h, data, batch_size=48).cpu().numpy(),
                                   P.loglikelihoods(fresh, data, batch_size=48).cpu().numpy(), rtol=1e-6)


@pytest.mark.parametrize("temperature", [1.0, 0.4])
def test_relaxed_sampling_matches_oracle(gpu, oracle, temperature):
    """Soft top-down pass (src/queries/sample.jl:37-51, :105-140, :262-284) with supplied noise
    on a DAG with shared sub-circuits and on an HCLT, row by row against the oracle; invariants
    of test/queries/sample_tests.jl:34-53."""
    torch, P = gpu
    O = oracle
    from helpers import random_dag, make_hclt, block_theta
    rng = np.random.default_rng(17)
    V, C, B = 7, 5, 6
    root = random_dag(V, C, rng, width=3)
    fc = O.bits_compile(root, C, V)
    bpc = _compile(P, root, V, C)
    n_sum = bpc.num_inner_params()
    noise = _gumbel(rng, (B, n_sum))
    out = P.gumbel_sample(bpc, B, temperature=temperature, node_noise=torch.from_numpy(noise).cuda()).cpu().numpy()
    assert out.shape == (B, V, C)
    np.testing.assert_allclose(out.sum(axis=2), 1.0, rtol=1e-4)
    pe = fc.sum_param_edges()
    for b in range(B):
        g = np.zeros(fc.n_edges, np.float64)
        g[pe] = noise[b]
        _, want = O.gumbel_soft(fc, g, temperature, double=True)
        np.testing.assert_allclose(out[b], want, rtol=1e-4, atol=1e-7)
    # no noise, temperature 1: the circuit's marginals
    import itertools
    allx = np.array(list(itertools.product(range(C), repeat=V)), np.uint8)
    p = np.exp(O.forward(fc, allx, double=True)[-1])
    plain = P.gumbel_sample(bpc, 2, temperature=1.0).cpu().numpy()
    for v in range(V):
        marg = np.array([p[allx[:, v] == c].sum() for c in range(C)])
        np.testing.assert_allclose(plain[0, v], marg, rtol=1e-4)
    assert np.array_equal(plain[0], plain[1])

    # HCLT: the K sum nodes of a tree node share the noise column of each hidden state.  Block
    # sizes run on the block form (two matrix contractions per tree node and 16 examples), other
    # sizes on the layered engine.
    star = np.array([-1, 0, 0, 0, 0, 0, 1, 2, 3, 4, 5], np.int32)    # five non-leaf children: split for the walks
    for Vh, K, Ch, Bh, tree in ((6, 16, 4, 3, None), (11, 32, 256, 37, None), (9, 64, 10, 16, None), (5, 8, 4, 3, None),
                                (7, 16, 200, 20, None), (6, 32, 20, 33, None),   # category tiles left out past C; a partial tile of whole words
                                (11, 16, 5, 9, star)):
        parent, theta, leaf, flat = make_hclt(Vh, K, Ch, 23 + K, parent=tree)
        h = P.hclt_from_clt(parent, Ch, K)
        h.set_params(block_theta(parent, K, theta), leaf)
        ch, _ = O.clt_children(parent)
        inner = [v for v in O.clt_bottom_up(parent) if ch[v]]
        hn = _gumbel(rng, (Bh, len(inner) * K))
        got = P.gumbel_sample(h, Bh, temperature=temperature, node_noise=torch.from_numpy(hn).cuda()).cpu().numpy()
        np.testing.assert_allclose(got.sum(axis=2), 1.0, rtol=1e-4)
        for b in range(Bh):
            g = np.zeros(flat.n_edges, np.float64)
            for r, v in enumerate(inner):
                nk = len(flat.meta["sum_node"][v])
                e0 = flat.meta["edge_of"][v]
                g[e0:e0 + nk * K] = np.tile(hn[b, r * K:(r + 1) * K], nk)
            _, want = O.gumbel_soft(flat, g, temperature, double=True)
            np.testing.assert_allclose(got[b], want, rtol=2e-4, atol=1e-7)
        # without noise at temperature 1: the marginals of the circuit, whatever the engine
        _, marg = O.gumbel_soft(flat, None, 1.0, double=True)
        plain = P.gumbel_sample(h, 2, temperature=1.0).cpu().numpy()
        np.testing.assert_allclose(plain[0], marg, rtol=2e-4, atol=1e-7)
        # a temperature below the block form's range takes the layered engine: same answer
        cold = P.gumbel_sample(h, 2, temperature=0.15, node_noise=torch.from_numpy(hn[:2].copy()).cuda()).cpu().numpy()
        for b in range(2):
            g = np.zeros(flat.n_edges, np.float64)
            for r, v in enumerate(inner):
                nk = len(flat.meta["sum_node"][v])
                e0 = flat.meta["edge_of"][v]
                g[e0:e0 + nk * K] = np.tile(hn[b, r * K:(r + 1) * K], nk)
            _, want = O.gumbel_soft(flat, g, 0.15, double=True)
            np.testing.assert_allclose(cold[b], want, rtol=1e-3, atol=1e-6)


def _row_oracle(O, fc, row, n_sum, norm):
    """The oracle circuit whose parameters are one row of a parameter matrix (with norm the leaf
    part of the row holds probabilities, which the oracle's leaf array then holds as they are)."""
    f = fc.copy()
    f.logp = f.logp.astype(np.float64)
    f.leaf_logp = f.leaf_logp.astype(np.float64)
    f.update_parameters(row.astype(np.float64))
    return f


@pytest.mark.parametrize("kind,R,norm", [("hclt", 1, False), ("hclt", 7, True), ("hclt", 64, False), ("dag", 7, False),
                                         ("dag", 64, True), ("hclt64", 5, True), ("hclt_c8", 7, False), ("hclt_c8", 33, True),
                                         ("hclt32_c12", 5, False), ("hclt64_c4", 3, True)])
def test_parameter_row_queries_match_oracle(gpu, oracle, kind, R, norm):
    """`kld`, `kld_backward` and `gumbel_sample` on a matrix of parameter rows (src/queries/kld.jl:164-206,
    :593-649, src/queries/sample.jl:338-383), all rows in one pass, log-parameters and probability-valued
    leaves (norm_params), row-major and column-major matrices: every row against the oracle on that row's
    parameters.  Tolerances: 1e-4 of the KL, 1e-4 of the largest gradient entry, 1e-4 on the soft samples."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta, random_dag, log_dirichlet
    rng = np.random.default_rng(100 + R)
    if kind.startswith("hclt"):
        # (category counts divisible by 4: the KL gradient of the rows also runs on the block kernels)
        V, K, C = {"hclt64": (9, 64, 5), "hclt": (13, 16, 6), "hclt_c8": (13, 16, 8), "hclt32_c12": (21, 32, 12),
                   "hclt64_c4": (7, 64, 4)}[kind]
        parent, theta, leaf, _ = make_hclt(V, K, C, 61)
        bpc = P.hclt_from_clt(parent, C, K)
        fc = O.bits_compile(O.hclt_dag(parent, K, C, theta, leaf), C, V)
    else:
        V, C = 8, 5
        root = random_dag(V, C, rng, width=3)
        bpc = _compile(P, root, V, C)
        fc = O.bits_compile(root, C, V)
    n, ns = bpc.num_parameters(), bpc.num_inner_params()
    sizes = bpc.table("pargroup_sizes")

    def draw_rows():
        rows = np.empty((R, n), np.float32)
        for r in range(R):
            pos = 0
            for sz in sizes:
                rows[r, pos:pos + sz] = log_dirichlet(rng, sz) if sz > 1 else 0.0
                pos += sz
            lf = np.exp(np.stack([log_dirichlet(rng, C) for _ in range((n - ns) // C)]))
            rows[r, ns:] = (lf if norm else np.log(lf)).reshape(-1)
        return rows

    p1, p2 = draw_rows(), draw_rows()
    want_kl, want_g1, want_g2 = [], [], []
    for r in range(R):
        f1, f2 = _row_oracle(O, fc, p1[r], ns, norm), _row_oracle(O, fc, p2[r], ns, norm)
        klds, ek = O.kld(f1, f2, double=True, norm_params=norm)
        _, eg1, eg2, lg1, lg2 = O.kld_backward(f1, f2, ek, double=True, norm_params=norm)
        want_kl.append(klds[-1])
        want_g1.append(_grads_in_param_order(fc, eg1, lg1))
        want_g2.append(_grads_in_param_order(fc, eg2, lg2))
    want_kl, want_g1, want_g2 = np.array(want_kl), np.stack(want_g1), np.stack(want_g2)
    # host matrices (row-major on the device)
    got = P.kld(bpc, p1, p2, norm_params=norm)
    assert got.shape == (R,) and np.abs(got - want_kl).max() < KLD_RTOL * np.abs(want_kl).max()
    g1, g2 = P.kld_backward(bpc, p1, p2, norm_params=norm)
    assert g1.shape == (R, n)
    assert np.abs(g1 - want_g1).max() < GRAD_RTOL * np.abs(want_g1).max()
    assert np.abs(g2 - want_g2).max() < GRAD_RTOL * np.abs(want_g2).max()
    # column-major device matrices, as Julia holds [rows, n]: same numbers, gradients come back in that layout
    t1 = torch.from_numpy(np.ascontiguousarray(p1.T)).cuda().t()
    t2 = torch.from_numpy(np.ascontiguousarray(p2.T)).cuda().t()
    assert R == 1 or t1.stride() == (1, R)
    np.testing.assert_array_equal(P.kld(bpc, t1, t2, norm_params=norm).cpu().numpy(), got)
    c1, c2 = P.kld_backward(bpc, t1, t2, norm_params=norm)
    assert R == 1 or c1.stride() == (1, R)
    np.testing.assert_array_equal(c1.cpu().numpy(), g1)
    np.testing.assert_array_equal(c2.cpu().numpy(), g2)
    # relaxed samples: one draw of noise per row and sum edge
    for T, with_noise in ((1.0, False), (0.6, True)):
        noise = _gumbel(rng, (R, ns)) if with_noise else None
        soft = P.gumbel_sample_rows(bpc, p1, temperature=T, noise=noise, norm_params=norm)
        assert soft.shape == (R, V, C)
        pe = fc.sum_param_edges()
        for r in range(0, R, max(1, R // 5)):
            f1 = _row_oracle(O, fc, p1[r], ns, norm)
            g = None
            if with_noise:
                g = np.zeros(fc.n_edges)
                g[pe] = noise[r]
            _, want = O.gumbel_soft(f1, g, T, double=True, norm_params=norm)
            np.testing.assert_allclose(soft[r], want, rtol=1e-4, atol=1e-7)
        # and back (src/queries/sample.jl:389-650): gradients of sum(soft * G) w.r.t. every parameter row,
        # per log-parameter and per probability (grad_wrt_logparams), row- and column-major
        G = rng.normal(size=(R, V, C)).astype(np.float32)
        for wrt_log in (True, False):
            back = P.gumbel_sample_backward_rows(bpc, p1, G, temperature=T, noise=noise, norm_params=norm,
                                                 grad_wrt_logparams=wrt_log)
            assert back.shape == (R, n)
            for r in range(0, R, max(1, R // 5)):
                f1 = _row_oracle(O, fc, p1[r], ns, norm)
                g = None
                if with_noise:
                    g = np.zeros(fc.n_edges)
                    g[pe] = noise[r]
                eg, lg = O.gumbel_soft_backward(f1, g, T, G[r], double=True, norm_params=norm, grad_wrt_logparams=wrt_log)
                want = _grads_in_param_order(fc, eg, lg)
                assert np.abs(back[r] - want).max() < GRAD_RTOL * np.abs(want).max(), (T, wrt_log, r)
        tb = P.gumbel_sample_backward_rows(bpc, t1, torch.from_numpy(G).cuda(), temperature=T,
                                           noise=None if noise is None else torch.from_numpy(noise).cuda(), norm_params=norm,
                                           grad_wrt_logparams=False)
        assert R == 1 or tb.stride() == (1, R)
        np.testing.assert_array_equal(tb.cpu().numpy(), back)
    # the circuit lends its structure only: its own parameters were not read or touched
    with pytest.raises(P.PcmError):
        P._lib.check(P._lib.lib.pcm_kld_rows(bpc.handle, None, None, n, 1, R, 0, None))


def test_prealloc_wrappers_run_all_rows_at_once(gpu, oracle):
    """`kld_with_prealloc`, `kld_backward_with_prealloc`, `gumbel_sample_with_prealloc`
    (src/utils/cuda_preallocation.jl:47-78,189-203) with one parameter vector per example and the
    arguments src/models/pc_vae.py:81-92 passes (norm_params = True for the sampler, a repeated prior
    for the KL), against the single-vector queries and the oracle."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta
    W = P.prealloc
    V, K, C, R = 6, 16, 5, 3
    parent, theta, leaf, fc = make_hclt(V, K, C, 31)
    bpc = P.hclt_from_clt(parent, C, K)
    bpc.set_params(block_theta(parent, K, theta), leaf)
    base = P.vectorize_parameters(bpc)
    rows1, rows2, fcs = [], [], []
    for r in range(R + 1):
        _, th, lf, f = make_hclt(V, K, C, 40 + r, parent=parent)
        c = P.hclt_from_clt(parent, C, K)
        c.set_params(block_theta(parent, K, th), lf)
        (rows2 if r == R else rows1).append(P.vectorize_parameters(c))
        fcs.append(f)
    p1, prior = np.stack(rows1), np.stack(rows2)
    with pytest.raises(RuntimeError):
        W.kld_with_prealloc(bpc, p1, prior)
    W.kld_preallocation(bpc, num_examples=R)
    klds = W.kld_with_prealloc(bpc, p1, prior)
    want = [O.kld(fcs[r], fcs[R], double=True)[0][-1] for r in range(R)]
    np.testing.assert_allclose(klds, want, rtol=KLD_RTOL)
    np.testing.assert_array_equal(P.vectorize_parameters(bpc), base)          # the circuit's own parameters come back
    g1, g2 = W.kld_backward_with_prealloc(bpc)
    assert g1.shape == g2.shape == p1.shape
    q = P.hclt_from_clt(parent, C, K)
    P.update_parameters(q, prior[0])
    P.update_parameters(bpc, p1[1])
    e1, e2 = P.kld_backward(bpc, q)
    P.update_parameters(bpc, base)
    np.testing.assert_allclose(g1[1], e1, rtol=1e-4, atol=1e-6)              # two engines: block chains / lane groups
    np.testing.assert_allclose(g2[1], e2, rtol=1e-4, atol=1e-6)
    with pytest.raises(ValueError):
        W.kld_with_prealloc(bpc, p1[:2], prior)                                # not the preallocated number of rows
    W.kld_free_mem()
    W.gumbel_sample_preallocation(bpc, num_examples=R, num_vars=V, par_buffer_size=C + 2)
    soft = W.gumbel_sample_with_prealloc(bpc, p1, temperature=1.0, no_gumbel=True)
    assert soft.shape == (R, V, C + 2) and np.all(soft[:, :, C:] == 0)
    np.testing.assert_allclose(soft.sum(-1), 1.0, rtol=1e-4)                   # a distribution per variable
    P.update_parameters(bpc, p1[2])
    direct = P.gumbel_sample(bpc, 1, temperature=1.0)[0].cpu().numpy()
    P.update_parameters(bpc, base)
    np.testing.assert_allclose(soft[2, :, :C], direct, rtol=1e-4, atol=1e-7)
    noisy = W.gumbel_sample_with_prealloc(bpc, p1, temperature=0.5, generator=torch.Generator(device="cuda").manual_seed(3))
    np.testing.assert_allclose(noisy.sum(-1), 1.0, rtol=1e-4)
    # what pc_vae.py:81-86 asks for: probability-valued leaves, no noise
    ns = bpc.num_inner_params()
    probs = p1.copy()
    probs[:, ns:] = np.exp(p1[:, ns:])
    as_vae = W.gumbel_sample_with_prealloc(bpc, probs, temperature=1.0, norm_params=True, no_gumbel=True)
    np.testing.assert_allclose(as_vae, soft, rtol=1e-5, atol=1e-7)
    with pytest.raises(RuntimeError):                                          # allocate_for_grad was not asked for
        W.gumbel_sample_backward_with_prealloc(bpc, np.zeros((R, V, C + 2), np.float32), temperature=1.0)
    W.gumbel_sample_free_mem()
    # the reverse pass through the wrappers (src/utils/cuda_preallocation.jl:205-218): central differences of
    # sum(soft * G) in float32 along a few sum parameters of row 1
    W.gumbel_sample_preallocation(bpc, num_examples=R, num_vars=V, par_buffer_size=C + 2, allocate_for_grad=True)
    G = np.random.default_rng(5).normal(size=(R, V, C + 2)).astype(np.float32)
    W.gumbel_sample_with_prealloc(bpc, probs, temperature=0.8, norm_params=True, no_gumbel=True)
    back = W.gumbel_sample_backward_with_prealloc(bpc, G, temperature=0.8, norm_params=True)
    assert back.shape == probs.shape
    for i in (0, 7, ns - 3):
        vals = []
        for h in (1e-2, -1e-2):
            q = probs.copy()
            q[1, i] += h
            vals.append(float((W.gumbel_sample_with_prealloc(bpc, q, temperature=0.8, norm_params=True, no_gumbel=True)[1] * G[1]).sum()))
        fd = (vals[0] - vals[1]) / 2e-2
        assert abs(back[1, i] - fd) < 2e-3 * max(1.0, abs(fd)), (i, back[1, i], fd)
    W.gumbel_sample_free_mem()
    # pc_vae.py:88-92: the prior repeated for every row
    W.kld_preallocation(bpc, num_examples=R)
    np.testing.assert_allclose(W.kld_with_prealloc(bpc, p1, np.repeat(prior, R, axis=0)), klds, rtol=1e-6)
    W.kld_free_mem()
    np.testing.assert_array_equal(P.vectorize_parameters(bpc), base)


def test_misaligned_noise_is_refused(gpu, oracle):
    """The block samplers read noise rows as 16-byte words: a pointer that is not 16-byte
    aligned is an argument error, not a launch."""
    torch, P = gpu
    from helpers import make_hclt, block_theta
    V, K, C, B = 6, 16, 8, 5
    parent, theta, leaf, _ = make_hclt(V, K, C, 3)
    h = P.hclt_from_clt(parent, C, K)
    h.set_params(block_theta(parent, K, theta), leaf)
    need = int(P._lib.lib.pcm_sample_noise_size(h.handle))
    flat = torch.zeros(B * need + 4, device="cuda")
    leafn = torch.zeros((B, V, C), device="cuda")
    shifted = flat[1:1 + B * need].view(B, need)            # contiguous, 4 bytes past an aligned address
    assert shifted.data_ptr() % 16 != 0
    with pytest.raises(P.PcmError):
        P.sample(h, shifted, leafn)
    with pytest.raises(P.PcmError):
        P.gumbel_sample(h, B, temperature=0.7, node_noise=shifted)
    aligned = flat[:B * need].view(B, need)
    assert P.sample(h, aligned, leafn).shape == (B, V)


@pytest.mark.parametrize("kind", ["hclt16", "hclt64", "hclt128", "hclt8", "dag", "star32"])
def test_adam_from_flows_matches_oracle(gpu, oracle, kind):
    """`compute_gradients` and the `adam` loop's step (src/sgd/adam.jl:27-61, :218-242, :305-325) on the block
    engines (lean / general walks, wide blocks), on a hidden size without block kernels and on a DAG: the
    gradient vector, then three steps of the sum parameters' and the input nodes' optimiser state, against
    the oracle.  Tolerance 1e-4 (gradient: of its largest entry)."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta, random_dag, correlated_data
    from pcmi355._lib import lib, check
    rng = np.random.default_rng(7)
    B = 50
    if kind == "dag":
        V, C = 7, 5
        root = random_dag(V, C, rng, width=3)
        bpc = _compile(P, root, V, C)
        fc = O.bits_compile(root, C, V)
        data = rng.integers(0, C, (B, V)).astype(np.uint8)
    else:
        K = int(kind[4:])
        V, C = 9, 6
        # star: a root with five non-leaf children, which the walk kernels split
        tree = np.array([-1, 0, 0, 0, 0, 0, 1, 2, 3, 4, 5], np.int32) if kind.startswith("star") else None
        V = V if tree is None else len(tree)
        parent, theta, leaf, _ = make_hclt(V, K, C, 17, parent=tree)
        bpc = P.hclt_from_clt(parent, C, K)
        bpc.set_params(block_theta(parent, K, theta), leaf)
        fc = O.bits_compile(O.hclt_dag(parent, K, C, theta, leaf), C, V)
        data = correlated_data(B, V, C, 18, parent)
    np.testing.assert_allclose(P.vectorize_parameters(bpc), fc.vectorize_parameters(), atol=1e-6)
    d = torch.from_numpy(data).cuda()
    ns, nl = bpc.num_inner_params(), bpc.num_input_params()
    pe = fc.sum_param_edges()
    sizes = bpc.table("pargroup_sizes")
    gp = np.concatenate([[0], np.cumsum(sizes)])
    # optimiser state on both sides
    params = fc.logp[pe].astype(np.float32).copy()
    m, v = np.zeros(ns, np.float32), np.zeros(ns, np.float32)
    aux_p = fc.leaf_logp.astype(np.float32).copy()      # the oracle keeps leaves in input-node order = parameter order
    aux_m, aux_v = np.zeros(nl, np.float32), np.zeros(nl, np.float32)
    dp, dm, dv = (torch.from_numpy(x.copy()).cuda() for x in (params, m, v))
    lp, lm, lv = (torch.from_numpy(x.copy()).cuda() for x in (aux_p, aux_m, aux_v))
    lr = 2e-2
    leaves_before = P.vectorize_parameters(bpc)[ns:].copy()
    for t in range(1, 4):
        P.probs_flows_circuit(bpc, d)
        mars = O.forward(fc, data)
        flows, ea = O.backward(fc, mars)
        lf = O.input_flows(fc, data, flows)
        want_grad = O.flow_gradients(fc, ea, B)[pe]
        got_grad = P.flow_gradients(bpc, B).cpu().numpy()
        assert np.abs(got_grad - want_grad).max() < 1e-4 * np.abs(want_grad).max()
        check(lib.pcm_adam_flow_step(bpc.handle, B, dp.data_ptr(), dm.data_ptr(), dv.data_ptr(), lp.data_ptr(), lm.data_ptr(),
                                     lv.data_ptr(), lr, 0.9, 0.999, 1e-8, t))
        O.leaf_adam(fc, lf, aux_p, aux_m, aux_v, lr, 0.9, 0.999, 1e-8, t)
        logp_new = fc.logp[pe].astype(np.float32).copy()
        O.adam_step(params, want_grad.astype(np.float32), m, v, lr, 0.9, 0.999, 1e-8, t, gp, logp_new)
        fc.logp = fc.logp.copy()
        fc.logp[pe] = logp_new
        np.testing.assert_allclose(dp.cpu().numpy(), params, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(lp.cpu().numpy(), aux_p, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(lm.cpu().numpy(), aux_m, rtol=1e-4, atol=1e-6)
        got = P.vectorize_parameters(bpc)
        # (m / sqrt(v) carries the gradient's 1e-4 over to parameters whose gradient is near zero: 5e-4 here)
        np.testing.assert_allclose(np.exp(got[:ns]), np.exp(logp_new), rtol=5e-4)
        np.testing.assert_array_equal(got[ns:], leaves_before)        # the source never writes the leaves back


def test_em_then_adam_raises_the_likelihood(gpu):
    """The sequence of test/sgd/adam_tests.jl:16-24 on the small single-channel configuration (64 variables,
    K = 16, 256 categories, 1024 examples): mini-batch EM epochs, then Adam epochs on the same data; every
    phase raises the training log-likelihood and the Adam phase ends above where EM left off."""
    torch, P = gpu
    from pcmi355 import workloads
    cfg = workloads.make_config("c1_hclt64_k16")
    bpc = P.hclt_from_clt(cfg["parent"], cfg["C"], cfg["K"])
    bpc.set_params(cfg["theta"], cfg["leaf"])
    d = torch.from_numpy(cfg["data"]).cuda()
    g = torch.Generator().manual_seed(1)
    em = P.mini_batch_em(bpc, d, 5, batch_size=256, pseudocount=0.1, param_inertia=0.1, param_inertia_end=0.9, generator=g)
    assert em[-1] > em[0]
    st = {}
    lls = P.adam(bpc, d, 6, batch_size=256, lr=1e-2, generator=g, state=st)
    assert len(lls) == 6 and st["opt_count"] == 24
    assert lls[-1] > lls[0] and lls[-1] > em[-1]
    final = float(P.loglikelihoods(bpc, d).mean().item())
    assert final > em[-1]


@pytest.mark.parametrize("shape", ["random", "wide_levels"])
def test_row_queries_on_the_block_form_agree_with_the_layer_kernels(gpu, oracle, shape):
    """The four row queries of an HCLT handle (block form, the row as a grid dimension) against the same circuit
    compiled from its DAG (per-layer kernels of the general form; same parameter order): a random tree with up to five
    children per node, and a complete binary tree of twelve levels, whose widest level (1024 tree nodes) no longer
    fits the chains' ring of vectors in LDS -- the ring is then in device memory, one per row."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, log_dirichlet
    rng = np.random.default_rng(77)
    if shape == "random":
        V, K, C, R = 57, 32, 12, 9
        parent, theta, leaf, _ = make_hclt(V, K, C, 78, max_children=5)
    else:
        V, K, C, R = 4095, 16, 4, 3
        parent = np.array([-1] + [(v - 1) // 2 for v in range(1, V)], np.int32)
        parent, theta, leaf, _ = make_hclt(V, K, C, 79, parent=parent)
    blk = P.hclt_from_clt(parent, C, K)
    gen = _compile(P, O.hclt_dag(parent, K, C, theta, leaf), V, C)
    n, ns = blk.num_parameters(), blk.num_inner_params()
    assert n == gen.num_parameters() and np.array_equal(blk.table("param2edge"), gen.table("param2edge"))
    sizes = blk.table("pargroup_sizes")

    def draw(norm):
        rows = np.empty((R, n), np.float32)
        for r in range(R):
            pos = 0
            for sz in sizes:
                rows[r, pos:pos + sz] = log_dirichlet(rng, sz) if sz > 1 else 0.0
                pos += sz
            lf = np.exp(np.stack([log_dirichlet(rng, C) for _ in range((n - ns) // C)]))
            rows[r, ns:] = (lf if norm else np.log(lf)).reshape(-1)
        return torch.from_numpy(rows).cuda()

    def close(a, b, what):
        a, b = a.cpu().numpy(), b.cpu().numpy()
        assert np.abs(a - b).max() < 1e-4 * np.abs(b).max(), what

    for norm in (False, True):
        p1, p2 = draw(norm), draw(norm)
        noise = torch.from_numpy(_gumbel(rng, (R, ns))).cuda()
        G = torch.from_numpy(rng.normal(size=(R, V, C)).astype(np.float32)).cuda()
        close(P.kld(blk, p1, p2, norm_params=norm), P.kld(gen, p1, p2, norm_params=norm), "kld")
        a, b = P.kld_backward(blk, p1, p2, norm_params=norm), P.kld_backward(gen, p1, p2, norm_params=norm)
        close(a[0], b[0], "kld gradient 1")
        close(a[1], b[1], "kld gradient 2")
        kw = dict(temperature=0.7, noise=noise, norm_params=norm)
        close(P.gumbel_sample_rows(blk, p1, **kw), P.gumbel_sample_rows(gen, p1, **kw), "relaxed samples")
        for wrt_log in (True, False):
            close(P.gumbel_sample_backward_rows(blk, p1, G, grad_wrt_logparams=wrt_log, **kw),
                  P.gumbel_sample_backward_rows(gen, p1, G, grad_wrt_logparams=wrt_log, **kw), "reverse pass")
