"""Committed golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from
the float64 oracle): the float32 oracle on the CPU and the HIP library through the C ABI on
the GPU must both reproduce them."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
LL_RTOL = 1e-4       # fp32 log-likelihoods, relative
PARAM_RTOL = 1e-4    # updated parameters compared as probabilities, relative
FLOW_RTOL = 2e-4     # aggregated flows, relative to the largest entry


def load(name):
    return dict(np.load(os.path.join(GOLD, name), allow_pickle=False))


def rel(a, b):
    return np.abs(np.asarray(a, np.float64) - b) / np.maximum(np.abs(b), 1e-30)


def _check_outputs(g, ll, params_after, kld, g1, g2, samples):
    assert rel(ll, g["ll"]).max() < LL_RTOL
    assert rel(np.exp(params_after), np.exp(g["params_after"])).max() < PARAM_RTOL
    assert abs(kld - g["kld"]) < 1e-4 * abs(g["kld"])
    assert np.abs(g1 - g["kld_grad1"]).max() < 1e-4 * np.abs(g["kld_grad1"]).max()
    assert np.abs(g2 - g["kld_grad2"]).max() < 1e-4 * np.abs(g["kld_grad2"]).max()
    assert np.array_equal(samples, g["samples"])


def test_fixtures_are_well_formed():
    s, m = load("soft_small.npz"), load("multihead_small.npz")
    assert s["evidence"].dtype == np.float32 and s["evidence"].shape == (24, 6, 5) and np.isfinite(s["ll"]).all()
    assert m["head_mask"].shape == (32, 3) and m["ll_heads"].shape == (32, 3) and m["keep"].sum() > 0
    h, d = load("hclt_small.npz"), load("dag_small.npz")
    assert h["data"].dtype == np.uint8 and h["samples"].dtype == np.uint8
    assert h["ll"].shape == h["idx"].shape and np.isfinite(h["ll"]).all() and (h["ll"] < 0).all()
    assert h["kld"] > 0 and d["kld"] > 0
    assert len(h["params_before"]) == len(h["params_after"]) == len(h["kld_grad1"])
    assert len(d["params_before"]) == len(d["params_after"]) == len(d["params2"])


def test_float32_oracle_reproduces_hclt_fixture(oracle):
    O = oracle
    g = load("hclt_small.npz")
    parent, K, C = g["parent"], int(g["K"]), int(g["C"])
    V = len(parent)
    fc = O.bits_compile(O.hclt_dag(parent, K, C, g["theta"], g["leaf"]), C, V)
    fc2 = O.bits_compile(O.hclt_dag(parent, K, C, g["theta2"], g["leaf2"]), C, V)
    assert np.array_equal(fc.vectorize_parameters(), g["params_before"])
    ll, logp, leaf, ea, lf = O.em_step(fc, g["data"], g["idx"], float(g["pseudocount"]), float(g["inertia"]))
    new = fc.copy()
    new.logp, new.leaf_logp = logp, leaf
    klds, ek = O.kld(fc, fc2)
    _, eg1, eg2, lg1, lg2 = O.kld_backward(fc, fc2, ek)
    pe = fc.sum_param_edges()
    cat = lambda e, l: np.concatenate([e[pe]] + [l[fc.in_off[n]:fc.in_off[n] + C] for n in fc.input_nodes()])
    # sampling on the reference-numbered circuit: noise column of a sum edge = (rank of its tree
    # node, hidden state); both are recovered from the direct builder, whose answer is stored
    assert np.abs(ea[fc.up_order()] - g["edge_aggr"]).max() < FLOW_RTOL * g["edge_aggr"].max()
    assert np.abs(lf - g["leaf_flow"]).max() < FLOW_RTOL * g["leaf_flow"].max()
    _check_outputs(g, ll, new.vectorize_parameters(), klds[-1], cat(eg1, lg1), cat(eg2, lg2), g["samples"])


def test_float32_oracle_reproduces_dag_fixture(oracle):
    O = oracle
    g = load("dag_small.npz")
    V, C = int(g["V"]), int(g["C"])
    # rebuild the DAG from its description
    nodes = []
    k = 0
    for i, t in enumerate(g["node_type"]):
        kids = [nodes[c] for c in g["child_idx"][g["child_ptr"][i]:g["child_ptr"][i + 1]]]
        if t == O.INPUT:
            nodes.append(O.input_node(int(g["input_var"][i]), g["input_logp"][k * C:(k + 1) * C]))
            k += 1
        elif t == O.SUM:
            nodes.append(O.summate(*kids, logps=g["sum_logp"][g["child_ptr"][i]:g["child_ptr"][i + 1]]))
        else:
            nodes.append(O.multiply(*kids))
    fc = O.bits_compile(nodes[-1], C, V)
    assert np.array_equal(fc.vectorize_parameters(), g["params_before"])
    fc2 = fc.copy()
    fc2.update_parameters(g["params2"])
    ll, logp, leaf, ea, lf = O.em_step(fc, g["data"], g["idx"], float(g["pseudocount"]), float(g["inertia"]))
    new = fc.copy()
    new.logp, new.leaf_logp = logp, leaf
    klds, ek = O.kld(fc, fc2)
    _, eg1, eg2, lg1, lg2 = O.kld_backward(fc, fc2, ek)
    pe = fc.sum_param_edges()
    cat = lambda e, l: np.concatenate([e[pe]] + [l[fc.in_off[n]:fc.in_off[n] + C] for n in fc.input_nodes()])
    slot = np.zeros(fc.n_edges, np.int64)
    slot[pe] = np.arange(len(pe))
    s = O.sample(fc, g["node_noise"], g["leaf_noise"], noise_slot=slot)
    assert np.abs(ea[fc.up_order()] - g["edge_aggr"]).max() < FLOW_RTOL * g["edge_aggr"].max()
    _check_outputs(g, ll, new.vectorize_parameters(), klds[-1], cat(eg1, lg1), cat(eg2, lg2), s)


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355
    return torch, pcmi355


@pytest.mark.gpu
def test_library_reproduces_hclt_fixture(gpu):
    torch, P = gpu
    import pcmi355._lib as L
    g = load("hclt_small.npz")
    K, C = int(g["K"]), int(g["C"])
    a = P.hclt_from_clt(g["parent"], C, K)
    a.set_params(g["theta"], g["leaf"])
    b = P.hclt_from_clt(g["parent"], C, K)
    b.set_params(g["theta2"], g["leaf2"])
    assert np.array_equal(P.vectorize_parameters(a), g["params_before"])
    kld = P.kld(a, b)
    g1, g2 = P.kld_backward(a, b)
    s = P.sample(a, torch.from_numpy(g["node_noise"]).cuda(), torch.from_numpy(g["leaf_noise"]).cuda()).cpu().numpy()
    d = torch.from_numpy(g["data"]).cuda()
    ids = torch.from_numpy(g["idx"]).cuda()
    ll = torch.empty(len(g["idx"]), device="cuda")
    L.check(L.lib.pcm_em_step(a.handle, d.data_ptr(), d.stride(0), d.stride(1), ids.data_ptr(), len(g["idx"]), 0.0,
                              float(g["pseudocount"]), float(g["inertia"]), ll.data_ptr()))
    _, lf = a.get_flows()
    _check_outputs(g, ll.cpu().numpy(), P.vectorize_parameters(a), kld, g1, g2, s)


@pytest.mark.gpu
def test_library_reproduces_dag_fixture(gpu):
    torch, P = gpu
    import pcmi355._lib as L
    g = load("dag_small.npz")
    V, C = int(g["V"]), int(g["C"])
    mk = lambda: P.compile_circuit(g["node_type"], g["child_ptr"], g["child_idx"], g["sum_logp"], g["input_var"],
                                   g["input_logp"], V, C)
    a, b = mk(), mk()
    assert np.array_equal(P.vectorize_parameters(a), g["params_before"])
    P.update_parameters(b, g["params2"])
    kld = P.kld(a, b)
    g1, g2 = P.kld_backward(a, b)
    s = P.sample(a, torch.from_numpy(g["node_noise"]).cuda(), torch.from_numpy(g["leaf_noise"]).cuda()).cpu().numpy()
    d = torch.from_numpy(g["data"]).cuda()
    ll = P.probs_flows_circuit(a, d, example_ids=g["idx"]).cpu().numpy()
    ea, lf = a.get_aggregates()
    assert np.abs(ea - g["edge_aggr"]).max() < FLOW_RTOL * g["edge_aggr"].max()
    assert np.abs(lf - g["leaf_flow"]).max() < FLOW_RTOL * g["leaf_flow"].max()
    L.check(L.lib.pcm_em_update(a.handle, float(g["pseudocount"]), float(g["inertia"])))
    _check_outputs(g, ll, P.vectorize_parameters(a), kld, g1, g2, s)


# ---- soft evidence and multi-head statistics -----------------------------------------------------

def _rebuild(O, g):
    """the oracle DAG of a stored description, in description order"""
    C = int(g["C"])
    nodes, k = [], 0
    for i, t in enumerate(g["node_type"]):
        kids = [nodes[c] for c in g["child_idx"][g["child_ptr"][i]:g["child_ptr"][i + 1]]]
        if t == O.INPUT:
            nodes.append(O.input_node(int(g["input_var"][i]), g["input_logp"][k * C:(k + 1) * C]))
            k += 1
        elif t == O.SUM:
            nodes.append(O.summate(*kids, logps=g["sum_logp"][g["child_ptr"][i]:g["child_ptr"][i + 1]]))
        else:
            nodes.append(O.multiply(*kids))
    return nodes


def test_float32_oracle_reproduces_soft_fixture(oracle):
    O = oracle
    h, g = load("hclt_small.npz"), load("soft_small.npz")
    parent, K, C = h["parent"], int(h["K"]), int(h["C"])
    fc = O.bits_compile(O.hclt_dag(parent, K, C, h["theta"], h["leaf"]), C, len(parent))
    mars = O.forward_soft(fc, g["evidence"])
    assert rel(mars[-1], g["ll"]).max() < LL_RTOL
    fl, ea = O.backward(fc, mars)
    counts = O.input_flows_soft(fc, g["evidence"], mars, fl)
    assert np.abs(ea[fc.up_order()] - g["edge_aggr"]).max() < FLOW_RTOL * g["edge_aggr"].max()
    assert np.abs(counts - g["leaf_flow"]).max() < FLOW_RTOL * g["leaf_flow"].max()
    np.testing.assert_allclose(g["leaf_flow"].sum(), 24 * 6, rtol=1e-9)          # one unit per example and variable


def test_dag_oracle_reproduces_multihead_fixture(oracle):
    import dag_oracle as D
    O = oracle
    g = load("multihead_small.npz")
    H = int(g["H"])
    nodes = _rebuild(O, g)
    heads = nodes[-H:]
    F, E, val = D.flows(heads, g["data"], g["head_mask"].astype(np.float64))
    np.testing.assert_allclose(np.stack([val[id(r)] for r in heads], 1), g["ll_heads"], rtol=1e-9)
    np.testing.assert_allclose([F[id(n)].sum() for n in nodes], g["node_flow"], rtol=1e-9)
    fc = O.bits_compile(O.summate(*heads), int(g["C"]), int(g["V"]))              # the flat oracle on the same circuit
    mars = O.forward(fc, g["data"], double=True)
    assert np.abs(np.sort(mars[:, 0])[-3:].sum()) > 0                               # sanity: finite values
    pruned = D.prune(heads, {k: v.sum() for k, v in E.items()}, float(g["prune_threshold"]) * len(g["data"]))
    pv = D.values(pruned, g["probe"])
    np.testing.assert_allclose(np.stack([pv[id(r)] for r in pruned], 1), g["ll_pruned"], rtol=1e-9)


@pytest.mark.gpu
def test_library_reproduces_soft_fixture(gpu):
    torch, P = gpu
    import pcmi355._lib as L
    h, g = load("hclt_small.npz"), load("soft_small.npz")
    a = P.hclt_from_clt(h["parent"], int(h["C"]), int(h["K"]))
    a.set_params(h["theta"], h["leaf"])
    ev = torch.from_numpy(g["evidence"]).cuda()
    ll = P.probs_flows_circuit(a, ev).cpu().numpy()
    assert rel(ll, g["ll"]).max() < LL_RTOL
    assert rel(P.loglikelihoods(a, ev).cpu().numpy(), g["ll"]).max() < LL_RTOL
    _, lf = a.get_flows()
    # the fixture holds the leaf statistics in parameter order; the permutation from the block form is
    # read off a circuit whose leaf "parameters" are their own block-form positions
    V, K, C = len(h["parent"]), int(h["K"]), int(h["C"])
    probe = P.hclt_from_clt(h["parent"], C, K)
    probe.set_params(None, -(1.0 + np.arange(V * K * C, dtype=np.float32)).reshape(V, K, C))
    at = (-P.vectorize_parameters(probe)[probe.num_inner_params():] - 1.0).astype(np.int64)
    assert np.abs(lf.reshape(-1)[at] - g["leaf_flow"]).max() < FLOW_RTOL * g["leaf_flow"].max()
    L.check(L.lib.pcm_em_update(a.handle, float(g["pseudocount"]), float(g["inertia"])))
    assert rel(np.exp(P.vectorize_parameters(a)), np.exp(g["params_after"])).max() < PARAM_RTOL


@pytest.mark.gpu
def test_library_reproduces_multihead_fixture(gpu):
    torch, P = gpu
    N = P.nodes
    g = load("multihead_small.npz")
    V, C, H = int(g["V"]), int(g["C"]), int(g["H"])
    # the stored description as a DAG of pcmi355.nodes, in description order
    nodes, k = [], 0
    for i, t in enumerate(g["node_type"]):
        kids = [nodes[c] for c in g["child_idx"][g["child_ptr"][i]:g["child_ptr"][i + 1]]]
        if t == N.INPUT:
            nodes.append(N.input_node(int(g["input_var"][i]), g["input_logp"][k * C:(k + 1) * C]))
            k += 1
        elif t == N.SUM:
            nodes.append(N.summate(kids, params=g["sum_logp"][g["child_ptr"][i]:g["child_ptr"][i + 1]]))
        else:
            nodes.append(N.multiply(kids))
    pcs = nodes[-H:]
    bpc = P.CuMultiHeadBitsProbCircuit(pcs, num_vars=V)
    assert [id(n) for n in bpc.nodes] == [id(n) for n in nodes]
    d, hm = torch.from_numpy(g["data"]).cuda(), torch.from_numpy(g["head_mask"]).cuda()
    assert rel(P.loglikelihoods(bpc, d).cpu().numpy(), g["ll_heads"]).max() < LL_RTOL
    P.probs_flows_circuit(bpc, d, head_mask=hm)
    sums = bpc.node_flow_sums()
    nodes_map, node2id = P.node_maps(bpc)
    for i, n in enumerate(nodes):
        f = node2id.get(id(n))
        if f is not None and nodes_map[f] is n:
            assert abs(sums[f - 1] - g["node_flow"][i]) < FLOW_RTOL * max(g["node_flow"].max(), 1.0), i
    pruned = P.prune_pc(pcs, d, hm, batch_size=len(g["data"]), prune_threshold=float(g["prune_threshold"]))
    kept = {id(n): len(n.inputs) for n in N.linearize(pruned)}
    want_edges = int(g["keep"].sum())
    got_edges = sum(len(n.inputs) for n in N.linearize(pruned) if N.issum(n) and len(n.inputs) > 1)
    assert got_edges <= want_edges + H * 2                              # a head pruned to one child gets a copy added
    out = P.CuMultiHeadBitsProbCircuit(pruned, num_vars=V)
    assert rel(P.loglikelihoods(out, torch.from_numpy(g["probe"]).cuda()).cpu().numpy(), g["ll_pruned"]).max() < LL_RTOL
