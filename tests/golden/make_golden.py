#!/usr/bin/env python3
"""Writes the golden fixtures of this directory from the float64 build of the CPU oracle
(after the oracle itself has been pinned by tests/test_oracle_pinning.py):

    python tests/golden/make_golden.py

hclt_small.npz     an HCLT (6 variables, 16 hidden states, 5 categories), 24 examples:
                   log-likelihoods, flows, one EM step, KL to a second parameter set and its
                   gradient, Gumbel-max samples for stored noise
dag_small.npz      a random DAG with shared sub-circuits in the description format of
                   pcm_circuit_create, with the same expected outputs
soft_small.npz     the HCLT of hclt_small.npz under soft evidence [24, 6, 5] (some categories ruled
                   out): log-likelihoods, edge and leaf statistics, one EM step
multihead_small.npz  a three-head circuit over a shared body with a soft head mask: per-head
                   log-likelihoods, node-flow sums per description node, edge statistics, and
                   the sum-node children that survive pruning at threshold 0.05
(written by `python tests/golden/make_golden.py extra`, which leaves the first two files alone)
Inputs are float32 (what the library receives); expected outputs are float64, except the
samples, which are bit-exact integers computed in float32 like the library does.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [os.path.join(HERE, "..", "..", "oracle"), os.path.join(HERE, "..")]
import pc_oracle as O                                                      # noqa: E402
from helpers import correlated_data, describe_dag, random_dag, block_theta  # noqa: E402


def gumbel(rng, shape):
    return (-np.log(-np.log(rng.random(shape).clip(1e-12, 1 - 1e-12)))).astype(np.float32)


def grads_in_param_order(fc, eg, lg):
    """Per-edge (CSR order) and per-leaf values -> parameter-vector order."""
    pe = fc.sum_param_edges()
    leaf = [lg[fc.in_off[n]:fc.in_off[n] + fc.C] for n in fc.input_nodes()]
    return np.concatenate([eg[pe]] + leaf)


def expected(fc, fc2, data, idx, pc, inertia):
    ll, logp, leaf, ea, lf = O.em_step(fc, data, idx, pc, inertia, double=True)
    klds, ek = O.kld(fc, fc2, double=True)
    _, eg1, eg2, lg1, lg2 = O.kld_backward(fc, fc2, ek, double=True)
    order = fc.up_order()
    return dict(ll=ll, params_after=grads_in_param_order(fc, logp, leaf), edge_aggr=ea[order], leaf_flow=lf, kld=klds[-1],
                kld_grad1=grads_in_param_order(fc, eg1, lg1), kld_grad2=grads_in_param_order(fc, eg2, lg2))


def main():
    rng = np.random.default_rng(20240)
    # ---- HCLT ----
    V, K, C, B = 6, 16, 5, 24
    parent = np.array([-1, 0, 0, 1, 1, 4], np.int32)
    theta, leaf = O.random_hclt_params(parent, K, C, rng)
    theta2, leaf2 = O.random_hclt_params(parent, K, C, rng)
    data = correlated_data(40, V, C, 7, parent)
    idx = rng.permutation(40)[:B].astype(np.int32)
    fc = O.bits_compile(O.hclt_dag(parent, K, C, theta, leaf), C, V)      # reference numbering
    fc2 = O.bits_compile(O.hclt_dag(parent, K, C, theta2, leaf2), C, V)
    exp = expected(fc, fc2, data, idx, 0.1, 0.9)
    ch, root = O.clt_children(parent)
    inner = [v for v in O.clt_bottom_up(parent) if ch[v]]
    node_noise = gumbel(rng, (B, len(inner) * K))
    leaf_noise = gumbel(rng, (B, V, C))
    flat = O.hclt_flat(parent, K, C, theta, leaf)
    slot = np.zeros(flat.n_edges, np.int64)
    for r, v in enumerate(inner):
        nk = len(flat.meta["sum_node"][v])
        e0 = flat.meta["edge_of"][v]
        slot[e0:e0 + nk * K] = np.tile(r * K + np.arange(K), nk)
    samples = O.sample(flat, node_noise, leaf_noise, noise_slot=slot)
    np.savez_compressed(os.path.join(HERE, "hclt_small.npz"), parent=parent, K=K, C=C,
                        theta=block_theta(parent, K, theta), leaf=leaf, theta2=block_theta(parent, K, theta2), leaf2=leaf2,
                        data=data, idx=idx, pseudocount=0.1, inertia=0.9, node_noise=node_noise, leaf_noise=leaf_noise,
                        samples=samples, params_before=fc.vectorize_parameters(), **exp)
    # ---- general DAG ----
    V, C, B = 7, 4, 24
    root = random_dag(V, C, rng, width=3)
    d = describe_dag([root])
    fc = O.bits_compile(root, C, V)
    fc2 = fc.copy()
    p2 = fc.vectorize_parameters().copy()
    t = fc.param_tables()
    pos = 0
    for s in t["pargroup_sizes"]:
        p2[pos:pos + s] = np.log(rng.dirichlet(np.ones(s)))
        pos += s
    lv = np.exp(p2[pos:].reshape(-1, C)) * rng.uniform(0.5, 1.5, size=(len(p2[pos:]) // C, C))
    p2[pos:] = np.log(lv / lv.sum(axis=1, keepdims=True)).reshape(-1)
    p2 = p2.astype(np.float32)
    fc2.update_parameters(p2)
    data = rng.integers(0, C, size=(40, V)).astype(np.uint8)
    idx = rng.permutation(40)[:B].astype(np.int32)
    exp = expected(fc, fc2, data, idx, 0.1, 0.9)
    n_sum = len(t["param2edge"])
    node_noise = gumbel(rng, (B, n_sum))
    leaf_noise = gumbel(rng, (B, V, C))
    slot = np.zeros(fc.n_edges, np.int64)
    slot[fc.sum_param_edges()] = np.arange(n_sum)
    samples = O.sample(fc, node_noise, leaf_noise, noise_slot=slot)
    np.savez_compressed(os.path.join(HERE, "dag_small.npz"), V=V, C=C, data=data, idx=idx, pseudocount=0.1, inertia=0.9,
                        params_before=fc.vectorize_parameters(), params2=p2, node_noise=node_noise,
                        leaf_noise=leaf_noise, samples=samples, **d, **exp)
    for f in ("hclt_small.npz", "dag_small.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


def extra():
    """soft_small.npz and multihead_small.npz (own seeds; the first two fixtures are not touched)."""
    import dag_oracle as D
    from helpers import log_dirichlet
    h = dict(np.load(os.path.join(HERE, "hclt_small.npz"), allow_pickle=False))
    parent, K, C = h["parent"], int(h["K"]), int(h["C"])
    V, B = len(parent), 24
    rng = np.random.default_rng(20241)
    ev = rng.normal(0, 2, (B, V, C)).astype(np.float32)
    ev[rng.random((B, V, C)) < 0.15] = -np.inf
    ev[:, :, 0] = np.where(np.isinf(ev).all(axis=2), 0.0, ev[:, :, 0])
    fc = O.bits_compile(O.hclt_dag(parent, K, C, h["theta"], h["leaf"]), C, V)
    assert np.array_equal(fc.vectorize_parameters(), h["params_before"])
    mars = O.forward_soft(fc, ev, double=True)
    fl, ea = O.backward(fc, mars, double=True)
    counts = O.input_flows_soft(fc, ev, mars, fl, double=True)
    logp, leaf = O.em_update(fc, ea, counts, 0.1, 0.9, double=True)
    new = fc.copy()
    new.logp, new.leaf_logp = logp.astype(np.float32), leaf.astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "soft_small.npz"), evidence=ev, ll=mars[-1], edge_aggr=ea[fc.up_order()],
                        leaf_flow=counts, params_after=grads_in_param_order(fc, logp, leaf), pseudocount=0.1, inertia=0.9)
    # ---- multi-head ----
    V, C, H, B = 6, 4, 3, 32
    root = random_dag(V, C, rng, width=3)
    while len(root.children) < 3:
        root = random_dag(V, C, rng, width=3)
    heads = [O.summate(*root.children, logps=log_dirichlet(rng, len(root.children))) for _ in range(H)]
    d = describe_dag(heads)
    data = rng.integers(0, C, size=(B, V)).astype(np.uint8)
    mask = np.zeros((B, H), np.float32)
    mask[np.arange(B), rng.integers(0, H, B)] = 1.0
    mask += (rng.random((B, H)) < 0.25) * rng.random((B, H)).astype(np.float32)
    F, E, val = D.flows(heads, data, mask.astype(np.float64))
    order = [n for n in D.topo(heads) if all(n is not r for r in heads)] + heads   # description order
    node_flow = np.array([F[id(n)].sum() for n in order])
    is_sum = np.array([n.kind == O.SUM for n in order])
    child_ptr = d["child_ptr"]
    edge_flow = np.zeros(child_ptr[-1])
    for i, n in enumerate(order):
        if n.kind == O.SUM:
            for q in range(len(n.children)):
                edge_flow[child_ptr[i] + q] = E[(id(n), q)].sum()
    keep = np.zeros(child_ptr[-1], np.uint8)
    for i, n in enumerate(order):
        if n.kind == O.SUM and len(n.children) > 1:
            k = edge_flow[child_ptr[i]:child_ptr[i + 1]] > 0.05 * B
            if not k.any():
                k[int(np.argmax(n.logps))] = True
            keep[child_ptr[i]:child_ptr[i + 1]] = k
    pruned = D.prune(heads, {k: v.sum() for k, v in E.items()}, 0.05 * B)
    probe = rng.integers(0, C, size=(16, V)).astype(np.uint8)
    pv = D.values(pruned, probe)
    np.savez_compressed(os.path.join(HERE, "multihead_small.npz"), V=V, C=C, H=H, data=data, head_mask=mask,
                        ll_heads=np.stack([val[id(r)] for r in heads], 1), node_flow=node_flow, is_sum=is_sum,
                        edge_flow=edge_flow, keep=keep, prune_threshold=0.05, probe=probe,
                        ll_pruned=np.stack([pv[id(r)] for r in pruned], 1), **d)
    for f in ("soft_small.npz", "multihead_small.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    extra() if sys.argv[1:] == ["extra"] else main()
