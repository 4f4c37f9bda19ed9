"""Shared builders for the parity tests (CPU side only: numpy + the oracle)."""
import numpy as np

import pc_oracle as O


def block_theta(parent, K, theta_dict):
    """{v: [K, K]} -> dense [V, K, K] (zeros for leaf tree nodes)."""
    V = len(parent)
    out = np.zeros((V, K, K), np.float32)
    for v, t in theta_dict.items():
        out[v] = t
    return out


def make_hclt(V, K, C, seed, kind="dirichlet", max_children=3, parent=None):
    rng = np.random.default_rng(seed)
    if parent is None:
        parent = O.random_tree(V, rng, max_children)
    theta, leaf = O.random_hclt_params(parent, K, C, rng, kind)
    fc = O.hclt_flat(parent, K, C, theta, leaf)
    return parent, theta, leaf, fc


def correlated_data(N, V, C, seed, parent=None):
    """uint8 data with tree-shaped dependence so flows are not uniform."""
    rng = np.random.default_rng(seed)
    x = np.zeros((N, V), np.int64)
    if parent is None:
        parent = np.arange(-1, V - 1)
    order = O.clt_bottom_up(parent)[::-1]
    for v in order:
        if parent[v] < 0:
            x[:, v] = rng.integers(0, C, N)
        else:
            step = rng.integers(-2, 3, N)
            fresh = rng.random(N) < 0.15
            x[:, v] = np.where(fresh, rng.integers(0, C, N), (x[:, parent[v]] + step) % C)
    return x.astype(np.uint8)


def oracle_em_reference(fc, data, idx, pseudocount, inertia):
    """One EM step on the oracle; returns LL, theta blocks, leaf [V,K,C], edge_aggr blocks, leaf flows."""
    ll, logp, leaf, ea, lf = O.em_step(fc, data, idx, pseudocount, inertia)
    K, C, V = fc.meta["K"], fc.C, fc.V
    new = fc.copy()
    new.logp = logp
    new.leaf_logp = leaf
    th, lf_new = O.hclt_block_params(new)
    return ll, th, lf_new, O.hclt_block_aggr(fc, ea), lf.reshape(V, K, C)


def rel_err(a, b, floor=1e-30):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return np.abs(a - b) / np.maximum(np.abs(b), floor)
