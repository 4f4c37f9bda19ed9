"""Structure learning (pairwise mutual information, Chow-Liu tree): the oracle against library
routines and closed forms (CPU), the HIP path against the oracle (GPU)."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.join(ROOT, "lvd-pg_amd"))

import structure_oracle as S  # noqa: E402


def _data(N, V, C, seed, corr=0.7):
    """Columns copied from their predecessor with probability `corr`, else uniform."""
    rng = np.random.default_rng(seed)
    x = np.zeros((N, V), np.uint8)
    x[:, 0] = rng.integers(0, C, N)
    for v in range(1, V):
        src = rng.integers(0, v)
        keep = rng.random(N) < corr
        x[:, v] = np.where(keep, x[:, src], rng.integers(0, C, N))
    return x


# ---- the oracle, pinned ------------------------------------------------------------------

def test_oracle_mi_matches_sklearn_without_pseudocount():
    from sklearn.metrics import mutual_info_score
    x = _data(500, 5, 6, 0)
    mi = S.pairwise_mi(x, 6, pseudocount=0.0)
    for u in range(5):
        for v in range(5):
            assert abs(mi[u, v] - mutual_info_score(x[:, u], x[:, v])) < 1e-10


def test_oracle_mi_closed_forms():
    rng = np.random.default_rng(1)
    N, C = 4000, 4
    a = rng.integers(0, C, N)
    b = rng.integers(0, C, N)
    x = np.stack([a, a, b], axis=1).astype(np.uint8)
    mi = S.pairwise_mi(x, C, pseudocount=0.0)
    p = np.bincount(a, minlength=C) / N
    H = -(p * np.log(p)).sum()
    assert abs(mi[0, 1] - H) < 1e-12 and abs(mi[0, 0] - H) < 1e-12      # MI(x, x) = H(x)
    assert 0 <= mi[0, 2] < 5e-3                                           # independent columns
    assert np.allclose(mi, mi.T)
    # the pseudocount enters as information.jl:52-58 says: every cell pc/C^2, every category pc/C, Z = N + pc
    pair, single = S.marginals(x.astype(np.int64), C, 0.5)
    assert abs(pair[0, 2].sum() - 1) < 1e-12 and abs(single[1].sum() - 1) < 1e-12
    assert abs(pair[0, 1][0, 1] - 0.5 / 16 / (N + 0.5)) < 1e-15           # an empty cell


def test_oracle_tree_is_a_maximum_spanning_tree_rooted_at_the_centre():
    from scipy.sparse.csgraph import minimum_spanning_tree
    x = _data(800, 12, 5, 2)
    mi = S.pairwise_mi(x, 5)
    parent = S.chow_liu_tree(mi)
    assert (parent < 0).sum() == 1
    w = mi.max() + 1.0 - mi
    np.fill_diagonal(w, 0)
    ref = minimum_spanning_tree(w).toarray()
    ref_weight = sum(mi[i, j] for i, j in zip(*np.nonzero(ref)))
    assert abs(S.tree_weight(mi, parent) - ref_weight) < 1e-9
    # path graph 0-1-2-3-4: the centre is 2; with six vertices the centres are 2 and 3 -> 2
    for V, root in ((5, 2), (6, 2)):
        m = np.zeros((V, V))
        for i in range(V - 1):
            m[i, i + 1] = m[i + 1, i] = 1.0
        p = S.chow_liu_tree(m)
        assert int(np.where(p < 0)[0][0]) == root


# ---- the C ABI on the host ----------------------------------------------------------------

def test_chow_liu_tree_host_entry_matches_oracle():
    import pcmi355 as P
    x = _data(600, 20, 4, 3)
    mi = S.pairwise_mi(x, 4).astype(np.float32)
    got = P.chow_liu_tree(mi)
    want = S.chow_liu_tree(mi.astype(np.float64))
    assert abs(S.tree_weight(mi, got) - S.tree_weight(mi, want)) < 1e-5
    assert np.array_equal(got, want)        # same tie rule, same centre
    with pytest.raises(P.PcmError):
        P.chow_liu_tree(np.full((3, 3), np.nan, np.float32))


# ---- the HIP path -------------------------------------------------------------------------

@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU box"
    import pcmi355
    return torch, pcmi355


@pytest.mark.gpu
@pytest.mark.parametrize("N,V,C,pc", [(300, 7, 5, 0.1), (1000, 9, 16, 0.0), (4097, 6, 256, 0.1), (64, 3, 2, 1.0),
                                      (5000, 4, 200, 0.1), (65535, 3, 256, 0.1), (65536, 3, 256, 0.1), (70001, 4, 256, 0.1),
                                      (140000, 3, 7, 0.0), (66000, 3, 200, 0.1), (12000, 5, 64, 0.1), (30000, 3, 256, 0.1)])
def test_pairwise_mi_matches_oracle(gpu, N, V, C, pc):
    """Tolerance: 1e-4 of the largest entry (float32 output of float64 sums).  Beyond 65535 examples
    the cells are counted in 32 bits, band by band of the first variable's categories (two bands at
    256 categories, one at 200 and 7)."""
    torch, P = gpu
    x = _data(N, V, C, N + V)
    want = S.pairwise_mi(x, C, pc)
    got = P.pairwise_MI(torch.from_numpy(x).cuda(), C, pc).cpu().numpy()
    assert np.abs(got - want).max() < 1e-4 * np.abs(want).max()
    assert np.array_equal(got, got.T)
    xt = torch.from_numpy(np.ascontiguousarray(x.T)).cuda().t()          # column-major, as Julia holds it
    assert np.array_equal(P.pairwise_MI(xt, C, pc).cpu().numpy(), got)


@pytest.mark.gpu
def test_learned_tree_and_hclt(gpu):
    torch, P = gpu
    x = _data(2000, 30, 8, 11)
    d = torch.from_numpy(x).cuda()
    mi = P.pairwise_MI(d, 8, 0.1).cpu().numpy()
    parent = P.learn_chow_liu_tree(d, 8, 0.1)
    want = S.chow_liu_tree(S.pairwise_mi(x, 8, 0.1))
    assert abs(S.tree_weight(mi, parent) - S.tree_weight(mi, want)) < 1e-3
    bpc = P.hclt(d, 16, num_cats=8)
    assert bpc.size("variables") == 30
    lls = P.mini_batch_em_with_reg(bpc, d, 3, batch_size=500, pseudocount=0.1, param_inertia=0.9, shuffle="none")
    assert lls[-1] > lls[0]


@pytest.mark.gpu
def test_hclt_over_variable_groups_and_for_colored_images(gpu):
    """`hclt(data, K, variable_groups)` and `hclt_for_colored_images` (src/structures/hclts.jl:7-98): the tree is
    learned on the groups' first variables, a tree node's leaf is the product of one categorical per variable of
    its group; the circuit is the one `hclt_pc` builds from that tree, it covers exactly the grouped variables,
    and it trains."""
    torch, P = gpu
    from pcmi355 import nodes as N
    nc, h, w, K, C, n = 3, 4, 4, 4, 6, 600
    x = _data(n, nc * h * w, C, 23)
    d = torch.from_numpy(x).cuda()
    for mode, offset in (("red_only", 0), ("green_only", h * w), ("blue_only", 2 * h * w), ("cat_channels", None)):
        pc, leaves = P.hclt_for_colored_images(d, nc, h, w, K, num_cats=C, mode=mode, patch_size=2)
        groups = (P.group_vars_by_cgrid(h, w, nc, 2, 2, 0) if offset is None else P.group_vars_by_grid(h, w, 1, 2, 2, offset))
        assert len(leaves) == len(groups) == 4 and all(len(l) == K for l in leaves)
        want_vars = sorted(v for g in groups for v in g[1])
        assert N.variables(pc) == want_vars and len(want_vars) == (4 * nc if offset is None else 4) * 4
        firsts = [g[0] for g in groups]
        clt = P.learn_chow_liu_tree(d[:, firsts].contiguous(), C, 0.1)
        same, _ = N.describe(P.hclt_pc(clt, C, K, groups))
        got, _ = N.describe(pc)
        for k in same:
            np.testing.assert_array_equal(got[k], same[k], err_msg=f"{mode} {k}")
        for i, g in enumerate(groups):                          # a leaf circuit: sum over the product of its group's inputs
            prod = leaves[i][0].inputs[0]
            assert [c.var for c in prod.inputs] == list(g[1])
    with pytest.raises(ValueError):
        P.hclt_for_colored_images(d, nc, h, w, K, num_cats=C, mode="grey")
    N.init_parameters(pc, perturbation=0.4, rng=np.random.default_rng(1))
    bpc = P.CuBitsProbCircuit(pc, nc * h * w)
    lls = P.mini_batch_em_with_reg(bpc, d, 3, batch_size=200, pseudocount=0.1, param_inertia=0.9, shuffle="none")
    assert lls[-1] > lls[0]


@pytest.mark.gpu
def test_pairwise_mi_full_size_properties(gpu):
    """4096 examples x 512 variables x 256 categories: symmetry, MI(x, x) = smoothed entropy
    identity against the oracle on a few pairs, duplicated column gives the same row."""
    torch, P = gpu
    from pcmi355 import workloads
    data = workloads.grf_images(4096, 16, 16, 2, 3.0, 0.8, seed=77)        # [4096, 512]
    data[:, 100] = data[:, 7]
    d = torch.from_numpy(data).cuda()
    mi = P.pairwise_MI(d, 256, 0.1).cpu().numpy()
    assert np.array_equal(mi, mi.T)
    assert np.allclose(mi[100], mi[7], rtol=0, atol=1e-6)
    sub = [0, 7, 100, 511]
    want = S.pairwise_mi(data[:, sub], 256, 0.1)
    assert np.abs(mi[np.ix_(sub, sub)] - want).max() < 1e-4 * np.abs(want).max()
