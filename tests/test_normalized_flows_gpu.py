"""GPU parity of the per-example normalised flows (`per_sample_normalized_flows`, src/queries/flow.jl:417-593),
`normalize_params` (src/misc.jl:448-498) and the `normalized_flows_with_prealloc` pipeline
(src/utils/cuda_preallocation.jl:292-308, the first call of src/models/pc_vae.py:77) against the CPU oracle, through
the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL = 1e-4     # exp(entry), i.e. the normalised flow itself, relative (float32 on both sides)


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


def _same(got, want, n_sum):
    """Sum entries: exp within RTOL (absolute floor 1e-8 + float32 rounding at the guards); input entries: 0, -inf
    and NaN in the same places."""
    g, w = np.exp(got[:, :n_sum].astype(np.float64)), np.exp(want[:, :n_sum].astype(np.float64))
    assert np.abs(g - w).max() < RTOL * np.maximum(w, 1e-4).max()
    assert (np.abs(g - w) / np.maximum(w, 1e-6)).max() < 1e-3
    gi, wi = got[:, n_sum:], want[:, n_sum:]
    assert np.array_equal(np.isnan(gi), np.isnan(wi))
    ok = ~np.isnan(wi)
    assert np.array_equal(gi[ok], wi[ok])


@pytest.mark.parametrize("as_written", [True, False])
def test_normalized_flows_match_the_oracle_on_a_dag(gpu, oracle, as_written):
    torch, P = gpu
    O = oracle
    from helpers import random_dag
    V, C, B = 7, 5, 150
    root = random_dag(V, C, np.random.default_rng(21), width=4)
    fc = O.bits_compile(root, C, V)
    c = _compile(P, root, V, C)
    data = np.random.default_rng(22).integers(0, C, size=(B, V)).astype(np.uint8)
    want = O.normalized_flows(fc, data, double=True, as_written=as_written)
    n_sum = len(fc.sum_param_edges())
    got = P.per_sample_normalized_flows(c, data, as_written=as_written)
    assert got.shape == want.shape == (B, c.num_parameters()) and got.dtype == np.float32
    _same(got, want, n_sum)
    # in batches, into a column-major matrix (Julia's layout) on the device
    d = torch.from_numpy(data).cuda()
    out = torch.empty((c.num_parameters(), B), dtype=torch.float32, device="cuda").t()
    got2 = P.per_sample_normalized_flows(c, d, batch_size=64, as_written=as_written, out=out)
    assert got2.data_ptr() == out.data_ptr() and out.stride() == (1, B)
    np.testing.assert_array_equal(out.cpu().numpy(), got)
    # the circuit's accumulators are not touched
    P.probs_flows_circuit(c, d)
    ea0, lf0 = c.get_aggregates()
    P.per_sample_normalized_flows(c, d[:40].contiguous(), as_written=as_written)
    ea1, lf1 = c.get_aggregates()
    np.testing.assert_array_equal(ea0, ea1)
    np.testing.assert_array_equal(lf0, lf1)


@pytest.mark.parametrize("V,K,C,B", [(9, 16, 6, 70), (14, 32, 17, 40), (6, 8, 4, 33)])
def test_normalized_flows_of_an_hclt(gpu, oracle, V, K, C, B):
    """An HCLT handle answers on its general form, in the parameter order of vectorize_parameters: against the
    oracle on the DAG compiled as the reference compiles it, and every sum node's shares add up to 1."""
    torch, P = gpu
    O = oracle
    from helpers import make_hclt, block_theta, correlated_data
    parent, theta, leaf, _ = make_hclt(V, K, C, V + K)
    fc = O.bits_compile(O.hclt_dag(parent, K, C, theta, leaf), C, V)
    c = P.hclt_from_clt(parent, C, K)
    c.set_params(block_theta(parent, K, theta), leaf)
    np.testing.assert_allclose(P.vectorize_parameters(c), fc.vectorize_parameters(), rtol=1e-6)
    data = correlated_data(B, V, C, 5, parent)
    want = O.normalized_flows(fc, data, double=True)
    got = P.per_sample_normalized_flows(c, data)
    n_sum = len(fc.sum_param_edges())
    _same(got, want, n_sum)
    sizes = c.table("pargroup_sizes")
    ends = np.cumsum(sizes)
    tot = np.add.reduceat(np.exp(got[:, :n_sum].astype(np.float64)), np.concatenate([[0], ends[:-1]]), axis=1)
    flows = O.backward(fc, O.forward(fc, data, double=True), double=True)[0]
    pe = fc.sum_param_edges()
    live = flows[fc.edge_parent()[pe][np.concatenate([[0], ends[:-1]])]].T > 1e-3     # [B, groups]
    assert np.abs(tot[live] - 1).max() < 1e-4
    # multi-head circuits have no such query
    mh = P.multihead_hclt_from_clt(parent, C, 16, 3)
    with pytest.raises(P.PcmError):
        P.per_sample_normalized_flows(mh, data)


def test_normalize_params_rows(gpu, oracle):
    torch, P = gpu
    O = oracle
    from helpers import random_dag
    V, C, R = 5, 4, 37
    root = random_dag(V, C, np.random.default_rng(31), width=3)
    fc = O.bits_compile(root, C, V)
    c = _compile(P, root, V, C)
    n = c.num_parameters()
    p = np.random.default_rng(32).normal(0, 2, size=(R, n)).astype(np.float32)
    want = O.normalize_params(fc, p, double=True)
    got = P.normalize_params(c, p)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=2e-6)
    # in place on a column-major device matrix, then undone
    t = torch.as_strided(torch.from_numpy(np.ascontiguousarray(p.T)).cuda(), (R, n), (1, R))
    same = P.normalize_params(c, t)
    assert same.data_ptr() == t.data_ptr()
    np.testing.assert_allclose(t.cpu().numpy(), want, rtol=1e-5, atol=2e-6)
    back = P.normalize_params(c, t, undo=True).cpu().numpy()
    np.testing.assert_allclose(back, O.normalize_params(fc, want, undo=True, double=True), rtol=1e-5, atol=3e-6)


def test_normalized_flows_with_prealloc_pipeline(gpu, oracle):
    """`normalized_flows_with_prealloc` (cuda_preallocation.jl:292-308): flows of the circuit over (x, z), matched sum
    parameters copied into a parameter matrix of the circuit over z, clamped to [-20, 0], normalised -- against the
    same steps on the oracle.  Here z = the first three variables and the mapping pairs the sum nodes of the z
    circuit with the first sum nodes of the joint circuit that have as many children (the reference derives the
    pairs from a node correspondence, src/utils/map_params.jl:47-126; any list of pairs exercises the path)."""
    torch, P = gpu
    O = oracle
    from pcmi355 import prealloc
    from helpers import random_dag
    C, B = 4, 60
    root_xz = random_dag(6, C, np.random.default_rng(41), width=4)
    root_z = random_dag(3, C, np.random.default_rng(42), width=4)
    fxz, fz = O.bits_compile(root_xz, C, 6), O.bits_compile(root_z, C, 3)
    cxz, cz = _compile(P, root_xz, 6, C), _compile(P, root_z, 3, C)

    def groups(fc):
        par = fc.edge_parent()[fc.sum_param_edges()]
        out, s = [], 0
        for n in range(1, len(par) + 1):
            if n == len(par) or par[n] != par[s]:
                out.append((s, n))
                s = n
        return out
    ids_z, ids_xz, used = [], [], set()
    for (a, b) in groups(fz):
        for gi, (u, v) in enumerate(groups(fxz)):
            if gi not in used and v - u == b - a:
                used.add(gi)
                ids_z += list(range(a + 1, b + 1))
                ids_xz += list(range(u + 1, v + 1))
                break
    assert len(ids_z) >= 4
    data = np.random.default_rng(43).integers(0, C, size=(B, 6)).astype(np.uint8)
    prealloc.normalized_flows_preallocation(cxz, cz, num_examples=B, num_vars=6, mbpc_mapping=(ids_z, ids_xz))
    got = prealloc.normalized_flows_with_prealloc(cxz, cz, data)
    prealloc.normalized_flows_free_mem()
    nf = O.normalized_flows(fxz, data, double=True)
    z = np.zeros((B, len(fz.vectorize_parameters())))
    z[:, np.array(ids_z) - 1] = nf[:, np.array(ids_xz) - 1]
    want = O.normalize_params(fz, np.clip(z, -20.0, 0.0), double=True)
    assert got.shape == want.shape and got.dtype == np.float32
    ns = len(fz.sum_param_edges())
    np.testing.assert_allclose(np.exp(got[:, :ns]), np.exp(want[:, :ns]), rtol=2e-4, atol=1e-7)
    np.testing.assert_allclose(got[:, ns:], want[:, ns:], rtol=1e-5)       # unmatched leaves: uniform
    with pytest.raises(RuntimeError):
        prealloc.normalized_flows_with_prealloc(cxz, cz, data)
