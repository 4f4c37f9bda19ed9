"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares,
argument errors are reported as status codes without touching a GPU, and the host-side
workload builders are deterministic and well-formed."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pcmi355.h")
LIB = os.path.join(ROOT, "lvd-pg_amd", "libpcmi355.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pcm_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def cdll():
    assert os.path.exists(LIB), "build the library first: python lvd-pg_amd/build.py"
    return ctypes.CDLL(LIB)


def test_header_declares_the_whole_path():
    names = declared_symbols()
    for must in ("pcm_hclt_create", "pcm_circuit_create", "pcm_loglikelihoods", "pcm_flows", "pcm_em_update",
                 "pcm_em_step", "pcm_kld", "pcm_kld_backward", "pcm_sample", "pcm_adam_step",
                 "pcm_vectorize_parameters", "pcm_update_parameters", "pcm_index_table", "pcm_free"):
        assert must in names
    assert len(names) >= 25


def test_library_exports_every_declared_symbol(cdll):
    missing = [n for n in declared_symbols() if not hasattr(cdll, n)]
    assert not missing, missing


def test_version_and_error_reporting_without_a_gpu(cdll):
    cdll.pcm_last_error.restype = ctypes.c_char_p
    assert cdll.pcm_version() >= 1
    out = ctypes.c_void_p()
    # null tree
    rc = cdll.pcm_hclt_create(None, 4, 16, 8, ctypes.byref(out))
    assert rc == -1 and out.value is None
    assert b"null" in cdll.pcm_last_error().lower() or len(cdll.pcm_last_error()) > 0
    # bad sizes and a malformed tree are rejected before any device work
    par = (ctypes.c_int32 * 3)(-1, 0, 0)
    assert cdll.pcm_hclt_create(par, 3, 0, 8, ctypes.byref(out)) == -2
    assert cdll.pcm_hclt_create(par, 3, 16, 300, ctypes.byref(out)) == -2
    two_roots = (ctypes.c_int32 * 3)(-1, -1, 0)
    assert cdll.pcm_hclt_create(two_roots, 3, 16, 8, ctypes.byref(out)) == -2
    cycle = (ctypes.c_int32 * 3)(-1, 2, 1)
    assert cdll.pcm_hclt_create(cycle, 3, 16, 8, ctypes.byref(out)) == -2
    # null handles
    cdll.pcm_size.restype = ctypes.c_int64
    assert cdll.pcm_size(None, 0) < 0
    assert cdll.pcm_em_update(None, ctypes.c_float(0.1), ctypes.c_float(0.9)) == -1
    assert cdll.pcm_free(None) == -1
    # a pointer the library never gave out is turned down without being touched
    stray = ctypes.create_string_buffer(64)
    h = ctypes.cast(stray, ctypes.c_void_p)
    assert cdll.pcm_size(h, 0) < 0
    assert cdll.pcm_em_update(h, ctypes.c_float(0.1), ctypes.c_float(0.9)) == -1
    assert cdll.pcm_free(h) == -1 and b"live" in cdll.pcm_last_error()
    assert stray.raw == bytes(64)
    # structure learning and soft evidence: argument errors come back as status codes
    i64, f32 = ctypes.c_int64, ctypes.c_float
    assert cdll.pcm_pairwise_mi(None, i64(1), i64(1), i64(10), 3, 4, f32(0.1), None, None) == -1
    assert cdll.pcm_chow_liu_tree(None, 3, None) == -1
    mi = (ctypes.c_float * 9)(0, 2, 1, 2, 0, 3, 1, 3, 0)
    parent = (ctypes.c_int32 * 3)()
    assert cdll.pcm_chow_liu_tree(mi, 3, parent) == 0
    assert list(parent) == [1, -1, 1]                     # path 0 - 1 - 2, rooted at its centre
    assert cdll.pcm_loglikelihoods_soft(None, None, i64(1), i64(1), i64(1), None, 4, None) == -1
    assert cdll.pcm_flows_soft(None, None, i64(1), i64(1), i64(1), None, 4, f32(0), None, None) == -1
    assert cdll.pcm_node_flow_sums(None, None, i64(0)) == -1
    assert cdll.pcm_hclt_create_multihead(par, 2, 16, 8, 5000, ctypes.byref(out)) == -2


def test_python_mirror_binds_every_symbol():
    import pcmi355._lib as L
    for n in declared_symbols():
        assert hasattr(L.lib, n), n


def test_julia_bindings_follow_the_header_and_the_ctypes_table():
    """lvd-pg_amd/julia/LibPCMI355.jl is what gen_bindings.py writes from the header, binds every entry point, and
    its argument types are the ones the ctypes table of the Python mirror uses (two independent readings of the
    header)."""
    import importlib.util
    import pcmi355._lib as L
    jdir = os.path.join(ROOT, "lvd-pg_amd", "julia")
    spec = importlib.util.spec_from_file_location("gen_bindings", os.path.join(jdir, "gen_bindings.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    text = open(os.path.join(jdir, "LibPCMI355.jl")).read()
    assert text == gen.render(open(HEADER).read()), "run python lvd-pg_amd/julia/gen_bindings.py"
    bound = dict(re.findall(r"ccall\(\(:(pcm_[a-z0-9_]+), libpcmi355\), \w+, \(([^)]*)\)", text))
    assert sorted(bound) == declared_symbols()

    def kind(t):
        if t in (ctypes.c_int32, ctypes.c_int):
            return "Int32"
        if t is ctypes.c_int64:
            return "Int64"
        if t is ctypes.c_float:
            return "Float32"
        return "Ptr"
    for name in declared_symbols():
        argtypes = getattr(L.lib, name).argtypes or []
        jl = [t.strip() for t in bound[name].split(",") if t.strip()]
        jl = ["Ptr" if t.startswith("Ptr{") else "Int32" if t == "Cint" else t for t in jl]
        assert jl == [kind(t) for t in argtypes], name


def test_workload_builders():
    from pcmi355 import workloads as W
    a = W.grf_images(64, 8, 8, 3, 2.0, 0.8, seed=5)
    b = W.grf_images(64, 8, 8, 3, 2.0, 0.8, seed=5)
    assert a.dtype == np.uint8 and a.shape == (64, 192) and np.array_equal(a, b)
    assert a.min() == 0 and a.max() == 255
    # neighbouring pixels are correlated, distant channels share the base field
    x = a.astype(np.float64)
    assert np.corrcoef(x[:, 0], x[:, 1])[0, 1] > 0.5
    parent = W.chow_liu_parent(a)
    assert (parent < 0).sum() == 1 and len(parent) == 192
    # a tree: every node reaches the root without cycles
    root = int(np.nonzero(parent < 0)[0][0])
    for v in range(192):
        seen, u = 0, v
        while u != root:
            u = parent[u]
            seen += 1
            assert seen <= 192
    st = W.tree_stats(parent)
    assert st["n_inner"] + st["n_leaf"] == 192 and st["depth"] >= 1
    th, lf = W.init_params(parent, 4, 6, 1)
    np.testing.assert_allclose(np.exp(th.astype(np.float64)).sum(-1), 1, rtol=1e-5)
    np.testing.assert_allclose(np.exp(lf.astype(np.float64)).sum(-1), 1, rtol=1e-5)
    ratio = np.exp(th.max(-1) - th.min(-1))
    assert ratio.max() <= 1.4 / 0.6 + 1e-3      # init_parameters(perturbation = 0.4)


def test_algorithmic_bytes_formula():
    """The step formula: 6 vectors of K floats per (inner tree node, example), the batch once, the sum parameters
    three times, the leaf tables five.  Per kernel: two vectors each for the backward walk and the statistics, ONE
    for the forward walk (its second vector, the value read as a child, never leaves LDS and is not HBM traffic)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    n_int, V, K, C, B = 2505, 3072, 32, 256, 4096
    ab = bench.algorithmic_bytes(n_int, V, K, C, B)
    edges = (n_int - 1) * K * K + K
    assert ab["step"] == n_int * 6 * K * 4 * B + V * B + 3 * 4 * edges + 5 * 4 * V * K * C
    assert ab["forward"] == n_int * 1 * K * 4 * B + V * B + 4 * edges + 4 * V * K * C
    assert ab["backward"] == n_int * 2 * K * 4 * B + V * B + 4 * edges + 4 * V * K * C


def test_describe_dag_is_topological():
    from helpers import describe_dag, random_dag, simple_multihead_circuit
    import pc_oracle as O
    d = describe_dag([random_dag(7, 3, np.random.default_rng(0), width=3)])
    n = len(d["node_type"])
    for i in range(n):
        kids = d["child_idx"][d["child_ptr"][i]:d["child_ptr"][i + 1]]
        assert (kids < i).all()
        assert (d["node_type"][i] == O.INPUT) == (len(kids) == 0)
    assert len(d["input_logp"]) == 3 * (d["node_type"] == O.INPUT).sum()
    heads = simple_multihead_circuit(5)
    d = describe_dag(heads)
    assert d["node_type"][-2:].tolist() == [O.SUM, O.SUM] and len(d["node_type"]) == 10
