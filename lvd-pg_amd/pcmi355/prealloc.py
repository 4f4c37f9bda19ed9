"""The `*_with_prealloc` wrappers of src/utils/cuda_preallocation.jl:1-230, through which the
reference's Python side (src/models/pc_vae.py:77-95, via PyJulia) reaches the KL recursion and the
relaxed sampler with one parameter vector per example, `params[R, num_parameters]`.

The library keeps its own scratch memory, so the `*_preallocation` / `*_free_mem` calls only record
and check the shapes the reference asserts (:50-51, :192-193).  A row of the parameter matrices is
one circuit's worth of parameters: the rows are run one after the other through the single-vector
entry points (`pcm_kld`, `pcm_kld_backward`, `pcm_sample_soft`) on two scratch copies of the
circuit's structure.  Host arrays in, host arrays out, as there.
"""
import numpy as np
import torch

from .queries import kld, kld_backward, gumbel_sample, update_parameters, vectorize_parameters

_state = {}


def _twin(mbpc):
    """a second circuit with the structure of `mbpc` (the q side of a KL)"""
    from .circuits import HcltCircuit, hclt_from_clt, compile_circuit
    if isinstance(mbpc, HcltCircuit):
        return hclt_from_clt(mbpc.clt_parent, mbpc.num_cats, mbpc.num_hidden_cats)
    if hasattr(mbpc, "nodes"):
        from .circuits import CuBitsProbCircuit
        return CuBitsProbCircuit(mbpc.pcs, mbpc.num_vars)
    raise ValueError("the circuit must come from hclt_from_clt or CuBitsProbCircuit")


def _rows(params, n, what):
    p = np.ascontiguousarray(params, dtype=np.float32)
    if p.ndim != 2 or p.shape[1] != n:
        raise ValueError(f"{what} must be [num_examples, {n}], got {p.shape}")
    return p


def kld_preallocation(mbpc, *, num_examples):
    _state["kld"] = dict(num_examples=int(num_examples), twin=_twin(mbpc), mbpc=mbpc, rows=None)


def kld_free_mem():
    _state.pop("kld", None)


def kld_with_prealloc(mbpc, params1, params2, *, norm_params=False):
    """`kld_with_prealloc(mbpc, params1, params2)` (:47-61): KL(row r of params1 || row r of
    params2) for every row, as a float32 host vector.  A single row of params2 is shared by all
    rows of params1 (the prior of src/models/pc_vae.py:88-90)."""
    if norm_params:
        raise NotImplementedError("norm_params = true is not supported")
    st = _state.get("kld")
    if st is None or st["mbpc"] is not mbpc:
        raise RuntimeError("call kld_preallocation(mbpc; num_examples) first")
    n = mbpc.num_parameters()
    p1, p2 = _rows(params1, n, "params1"), _rows(params2, n, "params2")
    if p1.shape[0] != st["num_examples"]:
        raise ValueError(f"preallocated for {st['num_examples']} examples, got {p1.shape[0]}")   # :50
    if p2.shape[0] not in (1, p1.shape[0]):
        raise ValueError("params2 must have one row or as many as params1")
    keep = vectorize_parameters(mbpc)
    out = np.empty(p1.shape[0], np.float32)
    try:
        for r in range(p1.shape[0]):
            update_parameters(mbpc, p1[r])
            if r == 0 or p2.shape[0] > 1:
                update_parameters(st["twin"], p2[min(r, p2.shape[0] - 1)])
            out[r] = kld(mbpc, st["twin"])
    finally:
        update_parameters(mbpc, keep)
    st["rows"] = (p1, p2)
    return out


def kld_backward_with_prealloc(mbpc, *, norm_params=False, grad_wrt_logparams=True):
    """`kld_backward_with_prealloc(mbpc)` (:63-78): gradients of the KLs of the last
    `kld_with_prealloc` call with respect to the log-parameters of both sides, two host matrices
    [num_examples, num_parameters]."""
    if norm_params or not grad_wrt_logparams:
        raise NotImplementedError("only grad_wrt_logparams = true, norm_params = false")
    st = _state.get("kld")
    if st is None or st["mbpc"] is not mbpc or st["rows"] is None:
        raise RuntimeError("call kld_with_prealloc first")
    p1, p2 = st["rows"]
    g1, g2 = np.empty_like(p1), np.empty_like(p1)
    keep = vectorize_parameters(mbpc)
    try:
        for r in range(p1.shape[0]):
            update_parameters(mbpc, p1[r])
            if r == 0 or p2.shape[0] > 1:
                update_parameters(st["twin"], p2[min(r, p2.shape[0] - 1)])
            g1[r], g2[r] = kld_backward(mbpc, st["twin"])
    finally:
        update_parameters(mbpc, keep)
    return g1, g2


def gumbel_sample_preallocation(mbpc, *, num_examples, num_vars, par_buffer_size, allocate_for_grad=False,
                                allocate_for_target=False):
    if allocate_for_grad or allocate_for_target:
        raise NotImplementedError("the reverse pass of the relaxed sampler is not built")
    if num_vars != mbpc.size("variables") or par_buffer_size < mbpc.size("categories"):
        raise ValueError("num_vars / par_buffer_size do not fit the circuit")
    _state["sample"] = dict(num_examples=int(num_examples), num_vars=int(num_vars), width=int(par_buffer_size), mbpc=mbpc)


def gumbel_sample_free_mem(allocate_for_grad=False, allocate_for_target=False):
    _state.pop("sample", None)


def gumbel_sample_with_prealloc(mbpc, params, *, temperature, no_gumbel=False, norm_params=False, generator=None):
    """`gumbel_sample_with_prealloc(mbpc, params; temperature, no_gumbel)` (:189-203): one relaxed
    sample per row of `params`, the soft assignment [num_examples, num_vars, par_buffer_size]
    (columns past the circuit's categories stay zero) as a host array.  The reference draws its
    Gumbel noise inside the kernel; here it is drawn with torch (`generator` for a fixed stream)."""
    if norm_params:
        raise NotImplementedError("norm_params = true is not supported")
    st = _state.get("sample")
    if st is None or st["mbpc"] is not mbpc:
        raise RuntimeError("call gumbel_sample_preallocation first")
    p = _rows(params, mbpc.num_parameters(), "params")
    if p.shape[0] != st["num_examples"]:
        raise ValueError(f"preallocated for {st['num_examples']} examples, got {p.shape[0]}")       # :192
    from ._lib import lib
    need = int(lib.pcm_sample_noise_size(mbpc.handle))
    C = mbpc.size("categories")
    out = np.zeros((p.shape[0], st["num_vars"], st["width"]), np.float32)
    keep = vectorize_parameters(mbpc)
    try:
        for r in range(p.shape[0]):
            update_parameters(mbpc, p[r])
            noise = None
            if not no_gumbel:
                u = torch.rand((1, need), device="cuda", generator=generator).clamp_(1e-10, 1 - 1e-7)
                noise = -torch.log(-torch.log(u))
            out[r, :, :C] = gumbel_sample(mbpc, 1, temperature=temperature, node_noise=noise)[0].cpu().numpy()
    finally:
        update_parameters(mbpc, keep)
    return out
