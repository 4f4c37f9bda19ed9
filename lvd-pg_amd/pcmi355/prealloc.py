"""The `*_with_prealloc` wrappers of src/utils/cuda_preallocation.jl:1-230, through which the
reference's Python side (src/models/pc_vae.py:77-95, via PyJulia) reaches the KL recursion and the
relaxed sampler with one parameter vector per example, `params[R, num_parameters]`.

The library keeps its own scratch memory, so the `*_preallocation` / `*_free_mem` calls only record
and check the shapes the reference asserts (:50-51, :192-193).  The parameter matrices go to the
device once and all their rows run in one pass of the row entry points (`pcm_kld_rows`,
`pcm_kld_backward_rows`, `pcm_gumbel_sample_rows`); the circuit only lends its structure, its own
parameters are neither read nor changed.  Host arrays in, host arrays out, as there.
"""
import numpy as np
import torch

from .queries import (kld, kld_backward, gumbel_sample_rows, gumbel_sample_backward_rows, _rows_on_device,
                      per_sample_normalized_flows, map_pc_parameters, normalize_params)

_state = {}


def kld_preallocation(mbpc, *, num_examples):
    _state["kld"] = dict(num_examples=int(num_examples), mbpc=mbpc, rows=None)


def kld_free_mem():
    _state.pop("kld", None)


def kld_with_prealloc(mbpc, params1, params2, *, norm_params=False):
    """`kld_with_prealloc(mbpc, params1, params2; norm_params)` (:47-61): KL(row r of params1 || row r
    of params2) for every row, as a float32 host vector.  A single row of params2 is shared by all
    rows of params1 (the prior of src/models/pc_vae.py:88-90)."""
    st = _state.get("kld")
    if st is None or st["mbpc"] is not mbpc:
        raise RuntimeError("call kld_preallocation(mbpc; num_examples) first")
    n = mbpc.num_parameters()
    p1, _ = _rows_on_device(params1, n, "params1")
    p2, _ = _rows_on_device(params2, n, "params2")
    if p1.shape[0] != st["num_examples"]:
        raise ValueError(f"preallocated for {st['num_examples']} examples, got {p1.shape[0]}")   # :50
    if p2.shape[0] not in (1, p1.shape[0]):
        raise ValueError("params2 must have one row or as many as params1")
    st["rows"] = (p1, p2)                      # the reference keeps both matrices on the device for the reverse pass
    return kld(mbpc, p1, p2, norm_params=norm_params).cpu().numpy()


def kld_backward_with_prealloc(mbpc, *, norm_params=False, grad_wrt_logparams=True):
    """`kld_backward_with_prealloc(mbpc; norm_params, grad_wrt_logparams)` (:63-78): gradients of the
    KLs of the last `kld_with_prealloc` call with respect to both parameter matrices, two host
    matrices [num_examples, num_parameters]."""
    st = _state.get("kld")
    if st is None or st["mbpc"] is not mbpc or st["rows"] is None:
        raise RuntimeError("call kld_with_prealloc first")
    p1, p2 = st["rows"]
    g1, g2 = kld_backward(mbpc, p1, p2, norm_params=norm_params, grad_wrt_logparams=grad_wrt_logparams)
    return g1.cpu().numpy(), g2.cpu().numpy()


def gumbel_sample_preallocation(mbpc, *, num_examples, num_vars, par_buffer_size, allocate_for_grad=False,
                                allocate_for_target=False):
    if allocate_for_target:
        raise NotImplementedError("gumbel_sample_target_with_prealloc (parameter targets) is not built")
    if num_vars != mbpc.size("variables") or par_buffer_size < mbpc.size("categories"):
        raise ValueError("num_vars / par_buffer_size do not fit the circuit")
    _state["sample"] = dict(num_examples=int(num_examples), num_vars=int(num_vars), width=int(par_buffer_size), mbpc=mbpc,
                            grad=bool(allocate_for_grad), last=None)


def gumbel_sample_free_mem(allocate_for_grad=False, allocate_for_target=False):
    _state.pop("sample", None)


def gumbel_sample_with_prealloc(mbpc, params, *, temperature, no_gumbel=False, norm_params=False, generator=None):
    """`gumbel_sample_with_prealloc(mbpc, params; temperature, no_gumbel, norm_params)` (:189-203): one
    relaxed sample per row of `params`, the soft assignment [num_examples, num_vars, par_buffer_size]
    (columns past the circuit's categories stay zero) as a host array.  The reference draws its
    Gumbel noise inside the kernel (src/queries/sample.jl:45: -log(-log(u * (1 - 1e-6) + 1e-6)), one
    draw per example and sum edge); here the same draws come from torch (`generator` for a fixed
    stream)."""
    st = _state.get("sample")
    if st is None or st["mbpc"] is not mbpc:
        raise RuntimeError("call gumbel_sample_preallocation first")
    p, _ = _rows_on_device(params, mbpc.num_parameters(), "params")
    if p.shape[0] != st["num_examples"]:
        raise ValueError(f"preallocated for {st['num_examples']} examples, got {p.shape[0]}")       # :192
    noise = None
    if not no_gumbel:
        u = torch.rand((p.shape[0], mbpc.num_inner_params()), device=p.device, generator=generator)
        noise = -torch.log(-torch.log(u * (1.0 - 1e-6) + 1e-6))
    soft = gumbel_sample_rows(mbpc, p, temperature=temperature, noise=noise, norm_params=norm_params)
    st["last"] = (p, noise)                      # the reverse pass runs on the same parameters and draws
    C = mbpc.size("categories")
    out = np.zeros((p.shape[0], st["num_vars"], st["width"]), np.float32)
    out[:, :, :C] = soft.cpu().numpy()
    return out


def gumbel_sample_backward_with_prealloc(mbpc, input_aggr_grads, *, temperature, norm_params=False, grad_wrt_logparams=True):
    """`gumbel_sample_backward_with_prealloc(mbpc, input_aggr_grads; temperature, norm_params,
    grad_wrt_logparams)` (:205-218): gradients with respect to the parameter rows of the last
    `gumbel_sample_with_prealloc` call, given the gradients [num_examples, num_vars, par_buffer_size] with
    respect to what it returned; a host matrix [num_examples, num_parameters]."""
    st = _state.get("sample")
    if st is None or st["mbpc"] is not mbpc or st["last"] is None:
        raise RuntimeError("call gumbel_sample_with_prealloc first")
    if not st["grad"]:
        raise RuntimeError("gumbel_sample_preallocation was called without allocate_for_grad")
    p, noise = st["last"]
    og = np.asarray(input_aggr_grads, np.float32)
    if og.shape != (p.shape[0], st["num_vars"], st["width"]):
        raise ValueError(f"input_aggr_grads must be {(p.shape[0], st['num_vars'], st['width'])}, got {og.shape}")
    C = mbpc.size("categories")
    g = gumbel_sample_backward_rows(mbpc, p, torch.from_numpy(np.ascontiguousarray(og[:, :, :C])).to(p.device),
                                    temperature=temperature, noise=noise, norm_params=norm_params,
                                    grad_wrt_logparams=grad_wrt_logparams)
    return g.cpu().numpy()


def normalized_flows_preallocation(mbpc_xz, mbpc_z, *, num_examples, num_vars, mbpc_mapping):
    """`normalized_flows_preallocation` (:236-263): records the shapes and the parameter mapping (ids of mbpc_z,
    ids of mbpc_xz; 1-based)."""
    _state["nflows"] = dict(num_examples=int(num_examples), num_vars=int(num_vars), xz=mbpc_xz, z=mbpc_z,
                            mapping=(np.asarray(mbpc_mapping[0], np.int64), np.asarray(mbpc_mapping[1], np.int64)))


def normalized_flows_free_mem():
    _state.pop("nflows", None)


def normalized_flows_with_prealloc(mbpc_xz, mbpc_z, data):
    """`normalized_flows_with_prealloc(mbpc_xz, mbpc_z, data)` (:292-308), the first call of
    src/models/pc_vae.py:77: the per-example normalised flows of the joint circuit over (x, z), the columns of the
    matched sum parameters copied into a parameter matrix of the circuit over z, clamped to [-20, 0], and
    normalised (`normalize_params`: the leaves of mbpc_z become probabilities, its sum parameters normalised
    log-parameters).  Host matrix [num_examples, num_parameters(mbpc_z)]."""
    st = _state.get("nflows")
    if st is None or st["xz"] is not mbpc_xz or st["z"] is not mbpc_z:
        raise RuntimeError("call normalized_flows_preallocation(mbpc_xz, mbpc_z; ...) first")
    data = np.asarray(data)
    if data.shape != (st["num_examples"], st["num_vars"]):
        raise ValueError(f"preallocated for {(st['num_examples'], st['num_vars'])}, got {data.shape}")
    d = torch.from_numpy(np.ascontiguousarray(data, np.uint8)).cuda()
    xz = per_sample_normalized_flows(mbpc_xz, d, batch_size=data.shape[0])
    z = map_pc_parameters(mbpc_z, mbpc_xz, xz, param_mapping=st["mapping"])
    z.clamp_(-20.0, 0.0)
    return normalize_params(mbpc_z, z).cpu().numpy()
