"""TEST INFRASTRUCTURE ONLY: Python face of the CPU oracle.

Holds (1) ctypes bindings to ``pc_oracle.c`` (float build and its double twin),
(2) a small-circuit restatement of how the reference flattens a circuit DAG into
nodes + (prime, sub) edges and derives its parameter-index tables, and (3) builders
for hidden Chow-Liu tree (HCLT) circuits.  Nothing in the product imports this module.

Reference lines restated here (paths relative to VariationalJuice.jl/):
  * src/structures/hclts.jl:100-145   -- `hclt_from_clt`: circuit shape of an HCLT
  * src/bits_circuit.jl:39-113        -- edge2param / param2edge / param2group /
                                         pargroup_sizes / innode2ncumparam tables
  * src/misc.jl:42-68                 -- parameter vector order: sum edges in up-edge
                                         order, then input nodes in creation order
  * test/bits_circuit_tests.jl:13-24, test/misc_tests.jl:14-62,
    test/queries/likelihood_tests.jl:24-37 -- node / edge numbering of the 3-variable
                                         fixture (the only numbering the reference pins)

The flattening itself lives in the un-vendored dependency ProbabilisticCircuits.jl
(`BitsProbCircuit`, v0.4.x API, no manifest in the reference).  Its published behaviour
is restated in `bits_compile`: depth-first post-order node numbering, pass-through of
single-child nodes, a two-child product whose children are plain nodes becomes a
(prime, sub) edge of its parent, larger products pair their children up into edges,
edges are grouped into layers by height.  Numbering beyond the fixture above is
"parity unpinned": no file in the reference fixes it.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass, field

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
INPUT, SUM, MUL = 0, 1, 2

_libs = {}


def build(force=False):
    """Compile pc_oracle.c into liborc32.so / liborc64.so next to this file."""
    src = os.path.join(HERE, "pc_oracle.c")
    for name, flag in (("liborc32.so", []), ("liborc64.so", ["-DREAL=double"])):
        out = os.path.join(HERE, name)
        if force or not os.path.exists(out) or os.path.getmtime(out) < os.path.getmtime(src):
            subprocess.check_call(
                ["gcc", "-O2", "-fopenmp", "-fPIC", "-shared", *flag, "-o", out, src, "-lm"])


def lib(double=False):
    key = "64" if double else "32"
    if key not in _libs:
        path = os.path.join(HERE, f"liborc{key}.so")
        if not os.path.exists(path) or os.path.getmtime(path) < os.path.getmtime(os.path.join(HERE, "pc_oracle.c")):
            build()   # absent, or older than its source
        _libs[key] = ctypes.CDLL(path)
        assert _libs[key].orc_real_size() == (8 if double else 4)
    return _libs[key]


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


@dataclass
class FlatCircuit:
    """Nodes in topological order (root last); edges grouped by parent (CSR)."""
    type: np.ndarray        # u8 [n]
    edge_ptr: np.ndarray    # i32 [n+1]
    prime: np.ndarray       # i32 [E]
    sub: np.ndarray         # i32 [E]  (-1: none)
    logp: np.ndarray        # f32 [E]  (0 on product edges)
    in_var: np.ndarray      # i32 [n]  (variable of an input node, else -1)
    in_off: np.ndarray      # i64 [n]  (offset of its C log-probs in leaf_logp, else -1)
    leaf_logp: np.ndarray   # f32 [n_inputs*C]
    C: int
    V: int
    meta: dict = field(default_factory=dict)

    @property
    def n_nodes(self):
        return len(self.type)

    @property
    def n_edges(self):
        return len(self.prime)

    def edge_parent(self):
        return np.repeat(np.arange(self.n_nodes, dtype=np.int32), np.diff(self.edge_ptr))

    def layers(self):
        """Height of every node: inputs 0, inner = 1 + max over prime/sub."""
        lay = np.zeros(self.n_nodes, dtype=np.int32)
        for n in range(self.n_nodes):
            e0, e1 = self.edge_ptr[n], self.edge_ptr[n + 1]
            if e1 > e0:
                m = lay[self.prime[e0:e1]].max()
                s = self.sub[e0:e1]
                if (s >= 0).any():
                    m = max(m, lay[s[s >= 0]].max())
                lay[n] = m + 1
        return lay

    def up_order(self):
        """Edge ids in the reference's up-edge order: by layer, then by parent id."""
        par = self.edge_parent()
        lay = self.layers()[par]
        return np.lexsort((np.arange(self.n_edges), par, lay)).astype(np.int64)

    def input_nodes(self):
        return np.nonzero(self.type == INPUT)[0].astype(np.int32)

    def param_tables(self):
        """src/bits_circuit.jl:39-113, 1-based like the reference's tests read them."""
        order = self.up_order()
        par = self.edge_parent()
        issum = self.type[par] == SUM
        edge2param = np.zeros(self.n_edges, dtype=np.int64)   # indexed by up-edge position
        param2edge, param2group, sizes = [], [], []
        group = 1
        for pos, e in enumerate(order):
            if not issum[e]:
                continue
            param2edge.append(pos + 1)
            edge2param[pos] = len(param2edge)
            param2group.append(group)
            last = (pos + 1 == len(order)) or par[order[pos + 1]] != par[e]
            if last:
                first_pos = pos
                while first_pos > 0 and par[order[first_pos - 1]] == par[e]:
                    first_pos -= 1
                sizes.append(pos - first_pos + 1)
                group += 1
        nin = len(self.input_nodes())
        return dict(edge2param=edge2param, param2edge=np.array(param2edge, dtype=np.int64),
                    param2group=np.array(param2group, dtype=np.int64),
                    pargroup_sizes=np.array(sizes, dtype=np.int64),
                    innode2ncumparam=np.cumsum(np.full(nin, self.C, dtype=np.int64)),
                    num_input_params=nin * self.C)

    def sum_param_edges(self):
        """CSR edge ids of the sum parameters, in parameter-vector order."""
        order = self.up_order()
        par = self.edge_parent()
        return order[self.type[par[order]] == SUM]

    def vectorize_parameters(self):
        """src/misc.jl:5-68: sum-edge log-params in up-edge order, then input nodes."""
        pe = self.sum_param_edges()
        leaf = [self.leaf_logp[self.in_off[n]:self.in_off[n] + self.C] for n in self.input_nodes()]
        return np.concatenate([self.logp[pe]] + leaf).astype(np.float32)

    def update_parameters(self, params):
        """src/misc.jl:73-135 (inverse of vectorize_parameters)."""
        pe = self.sum_param_edges()
        self.logp[pe] = params[:len(pe)]
        pos = len(pe)
        for n in self.input_nodes():
            self.leaf_logp[self.in_off[n]:self.in_off[n] + self.C] = params[pos:pos + self.C]
            pos += self.C

    def copy(self):
        return FlatCircuit(self.type, self.edge_ptr, self.prime, self.sub, self.logp.copy(),
                           self.in_var, self.in_off, self.leaf_logp.copy(), self.C, self.V,
                           dict(self.meta))


# ----------------------------------------------------------------------------------
# numeric kernels (ctypes)
# ----------------------------------------------------------------------------------

def _real(double):
    return np.float64 if double else np.float32


def forward(fc, data, idx=None, double=False):
    R = _real(double)
    data = np.ascontiguousarray(data, dtype=np.uint8)
    idx = np.arange(data.shape[0], dtype=np.int32) if idx is None else np.ascontiguousarray(idx, np.int32)
    B = len(idx)
    mars = np.empty((fc.n_nodes, B), dtype=R)
    logp = np.ascontiguousarray(fc.logp, dtype=R)
    leaf = np.ascontiguousarray(fc.leaf_logp, dtype=R)
    lib(double).orc_forward(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr), _p(fc.prime),
                            _p(fc.sub), _p(logp), _p(fc.in_var), _p(fc.in_off), _p(leaf),
                            _p(data), ctypes.c_int64(data.shape[1]), _p(idx), ctypes.c_int(B), _p(mars))
    return mars


def backward(fc, mars, edge_aggr=None, skip=None, root_ids=None, root_flow=None, double=False, fscale=1.0):
    """Node flows and (added to edge_aggr) edge flows summed over the batch.  fscale != 1: the tempered flows of
    `mini_batch_em_beta` (src-jl/learning/flow.jl:120-175, :204-300): every sum node's shares raised to 1 / fscale
    and normalised again."""
    R = _real(double)
    B = mars.shape[1]
    flows = np.empty((fc.n_nodes, B), dtype=R)
    if edge_aggr is None:
        edge_aggr = np.zeros(fc.n_edges, dtype=R)
    logp = np.ascontiguousarray(fc.logp, dtype=R)
    nr = 0 if root_ids is None else len(root_ids)
    rid = None if root_ids is None else np.ascontiguousarray(root_ids, np.int32)
    rfl = None if root_flow is None else np.ascontiguousarray(root_flow, R)
    if fscale != 1.0:
        lib(double).orc_backward_scaled(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr), _p(fc.prime),
                                        _p(fc.sub), _p(logp), _p(skip), _p(np.ascontiguousarray(mars, R)),
                                        ctypes.c_int(B), _p(flows), _p(edge_aggr), ctypes.c_int(nr), _p(rid), _p(rfl),
                                        (ctypes.c_double if double else ctypes.c_float)(fscale))
        return flows, edge_aggr
    lib(double).orc_backward(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr), _p(fc.prime),
                             _p(fc.sub), _p(logp), _p(skip), _p(np.ascontiguousarray(mars, R)),
                             ctypes.c_int(B), _p(flows), _p(edge_aggr), ctypes.c_int(nr), _p(rid), _p(rfl))
    return flows, edge_aggr


def input_flows(fc, data, flows, idx=None, leaf_flow=None, double=False):
    R = _real(double)
    data = np.ascontiguousarray(data, dtype=np.uint8)
    idx = np.arange(data.shape[0], dtype=np.int32) if idx is None else np.ascontiguousarray(idx, np.int32)
    if leaf_flow is None:
        leaf_flow = np.zeros(len(fc.leaf_logp), dtype=R)
    lib(double).orc_input_flows(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.in_var), _p(fc.in_off),
                                _p(data), ctypes.c_int64(data.shape[1]), _p(idx), ctypes.c_int(len(idx)),
                                _p(np.ascontiguousarray(flows, R)), _p(leaf_flow))
    return leaf_flow


def forward_soft(fc, ev, double=False):
    """ev [B, V, C] log-evidence -> node values [n_nodes, B]."""
    R = _real(double)
    ev = np.ascontiguousarray(ev, dtype=R)
    B, V, C = ev.shape
    assert C == fc.C
    mars = np.empty((fc.n_nodes, B), dtype=R)
    lib(double).orc_forward_soft(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr), _p(fc.prime), _p(fc.sub),
                                 _p(np.ascontiguousarray(fc.logp, dtype=R)), _p(fc.in_var), _p(fc.in_off),
                                 ctypes.c_int(C), _p(np.ascontiguousarray(fc.leaf_logp, dtype=R)), _p(ev),
                                 ctypes.c_int64(V), ctypes.c_int(B), _p(mars))
    return mars


def input_flows_soft(fc, ev, mars, flows, leaf_flow=None, double=False):
    R = _real(double)
    ev = np.ascontiguousarray(ev, dtype=R)
    B, V, C = ev.shape
    if leaf_flow is None:
        leaf_flow = np.zeros(len(fc.leaf_logp), dtype=R)
    lib(double).orc_input_flows_soft(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.in_var), _p(fc.in_off),
                                     ctypes.c_int(C), _p(np.ascontiguousarray(fc.leaf_logp, dtype=R)), _p(ev),
                                     ctypes.c_int64(V), ctypes.c_int(B), _p(np.ascontiguousarray(mars, R)),
                                     _p(np.ascontiguousarray(flows, R)), _p(leaf_flow))
    return leaf_flow


def soft_flow_counts(fc, data, flows, soft_reg, soft_reg_width, as_written=True, leaf_flow=None, double=False):
    """`soft_flow` over a batch (src/regularization/reg_flow.jl:3-22, called per input node and example by
    input_flows_circuit_with_reg_kernel, :24-48): an input node's flow goes to the observed category and to the
    categories of its window.  as_written: the lines as they stand, with the heap's entries -- LOG-probabilities -- in
    the shares and in the first term of `base`; otherwise the same lines on probabilities, i.e. the derivative of
    `soft_loglikelihood` (reg_likelihood.jl:4-14).  data [B, V] categories, flows [n_nodes, B]; returns the counts in
    the layout of fc.leaf_logp.  Plain loops: small cases only."""
    R = _real(double)
    leaf = np.asarray(fc.leaf_logp, dtype=R)
    out = np.zeros(len(leaf), dtype=R) if leaf_flow is None else leaf_flow
    s, C = R(soft_reg), fc.C
    for n in range(fc.n_nodes):
        if fc.type[n] != 0:
            continue
        v, off = int(fc.in_var[n]), int(fc.in_off[n])
        heap = leaf[off:off + C]
        for b in range(data.shape[0]):
            value = int(data[b, v])
            node_flow = R(flows[n, b])
            c_start = max(0, value - soft_reg_width // 2)
            c_end = min(c_start + soft_reg_width - 1, C - 1)
            sp = np.exp(heap[c_start:c_end + 1]).sum(dtype=R) / R(c_end - c_start + 1)
            q = heap if as_written else np.exp(heap)
            base = (R(1) - s) * q[value] + s * sp
            out[off + value] += (R(1) - s) * q[value] * node_flow / base
            for c in range(c_start, c_end + 1):
                out[off + c] += s / R(c_end - c_start + 1) * q[c] * node_flow / base
    return out


def em_update(fc, edge_aggr, leaf_flow, pseudocount, inertia, double=False, missing=False, return_aggr=False):
    """Returns the updated (logp, leaf_logp).  missing: the last row of every leaf table marks a missing value
    (log-probability 0; data carry category C - 1 where the reference has `missing`), and the flow it collected
    is the `missing_flow` of nodes/fixable_categorical_dist.jl:233-241.  return_aggr: also the edge statistics as the
    update leaves them -- `add_pseudocount` works in place (src/regularization/reg_em.jl:292), so under a flow memory
    the pseudocount of one update is part of what the next batch decays."""
    R = _real(double)
    logp = np.ascontiguousarray(fc.logp, dtype=R).copy()
    leaf = np.ascontiguousarray(fc.leaf_logp, dtype=R).copy()
    ea = np.ascontiguousarray(edge_aggr, dtype=R).copy()
    lf = np.ascontiguousarray(leaf_flow, dtype=R)
    rc = ctypes.c_double if double else ctypes.c_float
    lib(double).orc_em_update(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr), _p(logp), _p(ea),
                              _p(fc.in_off), ctypes.c_int(fc.C), _p(leaf), _p(lf),
                              rc(pseudocount), rc(inertia), ctypes.c_int(int(bool(missing))))
    if return_aggr:
        return logp, leaf, ea
    return logp, leaf


def em_step(fc, data, idx, pseudocount, inertia, double=False):
    """One mini-batch EM step in the order of src/regularization/reg_em.jl:276-299.
    Returns (per-example LL, new logp, new leaf_logp, edge_aggr, leaf_flow)."""
    mars = forward(fc, data, idx, double)
    flows, ea = backward(fc, mars, double=double)
    lf = input_flows(fc, data, flows, idx, double=double)
    logp, leaf = em_update(fc, ea, lf, pseudocount, inertia, double)
    return mars[-1].copy(), logp, leaf, ea, lf


def edge_flows(fc, mars, flows):
    """Per-example flows of the sum parameters, [n_sum_params, B] in parameter-vector order (the reference's
    `edge_flows[ex, edge]`, src/queries/flow.jl:49-60, :70-71): flow of the parent times
    exp(value of the edge's children + logp - value of the parent); 0 where the parent has no flow."""
    pe = fc.sum_param_edges()
    par = fc.edge_parent()[pe]
    R = mars.dtype
    em = mars[fc.prime[pe]] + fc.logp[pe].astype(R)[:, None]
    sub = fc.sub[pe]
    has = sub >= 0
    em[has] += mars[sub[has]]
    with np.errstate(invalid="ignore", over="ignore"):
        ef = flows[par] * np.exp(em - mars[par])
    ef[~(flows[par] > 0)] = 0
    return ef.astype(R), par


def normalized_flows(fc, data, idx=None, double=False, as_written=True):
    """`per_sample_normalized_flows(mbpc, data; batch_size)` (src/queries/flow.jl:417-464) -> [B, n_params] in
    parameter-vector order.  Sum parameters as `map_flows_kernel` writes them (:496-528): with f the edge flow
    and g the sum of the flows of the sum node's edges, log(f / (g + 1e-8) + 1e-8) (`par_groups` starts at 1e-8,
    :535).  Input parameters as `map_input_flows_kernel` (:549-593): log(f_c / sum_c f_c) of the node's
    per-example edge flows (`input_flows_circuit_kernel` :165-195), which hold the node's flow in ONE slot and 0
    elsewhere -- so the entries are 0 in that slot and -inf in the others, NaN (0/0) throughout where the node has
    no flow.  Which slot: `get_edge_flow` (src/nodes/fixable_categorical_dist.jl:162-176) compares the 0-based
    category with the 1-based parameter index, so as written the flow of category x sits in the slot of category
    x - 1 and category 0 leaves every slot empty (the test of test/queries/flow_tests.jl:54-64 has data value 1 in
    slot 1); as_written = False puts it in the slot of category x (what src/conditional_pc/flow.jl:244 does)."""
    R = _real(double)
    data = np.ascontiguousarray(data, dtype=np.uint8)
    idx = np.arange(data.shape[0], dtype=np.int32) if idx is None else np.ascontiguousarray(idx, np.int32)
    B = len(idx)
    mars = forward(fc, data, idx, double)
    flows, _ = backward(fc, mars, double=double)
    ef, par = edge_flows(fc, mars, flows)
    _, inv = np.unique(par, return_inverse=True)
    g = np.full((inv.max() + 1 if len(inv) else 0, B), 1e-8, dtype=R)
    np.add.at(g, inv, ef)
    with np.errstate(divide="ignore", invalid="ignore"):
        sums = np.log(ef / g[inv] + R(1e-8))
        leaves = []
        for n in fc.input_nodes():
            x = data[idx, fc.in_var[n]].astype(np.int64)
            slot = x - 1 if as_written else x
            f = np.zeros((fc.C, B), dtype=R)
            ok = slot >= 0
            f[slot[ok], np.nonzero(ok)[0]] = flows[n][ok]
            leaves.append(np.log(f / f.sum(axis=0, keepdims=True)))
    return np.concatenate([sums] + leaves, axis=0).T.astype(R)


def normalize_params(fc, params, undo=False, double=False):
    """`normalize_params(mbpc, params; undo)` (src/misc.jl:448-498) on rows [R, n_params] of parameter vectors.
    undo = False: every input node's C entries become exp(entry) / sum of them (`normalize_params_step`,
    :364-378: log-parameters -> probabilities) and every sum parameter logp - log(sum over its node of exp(logp))
    (`preprocess_inner_params_kernel`, :403-446).  undo = True: input entries p > 0 become log(p + 1e-6), others
    stay (`undo_normalize_params_step`, :380-393); the sum parameters go through the same normalisation."""
    R = _real(double)
    p = np.array(params, dtype=R, ndmin=2)
    pe = fc.sum_param_edges()
    ns = len(pe)
    par = fc.edge_parent()[pe]
    nin = len(fc.input_nodes())
    leaf = p[:, ns:].reshape(p.shape[0], nin, fc.C)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        if not undo:
            e = np.exp(leaf)
            leaf[...] = e / e.sum(axis=2, keepdims=True)
        else:
            leaf[...] = np.where(leaf > 0, np.log(leaf + R(1e-6)), leaf)
        if ns:
            _, inv = np.unique(par, return_inverse=True)
            cum = np.zeros((p.shape[0], inv.max() + 1), dtype=R)
            np.add.at(cum.T, inv, np.exp(p[:, :ns]).T)
            p[:, :ns] -= np.log(cum[:, inv])
    return p


def kld(fc1, fc2, double=False, norm_params=False):
    """norm_params: the circuits' leaf arrays hold probabilities (sum edges stay in log space)."""
    R = _real(double)
    klds = np.empty(fc1.n_nodes, dtype=R)
    ek = np.empty(fc1.n_edges, dtype=R)
    a = [np.ascontiguousarray(x, R) for x in (fc1.logp, fc2.logp, fc1.leaf_logp, fc2.leaf_logp)]
    lib(double).orc_kld(ctypes.c_int(fc1.n_nodes), _p(fc1.type), _p(fc1.edge_ptr), _p(fc1.prime),
                        _p(fc1.sub), _p(a[0]), _p(a[1]), _p(fc1.in_off), ctypes.c_int(fc1.C),
                        _p(a[2]), _p(a[3]), _p(klds), _p(ek), ctypes.c_int(int(norm_params)))
    return klds, ek


def kld_backward(fc1, fc2, edge_klds, analytic=False, double=False, norm_params=False):
    """norm_params: leaf arrays hold probabilities, leaf lines of fixable_categorical_dist.jl:216-217."""
    R = _real(double)
    a = [np.ascontiguousarray(x, R) for x in (fc1.logp, fc2.logp, fc1.leaf_logp, fc2.leaf_logp, edge_klds)]
    grads = np.empty(fc1.n_nodes, dtype=R)
    eg1 = np.zeros(fc1.n_edges, dtype=R)
    eg2 = np.zeros(fc1.n_edges, dtype=R)
    lg1 = np.zeros(len(fc1.leaf_logp), dtype=R)
    lg2 = np.zeros(len(fc1.leaf_logp), dtype=R)
    lib(double).orc_kld_backward(ctypes.c_int(fc1.n_nodes), _p(fc1.type), _p(fc1.edge_ptr), _p(fc1.prime),
                                 _p(fc1.sub), _p(a[0]), _p(a[1]), _p(fc1.in_off), ctypes.c_int(fc1.C),
                                 _p(a[2]), _p(a[3]), _p(a[4]), _p(grads), _p(eg1), _p(eg2), _p(lg1), _p(lg2),
                                 ctypes.c_int(2 if norm_params else int(analytic)))
    return grads, eg1, eg2, lg1, lg2


def sample(fc, edge_noise, leaf_noise, noise_slot=None, double=False):
    """edge_noise [B, stride], leaf_noise [B, V, C] -> uint8 [B, V]."""
    R = _real(double)
    en = np.ascontiguousarray(edge_noise, R)
    ln = np.ascontiguousarray(leaf_noise, R)
    B = en.shape[0]
    out = np.empty((B, fc.V), dtype=np.uint8)
    slot = None if noise_slot is None else np.ascontiguousarray(noise_slot, np.int64)
    lib(double).orc_sample(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr), _p(fc.prime), _p(fc.sub),
                           _p(np.ascontiguousarray(fc.logp, R)), _p(fc.in_var), _p(fc.in_off),
                           ctypes.c_int(fc.C), _p(np.ascontiguousarray(fc.leaf_logp, R)), _p(slot),
                           ctypes.c_int64(en.shape[1]), _p(en), _p(ln), ctypes.c_int64(fc.V),
                           ctypes.c_int(B), _p(out))
    return out


def gumbel_soft(fc, g, temperature, double=False, norm_params=False):
    R = _real(double)
    td = np.empty(fc.n_nodes, dtype=R)
    out = np.empty((fc.V, fc.C), dtype=R)
    gg = None if g is None else np.ascontiguousarray(g, R)
    rc = ctypes.c_double if double else ctypes.c_float
    lib(double).orc_gumbel_soft(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr), _p(fc.prime),
                                _p(fc.sub), _p(np.ascontiguousarray(fc.logp, R)), _p(fc.in_var),
                                _p(fc.in_off), ctypes.c_int(fc.C), _p(np.ascontiguousarray(fc.leaf_logp, R)),
                                _p(gg), rc(temperature), ctypes.c_int64(fc.V), _p(td), _p(out),
                                ctypes.c_int(int(norm_params)))
    return td, out


def gumbel_soft_backward(fc, g, temperature, out_grad, double=False, norm_params=False, grad_wrt_logparams=True):
    """Reverse pass of `gumbel_soft` (sample.jl:389-650): returns (edge_grad [n_edges] in CSR order,
    leaf_grad [n_leaf_params]) for the gradient `out_grad` [V, C] of a loss w.r.t. the soft output."""
    R = _real(double)
    td, _ = gumbel_soft(fc, g, temperature, double, norm_params)
    gg = None if g is None else np.ascontiguousarray(g, R)
    og = np.ascontiguousarray(out_grad, R)
    grads = np.zeros(fc.n_nodes, R)
    eg = np.zeros(fc.n_edges, R)
    lg = np.zeros(len(fc.leaf_logp), R)
    rc = ctypes.c_double if double else ctypes.c_float
    lib(double).orc_gumbel_soft_backward(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr), _p(fc.prime),
                                         _p(fc.sub), _p(np.ascontiguousarray(fc.logp, R)), _p(fc.in_var),
                                         _p(fc.in_off), ctypes.c_int(fc.C), _p(np.ascontiguousarray(fc.leaf_logp, R)),
                                         _p(gg), rc(temperature), _p(td), _p(og), ctypes.c_int(int(norm_params)),
                                         ctypes.c_int(int(grad_wrt_logparams)), _p(grads), _p(eg), _p(lg))
    return eg, lg


def adam_step(params, grad, m, v, lr, b1, b2, eps, t, group_ptr, logp_out, double=False):
    rc = ctypes.c_double if double else ctypes.c_float
    gp = np.ascontiguousarray(group_ptr, np.int64)
    lib(double).orc_adam_step(ctypes.c_int64(len(params)), _p(params), _p(grad), _p(m), _p(v), rc(lr), rc(b1),
                              rc(b2), rc(eps), ctypes.c_int(t), ctypes.c_int(len(gp) - 1), _p(gp), _p(logp_out))


def flow_gradients(fc, edge_aggr, batch_size, double=False):
    """sgd/adam.jl:27-61, 305-311: gradient of the mean LL w.r.t. unnormalised sum log-parameters,
    [n_edges] in CSR order (product edges keep their flow)."""
    R = _real(double)
    g = np.ascontiguousarray(edge_aggr, R).copy()
    rc = ctypes.c_double if double else ctypes.c_float
    lib(double).orc_flow_gradients(ctypes.c_int(fc.n_nodes), _p(fc.type), _p(fc.edge_ptr),
                                   _p(np.ascontiguousarray(fc.logp, R)), _p(g), rc(batch_size))
    return g


def leaf_adam(fc, leaf_flow, aux_p, aux_m, aux_v, lr, b1, b2, eps, t, double=False):
    """sgd/adam.jl:218-242 on every input node, in the order of fc.leaf_logp; the aux arrays are
    updated in place, the circuit's leaves are not."""
    R = _real(double)
    rc = ctypes.c_double if double else ctypes.c_float
    lib(double).orc_leaf_adam(ctypes.c_int64(len(fc.leaf_logp) // fc.C), ctypes.c_int(fc.C),
                              _p(np.ascontiguousarray(fc.leaf_logp, R)), _p(np.ascontiguousarray(leaf_flow, R)),
                              _p(aux_p), _p(aux_m), _p(aux_v), rc(lr), rc(b1), rc(b2), rc(eps), ctypes.c_int(t))


# ----------------------------------------------------------------------------------
# circuit DAGs and their flattening (small circuits)
# ----------------------------------------------------------------------------------

class Node:
    __slots__ = ("kind", "children", "logps", "var")

    def __init__(self, kind, children=(), logps=None, var=-1):
        self.kind, self.children, self.var = kind, list(children), var
        self.logps = None if logps is None else np.asarray(logps, dtype=np.float32)


def input_node(var, logps):
    return Node(INPUT, (), logps, var)


def summate(*children, logps=None):
    n = len(children)
    if logps is None:
        logps = np.full(n, -np.log(n), dtype=np.float32)
    return Node(SUM, children, logps)


def multiply(*children):
    return Node(MUL, children)


def bits_compile(root, C, V):
    """Flatten a DAG into a FlatCircuit (see the module docstring for what is restated)."""
    nparents = {}
    stack, seen = [root], set()
    while stack:
        n = stack.pop()
        if id(n) in seen:
            continue
        seen.add(id(n))
        for c in n.children:
            nparents[id(c)] = nparents.get(id(c), 0) + 1
            stack.append(c)

    types, in_var, in_off, leaf = [], [], [], []
    edges = {}          # node id -> list of (prime, sub, logp)
    memo = {}

    def new_node(kind, var=-1, off=-1):
        types.append(kind)
        in_var.append(var)
        in_off.append(off)
        return len(types) - 1

    def materialize(info):
        """info is ('node', id) or ('elem', prime, sub); return a node id."""
        if info[0] == "node":
            return info[1]
        nid = new_node(MUL)
        edges[nid] = [(info[1], info[2], 0.0)]
        return nid

    def visit(n):
        if id(n) in memo:
            return memo[id(n)]
        if n.kind == INPUT:
            off = len(leaf) * C
            leaf.append(n.logps)
            info = ("node", new_node(INPUT, n.var, off))
        else:
            infos = [visit(c) for c in n.children]
            if len(infos) == 1:
                info = infos[0]
            elif n.kind == SUM:
                es = []
                for i, lp in zip(infos, n.logps):
                    if i[0] == "elem":
                        es.append((i[1], i[2], float(lp)))
                    else:
                        es.append((i[1], -1, float(lp)))
                nid = new_node(SUM)
                edges[nid] = es
                info = ("node", nid)
            else:
                # children of a product must be nodes: an element child becomes a
                # product node of its own first
                ids = []
                for c, i in zip(n.children, infos):
                    if i[0] == "elem":
                        i = ("node", materialize(i))
                        memo[id(c)] = i
                    ids.append(i[1])
                if len(ids) == 2 and nparents.get(id(n), 0) <= 1:
                    info = ("elem", ids[0], ids[1])
                else:
                    nid = new_node(MUL)
                    edges[nid] = [(ids[k], ids[k + 1] if k + 1 < len(ids) else -1, 0.0)
                                  for k in range(0, len(ids), 2)]
                    info = ("node", nid)
        memo[id(n)] = info
        return info

    import sys
    old = sys.getrecursionlimit()
    sys.setrecursionlimit(max(old, 100000))
    try:
        info = visit(root)
    finally:
        sys.setrecursionlimit(old)
    materialize(info)
    n = len(types)
    edge_ptr = np.zeros(n + 1, dtype=np.int32)
    prime, sub, logp = [], [], []
    for i in range(n):
        for (p, s, lp) in edges.get(i, []):
            prime.append(p)
            sub.append(s)
            logp.append(lp)
        edge_ptr[i + 1] = len(prime)
    return FlatCircuit(np.array(types, np.uint8), edge_ptr, np.array(prime, np.int32),
                       np.array(sub, np.int32), np.array(logp, np.float32),
                       np.array(in_var, np.int32), np.array(in_off, np.int64),
                       np.concatenate(leaf).astype(np.float32) if leaf else np.zeros(0, np.float32), C, V)


# ----------------------------------------------------------------------------------
# HCLT
# ----------------------------------------------------------------------------------

def clt_children(parent):
    V = len(parent)
    ch = [[] for _ in range(V)]
    root = -1
    for v in range(V):
        if parent[v] < 0:
            root = v
        else:
            ch[parent[v]].append(v)
    return ch, root


def clt_bottom_up(parent):
    """Children before parents, root last (post-order of the rooted tree)."""
    ch, root = clt_children(parent)
    order, stack = [], [(root, 0)]
    while stack:
        v, i = stack.pop()
        if i < len(ch[v]):
            stack.append((v, i + 1))
            stack.append((ch[v][i], 0))
        else:
            order.append(v)
    return order


def hclt_dag(parent, K, C, theta, leaf):
    """src/structures/hclts.jl:100-145 with single-variable groups.

    theta[v] is the [K, K] log-parameter block of inner CLT node v (row k = sum node k,
    column j = hidden state j); only row 0 of the root's block is used (:137 takes
    circuits[1]).  leaf[v, j] are the C log-probs of `joined_leaves[v, j]`."""
    ch, root = clt_children(parent)
    V = len(parent)
    leaves = [[input_node(v, leaf[v, j]) for j in range(K)] for v in range(V)]
    circuits = [None] * V
    for v in clt_bottom_up(parent):
        if not ch[v]:
            circuits[v] = leaves[v]
            continue
        cc = [circuits[c] for c in ch[v]]
        if len(cc) > 1:
            cc = [summate(multiply(*[c[j] for c in cc])) for j in range(K)]
        else:
            cc = cc[0]
        circuits[v] = [summate(*[multiply(cc[j], leaves[v][j]) for j in range(K)], logps=theta[v][k])
                       for k in range(K)]
    return circuits[root][0]


def hclt_flat(parent, K, C, theta, leaf):
    """Same circuit as bits_compile(hclt_dag(...)) built directly (scales to thousands of
    variables).  Node order: all inputs (variable-major, then hidden state), then per CLT
    node bottom-up its K products (only if it has more than one child) and its K sums
    (1 for the root).  meta maps (v, k, j) to node and edge ids."""
    parent = np.asarray(parent)
    V = len(parent)
    ch, root = clt_children(parent)
    n_in = V * K
    types = [np.zeros(n_in, np.uint8)]
    in_var = [np.repeat(np.arange(V, dtype=np.int32), K)]
    in_off = [np.arange(n_in, dtype=np.int64) * C]
    nid = n_in
    prime, sub, logp, counts = [], [], [], [np.zeros(n_in, np.int32)]
    vec = {}       # CLT node -> node ids of its K output circuits
    sum_node = {}
    edge_of = {}
    ne = 0
    for v in clt_bottom_up(parent):
        if not ch[v]:
            vec[v] = np.arange(v * K, (v + 1) * K, dtype=np.int32)
            continue
        cvecs = [vec[c] for c in ch[v]]
        if len(cvecs) > 1:
            m = len(cvecs)
            ids = np.arange(nid, nid + K, dtype=np.int32)
            nid += K
            types.append(np.full(K, MUL, np.uint8))
            in_var.append(np.full(K, -1, np.int32))
            in_off.append(np.full(K, -1, np.int64))
            npair = (m + 1) // 2
            counts.append(np.full(K, npair, np.int32))
            pr = np.empty((K, npair), np.int32)
            sb = np.full((K, npair), -1, np.int32)
            for q in range(npair):
                pr[:, q] = cvecs[2 * q]
                if 2 * q + 1 < m:
                    sb[:, q] = cvecs[2 * q + 1]
            prime.append(pr.ravel())
            sub.append(sb.ravel())
            logp.append(np.zeros(K * npair, np.float32))
            ne += K * npair
            cvec = ids
        else:
            cvec = cvecs[0]
        nk = 1 if v == root else K
        ids = np.arange(nid, nid + nk, dtype=np.int32)
        nid += nk
        types.append(np.full(nk, SUM, np.uint8))
        in_var.append(np.full(nk, -1, np.int32))
        in_off.append(np.full(nk, -1, np.int64))
        counts.append(np.full(nk, K, np.int32))
        prime.append(np.tile(cvec, nk))
        sub.append(np.tile(np.arange(v * K, (v + 1) * K, dtype=np.int32), nk))
        logp.append(np.asarray(theta[v], np.float32)[:nk].ravel())
        edge_of[v] = ne
        ne += nk * K
        sum_node[v] = ids
        vec[v] = ids
    edge_ptr = np.concatenate([[0], np.cumsum(np.concatenate(counts))]).astype(np.int32)
    fc = FlatCircuit(np.concatenate(types), edge_ptr, np.concatenate(prime), np.concatenate(sub),
                     np.concatenate(logp), np.concatenate(in_var), np.concatenate(in_off),
                     np.ascontiguousarray(leaf, np.float32).reshape(-1).copy(), C, V)
    fc.meta = dict(K=K, root=root, sum_node=sum_node, edge_of=edge_of, children=ch)
    return fc


def hclt_block_params(fc):
    """theta blocks {v: [nk, K]} and leaf [V, K, C] read back from an hclt_flat circuit."""
    K = fc.meta["K"]
    th = {}
    for v, e0 in fc.meta["edge_of"].items():
        nk = len(fc.meta["sum_node"][v])
        th[v] = fc.logp[e0:e0 + nk * K].reshape(nk, K).copy()
    return th, fc.leaf_logp.reshape(fc.V, K, fc.C).copy()


def hclt_block_aggr(fc, edge_aggr):
    K = fc.meta["K"]
    out = {}
    for v, e0 in fc.meta["edge_of"].items():
        nk = len(fc.meta["sum_node"][v])
        out[v] = np.asarray(edge_aggr[e0:e0 + nk * K]).reshape(nk, K).copy()
    return out


def random_tree(V, rng, max_children=3):
    """A random rooted tree as a parent array (root = node 0 has parent -1)."""
    parent = np.full(V, -1, dtype=np.int32)
    nch = np.zeros(V, dtype=np.int32)
    for v in range(1, V):
        while True:
            p = int(rng.integers(0, v))
            if nch[p] < max_children:
                break
        parent[v] = p
        nch[p] += 1
    return parent


def random_hclt_params(parent, K, C, rng, kind="dirichlet"):
    """kind='dirichlet': normalised Exp(1) draws (Dirichlet(1)); kind='perturb': uniform
    (0.6, 1.4) normalised, the reference's init_params(perturbation = 0.4)
    (src/nodes/fixable_categorical_dist.jl:31-37)."""
    V = len(parent)

    def draw(shape):
        if kind == "dirichlet":
            x = rng.exponential(size=shape)
        else:
            x = rng.uniform(0.6, 1.4, size=shape)
        x = np.maximum(x, 1e-30)
        return np.log(x / x.sum(axis=-1, keepdims=True)).astype(np.float32)

    ch, _ = clt_children(parent)
    theta = {v: draw((K, K)) for v in range(V) if ch[v]}
    leaf = draw((V, K, C))
    return theta, leaf
