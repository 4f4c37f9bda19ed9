"""Structure changes driven by flows: `prune_pc` (src-jl/multi_head_pc/prune.jl:4-97) and
`grow_heads_by_flows` (src-jl/multi_head_pc/transformation.jl:94-279).  Both run the flow pass
of a multi-head circuit over a dataset on the device, read the accumulated statistics and
rebuild the DAG on the host."""
import numpy as np
import torch

from . import nodes as N
from .circuits import CuMultiHeadBitsProbCircuit, node_maps
from .queries import probs_flows_circuit


def _logsumexp(x):
    m = np.max(x)
    return m + np.log(np.sum(np.exp(x - m)))


def aggregate_edge_flows(mhbpc, data, head_mask, batch_size):
    """`edge_aggr` summed over the full batches of `data` (prune.jl:18-27: the trailing
    examples that do not fill a batch are left out, as there).  Returns (edge_aggr in up-edge
    order, number of examples covered)."""
    n = data.shape[0]
    num_batches = n // batch_size
    if num_batches < 1:
        raise ValueError("fewer examples than one batch")
    for b in range(num_batches):
        ids = torch.arange(b * batch_size, (b + 1) * batch_size, device=data.device, dtype=torch.int32)
        probs_flows_circuit(mhbpc, data, example_ids=ids, rate=0.0 if b == 0 else 1.0, head_mask=head_mask)
    ea, _ = mhbpc.get_aggregates()
    return ea, num_batches * batch_size


def aggregate_node_flows(mhbpc, data, head_mask, batch_size):
    """Mean flow per node over all examples (transformation.jl:112-124), [num_nodes]."""
    n = data.shape[0]
    total = np.zeros(mhbpc.num_nodes(), np.float64)
    for s in range(0, n, batch_size):
        ids = torch.arange(s, min(s + batch_size, n), device=data.device, dtype=torch.int32)
        probs_flows_circuit(mhbpc, data, example_ids=ids, rate=0.0, head_mask=head_mask)
        total += mhbpc.node_flow_sums()
    return (total / n).astype(np.float32)


def prune_pc(pcs, data, head_mask, *, batch_size, prune_threshold, mhbpc=None):
    """`prune_pc(pcs, data, head_mask; batch_size, prune_threshold)`: keeps the sum edges whose
    accumulated flow exceeds `prune_threshold * num_examples` (the most probable child where
    none does), renormalises, and returns the new heads.  A head left with one child gets a
    copy of it as a second child, as in the reference (prune.jl:88-96)."""
    pcs = list(pcs)
    if mhbpc is None:
        mhbpc = CuMultiHeadBitsProbCircuit(pcs)
    edge_aggr, _ = aggregate_edge_flows(mhbpc, data, head_mask, batch_size)
    keep = edge_aggr > prune_threshold * data.shape[0]
    nodes_map, _ = node_maps(mhbpc)
    parent = mhbpc.table("edge_parent")
    e2p = mhbpc.table("edge2param")
    kept = {}
    pos = 0
    while pos < len(parent):                       # an edge's rank in its parent's run is the child's index
        end = pos
        while end < len(parent) and parent[end] == parent[pos]:
            end += 1
        n = nodes_map.get(int(parent[pos]))
        if n is not None and n.kind == N.SUM and e2p[pos] > 0 and keep[pos:end].any():
            kept[id(n)] = np.nonzero(keep[pos:end])[0]
        pos = end

    def f_sum(n, ins):
        idx = kept.get(id(n), np.zeros(0, np.int64))
        if len(idx) == 0:                           # also a sum with one child: it has no edge of its own
            idx = np.array([int(np.argmax(n.params))])
        params = n.params[idx].astype(np.float32)
        params = params - np.float32(_logsumexp(params))
        return N.summate([ins[i] for i in idx], params=params)

    fake_root = N.summate(pcs)
    kept[id(fake_root)] = np.arange(len(pcs))
    root = N.foldup_aggregate(fake_root, lambda n: N.InputNode(n.var, n.logps), lambda n, ins: N.multiply(ins), f_sum)
    out = []
    for pc in root.inputs:
        if len(pc.inputs) == 1 and pc.inputs[0].kind == N.MUL:
            fake = N.multiply(pc.inputs[0].inputs)
            pc = N.summate(pc.inputs[0], fake)
        out.append(pc)
    return out


def _perturb_input(n, sigma, rng):
    """`perturb(n::PlainInputNode; sigma)` (transformation.jl:77-86)."""
    lp = n.logps.astype(np.float64) + np.log(np.clip(rng.normal(1.0, sigma, len(n.logps)), 0.1, 2.0))
    n.logps = (lp - _logsumexp(lp)).astype(np.float32)


def _perturb(params, sigma, rng):
    """`perturb(params; sigma)` (transformation.jl:88-94)."""
    p = np.asarray(params, np.float64) + np.log(np.clip(rng.normal(1.0, sigma, len(params)), 0.1, 10.0))
    return (p - _logsumexp(p)).astype(np.float32)


def grow_heads_by_flows(pcs, data, head_mask, *, batch_size, sigma=0.2, cross_term_discount=0.2,
                        node_selection_method="percentage", node_selection_args=None, mhbpc=None, rng=None):
    """`grow_heads_by_flows(pcs, data, head_mask; sigma, cross_term_discount,
    node_selection_method, node_selection_args, batch_size)`: the nodes that carry the most flow
    (the top `grow_frac` of all nodes by mean flow) are split into two perturbed copies; a sum
    node above a split child takes both copies, with the cross terms discounted where it is
    split itself or has a split parent; heads that were split add their second copy to the end
    of the returned list."""
    pcs = list(pcs)
    rng = np.random.default_rng() if rng is None else rng
    args = node_selection_args or {}
    if mhbpc is None:
        mhbpc = CuMultiHeadBitsProbCircuit(pcs)
    aggr = aggregate_node_flows(mhbpc, data, head_mask, batch_size)
    if node_selection_method != "percentage":
        raise ValueError(f"Unknown node selection method {node_selection_method}.")
    threshold = max(np.percentile(aggr, (1.0 - args["grow_frac"]) * 100.0), 1e-8)
    grow_flag = aggr >= threshold
    _, node2id = node_maps(mhbpc)

    def grows(n):
        f = node2id.get(id(n))
        return f is not None and bool(grow_flag[f - 1])

    has_grow_pars = set()
    for n in reversed(N.linearize(pcs)):
        if n.kind != N.INPUT and (grows(n) or id(n) in has_grow_pars):
            for c in n.inputs:
                has_grow_pars.add(id(c))

    log_d = np.float32(np.log(cross_term_discount))
    old2new = {}

    def mul_pair(n):
        ch = [old2new[id(c)] for c in n.inputs]
        return N.multiply([a for a, _ in ch]), N.multiply([a if b is None else b for a, b in ch])

    def doubled(n):
        """children with both copies of a split child, and the two parameter rows"""
        chs, p1, p2 = [], [], []
        for i, c in enumerate(n.inputs):
            a, b = old2new[id(c)]
            if b is None:
                chs.append(a); p1.append(n.params[i]); p2.append(n.params[i])
            else:
                chs += [a, b]
                p1 += [n.params[i], n.params[i] + log_d]
                p2 += [n.params[i] + log_d, n.params[i]]
        return chs, np.array(p1, np.float32), np.array(p2, np.float32)

    for n in N.linearize(pcs):
        if grows(n):
            if n.kind == N.INPUT:
                n1, n2 = N.InputNode(n.var, n.logps), N.InputNode(n.var, n.logps)
                _perturb_input(n1, sigma, rng)
                _perturb_input(n2, sigma, rng)
                old2new[id(n)] = (n1, n2)
            elif n.kind == N.SUM:
                chs, p1, p2 = doubled(n)
                old2new[id(n)] = (N.summate(chs, params=_perturb(p1, sigma, rng)), N.summate(chs, params=_perturb(p2, sigma, rng)))
            else:
                old2new[id(n)] = mul_pair(n)
        elif n.kind == N.INPUT:
            old2new[id(n)] = (n, None)
        elif n.kind == N.SUM:
            ch = [old2new[id(c)] for c in n.inputs]
            if all(b is None for _, b in ch):
                old2new[id(n)] = (N.summate(n.inputs, params=n.params), None)     # the old children, as the reference does
            elif id(n) in has_grow_pars:
                chs, p1, p2 = doubled(n)
                old2new[id(n)] = (N.summate(chs, params=_perturb(p1, sigma, rng)), N.summate(chs, params=_perturb(p2, sigma, rng)))
            else:
                chs, params = [], []
                for i, (a, b) in enumerate(ch):
                    if b is None:
                        chs.append(a); params.append(n.params[i])
                    else:
                        r = float(np.clip(rng.random(), 0.1, 0.9))
                        chs += [a, b]
                        params += [n.params[i] + np.log(r), n.params[i] + np.log(1.0 - r)]
                old2new[id(n)] = (N.summate(chs, params=_perturb(np.array(params), sigma, rng)), None)
        else:
            old2new[id(n)] = mul_pair(n)

    new_pcs = [old2new[id(p)][0] for p in pcs]
    grown = [old2new[id(p)][1] for p in pcs if old2new[id(p)][1] is not None]
    return new_pcs + grown
