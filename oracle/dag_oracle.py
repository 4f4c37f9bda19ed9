"""TEST INFRASTRUCTURE ONLY -- a CPU restatement, on the DAG itself (not on the flattened
circuit), of what the reference's flow-driven structure changes consume and do.  Nothing under
lvd-pg_amd/ may import this.

Works on the `Node` objects of pc_oracle.py (kind / children / logps / var), float64 throughout.

  values, flows        src-jl/multi_head_pc/likelihood.jl:3-18, flow.jl:7-109,141-176 restated as
                       the textbook recursion on the DAG: a sum's value is the logsumexp of
                       (log-weight + child value), a product's the sum of its children's;
                       head h of example b starts with flow mask[b, h]; the flow of a sum edge is
                       flow(parent) * exp(logp + value(child) - value(parent)), a product hands
                       its flow to every child.
                       Pinned (tests/test_transformations.py) by: values equal pc_oracle's
                       flat-circuit forward pass on random DAGs (a different algorithm on a
                       different data structure); the edge flows of a sum node add up to its node
                       flow; summed edge flows equal the central-difference derivative of the
                       total log-likelihood with respect to the edge's log-weight.
  prune                src-jl/multi_head_pc/prune.jl:29-96: keep the sum edges whose flow summed
                       over the data exceeds the threshold (the most probable child where none
                       does), renormalise; a head left with one child gets a copy of that product
                       as a second child.
                       Pinned by: a negative threshold returns a circuit with the same values;
                       the result is normalised (brute-force sum over all assignments of a tiny
                       circuit is 1); exactly the edges above the threshold survive.
Which of two equally probable children the fallback keeps follows numpy's argmax (first), as
Julia's `argmax` does.
"""
import numpy as np

import pc_oracle as O


def topo(roots):
    """children before parents, each node once"""
    order, seen = [], set()
    for r in roots:
        if id(r) in seen:
            continue
        stack = [(r, 0)]
        seen.add(id(r))
        while stack:
            n, i = stack[-1]
            if i < len(n.children):
                stack[-1] = (n, i + 1)
                c = n.children[i]
                if id(c) not in seen:
                    seen.add(id(c))
                    stack.append((c, 0))
            else:
                order.append(n)
                stack.pop()
    return order


def _lse(rows):
    m = np.max(rows, axis=0)
    safe = np.where(np.isfinite(m), m, 0.0)
    return safe + np.log(np.sum(np.exp(rows - safe), axis=0))


def values(roots, data):
    """{id(node): log value per example [B]} for categorical data [B, V]"""
    val = {}
    for n in topo(roots):
        if n.kind == O.INPUT:
            val[id(n)] = np.asarray(n.logps, np.float64)[data[:, n.var]]
        elif n.kind == O.MUL:
            val[id(n)] = np.sum([val[id(c)] for c in n.children], axis=0)
        else:
            val[id(n)] = _lse(np.stack([np.float64(n.logps[i]) + val[id(c)] for i, c in enumerate(n.children)]))
    return val


def flows(heads, data, mask):
    """(node flows {id: [B]}, edge flows {(id(sum), child index): [B]}, values)"""
    val = values(heads, data)
    B = data.shape[0]
    order = topo(heads)
    F = {id(n): np.zeros(B) for n in order}
    for h, r in enumerate(heads):
        F[id(r)] = F[id(r)] + np.asarray(mask[:, h], np.float64)
    E = {}
    for n in reversed(order):
        if n.kind == O.MUL:
            for c in n.children:
                F[id(c)] = F[id(c)] + F[id(n)]
        elif n.kind == O.SUM:
            for i, c in enumerate(n.children):
                with np.errstate(invalid="ignore"):
                    ef = F[id(n)] * np.exp(np.float64(n.logps[i]) + val[id(c)] - val[id(n)])
                ef = np.where(F[id(n)] > 0, ef, 0.0)
                E[(id(n), i)] = ef
                F[id(c)] = F[id(c)] + ef
    return F, E, val


def prune(heads, edge_flow_sums, threshold_count):
    """edge_flow_sums: {(id(sum), child index): flow summed over the data}"""
    new = {}
    for n in topo(heads):
        if n.kind == O.INPUT:
            new[id(n)] = O.input_node(n.var, np.array(n.logps, np.float32))
        elif n.kind == O.MUL:
            new[id(n)] = O.multiply(*[new[id(c)] for c in n.children])
        else:
            idx = [i for i in range(len(n.children)) if len(n.children) > 1 and edge_flow_sums.get((id(n), i), 0.0) > threshold_count]
            if not idx:
                idx = [int(np.argmax(n.logps))]
            lp = np.asarray(n.logps, np.float32)[idx]
            m = np.max(lp)
            lp = lp - np.float32(m + np.log(np.sum(np.exp(lp - m))))
            new[id(n)] = O.summate(*[new[id(n.children[i])] for i in idx], logps=lp)
    out = []
    for r in heads:
        pc = new[id(r)]
        if len(pc.children) == 1 and pc.children[0].kind == O.MUL:
            pc = O.summate(pc.children[0], O.multiply(*pc.children[0].children))
        out.append(pc)
    return out
