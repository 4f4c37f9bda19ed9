"""Circuits as DAGs on the host: what ProbabilisticCircuits.jl's `PlainSumNode`, `PlainMulNode`
and `PlainInputNode` are to the reference (its structure builders, `prune_pc` and
`grow_heads_by_flows` work on them and compile the result with `CuMultiHeadBitsProbCircuit`).
Variables and categories are 0-based here; log-parameters are float32.

Traversals are iterative: a Chow-Liu tree of a few thousand variables is deeper than Python's
recursion limit.
"""
import numpy as np

INPUT, SUM, MUL = 0, 1, 2


class ProbCircuit:
    __slots__ = ("inputs",)
    kind = None


class InputNode(ProbCircuit):
    """`PlainInputNode(var, Categorical(logps))`."""
    __slots__ = ("var", "logps")
    kind = INPUT

    def __init__(self, var, logps):
        self.inputs = []
        self.var = int(var)
        self.logps = np.array(logps, dtype=np.float32)
        if self.logps.ndim != 1 or len(self.logps) < 1:
            raise ValueError("logps must be a non-empty vector")


class SumNode(ProbCircuit):
    __slots__ = ("params",)
    kind = SUM

    def __init__(self, inputs, params=None):
        self.inputs = list(inputs)
        if not self.inputs:
            raise ValueError("a sum node needs children")
        n = len(self.inputs)
        self.params = np.full(n, -np.log(n), np.float32) if params is None else np.array(params, dtype=np.float32)
        if self.params.shape != (n,):
            raise ValueError(f"{n} children but {self.params.shape} parameters")


class MulNode(ProbCircuit):
    __slots__ = ()
    kind = MUL

    def __init__(self, inputs):
        self.inputs = list(inputs)
        if not self.inputs:
            raise ValueError("a product node needs children")


def _flat(children):
    if len(children) == 1 and isinstance(children[0], (list, tuple)):
        return list(children[0])
    return list(children)


def input_node(var, logps):
    return InputNode(var, logps)


def categorical(var, num_cats):
    """`PlainInputNode(var, Categorical(num_cats))`: uniform."""
    return InputNode(var, np.full(num_cats, -np.log(num_cats), np.float32))


def summate(*children, params=None):
    """`summate(children...)` / `summate(children::Vector)`: uniform parameters unless given."""
    return SumNode(_flat(children), params)


def multiply(*children):
    return MulNode(_flat(children))


def isinput(n):
    return n.kind == INPUT


def issum(n):
    return n.kind == SUM


def ismul(n):
    return n.kind == MUL


def isinner(n):
    return n.kind != INPUT


def children(n):
    return n.inputs


def num_children(n):
    return len(n.inputs)


def randvar(n):
    return n.var


def _roots(pcs):
    return list(pcs) if isinstance(pcs, (list, tuple)) else [pcs]


def linearize(pcs):
    """Every node reachable from the roots once, children before parents, depth-first from the
    first root with children in order (the order of `foreach`,
    src-jl/multi_head_pc/transformation.jl:9-32)."""
    order, seen = [], set()
    for r in _roots(pcs):
        if id(r) in seen:
            continue
        stack = [(r, 0)]
        seen.add(id(r))
        while stack:
            n, i = stack[-1]
            if i < len(n.inputs):
                stack[-1] = (n, i + 1)
                c = n.inputs[i]
                if id(c) not in seen:
                    seen.add(id(c))
                    stack.append((c, 0))
            else:
                order.append(n)
                stack.pop()
    return order


def foreach(f, pcs):
    for n in linearize(pcs):
        f(n)


def foreach_down(f, pcs):
    """Parents before children (transformation.jl:34-40)."""
    for n in reversed(linearize(pcs)):
        f(n)


def foldup_aggregate(root, f_input, f_mul, f_sum):
    """`foldup_aggregate(root, f_i, f_m, f_s, T)`: bottom-up fold with the children's results
    handed to the inner callbacks; every node is visited once."""
    out = {}
    for n in linearize(root):
        if n.kind == INPUT:
            out[id(n)] = f_input(n)
        else:
            ins = [out[id(c)] for c in n.inputs]
            out[id(n)] = f_mul(n, ins) if n.kind == MUL else f_sum(n, ins)
    return out[id(root)]


def num_nodes(pcs):
    return len(linearize(pcs))


def num_edges(pcs):
    return sum(len(n.inputs) for n in linearize(pcs))


def num_parameters(pcs):
    """Free parameters (transformation.jl:58-75): one less than the children of every sum node
    and the categories of every input node."""
    total = 0
    for n in linearize(pcs):
        if n.kind == SUM:
            total += len(n.params) - 1
        elif n.kind == INPUT:
            total += len(n.logps) - 1
    return total


def init_parameters(pcs, perturbation=0.0, rng=None):
    """`init_parameters(pc; perturbation)`: every sum node and every categorical gets weights
    drawn uniformly from [1 - perturbation, 1 + perturbation] and normalised
    (src/nodes/fixable_categorical_dist.jl:31-37 for the inputs; uniform when perturbation
    is 0)."""
    rng = np.random.default_rng() if rng is None else rng

    def draw(n):
        if perturbation == 0.0:
            return np.full(n, -np.log(n), np.float32)
        w = rng.uniform(1.0 - perturbation, 1.0 + perturbation, size=n)
        return np.log(w / w.sum()).astype(np.float32)

    for n in linearize(pcs):
        if n.kind == SUM:
            n.params = draw(len(n.params))
        elif n.kind == INPUT:
            n.logps = draw(len(n.logps))


def variables(pcs):
    return sorted({n.var for n in linearize(pcs) if n.kind == INPUT})


def describe(pcs):
    """The flat description `pcm_circuit_create` takes (children before parents, the roots
    last), plus the nodes in that order.  Several roots are the heads of a multi-head circuit
    and must be distinct nodes that are not each other's descendants' parents."""
    roots = _roots(pcs)
    root_ids = {id(r) for r in roots}
    if len(root_ids) != len(roots):
        raise ValueError("the heads must be distinct nodes")
    order = [n for n in linearize(roots) if id(n) not in root_ids] + roots
    index = {id(n): i for i, n in enumerate(order)}
    child_ptr = np.zeros(len(order) + 1, np.int32)
    child_idx, sum_logp, input_logp = [], [], []
    num_cats = None
    for i, n in enumerate(order):
        for q, c in enumerate(n.inputs):
            if index[id(c)] >= i:
                raise ValueError("a head is a descendant of another node of the circuit")
            child_idx.append(index[id(c)])
        if n.kind == SUM:
            if len(n.params) != len(n.inputs):
                raise ValueError("a sum node's parameters do not match its children")
            sum_logp.append(n.params)
        elif n.kind == MUL:
            sum_logp.append(np.zeros(len(n.inputs), np.float32))
        else:
            if num_cats is None:
                num_cats = len(n.logps)
            elif len(n.logps) != num_cats:
                raise ValueError("all input nodes must have the same number of categories")
            input_logp.append(n.logps)
        child_ptr[i + 1] = len(child_idx)
    if num_cats is None:
        raise ValueError("the circuit has no input nodes")
    desc = dict(node_type=np.array([n.kind for n in order], np.uint8), child_ptr=child_ptr,
                child_idx=np.array(child_idx, np.int32),
                sum_logp=(np.concatenate(sum_logp) if sum_logp else np.zeros(0)).astype(np.float32),
                input_var=np.array([n.var if n.kind == INPUT else -1 for n in order], np.int32),
                input_logp=np.concatenate(input_logp).astype(np.float32), num_cats=num_cats)
    return desc, order
