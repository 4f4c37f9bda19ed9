"""Circuits as `.jpc` text files: what `write(file, pc)` / `read(file, ProbCircuit)` of
ProbabilisticCircuits.jl are to the reference, and its two multi-head wrappers
(src-jl/multi_head_pc/io.jl:2-9: `write_mhpc` stores `summate(pcs...)`, `read_mhpc` returns the
children of the root it reads).

The format is line oriented.  Lines starting with `c` are comments; the first other line is
`jpc <number of nodes>`; then one line per node, children before parents, node ids from 0:

    L id vtree literal                      a literal of a binary variable (+v: true, -v: false)
    I id vtree variable value               an indicator (variable == value)
    B id vtree variable N p                 a binomial input
    C id vtree variable logp logp ...       a categorical input, one log-probability per category
    P id vtree n child child ...            a product node
    S id vtree n child logp child logp ...  a sum node, a log-parameter after every child

(`vtree` is the id of the node's vtree node, 0 for circuits without one.)  Variables are
1-based in the file and 0-based in `pcmi355.nodes`; the last node of the file is the root.
This module writes `C`, `P` and `S` lines -- the three node kinds these circuits have -- and
reads those and `L` (as a categorical over two categories with all mass on one); `I` and `B`
inputs have no counterpart among the input nodes of this library and are refused by name.

A file name ending in `.gz` is read and written through gzip, as the reference's test
fixtures are named (test/conditional_pc/custom_em_tests.jl:14).

The grammar above is the published one of ProbabilisticCircuits.jl 0.4; neither that package
nor any `.jpc` file ships with the reference, so files written here are checked against the
grammar and by reading them back, not against files the reference wrote.
"""
import gzip
import io as _io

import re

import numpy as np

from . import nodes as N

_HEADER = """c this file was saved by pcmi355 in the jpc format of ProbabilisticCircuits.jl
c ids of jpc nodes start at 0
c jpc nodes appear bottom-up, children before parents
c
c file syntax:
c jpc count-of-jpc-nodes
c L id-of-jpc-node id-of-vtree literal
c I id-of-jpc-node id-of-vtree variable indicator-value
c B id-of-jpc-node id-of-vtree variable binomial-N binomial-P
c C id-of-jpc-node id-of-vtree variable {log-probability}+
c P id-of-sum-jpc-node id-of-vtree number-of-children {child-id}+
c S id-of-product-jpc-node id-of-vtree number-of-children {child-id log-probability}+
c"""


def _open(file, mode):
    if hasattr(file, "read") or hasattr(file, "write"):
        return file, False
    name = str(file)
    if name.endswith(".gz"):
        return _io.TextIOWrapper(gzip.open(name, mode + "b"), encoding="ascii", newline="\n"), True
    return open(name, mode, encoding="ascii", newline="\n"), True


def _num(x):
    """Shortest text that reads back as the same float32 (`-Inf` as Julia prints it)."""
    x = np.float32(x)
    if np.isinf(x):
        return "-Inf" if x < 0 else "Inf"
    if np.isnan(x):
        raise ValueError("a parameter is NaN")
    return str(x)


def write_jpc(file, pc):
    """`write(file, pc)` with the jpc format: every node reachable from `pc` once, children
    before parents, `pc` itself last."""
    order = N.linearize(pc)
    ids = {id(n): i for i, n in enumerate(order)}
    f, close = _open(file, "w")
    try:
        out = [_HEADER, f"jpc {len(order)}"]
        for i, n in enumerate(order):
            if n.kind == N.INPUT:
                out.append(f"C {i} 0 {n.var + 1} " + " ".join(_num(p) for p in n.logps))
            elif n.kind == N.MUL:
                out.append(f"P {i} 0 {len(n.inputs)} " + " ".join(str(ids[id(c)]) for c in n.inputs))
            else:
                if len(n.params) != len(n.inputs):
                    raise ValueError("a sum node's parameters do not match its children")
                out.append(f"S {i} 0 {len(n.inputs)} " +
                           " ".join(f"{ids[id(c)]} {_num(p)}" for c, p in zip(n.inputs, n.params)))
        f.write("\n".join(out) + "\n")
    finally:
        if close:
            f.close()


_JULIA_F32 = re.compile(r"^[-+]?(\d+\.?\d*|\.\d+)f[-+]?\d+$")


def _logp(tok, where):
    """A log-probability token.  Besides what Python's float() reads, the spellings Julia prints for a Float32:
    an `f` exponent (`-1.0f-5`) and `-Inf32` (ProbabilisticCircuits.jl keeps parameters as Float32)."""
    t = tok.lower()
    if t in ("-inf", "-infinity", "-inf32", "-inf16"):
        return -np.inf
    if _JULIA_F32.match(t):
        t = t.replace("f", "e")
    try:
        return float(t)
    except ValueError:
        raise ValueError(f"{where}: '{tok}' is not a log-probability") from None


def read_jpc(file):
    """`read(file, ProbCircuit)`: the root (last node) of a `.jpc` file as `pcmi355.nodes` objects;
    a node named by several parents is one object, as in the file."""
    f, close = _open(file, "r")
    try:
        text = f.read()
    finally:
        if close:
            f.close()
    count, made = None, {}
    last = None
    for ln, line in enumerate(text.splitlines(), 1):
        tok = line.split()
        if not tok or tok[0] == "c":
            continue
        where = f"line {ln}"
        if count is None:
            if tok[0] != "jpc" or len(tok) != 2 or not tok[1].isdigit():
                raise ValueError(f"{where}: expected 'jpc <number of nodes>'")
            count = int(tok[1])
            continue
        kind = tok[0]
        if kind not in ("L", "I", "B", "C", "P", "S"):
            raise ValueError(f"{where}: unknown node kind '{kind}'")
        try:
            nid = int(tok[1])
            int(tok[2])   # vtree id: not used by circuits without a vtree
        except (IndexError, ValueError):
            raise ValueError(f"{where}: a node line starts with kind, node id and vtree id") from None
        if nid in made:
            raise ValueError(f"{where}: node {nid} is defined twice")
        if nid < 0 or nid >= count:
            raise ValueError(f"{where}: node id {nid} outside 0..{count - 1}")
        rest = tok[3:]

        def child(t):
            if not t.lstrip("-").isdigit() or int(t) not in made:
                raise ValueError(f"{where}: child '{t}' is not a node defined above")
            return made[int(t)]

        if kind == "C":
            if len(rest) < 2 or not rest[0].isdigit() or int(rest[0]) < 1:
                raise ValueError(f"{where}: C takes a variable (from 1) and its log-probabilities")
            node = N.InputNode(int(rest[0]) - 1, [_logp(t, where) for t in rest[1:]])
        elif kind == "L":
            if len(rest) != 1 or not rest[0].lstrip("-").isdigit() or int(rest[0]) == 0:
                raise ValueError(f"{where}: L takes one non-zero literal")
            lit = int(rest[0])
            node = N.InputNode(abs(lit) - 1, [-np.inf, 0.0] if lit > 0 else [0.0, -np.inf])
        elif kind in ("I", "B"):
            raise ValueError(f"{where}: {'indicator' if kind == 'I' else 'binomial'} inputs are not categorical input "
                             "nodes and cannot be read")
        else:
            if not rest or not rest[0].isdigit() or int(rest[0]) < 1:
                raise ValueError(f"{where}: {kind} takes its number of children first")
            n = int(rest[0])
            if kind == "P":
                if len(rest) != 1 + n:
                    raise ValueError(f"{where}: {n} children announced, {len(rest) - 1} ids given")
                node = N.MulNode([child(t) for t in rest[1:]])
            else:
                if len(rest) != 1 + 2 * n:
                    raise ValueError(f"{where}: {n} children announced, {len(rest) - 1} tokens of (child, log-parameter) given")
                node = N.SumNode([child(t) for t in rest[1::2]], [_logp(t, where) for t in rest[2::2]])
        made[nid] = node
        last = node
    if count is None:
        raise ValueError("no 'jpc <number of nodes>' line")
    if len(made) != count:
        raise ValueError(f"{count} nodes announced, {len(made)} defined")
    return last


def write_mhpc(file, pcs):
    """`write_mhpc(file, pcs)` (src-jl/multi_head_pc/io.jl:2-4): the heads of a multi-head circuit
    under one sum node."""
    write_jpc(file, N.summate(list(pcs)))


def read_mhpc(file):
    """`read_mhpc(file)` (src-jl/multi_head_pc/io.jl:6-9): the heads, in the order they were
    written."""
    root = read_jpc(file)
    if root.kind != N.SUM:
        raise ValueError("the root of a multi-head file is the sum node over its heads")
    return list(N.children(root))
