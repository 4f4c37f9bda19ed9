"""`.jpc` files (pcmi355.jpc_io): the grammar as published for ProbabilisticCircuits.jl, the
multi-head wrappers of src-jl/multi_head_pc/io.jl:2-9, and what a malformed file raises.  No
`.jpc` file ships with the reference, so the fixtures here are written out by hand from the
grammar; files the library writes are checked against that grammar and by reading them back."""
import gzip
import io
import re

import numpy as np
import pytest

from pcmi355 import nodes as N
from pcmi355.jpc_io import write_jpc, read_jpc, write_mhpc, read_mhpc
from pcmi355.structures import hclt_pc


def _same_circuit(a, b):
    da, oa = N.describe(a)
    db, ob = N.describe(b)
    assert da.keys() == db.keys()
    for k in da:
        np.testing.assert_array_equal(da[k], db[k], err_msg=k)


HAND_WRITTEN = """c a mixture of two fully factorised distributions over two ternary variables
c
jpc 7
C 0 0 1 -0.5108256 -1.609438 -1.609438
C 1 0 2 -1.203973 -1.203973 -0.9162907
P 2 0 2 0 1
C 3 0 1 -2.302585 -0.3566749 -1.609438
C 4 0 2 -Inf -0.6931472 -0.6931472
P 5 0 2 3 4
S 6 0 2 2 -0.3566749 5 -1.203973
"""


def test_a_file_written_out_by_hand_from_the_grammar():
    root = read_jpc(io.StringIO(HAND_WRITTEN))
    assert root.kind == N.SUM and [c.kind for c in root.inputs] == [N.MUL, N.MUL]
    np.testing.assert_array_equal(root.params, np.float32([-0.3566749, -1.203973]))
    a, b = root.inputs
    assert [(c.kind, c.var) for c in a.inputs] == [(N.INPUT, 0), (N.INPUT, 1)]    # variables are 1-based in the file
    assert [(c.kind, c.var) for c in b.inputs] == [(N.INPUT, 0), (N.INPUT, 1)]
    np.testing.assert_array_equal(a.inputs[0].logps, np.float32([-0.5108256, -1.609438, -1.609438]))
    np.testing.assert_array_equal(b.inputs[1].logps, np.float32([-np.inf, -0.6931472, -0.6931472]))
    # the distribution it stands for: 0.7 * p_a(x1) p_a(x2) + 0.3 * p_b(x1) p_b(x2), here at x = (1, 2)
    p = 0.7 * np.exp(-1.609438) * np.exp(-0.9162907) + 0.3 * np.exp(-0.3566749) * np.exp(-0.6931472)
    val = {}
    for n in N.linearize(root):
        if n.kind == N.INPUT:
            val[id(n)] = float(n.logps[(1, 2)[n.var]])
        elif n.kind == N.MUL:
            val[id(n)] = sum(val[id(c)] for c in n.inputs)
        else:
            val[id(n)] = float(np.log(sum(np.exp(val[id(c)] + w) for c, w in zip(n.inputs, n.params))))
    assert abs(np.exp(val[id(root)]) - p) < 1e-7


def test_log_parameters_in_julia_float32_spelling():
    """Julia prints a Float32 with an `f` exponent and its infinities as `Inf32`; a file written by the reference
    may hold both (ProbabilisticCircuits.jl keeps parameters as Float32)."""
    text = "c a file with Float32 tokens\njpc 4\nC 0 0 1 -1.0f-5 -Inf32 -2.5f0\nC 1 0 1 -Inf -11.512925f0 -1f1\nP 2 0 1 0\nS 3 0 2 2 -6.9077554f-1 2 -0.6955f0\n"
    root = read_jpc(io.StringIO(text))
    np.testing.assert_array_equal(root.params, np.float32([-0.69077554, -0.6955]))
    leaf = root.inputs[0].inputs[0]
    np.testing.assert_array_equal(leaf.logps, np.float32([-1.0e-5, -np.inf, -2.5]))
    with pytest.raises(ValueError, match="not a log-probability"):
        read_jpc(io.StringIO("jpc 1\nC 0 0 1 -1.0g-5 0.0\n"))


def test_literals_read_as_categoricals_over_two_values():
    root = read_jpc(io.StringIO("jpc 3\nL 0 0 2\nL 1 0 -1\nP 2 0 2 0 1\n"))
    pos, neg = root.inputs
    assert pos.var == 1 and neg.var == 0
    np.testing.assert_array_equal(pos.logps, np.float32([-np.inf, 0.0]))
    np.testing.assert_array_equal(neg.logps, np.float32([0.0, -np.inf]))


def test_what_is_written_follows_the_grammar_and_reads_back_as_the_same_circuit(tmp_path):
    rng = np.random.default_rng(5)
    parent = np.array([-1, 0, 0, 1, 1, 1, 2], np.int32)
    pc = hclt_pc(parent, 5, 3)
    N.init_parameters(pc, perturbation=0.4, rng=rng)
    first_input = next(n for n in N.linearize(pc) if n.kind == N.INPUT)
    first_input.logps[2] = -np.inf                       # a category of probability zero
    path = tmp_path / "c.jpc"
    write_jpc(path, pc)
    lines = [l for l in path.read_text().splitlines() if not l.startswith("c")]
    assert lines[0] == f"jpc {N.num_nodes(pc)}"
    num = r"(-?\d+(\.\d+)?([eE][-+]?\d+)?|-Inf)"
    pats = {"C": rf"C \d+ 0 [1-9]\d*( {num})+$", "P": r"P \d+ 0 \d+( \d+)+$", "S": rf"S \d+ 0 \d+( \d+ {num})+$"}
    for i, l in enumerate(lines[1:]):
        assert re.match(pats[l[0]], l), l
        assert int(l.split()[1]) == i                    # ids from 0, in file order
        if l[0] in "PS":                                 # children before parents, announced count is the real one
            tok = l.split()
            kids = tok[4:] if l[0] == "P" else tok[4::2]
            assert len(kids) == int(tok[3]) and all(int(k) < i for k in kids)
    assert any(" -Inf" in l for l in lines)
    back = read_jpc(path)
    _same_circuit(pc, back)
    assert N.num_nodes(back) == N.num_nodes(pc)          # shared nodes stay shared
    # and through gzip, by the file name
    gz = tmp_path / "c.jpc.gz"
    write_jpc(gz, pc)
    assert gzip.open(gz, "rt").read() == path.read_text()
    _same_circuit(pc, read_jpc(gz))


def test_multi_head_files_keep_heads_order_and_sharing(tmp_path):
    from helpers import simple_multihead_circuit, from_oracle_dag
    rng = np.random.default_rng(6)
    heads, _ = from_oracle_dag(simple_multihead_circuit(4, rng))
    heads[1].params = np.log(np.float32([0.25, 0.75]))
    path = tmp_path / "heads.jpc"
    write_mhpc(path, heads)
    back = read_mhpc(path)
    assert len(back) == len(heads)
    _same_circuit(heads, back)
    assert N.num_nodes(back) == N.num_nodes(heads)
    top = read_jpc(path)                                  # io.jl:2-4: one sum node over the heads
    assert top.kind == N.SUM and len(top.inputs) == len(heads)


@pytest.mark.parametrize("text,what", [
    ("C 0 0 1 -0.1 -2.0\n", "expected 'jpc"),
    ("jpc 2\nC 0 0 1 -0.1 -2.0\n", "2 nodes announced, 1 defined"),
    ("jpc 2\nC 0 0 1 -0.1 -2.0\nP 1 0 2 0 5\n", "child '5'"),
    ("jpc 2\nC 0 0 1 -0.1 -2.0\nS 1 0 2 0 -0.5\n", "2 children announced"),
    ("jpc 2\nC 0 0 1 -0.1 -2.0\nC 0 0 2 -0.1 -2.0\n", "defined twice"),
    ("jpc 1\nC 0 0 0 -0.1 -2.0\n", "variable (from 1)"),
    ("jpc 1\nC 0 0 1 -0.1 abc\n", "not a log-probability"),
    ("jpc 1\nI 0 0 1 3\n", "indicator inputs"),
    ("jpc 1\nB 0 0 1 10 0.3\n", "binomial inputs"),
    ("jpc 1\nX 0 0 1\n", "unknown node kind"),
    ("jpc 1\nC 4 0 1 -0.1 -2.0\n", "outside 0..0"),
])
def test_malformed_files_are_refused_by_line(text, what):
    with pytest.raises(ValueError, match=re.escape(what)):
        read_jpc(io.StringIO(text))
