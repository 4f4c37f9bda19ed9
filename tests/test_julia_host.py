"""lvd-pg_amd/julia/PCMI355.jl, the Julia host module with the reference's call signatures.  Julia is not installed
where these tests run, so this reads the file as text: every library call it makes names an entry point that the raw
bindings (LibPCMI355.jl, generated from the header) define, with as many arguments as that binding takes; blocks are
balanced; and every function of the reference's interface for this path is there under its own name."""
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
JDIR = os.path.join(os.path.dirname(HERE), "lvd-pg_amd", "julia")


def _strip(text):
    """Source without comments, docstrings and string literals."""
    text = re.sub(r'"""(?:.|\n)*?"""', '""', text)
    text = re.sub(r'"(?:\\.|[^"\\\n])*"', '""', text)
    return "\n".join(l.split("#", 1)[0] for l in text.splitlines())


def _call_args(src, start):
    """Number of top-level arguments of the call whose '(' is at src[start]."""
    depth, n, seen = 0, 0, False
    for i in range(start, len(src)):
        ch = src[i]
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
            if depth == 0:
                return n + (1 if seen else 0)
        elif ch == "," and depth == 1:
            n += 1
        elif depth == 1 and not ch.isspace():
            seen = True
    raise AssertionError("unbalanced call")


def test_host_module_calls_only_what_the_bindings_define():
    raw = open(os.path.join(JDIR, "LibPCMI355.jl")).read()
    arity = {m.group(1): (len([a for a in m.group(2).split(",") if a.strip()]))
             for m in re.finditer(r"^(pcm_\w+)\(([^)]*)\) =$", raw, re.M)}
    assert len(arity) > 40
    src = _strip(open(os.path.join(JDIR, "PCMI355.jl")).read())
    calls = list(re.finditer(r"LibPCMI355\.(pcm_\w+)\(", src))
    assert len(calls) > 20
    for m in calls:
        name = m.group(1)
        assert name in arity, f"{name} is not an entry point"
        got = _call_args(src, m.end() - 1)
        assert got == arity[name], f"{name}: called with {got} arguments, the binding takes {arity[name]}"


def test_host_module_blocks_are_balanced_and_has_the_reference_interface():
    src = _strip(open(os.path.join(JDIR, "PCMI355.jl")).read())
    opens = len(re.findall(r"(?<![\w.])(?:function|if|for|while|struct|module|let|begin|do|try)(?![\w!])", src))
    opens -= len(re.findall(r"mutable struct", src)) * 0          # `mutable struct` counts once (struct)
    ends = len(re.findall(r"(?<![\w.:])end(?![\w!])", src))
    assert opens == ends, (opens, ends)
    assert src.count("(") == src.count(")") and src.count("[") == src.count("]")
    for name in ("loglikelihoods", "loglikelihood", "probs_flows_circuit", "mini_batch_em_with_reg", "mini_batch_em_beta",
                 "mini_batch_em_for_multihead_pc", "vectorize_parameters", "update_parameters", "kld", "kld_backward",
                 "gumbel_sample", "gumbel_sample_backward", "per_sample_normalized_flows", "normalize_params", "hclt",
                 "hclt_from_clt", "pairwise_MI", "learn_chow_liu_tree", "num_parameters"):
        assert re.search(rf"^(?:function )?{name}\(", src, re.M), name
    # keyword arguments of the EM driver as the reference spells them (src/regularization/reg_em.jl:208-213)
    sig = src[src.index("function mini_batch_em_with_reg("):]
    sig = sig[:sig.index(")\n")]
    for kw in ("batch_size", "pseudocount", "soft_reg", "soft_reg_width", "ent_reg", "param_inertia", "param_inertia_end",
               "flow_memory", "shuffle", "verbose"):
        assert re.search(rf"\b{kw}\b", sig), kw
    # ... and of the interval driver (VariationalJuice.jl/src-jl/learning/em.jl:289-296)
    sig = src[src.index("function mini_batch_em_beta("):]
    sig = sig[:sig.index(")\n")]
    for kw in ("batch_size", "pseudocount", "soft_reg", "soft_reg_width", "param_inertia", "param_inertia_end", "flow_memory",
               "flow_memory_end", "shuffle", "update_interval", "fscale", "verbose"):
        assert re.search(rf"\b{kw}\b", sig), kw
    assert "CUDA" not in src and "AMDGPU" not in src
