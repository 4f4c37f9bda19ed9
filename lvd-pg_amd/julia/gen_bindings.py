"""Writes LibPCMI355.jl, the raw `ccall` of every entry point include/pcmi355.h declares, from the
header itself: `python lvd-pg_amd/julia/gen_bindings.py`.  One Julia function per entry point,
same name, same arguments in the same order; the functions that return a status keep returning
it (the caller's `check` turns it into an exception).  A maintainer of the Julia host writes the
reference's API over these.  The tests call `render()` and compare it with the committed file, so
the two cannot drift apart."""
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
HEADER = os.path.join(HERE, "..", "..", "include", "pcmi355.h")
OUT = os.path.join(HERE, "LibPCMI355.jl")

_SCALARS = {"int32_t": "Int32", "int64_t": "Int64", "float": "Float32", "int": "Cint", "uint8_t": "UInt8"}
_RETURNS = {"int": "Cint", "int64_t": "Int64", "const char*": "Cstring"}


def declarations(header_text):
    """[(return type, name, [(C type, argument name)])] in header order."""
    text = re.sub(r"/\*.*?\*/", "", header_text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    out = []
    for m in re.finditer(r"(?m)^(const char\*|int64_t|int)\s+(pcm_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text):
        ret, name, args = m.group(1), m.group(2), " ".join(m.group(3).split())
        params = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                am = re.match(r"(.*?)(\w+)$", a)
                params.append((am.group(1).strip().replace(" *", "*"), am.group(2)))
        out.append((ret, name, params))
    return out


def julia_type(ctype):
    t = ctype.replace("const ", "").strip()
    if t in _SCALARS:
        return _SCALARS[t]
    if t == "pcm_circuit**":
        return "Ptr{Ptr{Cvoid}}"
    if t in ("pcm_circuit*", "void*"):
        return "Ptr{Cvoid}"
    if t.endswith("*") and t[:-1] in _SCALARS:
        return "Ptr{%s}" % _SCALARS[t[:-1]]
    raise ValueError(f"no Julia type for '{ctype}'")


def render(header_text):
    lines = ["# Raw bindings of libpcmi355.so: one function per entry point of include/pcmi355.h, same name, same",
             "# arguments.  Written by gen_bindings.py from the header; do not edit by hand.",
             "#",
             "# Pointers named d_* are device addresses (e.g. `Ptr{Float32}(UInt(pointer(x)))` of a ROCArray), the others",
             "# are host arrays or `Ref`s; a null pointer is `C_NULL`.  Status codes are those of `enum pcm_status`;",
             "# `pcm_last_error()` has the message of the last failure on the calling thread.",
             "module LibPCMI355",
             "",
             'const libpcmi355 = get(ENV, "LIBPCMI355", joinpath(@__DIR__, "..", "libpcmi355.so"))',
             ""]
    for ret, name, params in declarations(header_text):
        names = ", ".join(p for _, p in params)
        types = ", ".join(julia_type(t) for t, _ in params)
        if len(params) == 1:
            types += ","
        call = f"ccall((:{name}, libpcmi355), {_RETURNS[ret]}, ({types})" + (f", {names})" if params else ")")
        lines.append(f"{name}({names}) =")
        lines.append(f"    {call}")
    lines += ["", "end # module", ""]
    return "\n".join(lines)


if __name__ == "__main__":
    with open(HEADER) as f:
        text = render(f.read())
    with open(OUT, "w") as f:
        f.write(text)
    print(f"wrote {OUT}")
