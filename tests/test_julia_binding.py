"""Keeps julia/EvoTreesHIP.jl in step with include/evotrees_hip.h without a Julia toolchain: every `ccall` of the module
is parsed and its argument tuple compared with the C prototype it binds (arity and types), the two mirrored structs
are compared field by field, and every `EvoTrees.<name>` the module touches must be tabulated in the integration notes."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
JL = os.path.join(ROOT, "julia", "EvoTreesHIP.jl")
HDR = os.path.join(ROOT, "include", "evotrees_hip.h")
INTEG = os.path.join(ROOT, "INTEGRATION.md")

# Julia ccall type -> canonical form
JL_SCALARS = {"Int64": "i64", "Cint": "i32", "Int32": "i32", "UInt8": "u8", "UInt64": "u64", "UInt32": "u32", "Cdouble": "f64",
              "Float64": "f64", "Float32": "f32", "Cfloat": "f32", "Bool": "u8", "Cvoid": "void", "Cstring": "ptr:char",
              "EvtParams": "evt_params", "EvtTreeOut": "evt_tree_out"}
C_SCALARS = {"int64_t": "i64", "int32_t": "i32", "int": "i32", "uint8_t": "u8", "uint64_t": "u64", "uint32_t": "u32", "double": "f64",
             "float": "f32", "void": "void", "char": "char", "evt_params": "evt_params", "evt_tree_out": "evt_tree_out"}


def strip_comments_c(s):
    s = re.sub(r"/\*.*?\*/", " ", s, flags=re.S)
    return re.sub(r"//[^\n]*", " ", s)


def strip_comments_jl(s):
    return "\n".join(line.split("#", 1)[0] if '"' not in line.split("#", 1)[0] or line.split("#", 1)[0].count('"') % 2 == 0 else line
                     for line in s.splitlines())


def split_top(s, sep=","):
    """Splits at separators that are not nested in (), {} or []."""
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "({[":
            depth += 1
        elif ch in ")}]":
            depth -= 1
        if ch == sep and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur)
    return [x.strip() for x in out]


def balanced(s, start):
    """Index just past the parenthesis that closes the one at s[start]."""
    depth = 0
    for i in range(start, len(s)):
        if s[i] == "(":
            depth += 1
        elif s[i] == ")":
            depth -= 1
            if depth == 0:
                return i + 1
    raise AssertionError("unbalanced parentheses")


def jl_type(t):
    t = t.strip()
    m = re.fullmatch(r"(Ptr|Ref)\{(.*)\}", t)
    if m:
        inner = jl_type(m.group(2))
        # an opaque handle is a pointer to void on both sides
        return "ptr:" + inner
    assert t in JL_SCALARS, "unknown Julia ccall type " + t
    return JL_SCALARS[t]


def c_type(decl):
    """Canonical type of one C parameter declaration (name dropped)."""
    d = decl.replace("const", " ").strip()
    stars = d.count("*")
    d = d.replace("*", " ")
    words = d.split()
    base = words[0]
    if base == "evt_handle":
        base, stars = "void", stars + 1
    else:
        assert base in C_SCALARS, "unknown C type in " + decl
        base = C_SCALARS[base]
    out = base
    for _ in range(stars):
        out = "ptr:" + out
    return out


def c_prototypes():
    s = strip_comments_c(open(HDR).read())
    protos = {}
    for m in re.finditer(r"\b(?:int|const char \*)\s*(evt_[a-z0-9_]+)\s*\(", s):
        end = balanced(s, m.end() - 1)
        args = s[m.end():end - 1].strip()
        protos[m.group(1)] = [] if args in ("", "void") else [c_type(a) for a in split_top(args)]
    return protos


def jl_ccalls():
    s = strip_comments_jl(open(JL).read())
    calls = []
    for m in re.finditer(r"ccall\(\(:(evt_[a-z0-9_]+), LIB\)", s):
        end = balanced(s, m.start() + len("ccall"))
        body = s[m.end():end - 1]
        parts = split_top(body)  # "", return type, (types...), args...
        parts = [p for p in parts if p != ""]
        ret, types = parts[0], parts[1]
        assert types.startswith("(") and types.endswith(")"), "argument tuple of " + m.group(1)
        tl = [t for t in split_top(types[1:-1]) if t]
        calls.append((m.group(1), ret.strip(), [jl_type(t) for t in tl], len(parts) - 2))
    return calls


def compatible(jl, c):
    if jl == c:
        return True
    # Vector{Bool} is handed over as bytes; a Ptr{Cvoid} may stand for any object pointer the caller leaves NULL
    if jl == "ptr:void" and c.startswith("ptr:"):
        return True
    return False


def test_every_ccall_matches_its_prototype():
    protos = c_prototypes()
    calls = jl_ccalls()
    assert len(calls) >= 20
    for name, ret, types, nargs in calls:
        assert name in protos, "%s is not declared in the header" % name
        want = protos[name]
        assert nargs == len(types), "%s: %d arguments passed for %d declared types" % (name, nargs, len(types))
        assert len(types) == len(want), "%s: ccall has %d arguments, the prototype %d" % (name, len(types), len(want))
        for k, (a, b) in enumerate(zip(types, want)):
            assert compatible(a, b), "%s argument %d: Julia %s, C %s" % (name, k + 1, a, b)
        assert ret == ("Cstring" if name == "evt_last_error" else "Cint"), name


def c_struct(name):
    s = strip_comments_c(open(HDR).read())
    m = re.search(r"typedef struct \{([^}]*)\}\s*" + name + r"\s*;", s)
    assert m, name
    fields = []
    for decl in m.group(1).split(";"):
        decl = decl.strip()
        if decl:
            fields.append((re.findall(r"[A-Za-z_0-9]+", decl)[-1], c_type(decl)))
    return fields


def jl_struct(name):
    s = strip_comments_jl(open(JL).read())
    m = re.search(r"\bstruct " + name + r"\b(.*?)\nend", s, flags=re.S)
    assert m, name
    fields = []
    for line in m.group(1).splitlines():
        line = line.strip()
        if "::" in line:
            f, t = line.split("::")
            fields.append((f.strip(), jl_type(t.strip())))
    return fields


def test_mirrored_structs_have_the_same_fields():
    for jl, c in (("EvtParams", "evt_params"), ("EvtTreeOut", "evt_tree_out")):
        a, b = jl_struct(jl), c_struct(c)
        assert [f for f, _ in a] == [f for f, _ in b], "%s: field names / order differ" % jl
        for (f, ta), (_, tb) in zip(a, b):
            assert compatible(ta, tb) or (ta, tb) == ("ptr:u8", "ptr:u8"), "%s.%s: Julia %s, C %s" % (jl, f, ta, tb)


def test_parser_notices_a_changed_prototype():
    """The guard itself: an argument added to a prototype, or a changed type, must be reported."""
    protos = c_prototypes()
    name, ret, types, nargs = next(c for c in jl_ccalls() if c[0] == "evt_grow_tree")
    assert len(types) == len(protos[name])
    assert not compatible("i32", "i64") and not compatible("ptr:f32", "ptr:f64") and not compatible("u8", "i32")
    assert len(types) != len(protos[name] + ["i32"])


def test_every_reference_name_is_tabulated():
    """Every EvoTrees.<name> the module extends or calls appears in the integration notes at the repository root."""
    s = strip_comments_jl(open(JL).read())
    names = set(re.findall(r"\bEvoTrees\.([A-Za-z_!][A-Za-z_0-9!]*)", s)) - {"Random", "Tables"}
    doc = open(INTEG).read()
    missing = sorted(n for n in names if n not in doc)
    assert not missing, "not tabulated in the integration notes: " + ", ".join(missing)
