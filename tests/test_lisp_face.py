"""Static checks of the Common Lisp face (cl-waffe2_amd/lisp/) against the C ABI.

No Common Lisp implementation exists where these tests run, so nothing here is
executed: the CFFI declarations of api.lisp are parsed and compared with
include/waffe2_hip.h -- every `defcfun` names a declared function, has its
number of arguments and, position by position, its class of C type; every
`defcstruct` lists the fields of its C struct in order and has its size (the
size the ctypes binding has, which the GPU tests exercise); every `+op+`
constant equals its enumerator.  A swapped or missing argument on that side
would otherwise first show as memory corruption on a user's machine.
"""
import ctypes as C
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "waffe2_hip.h")
LISP_DIR = os.path.join(ROOT, "cl-waffe2_amd", "lisp")
REFERENCE = "/root/reference"


# ---- the header ------------------------------------------------------------------------

def _header_text():
    text = open(HEADER).read()
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def c_class(ctype: str) -> str:
    t = ctype.replace("const", " ").strip()
    if "*" in t:
        return "pointer"
    t = " ".join(t.split())
    return {"long": "long", "int": "int", "int32_t": "int", "float": "float", "double": "double",
            "size_t": "size", "char": "char", "int64_t": "int64", "void": "void",
            "uint8_t": "u8", "int8_t": "i8", "uint16_t": "u16", "int16_t": "i16", "uint32_t": "u32"}[t]


def header_functions():
    """name -> (return class, [argument classes])"""
    out = {}
    for ret, name, args in re.findall(r"\b((?:const\s+)?[A-Za-z_0-9]+\s*\**)\s*(wf2hip_[a-z0-9_]+)\s*\(([^)]*)\)\s*;",
                                      _header_text()):
        args = args.strip()
        classes = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                # drop the parameter name: the last identifier that is not part of the type
                m = re.match(r"(.*?)([A-Za-z_][A-Za-z_0-9]*)$", a)
                ctype = m.group(1) if m and m.group(1).strip() else a
                classes.append(c_class(ctype))
        out[name] = (c_class(ret), classes)
    return out


def header_structs():
    """struct name -> [(field, ctype, count)] in declaration order"""
    out = {}
    for body, name in re.findall(r"typedef\s+struct\s+\w+\s*\{(.*?)\}\s*(wf2hip_\w+)\s*;", _header_text(), flags=re.S):
        fields = []
        for decl in body.split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            m = re.match(r"((?:const\s+)?\w+\s*\*?)\s*(.*)$", decl)
            ctype = m.group(1)
            for item in m.group(2).split(","):
                item = item.strip()
                am = re.match(r"(\w+)\[(\w+)\]$", item)
                if am:
                    count = am.group(2)
                    count = 8 if count == "WF2HIP_MAX_RANK" else int(count)
                    fields.append((am.group(1), ctype.strip(), count))
                else:
                    fields.append((item, ctype.strip(), 1))
        out[name] = fields
    return out


def header_enums():
    return {name: int(value) for name, value in re.findall(r"\b(WF2HIP_[A-Z0-9_]+)\s*=\s*(-?\d+)", _header_text())}


# ---- api.lisp --------------------------------------------------------------------------

def tokenize(text):
    """Strings, `;` comments, #| |# comments and #\\x characters handled before parentheses count."""
    tokens = []
    i, n = 0, len(text)
    while i < n:
        ch = text[i]
        if ch.isspace():
            i += 1
        elif ch == ";":
            while i < n and text[i] != "\n":
                i += 1
        elif text.startswith("#|", i):
            i = text.index("|#", i) + 2
        elif text.startswith("#\\", i):
            j = i + 3
            while j < n and (text[j].isalnum() or text[j] == "-"):
                j += 1
            tokens.append(text[i:j])
            i = j
        elif ch == '"':
            j = i + 1
            while text[j] != '"':
                j += 2 if text[j] == "\\" else 1
            tokens.append(text[i:j + 1])
            i = j + 1
        elif ch in "()":
            tokens.append(ch)
            i += 1
        elif ch in "'`,@":
            i += 1  # quote / quasiquote markers do not change the nesting
        else:
            j = i
            while j < n and not text[j].isspace() and text[j] not in '()";':
                j += 1
            tokens.append(text[i:j])
            i = j
    return tokens


def read_forms(text):
    """A minimal s-expression reader: nested lists of atoms (strings keep their quotes)."""
    tokens = tokenize(text)
    pos = 0

    def parse():
        nonlocal pos
        tok = tokens[pos]
        pos += 1
        if tok == "(":
            items = []
            while tokens[pos] != ")":
                items.append(parse())
            pos += 1
            return items
        return tok

    forms = []
    while pos < len(tokens):
        forms.append(parse())
    return forms


def walk(form):
    if isinstance(form, list):
        yield form
        for f in form:
            yield from walk(f)


def lisp_forms():
    forms = []
    for path in sorted(glob.glob(os.path.join(LISP_DIR, "*.lisp"))):
        forms += read_forms(open(path).read())
    return forms


def lisp_class(t) -> str:
    if isinstance(t, list):
        assert t[0] == ":pointer", t
        return "pointer"
    return {":pointer": "pointer", ":long": "long", ":int": "int", ":int32": "int", ":float": "float",
            ":double": "double", ":size": "size", ":char": "char", ":int64": "int64", ":string": "pointer"}[t]


def defcfuns():
    out = {}
    for f in (x for form in lisp_forms() for x in walk(form)):
        if f and f[0] == "defcfun":
            name = f[1].strip('"')
            out[name] = (lisp_class(f[2]), [lisp_class(a[1]) for a in f[3:]], [a[0] for a in f[3:]])
    return out


def defcstructs():
    out = {}
    for f in (x for form in lisp_forms() for x in walk(form)):
        if f and f[0] == "defcstruct":
            fields = []
            for item in f[2:]:
                if not isinstance(item, list):
                    continue  # a docstring
                count = int(item[item.index(":count") + 1]) if ":count" in item else 1
                fields.append((item[0], item[1], count))
            out[f[1]] = fields
    return out


# ---- the checks ------------------------------------------------------------------------

def test_every_defcfun_matches_its_prototype():
    protos = header_functions()
    assert len(protos) > 100
    funs = defcfuns()
    assert len(funs) >= 40
    for name, (ret, classes, argnames) in funs.items():
        assert name in protos, f"api.lisp binds {name}, which include/waffe2_hip.h does not declare"
        want_ret, want = protos[name]
        assert ret == want_ret, f"{name}: returns {ret} in Lisp, {want_ret} in C"
        assert len(classes) == len(want), f"{name}: {len(classes)} arguments in Lisp, {len(want)} in C"
        for i, (got, exp) in enumerate(zip(classes, want)):
            assert got == exp, f"{name}: argument {i} ({argnames[i]}) is {got} in Lisp, {exp} in C"


SIZES = {":int32": 4, ":int64": 8, ":float": 4, ":double": 8, ":pointer": 8}
C_TO_LISP = {"int32_t": ":int32", "int64_t": ":int64", "float": ":float", "double": ":double"}


def test_every_defcstruct_matches_its_struct(W):
    structs = header_structs()
    lisp = defcstructs()
    pairs = {"view2": ("wf2hip_view2", W.lib.View2), "view3": ("wf2hip_view3", W.lib.View3),
             "matmul-desc": ("wf2hip_matmul_desc", W.lib.MatmulDesc),
             "attention-desc": ("wf2hip_attention_desc", W.lib.AttentionDesc)}
    assert set(lisp) == set(pairs), set(lisp) ^ set(pairs)
    for lname, (cname, ctypes_struct) in pairs.items():
        cfields, lfields = structs[cname], lisp[lname]
        assert len(cfields) == len(lfields), (lname, len(cfields), len(lfields))
        offset = 0
        align = 1
        for (cf, ctype, ccount), (lf, ltype, lcount) in zip(cfields, lfields):
            assert lf.replace("-", "_") == cf, f"{lname}: field {lf} where the C struct has {cf}"
            want = ":pointer" if "*" in ctype else C_TO_LISP[ctype.replace("const", "").strip()]
            assert ltype == want, f"{lname}.{lf}: {ltype} in Lisp, {ctype} in C"
            assert lcount == ccount, f"{lname}.{lf}: count {lcount} in Lisp, {ccount} in C"
            size = SIZES[ltype]
            offset = -(-offset // size) * size  # natural alignment, as CFFI and the C compiler lay it out
            # the ctypes binding is what the GPU tests run against: same offset there
            assert getattr(ctypes_struct, cf).offset == offset, f"{lname}.{lf}: offset {offset} in Lisp"
            offset += size * lcount
            align = max(align, size)
        total = -(-offset // align) * align
        assert total == C.sizeof(ctypes_struct), f"{lname}: {total} bytes in Lisp, {C.sizeof(ctypes_struct)} in C"


def test_every_constant_equals_its_enumerator():
    enums = header_enums()
    consts = {}
    for f in (x for form in lisp_forms() for x in walk(form)):
        if f and f[0] == "defconstant" and re.fullmatch(r"\+[a-z0-9-]+\+", f[1]):
            consts[f[1]] = int(f[2])
    assert len(consts) >= 30
    for name, value in consts.items():
        cname = "WF2HIP_" + name.strip("+").upper().replace("-", "_")
        assert cname in enums, f"{name}: no enumerator {cname} in include/waffe2_hip.h"
        assert enums[cname] == value, f"{name} = {value} in Lisp, {cname} = {enums[cname]} in C"
    # dtype codes of dtype-info (tensor.lisp): (:double (values :double 8 1)) ...
    text = open(os.path.join(LISP_DIR, "tensor.lisp")).read()
    codes = dict(re.findall(r"\(:(double|int32|uint32|int16|uint16|int8|uint8) \(values :\w+ \d+ (\d+)\)\)", text))
    want = {"double": "F64", "int32": "I32", "uint32": "U32", "int16": "I16", "uint16": "U16", "int8": "I8",
            "uint8": "U8"}
    assert set(codes) == set(want)
    for k, v in codes.items():
        assert int(v) == enums["WF2HIP_" + want[k]], k


def test_every_called_binding_is_declared():
    """Every (wf2hip-...) call in the Lisp files has a defcfun (CFFI names them by
    replacing _ with -)."""
    declared = {name.replace("_", "-") for name in defcfuns()}
    used = set()
    for path in glob.glob(os.path.join(LISP_DIR, "*.lisp")):
        text = re.sub(r";[^\n]*", "", open(path).read())
        used |= set(re.findall(r"\((wf2hip-[a-z0-9-]+)", text))
    assert used, "no calls found"
    assert used <= declared, sorted(used - declared)


def test_every_call_passes_as_many_arguments_as_its_binding_takes():
    """(wf2hip-foo a b c) in the glue against the defcfun of wf2hip_foo: the same count."""
    arity = {name.replace("_", "-"): len(classes) for name, (_, classes, _) in defcfuns().items()}
    calls = 0
    for f in (x for form in lisp_forms() for x in walk(form)):
        if f and isinstance(f[0], str) and f[0] in arity:
            calls += 1
            assert len(f) - 1 == arity[f[0]], f"({f[0]} ...) is called with {len(f) - 1} arguments, " \
                                             f"its defcfun takes {arity[f[0]]}"
    assert calls >= 40


def test_nodes_of_the_fused_block_exist_on_both_faces(W):
    """The define-op nodes of fusion.lisp and the node names the Python mirror dispatches through."""
    ops = {f[1][0] for form in lisp_forms() for f in walk(form) if f and f[0] == "define-op"}
    want = {"HIP-Activation-Node", "HIP-Softmax-Node", "HIP-LayerNorm-Node", "HIP-Sum-Node", "HIP-Linear-Node",
            "HIP-Linear-Residual-Node", "HIP-Causal-Softmax-Node", "HIP-Attention-Node"}
    assert want <= ops, want - ops
    assert want <= set(W.nodes.NODE_NAMES), want - set(W.nodes.NODE_NAMES)
    bypassed = {f[2] for form in lisp_forms() for f in walk(form) if f and f[0] == "define-bypass"}
    assert {"cl-waffe2/base-impl:!sum", "cl-waffe2/base-impl:!mean", "cl-waffe2/nn:!softmax",
            "cl-waffe2/nn:!gelu", "cl-waffe2/nn:!relu"} <= bypassed


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference checkout is not on this machine")
def test_internal_symbols_exist_in_the_reference():
    """Symbols the glue reaches with `package::name` are not exported by cl-waffe2, so a
    rename upstream would only show at load time: each must be defined somewhere in the
    reference's sources (as text: nothing is loaded)."""
    wanted = set()
    for path in glob.glob(os.path.join(LISP_DIR, "*.lisp")):
        text = re.sub(r";[^\n]*", "", open(path).read())
        wanted |= set(re.findall(r"(cl-waffe2[a-z0-9./-]*)::([a-zA-Z0-9*%+<>=!?-]+)", text))
    assert wanted
    sources = ""
    for dirpath, _, files in os.walk(os.path.join(REFERENCE, "source")):
        for f in files:
            if f.endswith(".lisp"):
                sources += open(os.path.join(dirpath, f), errors="ignore").read().lower()
    missing = [f"{pkg}::{sym}" for pkg, sym in sorted(wanted) if sym.lower() not in sources]
    assert not missing, missing
