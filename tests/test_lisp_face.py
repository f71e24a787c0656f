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
        wanted |= set(re.findall(r"((?:cl-waffe2|gpt-2-example)[a-z0-9./-]*)::([a-zA-Z0-9*%+<>=!?-]+)", text))
    assert wanted and any(pkg == "gpt-2-example" for pkg, _ in wanted)
    sources = ""
    for top in ("source", "examples/gpt-2"):
        for dirpath, _, files in os.walk(os.path.join(REFERENCE, top)):
            for f in files:
                if f.endswith(".lisp"):
                    sources += open(os.path.join(dirpath, f), errors="ignore").read().lower()
    missing = [f"{pkg}::{sym}" for pkg, sym in sorted(wanted) if sym.lower() not in sources]
    assert not missing, missing


# ---- which operators the glue calls, and whether anything defines them --------------------------------------
# A small code walker: it knows the binding forms the glue uses (let, flet, loop, the CFFI and cl-waffe2 macros
# with their own syntax ...) well enough to tell a form in operator position from data, and returns the symbols
# found there.  It raises on a macro it does not know rather than guess.

def tokenize_quotes(text):
    """Like tokenize(), but ' ` , ,@ and #' stay as tokens of their own."""
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
        elif text.startswith("#'", i):
            tokens.append("#'")
            i += 2
        elif ch == '"':
            j = i + 1
            while text[j] != '"':
                j += 2 if text[j] == "\\" else 1
            tokens.append(text[i:j + 1])
            i = j + 1
        elif ch in "()'`":
            tokens.append(ch)
            i += 1
        elif ch == ",":
            if text.startswith(",@", i):
                tokens.append(",@")
                i += 2
            else:
                tokens.append(",")
                i += 1
        else:
            j = i
            while j < n and not text[j].isspace() and text[j] not in "()\";'`,":
                j += 1
            tokens.append(text[i:j])
            i = j
    return tokens


_WRAP = {"'": "quote", "`": "quasiquote", ",": "unquote", ",@": "unquote-splicing", "#'": "function"}


def read_forms_quotes(text):
    tokens = tokenize_quotes(text)
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
        if tok in _WRAP:
            return [_WRAP[tok], parse()]
        return tok

    forms = []
    while pos < len(tokens):
        forms.append(parse())
    return forms


def _is_symbol(x):
    return isinstance(x, str) and not (x.startswith('"') or x.startswith("#\\") or x.startswith(":") or
                                       x.startswith("#:") or re.fullmatch(r"[-+]?[0-9.]+(d0|e[0-9]+)?", x))


class Walker:
    def __init__(self):
        self.calls = []          # (operator, local function names in scope)
        self.where = []          # (kind of form, node name, :where form, :forward lambda list)
        self.options = []        # (macro, header options, body options)
        self.defined = set()     # operators the files define at top level
        self.bypassed = []       # (name, replacement) of define-bypass
        self.in_macro = 0        # inside a defmacro / macrolet body a quasiquoted form is code, elsewhere data

    def lambda_list(self, ll, env):
        for item in ll:
            if isinstance(item, list) and len(item) >= 2:  # (var default [supplied-p]) or ((keyword var) default)
                self.code(item[1], env)

    def body(self, forms, env):
        for f in forms:
            self.code(f, env)

    def plist_forms(self, items, env, kind, name):
        """:forward ((lambda list) body ...) and friends of define-op / define-impl-op / define-impl."""
        keys = []
        where = forward_ll = None
        for k, v in zip(items[::2], items[1::2]):
            keys.append(k.lower())
            if k.lower() in (":forward", ":backward"):
                self.lambda_list(v[0], env)
                self.body(v[1:], env)
                if k.lower() == ":forward":
                    forward_ll = v[0]
            elif k.lower() == ":where":
                where = v
            elif k.lower() == ":slots":
                for slot in v:
                    opts = slot[1:]
                    for ok, ov in zip(opts[::2], opts[1::2]):
                        if ok.lower() == ":initform":
                            self.code(ov, env)
                        if ok.lower() in (":accessor", ":reader", ":writer"):
                            self.defined.add(ov.lower())
        assert len(items) % 2 == 0, f"{kind} {name}: options are not keyword / value pairs"
        if where is not None:
            self.where.append((kind, name, where, forward_ll))
        return keys

    def code(self, f, env):
        if not isinstance(f, list) or not f:
            return
        head = f[0]
        if isinstance(head, list):      # ((lambda ...) args) or a list of forms in a template
            self.body(f, env)
            return
        if not _is_symbol(head):        # (:struct view2), (1 2 3), ("..." ...): data
            return
        h = head.lower()
        rest = f[1:]
        if h in ("quote", "declare", "declaim", "in-package", "defpackage", "defcfun", "defcstruct",
                 "define-foreign-library", "use-foreign-library", "defgeneric", "defstruct", "deftype"):
            if h == "defcfun":
                name = rest[0][1] if isinstance(rest[0], list) else rest[0].strip('"').replace("_", "-")
                self.defined.add(name.lower())
            if h == "defstruct":
                self.struct(rest)
            if h == "defgeneric":
                self.defined.add(rest[0].lower())
            return
        if h == "quasiquote":
            if self.in_macro:
                self.code(rest[0], env)
            else:
                self.unquoted(rest[0], env)
            return
        if h in ("unquote", "unquote-splicing"):
            self.code(rest[0], env)
            return
        if h == "function":
            if isinstance(rest[0], list):
                self.code(rest[0], env)
            else:
                self.calls.append((rest[0], env))
            return
        if h in ("let", "let*", "symbol-macrolet"):
            for b in rest[0]:
                if isinstance(b, list) and len(b) > 1:
                    self.code(b[1], env)
            self.body(rest[1:], env)
        elif h in ("flet", "labels", "macrolet"):
            names = frozenset(d[0].lower() for d in rest[0])
            inner = env | names
            self.in_macro += h == "macrolet"
            for d in rest[0]:
                self.lambda_list(d[1], inner)
                self.body(d[2:], inner if h != "flet" else env)
            self.in_macro -= h == "macrolet"
            self.body(rest[1:], inner)
        elif h == "lambda":
            self.lambda_list(rest[0], env)
            self.body(rest[1:], env)
        elif h in ("defun", "defmacro"):
            if isinstance(rest[0], str):
                self.defined.add(rest[0].lower())
            self.in_macro += h == "defmacro"
            self.lambda_list(rest[1], env)
            self.body(rest[2:], env)
            self.in_macro -= h == "defmacro"
        elif h == "defmethod":
            if isinstance(rest[0], str):
                self.defined.add(rest[0].lower())
            i = 1
            while not isinstance(rest[i], list):
                i += 1                  # qualifiers
            self.lambda_list([a for a in rest[i] if not (isinstance(a, list) and _is_symbol(a[0]) and
                                                       len(a) == 2 and not isinstance(a[1], list))], env)
            self.body(rest[i + 1:], env)
        elif h in ("defparameter", "defvar", "defconstant"):
            self.body(rest[1:2], env)
        elif h == "defclass":
            for slot in rest[2]:
                opts = slot[1:] if isinstance(slot, list) else []
                for ok, ov in zip(opts[::2], opts[1::2]):
                    if ok.lower() == ":initform":
                        self.code(ov, env)
                    if ok.lower() in (":accessor", ":reader", ":writer"):
                        self.defined.add(ov.lower())
        elif h == "define-condition":
            for slot in rest[2]:
                opts = slot[1:] if isinstance(slot, list) else []
                for ok, ov in zip(opts[::2], opts[1::2]):
                    if ok.lower() in (":accessor", ":reader"):
                        self.defined.add(ov.lower())
            for opt in rest[3:]:
                self.body(opt[1:], env)
        elif h == "cond":
            for clause in rest:
                self.body(clause, env)
        elif h in ("case", "ecase", "ccase", "typecase", "etypecase", "ctypecase"):
            self.code(rest[0], env)
            for clause in rest[1:]:
                self.body(clause[1:], env)
        elif h in ("multiple-value-bind", "destructuring-bind"):
            if h == "destructuring-bind":
                self.lambda_list(rest[0], env)
            self.code(rest[1], env)
            self.body(rest[2:], env)
        elif h in ("dolist", "dotimes"):
            self.body(rest[0][1:], env)
            self.body(rest[1:], env)
        elif h == "loop":
            skip = False
            for item in rest:
                if skip and isinstance(item, list):
                    skip = False        # a destructuring pattern after for / with
                    continue
                skip = isinstance(item, str) and item.lower() in ("for", "as", "with")
                self.code(item, env)
        elif h in ("with-slots",):
            self.code(rest[1], env)
            self.body(rest[2:], env)
        elif h == "handler-case":
            self.code(rest[0], env)
            for clause in rest[1:]:
                self.body(clause[2:], env)
        elif h == "the":
            self.code(rest[1], env)
        elif h == "eval-when":
            self.body(rest[1:], env)
        elif h in ("with-foreign-object", "cffi:with-foreign-object", "with-pointer-to-vector-data"):
            self.calls.append((head, env))
            self.body(rest[0][1:], env)
            self.body(rest[1:], env)
        elif h == "with-foreign-objects":
            self.calls.append((head, env))
            for b in rest[0]:
                self.body(b[1:], env)
            self.body(rest[1:], env)
        elif h == "with-foreign-pointer-as-string":
            self.calls.append((head, env))
            spec = rest[0][0] if isinstance(rest[0][0], list) else rest[0]
            self.body(spec[1:2], env)
            self.body(rest[1:], env)
        elif h in ("with-setting-save4bw", "with-reading-save4bw"):
            self.calls.append((head, env))
            if h == "with-setting-save4bw":
                for b in rest[0]:
                    self.code(b[1], env)
            self.body(rest[1:], env)
        elif h in ("define-op", "define-impl-op", "define-impl", "defnode"):
            self.calls.append((head, env))
            header = rest[0]
            name = header[0]
            if h in ("define-op", "defnode"):
                assert isinstance(header[1], list), f"{h} {name}: (self ...) expected"
                keys = self.plist_forms(header[2:], env, h, name)
                self.options.append((h, keys, []))
                self.defined.add(name.lower())
            else:
                hk = [k.lower() for k in header[1::2]]
                for v in header[2::2]:
                    self.code(v, env)
                keys = self.plist_forms(rest[1:], env, h, name)
                self.options.append((h, hk, keys))
        elif h == "define-bypass":
            self.calls.append((head, env))
            self.bypassed.append((rest[1], rest[2]))
        else:
            self.calls.append((head, env))
            self.body(rest, env)

    def unquoted(self, f, env):
        """A quasiquoted datum: only what is unquoted inside it is code."""
        if isinstance(f, list) and f:
            if f[0] in ("unquote", "unquote-splicing"):
                self.code(f[1], env)
            else:
                for x in f:
                    self.unquoted(x, env)

    def struct(self, rest):
        name = rest[0][0] if isinstance(rest[0], list) else rest[0]
        opts = rest[0][1:] if isinstance(rest[0], list) else []
        constructor = f"make-{name}"
        for o in opts:
            if isinstance(o, list) and o[0].lower() == ":constructor":
                constructor = o[1]
        self.defined |= {constructor.lower(), f"{name}-p".lower(), f"copy-{name}".lower()}
        for slot in rest[1:]:
            if isinstance(slot, str) and slot.startswith('"'):
                continue
            self.defined.add(f"{name}-{slot[0] if isinstance(slot, list) else slot}".lower())


def walk_glue():
    w = Walker()
    for path in sorted(glob.glob(os.path.join(LISP_DIR, "*.lisp"))):
        for form in read_forms_quotes(open(path).read()):
            w.code(form, frozenset())
    return w


def _bind(ll, args, out):
    """Required and &optional parameters of a macro lambda list (destructuring included) against a call's arguments."""
    i = 0
    for item in ll:
        if isinstance(item, str) and item.startswith("&"):
            if item.lower() == "&optional":
                continue
            break
        if i >= len(args):
            break
        if isinstance(item, list) and not (len(item) == 2 and isinstance(item[0], str) and isinstance(args[i], str)):
            if isinstance(args[i], list):
                _bind(item, args[i], out)
        else:
            out[(item[0] if isinstance(item, list) else item).lower()] = args[i]
        i += 1


def _exporting_macros(forms):
    """{macro name: (lambda list, [resolver])} for every defmacro / macrolet definition whose template says
    (export ',param): the resolver turns a call's bindings into the exported name -- the parameter itself, or
    a (symb a 'b ...) concatenation bound by a let inside the macro (source/base-impl/mathematics.lisp:13-20)."""
    found = {}
    for form in (x for f in forms for x in walk(f)):
        defs = []
        if form and form[0] == "defmacro" and len(form) > 3:
            defs = [form[1:]]
        elif form and form[0] == "macrolet" and len(form) > 1 and isinstance(form[1], list):
            defs = [d for d in form[1] if isinstance(d, list) and len(d) > 2]
        for d in defs:
            name, ll, body = d[0], d[1], d[2:]
            if not isinstance(name, str) or not isinstance(ll, list):
                continue
            lets = {}
            params = []
            for x in (y for b in body for y in walk(b)):
                if x and x[0] in ("let", "let*") and len(x) > 1 and isinstance(x[1], list):
                    for b in x[1]:
                        if isinstance(b, list) and len(b) == 2 and isinstance(b[1], list) and b[1] and b[1][0] == "symb":
                            lets[b[0].lower()] = b[1][1:]
                if len(x) == 2 and x[0] == "export" and isinstance(x[1], list) and x[1][0] == "quote" \
                        and isinstance(x[1][1], list) and x[1][1][0] == "unquote" and isinstance(x[1][1][1], str):
                    params.append(x[1][1][1].lower())
            if params:
                found[name.lower()] = (ll, params, lets)
    return found


def _literal_exports(forms):
    out = set()
    for x in (y for f in forms for y in walk(f)):
        if len(x) == 2 and x[0] == "export" and isinstance(x[1], list) and x[1][0] == "quote":
            what = x[1][1]
            for sym in (what if isinstance(what, list) else [what]):
                if isinstance(sym, str):
                    out.add(sym.lower())
    return out


def reference_packages():
    """{package name or nickname: set of exported names} from the reference's source/, read as text: the :export
    lists of every defpackage, the literal (export '(...)) forms of every file, and the names that macros export
    with (export ',name) for each of their invocations (source/base-impl/arithmetic.lisp:57-60,
    mathematics.lisp:13-20, package.lisp:86-89)."""
    packages, nick = {}, {}
    clean = lambda s: s.lstrip("#").lstrip(":").strip('"').lower()  # noqa: E731
    files = []
    for dirpath, _, names in os.walk(os.path.join(REFERENCE, "source")):
        for fn in sorted(names):
            if fn.endswith(".lisp"):
                files.append(os.path.join(dirpath, fn))
    parsed = {}
    for path in files:
        try:
            parsed[path] = read_forms_quotes(open(path, errors="ignore").read())
        except (IndexError, ValueError):
            continue  # a file this reader cannot follow (reader macros): none of the package files is one
    for path, forms in parsed.items():
        for form in forms:
            if not (isinstance(form, list) and form and isinstance(form[0], str) and form[0].lower() == "defpackage"):
                continue
            name = clean(form[1])
            exports = packages.setdefault(name, set())
            nick[name] = name
            for opt in form[2:]:
                if isinstance(opt, list) and opt and isinstance(opt[0], str):
                    if opt[0].lower() == ":nicknames":
                        for x in opt[1:]:
                            nick[clean(x)] = name
                    if opt[0].lower() == ":export":
                        exports |= {clean(x) for x in opt[1:] if isinstance(x, str)}
    by_package = {}
    for path, forms in parsed.items():
        current = None
        for form in forms:
            if isinstance(form, list) and len(form) == 2 and form[0] == "in-package" and isinstance(form[1], str):
                current = nick.get(clean(form[1]))
        if current:  # files of the reference hold one in-package each
            by_package.setdefault(current, []).append(forms)
    for pkg, file_forms in by_package.items():
        everything = [f for forms in file_forms for f in forms]
        packages[pkg] |= _literal_exports(everything)
        macros = _exporting_macros(everything)
        for call in (x for f in everything for x in walk(f)):
            if call and isinstance(call[0], str) and call[0].lower() in macros:
                ll, params, lets = macros[call[0].lower()]
                bound = {}
                _bind(ll, call[1:], bound)
                for p in params:
                    if isinstance(bound.get(p), str):
                        packages[pkg].add(bound[p].lower())
                    elif p in lets:
                        parts = []
                        for part in lets[p]:
                            if isinstance(part, list) and part[0] == "quote" and isinstance(part[1], str):
                                parts.append(part[1])
                            elif isinstance(part, str) and isinstance(bound.get(part.lower()), str):
                                parts.append(bound[part.lower()])
                            else:
                                parts = None
                                break
                        if parts:
                            packages[pkg].add("".join(parts).lower())
    for alias, name in nick.items():
        packages[alias] = packages[name]
    return packages


# What CFFI exports, of which the glue uses a part (cffi/src/package.lisp; CFFI is a Quicklisp dependency of the
# reference, cl-waffe2.asd, and not vendored in its tree).
CFFI_EXPORTS = {
    "defcfun", "defcstruct", "defcunion", "defctype", "defcenum", "defbitfield", "defcvar", "defcallback", "callback",
    "get-callback", "foreign-funcall", "foreign-funcall-pointer", "foreign-alloc", "foreign-free", "foreign-pointer",
    "foreign-slot-value", "foreign-slot-pointer", "foreign-slot-offset", "foreign-slot-names", "foreign-type-size",
    "foreign-type-alignment", "foreign-symbol-pointer", "foreign-enum-value", "foreign-enum-keyword",
    "foreign-bitfield-value", "foreign-bitfield-symbols", "foreign-string-alloc", "foreign-string-free",
    "foreign-string-to-lisp", "lisp-string-to-foreign", "with-foreign-object", "with-foreign-objects",
    "with-foreign-slots", "with-foreign-string", "with-foreign-strings", "with-foreign-pointer",
    "with-foreign-pointer-as-string", "with-pointer-to-vector-data", "make-shareable-byte-vector", "mem-ref", "mem-aref",
    "mem-aptr", "pointerp", "pointer-eq", "pointer-address", "make-pointer", "null-pointer", "null-pointer-p",
    "inc-pointer", "incf-pointer", "define-foreign-library", "use-foreign-library", "load-foreign-library",
    "load-foreign-library-error", "close-foreign-library", "reload-foreign-libraries", "foreign-library-loaded-p",
    "foreign-library-name", "foreign-library-pathname", "list-foreign-libraries", "convert-to-foreign",
    "convert-from-foreign", "free-converted-object", "translate-to-foreign", "translate-from-foreign",
    "free-translated-object", "define-foreign-type", "define-parse-method", "*foreign-library-directories*",
    "*darwin-framework-directories*", "*default-foreign-encoding*",
}


@pytest.fixture(scope="module")
def glue():
    return walk_glue()


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference checkout is not on this machine")
def test_every_operator_the_glue_calls_is_defined_somewhere(glue):
    """Every unqualified symbol in operator position is a COMMON-LISP symbol, defined in these files (defun, defmacro,
    defgeneric, defmethod, an accessor, a defcfun, a local flet / labels / macrolet), exported by CFFI, or exported
    by one of the packages package.lisp uses; every `pkg:name` is in that package's :export list
    (source/vm/generic-tensor/package.lisp, vm/nodes/package.lisp, base-impl/package.lisp, vm/package.lisp and the
    others, read as text)."""
    cl = pytest.importorskip("pygments.lexers._cl_builtins")
    common_lisp = set(cl.BUILTIN_FUNCTIONS) | set(cl.SPECIAL_FORMS) | set(cl.MACROS)
    assert {"car", "let", "defun", "loop", "setf", "handler-case"} <= common_lisp
    packages = reference_packages()
    package_form = next(f for f in lisp_forms() if f and f[0] == "defpackage")
    used = [u.lstrip(":").lower() for opt in package_form[2:] if opt[0] == ":use" for u in opt[1:]]
    assert used == ["cl", "cffi", "cl-waffe2/vm.generic-tensor", "cl-waffe2/vm.nodes", "cl-waffe2/base-impl", "cl-waffe2/vm"]
    inherited = set()
    for u in used[2:]:
        assert u in packages and packages[u], f"no defpackage with an :export list for {u} in the reference"
        inherited |= packages[u]
    unknown, unexported, checked = [], [], 0
    for op, env in glue.calls:
        name = op.lower()
        checked += 1
        if "::" in name:
            continue  # internal symbols: test_internal_symbols_exist_in_the_reference
        if ":" in name:
            pkg, sym = name.split(":")
            if pkg in ("cffi",):
                ok = sym in CFFI_EXPORTS
            elif pkg in ("asdf", "trivial-garbage"):
                ok = True  # Quicklisp dependencies of the reference (cl-waffe2.asd), not in its tree
            else:
                ok = pkg in packages and sym in packages[pkg]
            if not ok:
                unexported.append(op)
            continue
        if not (name in common_lisp or name in env or name in glue.defined or name in CFFI_EXPORTS or name in inherited):
            unknown.append(op)
    assert checked > 1200, checked
    assert not unknown, f"operators nothing defines: {sorted(set(unknown))}"
    assert not unexported, f"pkg:name that pkg does not export: {sorted(set(unexported))}"


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference checkout is not on this machine")
def test_bypassed_functions_and_extended_nodes_are_exported(glue):
    """define-bypass names an exported function of the reference and a replacement these files define; every node a
    define-impl-op / define-impl extends is exported by a package the glue uses (or defined here by define-op)."""
    packages = reference_packages()
    inherited = set().union(*(packages[p] for p in ("cl-waffe2/vm.generic-tensor", "cl-waffe2/vm.nodes",
                                                    "cl-waffe2/base-impl", "cl-waffe2/vm")))
    assert len(glue.bypassed) >= 5
    for name, replacement in glue.bypassed:
        pkg, sym = name.lower().split(":")
        assert sym in packages.get(pkg, ()), f"define-bypass: {name} is not exported"
        assert replacement.lower() in glue.defined, f"define-bypass: {replacement} is not defined here"
    extended = 0
    for form in (x for f in read_forms_quotes("\n".join(open(p).read() for p in sorted(glob.glob(os.path.join(LISP_DIR, "*.lisp")))))
                 for x in walk(f)):
        if form and isinstance(form[0], str) and form[0].lower() in ("define-impl-op", "define-impl"):
            node = form[1][0]
            if isinstance(node, list) or "::" in node:
                continue  # ,node inside a macrolet template: its uses are checked below; pkg::name: the test of internal symbols
            extended += 1
            assert node.lower() in inherited or node.lower() in glue.defined, f"{form[0]}: {node} is neither exported nor defined here"
        if form and isinstance(form[0], str) and form[0].lower() in ("define-arith", "define-math", "define-select", "define-unfold") \
                and not isinstance(form[1], list):
            extended += 1
            assert form[1].lower() in inherited, f"{form[0]}: {form[1]} is not exported by the reference"
    assert extended >= 36, extended


def _macro_keys(text, macro):
    """The &key names of `(defmacro <macro> ((name ... &key a b) &key c d) ...)` in the reference: header keys, body keys."""
    for form in read_forms(text):
        if isinstance(form, list) and len(form) > 2 and form[0] == "defmacro" and form[1] == macro:
            ll = form[2]

            def keys(items):
                out, on = [], False
                for it in items:
                    if isinstance(it, str) and it.startswith("&"):
                        on = it == "&key"
                    elif on:
                        out.append(":" + (it[0] if isinstance(it, list) else it).lower())
                return out
            return keys(ll[0]), keys(ll[1:])
    raise AssertionError(f"defmacro {macro} not found")


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference checkout is not on this machine")
def test_keyword_options_are_ones_the_reference_macros_take(glue):
    """define-op (source/vm/nodes/static-node.lisp:177), define-impl and define-impl-op
    (source/vm/nodes/defnode.lisp:428-671): every keyword the glue passes is named in the macro's lambda list."""
    defnode = open(os.path.join(REFERENCE, "source/vm/nodes/defnode.lisp")).read()
    static = open(os.path.join(REFERENCE, "source/vm/nodes/static-node.lisp")).read()
    allowed = {"define-op": _macro_keys(static, "define-op"), "define-impl": _macro_keys(defnode, "define-impl"),
               "define-impl-op": _macro_keys(defnode, "define-impl-op"), "defnode": _macro_keys(defnode, "defnode")}
    assert ":where" in allowed["define-op"][0] and ":forward" in allowed["define-op"][0]
    assert ":device" in allowed["define-impl-op"][0] and ":forward" in allowed["define-impl-op"][1]
    seen = 0
    for macro, header_keys, body_keys in glue.options:
        head_ok, body_ok = allowed[macro]
        for k in header_keys:
            seen += 1
            assert k in head_ok, f"{macro}: {k} is not in ({' '.join(head_ok)})"
        for k in body_keys:
            seen += 1
            assert k in body_ok, f"{macro}: {k} is not in ({' '.join(body_ok)})"
    assert seen >= 60, seen


def test_where_declarations_are_well_formed_and_match_forward(glue):
    """:where (X[rows cols] G[cols] ... -> OUT[rows cols]) of every define-op: brackets balance, exactly one ->, every
    operand is NAME[subscripts], the operands before -> are the arguments of :forward after `self` (same names, same
    order), and a name that appears after -> with other subscripts than before it is new there (the reference's
    grammar, source/vm/nodes/shape.lisp)."""
    assert len(glue.where) >= 8

    def flatten(x):
        return " ".join(flatten(i) if isinstance(i, list) else i for i in x)

    for kind, name, where, forward_ll in glue.where:
        text = flatten(where)
        assert text.count("[") == text.count("]"), f"{name}: unbalanced brackets in {text}"
        assert text.count("->") == 1, f"{name}: {text}"
        left, right = text.split("->")
        operand = re.compile(r"([A-Za-z][A-Za-z0-9*-]*)\[([^\[\]]*)\]")
        ins, outs = operand.findall(left), operand.findall(right)
        assert operand.sub("", left).strip() == "" and ins, f"{name}: {left!r} is not a list of NAME[...]"
        assert operand.sub("", right).strip() == "" and outs, f"{name}: {right!r} is not a list of NAME[...]"
        names = [n.lower() for n, _ in ins]
        assert len(set(names)) == len(names), f"{name}: an operand is declared twice"
        if forward_ll is not None:
            args = [a.lower() for a in forward_ll if not a.startswith("&")]
            assert args[0] == "self" and args[1:] == names, f"{name}: :forward takes {args[1:]}, :where declares {names}"
        declared = {s for _, subs in ins for s in subs.split()}
        for n, subs in outs:
            for s in subs.split():
                assert s in declared or s == "~" or s.isdigit(), f"{name}: {n}[{subs}] uses {s}, which no input declares"
