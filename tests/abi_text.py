"""Text-level readers for the two descriptions of the C ABI: `include/ophip.h` and the Rust side's
`rust_shim/operators/src/handle/hip/ffi.rs`.  Both are reduced to the same canonical form (Rust spelling of the
types), so that a test can compare them declaration by declaration without a C or a Rust compiler."""
import re

_SCALARS = {
    "void": "c_void", "int": "c_int", "unsigned": "c_uint", "char": "c_char", "float": "f32", "double": "f64", "size_t": "usize",
    "ptrdiff_t": "isize", "uint8_t": "u8", "uint16_t": "u16", "uint32_t": "u32", "uint64_t": "u64", "int32_t": "i32",
    "int64_t": "i64",
}
# typedefs of the header that are plain pointers; the Rust side may spell them either way
_POINTER_ALIASES = {"ophip_stream": "*mut c_void", "ophip_event": "*mut c_void", "ophip_graph": "*mut c_void"}


def _strip_c_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    return re.sub(r"(?m)^[ \t]*#(?:[^\n]*\\\n)*[^\n]*$", " ", text)  # preprocessor lines


def c_type(decl):
    """'const ophip_x *', 'void **' ... -> the Rust spelling ('*const ophip_x', '*mut *mut c_void')."""
    decl = decl.strip()
    stars = decl.count("*")
    base = decl.replace("*", " ").split()
    const = "const" in base
    base = [w for w in base if w not in ("const", "struct", "enum")]
    assert len(base) == 1, decl
    name = _SCALARS.get(base[0], base[0])
    if stars == 0:
        return _POINTER_ALIASES.get(name, name)
    name = _POINTER_ALIASES.get(name, name)
    # only the innermost level carries the const of the declarations this header uses
    out = ("*const " if const else "*mut ") + name
    for _ in range(stars - 1):
        out = "*mut " + out
    return out


def _c_param(p):
    """One C parameter or field declaration -> (name, canonical type)."""
    p = p.strip()
    m = re.match(r"(.*?)\(\s*\*\s*(\w+)\s*\)\s*\((.*)\)$", p)  # function pointer: ret (*name)(params)
    if m:
        ret, name, params = m.groups()
        args = ", ".join(_c_param(a)[1] for a in params.split(","))
        r = c_type(ret)
        return name, "extern \"C\" fn(%s)%s" % (args, "" if r == "c_void" else " -> " + r)
    m = re.match(r"(.*?)(\w+)\s*\[\s*(\d+)\s*\]$", p)  # array field
    if m:
        return m.group(2), "[%s; %s]" % (c_type(m.group(1)), m.group(3))
    m = re.match(r"(.*?)(\w+)$", p)
    assert m, p
    return m.group(2), c_type(m.group(1))


def parse_header(text):
    """-> (structs {name: [(field, type)]}, functions {name: (ret, [types])}, enums {name: {member: value}},
    opaque [names])."""
    text = _strip_c_comments(text)
    structs, functions, enums, opaque = {}, {}, {}, []
    for m in re.finditer(r"typedef\s+struct\s+(\w+)\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        fields = []
        for decl in m.group(2).split(";"):
            decl = " ".join(decl.split())
            if not decl:
                continue
            if "(" in decl:
                fields.append(_c_param(decl))
                continue
            first, *more = [d.strip() for d in decl.split(",")]
            name, ty = _c_param(first)
            fields.append((name, ty))
            fields += [(n, ty) for n in more]  # `int32_t a, b, c;`
        structs[m.group(3)] = fields
    for m in re.finditer(r"typedef\s+struct\s+(\w+)\s+(\w+)\s*;", text):
        opaque.append(m.group(2))
    for m in re.finditer(r"typedef\s+enum\s+(\w+)\s*\{(.*?)\}\s*(\w+)\s*;", text, flags=re.S):
        members, nxt = {}, 0
        for item in m.group(2).split(","):
            item = item.strip()
            if not item:
                continue
            if "=" in item:
                k, v = [s.strip() for s in item.split("=")]
                nxt = int(v, 0)
            else:
                k = item
            members[k] = nxt
            nxt += 1
        enums[m.group(3)] = members
    for m in re.finditer(r"OPHIP_API\s+(.*?)\b(ophip_\w+)\s*\((.*?)\)\s*;", text, flags=re.S):
        ret, name, params = m.groups()
        params = " ".join(params.split())
        args = [] if params in ("", "void") else [_c_param(a)[1] for a in params.split(",")]
        r = c_type(ret)
        functions[name] = ("" if r == "c_void" else r, args)
    return structs, functions, enums, opaque


def _rust_type(t):
    t = " ".join(t.split())
    return re.sub(r"\b(%s)\b" % "|".join(_POINTER_ALIASES), lambda m: _POINTER_ALIASES[m.group(1)], t)


def _split_top(s):
    """Split at commas that are not inside () or []."""
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([":
            depth += 1
        elif ch in ")]":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur)
    return out


def parse_rust_ffi(text):
    """-> (structs, functions, opaque) in the same form as parse_header, with the `verbs!` macro expanded."""
    text = re.sub(r"//[^\n]*", " ", text)
    structs, functions, opaque = {}, {}, []

    def take_fns(block, subst=None):
        for m in re.finditer(r"pub\s+fn\s+(\$?\w+)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", block, flags=re.S):
            name, params, ret = m.groups()
            args = []
            for a in _split_top(params):
                a = a.strip()
                if a:
                    args.append(a.split(":", 1)[1].strip())
            ret = (ret or "").strip()
            if subst:
                name = subst.get(name, name)
                args = [re.sub(r"\$\w+", lambda mm: subst[mm.group(0)], a) for a in args]
            functions[name] = (_rust_type(ret), [_rust_type(a) for a in args])

    macro = re.search(r"macro_rules!\s*verbs\s*\{(.*?)\n\}\n", text, flags=re.S)
    body = text
    if macro:
        body = text.replace(macro.group(0), "")
        params = re.findall(r"\$(\w+):ident", macro.group(1))
        call = re.search(r"verbs!\s*\{(.*?)\}", body, flags=re.S)
        for row in call.group(1).split(";"):
            names = [n.strip() for n in row.split(",") if n.strip()]
            if not names:
                continue
            assert len(names) == len(params), row
            subst = {"$" + p: n for p, n in zip(params, names)}
            take_fns(macro.group(1), subst)
            opaque.append(subst["$op"])
        body = body.replace(call.group(0), "")
    for m in re.finditer(r"pub\s+struct\s+(\w+)\s*\{(.*?)\}", body, flags=re.S):
        fields = []
        for f in _split_top(m.group(2)):
            f = f.strip()
            if not f:
                continue
            name, ty = f.split(":", 1)
            fields.append((name.replace("pub", "").strip(), _rust_type(ty)))
        if [n for n, _ in fields] == ["_opaque"]:
            opaque.append(m.group(1))
        else:
            structs[m.group(1)] = fields
    for m in re.finditer(r"extern\s+\"C\"\s*\{(.*?)\n\}", body, flags=re.S):
        take_fns(m.group(1))
    return structs, functions, opaque
