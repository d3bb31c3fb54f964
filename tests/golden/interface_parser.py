"""A small text parser for the C++ declarations that make up the operator / device interface:
free-function prototypes, plain structs with their fields, enum classes, typedefs of
template closures, and the member functions of a class.  It reads header TEXT only (nothing
is compiled or run).  `extract_reference_interface.py` applies it to the reference's headers
and writes interface.json; the CPU tests apply the same functions to this repository's
headers and compare."""
import re


def strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def norm_type(t):
    """One spelling per type: 'DataList const&' == 'const DataList&', no parameter names."""
    t = " ".join(t.replace("&", " & ").replace("*", " * ").split())
    m = re.match(r"^(\w[\w:<>]*) const (.*)$", t)          # east const -> west const
    if m:
        t = "const %s %s" % (m.group(1), m.group(2))
    t = t.replace(" &", "&").replace(" *", "*").replace("& ", "&").replace("* ", "*")
    return t.strip()


def _param_types(params):
    out = []
    for p in [q.strip() for q in params.split(",") if q.strip()]:
        p = re.sub(r"\s*=.*$", "", p)                       # default argument
        m = re.match(r"^(.*?[&*\s])(\w+)$", p)              # trailing parameter name
        if m and m.group(2) not in ("int", "float", "size_t", "bool", "Context", "DataList",
                                    "uint64_t", "unsigned", "double", "char", "const"):
            p = m.group(1)
        out.append(norm_type(p))
    return out


def free_functions(text, namespace):
    """{name: [parameter types]} of the `void name(...)` prototypes in `namespace X { ... }`."""
    text = strip_comments(text)
    m = re.search(r"namespace\s+%s\s*\{(.*?)\n\}" % namespace, text, flags=re.S)
    body = m.group(1) if m else ""
    return {f.group(1): _param_types(f.group(2))
            for f in re.finditer(r"\bvoid\s+(\w+)\s*\(([^)]*)\)\s*;", body)}


def structs(text):
    """{struct name: [[type, field], ...]} for plain and `template<int i>` structs, with the
    typedefs of template instances resolved to their own names; multi-declarator fields
    ('float mu, var;') are split."""
    text = strip_comments(text)
    found, templates = {}, set()
    for m in re.finditer(r"(template\s*<[^>]*>\s*)?struct\s+(\w+)\s*\{([^{}]*)\}\s*;", text):
        fields = []
        for decl in m.group(3).split(";"):
            decl = " ".join(decl.split())
            if not decl or "(" in decl:
                continue
            d = re.match(r"^(.*?)\s+([\w\s,]+)$", decl)
            for name in d.group(2).split(","):
                fields.append([norm_type(d.group(1)), name.strip()])
        found[m.group(2)] = fields
        if m.group(1):
            templates.add(m.group(2))
    for m in re.finditer(r"typedef\s+(\w+)\s*<[^>]*>\s+(\w+)\s*;", text):
        if m.group(1) in templates:
            found[m.group(2)] = found[m.group(1)]
    for t in templates:
        del found[t]
    return found


def enums(text):
    """{enum class name: [enumerators]}"""
    text = strip_comments(text)
    out = {}
    for m in re.finditer(r"enum\s+class\s+(\w+)\s*\{([^}]*)\}", text):
        out[m.group(1)] = [re.sub(r"\s*=.*$", "", e).strip() for e in m.group(2).split(",") if e.strip()]
    return out


def class_methods(text, cls):
    """Member functions of `class cls`: {name: {"ret", "params", "virtual", "pure", "const",
    "override", "access"}} (constructors, destructors and deleted members left out)."""
    text = strip_comments(text)
    m = re.search(r"class\s+%s\b[^{;]*\{" % cls, text)
    if not m:
        return None
    depth, i = 1, m.end()
    while depth and i < len(text):
        depth += {"{": 1, "}": -1}.get(text[i], 0)
        i += 1
    body = text[m.end(): i - 1]
    body = re.sub(r"\{[^{}]*\}", ";", body)                 # inline bodies and nested structs
    body = re.sub(r"\{[^{}]*\}", ";", body)
    base = re.search(r"class\s+%s\s*:\s*public\s+(\w+)" % cls, text)
    methods, access = {}, "private"
    for stmt in re.split(r";|(?=\b(?:public|protected|private)\s*:)", body):
        stmt = " ".join(stmt.split())
        a = re.match(r"^(public|protected|private)\s*:\s*(.*)$", stmt)
        if a:
            access, stmt = a.group(1), a.group(2)
        f = re.match(r"^(virtual\s+)?(static\s+)?([\w:<>,\s&*]+?)\s+(\w+)\s*\(([^)]*)\)\s*(const)?\s*"
                     r"(override)?\s*(=\s*0)?$", stmt)
        if not f or f.group(4) == cls or "delete" in stmt or "DISALLOW" in stmt:
            continue
        methods[f.group(4)] = {"ret": norm_type(f.group(3)), "params": _param_types(f.group(5)),
                               "virtual": bool(f.group(1)), "pure": bool(f.group(8)),
                               "const": bool(f.group(6)), "override": bool(f.group(7)),
                               "access": access}
    return {"base": base.group(1) if base else None, "methods": methods}
