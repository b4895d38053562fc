"""Function names a roc_shmem header declares, per side (__host__ / __device__), found by
expanding the header's own function-like macros textually.  Used to write
reference_api_names.json from the reference's public header and, in
tests/test_api_surface.py, to read the same from this repository's headers."""
import re


def names_of(paths):
    txt = "\n".join(open(p).read() for p in paths)
    txt = re.sub(r"//[^\n]*", "", txt)
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    txt = re.sub(r"\\\n", " ", txt)
    macros = {}
    for m in re.finditer(r"#define\s+(\w+)\(([^)]*)\)\s+(.*)", txt):
        macros[m.group(1)] = ([p.strip() for p in m.group(2).split(",")], m.group(3))
    host, device = set(), set()

    def collect(s):
        host.update(re.findall(r"__host__[^;({]*?\b(roc_shmemx?_\w+)\s*\(", s))
        device.update(re.findall(r"__device__[^;({]*?\b(roc_shmemx?_\w+)\s*\(", s))

    plain = re.sub(r"#define[^\n]*", "", txt)
    collect(plain)

    def expand(text, depth=0):
        for m in re.finditer(r"\b(\w+)\(([^()]*)\)", text):
            mac, args = m.group(1), [a.strip() for a in m.group(2).split(",")]
            if mac not in macros:
                continue
            params, body = macros[mac]
            if len(params) != len(args):
                continue
            for p, a in zip(params, args):
                p = re.escape(p)
                body = re.sub(r"##\s*%s\s*##" % p, a, body)
                body = re.sub(r"##\s*%s\b" % p, a, body)
                body = re.sub(r"\b%s\s*##" % p, a, body)
                body = re.sub(r"\b%s\b" % p, a, body)
            body = body.replace("##", "")
            collect(body)
            if depth < 3:
                expand(body, depth + 1)

    expand(plain)
    return sorted(host), sorted(device)


def _param_type(param):
    """'const T *source' -> 'const T *'; 'MPI_Comm comm = X' -> 'MPI_Comm'; 'int' -> 'int'."""
    param = param.split("=")[0].strip()
    m = re.match(r"^(.*?)(\b[A-Za-z_]\w*)?\s*$", param)
    head, last = m.group(1).strip(), m.group(2)
    words = param.replace("*", " * ").replace("&", " & ").split()
    type_words = {"const", "unsigned", "signed", "short", "int", "long", "char", "float", "double", "void",
                  "size_t", "ptrdiff_t", "int32_t", "int64_t", "uint32_t", "uint64_t", "bool"}
    if last is None or last in type_words or not head or (len(words) == 1):
        return " ".join(words)
    if re.match(r"^[\w\s]*$", head) and all(w in ("const",) for w in head.split()):
        return " ".join(words)          # 'const T' and the like: the last word is the type
    return " ".join(head.replace("*", " * ").replace("&", " & ").split())


def declarations_of(paths):
    """[(side, return type, name, [parameter types])] of every roc_shmem function declared."""
    txt = "\n".join(open(p).read() for p in paths)
    txt = re.sub(r"//[^\n]*", "", txt)
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    txt = re.sub(r"\\\n", " ", txt)
    macros = {}
    for m in re.finditer(r"#define\s+(\w+)\(([^)]*)\)\s+(.*)", txt):
        macros[m.group(1)] = ([p.strip() for p in m.group(2).split(",")], m.group(3))
    out = set()
    decl = re.compile(r"__(host|device)__\s+((?:ATTR_NO_INLINE\s+|inline\s+)*)([\w\s\*]+?)\s*\b(roc_shmemx?_\w+)\s*\(([^()]*)\)")

    def collect(s):
        for side, _, ret, name, params in decl.findall(s):
            ret = " ".join(ret.replace("*", " * ").split())
            ret = re.sub(r"\b(inline|ATTR_NO_INLINE)\b\s*", "", ret).strip()
            plist = [p for p in (q.strip() for q in params.split(",")) if p and p != "void"]
            out.add((side, ret, name, tuple(_param_type(p) for p in plist)))

    plain = re.sub(r"#define[^\n]*", "", txt)
    collect(plain)

    def expand(text, depth=0):
        for m in re.finditer(r"\b(\w+)\(([^()]*)\)", text):
            mac, args = m.group(1), [a.strip() for a in m.group(2).split(",")]
            if mac not in macros:
                continue
            params, body = macros[mac]
            if len(params) != len(args):
                continue
            for p, a in zip(params, args):
                p = re.escape(p)
                body = re.sub(r"##\s*%s\s*##" % p, a, body)
                body = re.sub(r"##\s*%s\b" % p, a, body)
                body = re.sub(r"\b%s\s*##" % p, a, body)
                body = re.sub(r"\b%s\b" % p, a, body)
            body = body.replace("##", "")
            collect(body)
            if depth < 3:
                expand(body, depth + 1)

    expand(plain)
    return sorted(out)
