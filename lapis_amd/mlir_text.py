"""A small reader of MLIR module text: enough structure to tell WHAT a function computes.

The reference lowers whatever module text it is given (python/lapis/KokkosBackend.py:83-127 runs it
through lapis-opt and lapis-translate).  The gfx950 module is prebuilt, so the front door has to
recognise the computation instead: this file parses a module into functions, statements and nested
regions and renders each function in a canonical form in which SSA names, comments, whitespace, the
order of constant definitions, static versus dynamic extents and the NAMES of the functions do not
appear.  Two functions with the same canonical form compute the same thing, operation for operation.
"""
import re

_OPEN = {"(": ")", "[": "]", "{": "}", "<": ">"}
_CLOSE = {v: k for k, v in _OPEN.items()}


class ParseError(Exception):
    pass


def strip_comments(text):
    return re.sub(r"//[^\n]*", "", text)


def _match(text, i):
    """Index just past the bracket that closes the one opening at text[i]; `->`, `>=`, `<=` are no brackets."""
    stack = [_OPEN[text[i]]]
    j = i + 1
    n = len(text)
    while j < n and stack:
        ch = text[j]
        if ch == '"':
            k = text.find('"', j + 1)
            if k < 0:
                raise ParseError("a string that does not end: %r" % text[j:j + 30])
            j = k + 1
            continue
        if ch in ">" and j > 0 and text[j - 1] == "-":
            j += 1
            continue
        if ch in "<>" and j + 1 < n and text[j + 1] == "=":
            j += 2
            continue
        if ch in _OPEN:
            # `<` opens a bracket only where a type or attribute can start
            if ch != "<" or re.search(r"[\w.#!]$", text[:j]):
                stack.append(_OPEN[ch])
        elif ch in _CLOSE and stack and ch == stack[-1]:
            stack.pop()
        j += 1
    if stack:
        raise ParseError("unbalanced %r" % text[i])
    return j


def split_top(text, sep=","):
    """Split at `sep` outside every bracket."""
    out, cur, i = [], "", 0
    while i < len(text):
        ch = text[i]
        if ch in _OPEN and (ch != "<" or re.search(r"[\w.#!]$", text[:i])):
            j = _match(text, i)
            cur += text[i:j]
            i = j
            continue
        if ch == "-" and text[i:i + 2] == "->":
            cur += "->"
            i += 2
            continue
        if ch == sep:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
        i += 1
    if cur.strip():
        out.append(cur.strip())
    return out


# ---- attribute aliases (#name = ...) -------------------------------------------------------------

def read_aliases(text):
    aliases = {}
    for m in re.finditer(r"^\s*(#[\w.$-]+)\s*=\s*", text, re.M):
        i = m.end()
        j = i
        while j < len(text) and text[j] != "\n":
            if text[j] in _OPEN and (text[j] != "<" or re.search(r"[\w.#!]$", text[:j])):
                j = _match(text, j)
            else:
                j += 1
        aliases[m.group(1)] = text[i:j].strip()
    return aliases


def encoding_kind(attr, aliases):
    """'csr' / 'csrv' for the two encodings the module implements with 32-bit positions and coordinates,
    else a description of what was found."""
    seen = set()
    while attr in aliases and attr not in seen:
        seen.add(attr)
        attr = aliases[attr]
    m = re.search(r"map\s*=\s*\(([^)]*)\)\s*->\s*\(([^)]*)\)", attr)
    if not m:
        return "sparse(%s)" % attr.strip()[:40]
    dims = [d.strip() for d in m.group(1).split(",")]
    levels = []
    for lv in m.group(2).split(","):
        if ":" not in lv:
            return "sparse(%s)" % m.group(2)
        d, fmt = [t.strip() for t in lv.split(":", 1)]
        levels.append((d, fmt))
    widths = dict(re.findall(r"(posWidth|crdWidth)\s*=\s*(\d+)", attr))
    if widths.get("posWidth") != "32" or widths.get("crdWidth") != "32":
        return "sparse(position/coordinate width other than 32)"
    order_ok = [d for d, _ in levels] == dims
    fmts = [f for _, f in levels]
    if order_ok and fmts == ["dense", "compressed"]:
        return "csr"
    if order_ok and fmts == ["dense", "compressed", "dense"]:
        return "csrv"
    return "sparse(%s)" % ", ".join("%s : %s" % lv for lv in levels)


def type_kind(ty, aliases):
    """Canonical kind of a value type: 'f64', 'index', 'vec:f64', 'mat:f32', 'csr:f64', 'dense3:f32', ..."""
    ty = ty.strip()
    m = re.match(r"tensor<(.*)>$", ty, re.S)
    if not m:
        return ty
    inner = split_top(m.group(1))
    shape = inner[0]
    dims = re.findall(r"(?:\?|\d+)x", shape)
    elem = re.sub(r"^(?:(?:\?|\d+)x)*", "", shape).strip()
    rank = len(dims)
    if len(inner) > 1:
        return "%s:%s" % (encoding_kind(inner[1], aliases), elem)
    return "%s:%s" % ({0: "scalar_tensor", 1: "vec", 2: "mat"}.get(rank, "dense%d" % rank), elem)


# ---- functions, statements, regions --------------------------------------------------------------

class Function:
    def __init__(self, name, private, args, results, body):
        self.name, self.private, self.args, self.results, self.body = name, private, args, results, body


class Statement:
    def __init__(self, results, op, head, regions):
        self.results, self.op, self.head, self.regions = results, op, head, regions


_STMT_START = re.compile(
    r"(?:(?P<res>%[\w.$-]+(?::\d+)?(?:\s*,\s*%[\w.$-]+(?::\d+)?)*)\s*=\s*)?"
    r"(?P<op>(?:[a-z_][\w]*\.)+[\w]+|return\b|call\b)")


def read_functions(text):
    text = strip_comments(text)
    funcs = []
    for m in re.finditer(r"func\.func\s+(private\s+)?@([\w$.-]+)\s*\(", text):
        i = m.end() - 1
        j = _match(text, i)
        args = []
        for a in split_top(text[i + 1:j - 1]):
            if ":" in a:
                nm, ty = a.split(":", 1)
                args.append((nm.strip(), ty.strip()))
            else:
                args.append((None, a.strip()))  # a declaration lists types only
        k = j
        while k < len(text) and text[k].isspace():
            k += 1
        results = []
        if text[k:k + 2] == "->":
            k += 2
            while text[k].isspace():
                k += 1
            if text[k] == "(":
                e = _match(text, k)
                results = split_top(text[k + 1:e - 1])
                k = e
            else:
                e = k
                while e < len(text) and text[e] not in "{\n":
                    if text[e] in _OPEN and (text[e] != "<" or re.search(r"[\w.#!]$", text[:e])):
                        e = _match(text, e)
                    else:
                        e += 1
                results = [text[k:e].strip()]
                k = e
        while k < len(text) and text[k].isspace():
            k += 1
        if text[k:k + 10] == "attributes":
            k = _match(text, text.index("{", k))
            while k < len(text) and text[k].isspace():
                k += 1
        body = None
        if k < len(text) and text[k] == "{":
            e = _match(text, k)
            body = text[k + 1:e - 1]
        funcs.append(Function(m.group(2), bool(m.group(1)), args, results, body))
    return funcs


def _is_region(inner):
    return bool(re.search(r"\^bb\d+|(?:^|\n|\s)(?:%[\w.$-]+[^=\n]*=\s*)?(?:[a-z_]\w*\.)+\w+\s|return\b", inner))


def read_region(text):
    """Statements of a region: each one's depth-0 text (`head`) and its nested regions."""
    stmts = []
    block_args = []
    i, n = 0, len(text)
    cur = None
    while i < n:
        ch = text[i]
        if ch.isspace():
            if cur:
                cur.head += " "
            i += 1
            continue
        if ch == "^":  # block label with its arguments
            m = re.match(r"\^bb\d+\s*(\(|:)", text[i:])
            if m and m.group(1) == "(":
                e = _match(text, i + m.end() - 1)
                block_args = [a.split(":")[0].strip() for a in split_top(text[i + m.end():e - 1])]
                i = e
                while i < n and text[i] in " :\t":
                    i += 1
            else:
                i += m.end() if m else 1
            continue
        m = _STMT_START.match(text, i)
        at_start = m and (cur is None or not re.search(r"[=,(:]\s*$", cur.head.rstrip() or " "))
        if at_start and not re.search(r"[\w#.!]$", text[:i]):
            res = [r.strip() for r in m.group("res").split(",")] if m.group("res") else []
            cur = Statement(res, m.group("op"), "", [])
            stmts.append(cur)
            i = m.end()
            continue
        if cur is None:
            raise ParseError("text before the first operation: %r" % text[i:i + 30])
        if ch in _OPEN and (ch != "<" or re.search(r"[\w.#!]$", text[:i])):
            e = _match(text, i)
            inner = text[i + 1:e - 1]
            if ch == "{" and _is_region(inner):
                sub, bargs = read_region(inner)
                cur.regions.append((bargs, sub))
                cur.head += " {region} "
            else:
                cur.head += text[i:e]
            i = e
            continue
        cur.head += ch
        i += 1
    return stmts, block_args


# ---- canonical form ------------------------------------------------------------------------------

_VALUE = re.compile(r"%[\w.$-]+(?:#\d+)?")


class Canonicalizer:
    """Renders functions with values numbered in order of definition and callees replaced by their own
    canonical form, so that equal text means equal computation."""

    def __init__(self, text):
        self.text = strip_comments(text)
        self.aliases = read_aliases(self.text)
        self.functions = {f.name: f for f in read_functions(self.text)}
        self._memo = {}

    def public(self):
        return [f for f in self.functions.values() if not f.private]

    def signature(self, f):
        return [type_kind(ty, self.aliases) for _, ty in f.args], [type_kind(t, self.aliases) for t in f.results]

    def canonical(self, name):
        if name in self._memo:
            return self._memo[name]
        f = self.functions[name]
        if f.body is None:
            raise ParseError("@%s has no body" % name)
        self._memo[name] = "<recursive>"
        env = {}
        for k, (nm, _) in enumerate(f.args):
            if nm:
                env[nm] = "a%d" % k
        args, results = self.signature(f)
        stmts, _ = read_region(f.body)
        counter = [0]
        lines = self._region(stmts, env, counter)
        out = "(%s)->(%s){%s}" % (",".join(args), ",".join(results), ";".join(lines))
        self._memo[name] = out
        return out

    def _resolve(self, attr):
        seen = set()
        while attr in self.aliases and attr not in seen:
            seen.add(attr)
            attr = self.aliases[attr]
        return attr

    def _head(self, head, env):
        # attribute aliases spelled out, types reduced to their kind, values renamed, blanks dropped
        head = re.sub(r"#[\w.$-]+", lambda m: self._resolve(m.group(0)) if m.group(0) in self.aliases else m.group(0),
                      head)
        head = re.sub(r"affine_map<\(([^)]*)\)\s*->\s*\(([^)]*)\)>", self._affine, head)
        head = re.sub(r',?\s*doc\s*=\s*"[^"]*"', "", head)
        out, i = "", 0
        while i < len(head):
            m = re.compile(r"tensor<").match(head, i)
            if m:
                e = _match(head, m.end() - 1)
                out += type_kind(head[i:e], self.aliases)
                i = e
                continue
            out += head[i]
            i += 1

        def val(m):
            v = m.group(0)
            base = v.split("#")[0]
            if base in env:
                return env[base] + (("#" + v.split("#")[1]) if "#" in v else "")
            return "?" + v
        out = _VALUE.sub(val, out)
        return re.sub(r"\s+", "", out)

    @staticmethod
    def _affine(m):
        dims = [d.strip() for d in m.group(1).split(",")]
        ren = {d: "d%d" % k for k, d in enumerate(dims) if d}
        res = [re.sub(r"\b[A-Za-z_]\w*\b", lambda t: ren.get(t.group(0), t.group(0)), r.strip())
               for r in m.group(2).split(",")]
        return "map(%d:%s)" % (len(dims), ",".join(res))

    def _region(self, stmts, env, counter):
        # constants are written into their uses; a constant nobody uses leaves no trace
        lines = []
        for s in stmts:
            if s.op == "arith.constant" and len(s.results) == 1:
                lit = re.sub(r"\s+", "", s.head)
                m = re.match(r"(-?[\d.eE+-]+|true|false):(\w+)", lit)
                if m and m.group(2)[0] in "fb":
                    lit = "%r:%s" % (float(m.group(1)), m.group(2))
                env[s.results[0]] = "const(%s)" % lit
                continue
            head = s.head
            callee = None
            if s.op in ("func.call", "call"):
                m = re.search(r"@([\w$.-]+)", head)
                if not m or m.group(1) not in self.functions:
                    raise ParseError("call of an unknown function in %r" % head[:60])
                callee = self.canonical(m.group(1))
                head = head.replace("@" + m.group(1), "@callee", 1)
            head_env = env
            carried = [m.group(1) for m in re.finditer(r"(%[\w.$-]+)\s*=\s*%", head) if m.group(1) not in env]
            if s.op == "scf.for":
                m = re.match(r"\s*(%[\w.$-]+)\s*=", head)
                if m and m.group(1) not in env and m.group(1) not in carried:
                    carried.insert(0, m.group(1))
            if carried:
                head_env = dict(env)
                for b in carried:
                    head_env[b] = "b%d" % counter[0]
                    counter[0] += 1
            text = self._head(head, head_env)
            regions = []
            for ri, (bargs, sub) in enumerate(s.regions):
                inner_env = dict(head_env) if ri == 0 else dict(env)
                for b in bargs:
                    inner_env[b] = "b%d" % counter[0]
                    counter[0] += 1
                regions.append("[" + ";".join(self._region(sub, inner_env, counter)) + "]")
            names = []
            for r in s.results:
                base, _, cnt = r.partition(":")
                env[base] = "v%d" % counter[0]
                names.append(env[base] + (":" + cnt if cnt else ""))
                counter[0] += 1
            line = "%s%s %s" % ((",".join(names) + "=") if names else "", s.op, text)
            if callee is not None:
                line += " callee=" + callee
            if regions:
                line += " " + " ".join(regions)
            lines.append(line)
        return lines
