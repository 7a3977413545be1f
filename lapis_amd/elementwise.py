"""What an elementwise body computes, as far as the kernel library can run it.

The body of a parallel `linalg.generic` (examples/pcg_solve.py:30-47 of the reference) or of a depth-1
`scf.parallel` loop (what DenseLinalgToParallelLoops.cpp:227-272 makes of it) is a handful of scalar
`arith` operations on the elements of the operands and on scalars defined outside.  Here such a body is
evaluated symbolically into a polynomial in the elements whose coefficients are expressions in the outside
scalars, and the polynomial is classified as one of the operations `include/lapis_hip.h` offers:

    a*x + b*y   -> ("axpby", a, x, b, y)          x*y      -> ("mult", x, y)
    a*x         -> ("scale", a, x)                x        -> ("copy", x)
    c           -> ("fill", c)

`x`, `y` are positions in the list of element variables the caller passed; `a`, `b`, `c` are coefficient
expressions (`evaluate` turns one into a number once the outside scalars are known).
"""
import re

_VALUE = re.compile(r"%[\w.$-]+(?:#\d+)?")


class Unsupported(Exception):
    pass


def _const(v):
    return ("const", float(v))


def _add(a, b):
    if a == _const(0.0):
        return b
    if b == _const(0.0):
        return a
    if a[0] == "const" and b[0] == "const":
        return _const(a[1] + b[1])
    return ("add", a, b)


def _mul(a, b):
    if a == _const(1.0):
        return b
    if b == _const(1.0):
        return a
    if a[0] == "const" and b[0] == "const":
        return _const(a[1] * b[1])
    return ("mul", a, b)


def _neg(a):
    return _const(-a[1]) if a[0] == "const" else ("neg", a)


def _div(a, b):
    if b == _const(1.0):
        return a
    if a[0] == "const" and b[0] == "const" and b[1] != 0.0:
        return _const(a[1] / b[1])
    return ("div", a, b)


def evaluate(expr, scalars, dtype=float):
    """Value of a coefficient expression; `scalars(name)` gives the value of an outside scalar.  The
    arithmetic is done in `dtype` (numpy.float32 for f32 bodies) so that products of scalars round as the
    body's own operations would."""
    kind = expr[0]
    if kind == "const":
        return dtype(expr[1])
    if kind == "name":
        return dtype(scalars(expr[1]))
    if kind == "neg":
        return dtype(-evaluate(expr[1], scalars, dtype))
    a, b = evaluate(expr[1], scalars, dtype), evaluate(expr[2], scalars, dtype)
    if kind == "add":
        return dtype(a + b)
    if kind == "mul":
        return dtype(a * b)
    if kind == "div":
        return dtype(a / b)
    raise Unsupported("coefficient expression %r" % (expr,))


def scalar_names(expr, out=None):
    out = set() if out is None else out
    if expr[0] == "name":
        out.add(expr[1])
    elif expr[0] != "const":
        for sub in expr[1:]:
            scalar_names(sub, out)
    return out


class Poly:
    """{monomial: coefficient expression}; a monomial is a sorted tuple of element-variable positions."""

    def __init__(self, terms=None):
        self.terms = dict(terms or {})

    @staticmethod
    def var(k):
        return Poly({(k,): _const(1.0)})

    @staticmethod
    def scalar(expr):
        return Poly({(): expr})

    def __add__(self, other):
        out = dict(self.terms)
        for m, c in other.terms.items():
            out[m] = _add(out[m], c) if m in out else c
        return Poly(out)

    def __neg__(self):
        return Poly({m: _neg(c) for m, c in self.terms.items()})

    def __mul__(self, other):
        out = {}
        for m1, c1 in self.terms.items():
            for m2, c2 in other.terms.items():
                m = tuple(sorted(m1 + m2))
                if len(m) > 2:
                    raise Unsupported("a product of more than two elements")
                c = _mul(c1, c2)
                out[m] = _add(out[m], c) if m in out else c
        return Poly(out)

    def over(self, other):
        if list(other.terms) != [()]:
            raise Unsupported("a division by an element")
        return Poly({m: _div(c, other.terms[()]) for m, c in self.terms.items()})


_BINARY = {"arith.addf": lambda a, b: a + b, "arith.subf": lambda a, b: a + (-b), "arith.mulf": lambda a, b: a * b,
           "arith.divf": lambda a, b: a.over(b)}


def polynomial(stmts, element_of, result_name):
    """Polynomial of `result_name` over the element variables.  `element_of(name)` gives the position of an
    element variable (a block argument, or the result of a load at the loop index) or None; every other
    name that is not defined by `stmts` is an outside scalar."""
    defined = {}
    for s in stmts:
        if s.regions:
            raise Unsupported("a nested region inside an elementwise body")
        for r in s.results:
            defined[r.split(":")[0]] = s

    def value(name):
        k = element_of(name)
        if k is not None:
            return Poly.var(k)
        if name not in defined:
            return Poly.scalar(("name", name))
        s = defined[name]
        ops = _VALUE.findall(s.head.split(":")[0])
        if s.op == "arith.constant":
            m = re.match(r"\s*(-?[\d.]+(?:[eE][-+]?\d+)?)\s*:", s.head)
            if not m:
                raise Unsupported("constant %r" % s.head.strip())
            return Poly.scalar(_const(m.group(1)))
        if s.op == "arith.negf" and len(ops) == 1:
            return -value(ops[0])
        if s.op in _BINARY and len(ops) == 2:
            return _BINARY[s.op](value(ops[0]), value(ops[1]))
        raise Unsupported("%s in an elementwise body" % s.op)

    return value(result_name)


def classify(poly):
    """One of the tuples listed at the top of the file, or Unsupported."""
    terms = {m: c for m, c in poly.terms.items() if c != _const(0.0)}
    monos = sorted(terms)
    if not monos:
        return ("fill", _const(0.0))
    if monos == [()]:
        return ("fill", terms[()])
    if len(monos) == 1 and len(monos[0]) == 1:
        (k,), c = monos[0], terms[monos[0]]
        return ("copy", k) if c == _const(1.0) else ("scale", c, k)
    if len(monos) == 1 and len(monos[0]) == 2:
        (i, j), c = monos[0], terms[monos[0]]
        if c != _const(1.0):
            raise Unsupported("a scaled product of two elements")
        return ("mult", i, j)
    if len(monos) == 2 and all(len(m) == 1 for m in monos):
        (i,), (j,) = monos
        return ("axpby", terms[(i,)], i, terms[(j,)], j)
    raise Unsupported("the elementwise body is none of a*x + b*y, a*x, x*y, x or a constant")
