"""Runs a module function operation by operation on the gfx950 kernel library.

The reference lowers ANY module made of `linalg` / `sparse_tensor` / `scf` / `arith` operations to loops and
emits a kernel per loop nest (python/lapis/KokkosBackend.py:83-127, Pipelines/KokkosPipelines.cpp:42-153).
The prebuilt module has whole functions for the computations of the reference's examples; this file covers
every other function written in the same vocabulary: it walks the function's statements and hands each one
to the entry point of `include/lapis_hip.h` that computes it, with all tensors resident on the device
between operations.

    linalg.matvec / linalg.matmul with a CSR operand     lapis_hip_spmv_csr_* / lapis_hip_spmm_csr_*
    linalg.dot                                            lapis_hip_dot_*_host (the scalar comes back to the host, as
                                                          the reference's parallel_reduce does, TranslateToKokkosCpp.cpp:1696-1705)
    linalg.fill / copy / add / sub / mul / div, and parallel linalg.generic bodies that are a*x + b*y, a*x,
    x*y, x or a constant (lapis_amd/elementwise.py)       lapis_hip_fill / copy / axpby / mult / div
    tensor.empty / splat / dim / extract, memref.alloc / dim / load / store / copy, scalar arith.* and math.sqrt,
    scf.while / for / if, func.call
    scf.parallel nests that lapis_amd/loop_mapping.py recognises: the CSR SpMV nest, the CSR x dense SpMM nest,
    depth-1 reductions (dot) and depth-1 elementwise loops

Anything else is refused when the module is compiled (`check`), with the operation named, as the reference
refuses what its pipeline cannot lower.

Tensor values are immutable in MLIR; an operation's `outs` operand is overwritten in place only when it is a
temporary this region made itself (tensor.empty, tensor.splat or the result of an earlier linalg operation)
that nothing mentions afterwards, otherwise the result gets a buffer of its own.  Memref operands are
buffers and are always updated in place.
"""
import re

import numpy

from . import elementwise as _ew
from . import loop_mapping as _lm
from . import mlir_text as _mt


class Refused(Exception):
    """The function uses something outside the vocabulary; the message names it."""


_NAME = r"%[\w.$-]+(?:#\d+)?"
def _ieee(fn):
    """Host scalars follow IEEE 754 as the emitted C++ does: x/0 is an infinity or a NaN, not an exception,
    and the maximum of a NaN and a number is a NaN."""
    def apply(a, b):
        f32 = isinstance(a, numpy.float32) and isinstance(b, numpy.float32)
        with numpy.errstate(all="ignore"):
            r = fn(numpy.float32(a) if f32 else numpy.float64(a), numpy.float32(b) if f32 else numpy.float64(b))
        return numpy.float32(r) if f32 else float(r)
    return apply


_FLOAT_BIN = {"arith.addf": lambda a, b: a + b, "arith.subf": lambda a, b: a - b, "arith.mulf": lambda a, b: a * b,
              "arith.divf": _ieee(numpy.divide), "arith.maximumf": _ieee(numpy.maximum),
              "arith.minimumf": _ieee(numpy.minimum)}
_INT_BIN = {"arith.addi": lambda a, b: a + b, "arith.subi": lambda a, b: a - b, "arith.muli": lambda a, b: a * b,
            "arith.divui": lambda a, b: a // b, "arith.divsi": lambda a, b: int(a / b) if b else 0,
            "arith.remui": lambda a, b: a % b, "arith.remsi": lambda a, b: a - b * int(a / b),
            "arith.andi": lambda a, b: a & b, "arith.ori": lambda a, b: a | b, "arith.xori": lambda a, b: a ^ b,
            "arith.maxsi": max, "arith.minsi": min, "arith.maxui": max, "arith.minui": min}
_CMPI = {"eq": lambda a, b: a == b, "ne": lambda a, b: a != b, "slt": lambda a, b: a < b, "sle": lambda a, b: a <= b,
         "sgt": lambda a, b: a > b, "sge": lambda a, b: a >= b, "ult": lambda a, b: a < b, "ule": lambda a, b: a <= b,
         "ugt": lambda a, b: a > b, "uge": lambda a, b: a >= b}
_CMPF = {"oeq": lambda a, b: a == b, "one": lambda a, b: a != b and a == a and b == b, "olt": lambda a, b: a < b,
         "ole": lambda a, b: a <= b, "ogt": lambda a, b: a > b, "oge": lambda a, b: a >= b,
         "ueq": lambda a, b: a == b or a != a or b != b, "une": lambda a, b: a != b,
         "ult": lambda a, b: not (a >= b), "ule": lambda a, b: not (a > b), "ugt": lambda a, b: not (a <= b),
         "uge": lambda a, b: not (a < b)}
_CASTS = ("arith.index_cast", "arith.index_castui", "arith.extui", "arith.extsi", "arith.trunci", "arith.sitofp",
          "arith.uitofp", "arith.fptosi", "arith.fptoui", "arith.extf", "arith.truncf")
_SCALAR_OPS = set(_FLOAT_BIN) | set(_INT_BIN) | set(_CASTS) | {
    "arith.constant", "arith.negf", "arith.cmpi", "arith.cmpf", "arith.select", "math.sqrt", "math.absf"}
_LINALG_NAMED = {"linalg.add": ("axpby", 1.0, 1.0), "linalg.sub": ("axpby", 1.0, -1.0), "linalg.mul": ("mult",),
                 "linalg.div": ("div",)}
_STRUCTURE = {"scf.while", "scf.for", "scf.if", "scf.condition", "scf.yield", "func.call", "call", "return",
              "func.return", "scf.parallel", "scf.reduce"}
_BUFFER_OPS = {"tensor.empty", "tensor.splat", "tensor.dim", "tensor.extract", "memref.alloc", "memref.alloca",
               "memref.dealloc", "memref.dim", "memref.load", "memref.store", "memref.copy", "linalg.fill",
               "linalg.copy", "linalg.dot", "linalg.matvec", "linalg.matmul", "linalg.generic",
               "bufferization.alloc_tensor"} | set(_LINALG_NAMED)
VOCABULARY = _SCALAR_OPS | _STRUCTURE | _BUFFER_OPS


class Csr:
    """A CSR operand on the device: the three buffers, the sizes, and the SpMV plan made at its first product."""

    def __init__(self, pos, crd, val, nrows, ncols):
        self.pos, self.crd, self.val, self.nrows, self.ncols = pos, crd, val, int(nrows), int(ncols)
        self.nnz = int(crd.shape[0])
        # the kernels index with what the buffers hold: sizes that do not agree must stop here, on the host
        if self.nrows < 0 or self.ncols < 0 or int(pos.shape[0]) != self.nrows + 1:
            raise ValueError("a %d x %d CSR operand needs %d positions, got %d" % (
                self.nrows, self.ncols, self.nrows + 1, int(pos.shape[0])))
        if int(val.shape[0]) != self.nnz:
            raise ValueError("a CSR operand with %d coordinates and %d values" % (self.nnz, int(val.shape[0])))
        self.plan = None
        self.products = 0

    def release(self):
        if self.plan is not None:
            self.plan.destroy()
            self.plan = None


class Cell:
    """A zero-dimensional memref: one scalar, kept on the host."""

    def __init__(self, value=0.0):
        self.value = value


def _same_size(what, *tensors):
    """The kernels take one element count for all their operands: refuse, on the host, operands that differ."""
    sizes = [int(t.numel()) for t in tensors]
    if len(set(sizes)) > 1:
        raise ValueError("%s over operands of %s elements" % (what, ", ".join(map(str, sizes))))


def _elem(ty):
    m = re.search(r"x?(f64|f32|i64|i32|i1|index)\s*(?:,|>)", ty)
    return m.group(1) if m else ty.strip()


def _shape_spec(ty):
    """Dimensions of a tensor / memref type as a list of ints and None (dynamic), and its element type."""
    m = re.match(r"\s*(?:tensor|memref)<(.*)>\s*$", ty, re.S)
    if not m:
        raise Refused("a value of type %s" % ty.strip())
    first = _mt.split_top(m.group(1))[0].strip()
    parts = first.split("x")
    return [None if p == "?" else int(p) for p in parts[:-1]], parts[-1].strip()


def _split_colon(text):
    """`names : types` split at the first depth-0 colon."""
    depth = 0
    for i, ch in enumerate(text):
        if ch in "<([{":
            depth += 1
        elif ch in ">)]}" and not (ch == ">" and i and text[i - 1] == "-"):
            depth -= 1
        elif ch == ":" and depth == 0 and text[i:i + 2] != "::":
            return text[:i], text[i + 1:]
    return text, ""


def _rsplit_colon(text):
    """`left : type` split at the LAST depth-0 colon."""
    depth, at = 0, -1
    for i, ch in enumerate(text):
        if ch in "<([{":
            depth += 1
        elif ch in ">)]}" and not (ch == ">" and text[i - 1] == "-"):
            depth -= 1
        elif ch == ":" and depth == 0:
            at = i
    return (text[:at], text[at + 1:]) if at >= 0 else (text, "")


def _group(head, keyword):
    """(names, types) inside `keyword( ... )` of a statement head, or ([], [])."""
    m = re.search(r"\b%s\s*\(" % keyword, head)
    if not m:
        return [], []
    i = m.end() - 1
    inner = head[i + 1:_mt._match(head, i) - 1]
    names, types = _split_colon(inner)
    return re.findall(_NAME, names), [t.strip() for t in _mt.split_top(types)] if types.strip() else []


def _mentions(stmt, out):
    out.update(re.findall(_NAME, stmt.head))
    for _, sub in stmt.regions:
        for s in sub:
            _mentions(s, out)
    return out


class Executor:
    def __init__(self, canonicalizer, torch_module=None, hip_module=None, device="cuda"):
        # `hip_module` / `device`: the tests of the host logic pass a stand-in for lapis_amd.hip that works on
        # CPU tensors; the product never does (KokkosBackend constructs Executor(canonicalizer))
        self.device = device
        self.c = canonicalizer
        self.aliases = canonicalizer.aliases
        self._parsed = {}
        self._torch = torch_module
        self._hip = hip_module

    # ---- lazily imported plumbing -----------------------------------------------------------------
    @property
    def torch(self):
        if self._torch is None:
            import torch
            self._torch = torch
        return self._torch

    @property
    def hip(self):
        if self._hip is None:
            from . import hip
            hip.init()
            self._hip = hip
        return self._hip

    def _function(self, name):
        if name not in self.c.functions:
            raise Refused("a call of @%s, which the module does not define" % name)
        f = self.c.functions[name]
        if f.body is None:
            raise Refused("a call of @%s, which is declared without a body" % name)
        if name not in self._parsed:
            stmts, _ = _mt.read_region(f.body)
            nests = {}
            if "scf.parallel" in f.body:
                for n in _lm.map_statements(stmts, hip_kernels=True):
                    nests[id(n.stmt)] = n
            self._parsed[name] = (stmts, nests)
        return f, self._parsed[name][0], self._parsed[name][1]

    # ---- what can be told without running -----------------------------------------------------------
    def check(self, name, _seen=None):
        """Raises Refused naming the first thing in @name (or a function it calls) that the library cannot run."""
        seen = _seen if _seen is not None else set()
        if name in seen:
            return
        seen.add(name)
        f, stmts, nests = self._function(name)
        for _, ty in f.args:
            self._check_type(ty)
        self._check_region(stmts, nests, seen, {nm: ty for nm, ty in f.args})

    def _check_type(self, ty):
        ty = ty.strip()
        if ty in ("f64", "f32", "index", "i64", "i32", "i1"):
            return
        kind = _mt.type_kind(ty, self.aliases) if ty.startswith("tensor<") else None
        if kind:
            if kind.startswith("sparse(") or kind.startswith("csrv"):
                raise Refused("an operand stored as %s; CSR with 32-bit positions and coordinates is what the kernel "
                              "library multiplies with" % kind)
            if kind.split(":")[1] not in ("f64", "f32"):
                raise Refused("a tensor of %s" % kind.split(":")[1])
            return
        if ty.startswith("memref<"):
            if "strided" in ty or "affine_map" in ty:
                raise Refused("a memref with a layout (%s)" % ty)
            return
        raise Refused("a value of type %s" % ty)

    def _check_region(self, stmts, nests, seen, arg_types):
        for s in stmts:
            if s.op not in VOCABULARY:
                raise Refused("the operation %s" % s.op)
            if s.op == "scf.parallel":
                n = nests.get(id(s))
                if n is None or not (n.csr_spmv or n.depth1 or n.csr_spmm):
                    raise Refused("a %s loop nest of depth %s that is none of the CSR SpMV nest, the CSR x dense SpMM "
                                  "nest, a depth-1 dot product or a depth-1 elementwise loop"
                                  % ((n.space, n.depth) if n is not None else ("nested", "?")))
                roles = n.csr_spmv or n.csr_spmm
                if roles:
                    what = "SpMV" if n.csr_spmv else "SpMM"
                    for role in ("pos", "crd"):
                        ty = arg_types.get(roles[role])
                        if ty is None or not re.match(r"memref<\?xi32>$", ty.replace(" ", "")):
                            raise Refused("the %s buffer of its %s nest is %s; the kernel library indexes with 32-bit "
                                          "positions and coordinates held in function arguments of type memref<?xi32>"
                                          % (role, what, ty or "not a function argument"))
                continue
            if s.op in ("func.call", "call"):
                m = re.search(r"@([\w$.-]+)", s.head)
                if not m:
                    raise Refused("an indirect call")
                self.check(m.group(1), seen)
            elif s.op in ("linalg.matvec", "linalg.matmul"):
                _, types = _group(s.head, "ins")
                if not types or not _mt.type_kind(types[0], self.aliases).startswith("csr:"):
                    raise Refused("%s whose first operand is not a CSR tensor with 32-bit positions and coordinates"
                                  % s.op)
                if len(types) > 1 and "#" in types[1]:
                    raise Refused("%s with a sparse second operand" % s.op)
            elif s.op == "linalg.generic":
                self._generic_plan(s)
            elif s.op == "arith.constant" and "dense" in s.head:
                raise Refused("a dense constant")
            if s.op != "linalg.generic":
                for _, sub in s.regions:
                    self._check_region(sub, nests, seen, arg_types)

    # ---- linalg.generic ------------------------------------------------------------------------------
    def _generic_plan(self, s):
        """("elementwise", call, n_ins) | ("matvec",) | ("matmul",) for a linalg.generic statement."""
        maps_m = re.search(r"indexing_maps\s*=\s*\[", s.head)
        iters = re.search(r"iterator_types\s*=\s*\[([^\]]*)\]", s.head)
        if not maps_m or not iters or len(s.regions) != 1:
            raise Refused("a linalg.generic without indexing maps, iterator types or a body")
        i = maps_m.end() - 1
        maps = []
        for a in _mt.split_top(s.head[i + 1:_mt._match(s.head, i) - 1]):
            a = a.strip()
            seen = set()
            while a in self.aliases and a not in seen:
                seen.add(a)
                a = self.aliases[a]
            m = re.search(r"\(([^)]*)\)\s*->\s*\(([^)]*)\)", a)
            if not m:
                raise Refused("an indexing map %s" % a)
            dims = [d.strip() for d in m.group(1).split(",") if d.strip()]
            maps.append(tuple(dims.index(r.strip()) if r.strip() in dims else r.strip()
                              for r in m.group(2).split(",") if r.strip()))
        kinds = re.findall(r"parallel|reduction", iters.group(1))
        ins, in_types = _group(s.head, "ins")
        outs, _ = _group(s.head, "outs")
        bargs, body = s.regions[0]
        if len(outs) != 1 or len(bargs) != len(ins) + 1 or not body or body[-1].op != "linalg.yield":
            raise Refused("a linalg.generic with %d outputs" % len(outs))
        yielded = re.findall(_NAME, body[-1].head)
        if len(yielded) != 1:
            raise Refused("a linalg.generic that yields %d values" % len(yielded))
        rank = len(kinds)
        ident = tuple(range(rank))
        if all(k == "parallel" for k in kinds) and all(m == ident for m in maps):
            for t in in_types:
                if "#" in t:
                    raise Refused("an elementwise linalg.generic over a sparse operand")
            try:
                poly = _ew.polynomial(body[:-1], lambda nm: bargs.index(nm) if nm in bargs else None, yielded[0])
                call = _ew.classify(poly)
            except _ew.Unsupported as e:
                raise Refused("a linalg.generic body the library has no kernel for: %s" % e)
            return ("elementwise", call, len(ins))
        # the two contractions, written as generics (examples/spmm_dcsr_opdsl.py:73-78 of the reference)
        if len(ins) == 2 and in_types and _mt.type_kind(in_types[0], self.aliases).startswith("csr:"):
            try:
                poly = _ew.polynomial(body[:-1], lambda nm: bargs.index(nm) if nm in bargs else None, yielded[0])
            except _ew.Unsupported as e:
                raise Refused("a contraction body the library has no kernel for: %s" % e)
            one = ("const", 1.0)
            if {k: c for k, c in poly.terms.items() if c != ("const", 0.0)} == {(0, 1): one, (2,): one}:
                if kinds == ["parallel", "reduction"] and maps == [(0, 1), (1,), (0,)]:
                    return ("matvec",)
                if kinds == ["parallel", "parallel", "reduction"] and maps == [(0, 2), (2, 1), (0, 1)]:
                    return ("matmul",)
        raise Refused("a linalg.generic that is neither elementwise over identity maps nor out += A*b with a CSR A")

    # ---- running --------------------------------------------------------------------------------------
    def run(self, name, args):
        """Results of @name for `args` (device tensors, Csr operands, host scalars), as a list."""
        f, stmts, nests = self._function(name)
        env = {}
        for (nm, _), v in zip(f.args, args):
            env[nm] = v
        kind, values = self._region(stmts, env, nests, owned=set())
        if kind != "return":
            raise RuntimeError("@%s ended without a return" % name)
        return values

    def _val(self, env, name):
        if name not in env:
            raise RuntimeError("value %s is used before it is defined" % name)
        return env[name]

    def _region(self, stmts, env, nests, owned):
        """Runs the statements; returns (terminator kind, its operand values)."""
        later = [None] * len(stmts)
        acc = set()
        for k in range(len(stmts) - 1, -1, -1):
            later[k] = set(acc)
            _mentions(stmts[k], acc)
        defined_here = set()
        for k, s in enumerate(stmts):
            op = s.op
            if op in ("return", "func.return", "scf.yield", "scf.condition"):
                names = re.findall(_NAME, _split_colon(s.head)[0])
                return op.split(".")[-1], [self._val(env, n) for n in names]
            can_overwrite = lambda nm: nm in owned and nm in defined_here and nm not in later[k]
            try:
                results = self._statement(s, env, nests, owned, can_overwrite)
            except ZeroDivisionError:
                raise RuntimeError("%s: integer division by zero" % op)
            except (AttributeError, TypeError, IndexError, KeyError) as e:
                # an operand that is not what the operation's types say (a scalar where a tensor is named, ...):
                # text MLIR's own verifier would not have let through
                raise RuntimeError("%s: an operand does not have the type the operation declares (%s: %s)" % (
                    op, type(e).__name__, e))
            names = []
            for r in s.results:
                if ":" in r:
                    base, cnt = r.split(":")
                    names += ["%s#%d" % (base, j) for j in range(int(cnt))]
                else:
                    names.append(r)
            if results is not None:
                if len(results) != len(names):
                    raise RuntimeError("%s gave %d values for %d results" % (op, len(results), len(names)))
                for nm, v in zip(names, results):
                    env[nm] = v
                    defined_here.add(nm)
        return "end", []

    # every handler returns the list of result values (or None for no results)
    def _statement(self, s, env, nests, owned, can_overwrite):
        op, head = s.op, s.head
        if op in _SCALAR_OPS:
            return [self._scalar(op, head, env)]
        if op == "scf.parallel":
            return self._nest(s, nests[id(s)], env)
        if op in ("func.call", "call"):
            callee = re.search(r"@([\w$.-]+)", head).group(1)
            i = head.index("(")
            names = re.findall(_NAME, head[i:_mt._match(head, i)])
            return self.run(callee, [self._val(env, n) for n in names])
        if op == "scf.while":
            return self._while(s, env, nests)
        if op == "scf.for":
            return self._for(s, env, nests)
        if op == "scf.if":
            cond = self._val(env, re.findall(_NAME, head)[0])
            if len(s.regions) < 2 and not cond:
                return None
            bargs, sub = s.regions[0 if cond else 1]
            kind, vals = self._region(sub, env, nests, set())
            return vals if s.results else None
        return self._buffer_op(s, env, owned, can_overwrite)

    def _scalar(self, op, head, env):
        left, ty = _split_colon(head)
        ty = ty.strip()
        if op == "arith.constant":
            tok = left.strip()
            if tok in ("true", "false"):
                return tok == "true"
            if ty in ("f64", "f32"):
                return numpy.float32(tok) if ty == "f32" else float(tok)
            return int(float(tok)) if ty != "i1" else bool(int(tok))
        names = re.findall(_NAME, left)
        vals = [self._val(env, n) for n in names]
        if op in _FLOAT_BIN:
            return _FLOAT_BIN[op](vals[0], vals[1])
        if op in _INT_BIN:
            return _INT_BIN[op](vals[0], vals[1])
        if op == "arith.negf":
            return -vals[0]
        if op == "math.sqrt":
            with numpy.errstate(all="ignore"):  # the root of a negative number is a NaN
                return numpy.sqrt(vals[0]) if isinstance(vals[0], numpy.floating) else float(numpy.sqrt(vals[0]))
        if op == "math.absf":
            return abs(vals[0])
        if op in ("arith.cmpi", "arith.cmpf"):
            pred = re.match(r"\s*(\w+)", left).group(1)
            return (_CMPI if op == "arith.cmpi" else _CMPF)[pred](vals[0], vals[1])
        if op == "arith.select":
            return vals[1] if vals[0] else vals[2]
        if op in _CASTS:
            target = ty.split("to")[-1].strip()
            if target == "f32":
                return numpy.float32(vals[0])
            if target == "f64":
                return float(vals[0])
            return int(vals[0])
        raise Refused("the operation %s" % op)

    # ---- structured control flow -----------------------------------------------------------------------
    def _while(self, s, env, nests):
        head = s.head
        i = head.index("(")
        inits = [p.split("=") for p in _mt.split_top(head[i + 1:_mt._match(head, i) - 1]) if "=" in p]
        before_names = [a.strip() for a, _ in inits]
        values = [self._val(env, b.strip()) for _, b in inits]
        (_, before), (after_args, after) = s.regions
        while True:
            e = dict(env)
            e.update(zip(before_names, values))
            kind, out = self._region(before, e, nests, set())
            if kind != "condition":
                raise RuntimeError("the first region of scf.while does not end in scf.condition")
            if not out[0]:
                return out[1:]
            e = dict(env)
            e.update(zip(after_args, out[1:]))
            kind, values = self._region(after, e, nests, set())
            if kind != "yield":
                raise RuntimeError("the second region of scf.while does not end in scf.yield")

    def _for(self, s, env, nests):
        m = re.match(r"\s*(%s)\s*=\s*(%s)\s*to\s*(%s)\s*step\s*(%s)" % ((_NAME,) * 4), s.head)
        if not m:
            raise Refused("an scf.for that is not `%i = lo to hi step st`")
        iv, lo, hi, st = m.group(1), self._val(env, m.group(2)), self._val(env, m.group(3)), self._val(env, m.group(4))
        carried_names, values = [], []
        im = re.search(r"iter_args\s*\(", s.head)
        if im:
            i = im.end() - 1
            for p in _mt.split_top(s.head[i + 1:_mt._match(s.head, i) - 1]):
                a, b = p.split("=")
                carried_names.append(a.strip())
                values.append(self._val(env, b.strip()))
        _, body = s.regions[0]
        for k in range(lo, hi, st):
            e = dict(env)
            e[iv] = k
            e.update(zip(carried_names, values))
            kind, out = self._region(body, e, nests, set())
            if carried_names:
                values = out
        return values if s.results else None

    # ---- tensors and memrefs ---------------------------------------------------------------------------
    def _new(self, shape, elem):
        torch = self.torch
        return torch.empty(tuple(int(d) for d in shape), dtype=torch.float64 if elem == "f64" else
                           torch.float32 if elem == "f32" else torch.int32, device=self.device)

    def _sizes(self, ty, dynamic):
        dims, elem = _shape_spec(ty)
        dyn = iter(dynamic)
        return [d if d is not None else int(next(dyn)) for d in dims], elem

    def _dest(self, nm, env, can_overwrite, keep_contents):
        """Buffer the result of a tensor operation goes to: the `outs` operand itself where that is allowed, else
        a new buffer (a copy of the operand when the operation reads it)."""
        t = self._val(env, nm)
        if can_overwrite(nm):
            return t
        return t.clone() if keep_contents else self.torch.empty_like(t)

    def _csr_product(self, A, x, y, k=None):
        hip = self.hip
        if k is None:
            if x.numel() != A.ncols or y.numel() != A.nrows:
                raise ValueError("a %d x %d matrix times a vector of %d elements into one of %d" % (
                    A.nrows, A.ncols, x.numel(), y.numel()))
        elif tuple(x.shape) != (A.ncols, k) or tuple(y.shape) != (A.nrows, k):
            raise ValueError("a %d x %d matrix times a %s matrix into a %s one" % (
                A.nrows, A.ncols, "x".join(map(str, x.shape)), "x".join(map(str, y.shape))))
        if A.plan is None:
            A.plan = hip.CsrPlan(A.nrows, A.ncols, A.pos, A.crd, value_bytes=A.val.element_size(), nnz=A.nnz)
        A.products += 1
        if k is None:
            if A.products == 6:  # a matrix multiplied with again and again: let the library decide on its blocked copy
                A.plan.analyze(A.crd, A.val)
            hip.spmv(A.plan, A.nrows, A.ncols, A.pos, A.crd, A.val, x, y)
        else:
            hip.spmm(A.nrows, A.ncols, A.pos, A.crd, A.val, x, y, plan=A.plan)
        return y

    def _elementwise(self, call, operands, dst, scalars):
        """dst = call(operands); `operands[k]` are flat device tensors, `scalars(name)` host values."""
        hip = self.hip
        f32 = dst.element_size() == 4
        dtype = numpy.float32 if f32 else float
        ev = lambda expr: float(_ew.evaluate(expr, scalars, dtype))
        kind = call[0]
        _same_size("an elementwise operation", dst, *operands)
        if kind == "fill":
            hip.fill(dst, ev(call[1]))
        elif kind == "copy":
            if operands[call[1]].data_ptr() != dst.data_ptr():
                hip.copy(operands[call[1]], dst)
        elif kind == "scale":
            x = operands[call[2]]
            hip.axpby(ev(call[1]), x, 0.0, x, dst)
        elif kind == "mult":
            hip.mult(operands[call[1]], operands[call[2]], dst)
        elif kind == "axpby":
            hip.axpby(ev(call[1]), operands[call[2]], ev(call[3]), operands[call[4]], dst)
        else:
            raise Refused("elementwise %s" % kind)
        return dst

    def _buffer_op(self, s, env, owned, can_overwrite):
        op, head = s.op, s.head
        torch, hip = self.torch, self.hip
        result_is_tensor = bool(s.results)
        own = lambda: owned.add(s.results[0]) if s.results else None
        if op in ("tensor.empty", "memref.alloc", "memref.alloca", "bufferization.alloc_tensor"):
            left, ty = _rsplit_colon(head)
            i = left.index("(")
            dyn = [self._val(env, n) for n in re.findall(_NAME, left[i:_mt._match(left, i)])]
            dims, elem = self._sizes(ty, dyn)
            own()
            if not dims:
                return [Cell(0.0)] if op.startswith("memref") else [0.0]
            return [self._new(dims, elem)]
        if op == "memref.dealloc":
            return None
        if op == "tensor.splat":
            left, ty = _rsplit_colon(head)
            names = re.findall(_NAME, left)
            dims, elem = self._sizes(ty, [self._val(env, n) for n in names[1:]])
            v = self._val(env, names[0])
            own()
            if not dims:
                return [v]
            t = self._new(dims, elem)
            hip.fill(t.view(-1), float(v))
            return [t]
        if op in ("tensor.dim", "memref.dim"):
            names = re.findall(_NAME, _split_colon(head)[0])
            t, d = self._val(env, names[0]), self._val(env, names[1])
            if isinstance(t, Csr):
                return [(t.nrows, t.ncols)[d]]
            return [int(t.shape[d])]
        if op in ("tensor.extract", "memref.load"):
            names = re.findall(_NAME, _split_colon(head)[0])
            t = self._val(env, names[0])
            idx = [self._val(env, n) for n in names[1:]]
            if isinstance(t, Cell):
                return [t.value]
            if not isinstance(t, torch.Tensor):  # a zero-dimensional tensor is kept as a host scalar
                return [t]
            v = t[tuple(idx)].item()  # waits for the kernels that produce it
            return [numpy.float32(v) if t.dtype == torch.float32 else v]
        if op == "memref.store":
            names = re.findall(_NAME, _split_colon(head)[0])
            v, t = self._val(env, names[0]), self._val(env, names[1])
            if isinstance(t, Cell):
                t.value = v
            else:
                t[tuple(self._val(env, n) for n in names[2:])] = v
            return None
        if op == "memref.copy":
            names = re.findall(_NAME, _split_colon(head)[0])
            src, dst = self._val(env, names[0]), self._val(env, names[1])
            if isinstance(dst, Cell):
                dst.value = src.value
            else:
                dst.copy_(src)
            return None

        ins, in_types = _group(head, "ins")
        outs, out_types = _group(head, "outs")
        if len(outs) != 1:
            raise Refused("%s with %d outputs" % (op, len(outs)))
        out_nm = outs[0]
        out_v = self._val(env, out_nm)
        scalar_out = not isinstance(out_v, torch.Tensor)  # a zero-dimensional tensor (host scalar) or a Cell
        in_vals = [self._val(env, n) for n in ins]
        in_place = not result_is_tensor  # memref semantics
        flat = lambda t: t.reshape(-1)

        def dest(keep):
            if in_place:
                return out_v
            own()
            return self._dest(out_nm, env, can_overwrite, keep)

        def give(t):
            return [t] if result_is_tensor else None

        if op == "linalg.fill":
            if scalar_out:
                if isinstance(out_v, Cell):
                    out_v.value = in_vals[0]
                    return None
                return [in_vals[0]]
            d = dest(False)
            hip.fill(flat(d), float(in_vals[0]))
            return give(d)
        if op == "linalg.copy":
            if scalar_out:
                return [in_vals[0]]
            d = dest(False)
            if d.data_ptr() != in_vals[0].data_ptr():
                _same_size("linalg.copy", in_vals[0], d)
                hip.copy(flat(in_vals[0]), flat(d))
            return give(d)
        if op == "linalg.dot":
            init = out_v.value if isinstance(out_v, Cell) else out_v
            _same_size("linalg.dot", in_vals[0], in_vals[1])
            r = hip.dot_host(flat(in_vals[0]), flat(in_vals[1]), float(init))
            r = numpy.float32(r) if in_vals[0].element_size() == 4 else r
            if isinstance(out_v, Cell):
                out_v.value = r
                return None
            return [r]
        plan = self._generic_plan(s) if op == "linalg.generic" else None
        if op == "linalg.matvec" or plan == ("matvec",):
            d = dest(True)
            self._csr_product(in_vals[0], in_vals[1], d)
            return give(d)
        if op == "linalg.matmul" or plan == ("matmul",):
            d = dest(True)
            self._csr_product(in_vals[0], in_vals[1], d, k=int(in_vals[1].shape[1]))
            return give(d)
        if op in _LINALG_NAMED:
            spec = _LINALG_NAMED[op]
            d = dest(False)
            a, b = flat(in_vals[0]), flat(in_vals[1])
            _same_size(op, a, b, d)
            if spec[0] == "axpby":
                hip.axpby(spec[1], a, spec[2], b, flat(d))
            elif spec[0] == "mult":
                hip.mult(a, b, flat(d))
            else:
                hip.div(a, b, flat(d))
            return give(d)
        if op == "linalg.generic":
            _, call, n_ins = plan
            operands = in_vals + [out_v]
            reads_out = any(isinstance(c, int) and c == n_ins for c in call[1:])
            if scalar_out:
                raise Refused("an elementwise linalg.generic over zero-dimensional tensors")
            d = dest(reads_out)
            if reads_out:
                operands[n_ins] = d
            self._elementwise(call, [flat(o) for o in operands], flat(d), lambda nm: self._val(env, nm))
            return give(d)
        raise Refused("the operation %s" % op)

    # ---- loop nests the library has kernels for ----------------------------------------------------------
    def _nest(self, s, n, env):
        hip = self.hip
        if n.csr_spmv:
            r = n.csr_spmv
            y, pos, crd, val, x = (self._val(env, r[k]) for k in ("y", "pos", "crd", "val", "x"))
            A = self._csr_for(pos, crd, val, int(y.shape[0]), int(x.shape[0]))
            self._csr_product(A, x, y)
            return None
        if n.csr_spmm:
            r = n.csr_spmm
            C, pos, crd, val, B = (self._val(env, r[k]) for k in ("C", "pos", "crd", "val", "B"))
            A = self._csr_for(pos, crd, val, int(C.shape[0]), int(B.shape[0]))
            self._csr_product(A, B, C, k=int(B.shape[1]))
            return None
        d = n.depth1
        count = self._val(env, d["n"]) if d["n"] in env else int(d["n"])
        if count < 0 or any(int(self._val(env, a).shape[0]) < count
                            for a in ([d["x"], d["y"]] if d["kind"] == "dot" else list(d["arrays"]) + [d["dst"]])):
            raise ValueError("a loop over %d elements of a shorter buffer" % count)
        if d["kind"] == "dot":
            x, y = self._val(env, d["x"])[:count], self._val(env, d["y"])[:count]
            r = hip.dot_host(x, y, float(self._val(env, d["init"])))
            return [numpy.float32(r) if x.element_size() == 4 else r]
        arrays = [self._val(env, a)[:count] for a in d["arrays"]]
        self._elementwise(d["call"], arrays, self._val(env, d["dst"])[:count], lambda nm: self._val(env, nm))
        return None

    def _csr_for(self, pos, crd, val, nrows, ncols):
        """The Csr (and its plan) of a matrix given as three memrefs; kept while the same buffers come back."""
        key = (pos.data_ptr(), crd.data_ptr(), val.data_ptr(), nrows, ncols, int(crd.shape[0]))
        cache = self.__dict__.setdefault("_csr_cache", {})
        if key not in cache:
            for old in cache.values():
                old.release()
            cache.clear()
            cache[key] = Csr(pos, crd, val, nrows, ncols)
        return cache[key]

    def release(self):
        for A in self.__dict__.get("_csr_cache", {}).values():
            A.release()
        self.__dict__.get("_csr_cache", {}).clear()
