"""Which Kokkos level every loop of an `scf.parallel` nest gets: the decision of the reference's
`kokkos-loop-mapping` pass (mlir/lib/Dialect/Kokkos/Transforms/KokkosLoopMapping.cpp:829-965), taken here
from the module TEXT, without MLIR.

The pass rewrites IR; this file only DECIDES, and reports the decision as a tree:

* a top-level nest runs on the device unless it calls a function or allocates / frees memory inside
  (`:844-855`); on the host, or with one level of parallelism, the outer loop is a RangePolicy /
  MDRangePolicy loop and every inner `scf.parallel` becomes sequential (`:871-887`);
* two levels: the outer loop is a `thread_parallel` (a TeamPolicy with one Kokkos thread per iteration),
  every inner loop a ThreadVector loop (`:888-921`); this is the CSR SpMV shape;
* three or more: `team_parallel`, then TeamThread for a child that has parallel loops of its own and
  TeamVector for one that has none; below a TeamThread loop the innermost loops are ThreadVector and the
  ones between are sequential (`mapNestedLoopsImpl`, `:761-808`);
* stores, atomic updates and reduction updates that do not sit in a vector loop are wrapped in a
  `single`: per team outside every thread loop, per thread inside one (`insertSingleWraps`, `:680-724`);
* in a `team_parallel`, a barrier follows every TeamThread / TeamVector loop without results and every
  per-team `single` without results (`insertTeamSynchronization`, `:732-758`);
* the vector-length (and team-size) hint is the largest product of upper bounds over the loops of that
  level, where a bound is either defined outside the nest or follows the CSR pattern
  `R[i+1] - R[i]` with `i` the outer induction variable, for which the mean row length
  `(R[N] - R[0] + N - 1) / N` stands in (`estimateParallelism`, `:132-343`).

`mapped_summary` reads the same tree back from text the pass has already rewritten (the reference's
`tests/Dialect/Kokkos/loop_mapping_*.mlir.gold`), which is how the tests pin the rules.
"""
import re

from . import elementwise as _ew
from . import mlir_text as _mt

HOST, DEVICE, TEAM_HANDLE = 0, 1, 2                       # executionSpace attribute values
RANGE_POLICY, TEAM_VECTOR, TEAM_THREAD, THREAD_VECTOR = 0, 1, 2, 3   # parallelLevel attribute values
PER_TEAM, PER_THREAD = 0, 1                               # level of a kokkos.single

_HOST_ONLY = ("func.call", "call", "memref.alloc", "memref.alloca", "memref.dealloc", "memref.realloc")
_NEEDS_SINGLE = ("memref.store", "memref.atomic_rmw")
_CASTS = ("arith.index_cast", "arith.index_castui", "arith.extui")


class Node:
    """One structural operation of the mapped nest."""

    def __init__(self, kind, **attrs):
        self.kind, self.attrs, self.children = kind, attrs, []

    def summary(self):
        head = self.kind
        for key in ("space", "level", "ivs", "results"):
            if key in self.attrs:
                head += " %s=%s" % (key, self.attrs[key])
        if self.children:
            return (head, tuple(c.summary() for c in self.children))
        return head


class _Loop:
    def __init__(self, stmt, parent):
        self.stmt, self.parent = stmt, parent
        head = stmt.head
        m = re.match(r"\s*\(([^)]*)\)\s*=\s*\(([^)]*)\)\s*to\s*\(([^)]*)\)\s*step\s*\(([^)]*)\)", head)
        if not m:
            raise _mt.ParseError("scf.parallel without (ivs) = (lb) to (ub) step (st): %r" % head[:60])
        self.ivs = [v.strip() for v in m.group(1).split(",")]
        self.upper = [v.strip() for v in m.group(3).split(",")]
        self.results = len(stmt.results)
        self.body = stmt.regions[0][1] if stmt.regions else []
        self.inner = []    # scf.parallel loops directly nested (through any other region-holding op)
        self.levels = 1


def _walk_loops(stmts, parent, out):
    for s in stmts:
        if s.op == "scf.parallel":
            loop = _Loop(s, parent)
            out.append(loop)
            if parent is not None:
                parent.inner.append(loop)
            _walk_loops(loop.body, loop, out)
        else:
            for _, sub in s.regions:
                _walk_loops(sub, parent, out)


def _contains(stmts, ops):
    for s in stmts:
        if s.op in ops:
            return True
        for _, sub in s.regions:
            if _contains(sub, ops):
                return True
    return False


def _set_levels(loop):
    for c in loop.inner:
        _set_levels(c)
    loop.levels = 1 + max([c.levels for c in loop.inner], default=0)


class NestMapping:
    """The decision for one top-level nest: `.space`, `.depth`, `.tree` (a Node), the hints."""

    def __init__(self, space, depth, tree, vector_length_hint, team_size_hint):
        self.space, self.depth, self.tree = space, depth, tree
        self.vector_length_hint, self.team_size_hint = vector_length_hint, team_size_hint
        self.csr_spmv = None   # {"y", "pos", "crd", "val", "x", "elem"} when the nest is the CSR SpMV nest
        self.depth1 = None     # match_depth1: a dot or an elementwise loop the kernel library has an entry for
        self.csr_spmm = None   # match_csr_spmm: the CSR x dense SpMM nest
        self.stmt = None       # the scf.parallel statement of the nest

    def summary(self):
        return self.tree.summary()


class _Mapper:
    def __init__(self, func_stmts):
        self.defs = {}
        self._index(func_stmts, None)

    def _index(self, stmts, owner):
        for s in stmts:
            for r in s.results:
                self.defs[r.split(":")[0]] = (s, owner)
            for _, sub in s.regions:
                self._index(sub, s)

    # -- hints ------------------------------------------------------------------------------------
    def _follow_cast(self, v):
        while v in self.defs and self.defs[v][0].op in _CASTS:
            v = _mt._VALUE.search(self.defs[v][0].head).group(0)
        return v

    def _operands(self, stmt):
        return _mt._VALUE.findall(stmt.head.split(":")[0])

    def _is_one(self, v):
        v = self._follow_cast(v)
        return v in self.defs and self.defs[v][0].op == "arith.constant" and \
            re.match(r"\s*1\s*:", self.defs[v][0].head) is not None

    def _bound_estimate(self, bound, top, nested):
        """Expression for one upper bound of `nested`, or None when it follows no known pattern."""
        b = self._follow_cast(bound)
        inner = []
        self._collect(top, inner)
        if any(b in l.ivs for l in [top] + inner):
            return None                                 # an induction variable of the nest itself
        if b not in self.defs or not self._inside(self.defs[b][0], top):
            return b                                    # defined outside the nest: loop invariant
        if nested.parent is not top or len(top.ivs) != 1:
            return None
        sub, owner = self.defs[b]
        if sub.op != "arith.subi":
            return None
        ops = self._operands(sub)
        if len(ops) != 2:
            return None
        hi, lo = self._follow_cast(ops[0]), self._follow_cast(ops[1])
        if hi not in self.defs or lo not in self.defs:
            return None
        (hs, hown), (ls, lown) = self.defs[hi], self.defs[lo]
        if hs.op != "memref.load" or ls.op != "memref.load" or hown is not top.stmt or lown is not top.stmt:
            return None
        hm = re.match(r"\s*(%[\w.$-]+)\s*\[([^\]]*)\]", hs.head)
        lm = re.match(r"\s*(%[\w.$-]+)\s*\[([^\]]*)\]", ls.head)
        if not hm or not lm or hm.group(1) != lm.group(1) or "," in lm.group(2) or "," in hm.group(2):
            return None
        i = top.ivs[0]
        if self._follow_cast(lm.group(2).strip()) != i:
            return None
        nxt = self._follow_cast(hm.group(2).strip())
        if nxt not in self.defs or self.defs[nxt][0].op != "arith.addi":
            return None
        a, c = self._operands(self.defs[nxt][0])
        if not ((self._follow_cast(a) == i and self._is_one(c)) or (self._follow_cast(c) == i and self._is_one(a))):
            return None
        n = top.upper[0]
        r = hm.group(1)
        return "divui(subi(addi(subi(load(%s,%s),load(%s,0)),%s),1),%s)" % (r, n, r, n, n)

    def _inside(self, stmt, loop):
        """Is stmt (strictly) inside loop's body?"""
        def has(stmts):
            for s in stmts:
                if s is stmt:
                    return True
                for _, sub in s.regions:
                    if has(sub):
                        return True
            return False
        return has(loop.body)

    def _estimate(self, top, loops):
        best = []
        for nested in loops:
            parts = [self._bound_estimate(b, top, nested) for b in nested.upper]
            if parts and all(p is not None for p in parts):
                best.append("*".join(parts))
        if not best:
            return None
        return best[0] if len(best) == 1 else "maxui(%s)" % ",".join(best)

    # -- the CSR SpMV nest --------------------------------------------------------------------------
    def match_csr_spmv(self, top):
        """The five buffers of `y[i] = y[i] + sum_j val[pos[i]+j] * x[crd[pos[i]+j]]`, j < pos[i+1]-pos[i],
        when `top` is exactly that nest (tests/Dialect/Kokkos/loop_mapping_2.mlir of the reference, with
        index casts wherever positions and coordinates are narrower than index), else None."""
        if len(top.ivs) != 1 or top.results or len(top.inner) != 1 or top.levels != 2:
            return None
        inner = top.inner[0]
        allowed = ("memref.load", "arith.addi", "arith.subi", "scf.parallel", "memref.store", "scf.reduce") + _CASTS
        if any(s.op not in allowed for s in top.body) or inner.stmt not in top.body:
            return None
        if len(inner.ivs) != 1 or inner.results != 1 or sum(s.op == "memref.store" for s in top.body) != 1:
            return None
        est = self._bound_estimate(inner.upper[0], top, inner)
        if est is None or not est.startswith("divui("):
            return None
        i, j = top.ivs[0], inner.ivs[0]

        def load(v):
            """(memref, index value) of a one-dimensional memref.load that defines v (casts followed)."""
            v = self._follow_cast(v)
            if v not in self.defs or self.defs[v][0].op != "memref.load":
                return None
            m = re.match(r"\s*(%[\w.$-]+)\s*\[\s*(%[\w.$-]+)\s*\]", self.defs[v][0].head)
            return (m.group(1), self._follow_cast(m.group(2))) if m else None

        sub = self.defs[self._follow_cast(inner.upper[0])][0]
        lo_value = self._follow_cast(self._operands(sub)[1])          # pos[i]
        pos = load(lo_value)[0]
        # init (%y0): the reduction starts from y[i]
        m = re.search(r"init\s*\(\s*(%[\w.$-]+)\s*\)\s*->\s*(\w+)", inner.stmt.head)
        if not m:
            return None
        y0, elem = load(m.group(1)), m.group(2)
        if not y0 or y0[1] != i or elem not in ("f64", "f32"):
            return None
        body_ops = ("memref.load", "arith.addi", "arith.mulf", "scf.reduce") + _CASTS
        if any(s.op not in body_ops for s in inner.body):
            return None
        reduces = [s for s in inner.body if s.op == "scf.reduce"]
        if len(reduces) != 1 or len(reduces[0].regions) != 1:
            return None
        bargs, comb = reduces[0].regions[0]
        if len(comb) != 2 or comb[0].op != "arith.addf" or sorted(self._operands(comb[0])) != sorted(bargs):
            return None
        prod = _mt._VALUE.search(reduces[0].head).group(0)
        if prod not in self.defs or self.defs[prod][0].op != "arith.mulf":
            return None
        a, b = self._operands(self.defs[prod][0])

        def is_entry(idx):          # pos[i] + j
            if idx not in self.defs or self.defs[idx][0].op != "arith.addi":
                return False
            p, q = [self._follow_cast(o) for o in self._operands(self.defs[idx][0])]
            return (p == lo_value and q == j) or (q == lo_value and p == j)

        def via_crd(v):             # x[crd[pos[i] + j]]
            g = load(v)
            if not g:
                return None
            c = load(g[1])
            return (g[0], c[0]) if c and is_entry(c[1]) else None

        la, lb = load(a), load(b)
        if not la or not lb:
            return None
        xc = via_crd(b)
        vload = la
        if not xc:
            xc, vload = via_crd(a), lb
        if not xc or not is_entry(vload[1]):
            return None
        store = next(s for s in top.body if s.op == "memref.store")
        m = re.match(r"\s*(%[\w.$-]+)\s*,\s*(%[\w.$-]+)\s*\[\s*(%[\w.$-]+)\s*\]", store.head)
        if not m or m.group(1) != inner.stmt.results[0] or m.group(2) != y0[0] or self._follow_cast(m.group(3)) != i:
            return None
        return {"y": y0[0], "pos": pos, "crd": xc[1], "val": vload[0], "x": xc[0], "elem": elem}


    # -- depth-1 nests the kernel library runs: dot, axpby / mult / scale / copy / fill --------------
    def _load_at(self, name, iv):
        """Memref of a one-dimensional `memref.load <m>[<iv>]` that defines `name` (casts followed), else None."""
        name = self._follow_cast(name)
        if name not in self.defs or self.defs[name][0].op != "memref.load":
            return None
        m = re.match(r"\s*(%[\w.$-]+)\s*\[\s*(%[\w.$-]+)\s*\]", self.defs[name][0].head)
        if not m or self._follow_cast(m.group(2)) != iv:
            return None
        return m.group(1)

    def match_depth1(self, top):
        """What a one-level `scf.parallel` over one induction variable computes, if it is a loop the library
        has an entry point for (the loops DenseLinalgToParallelLoops.cpp:227-272,349-393 of the reference
        makes of linalg.dot, linalg.fill, linalg.copy and parallel linalg.generic), else None:

        {"kind": "dot", "x", "y", "init", "result", "elem", "n"}  or
        {"kind": "axpby" | "scale" | "mult" | "copy" | "fill", "dst", "arrays", "call", "elem", "n"}
        with `call` the classification of lapis_amd/elementwise.py over `arrays`."""
        if len(top.ivs) != 1 or top.levels != 1 or top.inner:
            return None
        iv, n = top.ivs[0], top.upper[0]
        arrays = []

        def element_of(name):
            m = self._load_at(name, iv)
            if m is None:
                return None
            if m not in arrays:
                arrays.append(m)
            return arrays.index(m)

        body = [s for s in top.body if s.op not in ("scf.yield",)]
        loads = [s for s in body if s.op == "memref.load"]
        for s in loads:  # every load is an element at the loop index
            mm = re.match(r"\s*(%[\w.$-]+)\s*\[\s*(%[\w.$-]+)\s*\]", s.head)
            if not mm or self._follow_cast(mm.group(2)) != iv:
                return None
        arith = [s for s in body if s.op.startswith("arith.")]
        stores = [s for s in body if s.op == "memref.store"]
        reduces = [s for s in body if s.op == "scf.reduce"]
        if len(loads) + len(arith) + len(stores) + len(reduces) != len(body):
            return None
        try:
            if top.results == 1:  # a reduction: init + sum x[i] * y[i]
                m = re.search(r"init\s*\(\s*(%[\w.$-]+)\s*\)\s*->\s*(\w+)", top.stmt.head)
                if not m or stores or len(reduces) != 1 or len(reduces[0].regions) != 1 or m.group(2) not in ("f64", "f32"):
                    return None
                bargs, comb = reduces[0].regions[0]
                if len(comb) != 2 or comb[0].op != "arith.addf" or sorted(self._operands(comb[0])) != sorted(bargs):
                    return None
                reduced = _mt._VALUE.search(reduces[0].head).group(0)
                poly = _ew.polynomial(arith, element_of, reduced)
                terms = {k: c for k, c in poly.terms.items() if c != ("const", 0.0)}
                if len(terms) != 1:
                    return None
                (mono, coeff), = terms.items()
                if len(mono) != 2 or coeff != ("const", 1.0):
                    return None
                return {"kind": "dot", "x": arrays[mono[0]], "y": arrays[mono[1]], "init": m.group(1),
                        "result": top.stmt.results[0], "elem": m.group(2), "n": n}
            if top.results or len(stores) != 1 or any(r.regions for r in reduces):
                return None
            m = re.match(r"\s*(%[\w.$-]+)\s*,\s*(%[\w.$-]+)\s*\[\s*(%[\w.$-]+)\s*\]\s*:\s*memref<\?x(\w+)>", stores[0].head)
            if not m or self._follow_cast(m.group(3)) != iv or m.group(4) not in ("f64", "f32"):
                return None
            call = _ew.classify(_ew.polynomial(arith, element_of, m.group(1)))
        except _ew.Unsupported:
            return None
        # coefficients have to be loop invariant: defined outside the nest
        for expr in [c for c in call[1:] if isinstance(c, tuple)]:
            for nm in _ew.scalar_names(expr):
                if nm in self.defs and self._inside(self.defs[nm][0], top):
                    return None
        return {"kind": call[0], "dst": m.group(2), "arrays": list(arrays), "call": call, "elem": m.group(4), "n": n}

    # -- the CSR x dense SpMM nest ------------------------------------------------------------------
    def match_csr_spmm(self, top):
        """Buffers of `C[i,j] += sum_kk val[kk] * B[crd[kk], j]`, kk in [pos[i], pos[i+1]), when `top` is that
        nest with the rows parallel, the compressed loop sequential (`scf.for`) and the dense column loop
        either kind -- what the sparsifier leaves for CSR x dense matmul (examples/spmm_dcsr_opdsl.py:73-110)
        under the strategies that do not parallelise the reduction (Pipelines/Passes.h:41-56) -- else None:
        {"C", "pos", "crd", "val", "B", "elem", "rows", "k"}."""
        if len(top.ivs) != 1 or top.results:
            return None
        i = top.ivs[0]
        fors = [s for s in top.body if s.op == "scf.for"]
        if len(fors) != 1 or any(s.op not in ("memref.load", "arith.addi", "scf.for", "scf.reduce", "scf.yield") + _CASTS
                                 for s in top.body):
            return None
        outer = fors[0]
        m = re.match(r"\s*(%[\w.$-]+)\s*=\s*(%[\w.$-]+)\s*to\s*(%[\w.$-]+)\s*step\s*(%[\w.$-]+)", outer.head)
        if not m or not self._is_one(m.group(4)) or "iter_args" in outer.head:
            return None
        kk, lo, hi = m.group(1), self._follow_cast(m.group(2)), self._follow_cast(m.group(3))

        def load1(v):
            v = self._follow_cast(v)
            if v not in self.defs or self.defs[v][0].op != "memref.load":
                return None
            mm = re.match(r"\s*(%[\w.$-]+)\s*\[\s*(%[\w.$-]+)\s*\]", self.defs[v][0].head)
            return (mm.group(1), self._follow_cast(mm.group(2))) if mm else None

        plo, phi = load1(lo), load1(hi)
        if not plo or not phi or plo[0] != phi[0] or plo[1] != i:
            return None
        nxt = phi[1]
        if nxt not in self.defs or self.defs[nxt][0].op != "arith.addi":
            return None
        a, c = self._operands(self.defs[nxt][0])
        if not ((self._follow_cast(a) == i and self._is_one(c)) or (self._follow_cast(c) == i and self._is_one(a))):
            return None
        mid = outer.regions[0][1]
        inner = [s for s in mid if s.op in ("scf.for", "scf.parallel")]
        if len(inner) != 1 or any(s.op not in ("memref.load", "scf.for", "scf.parallel", "scf.yield") + _CASTS for s in mid):
            return None
        jl = inner[0]
        if jl.op == "scf.for":
            mj = re.match(r"\s*(%[\w.$-]+)\s*=\s*(%[\w.$-]+)\s*to\s*(%[\w.$-]+)\s*step\s*(%[\w.$-]+)", jl.head)
            if not mj or not self._is_one(mj.group(4)) or "iter_args" in jl.head:
                return None
            j, kcols = mj.group(1), mj.group(3)
        else:
            mj = re.match(r"\s*\(\s*(%[\w.$-]+)\s*\)\s*=\s*\([^)]*\)\s*to\s*\(\s*(%[\w.$-]+)\s*\)\s*step\s*\(\s*(%[\w.$-]+)\s*\)", jl.head)
            if not mj or not self._is_one(mj.group(3)) or jl.results:
                return None
            j, kcols = mj.group(1), mj.group(2)
        jbody = jl.regions[0][1]
        if any(s.op not in ("memref.load", "arith.mulf", "arith.addf", "memref.store", "scf.yield", "scf.reduce") + _CASTS
               for s in jbody):
            return None
        stores = [s for s in jbody if s.op == "memref.store"]
        if len(stores) != 1:
            return None

        def load2(v):
            v = self._follow_cast(v)
            if v not in self.defs or self.defs[v][0].op != "memref.load":
                return None
            mm = re.match(r"\s*(%[\w.$-]+)\s*\[\s*(%[\w.$-]+)\s*,\s*(%[\w.$-]+)\s*\]", self.defs[v][0].head)
            return (mm.group(1), self._follow_cast(mm.group(2)), self._follow_cast(mm.group(3))) if mm else None

        ms = re.match(r"\s*(%[\w.$-]+)\s*,\s*(%[\w.$-]+)\s*\[\s*(%[\w.$-]+)\s*,\s*(%[\w.$-]+)\s*\]\s*:\s*memref<\?x\?x(\w+)>",
                      stores[0].head)
        if not ms or self._follow_cast(ms.group(3)) != i or self._follow_cast(ms.group(4)) != j:
            return None
        total, C, elem = ms.group(1), ms.group(2), ms.group(5)
        if elem not in ("f64", "f32") or total not in self.defs or self.defs[total][0].op != "arith.addf":
            return None
        t0, t1 = self._operands(self.defs[total][0])
        old, prod = (t0, t1) if load2(t0) else (t1, t0)
        lold = load2(old)
        if not lold or lold != (C, i, j) or prod not in self.defs or self.defs[prod][0].op != "arith.mulf":
            return None
        p0, p1 = self._operands(self.defs[prod][0])
        vname, bname = (p0, p1) if load1(p0) else (p1, p0)
        lv, lb = load1(vname), load2(bname)
        if not lv or not lb or lv[1] != kk or lb[2] != j:
            return None
        lc = load1(lb[1])
        if not lc or lc[1] != kk:
            return None
        return {"C": C, "pos": plo[0], "crd": lc[0], "val": lv[0], "B": lb[0], "elem": elem, "rows": top.upper[0],
                "k": kcols}

    # -- the tree -----------------------------------------------------------------------------------
    def map_nest(self, top, hip_kernels=False):
        offload = not _contains(top.body, _HOST_ONLY)
        space = DEVICE if offload else HOST
        depth = top.levels
        level_of = {}
        if space == HOST or depth == 1:
            level_of[id(top)] = ("range", space, RANGE_POLICY)
            self._mark(top, lambda l: ("for",), level_of)
        elif depth == 2:
            level_of[id(top)] = ("thread",)
            self._mark(top, lambda l: ("range", TEAM_HANDLE, THREAD_VECTOR), level_of)
        else:
            level_of[id(top)] = ("team",)
            self._map_nested(top, 2, level_of)
        tree = self._build(top, level_of, in_team=False, in_thread=False, in_vector=False, team_sync=depth >= 3 and space == DEVICE)
        vec = team = None
        if space == DEVICE and depth >= 2:
            all_loops = []
            self._collect(top, all_loops)
            vec = self._estimate(top, [l for l in all_loops if level_of.get(id(l)) == ("range", TEAM_HANDLE, THREAD_VECTOR)])
            if depth >= 3:
                team = self._estimate(top, [l for l in all_loops if level_of.get(id(l)) == ("range", TEAM_HANDLE, TEAM_THREAD)])
        mapping = NestMapping("device" if offload else "host", depth, tree, vec, team)
        mapping.csr_spmv = self.match_csr_spmv(top) if space == DEVICE else None
        mapping.depth1 = self.match_depth1(top) if space == DEVICE and depth == 1 else None
        mapping.csr_spmm = self.match_csr_spmm(top) if space == DEVICE and not mapping.csr_spmv else None
        if hip_kernels and mapping.csr_spmv:
            # the kernel library takes this nest over; its plan reads the row statistics once, so no estimate
            # (and with it no host read of the positions) is left before the launch
            mapping.vector_length_hint = None
        return mapping

    def _collect(self, loop, out):
        for c in loop.inner:
            out.append(c)
            self._collect(c, out)

    def _mark(self, loop, what, level_of):
        for c in loop.inner:
            level_of[id(c)] = what(c)
            self._mark(c, what, level_of)

    def _map_nested(self, loop, remaining, level_of):
        for child in loop.inner:
            sequential = remaining == 1 and child.levels > 1
            self._map_nested(child, remaining - (0 if sequential else 1), level_of)
            if sequential:
                level_of[id(child)] = ("for",)
            elif remaining == 2:
                level_of[id(child)] = ("range", TEAM_HANDLE, TEAM_VECTOR if child.levels == 1 else TEAM_THREAD)
            else:
                level_of[id(child)] = ("range", TEAM_HANDLE, THREAD_VECTOR)

    def _build(self, loop, level_of, in_team, in_thread, in_vector, team_sync):
        what = level_of[id(loop)]
        if what[0] == "team":
            node = Node("team_parallel", results=loop.results)
            in_team, in_thread, in_vector = True, False, False
        elif what[0] == "thread":
            node = Node("thread_parallel", results=loop.results)
            in_thread, in_vector = True, False
        elif what[0] == "range":
            node = Node("range_parallel", space=what[1], level=what[2], ivs=len(loop.ivs), results=loop.results)
            if what[2] == TEAM_THREAD:
                in_thread = True
            in_vector = what[2] in (THREAD_VECTOR, TEAM_VECTOR)
        else:
            node = Node("for")
        parallel = what[0] != "for"
        self._body(loop.body, node, loop, level_of, in_team, in_thread, in_vector, team_sync, parallel)
        return node

    def _wrap(self, op_node, in_team, in_thread, in_vector, team_sync, out):
        if in_team and not in_thread:
            single = Node("single", level=PER_TEAM)
            single.children.append(op_node)
            out.append(single)
            if team_sync:
                out.append(Node("team_barrier"))
        elif in_thread and not in_vector:
            single = Node("single", level=PER_THREAD)
            single.children.append(op_node)
            out.append(single)
        else:
            out.append(op_node)

    def _body(self, stmts, node, loop, level_of, in_team, in_thread, in_vector, team_sync, parallel):
        for s in stmts:
            if s.op == "scf.parallel":
                inner = next(c for c in loop.inner if c.stmt is s) if any(c.stmt is s for c in loop.inner) else None
                if inner is None:   # nested through another region-holding op: find it anywhere below
                    inner = self._find(loop, s)
                child = self._build(inner, level_of, in_team, in_thread, in_vector, team_sync)
                node.children.append(child)
                what = level_of[id(inner)]
                if team_sync and what[0] == "range" and what[2] in (TEAM_THREAD, TEAM_VECTOR) and inner.results == 0:
                    node.children.append(Node("team_barrier"))
            elif s.op == "scf.reduce":
                # one update per reduced value; a loop that became sequential carries its value instead
                count = len(s.regions)
                if parallel:
                    for _ in range(count):
                        self._wrap(Node("update_reduction"), in_team, in_thread, in_vector, team_sync, node.children)
            elif s.op in _NEEDS_SINGLE:
                self._wrap(Node(s.op.split(".")[1]), in_team, in_thread, in_vector, team_sync, node.children)
            elif s.regions:
                holder = Node(s.op.split(".")[-1]) if s.op == "scf.for" else Node(s.op)
                for _, sub in s.regions:
                    self._body(sub, holder, loop, level_of, in_team, in_thread, in_vector, team_sync, parallel)
                if holder.children:
                    node.children.append(holder)

    def _find(self, loop, stmt):
        for c in loop.inner:
            if c.stmt is stmt:
                return c
            got = self._find(c, stmt)
            if got is not None:
                return got
        return None


def map_function_body(body_text, hip_kernels=False):
    """[NestMapping] for the top-level scf.parallel nests of one function body, in program order.
    `hip_kernels`: a nest that is the CSR SpMV nest goes to the kernel library and gets no estimate."""
    stmts, _ = _mt.read_region(body_text)
    return map_statements(stmts, hip_kernels)


def map_statements(stmts, hip_kernels=False):
    """map_function_body for a body that is already read: `.stmt` of every NestMapping is the caller's own
    `scf.parallel` Statement object."""
    loops = []
    _walk_loops(stmts, None, loops)
    tops = [l for l in loops if l.parent is None]
    for t in tops:
        _set_levels(t)
    mapper = _Mapper(stmts)
    out = []
    for t in tops:
        mapping = mapper.map_nest(t, hip_kernels)
        mapping.stmt = t.stmt
        out.append(mapping)
    return out


def map_module(text, hip_kernels=False):
    """{function name: [NestMapping, ...]} for every function with a body."""
    out = {}
    for f in _mt.read_functions(text):
        if f.body is not None:
            out[f.name] = map_function_body(f.body, hip_kernels)
    return out


# ---- reading a module the pass has already rewritten -------------------------------------------------

def _normalise_generic(text):
    text = _mt.strip_comments(text)
    text = re.sub(r'"(kokkos\.[\w.]+)"', r"\1", text)
    return text.replace("({", "{").replace("})", "}")


def _attr(head, name):
    m = re.search(name + r"\s*=\s*(\d+)", head)
    return int(m.group(1)) if m else None


def _mapped_nodes(stmts, out):
    for s in stmts:
        if s.op == "kokkos.range_parallel":
            m = re.match(r"\s*\(([^)]*)\)", s.head)
            node = Node("range_parallel", space=_attr(s.head, "executionSpace"), level=_attr(s.head, "parallelLevel"),
                        ivs=len(m.group(1).split(",")), results=len(s.results))
        elif s.op in ("kokkos.thread_parallel", "kokkos.team_parallel"):
            node = Node(s.op.split(".")[1], results=len(s.results))
        elif s.op == "kokkos.single":
            node = Node("single", level=_attr(s.head, "level"))
        elif s.op == "kokkos.team_barrier":
            out.append(Node("team_barrier"))
            continue
        elif s.op == "kokkos.update_reduction":
            out.append(Node("update_reduction"))      # its region is the combiner, not part of the structure
            continue
        elif s.op in _NEEDS_SINGLE:
            out.append(Node(s.op.split(".")[1]))
            continue
        elif s.op == "scf.for":
            node = Node("for")
        elif s.regions:
            node = Node(s.op)
        else:
            continue
        for _, sub in s.regions:
            _mapped_nodes(sub, node.children)
        if node.kind in ("for",) or not node.kind.startswith(("scf.", "memref.", "arith.")) or node.children:
            out.append(node)


def mapped_summary(text):
    """{function name: [summary of each top-level kokkos loop]} of text the mapping pass produced."""
    text = _normalise_generic(text)
    out = {}
    for f in _mt.read_functions(text):
        if f.body is None:
            continue
        stmts, _ = _mt.read_region(f.body)
        nodes = []
        _mapped_nodes(stmts, nodes)
        out[f.name] = [n.summary() for n in nodes if n.kind in ("range_parallel", "thread_parallel", "team_parallel")]
    return out


def mapped_hints(text):
    """{function name: [(vector length hint, team size hint) per thread_parallel / team_parallel]} of mapped
    text, each hint written out as an expression over values defined before the loop (None = constant 0 =
    no hint)."""
    text = _normalise_generic(text)
    out = {}
    for f in _mt.read_functions(text):
        if f.body is None:
            continue
        stmts, _ = _mt.read_region(f.body)
        defs = {}
        for s in stmts:
            for r in s.results:
                defs[r.split(":")[0]] = s

        def expr(v):
            if v not in defs:
                return v
            s = defs[v]
            ops = _mt._VALUE.findall(s.head.split(":")[0])
            if s.op == "arith.constant":
                return re.match(r"\s*(-?\w+)", s.head).group(1)
            if s.op in _CASTS:
                return expr(ops[0])
            if s.op == "memref.load":
                return "load(%s)" % ",".join(expr(o) for o in ops)
            if s.op == "memref.dim":
                return v
            return "%s(%s)" % (s.op.split(".")[1], ",".join(expr(o) for o in ops))

        hints = []
        for s in stmts:
            if s.op in ("kokkos.thread_parallel", "kokkos.team_parallel"):
                ops = _mt._VALUE.findall(s.head.split("{region}")[0])
                ex = [expr(o) for o in ops]
                ex = [None if e == "0" else e for e in ex]
                hints.append((ex[1], None) if s.op == "kokkos.thread_parallel" else (ex[2], ex[1]))
        out[f.name] = hints
    return out
