"""``KokkosBackend``-shaped front door: ``KokkosBackend(...).compile(module)`` returns a
``LAPISModule``, as python/lapis/KokkosBackend.py:13,83 of the reference does, so an
example script runs with only its import line changed::

    from lapis_amd import KokkosBackend          # was: from lapis import KokkosBackend
    backend = KokkosBackend.KokkosBackend(decompose_tensors=True)
    module_kokkos = backend.compile(moduleText)
    module_kokkos.spmv(rowptrs, colinds, values, ((m, n), (len(rowptrs), len(colinds), len(values))), x, y)

Nothing is compiled at run time: there is no MLIR here.  ``compile`` reads the
signatures of the module's public functions, checks each one against the catalogue
of functions the prebuilt gfx950 module implements (the CSR SpMV / SpMM / CG path)
and binds them.  A module asking for anything else raises, with the reference's own
message for a failed lowering.
"""
import os
import re

from . import module as _module

# public function name -> (kind, result count); `main` is renamed as the emitter does
# (TranslateToKokkosCpp.cpp:2351-2355)
_FUNC_RE = re.compile(r"func\.func\s+(private\s+)?@([A-Za-z_][\w$.]*)\s*\(([^)]*)\)\s*(?:->\s*(\([^)]*\)|[^\s{]+(?:\s*<[^{]*>)?))?", re.S)


def _public_functions(text):
    funcs = []
    for m in _FUNC_RE.finditer(text):
        if m.group(1):
            continue
        name = m.group(2)
        args = [a.strip() for a in _split_top(m.group(3))] if m.group(3).strip() else []
        funcs.append((name, args, bool(m.group(4))))
    return funcs


def _split_top(s):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "<([{":
            depth += 1
        elif ch in ">)]}":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur)
    return out


def _classify(arg):
    """'csr' for a 2-D tensor with an encoding attribute, 'vec'/'mat' for dense tensors, 'scalar' otherwise."""
    m = re.search(r"tensor<([^>]*)", arg)
    if not m:
        return "scalar"
    body = m.group(1)
    dims = body.count("x")
    if "#" in arg.split("tensor<", 1)[1]:
        return "csr" if dims == 2 else ("csrv" if dims == 3 else "sparse")
    return {1: "vec", 2: "mat"}.get(dims, "dense%d" % dims)


# what the prebuilt module implements: name -> argument kinds
_CATALOGUE = {
    "spmv": ["csr", "vec", "vec"],
    "lapis_main": ["csr", "vec"],
    "pcg": ["csr", "vec", "vec", "scalar", "scalar"],
    "spmm": ["csr", "mat", "mat"],
    "plus_norm": ["vec", "vec"],
    "mht": ["csr", "vec", "vec", "scalar", "scalar", "scalar"],
    "normalize_mom2": ["vec", "vec"],
    "pte_local_bspmm": ["csrv", "dense3"],
}


class KokkosBackend:
    """Same constructor as the reference's class (python/lapis/KokkosBackend.py:13)."""

    def __init__(self, decompose_tensors=False, parallel_strategy="any-storage-any-loop", dump_mlir=False,
                 index_instance=0, num_instances=0, ws=os.getcwd()):
        self.dump_mlir = dump_mlir
        self.ws = ws
        self.index_instance = index_instance
        self.num_instances = num_instances
        self.decompose_tensors = decompose_tensors
        self.parallel_strategy = parallel_strategy
        self.package_name = "lapis_package" if index_instance == 0 else "lapis_package_" + str(index_instance)

    def bind(self, moduleText):
        """Names of the module's public functions after checking them against the catalogue."""
        funcs = _public_functions(moduleText)
        if not funcs:
            raise Exception("Lowering to Kokkos dialect failed.")
        names = []
        self.unbound = []
        for name, args, has_result in funcs:
            bound = "lapis_main" if name == "main" else name
            kinds = [_classify(a) for a in args]
            if bound not in _CATALOGUE and not has_result:
                # a helper that returns nothing (the sparse_tensor.print wrapper of examples/bspmm.py:54-58):
                # compiled by the reference, not implemented here; the rest of the module still binds
                self.unbound.append(bound)
                continue
            if bound not in _CATALOGUE or _CATALOGUE[bound] != kinds:
                raise Exception("Lowering to Kokkos dialect failed.\nfunction @%s(%s) is outside the CSR SpMV / SpMM / CG "
                                "path the gfx950 module implements" % (name, ", ".join(kinds)))
            if ("csr" in kinds or "csrv" in kinds) and not self.decompose_tensors:
                raise Exception("Lowering to Kokkos dialect failed.\n@%s takes a sparse tensor: pass decompose_tensors=True "
                                "(positions, coordinates, values and the storage specifier as separate arguments)" % name)
            names.append(bound)
        return names

    def compile(self, module):
        moduleText = str(module)
        if self.dump_mlir:
            print("== High-Level ==")
            print(moduleText)
        names = self.bind(moduleText)
        mod = _module.LAPISModule()
        mod.bound_functions = names
        for name in self.unbound:
            def _not_implemented(*args, _name=name, **kwargs):
                raise NotImplementedError("@%s is outside the CSR SpMV / SpMM / CG path the gfx950 module implements" % _name)
            setattr(mod, name, _not_implemented)
        return mod
