"""``KokkosBackend``-shaped front door: ``KokkosBackend(...).compile(module)`` returns a
``LAPISModule``, as python/lapis/KokkosBackend.py:13,83 of the reference does, so an
example script runs with only its import line changed::

    from lapis_amd import KokkosBackend          # was: from lapis import KokkosBackend
    backend = KokkosBackend.KokkosBackend(decompose_tensors=True)
    module_kokkos = backend.compile(moduleText)
    module_kokkos.spmv(rowptrs, colinds, values, ((m, n), (len(rowptrs), len(colinds), len(values))), x, y)

Nothing is compiled at run time: there is no MLIR here.  ``compile`` reads the module, reduces every
public function (with the private functions it calls) to a canonical form that keeps the operations and
their data flow and drops every name (lapis_amd/mlir_text.py), and looks that form up among the
computations the prebuilt gfx950 module implements (lapis_amd/catalogue.py).  A function binds because
of WHAT it computes: ``@matvec`` doing ``linalg.matvec`` on a CSR operand binds to the SpMV entry point
under its own name, while a ``@spmv`` that multiplies by the transpose, or takes a CSC operand, is
refused with the reference's message for a failed lowering.
"""
import os

from . import catalogue as _catalogue
from . import mlir_text as _mt
from . import module as _module

_LOWERING_FAILED = "Lowering to Kokkos dialect failed."

_catalogue_forms = None


def _forms():
    """canonical form -> entry point of the prebuilt module"""
    global _catalogue_forms
    if _catalogue_forms is None:
        forms = {}
        for entry, text in _catalogue.entries():
            forms[_mt.Canonicalizer(text).canonical("f")] = entry
        _catalogue_forms = forms
    return _catalogue_forms


def _public_functions(text):
    """(name, argument kinds, has a result) of the module's public functions."""
    c = _mt.Canonicalizer(text)
    return [(f.name, c.signature(f)[0], bool(f.results)) for f in c.public()]


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
        """{method name: entry point of the prebuilt module} for the module's public functions.

        The method name is the function's own (``main`` becomes ``lapis_main`` as in the emitter,
        TranslateToKokkosCpp.cpp:2351-2355); the entry point is found by what the function computes."""
        try:
            c = _mt.Canonicalizer(moduleText)
            public = c.public()
        except _mt.ParseError as e:
            raise Exception(_LOWERING_FAILED + "\nthe module text could not be read: %s" % e)
        if not public:
            raise Exception(_LOWERING_FAILED)
        bound = {}
        self.unbound = []
        for f in public:
            method = "lapis_main" if f.name == "main" else f.name
            kinds, results = c.signature(f)
            if f.body is None:
                raise Exception(_LOWERING_FAILED + "\n@%s is declared without a body" % f.name)
            try:
                form = c.canonical(f.name)
            except _mt.ParseError as e:
                raise Exception(_LOWERING_FAILED + "\n@%s could not be read: %s" % (f.name, e))
            entry = _forms().get(form)
            if entry is None:
                if not results:
                    # a helper that returns nothing (the sparse_tensor.print wrapper of examples/bspmm.py:54-58):
                    # compiled by the reference, not implemented here; the rest of the module still binds
                    self.unbound.append(method)
                    continue
                sparse = [k for k in kinds if k.startswith("sparse(")]
                why = ("its sparse operand is stored as %s; the module implements CSR and CSRV with 32-bit positions "
                       "and coordinates" % sparse[0][7:-1]) if sparse else \
                    "what it computes is not one of the CSR SpMV / SpMM / CG functions the gfx950 module implements"
                raise Exception("%s\nfunction @%s(%s): %s" % (_LOWERING_FAILED, f.name, ", ".join(kinds), why))
            if any(k.startswith(("csr:", "csrv:")) for k in kinds) and not self.decompose_tensors:
                raise Exception(_LOWERING_FAILED + "\n@%s takes a sparse tensor: pass decompose_tensors=True "
                                "(positions, coordinates, values and the storage specifier as separate arguments)" % f.name)
            bound[method] = entry
        return bound

    def compile(self, module):
        moduleText = str(module)
        if self.dump_mlir:
            print("== High-Level ==")
            print(moduleText)
        bound = self.bind(moduleText)
        mod = _module.LAPISModule()
        mod.bound_functions = sorted(bound)
        for method, entry in bound.items():
            if method != entry:
                setattr(mod, method, getattr(mod, entry))  # the function's own name, the entry its body calls for
        for name in self.unbound:
            def _not_implemented(*args, _name=name, **kwargs):
                raise NotImplementedError("@%s is outside the CSR SpMV / SpMM / CG path the gfx950 module implements" % _name)
            setattr(mod, name, _not_implemented)
        return mod
