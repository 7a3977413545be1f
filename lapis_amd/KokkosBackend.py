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

A module that is already lowered to loops binds too: a function whose one `scf.parallel` nest is the CSR
SpMV nest the sparsifier produces (lapis_amd/loop_mapping.py decides the Kokkos level of every loop by the
rules of the reference's loop-mapping pass and recognises that nest) is bound to the SpMV entry point, with
its memref arguments routed by the ROLE each plays in the nest (y, positions, coordinates, values, x).

Every other function made of the path's vocabulary -- `linalg.matvec` / `matmul` on CSR operands, `linalg.dot`,
fill, copy, elementwise `linalg.generic` bodies, `tensor.*`, scalar `arith` / `math.sqrt`, `scf.while` / `for` /
`if`, calls of private functions, and loop nests the kernel library has entry points for -- is run operation by
operation on device-resident tensors (lapis_amd/executor.py): a CG written with other helper functions, an
SpMV followed by an axpby, a Richardson iteration bind although no whole-function entry point exists for them.
A function that uses anything else is refused, with the operation named.
"""
import os

import re

from . import catalogue as _catalogue
from . import executor as _executor
from . import loop_mapping as _lm
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


def _spmv_by_role(mod, order):
    """Method for a loop-level SpMV function: memref arguments in the function's own order, y updated in place."""
    def method(*args):
        if len(args) != 5:
            raise TypeError("expected 5 memref arguments, got %d" % len(args))
        y, pos, crd, val, x = (args[order[r]] for r in ("y", "pos", "crd", "val", "x"))
        mod.spmv(pos, crd, val, ((len(y), len(x)), (len(pos), len(crd), len(val))), x, y)
    return method


def _run_by_operation(mod, ex, c, fname, decompose_tensors):
    """Method for a function the executor runs operation by operation.  Arguments as the reference's wrapper
    takes them (TranslateToKokkosCpp.cpp:2757-2977): a sparse tensor as positions, coordinates, values and the
    specifier ((rows, columns), (len(pos), len(crd), len(val))), dense tensors and memrefs as numpy arrays,
    scalars as Python numbers.  Tensor results come back as new numpy arrays, memref arguments are updated
    in place; one result is returned as itself, several as a tuple."""
    f = c.functions[fname]
    kinds, _ = c.signature(f)
    types = [ty for _, ty in f.args]

    def method(*params, _keep=mod):
        import numpy
        import torch
        params = list(params)
        args, written = [], []
        np_of = {"f64": numpy.float64, "f32": numpy.float32, "i32": numpy.int32, "i64": numpy.int64, "index": numpy.int64}

        def up(a, elem):
            return torch.from_numpy(numpy.array(a, dtype=np_of[elem], order="C")).to(ex.device)

        def take():
            if not params:
                raise TypeError("@%s: too few arguments" % fname)
            return params.pop(0)

        for kind, ty in zip(kinds, types):
            ty = ty.strip()
            if kind.startswith("csr:"):
                if not decompose_tensors:
                    raise TypeError("@%s takes a sparse tensor: compile with decompose_tensors=True" % fname)
                pos, crd, val, spec = take(), take(), take(), take()
                args.append(_executor.Csr(up(pos, "i32"), up(crd, "i32"), up(val, kind[4:]), spec[0][0], spec[0][1]))
            elif ty.startswith("tensor<"):
                dims, elem = _executor._shape_spec(ty)
                a = take()
                args.append(up(a, elem) if dims else (numpy.float32(a) if elem == "f32" else float(a)))
            elif ty.startswith("memref<"):
                dims, elem = _executor._shape_spec(ty)
                a = take()
                if not dims:
                    args.append(_executor.Cell(numpy.asarray(a).reshape(-1)[0]))
                    written.append((a, args[-1]))
                else:
                    args.append(up(a, elem))
                    if elem in ("f64", "f32"):
                        written.append((a, args[-1]))
            elif ty in ("f64", "f32"):
                a = take()
                args.append(numpy.float32(a) if ty == "f32" else float(a))
            else:
                args.append(int(take()))
        if params:
            raise TypeError("@%s: %d arguments too many" % (fname, len(params)))
        try:
            results = ex.run(fname, args)
            out = []
            for r in results:
                if isinstance(r, torch.Tensor):
                    out.append(r.cpu().numpy())
                elif isinstance(r, _executor.Cell):
                    out.append(r.value)
                else:
                    out.append(r.item() if isinstance(r, numpy.generic) and not isinstance(r, numpy.floating) else r)
            for host, dev in written:
                if isinstance(dev, _executor.Cell):
                    numpy.asarray(host).reshape(-1)[0] = dev.value
                elif isinstance(host, numpy.ndarray) and host.flags.writeable:
                    numpy.copyto(host, dev.cpu().numpy().reshape(host.shape))
        finally:
            for a in args:
                if isinstance(a, _executor.Csr):
                    a.release()
            ex.release()
        if not out:
            return None
        return out[0] if len(out) == 1 else tuple(out)
    return method


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
        TranslateToKokkosCpp.cpp:2351-2355); the entry point is found by what the function computes.
        Text that cannot be read as MLIR fails like any other module the reference cannot lower
        (python/lapis/KokkosBackend.py:36), whatever the reader stumbled over."""
        try:
            return self._bind(moduleText)
        except (_mt.ParseError, ValueError, IndexError, KeyError, AttributeError, RecursionError) as e:
            raise Exception(_LOWERING_FAILED + "\nthe module text could not be read: %s%s" % (
                "" if isinstance(e, _mt.ParseError) else type(e).__name__ + ": ", e))

    def _bind(self, moduleText):
        try:
            c = _mt.Canonicalizer(moduleText)
            public = c.public()
        except _mt.ParseError as e:
            raise Exception(_LOWERING_FAILED + "\nthe module text could not be read: %s" % e)
        if not public:
            raise Exception(_LOWERING_FAILED)
        bound = {}
        self._canonicalizer = c
        self._executor = None
        self.unbound = []
        self.loop_mapping = {}   # function name -> loop_mapping.NestMapping of a function bound at loop level
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
                entry, why_not = self._loop_level_entry(f)
            if entry is None and (results or f.args):
                # no whole-function entry point: operation by operation, if every operation has one
                try:
                    self.executor(c).check(f.name)
                    entry = ("exec", f.name)
                except _executor.Refused as e:
                    if not (not results and "sparse_tensor.print" in f.body):
                        sparse = [k for k in kinds if k.startswith("sparse(")]
                        raise Exception("%s\nfunction @%s(%s): it uses %s%s" % (
                            _LOWERING_FAILED, f.name, ", ".join(kinds), e,
                            "" if not why_not else "; as one loop nest: " + why_not))
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

    def executor(self, c=None):
        if getattr(self, "_executor", None) is None:
            self._executor = _executor.Executor(c or self._canonicalizer)
        return self._executor

    def _loop_level_entry(self, f):
        """(("loops:spmv", {role: argument index}), None) when @f is one CSR SpMV loop nest over 32-bit
        positions and coordinates and nothing else; (None, reason) for any other function made of loops;
        (None, None) for a function without `scf.parallel`."""
        if "scf.parallel" not in f.body:
            return None, None
        try:
            nests = _lm.map_function_body(f.body, hip_kernels=True)
        except (_mt.ParseError, AttributeError, ValueError) as e:
            return None, "its loops could not be read: %s" % e
        described = "; ".join("%s nest of depth %d" % (n.space, n.depth) for n in nests)
        if len(nests) != 1 or not nests[0].csr_spmv or f.results:
            return None, ("its loops (%s) are not the one CSR SpMV nest y[i] += sum_j val[pos[i]+j] * x[crd[pos[i]+j]] "
                          "the gfx950 module implements" % described)
        roles = nests[0].csr_spmv
        stmts, _ = _mt.read_region(f.body)
        if any(s.op not in ("arith.constant", "memref.dim", "scf.parallel", "return", "func.return") for s in stmts):
            return None, "it does more than the one CSR SpMV nest"
        names = [nm for nm, _ in f.args]
        types = dict(f.args)
        order = {}
        for role in ("y", "pos", "crd", "val", "x"):
            if roles[role] not in names:
                return None, "the %s buffer of its SpMV nest is not a function argument" % role
            order[role] = names.index(roles[role])
            want = "i32" if role in ("pos", "crd") else roles["elem"]
            have = types[roles[role]].replace(" ", "")
            if not re.match(r"memref<\?x%s>$" % want, have):
                return None, ("the %s buffer of its SpMV nest is %s; the module implements 32-bit positions and "
                              "coordinates and contiguous one-dimensional memref<?x%s>" % (role, have, want))
        if len(set(order.values())) != 5:
            return None, "two buffers of its SpMV nest are the same argument"
        self.loop_mapping[f.name] = nests[0]
        return ("loops:spmv", order), None

    def compile(self, module):
        moduleText = str(module)
        if self.dump_mlir:
            print("== High-Level ==")
            print(moduleText)
        bound = self.bind(moduleText)
        mod = _module.LAPISModule()
        mod.bound_functions = sorted(bound)
        # python/lapis/KokkosBackend.py:21-24,113-114: the package of instance k is lapis_package_k, and only the
        # last of `num_instances` modules is emitted with --finalize (it shuts Kokkos down).  Here every module
        # shares one prebuilt library whose lapis_initialize / lapis_finalize count the live modules, so the
        # runtime goes down with the last module whichever index it has; the two attributes record what the
        # reference would have generated.
        mod.package_name = self.package_name
        mod.finalizes_runtime = self.num_instances == 0 or self.index_instance == self.num_instances - 1
        for method, entry in bound.items():
            if isinstance(entry, tuple) and entry[0] == "exec":
                setattr(mod, method, _run_by_operation(mod, self.executor(), self._canonicalizer, entry[1],
                                                       self.decompose_tensors))
            elif isinstance(entry, tuple):
                setattr(mod, method, _spmv_by_role(mod, entry[1]))
            elif method != entry:
                setattr(mod, method, getattr(mod, entry))  # the function's own name, the entry its body calls for
        for name in self.unbound:
            def _not_implemented(*args, _name=name, **kwargs):
                raise NotImplementedError("@%s is outside the CSR SpMV / SpMM / CG path the gfx950 module implements" % _name)
            setattr(mod, name, _not_implemented)
        return mod
