"""ctypes descriptors for MLIR ranked memrefs over numpy arrays.

The wrappers the reference emits import these helpers from ``mlir.runtime``
(TranslateToKokkosCpp.cpp:4397, used at :2897-2962); that package is not a
dependency here, so the three functions the wrappers use are provided with the
same names and meaning: ``make_nd_memref_descriptor``,
``get_ranked_memref_descriptor`` and ``ranked_memref_to_numpy``.
The layout is StridedMemRefType<T,N> of LAPISSupport.hpp:7-14:
``{T* basePtr; T* data; int64 offset; int64 sizes[N]; int64 strides[N]}``.
"""
import ctypes

import numpy as np

_CACHE = {}


def make_nd_memref_descriptor(rank, ctype):
    """Descriptor class of a rank-``rank`` memref with element type ``ctype``."""
    key = (rank, ctype)
    cls = _CACHE.get(key)
    if cls is None:
        fields = [("allocated", ctypes.POINTER(ctype)), ("aligned", ctypes.POINTER(ctype)), ("offset", ctypes.c_longlong)]
        if rank > 0:
            fields += [("shape", ctypes.c_longlong * rank), ("strides", ctypes.c_longlong * rank)]
        cls = type("MemRefDescriptor_%d_%s" % (rank, ctype.__name__), (ctypes.Structure,), {"_fields_": fields})
        _CACHE[key] = cls
    return cls


def get_ranked_memref_descriptor(array):
    """Descriptor aliasing a numpy array (strides in elements, as MLIR counts them)."""
    array = np.asarray(array)
    ctype = np.ctypeslib.as_ctypes_type(array.dtype)
    desc = make_nd_memref_descriptor(array.ndim, ctype)()
    ptr = ctypes.cast(ctypes.c_void_p(array.ctypes.data), ctypes.POINTER(ctype))
    desc.allocated = ptr
    desc.aligned = ptr
    desc.offset = 0
    if array.ndim > 0:
        desc.shape = (ctypes.c_longlong * array.ndim)(*array.shape)
        desc.strides = (ctypes.c_longlong * array.ndim)(*[s // array.itemsize for s in array.strides])
    desc._keepalive = array
    return desc


def ranked_memref_to_numpy(desc):
    """numpy view aliasing the memory a descriptor points at (no copy, no ownership).

    Takes a pointer to a descriptor, as the emitted wrappers pass it (``ret0[0]``), or
    the descriptor itself."""
    if not hasattr(desc, "aligned"):
        desc = desc[0]
    rank = len(desc.shape) if hasattr(desc, "shape") else 0
    shape = tuple(desc.shape) if rank else ()
    ctype = type(desc.aligned.contents) if bool(desc.aligned) else desc._fields_[1][1]._type_
    dtype = np.dtype(ctype)
    count = int(np.prod(shape)) if rank else 1
    if count == 0 or not bool(desc.aligned):
        return np.zeros(shape, dtype=dtype)
    base = ctypes.addressof(desc.aligned.contents) + desc.offset * dtype.itemsize
    extent = 1 + sum((s - 1) * st for s, st in zip(shape, desc.strides)) if rank else 1
    flat = np.ctypeslib.as_array((ctype * extent).from_address(base))
    if rank == 0:
        return flat.reshape(())
    return np.lib.stride_tricks.as_strided(flat, shape=shape, strides=[st * dtype.itemsize for st in desc.strides])
